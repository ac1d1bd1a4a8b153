"""Plans that checksum the image while they copy it (plan option ``crc_chunk_kib``): the bytes moved are the same as
without the option, and the per-chunk CRC-32C values equal those of the stand-alone checksum pass and of the CPU
oracle's C routine - for every source/target misalignment, for chunks of 64 KiB to 32 MiB (one to 512 workgroups per
group), with record headers, item edges, strided views and a short last chunk in the image."""

import numpy as np
import pytest
import torch

from oracle import mlf_format as oracle_fmt

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _oracle_chunks(oracle_c, raw: bytes, chunk: int) -> np.ndarray:
    want = np.zeros(-(-len(raw) // chunk), dtype=np.uint32)
    oracle_c.oracle_crc32c_chunks(raw, len(raw), chunk, want.ctypes.data)
    return want


def _misaligned_tensors(sizes, seed):
    """Contiguous uint8 device tensors whose addresses are off the 16-byte grid by 0, 1, 2 ... bytes."""
    gen = torch.Generator(device=DEV).manual_seed(seed)
    out = []
    for k, n in enumerate(sizes):
        parent = torch.randint(0, 256, (n + 64,), dtype=torch.uint8, device=DEV, generator=gen)
        t = parent[k % 16 : k % 16 + n]
        assert t.data_ptr() % 16 == (parent.data_ptr() + k % 16) % 16
        out.append(t)
    return out


@pytest.mark.parametrize("chunk", [65536, 1 << 20, 4 << 20, 32 << 20])
def test_pack_with_checksums_matches_plain_pack_and_oracle(chunk, oracle_c):
    from ml_flashpoint.hip import plan as P

    # 17 tensors of 0.3 .. 9 MB at every byte misalignment; record headers in between put the payloads at odd offsets
    sizes = [(300 << 10) + 4099 * k + (k % 5) * (1 << 21) for k in range(17)]
    if chunk == 32 << 20:
        sizes += [(40 << 20) + 7]  # room for a whole group of 512 workgroups
    tensors = _misaligned_tensors(sizes, seed=3)
    layout = P.build_save_layout(tensors)
    plain = P.Plan(layout.items, layout.blob, layout.image_bytes)
    fused = P.Plan(layout.items, layout.blob, layout.image_bytes, crc_chunk_bytes=chunk)
    info = fused.info
    assert info.crc_chunks == -(-layout.image_bytes // chunk)
    assert info.fused_crc_bytes > 0.5 * layout.image_bytes if chunk <= (4 << 20) else info.fused_crc_bytes >= (32 << 20)
    image_a = torch.full((layout.image_bytes + 512,), 0xAB, dtype=torch.uint8, device=DEV)
    image_b = torch.full((layout.image_bytes + 512,), 0xCD, dtype=torch.uint8, device=DEV)
    plain.pack(image_a)
    fused.pack(image_b)
    got = fused.crc_values()
    torch.cuda.synchronize()
    assert torch.equal(image_a[: layout.image_bytes], image_b[: layout.image_bytes])
    assert bool((image_b[layout.image_bytes :] == 0xCD).all()), "pack wrote past the end of the image"
    raw = image_b[: layout.image_bytes].cpu().numpy().tobytes()
    want, spans = oracle_fmt.data_section([t.cpu() for t in tensors])
    assert raw == want and layout.spans == spans
    assert got.tolist() == P.crc32c_device(image_b, layout.image_bytes, chunk).tolist()
    assert got.tolist() == _oracle_chunks(oracle_c, raw, chunk).tolist()
    # a second launch of the same plan over changed tensors: new bytes, new values, nothing left over
    for t in tensors:
        t.add_(1)
    fused.pack(image_b)
    got2 = fused.crc_values()
    raw2 = image_b[: layout.image_bytes].cpu().numpy().tobytes()
    assert raw2 == oracle_fmt.data_section([t.cpu() for t in tensors])[0]
    assert got2.tolist() == _oracle_chunks(oracle_c, raw2, chunk).tolist() and got2.tolist() != got.tolist()


def test_pack_with_checksums_mixed_items(oracle_c):
    """Small items, strided and transposed views, host-resident items and byte blobs beside large contiguous ones."""
    from ml_flashpoint.hip import plan as P

    gen = torch.Generator(device=DEV).manual_seed(5)
    big = torch.randint(0, 256, (6 << 20,), dtype=torch.uint8, device=DEV, generator=gen)
    base = torch.randint(0, 2**15, (1024, 768), dtype=torch.int16, device=DEV, generator=gen)
    tensors = [
        torch.randn(3, 5, device=DEV, generator=gen),
        big[3:].view(torch.uint8),
        base.t(),
        base[:, ::2],
        torch.randn(700_001, device=DEV, generator=gen).to(torch.bfloat16),
        torch.arange(40_000, dtype=torch.int64),  # host-resident: rides in the blob
        base[16:528],
        torch.randn(1 << 20, device=DEV, generator=gen),
    ]
    blobs = [b"", bytes(range(256)) * 300, b"tail"]
    layout = P.build_save_layout(tensors, blobs)
    chunk = 1 << 20
    fused = P.Plan(layout.items, layout.blob, layout.image_bytes, crc_chunk_bytes=chunk)
    image = torch.zeros(layout.image_bytes, dtype=torch.uint8, device=DEV)
    fused.pack(image)
    got = fused.crc_values()
    raw = image.cpu().numpy().tobytes()
    assert raw == oracle_fmt.data_section([t.cpu() for t in tensors], blobs)[0]
    assert got.tolist() == _oracle_chunks(oracle_c, raw, chunk).tolist()
    info = fused.info
    assert info.fused_crc_bytes > 0 and info.n_strided_items > 0 and info.n_transposed_items > 0


@pytest.mark.parametrize("nbytes", [1, 4095, 65535, 65536, 65537, (1 << 20) - 1, (1 << 20) + 4096, (3 << 20) + 12345])
def test_pack_with_checksums_small_images(nbytes, oracle_c):
    from ml_flashpoint.hip import plan as P

    gen = torch.Generator(device=DEV).manual_seed(nbytes)
    t = torch.randint(0, 256, (nbytes,), dtype=torch.uint8, device=DEV, generator=gen)
    layout = P.build_save_layout([t])
    for chunk in (65536, 1 << 20):
        fused = P.Plan(layout.items, layout.blob, layout.image_bytes, crc_chunk_bytes=chunk)
        image = torch.zeros(layout.image_bytes, dtype=torch.uint8, device=DEV)
        fused.pack(image)
        raw = image.cpu().numpy().tobytes()
        assert fused.crc_values().tolist() == _oracle_chunks(oracle_c, raw, chunk).tolist()


def test_one_item_beyond_4_gib_with_checksums():
    """A single tensor of 5 GiB + 12 345 bytes at a byte-misaligned address: positions inside the item pass 2^32.
    The fused pack moves what the plain pack moves, its per-chunk values equal the stand-alone pass over the image
    (itself held to the host's CRC at 8.5 GiB elsewhere), and the fused unpack brings the tensor back and reports
    the same values."""
    from ml_flashpoint.hip import plan as P

    need = 4 * (5 << 30) + (2 << 30)
    if torch.cuda.mem_get_info()[0] < need:
        pytest.skip("not enough free device memory")
    n = 5 * (1 << 30) + 12345
    gen = torch.Generator(device=DEV).manual_seed(41)
    parent = torch.randint(0, 256, (n + 64,), dtype=torch.uint8, device=DEV, generator=gen)
    tensor = parent[3 : 3 + n]
    layout = P.build_save_layout([tensor])
    chunk = 32 << 20
    plain = P.Plan(layout.items, layout.blob, layout.image_bytes)
    fused = P.Plan(layout.items, layout.blob, layout.image_bytes, crc_chunk_bytes=chunk)
    assert fused.info.fused_crc_bytes > (1 << 32)
    image_a = torch.zeros(layout.image_bytes, dtype=torch.uint8, device=DEV)
    image_b = torch.full((layout.image_bytes + 512,), 0xCD, dtype=torch.uint8, device=DEV)
    plain.pack(image_a)
    fused.pack(image_b)
    got = fused.crc_values()
    torch.cuda.synchronize()
    assert torch.equal(image_a, image_b[: layout.image_bytes])
    assert bool((image_b[layout.image_bytes :] == 0xCD).all()), "pack wrote past the end of the image"
    want = P.crc32c_device(image_b, layout.image_bytes, chunk)
    assert len(got) == -(-layout.image_bytes // chunk) and got.tolist() == want.tolist()
    del image_a, plain, fused
    back = torch.full((n + 64,), 0x5A, dtype=torch.uint8, device=DEV)
    table = P.ItemTable()
    (offset, length), = layout.spans
    table.add_contiguous(back.data_ptr() + 7, offset + length - n, 1, n)
    unpacker = P.Plan(table.to_array(), b"", layout.image_bytes, align_to_tensor=True, crc_chunk_bytes=chunk)
    unpacker.unpack(image_b)
    got = unpacker.crc_values()
    torch.cuda.synchronize()
    assert got.tolist() == want.tolist()
    assert torch.equal(back[7 : 7 + n], tensor)
    assert bool((back[:7] == 0x5A).all()) and bool((back[7 + n :] == 0x5A).all()), "guard bytes"


@pytest.mark.parametrize("chunk", [65536, 1 << 20, 32 << 20])
def test_unpack_with_checksums_restores_and_reports_the_images_values(chunk, oracle_c):
    from ml_flashpoint.hip import plan as P

    sizes = [(200 << 10) + 8191 * k + (k % 3) * (3 << 20) for k in range(16)]
    if chunk == 32 << 20:
        sizes += [(36 << 20) + 3]
    source = _misaligned_tensors(sizes, seed=11)
    layout = P.build_save_layout(source)
    packer = P.Plan(layout.items, layout.blob, layout.image_bytes)
    image = torch.zeros(layout.image_bytes, dtype=torch.uint8, device=DEV)
    packer.pack(image)
    torch.cuda.synchronize()
    raw = image.cpu().numpy().tobytes()
    want = _oracle_chunks(oracle_c, raw, chunk)
    # targets at other misalignments than the sources, with guard bytes around them
    parents = [torch.full((n + 96,), 0x5A, dtype=torch.uint8, device=DEV) for n in sizes]
    targets = [p[32 + (5 * k + 1) % 16 : 32 + (5 * k + 1) % 16 + n] for k, (p, n) in enumerate(zip(parents, sizes))]
    table = P.ItemTable()
    for (offset, length), t in zip(layout.spans, targets):
        n = t.numel()
        table.add_contiguous(t.data_ptr(), offset + length - n, 1, n)
    for align_to_tensor in (True, False):
        for p in parents:
            p.fill_(0x5A)
        plan = P.Plan(table.to_array(), b"", layout.image_bytes, align_to_tensor=align_to_tensor, crc_chunk_bytes=chunk)
        plan.unpack(image)
        got = plan.crc_values()
        torch.cuda.synchronize()
        assert got.tolist() == want.tolist()
        for k, (p, t, s) in enumerate(zip(parents, targets, source)):
            assert torch.equal(t, s), k
            lo = 32 + (5 * k + 1) % 16
            assert bool((p[:lo] == 0x5A).all()) and bool((p[lo + t.numel() :] == 0x5A).all()), f"guard bytes of {k}"
    # a flipped bit in the image shows up in exactly the chunk it lies in
    at = layout.image_bytes // 2
    image[at] ^= 0x10
    plan.unpack(image)
    bad = plan.crc_values()
    assert (bad != want).nonzero()[0].tolist() == [at // chunk]


@pytest.mark.parametrize("align_to_tensor", [True, False])
def test_unpack_with_checksums_one_record_into_two_targets(align_to_tensor, oracle_c):
    """Two items of an unpack plan may read the same range of the image (one stored tensor restored into two targets,
    wholly or in part).  With checksums on, every target is written and the chunk values are those of the image."""
    from ml_flashpoint.hip import plan as P

    sizes = [(1 << 20) + 77, (3 << 20) + 5, 600_001]
    source = _misaligned_tensors(sizes, seed=23)
    layout = P.build_save_layout(source)
    image = torch.zeros(layout.image_bytes, dtype=torch.uint8, device=DEV)
    P.Plan(layout.items, layout.blob, layout.image_bytes).pack(image)
    torch.cuda.synchronize()
    chunk = 1 << 20
    want = _oracle_chunks(oracle_c, image.cpu().numpy().tobytes(), chunk)
    payload_at = [offset + length - n for (offset, length), n in zip(layout.spans, sizes)]
    # (record, first byte of the record's payload, length): the whole of record 1 twice, then a part of it that
    # starts inside a 64 KiB piece another target already owns, then records 0 and 2 once each
    wanted = [(1, 0, sizes[1]), (1, 0, sizes[1]), (1, 70_001, 2 << 20), (0, 0, sizes[0]), (2, 0, sizes[2])]
    parents = [torch.full((n + 96,), 0x5A, dtype=torch.uint8, device=DEV) for _, _, n in wanted]
    targets = [p[32 + (3 * k) % 16 :][:n] for k, (p, (_, _, n)) in enumerate(zip(parents, wanted))]
    table = P.ItemTable()
    for t, (rec, first, n) in zip(targets, wanted):
        table.add_contiguous(t.data_ptr(), payload_at[rec] + first, 1, n)
    plan = P.Plan(table.to_array(), b"", layout.image_bytes, align_to_tensor=align_to_tensor, crc_chunk_bytes=chunk)
    assert plan.info.fused_crc_bytes <= layout.image_bytes  # no piece of the image is counted twice
    plan.unpack(image)
    got = plan.crc_values()
    torch.cuda.synchronize()
    assert got.tolist() == want.tolist()
    for k, (p, t, (rec, first, n)) in enumerate(zip(parents, targets, wanted)):
        assert torch.equal(t, source[rec][first : first + n]), k
        lo = 32 + (3 * k) % 16
        assert bool((p[:lo] == 0x5A).all()) and bool((p[lo + n :] == 0x5A).all()), f"guard bytes of {k}"


def test_checksum_option_argument_checks():
    from ml_flashpoint.hip import _lib
    from ml_flashpoint.hip import plan as P

    t = torch.zeros(1 << 16, dtype=torch.uint8, device=DEV)
    layout = P.build_save_layout([t])
    with pytest.raises(ValueError):
        P.Plan(layout.items, layout.blob, layout.image_bytes, crc_chunk_bytes=1000)
    plain = P.Plan(layout.items, layout.blob, layout.image_bytes)
    out = np.zeros(4, dtype=np.uint32)
    assert _lib.load().mlf_plan_crc_values(plain._handle, out.ctypes.data, 4) != 0
    fused = P.Plan(layout.items, layout.blob, layout.image_bytes, crc_chunk_bytes=65536)
    assert _lib.load().mlf_plan_crc_values(fused._handle, out.ctypes.data, 4) != 0  # not launched yet
    assert b"not been launched" in _lib.load().mlf_hip_last_error()


@pytest.mark.filterwarnings("ignore:torch.distributed is disabled")
@pytest.mark.parametrize("background_write", [False, True])
def test_saver_and_loader_checksum_modes_agree(shm_dir, background_write):
    """The saver's two ways to the sidecar (a pass beside the transfer, or inside the pack kernel) write the same
    object and the same sidecar; the loader's two ways to check it (inside the unpack kernel, or a pass before it)
    restore the same bits and reject the same corrupted chunk."""
    import concurrent.futures
    import os
    import threading

    import torch.distributed.checkpoint as dcp

    import workloads
    from ml_flashpoint.adapter.pytorch.memory_storage_reader import MemoryStorageReader
    from ml_flashpoint.adapter.pytorch.memory_storage_writer import MemoryStorageWriter
    from ml_flashpoint.checkpoint_object_manager.buffer_metadata import METADATA_SIZE
    from ml_flashpoint.checkpoint_object_manager.checkpoint_object_manager import CheckpointObjectManager
    from ml_flashpoint.core.checkpoint_loader import DefaultMLFlashpointCheckpointLoader
    from ml_flashpoint.core.checkpoint_saver import DefaultMLFlashpointCheckpointSaver
    from ml_flashpoint.hip import integrity

    class LocalManager:
        def dict(self):
            return {}

        def Event(self):
            return threading.Event()

    fut = concurrent.futures.Future()
    fut.set_result(LocalManager())
    CheckpointObjectManager._worker_pool = None
    sd = workloads.llama3_8b_shard(DEV, layers=2, d=512, ffn=1792, kv=128, vocab=8000)
    sd["extra.step"] = 7  # a pickled object behind the tensors
    chunk = 1 << 20
    files, sidecars = {}, {}
    for mode in ("beside", "fused"):
        saver = DefaultMLFlashpointCheckpointSaver(lambda: 0, lambda: 0, lambda: None, CheckpointObjectManager(), None,
                                                   initial_buffer_size_bytes=1 << 20, crc_chunk_bytes=chunk, crc_mode=mode,
                                                   background_write=background_write)
        for step in (1, 2):  # the second save of a mode runs on the kept plan
            ckpt = os.path.join(shm_dir, mode, f"step-{step}_ckpt")
            dcp.save(sd, checkpoint_id=ckpt, storage_writer=MemoryStorageWriter(saver, fut), no_dist=True)
            obj = os.path.join(ckpt, "__0__0_src0.distcp")
            files[mode, step] = open(obj, "rb").read()
            sidecars[mode, step] = integrity.read_sidecar(obj)
        assert saver.last_save_stats.get("plans_reused") == 1
    assert files["beside", 1] == files["fused", 1] == files["fused", 2]
    want = sidecars["beside", 1]
    assert want is not None and want[0] == chunk and want[1] == len(files["beside", 1]) - METADATA_SIZE
    for key, got in sidecars.items():
        assert got[:2] == want[:2] and got[2].tolist() == want[2].tolist(), key
    with pytest.raises(ValueError):
        DefaultMLFlashpointCheckpointSaver(lambda: 0, lambda: 0, lambda: None, CheckpointObjectManager(), None, crc_mode="x")

    ckpt = os.path.join(shm_dir, "fused", "step-2_ckpt")
    obj = os.path.join(ckpt, "__0__0_src0.distcp")
    originals = {k: v.clone() for k, v in sd.items() if isinstance(v, torch.Tensor)}
    for mode in ("fused", "before"):
        loader = DefaultMLFlashpointCheckpointLoader(CheckpointObjectManager(), None, crc_mode=mode)
        target = {k: (torch.zeros_like(v) if isinstance(v, torch.Tensor) else None) for k, v in sd.items()}
        dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, loader), no_dist=True)
        assert target["extra.step"] == 7
        assert all(torch.equal(target[k].view(torch.uint8), v.view(torch.uint8)) for k, v in originals.items()), mode
    at = METADATA_SIZE + 5 * chunk + 4321
    with open(obj, "r+b") as f:
        f.seek(at)
        byte = f.read(1)
        f.seek(at)
        f.write(bytes([byte[0] ^ 0x01]))
    for mode in ("fused", "before"):
        loader = DefaultMLFlashpointCheckpointLoader(CheckpointObjectManager(), None, crc_mode=mode)
        target = {k: (torch.zeros_like(v) if isinstance(v, torch.Tensor) else None) for k, v in sd.items()}
        with pytest.raises(BaseException) as exc:
            dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, loader), no_dist=True)
        cause = exc.value.failures[0][0] if hasattr(exc.value, "failures") else exc.value
        assert isinstance(cause, integrity.ChecksumMismatchError) and "chunk(s) [5]" in str(cause), mode
        if mode == "before":  # nothing was written before the mismatch was found
            assert all(not bool(v.any()) for v in target.values() if isinstance(v, torch.Tensor))


def test_two_saves_prepared_before_either_is_written_keep_their_own_checksums(shm_dir):
    """A kept plan holds the checksums of its last launch only.  When the next save is prepared (and the plan launched
    again, over changed tensors) before the previous one has been written, the previous one's values must have left
    the plan: each object's sidecar describes that object's bytes."""
    import ctypes
    import os

    from torch.distributed.checkpoint.planner_helpers import _create_write_items

    from ml_flashpoint.checkpoint_object_manager.buffer_metadata import METADATA_SIZE
    from ml_flashpoint.checkpoint_object_manager.checkpoint_object_manager import CheckpointObjectManager
    from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId
    from ml_flashpoint.core.checkpoint_saver import DefaultMLFlashpointCheckpointSaver
    from ml_flashpoint.hip import integrity
    from ml_flashpoint.hip import plan as P

    class Resolver:
        def __init__(self, data):
            self.data = data

        def resolve_data(self, item):
            return self.data[item.index.fqn]

    g = torch.Generator().manual_seed(3)
    data = {f"w{i}": torch.randn(300_000, generator=g).to(DEV) for i in range(4)}  # 4.8 MB: whole 64 KiB pieces
    items = [wi for k, v in data.items() for wi in _create_write_items(k, v)]
    CheckpointObjectManager._worker_pool = None
    saver = DefaultMLFlashpointCheckpointSaver(lambda: 0, lambda: 0, lambda: None, CheckpointObjectManager(), None,
                                               initial_buffer_size_bytes=1 << 20, crc_chunk_bytes=1 << 16, crc_mode="fused")
    cids = [CheckpointContainerId(os.path.join(shm_dir, f"step-{n}_ckpt")) for n in (1, 2)]
    first = saver.prepare_write_data(cids[0], items, Resolver(data), "data", 1)
    for v in data.values():
        v.mul_(-3.0)  # the next step's values
    second = saver.prepare_write_data(cids[1], items, Resolver(data), "data", 1)
    assert saver.last_save_stats.get("plans_reused") == 1
    saver.write_data(cids[0], first, replicate_after_write=False, thread_count=1)
    saver.write_data(cids[1], second, replicate_after_write=False, thread_count=1)
    raws = []
    for cid in cids:
        path = os.path.join(cid.data, "data_0_src0.distcp")
        raw = open(path, "rb").read()
        raws.append(raw)
        chunk, nbytes, crcs = integrity.read_sidecar(path)
        assert nbytes == len(raw) - METADATA_SIZE
        for k, c in enumerate(crcs):
            piece = raw[METADATA_SIZE + k * chunk : METADATA_SIZE + (k + 1) * chunk]
            buf = ctypes.create_string_buffer(piece, len(piece))
            assert P.crc32c_host(ctypes.addressof(buf), len(piece)) == int(c), (cid.data, k)
    assert raws[0] != raws[1]


@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_checksums_of_a_piece_cut_on_the_sections_chunk_grid(seed, oracle_c):
    """``crc32c_device_cut``: a piece of a data section lies somewhere in a device buffer (same position modulo 16 as in
    the section) and, already, in host memory; its checksums come back cut where the section's chunks end - the
    first part may start off the 16-byte grid the kernels read on, its leading bytes are then taken on the host."""
    import ctypes

    from ml_flashpoint.hip import integrity
    from ml_flashpoint.hip import plan as P

    rng = np.random.default_rng(seed)
    chunk = 65536
    for _ in range(6):
        data_off = int(rng.integers(0, 5 * chunk))
        nbytes = int(rng.integers(1, 4 * chunk))
        if seed == 3:
            nbytes = int(rng.integers(1, 40))  # pieces shorter than a vector
        buf_off = data_off % 16 + 16 * int(rng.integers(0, 300))
        host = rng.integers(0, 256, nbytes, dtype=np.uint8)
        buf = torch.zeros(buf_off + nbytes + 64, dtype=torch.uint8, device=DEV)
        buf[buf_off : buf_off + nbytes] = torch.from_numpy(host).to(DEV)
        got = P.crc32c_device_cut(buf, buf_off, data_off, nbytes, chunk, host.ctypes.data)
        parts = integrity.ChunkChecksums.cuts(data_off, nbytes, chunk)
        want = [oracle_c.oracle_crc32c(host[first - data_off : first - data_off + n].tobytes(), n) for first, n in parts]
        assert got == want, (data_off, nbytes, buf_off)
    with pytest.raises(ValueError, match="modulo 16"):
        P.crc32c_device_cut(torch.zeros(256, dtype=torch.uint8, device=DEV), 1, 0, 100, chunk, 0)
