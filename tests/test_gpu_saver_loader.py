"""GPU parity of the saver/loader plug-ins behind the DCP adapters: file bytes and restored tensors are compared
with the CPU oracle on the same seeded state dicts (bit-exact)."""

import concurrent.futures
import ctypes
import io
import os
import pickle
import threading

import pytest
import torch
import torch.distributed.checkpoint as dcp
import torch.multiprocessing as torch_mp
from torch.distributed.checkpoint.filesystem import _StorageInfo
from torch.distributed.checkpoint.metadata import MetadataIndex
from torch.distributed.checkpoint.planner import LoadItemType, ReadItem, WriteItemType

import workloads
from ml_flashpoint.adapter.pytorch.memory_storage_reader import MemoryStorageReader
from ml_flashpoint.adapter.pytorch.memory_storage_writer import MemoryStorageWriter
from ml_flashpoint.checkpoint_object_manager.buffer_metadata import METADATA_SIZE
from ml_flashpoint.checkpoint_object_manager.checkpoint_object_manager import CheckpointObjectManager
from ml_flashpoint.core.buffer_pool import BufferPoolConfig
from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId, CheckpointObjectId
from oracle import mlf_format as fmt
from oracle.cpu_path import OracleCheckpointLoader, OracleCheckpointSaver

pytestmark = [pytest.mark.gpu, pytest.mark.filterwarnings("ignore:torch.distributed is disabled")]
DEV = "cuda:0"


@pytest.fixture(scope="module")
def manager_future():
    mgr = torch_mp.get_context("spawn").Manager()
    fut = concurrent.futures.Future()
    fut.set_result(mgr)
    yield fut
    mgr.shutdown()


@pytest.fixture(autouse=True)
def _fresh_pool():
    CheckpointObjectManager._worker_pool = None
    yield
    CheckpointObjectManager().teardown_pool()


def _saver(manager=None, **kw):
    from ml_flashpoint.core.checkpoint_saver import DefaultMLFlashpointCheckpointSaver

    return DefaultMLFlashpointCheckpointSaver(
        global_rank_getter=lambda: 0,
        local_rank_getter=lambda: 0,
        global_barrier_func=lambda: None,
        ckpt_obj_manager=manager or CheckpointObjectManager(),
        replication_manager=None,
        initial_buffer_size_bytes=kw.pop("initial_buffer_size_bytes", 1 << 20),
        **kw,
    )


def _loader(**kw):
    from ml_flashpoint.core.checkpoint_loader import DefaultMLFlashpointCheckpointLoader

    return DefaultMLFlashpointCheckpointLoader(CheckpointObjectManager(), None, **kw)


def _bits(t):
    return t.detach().cpu().contiguous().reshape(-1).view(torch.uint8)


def _expected_file(sd_cpu, metadata, raw):
    """Oracle image for the item order the plan chose; byte blobs (pickled non-tensors) are taken as written."""
    by_offset = sorted(metadata.storage_data.items(), key=lambda kv: kv[1].offset)
    tensors = [sd_cpu[i.fqn] for i, _ in by_offset if isinstance(sd_cpu[i.fqn], torch.Tensor)]
    blobs = [raw[METADATA_SIZE + s.offset : METADATA_SIZE + s.offset + s.length] for i, s in by_offset
             if not isinstance(sd_cpu[i.fqn], torch.Tensor)]
    image, spans = fmt.file_image(tensors, blobs)
    return image, spans, [(s.offset, s.length) for _, s in by_offset]


def _mixed_state_dict():
    g = torch.Generator().manual_seed(99)
    rb = lambda n: torch.randint(0, 256, (n,), dtype=torch.uint8, generator=g)  # noqa: E731
    base = rb(64 * 96 * 2).view(torch.bfloat16).reshape(64, 96)
    sd = {
        "w.fp32": torch.randn(257, 33, generator=g) * 0.02,
        "w.bf16": rb(1000 * 2).view(torch.bfloat16).reshape(10, 100),
        "w.fp8": rb(4096).view(torch.float8_e4m3fn).reshape(64, 64),
        "w.i64": torch.randint(-(2**62), 2**62, (513,), generator=g),
        "w.scalar": torch.tensor(3.25),
        "w.empty": torch.empty(0, 7),
        "w.bool": torch.rand(40, generator=g) > 0.5,
        "v.transposed": base.t(),
        "v.cols": base[:, ::2],
        "v.rows": base[16:48],
        "obj.step": 123,
        "obj.cfg": "lr=1e-3;name=x",
    }
    return sd


def _to_dev(sd, keep_on_host=()):
    out = {}
    for k, v in sd.items():
        if isinstance(v, torch.Tensor) and k not in keep_on_host:
            if v.is_contiguous():
                out[k] = v.to(DEV)
            else:  # rebuild the same view over a device copy of the base
                base = torch.empty(v.untyped_storage().size(), dtype=torch.uint8)
                base.untyped_storage().copy_(v.untyped_storage())
                dev_base = base.to(DEV)
                out[k] = torch.as_strided(dev_base.view(v.dtype), v.shape, v.stride(), v.storage_offset())
        else:
            out[k] = v
    return out


def test_dcp_save_bytes_equal_oracle_and_load_is_bit_exact(shm_dir, manager_future):
    sd_cpu = _mixed_state_dict()
    sd_dev = _to_dev(sd_cpu, keep_on_host=("w.i64",))  # one host-resident tensor among device tensors
    ckpt = os.path.join(shm_dir, "step-5_ckpt")
    saver = _saver()
    dcp.save(sd_dev, checkpoint_id=ckpt, storage_writer=MemoryStorageWriter(saver, manager_future), no_dist=True)
    assert sorted(os.listdir(ckpt)) == [".metadata", "__0__0_src0.distcp"]
    raw = open(os.path.join(ckpt, "__0__0_src0.distcp"), "rb").read()
    metadata = pickle.load(open(os.path.join(ckpt, ".metadata"), "rb"))
    image, spans, got_spans = _expected_file(sd_cpu, metadata, raw)
    assert raw == image and got_spans == spans
    assert saver.last_save_stats["d2h_bytes"] == len(raw) - METADATA_SIZE

    # the oracle's CPU saver writes the very same file for the host copy of the state dict
    ckpt2 = os.path.join(shm_dir, "oracle", "step-5_ckpt")
    dcp.save(sd_cpu, checkpoint_id=ckpt2, storage_writer=MemoryStorageWriter(OracleCheckpointSaver(), manager_future), no_dist=True)
    assert open(os.path.join(ckpt2, "__0__0_src0.distcp"), "rb").read() == raw

    for src_ckpt in (ckpt, ckpt2):  # restore from our file and from the oracle's file
        target = {}
        for k, v in sd_dev.items():
            if isinstance(v, torch.Tensor):
                # (zeroed as bytes: torch has no fill kernel for the fp8 and packed fp4 dtypes)
                target[k] = torch.zeros(v.numel() * v.element_size(), dtype=torch.uint8, device=v.device).view(v.dtype).reshape(v.shape)
            else:
                target[k] = None
        loader = _loader()
        dcp.load(target, checkpoint_id=src_ckpt, storage_reader=MemoryStorageReader(src_ckpt, loader), no_dist=True)
        assert target["obj.step"] == 123 and target["obj.cfg"] == "lr=1e-3;name=x"
        for k, v in sd_cpu.items():
            if isinstance(v, torch.Tensor):
                assert torch.equal(_bits(target[k]), _bits(v)), k
        assert loader.last_load_stats["device_items"] >= 8 and loader.last_load_stats["host_items"] == 1
        # (an object with a host-resident target among the device targets is not uploaded ahead of the parse: what
        # the device needs of it is known only once the targets are)
        assert "upload_began_before_parse" not in loader.last_load_stats

    # and the oracle's CPU loader restores our file
    target = {k: (torch.zeros_like(v) if isinstance(v, torch.Tensor) else None) for k, v in sd_cpu.items()}
    dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, OracleCheckpointLoader()), no_dist=True)
    for k, v in sd_cpu.items():
        if isinstance(v, torch.Tensor):
            assert torch.equal(_bits(target[k]), _bits(v)), k


def test_gpt2_small_config_on_device(shm_dir, manager_future):
    """The GPT-2-small-shaped fp32 state dict (the benchmark's CPU-runnable configuration), resident on the GPU, saved by the gfx950 saver: same bytes as the oracle."""
    sd_dev = workloads.gpt2_small(device=DEV, layers=3, d=256, vocab=5003, ctx=128)
    sd_cpu = {k: v.cpu() for k, v in sd_dev.items()}
    ckpt = os.path.join(shm_dir, "step-1_ckpt")
    dcp.save(sd_dev, checkpoint_id=ckpt, storage_writer=MemoryStorageWriter(_saver(), manager_future), no_dist=True)
    raw = open(os.path.join(ckpt, "__0__0_src0.distcp"), "rb").read()
    metadata = pickle.load(open(os.path.join(ckpt, ".metadata"), "rb"))
    image, spans, got_spans = _expected_file(sd_cpu, metadata, raw)
    assert raw == image and got_spans == spans
    target = {k: torch.zeros_like(v) for k, v in sd_dev.items()}
    dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, _loader()), no_dist=True)
    assert all(torch.equal(target[k].view(torch.int32), sd_dev[k].view(torch.int32)) for k in sd_dev)


def test_megatron_style_sequence_with_pool_and_finalize(shm_dir, manager_future):
    """initialize -> prepare buckets (pack) -> generic stage step -> write -> finish -> finalize, into pooled buffers,
    twice (the second save reuses a pool buffer and removes the first step)."""
    from torch.distributed.checkpoint import DefaultSavePlanner

    pool_cfg = BufferPoolConfig(os.path.join(shm_dir, "pool"), 0, 2, METADATA_SIZE + 4096)
    manager = CheckpointObjectManager(pool_cfg)
    saver = _saver(manager)
    sd_cpu = {k: v for k, v in _mixed_state_dict().items() if isinstance(v, torch.Tensor)}
    sd_dev = _to_dev(sd_cpu)
    for step in (10, 20):
        cid = CheckpointContainerId(os.path.join(shm_dir, "run", f"step-{step}_ckpt"))
        saver.initialize_checkpoint(cid)
        marker = f"{cid}__0__unfinished"
        assert os.path.exists(marker)
        writer = MemoryStorageWriter(saver, manager_future)
        writer.reset(cid.data)
        planner = DefaultSavePlanner()
        planner.set_up_planner(sd_dev, is_coordinator=True)
        local = writer.prepare_local_plan(planner.create_local_plan())
        plans, metadata = planner.create_global_plan([local])
        plan = planner.finish_plan(writer.prepare_global_plan(plans)[0])
        buckets = writer.prepare_write_data_buckets(cid, plan, planner)
        staged = MemoryStorageWriter.stage_write_data_buckets(cid, buckets, non_blocking=True)
        assert all(a is b for (_, a), (_, b) in zip(buckets[0].tensor_data, staged[0].tensor_data))
        for t in sd_dev.values():  # training may overwrite the live tensors as soon as staging returned
            if t.numel() and t.is_contiguous() and t.dtype not in (torch.bool, torch.float8_e4m3fn):
                t.add_(1)
        results = writer.write_staged_data_buckets(cid, staged, replicate_after_write=False).wait()
        assert writer.get_write_results(cid) is not None
        writer.finish_checkpoint(cid, metadata, [results])
        open(os.path.join(cid.data, "common.pt"), "wb").write(b"common state, written by the strategy")
        proc = saver.finalize_checkpoint(cid)
        assert not os.path.exists(marker)
        if proc is not None:
            proc.wait()
        obj = os.path.join(cid.data, "__0__0_src0.distcp")
        assert os.path.islink(obj)
        raw = open(obj, "rb").read()
        md = pickle.load(open(os.path.join(cid.data, ".metadata"), "rb"))
        image, spans, got_spans = _expected_file(sd_cpu, md, raw)
        assert raw == image and got_spans == spans  # the bytes are those of the moment prepare returned
        sd_cpu = {k: v.cpu() for k, v in sd_dev.items()}  # what the next save must capture
    assert not os.path.exists(os.path.join(shm_dir, "run", "step-10_ckpt"))
    assert _loader().get_latest_complete_checkpoint(CheckpointContainerId(os.path.join(shm_dir, "run"))).data.endswith("step-20_ckpt")


def test_metadata_object_is_pickled_while_the_data_is_written(shm_dir, manager_future, monkeypatch):
    """A save that one process plans, writes and finishes: the metadata object is pickled on a thread while the image
    crosses the link, and ``finish_write`` only writes those bytes - the same file as the ordinary way produces.  If
    what the write reported differs from what was predicted, or another metadata object arrives, the ordinary way
    is taken."""
    from torch.distributed.checkpoint import DefaultSavePlanner
    from torch.distributed.checkpoint.utils import _DistWrapper

    from ml_flashpoint.adapter.pytorch import custom_state_dict_saver as three_calls

    sd_dev = {k: v for k, v in _to_dev(_mixed_state_dict()).items()}
    saver = _saver()
    dist = _DistWrapper(None, False, 0)
    calls = []
    real_bytes, real_object = saver.write_metadata_bytes, saver.write_metadata
    monkeypatch.setattr(saver, "write_metadata_bytes", lambda *a, **k: (calls.append("bytes"), real_bytes(*a, **k))[1])
    monkeypatch.setattr(saver, "write_metadata", lambda *a, **k: (calls.append("object"), real_object(*a, **k))[1])

    def save(step, tamper=None):
        cid = CheckpointContainerId(os.path.join(shm_dir, f"step-{step}_ckpt"))
        writer = MemoryStorageWriter(saver, manager_future)
        writer.reset(cid.data)
        buckets, metadata, *_ = three_calls.generate_plan(cid, sd_dev, writer, DefaultSavePlanner(), dist)
        staged = MemoryStorageWriter.stage_write_data_buckets(cid, buckets)
        three_calls.write_data(cid, writer, staged, replicate_after_write=False)
        if tamper == "other-object":
            metadata = pickle.loads(pickle.dumps(metadata))
        three_calls.finish_write(cid, writer, metadata, dist)
        return cid, writer

    cid, writer = save(1)
    assert calls == ["bytes"]
    early = pickle.load(open(os.path.join(cid.data, ".metadata"), "rb"))
    assert early.storage_meta.checkpoint_id == cid.data and early.storage_meta.save_id == writer._current_save_id
    cid2, _ = save(2, tamper="other-object")
    assert calls == ["bytes", "object"]
    late = pickle.load(open(os.path.join(cid2.data, ".metadata"), "rb"))
    assert early.state_dict_metadata == late.state_dict_metadata and early.storage_data == late.storage_data
    assert early.planner_data == late.planner_data
    # the object the early bytes describe is the one that was written: it loads
    target = {k: (torch.zeros_like(v) if isinstance(v, torch.Tensor) and v.dtype != torch.float8_e4m3fn else
                  (torch.zeros(v.shape, dtype=torch.uint8, device=v.device).view(v.dtype) if isinstance(v, torch.Tensor) else None))
              for k, v in sd_dev.items()}
    dcp.load(target, checkpoint_id=cid.data, storage_reader=MemoryStorageReader(cid.data, _loader()), no_dist=True)
    assert all(torch.equal(_bits(target[k]), _bits(v)) for k, v in sd_dev.items() if isinstance(v, torch.Tensor))
    assert target["obj.step"] == 123


@pytest.mark.parametrize("crc_mode", ["beside", "fused", "host"])
def test_crc_sidecar_written_and_corruption_detected(shm_dir, manager_future, crc_mode):
    """Whoever takes the checksums of a save - a pass of kernels beside the transfer, the pack kernel itself, or the
    host threads that move the image into the buffer - the sidecar holds the CRC-32C of the bytes in the file."""
    from ml_flashpoint.hip import integrity

    sd = {"a": torch.randn(300_000, device=DEV), "b": torch.randn(7, 9, device=DEV).to(torch.bfloat16)}
    ckpt = os.path.join(shm_dir, "step-2_ckpt")
    dcp.save(sd, checkpoint_id=ckpt, storage_writer=MemoryStorageWriter(
        _saver(crc_chunk_bytes=1 << 18, crc_mode=crc_mode), manager_future), no_dist=True)
    obj = os.path.join(ckpt, "__0__0_src0.distcp")
    chunk, nbytes, crcs = integrity.read_sidecar(obj)
    raw = open(obj, "rb").read()
    assert chunk == 1 << 18 and nbytes == len(raw) - METADATA_SIZE and len(crcs) == -(-nbytes // chunk)
    import ctypes

    from ml_flashpoint.hip import plan as P

    for k, c in enumerate(crcs):  # the GPU's values are the CRCs of the bytes that landed in the file
        piece = raw[METADATA_SIZE + k * chunk : METADATA_SIZE + (k + 1) * chunk]
        buf = ctypes.create_string_buffer(piece, len(piece))
        assert P.crc32c_host(ctypes.addressof(buf), len(piece)) == int(c)
    target = {k: torch.zeros_like(v) for k, v in sd.items()}
    dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, _loader()), no_dist=True)
    assert all(torch.equal(target[k], sd[k]) for k in sd)
    with open(obj, "r+b") as f:  # flip one payload bit in the third chunk
        f.seek(METADATA_SIZE + 2 * chunk + 1000)
        byte = f.read(1)
        f.seek(-1, os.SEEK_CUR)
        f.write(bytes([byte[0] ^ 0x10]))
    with pytest.raises(BaseException) as exc:
        dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, _loader()), no_dist=True)
    cause = exc.value.failures[0][0] if hasattr(exc.value, "failures") else exc.value
    assert isinstance(cause, integrity.ChecksumMismatchError) and "chunk(s) [2]" in str(cause)
    dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, _loader(verify_crc=False)), no_dist=True)
    # the same object written again without checksums: the old sidecar must not outlive the bytes it described
    dcp.save(sd, checkpoint_id=ckpt, storage_writer=MemoryStorageWriter(_saver(), manager_future), no_dist=True)
    assert integrity.read_sidecar(obj) is None and not os.path.exists(integrity.sidecar_path(obj))
    dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, _loader()), no_dist=True)
    assert all(torch.equal(target[k], sd[k]) for k in sd)


@pytest.mark.parametrize("save_file_io,load_file_io", [(False, False), (False, True), (True, False), (True, True)])
def test_mapping_and_file_descriptor_io_write_and_read_the_same_object(shm_dir, manager_future, save_file_io, load_file_io):
    """The host end of a transfer is either the MAP_SHARED mapping (memcpy) or the file descriptor (pwrite / pread);
    every combination produces the oracle's bytes, a valid checksum sidecar, and a bit-exact restore."""
    from ml_flashpoint.hip import integrity

    sd_cpu = _mixed_state_dict()
    sd_cpu["w.big"] = torch.randn(3_000_001, generator=torch.Generator().manual_seed(3))
    sd_dev = _to_dev(sd_cpu)
    ckpt = os.path.join(shm_dir, "step-3_ckpt")
    saver = _saver(use_file_io=save_file_io, crc_chunk_bytes=1 << 20)
    dcp.save(sd_dev, checkpoint_id=ckpt, storage_writer=MemoryStorageWriter(saver, manager_future), no_dist=True)
    obj = os.path.join(ckpt, "__0__0_src0.distcp")
    raw = open(obj, "rb").read()
    metadata = pickle.load(open(os.path.join(ckpt, ".metadata"), "rb"))
    image, spans, got_spans = _expected_file(sd_cpu, metadata, raw)
    assert raw == image and got_spans == spans
    chunk, nbytes, crcs = integrity.read_sidecar(obj)
    assert nbytes == len(raw) - METADATA_SIZE and len(crcs) == -(-nbytes // chunk)
    target = {k: (torch.zeros_like(v) if isinstance(v, torch.Tensor) else None) for k, v in sd_dev.items()}
    loader = _loader(use_file_io=load_file_io)
    dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, loader), no_dist=True)
    for k, v in sd_cpu.items():
        if isinstance(v, torch.Tensor):
            assert torch.equal(_bits(target[k]), _bits(v)), k


def test_stage_data_returns_host_copies(shm_dir):
    sd_cpu = _mixed_state_dict()
    sd_dev = _to_dev(sd_cpu, keep_on_host=("w.i64",))
    staged = _saver().stage_data(CheckpointContainerId(os.path.join(shm_dir, "step-1_ckpt")), sd_dev)
    assert list(staged) == list(sd_dev)
    for k, v in sd_cpu.items():
        if isinstance(v, torch.Tensor):
            assert staged[k].device.type == "cpu" and staged[k].shape == v.shape and staged[k].dtype == v.dtype
            assert torch.equal(_bits(staged[k]), _bits(v)), k
        else:
            assert staged[k] == v
    assert staged["w.i64"] is sd_dev["w.i64"]


class _Resolver:
    def __init__(self, data):
        self.data = data

    def resolve_data(self, item):
        return self.data[item.index.fqn]


class _Planner:
    """Minimal LoadPlanner stand-in: hands out targets by fqn and records commits / loaded bytes."""

    def __init__(self, targets):
        self.targets, self.committed, self.loaded = targets, [], {}

    def resolve_tensor(self, req):
        return self.targets[req.dest_index.fqn]

    def commit_tensor(self, req, tensor):
        self.committed.append(req.dest_index.fqn)

    def load_bytes(self, req, value):
        self.loaded[req.dest_index.fqn] = value.read()


def _write_direct(shm_dir, data, bucket_count=1):
    saver = _saver()
    cid = CheckpointContainerId(os.path.join(shm_dir, "step-7_ckpt"))
    from torch.distributed.checkpoint.planner_helpers import _create_write_items

    items = [wi for k, v in data.items() for wi in _create_write_items(k, v)]
    assert all((wi.type == WriteItemType.BYTE_IO) == isinstance(data[wi.index.fqn], io.BytesIO) for wi in items)
    buckets = saver.prepare_write_data(cid, items, _Resolver(data), "data", bucket_count)
    results = saver.write_data(cid, buckets, replicate_after_write=False, thread_count=bucket_count)
    return cid, buckets, {r.index.fqn: r.storage_data for r in results}


def test_direct_saver_calls_offsets_names_and_sub_box_reads(shm_dir):
    g = torch.Generator().manual_seed(5)
    stored = torch.randn(12, 20, 10, generator=g)
    data = {"t3": stored.to(DEV), "blob": io.BytesIO(b"some-bytes"), "t1": torch.arange(20, dtype=torch.float32, device=DEV)}
    cid, buckets, info = _write_direct(shm_dir, data)
    assert [b.object_name for b in buckets] == ["data_0_src0.distcp"]
    hdr3 = len(fmt.header_bytes("float32", (12, 20, 10)))
    hdr1 = len(fmt.header_bytes("float32", (20,)))
    assert (info["t3"].offset, info["t3"].length) == (0, hdr3 + stored.numel() * 4)  # tensors first ...
    assert (info["t1"].offset, info["t1"].length) == (info["t3"].length, hdr1 + 80)
    assert (info["blob"].offset, info["blob"].length) == (info["t3"].length + info["t1"].length, 10)  # ... then blobs
    oid = CheckpointObjectId.from_container(cid, "data_0_src0.distcp")
    assert os.path.getsize(oid.data) == METADATA_SIZE + info["blob"].offset + 10

    storage = {0: info["t3"], 1: info["t1"], 2: info["blob"]}
    parent = torch.zeros(2, 4, 5, device=DEV)
    targets = {"box": parent[:, ::2, 3:], "slice": torch.zeros(10, device=DEV), "host": torch.zeros(8, 15, 10), "blob": None}
    reqs = [
        ReadItem(type=LoadItemType.TENSOR, dest_index=MetadataIndex("box"), dest_offsets=torch.Size([0, 0, 0]), storage_index=0,
                 storage_offsets=torch.Size([1, 0, 3]), lengths=torch.Size([2, 2, 2])),
        ReadItem(type=LoadItemType.TENSOR, dest_index=MetadataIndex("slice"), dest_offsets=torch.Size([0]), storage_index=1,
                 storage_offsets=torch.Size([5]), lengths=torch.Size([10])),
        ReadItem(type=LoadItemType.TENSOR, dest_index=MetadataIndex("host"), dest_offsets=torch.Size([0, 0, 0]), storage_index=0,
                 storage_offsets=torch.Size([4, 5, 0]), lengths=torch.Size([8, 15, 10])),
        ReadItem(type=LoadItemType.BYTE_IO, dest_index=MetadataIndex("blob"), dest_offsets=torch.Size([0]), storage_index=2,
                 storage_offsets=torch.Size([0]), lengths=torch.Size([0])),
    ]
    planner = _Planner(targets)
    _loader().read_data(oid, reqs, planner, storage)
    assert torch.equal(targets["box"].cpu(), stored[1:3, 0:2, 3:5])
    assert torch.equal(targets["slice"].cpu(), torch.arange(5, 15, dtype=torch.float32))  # the reference's known answer
    assert torch.equal(targets["host"], stored[4:12, 5:20, :])
    assert planner.loaded == {"blob": b"some-bytes"} and sorted(planner.committed) == ["box", "host", "slice"]
    assert float(parent[:, 1::2].abs().sum()) == 0 and float(parent[:, :, :3].abs().sum()) == 0

    with pytest.raises(AssertionError, match="mismatch sizes"):
        _loader().read_data(oid, [reqs[1]], _Planner({"slice": torch.zeros(11, device=DEV)}), storage)
    with pytest.raises(FileNotFoundError, match="does not exist on any node in the cluster"):
        _loader().read_data(CheckpointObjectId(oid.data + ".gone"), reqs, planner, storage)


def test_targets_of_another_dtype_are_converted_as_copy_does(shm_dir):
    """The reference ends a read with ``target.copy_(stored)`` (checkpoint_loader.py:335), which converts between
    dtypes; a device target of another dtype gets the same values here, converted on the device."""
    g = torch.Generator().manual_seed(9)
    w = torch.randn(40, 30, generator=g)
    steps = torch.arange(-50, 50, dtype=torch.int64)
    data = {"w": w.to(DEV), "steps": steps.to(DEV), "same": w[:5].clone().to(DEV)}
    cid, _, info = _write_direct(shm_dir, data)
    oid = CheckpointObjectId.from_container(cid, "data_0_src0.distcp")
    storage = {0: info["w"], 1: info["steps"], 2: info["same"]}
    parent = torch.zeros(30, 40, dtype=torch.float64, device=DEV)
    targets = {
        "w_bf16": torch.zeros(40, 30, dtype=torch.bfloat16, device=DEV),
        "w_f64_view": parent.t(),                                          # non-contiguous target of another dtype
        "box_f16": torch.zeros(10, 7, dtype=torch.float16, device=DEV),    # sub-box of the stored tensor
        "steps_f32": torch.zeros(100, dtype=torch.float32, device=DEV),
        "same": torch.zeros(5, 30, device=DEV),
    }
    whole = lambda name, idx, shape: ReadItem(  # noqa: E731
        type=LoadItemType.TENSOR, dest_index=MetadataIndex(name), dest_offsets=torch.Size([0] * len(shape)),
        storage_index=idx, storage_offsets=torch.Size([0] * len(shape)), lengths=torch.Size(shape))
    reqs = [
        whole("w_bf16", 0, (40, 30)),
        whole("w_f64_view", 0, (40, 30)),
        ReadItem(type=LoadItemType.TENSOR, dest_index=MetadataIndex("box_f16"), dest_offsets=torch.Size([0, 0]),
                 storage_index=0, storage_offsets=torch.Size([20, 3]), lengths=torch.Size([10, 7])),
        whole("steps_f32", 1, (100,)),
        whole("same", 2, (5, 30)),
    ]
    planner = _Planner(targets)
    _loader().read_data(oid, reqs, planner, storage)
    assert torch.equal(targets["w_bf16"].cpu(), w.to(torch.bfloat16))
    assert torch.equal(parent.cpu(), w.to(torch.float64).t())
    assert torch.equal(targets["box_f16"].cpu(), w[20:30, 3:10].to(torch.float16))
    assert torch.equal(targets["steps_f32"].cpu(), steps.to(torch.float32))
    assert torch.equal(targets["same"].cpu(), w[:5])
    assert sorted(planner.committed) == sorted(targets)


def test_multiple_buckets_and_overwrite_of_existing_object(shm_dir):
    data = {f"t{i}": torch.full((1000 + i,), float(i), device=DEV) for i in range(5)}
    data["b0"], data["b1"] = io.BytesIO(b"zero"), io.BytesIO(b"one")
    cid, buckets, info = _write_direct(shm_dir, data, bucket_count=3)
    names = sorted(b.object_name for b in buckets)
    assert names == ["data_0_src0.distcp", "data_1_src0.distcp", "data_2_src0.distcp"]
    assert sum(len(b.tensor_data) + len(b.bytesio_data) for b in buckets) == 7
    for b in buckets:  # every object parses as a sequence of records + blobs the oracle agrees with
        raw = open(b.object_id.data, "rb").read()
        tensors = [data[i.index.fqn].cpu() for i, _ in b.tensor_data]
        blobs = [d.getvalue() for _, d in b.bytesio_data]
        assert raw == fmt.file_image(tensors, blobs)[0]
    _write_direct(shm_dir, {"t0": torch.ones(3, device=DEV)})  # same object id again: overwritten, not an error
    raw = open(os.path.join(cid.data, "data_0_src0.distcp"), "rb").read()
    assert raw == fmt.file_image([torch.ones(3)])[0]


@pytest.mark.parametrize("crc_mode", ["host", "beside"])
def test_object_larger_than_the_hbm_limit_is_saved_window_by_window(shm_dir, manager_future, crc_mode):
    """With ``max_image_bytes`` far below the object size the saver packs and sends windows of records through
    one small device buffer; the file is the same."""
    sd_cpu = {k: v for k, v in _mixed_state_dict().items()}
    sd_cpu["big"] = torch.arange(200_000, dtype=torch.float32)  # one record larger than the limit
    sd_dev = _to_dev(sd_cpu, keep_on_host=("w.i64",))
    ckpt = os.path.join(shm_dir, "step-8_ckpt")
    saver = _saver(max_image_bytes=64 << 10, crc_chunk_bytes=1 << 16, crc_mode=crc_mode)
    dcp.save(sd_dev, checkpoint_id=ckpt, storage_writer=MemoryStorageWriter(saver, manager_future), no_dist=True)
    assert saver.last_save_stats["windows"] >= 4
    raw = open(os.path.join(ckpt, "__0__0_src0.distcp"), "rb").read()
    metadata = pickle.load(open(os.path.join(ckpt, ".metadata"), "rb"))
    image, spans, got_spans = _expected_file(sd_cpu, metadata, raw)
    assert raw == image and got_spans == spans
    # windows end where records end, not where checksum chunks end: the sidecar is joined from the checksums of the
    # parts of each window - taken by the host threads as they copy the window, or by kernels; every value is the
    # host's for that chunk of the file, and the GPU check of an ordinary restore accepts it
    from ml_flashpoint.hip import integrity
    from ml_flashpoint.hip import plan as P

    chunk, nbytes, crcs = integrity.read_sidecar(os.path.join(ckpt, "__0__0_src0.distcp"))
    assert chunk == 1 << 16 and nbytes == len(raw) - METADATA_SIZE and len(crcs) == -(-nbytes // chunk)
    for k, c in enumerate(crcs):
        piece = raw[METADATA_SIZE + k * chunk : METADATA_SIZE + (k + 1) * chunk]
        buf = ctypes.create_string_buffer(piece, len(piece))
        assert P.crc32c_host(ctypes.addressof(buf), len(piece)) == int(c), k
    target = {k: (torch.zeros_like(v) if isinstance(v, torch.Tensor) and v.dtype != torch.float8_e4m3fn else
                  (torch.zeros(v.shape, dtype=torch.uint8, device=v.device).view(v.dtype) if isinstance(v, torch.Tensor) else None))
              for k, v in sd_dev.items()}
    loader = _loader()
    dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, loader), no_dist=True)
    assert "windows" not in loader.last_load_stats
    for k, v in sd_cpu.items():
        if isinstance(v, torch.Tensor):
            assert torch.equal(_bits(target[k]), _bits(v)), k


def test_windowed_save_keeps_the_end_of_the_object_resident_and_sends_it_behind_the_blocking_part(shm_dir):
    """With room for part of the image only, the records at the end of the object stay in HBM as a snapshot and are
    sent by a thread after ``prepare_write_data`` has returned; the records before them go window by window inside
    it.  Overwriting every live tensor right after that call must not change what lands in the file."""
    from torch.distributed.checkpoint.planner_helpers import _create_write_items

    from ml_flashpoint.hip import integrity
    from ml_flashpoint.hip import plan as P

    g = torch.Generator().manual_seed(31)
    data_cpu = {f"t{i:02d}": torch.randn(40_000 + 1_000 * i, generator=g) for i in range(14)}  # 2.6 MB
    data_cpu["blob"] = io.BytesIO(b"x" * 1000)
    data = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in data_cpu.items()}
    saver = _saver(max_image_bytes=2 << 20, crc_chunk_bytes=1 << 16)  # windows of 256 KiB through two buffers
    cid = CheckpointContainerId(os.path.join(shm_dir, "step-12_ckpt"))
    items = [wi for k, v in data.items() for wi in _create_write_items(k, v)]
    buckets = saver.prepare_write_data(cid, items, _Resolver(data), "data", 1)
    stats = saver.last_save_stats
    assert stats["windows"] >= 3 and stats["window_buffers"] == 2 and (1 << 20) < stats["resident_bytes"] < (2 << 20)
    for v in data.values():  # the training step goes on
        if isinstance(v, torch.Tensor):
            v.fill_(-1.0)
    torch.cuda.synchronize()
    results = saver.write_data(cid, buckets, replicate_after_write=False, thread_count=1)
    assert saver.last_save_stats["d2h_bytes"] == sum(r.size_in_bytes for r in results)
    path = os.path.join(cid.data, "data_0_src0.distcp")
    raw = open(path, "rb").read()
    order = sorted(results, key=lambda r: r.storage_data.offset)
    tensors = [data_cpu[r.index.fqn] for r in order if r.index.fqn != "blob"]
    assert raw == fmt.file_image(tensors, [b"x" * 1000])[0]
    chunk, nbytes, crcs = integrity.read_sidecar(path)
    assert nbytes == len(raw) - METADATA_SIZE and len(crcs) == -(-nbytes // chunk)
    for k, c in enumerate(crcs):
        piece = raw[METADATA_SIZE + k * chunk : METADATA_SIZE + (k + 1) * chunk]
        buf = ctypes.create_string_buffer(piece, len(piece))
        assert P.crc32c_host(ctypes.addressof(buf), len(piece)) == int(c), k
    with pytest.raises(ValueError, match="already written"):
        saver.write_data(cid, buckets, replicate_after_write=False, thread_count=1)


def test_windowed_save_reports_a_failure_of_the_part_that_follows(shm_dir, monkeypatch):
    """The resident part is written by a thread; what goes wrong there reaches ``write_data``, and the saver stays
    usable."""
    from torch.distributed.checkpoint.planner_helpers import _create_write_items

    from ml_flashpoint.hip import integrity

    data = {f"t{i}": torch.full((50_000,), float(i), device=DEV) for i in range(10)}
    saver = _saver(max_image_bytes=1 << 20, crc_chunk_bytes=1 << 16)
    items = [wi for k, v in data.items() for wi in _create_write_items(k, v)]

    def refuse(*a, **kw):
        raise OSError("no room for the sidecar")

    monkeypatch.setattr(integrity, "write_sidecar", refuse)
    cid = CheckpointContainerId(os.path.join(shm_dir, "step-13_ckpt"))
    buckets = saver.prepare_write_data(cid, items, _Resolver(data), "data", 1)
    assert saver.last_save_stats["resident_bytes"] > 0
    with pytest.raises(RuntimeError, match="no room for the sidecar"):
        saver.write_data(cid, buckets, replicate_after_write=False, thread_count=1)
    monkeypatch.undo()
    cid = CheckpointContainerId(os.path.join(shm_dir, "step-14_ckpt"))
    buckets = saver.prepare_write_data(cid, items, _Resolver(data), "data", 1)
    results = saver.write_data(cid, buckets, replicate_after_write=False, thread_count=1)
    raw = open(os.path.join(cid.data, "data_0_src0.distcp"), "rb").read()
    order = sorted(results, key=lambda r: r.storage_data.offset)
    assert raw == fmt.file_image([data[r.index.fqn].cpu() for r in order])[0]


@pytest.mark.parametrize("crc_mode", ["host", "beside"])
@pytest.mark.parametrize("background_write", [False, True])
def test_image_is_held_in_pieces_when_no_single_block_is_to_be_had(shm_dir, manager_future, monkeypatch, background_write,
                                                                   crc_mode):
    """Free device memory that is not in one block (the usual state of a long-running job): the image is packed into
    several smaller buffers, all resident, and sent piece by piece - same file, valid sidecar, and still an
    asynchronous save - instead of failing or falling back to the blocking window-by-window mode."""
    from ml_flashpoint.hip import checkpoint_saver as saver_mod
    from ml_flashpoint.hip import integrity
    from ml_flashpoint.hip import plan as P

    sd_cpu = _mixed_state_dict()
    sd_cpu["big"] = torch.arange(100_000, dtype=torch.float32)  # a record larger than a piece: a piece of its own
    for i in range(8):
        sd_cpu[f"mid.{i}"] = torch.full((60_000,), float(i))
    sd_dev = _to_dev(sd_cpu)
    real = P.try_allocate
    refused = []

    def fragmented(nbytes, device):  # no block above 512 KiB
        if nbytes > (1 << 19):
            refused.append(nbytes)
            return None
        return real(nbytes, device)

    monkeypatch.setattr(P, "try_allocate", fragmented)
    monkeypatch.setattr(saver_mod, "_IMAGE_PIECE_BYTES", 1 << 18)
    saver = _saver(crc_chunk_bytes=1 << 16, background_write=background_write, crc_mode=crc_mode)
    ckpt = os.path.join(shm_dir, "step-6_ckpt")
    dcp.save(sd_dev, checkpoint_id=ckpt, storage_writer=MemoryStorageWriter(saver, manager_future), no_dist=True)
    obj = os.path.join(ckpt, "__0__0_src0.distcp")
    raw = open(obj, "rb").read()
    metadata = pickle.load(open(os.path.join(ckpt, ".metadata"), "rb"))
    image, spans, got_spans = _expected_file(sd_cpu, metadata, raw)
    assert raw == image and got_spans == spans
    assert refused == [len(raw) - METADATA_SIZE]  # the one image was asked for, once
    assert saver.last_save_stats["image_pieces"] >= 4 and "windows" not in saver.last_save_stats
    chunk, nbytes, crcs = integrity.read_sidecar(obj)
    assert nbytes == len(raw) - METADATA_SIZE
    for k, c in enumerate(crcs):
        piece = raw[METADATA_SIZE + k * chunk : METADATA_SIZE + (k + 1) * chunk]
        buf = ctypes.create_string_buffer(piece, len(piece))
        assert P.crc32c_host(ctypes.addressof(buf), len(piece)) == int(c)


@pytest.mark.parametrize("load_file_io", [True, False])
def test_restore_larger_than_the_hbm_limit_goes_window_by_window(shm_dir, manager_future, load_file_io):
    """With ``max_image_bytes`` far below the object size the loader uploads and unpacks windows of rows through
    one small device buffer (contiguous rows larger than a window are cut); the restored bits are the same, the
    CRC sidecar is still honoured (windows start on checksum chunks and are checked before they are unpacked), and a
    strided target that spans more than a window is restored through boxes that fit."""
    from ml_flashpoint.hip import integrity

    sd_cpu = dict(_mixed_state_dict())
    sd_cpu["big"] = torch.arange(200_000, dtype=torch.float32)          # 800 kB: several windows of its own
    sd_cpu["wide"] = torch.arange(512 * 300, dtype=torch.int32).reshape(512, 300)
    sd_dev = _to_dev(sd_cpu, keep_on_host=("w.i64",))
    ckpt = os.path.join(shm_dir, "step-9_ckpt")
    dcp.save(sd_dev, checkpoint_id=ckpt, storage_writer=MemoryStorageWriter(_saver(crc_chunk_bytes=1 << 16), manager_future),
             no_dist=True)

    def targets(transposed_wide=False):
        out = {}
        for k, v in sd_dev.items():
            if not isinstance(v, torch.Tensor):
                out[k] = None
            elif v.dtype == torch.float8_e4m3fn:
                out[k] = torch.zeros(v.shape, dtype=torch.uint8, device=v.device).view(torch.float8_e4m3fn)
            else:
                out[k] = torch.zeros(v.shape, dtype=v.dtype, device=v.device)
        if transposed_wide:  # a strided target: its row cannot be cut into windows
            out["wide"] = torch.zeros(300, 512, dtype=torch.int32, device=DEV).t()
        return out

    loader = _loader(max_image_bytes=256 << 10, use_file_io=load_file_io)
    target = targets()
    dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, loader), no_dist=True)
    assert loader.last_load_stats["windows"] >= 5
    assert target["obj.step"] == 123
    for k, v in sd_cpu.items():
        if isinstance(v, torch.Tensor):
            assert torch.equal(_bits(target[k]), _bits(v)), k

    # a strided target small enough for one window is fine ...
    target = targets(transposed_wide=True)
    roomy = _loader(max_image_bytes=700 << 10, use_file_io=load_file_io)
    dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, roomy), no_dist=True)
    assert roomy.last_load_stats["windows"] >= 2 and torch.equal(target["wide"].cpu(), sd_cpu["wide"])
    # ... one that is larger than a window is cut into boxes that fit, as torch's ``copy_`` would take any target
    target = targets(transposed_wide=True)
    dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, loader), no_dist=True)
    assert loader.last_load_stats["windows"] >= 5 and torch.equal(target["wide"].cpu(), sd_cpu["wide"])
    for k, v in sd_cpu.items():
        if isinstance(v, torch.Tensor):
            assert torch.equal(_bits(target[k]), _bits(v)), k

    obj = os.path.join(ckpt, "__0__0_src0.distcp")
    assert loader.last_load_stats.get("crc_s", 0.0) >= 0.0
    with open(obj, "r+b") as f:  # one flipped bit: found by the window that holds its chunk
        f.seek(METADATA_SIZE + 5 * (1 << 16) + 77)
        byte = f.read(1)
        f.seek(-1, os.SEEK_CUR)
        f.write(bytes([byte[0] ^ 0x01]))
    assert _loader()._crc_mode == "before"
    for mode in ("fused", "before"):
        picky = _loader(max_image_bytes=256 << 10, use_file_io=load_file_io, crc_mode=mode)
        victim = targets()
        with pytest.raises(BaseException) as exc:
            dcp.load(victim, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, picky), no_dist=True)
        cause = exc.value.failures[0][0] if hasattr(exc.value, "failures") else exc.value
        assert isinstance(cause, integrity.ChecksumMismatchError) and "chunk(s) [5]" in str(cause), mode
        if mode == "before":
            # every window is checked before it is unpacked: what the earlier windows brought is in place, the window
            # with the flipped bit and everything behind it never reached a target - no byte of any target is
            # anything but its old value (zero) or the checkpoint's
            touched = 0
            for k, v in sd_cpu.items():
                if isinstance(v, torch.Tensor) and v.numel():
                    got, want = _bits(victim[k]), _bits(v)
                    assert bool(((got == 0) | (got == want)).all()), k
                    touched += int(bool(got.any()))
            assert 0 < touched < sum(1 for v in sd_cpu.values() if isinstance(v, torch.Tensor) and v.numel())
            metadata = pickle.load(open(os.path.join(ckpt, ".metadata"), "rb"))
            at = 5 * (1 << 16) + 77  # the flipped byte: its tensor's byte there is still the old one
            hit = [(i.fqn, at - (st.offset + st.length - _bits(sd_cpu[i.fqn]).numel()))
                   for i, st in metadata.storage_data.items()
                   if isinstance(sd_cpu[i.fqn], torch.Tensor) and st.offset <= at < st.offset + st.length]
            for fqn, pos in hit:
                if pos >= 0:
                    assert int(_bits(victim[fqn])[pos]) == 0, fqn
    with open(obj, "r+b") as f:  # the last chunk of the object, which no window holds completely: found on the host
        f.seek(-3, os.SEEK_END)
        byte = f.read(1)
        f.seek(-1, os.SEEK_CUR)
        f.write(bytes([byte[0] ^ 0x80]))
    with open(obj, "r+b") as f:  # (the first flip undone)
        f.seek(METADATA_SIZE + 5 * (1 << 16) + 77)
        byte = f.read(1)
        f.seek(-1, os.SEEK_CUR)
        f.write(bytes([byte[0] ^ 0x01]))
    with pytest.raises(BaseException) as exc:
        dcp.load(targets(), checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, loader), no_dist=True)
    cause = exc.value.failures[0][0] if hasattr(exc.value, "failures") else exc.value
    n_chunks = -(-(os.path.getsize(obj) - METADATA_SIZE) // (1 << 16))
    assert isinstance(cause, integrity.ChecksumMismatchError) and f"chunk(s) [{n_chunks - 1}]" in str(cause)


def test_restore_goes_through_a_smaller_buffer_when_no_single_block_is_to_be_had(shm_dir, manager_future, monkeypatch):
    """The loader asks for one buffer for the whole range; when the allocator has no block of that size it halves
    its request until it gets one (two, to alternate between, if it can have them) and restores window by window
    through them - same tensors."""
    from ml_flashpoint.hip import plan as P

    sd_cpu = {f"t{i}": torch.randn(50_000, generator=torch.Generator().manual_seed(i)) for i in range(12)}  # 2.4 MB
    sd_dev = _to_dev(sd_cpu)
    ckpt = os.path.join(shm_dir, "step-8_ckpt")
    dcp.save(sd_dev, checkpoint_id=ckpt, storage_writer=MemoryStorageWriter(_saver(crc_chunk_bytes=1 << 16), manager_future), no_dist=True)
    real, asked = P.try_allocate, []

    def fragmented(nbytes, device):  # no block above 512 KiB
        asked.append(nbytes)
        return real(nbytes, device) if nbytes <= (1 << 19) else None

    monkeypatch.setattr(P, "try_allocate", fragmented)
    target = {k: torch.zeros_like(v) for k, v in sd_dev.items()}
    loader = _loader()
    dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, loader), no_dist=True)
    assert all(torch.equal(target[k].cpu(), sd_cpu[k]) for k in sd_cpu)
    assert len(asked) >= 3 and asked == sorted(asked, reverse=True) and asked[-1] <= (1 << 19)
    assert loader.last_load_stats["windows"] >= 5


@pytest.mark.parametrize("load_file_io", [True, False])
def test_truncated_object_is_refused_before_anything_is_read(shm_dir, manager_future, load_file_io):
    """An object cut short after it was written (its metadata block still records the full length) must end in an
    error, in both IO modes - not in a read past the end of the file or of its mapping."""
    sd = {"a": torch.randn(300_000, device=DEV), "b": torch.ones(1000, device=DEV)}
    ckpt = os.path.join(shm_dir, "step-3_ckpt")
    dcp.save(sd, checkpoint_id=ckpt, storage_writer=MemoryStorageWriter(_saver(), manager_future), no_dist=True)
    obj = os.path.join(ckpt, "__0__0_src0.distcp")
    os.truncate(obj, os.path.getsize(obj) - 70_000)
    target = {k: torch.zeros_like(v) for k, v in sd.items()}
    with pytest.raises(BaseException) as exc:
        dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, _loader(use_file_io=load_file_io)), no_dist=True)
    cause = exc.value.failures[0][0] if hasattr(exc.value, "failures") else exc.value
    assert isinstance(cause, ValueError) and "is truncated" in str(cause)
    assert all(float(t.abs().sum()) == 0 for t in target.values())


def test_several_objects_are_written_and_read_back_concurrently(shm_dir, manager_future):
    """``thread_count=3`` splits a save into three objects; the reader then hands each object to the loader on a
    thread of its own, so three ``read_data`` calls share one copy engine and one device."""
    g = torch.Generator().manual_seed(17)
    sd_cpu = {f"p{i}": torch.randn(40_000 + 1111 * i, generator=g) for i in range(9)}
    sd_cpu["view"] = torch.randn(300, 200, generator=g).t()
    sd_cpu["note"] = "three objects"
    sd_dev = _to_dev(sd_cpu)
    ckpt = os.path.join(shm_dir, "step-6_ckpt")
    saver = _saver(crc_chunk_bytes=1 << 16)
    dcp.save(sd_dev, checkpoint_id=ckpt, storage_writer=MemoryStorageWriter(saver, manager_future, thread_count=3), no_dist=True)
    objects = sorted(n for n in os.listdir(ckpt) if n.endswith(".distcp"))
    assert objects == ["__0__0_src0.distcp", "__0__1_src0.distcp", "__0__2_src0.distcp"]
    metadata = pickle.load(open(os.path.join(ckpt, ".metadata"), "rb"))
    for name in objects:  # each object is the oracle's image of the items the plan put there, in offset order
        here = sorted(((i, s) for i, s in metadata.storage_data.items() if s.relative_path == name), key=lambda kv: kv[1].offset)
        raw = open(os.path.join(ckpt, name), "rb").read()
        tensors = [sd_cpu[i.fqn] for i, _ in here if isinstance(sd_cpu[i.fqn], torch.Tensor)]
        blobs = [raw[METADATA_SIZE + s.offset : METADATA_SIZE + s.offset + s.length] for i, s in here
                 if not isinstance(sd_cpu[i.fqn], torch.Tensor)]
        assert raw == fmt.file_image(tensors, blobs)[0]
    for _ in range(3):  # the interleaving of the three reader threads differs from run to run
        target = {k: (torch.zeros(v.shape, dtype=v.dtype, device=DEV) if isinstance(v, torch.Tensor) else None)
                  for k, v in sd_cpu.items()}
        loader = _loader()
        dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, loader), no_dist=True)
        assert target["note"] == "three objects"
        for k, v in sd_cpu.items():
            if isinstance(v, torch.Tensor):
                assert torch.equal(_bits(target[k]), _bits(v)), k


def test_plans_are_kept_from_save_to_save_and_rebuilt_when_the_tensors_change(shm_dir, manager_future):
    """The second save of the same tensors reuses layout and device tables; new values, a new step counter (host
    tensor) and new pickled objects of the same length only refresh bytes.  A changed shape, address or blob length
    rebuilds.  Every file is the oracle's image of what was live at that save."""
    g = torch.Generator().manual_seed(23)
    sd_cpu = dict(_mixed_state_dict())
    sd_cpu["opt.step"] = torch.tensor([1, 0, 0], dtype=torch.int64)      # stays on the host: its bytes change per save
    sd_dev = _to_dev(sd_cpu, keep_on_host=("w.i64", "opt.step"))
    saver = _saver()

    def save(step, sd_d):
        ckpt = os.path.join(shm_dir, f"step-{step}_ckpt")
        dcp.save(sd_d, checkpoint_id=ckpt, storage_writer=MemoryStorageWriter(saver, manager_future), no_dist=True)
        raw = open(os.path.join(ckpt, "__0__0_src0.distcp"), "rb").read()
        metadata = pickle.load(open(os.path.join(ckpt, ".metadata"), "rb"))
        host = {k: (v.cpu() if isinstance(v, torch.Tensor) else v) for k, v in sd_d.items()}
        image, spans, got_spans = _expected_file(host, metadata, raw)
        assert raw == image and got_spans == spans, f"save {step}"
        return dict(saver.last_save_stats)

    assert "plans_reused" not in save(1, sd_dev)
    for step in (2, 3):  # training moves on: new values everywhere, same tensors
        for k, v in sd_dev.items():
            if isinstance(v, torch.Tensor) and v.is_floating_point() and v.dtype not in (torch.float8_e4m3fn,):
                v.mul_(-1.5).add_(float(step))
        sd_dev["opt.step"][0] = step
        sd_dev["obj.step"] = 123 + step                     # pickles to the same number of bytes
        assert save(step, sd_dev)["plans_reused"] == 1
    sd_dev["obj.cfg"] = "lr=1e-4;name=a-longer-one"          # serialises into the same (padded) number of bytes
    assert save(4, sd_dev)["plans_reused"] == 1
    sd_dev["obj.cfg"] = "lr=1e-4;" + "x" * 300                # a blob of another length moves what lies behind it
    assert "plans_reused" not in save(40, sd_dev)
    assert save(5, sd_dev)["plans_reused"] == 1
    sd_dev["w.fp32"] = torch.randn(129, 66, generator=g).to(DEV)  # same byte count, another shape and address
    assert "plans_reused" not in save(6, sd_dev)
    assert save(7, sd_dev)["plans_reused"] == 1
    saver.release_device_memory()                               # drops the kept plans too
    assert "plans_reused" not in save(8, sd_dev)
    fresh = _saver(reuse_plans=False)
    saver = fresh
    assert "plans_reused" not in save(9, sd_dev) and "plans_reused" not in save(10, sd_dev)


@pytest.mark.parametrize("crc_mode", ["host", "beside"])
@pytest.mark.parametrize("background_write", [False, True])
def test_large_host_resident_tensors_go_from_host_memory_into_the_buffer(shm_dir, manager_future, background_write, crc_mode):
    """A state dict with part of it kept in host memory (offloaded optimizer state): the large host tensors never visit
    the device - the image holds the rest, in runs that are sent to their places around them - and the file is still
    the oracle's, byte for byte, with a valid checksum sidecar; a second save through the kept plan picks up the
    host tensors' new contents; the file restores into device and host targets alike."""
    from ml_flashpoint.hip import integrity
    from ml_flashpoint.hip import plan as P

    g = torch.Generator().manual_seed(21)
    sd_cpu = {
        "dev.w": torch.randn(300, 1000, generator=g),
        "host.m": torch.randn(700, 800, generator=g),                       # 2.2 MB, stays on the host
        "dev.b": torch.randn(4097, generator=g).to(torch.bfloat16),
        "host.v_view": torch.randn(900, 600, generator=g).t(),              # 2.2 MB, a strided view on the host
        "host.small": torch.arange(50, dtype=torch.int64),                  # rides in the image with the headers
        "dev.tail": torch.randint(0, 255, (70001,), dtype=torch.uint8, generator=g),
        "host.last": torch.randn(1 << 18, generator=g),                     # 1 MiB, host, possibly the last record
        "obj.step": 7,
        "obj.big": bytes(range(256)) * 1600,                                # a 400 KiB pickled object: host to buffer too
    }
    on_host = {k for k in sd_cpu if k.startswith("host.")}
    sd = {k: (v.to(DEV) if isinstance(v, torch.Tensor) and k not in on_host else v) for k, v in sd_cpu.items()}
    saver = _saver(crc_chunk_bytes=1 << 18, background_write=background_write, crc_mode=crc_mode)
    big_host_bytes = sum(sd_cpu[k].numel() * sd_cpu[k].element_size() for k in ("host.m", "host.v_view", "host.last"))
    for step in (1, 2):
        ckpt = os.path.join(shm_dir, f"step-{step}_ckpt")
        dcp.save(sd, checkpoint_id=ckpt, storage_writer=MemoryStorageWriter(saver, manager_future), no_dist=True)
        obj = os.path.join(ckpt, "__0__0_src0.distcp")
        raw = open(obj, "rb").read()
        metadata = pickle.load(open(os.path.join(ckpt, ".metadata"), "rb"))
        image, spans, got_spans = _expected_file(sd_cpu, metadata, raw)
        assert raw == image and got_spans == spans
        if not background_write:  # (the background thread keeps its own transfer statistics)
            stats = saver.last_save_stats
            pickled = stats["host_copy_bytes"] - big_host_bytes  # torch.save of the 400 KiB bytes object
            assert 409_600 < pickled < 2 * 409_600  # (its pickle protocol writes bytes as text, about 1.5 x)
            assert stats["d2h_bytes"] == len(raw) - METADATA_SIZE - stats["host_copy_bytes"] == stats["image_bytes"]
            assert stats.get("plans_reused", 0) == (1 if step == 2 else 0)
        chunk, nbytes, crcs = integrity.read_sidecar(obj)
        assert nbytes == len(raw) - METADATA_SIZE
        for k, c in enumerate(crcs):
            piece = raw[METADATA_SIZE + k * chunk : METADATA_SIZE + (k + 1) * chunk]
            buf = ctypes.create_string_buffer(piece, len(piece))
            assert P.crc32c_host(ctypes.addressof(buf), len(piece)) == int(c)
        target = {k: (torch.zeros(v.shape, dtype=v.dtype, device=sd[k].device) if isinstance(v, torch.Tensor) else None)
                  for k, v in sd_cpu.items()}
        dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, _loader()), no_dist=True)
        assert target["obj.step"] == 7 and target["obj.big"] == sd_cpu["obj.big"]
        for k, v in sd_cpu.items():
            if isinstance(v, torch.Tensor):
                assert torch.equal(_bits(target[k]), _bits(v)), k
        # once more with the large host-resident targets read from the file by the copy engine's threads (as
        # targets of 8 MiB and more are), the small one by ``copy_``
        from ml_flashpoint.hip import checkpoint_loader as loader_mod

        for v in target.values():
            if isinstance(v, torch.Tensor):
                v.zero_()
        threshold = loader_mod._HOST_COPY_ON_THE_ENGINE_FROM
        loader_mod._HOST_COPY_ON_THE_ENGINE_FROM = 1 << 19
        try:
            dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, _loader()), no_dist=True)
        finally:
            loader_mod._HOST_COPY_ON_THE_ENGINE_FROM = threshold
        for k, v in sd_cpu.items():
            if isinstance(v, torch.Tensor):
                assert torch.equal(_bits(target[k]), _bits(v)), k
        # the next step's values, in place: on the host for the host tensors, on the device for the others
        for k in ("host.m", "host.v_view", "host.small", "dev.w"):
            sd_cpu[k].mul_(3).add_(1)
        sd["dev.w"].mul_(3).add_(1)
    saver.release_device_memory()


def test_host_tensors_can_be_snapshotted_inside_the_blocking_part(shm_dir):
    """With ``snapshot_host_tensors=True`` the staged object holds clones of the large host tensors: what is written
    is what they held when ``prepare_write_data`` returned, whatever happens to them before ``write_data``."""
    from torch.distributed.checkpoint.planner_helpers import _create_write_items

    host = torch.arange(1 << 17, dtype=torch.float32)  # 512 KiB on the host
    data = {"host": host, "dev": torch.ones(1000, device=DEV)}
    before = host.clone()
    for snapshot in (True, False):
        saver = _saver(snapshot_host_tensors=snapshot)
        cid = CheckpointContainerId(os.path.join(shm_dir, f"step-{int(snapshot)}_ckpt"))
        items = [wi for k, v in data.items() for wi in _create_write_items(k, v)]
        buckets = saver.prepare_write_data(cid, items, _Resolver(data), "data", 1)
        host.add_(1.0)  # the training loop moves on before the transfer
        results = saver.write_data(cid, buckets, replicate_after_write=False)
        where = {r.index.fqn: r.storage_data for r in results}["host"]
        raw = open(os.path.join(cid.data, "data_0_src0.distcp"), "rb").read()
        payload = raw[METADATA_SIZE + where.offset + where.length - host.numel() * 4 : METADATA_SIZE + where.offset + where.length]
        assert payload == (before if snapshot else host).numpy().tobytes()
        before = host.clone()


@pytest.mark.parametrize("side_by_side", [True, False])
@pytest.mark.parametrize("with_sidecar", [False, True])
def test_a_partial_read_uploads_only_what_it_needs(shm_dir, monkeypatch, with_sidecar, side_by_side):
    """Asking for two of sixteen tensors (weights without the optimizer state, say) uploads two neighbourhoods, not
    the object; with a sidecar exactly the chunks that are read are checked: damage inside them is found, damage
    elsewhere is not looked at."""
    from torch.distributed.checkpoint.planner_helpers import _create_write_items

    from ml_flashpoint.hip import checkpoint_loader as loader_mod
    from ml_flashpoint.hip import integrity

    monkeypatch.setattr(loader_mod, "_PARTIAL_READ_MIN_SAVING", 1 << 20)
    monkeypatch.setattr(loader_mod, "_PARTIAL_READ_GAP", 1 << 16)
    if not side_by_side:  # no block for both neighbourhoods at once: they pass through one buffer in turn
        from ml_flashpoint.hip import plan as plan_mod

        real_allocate = plan_mod.try_allocate
        monkeypatch.setattr(plan_mod, "try_allocate", lambda n, device: real_allocate(n, device) if n <= 400_000 else None)
    g = torch.Generator().manual_seed(33)
    data_cpu = {f"t{i:02d}": torch.randn(1 << 16, generator=g) for i in range(16)}  # 256 KiB each, 4 MiB together
    data = {k: v.to(DEV) for k, v in data_cpu.items()}
    saver = _saver(crc_chunk_bytes=(1 << 16) if with_sidecar else 0)
    cid = CheckpointContainerId(os.path.join(shm_dir, "step-9_ckpt"))
    items = [wi for k, v in data.items() for wi in _create_write_items(k, v)]
    buckets = saver.prepare_write_data(cid, items, _Resolver(data), "data", 1)
    info = {r.index.fqn: r.storage_data for r in saver.write_data(cid, buckets, replicate_after_write=False)}
    oid = CheckpointObjectId.from_container(cid, "data_0_src0.distcp")
    by_offset = sorted(info, key=lambda k: info[k].offset)
    wanted = [by_offset[2], by_offset[11]]  # far apart in the object
    storage = {n: info[k] for n, k in enumerate(wanted)}

    def read():
        targets = {k: torch.zeros(1 << 16, device=DEV) for k in wanted}
        reqs = [ReadItem(type=LoadItemType.TENSOR, dest_index=MetadataIndex(k), dest_offsets=torch.Size([0]), storage_index=n,
                         storage_offsets=torch.Size([0]), lengths=torch.Size([1 << 16])) for n, k in enumerate(wanted)]
        loader = _loader()
        loader.read_data(oid, reqs, _Planner(targets), storage)
        return targets, loader.last_load_stats

    targets, stats = read()
    assert all(torch.equal(targets[k].cpu(), data_cpu[k]) for k in wanted)
    assert stats["partial_read_ranges"] == 2 and "upload_began_before_parse" not in stats
    assert stats["h2d_bytes"] <= 2 * ((1 << 18) + (3 << 16))  # two tensors and at most a chunk or two around each
    untouched = info[by_offset[7]]
    with open(oid.data, "r+b") as f:  # damage in a tensor nobody asked for
        f.seek(METADATA_SIZE + untouched.offset + 5000)
        f.write(b"\xff\x00\xff")
    targets, _ = read()
    assert all(torch.equal(targets[k].cpu(), data_cpu[k]) for k in wanted)
    hit = info[wanted[1]]
    with open(oid.data, "r+b") as f:  # damage in a tensor that is asked for
        f.seek(METADATA_SIZE + hit.offset + hit.length - 1000)
        byte = f.read(1)
        f.seek(-1, os.SEEK_CUR)
        f.write(bytes([byte[0] ^ 0x01]))
    if with_sidecar:
        with pytest.raises(integrity.ChecksumMismatchError, match=rf"chunk\(s\) \[{(hit.offset + hit.length - 1000) // (1 << 16)}\]"):
            read()
    else:
        targets, _ = read()
        assert torch.equal(targets[wanted[0]].cpu(), data_cpu[wanted[0]]) and not torch.equal(targets[wanted[1]].cpu(), data_cpu[wanted[1]])


def test_legacy_torch_save_objects_are_still_readable(shm_dir):
    """An object whose signature is TORCH___ holds torch.save records; the loader reads it on the host."""
    from ml_flashpoint.core.defaults import CheckpointFormat

    t = torch.tensor([4.0, 5.0, 6.0])
    oid = CheckpointObjectId(os.path.join(shm_dir, "step-1_ckpt", "legacy.distcp"))
    with CheckpointObjectManager().acquire_buffer(oid, 1 << 16) as w:
        w.set_format_signature(CheckpointFormat.TORCH_SAVE)
        torch.save(t, w)
        length = w.tell()
    target = torch.zeros(3, device=DEV)
    req = ReadItem(type=LoadItemType.TENSOR, dest_index=MetadataIndex("x"), dest_offsets=torch.Size([0]), storage_index=0,
                   storage_offsets=torch.Size([0]), lengths=torch.Size([3]))
    _loader().read_data(oid, [req], _Planner({"x": target}), {0: _StorageInfo("legacy.distcp", 0, length)})
    assert torch.equal(target.cpu(), t)


def test_legacy_format_and_blob_only_objects_are_written_on_the_host(shm_dir, manager_future):
    """``use_optimized_save=False`` (torch.save records, as the reference writes them) with the tensors on the device:
    the generic staging step brings them to the host, the object carries the legacy signature and loads back through
    the loader; a state dict of non-tensors only becomes an object of byte blobs without any image."""
    sd_cpu = {k: v for k, v in _mixed_state_dict().items() if not (isinstance(v, torch.Tensor) and v.dtype == torch.float8_e4m3fn)}
    sd_dev = _to_dev(sd_cpu)
    saver = _saver(use_optimized_save=False, crc_chunk_bytes=1 << 16)
    ckpt = os.path.join(shm_dir, "step-1_ckpt")
    dcp.save(sd_dev, checkpoint_id=ckpt, storage_writer=MemoryStorageWriter(saver, manager_future), no_dist=True)
    raw = open(os.path.join(ckpt, "__0__0_src0.distcp"), "rb").read()
    assert raw[8:16] == b"TORCH___" and saver.last_save_stats.get("objects", 0) == 0  # nothing was packed
    metadata = pickle.load(open(os.path.join(ckpt, ".metadata"), "rb"))
    for index, info in metadata.storage_data.items():
        if isinstance(sd_cpu[index.fqn], torch.Tensor):
            record = raw[METADATA_SIZE + info.offset : METADATA_SIZE + info.offset + info.length]
            got = torch.load(io.BytesIO(record), weights_only=True, map_location="cpu")
            assert torch.equal(_bits(got), _bits(sd_cpu[index.fqn])), index.fqn
    target = {k: (torch.zeros_like(v) if isinstance(v, torch.Tensor) else None) for k, v in sd_dev.items()}
    dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, _loader()), no_dist=True)
    assert all(torch.equal(_bits(target[k]), _bits(v)) for k, v in sd_cpu.items() if isinstance(v, torch.Tensor))
    assert target["obj.step"] == 123
    # byte blobs only, default format
    saver = _saver()
    ckpt2 = os.path.join(shm_dir, "step-2_ckpt")
    only_objects = {"a": 1, "b": "two", "c": 3.5}
    dcp.save(only_objects, checkpoint_id=ckpt2, storage_writer=MemoryStorageWriter(saver, manager_future), no_dist=True)
    assert saver.last_save_stats.get("objects", 0) == 0 and saver._engine is None  # no image, no copy engine
    target = {"a": None, "b": None, "c": None}
    dcp.load(target, checkpoint_id=ckpt2, storage_reader=MemoryStorageReader(ckpt2, _loader()), no_dist=True)
    assert target == only_objects


def test_blocking_stage_call_waits_for_the_pack(shm_dir, manager_future):
    """``stage_write_data_buckets(non_blocking=False)``: the reference's blocking copies return with the data staged;
    with placeholders the call returns once the pack that read the live tensors has finished."""
    from torch.distributed.checkpoint import DefaultSavePlanner
    from torch.distributed.checkpoint.utils import _DistWrapper

    from ml_flashpoint.adapter.pytorch import custom_state_dict_saver as three_calls

    sd = {"w": torch.randn(64 << 20, device=DEV)}
    want = sd["w"].cpu()
    saver = _saver()
    cid = CheckpointContainerId(os.path.join(shm_dir, "step-1_ckpt"))
    writer = MemoryStorageWriter(saver, manager_future)
    writer.reset(cid.data)
    dist = _DistWrapper(None, False, 0)
    buckets, metadata, *_ = three_calls.generate_plan(cid, sd, writer, DefaultSavePlanner(), dist)
    staged = MemoryStorageWriter.stage_write_data_buckets(cid, buckets, non_blocking=False)
    event = buckets[0].tensor_data[0][1].staged.packed_event
    assert event.query(), "the call returned before the pack had finished"
    sd["w"].zero_()  # the live tensor may be overwritten now
    three_calls.write_data(cid, writer, staged, replicate_after_write=False)
    three_calls.finish_write(cid, writer, metadata, dist)
    raw = open(os.path.join(cid.data, "__0__0_src0.distcp"), "rb").read()
    assert raw == fmt.file_image([want])[0]


def test_saver_is_picklable():
    from ml_flashpoint.hip.checkpoint_saver import HipMLFlashpointCheckpointSaver

    s = HipMLFlashpointCheckpointSaver(_zero, _zero, _none, CheckpointObjectManager(), replication_manager=object())
    clone = pickle.loads(pickle.dumps(s))
    assert clone._replication_manager is None and clone._engine is None
    with pytest.raises(RuntimeError, match="ReplicationManager is not available"):
        clone.async_replicate_object(CheckpointObjectId("/x/y"))


def _zero():
    return 0


def _none():
    return None


def test_large_ranges_go_through_two_alternating_buffers_by_choice(shm_dir, manager_future, monkeypatch):
    """A range from a certain size on is restored through two modest buffers even when one buffer for all of it
    could be had: a window is unpacked while the next one is uploaded.  Same tensors, the sidecar checked window by
    window (a flipped bit is found), and ``pipelined_restore=False`` keeps the one image."""
    from ml_flashpoint.hip import checkpoint_loader as loader_mod
    from ml_flashpoint.hip import integrity

    monkeypatch.setattr(loader_mod, "_PIPELINED_FROM_BYTES", 1 << 20)
    monkeypatch.setattr(loader_mod, "_PIPELINED_MIN_BYTES", 1 << 20)
    assert loader_mod._PIPELINED_MIN_BYTES // 2 > loader_mod._PIPELINED_MIN_WINDOW
    sd_cpu = {f"t{i:02d}": torch.randn(90_000 + 777 * i, generator=torch.Generator().manual_seed(i)) for i in range(16)}
    sd_cpu["v.t"] = torch.arange(300 * 200, dtype=torch.int32).reshape(300, 200)
    sd_cpu["step"] = 5
    sd_dev = _to_dev(sd_cpu)
    ckpt = os.path.join(shm_dir, "step-21_ckpt")
    dcp.save(sd_dev, checkpoint_id=ckpt, storage_writer=MemoryStorageWriter(_saver(crc_chunk_bytes=1 << 16), manager_future), no_dist=True)

    def targets():
        out = {k: (torch.zeros_like(v) if isinstance(v, torch.Tensor) else None) for k, v in sd_dev.items()}
        out["v.t"] = torch.zeros(200, 300, dtype=torch.int32, device=DEV).t()  # a strided target: its row stays whole
        return out

    loader = _loader()
    target = targets()
    dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, loader), no_dist=True)
    assert loader.last_load_stats["windows"] >= 4 and target["step"] == 5
    assert all(torch.equal(target[k].cpu(), v) for k, v in sd_cpu.items() if isinstance(v, torch.Tensor))
    whole = _loader(pipelined_restore=False)
    target = targets()
    dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, whole), no_dist=True)
    assert "windows" not in whole.last_load_stats
    assert all(torch.equal(target[k].cpu(), v) for k, v in sd_cpu.items() if isinstance(v, torch.Tensor))

    obj = os.path.join(ckpt, "__0__0_src0.distcp")
    with open(obj, "r+b") as f:
        f.seek(METADATA_SIZE + 9 * (1 << 16) + 5)
        byte = f.read(1)
        f.seek(-1, os.SEEK_CUR)
        f.write(bytes([byte[0] ^ 0x10]))
    with pytest.raises(BaseException) as exc:
        dcp.load(targets(), checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, loader), no_dist=True)
    cause = exc.value.failures[0][0] if hasattr(exc.value, "failures") else exc.value
    assert isinstance(cause, integrity.ChecksumMismatchError) and "chunk(s) [9]" in str(cause)


def test_a_failed_upload_in_a_pipelined_restore_is_reported_and_the_loader_stays_usable(shm_dir, manager_future, monkeypatch):
    """The upload of a later window fails on the helper thread (forced from the host; every kernel that was launched
    still runs to its end): the restore raises that error, commits nothing, and the same loader restores the object
    correctly afterwards."""
    from ml_flashpoint.hip import checkpoint_loader as loader_mod

    monkeypatch.setattr(loader_mod, "_PIPELINED_FROM_BYTES", 1 << 20)
    monkeypatch.setattr(loader_mod, "_PIPELINED_MIN_BYTES", 1 << 20)
    sd_cpu = {f"t{i:02d}": torch.randn(90_000 + 777 * i, generator=torch.Generator().manual_seed(100 + i)) for i in range(16)}
    sd_dev = _to_dev(sd_cpu)
    ckpt = os.path.join(shm_dir, "step-22_ckpt")
    dcp.save(sd_dev, checkpoint_id=ckpt, storage_writer=MemoryStorageWriter(_saver(crc_chunk_bytes=1 << 16), manager_future), no_dist=True)

    loader = _loader()
    real_upload = loader._upload
    calls = []

    def failing_upload(*args, **kwargs):
        calls.append(1)
        if len(calls) == 3:
            raise OSError("injected: the third window could not be read")
        return real_upload(*args, **kwargs)

    committed = []

    class Planner(dcp.DefaultLoadPlanner):
        def commit_tensor(self, read_item, tensor):
            committed.append(read_item.dest_index.fqn)
            return super().commit_tensor(read_item, tensor)

    monkeypatch.setattr(loader, "_upload", failing_upload)
    target = {k: torch.zeros_like(v) for k, v in sd_dev.items()}
    with pytest.raises(BaseException) as exc:
        dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, loader), planner=Planner(), no_dist=True)
    cause = exc.value.failures[0][0] if hasattr(exc.value, "failures") else exc.value
    assert isinstance(cause, OSError) and "injected" in str(cause)
    assert len(calls) >= 3 and committed == []
    torch.cuda.synchronize()

    monkeypatch.setattr(loader, "_upload", real_upload)
    target = {k: torch.zeros_like(v) for k, v in sd_dev.items()}
    dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, loader), planner=Planner(), no_dist=True)
    assert loader.last_load_stats["windows"] >= 4 and sorted(committed) == sorted(sd_cpu)
    assert all(torch.equal(target[k].cpu(), v) for k, v in sd_cpu.items())


@pytest.mark.parametrize("with_sidecar", [True, False])
def test_an_upload_that_began_before_the_headers_were_parsed_and_fails_is_reported(shm_dir, manager_future, monkeypatch,
                                                                                  with_sidecar):
    """The range that holds the requested records is uploaded on a thread while the headers are parsed.  If that
    upload fails (forced from the host), the restore raises its error, commits nothing and leaves nothing running
    that still reads the object; a corrupt object is found before a target is touched; the loader stays usable."""
    from ml_flashpoint.hip import integrity

    sd_cpu = {f"t{i:02d}": torch.randn(40_000 + 333 * i, generator=torch.Generator().manual_seed(7 + i)) for i in range(12)}
    sd_dev = _to_dev(sd_cpu)
    ckpt = os.path.join(shm_dir, "step-31_ckpt")
    dcp.save(sd_dev, checkpoint_id=ckpt, storage_writer=MemoryStorageWriter(
        _saver(crc_chunk_bytes=(1 << 16) if with_sidecar else 0), manager_future), no_dist=True)
    loader = _loader()
    real_upload = loader._upload
    threads = []

    def failing_upload(*args, **kwargs):
        threads.append(threading.current_thread().name)
        raise OSError("injected: the object could not be read")

    committed = []

    class Planner(dcp.DefaultLoadPlanner):
        def commit_tensor(self, read_item, tensor):
            committed.append(read_item.dest_index.fqn)
            return super().commit_tensor(read_item, tensor)

    monkeypatch.setattr(loader, "_upload", failing_upload)
    target = {k: torch.full_like(v, 5.0) for k, v in sd_dev.items()}
    with pytest.raises(BaseException) as exc:
        dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, loader), planner=Planner(), no_dist=True)
    cause = exc.value.failures[0][0] if hasattr(exc.value, "failures") else exc.value
    assert isinstance(cause, OSError) and "injected" in str(cause)
    assert threads == ["mlf-early-upload"] and committed == []
    assert not any(t.name == "mlf-early-upload" for t in threading.enumerate())
    assert all(bool((v == 5.0).all()) for v in target.values())

    monkeypatch.setattr(loader, "_upload", real_upload)
    dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, loader), planner=Planner(), no_dist=True)
    assert loader.last_load_stats["upload_began_before_parse"] == 1 and sorted(committed) == sorted(sd_cpu)
    assert all(torch.equal(target[k].cpu(), v) for k, v in sd_cpu.items())
    if with_sidecar:  # one flipped bit: found by the pass over the uploaded range, before any target is written
        obj = os.path.join(ckpt, "__0__0_src0.distcp")
        with open(obj, "r+b") as f:
            f.seek(METADATA_SIZE + 100_000)
            byte = f.read(1)
            f.seek(-1, os.SEEK_CUR)
            f.write(bytes([byte[0] ^ 0x04]))
        target = {k: torch.full_like(v, 5.0) for k, v in sd_dev.items()}
        with pytest.raises(BaseException) as exc:
            dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, loader), no_dist=True)
        cause = exc.value.failures[0][0] if hasattr(exc.value, "failures") else exc.value
        assert isinstance(cause, integrity.ChecksumMismatchError)
        torch.cuda.synchronize()
        assert all(bool((v == 5.0).all()) for v in target.values())


def test_tied_and_overlapping_tensors_are_saved_once_per_name_and_restored_into_shared_storage(shm_dir, manager_future):
    """Tied weights (one tensor under two names), a slice of it under a third and a view of its transpose: every
    name gets its own record, as the reference's per-item loop writes them (checkpoint_saver.py:667-698); restoring
    into targets that share storage the same way writes the same bytes through every alias."""
    g = torch.Generator().manual_seed(7)
    w_cpu = torch.randn(96, 160, generator=g)
    other_cpu = torch.randn(50_000, generator=g)

    def tied(w, other):
        return {"embed.weight": w, "lm_head.weight": w, "embed.first_rows": w[:40], "embed.transposed": w.t(),
                "other": other, "step": 9}

    sd_cpu, sd_dev = tied(w_cpu, other_cpu), tied(w_cpu.to(DEV), other_cpu.to(DEV))
    ckpt = os.path.join(shm_dir, "step-31_ckpt")
    dcp.save(sd_dev, checkpoint_id=ckpt, storage_writer=MemoryStorageWriter(_saver(crc_chunk_bytes=1 << 16), manager_future),
             no_dist=True)
    raw = open(os.path.join(ckpt, "__0__0_src0.distcp"), "rb").read()
    metadata = pickle.load(open(os.path.join(ckpt, ".metadata"), "rb"))
    image, spans, got_spans = _expected_file(sd_cpu, metadata, raw)
    assert raw == image and got_spans == spans
    assert len([i for i in metadata.storage_data if i.fqn.startswith(("embed", "lm_head"))]) == 4

    target = tied(torch.zeros(96, 160, device=DEV), torch.zeros(50_000, device=DEV))
    target["step"] = None
    dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, _loader()), no_dist=True)
    assert target["step"] == 9 and target["lm_head.weight"].data_ptr() == target["embed.weight"].data_ptr()
    for k, v in sd_cpu.items():
        if isinstance(v, torch.Tensor):
            assert torch.equal(_bits(target[k]), _bits(v)), k


def test_a_real_module_and_optimizer_state_round_trip(shm_dir, manager_future):
    """What a training script hands over: ``module.state_dict(keep_vars=True)`` (Parameters that require grad, a
    channels-last convolution weight, buffers, an integer counter) and ``optimizer.state_dict()`` (nested dicts, lists
    of hyper-parameters, per-parameter moments, 0-dim step tensors).  The object equals the oracle's image of the same
    state on the host, and a second model and optimizer loaded from it hold the same bits: weights, buffers, moments,
    step counts, hyper-parameters."""
    torch.manual_seed(3)

    def build():
        model = torch.nn.Sequential(
            torch.nn.Conv2d(3, 8, 3, padding=1), torch.nn.BatchNorm2d(8), torch.nn.Flatten(), torch.nn.Linear(8 * 6 * 6, 10)
        ).to(DEV).to(memory_format=torch.channels_last)
        return model, torch.optim.AdamW(model.parameters(), lr=1e-2)

    def step(model, optim, seed):
        x = torch.randn(4, 3, 6, 6, generator=torch.Generator().manual_seed(seed)).to(DEV)
        optim.zero_grad()
        model(x).square().mean().backward()
        optim.step()

    model, optim = build()
    for seed in (1, 2):
        step(model, optim, seed)
    sd = {"model": model.state_dict(keep_vars=True), "optim": optim.state_dict()}
    assert sd["model"]["0.weight"].requires_grad and not sd["model"]["0.weight"].is_contiguous()
    ckpt = os.path.join(shm_dir, "step-41_ckpt")
    dcp.save(sd, checkpoint_id=ckpt, storage_writer=MemoryStorageWriter(_saver(crc_chunk_bytes=1 << 16), manager_future),
             no_dist=True)
    raw = open(os.path.join(ckpt, "__0__0_src0.distcp"), "rb").read()
    metadata = pickle.load(open(os.path.join(ckpt, ".metadata"), "rb"))
    from torch.distributed.checkpoint._nested_dict import flatten_state_dict

    flat, _ = flatten_state_dict(sd)
    flat_cpu = {k: (v.detach().cpu() if isinstance(v, torch.Tensor) else v) for k, v in flat.items()}
    image, spans, got_spans = _expected_file(flat_cpu, metadata, raw)
    assert raw == image and got_spans == spans

    model2, optim2 = build()
    step(model2, optim2, 77)  # gives the second optimizer its state entries (other values)
    sd2 = {"model": model2.state_dict(keep_vars=True), "optim": optim2.state_dict()}
    dcp.load(sd2, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, _loader()), no_dist=True)
    optim2.load_state_dict(sd2["optim"])
    for (k, a), b in zip(model.state_dict().items(), model2.state_dict().values()):
        assert torch.equal(_bits(a), _bits(b)), k
    want, got = optim.state_dict(), optim2.state_dict()
    assert got["param_groups"] == want["param_groups"] and got["state"].keys() == want["state"].keys()
    for index, moments in want["state"].items():
        assert moments.keys() == got["state"][index].keys()
        for name, value in moments.items():
            assert torch.equal(_bits(value), _bits(got["state"][index][name])), (index, name)
    assert int(got["state"][0]["step"]) == 2  # (the second optimizer had taken one step of its own)


def test_mx_quantized_weights_round_trip(shm_dir, manager_future):
    """Weights in the MX formats the MI355X computes in: packed fp4 pairs (``float4_e2m1fn_x2``), fp8, and their
    ``float8_e8m0fnu`` block scales (one per 32 values), beside a bf16 tensor.  The object equals the oracle's image of
    the host copies and the restore is bit-exact (targets are zeroed as bytes: torch fills none of these dtypes)."""
    g = torch.Generator().manual_seed(17)
    rb = lambda n: torch.randint(0, 256, (n,), dtype=torch.uint8, generator=g)  # noqa: E731
    rows, cols = 384, 1024
    sd_cpu = {
        "proj.weight_fp4": rb(rows * cols // 2).view(torch.float4_e2m1fn_x2).reshape(rows, cols // 2),
        "proj.weight_fp4_scale": rb(rows * cols // 32).view(torch.float8_e8m0fnu).reshape(rows, cols // 32),
        "gate.weight_fp8": rb(rows * cols).view(torch.float8_e4m3fn).reshape(rows, cols),
        "gate.weight_fp8_scale": rb(rows * cols // 32).view(torch.float8_e8m0fnu).reshape(rows, cols // 32),
        "norm.weight": rb(cols * 2).view(torch.bfloat16),
        "step": 3,
    }
    sd_dev = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in sd_cpu.items()}
    ckpt = os.path.join(shm_dir, "step-51_ckpt")
    dcp.save(sd_dev, checkpoint_id=ckpt, storage_writer=MemoryStorageWriter(_saver(crc_chunk_bytes=1 << 16), manager_future),
             no_dist=True)
    raw = open(os.path.join(ckpt, "__0__0_src0.distcp"), "rb").read()
    metadata = pickle.load(open(os.path.join(ckpt, ".metadata"), "rb"))
    image, spans, got_spans = _expected_file(sd_cpu, metadata, raw)
    assert raw == image and got_spans == spans
    target = {k: (torch.zeros(v.numel() * v.element_size(), dtype=torch.uint8, device=DEV).view(v.dtype).reshape(v.shape)
                  if isinstance(v, torch.Tensor) else None) for k, v in sd_cpu.items()}
    dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, _loader()), no_dist=True)
    assert target["step"] == 3
    for k, v in sd_cpu.items():
        if isinstance(v, torch.Tensor):
            assert target[k].dtype == v.dtype and torch.equal(target[k].cpu().view(torch.uint8), v.view(torch.uint8)), k


def test_views_of_more_dimensions_than_a_descriptor_holds(shm_dir, manager_future):
    """Sources and targets of rank 9 that are not contiguous: a permutation that merges into fewer dimensions goes
    through the kernels as it is, one that does not is staged through a contiguous copy on the device (the saver) or
    restored into a contiguous stand-in and scattered by ``copy_`` (the loader) - as the reference's ``copy_`` takes
    any view (checkpoint_saver.py:797-800, checkpoint_loader.py:331-336).  Bytes against the oracle's index walk."""
    g = torch.Generator().manual_seed(21)
    base = torch.randint(-(2**15), 2**15, (2, 3, 2, 2, 3, 2, 2, 3, 2), dtype=torch.int16, generator=g)
    scattered = base.permute(8, 7, 6, 5, 4, 3, 2, 1, 0)       # nine dimensions, none of which merge
    mergeable = base.permute(0, 1, 2, 3, 4, 5, 6, 8, 7)       # the first seven merge into one
    wide = torch.randint(0, 255, (2, 2, 2, 2, 2, 2, 2, 2, 2, 2, 3), dtype=torch.uint8, generator=g)[..., ::2]  # rank 11
    sd_cpu = {"scattered": scattered, "mergeable": mergeable, "wide": wide, "plain": torch.arange(10.0)}
    sd_dev = _to_dev(sd_cpu)
    assert not sd_dev["scattered"].is_contiguous() and sd_dev["scattered"].dim() == 9
    ckpt = os.path.join(shm_dir, "step-3_ckpt")
    saver = _saver()
    for _ in range(2):  # the second save rebuilds the plan of an object that holds a staged copy
        dcp.save(sd_dev, checkpoint_id=ckpt, storage_writer=MemoryStorageWriter(saver, manager_future), no_dist=True)
    raw = open(os.path.join(ckpt, "__0__0_src0.distcp"), "rb").read()
    metadata = pickle.load(open(os.path.join(ckpt, ".metadata"), "rb"))
    for index, where in metadata.storage_data.items():
        want = fmt.payload_bytes_bruteforce(sd_cpu[index.fqn])
        got = raw[METADATA_SIZE + where.offset + where.length - len(want) : METADATA_SIZE + where.offset + where.length]
        assert got == want, index.fqn
    image, _, _ = _expected_file(sd_cpu, metadata, raw)
    assert raw == image
    # back into views of the same kinds (over zeroed storage), and into plain tensors
    zero = torch.zeros(base.shape, dtype=torch.int16, device=DEV)
    wide_zero = torch.zeros(wide.shape[:-1] + (3,), dtype=torch.uint8, device=DEV)
    target = {"scattered": zero.permute(8, 7, 6, 5, 4, 3, 2, 1, 0),
              "mergeable": torch.zeros(base.shape, dtype=torch.int16, device=DEV).permute(0, 1, 2, 3, 4, 5, 6, 8, 7),
              "wide": wide_zero[..., ::2], "plain": torch.zeros(10, device=DEV)}
    dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, _loader()), no_dist=True)
    for k, v in sd_cpu.items():
        assert torch.equal(target[k].cpu(), v), k
    assert torch.equal(zero.cpu(), base), "the scatter went through the view into its storage"
    assert not bool(wide_zero[..., 1].any()), "the columns the view skips stay untouched"
