"""The benchmark's four device-resident configurations at their full sizes through the gfx950 saver and loader:
the Llama-3-8B shard (1 164 tensors, 112.4 GB), 20 000 small tensors, the Mixtral expert shard (92.9 GB) and 2 000
non-contiguous views of shared parents.

At these sizes a second copy of the data cannot be held for a byte-by-byte comparison with the CPU oracle, so the
file is checked through properties that do not depend on size: every record header and every offset against the
oracle's closed forms (offset of the first record 0, every next one where the previous ends, length = header +
payload, as the reference's own tests assert at tests/core/test_checkpoint_saver.py:1297-1307,1394-1431), the payload
of a sample of records against the live tensors' bytes (for a view: the bytes of ``t.contiguous()``), the CRC-32C of
every chunk of the file (host instruction, and the oracle's table-driven C routine on a sample) against the value the
GPU computed from the packed image, the whole-file CRC as the combination of the chunk CRCs, and the restored
tensors against order-sensitive fingerprints of the originals.
"""

import concurrent.futures
import ctypes
import mmap
import os
import pickle

import numpy as np
import pytest
import torch
import torch.distributed.checkpoint as dcp

import workloads
from ml_flashpoint.adapter.pytorch.memory_storage_reader import MemoryStorageReader
from ml_flashpoint.adapter.pytorch.memory_storage_writer import MemoryStorageWriter
from ml_flashpoint.checkpoint_object_manager.buffer_metadata import METADATA_SIZE
from ml_flashpoint.checkpoint_object_manager.checkpoint_object_manager import CheckpointObjectManager
from oracle import mlf_format as fmt

pytestmark = [pytest.mark.gpu, pytest.mark.filterwarnings("ignore:torch.distributed is disabled")]
DEV = "cuda:0"
CHUNK = 32 << 20


class _LocalManager:
    """In-process stand-in for the multiprocessing manager the writer keeps its results in."""

    def dict(self):
        return {}

    def Event(self):
        import threading

        return threading.Event()


def _build(config):
    """(state dict, objects to keep alive, expected tensor count, expected payload bytes or None)."""
    if config == "llama3-8b-shard":
        return workloads.llama3_8b_shard(DEV), None, 1164, 112_423_657_472
    if config == "many-small":
        return workloads.many_small(DEV), None, 20000, None
    if config == "mixtral-expert-shard":
        return workloads.mixtral_expert_shard(DEV), None, 32 * (7 + 8 * 3), None
    sd, parents = workloads.strided_views(DEV)
    return sd, parents, 2000, None


# free HBM (state + image) and tmpfs the configuration needs; the test is skipped where the box has less
NEEDS = {"llama3-8b-shard": (240e9, 125e9), "many-small": (20e9, 10e9), "mixtral-expert-shard": (200e9, 100e9),
         "strided-views": (60e9, 25e9)}


@pytest.mark.parametrize("config,limit_gb", [("llama3-8b-shard", None), ("many-small", None), ("mixtral-expert-shard", None),
                                             ("strided-views", None),
                                             # room for part of the image only: windows, a resident end, windowed restore
                                             ("llama3-8b-shard", 40), ("strided-views", 3)])
def test_full_size_properties(config, limit_gb, shm_dir, oracle_c):
    from ml_flashpoint.core.checkpoint_loader import DefaultMLFlashpointCheckpointLoader
    from ml_flashpoint.core.checkpoint_saver import DefaultMLFlashpointCheckpointSaver
    from ml_flashpoint.hip import integrity
    from ml_flashpoint.hip import plan as P

    torch.cuda.empty_cache()
    free, _ = torch.cuda.mem_get_info()
    st = os.statvfs(shm_dir)
    need_hbm, need_tmpfs = NEEDS[config]
    if free < need_hbm or st.f_bavail * st.f_frsize < need_tmpfs:
        pytest.skip(f"needs {need_hbm / 1e9:.0f} GB of free HBM and {need_tmpfs / 1e9:.0f} GB of tmpfs")
    sd, keep_alive, n_tensors, want_payload = _build(config)
    payload = workloads.payload_bytes(sd)
    assert len(sd) == n_tensors and (want_payload is None or payload == want_payload)
    if config == "strided-views":
        kinds = {(t.dtype, t.stride(-1) == 1, t.is_contiguous()) for t in sd.values()}
        assert len({d for d, _, _ in kinds}) == 3 and not all(c for _, _, c in kinds)  # three dtypes, real views
    prints = {k: workloads.fingerprint(v) for k, v in sd.items()}

    CheckpointObjectManager._worker_pool = None
    manager = CheckpointObjectManager()
    limit = int(limit_gb * 1e9) if limit_gb else None
    saver = DefaultMLFlashpointCheckpointSaver(lambda: 0, lambda: 0, lambda: None, manager, None,
                                               initial_buffer_size_bytes=1 << 20, crc_chunk_bytes=CHUNK,
                                               max_image_bytes=limit)
    fut = concurrent.futures.Future()
    fut.set_result(_LocalManager())
    ckpt = os.path.join(shm_dir, "step-1_ckpt")
    dcp.save(sd, checkpoint_id=ckpt, storage_writer=MemoryStorageWriter(saver, fut), no_dist=True)
    if limit:
        assert saver.last_save_stats["windows"] >= 2 and limit // 2 < saver.last_save_stats["resident_bytes"] < limit
    saver.release_device_memory()
    obj = os.path.join(ckpt, "__0__0_src0.distcp")
    metadata = pickle.load(open(os.path.join(ckpt, ".metadata"), "rb"))

    # -- offsets, lengths and headers: the oracle's closed forms, record by record ------------------------------
    by_offset = sorted(metadata.storage_data.items(), key=lambda kv: kv[1].offset)
    assert len(by_offset) == len(sd)
    fd = os.open(obj, os.O_RDONLY)
    try:
        pos = 0
        header_total = 0
        for index, info in by_offset:
            t = sd[index.fqn]
            header = fmt.header_bytes(fmt.dtype_name(t.dtype), tuple(t.shape))
            assert (info.offset, info.length) == (pos, len(header) + t.numel() * t.element_size()), index.fqn
            assert os.pread(fd, len(header), METADATA_SIZE + pos) == header, index.fqn
            pos += info.length
            header_total += len(header)
        data_bytes = pos
        assert os.fstat(fd).st_size == METADATA_SIZE + data_bytes
        assert os.pread(fd, METADATA_SIZE, 0) == fmt.metadata_block(data_bytes)
        assert data_bytes - payload == header_total

        # -- payload of a sample of records (first, last, smallest, largest, a few in between) -------------------
        order = [i.fqn for i, _ in by_offset]
        sample = {order[0], order[-1], order[len(order) // 3], order[len(order) // 2], order[2 * len(order) // 3],
                  min(sd, key=lambda k: sd[k].numel()), max(sd, key=lambda k: sd[k].numel())}
        if config == "llama3-8b-shard":
            sample |= {"model.model.layers.17.mlp.down_proj.weight", "optimizer.master.lm_head.weight",
                       "optimizer.exp_avg_sq.model.layers.31.self_attn.k_proj.weight"}
        if config == "strided-views":  # one of every (dtype, view kind) pair
            n_parents = len(keep_alive)  # view i: parent i % n_parents (dtype by parent % 3), kind (i // n_parents) % 3
            sample |= {f"views.{p + n_parents * k}" for p in range(3) for k in range(3)}
        where = {i.fqn: s for i, s in by_offset}
        for fqn in sorted(sample):
            t = sd[fqn]
            nbytes = t.numel() * t.element_size()
            start = METADATA_SIZE + where[fqn].offset + where[fqn].length - nbytes
            got = np.empty(nbytes, dtype=np.uint8)
            done = 0
            while done < nbytes:
                done += os.preadv(fd, [memoryview(got)[done:]], start + done)
            want = t.contiguous().cpu().reshape(-1).view(torch.uint8).numpy()  # the logical tensor, row-major
            assert np.array_equal(got, want), fqn
            del got, want

        # -- every chunk's CRC-32C: GPU value (from the packed image) == CRC of the bytes that reached the file ---
        chunk, recorded_bytes, crcs = integrity.read_sidecar(obj)
        assert (chunk, recorded_bytes, len(crcs)) == (CHUNK, data_bytes, -(-data_bytes // CHUNK))
        mm = mmap.mmap(fd, 0, prot=mmap.PROT_READ)
        try:
            view = np.frombuffer(mm, dtype=np.uint8)
            base = view.ctypes.data + METADATA_SIZE

            def host_crc(k):
                return P.crc32c_host(base + k * CHUNK, min(CHUNK, data_bytes - k * CHUNK))

            with concurrent.futures.ThreadPoolExecutor(16) as pool:
                host = list(pool.map(host_crc, range(len(crcs))))
            bad = [k for k, (a, b) in enumerate(zip(host, crcs)) if a != int(b)]
            assert not bad, f"chunks whose file bytes differ from the packed image: {bad[:8]}"
            for k in (0, len(crcs) // 2, len(crcs) - 1):  # the oracle's table-driven routine on a sample of chunks
                n = min(CHUNK, data_bytes - k * CHUNK)
                assert oracle_c.oracle_crc32c(ctypes.cast(base + k * CHUNK, ctypes.c_char_p), n) == int(crcs[k])
            # checksum of checksums: combining the last chunks' CRCs gives the CRC of their concatenation
            tail = min(4, len(crcs))
            whole = int(crcs[-tail])
            for k in range(len(crcs) - tail + 1, len(crcs)):
                whole = P.crc32c_combine(whole, int(crcs[k]), min(CHUNK, data_bytes - k * CHUNK))
            start = (len(crcs) - tail) * CHUNK
            assert whole == P.crc32c_host(base + start, data_bytes - start)
        finally:
            view = None
            mm.close()
    finally:
        os.close(fd)

    # -- restore into zeroed tensors: bit patterns equal the originals' ------------------------------------------
    for v in sd.values():
        v.zero_() if v.is_contiguous() else v.fill_(0)
    loader = DefaultMLFlashpointCheckpointLoader(manager, None, max_image_bytes=limit)
    dcp.load(sd, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, loader), no_dist=True)
    torch.cuda.synchronize()
    if limit or payload >= (8 << 30):
        assert loader.last_load_stats["windows"] >= 2
    wrong = [k for k, v in sd.items() if workloads.fingerprint(v) != prints[k]]
    assert not wrong, wrong[:5]
    assert loader.last_load_stats["device_items"] == len(sd)
    loader_engine = getattr(loader, "_engine", None)
    if loader_engine is not None:
        loader_engine.destroy()
    del sd, keep_alive
    torch.cuda.empty_cache()
