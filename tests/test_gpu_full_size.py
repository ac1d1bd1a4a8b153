"""The Llama-3-8B shard at its full size (1 164 tensors, 112.4 GB) through the gfx950 saver and loader.

At this size a second copy of the data cannot be held for a byte-by-byte comparison with the CPU oracle, so the
file is checked through properties that do not depend on size: every record header and every offset against the
oracle's closed forms, the payload of a sample of records against the live tensors' bytes, the CRC-32C of every
chunk of the file (host instruction, and the oracle's table-driven C routine on a sample) against the value the GPU
computed from the packed image, the whole-file CRC as the combination of the chunk CRCs, and the restored tensors
against order-sensitive fingerprints of the originals.
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


def test_llama3_8b_shard_full_size_properties(shm_dir, oracle_c):
    from ml_flashpoint.core.checkpoint_loader import DefaultMLFlashpointCheckpointLoader
    from ml_flashpoint.core.checkpoint_saver import DefaultMLFlashpointCheckpointSaver
    from ml_flashpoint.hip import integrity
    from ml_flashpoint.hip import plan as P

    torch.cuda.empty_cache()
    free, _ = torch.cuda.mem_get_info()
    st = os.statvfs(shm_dir)
    if free < 240e9 or st.f_bavail * st.f_frsize < 125e9:
        pytest.skip("needs 240 GB of free HBM and 125 GB of tmpfs")
    sd = workloads.llama3_8b_shard(DEV)
    payload = workloads.payload_bytes(sd)
    assert len(sd) == 1164 and payload == 112_423_657_472
    prints = {k: workloads.fingerprint(v) for k, v in sd.items()}

    CheckpointObjectManager._worker_pool = None
    manager = CheckpointObjectManager()
    saver = DefaultMLFlashpointCheckpointSaver(lambda: 0, lambda: 0, lambda: None, manager, None,
                                               initial_buffer_size_bytes=1 << 20, crc_chunk_bytes=CHUNK)
    fut = concurrent.futures.Future()
    fut.set_result(_LocalManager())
    ckpt = os.path.join(shm_dir, "step-1_ckpt")
    dcp.save(sd, checkpoint_id=ckpt, storage_writer=MemoryStorageWriter(saver, fut), no_dist=True)
    saver.release_device_memory()
    obj = os.path.join(ckpt, "__0__0_src0.distcp")
    metadata = pickle.load(open(os.path.join(ckpt, ".metadata"), "rb"))

    # -- offsets, lengths and headers: the oracle's closed forms, record by record ------------------------------
    by_offset = sorted(metadata.storage_data.items(), key=lambda kv: kv[1].offset)
    assert len(by_offset) == len(sd)
    fd = os.open(obj, os.O_RDONLY)
    try:
        pos = 0
        for index, info in by_offset:
            t = sd[index.fqn]
            header = fmt.header_bytes(fmt.dtype_name(t.dtype), tuple(t.shape))
            assert (info.offset, info.length) == (pos, len(header) + t.numel() * t.element_size()), index.fqn
            assert os.pread(fd, len(header), METADATA_SIZE + pos) == header, index.fqn
            pos += info.length
        data_bytes = pos
        assert os.fstat(fd).st_size == METADATA_SIZE + data_bytes
        assert os.pread(fd, METADATA_SIZE, 0) == fmt.metadata_block(data_bytes)
        assert data_bytes - payload == sum(len(fmt.header_bytes(fmt.dtype_name(t.dtype), tuple(t.shape))) for t in sd.values())

        # -- payload of a sample of records (first, last, smallest, one of the largest, a few in between) -------
        order = [i.fqn for i, _ in by_offset]
        sample = {order[0], order[-1], order[len(order) // 3], order[len(order) // 2], order[2 * len(order) // 3],
                  min(sd, key=lambda k: sd[k].numel()), "model.model.layers.17.mlp.down_proj.weight",
                  "optimizer.exp_avg_sq.model.layers.31.self_attn.k_proj.weight", "optimizer.master.lm_head.weight"}
        where = {i.fqn: s for i, s in by_offset}
        for fqn in sample:
            t = sd[fqn]
            nbytes = t.numel() * t.element_size()
            start = METADATA_SIZE + where[fqn].offset + where[fqn].length - nbytes
            got = np.empty(nbytes, dtype=np.uint8)
            done = 0
            while done < nbytes:
                done += os.preadv(fd, [memoryview(got)[done:]], start + done)
            assert np.array_equal(got, t.cpu().reshape(-1).view(torch.uint8).numpy()), fqn
            del got

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
            tail = 4
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
        v.zero_()
    loader = DefaultMLFlashpointCheckpointLoader(manager, None)
    dcp.load(sd, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, loader), no_dist=True)
    torch.cuda.synchronize()
    wrong = [k for k, v in sd.items() if workloads.fingerprint(v) != prints[k]]
    assert not wrong, wrong[:5]
    assert loader.last_load_stats["device_items"] == len(sd)
    del sd
    torch.cuda.empty_cache()
