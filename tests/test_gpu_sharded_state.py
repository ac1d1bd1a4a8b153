"""Sharded state, as Megatron's strategies hand it to DCP: ``ShardedTensor`` values whose local shards live in HBM,
saved and loaded with a process group in place (one rank; ``gloo``, so every collective moves pickled objects through
host memory and no device tensor ever reaches it).

The body runs in a child process of its own: a process group is process-wide state that the other tests, which call
``dcp.save(..., no_dist=True)``, must not see.  The child writes with the gfx950 saver, compares the object with the
oracle's image of the same shards, then loads into a target that is sharded the other way (every target shard reads a
sub-box of both stored shards) and compares with the full tensor.
"""

import os
import subprocess
import sys
import textwrap

import pytest

pytestmark = pytest.mark.gpu

_CHILD = textwrap.dedent(
    '''
    import concurrent.futures, os, pickle, sys, threading
    import torch
    import torch.distributed as dist
    import torch.distributed.checkpoint as dcp
    from torch.distributed._shard.sharded_tensor import Shard, ShardedTensor, ShardMetadata

    root, port = sys.argv[1], sys.argv[2]
    dist.init_process_group("gloo", init_method=f"tcp://127.0.0.1:{port}", rank=0, world_size=1)
    from ml_flashpoint.adapter.pytorch.memory_storage_reader import MemoryStorageReader
    from ml_flashpoint.adapter.pytorch.memory_storage_writer import MemoryStorageWriter
    from ml_flashpoint.checkpoint_object_manager.buffer_metadata import METADATA_SIZE
    from ml_flashpoint.checkpoint_object_manager.checkpoint_object_manager import CheckpointObjectManager
    from ml_flashpoint.hip.checkpoint_loader import HipMLFlashpointCheckpointLoader
    from ml_flashpoint.hip.checkpoint_saver import HipMLFlashpointCheckpointSaver
    from oracle import mlf_format as fmt

    DEV = "cuda:0"

    class LocalManager:  # the two factory methods the writer uses of a multiprocessing manager
        def dict(self):
            return {}

        def Event(self):
            return threading.Event()

    fut = concurrent.futures.Future()
    fut.set_result(LocalManager())

    def sharded(full, boxes):
        """``full`` as a ShardedTensor whose local shards are the given (offsets, sizes) boxes, each its own
        contiguous device tensor."""
        shards = []
        for offsets, sizes in boxes:
            index = tuple(slice(o, o + n) for o, n in zip(offsets, sizes))
            local = full[index].to(DEV).contiguous()
            shards.append(Shard(local, ShardMetadata(shard_offsets=list(offsets), shard_sizes=list(sizes),
                                                     placement=f"rank:0/{DEV}")))
        return ShardedTensor._init_from_local_shards(shards, tuple(full.shape))

    g = torch.Generator().manual_seed(5)
    full = torch.randn(64, 48, generator=g)
    bias = torch.randn(300, generator=g).to(torch.bfloat16)
    by_rows = [((0, 0), (32, 48)), ((32, 0), (32, 48))]
    by_cols = [((0, 0), (64, 20)), ((0, 20), (64, 28))]
    sd = {"w": sharded(full, by_rows), "bias": bias.to(DEV), "step": 4}

    saver = HipMLFlashpointCheckpointSaver(lambda: 0, lambda: 0, dist.barrier, CheckpointObjectManager(), None,
                                           initial_buffer_size_bytes=1 << 20, crc_chunk_bytes=1 << 16)
    ckpt = os.path.join(root, "step-8_ckpt")
    dcp.save(sd, checkpoint_id=ckpt, storage_writer=MemoryStorageWriter(saver, fut))
    assert sorted(os.listdir(ckpt)) == [".metadata", "__0__0_src0.distcp"], os.listdir(ckpt)
    raw = open(os.path.join(ckpt, "__0__0_src0.distcp"), "rb").read()
    metadata = pickle.load(open(os.path.join(ckpt, ".metadata"), "rb"))
    chunks = metadata.state_dict_metadata["w"].chunks
    assert [(tuple(c.offsets), tuple(c.sizes)) for c in chunks] == by_rows and tuple(metadata.state_dict_metadata["w"].size) == (64, 48)

    def stored(index):  # the host copy of what lies behind a metadata index
        if index.fqn == "w":
            (r0, c0), = [tuple(index.offset)]
            sizes = dict(by_rows)[(r0, c0)]
            return full[r0 : r0 + sizes[0], c0 : c0 + sizes[1]].contiguous()
        return bias if index.fqn == "bias" else None

    by_offset = sorted(metadata.storage_data.items(), key=lambda kv: kv[1].offset)
    tensors = [stored(i) for i, _ in by_offset if stored(i) is not None]
    blobs = [raw[METADATA_SIZE + s.offset : METADATA_SIZE + s.offset + s.length] for i, s in by_offset if stored(i) is None]
    image, spans = fmt.file_image(tensors, blobs)
    assert raw == image and [(s.offset, s.length) for _, s in by_offset] == spans
    assert len(tensors) == 3 and len(blobs) == 1

    # loaded into a target that is cut the other way: each target shard takes a sub-box of both stored shards
    target = {"w": sharded(torch.zeros(64, 48), by_cols), "bias": torch.zeros(300, dtype=torch.bfloat16, device=DEV), "step": None}
    loader = HipMLFlashpointCheckpointLoader(CheckpointObjectManager(), None)
    dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, loader))
    assert target["step"] == 4 and torch.equal(target["bias"].cpu().view(torch.int16), bias.view(torch.int16))
    for shard, (offsets, sizes) in zip(target["w"].local_shards(), by_cols):
        want = full[offsets[0] : offsets[0] + sizes[0], offsets[1] : offsets[1] + sizes[1]]
        assert shard.tensor.is_cuda and torch.equal(shard.tensor.cpu(), want), offsets
    assert loader.last_load_stats["device_items"] == 5  # 2 x 2 sub-boxes and the bias
    saver.finalize_checkpoint(__import__("ml_flashpoint.core.checkpoint_id_types", fromlist=["x"]).CheckpointContainerId(ckpt))
    dist.destroy_process_group()
    print("SHARDED-STATE-OK", flush=True)
    '''
)


def test_sharded_tensors_are_saved_per_shard_and_loaded_into_another_sharding(shm_dir):
    import socket

    with socket.socket() as s:
        s.bind(("127.0.0.1", 0))
        port = s.getsockname()[1]
    repo = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ)
    env["PYTHONPATH"] = os.pathsep.join([repo, os.path.join(repo, "ml-flashpoint_amd"), env.get("PYTHONPATH", "")])
    done = subprocess.run([sys.executable, "-u", "-c", _CHILD, shm_dir, str(port)], env=env, capture_output=True, text=True,
                          timeout=150)
    assert done.returncode == 0 and "SHARDED-STATE-OK" in done.stdout, (done.stdout[-2000:], done.stderr[-4000:])
