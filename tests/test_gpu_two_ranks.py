"""Two ranks through the three-call save (``generate_plan`` -> ``write_data`` -> ``finish_write``), three saves in
a row, as the reference's Megatron strategy drives it (src/ml_flashpoint/adapter/pytorch/custom_state_dict_saver.py
:42-145,177-215): the plan goes through the coordinator's reduce-scatter, every rank writes its own object
(``__<rank>__0_src<rank>.distcp``), the write results are gathered and broadcast, and the first rank of the node writes
the one metadata object.

Two fresh processes form a ``gloo`` group (object collectives only: what they move are pickled plans and results in
host memory; no device tensor is handed to it) and share the one GPU.  Each compares its object with the oracle's image
of the tensors it held when the save was staged, then both load the checkpoint back.  From the second save on the
metadata object is pickled while the data is in flight, the other rank's part predicted from the previous save; the
third save runs on the validated plan cache.
"""

import os
import socket
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
    from torch.distributed.checkpoint.default_planner import DefaultSavePlanner
    from torch.distributed.checkpoint.utils import _DistWrapper

    root, port, rank = sys.argv[1], sys.argv[2], int(sys.argv[3])
    dist.init_process_group("gloo", init_method=f"tcp://127.0.0.1:{port}", rank=rank, world_size=2)
    from ml_flashpoint.adapter.pytorch import custom_state_dict_saver as three_calls
    from ml_flashpoint.adapter.pytorch.memory_storage_reader import MemoryStorageReader
    from ml_flashpoint.adapter.pytorch.memory_storage_writer import MemoryStorageWriter
    from ml_flashpoint.checkpoint_object_manager.checkpoint_object_manager import CheckpointObjectManager
    from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId
    from ml_flashpoint.hip.checkpoint_loader import HipMLFlashpointCheckpointLoader
    from ml_flashpoint.hip.checkpoint_saver import HipMLFlashpointCheckpointSaver
    from oracle import mlf_format as fmt

    DEV = "cuda:0"
    assert dist.get_node_local_rank(fallback_rank=0) == rank  # LOCAL_RANK: rank 0 writes the node's metadata object

    class LocalManager:  # the two factory methods the writer uses of a multiprocessing manager
        def dict(self):
            return {}

        def Event(self):
            return threading.Event()

    fut = concurrent.futures.Future()
    fut.set_result(LocalManager())

    g = torch.Generator().manual_seed(100 + rank)
    base = torch.randint(0, 2**15, (96, 80), dtype=torch.int16, generator=g).to(DEV)
    sd = {  # every rank owns its own names, like the stages of a pipeline
        f"stage{rank}.w": torch.randn(300 + 17 * rank, 64, generator=g).to(DEV),
        f"stage{rank}.b": torch.randn(1000 + rank, generator=g).to(torch.bfloat16).to(DEV),
        f"stage{rank}.t": base.t(),
        f"stage{rank}.cols": base[:, ::2],
        f"stage{rank}.step": 10 * rank,
    }
    mine = f"__{rank}__0_src{rank}.distcp"
    saver = HipMLFlashpointCheckpointSaver(lambda: rank, lambda: rank, dist.barrier, CheckpointObjectManager(), None,
                                           initial_buffer_size_bytes=1 << 20, crc_chunk_bytes=1 << 16)
    wrapper = _DistWrapper(None, True, 0)
    cached, metadata, early, respliced = None, None, [], []
    for step in (1, 2, 3):
        cid = CheckpointContainerId(os.path.join(root, f"step-{step}_ckpt"))
        writer = MemoryStorageWriter(saver, fut)
        writer.reset(cid.data)
        buckets, md, central, local, validated = three_calls.generate_plan(cid, sd, writer, DefaultSavePlanner(), wrapper, cached)
        assert (md is None) == (step == 3), "the third save runs on the validated cache"
        metadata = md if md is not None else metadata
        cached = (central, local, validated)
        staged = MemoryStorageWriter.stage_write_data_buckets(cid, buckets, non_blocking=True)
        held = {k: (v.detach().cpu().contiguous() if isinstance(v, torch.Tensor) else v) for k, v in sd.items()}
        for v in sd.values():  # the training step goes on while the image crosses the link
            if isinstance(v, torch.Tensor) and v.is_contiguous():
                v.mul_(-1)
        base.add_(step)
        three_calls.write_data(cid, writer, staged, replicate_after_write=False)
        three_calls.finish_write(cid, writer, metadata, wrapper)
        early.append(writer.early_metadata_used)
        respliced.append(writer.early_metadata_respliced)
        dist.barrier()
        assert sorted(os.listdir(cid.data)) == [".metadata", "__0__0_src0.distcp", "__1__0_src1.distcp"], os.listdir(cid.data)
        written = pickle.load(open(os.path.join(cid.data, ".metadata"), "rb"))
        assert written.storage_meta.checkpoint_id == cid.data and written.storage_meta.save_id == (
            writer._current_save_id if rank == 0 else written.storage_meta.save_id)
        assert {s.relative_path for s in written.storage_data.values()} == {"__0__0_src0.distcp", "__1__0_src1.distcp"}
        own = sorted(((i, s) for i, s in written.storage_data.items() if s.relative_path == mine), key=lambda kv: kv[1].offset)
        assert {i.fqn for i, _ in own} == set(sd), "every rank's items are in the one metadata object, under its object"
        raw = open(os.path.join(cid.data, mine), "rb").read()
        tensors = [held[i.fqn] for i, _ in own if isinstance(held[i.fqn], torch.Tensor)]
        blobs = [raw[4096 + s.offset : 4096 + s.offset + s.length] for i, s in own if not isinstance(held[i.fqn], torch.Tensor)]
        image, spans = fmt.file_image(tensors, blobs)
        assert raw == image and [(s.offset, s.length) for _, s in own] == spans, f"step {step}: object differs from the oracle's image"
        # both ranks load what they own from the checkpoint of this step
        target = {k: (torch.zeros_like(v) if isinstance(v, torch.Tensor) else None) for k, v in held.items()}
        target = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in target.items()}
        loader = HipMLFlashpointCheckpointLoader(CheckpointObjectManager(), None, global_rank_getter=lambda: rank,
                                                 local_rank_getter=lambda: rank)
        dcp.load(target, checkpoint_id=cid.data, storage_reader=MemoryStorageReader(cid.data, loader))
        for k, v in held.items():
            if isinstance(v, torch.Tensor):
                assert torch.equal(target[k].cpu().reshape(-1).view(torch.uint8), v.reshape(-1).view(torch.uint8)), (step, k)
            else:
                assert target[k] == v
        dist.barrier()
        saver.finalize_checkpoint(cid)
    if rank == 0:
        # the metadata object of the second and third save was pickled while their data was in flight, the other
        # rank's results predicted from the save before; the first save had nothing to go by
        assert early == [False, True, True], early
        # and on the kept plan of the third save nothing was pickled: the second save's bytes, storage_meta exchanged
        assert respliced == [False, False, True], respliced
        assert set(saver.last_write_locations) == set(written.storage_data)
    else:
        assert early == [False, False, False] and saver.last_write_locations is None  # never writes a metadata object
    dist.barrier()
    dist.destroy_process_group()
    print(f"TWO-RANKS-OK {rank}", flush=True)
    '''
)


def test_two_ranks_plan_write_and_finish_three_saves(shm_dir):
    with socket.socket() as s:
        s.bind(("127.0.0.1", 0))
        port = s.getsockname()[1]
    repo = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    children = []
    for rank in (0, 1):
        env = dict(os.environ)
        env["PYTHONPATH"] = os.pathsep.join([repo, os.path.join(repo, "ml-flashpoint_amd"), env.get("PYTHONPATH", "")])
        env["LOCAL_RANK"] = str(rank)
        children.append(subprocess.Popen([sys.executable, "-u", "-c", _CHILD, shm_dir, str(port), str(rank)], env=env,
                                         stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True))
    outputs = []
    try:
        for child in children:
            outputs.append(child.communicate(timeout=170))
    finally:
        for child in children:
            if child.poll() is None:
                child.kill()
    for rank, (child, (out, err)) in enumerate(zip(children, outputs)):
        assert child.returncode == 0 and f"TWO-RANKS-OK {rank}" in out, (rank, out[-2000:], err[-4000:])
