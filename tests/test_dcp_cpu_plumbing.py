"""The benchmark's CPU-runnable configuration: a GPT-2-small-shaped fp32 state dict goes through the PyTorch DCP adapters into
buffer files and back, bit-exactly, with the CPU oracle's saver/loader as the plug-ins.

This exercises the host logic of the adapters (plan -> buckets -> results -> metadata -> read plan) without a GPU and
pins the file bytes the oracle produces through that plumbing against the closed-form ``file_image``.
"""

import concurrent.futures
import os
import pickle

import pytest
import torch
import torch.distributed.checkpoint as dcp
import torch.multiprocessing as torch_mp

import workloads
from ml_flashpoint.adapter.pytorch.memory_storage_reader import MemoryStorageReader
from ml_flashpoint.adapter.pytorch.memory_storage_writer import MemoryStorageWriter, _StorageDataContext
from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId
from oracle import mlf_format as fmt
from oracle.cpu_path import OracleCheckpointLoader, OracleCheckpointSaver

pytestmark = pytest.mark.filterwarnings("ignore:torch.distributed is disabled")


@pytest.fixture(scope="module")
def manager_future():
    mgr = torch_mp.get_context("spawn").Manager()
    fut = concurrent.futures.Future()
    fut.set_result(mgr)
    yield fut
    mgr.shutdown()


def _bits(t):
    return t.detach().cpu().contiguous().reshape(-1).view(torch.uint8)


@pytest.mark.parametrize("full", [False, True], ids=["2-layer", "gpt2-small-124M"])
def test_config1_round_trip_through_dcp_adapters(full, shm_dir, manager_future):
    sd = workloads.gpt2_small() if full else workloads.gpt2_small(layers=2, d=64, vocab=1000, ctx=32)
    if full:
        assert len(sd) == 148 and sum(t.numel() for t in sd.values()) == 124_439_808
    sd["extra.step"] = 17  # a non-tensor entry travels as a pickled byte blob
    ckpt = os.path.join(shm_dir, "step-3_ckpt")
    writer = MemoryStorageWriter(OracleCheckpointSaver(initial_buffer_size_bytes=workloads.payload_bytes(sd) + (1 << 20)),
                                 manager_future)
    dcp.save(sd, checkpoint_id=ckpt, storage_writer=writer, no_dist=True)

    assert sorted(os.listdir(ckpt)) == [".metadata", "__0__0_src0.distcp"]
    assert os.path.exists(ckpt + "__0__unfinished")  # plain dcp.save never finalizes
    metadata = pickle.load(open(os.path.join(ckpt, ".metadata"), "rb"))
    assert metadata.storage_meta.checkpoint_id == ckpt and metadata.storage_meta.save_id.startswith("memwritersave_")

    # the file is exactly metadata block + records in plan order, and storage_data points at each record
    raw = open(os.path.join(ckpt, "__0__0_src0.distcp"), "rb").read()
    by_offset = sorted(metadata.storage_data.items(), key=lambda kv: kv[1].offset)
    tensors = [sd[idx.fqn] for idx, _ in by_offset if isinstance(sd[idx.fqn], torch.Tensor)]
    blob_infos = [info for idx, info in by_offset if not isinstance(sd[idx.fqn], torch.Tensor)]
    blobs = [raw[4096 + i.offset : 4096 + i.offset + i.length] for i in blob_infos]
    image, spans = fmt.file_image(tensors, blobs)
    assert raw == image
    assert [(i.offset, i.length) for _, i in by_offset] == spans
    assert all(i.relative_path == "__0__0_src0.distcp" for _, i in by_offset)

    target = {k: (torch.zeros_like(v) if isinstance(v, torch.Tensor) else 0) for k, v in sd.items()}
    dcp.load(target, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, OracleCheckpointLoader()), no_dist=True)
    assert target["extra.step"] == 17
    for k, v in sd.items():
        if isinstance(v, torch.Tensor):
            assert torch.equal(_bits(target[k]), _bits(v)), k


def test_writer_contract_details(shm_dir, manager_future):
    saver = OracleCheckpointSaver()
    writer = MemoryStorageWriter(saver, manager_future, thread_count=0)
    assert writer._thread_count == 1 and writer.path is None and writer.current_checkpoint_id is None
    with pytest.raises(ValueError, match="has not been reset"):
        writer.storage_meta()
    with pytest.raises(ValueError):
        writer.reset("relative/path")
    ckpt = os.path.join(shm_dir, "step-9_ckpt")
    writer.reset(ckpt)
    first_id = writer.storage_meta().save_id
    writer.reset(ckpt)
    assert writer.storage_meta().save_id != first_id and writer.path == ckpt
    assert MemoryStorageWriter.validate_checkpoint_id(ckpt) and not MemoryStorageWriter.validate_checkpoint_id("nope")

    from torch.distributed.checkpoint import SavePlan

    plans = writer.prepare_global_plan([SavePlan([]), SavePlan([])])
    assert [p.storage_data for p in plans] == [_StorageDataContext("__0_"), _StorageDataContext("__1_")]
    with pytest.raises(ValueError, match="prepare_global_plan was not called"):
        writer.write_data(SavePlan([]), planner=None)
    with pytest.raises(RuntimeError, match="results\\[1\\] is None"):
        writer.finish_checkpoint(CheckpointContainerId(ckpt), metadata=None, results=[[], None])

    clone = pickle.loads(pickle.dumps(writer))  # crosses into worker processes without the manager
    assert clone._main_process_torchmp_manager_future is None and clone.path == ckpt

    cid = CheckpointContainerId(ckpt)
    writer._write_events_per_checkpoint_id[cid] = manager_future.result().Event()
    with pytest.raises(RuntimeError, match="Event was never set"):
        writer.get_write_results(cid, wait_timeout_sec=0.05)
    with pytest.raises(KeyError):
        writer.get_write_results(CheckpointContainerId(ckpt + "x"), wait_timeout_sec=0.05)


def test_reader_groups_items_per_file_and_propagates_errors(shm_dir, manager_future):
    sd = {"a": torch.arange(10.0), "b": torch.ones(3, 3)}
    ckpt = os.path.join(shm_dir, "step-1_ckpt")
    dcp.save(sd, checkpoint_id=ckpt, storage_writer=MemoryStorageWriter(OracleCheckpointSaver(), manager_future), no_dist=True)
    os.remove(os.path.join(ckpt, "__0__0_src0.distcp"))
    out = {"a": torch.zeros(10), "b": torch.zeros(3, 3)}
    with pytest.raises(BaseException) as exc:  # DCP's CheckpointException is a BaseException
        dcp.load(out, checkpoint_id=ckpt, storage_reader=MemoryStorageReader(ckpt, OracleCheckpointLoader()), no_dist=True)
    cause = exc.value.failures[0][0] if hasattr(exc.value, "failures") else exc.value  # DCP wraps per-rank failures
    assert isinstance(cause, FileNotFoundError) and "does not exist on any node in the cluster" in str(cause)
    reader = MemoryStorageReader(ckpt, OracleCheckpointLoader())
    md = reader.read_metadata()
    assert md.storage_meta.load_id.startswith("memreaderload_")
    md.storage_data = None
    with pytest.raises(ValueError, match="storage_data cannot be None"):
        reader.set_up_storage_reader(md, True)
