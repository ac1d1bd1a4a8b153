"""Asynchronous saves with the gfx950 saver: the transfer runs on a background thread of the process that owns the
GPU; ``write_data`` - in the same process or in a spawned worker that received the pickled buckets - only waits."""

import concurrent.futures
import os
import pickle
import time

import pytest
import torch
import torch.multiprocessing as torch_mp
from torch.distributed.checkpoint import DefaultSavePlanner
from torch.distributed.checkpoint.utils import _DistWrapper

from ml_flashpoint.adapter.pytorch import custom_state_dict_saver as statedictsaver
from ml_flashpoint.adapter.pytorch.memory_storage_writer import MemoryStorageWriter
from ml_flashpoint.checkpoint_object_manager.checkpoint_object_manager import CheckpointObjectManager
from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId
from oracle import mlf_format as fmt

pytestmark = [pytest.mark.gpu, pytest.mark.filterwarnings("ignore:torch.distributed is disabled")]
DEV = "cuda:0"


def _zero():
    return 0


def _none():
    return None


def worker_write(checkpoint_id, writer, buckets):
    """What an async framework's worker process runs: the write phase, nothing else.  Never touches the GPU."""
    return statedictsaver.write_data(checkpoint_id, writer, buckets, replicate_after_write=False)


@pytest.fixture(scope="module")
def manager_future():
    mgr = torch_mp.get_context("spawn").Manager()
    fut = concurrent.futures.Future()
    fut.set_result(mgr)
    yield fut
    mgr.shutdown()


def _make_saver(**kw):
    from ml_flashpoint.hip.checkpoint_saver import HipMLFlashpointCheckpointSaver

    CheckpointObjectManager._worker_pool = None
    return HipMLFlashpointCheckpointSaver(_zero, _zero, _none, CheckpointObjectManager(), None,
                                          initial_buffer_size_bytes=1 << 20, **kw)


def _state_dict():
    g = torch.Generator(device=DEV).manual_seed(3)
    return {f"layer.{i}.w": torch.randn(1 << 18, generator=g, device=DEV) for i in range(8)}


def _check_files(cid, snapshot):
    raw = open(os.path.join(cid.data, "__0__0_src0.distcp"), "rb").read()
    md = pickle.load(open(os.path.join(cid.data, ".metadata"), "rb"))
    order = [i.fqn for i, _ in sorted(md.storage_data.items(), key=lambda kv: kv[1].offset)]
    assert raw == fmt.file_image([snapshot[k] for k in order])[0]


def test_inline_staged_image_refuses_to_cross_a_process_boundary(shm_dir, manager_future):
    saver = _make_saver()
    cid = CheckpointContainerId(os.path.join(shm_dir, "step-1_ckpt"))
    writer = MemoryStorageWriter(saver, manager_future)
    writer.reset(cid.data)
    buckets, *_ = statedictsaver.generate_plan(cid, _state_dict(), writer, DefaultSavePlanner(), _DistWrapper(None, False, 0))
    with pytest.raises(pickle.PicklingError, match="background_write=True"):
        pickle.dumps(buckets)
    statedictsaver.write_data(cid, writer, buckets, replicate_after_write=False)  # in-process it is fine


def test_background_write_in_process_overlaps_with_training(shm_dir, manager_future):
    saver = _make_saver(background_write=True)
    dist = _DistWrapper(None, False, 0)
    sd = _state_dict()
    cid = CheckpointContainerId(os.path.join(shm_dir, "step-2_ckpt"))
    saver.initialize_checkpoint(cid)
    writer = MemoryStorageWriter(saver, manager_future)
    writer.reset(cid.data)
    buckets, metadata, *_ = statedictsaver.generate_plan(cid, sd, writer, DefaultSavePlanner(), dist)
    staged = MemoryStorageWriter.stage_write_data_buckets(cid, buckets, non_blocking=True)  # ends the blocking part
    snapshot = {k: v.cpu() for k, v in sd.items()}
    for v in sd.values():  # "training" overwrites the live tensors while the transfer is in flight
        v.mul_(-3.0)
    results = statedictsaver.write_data(cid, writer, staged, replicate_after_write=False)
    assert len(results) == len(sd)
    statedictsaver.finish_write(cid, writer, metadata, dist)
    saver.finalize_checkpoint(cid)
    _check_files(cid, snapshot)
    with pytest.raises(ValueError, match="already written"):
        saver.write_data(cid, staged, replicate_after_write=False)


def test_worker_process_waits_for_the_gpu_owning_process(shm_dir, manager_future):
    """Megatron-style: buckets (and the writer, minus its manager) are pickled into a spawned worker that runs the
    write phase; the parent's background thread moves the bytes; results come back through the manager proxies."""
    saver = _make_saver(background_write=True)
    dist = _DistWrapper(None, False, 0)
    sd = _state_dict()
    cid = CheckpointContainerId(os.path.join(shm_dir, "step-3_ckpt"))
    saver.initialize_checkpoint(cid)
    writer = MemoryStorageWriter(saver, manager_future)
    writer.reset(cid.data)
    buckets, metadata, *_ = statedictsaver.generate_plan(cid, sd, writer, DefaultSavePlanner(), dist)
    staged = MemoryStorageWriter.stage_write_data_buckets(cid, buckets, non_blocking=True)
    snapshot = {k: v.cpu() for k, v in sd.items()}
    for v in sd.values():
        v.zero_()
    ctx = torch_mp.get_context("spawn")
    with concurrent.futures.ProcessPoolExecutor(max_workers=1, mp_context=ctx) as pool:
        worker_results = pool.submit(worker_write, cid, writer, staged).result(timeout=120)
    assert [r.index.fqn for r in worker_results] == [r.index.fqn for r in writer.get_write_results(cid)]
    statedictsaver.finish_write(cid, writer, metadata, dist)  # reads the results the worker published
    saver.finalize_checkpoint(cid)
    _check_files(cid, snapshot)


def test_failure_in_the_background_write_reaches_the_waiter(shm_dir, manager_future, monkeypatch):
    saver = _make_saver(background_write=True)
    cid = CheckpointContainerId(os.path.join(shm_dir, "step-4_ckpt"))
    writer = MemoryStorageWriter(saver, manager_future)
    writer.reset(cid.data)

    def boom(*a, **kw):
        raise OSError("no space left on device (injected)")

    monkeypatch.setattr(saver._chkpt_obj_manager, "acquire_buffer", boom)
    buckets, *_ = statedictsaver.generate_plan(cid, _state_dict(), writer, DefaultSavePlanner(), _DistWrapper(None, False, 0))
    remote = pickle.loads(pickle.dumps(buckets))  # what a worker would hold
    with pytest.raises(RuntimeError, match="injected"):
        saver.write_data(cid, remote, replicate_after_write=False)
    with pytest.raises(RuntimeError, match="injected"):
        saver.write_data(cid, buckets, replicate_after_write=False)


def test_next_save_does_not_wait_for_the_previous_transfer(shm_dir, manager_future):
    """The blocking part of a save ends when *its* pack has finished: staging waits for the event behind that pack,
    not for the whole device, so a checkpoint that is still crossing the host link does not hold up the next one."""
    saver = _make_saver(background_write=True)
    dist = _DistWrapper(None, False, 0)
    big = {f"big.{i}": torch.full((1 << 28,), float(i), device=DEV) for i in range(6)}  # 6 GiB: >= 0.1 s on the link
    small = _state_dict()

    def begin(step, sd):
        cid = CheckpointContainerId(os.path.join(shm_dir, f"step-{step}_ckpt"))
        saver.initialize_checkpoint(cid)
        writer = MemoryStorageWriter(saver, manager_future)
        writer.reset(cid.data)
        buckets, metadata, *_ = statedictsaver.generate_plan(cid, sd, writer, DefaultSavePlanner(), dist)
        staged = MemoryStorageWriter.stage_write_data_buckets(cid, buckets, non_blocking=True)
        return cid, writer, metadata, staged

    first = begin(10, big)
    first_transfer = saver._staged_of(first[3][0]).future
    t0 = time.perf_counter()
    second = begin(11, small)
    blocked_s = time.perf_counter() - t0
    assert not first_transfer.done(), "the second save's blocking part outlasted the first save's transfer"
    assert blocked_s < 0.25
    snapshot = {k: v.cpu() for k, v in small.items()}
    for v in small.values():
        v.add_(1.0)
    def complete(cid, writer, metadata, staged):
        statedictsaver.write_data(cid, writer, staged, replicate_after_write=False)
        statedictsaver.finish_write(cid, writer, metadata, dist)
        saver.finalize_checkpoint(cid)

    complete(*first)
    with open(os.path.join(first[0].data, "__0__0_src0.distcp"), "rb") as raw:
        raw.seek(-(1 << 20), os.SEEK_END)
        assert raw.read() == torch.full((1 << 18,), 5.0).numpy().tobytes()  # the tail of the last big tensor
    complete(*second)  # finalizing the newer checkpoint removes the older one in the background
    _check_files(second[0], snapshot)


def test_a_follower_can_forward_the_object_while_it_is_still_being_written(shm_dir, manager_future):
    """The staged object publishes how much of its image has reached the buffer file; a follower that reads the file
    behind that mark (what a replication sender would do instead of waiting for the whole object) ends up with the
    object's data section, and has seen the transfer under way."""
    from ml_flashpoint.checkpoint_object_manager.buffer_metadata import METADATA_SIZE

    saver = _make_saver(background_write=True)
    sd = {f"big.{i}": torch.randn(1 << 28, device=DEV) for i in range(2)}  # 2 GiB: some 65 slots of 32 MiB
    cid = CheckpointContainerId(os.path.join(shm_dir, "step-20_ckpt"))
    saver.initialize_checkpoint(cid)
    writer = MemoryStorageWriter(saver, manager_future)
    writer.reset(cid.data)
    dist = _DistWrapper(None, False, 0)
    buckets, metadata, *_ = statedictsaver.generate_plan(cid, sd, writer, DefaultSavePlanner(), dist)
    staged = saver._staged_of(buckets[0])
    total = staged.layout.image_bytes
    path = str(buckets[0].object_id)
    marks, replica = [], bytearray()
    deadline = time.perf_counter() + 60
    fd = None
    while len(replica) < total and time.perf_counter() < deadline:
        mark = staged.landed_bytes()
        if mark > len(replica):
            fd = fd if fd is not None else os.open(path, os.O_RDONLY)
            marks.append(mark)
            replica += os.pread(fd, mark - len(replica), METADATA_SIZE + staged.data_offset + len(replica))
        else:
            time.sleep(0.001)
    assert len(replica) == total and marks == sorted(marks)
    assert len(marks) >= 3, "the follower only ever saw the finished object"
    statedictsaver.write_data(cid, writer, buckets, replicate_after_write=False)
    statedictsaver.finish_write(cid, writer, metadata, dist)
    saver.finalize_checkpoint(cid)
    os.close(fd)
    with open(path, "rb") as f:
        f.seek(METADATA_SIZE)
        assert f.read() == replica
