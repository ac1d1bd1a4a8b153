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


def test_worker_process_waits_for_a_save_that_had_room_for_part_of_the_image_only(shm_dir, manager_future):
    """With room for part of the image the blocking part sends windows and a thread of the parent sends the resident
    end; a spawned worker that received the buckets waits for that thread's outcome like for any background write."""
    saver = _make_saver(max_image_bytes=4 << 20, crc_chunk_bytes=1 << 16)  # the object holds 8 MiB
    dist = _DistWrapper(None, False, 0)
    sd = _state_dict()
    cid = CheckpointContainerId(os.path.join(shm_dir, "step-4_ckpt"))
    saver.initialize_checkpoint(cid)
    writer = MemoryStorageWriter(saver, manager_future)
    writer.reset(cid.data)
    buckets, metadata, *_ = statedictsaver.generate_plan(cid, sd, writer, DefaultSavePlanner(), dist)
    assert saver.last_save_stats["windows"] >= 2 and saver.last_save_stats["resident_bytes"] > 0
    staged = MemoryStorageWriter.stage_write_data_buckets(cid, buckets, non_blocking=True)
    snapshot = {k: v.cpu() for k, v in sd.items()}
    for v in sd.values():
        v.zero_()
    ctx = torch_mp.get_context("spawn")
    with concurrent.futures.ProcessPoolExecutor(max_workers=1, mp_context=ctx) as pool:
        worker_results = pool.submit(worker_write, cid, writer, staged).result(timeout=120)
    assert len(worker_results) == len(sd)
    statedictsaver.finish_write(cid, writer, metadata, dist)
    saver.finalize_checkpoint(cid)
    _check_files(cid, snapshot)


def test_engine_streams_follow_the_stream_the_save_runs_on(shm_dir, manager_future):
    """``warm_up`` moves the copy engine's streams off the hardware queue of the stream that is current then; a save
    that later runs on another stream adds that one - and writes the same bytes."""
    saver = _make_saver(background_write=True)
    saver.warm_up()
    assert saver._engine_clear_of == {torch.cuda.current_stream().cuda_stream}
    saver.warm_up()  # nothing to do twice
    dist = _DistWrapper(None, False, 0)
    sd = _state_dict()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    cid = CheckpointContainerId(os.path.join(shm_dir, "step-5_ckpt"))
    saver.initialize_checkpoint(cid)
    writer = MemoryStorageWriter(saver, manager_future)
    writer.reset(cid.data)
    with torch.cuda.stream(side):
        buckets, metadata, *_ = statedictsaver.generate_plan(cid, sd, writer, DefaultSavePlanner(), dist)
        staged = MemoryStorageWriter.stage_write_data_buckets(cid, buckets, non_blocking=True)
    assert saver._engine_clear_of == {torch.cuda.current_stream().cuda_stream, side.cuda_stream}
    snapshot = {k: v.cpu() for k, v in sd.items()}
    statedictsaver.write_data(cid, writer, staged, replicate_after_write=False)
    statedictsaver.finish_write(cid, writer, metadata, dist)
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
    second = begin(11, small)
    # order, not a duration: the second save was planned, packed and staged while the first was still on the link
    assert not first_transfer.done(), "the second save's blocking part outlasted the first save's transfer"
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


def test_replication_manager_that_follows_the_transfer(shm_dir, manager_future):
    """A replication manager with ``async_replicate_streaming`` is handed the object when its transfer begins: a
    follower thread copies the metadata block and then whatever prefix of the data section the counter announces
    into a second file, and ends with a byte-identical replica - identical, too, to the oracle's image.  A manager
    without the method gets the reference's call after the write; a transfer that fails tells the follower so."""
    import concurrent.futures
    import threading

    from ml_flashpoint.checkpoint_object_manager.buffer_metadata import METADATA_SIZE

    class FollowingManager:
        def __init__(self, replica_dir):
            self.replica_dir, self.calls, self.after_write, self.threads, self.errors = replica_dir, [], [], [], []

        def async_replicate(self, buffer_io):
            self.after_write.append(buffer_io.buffer_obj.get_id())
            buffer_io.close()
            return []

        def async_replicate_streaming(self, object_id, data_offset, landed_counter, total, *, outcome):
            self.calls.append((str(object_id), data_offset, total))
            done = concurrent.futures.Future()
            target = os.path.join(self.replica_dir, os.path.basename(str(object_id)))

            def follow():
                try:
                    seen, have = [], 0
                    with open(str(object_id), "rb") as src, open(target, "wb") as dst:
                        dst.write(os.pread(src.fileno(), data_offset, 0))  # the metadata block is final already
                        while have < total:
                            now = landed_counter()
                            if now > have:
                                seen.append(now)
                                dst.write(os.pread(src.fileno(), now - have, data_offset + have))
                                have = now
                            elif outcome.done():
                                outcome.result()  # raises if the transfer failed
                                if landed_counter() == have:
                                    break
                            else:
                                time.sleep(0.0002)
                    done.set_result(seen)
                except BaseException as e:
                    self.errors.append(e)
                    done.set_exception(e)

            thread = threading.Thread(target=follow, daemon=True)
            thread.start()
            self.threads.append(thread)
            return [done]

    import torch.distributed.checkpoint as dcp

    from ml_flashpoint.hip.checkpoint_saver import EngineConfig, HipMLFlashpointCheckpointSaver

    def _saver(replication_manager, **kw):
        CheckpointObjectManager._worker_pool = None
        return HipMLFlashpointCheckpointSaver(_zero, _zero, _none, CheckpointObjectManager(), replication_manager,
                                              initial_buffer_size_bytes=1 << 20, **kw)

    replica_dir = os.path.join(shm_dir, "replica")
    os.makedirs(replica_dir)
    manager = FollowingManager(replica_dir)
    g = torch.Generator(device=DEV).manual_seed(17)
    sd = {f"layer.{i}.w": torch.randn(3 << 20, generator=g, device=DEV) for i in range(8)}  # 96 MiB
    sd_cpu = {k: v.cpu() for k, v in sd.items()}
    saver = _saver(manager, crc_chunk_bytes=1 << 20, engine_config=EngineConfig(slot_bytes=1 << 20, n_slots=3, copy_threads=4))
    ckpt = os.path.join(shm_dir, "step-1_ckpt")
    dcp.save(sd, checkpoint_id=ckpt, storage_writer=MemoryStorageWriter(saver, manager_future), no_dist=True)
    for thread in manager.threads:
        thread.join(30)
    obj = os.path.join(ckpt, "__0__0_src0.distcp")
    assert not manager.errors and not manager.after_write
    assert [c[0] for c in manager.calls] == [obj] and manager.calls[0][1] == METADATA_SIZE
    raw = open(obj, "rb").read()
    assert manager.calls[0][2] == len(raw) - METADATA_SIZE
    replica = open(os.path.join(replica_dir, "__0__0_src0.distcp"), "rb").read()
    metadata = pickle.load(open(os.path.join(ckpt, ".metadata"), "rb"))
    order = [i.fqn for i, _ in sorted(metadata.storage_data.items(), key=lambda kv: kv[1].offset)]
    want, _ = fmt.file_image([sd_cpu[k] for k in order])
    assert raw == want and replica == want
    # a manager without the method: the reference's hand-over after the write
    class PlainManager:
        def __init__(self):
            self.after_write = []

        def async_replicate(self, buffer_io):
            self.after_write.append(buffer_io.buffer_obj.get_id())
            buffer_io.close()
            return []

    plain = PlainManager()
    ckpt2 = os.path.join(shm_dir, "step-2_ckpt")
    dcp.save(sd, checkpoint_id=ckpt2, storage_writer=MemoryStorageWriter(_saver(plain), manager_future), no_dist=True)
    assert plain.after_write == [os.path.join(ckpt2, "__0__0_src0.distcp")]


def test_discovery_with_checksums_of_objects_written_on_the_gpu(shm_dir, manager_future):
    """Two steps saved by the gfx950 saver with checksums; a byte of the newer step's object is flipped afterwards.
    Recovery discovery that verifies while choosing (host-side check against the sidecars the GPU produced, collectives
    injected) picks the older step; discovery that only looks at what is present, as the reference's, the newer one.
    The sidecars lie outside the containers, so no lister takes them for objects."""
    import torch.distributed.checkpoint as dcp

    from ml_flashpoint.checkpoint_object_manager.buffer_metadata import METADATA_SIZE
    from ml_flashpoint.hip import integrity
    from ml_flashpoint.hip.checkpoint_loader import HipMLFlashpointCheckpointLoader
    from ml_flashpoint.hip.checkpoint_saver import HipMLFlashpointCheckpointSaver

    CheckpointObjectManager._worker_pool = None
    base = os.path.join(shm_dir, "job")
    for crc_mode, step in (("beside", 1), ("fused", 2)):
        saver = HipMLFlashpointCheckpointSaver(_zero, _zero, _none, CheckpointObjectManager(), None,
                                               initial_buffer_size_bytes=1 << 20, crc_chunk_bytes=1 << 16, crc_mode=crc_mode)
        cid = CheckpointContainerId(os.path.join(base, f"step-{step}_ckpt"))
        sd = _state_dict()
        dcp.save(sd, checkpoint_id=cid.data, storage_writer=MemoryStorageWriter(saver, manager_future), no_dist=True)
        saver._remove_dirty_checkpoint_marker(cid)  # plain dcp.save leaves the marker to the strategy's finalize step
        assert sorted(os.listdir(cid.data)) == [".metadata", "__0__0_src0.distcp"]  # no sidecar in the container
        assert os.path.exists(integrity.sidecar_path(os.path.join(cid.data, "__0__0_src0.distcp")))
    assert sorted(os.listdir(base)) == [".mlf_crc32c", "step-1_ckpt", "step-2_ckpt"]

    calls = {"gather": 0, "broadcast": 0}

    def all_gather(out_list, obj):
        calls["gather"] += 1
        out_list[0] = obj

    def broadcast(obj_list, src=0):
        calls["broadcast"] += 1

    def loader(**kw):
        made = HipMLFlashpointCheckpointLoader(CheckpointObjectManager(), None, all_gather_object_func=all_gather,
                                               broadcast_object_list_func=broadcast, **kw)
        made.common_state_object_name = None  # written by plain dcp.save: no common.pt
        return made

    base_id = CheckpointContainerId(base)
    assert loader(verify_on_discovery=True).get_latest_complete_checkpoint(base_id).data.endswith("step-2_ckpt")
    newer = os.path.join(base, "step-2_ckpt", "__0__0_src0.distcp")
    with open(newer, "r+b") as f:
        f.seek(METADATA_SIZE + 3 * (1 << 16) + 99)
        byte = f.read(1)
        f.seek(-1, os.SEEK_CUR)
        f.write(bytes([byte[0] ^ 0x40]))
    assert loader().get_latest_complete_checkpoint(base_id).data.endswith("step-2_ckpt")
    checking = loader(verify_on_discovery=True)
    assert checking.get_latest_complete_checkpoint(base_id).data.endswith("step-1_ckpt")
    assert calls["gather"] >= 4 and calls["broadcast"] >= 2
    # the older step restores; the corrupted one is refused by the restore as well
    target = {k: torch.zeros_like(v) for k, v in _state_dict().items()}
    older = os.path.join(base, "step-1_ckpt")
    from ml_flashpoint.adapter.pytorch.memory_storage_reader import MemoryStorageReader

    dcp.load(target, checkpoint_id=older, storage_reader=MemoryStorageReader(older, checking), no_dist=True)
    assert all(torch.equal(target[k], v) for k, v in _state_dict().items())
    with pytest.raises(BaseException) as exc:
        bad = os.path.join(base, "step-2_ckpt")
        dcp.load(target, checkpoint_id=bad, storage_reader=MemoryStorageReader(bad, checking), no_dist=True)
    cause = exc.value.failures[0][0] if hasattr(exc.value, "failures") else exc.value
    assert isinstance(cause, integrity.ChecksumMismatchError) and "chunk(s) [3]" in str(cause)
    # finalize of a later step removes an older step's sidecars along with the step
    saver = HipMLFlashpointCheckpointSaver(_zero, _zero, _none, CheckpointObjectManager(), None)
    proc = saver._remove_older_checkpoints(CheckpointContainerId(os.path.join(base, "step-2_ckpt")))
    proc.wait()
    assert sorted(os.listdir(base)) == [".mlf_crc32c", "step-2_ckpt"]
    assert os.listdir(os.path.join(base, ".mlf_crc32c")) == ["step-2_ckpt"]
