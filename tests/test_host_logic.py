"""Host-side duties of the saver/loader plug-ins and the small core types, on the CPU (no kernel is launched).

Expectations are those of the reference's tests (tests/core/test_checkpoint_saver.py: markers :324-384, metadata
:1760-1867, removal of older steps :2014-2155; tests/core/test_checkpoint_id_types.py; tests/core/test_checkpoint_loader.py
discovery of complete steps), re-expressed against this package.
"""

import os
import pickle
import subprocess

import pytest
import torch
from torch.distributed.checkpoint.metadata import Metadata

from ml_flashpoint.checkpoint_object_manager.checkpoint_object_manager import CheckpointObjectManager
from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId, CheckpointObjectId
from ml_flashpoint.core.checkpoint_loader import DefaultMLFlashpointCheckpointLoader, MLFlashpointCheckpointLoader
from ml_flashpoint.core.checkpoint_saver import (
    DEFAULT_INITIAL_BUFFER_SIZE_BYTES,
    DefaultMLFlashpointCheckpointSaver,
    MLFlashpointCheckpointSaver,
    ObjectWriteBucket,
)
from ml_flashpoint.core.defaults import CheckpointFormat, default_metadata_object_name
from ml_flashpoint.core.hfid import generate_hfid
from ml_flashpoint.core.tensor_header import TensorHeader


def make_saver(local_rank=0, barrier=None, **kw):
    calls = []
    saver = DefaultMLFlashpointCheckpointSaver(
        global_rank_getter=lambda: 3,
        local_rank_getter=lambda: local_rank,
        global_barrier_func=barrier or (lambda: calls.append("barrier")),
        ckpt_obj_manager=CheckpointObjectManager(),
        replication_manager=None,
        **kw,
    )
    saver._test_calls = calls
    return saver


def test_plugin_classes_and_defaults():
    assert DEFAULT_INITIAL_BUFFER_SIZE_BYTES == 16 * 1024**3
    assert issubclass(DefaultMLFlashpointCheckpointSaver, MLFlashpointCheckpointSaver)
    assert issubclass(DefaultMLFlashpointCheckpointLoader, MLFlashpointCheckpointLoader)
    assert CheckpointFormat.MLF_FORMAT == b"MLF_TENS" and CheckpointFormat.TORCH_SAVE == b"TORCH___"
    assert default_metadata_object_name() == ".metadata"
    with pytest.raises(TypeError):
        MLFlashpointCheckpointSaver()  # abstract


@pytest.mark.parametrize("local_rank", [0, 5])
def test_dirty_marker_lifecycle(tmp_path, local_rank):
    saver = make_saver(local_rank)
    cid = CheckpointContainerId(str(tmp_path / "job" / "step-7_ckpt"))
    marker = f"{cid}__{local_rank}__unfinished"
    saver.initialize_checkpoint(cid)
    assert os.path.isfile(marker) and os.path.getsize(marker) == 0 and os.path.isdir(cid.data)
    saver.initialize_checkpoint(cid)  # idempotent
    assert CheckpointContainerId.get_dirty_version_checkpoint_container_pattern().match(os.path.basename(marker))
    proc = saver.finalize_checkpoint(cid)
    assert not os.path.exists(marker) and saver._test_calls == ["barrier"]
    assert proc is None  # nothing older to delete (and only local rank 0 would)
    saver.finalize_checkpoint(cid)  # marker already gone: a warning, not an error
    assert saver._get_dirty_marker_file_path(CheckpointContainerId(cid.data + "/")) == marker


def test_write_metadata_is_atomic_and_round_trips(tmp_path):
    saver = make_saver()
    cid = CheckpointContainerId(str(tmp_path / "step-1_ckpt"))
    md = Metadata(state_dict_metadata={}, planner_data={"k": 1}, storage_data={"a": 2})
    saver.write_metadata(cid, md)
    assert sorted(os.listdir(cid.data)) == [".metadata"]  # the .tmp file was renamed away
    loader = DefaultMLFlashpointCheckpointLoader(CheckpointObjectManager(), None)
    back = loader.read_metadata(cid)
    assert back.planner_data == {"k": 1} and back.storage_data == {"a": 2}
    saver.write_metadata(cid, md, md_object_name="nested/custom.md")
    assert pickle.load(open(os.path.join(cid.data, "nested", "custom.md"), "rb")).planner_data == {"k": 1}
    with pytest.raises(FileNotFoundError):
        loader.read_metadata(cid, object_name="absent")


@pytest.mark.parametrize(
    "older_than_step, steps, expected_deleted",
    [
        (3, [1, 2, 3, 4, 5], [1, 2]),
        (10, [1, 5, 9, 10, 11], [1, 5, 9]),
        (100, [1, 10, 99, 100, 101], [1, 10, 99]),
        (1, [1, 2, 3], []),
        (5, [1, 2, 3, 4], [1, 2, 3, 4]),
        (10, [1, 5, 9, 10, 11, "invalid", "step-abc_ckpt", "step-10_ckpt_extra", "step--100_ckpt", "step-3.14_ckpt"], [1, 5, 9]),
    ],
)
def test_finalize_removes_only_older_well_formed_steps(tmp_path, older_than_step, steps, expected_deleted):
    base = tmp_path / "checkpoints"
    created = []
    for s in steps:
        name = CheckpointContainerId.format_version_container(s) if isinstance(s, int) else s
        os.makedirs(base / name)
        created.append(str(base / name))
    (base / "step-0_ckpt_file").write_text("a file, not a directory")
    saver = make_saver(local_rank=0)
    cid = CheckpointContainerId(str(base / CheckpointContainerId.format_version_container(older_than_step)))
    os.makedirs(cid.data, exist_ok=True)
    proc = saver.finalize_checkpoint(cid)
    if expected_deleted:
        assert isinstance(proc, subprocess.Popen)
        proc.wait()
    else:
        assert proc is None
    gone = {str(base / CheckpointContainerId.format_version_container(s)) for s in expected_deleted}
    for d in created:
        assert os.path.exists(d) != (d in gone), d
    assert make_saver(local_rank=1).finalize_checkpoint(cid) is None  # only local rank 0 cleans up
    assert saver._remove_older_checkpoints(CheckpointContainerId(str(base / "not-a-step"))) is None


def test_saver_crosses_process_boundaries_as_configuration_only(tmp_path):
    saver = make_saver(initial_buffer_size_bytes=123, crc_chunk_bytes=1 << 20)
    saver._barrier_func = None  # lambdas do not pickle; the reference's users pass module-level callables
    saver._global_rank_getter = saver._local_rank_getter = None
    saver._test_calls = None
    clone = pickle.loads(pickle.dumps(saver))
    assert clone._initial_buffer_size_bytes == 123 and clone._crc_chunk_bytes == 1 << 20
    assert clone._replication_manager is None and clone._engine is None and clone.kernel_events == []


# ---- ids, hfid, header type -------------------------------------------------------------------------------------
def test_checkpoint_ids():
    c = CheckpointContainerId("/a/b/step-12_ckpt///")
    assert c.data == "/a/b/step-12_ckpt" and str(c) == c.data
    assert CheckpointContainerId.parse_version_container_step("step-12_ckpt") == 12
    for bad in ("step-12", "step-x_ckpt", "xstep-1_ckpt", "step-1_ckpt_", "step--1_ckpt"):
        assert CheckpointContainerId.parse_version_container_step(bad) is None
    assert CheckpointContainerId.format_version_container(7) == "step-7_ckpt"
    assert c.get_parent().data == "/a/b" and c.get_parent(2).data == "/a" and c.get_parent(3) is None
    with pytest.raises(ValueError, match="levels_up"):
        c.get_parent(0)
    for bad, msg in (("a/b", "must begin with '/'"), ("/a//b", "cannot be empty"), ("/a/b.", "cannot end with a '.'"), ("/", "root path")):
        with pytest.raises(ValueError, match=msg):
            CheckpointContainerId(bad)
    with pytest.raises(ValueError, match="not a valid leaf ID"):
        CheckpointObjectId("/")
    o = CheckpointObjectId.from_container(c, " /data_0_src3.distcp/ ")
    assert o.data == "/a/b/step-12_ckpt/data_0_src3.distcp" and o.get_parent() == c
    with pytest.raises(ValueError, match="must not be empty"):
        CheckpointObjectId.from_container(c, " // ")
    with pytest.raises(TypeError):
        CheckpointObjectId.from_container("/a", "x")
    assert CheckpointContainerId.create_child(c, "/").data == c.data
    assert CheckpointContainerId.create_child(c, "/sub/dir/").data == c.data + "/sub/dir"
    assert c == "/a/b/step-12_ckpt" and hash(c) == hash(CheckpointContainerId("/a/b/step-12_ckpt"))  # dict keys


def test_hfid():
    a, b = generate_hfid("memwritersave"), generate_hfid("memwritersave")
    assert a != b and a.startswith("memwritersave_") and len(a.split("_")[1]) == 32
    for bad in ("", "Has_Upper", "with-dash", "sp ace"):
        with pytest.raises(ValueError):
            generate_hfid(bad)


def test_tensor_header_round_trip_and_length_prefix():
    h = TensorHeader(dtype=torch.bfloat16, shape=torch.Size([4, 0, 3]))
    raw = h.to_bytes()
    assert int.from_bytes(raw[:4], "little") == len(raw) - 4
    back, used = TensorHeader.from_bytes(raw + b"trailing payload")
    assert used == len(raw) and back == h and isinstance(back.shape, torch.Size)


def test_bucket_dataclass_is_replaceable():
    import dataclasses

    b = ObjectWriteBucket(CheckpointObjectId("/x/y"), "y", [], [])
    c = dataclasses.replace(b, tensor_data=[("item", "tensor")])
    assert c.object_id == b.object_id and c.tensor_data and not b.tensor_data


def test_gc_pause_is_reentrant_and_restores_the_previous_state():
    import gc
    import threading

    from ml_flashpoint.core.utils import gc_paused

    assert gc.isenabled()
    with gc_paused():
        assert not gc.isenabled()
        with gc_paused():  # nested
            assert not gc.isenabled()
        assert not gc.isenabled()

        def other_thread():  # another thread entering and leaving while the outer pause lasts does not end it
            with gc_paused():
                pass

        t = threading.Thread(target=other_thread)
        t.start()
        t.join()
        assert not gc.isenabled()
    assert gc.isenabled()
    with pytest.raises(ValueError):
        with gc_paused():
            raise ValueError("the collector comes back on after an exception")
    assert gc.isenabled()

    @gc_paused()
    def decorated():
        return gc.isenabled()

    assert decorated() is False and decorated() is False and gc.isenabled()
    gc.disable()  # a caller who runs with the collector off keeps it off
    try:
        with gc_paused():
            pass
        assert not gc.isenabled()
    finally:
        gc.enable()


def test_copy_threads_default_follows_the_cpus_available(monkeypatch):
    from ml_flashpoint.hip.checkpoint_saver import EngineConfig

    assert EngineConfig(copy_threads=5).resolved_copy_threads() == 5
    monkeypatch.setattr(os, "sched_getaffinity", lambda pid: set(range(64)))
    assert EngineConfig().resolved_copy_threads() == 16
    monkeypatch.setattr(os, "sched_getaffinity", lambda pid: {0, 1, 2})
    assert EngineConfig().resolved_copy_threads() == 3


def test_partial_read_clusters_are_cut_on_the_right_boundaries(monkeypatch):
    """Pure host arithmetic of the loader: which ranges of an object a partial read uploads."""
    from ml_flashpoint.hip import checkpoint_loader as loader_mod

    monkeypatch.setattr(loader_mod, "_PARTIAL_READ_GAP", 1000)
    cluster = loader_mod.HipMLFlashpointCheckpointLoader._clusters_of
    rows = [(50_000, 51_000, True, "c"), (5_000, 6_000, True, "a"), (6_500, 9_000, False, "b"), (100_000, 100_010, True, "d")]
    # without a sidecar: starts on 4096-byte upload boundaries, ends where the last row ends
    got = cluster(rows, None, 200_000)
    assert [(lo, hi, [r[3] for r in members]) for lo, hi, members in got] == [
        (4096, 9_000, ["a", "b"]), (49_152, 51_000, ["c"]), (98_304, 100_010, ["d"])]
    # with a sidecar: whole checksum chunks, the last one cut at the end of the written data; ranges that come to
    # touch after rounding are one
    got = cluster(rows, 65536, 100_020)
    assert [(lo, hi, [r[3] for r in members]) for lo, hi, members in got] == [(0, 100_020, ["a", "b", "c", "d"])]
    monkeypatch.setattr(loader_mod, "_PARTIAL_READ_GAP", 0)
    assert [(lo, hi) for lo, hi, _ in cluster(rows, 8192, 200_000)] == [(0, 16_384), (49_152, 57_344), (98_304, 106_496)]


def test_a_forked_child_starts_with_free_locks_and_a_running_collector():
    """An async framework forks its worker from the training process at any moment: the child must not inherit a
    held lock (the thread that held it does not exist there) or a collector that was paused by such a thread."""
    import gc
    import os

    from ml_flashpoint.checkpoint_object_manager.checkpoint_object_manager import CheckpointObjectManager
    from ml_flashpoint.core import utils

    assert gc.isenabled()
    with utils.gc_paused():
        utils._gc_pause_lock.acquire()  # as if another thread were inside the bookkeeping right now
        CheckpointObjectManager._worker_pool_lock.acquire()
        try:
            pid = os.fork()
            if pid == 0:
                ok = False
                try:
                    free = utils._gc_pause_lock.acquire(timeout=2) and CheckpointObjectManager._worker_pool_lock.acquire(timeout=2)
                    utils._gc_pause_lock.release()
                    with utils.gc_paused():
                        paused = not gc.isenabled()
                    ok = bool(free) and paused and gc.isenabled() and utils._gc_pause_depth == 0
                finally:
                    os._exit(0 if ok else 1)
            _, status = os.waitpid(pid, 0)
        finally:
            utils._gc_pause_lock.release()
            CheckpointObjectManager._worker_pool_lock.release()
    assert os.WIFEXITED(status) and os.WEXITSTATUS(status) == 0
    assert gc.isenabled()


def test_bench_refuses_more_than_one_gpu():
    """The benchmark measures one GPU's share of the path; asked for more it says so and exits, before any GPU work."""
    import sys

    bench = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bench.py")
    done = subprocess.run([sys.executable, bench, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert done.returncode == 2
    assert "one GPU" in done.stderr + done.stdout


def test_result_markers_of_dead_writer_processes_are_swept(tmp_path, monkeypatch):
    """A background writer hands its results to a waiter in another process through a marker file in the temporary
    directory; a writer that died leaves it behind.  Markers whose process no longer exists go when a saver is
    made; those of live processes stay."""
    import os
    import subprocess
    import sys
    import tempfile

    from ml_flashpoint.hip import checkpoint_saver as hip_saver

    monkeypatch.setattr(tempfile, "tempdir", str(tmp_path))
    gone = subprocess.Popen([sys.executable, "-c", "pass"])
    gone.wait()
    dead = [tmp_path / f"mlf_write_{gone.pid}_abc.done", tmp_path / f"mlf_write_{gone.pid}_abc.done.tmp"]
    alive = [tmp_path / f"mlf_write_{os.getpid()}_own.done", tmp_path / f"mlf_write_{os.getppid()}_parent.done",
             tmp_path / "mlf_write_notapid_x.done", tmp_path / "unrelated.done"]
    for path in dead + alive:
        path.write_bytes(b"x")
    assert hip_saver._sweep_stale_markers() == 2
    assert not any(p.exists() for p in dead) and all(p.exists() for p in alive)
