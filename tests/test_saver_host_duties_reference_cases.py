"""Host-only duties of the saver - dirty marker, container directory, finalize order, removal of older steps,
replication hand-off, pickling - case by case as the reference's suite states them
(tests/core/test_checkpoint_saver.py:324-700, :1880-2155, :2157-2240), against the gfx950 saver class.  None of this
touches the GPU, so it runs everywhere."""

import builtins
import concurrent.futures
import os
import pickle
import subprocess
from unittest import mock

import pytest
import torch

from ml_flashpoint.checkpoint_object_manager.buffer_io import BufferIO
from ml_flashpoint.checkpoint_object_manager.checkpoint_object_manager import CheckpointObjectManager
from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId, CheckpointObjectId
from ml_flashpoint.hip import checkpoint_saver as saver_module
from ml_flashpoint.hip.checkpoint_saver import HipMLFlashpointCheckpointSaver


def _zero():
    return 0


def _none():
    return None


def _saver(local_rank=0, global_rank=0, barrier=None, replication_manager=None, **kw):
    CheckpointObjectManager._worker_pool = None
    return HipMLFlashpointCheckpointSaver(
        global_rank_getter=lambda: global_rank, local_rank_getter=lambda: local_rank,
        global_barrier_func=barrier or (lambda: None), ckpt_obj_manager=CheckpointObjectManager(),
        replication_manager=replication_manager, **kw)


# ---- dirty marker and container directory (:324-560) ---------------------------------------------------------------------
@pytest.mark.parametrize("suffix", ["checkpoint_test", "checkpoint_test/"])
def test_marker_path(tmp_path, suffix):
    saver = _saver(local_rank=123)
    cid_str = f"{tmp_path}/{suffix}"
    assert saver._get_dirty_marker_file_path(CheckpointContainerId(cid_str)) == f"{cid_str.rstrip('/')}__123__unfinished"
    root = mock.MagicMock(spec=CheckpointContainerId)
    root.__str__.return_value = "/"
    with pytest.raises(ValueError, match="CheckpointContainerId cannot be the root path '/'"):
        saver._get_dirty_marker_file_path(root)


@pytest.mark.parametrize("local_rank, global_rank", [(0, 0), (1, 0), (0, 1), (1, 1), (2, 5), (8, 0)])
def test_initialize_creates_marker_and_directory(tmp_path, local_rank, global_rank):
    saver = _saver(local_rank, global_rank)
    cid = CheckpointContainerId(f"{tmp_path}/subdir/checkpoint_init_{local_rank}_{global_rank}")  # parent missing too
    marker = f"{cid}__{local_rank}__unfinished"
    saver.initialize_checkpoint(cid)
    saver.initialize_checkpoint(cid)                           # again: harmless
    assert os.path.isfile(marker) and os.path.isdir(cid.data) and os.path.isdir(os.path.dirname(marker))


def test_initialize_keeps_what_the_directory_already_holds(tmp_path):
    cid = CheckpointContainerId(f"{tmp_path}/checkpoint_init_dir")
    os.makedirs(cid.data)
    kept = CheckpointObjectId.from_container(cid, "test_file.txt")
    with open(kept.data, "w") as f:
        f.writelines(["hello\n", "world"])
    _saver(local_rank=1).initialize_checkpoint(cid)
    assert os.path.isdir(cid.data) and open(kept.data).readlines() == ["hello\n", "world"]


def test_marker_comes_first_so_a_failing_marker_leaves_no_directory(tmp_path, monkeypatch):
    """A checkpoint directory without its marker would count as complete; the marker is therefore created before
    the directory, and if it cannot be created the directory must not appear."""
    cid = CheckpointContainerId(f"{tmp_path}/checkpoint_init_fail")
    marker = f"{cid}__0__unfinished"
    real_open = builtins.open

    def failing_open(file, *args, **kwargs):
        if file == marker:
            raise IOError("Test error: Failed to create dirty marker")
        return real_open(file, *args, **kwargs)

    monkeypatch.setattr(builtins, "open", failing_open)
    with pytest.raises(IOError, match="Test error: Failed to create dirty marker"):
        _saver().initialize_checkpoint(cid)
    assert not os.path.exists(cid.data)


# ---- finalize (:562-700) -----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("global_rank, local_rank", [(0, 0), (0, 1), (1, 0), (1, 1), (5, 2)])
@pytest.mark.parametrize("marker_exists", [True, False])
def test_finalize_removes_the_marker_and_nothing_else(tmp_path, global_rank, local_rank, marker_exists):
    cid = CheckpointContainerId(f"{tmp_path}/checkpoint_finalizetest_{local_rank}_{global_rank}")
    data = CheckpointObjectId.from_container(cid, "test_file.txt")
    marker = f"{cid}__{local_rank}__unfinished"
    os.makedirs(cid.data)
    with open(data.data, "w") as f:
        f.writelines(["hello\n", "world"])
    if marker_exists:
        open(marker, "w").close()
    _saver(local_rank, global_rank).finalize_checkpoint(cid)   # a missing marker is worth a warning only
    assert not os.path.exists(marker) and open(data.data).readlines() == ["hello\n", "world"]


def test_finalize_order_marker_then_barrier_then_cleanup(tmp_path):
    order = mock.Mock()
    saver = _saver(barrier=order.barrier)
    cid = CheckpointContainerId(f"{tmp_path}/checkpoint_finalize_barrier")
    with mock.patch.object(saver, "_remove_dirty_checkpoint_marker", order.remove_dirty), \
            mock.patch.object(saver, "_remove_older_checkpoints", order.remove_older):
        result = saver.finalize_checkpoint(cid)
    assert order.mock_calls == [mock.call.remove_dirty(cid), mock.call.barrier(), mock.call.remove_older(older_than=cid)]
    assert result is order.remove_older.return_value


@pytest.mark.parametrize("local_rank", [0, 1, 5])
def test_only_local_rank_0_removes_older_steps(tmp_path, local_rank):
    base = tmp_path / "checkpoints"
    for step in (100, 200, 300, 400):
        os.makedirs(base / f"step-{step}_ckpt")
    proc = _saver(local_rank).finalize_checkpoint(CheckpointContainerId(str(base / "step-300_ckpt")))
    if local_rank == 0:
        assert isinstance(proc, subprocess.Popen)
        proc.wait()
    else:
        assert proc is None
    assert os.path.exists(base / "step-100_ckpt") == (local_rank != 0)
    assert os.path.exists(base / "step-200_ckpt") == (local_rank != 0)
    assert os.path.exists(base / "step-300_ckpt") and os.path.exists(base / "step-400_ckpt")


# ---- removal of older steps (:1880-2155) ------------------------------------------------------------------------------------
def test_remove_older_leaves_everything_that_is_not_an_older_step(tmp_path):
    base = tmp_path / "checkpoints"
    base.mkdir()
    saver = _saver()
    assert saver._remove_older_checkpoints(older_than=CheckpointContainerId(str(base / "step-100_ckpt"))) is None
    assert os.listdir(base) == []                              # an empty base stays empty
    for step in (100, 200):
        os.makedirs(base / f"step-{step}_ckpt")
    (base / "some_file.txt").write_text("hello")
    os.makedirs(base / "not_a_checkpoint")
    assert saver._remove_older_checkpoints(older_than=CheckpointContainerId(str(base / "step-100_ckpt"))) is None
    with mock.patch("subprocess.Popen") as popen:              # an id that is not a step: nothing is attempted
        saver._remove_older_checkpoints(older_than=CheckpointContainerId(str(base / "invalid-step")))
        popen.assert_not_called()
    proc = saver._remove_older_checkpoints(older_than=CheckpointContainerId(str(base / "step-300_ckpt")))
    proc.wait()
    assert sorted(os.listdir(base)) == ["not_a_checkpoint", "some_file.txt"]


def test_remove_older_survives_a_failing_deletion(tmp_path, monkeypatch):
    base = tmp_path / "checkpoints"
    doomed = [str(base / "step-100_ckpt"), str(base / "step-200_ckpt")]
    for d in doomed:
        os.makedirs(d)
    logged = mock.MagicMock()
    monkeypatch.setattr(saver_module, "_LOGGER", logged)
    with mock.patch("subprocess.Popen", side_effect=IOError("Mocked deletion failure")) as popen:
        assert _saver()._remove_older_checkpoints(older_than=CheckpointContainerId(str(base / "step-300_ckpt"))) is None
        popen.assert_called_once()
    command = popen.call_args.args[0]
    assert command[:2] == ["rm", "-rf"] and set(command[2:]) == set(doomed)
    assert all(os.path.exists(d) for d in doomed)
    logged.exception.assert_called_once()


@pytest.mark.parametrize("older_than, steps, expected_deleted", [
    (10, [1, 5, 10, 15], [1, 5]),
    (9, [1, 5, 8, 9, 10], [1, 5, 8]),
    (99, [1, 10, 98, 99, 100], [1, 10, 98]),
    (5, [5, 6, 7], []),
])
def test_remove_older_compares_steps_as_numbers(tmp_path, older_than, steps, expected_deleted):
    base = tmp_path / "checkpoints"
    for s in steps:
        os.makedirs(base / f"step-{s}_ckpt")
    proc = _saver()._remove_older_checkpoints(older_than=CheckpointContainerId(str(base / f"step-{older_than}_ckpt")))
    if proc is not None:
        proc.wait()
    assert sorted(os.listdir(base)) == sorted(f"step-{s}_ckpt" for s in steps if s not in expected_deleted)


# ---- replication hand-off and pickling (:2157-2240) ----------------------------------------------------------------------
def test_async_replicate_object_hands_over_a_read_only_stream(tmp_path):
    replication = mock.MagicMock()
    saver = _saver(replication_manager=replication)
    oid = CheckpointObjectId.from_container(CheckpointContainerId(f"{tmp_path}/c1"), "obj1")
    with saver._chkpt_obj_manager.acquire_buffer(oid, 1024) as f:
        f.write(b"test_async_replicate_object data")
    futures = [concurrent.futures.Future() for _ in range(3)]
    replication.async_replicate.return_value = futures
    assert saver.async_replicate_object(oid) is futures
    assert replication.async_replicate.call_count == 1
    handed = replication.async_replicate.call_args.args[0]
    assert isinstance(handed, BufferIO) and handed.buffer_obj.get_id() == str(oid)
    assert handed.read() == b"test_async_replicate_object data"
    handed.close()
    saver._replication_manager = None                          # as after unpickling in a worker
    with pytest.raises(RuntimeError, match="ReplicationManager is not available"):
        saver.async_replicate_object(oid)


def test_pickling_keeps_configuration_and_callables_but_not_the_replication_manager():
    CheckpointObjectManager._worker_pool = None
    saver = HipMLFlashpointCheckpointSaver(_zero, _zero, _none, CheckpointObjectManager(), replication_manager=object(),
                                           initial_buffer_size_bytes=1024)
    clone = pickle.loads(pickle.dumps(saver))
    assert clone._replication_manager is None and clone._initial_buffer_size_bytes == 1024
    assert clone._use_optimized_save is True and clone._global_rank_getter() == 0 and clone._plan_cache == {}
    legacy = HipMLFlashpointCheckpointSaver(_zero, _zero, _none, CheckpointObjectManager(), None, use_optimized_save=False)
    assert pickle.loads(pickle.dumps(legacy))._use_optimized_save is False  # (tests/core/test_checkpoint_saver.py:2207-2218)


def test_write_data_with_optimized_save_false(tmp_path):
    """The reference's case (tests/core/test_checkpoint_saver.py:188-230), same input: an object written with
    ``use_optimized_save=False`` does not carry the MLF signature and its data section loads with ``torch.load``.
    Plus what that case leaves out: offsets and lengths of several records, byte blobs behind the tensors, and the
    loader reading such an object back."""
    import io

    from torch.distributed.checkpoint.metadata import MetadataIndex
    from torch.distributed.checkpoint.planner import WriteItem, WriteItemType

    from ml_flashpoint.checkpoint_object_manager.buffer_metadata import METADATA_SIZE
    from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId
    from ml_flashpoint.core.defaults import CheckpointFormat

    class Resolver:
        def __init__(self, data):
            self.data = data

        def resolve_data(self, item):
            return self.data[item.index]

    CheckpointObjectManager._worker_pool = None
    manager = CheckpointObjectManager()
    saver = HipMLFlashpointCheckpointSaver(_zero, _zero, _none, manager, None, initial_buffer_size_bytes=1 << 20,
                                           use_optimized_save=False)
    checkpoint_id = CheckpointContainerId(str(tmp_path / "ckpt_opt_false"))
    tensor = torch.tensor([1, 2, 3], dtype=torch.int32)
    view = torch.arange(24, dtype=torch.float32).reshape(4, 6)[:, ::2]
    blob = io.BytesIO(b"pickled step counter")
    data = {MetadataIndex("item_0"): tensor, MetadataIndex("item_1"): view, MetadataIndex("item_2"): blob}
    items = [WriteItem(index=i, type=WriteItemType.BYTE_IO if isinstance(v, io.BytesIO) else WriteItemType.TENSOR)
             for i, v in data.items()]
    buckets = saver.prepare_write_data(checkpoint_id, items, Resolver(data), object_name_prefix="data", bucket_count=1)
    assert len(buckets) == 1 and buckets[0].object_name == "data_0_src0.distcp"
    assert all(isinstance(t, torch.Tensor) for _, t in buckets[0].tensor_data)  # real tensors, no placeholders
    results = saver.write_data(checkpoint_id, buckets, replicate_after_write=False)
    raw = open(buckets[0].object_id.data, "rb").read()
    assert raw[8:16] == CheckpointFormat.TORCH_SAVE != CheckpointFormat.MLF_FORMAT
    section = raw[METADATA_SIZE:]
    assert torch.equal(torch.load(io.BytesIO(section), weights_only=False), tensor)  # the reference's assertion
    by_name = {r.index.fqn: r.storage_data for r in results}
    assert by_name["item_0"].offset == 0 and by_name["item_1"].offset == by_name["item_0"].length
    assert by_name["item_2"].offset == by_name["item_1"].offset + by_name["item_1"].length
    assert by_name["item_2"].offset + by_name["item_2"].length == len(section)
    second = section[by_name["item_1"].offset : by_name["item_1"].offset + by_name["item_1"].length]
    assert torch.equal(torch.load(io.BytesIO(second), weights_only=True), view)
    assert section[by_name["item_2"].offset :] == b"pickled step counter"
