"""``MemoryStorageWriter`` behaviour, case by case as the reference's suite states it
(tests/adapter/pytorch/test_memory_storage_writer.py:55-1640), with a ``unittest.mock`` saver in the saver's place.
Waits that the reference lets run into its 15 s default are given a short timeout here."""

import concurrent.futures
import dataclasses
import pickle
import re
import threading
import time
from unittest import mock

import pytest
import torch
from torch import multiprocessing as torch_mp
from torch.distributed.checkpoint import Metadata, SavePlan, WriteItem
from torch.distributed.checkpoint import metadata as torchdistmeta
from torch.distributed.checkpoint.planner import WriteItemType
from torch.distributed.checkpoint.storage import WriteResult
from torch.futures import Future as TorchFuture

from ml_flashpoint.adapter.pytorch.memory_storage_writer import MemoryStorageWriter, _StorageDataContext
from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId, CheckpointObjectId
from ml_flashpoint.core.checkpoint_saver import (
    DefaultMLFlashpointCheckpointSaver,
    MLFlashpointCheckpointSaver,
    ObjectWriteBucket,
)

RESET_ERROR = re.escape("MemoryStorageWriter has not been reset. Call reset() before using this method.")
PREFIX_ERROR = re.escape("SavePlan.storage_data is not a valid _StorageDataContext or prefix is empty.")
IDX = torchdistmeta.MetadataIndex


def _zero():
    return 0


def _none():
    return None


class DummyObjectManager:
    pass


class DummyReplicationManager:
    pass


@pytest.fixture(scope="module")
def mp_manager_future():
    manager = torch_mp.Manager()
    future = concurrent.futures.Future()
    future.set_result(manager)
    yield future
    manager.shutdown()


@pytest.fixture
def saver():
    return mock.MagicMock(spec=MLFlashpointCheckpointSaver)


@pytest.fixture
def writer(saver, mp_manager_future):
    return MemoryStorageWriter(checkpoint_saver=saver, mp_manager_future=mp_manager_future)


def _wr(name, size=10):
    return WriteResult(index=IDX(name), size_in_bytes=size, storage_data=f"data_{name}")


def _items(*kinds):
    return [WriteItem(index=IDX(chr(ord("a") + i)), type=k) for i, k in enumerate(kinds)]


def _buckets(checkpoint_id, count=3):
    return [
        ObjectWriteBucket(
            object_id=CheckpointObjectId(f"{checkpoint_id.data}/obj_{i}"),
            object_name=f"obj_{i}",
            bytesio_data=[(WriteItem(index=IDX(f"bytes_{i}"), type=WriteItemType.BYTE_IO), b"some_bytes_data")],
            tensor_data=[(WriteItem(index=IDX(f"tensor_{i}"), type=WriteItemType.TENSOR), torch.tensor([i, i + 1, i + 2]))],
        )
        for i in range(count)
    ]


def _signal(writer, checkpoint_id, results):
    """What a finished write leaves behind in the shared state."""
    writer._write_results_per_checkpoint_id[checkpoint_id] = results
    writer._write_events_per_checkpoint_id[checkpoint_id] = writer._main_process_torchmp_manager_future.result().Event()
    writer._write_events_per_checkpoint_id[checkpoint_id].set()


# ---- construction, reset, identity (:69-318) ------------------------------------------------------------------------------
def test_construction(saver, mp_manager_future):
    w = MemoryStorageWriter(checkpoint_saver=saver, mp_manager_future=mp_manager_future)
    assert w._checkpoint_saver is saver and w._main_process_torchmp_manager_future is mp_manager_future
    assert w._write_events_per_checkpoint_id is None and w._write_results_per_checkpoint_id is None
    assert w._thread_count == 1 and w.current_checkpoint_id is None and w.path is None
    for given, kept in ((5, 5), (1, 1), (0, 1), (-1, 1), (-10, 1)):
        assert MemoryStorageWriter(saver, mp_manager_future, thread_count=given)._thread_count == kept
    w.set_up_storage_writer(is_coordinator=True)
    w.set_up_storage_writer(is_coordinator=False)


def test_validate_checkpoint_id():
    assert MemoryStorageWriter.validate_checkpoint_id("/valid/path") is True
    assert MemoryStorageWriter.validate_checkpoint_id("/valid/path/with/number/123") is True
    assert MemoryStorageWriter.validate_checkpoint_id("invalid/path") is False
    assert MemoryStorageWriter.validate_checkpoint_id(123) is False
    assert MemoryStorageWriter.validate_checkpoint_id(None) is False


def test_reset_sets_id_and_a_fresh_save_id(writer):
    writer.reset("/test_checkpoint")
    assert writer._current_checkpoint_id.data == "/test_checkpoint" and writer.path == "/test_checkpoint"
    first = writer._current_save_id
    assert isinstance(first, str) and first.startswith("memwritersave") and len(first) > len("memwritersave")
    writer.reset("/new_test_checkpoint")
    assert isinstance(writer.current_checkpoint_id, CheckpointContainerId)
    assert writer.current_checkpoint_id == CheckpointContainerId("/new_test_checkpoint")
    assert writer._current_save_id.startswith("memwritersave") and writer._current_save_id != first
    assert writer.storage_meta() == torchdistmeta.StorageMeta(checkpoint_id="/new_test_checkpoint",
                                                              save_id=writer._current_save_id)
    with pytest.raises(ValueError, match="A CheckpointContainerId must begin with '/'"):
        writer.reset("invalid/id")


def test_calls_before_reset(writer):
    plan = SavePlan(items=_items(WriteItemType.TENSOR, WriteItemType.BYTE_IO))
    for call in (writer.storage_meta, lambda: writer.prepare_local_plan(plan),
                 lambda: writer.write_data(mock.MagicMock(), mock.MagicMock()),
                 lambda: writer.finish(Metadata(state_dict_metadata={}), [])):
        with pytest.raises(ValueError, match=RESET_ERROR):
            call()


@pytest.mark.parametrize("events_unset, has_future, expect_init",
                         [(True, True, True), (True, False, False), (False, True, False), (False, False, False)])
def test_reset_creates_the_shared_state_once(saver, mp_manager_future, events_unset, has_future, expect_init):
    future = mock.MagicMock(wraps=mp_manager_future) if has_future else None
    w = MemoryStorageWriter(checkpoint_saver=saver, mp_manager_future=future)
    if not events_unset:
        manager = mp_manager_future.result()
        w._write_events_per_checkpoint_id, w._write_results_per_checkpoint_id = manager.dict(), manager.dict()
    w.reset("/test_checkpoint")
    if expect_init:
        assert type(w._write_events_per_checkpoint_id).__name__ == "DictProxy" and len(w._write_events_per_checkpoint_id) == 0
        assert type(w._write_results_per_checkpoint_id).__name__ == "DictProxy" and len(w._write_results_per_checkpoint_id) == 0
        future.result.assert_called_once()
    else:
        assert (w._write_events_per_checkpoint_id is None) == events_unset
        if future is not None:
            future.result.assert_not_called()


# ---- plans (:320-391) ----------------------------------------------------------------------------------------------------
def test_prepare_local_plan_starts_the_checkpoint(writer, saver):
    writer.reset("/test_checkpoint_prepare_local")
    plan = SavePlan(items=_items(WriteItemType.TENSOR, WriteItemType.BYTE_IO))
    assert writer.prepare_local_plan(plan) is plan
    saver.initialize_checkpoint.assert_called_once_with(writer._current_checkpoint_id)
    saver.initialize_checkpoint.side_effect = RuntimeError("Init failed")
    with pytest.raises(RuntimeError, match="Init failed"):
        writer.prepare_local_plan(plan)


def test_prepare_global_plan_numbers_the_prefixes(writer):
    item1, item2 = _items(WriteItemType.TENSOR, WriteItemType.TENSOR)
    new_plans = writer.prepare_global_plan([SavePlan(items=[item1]), SavePlan(items=[item2])])
    assert [type(p.storage_data) for p in new_plans] == [_StorageDataContext] * 2
    assert [p.storage_data.prefix for p in new_plans] == ["__0_", "__1_"]
    assert new_plans[0].items == [item1] and new_plans[1].items == [item2]


# ---- stage / buckets (:393-613) ------------------------------------------------------------------------------------------
def test_stage_of_a_state_dict_on_the_host(writer):
    state_dict = {"a": torch.tensor([1, 2, 3], device="cpu"), "b": "a string", "c": 123}
    staged = writer.stage(state_dict)
    assert staged["a"].device == torch.device("cpu") and torch.equal(staged["a"], state_dict["a"])
    assert staged["b"] == "a string" and staged["c"] == 123 and len(staged) == 3


@pytest.mark.parametrize("thread_count", [1, 4, 8])
def test_prepare_write_data_buckets_registers_an_event_and_asks_the_saver(saver, mp_manager_future, thread_count):
    w = MemoryStorageWriter(checkpoint_saver=saver, mp_manager_future=mp_manager_future, thread_count=thread_count)
    cid = CheckpointContainerId("/test_checkpoint_with_thread_count")
    plan = SavePlan(items=[], storage_data=_StorageDataContext(prefix="__0_"))
    planner = mock.MagicMock()
    saver.prepare_write_data.return_value = expected = _buckets(cid)
    w.reset(cid.data)
    assert w.prepare_write_data_buckets(cid, plan, planner) == expected
    assert cid in w._write_events_per_checkpoint_id and not w._write_events_per_checkpoint_id[cid].is_set()
    saver.prepare_write_data.assert_called_once_with(cid, plan.items, planner, "__0_", bucket_count=thread_count)


def test_stage_write_data_buckets_is_static_and_keeps_host_tensors():
    cid = CheckpointContainerId("/test_checkpoint")
    buckets = _buckets(cid)
    with mock.patch("torch.cuda.is_available", return_value=False), mock.patch("torch.cuda.synchronize") as sync:
        staged = MemoryStorageWriter.stage_write_data_buckets(cid, buckets, non_blocking=True)
        sync.assert_not_called()                             # nothing to wait for without a device
    assert len(staged) == len(buckets)
    for got, original in zip(staged, buckets):
        assert got is not original and got.object_id == original.object_id and got.bytesio_data == original.bytesio_data
        assert got.tensor_data[0][1].device == torch.device("cpu")
        assert torch.equal(got.tensor_data[0][1], original.tensor_data[0][1])
    with mock.patch("torch.cuda.is_available", return_value=True), mock.patch("torch.cuda.synchronize") as sync:
        MemoryStorageWriter.stage_write_data_buckets(cid, buckets, non_blocking=True)
        sync.assert_called_once()                            # the one wait that ends the blocking part of a save
        MemoryStorageWriter.stage_write_data_buckets(cid, buckets, non_blocking=False)
        sync.assert_called_once()


def test_stage_waits_for_the_packs_of_placeholders_instead_of_the_device():
    """Entries that stand for an image already being packed offer ``wait_until_packed``; when all of them do, those
    waits (one per image) replace the device-wide synchronize.  (Not in the reference: its entries are tensors.)"""

    class Placeholder:
        def __init__(self, staged):
            self.staged = staged

        def to(self, **kwargs):
            return self

        def wait_until_packed(self):
            self.staged.append("waited")

    cid = CheckpointContainerId("/test_checkpoint")
    image_a, image_b = [], []
    buckets = _buckets(cid, count=2)
    buckets[0].tensor_data = [(buckets[0].tensor_data[0][0], Placeholder(image_a)), (mock.MagicMock(), Placeholder(image_a))]
    buckets[1].tensor_data = [(buckets[1].tensor_data[0][0], Placeholder(image_b))]
    with mock.patch("torch.cuda.is_available", return_value=True), mock.patch("torch.cuda.synchronize") as sync:
        staged = MemoryStorageWriter.stage_write_data_buckets(cid, buckets, non_blocking=True)
        sync.assert_not_called()
        assert image_a == ["waited"] and image_b == ["waited"]          # once per image, not once per entry
        assert staged[0].tensor_data[0][1] is buckets[0].tensor_data[0][1]
        buckets[1].tensor_data.append((mock.MagicMock(), torch.tensor([1])))  # one real tensor among them
        MemoryStorageWriter.stage_write_data_buckets(cid, buckets, non_blocking=True)
        sync.assert_called_once()
        assert image_a == ["waited"] and image_b == ["waited"]


# ---- write_staged_data_buckets / write_data (:615-888) --------------------------------------------------------------------
@pytest.mark.parametrize("thread_count", [1, 4, 8])
def test_write_staged_data_buckets(saver, mp_manager_future, thread_count):
    w = MemoryStorageWriter(checkpoint_saver=saver, mp_manager_future=mp_manager_future, thread_count=thread_count)
    cid = CheckpointContainerId("/test_checkpoint_explicit_thread_count")
    w.reset(cid.data)
    staged = _buckets(cid)
    saver.write_data.return_value = expected = [_wr("a")]
    w.prepare_write_data_buckets(cid, SavePlan(items=[], storage_data=_StorageDataContext(prefix="__0_")), mock.MagicMock())
    future = w.write_staged_data_buckets(cid, staged, replicate_after_write=False)
    saver.write_data.assert_called_once_with(cid, write_buckets=staged, thread_count=thread_count, replicate_after_write=False)
    assert w._write_events_per_checkpoint_id[cid].is_set() and future.wait() == expected
    assert w.get_write_results(cid) == expected


def test_write_staged_data_buckets_failure_leaves_the_event_unset(writer, saver):
    cid = CheckpointContainerId("/test_checkpoint")
    writer.reset(cid.data)
    staged = _buckets(cid)
    saver.write_data.side_effect = RuntimeError("Saver write failed")
    writer.prepare_write_data_buckets(cid, SavePlan(items=[], storage_data=_StorageDataContext(prefix="__0_")), mock.MagicMock())
    with pytest.raises(RuntimeError, match="Saver write failed"):
        writer.write_staged_data_buckets(cid, staged, replicate_after_write=False)
    saver.write_data.assert_called_once_with(cid, write_buckets=staged, thread_count=1, replicate_after_write=False)
    assert not writer._write_events_per_checkpoint_id[cid].is_set()


def test_write_data_prepares_then_writes_with_replication_on(writer):
    cid = CheckpointContainerId("/test_checkpoint_write_data")
    writer.reset(cid.data)
    plan = SavePlan(items=_items(WriteItemType.TENSOR, WriteItemType.BYTE_IO), storage_data=_StorageDataContext(prefix="__0_"))
    planner, buckets, done = mock.MagicMock(), _buckets(cid), TorchFuture()
    done.set_result([_wr("a")])
    with mock.patch.object(writer, "prepare_write_data_buckets", return_value=buckets) as prepare, \
            mock.patch.object(writer, "write_staged_data_buckets", return_value=done) as write:
        assert writer.write_data(plan, planner).wait() == [_wr("a")]
        prepare.assert_called_once_with(cid, plan, planner)
        write.assert_called_once_with(cid, buckets, replicate_after_write=True)


def test_write_data_needs_a_prefixed_plan(writer, saver):
    writer.reset("/test_checkpoint_write_data_fail")
    plan = SavePlan(items=_items(WriteItemType.TENSOR))
    with pytest.raises(ValueError, match=PREFIX_ERROR):
        writer.write_data(plan, mock.MagicMock())
    with pytest.raises(ValueError, match=PREFIX_ERROR):
        writer.write_data(dataclasses.replace(plan, storage_data=_StorageDataContext(prefix="")), mock.MagicMock())
    saver.write_data.assert_not_called()


def _fork_and_wait(target, args):
    process = torch_mp.get_context("fork").Process(target=target, args=args)
    process.start()
    process.join(60)
    assert process.exitcode == 0


def test_results_written_in_another_process_are_seen_here(writer, saver):
    cid = CheckpointContainerId("/test_write_data_multiprocess")
    writer.reset(cid.data)
    saver.write_data.return_value = expected = [_wr("a"), _wr("b", 20)]
    plan = writer.prepare_global_plan([SavePlan(items=_items(WriteItemType.TENSOR, WriteItemType.BYTE_IO))])[0]
    _fork_and_wait(writer.write_data, (plan, mock.MagicMock()))
    assert writer.get_write_results(cid) == expected
    cid2 = CheckpointContainerId("/test_write_staged_multiprocess")
    writer.reset(cid2.data)
    writer.prepare_write_data_buckets(cid2, plan, mock.MagicMock())
    _fork_and_wait(writer.write_staged_data_buckets, (cid2, _buckets(cid2), False))
    assert writer.get_write_results(cid2) == expected


# ---- finish / finish_checkpoint (:890-1085, :1352-1411) --------------------------------------------------------------------
@pytest.mark.parametrize("results, expected", [
    ([[_wr("a")], [_wr("b", 20)]], {IDX("a"): "data_a", IDX("b"): "data_b"}),
    ([], {}),
    ([[_wr("a")], []], {IDX("a"): "data_a"}),
    ([[WriteResult(IDX("a"), 10, "data_a1"), WriteResult(IDX("a"), 20, "data_a2")]], {IDX("a"): "data_a2"}),
], ids=["two-ranks", "none", "one-empty", "duplicate-index-last-wins"])
def test_finish_fills_the_metadata_and_writes_it(writer, saver, results, expected):
    writer.reset("/test_checkpoint_finish")
    metadata = Metadata(state_dict_metadata={})
    meta = writer.storage_meta()
    writer.finish(metadata, results)
    assert metadata.storage_data == expected and metadata.storage_meta == meta
    saver.write_metadata.assert_called_once_with(writer._current_checkpoint_id, metadata)


def test_finish_uses_its_argument_and_drops_the_stored_results(writer, saver):
    cid = CheckpointContainerId("/test_finish_uses_arg")
    writer.reset(cid.data)
    _signal(writer, cid, [_wr("a")])
    metadata = Metadata(state_dict_metadata={})
    writer.finish(metadata, [[_wr("b", 20)]])
    assert metadata.storage_data == {IDX("b"): "data_b"}
    assert writer.get_write_results(cid) is None              # consumed
    saver.write_metadata.side_effect = RuntimeError("Metadata write failed")
    with pytest.raises(RuntimeError, match="Metadata write failed"):
        writer.finish(Metadata(state_dict_metadata={}), [])


def test_finish_checkpoint_with_an_explicit_id(writer, saver):
    cid = CheckpointContainerId("/test_checkpoint_finish")
    writer.reset(cid.data)
    writer._write_results_per_checkpoint_id[cid] = [WriteResult(IDX("dummy"), 0, "")]
    metadata = Metadata(state_dict_metadata={})
    writer.finish_checkpoint(cid, metadata, [[_wr("a")], [_wr("b", 20)]])
    assert metadata.storage_data == {IDX("a"): "data_a", IDX("b"): "data_b"} and metadata.storage_meta == writer.storage_meta()
    saver.write_metadata.assert_called_once_with(cid, metadata)
    assert cid not in writer._write_results_per_checkpoint_id
    writer.finish_checkpoint(cid, Metadata(state_dict_metadata={}), [])   # nothing stored: still fine
    assert cid not in writer._write_results_per_checkpoint_id


def test_finish_checkpoint_failures_keep_the_stored_results(writer, saver):
    cid = CheckpointContainerId("/test_checkpoint_finish_inner_none")
    writer.reset(cid.data)
    writer._write_results_per_checkpoint_id[cid] = []
    with pytest.raises(RuntimeError, match=re.escape("finish: write results[1] is None!")):
        writer.finish_checkpoint(cid, Metadata(state_dict_metadata={}), [[_wr("a")], None, []])
    saver.write_metadata.assert_not_called()
    assert cid in writer._write_results_per_checkpoint_id
    saver.write_metadata.side_effect = RuntimeError("Metadata write failed")
    with pytest.raises(RuntimeError, match="Metadata write failed"):
        writer.finish_checkpoint(cid, Metadata(state_dict_metadata={}), [])
    assert cid in writer._write_results_per_checkpoint_id


# ---- results per checkpoint id (:1087-1350, :1499-1564) ---------------------------------------------------------------------
def test_results_are_kept_per_checkpoint_id(writer, saver):
    cid1, cid2 = CheckpointContainerId("/test_checkpoint_diff1"), CheckpointContainerId("/test_checkpoint_diff2")
    writer.reset(cid1.data)
    plan = writer.prepare_global_plan([SavePlan(items=_items(WriteItemType.TENSOR, WriteItemType.BYTE_IO))])[0]
    saver.write_data.return_value = [_wr("a")]
    writer.write_data(plan, mock.MagicMock()).wait()
    saver.write_data.assert_called_once_with(cid1, write_buckets=saver.prepare_write_data.return_value, thread_count=1,
                                             replicate_after_write=True)
    assert writer.get_write_results(cid1) == [_wr("a")]
    saver.write_data.return_value = [_wr("b", 20)]
    writer.write_data(plan, mock.MagicMock()).wait()
    assert writer.get_write_results(cid1) == [_wr("b", 20)]   # a second write of the same id replaces the first
    writer.reset(cid2.data)                                    # reset keeps what other ids stored
    saver.write_data.return_value = []
    writer.write_data(plan, mock.MagicMock()).wait()
    assert writer.get_write_results(cid1) == [_wr("b", 20)] and writer.get_write_results(cid2) == []
    assert writer._current_checkpoint_id == cid2


def test_get_write_results_hands_out_copies_and_rejects_unknown_ids(writer):
    cid = CheckpointContainerId("/test_get_copy")
    writer.reset(cid.data)
    _signal(writer, cid, [_wr("a")])
    got = writer.get_write_results(cid)
    got.append(_wr("b", 20))
    assert writer.get_write_results(cid) == [_wr("a")]
    writer.reset("/non_existent_id")
    with pytest.raises(KeyError):
        writer.get_write_results(CheckpointContainerId("/non_existent_id"))


def test_get_write_results_waits_for_the_write(writer, saver):
    cid = CheckpointContainerId("/test_get_write_results_wait")
    writer.reset(cid.data)
    writer._write_events_per_checkpoint_id[cid] = writer._main_process_torchmp_manager_future.result().Event()

    def finish_later():
        time.sleep(0.3)
        writer._write_results_per_checkpoint_id[cid] = [_wr("a")]
        writer._write_events_per_checkpoint_id[cid].set()

    thread = threading.Thread(target=finish_later)
    thread.start()
    assert writer.get_write_results(cid) == [_wr("a")]
    thread.join()
    late = CheckpointContainerId("/test_get_write_results_timeout")
    writer.reset(late.data)
    writer._write_events_per_checkpoint_id[late] = writer._main_process_torchmp_manager_future.result().Event()
    message = ("Event was never set for checkpoint_id '%s', meaning we cannot confirm that the write has "
               "completed, and its results are available." % late)
    with pytest.raises(RuntimeError, match=re.escape(message)):
        writer.get_write_results(late, wait_timeout_sec=0.2)
    saver.write_data.assert_not_called()


def test_a_failed_write_is_never_signalled(writer, saver):
    cid = CheckpointContainerId("/test_checkpoint_exc")
    writer.reset(cid.data)
    plan = writer.prepare_global_plan([SavePlan(items=_items(WriteItemType.TENSOR, WriteItemType.BYTE_IO))])[0]
    saver.write_data.side_effect = RuntimeError("Saver failed")
    with pytest.raises(RuntimeError, match="Saver failed"):
        writer.write_data(plan, mock.MagicMock()).wait()
    with pytest.raises(RuntimeError, match=re.escape("Event was never set for checkpoint_id '%s'" % cid)):
        writer.get_write_results(cid, wait_timeout_sec=0)


# ---- replication and pickling (:1443-1497, :1566-1596) ------------------------------------------------------------------------
def test_replicate_written_objects_collects_every_future(writer, saver):
    object_ids = {CheckpointObjectId.from_container(CheckpointContainerId("/c1"), "obj1"),
                  CheckpointObjectId.from_container(CheckpointContainerId("/c1"), "obj2"),
                  CheckpointObjectId.from_container(CheckpointContainerId("/c2"), "obj3")}
    futures = [concurrent.futures.Future() for _ in range(6)]
    saver.async_replicate_object.side_effect = [futures[0:2], futures[2:5], futures[5:6]]
    assert writer.replicate_written_objects(object_ids) == futures
    assert {c.args[0] for c in saver.async_replicate_object.call_args_list} == object_ids
    assert saver.async_replicate_object.call_count == 3


def test_pickling_leaves_the_manager_and_the_replication_manager_behind(mp_manager_future):
    saver = DefaultMLFlashpointCheckpointSaver(
        global_rank_getter=_zero, local_rank_getter=_zero, global_barrier_func=_none,
        ckpt_obj_manager=DummyObjectManager(), replication_manager=DummyReplicationManager())
    clone = pickle.loads(pickle.dumps(MemoryStorageWriter(checkpoint_saver=saver, mp_manager_future=mp_manager_future)))
    assert clone._main_process_torchmp_manager_future is None
    assert isinstance(clone._checkpoint_saver, DefaultMLFlashpointCheckpointSaver)
    assert clone._checkpoint_saver._initial_buffer_size_bytes == saver._initial_buffer_size_bytes
    assert isinstance(clone._checkpoint_saver._chkpt_obj_manager, DummyObjectManager)
    assert clone._checkpoint_saver._replication_manager is None
