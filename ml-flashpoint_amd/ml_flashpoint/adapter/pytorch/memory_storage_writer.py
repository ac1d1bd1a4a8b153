"""DCP ``StorageWriter`` whose storage is a set of checkpoint buffer objects filled by a saver plug-in.

The public surface is the one the reference's adapter has (src/ml_flashpoint/adapter/pytorch/memory_storage_writer.py
:53-401), because DCP, the three-call saver (``custom_state_dict_saver``) and async frameworks call it:

* classic DCP:  ``reset -> prepare_local_plan -> prepare_global_plan -> write_data -> finish``
* split form:   ``prepare_write_data_buckets`` (training process; with the gfx950 saver this is where the image is
                packed) -> ``stage_write_data_buckets`` (static; ends the blocking part) ->
                ``write_staged_data_buckets`` (possibly another process) -> ``get_write_results`` ->
                ``finish_checkpoint``

What crosses the process boundary in the split form is kept in one place, ``_WriteLedger``: per checkpoint id a
completion event and the list of write results, both held by a ``torch.multiprocessing`` manager.
"""

from __future__ import annotations

import concurrent.futures
import dataclasses
import logging
import os
import pickle
import threading
import time

import torch
from torch.distributed.checkpoint import staging
from torch.distributed.checkpoint.metadata import STATE_DICT_TYPE, Metadata, StorageMeta
from torch.distributed.checkpoint.planner import SavePlan, SavePlanner
from torch.distributed.checkpoint.storage import StorageWriter, WriteResult
from torch.futures import Future as TorchFuture
from typing_extensions import override

from ml_flashpoint.core import utils
from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId, CheckpointObjectId
from ml_flashpoint.core.checkpoint_saver import MLFlashpointCheckpointSaver, ObjectWriteBucket
from ml_flashpoint.core.hfid import generate_hfid
from ml_flashpoint.core.mlf_logging import get_logger

_LOGGER = get_logger(__name__)
_timed = utils.log_execution_time

_NOT_RESET = "MemoryStorageWriter has not been reset. Call reset() before using this method."
_BAD_PLAN = (
    "SavePlan.storage_data is not a valid _StorageDataContext or prefix is empty. "
    "This is likely because prepare_global_plan was not called on this SavePlan."
)
_NEVER_SIGNALLED = (
    "Event was never set for checkpoint_id '%s', meaning we cannot confirm that the write "
    "has completed, and its results are available."
)
_MISSING_RANK_RESULTS = (
    "finish: write results[%d] is None! This suggests an error in producing or gathering "
    "the write_results list from that local rank (%d)."
)


@dataclasses.dataclass
class _StorageDataContext:
    """What ``prepare_global_plan`` attaches to each rank's plan: the prefix of that plan's object names."""

    prefix: str


def _pack_waits(write_buckets: list[ObjectWriteBucket]):
    """One ``wait_until_packed`` callable per packed image if every tensor entry of every bucket is a placeholder
    that has one, else None.  Waiting for the events behind the packs is enough to know that the live tensors may be
    overwritten, and unlike a device-wide synchronize it does not also wait for an earlier checkpoint that is
    still crossing the host link."""
    per_image = {}
    for bucket in write_buckets:
        for _, entry in bucket.tensor_data:
            wait = getattr(entry, "wait_until_packed", None)
            if wait is None:
                return None
            per_image.setdefault(id(getattr(entry, "staged", entry)), wait)
    return list(per_image.values())


class _WriteLedger:
    """Completion events and write results per checkpoint id, shared between the process that prepares a save and
    the one that writes it.  Empty until ``open`` is given a manager; a ledger that travelled to another process
    keeps working through its proxies but cannot create new events there."""

    def __init__(self):
        self.events = None   # manager dict: CheckpointContainerId -> manager Event
        self.results = None  # manager dict: CheckpointContainerId -> list[WriteResult]

    def open(self, manager) -> None:
        self.events, self.results = manager.dict(), manager.dict()

    def expect(self, checkpoint_id: CheckpointContainerId, manager_future) -> None:
        if checkpoint_id not in self.events:
            self.events[checkpoint_id] = manager_future.result().Event()

    def publish(self, checkpoint_id: CheckpointContainerId, results: list[WriteResult]) -> None:
        self.results[checkpoint_id] = results
        self.events[checkpoint_id].set()

    def wait(self, checkpoint_id: CheckpointContainerId, timeout_s: float) -> bool:
        return self.events[checkpoint_id].wait(timeout=timeout_s)


_STORAGE_META_KEY = b"\x8c\x0cstorage_meta"  # SHORT_BINUNICODE, length 12: the field's name as a key of the state dict


def _last_frame(pickled: bytes) -> int | None:
    """Offset of the FRAME opcode (protocol 4: 0x95 + eight bytes of length) that runs to the end of ``pickled``."""
    at = len(pickled)
    while True:
        at = pickled.rfind(b"\x95", 0, at)
        if at < 0:
            return None
        if at + 9 <= len(pickled) and int.from_bytes(pickled[at + 1 : at + 9], "little") == len(pickled) - at - 9:
            return at


def repickled_with_storage_meta(pickled: bytes, metadata: Metadata, old: StorageMeta, new: StorageMeta) -> bytes | None:
    """``pickle.dumps`` of a metadata object that differs from the one ``pickled`` was made from in ``storage_meta``
    only (``old`` there, ``new`` now) - without pickling its tens of thousands of entries again - or None where that
    cannot be done safely.

    A dataclass is pickled field by field in declaration order, and ``storage_meta`` comes after the two big
    dictionaries, so everything up to its key is the same stream of opcodes for both objects.  What follows the key
    is taken from the pickle of a stand-in with empty dictionaries, once with ``old`` and once with ``new``.  A tail
    may only be moved from one pickle into another if it does not depend on how many objects were memoized before it
    (back-references carry explicit memo numbers).  For ``old`` that is shown by the stand-in's tail being byte for
    byte the tail of ``pickled``; for ``new`` by a second stand-in, with some hundred more memo entries in front,
    giving the same tail.  Anything else - a tail that refers back into the dictionaries or to an object of its own,
    another field order - ends in None, never in wrong bytes.  The length of the last frame is corrected."""
    try:
        stand_in = dataclasses.replace(metadata, state_dict_metadata={}, planner_data=None, storage_data={})
        shifted = dataclasses.replace(stand_in, state_dict_metadata={f"k{i}": i for i in range(300)})
        tail_old, tail_new, tail_new_shifted = (
            pickle.dumps(dataclasses.replace(base, storage_meta=meta), protocol=pickle.DEFAULT_PROTOCOL)
            for base, meta in ((stand_in, old), (stand_in, new), (shifted, new)))
    except Exception:
        return None
    cut, cut_old, cut_new, cut_shifted = (b.rfind(_STORAGE_META_KEY) for b in (pickled, tail_old, tail_new, tail_new_shifted))
    if min(cut, cut_old, cut_new, cut_shifted) < 0 or pickled[cut:] != tail_old[cut_old:] \
            or tail_new[cut_new:] != tail_new_shifted[cut_shifted:]:
        return None
    frame = _last_frame(pickled)
    if frame is None or frame + 9 > cut:
        return None  # unframed, or the tail is spread over two frames
    tail = tail_new[cut_new:]
    length = len(pickled) - frame - 9 + len(tail) - (len(pickled) - cut)
    return b"".join((pickled[:frame], b"\x95", length.to_bytes(8, "little"), pickled[frame + 9 : cut], tail))


class _EarlyMetadata:
    """The checkpoint's metadata object pickled while its data is still on the way to the buffer.

    Where every item ends up is decided when the object is laid out, long before the last byte is written, so the
    metadata object - whose pickling takes 150 ms for 20 000 tensors - need not wait for the write.  This rank's
    part of it is predicted from the layout; with several ranks the others' parts are taken to be what they were in
    the previous save (the same plan puts the same items at the same offsets of objects of the same names), which
    the rank that writes the metadata object saw when it finished that save.  ``finish_checkpoint`` uses the bytes
    only if they describe exactly what all ranks then reported; otherwise it pickles again, as without this.

    ``before``: ``(metadata, where, storage_meta, bytes)`` of the last metadata object this process wrote.  When it
    was the same metadata object with every item in the same place - the steady state of a run that keeps its DCP
    plan - the new bytes are the old ones with the ``storage_meta`` part exchanged
    (``repickled_with_storage_meta``), which takes a millisecond instead of the pickling."""

    def __init__(self, checkpoint_id, metadata: Metadata, where: dict, storage_meta, before=None):
        self.checkpoint_id, self.metadata, self.where, self.storage_meta = checkpoint_id, metadata, where, storage_meta
        self.payload: bytes | None = None
        self.respliced = False
        self.predicted, self.others_as_before = None, False  # what `where` was made from (set by whoever made it)
        self._before = before
        self._thread = threading.Thread(target=self._run, name="mlf-early-metadata", daemon=True)
        self._thread.start()

    def _run(self):
        try:
            with utils.gc_paused():
                before, self._before = self._before, None
                if before is not None and before[0] is self.metadata and (before[1] is self.where or before[1] == self.where):
                    self.payload = repickled_with_storage_meta(before[3], self.metadata, before[2], self.storage_meta)
                    self.respliced = self.payload is not None
                if self.payload is None:
                    filled = dataclasses.replace(self.metadata, storage_data=self.where, storage_meta=self.storage_meta)
                    self.payload = pickle.dumps(filled)
        except Exception:  # the ordinary path takes over
            _LOGGER.warning("could not pickle the metadata object ahead of time", exc_info=True)

    def result_for(self, checkpoint_id, metadata: Metadata, where: dict, storage_meta) -> bytes | None:
        self._thread.join()
        same = (self.payload is not None and checkpoint_id == self.checkpoint_id and metadata is self.metadata
                and storage_meta == self.storage_meta and where == self.where)
        return self.payload if same else None


class MemoryStorageWriter(StorageWriter, staging.BlockingAsyncStager):
    def __init__(
        self,
        checkpoint_saver: MLFlashpointCheckpointSaver,
        mp_manager_future: concurrent.futures.Future,
        thread_count: int = 1,
    ):
        """``mp_manager_future`` resolves to a ``torch.multiprocessing`` manager (best created with the 'spawn'
        context) of the main process; it is consulted lazily and never pickled.  ``thread_count`` is both the
        number of objects a save is split into and the saver's writer-thread count; values below 1 mean 1."""
        super().__init__()
        if thread_count < 1:
            _LOGGER.warning("thread_count must be >= 1, but was %d. Setting to 1.", thread_count)
        self._thread_count = max(thread_count, 1)
        self._checkpoint_saver = checkpoint_saver
        self._main_process_torchmp_manager_future = mp_manager_future
        self._ledger = _WriteLedger()
        self._current_checkpoint_id: CheckpointContainerId | None = None
        self._current_save_id: str | None = None
        self._expected_metadata: Metadata | None = None  # see expect_metadata
        self._others_as_before = False
        self._early_metadata: _EarlyMetadata | None = None
        self.early_metadata_used = False  # the last finish_checkpoint wrote bytes that were pickled ahead of time
        self.early_metadata_respliced = False  # ... and those were the previous save's with storage_meta exchanged

    # the ledger's two dicts under the names other code (and the reference's tests) know them by
    @property
    def _write_events_per_checkpoint_id(self):
        return self._ledger.events

    @_write_events_per_checkpoint_id.setter
    def _write_events_per_checkpoint_id(self, value):
        self._ledger.events = value

    @property
    def _write_results_per_checkpoint_id(self):
        return self._ledger.results

    @_write_results_per_checkpoint_id.setter
    def _write_results_per_checkpoint_id(self, value):
        self._ledger.results = value

    def __getstate__(self):
        left_behind = ("_main_process_torchmp_manager_future", "_expected_metadata", "_early_metadata")  # (re-set below)
        return {k: v for k, v in self.__dict__.items() if k not in left_behind}

    def __setstate__(self, state):
        self.__dict__.update(state, _main_process_torchmp_manager_future=None, _expected_metadata=None,
                             _early_metadata=None)
        self._others_as_before = False

    def expect_metadata(self, metadata: Metadata | None, others_as_before: bool | None = None) -> None:
        """Tells the writer which metadata object ``finish_checkpoint`` is going to be called with, in the process
        that is going to call it: the writer may then pickle it while the data is still being written (see
        ``_EarlyMetadata``).  ``others_as_before``: other ranks contribute write results too, and they are predicted
        to be what the previous ``finish_checkpoint`` of this writer's saver saw (default: whether the process group
        has more than one rank); no prediction, and no early pickling, on the first save.  Optional; without it, or
        in a process that received the writer by pickling, nothing changes."""
        self._expected_metadata = metadata
        if others_as_before is None:
            dist = torch.distributed
            others_as_before = dist.is_available() and dist.is_initialized() and dist.get_world_size() > 1
        self._others_as_before = bool(others_as_before)

    # ---- identity of the save in progress ------------------------------------------------------------------------
    def _require_reset(self) -> CheckpointContainerId:
        if self._current_checkpoint_id is None:
            raise ValueError(_NOT_RESET)
        return self._current_checkpoint_id

    _check_checkpoint_id = _require_reset

    @property
    def current_checkpoint_id(self) -> CheckpointContainerId | None:
        return self._current_checkpoint_id

    @property
    def path(self) -> str | None:
        current = self._current_checkpoint_id
        return current.data if current is not None else None

    @property
    def checkpoint_saver(self) -> MLFlashpointCheckpointSaver:
        return self._checkpoint_saver

    @override
    def reset(self, checkpoint_id: str | os.PathLike | None = None) -> None:
        """Starts a save: new id, new save id.  Entries of earlier ids stay in the ledger."""
        self._current_checkpoint_id = CheckpointContainerId(checkpoint_id)
        self._current_save_id = generate_hfid("memwritersave")
        have_manager = self._main_process_torchmp_manager_future is not None
        if self._ledger.events is None and have_manager:
            self._ledger.open(self._main_process_torchmp_manager_future.result())

    def storage_meta(self) -> StorageMeta | None:
        return StorageMeta(checkpoint_id=self._require_reset().data, save_id=self._current_save_id)

    @classmethod
    @override
    def validate_checkpoint_id(cls, checkpoint_id: str | os.PathLike) -> bool:
        try:
            CheckpointContainerId(checkpoint_id)
        except Exception as e:
            _LOGGER.warning("Unable to validate checkpoint_id: %s, %s", checkpoint_id, e)
            return False
        return True

    # ---- planning hooks --------------------------------------------------------------------------------------------
    @override
    def set_up_storage_writer(self, is_coordinator: bool) -> None:
        """Nothing to set up: objects are created when they are written."""

    @override
    @_timed(logger=_LOGGER, name="prepare_local_plan")
    def prepare_local_plan(self, plan: SavePlan) -> SavePlan:
        self._checkpoint_saver.initialize_checkpoint(self._require_reset())  # marks the checkpoint as unfinished
        return plan

    @override
    @_timed(logger=_LOGGER, name="prepare_global_plan")
    def prepare_global_plan(self, plans: list[SavePlan]) -> list[SavePlan]:
        numbered = []
        for rank_position, plan in enumerate(plans):
            context = _StorageDataContext(prefix=f"__{rank_position}_")
            numbered.append(dataclasses.replace(plan, storage_data=context))
        return numbered

    # ---- the write, whole or in three parts ----------------------------------------------------------------------
    @override
    @_timed(logger=_LOGGER, name="stage", level=logging.INFO)
    def stage(self, state_dict: STATE_DICT_TYPE) -> STATE_DICT_TYPE:
        return super().stage(state_dict)

    @override
    @_timed(logger=_LOGGER, name="write_data", level=logging.INFO)
    def write_data(self, plan: SavePlan, planner: SavePlanner) -> TorchFuture[list[WriteResult]]:
        checkpoint_id = self._require_reset()
        context = plan.storage_data
        if not (isinstance(context, _StorageDataContext) and context.prefix):
            raise ValueError(_BAD_PLAN)
        write_buckets = self.prepare_write_data_buckets(checkpoint_id, plan, planner)
        return self.write_staged_data_buckets(checkpoint_id, write_buckets, replicate_after_write=True)

    @_timed(logger=_LOGGER, name="prepare_write_data_buckets")
    def prepare_write_data_buckets(
        self, checkpoint_id: CheckpointContainerId, plan: SavePlan, planner: SavePlanner
    ) -> list[ObjectWriteBucket]:
        """Registers the completion event of ``checkpoint_id`` (only the main process can create one) and lets the
        saver turn the plan into one bucket per object."""
        self._ledger.expect(checkpoint_id, self._main_process_torchmp_manager_future)
        return self._checkpoint_saver.prepare_write_data(
            checkpoint_id, plan.items, planner, plan.storage_data.prefix, bucket_count=self._thread_count
        )

    @staticmethod
    @_timed(logger=_LOGGER, name="stage_write_data_buckets", level=logging.INFO)
    @utils.gc_paused()
    def stage_write_data_buckets(
        _: CheckpointContainerId, write_buckets: list[ObjectWriteBucket], non_blocking: bool = True
    ):
        """Returns buckets that no longer depend on live training tensors.  Static, because async frameworks call
        it on the class.  A bucket prepared by the gfx950 saver holds placeholders for an image that is already
        being packed in HBM: their ``.to()`` is the identity, and the device synchronize below is then the moment
        the training stream may overwrite its tensors again."""

        def on_host(pairs):
            return [(item, tensor.to(device="cpu", non_blocking=non_blocking)) for item, tensor in pairs]

        staged = [dataclasses.replace(bucket, tensor_data=on_host(bucket.tensor_data)) for bucket in write_buckets]
        if torch.cuda.is_available():
            waits = _pack_waits(write_buckets)
            if waits is not None:
                # placeholders: whether the caller asked for blocking copies or not, the live tensors may be
                # overwritten once this returns, so the packs that read them must have finished
                for wait in waits:
                    wait()
            elif non_blocking:
                torch.cuda.synchronize()
        return staged

    @_timed(logger=_LOGGER, name="write_staged_write_buckets", level=logging.INFO)
    @utils.gc_paused()
    def write_staged_data_buckets(
        self,
        checkpoint_id: CheckpointContainerId,
        staged_write_buckets: list[ObjectWriteBucket],
        replicate_after_write: bool,
    ) -> TorchFuture[list[WriteResult]]:
        """Synchronous write of prepared buckets; publishes the results for ``get_write_results`` (in whichever
        process that is called) and also returns them in a completed future.  A failing write publishes nothing."""
        began = time.perf_counter()
        self._start_early_metadata(checkpoint_id, staged_write_buckets)
        outcome = self._checkpoint_saver.write_data(
            checkpoint_id,
            write_buckets=staged_write_buckets,
            thread_count=self._thread_count,
            replicate_after_write=replicate_after_write,
        )
        utils.log_rate(_LOGGER, "Written", sum(r.size_in_bytes for r in outcome), time.perf_counter() - began,
                       len(staged_write_buckets), "buckets")
        self._ledger.publish(checkpoint_id, outcome)
        done: TorchFuture = TorchFuture()
        done.set_result(outcome)
        return done

    def _start_early_metadata(self, checkpoint_id, buckets) -> None:
        self._early_metadata = None
        metadata, predict = self._expected_metadata, getattr(self._checkpoint_saver, "predict_write_results", None)
        if metadata is None or predict is None or self._current_checkpoint_id != checkpoint_id:
            return
        try:
            predicted = predict(buckets)
        except Exception:
            _LOGGER.warning("could not predict the write results", exc_info=True)
            return
        if predicted is None:
            return
        others = None
        if self._others_as_before:
            others = getattr(self._checkpoint_saver, "last_write_locations", None)
            if not others:
                return  # nothing to go by yet
        # (metadata, where, storage_meta, bytes, the predicted results and the other ranks' part that `where` was
        # made from) of the last metadata object written: a saver that keeps its plans predicts the same result
        # objects again, and then `where` need not be built anew either
        before = getattr(self._checkpoint_saver, "last_metadata_pickle", None)
        if before is not None and before[5] is others and len(before[4]) == len(predicted) \
                and all(a is b for a, b in zip(before[4], predicted)):
            where = before[1]
        else:
            where = {result.index: result.storage_data for result in predicted}
            if others is not None:
                where = {**others, **where}
        self._early_metadata = _EarlyMetadata(checkpoint_id, metadata, where, self.storage_meta(), before)
        self._early_metadata.predicted, self._early_metadata.others_as_before = predicted, others is not None

    @_timed(logger=_LOGGER, name="get_write_results")
    def get_write_results(
        self, checkpoint_id: CheckpointContainerId, wait_timeout_sec: float = 15.0
    ) -> list[WriteResult]:
        """Results of the write of ``checkpoint_id`` once it has been signalled: ``KeyError`` when no write was ever
        prepared for that id, ``RuntimeError`` when the signal does not come within ``wait_timeout_sec``."""
        if self._ledger.wait(checkpoint_id, wait_timeout_sec):
            return self._ledger.results.get(checkpoint_id)
        complaint = _NEVER_SIGNALLED % checkpoint_id
        _LOGGER.error(complaint)
        raise RuntimeError(complaint)

    def replicate_written_objects(self, object_ids: set[CheckpointObjectId]) -> list[concurrent.futures.Future]:
        replicate = self._checkpoint_saver.async_replicate_object
        return [future for object_id in object_ids for future in replicate(object_id)]

    # ---- completion --------------------------------------------------------------------------------------------------
    @override
    @_timed(logger=_LOGGER, name="finish")
    def finish(self, metadata: Metadata, results: list[list[WriteResult]]) -> None:
        self.finish_checkpoint(self._require_reset(), metadata, results)

    @_timed(logger=_LOGGER, name="finish_checkpoint", level=logging.INFO)
    @utils.gc_paused()
    def finish_checkpoint(
        self, checkpoint_id: CheckpointContainerId, metadata: Metadata, results: list[list[WriteResult]]
    ) -> None:
        """``finish`` for an explicit id (saves of several ids may overlap): records where every item went, writes
        the metadata object, then forgets the stored results of that id.  Nothing is forgotten on failure."""
        where = {}
        for position, rank_results in enumerate(results):
            if rank_results is None:
                complaint = _MISSING_RANK_RESULTS % (position, position)
                _LOGGER.error(complaint)
                raise RuntimeError(complaint)
            where.update((result.index, result.storage_data) for result in rank_results)  # a repeated index: last wins
        metadata.storage_data, metadata.storage_meta = where, self.storage_meta()
        early, self._early_metadata = self._early_metadata, None
        ready = early.result_for(checkpoint_id, metadata, where, metadata.storage_meta) if early is not None else None
        write_bytes = getattr(self._checkpoint_saver, "write_metadata_bytes", None)
        self.early_metadata_used = ready is not None and write_bytes is not None
        self.early_metadata_respliced = self.early_metadata_used and early.respliced
        if self.early_metadata_used:
            write_bytes(checkpoint_id, ready)  # pickled while the data was being written: same bytes, no wait
        else:
            self._checkpoint_saver.write_metadata(checkpoint_id, metadata)
        try:  # what the next save's prediction of the other ranks' results goes by (writers come and go, savers stay)
            if self.early_metadata_used and hasattr(self._checkpoint_saver, "last_metadata_pickle"):
                # the early bytes were right, so early.where says what `where` says: kept as the record of where
                # everything went, it is also the very dict the next save's prediction starts from, and that save
                # can tell by identity that nothing has moved
                where = early.where
                self._checkpoint_saver.last_metadata_pickle = (
                    metadata, where, metadata.storage_meta, ready, early.predicted, where if early.others_as_before else None)
            self._checkpoint_saver.last_write_locations = where
        except AttributeError:
            pass
        if self._ledger.results is not None:
            self._ledger.results.pop(checkpoint_id, None)
