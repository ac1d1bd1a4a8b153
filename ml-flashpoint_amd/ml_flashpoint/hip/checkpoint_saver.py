"""gfx950 implementation of the saver plug-in interface.

Where the reference's default saver copies tensor by tensor (``Tensor.to("cpu")``, then header +
``frombuffer().copy_()`` into the mapping; src/ml_flashpoint/core/checkpoint_saver.py:347-360,622-707,764-800),
this saver

1. lays the whole object out on the host (same record format, same offsets),
2. packs every device tensor and every header into a byte-exact *image* of the object's data section in HBM with
   one batched kernel launch (``prepare_write_data`` - the training stream is free again once that kernel ends),
3. streams the image into the mapped buffer file through pinned slots (``write_data``),

so the bytes on tmpfs are identical to the reference's while the blocking part shrinks to an HBM-to-HBM copy.
Host-only duties (dirty marker, metadata file, finalize + removal of older steps) are kept as the reference has
them (checkpoint_saver.py:340-343,533-619,709-762).
"""

import concurrent.futures
import contextlib
import ctypes
import dataclasses
import logging
import os
import pickle
import subprocess
import sys
import tempfile
import threading
import time
import uuid
import weakref
from typing import Callable, Optional, Union

import numpy as np
import torch
from torch.distributed.checkpoint import metadata as torchdistmeta
from torch.distributed.checkpoint.filesystem import _split_by_size_and_type, _StorageInfo
from torch.distributed.checkpoint.planner import WriteItem, WriteItemType
from torch.distributed.checkpoint.storage import WriteResult
from typing_extensions import override

from ml_flashpoint.checkpoint_object_manager.buffer_metadata import METADATA_SIZE
from ml_flashpoint.checkpoint_object_manager.checkpoint_object_manager import CheckpointObjectManager
from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId, CheckpointObjectId
from ml_flashpoint.core.checkpoint_saver import (
    _DEFAULT_OBJ_NAME_SUFFIX,
    DEFAULT_INITIAL_BUFFER_SIZE_BYTES,
    MLFlashpointCheckpointSaver,
    ObjectWriteBucket,
    WriteItemResolver,
)
from ml_flashpoint.core.defaults import DIRTY_MARKER_SUFFIX, CheckpointFormat, default_metadata_object_name
from ml_flashpoint.core.mlf_logging import get_logger
from ml_flashpoint.core.utils import gc_paused, log_execution_time
from ml_flashpoint.hip import _lib, integrity
from ml_flashpoint.hip import plan as hip_plan

_LOGGER = get_logger(__name__)

_STAGE_ALIGN = 64


@dataclasses.dataclass
class EngineConfig:
    """Shape of the pinned ring between HBM and the buffer file.  Small on purpose: while the ring stays in the
    host's caches, filling a slot and reading it back out cost no DRAM bandwidth (a ring of 256 MiB was measured a
    third slower on the restore side than one of 96 MiB)."""

    slot_bytes: int = 32 << 20
    n_slots: int = 3
    # host threads that move a slot to/from the buffer file; 0 = the CPUs this process may run on, at most 16
    # (reading a tmpfs file back at link speed takes ~12 of them, writing the mapping ~6)
    copy_threads: int = 0

    def resolved_copy_threads(self) -> int:
        if self.copy_threads > 0:
            return self.copy_threads
        try:
            cpus = len(os.sched_getaffinity(0))
        except (AttributeError, OSError):
            cpus = os.cpu_count() or 1
        return max(1, min(16, cpus))


# host-resident tensors of at least this many bytes go from host memory straight into the buffer; smaller ones ride
# in the image with the headers (one copy more, no extra pieces in the transfer)
_HOST_DIRECT_MIN_BYTES = 256 << 10

# when the allocator has no single block for an object's image, the image is held in pieces of about this size
_IMAGE_PIECE_BYTES = 8 << 30

# a window or piece of an image starts this many bytes (modulo) into its device buffer as into the image
_WINDOW_PAD = 4096
# the buffer that the windows of an image too large for HBM pass through: a quarter of the limit, at most this
_WINDOW_BUFFER_BYTES = 8 << 30
# ... in two halves that alternate (one packed while the other crosses the link) where a half is at least this large
_WINDOW_PAIR_MIN_BYTES = 64 << 10

_FUSED_VALUES_LOCK = threading.Lock()

_MAX_KEPT_PLANS = 64  # objects per save are few (one per writer thread); beyond this the oldest is rebuilt


class _KeptPlan:
    """Layout and device tables of one object, kept for the next save of the same tensors."""

    def __init__(self, key, layout: hip_plan.SaveLayout, plan: hip_plan.Plan, device: torch.device):
        self.key, self.plan, self.device = key, plan, device
        # the table has the device addresses and host tensors are looked up again by index: hold no tensors
        self.layout = dataclasses.replace(layout, device_tensors=[], host_tensors=[])
        self.blob = layout.blob
        # with checksums folded into the pack: the object of the last launch, until its values have been taken (a
        # plan holds the values of its last launch only)
        self.last_staged: Optional[weakref.ReferenceType] = None
        # (object name, the save's items, their WriteResults): a save planned from a kept DCP plan brings the very
        # same items again, and the layout is this one's, so the results are the same objects from save to save
        self.results: Optional[tuple] = None

    def refreshed_blob(self, tensors, blobs) -> Optional[bytes]:
        """The blob with the current bytes of its variable parts, or None if nothing changed since last time."""
        parts = self.layout.variable_parts
        if not parts:
            return None
        fresh = bytearray(self.blob)
        for offset, nbytes, kind, index in parts:
            data = hip_plan.host_tensor_bytes(tensors[index]) if kind == "tensor" else blobs[index]
            assert len(data) == nbytes
            fresh[offset : offset + nbytes] = data
        if fresh == self.blob:
            return None
        self.blob = bytes(fresh)
        return self.blob


class StagedObject:
    """Image of one checkpoint object in HBM, with the layout that produced it.

    With a background writer (``background_write=True``) the transfer into the buffer object starts as soon as the
    pack is enqueued and ``future`` resolves to the object's WriteResults.  Such an object may cross a process
    boundary: what arrives on the other side is a ``RemoteStagedObject`` that only waits for the transfer - the HIP
    context, the image and the buffer stay with the process that owns the GPU."""

    def __init__(self, layout: hip_plan.SaveLayout, plan: Optional[hip_plan.Plan], image: Optional[torch.Tensor],
                 device_index: int, stream: int, items: list):
        self.layout = layout
        self.plan = plan
        self.image = image
        self.device_index = device_index
        self.stream = stream
        self.items = items  # WriteItems in span order: tensors, then byte blobs
        self.consumed = False
        self.future: Optional[concurrent.futures.Future] = None
        self.done_marker: Optional[str] = None
        self.collected = False
        self.packed_event: Optional[torch.cuda.Event] = None  # recorded behind the pack on the producer's stream
        self.owns_plan = True  # False: the plan is kept by the saver for the next save
        self._landed = ctypes.c_uint64(0)  # kept current by the copy engine while the image crosses the link
        self.data_offset: Optional[int] = None  # position of the image's first byte in the object's data section
        # an image that is held in several device buffers: [(plan, buffer, first image byte, end)], in order
        self.pieces: Optional[list] = None
        self.fused_crcs = None  # chunk checksums out of the pack, once taken from the plan
        self.kept: Optional[_KeptPlan] = None  # the kept plan this object was packed with, if any
        self._results: Optional[tuple] = None  # (object name, WriteResults), once made

    def landed_bytes(self) -> int:
        """Leading bytes of the image that are in place in the buffer file (from byte 4096 + ``data_offset`` of the
        file on; ``data_offset`` is None until the transfer has begun).  Grows while the transfer runs: a sender
        that forwards the object to a replica can follow it instead of waiting for the whole object, which is
        when the reference starts (checkpoint_saver.py:700-707)."""
        return int(self._landed.value)

    def __reduce__(self):
        if self.future is None or self.done_marker is None:
            raise pickle.PicklingError(
                "a packed checkpoint image lives in this process's GPU memory and cannot be sent to another process; "
                "construct the saver with background_write=True so that this process writes it and the other one "
                "only waits for the result"
            )
        return (RemoteStagedObject, (self.done_marker,))


class RemoteStagedObject:
    """What a ``StagedObject`` becomes in another process: the path of the marker file through which the owning
    process reports the outcome (the pickled WriteResults, or the error text)."""

    def __init__(self, done_marker: str):
        self.done_marker = done_marker
        self.consumed = False

    def wait(self, timeout_s: float) -> list:
        deadline = time.monotonic() + timeout_s
        delay = 0.0005
        while not os.path.exists(self.done_marker):
            if time.monotonic() > deadline:
                raise RuntimeError(
                    f"timed out after {timeout_s:.0f} s waiting for the GPU-owning process to finish writing "
                    f"(marker '{self.done_marker}' never appeared)"
                )
            time.sleep(delay)
            delay = min(delay * 2, 0.01)
        with open(self.done_marker, "rb") as f:
            ok, payload = pickle.load(f)
        try:
            os.remove(self.done_marker)
        except OSError:
            pass
        if not ok:
            raise RuntimeError(f"writing the checkpoint object failed in the GPU-owning process: {payload}")
        return payload


class StagedTensorRef:
    """Placeholder that replaces a tensor in ``ObjectWriteBucket.tensor_data`` once its bytes are in the image.

    Generic staging code that calls ``tensor.to("cpu")`` on bucket entries gets the same object back: there is
    nothing left to move, the bytes already sit in the packed image.
    """

    __slots__ = ("staged", "index", "dtype", "shape")
    device = torch.device("cpu")
    is_cuda = False

    def __init__(self, staged: StagedObject, index: int, dtype: torch.dtype, shape: torch.Size):
        self.staged, self.index, self.dtype, self.shape = staged, index, dtype, shape

    def to(self, *args, **kwargs):
        return self

    def detach(self):
        return self

    def wait_until_packed(self) -> None:
        """Returns once the pack that read this tensor has finished, i.e. once the live tensor may be overwritten.
        Staging code that finds this method on every entry can call it instead of synchronizing the whole device,
        which would also wait for an earlier checkpoint that is still crossing the host link."""
        event = getattr(self.staged, "packed_event", None)
        if event is not None:
            event.synchronize()

    def numel(self) -> int:
        return self.shape.numel()

    def element_size(self) -> int:
        return torch.empty((), dtype=self.dtype).element_size()


_MARKER_PREFIX, _MARKER_SUFFIXES = "mlf_write_", (".done", ".done.tmp")


def _sweep_stale_markers() -> int:
    """Removes the result markers (``mlf_write_<pid>_<id>.done`` in the temporary directory) of writer processes that
    no longer exist: a writer that crashed between writing its marker and its waiter reading it leaves the file
    behind, and nothing else would ever take it away.  Markers of live processes are left alone, whoever they
    belong to.  Returns the number of files removed."""
    removed = 0
    try:
        names = os.listdir(tempfile.gettempdir())
    except OSError:
        return 0
    for name in names:
        if not (name.startswith(_MARKER_PREFIX) and name.endswith(_MARKER_SUFFIXES)):
            continue
        pid = name[len(_MARKER_PREFIX):].split("_", 1)[0]
        if not pid.isdigit() or int(pid) == os.getpid():
            continue
        try:
            os.kill(int(pid), 0)  # signal 0: existence check only
            continue
        except ProcessLookupError:
            pass
        except OSError:  # it exists but is not ours to signal: not ours to clean up after either
            continue
        try:
            os.remove(os.path.join(tempfile.gettempdir(), name))
            removed += 1
        except OSError:
            pass
    return removed


class HipMLFlashpointCheckpointSaver(MLFlashpointCheckpointSaver):
    def __init__(
        self,
        global_rank_getter: Callable[[], int],
        local_rank_getter: Callable[[], int],
        global_barrier_func: Callable[[], None],
        ckpt_obj_manager: CheckpointObjectManager,
        replication_manager=None,
        initial_buffer_size_bytes: int = DEFAULT_INITIAL_BUFFER_SIZE_BYTES,
        use_optimized_save: bool = True,
        *,
        engine_config: Optional[EngineConfig] = None,
        tile_bytes: int = 0,
        block_threads: int = 0,
        crc_chunk_bytes: int = 0,
        crc_mode: str = "host",
        use_file_io: bool = False,
        background_write: bool = False,
        remote_wait_timeout_s: float = 1800.0,
        max_image_bytes: Optional[int] = None,
        reuse_plans: bool = True,
        snapshot_host_tensors: bool = False,
    ):
        """Same positional arguments as the reference's default saver (checkpoint_saver.py:290-321);
        ``use_optimized_save=False`` writes the legacy format (``torch.save`` records) on the host, as the reference does.

        Keyword-only extras: ``engine_config`` (pinned ring), ``tile_bytes`` / ``block_threads`` (pack kernel work
        split, 0 = library default), ``crc_chunk_bytes`` (> 0: compute a CRC-32C per chunk of every object on the
        GPU and keep it beside the object), ``crc_mode`` (where those checksums are computed: ``"host"``, the default - by the
        copy engine's host threads as they move the pinned slots into the buffer, crc32 instructions beside the
        copy loop: no kernel, no second read of the image, nothing added to the blocking part, and on the hosts
        measured no slower than the plain copy; the same holds for objects that leave in several transfers (pieces,
        windows, host-resident items between the runs of the image), whose parts' checksums are joined per chunk;
        ``"beside"`` - a pass of kernels over the finished image, on the copy engine's third
        stream while the image crosses the link: nothing added to the blocking part either, but the image is read
        from device memory a second time; ``"fused"`` - inside the pack kernel, which then runs about 12 % longer),
        ``use_file_io`` (False, the default: the host threads memcpy the
        pinned slots into the mapping, whose page-table entries a pooled buffer keeps from save to save; True: they
        pwrite() through the file descriptor, which tmpfs serialises on the inode lock - measured 5x slower),
        ``background_write`` (True: ``prepare_write_data`` also starts the transfer into the buffer object on a
        background thread of this process; ``write_data`` - here or in a worker process that received the buckets -
        then only waits for it, for at most ``remote_wait_timeout_s`` across processes), ``max_image_bytes`` (largest
        image to hold in HBM at once; default: what is free on the device.  Of a larger object the end stays resident
        and follows on a thread, the rest is packed and sent window by window inside ``prepare_write_data``, which
        blocks for that part of the transfer), ``reuse_plans`` (keep
        the layout and the device-resident tables of every object from one save to the next and use them again
        when the tensors' addresses, shapes, strides and dtypes are the same; only the bytes of host-resident items
        are refreshed.  With 20 000 tensors this takes 60 ms out of the blocking part of each save after the first),
        ``snapshot_host_tensors`` (large host-resident tensors are copied from where they are into the buffer while
        the transfer runs, as the reference copies them while it writes; True: they are cloned inside
        ``prepare_write_data`` instead, for training loops that update them before the transfer has ended).
        """
        _lib.load()  # fail now, loudly, if the native library is not there
        _sweep_stale_markers()
        self._global_rank_getter = global_rank_getter
        self._local_rank_getter = local_rank_getter
        self._barrier_func = global_barrier_func
        self._chkpt_obj_manager = ckpt_obj_manager
        self._replication_manager = replication_manager
        self._initial_buffer_size_bytes = initial_buffer_size_bytes
        # False: the legacy object format, one ``torch.save`` record per tensor.  Those records are produced by
        # torch's serializer, on the host, as in the reference (checkpoint_saver.py:662-673); the kernels are not
        # involved and the blocking part of such a save is the generic ``.to("cpu")`` staging.
        self._use_optimized_save = use_optimized_save
        self._engine_config = engine_config or EngineConfig()
        self._tile_bytes = tile_bytes
        self._block_threads = block_threads
        if crc_mode not in ("beside", "fused", "host"):
            raise ValueError("crc_mode must be 'beside', 'fused' or 'host'")
        if crc_chunk_bytes % 65536:
            raise ValueError("crc_chunk_bytes must be a multiple of 65536")
        self._crc_chunk_bytes = crc_chunk_bytes
        self._crc_mode = crc_mode
        self._use_file_io = use_file_io
        self._background_write = background_write
        self._remote_wait_timeout_s = remote_wait_timeout_s
        self._max_image_bytes = max_image_bytes
        self._reuse_plans = reuse_plans
        self._snapshot_host_tensors = snapshot_host_tensors
        self._init_runtime_state()

    def _init_runtime_state(self):
        self._engine: Optional[hip_plan.CopyEngine] = None
        self._engine_clear_of: Optional[set] = None  # the streams whose hardware queues the engine's streams avoid
        self._engine_lock = threading.Lock()
        self.last_save_stats: dict = {}
        # set to True to bracket every pack launch with timing events on its stream; (start, end, payload bytes)
        # tuples are appended to kernel_events for the caller to read after a synchronize
        self.record_kernel_events = False
        self.kernel_events: list = []
        self._plan_cache: dict = {}  # object name -> _KeptPlan
        # Kept for the adapter from save to save (writers are made anew for every save, the saver stays): where every
        # rank's items went in the last save that this process finished, and the metadata object of the last planning
        # save - what the next save's metadata object is pickled from while its data is still in flight.
        self.last_write_locations: Optional[dict] = None
        self.last_global_metadata = None
        self.last_metadata_pickle = None  # (see MemoryStorageWriter: the bytes of the last metadata object written)

    # ---- pickling: only configuration crosses a process boundary --------------------------------------
    def __getstate__(self):
        state = self.__dict__.copy()
        for key in ("_replication_manager", "_engine", "_engine_clear_of", "_engine_lock", "last_save_stats", "kernel_events",
                    "_plan_cache", "last_write_locations", "last_global_metadata", "last_metadata_pickle"):
            state.pop(key, None)
        return state

    def __setstate__(self, state):
        self.__dict__.update(state)
        self._replication_manager = None
        self._init_runtime_state()

    def _get_engine(self) -> hip_plan.CopyEngine:
        with self._engine_lock:
            if self._engine is None:
                cfg = self._engine_config
                self._engine = hip_plan.CopyEngine(cfg.slot_bytes, cfg.n_slots, cfg.resolved_copy_threads())
                self._engine.set_host_checksums(self._crc_mode == "host")
            return self._engine

    def warm_up(self, device: Optional[torch.device] = None, also_avoid: tuple = ()) -> None:
        """Creates the copy engine (pinned slots, streams, threads) and moves its streams off the hardware queue of
        the stream that is current on ``device`` now - the one the training step runs on: HIP spreads a process's
        streams over a few hardware queues, and a copy stream that shares its queue with a stream that is kept full
        waits behind that stream's kernels (measured: 10-13 GB/s instead of 53-56 beside back-to-back GEMMs).  The
        first ``prepare_write_data`` does this by itself, inside its blocking part (30-50 ms, once - again if a
        later save finds another stream current - and it waits for the stream to drain); a job that calls
        ``warm_up`` at start-up spares its first save that.  ``also_avoid``: other streams of the job that are kept
        busy (``torch.cuda.Stream`` objects or raw handles)."""
        device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
        wanted = {torch.cuda.current_stream(device).cuda_stream} | {getattr(s, "cuda_stream", s) for s in also_avoid}
        with self._engine_lock:
            if self._engine_clear_of is not None and wanted <= self._engine_clear_of:
                return
            wanted |= self._engine_clear_of or set()
        with torch.cuda.device(device):
            _lib.check(_lib.load().mlf_hip_set_device(device.index or 0), "mlf_hip_set_device")
            left = self._get_engine().avoid_stream(*sorted(wanted))
        if left:
            _LOGGER.warning("%d of the copy engine's streams share a hardware queue with a stream of the training step: "
                            "transfers beside a busy device will be slow (more queues: GPU_MAX_HW_QUEUES)", left)
        with self._engine_lock:
            self._engine_clear_of = wanted | (self._engine_clear_of or set())

    # ---- dirty marker / directory ----------------------------------------------------------------------
    @override
    @log_execution_time(logger=_LOGGER, name="initialize_checkpoint")
    def initialize_checkpoint(self, checkpoint_id: CheckpointContainerId) -> None:
        self._create_dirty_checkpoint_marker(checkpoint_id)
        os.makedirs(checkpoint_id.data, exist_ok=True)

    def _get_dirty_marker_file_path(self, checkpoint_id: CheckpointContainerId) -> str:
        if str(checkpoint_id) == "/":
            raise ValueError("CheckpointContainerId cannot be the root path '/'")
        return f"{str(checkpoint_id).rstrip('/')}__{self._local_rank_getter()}__{DIRTY_MARKER_SUFFIX}"

    def _create_dirty_checkpoint_marker(self, checkpoint_id: CheckpointContainerId) -> None:
        path = self._get_dirty_marker_file_path(checkpoint_id)
        os.makedirs(os.path.dirname(path), exist_ok=True)
        with open(path, "w"):
            pass

    def _remove_dirty_checkpoint_marker(self, checkpoint_id: CheckpointContainerId) -> None:
        path = self._get_dirty_marker_file_path(checkpoint_id)
        if not os.path.exists(path):
            _LOGGER.warning("Dirty marker file path: '%s' does not exist, skipping removal.", path)
            return
        os.remove(path)

    # ---- stage_data ---------------------------------------------------------------------------------
    @override
    @log_execution_time(logger=_LOGGER, name="stage_data", level=logging.INFO)
    def stage_data(self, checkpoint_id: CheckpointContainerId, state_dict: dict, non_blocking: bool = True) -> dict:
        """Host-resident copy of a flat state dict: one batched gather in HBM and one pinned-ring transfer into a
        single host arena, instead of one pageable D2H copy per tensor.  Host tensors and non-tensors pass through.
        Blocking either way (``non_blocking`` is accepted for interface compatibility)."""
        device_entries = [(k, v) for k, v in state_dict.items() if isinstance(v, torch.Tensor) and v.device.type != "cpu"]
        staged = dict(state_dict)
        by_device: dict = {}
        for k, v in device_entries:
            by_device.setdefault(v.device, []).append((k, v))
        for device, entries in by_device.items():
            table = hip_plan.ItemTable()
            offsets, pos = [], 0
            for _, t in entries:
                offsets.append(pos)
                nbytes = t.numel() * t.element_size()
                if nbytes:
                    shape, stride = tuple(t.shape), tuple(t.stride())
                    if len(shape) > _lib.MAX_DIMS and t.is_contiguous():
                        shape, stride = (t.numel(),), (1,)
                    table.add_device(t.data_ptr(), pos, t.element_size(), shape, stride)
                pos = (pos + nbytes + _STAGE_ALIGN - 1) // _STAGE_ALIGN * _STAGE_ALIGN
            arena = torch.empty(max(pos, 1), dtype=torch.uint8)
            if pos:
                with torch.cuda.device(device):
                    _lib.check(_lib.load().mlf_hip_set_device(device.index or 0), "mlf_hip_set_device")
                    plan = hip_plan.Plan(table.to_array(), b"", pos, tile_bytes=self._tile_bytes,
                                         block_threads=self._block_threads)
                    image = torch.empty(pos, dtype=torch.uint8, device=device)
                    stream = torch.cuda.current_stream(device).cuda_stream
                    plan.pack(image, stream)
                    self._get_engine().d2h(image.data_ptr(), arena.data_ptr(), pos, stream)
                    plan.destroy()
            for (k, t), off in zip(entries, offsets):
                n = t.numel()
                if n == 0:
                    staged[k] = torch.empty(t.shape, dtype=t.dtype)
                else:
                    staged[k] = arena[off : off + n * t.element_size()].view(t.dtype).reshape(t.shape)
        return staged

    # ---- prepare_write_data (+ the pack) ------------------------------------------------------------
    @override
    @log_execution_time(logger=_LOGGER, name="prepare_write_data")
    def prepare_write_data(
        self,
        checkpoint_id: CheckpointContainerId,
        write_items: list[WriteItem],
        write_item_resolver: WriteItemResolver,
        object_name_prefix: str,
        bucket_count: int,
    ) -> list[ObjectWriteBucket]:
        """Groups the items exactly as the reference does (same bucketing routine, same object names) and, per
        object, enqueues the pack of its image on the current stream.  The returned buckets carry
        ``StagedTensorRef`` placeholders; ``write_data`` finds the image through them."""
        with gc_paused():
            return self._prepare_write_data(checkpoint_id, write_items, write_item_resolver, object_name_prefix, bucket_count)

    def _prepare_write_data(self, checkpoint_id, write_items, write_item_resolver, object_name_prefix, bucket_count):
        t_start = time.perf_counter()
        bucket_count = max(bucket_count, 1)
        rank = self._global_rank_getter()
        write_buckets: list[ObjectWriteBucket] = []
        stats = {"plan_build_s": 0.0, "objects": 0, "device_payload_bytes": 0, "image_bytes": 0}
        for bucket in _split_by_size_and_type(bucket_count, write_items):
            if not bucket:
                continue
            bytes_data = [
                (item, write_item_resolver.resolve_data(item)) for item in bucket if item.type == WriteItemType.BYTE_IO
            ]
            tensor_data = [
                (item, write_item_resolver.resolve_data(item).detach()) for item in bucket if item.type != WriteItemType.BYTE_IO
            ]
            if not bytes_data and not tensor_data:
                continue
            object_name = f"{object_name_prefix}_{len(write_buckets)}_src{rank}{_DEFAULT_OBJ_NAME_SUFFIX}"
            object_id = CheckpointObjectId.from_container(checkpoint_id, object_name)
            if not self._use_optimized_save or not tensor_data:
                # torch.save records, or an object of byte blobs only: written on the host by write_data, nothing
                # to pack.  Host views are copied now, as the reference does (checkpoint_saver.py:390-398).
                tensor_data = [(item, self._clone_if_needed(t)) for item, t in tensor_data]
                write_buckets.append(ObjectWriteBucket(object_id=object_id, object_name=object_name,
                                                       bytesio_data=bytes_data, tensor_data=tensor_data))
                continue
            staged = self._stage_object(tensor_data, bytes_data, stats, object_id, object_name)
            refs = [
                (item, StagedTensorRef(staged, i, t.dtype, t.shape)) for i, (item, t) in enumerate(tensor_data)
            ]
            bucket_out = ObjectWriteBucket(object_id=object_id, object_name=object_name, bytesio_data=bytes_data,
                                           tensor_data=refs)
            write_buckets.append(bucket_out)
            if self._background_write and refs and staged.future is None:
                self._start_background_write(staged, bucket_out)
        stats["prepare_s"] = time.perf_counter() - t_start
        self.last_save_stats = stats
        return write_buckets

    @staticmethod
    def _clone_if_needed(tensor: torch.Tensor) -> torch.Tensor:
        if tensor.device.type != "cpu":
            return tensor
        is_view = tensor.untyped_storage().size() != tensor.numel() * tensor.element_size()
        return (tensor.clone() if is_view else tensor).contiguous()

    def _image_limit(self, device: torch.device) -> int:
        """Bytes of HBM an image may take: the explicit limit, or what the device and torch's allocator have free
        (minus a margin for the tables and for whatever the training step allocates next)."""
        if self._max_image_bytes is not None:
            return self._max_image_bytes
        free, _ = torch.cuda.mem_get_info(device)
        cached = torch.cuda.memory_reserved(device) - torch.cuda.memory_allocated(device)
        return max(free + cached - (2 << 30), 64 << 20)

    def _stage_object(self, tensor_data, bytes_data, stats: dict, object_id=None, object_name=None) -> StagedObject:
        blobs = []
        for _, data in bytes_data:
            data.seek(0)
            blobs.append(data.read())
        tensors = [t for _, t in tensor_data]
        t0 = time.perf_counter()
        for i, t in enumerate(tensors):
            if t.dim() > _lib.MAX_DIMS and t.device.type != "cpu" and not t.is_contiguous() \
                    and not hip_plan.describable(tuple(t.shape), tuple(t.stride())):
                # A view of more dimensions than a descriptor holds, also after merging neighbours: made contiguous
                # on the device, on the stream the pack follows on, and packed from there as one run - what the
                # reference's ``copy_`` into the buffer does on the host (checkpoint_saver.py:797-800).  The copy is
                # a new tensor at every save, so such an object's plan is rebuilt every time.
                tensors[i] = t.contiguous()
        key = self._plan_key(tensors, blobs) if self._reuse_plans and object_name is not None else None
        kept = self._plan_cache.get(object_name) if key is not None else None
        if kept is not None and kept.key != key:
            self._drop_kept_plan(object_name)
            kept = None
        if kept is not None:
            device = kept.device
            fresh_blob = kept.refreshed_blob(tensors, blobs)
            layout = dataclasses.replace(kept.layout, blob=kept.blob,
                                         device_tensors=[t for t in tensors if t.device.type != "cpu"],
                                         host_tensors=[tensors[i] if i >= 0 else blobs[-1 - i]
                                                       for _, _, i in kept.layout.host_spans])
        else:
            # through the file descriptor (pwrite) everything goes through the image; the direct host copy
            # writes into the mapping
            layout = hip_plan.build_save_layout(tensors, blobs,
                                                None if self._use_file_io else _HOST_DIRECT_MIN_BYTES)
            device = next((t.device for t in tensors if t.device.type != "cpu"), None)
            if any(t.device != device for t in tensors if t.device.type != "cpu"):
                raise ValueError("all device tensors of one checkpoint object must live on the same device")
            if device is None:
                device = torch.device("cuda", torch.cuda.current_device())
        if layout.host_tensors and self._snapshot_host_tensors:
            layout.host_tensors = [t.detach().clone(memory_format=torch.contiguous_format) if isinstance(t, torch.Tensor)
                                   else t for t in layout.host_tensors]  # (byte blobs are immutable as they are)
        items = [item for item, _ in tensor_data] + [item for item, _ in bytes_data]
        plan = image = packed = None
        stream = 0
        clear_of = self._engine_clear_of  # (one read: warm_up replaces the set, it never changes one in place)
        if layout.image_bytes and (clear_of is None or torch.cuda.current_stream(device).cuda_stream not in clear_of):
            self.warm_up(device)  # the engine's streams off the hardware queue of the stream the pack runs on
        if layout.image_bytes and object_id is not None:
            if layout.image_bytes <= self._image_limit(device):
                with torch.cuda.device(device):
                    image = hip_plan.try_allocate(layout.image_bytes, device)
            if image is None:
                # no room for the image in one block: in pieces, all resident, if the device has that much left
                # in smaller blocks (the save stays asynchronous); else window by window through one buffer
                self._drop_kept_plan(object_name)
                if layout.host_spans:  # both modes send one image, whole: lay the host items out inside it
                    layout = hip_plan.build_save_layout(tensors, blobs)
                staged = self._stage_in_pieces(layout, items, device, stats)
                if staged is not None:
                    return staged
                return self._stage_windowed(layout, items, object_id, object_name, device, stats)
        if layout.image_bytes:
            with torch.cuda.device(device):
                _lib.check(_lib.load().mlf_hip_set_device(device.index or 0), "mlf_hip_set_device")
                stream = torch.cuda.current_stream(device).cuda_stream
                if kept is not None:
                    plan = kept.plan
                    earlier = kept.last_staged() if kept.last_staged is not None else None
                    if earlier is not None and earlier.plan is plan:
                        # a save that is still waiting to be written: its checksums leave the plan before this
                        # launch overwrites them
                        self._fused_checksums(earlier)
                    if fresh_blob is not None:  # step counters, RNG state, pickled objects: new bytes, same places
                        plan.update_blob(fresh_blob, stream)
                    stats["plans_reused"] = stats.get("plans_reused", 0) + 1
                else:
                    # checksums inside the pack only where one image is the whole data section
                    fused = self._crc_chunk_bytes if self._crc_mode == "fused" and not layout.host_spans else 0
                    plan = hip_plan.Plan(layout.items, layout.blob, layout.image_bytes, tile_bytes=self._tile_bytes,
                                         block_threads=self._block_threads, crc_chunk_bytes=fused)
                    if key is not None:
                        self._keep_plan(object_name, _KeptPlan(key, layout, plan, device))
                if image is None:
                    image = torch.empty(layout.image_bytes, dtype=torch.uint8, device=device)
                stats["plan_build_s"] += time.perf_counter() - t0
                if self.record_kernel_events:
                    begin, packed = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    begin.record()
                    plan.pack(image, stream)
                    packed.record()
                    self.kernel_events.append((begin, packed, layout.device_payload_bytes))
                else:
                    plan.pack(image, stream)
                    packed = torch.cuda.Event()
                    packed.record()
        stats["objects"] += 1
        stats["device_payload_bytes"] += layout.device_payload_bytes
        stats["image_bytes"] += layout.image_bytes
        staged = StagedObject(layout, plan, image, device.index or 0, stream, items)
        staged.packed_event = packed if layout.image_bytes else None
        staged.owns_plan = key is None  # with a key the plan went into, or came out of, the kept plans
        staged.kept = self._plan_cache.get(object_name) if key is not None and plan is not None else None
        if staged.kept is not None and staged.kept.plan is not plan:
            staged.kept = None
        if plan is not None and plan.crc_chunk_bytes and key is not None:
            holder = self._plan_cache.get(object_name)
            if holder is not None and holder.plan is plan:
                holder.last_staged = weakref.ref(staged)
        return staged

    # ---- plans kept from save to save ---------------------------------------------------------------------
    def _plan_key(self, tensors, blobs) -> tuple:
        """Everything the layout and the device tables of an object depend on - and nothing that changes from one
        save of the same model to the next: addresses, dtypes, shapes (strides where they matter), the lengths of
        the byte blobs, the work-split options.  Contents are not part of it."""
        parts = []
        for t in tensors:
            where = t.device
            if where.type == "cpu":
                parts.append((None, t.dtype, t.shape))
            elif t.is_contiguous():
                parts.append((where.index, t.data_ptr(), t.dtype, t.shape))
            else:
                parts.append((where.index, t.data_ptr(), t.dtype, t.shape, t.stride()))
        return (tuple(parts), tuple(len(b) for b in blobs), self._tile_bytes, self._block_threads,
                self._crc_chunk_bytes if self._crc_mode == "fused" else 0)

    def _keep_plan(self, object_name: str, kept: "_KeptPlan") -> None:
        while len(self._plan_cache) >= _MAX_KEPT_PLANS:
            self._drop_kept_plan(next(iter(self._plan_cache)))
        self._plan_cache[object_name] = kept

    def _drop_kept_plan(self, object_name) -> None:
        kept = self._plan_cache.pop(object_name, None)
        if kept is not None:
            kept.plan.destroy()  # releasing device memory waits for the kernels that still use it

    @staticmethod
    def _blob_of_rows(rows: np.ndarray, blob: bytes) -> bytes:
        """The part of the host blob that the blob items among ``rows`` refer to, their offsets rebased onto it: a
        plan uploads its blob whole, and the blob of an object with host-resident tensors laid out inside its image
        is as large as those tensors together - more than a window's plan may bring to a device that is short of
        room.  ``rows`` is changed in place."""
        from_blob = rows["kind"] == hip_plan.ITEM_BLOB
        if not from_blob.any():
            return b""
        first = int(rows["ptr"][from_blob].min())
        end = int((rows["ptr"][from_blob] + rows["nbytes"][from_blob]).max())
        rows["ptr"][from_blob] -= first
        return blob[first:end]

    @staticmethod
    def _windows_of(layout: hip_plan.SaveLayout, limit: int, stop: Optional[int] = None) -> list:
        """Consecutive rows of the layout's table (the first ``stop`` of them) grouped into windows of at most
        ``limit`` image bytes (a single larger row gets a window of its own): [(first row, end row, first image
        byte, end)]."""
        arr = layout.items
        ends = (arr["image_off"] + arr["nbytes"]).tolist()
        starts = arr["image_off"].tolist()
        windows, r0, n = [], 0, len(arr) if stop is None else stop
        while r0 < n:
            r1 = r0 + 1
            while r1 < n and ends[r1] - starts[r0] <= limit:
                r1 += 1
            windows.append((r0, r1, starts[r0], ends[r1 - 1]))
            r0 = r1
        return windows

    def _stage_in_pieces(self, layout, items, device, stats: dict) -> Optional[StagedObject]:
        """The image in several device buffers, all packed now: for a device whose free memory is there but not in
        one block.  The transfer sends them one after the other, so the save is as asynchronous as with one
        image.  None (and nothing allocated) if the buffers cannot be had either."""
        if self._max_image_bytes is not None and layout.image_bytes > self._max_image_bytes:
            return None
        windows = self._windows_of(layout, _IMAGE_PIECE_BYTES)
        with torch.cuda.device(device):
            _lib.check(_lib.load().mlf_hip_set_device(device.index or 0), "mlf_hip_set_device")
            buffers = []
            for _, _, begin, end in windows:
                buffers.append(hip_plan.try_allocate(begin % _WINDOW_PAD + end - begin, device))
                if buffers[-1] is None:
                    del buffers
                    return None
            if self._max_image_bytes is None and torch.cuda.mem_get_info(device)[0] < (1 << 30):
                del buffers  # that would leave the training step nothing to allocate from
                torch.cuda.empty_cache()
                return None
            _LOGGER.warning("no single block of %d bytes of device memory: the checkpoint image is held in %d pieces",
                            layout.image_bytes, len(windows))
            stream = torch.cuda.current_stream(device).cuda_stream
            pieces = []
            t0 = time.perf_counter()
            begin_event = torch.cuda.Event(enable_timing=True) if self.record_kernel_events else None
            if begin_event is not None:
                begin_event.record()
            for (r0, r1, begin, end), buf in zip(windows, buffers):
                pad = begin % _WINDOW_PAD  # as in _stage_windowed
                sub = layout.items[r0:r1].copy()
                sub["image_off"] -= begin - pad
                plan = hip_plan.Plan(sub, self._blob_of_rows(sub, layout.blob), pad + end - begin,
                                     tile_bytes=self._tile_bytes, block_threads=self._block_threads)
                plan.pack(buf, stream)
                pieces.append((plan, buf, begin, end))
            packed = torch.cuda.Event(enable_timing=self.record_kernel_events)
            packed.record()
            if begin_event is not None:
                self.kernel_events.append((begin_event, packed, layout.device_payload_bytes))
            stats["plan_build_s"] += time.perf_counter() - t0
        stats["objects"] += 1
        stats["image_pieces"] = stats.get("image_pieces", 0) + len(pieces)
        stats["device_payload_bytes"] += layout.device_payload_bytes
        stats["image_bytes"] += layout.image_bytes
        staged = StagedObject(layout, None, None, device.index or 0, stream, items)
        staged.pieces = pieces
        staged.packed_event = packed
        return staged

    def _stage_windowed(self, layout, items, object_id, object_name, device, stats: dict) -> StagedObject:
        """Fallback for an object whose image does not fit in HBM beside the live state.  The records at the end of
        the object, as many as the limit holds beside the window buffers (a quarter of it, at most 8 GiB), are packed
        into an image that stays resident, like the image of an ordinary save; the records before them are grouped
        into windows (a single larger record gets a window of its own) that pass through two alternating buffers:
        one is packed while the other crosses the link.  One thread of this process sends everything, in order -
        windows, then the resident image - checksums what it sent and closes the buffer; this call returns when the
        last window has been packed, i.e. when nothing reads the live tensors any more.  Blocking time: about
        (image - resident part - two windows) / link rate."""
        _LOGGER.warning("checkpoint image of %d bytes exceeds the HBM limit; saving '%s' window by window (blocking)",
                        layout.image_bytes, object_id)
        arr = layout.items
        limit = self._max_image_bytes
        if limit is None:  # what the driver reports free now, the allocator's unused segments included
            torch.cuda.empty_cache()
            limit = max(torch.cuda.mem_get_info(device)[0] - (2 << 30), 64 << 20)
        limit = max(limit, 1)
        nbytes = layout.image_bytes
        starts = arr["image_off"].tolist()
        ends = (arr["image_off"] + arr["nbytes"]).tolist()
        xfer = {"d2h_s": 0.0, "d2h_wait_s": 0.0, "d2h_bytes": 0}
        staged = StagedObject(layout, None, None, device.index or 0, 0, items)
        staged.consumed = True
        staged.future = concurrent.futures.Future()
        staged.done_marker = os.path.join(tempfile.gettempdir(), f"mlf_write_{os.getpid()}_{uuid.uuid4().hex}.done")
        held = contextlib.ExitStack()  # the buffer stays open until the last byte has been written
        sender = concurrent.futures.ThreadPoolExecutor(max_workers=1, thread_name_prefix=f"mlf-write-{object_name}")
        sent: list = []  # one future per window, in order
        made: list = []  # every plan built here; released at the end (freeing device memory waits for the whole device)
        try:
            writer = held.enter_context(
                self._chkpt_obj_manager.acquire_buffer(object_id, max(self._initial_buffer_size_bytes, nbytes)))
            writer.set_format_signature(CheckpointFormat.MLF_FORMAT)
            ensure = getattr(writer, "ensure_capacity", None)
            if ensure is not None:
                ensure(nbytes)
            with torch.cuda.device(device):
                _lib.check(_lib.load().mlf_hip_set_device(device.index or 0), "mlf_hip_set_device")
                start = writer.tell()
                writer.next_buffer_slice(nbytes).release()
                stream = torch.cuda.current_stream(device).cuda_stream
                engine = self._get_engine()
                sums = integrity.ChunkChecksums(self._crc_chunk_bytes, nbytes) if self._crc_chunk_bytes and nbytes else None
                # checksum kernels go to the engine's checksum stream: the training step's kernels are queued on the pack's
                side = engine.checksum_stream

                def pack_rows(r0, r1, begin, end, buf):
                    """Rows [r0, r1) = image bytes [begin, end) into ``buf``.  They lie in the buffer where they lie
                    in the image modulo the pad, so that tiles and checksum chunks are cut on the same grid as in
                    an image held whole.  Returns the plan, the pad and the event recorded behind the pack."""
                    pad = begin % _WINDOW_PAD
                    sub = arr[r0:r1].copy()
                    sub["image_off"] -= begin - pad
                    plan = hip_plan.Plan(sub, self._blob_of_rows(sub, layout.blob), pad + end - begin,
                                         tile_bytes=self._tile_bytes, block_threads=self._block_threads)
                    made.append(plan)
                    if self.record_kernel_events:
                        t_begin, packed = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                        t_begin.record()
                        plan.pack(buf, stream)
                        packed.record()
                        self.kernel_events.append(
                            (t_begin, packed, int(sub["nbytes"][sub["kind"] == hip_plan.ITEM_DEVICE].sum())))
                    else:
                        plan.pack(buf, stream)
                        packed = torch.cuda.Event()
                        packed.record()
                    return plan, pad, packed

                def send(plan, buf, pad, begin, end, packed):
                    """On the sender's thread: [begin, end) out of ``buf`` into the file, its checksums, the plan's
                    end.  Windows end where records end, not where checksum chunks end: the parts are checksummed
                    where they lie in the buffer and joined per chunk."""
                    with torch.cuda.device(device):
                        _lib.check(_lib.load().mlf_hip_set_device(device.index or 0), "mlf_hip_set_device")
                        dst = writer.data_address(start + begin)
                        if sums is not None and self._crc_mode == "host":
                            # the threads that copy the window into the file take its checksums as they go
                            st, values = engine.d2h_cut(buf.data_ptr() + pad, dst, end - begin, begin, self._crc_chunk_bytes,
                                                        ready_event=packed.cuda_event)
                            sums.add(begin, end - begin, values)
                        else:
                            st, _ = engine.d2h_gated(buf.data_ptr() + pad, dst, end - begin, packed.cuda_event, 0,
                                                     ctypes.c_uint64(0))
                        xfer["d2h_s"] += st.seconds
                        xfer["d2h_bytes"] += end - begin
                        if sums is not None and self._crc_mode != "host":
                            t0 = time.perf_counter()
                            sums.add(begin, end - begin, hip_plan.crc32c_device_cut(
                                buf, pad, begin, end - begin, self._crc_chunk_bytes, dst, side))
                            xfer["crc_s"] = xfer.get("crc_s", 0.0) + time.perf_counter() - t0

                # the resident part: the longest run of records at the end that fits beside the window buffers
                cycle = max(min(limit // 4, _WINDOW_BUFFER_BYTES), 1)
                room = limit - cycle - 3 * _WINDOW_PAD
                tail_row = len(arr)
                while tail_row > 0 and ends[-1] - starts[tail_row - 1] <= room:
                    tail_row -= 1
                tail = None  # arguments of its send()
                if 0 < tail_row < len(arr):
                    tail_begin = starts[tail_row]
                    image = hip_plan.try_allocate(tail_begin % _WINDOW_PAD + nbytes - tail_begin, device)
                    if image is not None:
                        plan, pad, packed = pack_rows(tail_row, len(arr), tail_begin, nbytes, image)
                        tail = (plan, image, pad, tail_begin, nbytes, packed)
                if tail is None:
                    tail_row, cycle = len(arr), limit
                # two buffers of half the size where that leaves windows worth sending, else one
                windows = self._windows_of(layout, cycle // 2, tail_row) if cycle // 2 >= _WINDOW_PAIR_MIN_BYTES else None
                largest = max((e - b for _, _, b, e in windows), default=0) if windows else 0
                if windows and 2 * (largest + _WINDOW_PAD) <= cycle + 2 * _WINDOW_PAD:
                    buffers = [torch.empty(largest + _WINDOW_PAD, dtype=torch.uint8, device=device) for _ in range(2)]
                else:
                    windows = self._windows_of(layout, cycle, tail_row)
                    buffers = [torch.empty(max(e - b for _, _, b, e in windows) + _WINDOW_PAD, dtype=torch.uint8, device=device)]
                for k, (r0, r1, begin, end) in enumerate(windows):
                    if k >= len(buffers):
                        sent[k - len(buffers)].result()  # the buffer's previous window has left it
                    buf = buffers[k % len(buffers)]
                    plan, pad, packed = pack_rows(r0, r1, begin, end, buf)
                    sent.append(sender.submit(send, plan, buf, pad, begin, end, packed))
                    staged.packed_event = packed  # the live tensors are not read after the last of these
        except BaseException:
            sender.shutdown(wait=True)
            for plan in made:
                plan.destroy()
            held.__exit__(*sys.exc_info())
            raise

        def finish():
            """After the last window: the resident part, the sidecar, the buffer's close, the outcome."""
            try:
                with held:
                    for done in sent:
                        done.result()
                    if tail is not None:
                        send(*tail)
                if sums is not None:
                    integrity.write_sidecar(str(object_id), self._crc_chunk_bytes, nbytes, sums.result())
                else:
                    integrity.remove_sidecar(str(object_id))
                outcome = (True, self._results_of(staged, object_name))
            except BaseException as e:  # reported to whoever waits; a thread must not die silently
                _LOGGER.exception("Windowed write of '%s' failed", object_id)
                outcome = (False, f"{type(e).__name__}: {e}")
            for plan in made:
                plan.destroy()
            stats.update({k: stats.get(k, 0) + v for k, v in xfer.items()})  # (the dict last_save_stats refers to)
            try:
                tmp = staged.done_marker + ".tmp"
                with open(tmp, "wb") as f:
                    pickle.dump(outcome, f)
                os.rename(tmp, staged.done_marker)
            finally:
                if outcome[0]:
                    staged.future.set_result(outcome[1])
                else:
                    staged.future.set_exception(RuntimeError(outcome[1]))

        stats["objects"] += 1
        stats["windows"] = stats.get("windows", 0) + len(windows)
        stats["window_buffers"] = len(buffers)
        stats["device_payload_bytes"] += layout.device_payload_bytes
        stats["image_bytes"] += nbytes
        if tail is not None:
            stats["resident_bytes"] = stats.get("resident_bytes", 0) + nbytes - tail[3]
        sender.submit(finish)
        sender.shutdown(wait=False)  # the thread ends when finish() has run
        return staged

    @staticmethod
    def _results_of(staged: StagedObject, object_name: str) -> list[WriteResult]:
        """One WriteResult per item of the object, from its layout.  Made once per staged object: the prediction that
        lets the metadata object be pickled early and the write itself ask for the same list (20 ms apiece at
        20 000 items) - and once per kept plan while the saves bring the same items (a kept DCP plan): callers get
        the same list and the same result objects again and must not change them."""
        made = staged._results
        if made is not None and made[0] == object_name:
            return made[1]
        kept = staged.kept
        before = kept.results if kept is not None else None
        if before is not None and before[0] == object_name and len(before[1]) == len(staged.items) \
                and all(a is b for a, b in zip(before[1], staged.items)):
            staged._results = (object_name, before[2])
            return before[2]
        results = [
            WriteResult(
                index=item.index,
                size_in_bytes=length,
                storage_data=_StorageInfo(relative_path=object_name, offset=offset, length=length),
            )
            for item, (offset, length) in zip(staged.items, staged.layout.spans)
        ]
        staged._results = (object_name, results)
        if kept is not None:
            kept.results = (object_name, list(staged.items), results)
        return results

    # ---- write_data -----------------------------------------------------------------------------
    @override
    @log_execution_time(logger=_LOGGER, name="write_data", level=logging.INFO)
    def write_data(
        self,
        checkpoint_id: CheckpointContainerId,
        write_buckets: list[ObjectWriteBucket],
        replicate_after_write: bool,
        thread_count: int = 1,
    ) -> list[WriteResult]:
        """Moves each bucket's image into its buffer object and returns the WriteResults.

        Buckets are processed one after another on the calling thread: the transfer is link-bound and the copy
        engine already spreads the host-side copy over its own threads, so ``thread_count`` adds nothing here.
        Buckets that still hold plain tensors (not produced by ``prepare_write_data`` of this class) are packed
        first."""
        all_results: list[WriteResult] = []
        errors: list[Exception] = []
        xfer = {"d2h_s": 0.0, "d2h_wait_s": 0.0, "d2h_bytes": 0, "crc_s": 0.0}
        for bucket in write_buckets:
            try:
                with gc_paused():
                    all_results.extend(self._write_bucket(bucket, replicate_after_write, xfer))
            except Exception as e:  # collected, first one re-raised: same contract as the reference's workers
                _LOGGER.exception("Error writing object '%s'", bucket.object_id)
                errors.append(e)
        # (a save that went window by window has counted its transfers already)
        self.last_save_stats = {**self.last_save_stats, **{k: self.last_save_stats.get(k, 0) + v for k, v in xfer.items()}}
        if errors:
            raise errors[0]
        return all_results

    def _staged_of(self, bucket: ObjectWriteBucket):
        refs = [t for _, t in bucket.tensor_data]
        if refs and all(isinstance(r, StagedTensorRef) for r in refs):
            staged = refs[0].staged
            in_flight = isinstance(staged, RemoteStagedObject) or staged.future is not None
            if all(r.staged is staged for r in refs) and (in_flight or not staged.consumed):
                return staged
            raise ValueError(f"bucket for '{bucket.object_id}' refers to a staged image that was already written")
        if any(isinstance(r, StagedTensorRef) for r in refs):
            raise ValueError("bucket mixes staged placeholders and tensors")
        return self._stage_object(bucket.tensor_data, bucket.bytesio_data, {"plan_build_s": 0.0, "objects": 0,
                                                                            "device_payload_bytes": 0, "image_bytes": 0})

    def _start_background_write(self, staged: StagedObject, bucket: ObjectWriteBucket) -> None:
        """Runs the transfer of ``bucket`` on a thread of this process and publishes the outcome twice: through
        ``staged.future`` (same process) and through a marker file (for a process that received the bucket)."""
        staged.future = concurrent.futures.Future()
        staged.done_marker = os.path.join(tempfile.gettempdir(), f"mlf_write_{os.getpid()}_{uuid.uuid4().hex}.done")

        def run():
            try:
                results = self._transfer_bucket(staged, bucket, {"d2h_s": 0.0, "d2h_wait_s": 0.0, "d2h_bytes": 0})
                outcome = (True, results)
            except BaseException as e:  # reported to whoever waits; the thread itself must not die silently
                _LOGGER.exception("Background write of '%s' failed", bucket.object_id)
                outcome = (False, f"{type(e).__name__}: {e}")
            try:
                tmp = staged.done_marker + ".tmp"
                with open(tmp, "wb") as f:
                    pickle.dump(outcome, f)
                os.rename(tmp, staged.done_marker)
            finally:
                if outcome[0]:
                    staged.future.set_result(outcome[1])
                else:
                    staged.future.set_exception(RuntimeError(outcome[1]))

        threading.Thread(target=run, name=f"mlf-write-{bucket.object_name}", daemon=True).start()

    def _write_bucket_on_host(self, bucket: ObjectWriteBucket, replicate_after_write: bool) -> list[WriteResult]:
        """An object that the kernels have no part in: ``torch.save`` records (``use_optimized_save=False``) and/or
        byte blobs, written through the buffer's file interface, tensors first (checkpoint_saver.py:655-698)."""
        results: list[WriteResult] = []
        with self._chkpt_obj_manager.acquire_buffer(bucket.object_id, self._initial_buffer_size_bytes) as writer:
            legacy = not self._use_optimized_save
            writer.set_format_signature(CheckpointFormat.TORCH_SAVE if legacy else CheckpointFormat.MLF_FORMAT)

            def record(item, write):
                offset = writer.tell()
                write()
                length = writer.tell() - offset
                results.append(WriteResult(index=item.index, size_in_bytes=length,
                                           storage_data=_StorageInfo(relative_path=bucket.object_name, offset=offset, length=length)))

            for item, tensor in bucket.tensor_data:
                record(item, lambda: torch.save(tensor, writer))
            for item, data in bucket.bytesio_data:
                data.seek(0)
                record(item, lambda: writer.write(data.read()))
            nbytes = writer.tell()
            crcs = self._host_side_checksums(writer, 0, nbytes) if nbytes else None
        if crcs is not None:
            integrity.write_sidecar(str(bucket.object_id), self._crc_chunk_bytes, nbytes, crcs)
        else:
            integrity.remove_sidecar(str(bucket.object_id))
        if replicate_after_write and self._replication_manager is not None:
            self.async_replicate_object(bucket.object_id)
        return results

    def _write_bucket(self, bucket: ObjectWriteBucket, replicate_after_write: bool, xfer: dict) -> list[WriteResult]:
        if not bucket.tensor_data or (not self._use_optimized_save and not any(
                isinstance(t, StagedTensorRef) for _, t in bucket.tensor_data)):
            return self._write_bucket_on_host(bucket, replicate_after_write)
        staged = self._staged_of(bucket)
        if isinstance(staged, RemoteStagedObject):
            # this process only received the bucket: the process that owns the GPU is writing it
            if staged.consumed:
                raise ValueError(f"bucket for '{bucket.object_id}' was already written")
            staged.consumed = True
            return staged.wait(self._remote_wait_timeout_s)
        if staged.future is not None:
            if staged.collected:
                raise ValueError(f"bucket for '{bucket.object_id}' was already written")
            staged.collected = True
            results = staged.future.result()
            try:
                os.remove(staged.done_marker)
            except OSError:
                pass
        else:
            streaming = getattr(self._replication_manager, "async_replicate_streaming", None) if replicate_after_write else None
            results = self._transfer_bucket(staged, bucket, xfer, streaming)
            if streaming is not None:
                return results  # the replication manager has been following the transfer since it began
        if replicate_after_write and self._replication_manager is not None:
            # without a replication manager (single node, or this package used on its own) there is no peer to
            # send to; an explicit async_replicate_object() call still raises
            self.async_replicate_object(bucket.object_id)
        return results

    def _transfer_bucket(self, staged: StagedObject, bucket: ObjectWriteBucket, xfer: dict,
                         streaming=None) -> list[WriteResult]:
        """``streaming``: a replication manager's ``async_replicate_streaming``, called when the transfer begins
        (see ``_announce_transfer``)."""
        outcome: Optional[concurrent.futures.Future] = concurrent.futures.Future() if streaming is not None else None
        try:
            results = self._transfer_bucket_inner(staged, bucket, xfer, streaming, outcome)
        except BaseException as e:
            if outcome is not None and not outcome.done():
                outcome.set_exception(e)  # whoever follows the transfer learns that it will not complete
            raise
        if outcome is not None and not outcome.done():
            outcome.set_result(True)
        return results

    def _announce_transfer(self, streaming, bucket: ObjectWriteBucket, staged: StagedObject, start: int, nbytes: int,
                           outcome: concurrent.futures.Future) -> None:
        """Hands the object to a replication manager that can forward it while it is still being written, where
        the reference hands it over after the write (checkpoint_saver.py:700-707 -> replication_manager.py:248-300).
        The manager is told: the object, the file offset of its data section's first byte (the 4096-byte metadata
        block in front of it is final at this point), a callable that returns how many leading bytes of the data
        section are in place - it only grows - their total, and a future that resolves when the transfer has ended
        (its exception if it failed: the counter then stops short of the total)."""
        try:
            streaming(bucket.object_id, METADATA_SIZE + start, staged.landed_bytes, nbytes, outcome=outcome)
        except Exception:
            _LOGGER.exception("async_replicate_streaming failed for '%s'; the object is written all the same", bucket.object_id)

    def _transfer_bucket_inner(self, staged: StagedObject, bucket: ObjectWriteBucket, xfer: dict, streaming,
                               outcome) -> list[WriteResult]:
        layout = staged.layout
        nbytes = layout.data_bytes
        crcs = None
        marks = [time.perf_counter()]  # -> buffer ready -> bytes in place -> buffer closed -> sidecar -> results
        with self._chkpt_obj_manager.acquire_buffer(
            bucket.object_id, max(self._initial_buffer_size_bytes, nbytes, 1)
        ) as writer:
            writer.set_format_signature(CheckpointFormat.MLF_FORMAT)
            if nbytes:
                ensure = getattr(writer, "ensure_capacity", None)
                if ensure is not None:
                    ensure(nbytes)  # pooled buffers grow once, to the exact total
                reserve = getattr(writer, "reserve", None)
                if reserve is not None:
                    reserve(nbytes)  # pages allocated ahead of the copy threads (first use of a buffer file only)
                marks.append(time.perf_counter())
                with torch.cuda.device(staged.device_index):
                    _lib.check(_lib.load().mlf_hip_set_device(staged.device_index), "mlf_hip_set_device")
                    start = writer.tell()
                    writer.next_buffer_slice(nbytes).release()  # bounds check + position/high-water mark
                    staged.data_offset = start
                    staged._landed.value = 0
                    if streaming is not None:
                        self._announce_transfer(streaming, bucket, staged, start, nbytes, outcome)
                    fd = writer.fileno() if self._use_file_io else -1
                    engine = self._get_engine()
                    if staged.pieces is not None:
                        crcs = self._transfer_image_pieces(staged, writer, start, xfer)
                    elif layout.host_spans:
                        crcs = self._transfer_in_pieces(staged, writer, start, xfer)
                    elif fd >= 0:
                        if staged.plan is not None and staged.plan.crc_chunk_bytes:
                            crcs = self._fused_checksums(staged)
                        elif self._crc_chunk_bytes:
                            crcs = hip_plan.crc32c_device(staged.image, nbytes, self._crc_chunk_bytes, staged.stream)
                        st = engine.d2h_fd(staged.image.data_ptr(), fd, METADATA_SIZE + start, nbytes, staged.stream)
                        self._count_transfer(xfer, st, nbytes)
                    elif staged.plan is not None and staged.plan.crc_chunk_bytes:
                        # the pack folded the checksums: take them now, before the plan (kept for the next save) is
                        # launched again
                        t0 = time.perf_counter()
                        crcs = self._fused_checksums(staged)
                        xfer["crc_s"] = xfer.get("crc_s", 0.0) + time.perf_counter() - t0
                        st, _ = self._send_image(engine, staged, writer.data_address(start), nbytes, 0)
                        self._count_transfer(xfer, st, nbytes)
                    else:
                        # checksum kernels (if asked for) run on the engine's third stream while the chunks cross
                        # the link; the engine keeps the object's progress counter current
                        st, crcs = self._send_image(engine, staged, writer.data_address(start), nbytes,
                                                    self._crc_chunk_bytes)
                        self._count_transfer(xfer, st, nbytes)
                    staged._landed.value = nbytes
                marks.append(time.perf_counter())
            elif streaming is not None:  # an object without data: nothing to follow, but it is to be replicated
                self._announce_transfer(streaming, bucket, staged, 0, 0, outcome)
        staged.consumed = True
        staged.image = None
        if staged.plan is not None and staged.owns_plan:
            staged.plan.destroy()
        staged.plan = None
        marks.append(time.perf_counter())
        if crcs is not None:
            integrity.write_sidecar(str(bucket.object_id), self._crc_chunk_bytes, nbytes, crcs)
        else:
            integrity.remove_sidecar(str(bucket.object_id))
        marks.append(time.perf_counter())
        results = self._results_of(staged, bucket.object_name)
        marks.append(time.perf_counter())
        if len(marks) == 6:  # host time of a write around the transfer itself, for whoever reads last_save_stats
            for name, a, b in (("acquire_s", 0, 1), ("close_s", 2, 3), ("sidecar_s", 3, 4), ("results_s", 4, 5)):
                xfer[name] = xfer.get(name, 0.0) + marks[b] - marks[a]
        return results

    @staticmethod
    def _fused_checksums(staged: StagedObject):
        """The chunk checksums that the pack of ``staged`` left in its plan - unless a later save has launched the
        same (kept) plan since and moved them into ``staged`` before it did."""
        with _FUSED_VALUES_LOCK:  # the writer's thread and the next save's launch may both come for them
            if staged.fused_crcs is None:
                staged.fused_crcs = staged.plan.crc_values()
        return staged.fused_crcs

    @staticmethod
    def _send_image(engine, staged: StagedObject, dst_host_ptr: int, nbytes: int, crc_chunk_bytes: int):
        """The image into the buffer.  The copies wait for the event recorded behind the pack, so a transfer that
        runs on a background thread is not held up by what the training step has put on that stream since."""
        event = staged.packed_event
        if event is not None:
            return engine.d2h_gated(staged.image.data_ptr(), dst_host_ptr, nbytes, event.cuda_event, crc_chunk_bytes,
                                    staged._landed)
        return engine.d2h_watched(staged.image.data_ptr(), dst_host_ptr, nbytes, staged.stream, crc_chunk_bytes,
                                  staged._landed)

    @staticmethod
    def _count_transfer(xfer: dict, st, nbytes: int) -> None:
        xfer["d2h_s"] += st.seconds
        xfer["d2h_wait_s"] += st.wait_seconds
        xfer["d2h_bytes"] += nbytes

    def _host_side_checksums(self, writer, start: int, nbytes: int):
        """Chunk checksums of a data section that was not sent as one image: taken from the pages just written."""
        fd = writer.fileno() if self._crc_chunk_bytes else -1
        if fd < 0:
            return None
        return hip_plan.crc32c_file(fd, METADATA_SIZE + start, nbytes, self._crc_chunk_bytes,
                                    self._engine_config.resolved_copy_threads())

    def _transfer_image_pieces(self, staged: StagedObject, writer, start: int, xfer: dict):
        """The transfer of an image that is held in several device buffers: one after the other, each released as
        soon as it has been sent."""
        engine = self._get_engine()
        nbytes = staged.layout.data_bytes
        sums = integrity.ChunkChecksums(self._crc_chunk_bytes, nbytes) if self._crc_chunk_bytes and nbytes else None
        # the checksum kernels go to the engine's checksum stream: this may be a background thread, and the training
        # step's kernels are queued on the stream the pack ran on
        side = engine.checksum_stream
        spent = []
        for k, (plan, buf, begin, end) in enumerate(staged.pieces):
            pad = begin % _WINDOW_PAD
            dst = writer.data_address(start + begin)
            on_host = sums is not None and self._crc_mode == "host"
            if on_host:
                st, values = engine.d2h_cut(
                    buf.data_ptr() + pad, dst, end - begin, begin, self._crc_chunk_bytes, producer_stream=staged.stream,
                    ready_event=staged.packed_event.cuda_event if staged.packed_event is not None else None)
                sums.add(begin, end - begin, values)
            elif staged.packed_event is not None:
                st, _ = engine.d2h_gated(buf.data_ptr() + pad, dst, end - begin, staged.packed_event.cuda_event, 0,
                                         ctypes.c_uint64(0))
            else:
                st = engine.d2h(buf.data_ptr() + pad, dst, end - begin, staged.stream)
            self._count_transfer(xfer, st, end - begin)
            if sums is not None and not on_host:
                # the piece has left the device, so its pack is over: the side stream may read it at once
                t0 = time.perf_counter()
                sums.add(begin, end - begin, hip_plan.crc32c_device_cut(buf, pad, begin, end - begin,
                                                                         self._crc_chunk_bytes, dst, side))
                xfer["crc_s"] = xfer.get("crc_s", 0.0) + time.perf_counter() - t0
            staged._landed.value = end
            staged.pieces[k] = None
            spent.append(plan)
            del buf  # back to the allocator now: the training step may want the room
        staged.pieces = None
        for plan in spent:  # at the end: releasing device memory waits for the whole device, busy as it may be
            plan.destroy()
        return sums.result() if sums is not None else None

    def _transfer_in_pieces(self, staged: StagedObject, writer, start: int, xfer: dict):
        """The transfer of an object some of whose tensors live in host memory: the runs of the image between them
        cross the host link, the host-resident payloads are copied from where they are into their places in the
        buffer, in the order of the data section.  Returns the chunk checksums or None: taken by the host threads as
        they move each piece (``crc_mode="host"``), else from the pages just written - the image alone is not the
        object, so the kernels cannot give them."""
        layout = staged.layout
        engine = self._get_engine()
        chunk = self._crc_chunk_bytes
        sums = integrity.ChunkChecksums(chunk, layout.data_bytes) if chunk and self._crc_mode == "host" else None
        pieces = [(data_off, n, image_off, None) for image_off, data_off, n in layout.segments]
        pieces += [(data_off, n, None, t) for (data_off, n, _), t in zip(layout.host_spans, layout.host_tensors)]
        t_host = 0.0
        for data_off, n, image_off, tensor in sorted(pieces, key=lambda piece: piece[0]):
            dst = writer.data_address(start + data_off)
            if tensor is None:
                if sums is not None:
                    st, values = engine.d2h_cut(staged.image.data_ptr() + image_off, dst, n, data_off, chunk,
                                                producer_stream=staged.stream)
                    sums.add(data_off, n, values)
                else:
                    st = engine.d2h(staged.image.data_ptr() + image_off, dst, n, staged.stream)
                self._count_transfer(xfer, st, n)
            else:
                t0 = time.perf_counter()
                if isinstance(tensor, torch.Tensor):
                    source = tensor.detach().contiguous()  # a copy only if the tensor is a strided view
                    assert source.numel() * source.element_size() == n
                    address = source.data_ptr()
                else:  # the bytes of a large pickled object
                    source = np.frombuffer(tensor, dtype=np.uint8)
                    assert source.size == n
                    address = source.ctypes.data
                if sums is not None:
                    sums.add(data_off, n, engine.host_copy_cut(dst, address, n, data_off, chunk))
                else:
                    engine.host_copy(dst, address, n)
                t_host += time.perf_counter() - t0
                xfer["host_copy_bytes"] = xfer.get("host_copy_bytes", 0) + n
            staged._landed.value = data_off + n
        xfer["host_copy_s"] = xfer.get("host_copy_s", 0.0) + t_host
        return sums.result() if sums is not None else self._host_side_checksums(writer, start, layout.data_bytes)

    # ---- replication hand-off, metadata, finalize (host logic kept as in the reference) -------------------
    @log_execution_time(logger=_LOGGER, name="async_replicate_object")
    def async_replicate_object(self, object_id: CheckpointObjectId) -> list[concurrent.futures.Future]:
        if self._replication_manager is None:
            raise RuntimeError("ReplicationManager is not available (None). Cannot replicate object.")
        return self._replication_manager.async_replicate(self._chkpt_obj_manager.get_buffer(object_id))

    @override
    @log_execution_time(logger=_LOGGER, name="write_metadata")
    def write_metadata(
        self,
        checkpoint_id: CheckpointContainerId,
        metadata: torchdistmeta.Metadata,
        md_object_name: str = default_metadata_object_name(),
    ):
        final_path = os.path.join(checkpoint_id.data, md_object_name)
        tmp_path = final_path + ".tmp"
        os.makedirs(os.path.dirname(final_path), exist_ok=True)
        with open(tmp_path, "wb") as f, gc_paused():
            pickle.dump(metadata, f)
        os.rename(tmp_path, final_path)

    def write_metadata_bytes(self, checkpoint_id: CheckpointContainerId, pickled: bytes,
                             md_object_name: str = default_metadata_object_name()) -> None:
        """``write_metadata`` for a metadata object that has been pickled already (same temporary name, same
        rename)."""
        final_path = os.path.join(checkpoint_id.data, md_object_name)
        tmp_path = final_path + ".tmp"
        os.makedirs(os.path.dirname(final_path), exist_ok=True)
        with open(tmp_path, "wb") as f:
            f.write(pickled)
        os.rename(tmp_path, final_path)

    def predict_write_results(self, write_buckets: list[ObjectWriteBucket]) -> Optional[list[WriteResult]]:
        """What ``write_data`` is going to return for buckets this saver prepared in this process - offsets and
        lengths are fixed when an object is laid out - or None if any bucket is not of that kind."""
        results: list[WriteResult] = []
        for bucket in write_buckets:
            refs = [t for _, t in bucket.tensor_data]
            if not refs or not all(isinstance(r, StagedTensorRef) for r in refs):
                return None
            staged = refs[0].staged
            if not isinstance(staged, StagedObject) or any(r.staged is not staged for r in refs):
                return None
            results.extend(self._results_of(staged, bucket.object_name))
        return results

    @override
    @log_execution_time(logger=_LOGGER, name="finalize_checkpoint")
    def finalize_checkpoint(self, checkpoint_id: CheckpointContainerId) -> Union[subprocess.Popen, None]:
        self._remove_dirty_checkpoint_marker(checkpoint_id)
        self._barrier_func()
        if self._local_rank_getter() == 0:
            return self._remove_older_checkpoints(older_than=checkpoint_id)
        return None

    def _remove_older_checkpoints(self, older_than: CheckpointContainerId) -> Optional[subprocess.Popen]:
        parent = os.path.dirname(older_than.data)
        limit = CheckpointContainerId.parse_version_container_step(os.path.basename(older_than.data))
        if limit is None:
            _LOGGER.warning("Could not parse step from 'older_than' checkpoint container: '%s'. "
                            "Skipping removal of older checkpoints.", older_than)
            return None
        doomed = []
        for name in os.listdir(parent):
            step = CheckpointContainerId.parse_version_container_step(name)
            path = os.path.join(parent, name)
            if step is not None and step < limit and os.path.isdir(path):
                doomed.append(path)
                sidecars = integrity.sidecar_dir(path)  # the checksums of a removed step go with it
                if os.path.isdir(sidecars):
                    doomed.append(sidecars)
        if not doomed:
            return None
        try:
            # detached `rm -rf`: does not hold the GIL and survives signals sent to the training job's group
            return subprocess.Popen(["rm", "-rf"] + doomed, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL,
                                    start_new_session=True)
        except Exception as e:
            _LOGGER.exception("Background deletion of old checkpoints failed: %s", e)
            return None

    def release_device_memory(self) -> None:
        """Destroys the copy engine (pinned slots, streams) and the plans kept for reuse; both are rebuilt on the
        next save."""
        for name in list(self._plan_cache):
            self._drop_kept_plan(name)
        with self._engine_lock:
            if self._engine is not None:
                self._engine.destroy()
                self._engine = None
                self._engine_clear_of = None
