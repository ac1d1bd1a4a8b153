"""gfx950 implementation of the loader plug-in interface.

The reference reads item by item: ``read()`` copies the record out of the mapping, ``torch.frombuffer`` wraps it,
``narrow_tensor_by_index`` selects the requested box and ``target.copy_()`` moves it (pageable H2D when the target
is on the GPU); src/ml_flashpoint/core/checkpoint_loader.py:177-219,300-336.  Here, per object:

1. record headers are parsed straight from the mapping (a few hundred bytes per item, no payload copy),
2. the byte range that covers all requested payloads is streamed into HBM through pinned slots,
3. one batched scatter kernel writes every requested box into its target tensor, whatever the target's strides.

Items whose target lives on the host, byte-blob items, and objects in the legacy ``torch.save`` format are served
on the host, the way the reference serves them.
"""

import concurrent.futures
import io
import logging
import os
import pickle
import struct
import threading
import time
import warnings
from pathlib import Path
from typing import IO, Callable, List, Optional, cast

import numpy as np
import torch
from torch.distributed._shard._utils import narrow_tensor_by_index
from torch.distributed.checkpoint import Metadata
from torch.distributed.checkpoint.filesystem import _StorageInfo
from torch.distributed.checkpoint.planner import LoadItemType, LoadPlanner, ReadItem
from torch.distributed.checkpoint.utils import _create_file_view
from typing_extensions import override

from ml_flashpoint.checkpoint_object_manager.buffer_metadata import METADATA_SIZE
from ml_flashpoint.checkpoint_object_manager.checkpoint_object_manager import CheckpointObjectManager
from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId, CheckpointObjectId
from ml_flashpoint.core.checkpoint_discovery import CheckpointDiscoveryMixin
from ml_flashpoint.core.checkpoint_loader import MLFlashpointCheckpointLoader
from ml_flashpoint.core.defaults import CheckpointFormat, default_metadata_object_name
from ml_flashpoint.core.mlf_logging import get_logger
from ml_flashpoint.core.utils import gc_paused, log_execution_time
from ml_flashpoint.hip import _lib, integrity
from ml_flashpoint.hip import plan as hip_plan
from ml_flashpoint.hip.checkpoint_saver import EngineConfig

_LOGGER = get_logger(__name__)

_MAX_HEADER_LEN = 1024 * 1024  # a larger "length" means the record is not in the MLF_TENS format
_UPLOAD_ALIGN = 4096
# A read that asks for part of an object (the weights out of weights + optimizer state, say) uploads only the
# neighbourhoods of what it asks for, when that leaves out at least this much; requested ranges closer than the gap
# are fetched together (a range costs about 0.3 ms to set up, the time 17 MB take on the link; measured on the
# weights of the 112 GB shard: 16 MiB 0.41 s, 128 MiB 0.47 s).
_PARTIAL_READ_MIN_SAVING = 256 << 20
# a host-resident target of at least this size is filled by the copy engine's threads instead of one ``copy_``
_HOST_COPY_ON_THE_ENGINE_FROM = 8 << 20
# neighbourhoods that share a device buffer start on this boundary in it (uploads to less aligned device addresses
# were measured at half the link's rate)
_SLICE_ALIGN = 2 << 20
_PARTIAL_READ_GAP = 16 << 20
# a restore through windows alternates between two device buffers (one is unpacked while the other is filled) when
# each can hold at least this much
_PIPELINED_MIN_WINDOW = 128 << 10
# a range of at least _PIPELINED_FROM_BYTES is restored through two alternating buffers by choice: a quarter of the
# range for both together, within these bounds (measured on the 112 GB shard: 2 x 16 GB 2.03 s, 2 x 8 GB 2.055 s,
# 2 x 2 GB 2.095 s, one image of 112 GB 2.06-2.10 s)
_PIPELINED_FROM_BYTES = 8 << 30
_PIPELINED_MIN_BYTES = 2 << 30
_PIPELINED_MAX_BYTES = 32 << 30
_U32 = struct.Struct("<I")
_HEADER_CACHE: dict = {}  # header pickle bytes -> (dtype, shape, stored payload bytes)
_ESZ_CACHE: dict = {}


def _element_size(dtype: torch.dtype) -> int:
    esz = _ESZ_CACHE.get(dtype)
    if esz is None:
        esz = _ESZ_CACHE[dtype] = torch.empty((), dtype=dtype).element_size()
    return esz


class HipMLFlashpointCheckpointLoader(CheckpointDiscoveryMixin, MLFlashpointCheckpointLoader):
    def __init__(
        self,
        checkpoint_object_manager: CheckpointObjectManager,
        replication_manager=None,
        *,
        global_rank_getter: Callable[[], int] = lambda: 0,
        local_rank_getter: Callable[[], int] = lambda: 0,
        broadcast_object_list_func: Optional[Callable[..., None]] = None,
        all_gather_object_func: Optional[Callable[..., None]] = None,
        world_size_getter: Callable[[], int] = lambda: 1,
        engine_config: Optional[EngineConfig] = None,
        tile_bytes: int = 0,
        block_threads: int = 0,
        verify_crc: bool = True,
        crc_mode: str = "before",
        use_file_io: bool = True,
        verify_on_discovery: bool = False,
        max_image_bytes: Optional[int] = None,
        pipelined_restore: bool = True,
    ):
        """Arguments as the reference's default loader (checkpoint_loader.py:126-158), plus the copy-engine and
        kernel work-split knobs, ``verify_crc`` (check the CRC-32C sidecar of an object, when it has one, while
        restoring it), ``crc_mode`` (when it is checked.  ``"before"``, the default: no byte reaches a target, or the
        planner, before the chunk it lies in has been checked - a checksum pass over every uploaded range or window
        ahead of its unpack, a host-side check ahead of every item that is served on the host; after a
        ``ChecksumMismatchError`` the targets hold what they held before, or, where earlier windows of the object
        had already passed, verified bytes of this checkpoint - never corrupt ones.  ``"fused"``: the unpack kernel
        folds the checksums of the image it scatters, so the image is read once, and a mismatch is reported after
        the targets were written - for callers that discard the targets on any error) and
        ``verify_on_discovery`` (also check it, on the host, while choosing the checkpoint to
        recover from, so that a corrupted copy counts as missing) and ``max_image_bytes`` (largest range of an
        object that is uploaded to HBM in one piece; default: what the device has free minus 2 GiB.  A larger
        range is restored window by window through buffers of that size together) and ``pipelined_restore`` (a
        range of 8 GiB or more goes through two alternating buffers - a quarter of the range together, 32 GiB at
        most - by choice: one window is unpacked while the next crosses the link, and the restore needs that much
        HBM instead of room for the whole range.  False: one buffer for the whole range where it fits)."""
        _lib.load()
        self._checkpoint_object_manager = checkpoint_object_manager
        self._replication_manager = replication_manager
        self._global_rank_getter = global_rank_getter
        self._local_rank_getter = local_rank_getter
        self._broadcast_object_list_func = broadcast_object_list_func
        self._all_gather_object_func = all_gather_object_func
        self._world_size_getter = world_size_getter
        self._engine_config = engine_config or EngineConfig()
        self._tile_bytes = tile_bytes
        self._block_threads = block_threads
        self._verify_crc = verify_crc
        if crc_mode not in ("fused", "before"):
            raise ValueError("crc_mode must be 'fused' or 'before'")
        self._crc_mode = crc_mode
        # pread() the buffer file into the pinned slots instead of reading through the (fresh, read-only) mapping:
        # reads of tmpfs run in parallel, and no page-table entry per 4 KiB has to be built and torn down
        self._use_file_io = use_file_io
        self.verify_on_discovery = verify_on_discovery
        self._max_image_bytes = max_image_bytes
        self._pipelined_restore = pipelined_restore
        self._engine: Optional[hip_plan.CopyEngine] = None
        self._engine_clear_of: Optional[int] = None
        self._engine_lock = threading.Lock()
        self._stats_local = threading.local()  # read_data runs on one executor thread per object
        self._init_discovery()
        self.last_load_stats: dict = {}
        # set to True to bracket every unpack launch with timing events; see the saver's attribute of the same name
        self.record_kernel_events = False
        self.kernel_events: list = []

    @property
    def _stats_in_progress(self) -> dict:
        stats = getattr(self._stats_local, "current", None)
        if stats is None:
            stats = self._stats_local.current = {}
        return stats

    def _get_engine(self) -> hip_plan.CopyEngine:
        with self._engine_lock:  # read_data runs on one executor thread per object
            if self._engine is None:
                cfg = self._engine_config
                self._engine = hip_plan.CopyEngine(cfg.slot_bytes, cfg.n_slots, cfg.resolved_copy_threads())
            return self._engine

    def _keep_clear_of(self, device: torch.device) -> None:
        """Once per engine: its streams off the hardware queue of the stream that is current on ``device`` (the one the
        unpack runs on, and whatever else the process keeps busy there); see the saver's ``warm_up``."""
        engine = self._get_engine()
        with self._engine_lock:
            if self._engine_clear_of is not None:
                return
            self._engine_clear_of = torch.cuda.current_stream(device).cuda_stream
        left = engine.avoid_stream(self._engine_clear_of)
        if left:
            _LOGGER.warning("%d of the copy engine's streams share a hardware queue with the current stream", left)

    @override
    @log_execution_time(logger=_LOGGER, name="read_metadata")
    def read_metadata(
        self,
        checkpoint_id: CheckpointContainerId,
        object_name: str = default_metadata_object_name(),
    ) -> Metadata:
        path = Path(checkpoint_id.data) / object_name
        try:
            with open(path, "rb") as f, gc_paused():  # unpickling creates ~5 objects per item and no cycles
                return pickle.load(f)
        except Exception:
            _LOGGER.exception("Error reading metadata from '%s'", path)
            raise

    # ---- host-side record access ----------------------------------------------------------------------
    def read_tensor(self, buffer_slice: IO[bytes], req: ReadItem, use_optimized_loader: bool = False) -> torch.Tensor:
        """Host read of one record into a CPU tensor, narrowed to the requested box.  Used for host-resident
        targets and for objects in the legacy format (same steps as checkpoint_loader.py:177-219)."""
        pos = buffer_slice.tell()
        tensor: Optional[torch.Tensor] = None
        if use_optimized_loader:
            raw_len = buffer_slice.read(4)
            if len(raw_len) == 4:
                (header_len,) = struct.unpack("<I", raw_len)
                if header_len < _MAX_HEADER_LEN:
                    try:
                        header = pickle.loads(buffer_slice.read(header_len))
                        data = buffer_slice.read()
                        with warnings.catch_warnings():  # `data` is immutable and the tensor over it is only read
                            warnings.filterwarnings("ignore", message="The given buffer is not writable")
                            tensor = torch.frombuffer(data, dtype=header.dtype).reshape(header.shape)
                    except Exception:
                        _LOGGER.exception("Failed to parse tensor header")
                        raise
        if tensor is None:
            buffer_slice.seek(pos)
            tensor = cast(torch.Tensor, torch.load(cast(IO[bytes], buffer_slice), map_location="cpu", weights_only=True))
        return narrow_tensor_by_index(tensor, req.storage_offsets, req.lengths)

    @staticmethod
    def _parse_header(view: memoryview, offset: int, length: int):
        """(dtype, shape, payload offset) of the record at data-section ``offset``; None if it is not MLF_TENS.
        Identical header bytes (same dtype and shape) are unpickled once."""
        base = METADATA_SIZE + offset
        if length < 4:
            return None
        (header_len,) = _U32.unpack_from(view, base)
        if header_len >= _MAX_HEADER_LEN or 4 + header_len > length:
            return None
        raw = bytes(view[base + 4 : base + 4 + header_len])
        parsed = _HEADER_CACHE.get(raw)
        if parsed is None:
            header = pickle.loads(raw)
            parsed = (header.dtype, header.shape, header.shape.numel() * _element_size(header.dtype))
            if len(_HEADER_CACHE) < 1 << 16:
                _HEADER_CACHE[raw] = parsed
        return parsed[0], parsed[1], offset + 4 + header_len, parsed[2]

    @staticmethod
    def _payload_view(whole: memoryview, written: int, object_id, req, dtype, shape, payload_off: int, stored_bytes: int):
        """A host tensor over a record's payload where it lies in the (read-only) mapping: nothing is copied."""
        if payload_off + stored_bytes > written:
            raise ValueError(f"req {req.storage_index}: record reaches past the written data of '{object_id.data}'")
        if stored_bytes == 0:
            return torch.empty(shape, dtype=dtype)
        with warnings.catch_warnings():  # the mapping is read-only and the tensor over it is only read
            warnings.filterwarnings("ignore", message="The given buffer is not writable")
            flat = torch.frombuffer(whole, dtype=dtype, count=shape.numel(), offset=METADATA_SIZE + payload_off)
        return flat.reshape(shape)

    # ---- read_data ------------------------------------------------------------------------------------
    @override
    @log_execution_time(logger=_LOGGER, name="read_data", level=logging.INFO)
    def read_data(
        self,
        checkpoint_object_id: CheckpointObjectId,
        read_items: List[ReadItem],
        planner: LoadPlanner,
        storage_data: dict[int, _StorageInfo],
    ) -> None:
        if not os.path.exists(checkpoint_object_id.data) and not self._try_retrieve_object_if_missing(checkpoint_object_id):
            msg = f"Checkpoint object '{checkpoint_object_id.data}' does not exist on any node in the cluster"
            _LOGGER.error(msg)
            raise FileNotFoundError(msg)
        t_start = time.perf_counter()
        stats = {"h2d_s": 0.0, "h2d_bytes": 0, "device_payload_bytes": 0, "host_items": 0, "device_items": 0}
        self._stats_local.current = stats
        with gc_paused(), self._checkpoint_object_manager.get_buffer(checkpoint_object_id) as stream:
            recorded, held = stream.len_written_data, stream.buffer_obj.get_capacity() - METADATA_SIZE
            if recorded > held:  # cut short after it was written: never read past the end of the file or its mapping
                raise ValueError(f"'{checkpoint_object_id.data}' is truncated: its metadata block records {recorded} "
                                 f"bytes of data, the file holds {held}")
            optimized = stream.format_signature == CheckpointFormat.MLF_FORMAT
            whole = stream.raw_view()
            sidecar = integrity.read_sidecar(checkpoint_object_id.data) if self._verify_crc else None
            if sidecar is not None and sidecar[1] != recorded:
                raise integrity.ChecksumMismatchError(
                    f"'{checkpoint_object_id.data}': sidecar covers {sidecar[1]} bytes, object holds {recorded}")
            host_checked: set = set()  # chunks already checked on the host for items served there

            def check_on_host_first(offset: int, length: int) -> None:
                """crc_mode "before": the chunks an item lies in are checked before the item is handed out."""
                if sidecar is None or self._crc_mode != "before" or length <= 0:
                    return
                chunk = sidecar[0]
                todo = sorted(set(range(offset // chunk, (offset + length - 1) // chunk + 1)) - host_checked)
                self._check_on_host(checkpoint_object_id, stream, sidecar, todo)
                host_checked.update(todo)

            resolved: dict = {}  # id(request) -> target, for the requests whose target was looked at ahead of time
            early = self._start_early_upload(stream, read_items, planner, storage_data, recorded, sidecar, stats,
                                             resolved) if optimized else None
            try:
                self._serve_items(checkpoint_object_id, stream, read_items, planner, storage_data, optimized, whole,
                                  recorded, sidecar, check_on_host_first, stats, early, resolved)
            finally:
                if early is not None:  # the file and its mapping are closed below: nothing may still be reading them
                    concurrent.futures.wait([early[1]])
        stats["read_s"] = time.perf_counter() - t_start
        self.last_load_stats = stats

    def _start_early_upload(self, stream, read_items, planner, storage_data, recorded: int, sidecar, stats,
                            resolved: dict):
        """Where the records that are asked for lie in the object is known from the checkpoint's metadata, so when
        they are going to be read through one device buffer in one piece - the whole data section if the object has
        checksums - the upload can begin before the record headers are parsed and the targets resolved (5 us per
        item on the host: 110 ms for 20 000 items, beside an upload of 150 ms).  Returns ``(buffer, future of the
        upload, device, first byte, end)`` when the read is certain to be of that kind, else None.  Targets it had to
        resolve to learn the device are left in ``resolved`` (a planner is asked for every target once)."""
        asked = {req.storage_index: storage_data[req.storage_index]
                 for req in read_items if req.type != LoadItemType.BYTE_IO}
        if not asked or recorded <= 0:
            return None
        if sidecar is not None:
            lo, hi = 0, recorded  # checksums cover the whole data section
        else:
            lo = min(info.offset for info in asked.values()) // _UPLOAD_ALIGN * _UPLOAD_ALIGN
            hi = min(max(info.offset + info.length for info in asked.values()), recorded)
        span = hi - lo
        if span <= 0 or (span >= _PIPELINED_FROM_BYTES and self._pipelined_restore):
            return None
        # a read that leaves out enough of the range to be worth several smaller uploads is decided on later
        if span - sum(info.length for info in asked.values()) + 256 * len(asked) >= _PARTIAL_READ_MIN_SAVING:
            return None
        # the device the targets live on: a sample of the requests says.  An object with host-resident targets among
        # them is left to the ordinary way, which uploads only what the device targets need.
        wanted = [req for req in read_items if req.type != LoadItemType.BYTE_IO]
        device = None
        for req in wanted[:: max(1, len(wanted) // 32)][:33]:
            resolved[id(req)] = planner.resolve_tensor(req).detach()
            if device is None:
                device = resolved[id(req)].device
            if resolved[id(req)].device != device or device.type == "cpu":
                return None
        with torch.cuda.device(device):
            _lib.check(_lib.load().mlf_hip_set_device(device.index or 0), "mlf_hip_set_device")
            self._keep_clear_of(device)
            image = hip_plan.try_allocate(span, device) if span <= self._image_limit(device) else None
            if image is None:
                return None
            cur = torch.cuda.current_stream(device)
        done: concurrent.futures.Future = concurrent.futures.Future()

        def run():
            try:
                self._upload(stream, lo, image, span, cur, stats)
                done.set_result(None)
            except BaseException as e:  # handed to whoever waits for the bytes
                done.set_exception(e)

        threading.Thread(target=run, name="mlf-early-upload", daemon=True).start()
        stats["upload_began_before_parse"] = 1
        return image, done, device, lo, hi

    def _serve_items(self, checkpoint_object_id, stream, read_items, planner, storage_data, optimized, whole, recorded,
                     sidecar, check_on_host_first, stats, early, resolved: dict) -> None:
        """Items for the host are served one by one; those for the device are collected and restored together."""
        device_reqs = []  # (req, target, dtype, shape, payload_off, stored payload bytes)
        t_parse = time.perf_counter()
        for req in read_items:
            item_md = storage_data[req.storage_index]
            if req.type == LoadItemType.BYTE_IO:
                check_on_host_first(item_md.offset, item_md.length)
                view = cast(IO[bytes], _create_file_view(stream, item_md.offset, item_md.length))
                data = io.BytesIO(view.read(item_md.length))
                data.seek(0)
                planner.load_bytes(req, data)
                continue
            target = resolved.pop(id(req), None)
            if target is None:
                target = planner.resolve_tensor(req).detach()
            parsed = self._parse_header(whole, item_md.offset, item_md.length) if optimized else None
            if parsed is not None and target.device.type == "cpu":
                # host-resident target: one copy, from a tensor laid over the record's payload in the mapping
                # into the target (the reference reads the record into a bytes object first,
                # checkpoint_loader.py:195-208)
                check_on_host_first(item_md.offset, item_md.length)
                tensor = self._payload_view(whole, recorded, checkpoint_object_id, req, *parsed)
                tensor = narrow_tensor_by_index(tensor, req.storage_offsets, req.lengths)
                assert target.size() == tensor.size(), (
                    f"req {req.storage_index} mismatch sizes {target.size()} vs {tensor.size()}"
                )
                nbytes = tensor.numel() * tensor.element_size()
                if (nbytes >= _HOST_COPY_ON_THE_ENGINE_FROM and tensor.dtype == target.dtype and tensor.is_contiguous()
                        and target.is_contiguous()):
                    # a large one (optimizer state kept in host memory): read from the file by the copy engine's
                    # threads, straight into the target - a copy out of the mapping would take a page fault per
                    # 4 KiB of it
                    first = tensor.data_ptr() - (stream.data_address(0) - METADATA_SIZE)  # its place in the file
                    self._get_engine().read_file(stream.fileno(), first, target.data_ptr(), nbytes)
                else:
                    target.copy_(tensor)
                planner.commit_tensor(req, target)
                stats["host_items"] += 1
                continue
            if parsed is None:
                check_on_host_first(item_md.offset, item_md.length)
                view = cast(IO[bytes], _create_file_view(stream, item_md.offset, item_md.length))
                tensor = self.read_tensor(view, req, use_optimized_loader=optimized)
                assert target.size() == tensor.size(), (
                    f"req {req.storage_index} mismatch sizes {target.size()} vs {tensor.size()}"
                )
                target.copy_(tensor)
                planner.commit_tensor(req, target)
                stats["host_items"] += 1
                continue
            device_reqs.append((req, target) + parsed)
        stats["parse_s"] = time.perf_counter() - t_parse  # headers parsed, targets resolved, host items served
        if device_reqs:
            self._read_device_items(checkpoint_object_id, stream, device_reqs, planner, stats, sidecar, early)

    def _image_limit(self, device: torch.device) -> int:
        """Bytes of HBM one uploaded range may take: the explicit limit, or what the device and torch's allocator
        have free minus a margin for the tables and for whatever else allocates while the restore runs."""
        if self._max_image_bytes is not None:
            return max(self._max_image_bytes, 1)
        free, _ = torch.cuda.mem_get_info(device)
        cached = torch.cuda.memory_reserved(device) - torch.cuda.memory_allocated(device)
        return max(free + cached - (2 << 30), 64 << 20)

    def _read_device_items(self, object_id, stream, device_reqs, planner, stats, sidecar, early=None) -> None:
        devices = {t.device for _, t, *_ in device_reqs}
        if len(devices) != 1 or (early is not None and early[2] not in devices):
            raise ValueError("all device targets of one checkpoint object must live on the same device")
        device = devices.pop()
        written = stream.len_written_data

        # Every request becomes one row: where its bytes lie in the data section ([first, last), absolute for now)
        # and how to add it to a descriptor table once the offset of the uploaded range is known.  A request for a
        # whole stored tensor into a contiguous target (the common case) is one run of bytes; anything else is a box
        # over the stored C-contiguous payload (offsets/strides) with the target's strides on the other side.
        t_rows = time.perf_counter()
        rows = []  # (first, last, contiguous?, table arguments)
        conversions = []  # (target, buffer of the stored dtype): the reference's `copy_` converts, so this does too
        for req, target, dtype, shape, payload_off, stored_bytes in device_reqs:
            if target.dtype != dtype or (target.dim() > _lib.MAX_DIMS and not target.is_contiguous()
                                         and not hip_plan.describable(tuple(target.shape), tuple(target.stride()))):
                # restored bit-exact into a contiguous buffer of the stored dtype; torch's ``copy_`` converts, or
                # scatters into a view of more dimensions than a descriptor holds, on the device afterwards, on the
                # stream the unpack runs on (checkpoint_loader.py:335 does the same ``copy_`` on the host)
                stored_as = torch.empty(target.size(), dtype=dtype, device=device)
                conversions.append((target, stored_as))
                target = stored_as
            if payload_off + stored_bytes > written:
                raise ValueError(f"req {req.storage_index}: record reaches past the written data of '{object_id.data}'")
            esz = _element_size(dtype)
            ndim = len(shape)
            req_lengths = req.lengths
            # a dimension is narrowed only where the requested length is smaller than the stored size
            narrowed = any(l < sz for l, sz in zip(req_lengths, shape))
            if not narrowed:
                assert target.size() == shape, f"req {req.storage_index} mismatch sizes {target.size()} vs {shape}"
                if stored_bytes == 0:
                    continue
                first, last = payload_off, payload_off + stored_bytes
                if target.is_contiguous():
                    rows.append((first, last, True, (target.data_ptr(), esz)))
                else:  # (a view of too many dimensions was replaced by a contiguous stand-in above)
                    rows.append((first, last, False, (target.data_ptr(), esz, tuple(shape), tuple(target.stride()), None)))
            else:
                stored_strides = hip_plan._contiguous_strides(tuple(shape))
                lengths = [l if l < sz else sz for l, sz in zip(req_lengths, shape)]
                offsets = [o if l < sz else 0 for o, l, sz in zip(req.storage_offsets, req_lengths, shape)]
                lengths += list(shape[len(lengths):])
                offsets += [0] * (ndim - len(offsets))
                box_shape = torch.Size(lengths)
                assert target.size() == box_shape, f"req {req.storage_index} mismatch sizes {target.size()} vs {box_shape}"
                numel = box_shape.numel()
                if numel == 0:
                    continue
                box = (tuple(lengths), tuple(target.stride()), tuple(stored_strides))
                if ndim > _lib.MAX_DIMS:
                    box = hip_plan.collapse_dims(*box)
                    if len(box[0]) > _lib.MAX_DIMS:
                        # a box that is narrowed in so many dimensions that no merging helps: into a contiguous
                        # stand-in of the box's shape first (its strides merge wherever the stored ones do)
                        stored_as = torch.empty(box_shape, dtype=dtype, device=device)
                        conversions.append((target, stored_as))
                        target = stored_as
                        box = hip_plan.collapse_dims(tuple(lengths), tuple(target.stride()), tuple(stored_strides))
                        if len(box[0]) > _lib.MAX_DIMS:
                            raise ValueError(f"req {req.storage_index}: a sub-box of {len(box[0])} dimensions after merging "
                                             f"does not fit the descriptor table's {_lib.MAX_DIMS}")
                first = payload_off + sum(o * st for o, st in zip(offsets, stored_strides)) * esz
                last = first + (sum((l - 1) * st for l, st in zip(lengths, stored_strides)) + 1) * esz
                rows.append((first, last, False, (target.data_ptr(), esz) + box))
                stored_bytes = numel * esz
            stats["device_payload_bytes"] += stored_bytes
        stats["table_s"] = time.perf_counter() - t_rows
        if rows:
            lo = min(r[0] for r in rows)
            hi = max(r[1] for r in rows)
            if sidecar is not None:
                lo, hi = 0, written  # checksums cover the whole data section
            lo = lo // _UPLOAD_ALIGN * _UPLOAD_ALIGN
            clusters = None
            if early is not None and early[3] <= lo and hi <= early[4]:  # the range is already on its way into a buffer
                with torch.cuda.device(device):
                    self._restore_range(object_id, stream, device, rows, early[3], early[4], sidecar, stats, early[0], early[1])
                    for target, stored_as in conversions:
                        target.copy_(stored_as)
                rows = []
            elif (hi - lo) - sum(r[1] - r[0] for r in rows) >= _PARTIAL_READ_MIN_SAVING:
                clusters = self._clusters_of(rows, sidecar[0] if sidecar is not None else None, written)
                if (hi - lo) - sum(c_hi - c_lo for c_lo, c_hi, _ in clusters) < _PARTIAL_READ_MIN_SAVING:
                    clusters = None
        if rows:
            with torch.cuda.device(device):
                _lib.check(_lib.load().mlf_hip_set_device(device.index or 0), "mlf_hip_set_device")
                self._keep_clear_of(device)
                limit = self._image_limit(device)
                # one buffer for the range (or for the largest neighbourhood of a partial read) if the allocator
                # has a block of that size; through a smaller buffer, window by window, if it has not
                image = None
                if clusters is not None:
                    # all neighbourhoods side by side in one buffer (one unpack for all of them), or one after
                    # the other through a buffer for the largest
                    for need in (sum(-(-(c_hi - c_lo) // _SLICE_ALIGN) * _SLICE_ALIGN for c_lo, c_hi, _ in clusters),
                                 max(c_hi - c_lo for c_lo, c_hi, _ in clusters)):
                        image = hip_plan.try_allocate(need, device) if need <= limit else None
                        if image is not None:
                            break
                    need = min(need, limit)
                else:
                    need = hi - lo
                    through = self._pipelined_limit(need, limit, rows, sidecar)
                    if through:
                        # a large range by choice through two modest buffers: one window is unpacked while the next
                        # crosses the link, and the restore needs that much HBM instead of room for the whole range
                        self._restore_windowed(object_id, stream, device, rows, through, sidecar, stats, by_choice=True)
                        image = False
                    else:
                        image = hip_plan.try_allocate(need, device) if need <= limit else None
                if image is False:
                    pass
                elif image is None:
                    self._restore_windowed(object_id, stream, device, rows, min(limit, need), sidecar, stats)
                elif clusters is not None:
                    self._restore_clusters(object_id, stream, device, clusters, sidecar, stats, image)
                else:
                    self._restore_range(object_id, stream, device, rows, lo, hi, sidecar, stats, image)
                del image
                for target, stored_as in conversions:
                    target.copy_(stored_as)
        t_commit = time.perf_counter()
        for req, target, *_ in device_reqs:
            planner.commit_tensor(req, target)
        stats["commit_s"] = time.perf_counter() - t_commit
        stats["device_items"] += len(device_reqs)

    @staticmethod
    def _table_of(rows, lo: int):
        """Descriptor table of ``rows`` for a buffer that holds the data section from byte ``lo`` on."""
        table = hip_plan.ItemTable()
        for first, last, contiguous, args in rows:
            if contiguous:
                ptr, esz = args
                table.add_contiguous(ptr, first - lo, esz, last - first)
            else:
                ptr, esz, shape, strides, image_strides = args
                table.add_device(ptr, first - lo, esz, shape, strides, image_stride=image_strides)
        return table.to_array()

    def _upload(self, stream, lo: int, image: torch.Tensor, span: int, cur, stats) -> None:
        fd = stream.fileno() if self._use_file_io else -1
        if fd >= 0:
            st = self._get_engine().h2d_fd(fd, METADATA_SIZE + lo, image.data_ptr(), span, cur.cuda_stream)
        else:
            st = self._get_engine().h2d(stream.data_address(lo), image.data_ptr(), span, cur.cuda_stream)
        stats["h2d_s"] += st.seconds
        stats["h2d_host_s"] = stats.get("h2d_host_s", 0.0) + st.wait_seconds  # filling the pinned slots
        stats["h2d_bytes"] += span

    def _unpack_plan(self, items, span: int, crc_chunk_bytes: int = 0, booked_as: str = "unpack_plan_s") -> hip_plan.Plan:
        t0 = time.perf_counter()
        plan = hip_plan.Plan(items, b"", span, tile_bytes=self._tile_bytes, block_threads=self._block_threads,
                             align_to_tensor=True, crc_chunk_bytes=crc_chunk_bytes)
        stats = self._stats_in_progress
        stats[booked_as] = stats.get(booked_as, 0.0) + time.perf_counter() - t0
        return plan

    def _launch_unpack(self, plan: hip_plan.Plan, image: torch.Tensor, cur, payload_bytes: int) -> torch.cuda.Event:
        """Enqueues the unpack on ``cur`` and returns the event recorded behind it: until it has passed, the image
        is still being read and the plan's tables are in use."""
        if self.record_kernel_events:
            begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            begin.record(cur)
            plan.unpack(image, cur.cuda_stream)
            end.record(cur)
            self.kernel_events.append((begin, end, payload_bytes))
            return end
        plan.unpack(image, cur.cuda_stream)
        done = torch.cuda.Event()
        done.record(cur)
        return done

    def _unpack(self, items, image: torch.Tensor, span: int, cur, payload_bytes: int, crc_chunk_bytes: int = 0):
        """Launches the unpack of ``items`` out of ``image`` and waits for it: the targets are complete, and the
        image may be reused or freed, when this returns.  With ``crc_chunk_bytes`` the unpack kernel also folds the
        CRC-32C of every chunk of the image; those values are returned."""
        plan = self._unpack_plan(items, span, crc_chunk_bytes)
        stats = self._stats_in_progress
        t0 = time.perf_counter()
        try:
            if self.record_kernel_events:
                begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                begin.record(cur)
                plan.unpack(image, cur.cuda_stream)
                end.record(cur)
                self.kernel_events.append((begin, end, payload_bytes))
            else:
                plan.unpack(image, cur.cuda_stream)
            cur.synchronize()
            stats["unpack_s"] = stats.get("unpack_s", 0.0) + time.perf_counter() - t0
            return plan.crc_values() if crc_chunk_bytes else None
        finally:
            plan.destroy()

    def _restore_range(self, object_id, stream, device, rows, lo, hi, sidecar, stats, image, uploaded=None) -> None:
        """One upload of [lo, hi) into ``image`` (``uploaded``: the future of one that was started earlier),
        checksum on the GPU if the object has a sidecar, one unpack."""
        span = hi - lo
        cur = torch.cuda.current_stream(device)
        if uploaded is not None:
            uploaded.result()
        else:
            self._upload(stream, lo, image, span, cur, stats)
        if sidecar is not None:
            chunk_bytes, data_bytes, want = sidecar
            if self._crc_mode == "fused" and chunk_bytes % 65536 == 0 and data_bytes == span:
                got = self._unpack(self._table_of(rows, lo), image, span, cur, stats["device_payload_bytes"], chunk_bytes)
                self._compare_checksums(object_id, got, want, chunk_bytes)
                return
            t0 = time.perf_counter()
            got = hip_plan.crc32c_device(image, data_bytes, chunk_bytes, cur.cuda_stream)
            stats["crc_s"] = stats.get("crc_s", 0.0) + time.perf_counter() - t0
            self._compare_checksums(object_id, got, want, chunk_bytes)
        self._unpack(self._table_of(rows, lo), image, span, cur, stats["device_payload_bytes"])

    @staticmethod
    def _compare_checksums(object_id, got, want, chunk_bytes, first_chunk: int = 0, n_chunks: Optional[int] = None) -> None:
        bad = [first_chunk + int(i) for i in (got != want).nonzero()[0]]
        if bad:
            raise integrity.ChecksumMismatchError(
                f"'{object_id.data}': CRC-32C mismatch in chunk(s) {bad[:8]} of {n_chunks if n_chunks is not None else len(want)} "
                f"(chunk size {chunk_bytes})")

    @staticmethod
    def _clusters_of(rows, chunk_bytes: Optional[int], written: int):
        """Groups the requested rows into ranges of the data section that are worth one upload each: rows closer than
        the gap go together; a range starts and ends on upload boundaries - on checksum chunks when the object has a
        sidecar, so that every chunk that is read can be checked.  Returns [(lo, hi, rows)], ascending, disjoint."""
        align = chunk_bytes or _UPLOAD_ALIGN
        clusters = []
        for row in sorted(rows, key=lambda r: r[0]):
            lo = row[0] // align * align
            hi = min(-(-row[1] // align) * align, written) if chunk_bytes else row[1]
            if clusters and lo - clusters[-1][1] <= _PARTIAL_READ_GAP:
                clusters[-1][1] = max(clusters[-1][1], hi)
                clusters[-1][2].append(row)
            else:
                clusters.append([lo, hi, [row]])
        return [(lo, hi, members) for lo, hi, members in clusters]

    def _restore_clusters(self, object_id, stream, device, clusters, sidecar, stats, image) -> None:
        """A partial read: every cluster is uploaded into ``image`` and checked against the sidecar's values for
        exactly the chunks it covers.  If ``image`` has room for all clusters they lie side by side and one unpack
        serves them all; otherwise they pass through it one at a time.  What the request does not touch is
        neither read nor checked."""
        cur = torch.cuda.current_stream(device)
        bases, at = [], 0
        for lo, hi, _ in clusters:
            bases.append(at)
            at += -(-(hi - lo) // _SLICE_ALIGN) * _SLICE_ALIGN
        together = at <= image.numel()
        chunk_bytes, want = (sidecar[0], sidecar[2]) if sidecar is not None else (0, None)
        # side by side, every neighbourhood starting on a chunk boundary of the buffer: one checksum pass over the
        # buffer yields all their chunks (and some over the padding between them, which nobody looks at)
        one_pass = together and sidecar is not None and all(base % chunk_bytes == 0 for base in bases)
        tables = []
        for (lo, hi, members), base in zip(clusters, bases if together else [0] * len(clusters)):
            span = hi - lo
            part = image[base : base + span]
            self._upload(stream, lo, part, span, cur, stats)
            if sidecar is not None and not one_pass:
                got = hip_plan.crc32c_device(part, span, chunk_bytes, cur.cuda_stream)
                first = lo // chunk_bytes
                self._compare_checksums(object_id, got, want[first : first + len(got)], chunk_bytes, first, len(want))
            if together:
                tables.append(self._table_of(members, lo - base))
            else:
                self._unpack(self._table_of(members, lo), image, span, cur, sum(r[1] - r[0] for r in members if r[2]))
        if one_pass:
            last_lo, last_hi, _ = clusters[-1]
            got = hip_plan.crc32c_device(image, bases[-1] + (last_hi - last_lo), chunk_bytes, cur.cuda_stream)
            for (lo, hi, _), base in zip(clusters, bases):
                n, first = -(-(hi - lo) // chunk_bytes), lo // chunk_bytes
                at_buffer = base // chunk_bytes
                self._compare_checksums(object_id, got[at_buffer : at_buffer + n], want[first : first + n], chunk_bytes,
                                        first, len(want))
        if together:
            self._unpack(np.concatenate(tables), image, at, cur, stats["device_payload_bytes"])
        stats["partial_read_ranges"] = stats.get("partial_read_ranges", 0) + len(clusters)

    def _pipelined_limit(self, need: int, limit: int, rows, sidecar) -> int:
        """HBM to restore a range of ``need`` bytes through, in two alternating buffers, when that is the better way
        (0 when one buffer for the whole range is): the range is large, the checksums can be checked window by
        window, and no row that must stay whole is larger than a window."""
        if need < _PIPELINED_FROM_BYTES or not self._pipelined_restore:
            return 0
        chunk_bytes = 0
        if sidecar is not None:
            chunk_bytes = sidecar[0]
            if chunk_bytes % (65536 if self._crc_mode == "fused" else _UPLOAD_ALIGN):
                return 0
        through = min(limit, max(_PIPELINED_MIN_BYTES, min(_PIPELINED_MAX_BYTES, need // 4)))
        window = through // 2 - 2 * max(chunk_bytes, _UPLOAD_ALIGN)
        uncut = max((r[1] - r[0] for r in rows if not r[2]), default=0)
        if window < max(uncut, 4 * chunk_bytes, _PIPELINED_MIN_WINDOW):
            return 0
        return through

    def _restore_windowed(self, object_id, stream, device, rows, limit, sidecar, stats, by_choice: bool = False) -> None:
        """Fallback for an object whose requested range does not fit in HBM beside the live state: the rows are
        sorted by position and restored window by window through one device buffer of at most ``limit`` bytes.  A
        contiguous row larger than a window is cut into pieces, a strided one or a sub-box into smaller boxes.

        With a sidecar every window starts on a checksum chunk.  ``crc_mode="before"``: a window is uploaded up to the
        end of the last chunk its rows touch, a checksum pass over the window runs first, and the window is unpacked
        only if every chunk matches - the next window is already crossing the link meanwhile; a chunk that two
        windows share is uploaded and checked twice.  ``crc_mode="fused"``: the unpack of a window yields the
        checksums of the chunks it holds completely; a chunk that a window ends in is held completely by the next
        window when the rows continue there; chunks that no window holds completely (where the rows do not continue;
        those of byte blobs behind the tensors) are checked on the host at the end, and a mismatch raises before any
        tensor is committed, after targets were written.  With a buffer too small for either, the whole object is
        checked on the host first."""
        if not by_choice:
            _LOGGER.warning("requested range of '%s' exceeds the HBM limit of %d bytes; restoring window by window",
                            object_id, limit)
        chunk_bytes, data_bytes, want = sidecar if sidecar is not None else (0, 0, None)
        # Two buffers of half the limit each, so that a window is unpacked while the next one crosses the link; one
        # buffer of whatever the allocator still has when it cannot give two.
        buffers = []
        uncut = max((r[1] - r[0] for r in rows if not r[2]), default=0)  # a strided row must fit a window whole
        while not buffers:
            if limit - _UPLOAD_ALIGN < 65536:
                if self._max_image_bytes is not None:
                    raise ValueError(f"max_image_bytes={self._max_image_bytes} is too small to restore anything")
                raise torch.OutOfMemoryError(f"no device buffer to restore '{object_id.data}' through")
            half = limit // 2 // _UPLOAD_ALIGN * _UPLOAD_ALIGN
            if half - max(chunk_bytes, _UPLOAD_ALIGN) >= max(_PIPELINED_MIN_WINDOW, uncut):
                first = hip_plan.try_allocate(half, device)
                if first is not None:
                    second = hip_plan.try_allocate(half, device)
                    buffers = [first] if second is None else [first, second]
                limit = half
            else:
                one = hip_plan.try_allocate(limit, device)
                if one is not None:
                    buffers = [one]
                else:
                    limit //= 2
        fused = self._crc_mode == "fused"
        on_device = (sidecar is not None and chunk_bytes % (65536 if fused else _UPLOAD_ALIGN) == 0
                     and limit >= 4 * chunk_bytes)
        check_first = on_device and not fused  # a checksum pass over every window ahead of its unpack
        if sidecar is not None and not on_device:
            self._check_on_host(object_id, stream, sidecar, range(len(want)))
        align = chunk_bytes if on_device else _UPLOAD_ALIGN

        # a window starts on an upload boundary at or below its first row and, where it is checked before it is
        # unpacked, ends on the chunk boundary at or above its last row (or where the data section ends)
        def start_of(first: int) -> int:
            return first // align * align

        def end_of(last: int) -> int:
            return min(-(-last // chunk_bytes) * chunk_bytes, data_bytes) if check_first else last

        piece = (limit - (2 if check_first else 1) * align) // 65536 * 65536  # a multiple of every element size
        pieces = []
        for first, last, contiguous, args in sorted(rows, key=lambda r: r[0]):
            if end_of(last) - start_of(first) <= limit:
                pieces.append((first, last, contiguous, args))
            elif contiguous:
                ptr, esz = args
                for begin in range(first, last, piece):
                    pieces.append((begin, min(begin + piece, last), True, (ptr + (begin - first), esz)))
            else:
                # a strided target or a sub-box whose bytes span more of the image than a window holds: cut along its
                # outermost dimension (then the next one) into boxes that do
                pieces.extend(self._cut_box(first, args, piece))
        windows, current, lo = [], [], 0
        for row in pieces:
            if current and end_of(row[1]) - lo > limit:
                windows.append((lo, current))
                current = []
            if not current:
                lo = start_of(row[0])
            current.append(row)
        windows.append((lo, current))
        cur = torch.cuda.current_stream(device)
        checked = set()
        # The upload of window k+1 runs on a helper thread (the engine call returns when the bytes are in HBM) while
        # this thread builds the tables of window k and launches its unpack; a buffer is reused once the unpack that
        # read it has passed.  Plans stay alive until their checksums have been taken.
        in_use = [None] * len(buffers)  # event behind the last unpack out of each buffer
        launched = []  # (plan, first chunk, complete chunks, event)
        stats_local = self._stats_in_progress

        def span_of(k):
            lo_k, rows_k = windows[k]
            return end_of(max(r[1] for r in rows_k)) - lo_k

        def upload(k):
            self._stats_local.current = stats_local  # (the helper thread books its transfer to this restore)
            self._upload(stream, windows[k][0], buffers[k % len(buffers)], span_of(k), cur, stats)

        try:
            with concurrent.futures.ThreadPoolExecutor(max_workers=1, thread_name_prefix="mlf-upload") as helper:
                pending = helper.submit(upload, 0)
                for k, (lo, window_rows) in enumerate(windows):
                    span = span_of(k)
                    # (built while the window is on its way: not a part of the restore's length)
                    plan = self._unpack_plan(self._table_of(window_rows, lo), span, chunk_bytes if on_device and fused else 0,
                                             booked_as="unpack_plan_s" if len(buffers) == 1 and k else "unpack_plan_beside_h2d_s")
                    launched.append([plan, 0, 0, None])
                    pending.result()
                    if check_first and len(buffers) == 1:
                        self._check_window(object_id, buffers[0], lo, span, sidecar, cur, checked)
                    if k + 1 < len(windows):
                        nxt = (k + 1) % len(buffers)
                        if len(buffers) == 1:  # the one buffer: nothing to overlap, the unpack goes first
                            launched[-1][3] = self._launch_unpack(plan, buffers[0], cur,
                                                                  sum(r[1] - r[0] for r in window_rows if r[2]))
                            launched[-1][3].synchronize()
                        elif in_use[nxt] is not None:
                            in_use[nxt].synchronize()
                        pending = helper.submit(upload, k + 1)
                    if check_first and len(buffers) > 1:  # while the next window is on its way
                        self._check_window(object_id, buffers[k % len(buffers)], lo, span, sidecar, cur, checked)
                    if launched[-1][3] is None:
                        launched[-1][3] = self._launch_unpack(plan, buffers[k % len(buffers)], cur,
                                                              sum(r[1] - r[0] for r in window_rows if r[2]))
                    in_use[k % len(buffers)] = launched[-1][3]
                    if on_device and fused:
                        first = lo // chunk_bytes
                        whole = span // chunk_bytes + (1 if lo + span == data_bytes and span % chunk_bytes else 0)
                        launched[-1][1:3] = [first, whole]
            t0 = time.perf_counter()
            cur.synchronize()
            stats["unpack_s"] = stats.get("unpack_s", 0.0) + time.perf_counter() - t0
            for plan, first, whole, _ in launched:
                if on_device and fused:
                    got = plan.crc_values()
                    self._compare_checksums(object_id, got[:whole], want[first : first + whole], chunk_bytes, first, len(want))
                    checked.update(range(first, first + whole))
        finally:
            cur.synchronize()  # nothing reads the buffers or the tables after this
            for entry in launched:
                entry[0].destroy()
        if on_device:  # what no window held completely: chunks where the rows do not continue, and those of byte blobs
            self._check_on_host(object_id, stream, sidecar, sorted(set(range(len(want))) - checked))
        stats["windows"] = stats.get("windows", 0) + len(windows)

    @staticmethod
    def _cut_box(first: int, args, usable: int):
        """Cuts a strided row - (target address, element size, shape, target strides, image strides or None), whose
        element 0 lies at data-section byte ``first`` - into rows of the same kind that each span at most ``usable``
        bytes of the image: slabs along the first dimension that has more than one index, and slabs of those along
        the next one where a single index is still too much.  Down to single elements if it must be."""
        ptr, esz, shape, strides, image_strides = args
        if image_strides is None:
            image_strides = tuple(hip_plan._contiguous_strides(shape))

        def span(box_shape):
            return (sum((n - 1) * st for n, st in zip(box_shape, image_strides)) + 1) * esz

        if span(shape) <= usable:
            return [(first, first + span(shape), False, (ptr, esz, tuple(shape), tuple(strides), tuple(image_strides)))]
        d = next(i for i, n in enumerate(shape) if n > 1)  # (a single element never exceeds a window)
        one = span(shape[:d] + (1,) + shape[d + 1:])
        per = (usable - one) // (image_strides[d] * esz) + 1 if one <= usable else 1
        out = []
        for i0 in range(0, shape[d], per):
            sub = shape[:d] + (min(per, shape[d] - i0),) + shape[d + 1:]
            out.extend(HipMLFlashpointCheckpointLoader._cut_box(
                first + i0 * image_strides[d] * esz, (ptr + i0 * strides[d] * esz, esz, sub, strides, image_strides), usable))
        return out

    def _check_window(self, object_id, buffer: torch.Tensor, lo: int, span: int, sidecar, cur, checked: set) -> None:
        """Checksum pass over a window that starts on a chunk boundary and ends on one (or where the data section
        ends), compared with the sidecar before anything is unpacked from it."""
        chunk_bytes, _, want = sidecar
        t0 = time.perf_counter()
        got = hip_plan.crc32c_device(buffer, span, chunk_bytes, cur.cuda_stream)
        stats = self._stats_in_progress
        stats["crc_s"] = stats.get("crc_s", 0.0) + time.perf_counter() - t0
        first = lo // chunk_bytes
        self._compare_checksums(object_id, got, want[first : first + len(got)], chunk_bytes, first, len(want))
        checked.update(range(first, first + len(got)))

    def _check_on_host(self, object_id, stream, sidecar, chunks) -> None:
        """Compares the given chunks of an object's data section with its sidecar, reading them on the host."""
        chunk_bytes, data_bytes, want = sidecar
        chunks = list(chunks)
        if not chunks:
            return
        t0 = time.perf_counter()
        fd = stream.fileno()
        own_fd = fd < 0
        if own_fd:
            fd = os.open(object_id.data, os.O_RDONLY)
        try:
            threads = self._engine_config.resolved_copy_threads()
            if chunks == list(range(chunks[0], chunks[-1] + 1)):  # one run: one threaded pass
                first = chunks[0] * chunk_bytes
                length = min((chunks[-1] + 1) * chunk_bytes, data_bytes) - first
                got = hip_plan.crc32c_file(fd, METADATA_SIZE + first, length, chunk_bytes, threads)
                self._compare_checksums(object_id, got, want[chunks[0] : chunks[-1] + 1], chunk_bytes, chunks[0], len(want))
            else:
                for k in chunks:
                    length = min((k + 1) * chunk_bytes, data_bytes) - k * chunk_bytes
                    got = hip_plan.crc32c_file(fd, METADATA_SIZE + k * chunk_bytes, length, chunk_bytes, threads)
                    self._compare_checksums(object_id, got, want[k : k + 1], chunk_bytes, k, len(want))
        finally:
            if own_fd:
                os.close(fd)
        stats = self._stats_in_progress
        stats["crc_s"] = stats.get("crc_s", 0.0) + time.perf_counter() - t0

    # ---- discovery (core/checkpoint_discovery.py) ----------------------------------------------------------
    def _object_is_intact(self, path: str) -> bool:
        """False when the object has a CRC-32C sidecar and its data section no longer matches it (host-side
        check: pread + SSE4.2, no GPU).  Objects without a sidecar, and the sidecars themselves, pass."""
        sidecar = integrity.read_sidecar(path)
        if sidecar is None:
            return True
        chunk_bytes, data_bytes, want = sidecar
        try:
            fd = os.open(path, os.O_RDONLY)
        except OSError:
            return False
        try:
            if os.fstat(fd).st_size != METADATA_SIZE + data_bytes:
                return False
            got = hip_plan.crc32c_file(fd, METADATA_SIZE, data_bytes, chunk_bytes, self._engine_config.resolved_copy_threads())
        except _lib.HipError:
            return False
        finally:
            os.close(fd)
        return bool((got == want).all())
