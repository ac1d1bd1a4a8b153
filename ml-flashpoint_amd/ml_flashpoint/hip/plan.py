"""Python face of the native plan / copy-engine / CRC entry points, plus the host-side layout rules.

The *layout* of a checkpoint object's data section is decided here, on the host, and is exactly the reference's:
records ``<u32 len><pickled TensorHeader><payload>`` back to back from offset 0, tensors first, then byte blobs
(reference: src/ml_flashpoint/core/checkpoint_saver.py:667-698,764-800).  The bytes themselves are moved by the
gfx950 kernels: this module only fills the descriptor table that drives them.
"""

import ctypes
import dataclasses
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ml_flashpoint.core.tensor_header import TensorHeader
from ml_flashpoint.hip import _lib
from ml_flashpoint.hip._lib import ITEM_BLOB, ITEM_DEVICE, ITEM_DTYPE, MAX_DIMS

_HEADER_CACHE: Dict[Tuple[torch.dtype, Tuple[int, ...]], bytes] = {}


def header_bytes(dtype: torch.dtype, shape: Sequence[int]) -> bytes:
    """``TensorHeader(dtype, shape).to_bytes()``, memoised: a state dict repeats few distinct (dtype, shape)."""
    key = (dtype, tuple(shape))
    raw = _HEADER_CACHE.get(key)
    if raw is None:
        raw = TensorHeader(dtype=dtype, shape=torch.Size(key[1])).to_bytes()
        if len(_HEADER_CACHE) < 1 << 16:
            _HEADER_CACHE[key] = raw
    return raw


def _contiguous_strides(shape: Sequence[int]) -> List[int]:
    strides = [1] * len(shape)
    for d in range(len(shape) - 2, -1, -1):
        strides[d] = strides[d + 1] * shape[d + 1]
    return strides


def collapse_dims(shape: Sequence[int], stride: Sequence[int],
                  image_stride: Optional[Sequence[int]] = None) -> Tuple[tuple, tuple, tuple]:
    """The same elements at the same places described with as few dimensions as possible: dimensions of extent 1
    dropped, neighbours merged where stepping the outer one equals walking off the end of the inner one on both
    sides.  ``image_stride`` None: the C-contiguous strides of ``shape``.  Strides in elements."""
    if image_stride is None:
        image_stride = _contiguous_strides(shape)
    out: List[List[int]] = []
    for n, ts, im in zip(shape, stride, image_stride):
        if n == 1:
            continue
        if out and out[-1][1] == ts * n and out[-1][2] == im * n:
            out[-1] = [out[-1][0] * n, ts, im]
        else:
            out.append([n, ts, im])
    return tuple(d[0] for d in out), tuple(d[1] for d in out), tuple(d[2] for d in out)


def describable(shape: Sequence[int], stride: Sequence[int], image_stride: Optional[Sequence[int]] = None) -> bool:
    """Whether a strided item fits the descriptor table's ``MAX_DIMS`` dimensions (after ``collapse_dims``)."""
    return len(shape) <= MAX_DIMS or len(collapse_dims(shape, stride, image_stride)[0]) <= MAX_DIMS


class ItemTable:
    """Column-wise builder of an ``mlf_item`` array.

    Scalar columns are plain Python lists turned into numpy columns in one go; contiguous device items are stored
    as 1-D (numel,) with unit strides, so only genuinely strided items carry per-dimension rows."""

    def __init__(self):
        self.ptr: List[int] = []
        self.image_off: List[int] = []
        self.nbytes: List[int] = []
        self.kind: List[int] = []
        self.elem_size: List[int] = []
        self._strided: List[tuple] = []  # (row, shape, stride, image_stride)

    def __len__(self):
        return len(self.ptr)

    def add_blob(self, blob_off: int, image_off: int, nbytes: int) -> None:
        self.ptr.append(blob_off)
        self.image_off.append(image_off)
        self.nbytes.append(nbytes)
        self.kind.append(ITEM_BLOB)
        self.elem_size.append(1)

    def add_contiguous(self, ptr: int, image_off: int, elem_size: int, nbytes: int) -> None:
        """Device item that is one run of bytes on both sides."""
        self.ptr.append(ptr)
        self.image_off.append(image_off)
        self.nbytes.append(nbytes)
        self.kind.append(ITEM_DEVICE)
        self.elem_size.append(elem_size)

    def add_device(
        self,
        ptr: int,
        image_off: int,
        elem_size: int,
        shape: Sequence[int],
        stride: Sequence[int],
        image_stride: Optional[Sequence[int]] = None,
    ) -> None:
        numel = 1
        for s in shape:
            numel *= s
        if image_stride is None:
            image_stride = _contiguous_strides(shape)
        if len(shape) > MAX_DIMS:
            # more dimensions than a table row holds: most such views are fewer once neighbours are merged; callers
            # stage the rest through a contiguous copy (see ``describable``)
            shape, stride, image_stride = collapse_dims(shape, stride, image_stride)
            if len(shape) > MAX_DIMS:
                raise ValueError(f"a strided item of {len(shape)} dimensions after merging does not fit the descriptor "
                                 f"table's {MAX_DIMS}; stage it through a contiguous copy")
        self._strided.append((len(self.ptr), tuple(shape), tuple(stride), tuple(image_stride)))
        self.add_contiguous(ptr, image_off, elem_size, numel * elem_size)

    def to_array(self) -> np.ndarray:
        n = len(self.ptr)
        arr = np.zeros(n, dtype=ITEM_DTYPE)
        if n == 0:
            return arr
        arr["ptr"] = self.ptr
        arr["image_off"] = self.image_off
        nbytes = np.array(self.nbytes, dtype=np.uint64)
        arr["nbytes"] = nbytes
        arr["kind"] = self.kind
        esz = np.array(self.elem_size, dtype=np.uint32)
        arr["elem_size"] = esz
        # default description of every item: one dimension of numel elements, unit strides
        arr["ndim"] = 1
        arr["shape"][:, 0] = nbytes // esz
        arr["stride"][:, 0] = 1
        arr["image_stride"][:, 0] = 1
        for row, shape, stride, image_stride in self._strided:
            k = len(shape)
            item = arr[row]
            item["ndim"] = k
            item["shape"][:k] = shape
            item["stride"][:k] = stride
            item["image_stride"][:k] = image_stride
            if k == 0:
                item["shape"][0] = 0
                item["stride"][0] = 0
                item["image_stride"][0] = 0
        return arr


def host_tensor_bytes(t: torch.Tensor) -> bytes:
    """C-contiguous bytes of a host-resident tensor (what its record's payload is)."""
    return t.detach().contiguous().reshape(-1).view(torch.uint8).numpy().tobytes()


@dataclasses.dataclass
class SaveLayout:
    """Where every item of one checkpoint object lies, and the table that packs it.

    ``image_bytes`` is what the image takes in HBM, ``data_bytes`` what the object's data section takes in the buffer
    file.  They differ only when large host-resident tensors go from host memory straight into the buffer
    (``host_spans``): their payloads are left out of the image, which then consists of ``segments`` - runs of image
    bytes that belong at consecutive offsets of the data section."""

    image_bytes: int
    spans: List[Tuple[int, int]]  # (data offset, length) of each record: tensors in order, then byte blobs in order
    items: np.ndarray
    blob: bytes
    device_payload_bytes: int
    device_tensors: List[torch.Tensor]  # kept alive while the plan may run
    # pieces of the blob whose bytes are not determined by dtypes and shapes: (blob offset, nbytes, "tensor" | "blob",
    # index into the tensors / blobs argument).  A layout that is reused for the next save refreshes exactly these.
    variable_parts: List[Tuple[int, int, str, int]] = dataclasses.field(default_factory=list)
    data_bytes: int = -1  # -1: same as image_bytes
    # (data offset, nbytes, index): index >= 0 into the tensors, -1 - k for byte blob k
    host_spans: List[Tuple[int, int, int]] = dataclasses.field(default_factory=list)
    host_tensors: list = dataclasses.field(default_factory=list)  # one source per host span: a tensor, or the blob's bytes
    segments: List[Tuple[int, int, int]] = dataclasses.field(default_factory=list)  # (image offset, data offset, nbytes)

    def __post_init__(self):
        if self.data_bytes < 0:
            self.data_bytes = self.image_bytes


def build_save_layout(tensors: Sequence[torch.Tensor], blobs: Sequence[bytes] = (),
                      host_direct_min: Optional[int] = None) -> SaveLayout:
    """Lays out records for ``tensors`` (device or host) followed by ``blobs`` and returns the descriptor table.

    Device tensors become DEVICE items (any strides; the image side is the C-contiguous payload).  Record headers,
    payloads of host-resident tensors and byte blobs are collected into one host blob that the plan uploads once -
    except host-resident tensors and byte blobs of at least ``host_direct_min`` bytes (None: no such exception),
    which never visit the device: the layout only notes where in the data section they belong (``host_spans``).
    """
    table = ItemTable()
    blob = bytearray()
    spans: List[Tuple[int, int]] = []
    keep: List[torch.Tensor] = []
    variable: List[Tuple[int, int, str, int]] = []
    host_spans: List[Tuple[int, int, int]] = []
    host_tensors: List[torch.Tensor] = []
    pos = 0   # in the data section
    ipos = 0  # in the image
    device_bytes = 0
    for index, t in enumerate(tensors):
        start = pos
        hdr = header_bytes(t.dtype, t.shape)
        table.add_blob(len(blob), ipos, len(hdr))
        blob += hdr
        pos += len(hdr)
        ipos += len(hdr)
        nbytes = t.numel() * t.element_size()
        if nbytes:
            if t.device.type == "cpu" and host_direct_min is not None and nbytes >= host_direct_min:
                # large host-resident item (an optimizer state kept in host memory ...): host to buffer directly
                host_spans.append((pos, nbytes, index))
                host_tensors.append(t)
            elif t.device.type == "cpu":
                # host-resident item (step counters, RNG state ...): its bytes travel with the headers
                variable.append((len(blob), nbytes, "tensor", index))
                table.add_blob(len(blob), ipos, nbytes)
                blob += host_tensor_bytes(t)
                ipos += nbytes
            else:
                if t.is_contiguous():
                    table.add_contiguous(t.data_ptr(), ipos, t.element_size(), nbytes)
                else:
                    table.add_device(t.data_ptr(), ipos, t.element_size(), tuple(t.shape), tuple(t.stride()))
                keep.append(t)
                device_bytes += nbytes
                ipos += nbytes
            pos += nbytes
        spans.append((start, pos - start))
    for index, data in enumerate(blobs):
        if host_direct_min is not None and len(data) >= max(host_direct_min, 1):
            host_spans.append((pos, len(data), -1 - index))  # a large pickled object: host to buffer, like a tensor
            host_tensors.append(data)
        elif len(data):
            variable.append((len(blob), len(data), "blob", index))
            table.add_blob(len(blob), ipos, len(data))
            blob += data
            ipos += len(data)
        spans.append((pos, len(data)))
        pos += len(data)
    segments: List[Tuple[int, int, int]] = []
    image_at = data_at = 0
    for offset, nbytes, _ in host_spans:
        if offset > data_at:
            segments.append((image_at, data_at, offset - data_at))
            image_at += offset - data_at
        data_at = offset + nbytes
    if pos > data_at:
        segments.append((image_at, data_at, pos - data_at))
        image_at += pos - data_at
    assert image_at == ipos
    return SaveLayout(
        image_bytes=ipos,
        spans=spans,
        items=table.to_array(),
        blob=bytes(blob),
        device_payload_bytes=device_bytes,
        device_tensors=keep,
        variable_parts=variable,
        data_bytes=pos,
        host_spans=host_spans,
        host_tensors=host_tensors,
        segments=segments,
    )


def try_allocate(nbytes: int, device) -> Optional[torch.Tensor]:
    """A ``uint8`` device buffer of ``nbytes`` from torch's allocator, or None if it cannot provide one piece of
    that size - also not after handing its unused segments back to the driver.  (A long-running job's free memory
    is rarely one piece: what the device reports as free says little about the largest block to be had.)"""
    for attempt in (0, 1):
        try:
            return torch.empty(nbytes, dtype=torch.uint8, device=device)
        except torch.OutOfMemoryError:
            if attempt == 0:
                torch.cuda.empty_cache()
    return None


class Plan:
    """Owns a native ``mlf_plan``: device-resident descriptor and work tables for one set of items."""

    def __init__(
        self,
        items: np.ndarray,
        blob: bytes,
        image_bytes: int,
        *,
        tile_bytes: int = 0,
        block_threads: int = 0,
        align_to_tensor: bool = False,
        unroll: int = 0,
        grid_x_log2: int = 0,
        crc_chunk_bytes: int = 0,
    ):
        """``crc_chunk_bytes`` > 0 (a multiple of 64 KiB): every pack / unpack launch also yields the CRC-32C of each
        chunk of that size of the image, folded inside the copy kernel where a contiguous item covers whole 64 KiB
        pieces of the image (``crc_values``)."""
        lib = _lib.load()
        assert items.dtype == ITEM_DTYPE and items.flags["C_CONTIGUOUS"]
        if crc_chunk_bytes % 65536:
            raise ValueError("crc_chunk_bytes must be a multiple of 65536")
        opts = _lib.PlanOpts(tile_bytes, block_threads, 1 if align_to_tensor else 0, unroll, grid_x_log2,
                             crc_chunk_bytes >> 10)
        handle = ctypes.c_void_p()
        blob_buf = (ctypes.c_char * len(blob)).from_buffer_copy(blob) if blob else None
        _lib.check(
            lib.mlf_plan_create(
                items.ctypes.data if len(items) else None,
                len(items),
                ctypes.addressof(blob_buf) if blob_buf is not None else None,
                len(blob),
                image_bytes,
                ctypes.byref(opts),
                ctypes.byref(handle),
            ),
            "mlf_plan_create",
        )
        self._handle = handle
        self.image_bytes = image_bytes
        self.crc_chunk_bytes = crc_chunk_bytes if image_bytes else 0

    def crc_values(self) -> np.ndarray:
        """Per-chunk CRC-32C of the image moved by the most recent launch (waits for that launch's checksum work)."""
        if self._handle is None:
            raise ValueError("plan already destroyed")
        if not self.crc_chunk_bytes:
            return np.zeros(0, dtype=np.uint32)
        n = -(-self.image_bytes // self.crc_chunk_bytes)
        out = np.zeros(n, dtype=np.uint32)
        _lib.check(_lib.load().mlf_plan_crc_values(self._handle, out.ctypes.data, n), "mlf_plan_crc_values")
        return out

    @property
    def info(self) -> _lib.PlanInfo:
        out = _lib.PlanInfo()
        _lib.check(_lib.load().mlf_plan_get_info(self._handle, ctypes.byref(out)), "mlf_plan_get_info")
        return out

    def update_blob(self, blob: bytes, stream: int) -> None:
        """New bytes (same length) for the blob of a plan that is kept across saves; ordered on ``stream``."""
        if self._handle is None:
            raise ValueError("plan already destroyed")
        buf = (ctypes.c_char * len(blob)).from_buffer_copy(blob) if blob else None
        _lib.check(
            _lib.load().mlf_plan_update_blob(self._handle, ctypes.addressof(buf) if buf is not None else None,
                                             len(blob), stream),
            "mlf_plan_update_blob",
        )

    def pack(self, image: torch.Tensor, stream: Optional[int] = None) -> None:
        """Enqueues tensors -> image on ``stream`` (default: torch's current stream)."""
        self._launch(_lib.load().mlf_pack_launch, image, stream, "mlf_pack_launch")

    def unpack(self, image: torch.Tensor, stream: Optional[int] = None) -> None:
        """Enqueues image -> tensors on ``stream`` (default: torch's current stream)."""
        self._launch(_lib.load().mlf_unpack_launch, image, stream, "mlf_unpack_launch")

    def _launch(self, fn, image: torch.Tensor, stream: Optional[int], what: str) -> None:
        if self._handle is None:
            raise ValueError("plan already destroyed")
        if image.dtype != torch.uint8 or not image.is_contiguous() or image.device.type != "cuda":
            raise ValueError("image must be a contiguous uint8 device tensor")
        if image.numel() < self.image_bytes:
            raise ValueError(f"image holds {image.numel()} bytes, plan needs {self.image_bytes}")
        if stream is None:
            stream = torch.cuda.current_stream(image.device).cuda_stream
        _lib.check(fn(self._handle, image.data_ptr() if image.numel() else None, stream), what)

    def destroy(self) -> None:
        if getattr(self, "_handle", None) is not None:
            _lib.load().mlf_plan_destroy(self._handle)
            self._handle = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


class CopyEngine:
    """Ring of pinned slots + copy streams + host threads between device images and pageable host memory."""

    def __init__(self, slot_bytes: int = 32 << 20, n_slots: int = 3, n_threads: int = 8):
        handle = ctypes.c_void_p()
        _lib.check(_lib.load().mlf_engine_create(slot_bytes, n_slots, n_threads, ctypes.byref(handle)), "mlf_engine_create")
        self._handle = handle
        self.slot_bytes, self.n_slots, self.n_threads = slot_bytes, n_slots, n_threads

    def set_host_checksums(self, on: bool) -> None:
        """Who takes the checksums of the ``d2h_*`` calls that ask for them: the host threads as they move the
        slots (True), or kernels that read the image once more beside the copies (False, the state of a new engine)."""
        _lib.check(_lib.load().mlf_engine_set_host_checksums(self._handle, 1 if on else 0), "mlf_engine_set_host_checksums")

    def d2h(self, src_dev_ptr: int, dst_host_ptr: int, nbytes: int, producer_stream: int = 0) -> _lib.XferStats:
        stats = _lib.XferStats()
        _lib.check(
            _lib.load().mlf_engine_d2h(self._handle, src_dev_ptr, dst_host_ptr, nbytes, producer_stream, ctypes.byref(stats)),
            "mlf_engine_d2h",
        )
        return stats

    def d2h_crc(self, src_dev_ptr: int, dst_host_ptr: int, nbytes: int, producer_stream: int, crc_chunk_bytes: int):
        """``d2h`` plus a CRC-32C per ``crc_chunk_bytes`` piece of the source, computed beside the copies.
        Returns (stats, uint32 array of chunk checksums)."""
        stats = _lib.XferStats()
        n_chunks = (nbytes + crc_chunk_bytes - 1) // crc_chunk_bytes
        crcs = np.zeros(max(n_chunks, 1), dtype=np.uint32)
        _lib.check(
            _lib.load().mlf_engine_d2h_crc(self._handle, src_dev_ptr, dst_host_ptr, nbytes, producer_stream, crc_chunk_bytes,
                                           crcs.ctypes.data, len(crcs), ctypes.byref(stats)),
            "mlf_engine_d2h_crc",
        )
        return stats, crcs[:n_chunks]

    def d2h_watched(self, src_dev_ptr: int, dst_host_ptr: int, nbytes: int, producer_stream: int, crc_chunk_bytes: int,
                    landed: "ctypes.c_uint64"):
        """``d2h_crc`` (``crc_chunk_bytes`` 0: no checksums) that keeps ``landed`` at the number of leading bytes
        that have reached the destination, for a reader on another thread.  Returns (stats, checksums or None)."""
        stats = _lib.XferStats()
        n_chunks = (nbytes + crc_chunk_bytes - 1) // crc_chunk_bytes if crc_chunk_bytes else 0
        crcs = np.zeros(max(n_chunks, 1), dtype=np.uint32)
        _lib.check(
            _lib.load().mlf_engine_d2h_watched(self._handle, src_dev_ptr, dst_host_ptr, nbytes, producer_stream,
                                               crc_chunk_bytes, crcs.ctypes.data, len(crcs), ctypes.addressof(landed),
                                               ctypes.byref(stats)),
            "mlf_engine_d2h_watched",
        )
        return stats, (crcs[:n_chunks] if crc_chunk_bytes else None)

    def d2h_gated(self, src_dev_ptr: int, dst_host_ptr: int, nbytes: int, ready_event: Optional[int],
                  crc_chunk_bytes: int, landed: "ctypes.c_uint64"):
        """``d2h_watched`` that waits for an event (a raw ``hipEvent_t``, e.g. ``torch.cuda.Event.cuda_event``, recorded
        behind the pack; None: does not wait) instead of for everything on the producer's stream."""
        stats = _lib.XferStats()
        n_chunks = (nbytes + crc_chunk_bytes - 1) // crc_chunk_bytes if crc_chunk_bytes else 0
        crcs = np.zeros(max(n_chunks, 1), dtype=np.uint32)
        _lib.check(
            _lib.load().mlf_engine_d2h_gated(self._handle, src_dev_ptr, dst_host_ptr, nbytes, ready_event,
                                             crc_chunk_bytes, crcs.ctypes.data, len(crcs), ctypes.addressof(landed),
                                             ctypes.byref(stats)),
            "mlf_engine_d2h_gated",
        )
        return stats, (crcs[:n_chunks] if crc_chunk_bytes else None)

    def link_probe(self, dev_ptr: int, nbytes: int, to_host: bool) -> float:
        """Seconds to move ``nbytes`` between device memory and the engine's pinned slots with nothing behind them:
        the host link's own rate for this engine's slot size and streams."""
        seconds = ctypes.c_double(0.0)
        _lib.check(_lib.load().mlf_engine_link_probe(self._handle, dev_ptr, nbytes, 1 if to_host else 0,
                                                     ctypes.byref(seconds)), "mlf_engine_link_probe")
        return seconds.value

    @staticmethod
    def _cut_count(nbytes: int, crc_chunk_bytes: int, first_part_bytes: int) -> int:
        head = min(first_part_bytes, nbytes)
        return (1 if head else 0) + -(-(nbytes - head) // crc_chunk_bytes)

    def d2h_cut(self, src_dev_ptr: int, dst_host_ptr: int, nbytes: int, data_off: int, crc_chunk_bytes: int,
                producer_stream: int = 0, ready_event: Optional[int] = None, landed: "Optional[ctypes.c_uint64]" = None):
        """A piece of a data section, from byte ``data_off`` of the section on, device to host, with the checksums of
        the piece taken by the host threads as they copy and cut where the section's chunks end: one value per part
        of ``integrity.ChunkChecksums.cuts(data_off, nbytes, crc_chunk_bytes)``.  The copies wait for ``ready_event``
        if given, else for what ``producer_stream`` holds now.  Returns (stats, list of values)."""
        stats = _lib.XferStats()
        first = -data_off % crc_chunk_bytes
        n = self._cut_count(nbytes, crc_chunk_bytes, first)
        crcs = np.zeros(max(n, 1), dtype=np.uint32)
        _lib.check(
            _lib.load().mlf_engine_d2h_cut(self._handle, src_dev_ptr, dst_host_ptr, nbytes, producer_stream, ready_event,
                                           crc_chunk_bytes, first, crcs.ctypes.data, len(crcs),
                                           ctypes.addressof(landed) if landed is not None else None, ctypes.byref(stats)),
            "mlf_engine_d2h_cut",
        )
        return stats, [int(v) for v in crcs[:n]]

    def host_copy_cut(self, dst_host_ptr: int, src_host_ptr: int, nbytes: int, data_off: int, crc_chunk_bytes: int) -> list:
        """``host_copy`` of a piece of a data section that also yields the piece's checksums, cut like ``d2h_cut``'s."""
        first = -data_off % crc_chunk_bytes
        n = self._cut_count(nbytes, crc_chunk_bytes, first)
        crcs = np.zeros(max(n, 1), dtype=np.uint32)
        _lib.check(_lib.load().mlf_engine_host_copy_cut(self._handle, dst_host_ptr, src_host_ptr, nbytes, crc_chunk_bytes,
                                                        first, crcs.ctypes.data, len(crcs)), "mlf_engine_host_copy_cut")
        return [int(v) for v in crcs[:n]]

    def read_file(self, fd: int, file_offset: int, dst_host_ptr: int, nbytes: int) -> None:
        """A range of a file into host memory, by ``pread`` on the engine's threads."""
        _lib.check(_lib.load().mlf_engine_read_file(self._handle, fd, file_offset, dst_host_ptr, nbytes), "mlf_engine_read_file")

    def host_copy(self, dst_host_ptr: int, src_host_ptr: int, nbytes: int) -> None:
        """Host memory to host memory on the engine's threads (checkpoint items that are resident on the host)."""
        _lib.check(_lib.load().mlf_engine_host_copy(self._handle, dst_host_ptr, src_host_ptr, nbytes), "mlf_engine_host_copy")

    def avoid_stream(self, *busy_streams: int) -> int:
        """Moves the engine's streams off the hardware queues of ``busy_streams`` (raw ``hipStream_t`` values: the
        streams the training step runs on), where they would wait behind those streams' kernels; waits for them to
        drain while it tests.  Returns how many of the engine's three streams could not be moved."""
        left = ctypes.c_uint32(0)
        handles = (ctypes.c_void_p * len(busy_streams))(*busy_streams)
        _lib.check(_lib.load().mlf_engine_avoid_streams(self._handle, handles, len(busy_streams), ctypes.byref(left)),
                   "mlf_engine_avoid_streams")
        return int(left.value)

    @property
    def checksum_stream(self) -> int:
        """The engine's checksum stream (raw ``hipStream_t``), for checksum calls between its transfers."""
        return int(_lib.load().mlf_engine_checksum_stream(self._handle) or 0)

    def h2d(self, src_host_ptr: int, dst_dev_ptr: int, nbytes: int, consumer_stream: int = 0) -> _lib.XferStats:
        stats = _lib.XferStats()
        _lib.check(
            _lib.load().mlf_engine_h2d(self._handle, src_host_ptr, dst_dev_ptr, nbytes, consumer_stream, ctypes.byref(stats)),
            "mlf_engine_h2d",
        )
        return stats

    def d2h_fd(self, src_dev_ptr: int, fd: int, file_offset: int, nbytes: int, producer_stream: int = 0) -> _lib.XferStats:
        """Device -> byte range of an open file (pwrite from the pinned slots)."""
        stats = _lib.XferStats()
        _lib.check(
            _lib.load().mlf_engine_d2h_fd(self._handle, src_dev_ptr, fd, file_offset, nbytes, producer_stream, ctypes.byref(stats)),
            "mlf_engine_d2h_fd",
        )
        return stats

    def h2d_fd(self, fd: int, file_offset: int, dst_dev_ptr: int, nbytes: int, consumer_stream: int = 0) -> _lib.XferStats:
        """Byte range of an open file -> device (pread into the pinned slots)."""
        stats = _lib.XferStats()
        _lib.check(
            _lib.load().mlf_engine_h2d_fd(self._handle, fd, file_offset, dst_dev_ptr, nbytes, consumer_stream, ctypes.byref(stats)),
            "mlf_engine_h2d_fd",
        )
        return stats

    def destroy(self) -> None:
        if getattr(self, "_handle", None) is not None:
            _lib.load().mlf_engine_destroy(self._handle)
            self._handle = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


def crc32c_device(buf: torch.Tensor, nbytes: int, chunk_bytes: int, stream: Optional[int] = None) -> np.ndarray:
    """CRC-32C of each ``chunk_bytes`` piece of the first ``nbytes`` of a device uint8 tensor."""
    if nbytes == 0:
        return np.zeros(0, dtype=np.uint32)
    if stream is None:
        stream = torch.cuda.current_stream(buf.device).cuda_stream
    n_chunks = (nbytes + chunk_bytes - 1) // chunk_bytes
    out = np.zeros(n_chunks, dtype=np.uint32)
    _lib.check(
        _lib.load().mlf_crc32c_device(buf.data_ptr(), nbytes, chunk_bytes, out.ctypes.data, n_chunks, stream),
        "mlf_crc32c_device",
    )
    return out


def crc32c_device_cut(buf: torch.Tensor, buf_off: int, data_off: int, nbytes: int, chunk_bytes: int, host_ptr: int,
                      stream: Optional[int] = None) -> list:
    """CRC-32C of ``nbytes`` bytes of a data section, from byte ``data_off`` on, cut where the section's checksum
    chunks end: one value per part of ``integrity.ChunkChecksums.cuts(data_off, nbytes, chunk_bytes)``.  The bytes
    lie at ``buf[buf_off:]`` on the device and, already, at ``host_ptr`` on the host; buffer positions and section
    positions must agree modulo 16, so that chunk boundaries are 16-byte aligned on the device (the checksum
    kernels read vectors).  Only a first part that starts off that grid needs the host copy: its leading bytes, at
    most 15, are checksummed there and joined with the device's value for the rest."""
    if nbytes == 0:
        return []
    base = buf.data_ptr() + buf_off
    if (base - data_off) % 16:
        raise ValueError("buffer and data section positions differ modulo 16")
    values = []
    head = min(nbytes, -data_off % chunk_bytes)
    if head:
        skip = min(head, -base % 16)
        value = crc32c_host(host_ptr, skip) if skip else None
        if head > skip:
            on_device = int(crc32c_device(buf[buf_off + skip : buf_off + head], head - skip, chunk_bytes, stream)[0])
            value = on_device if value is None else crc32c_combine(value, on_device, head - skip)
        values.append(value)
    if nbytes > head:
        values.extend(int(v) for v in crc32c_device(buf[buf_off + head : buf_off + nbytes], nbytes - head, chunk_bytes, stream))
    return values


def crc32c_host(ptr: int, nbytes: int) -> int:
    return int(_lib.load().mlf_crc32c_host(ptr, nbytes))


def crc32c_combine(crc_a: int, crc_b: int, len_b: int) -> int:
    return int(_lib.load().mlf_crc32c_combine(crc_a, crc_b, len_b))


def crc32c_file(fd: int, file_offset: int, nbytes: int, chunk_bytes: int, threads: int = 8) -> np.ndarray:
    """CRC-32C of each ``chunk_bytes`` piece of a byte range of an open file, computed on the host."""
    n_chunks = (nbytes + chunk_bytes - 1) // chunk_bytes if nbytes else 0
    out = np.zeros(n_chunks, dtype=np.uint32)
    if n_chunks:
        _lib.check(_lib.load().mlf_crc32c_file(fd, file_offset, nbytes, chunk_bytes, out.ctypes.data, n_chunks, threads),
                   "mlf_crc32c_file")
    return out
