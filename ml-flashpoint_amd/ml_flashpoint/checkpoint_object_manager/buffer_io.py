"""File-like stream over a ``BufferObject`` mapping.

Positions are relative to the data section, which starts after the 4096-byte metadata block.  The block's
``len_written_data`` is a high-water mark of what was written; reads never go past it.  Interface, error types
and messages follow the reference (src/ml_flashpoint/checkpoint_object_manager/buffer_io.py:26-530).
"""

import io
from typing import Union

from ml_flashpoint.checkpoint_object_manager.buffer_object.buffer_object_ext import BufferObject
from ml_flashpoint.core.mlf_logging import get_logger

from .buffer_metadata import METADATA_SIZE, BufferMetadataType

_LOGGER = get_logger(__name__)

_RO_OPS = frozenset(("read", "readinto", "seek"))
_RW_OPS = frozenset(("write", "read", "readinto", "seek"))


class BufferIO:
    """I/O operations on a BufferObject."""

    def __init__(self, buffer_obj: BufferObject):
        if buffer_obj.closed:
            raise ValueError("Cannot initialize BufferIO with a closed BufferObject.")
        self.buffer_obj = buffer_obj
        self._pos = 0
        try:
            self._mv = memoryview(buffer_obj)
        except TypeError:
            raise ValueError("Underlying BufferObject does not support the buffer protocol.")
        if len(self._mv) < METADATA_SIZE:
            raise ValueError(f"Buffer size must be at least {METADATA_SIZE} bytes.")
        self._bind_metadata()

    def _bind_metadata(self) -> None:
        head = self._mv[:METADATA_SIZE]
        try:
            if self.buffer_obj.is_readonly:
                # a read-only mapping cannot back a live ctypes view: keep a private copy
                self._metadata = BufferMetadataType.from_buffer_copy(head)
            else:
                self._metadata = BufferMetadataType.from_buffer(head)
        except Exception as e:
            raise IOError(f"Could not initialize metadata from buffer: {e}") from e

    # ---- state checks ---------------------------------------------------------------------------------
    def _check_validity(self, operation: str = None) -> None:
        if self.closed:
            raise ValueError("I/O operation on a closed BufferIO object")
        if operation is None:
            return
        if self.buffer_obj.is_readonly:
            if operation not in _RO_OPS:
                raise TypeError(f"Operation '{operation}' is not supported in read-only mode.")
        elif operation not in _RW_OPS:
            raise TypeError(f"Operation '{operation}' is not supported in read-write mode.")

    def _update_written_data_length(self, new_length: int) -> None:
        if new_length > self._metadata.len_written_data:
            self._metadata.len_written_data = new_length

    # ---- stream interface -----------------------------------------------------------------------------
    def write(self, data: bytes) -> int:
        self._check_validity("write")
        n = len(data)
        if n == 0:
            return 0
        start = METADATA_SIZE + self._pos
        if start + n > len(self._mv):
            raise ValueError(
                "Write operation exceeds buffer capacity. "
                f"Attempted to write {n} bytes at position {self._pos} "
                f"which would exceed the total capacity of {len(self._mv)}."
            )
        self._mv[start : start + n] = data
        self._pos += n
        self._update_written_data_length(self._pos)
        return n

    def _readable(self, size: int) -> int:
        avail = self._metadata.len_written_data - self._pos
        if avail <= 0:
            return 0
        return avail if size < 0 else min(size, avail)

    def read(self, size: int = -1) -> bytes:
        self._check_validity("read")
        n = self._readable(size)
        if n <= 0:
            return b""
        start = METADATA_SIZE + self._pos
        out = self._mv[start : start + n].tobytes()
        self._pos += n
        return out

    def readinto(self, b: Union[bytearray, memoryview]) -> int:
        self._check_validity("readinto")
        if not isinstance(b, (bytearray, memoryview)) or (isinstance(b, memoryview) and b.readonly):
            raise TypeError(f"readinto() argument must be a writable bytes-like object, not {type(b).__name__}")
        if len(b) == 0:
            return 0
        n = self._readable(len(b))
        if n <= 0:
            return 0
        start = METADATA_SIZE + self._pos
        try:
            b[:n] = self._mv[start : start + n]
        except Exception as e:
            raise OSError(f"Failed to read data into buffer from slice [{start}:{start + n}]") from e
        self._pos += n
        return n

    def seek(self, offset: int, whence: int = io.SEEK_SET) -> int:
        self._check_validity("seek")
        if whence == io.SEEK_SET:
            target = offset
        elif whence == io.SEEK_CUR:
            target = self._pos + offset
        elif whence == io.SEEK_END:
            target = self._metadata.len_written_data + offset
        else:
            raise ValueError(f"invalid whence value ({whence})")
        if target < 0:
            raise ValueError(f"Negative seek position is not allowed ({target})")
        self._pos = target
        return target

    def tell(self) -> int:
        self._check_validity()
        return self._pos

    def flush(self) -> None:
        self._check_validity()

    def next_buffer_slice(self, size: int) -> memoryview:
        """Writable view of the next ``size`` bytes; advances position and high-water mark (zero-copy writes)."""
        self._check_validity("write")
        if size < 0:
            raise ValueError(f"Size must be non-negative, got {size}")
        start = METADATA_SIZE + self._pos
        if start + size > len(self._mv):
            raise ValueError(
                f"Requested slice (size={size}) exceeds buffer capacity "
                f"(pos={self._pos}, cap={len(self._mv) - METADATA_SIZE})"
            )
        view = self._mv[start : start + size]
        self._pos += size
        self._update_written_data_length(self._pos)
        return view

    # ---- lifecycle ------------------------------------------------------------------------------------
    def _drop_views(self) -> None:
        self._metadata = None  # the ctypes view holds an export on the memoryview: drop it first
        if self._mv is not None:
            try:
                self._mv.release()
            except BufferError:
                pass  # a caller still holds a slice; the mapping goes away regardless
            self._mv = None

    def close(self, truncate: bool = True) -> None:
        if self.closed:
            return
        try:
            if truncate and not self.is_readonly:
                final_size = METADATA_SIZE + self._metadata.len_written_data
                self._drop_views()
                self.buffer_obj.close(truncate_size=final_size)
            else:
                self._drop_views()
                self.buffer_obj.close()
        finally:
            self._drop_views()
            self.buffer_obj = None
            self._pos = -1

    def resize(self, new_size: int) -> None:
        """Resizes the mapping to ``new_size`` bytes (metadata block included); the mapping may move."""
        self._check_validity("write")
        if new_size < METADATA_SIZE:
            raise ValueError(f"New size must be at least {METADATA_SIZE} bytes, got {new_size}.")
        self._drop_views()
        self.buffer_obj.resize(new_size)
        try:
            self._mv = memoryview(self.buffer_obj)
        except Exception:
            raise ValueError("Failed to recreate memoryview after resize.")
        self._bind_metadata()

    # ---- properties -----------------------------------------------------------------------------------
    @property
    def closed(self) -> bool:
        return self.buffer_obj is None or self.buffer_obj.closed

    @property
    def is_readonly(self) -> bool:
        self._check_validity()
        return self.buffer_obj.is_readonly

    @property
    def format_signature(self) -> bytes:
        self._check_validity()
        return self._metadata.format_signature

    def set_format_signature(self, signature: bytes) -> None:
        self._check_validity("write")
        if len(signature) > 8:
            raise ValueError(f"Format signature must be at most 8 bytes, got {len(signature)}")
        self._metadata.format_signature = signature

    @property
    def len_written_data(self) -> int:
        """High-water mark of the data section, in bytes."""
        self._check_validity()
        return self._metadata.len_written_data

    def raw_view(self) -> memoryview:
        """The whole mapping, metadata block included (no copy).  Valid until close() or resize()."""
        self._check_validity()
        return self._mv

    def data_address(self, pos: int = 0) -> int:
        """Raw address of data-section byte ``pos`` (for native copy engines that write around the stream)."""
        self._check_validity()
        return self.buffer_obj.get_data_ptr() + METADATA_SIZE + pos

    def reserve(self, nbytes: int) -> None:
        """Has the file system allocate the pages of the next ``nbytes`` of the data section now (they are zero
        until written).  For writers that know what they are about to fill: page allocation inside a page fault is
        several times slower than ahead of time.  A no-op where the buffer object cannot do it."""
        self._check_validity("write")
        ahead = getattr(self.buffer_obj, "reserve", None)
        if ahead is not None and nbytes > 0:
            ahead(METADATA_SIZE + self._pos, nbytes)

    def fileno(self) -> int:
        """Descriptor of the mapped file, for engines that read/write the file directly; -1 if the underlying
        buffer object does not expose one."""
        self._check_validity()
        getter = getattr(self.buffer_obj, "fileno", None)
        return getter() if getter is not None else -1

    def __enter__(self):
        self._check_validity()
        return self

    def __exit__(self, exc_type, exc_value, traceback):
        self.close()
