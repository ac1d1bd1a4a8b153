"""Per-rank pool of persistent, pre-allocated buffer files.

A checkpoint object acquired through the pool is a *symlink* to one of ``num_buffers`` files named
``buffer_<rank>_<idx>.dist``.  The mapping of a pool file stays open across checkpoints, so its pages stay
resident: after the first save a buffer is written without page faults.  A buffer returns to the free list
when its symlink no longer resolves.  Semantics follow the reference (src/ml_flashpoint/core/buffer_pool.py:35-342).
"""

import logging
import os
import threading
from dataclasses import dataclass
from typing import Dict, List, Optional

from ml_flashpoint.checkpoint_object_manager.buffer_io import BufferIO
from ml_flashpoint.checkpoint_object_manager.buffer_metadata import METADATA_SIZE
from ml_flashpoint.checkpoint_object_manager.buffer_object.buffer_object_ext import BufferObject
from ml_flashpoint.core.mlf_logging import get_logger
from ml_flashpoint.core.utils import log_execution_time

_LOGGER = get_logger(__name__)

PADDING_SIZE = 1024 * 1024
RESIZE_FACTOR = 1.1


class PooledBufferIO:
    """Proxy handed to writers: ``close()`` releases the proxy but keeps the pool's mapping alive, and writes
    grow the file on demand instead of failing."""

    def __init__(self, buffer_io: BufferIO):
        self._buffer_io = buffer_io
        self._closed = False

    def __getattr__(self, name):
        if self._closed:
            _LOGGER.warning("PooledBufferIO: Accessing closed buffer")
        return getattr(self._buffer_io, name)

    @log_execution_time(logger=_LOGGER, name="close", level=logging.INFO)
    def close(self, truncate: bool = True):
        if self._closed:
            return
        self._closed = True
        if not truncate or self._buffer_io.is_readonly:
            return
        try:
            wanted = METADATA_SIZE + self._buffer_io._metadata.len_written_data
            if wanted != len(self._buffer_io._mv):
                self._buffer_io.resize(wanted)
        except Exception:
            _LOGGER.warning("PooledBufferIO: Failed to truncate buffer during close.", exc_info=True)

    @property
    def closed(self) -> bool:
        return self._closed or self._buffer_io.closed

    def __enter__(self):
        return self

    def __exit__(self, exc_type, exc_value, traceback):
        self.close()

    def _auto_resize(self, required_bytes: int):
        """Grows the file so that ``required_bytes`` more fit at the current position: the larger of +10 % and
        exact need + 1 MiB."""
        capacity = self._buffer_io.buffer_obj.get_capacity()
        needed = METADATA_SIZE + self._buffer_io.tell() + required_bytes
        self._buffer_io.resize(int(max(capacity * RESIZE_FACTOR, needed + PADDING_SIZE)))

    def ensure_capacity(self, required_bytes: int) -> None:
        """Grows the file once, up front, when the total to be written from the current position is known."""
        if METADATA_SIZE + self._buffer_io.tell() + required_bytes > self._buffer_io.buffer_obj.get_capacity():
            self._auto_resize(required_bytes)

    def write(self, data: bytes) -> int:
        self.ensure_capacity(len(data))
        return self._buffer_io.write(data)

    def next_buffer_slice(self, size: int) -> memoryview:
        self.ensure_capacity(size)
        return self._buffer_io.next_buffer_slice(size)


@dataclass
class BufferPoolConfig:
    pool_dir_path: str
    rank: int
    num_buffers: int
    buffer_size: int

    def __post_init__(self):
        if not self.pool_dir_path:
            raise ValueError("pool_dir_path must be provided in BufferPoolConfig")
        for field in ("rank", "num_buffers", "buffer_size"):
            value = getattr(self, field)
            if not isinstance(value, int) or value < 0:
                raise ValueError(f"{field} must be a non-negative integer in BufferPoolConfig")


class BufferPool:
    def __init__(self, pool_dir_path: str, rank: int = 0, num_buffers: int = 3, buffer_size: int = 0):
        if num_buffers <= 0:
            raise ValueError(f"Number of buffers must be positive. Got {num_buffers}.")
        if buffer_size <= 0:
            raise ValueError(f"Buffer size must be positive. Got {buffer_size}.")
        if not pool_dir_path:
            raise ValueError("Pool directory path must be provided.")
        self.pool_dir = pool_dir_path
        self.rank = rank
        self.num_buffers = num_buffers
        self.buffer_size = buffer_size
        self.free_buffers: List[BufferIO] = []
        self.active_buffers: Dict[str, tuple[BufferIO, str]] = {}  # pool file path -> (stream, symlink path)
        self._lock = threading.Lock()
        os.makedirs(self.pool_dir, exist_ok=True)
        self._preallocate_buffers()

    def _preallocate_buffers(self) -> None:
        for idx in range(self.num_buffers):
            path = os.path.join(self.pool_dir, f"buffer_{self.rank}_{idx}.dist")
            self.free_buffers.append(BufferIO(BufferObject(path, self.buffer_size, overwrite=True)))

    @log_execution_time(logger=_LOGGER, name="acquire", level=logging.INFO)
    def acquire(self, associated_symlink: Optional[str] = None) -> PooledBufferIO:
        """Hands out a free pool buffer and links ``associated_symlink`` to it; raises RuntimeError when all
        buffers are in use."""
        with self._lock:
            self._gc()
            if not self.free_buffers:
                raise RuntimeError(f"BufferPool exhausted. All {self.num_buffers} buffers are in use.")
            candidate = self.free_buffers.pop()
            try:
                return PooledBufferIO(self._reuse_buffer(candidate, associated_symlink))
            except Exception:
                self.active_buffers.pop(candidate.buffer_obj.get_id(), None)
                self.free_buffers.append(candidate)
                raise

    def _gc(self) -> None:
        """Frees buffers whose symlink is gone or dangling (``exists`` follows the link on purpose)."""
        stale = [path for path, (_, link) in self.active_buffers.items() if link and not os.path.exists(link)]
        for path in stale:
            stream, _ = self.active_buffers.pop(path)
            self.free_buffers.append(stream)

    @log_execution_time(logger=_LOGGER, name="_reuse_buffer", level=logging.INFO)
    def _reuse_buffer(self, buffer_io: BufferIO, symlink: Optional[str]) -> BufferIO:
        buffer_io.seek(0)
        buffer_io._metadata.len_written_data = 0
        path = buffer_io.buffer_obj.get_id()
        self.active_buffers[path] = (buffer_io, symlink)
        if symlink:
            os.symlink(path, symlink)
        return buffer_io

    def teardown(self) -> None:
        """Closes every mapping; the files stay on disk."""
        with self._lock:
            streams = list(self.free_buffers) + [s for s, _ in self.active_buffers.values()]
            self.free_buffers.clear()
            self.active_buffers.clear()
            for stream in streams:
                try:
                    stream.close(truncate=True)
                except Exception:
                    _LOGGER.warning("PooledBufferIO: Failed to close buffer during teardown.", exc_info=True)
