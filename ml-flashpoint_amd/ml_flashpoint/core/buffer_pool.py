"""A rank's pool of long-lived buffer files, and the stream type it hands out.

Why a pool: a checkpoint object written into a fresh tmpfs file pays for page allocation (4-9 GB/s on the MI355X
host, against 57 GB/s for the link), a file whose mapping stays open from save to save does not.  So the pool
creates ``num_buffers`` files ``buffer_<rank>_<idx>.dist`` once, keeps them mapped, and a checkpoint object
"acquired" from it is only a symlink to one of them.  Deleting the object (the symlink) is what gives the file
back: the pool notices on its next ``acquire``.

Behaviour, names and messages are the reference's (src/ml_flashpoint/core/buffer_pool.py:35-342); ``ensure_capacity``
is an addition for writers that know the total size up front, and so is ``prefault``: the reference creates its pool
files sparse (buffer_pool.py:324-342) and the first checkpoint into each pays for its pages - 10 s for a 112 GB
object against 2 s from then on.  With ``prefault`` (off unless asked for: it commits ``num_buffers x buffer_size``
of host memory, where sparse files only ever hold what was written) a background thread allocates and maps the
pages of every pool file right after the pool is created; a buffer is not lent out before its own file is done.
The step is skipped, with a warning, when the file system or the host does not have that much memory to spare.
"""

from __future__ import annotations

import dataclasses
import logging
import os
import threading
from typing import NamedTuple

from ml_flashpoint.checkpoint_object_manager.buffer_io import BufferIO
from ml_flashpoint.checkpoint_object_manager.buffer_metadata import METADATA_SIZE
from ml_flashpoint.checkpoint_object_manager.buffer_object.buffer_object_ext import BufferObject
from ml_flashpoint.core import utils
from ml_flashpoint.core.mlf_logging import get_logger

_LOGGER = get_logger(__name__)

# growth rule of a pooled stream that runs out of room: at least 10 % more, and at least 1 MiB beyond what is needed
RESIZE_FACTOR = 1.1
PADDING_SIZE = 1 << 20


class PooledBufferIO:
    """A ``BufferIO`` on loan from the pool.  Everything not defined here goes straight to the underlying stream.
    Two things differ: writing past the end grows the file instead of failing, and ``close`` ends the loan without
    unmapping - it only cuts the file to what was written, so readers of the symlink see an object of exact size."""

    def __init__(self, buffer_io: BufferIO):
        self._buffer_io = buffer_io
        self._closed = False

    def __getattr__(self, name):  # only reached for names this class does not define
        if self._closed:
            _LOGGER.warning("PooledBufferIO: Accessing closed buffer")
        return getattr(self._buffer_io, name)

    def __enter__(self):
        return self

    def __exit__(self, exc_type, exc_value, traceback):
        self.close()

    @property
    def closed(self) -> bool:
        return self._closed or self._buffer_io.closed

    @utils.log_execution_time(logger=_LOGGER, name="close", level=logging.INFO)
    def close(self, truncate: bool = True):
        already, self._closed = self._closed, True
        if already or not truncate or self._buffer_io.is_readonly:
            return
        try:
            exact = METADATA_SIZE + self._buffer_io._metadata.len_written_data
            if len(self._buffer_io._mv) != exact:
                self._buffer_io.resize(exact)
        except Exception:
            _LOGGER.warning("PooledBufferIO: Failed to truncate buffer during close.", exc_info=True)

    # ---- growing ----------------------------------------------------------------------------------------------------
    def _missing_room(self, more_bytes: int) -> bool:
        stream = self._buffer_io
        return METADATA_SIZE + stream.tell() + more_bytes > stream.buffer_obj.get_capacity()

    def _auto_resize(self, required_bytes: int):
        stream = self._buffer_io
        by_factor = stream.buffer_obj.get_capacity() * RESIZE_FACTOR
        by_need = METADATA_SIZE + stream.tell() + required_bytes + PADDING_SIZE
        stream.resize(int(max(by_factor, by_need)))

    def ensure_capacity(self, required_bytes: int) -> None:
        """Makes room for ``required_bytes`` at the current position in one step (one remap instead of several)."""
        if self._missing_room(required_bytes):
            self._auto_resize(required_bytes)

    def write(self, data: bytes) -> int:
        self.ensure_capacity(len(data))
        return self._buffer_io.write(data)

    def next_buffer_slice(self, size: int) -> memoryview:
        self.ensure_capacity(size)
        return self._buffer_io.next_buffer_slice(size)


@dataclasses.dataclass
class BufferPoolConfig:
    """Picklable description of a pool; the pool itself is created lazily in the process that writes."""

    pool_dir_path: str
    rank: int
    num_buffers: int
    buffer_size: int
    # allocate and map the pool files' pages in the background, right after creating them: num_buffers x buffer_size
    # of host memory from then on, so it is for the caller to ask for
    prefault: bool = False

    def __post_init__(self):
        if not self.pool_dir_path:
            raise ValueError("pool_dir_path must be provided in BufferPoolConfig")
        for name in ("rank", "num_buffers", "buffer_size"):
            given = getattr(self, name)
            if not (isinstance(given, int) and given >= 0):
                raise ValueError(f"{name} must be a non-negative integer in BufferPoolConfig")


class _Loan(NamedTuple):
    stream: BufferIO
    symlink: str | None  # None while the borrower has not named its object yet: never reclaimed


# pool files smaller than this are not worth a background thread: their pages cost microseconds
_PREFAULT_MIN_BYTES = 64 << 20


def _spare_bytes(directory: str) -> int:
    """What a prefault may commit: the smaller of the file system's free space and the host's available memory (a
    tmpfs reports its size limit, not what the host can still back), less a tenth of either for everybody else."""
    stat = os.statvfs(directory)
    spare = stat.f_bavail * stat.f_frsize
    try:
        with open("/proc/meminfo") as f:
            for line in f:
                if line.startswith("MemAvailable:"):
                    spare = min(spare, int(line.split()[1]) * 1024)
                    break
    except OSError:
        pass
    return spare - spare // 10


class BufferPool:
    def __init__(self, pool_dir_path: str, rank: int = 0, num_buffers: int = 3, buffer_size: int = 0,
                 prefault: bool = False, prefault_threads: int = 8):
        if num_buffers <= 0:
            raise ValueError(f"Number of buffers must be positive. Got {num_buffers}.")
        if buffer_size <= 0:
            raise ValueError(f"Buffer size must be positive. Got {buffer_size}.")
        if not pool_dir_path:
            raise ValueError("Pool directory path must be provided.")
        self.pool_dir, self.rank, self.num_buffers, self.buffer_size = pool_dir_path, rank, num_buffers, buffer_size
        self._lock = threading.Lock()
        self.active_buffers: dict[str, _Loan] = {}  # pool file path -> who has it
        os.makedirs(pool_dir_path, exist_ok=True)
        self.free_buffers: list[BufferIO] = [self._create(index) for index in range(num_buffers)]
        self._prefault_threads = prefault_threads
        self._prefaulted: dict[str, threading.Event] = {}  # pool file path -> set once its pages are in place
        self._prefault_worker: threading.Thread | None = None
        self.prefault_seconds = 0.0
        if prefault:
            self.start_prefault()

    def _create(self, index: int) -> BufferIO:
        path = os.path.join(self.pool_dir, f"buffer_{self.rank}_{index}.dist")
        return BufferIO(BufferObject(path, self.buffer_size, overwrite=True))

    def _preallocate_buffers(self) -> None:
        """(Re)creates the pool files; all of them must be free."""
        self.wait_prefault()
        self.free_buffers = [self._create(index) for index in range(self.num_buffers)]

    def start_prefault(self) -> None:
        """Pages and page-table entries of every free pool file, on a background thread, in the order in which the
        files will be lent out.  Best effort: a failure (a file system too small for all of them, say) is logged and
        the pages are left to the first save, as without this step.  Does nothing for files too small to matter, or
        when it is already running."""
        if self.buffer_size < _PREFAULT_MIN_BYTES or self._prefault_worker is not None:
            return
        order = list(reversed(self.free_buffers))  # acquire() pops from the end
        wanted = sum(stream.buffer_obj.get_capacity() for stream in order)
        spare = _spare_bytes(self.pool_dir)
        if wanted > spare:
            _LOGGER.warning("BufferPool: not prefaulting %d bytes of pool files in '%s': only %d bytes to spare; "
                            "their pages are left to the saves that fill them.", wanted, self.pool_dir, spare)
            return
        for stream in order:
            self._prefaulted[stream.buffer_obj.get_id()] = threading.Event()

        def run():
            import time

            t0 = time.perf_counter()
            for stream in order:
                pool_file = stream.buffer_obj.get_id()
                try:
                    ahead = getattr(stream.buffer_obj, "prefault", None)
                    if ahead is not None and not stream.closed:
                        ahead(0, stream.buffer_obj.get_capacity(), self._prefault_threads)
                except Exception:
                    _LOGGER.warning("BufferPool: could not prefault '%s'; its pages are left to the first save.",
                                    pool_file, exc_info=True)
                finally:
                    self._prefaulted[pool_file].set()
            self.prefault_seconds = time.perf_counter() - t0

        self._prefault_worker = threading.Thread(target=run, name="mlf-pool-prefault", daemon=True)
        self._prefault_worker.start()

    def wait_prefault(self) -> float:
        """Returns once the background page allocation (if any) has finished; the seconds it took."""
        worker = self._prefault_worker
        if worker is not None:
            worker.join()
        return self.prefault_seconds

    @utils.log_execution_time(logger=_LOGGER, name="acquire", level=logging.INFO)
    def acquire(self, associated_symlink: str | None = None) -> PooledBufferIO:
        """Lends out a free buffer, rewound and empty, and creates ``associated_symlink`` pointing at its file.
        ``RuntimeError`` when every buffer is on loan; if the link cannot be created the buffer stays free and the
        ``OSError`` is the caller's."""
        with self._lock:
            self._gc()
            if not self.free_buffers:
                raise RuntimeError(f"BufferPool exhausted. All {self.num_buffers} buffers are in use.")
            stream = self.free_buffers.pop()
            pool_file = stream.buffer_obj.get_id()
            self.active_buffers[pool_file] = _Loan(stream, None)  # taken; without a name it is never reclaimed
        ready = self._prefaulted.get(pool_file)
        if ready is not None:
            # the background thread is still mapping this file's pages: it may not be resized yet.  Waited for
            # outside the lock, so that other acquires and the reclaiming of deleted objects go on meanwhile.
            ready.wait()
        with self._lock:
            try:
                self._reuse_buffer(stream, associated_symlink)
            except Exception:
                self.active_buffers.pop(pool_file, None)
                self.free_buffers.append(stream)
                raise
            return PooledBufferIO(stream)

    @utils.log_execution_time(logger=_LOGGER, name="_reuse_buffer", level=logging.INFO)
    def _reuse_buffer(self, buffer_io: BufferIO, symlink: str | None) -> BufferIO:
        buffer_io.seek(0)
        buffer_io._metadata.len_written_data = 0
        pool_file = buffer_io.buffer_obj.get_id()
        self.active_buffers[pool_file] = _Loan(buffer_io, symlink)
        if symlink:
            os.symlink(pool_file, symlink)
        return buffer_io

    def _gc(self) -> None:
        """Takes back every buffer whose symlink no longer leads anywhere (``os.path.exists`` follows links, so a
        deleted link and a dangling one count alike)."""
        for pool_file, loan in list(self.active_buffers.items()):
            if loan.symlink and not os.path.exists(loan.symlink):
                del self.active_buffers[pool_file]
                self.free_buffers.append(loan.stream)

    def teardown(self) -> None:
        """Unmaps everything, on loan or not; the files stay where they are."""
        self.wait_prefault()
        with self._lock:
            streams = self.free_buffers + [loan.stream for loan in self.active_buffers.values()]
            self.free_buffers, self.active_buffers = [], {}
        for stream in streams:
            try:
                stream.close(truncate=True)
            except Exception:
                _LOGGER.warning("PooledBufferIO: Failed to close buffer during teardown.", exc_info=True)
