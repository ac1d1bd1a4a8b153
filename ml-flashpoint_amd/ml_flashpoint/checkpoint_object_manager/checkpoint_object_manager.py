"""Where checkpoint buffers come from and go to: create (``acquire_buffer``), open read-only (``get_buffer``), close,
delete.  One instance per saver/loader; the buffer pool behind it is one per process.

Behaviour, names and messages are the reference's (src/ml_flashpoint/checkpoint_object_manager/
checkpoint_object_manager.py:30-284).  What matters for the MI355X path: an acquired buffer is preferably a pooled one
(a symlink to a file whose mapping and pages outlive the checkpoint, see ``core/buffer_pool.py``), and only if the
pool has none left a file of its own, whose pages are then faulted in while the image arrives.
"""

from __future__ import annotations

import os
import shutil
import threading
from typing import ClassVar

from ml_flashpoint.checkpoint_object_manager.buffer_io import BufferIO
from ml_flashpoint.checkpoint_object_manager.buffer_metadata import METADATA_SIZE
from ml_flashpoint.checkpoint_object_manager.buffer_object.buffer_object_ext import BufferObject
from ml_flashpoint.core.buffer_pool import BufferPool, BufferPoolConfig
from ml_flashpoint.core.checkpoint_id_types import CheckpointContainerId, CheckpointObjectId
from ml_flashpoint.core.mlf_logging import get_logger

_LOGGER = get_logger(__name__)


class CheckpointObjectManager:
    # The pool belongs to the process, not to a manager: managers are pickled into worker processes (where the first
    # acquire creates that process's pool from the configuration) and several of them may coexist.
    _worker_pool: ClassVar[BufferPool | None] = None
    _worker_pool_lock: ClassVar[threading.Lock] = threading.Lock()

    def __init__(self, pool_config: BufferPoolConfig | None = None):
        self._pool_config = pool_config

    # ---- the process-wide pool ----------------------------------------------------------------------------------
    def _get_or_create_buffer_pool(self) -> BufferPool | None:
        """This process's pool; created on first use if this manager has a configuration.  None without one, and
        None (with the failure logged) if creating it fails - callers then fall back to stand-alone files."""
        owner = CheckpointObjectManager
        if owner._worker_pool or not self._pool_config:
            return owner._worker_pool or None
        with owner._worker_pool_lock:
            if owner._worker_pool is None:
                try:
                    wanted = self._pool_config
                    owner._worker_pool = BufferPool(pool_dir_path=wanted.pool_dir_path, rank=wanted.rank,
                                                    num_buffers=wanted.num_buffers, buffer_size=wanted.buffer_size)
                    if getattr(wanted, "prefault", False):
                        owner._worker_pool.start_prefault()
                except Exception:
                    _LOGGER.exception("Failed to initialize BufferPool")
            return owner._worker_pool

    def warm_up_pool(self, wait: bool = False) -> float:
        """Creates this process's pool now instead of at the first ``acquire_buffer``, so that the background
        allocation of its files' pages (``BufferPoolConfig.prefault``) runs while the job is still starting up.
        ``wait``: return only when that has finished.  Returns the seconds the allocation has taken so far (0.0
        without a pool, or while it is still running and ``wait`` is false)."""
        pool = self._get_or_create_buffer_pool()
        if pool is None:
            return 0.0
        return pool.wait_prefault() if wait else pool.prefault_seconds

    def teardown_pool(self):
        owner = CheckpointObjectManager
        with owner._worker_pool_lock:
            pool, owner._worker_pool = owner._worker_pool, None
        if pool is None:
            return
        try:
            pool.teardown()
        except Exception as e:
            _LOGGER.debug("Failed to teardown BufferPool: %s", e)

    # ---- buffers ------------------------------------------------------------------------------------------------
    def acquire_buffer(self, object_id: CheckpointObjectId, buffer_size: int, overwrite: bool = True) -> "BufferIO":
        """A writable stream for a new object with room for ``buffer_size`` bytes of data (the 4096-byte metadata
        block comes on top; a pooled buffer may be smaller and grows as it is written).  An existing object is
        replaced, or ``FileExistsError`` with ``overwrite=False``; any other failure to create the buffer is a
        ``RuntimeError`` that names the object."""
        if buffer_size <= 0:
            raise ValueError("Buffer size must be a positive integer.")
        path = str(object_id)
        try:
            os.makedirs(os.path.dirname(path), exist_ok=True)
            if os.path.exists(path):
                if not overwrite:
                    raise FileExistsError(f"File {object_id} already exists and overwrite=False")
                self.delete_object(object_id)
            pool = self._get_or_create_buffer_pool()
            if pool:
                return pool.acquire(associated_symlink=path)
        except RuntimeError:  # every pooled buffer is taken
            _LOGGER.debug("BufferPool exhausted. Falling back to standalone buffer creation.")
        try:
            return BufferIO(BufferObject(path, METADATA_SIZE + buffer_size, overwrite))
        except Exception as e:
            _LOGGER.exception("Failed to create buffer for object_id='%s'", object_id)
            raise RuntimeError(f"Failed to create buffer for '{object_id}'") from e

    def get_buffer(self, object_id: CheckpointObjectId) -> "BufferIO | None":
        """A read-only stream over an existing object, or None if it cannot be opened as one (missing, a directory,
        shorter than a metadata block, ...)."""
        try:
            return BufferIO(BufferObject(str(object_id)))
        except (OSError, ValueError, RuntimeError):
            _LOGGER.exception("Could not open buffer '%s'. Returning None.", object_id)
        return None

    def close_buffer(self, buffer_io: BufferIO, skip_close_if_symlink: bool = False, truncate: bool = True) -> None:
        """Closes an open ``BufferIO`` (anything else is ignored with a warning).  ``skip_close_if_symlink`` leaves a
        stream whose object is a symlink - a pooled buffer - open for its owner."""
        if not isinstance(buffer_io, BufferIO) or buffer_io.closed:
            _LOGGER.warning("Attempted to close an invalid or already-closed buffer. Ignoring.")
        elif not (skip_close_if_symlink and os.path.islink(buffer_io.buffer_obj.get_id())):
            buffer_io.close(truncate=truncate)

    # ---- deletion -------------------------------------------------------------------------------------------------
    def delete_object(self, object_id: CheckpointObjectId) -> None:
        """Removes the object's file or symlink (a dangling symlink too); a missing one is only worth a warning."""
        path = str(object_id)
        if not os.path.lexists(path):
            _LOGGER.warning("Object '%s' does not exist. Nothing to delete.", path)
            return
        os.remove(path)

    def delete_container(self, container_id: CheckpointContainerId) -> None:
        """Removes a container directory with everything in it.  Files that vanish while it runs (another rank is
        deleting the same tree) are passed over; a path that is not a directory is left alone."""
        path = str(container_id)
        if not os.path.isdir(path):
            _LOGGER.warning("Container '%s' is not a directory or does not exist. Nothing to delete from disk.", path)
            return

        def unless_already_gone(function, failed_path, exc_info):
            if not isinstance(exc_info[1], FileNotFoundError):
                raise exc_info[1]

        shutil.rmtree(path, onerror=unless_already_gone)


def _fresh_pool_lock_after_fork() -> None:
    """The class-level lock may have been held by a thread of the parent that the forked child does not have."""
    CheckpointObjectManager._worker_pool_lock = threading.Lock()


if hasattr(os, "register_at_fork"):
    os.register_at_fork(after_in_child=_fresh_pool_lock_after_fork)
