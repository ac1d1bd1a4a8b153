"""Small helpers shared by the save/restore path (reference: src/ml_flashpoint/core/utils.py:27-159)."""

import contextlib
import gc
import logging
import os
import threading
import time

import torch

_ENV_PREFIX = "MLFLASHPOINT_"


def get_env_var_prefix() -> str:
    return _ENV_PREFIX


def get_env_val_str(env_var_name: str, default_val: str) -> str:
    return os.environ.get(_ENV_PREFIX + env_var_name, default_val)


def get_env_val_int(env_var_name: str, default_val: int) -> int:
    raw = os.environ.get(_ENV_PREFIX + env_var_name)
    if raw is None:
        return default_val
    try:
        return int(raw)
    except ValueError:
        return default_val


def get_env_val_bool(env_var_name: str, default_val: bool) -> bool:
    raw = os.environ.get(_ENV_PREFIX + env_var_name)
    if raw is None:
        return default_val
    return raw.strip().lower() in ("1", "true", "yes", "on")


def get_accelerator_count() -> int:
    """Accelerators visible to this process (0 without a GPU)."""
    try:
        return torch.cuda.device_count()
    except Exception:
        return 0


def get_num_of_nodes() -> int:
    for var in ("NNODES", "SLURM_NNODES"):
        raw = os.environ.get(var)
        if raw:
            try:
                return max(int(raw), 1)
            except ValueError:
                pass
    return 1


@contextlib.contextmanager
def log_execution_time(logger: logging.Logger, name: str, level: int = logging.DEBUG):
    """Context manager *and* decorator that logs ``"<name> took <sec>s"`` (format kept: log parsers rely on it)."""
    start = time.perf_counter()
    try:
        yield
    finally:
        if logger.isEnabledFor(level):
            logger.log(level, "%s took %.4fs", name, time.perf_counter() - start)


def log_rate(logger: logging.Logger, verb: str, nbytes: int, seconds: float, count: int, what: str) -> None:
    """One INFO line ``"<verb> N bytes in S s (R GB/s) from C <what>"`` for a finished transfer."""
    if seconds > 0:
        logger.info("%s %d bytes in %.4f s (%.2f GB/s) from %d %s", verb, nbytes, seconds, nbytes / 1e9 / seconds, count, what)


_gc_pause_lock = threading.Lock()
_gc_pause_depth = 0
_gc_was_enabled = False


def _fresh_gc_pause_state_after_fork() -> None:
    """A forked child (an async framework's worker) inherits the lock in whatever state some other thread of the parent
    left it, and none of those threads: start over with a free lock, no pause in progress, and the collector as it
    was before the pause the fork may have fallen into."""
    global _gc_pause_lock, _gc_pause_depth
    if _gc_pause_depth > 0 and _gc_was_enabled:
        gc.enable()
    _gc_pause_lock = threading.Lock()
    _gc_pause_depth = 0


if hasattr(os, "register_at_fork"):
    os.register_at_fork(after_in_child=_fresh_gc_pause_state_after_fork)


@contextlib.contextmanager
def gc_paused():
    """Suspends the cyclic garbage collector for the duration of the block (re-entrant, thread-safe, restores the
    previous state).  The save and restore paths build tens of thousands of short-lived tuples and descriptors per
    checkpoint; every few hundred allocations CPython then walks the young generations, and periodically all live
    containers of the process, which more than doubles the planning time of a 20 000-tensor checkpoint.  Nothing
    built there forms reference cycles, so plain reference counting frees it."""
    global _gc_pause_depth, _gc_was_enabled
    with _gc_pause_lock:
        if _gc_pause_depth == 0:
            _gc_was_enabled = gc.isenabled()
            gc.disable()
        _gc_pause_depth += 1
    try:
        yield
    finally:
        with _gc_pause_lock:
            _gc_pause_depth -= 1
            if _gc_pause_depth == 0 and _gc_was_enabled:
                gc.enable()
