"""Shared test setup: import paths, the ``gpu`` marker, and helpers to reach the oracle's C library."""

import ctypes
import os
import subprocess
import sys

import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG_ROOT = os.path.join(REPO, "ml-flashpoint_amd")
for p in (REPO, PKG_ROOT):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    try:
        import torch

        has_gpu = torch.cuda.is_available()
    except Exception:
        has_gpu = False
    if has_gpu:
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def oracle_c():
    """The oracle's C restatements (oracle/crc32c.c), built on demand where a compiler is present."""
    so = os.path.join(REPO, "oracle", "_build", "liboracle.so")
    if not os.path.exists(so):
        subprocess.check_call(["make", "-C", os.path.join(REPO, "oracle")])
    lib = ctypes.CDLL(so)
    lib.oracle_crc32c.restype = ctypes.c_uint32
    lib.oracle_crc32c.argtypes = [ctypes.c_char_p, ctypes.c_size_t]
    lib.oracle_crc32c_bitwise.restype = ctypes.c_uint32
    lib.oracle_crc32c_bitwise.argtypes = [ctypes.c_char_p, ctypes.c_size_t]
    lib.oracle_crc32c_chunks.restype = None
    lib.oracle_crc32c_chunks.argtypes = [ctypes.c_char_p, ctypes.c_size_t, ctypes.c_size_t, ctypes.c_void_p]
    lib.oracle_crc32c_combine.restype = ctypes.c_uint32
    lib.oracle_crc32c_combine.argtypes = [ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint64]
    return lib


@pytest.fixture
def shm_dir(tmp_path_factory):
    """A scratch directory on tmpfs when /dev/shm exists (the buffer files are meant to live there)."""
    import shutil
    import tempfile

    base = "/dev/shm" if os.path.isdir("/dev/shm") and os.access("/dev/shm", os.W_OK) else None
    d = tempfile.mkdtemp(prefix="mlf_test_", dir=base)
    yield d
    shutil.rmtree(d, ignore_errors=True)
