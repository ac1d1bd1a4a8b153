"""The C-ABI libraries load without a GPU and export every entry point the headers declare.

No kernel is launched here; only host-side entry points are called.
"""

import ctypes
import os
import re

import numpy as np
import pytest

from conftest import PKG_ROOT, REPO

LIB_DIR = os.path.join(PKG_ROOT, "lib")


def _declared(header):
    text = open(os.path.join(REPO, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mlf_[a-z0-9_]+)\s*\(", text)))


@pytest.mark.parametrize("header,lib", [("mlf_buffer.h", "libmlf_buffer.so"), ("mlf_hip.h", "libmlf_hip.so")])
def test_library_exports_every_declared_symbol(header, lib):
    names = _declared(header)
    assert len(names) >= 10
    handle = ctypes.CDLL(os.path.join(LIB_DIR, lib))
    missing = [n for n in names if not hasattr(handle, n)]
    assert not missing, f"{lib} lacks {missing}"


def test_python_binding_covers_the_hip_header():
    from ml_flashpoint.hip import _lib

    assert sorted(_lib.exported_symbols()) == _declared("mlf_hip.h")
    _lib.load()  # resolves every symbol and sets its signature


def test_item_struct_layout_matches_the_header():
    from ml_flashpoint.hip import _lib

    offsets = {name: _lib.ITEM_DTYPE.fields[name][1] for name in _lib.ITEM_DTYPE.names}
    assert offsets == {"ptr": 0, "image_off": 8, "nbytes": 16, "kind": 24, "elem_size": 28, "ndim": 32,
                       "reserved": 36, "shape": 40, "stride": 104, "image_stride": 168}
    assert _lib.ITEM_DTYPE.itemsize == 232


def test_host_crc_and_combine_entry_points(oracle_c):
    from ml_flashpoint.hip import plan as P

    rng = np.random.default_rng(9)
    for n in (0, 1, 7, 8, 9, 63, 1000, 65537):
        data = rng.bytes(n)
        buf = ctypes.create_string_buffer(data, max(n, 1))
        assert P.crc32c_host(ctypes.addressof(buf), n) == oracle_c.oracle_crc32c(data, n)
    a, b = rng.bytes(1234), rng.bytes(77)
    whole = oracle_c.oracle_crc32c(a + b, len(a + b))
    assert P.crc32c_combine(oracle_c.oracle_crc32c(a, len(a)), oracle_c.oracle_crc32c(b, len(b)), len(b)) == whole
    assert P.crc32c_combine(0x12345678, 0, 0) == 0x12345678


def test_host_parallel_memcpy():
    lib = ctypes.CDLL(os.path.join(LIB_DIR, "libmlf_buffer.so"))
    lib.mlf_host_parallel_memcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
    rng = np.random.default_rng(4)
    for n in (0, 1, 4095, (9 << 20) + 17):
        src = np.frombuffer(rng.bytes(n), dtype=np.uint8).copy()
        dst = np.zeros(n + 8, dtype=np.uint8)
        assert lib.mlf_host_parallel_memcpy(dst.ctypes.data, src.ctypes.data, n, 4) == 0
        assert (dst[:n] == src).all() and not dst[n:].any()


def test_hip_saver_refuses_to_exist_without_the_library(monkeypatch, tmp_path):
    from ml_flashpoint.hip import _lib

    monkeypatch.setattr(_lib, "_LIB", None)
    monkeypatch.setenv("MLF_HIP_LIBRARY", str(tmp_path / "nope.so"))
    from ml_flashpoint.checkpoint_object_manager.checkpoint_object_manager import CheckpointObjectManager
    from ml_flashpoint.hip.checkpoint_saver import HipMLFlashpointCheckpointSaver

    with pytest.raises(ImportError, match="HIP data-path library not found"):
        HipMLFlashpointCheckpointSaver(lambda: 0, lambda: 0, lambda: None, CheckpointObjectManager())
