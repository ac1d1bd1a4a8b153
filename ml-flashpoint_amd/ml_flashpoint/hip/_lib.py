"""ctypes binding of ``libmlf_hip.so`` (declared in ``include/mlf_hip.h``).

Loading is strict: if the library is missing or a symbol cannot be resolved, importing the HIP saver/loader
fails with an ImportError that says how to build it.  There is no CPU fallback behind these calls.
"""

import ctypes
import os
from typing import Optional

import numpy as np

MAX_DIMS = 8
ITEM_DEVICE = 0
ITEM_BLOB = 1

# numpy mirror of ``struct mlf_item`` (232 bytes, natural alignment, no padding)
ITEM_DTYPE = np.dtype(
    [
        ("ptr", "<u8"),
        ("image_off", "<u8"),
        ("nbytes", "<u8"),
        ("kind", "<u4"),
        ("elem_size", "<u4"),
        ("ndim", "<u4"),
        ("reserved", "<u4"),
        ("shape", "<i8", (MAX_DIMS,)),
        ("stride", "<i8", (MAX_DIMS,)),
        ("image_stride", "<i8", (MAX_DIMS,)),
    ]
)
assert ITEM_DTYPE.itemsize == 232


class PlanOpts(ctypes.Structure):
    _fields_ = [
        ("tile_bytes", ctypes.c_uint32),
        ("block_threads", ctypes.c_uint32),
        ("align_to_tensor", ctypes.c_uint32),
        ("unroll", ctypes.c_uint32),
        ("grid_x_log2", ctypes.c_uint32),
        ("crc_chunk_kib", ctypes.c_uint32),
    ]


class PlanInfo(ctypes.Structure):
    _fields_ = [
        (name, ctypes.c_uint64)
        for name in (
            "n_items",
            "n_flat_tiles",
            "n_strided_items",
            "n_strided_work",
            "n_transposed_items",
            "n_transposed_work",
            "device_bytes",
            "blob_bytes",
            "image_bytes",
            "table_bytes",
            "n_small_items",
            "fused_crc_bytes",
            "crc_chunks",
        )
    ]


class XferStats(ctypes.Structure):
    _fields_ = [
        ("seconds", ctypes.c_double),
        ("wait_seconds", ctypes.c_double),
        ("bytes", ctypes.c_uint64),
        ("chunks", ctypes.c_uint64),
    ]


_VP = ctypes.c_void_p
_U64 = ctypes.c_uint64
_U32 = ctypes.c_uint32
_INT = ctypes.c_int

_SIGNATURES = {
    "mlf_hip_last_error": (ctypes.c_char_p, []),
    "mlf_hip_device_count": (_INT, [ctypes.POINTER(_INT)]),
    "mlf_hip_set_device": (_INT, [_INT]),
    "mlf_hip_mem_info": (_INT, [ctypes.POINTER(_U64), ctypes.POINTER(_U64)]),
    "mlf_plan_create": (_INT, [_VP, _U64, _VP, _U64, _U64, ctypes.POINTER(PlanOpts), ctypes.POINTER(_VP)]),
    "mlf_plan_destroy": (_INT, [_VP]),
    "mlf_plan_get_info": (_INT, [_VP, ctypes.POINTER(PlanInfo)]),
    "mlf_plan_update_blob": (_INT, [_VP, _VP, _U64, _VP]),
    "mlf_plan_crc_values": (_INT, [_VP, _VP, _U64]),
    "mlf_pack_launch": (_INT, [_VP, _VP, _VP]),
    "mlf_unpack_launch": (_INT, [_VP, _VP, _VP]),
    "mlf_crc32c_device": (_INT, [_VP, _U64, _U64, _VP, _U64, _VP]),
    "mlf_crc32c_device_noalloc": (_INT, [_VP, _U64, _U64, _VP, _U64, _VP]),
    "mlf_crc32c_host": (_U32, [_VP, _U64]),
    "mlf_crc32c_combine": (_U32, [_U32, _U32, _U64]),
    "mlf_crc32c_file": (_INT, [_INT, _U64, _U64, _U64, _VP, _U64, _U32]),
    "mlf_engine_create": (_INT, [_U64, _U32, _U32, ctypes.POINTER(_VP)]),
    "mlf_engine_destroy": (_INT, [_VP]),
    "mlf_engine_d2h": (_INT, [_VP, _VP, _VP, _U64, _VP, ctypes.POINTER(XferStats)]),
    "mlf_engine_h2d": (_INT, [_VP, _VP, _VP, _U64, _VP, ctypes.POINTER(XferStats)]),
    "mlf_engine_d2h_crc": (_INT, [_VP, _VP, _VP, _U64, _VP, _U64, _VP, _U64, ctypes.POINTER(XferStats)]),
    "mlf_engine_d2h_watched": (_INT, [_VP, _VP, _VP, _U64, _VP, _U64, _VP, _U64, _VP, ctypes.POINTER(XferStats)]),
    "mlf_engine_d2h_gated": (_INT, [_VP, _VP, _VP, _U64, _VP, _U64, _VP, _U64, _VP, ctypes.POINTER(XferStats)]),
    "mlf_engine_link_probe": (_INT, [_VP, _VP, _U64, _INT, ctypes.POINTER(ctypes.c_double)]),
    "mlf_engine_avoid_streams": (_INT, [_VP, ctypes.POINTER(_VP), _U32, ctypes.POINTER(_U32)]),
    "mlf_engine_checksum_stream": (_VP, [_VP]),
    "mlf_engine_set_host_checksums": (_INT, [_VP, _INT]),
    "mlf_engine_d2h_cut": (_INT, [_VP, _VP, _VP, _U64, _VP, _VP, _U64, _U64, _VP, _U64, _VP, ctypes.POINTER(XferStats)]),
    "mlf_engine_host_copy_cut": (_INT, [_VP, _VP, _VP, _U64, _U64, _U64, _VP, _U64]),
    "mlf_engine_read_file": (_INT, [_VP, _INT, _U64, _VP, _U64]),
    "mlf_engine_host_copy": (_INT, [_VP, _VP, _VP, _U64]),
    "mlf_engine_d2h_fd": (_INT, [_VP, _VP, _INT, _U64, _U64, _VP, ctypes.POINTER(XferStats)]),
    "mlf_engine_h2d_fd": (_INT, [_VP, _INT, _U64, _VP, _U64, _VP, ctypes.POINTER(XferStats)]),
}

_LIB: Optional[ctypes.CDLL] = None


def library_path() -> str:
    here = os.path.dirname(os.path.abspath(__file__))
    return os.environ.get("MLF_HIP_LIBRARY", os.path.normpath(os.path.join(here, "..", "..", "lib", "libmlf_hip.so")))


def exported_symbols():
    return tuple(_SIGNATURES)


def load() -> ctypes.CDLL:
    """Returns the loaded library; raises ImportError if it cannot be loaded (no fallback)."""
    global _LIB
    if _LIB is not None:
        return _LIB
    path = library_path()
    if not os.path.exists(path):
        raise ImportError(
            f"HIP data-path library not found at {path}. Build it with `make -C ml-flashpoint_amd/csrc all` "
            "(hipcc, --offload-arch=gfx950)."
        )
    try:
        lib = ctypes.CDLL(path)
    except OSError as e:
        raise ImportError(f"could not load {path}: {e}") from e
    for name, (restype, argtypes) in _SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError as e:
            raise ImportError(f"{path} does not export {name}") from e
        fn.restype = restype
        fn.argtypes = argtypes
    _LIB = lib
    return lib


class HipError(RuntimeError):
    pass


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().mlf_hip_last_error().decode("utf-8", "replace")
        raise HipError(f"{what} failed (code {rc}): {msg}")
