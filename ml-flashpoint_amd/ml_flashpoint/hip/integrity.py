"""CRC-32C sidecar of a checkpoint object.

The reference has no checksum and its readers ignore unknown files, so the per-chunk CRCs computed on the GPU are
kept *beside* the object (``.<object name>.crc32c`` in the same directory) and never inside it: the object's bytes
stay identical to the reference's.  Layout (little-endian): ``8s magic, u64 chunk_bytes, u64 data_bytes,
u64 n_chunks, u32[n_chunks]``.
"""

import os
import struct
from typing import Optional, Tuple

import numpy as np

_MAGIC = b"MLFCRC1\x00"
_HEAD = struct.Struct("<8sQQQ")


def sidecar_path(object_path: str) -> str:
    d, name = os.path.split(object_path)
    return os.path.join(d, f".{name}.crc32c")


def write_sidecar(object_path: str, chunk_bytes: int, data_bytes: int, crcs: np.ndarray) -> None:
    path = sidecar_path(object_path)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(_HEAD.pack(_MAGIC, chunk_bytes, data_bytes, len(crcs)))
        f.write(np.ascontiguousarray(crcs, dtype="<u4").tobytes())
    os.rename(tmp, path)


def remove_sidecar(object_path: str) -> None:
    """Drops the sidecar of an object that has just been rewritten without checksums: an old one would condemn it."""
    try:
        os.unlink(sidecar_path(object_path))
    except FileNotFoundError:
        pass


def read_sidecar(object_path: str) -> Optional[Tuple[int, int, np.ndarray]]:
    """Returns (chunk_bytes, data_bytes, crcs) or None if the object has no (valid) sidecar."""
    path = sidecar_path(object_path)
    try:
        with open(path, "rb") as f:
            raw = f.read()
    except OSError:
        return None
    if len(raw) < _HEAD.size:
        return None
    magic, chunk_bytes, data_bytes, n = _HEAD.unpack_from(raw, 0)
    if magic != _MAGIC or len(raw) != _HEAD.size + 4 * n:
        return None
    return chunk_bytes, data_bytes, np.frombuffer(raw, dtype="<u4", offset=_HEAD.size).copy()


class ChecksumMismatchError(RuntimeError):
    """A restored object's bytes do not match the CRC-32C recorded when it was saved."""
