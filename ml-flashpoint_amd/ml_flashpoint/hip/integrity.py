"""CRC-32C sidecar of a checkpoint object.

The reference has no checksum, so the per-chunk CRCs computed on the GPU never go inside the object (its bytes stay
identical to the reference's) - and not inside its container directory either: the reference's recovery discovery
lists every entry of a container as an object of the checkpoint (src/ml_flashpoint/core/checkpoint_loader.py:601-603)
and would offer, plan and fetch a sidecar like one.  A sidecar lives beside the container instead:

    <base>/step-N_ckpt/<object name>                          the object
    <base>/.mlf_crc32c/step-N_ckpt/<object name>.crc32c       its sidecar

(the directory name does not match ``step-<N>_ckpt``, so the scan for candidate checkpoints,
checkpoint_loader.py:532-547, passes over it).  A copy of an object that arrived on another node through the
reference's transfer service has no sidecar there and is accepted unchecked, like any object without one; a
replication manager that wants replicas to be verifiable sends ``sidecar_path(object)`` along with the object.

Layout (little-endian): ``8s magic, u64 chunk_bytes, u64 data_bytes, u64 n_chunks, u32[n_chunks]``.
"""

import os
import struct
from typing import Optional, Tuple

import numpy as np

_MAGIC = b"MLFCRC1\x00"
_HEAD = struct.Struct("<8sQQQ")


SIDECAR_DIR = ".mlf_crc32c"


def sidecar_dir(container_path: str) -> str:
    """Where the sidecars of a container's objects are kept: beside the container, not in it."""
    base, container = os.path.split(os.path.normpath(container_path))
    return os.path.join(base, SIDECAR_DIR, container)


def sidecar_path(object_path: str) -> str:
    container, name = os.path.split(object_path)
    return os.path.join(sidecar_dir(container), f"{name}.crc32c")


def write_sidecar(object_path: str, chunk_bytes: int, data_bytes: int, crcs: np.ndarray) -> None:
    path = sidecar_path(object_path)
    os.makedirs(os.path.dirname(path), exist_ok=True)
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
