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


class ChunkChecksums:
    """Per-chunk CRC-32C of a data section that is checksummed piece by piece.

    An object that leaves the device in several transfers (windows, pieces) is cut where records end, not where
    checksum chunks end.  Each piece is checksummed where it lies, cut on the chunk grid of the data section - the
    first value covers the bytes up to the next chunk boundary, the following ones whole chunks, the last one what
    is left - and the values of the parts of one chunk are joined here: crc(A || B) = crc(A) * x^(8 |B|) + crc(B)
    over GF(2), the law ``mlf_crc32c_combine`` implements.  Pieces must arrive in ascending order and without gaps;
    ``result`` refuses an incomplete section."""

    def __init__(self, chunk_bytes: int, data_bytes: int, combine=None):
        if chunk_bytes <= 0:
            raise ValueError("chunk_bytes must be positive")
        if combine is None:
            from ml_flashpoint.hip import plan as hip_plan

            combine = hip_plan.crc32c_combine
        self._combine = combine
        self.chunk_bytes, self.data_bytes = chunk_bytes, data_bytes
        self._values = np.zeros(-(-data_bytes // chunk_bytes), dtype=np.uint32)
        self._at = 0  # the section is covered up to here

    @staticmethod
    def cuts(offset: int, nbytes: int, chunk_bytes: int) -> list:
        """[(first byte, length)] of the parts of [offset, offset + nbytes) between chunk boundaries."""
        parts, at, end = [], offset, offset + nbytes
        while at < end:
            stop = min((at // chunk_bytes + 1) * chunk_bytes, end)
            parts.append((at, stop - at))
            at = stop
        return parts

    def add(self, offset: int, nbytes: int, values) -> None:
        """``values``: one CRC-32C per part of ``cuts(offset, nbytes, chunk_bytes)``."""
        if offset != self._at:
            raise ValueError(f"piece at {offset} does not continue the section, which is covered up to {self._at}")
        parts = self.cuts(offset, nbytes, self.chunk_bytes)
        if len(values) != len(parts):
            raise ValueError(f"{len(values)} checksums for {len(parts)} parts")
        for (first, length), value in zip(parts, values):
            k = first // self.chunk_bytes
            if first % self.chunk_bytes == 0:
                self._values[k] = int(value)
            else:
                self._values[k] = self._combine(int(self._values[k]), int(value), length)
        self._at = offset + nbytes

    def result(self) -> np.ndarray:
        if self._at != self.data_bytes:
            raise ValueError(f"checksums cover {self._at} of {self.data_bytes} bytes")
        return self._values
