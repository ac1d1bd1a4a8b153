"""Record header of the MLF_TENS format: ``<u32 little-endian length><pickle of TensorHeader>``.

The pickle embeds this module's qualified name and the field order ``dtype, shape``; both are part of the
byte format (reference: src/ml_flashpoint/core/tensor_header.py:23-56).  The protocol is pinned to 4, the
default of CPython 3.8-3.13 which the reference relies on implicitly.
"""

import dataclasses
import pickle
import struct
from typing import Tuple

import torch

_PICKLE_PROTOCOL = 4
_LEN = struct.Struct("<I")


@dataclasses.dataclass
class TensorHeader:
    dtype: torch.dtype
    shape: torch.Size

    def to_bytes(self) -> bytes:
        body = pickle.dumps(self, protocol=_PICKLE_PROTOCOL)
        return _LEN.pack(len(body)) + body

    @classmethod
    def from_bytes(cls, buffer: bytes) -> Tuple["TensorHeader", int]:
        (n,) = _LEN.unpack_from(buffer, 0)
        end = _LEN.size + n
        return pickle.loads(buffer[_LEN.size : end]), end
