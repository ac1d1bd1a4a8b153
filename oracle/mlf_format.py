"""CPU oracle, part 1: the byte format of an ML Flashpoint checkpoint object, restated from first principles.

TEST INFRASTRUCTURE ONLY.  Nothing under ``oracle/`` is imported by the shipped package; only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may use it, as the checker.

Each function restates one piece of the reference and says which lines it follows:

* ``metadata_block``   - checkpoint_object_manager/buffer_metadata.py:18-37 (4096-byte packed little-endian block)
* ``header_bytes``     - core/tensor_header.py:30-39, i.e. ``<u32 len> + pickle.dumps(TensorHeader(dtype, shape))``
                         written out opcode by opcode (CPython protocol 4), *without* calling pickle
* ``payload_bytes``    - core/checkpoint_saver.py:786-800: C-contiguous, row-major, native little-endian bytes of
                         the logical tensor; strides are not stored; zero-size tensors have no payload
* ``data_section``     - core/checkpoint_saver.py:667-698: tensors first, then byte blobs, back to back from data
                         offset 0; offset/length bookkeeping of each item
* ``file_image``       - buffer_io.py:360-383: file = metadata block + data section, truncated to 4096 + written
* ``parse_record`` / ``read_item`` - core/checkpoint_loader.py:177-219 (header parse, reshape, narrow by index)

How it is pinned (see tests/test_oracle_*.py): ``header_bytes`` against 24 golden vectors produced by the reference's
own ``TensorHeader.to_bytes`` (tests/golden/tensor_header_vectors.json) and against ``pickle.loads`` round trips;
``metadata_block`` against ``struct`` closed forms; ``payload_bytes`` against ``numpy.tobytes`` for the dtypes numpy
has and against hand-written byte strings for bf16/fp8; ``data_section`` against the offset invariants the reference's
tests assert (tests/core/test_checkpoint_saver.py:1297-1307,1394-1431); ``read_item`` against the reference's
known-answer sub-box reads (tests/core/test_checkpoint_loader.py:223-302).
"""

import struct
import warnings
from typing import List, Sequence, Tuple

import numpy as np
import torch

METADATA_SIZE = 4096
SIGNATURE_MLF = b"MLF_TENS"
SIGNATURE_TORCH = b"TORCH___"
_HEADER_MODULE = "ml_flashpoint.core.tensor_header"
_HEADER_CLASS = "TensorHeader"


# ---- metadata block -------------------------------------------------------------------------------------------
def metadata_block(len_written_data: int, signature: bytes = SIGNATURE_MLF) -> bytes:
    if len(signature) > 8:
        raise ValueError("signature longer than 8 bytes")
    return struct.pack("<Q8s", len_written_data, signature) + bytes(METADATA_SIZE - 16)


# ---- record header (hand-rolled protocol-4 pickle) ------------------------------------------------------------
_MEMOIZE = b"\x94"


def _short_str(s: str) -> bytes:
    raw = s.encode("utf-8")
    assert len(raw) < 256
    return b"\x8c" + bytes([len(raw)]) + raw + _MEMOIZE  # SHORT_BINUNICODE + MEMOIZE


def _global(module: str, name: str) -> bytes:
    return _short_str(module) + _short_str(name) + b"\x93" + _MEMOIZE  # STACK_GLOBAL + MEMOIZE


def _int(v: int) -> bytes:
    if v < 0:
        raise ValueError("negative dimension")
    if v < 1 << 8:
        return b"K" + bytes([v])  # BININT1
    if v < 1 << 16:
        return b"M" + struct.pack("<H", v)  # BININT2
    if v < 1 << 31:
        return b"J" + struct.pack("<i", v)  # BININT
    nbytes = (v.bit_length() >> 3) + 1  # two's complement, room for the sign bit
    return b"\x8a" + bytes([nbytes]) + v.to_bytes(nbytes, "little", signed=True)  # LONG1


def _tuple(items: Sequence[int]) -> bytes:
    body = b"".join(_int(v) for v in items)
    n = len(items)
    if n == 0:
        return b")"  # EMPTY_TUPLE, never memoized
    if n <= 3:
        return body + (b"\x85", b"\x86", b"\x87")[n - 1] + _MEMOIZE  # TUPLE1/2/3
    return b"(" + body + b"t" + _MEMOIZE  # MARK ... TUPLE


def header_pickle(dtype_name: str, shape: Sequence[int]) -> bytes:
    frame = (
        _global(_HEADER_MODULE, _HEADER_CLASS)
        + b")"  # EMPTY_TUPLE (args of cls.__new__)
        + b"\x81"  # NEWOBJ
        + _MEMOIZE
        + b"}"  # EMPTY_DICT (instance state)
        + _MEMOIZE
        + b"("  # MARK
        + _short_str("dtype")
        + _global("torch", dtype_name)
        + _short_str("shape")
        + _global("torch", "Size")
        + _tuple(shape)
        + b"\x85"  # TUPLE1: the argument tuple of torch.Size(...)
        + _MEMOIZE
        + b"R"  # REDUCE
        + _MEMOIZE
        + b"u"  # SETITEMS
        + b"b"  # BUILD
        + b"."  # STOP
    )
    return b"\x80\x04\x95" + struct.pack("<Q", len(frame)) + frame


def header_bytes(dtype_name: str, shape: Sequence[int]) -> bytes:
    body = header_pickle(dtype_name, shape)
    return struct.pack("<I", len(body)) + body


def dtype_name(dtype: torch.dtype) -> str:
    return str(dtype).split(".", 1)[1]


# ---- payload --------------------------------------------------------------------------------------------------
def payload_bytes(t: torch.Tensor) -> bytes:
    """Row-major bytes of the logical tensor, element by element in index order."""
    if t.numel() == 0:
        return b""
    flat = t.detach().to("cpu").contiguous().reshape(-1)
    if flat.stride(0) != 1:  # a one-element tensor keeps whatever stride its view had
        flat = torch.empty(flat.shape, dtype=flat.dtype, device=flat.device).copy_(flat)
    return flat.view(torch.uint8).numpy().tobytes()


def payload_bytes_bruteforce(t: torch.Tensor) -> bytes:
    """Same bytes, produced one element at a time by explicit index arithmetic over (shape, stride, storage
    offset).  Small tensors only; used to pin ``payload_bytes`` and the strided-gather kernels on views."""
    t = t.detach().to("cpu")
    esz = t.element_size()
    storage = np.frombuffer(bytes(t.untyped_storage()), dtype=np.uint8) if t.untyped_storage().size() else np.zeros(0, np.uint8)
    shape, stride, base = list(t.shape), list(t.stride()), t.storage_offset()
    out = bytearray()
    idx = [0] * len(shape)
    for _ in range(t.numel()):
        elem = base + sum(i * s for i, s in zip(idx, stride))
        out += storage[elem * esz : (elem + 1) * esz].tobytes()
        for d in reversed(range(len(shape))):
            idx[d] += 1
            if idx[d] < shape[d]:
                break
            idx[d] = 0
    return bytes(out)


# ---- data section ---------------------------------------------------------------------------------------------
def record_bytes(t: torch.Tensor) -> bytes:
    return header_bytes(dtype_name(t.dtype), tuple(t.shape)) + payload_bytes(t)


def data_section(tensors: Sequence[torch.Tensor], blobs: Sequence[bytes] = ()) -> Tuple[bytes, List[Tuple[int, int]]]:
    """Returns (data-section bytes, [(offset, length)] per item: tensors in order, then blobs in order)."""
    out = bytearray()
    spans = []
    for t in tensors:
        start = len(out)
        out += record_bytes(t)
        spans.append((start, len(out) - start))
    for blob in blobs:
        start = len(out)
        out += blob
        spans.append((start, len(out) - start))
    return bytes(out), spans


def file_image(tensors: Sequence[torch.Tensor], blobs: Sequence[bytes] = ()) -> Tuple[bytes, List[Tuple[int, int]]]:
    data, spans = data_section(tensors, blobs)
    return metadata_block(len(data), SIGNATURE_MLF) + data, spans


# ---- reading --------------------------------------------------------------------------------------------------
def parse_record(record: bytes) -> Tuple[torch.dtype, Tuple[int, ...], bytes]:
    """Splits one MLF_TENS record into (dtype, shape, payload).  The header pickle is decoded with a tiny
    interpreter for exactly the opcodes ``header_pickle`` emits, so no class needs to be importable."""
    (hlen,) = struct.unpack_from("<I", record, 0)
    if hlen >= 1 << 20:
        raise ValueError("header length implausible: not an MLF_TENS record")
    p = record[4 : 4 + hlen]
    strings, ints = [], []
    i = 11  # PROTO(2) + FRAME(9)
    while i < len(p):
        op = p[i : i + 1]
        i += 1
        if op == b"\x8c":
            n = p[i]
            strings.append(p[i + 1 : i + 1 + n].decode())
            i += 1 + n
        elif op == b"K":
            ints.append(p[i])
            i += 1
        elif op == b"M":
            ints.append(struct.unpack_from("<H", p, i)[0])
            i += 2
        elif op == b"J":
            ints.append(struct.unpack_from("<i", p, i)[0])
            i += 4
        elif op == b"\x8a":
            n = p[i]
            ints.append(int.from_bytes(p[i + 1 : i + 1 + n], "little", signed=True))
            i += 1 + n
        elif op == b".":
            break
    if strings[:2] != [_HEADER_MODULE, _HEADER_CLASS] or strings[2] != "dtype" or strings[5] != "shape":
        raise ValueError("unexpected header pickle layout")
    return getattr(torch, strings[4]), tuple(ints), memoryview(record)[4 + hlen :]  # a view: no second copy


def read_item(record: bytes, storage_offsets: Sequence[int], lengths: Sequence[int]) -> torch.Tensor:
    """CPU tensor for one read request: stored tensor, narrowed per dimension where length < size."""
    dtype, shape, payload = parse_record(record)
    if len(payload) == 0:
        t = torch.empty(shape, dtype=dtype)
    else:
        with warnings.catch_warnings():  # frombuffer over read-only bytes, exactly as the reference does
            warnings.simplefilter("ignore")
            t = torch.frombuffer(payload, dtype=dtype).reshape(shape)
    for dim, (off, length) in enumerate(zip(storage_offsets, lengths)):
        if length < t.size(dim):
            t = t.narrow(dim, off, length)
    return t
