"""Pins the CPU oracle (oracle/mlf_format.py, oracle/crc32c.c) and the package's own header writer.

Sources of truth, in order: vectors produced by the reference's own ``TensorHeader.to_bytes``
(tests/golden/tensor_header_vectors.json), the known answers the reference's tests hold
(tests/core/test_checkpoint_loader.py:223-302 sub-box reads; tests/core/test_checkpoint_saver.py:1297-1307,1394-1431
offset rules), published vectors (RFC 3720 B.4), closed forms (``struct``), library routines (``numpy.tobytes``,
``pickle.loads``) and brute force on tiny inputs.
"""

import json
import os
import pickle
import struct

import numpy as np
import pytest
import torch
from hypothesis import given, settings
from hypothesis import strategies as st

from ml_flashpoint.core.tensor_header import TensorHeader
from oracle import mlf_format as fmt

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "tensor_header_vectors.json")))["vectors"]


@pytest.mark.parametrize("case", GOLDEN, ids=lambda c: f"{c['dtype']}-{'x'.join(map(str, c['shape'])) or 'scalar'}")
def test_header_bytes_match_reference_vectors(case):
    want = bytes.fromhex(case["hex"])
    assert fmt.header_bytes(case["dtype"], case["shape"]) == want  # oracle: hand-rolled pickle
    dtype = getattr(torch, case["dtype"])
    assert TensorHeader(dtype=dtype, shape=torch.Size(case["shape"])).to_bytes() == want  # package: pickle.dumps


@pytest.mark.parametrize("case", GOLDEN[:8], ids=lambda c: c["dtype"])
def test_header_vectors_unpickle_to_the_package_class(case):
    raw = bytes.fromhex(case["hex"])
    header, consumed = TensorHeader.from_bytes(raw + b"payload")
    assert consumed == len(raw)
    assert isinstance(header, TensorHeader)
    assert header.dtype == getattr(torch, case["dtype"]) and list(header.shape) == case["shape"]
    assert isinstance(header.shape, torch.Size)


@settings(max_examples=200, deadline=None)
@given(
    st.sampled_from(["float32", "bfloat16", "int64", "uint8", "float8_e4m3fn", "bool", "complex64", "uint16", "uint64",
                     "float8_e5m2", "float8_e4m3fnuz", "float8_e5m2fnuz", "complex128", "float64", "int8"]),
    st.lists(st.one_of(st.integers(0, 300), st.integers(0, 1 << 40)), min_size=0, max_size=9),
)
def test_header_pickle_closed_form_equals_cpython_pickler(dtype_name, shape):
    """Beyond the golden cases: the oracle's opcode writer and CPython's pickler agree for any shape, and the
    oracle's reader inverts it."""
    ours = fmt.header_bytes(dtype_name, shape)
    theirs = TensorHeader(dtype=getattr(torch, dtype_name), shape=torch.Size(shape)).to_bytes()
    assert ours == theirs
    (n,) = struct.unpack_from("<I", ours, 0)
    assert n == len(ours) - 4
    loaded = pickle.loads(ours[4:])
    assert loaded.dtype == getattr(torch, dtype_name) and tuple(loaded.shape) == tuple(shape)
    dtype, parsed_shape, payload = fmt.parse_record(ours + b"\x01\x02")
    assert dtype == getattr(torch, dtype_name) and parsed_shape == tuple(shape) and payload == b"\x01\x02"


def test_metadata_block_closed_form():
    block = fmt.metadata_block(0x0102030405060708, b"MLF_TENS")
    assert len(block) == 4096
    assert block[:8] == bytes([8, 7, 6, 5, 4, 3, 2, 1])  # u64 little-endian at offset 0
    assert block[8:16] == b"MLF_TENS"
    assert block[16:] == bytes(4080)
    assert fmt.metadata_block(5, b"AB")[8:16] == b"AB" + bytes(6)
    with pytest.raises(ValueError):
        fmt.metadata_block(0, b"123456789")


@pytest.mark.parametrize("dtype", [torch.int32, torch.float32, torch.float16, torch.int64, torch.uint8, torch.float64])
def test_payload_is_numpy_tobytes_for_numpy_dtypes(dtype):
    t = (torch.arange(60, dtype=torch.float64) * 1.5 - 7).to(dtype).reshape(3, 4, 5)
    assert fmt.payload_bytes(t) == t.numpy().tobytes()
    view = t.permute(2, 0, 1)[1:, :, ::2]
    assert fmt.payload_bytes(view) == np.ascontiguousarray(view.numpy()).tobytes()
    assert fmt.payload_bytes_bruteforce(view) == np.ascontiguousarray(view.numpy()).tobytes()


def test_payload_of_types_numpy_lacks_is_written_out_by_hand():
    bf = torch.tensor([1.0, -2.0, 0.5], dtype=torch.bfloat16)  # 0x3F80, 0xC000, 0x3F00
    assert fmt.payload_bytes(bf) == bytes([0x80, 0x3F, 0x00, 0xC0, 0x00, 0x3F])
    f8 = torch.tensor([1.0, -1.0, 0.0], dtype=torch.float8_e4m3fn)  # 0x38, 0xB8, 0x00
    assert fmt.payload_bytes(f8) == bytes([0x38, 0xB8, 0x00])
    assert fmt.payload_bytes(torch.empty(0, 3)) == b""
    assert fmt.payload_bytes(torch.tensor(7, dtype=torch.int16)) == b"\x07\x00"


def test_data_section_offsets_follow_the_reference_rules():
    """offset_0 = 0, offset_{i+1} = offset_i + length_i, length = 4 + len(pickle) + nbytes, tensors before blobs."""
    tensors = [torch.ones(2, 2), torch.arange(10, dtype=torch.int64), torch.empty(0), torch.tensor(3.0)]
    blobs = [b"abc", b"", b"0123456789"]
    data, spans = fmt.data_section(tensors, blobs)
    pos = 0
    for t, (off, length) in zip(tensors, spans):
        hdr = fmt.header_bytes(fmt.dtype_name(t.dtype), tuple(t.shape))
        assert off == pos and length == len(hdr) + t.numel() * t.element_size()
        assert data[off : off + len(hdr)] == hdr
        pos += length
    for b, (off, length) in zip(blobs, spans[len(tensors) :]):
        assert (off, length) == (pos, len(b)) and data[off : off + length] == b
        pos += length
    assert pos == len(data)
    image, _ = fmt.file_image(tensors, blobs)
    assert image[:4096] == fmt.metadata_block(len(data)) and image[4096:] == data
    assert spans[0][1] == 4 + 135 + 16  # float32 (2, 2): the 135-byte pickle measured on the reference's class


def _record(t):
    return fmt.header_bytes(fmt.dtype_name(t.dtype), tuple(t.shape)) + t.numpy().tobytes()


def test_read_item_known_answers_from_the_reference_tests():
    # 1-D: slice [5, 15) of arange(20)
    got = fmt.read_item(_record(torch.arange(20, dtype=torch.float32)), (5,), (10,))
    assert got.dtype == torch.float32 and torch.equal(got, torch.arange(5, 15, dtype=torch.float32))
    # 2-D: 2x3 box at (1, 2) of a 4x5 arange
    got = fmt.read_item(_record(torch.arange(20, dtype=torch.int64).reshape(4, 5)), (1, 2), (2, 3))
    assert torch.equal(got, torch.tensor([[7, 8, 9], [12, 13, 14]], dtype=torch.int64))
    # 3-D: 2x2x2 box at (1, 0, 3) of a 3x4x5 arange
    got = fmt.read_item(_record(torch.arange(60, dtype=torch.float32).reshape(3, 4, 5)), (1, 0, 3), (2, 2, 2))
    want = torch.tensor([[[23.0, 24.0], [28.0, 29.0]], [[43.0, 44.0], [48.0, 49.0]]])
    assert torch.equal(got, want)
    # full tensor: lengths equal to the sizes leave it alone whatever the offsets say
    got = fmt.read_item(_record(torch.tensor([1, 2, 3], dtype=torch.int32)), (0,), (3,))
    assert torch.equal(got, torch.tensor([1, 2, 3], dtype=torch.int32))


def test_read_item_agrees_with_torch_narrow_helper():
    from torch.distributed._shard._utils import narrow_tensor_by_index

    t = torch.arange(2 * 7 * 9, dtype=torch.int32).reshape(2, 7, 9)
    for offsets, lengths in [((0, 0, 0), (2, 7, 9)), ((1, 2, 3), (1, 4, 5)), ((0, 6, 8), (2, 1, 1)), ((5, 5, 5), (2, 7, 9))]:
        assert torch.equal(fmt.read_item(_record(t), offsets, lengths), narrow_tensor_by_index(t, offsets, lengths))


RFC3720 = [
    (b"123456789", 0xE3069283),
    (bytes(32), 0x8A9136AA),
    (b"\xff" * 32, 0x62A8AB43),
    (bytes(range(32)), 0x46DD794E),
    (bytes(range(31, -1, -1)), 0x113FDB5C),
]


@pytest.mark.parametrize("data,want", RFC3720)
def test_oracle_crc32c_known_vectors(oracle_c, data, want):
    assert oracle_c.oracle_crc32c(data, len(data)) == want
    assert oracle_c.oracle_crc32c_bitwise(data, len(data)) == want


def test_oracle_crc32c_empty_and_combine_by_brute_force(oracle_c):
    assert oracle_c.oracle_crc32c(b"", 0) == 0
    rng = np.random.default_rng(3)
    for la, lb in [(0, 5), (5, 0), (1, 1), (7, 64), (100, 3), (33, 1000)]:
        a, b = rng.bytes(la), rng.bytes(lb)
        whole = oracle_c.oracle_crc32c(a + b, la + lb)
        assert oracle_c.oracle_crc32c_combine(oracle_c.oracle_crc32c(a, la), oracle_c.oracle_crc32c(b, lb), lb) == whole
    out = np.zeros(3, dtype=np.uint32)
    data = rng.bytes(2500)
    oracle_c.oracle_crc32c_chunks(data, 2500, 1000, out.ctypes.data)
    assert out.tolist() == [oracle_c.oracle_crc32c(data[i : i + 1000], len(data[i : i + 1000])) for i in (0, 1000, 2000)]
