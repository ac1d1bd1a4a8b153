"""Host-side layout rules of the gfx950 saver (``hip/plan.py``), checked without a GPU.

The descriptor table is built on the host from addresses, shapes and strides only, so the whole rule set - record
order, header bytes, offsets with no padding, blobs behind the tensors, what becomes a contiguous run and what a
strided descriptor - can be compared with the oracle on CPU tensors.  (For host-resident tensors the payload
travels in the plan's blob, which then *is* the data section - unless they are large, when they stay out of the image
altogether; for device tensors only the table rows differ.)"""

import numpy as np
import pytest
import torch
from hypothesis import given, settings
from hypothesis import strategies as st

from ml_flashpoint.hip import _lib
from ml_flashpoint.hip import plan as P
from oracle import mlf_format as fmt

DTYPES = [torch.uint8, torch.bool, torch.int16, torch.bfloat16, torch.float16, torch.float32, torch.int64,
          torch.float64, torch.complex64]


def _tensor(draw_ints, dtype, shape):
    numel = int(np.prod(shape)) if shape else 1
    esz = torch.empty((), dtype=dtype).element_size()
    raw = torch.tensor(draw_ints(numel * esz), dtype=torch.uint8) if numel else torch.empty(0, dtype=torch.uint8)
    if dtype == torch.bool:
        return (raw[:numel] & 1).to(torch.bool).reshape(shape)
    return raw.view(dtype).reshape(shape)


@settings(max_examples=60, deadline=None)
@given(st.data())
def test_layout_of_host_tensors_is_the_oracles_data_section(data):
    n = data.draw(st.integers(0, 6))
    tensors = []
    for _ in range(n):
        dtype = data.draw(st.sampled_from(DTYPES))
        shape = tuple(data.draw(st.lists(st.integers(0, 5), min_size=0, max_size=4)))
        t = _tensor(lambda k: data.draw(st.lists(st.integers(0, 255), min_size=k, max_size=k)), dtype, shape)
        if t.dim() >= 2 and data.draw(st.booleans()):
            t = t.transpose(0, -1)  # host views are laid out by value, like everything else
        tensors.append(t)
    blobs = data.draw(st.lists(st.binary(min_size=0, max_size=40), min_size=0, max_size=3))
    layout = P.build_save_layout(tensors, blobs)
    want, spans = fmt.data_section(tensors, blobs)
    assert layout.spans == spans and layout.image_bytes == len(want)
    assert layout.blob == want                              # every item is host-resident: the blob is the image
    items = layout.items
    assert (items["kind"] == _lib.ITEM_BLOB).all() and layout.device_payload_bytes == 0
    # the rows tile the image exactly: consecutive, no gaps, no overlap, blob offsets in step with image offsets
    assert int(items["nbytes"].sum()) == len(want)
    if len(items):
        ends = items["image_off"] + items["nbytes"]
        assert items["image_off"][0] == 0 and (items["image_off"][1:] == ends[:-1]).all()
        assert (items["ptr"] == items["image_off"]).all()


@settings(max_examples=60, deadline=None)
@given(st.data())
def test_host_tensors_above_the_threshold_are_left_out_of_the_image(data):
    """With a threshold, large host tensors are only noted (``host_spans``); the image holds everything else in
    ``segments``.  Putting the segments and the host payloads where the layout says reproduces the oracle's data
    section, the records' spans are those of the layout without a threshold, and nothing overlaps or is left out."""
    threshold = data.draw(st.sampled_from([1, 16, 64]))
    tensors = []
    for _ in range(data.draw(st.integers(0, 7))):
        dtype = data.draw(st.sampled_from(DTYPES))
        shape = tuple(data.draw(st.lists(st.integers(0, 6), min_size=0, max_size=3)))
        t = _tensor(lambda k: data.draw(st.lists(st.integers(0, 255), min_size=k, max_size=k)), dtype, shape)
        if t.dim() >= 2 and data.draw(st.booleans()):
            t = t.transpose(0, -1)
        tensors.append(t)
    blobs = data.draw(st.lists(st.binary(min_size=0, max_size=40), min_size=0, max_size=2))
    layout = P.build_save_layout(tensors, blobs, host_direct_min=threshold)
    want, spans = fmt.data_section(tensors, blobs)
    assert layout.spans == spans and layout.data_bytes == len(want)
    big = [i for i, t in enumerate(tensors) if t.numel() * t.element_size() >= threshold]
    big += [-1 - k for k, b in enumerate(blobs) if len(b) >= threshold]  # byte blobs follow the same rule
    assert [i for _, _, i in layout.host_spans] == big
    assert [id(t) for t in layout.host_tensors] == [id(tensors[i]) if i >= 0 else id(blobs[-1 - i]) for i in big]
    assert layout.image_bytes == len(want) - sum(n for _, n, _ in layout.host_spans)
    # the image, as the pack kernel would fill it from the table (every row is a piece of the blob here)
    image = bytearray(layout.image_bytes)
    for row in layout.items:
        assert row["kind"] == _lib.ITEM_BLOB
        image[int(row["image_off"]) : int(row["image_off"] + row["nbytes"])] = layout.blob[int(row["ptr"]) : int(row["ptr"] + row["nbytes"])]
    built = bytearray(b"\xEE" * len(want))
    covered = 0
    for image_off, data_off, n in layout.segments:
        built[data_off : data_off + n] = image[image_off : image_off + n]
        covered += n
    for (data_off, n, _), t in zip(layout.host_spans, layout.host_tensors):
        built[data_off : data_off + n] = P.host_tensor_bytes(t) if isinstance(t, torch.Tensor) else t
        covered += n
    assert covered == len(want) and bytes(built) == want
    pieces = sorted([(d, n) for _, d, n in layout.segments] + [(d, n) for d, n, _ in layout.host_spans])
    assert all(a[0] + a[1] == b[0] for a, b in zip(pieces, pieces[1:])) and (not pieces or pieces[0][0] == 0)
    assert [io for io, _, _ in layout.segments] == [sum(n for _, _, n in layout.segments[:k]) for k in range(len(layout.segments))]


class _FakeDeviceTensor:
    """Quacks like a device tensor for the layout builder: an address, a shape, strides - no memory behind it."""

    def __init__(self, like: torch.Tensor, address: int):
        self._like, self._address = like, address
        self.dtype, self.shape = like.dtype, like.shape
        self.device = torch.device("cuda", 0)

    def numel(self):
        return self._like.numel()

    def element_size(self):
        return self._like.element_size()

    def is_contiguous(self):
        return self._like.is_contiguous()

    def stride(self):
        return self._like.stride()

    def data_ptr(self):
        return self._address


def test_device_rows_carry_address_and_strides_and_headers_stay_in_the_blob():
    base = torch.arange(6 * 8, dtype=torch.float32).reshape(6, 8)
    views = [base, base.t(), base[:, ::2], base[2:5], torch.empty(0, 3), torch.tensor(7, dtype=torch.int64)]
    fakes = [_FakeDeviceTensor(v, 0x7F0000000000 + 4096 * k) for k, v in enumerate(views)]
    layout = P.build_save_layout(fakes, [b"tail"])
    want, spans = fmt.data_section(views, [b"tail"])
    assert layout.spans == spans and layout.image_bytes == len(want)
    items = layout.items
    rows = [r for r in items if r["kind"] == _lib.ITEM_DEVICE]
    assert len(rows) == 5                                    # the zero-size tensor has a header and nothing else
    by_addr = {int(r["ptr"]): r for r in rows}
    for k, v in enumerate(views):
        if v.numel() == 0:
            continue
        r = by_addr[0x7F0000000000 + 4096 * k]
        off, length = spans[k]
        assert int(r["image_off"]) == off + length - v.numel() * v.element_size()   # payload sits behind the header
        assert int(r["nbytes"]) == v.numel() * v.element_size() and int(r["elem_size"]) == v.element_size()
        if v.is_contiguous():
            assert int(r["ndim"]) == 1 and int(r["shape"][0]) == v.numel() and int(r["stride"][0]) == 1
        else:
            d = v.dim()
            assert int(r["ndim"]) == d and tuple(r["shape"][:d]) == tuple(v.shape) and tuple(r["stride"][:d]) == v.stride()
            assert tuple(r["image_stride"][:d]) == tuple(torch.empty(v.shape).stride())  # C-contiguous in the image
    # headers and the byte blob, in image order, are what the blob holds
    blob_rows = [r for r in items if r["kind"] == _lib.ITEM_BLOB]
    pieces = b"".join(layout.blob[int(r["ptr"]): int(r["ptr"]) + int(r["nbytes"])] for r in blob_rows)
    assert pieces == b"".join(fmt.header_bytes(fmt.dtype_name(v.dtype), tuple(v.shape)) for v in views) + b"tail"
    for r in blob_rows:
        assert want[int(r["image_off"]): int(r["image_off"]) + int(r["nbytes"])] == \
            layout.blob[int(r["ptr"]): int(r["ptr"]) + int(r["nbytes"])]
    assert layout.device_payload_bytes == sum(v.numel() * v.element_size() for v in views)


def test_rank_limit_of_strided_rows():
    nine = torch.zeros((2,) * 9)
    P.build_save_layout([_FakeDeviceTensor(nine, 4096)])                    # contiguous: a run of bytes, any rank
    with pytest.raises(NotImplementedError, match="rank > 8"):
        P.build_save_layout([_FakeDeviceTensor(nine.transpose(0, 8), 4096)])
