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
    # a view whose neighbouring dimensions merge fits a descriptor whatever its rank ...
    layout = P.build_save_layout([_FakeDeviceTensor(nine.transpose(7, 8), 4096)])
    row = layout.items[-1]
    assert int(row["ndim"]) == 3 and row["shape"][:3].tolist() == [128, 2, 2] and row["stride"][:3].tolist() == [4, 1, 2]
    # ... one that stays above eight dimensions is for the caller to stage through a contiguous copy
    assert P.describable(tuple(nine.transpose(7, 8).shape), tuple(nine.transpose(7, 8).stride()))
    reversed_dims = nine.permute(*range(8, -1, -1))
    assert not P.describable(tuple(reversed_dims.shape), tuple(reversed_dims.stride()))
    with pytest.raises(ValueError, match="contiguous copy"):
        P.build_save_layout([_FakeDeviceTensor(reversed_dims, 4096)])


@settings(max_examples=60, deadline=None)
@given(st.data())
def test_merged_dimensions_address_the_same_elements(data):
    """``collapse_dims``: the merged description visits the same (tensor element, image element) pairs in the same
    order as the original one."""
    ndim = data.draw(st.integers(1, 10))
    shape = tuple(data.draw(st.integers(1, 3)) for _ in range(ndim))
    parent = torch.zeros(tuple(n + data.draw(st.integers(0, 1)) for n in shape))
    view = parent[tuple(slice(0, n) for n in shape)].permute(*data.draw(st.permutations(range(ndim))))
    shape, stride = tuple(view.shape), tuple(view.stride())
    image = tuple(P._contiguous_strides(shape))
    if data.draw(st.booleans()):  # the stored side of a sub-box read: strides of a larger C-contiguous tensor
        image = tuple(P._contiguous_strides(tuple(n + 1 for n in shape)))

    def pairs(shape, stride, image):
        out = []
        for idx in np.ndindex(*shape) if shape else [()]:
            out.append((sum(i * s for i, s in zip(idx, stride)), sum(i * s for i, s in zip(idx, image))))
        return out

    merged = P.collapse_dims(shape, stride, image)
    assert len(merged[0]) <= len(shape) and all(n > 1 for n in merged[0])
    assert pairs(*merged) == pairs(shape, stride, image)


@settings(max_examples=60, deadline=None)
@given(st.data())
def test_oversize_strided_rows_are_cut_into_boxes_that_cover_them_exactly(data):
    """The loader's ``_cut_box``: every piece spans at most the given number of image bytes, and together the pieces
    map exactly the original row's image bytes to the original target addresses."""
    from ml_flashpoint.hip.checkpoint_loader import HipMLFlashpointCheckpointLoader as Loader

    ndim = data.draw(st.integers(1, 4))
    shape = tuple(data.draw(st.integers(1, 5)) for _ in range(ndim))
    esz = data.draw(st.sampled_from([1, 2, 4]))
    target = torch.zeros(tuple(n + 1 for n in shape)).permute(*data.draw(st.permutations(range(ndim))))
    strides = tuple(target.stride())[:ndim]
    stored = tuple(P._contiguous_strides(tuple(n + data.draw(st.integers(0, 2)) for n in shape)))
    image_strides = data.draw(st.sampled_from([None, stored]))
    first, ptr = data.draw(st.integers(0, 1000)), 1 << 20
    usable = data.draw(st.integers(esz, 64 * esz))

    def mapping(row):
        begin, end, contiguous, (p, e, shp, st_t, st_i) = row
        st_i = st_i if st_i is not None else tuple(P._contiguous_strides(shp))
        assert not contiguous and end - begin == (sum((n - 1) * s for n, s in zip(shp, st_i)) + 1) * e
        return {begin + sum(i * s for i, s in zip(idx, st_i)) * e: p + sum(i * s for i, s in zip(idx, st_t)) * e
                for idx in np.ndindex(*shp)}

    whole = mapping(Loader._cut_box(first, (ptr, esz, shape, strides, image_strides), 1 << 40)[0])
    pieces = Loader._cut_box(first, (ptr, esz, shape, strides, image_strides), usable)
    got = {}
    for piece in pieces:
        assert piece[1] - piece[0] <= usable
        part = mapping(piece)
        assert not set(part) & set(got)
        got.update(part)
    assert got == whole
