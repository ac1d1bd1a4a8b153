"""GPU parity of the C-ABI kernels against the CPU oracle: pack, unpack, CRC-32C, copy engine.

Bit-exact is the bar everywhere (byte movement and integer arithmetic only).
"""

import ctypes

import numpy as np
import pytest
import torch

from oracle import mlf_format as oracle_fmt

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _rand_tensor(gen, shape, dtype):
    """Seeded tensor whose *bytes* are uniform random (so every bit pattern, NaNs included, must survive)."""
    numel = int(np.prod(shape)) if len(shape) else 1
    esz = torch.empty((), dtype=dtype).element_size()
    raw = torch.randint(0, 256, (max(numel, 1) * esz,), dtype=torch.uint8, generator=gen)
    return raw[: numel * esz].view(dtype).reshape(shape).clone()


def _pack_image(tensors, blobs=(), **plan_kw):
    from ml_flashpoint.hip import plan as P

    layout = P.build_save_layout(tensors, blobs)
    plan = P.Plan(layout.items, layout.blob, layout.image_bytes, **plan_kw)
    image = torch.empty(max(layout.image_bytes, 1) + 512, dtype=torch.uint8, device=DEV)
    image.fill_(0xAB)
    plan.pack(image)
    torch.cuda.synchronize()
    host = image.cpu().numpy()
    assert (host[layout.image_bytes :] == 0xAB).all(), "pack wrote past the end of the image"
    return layout, plan, image, host[: layout.image_bytes].tobytes()


MIXED = [
    ((), torch.float32),
    ((0,), torch.float32),
    ((1,), torch.int64),
    ((2, 2), torch.float32),
    ((7,), torch.bfloat16),
    ((13, 5), torch.float16),
    ((3, 5, 7), torch.int32),
    ((1023,), torch.uint8),
    ((1025,), torch.int8),
    ((17,), torch.bool),
    ((64, 257), torch.float8_e4m3fn),
    ((300, 1001), torch.bfloat16),
    ((4, 0, 3), torch.int16),
    ((2, 3), torch.complex64),
    ((5,), torch.complex128),
    ((33,), torch.uint16),
    ((9, 11), torch.uint32),
    ((1027,), torch.uint64),
    ((129, 3), torch.float8_e5m2),
    ((4099,), torch.float8_e4m3fnuz),
    ((2, 515), torch.float8_e5m2fnuz),
    ((4097,), torch.float8_e8m0fnu),  # the block scales of the MX formats
    ((96, 1040), torch.float4_e2m1fn_x2),  # two fp4 values per byte
    ((1 << 20,), torch.float32),
    ((777, 513), torch.float64),
]


def test_pack_contiguous_mixed_dtypes_matches_oracle():
    gen = torch.Generator().manual_seed(11)
    cpu = [_rand_tensor(gen, s, d) for s, d in MIXED]
    dev = [t.to(DEV) for t in cpu]
    blobs = [b"", b"x", bytes(range(256)) * 5]
    layout, plan, image, got = _pack_image(dev, blobs)
    want, spans = oracle_fmt.data_section(cpu, blobs)
    assert layout.spans == spans
    assert got == want


@pytest.mark.parametrize("tile_bytes,threads", [(1024, 64), (4096, 256), (65536, 512), (1 << 20, 1024)])
def test_pack_tile_and_block_shapes(tile_bytes, threads):
    gen = torch.Generator().manual_seed(12)
    cpu = [_rand_tensor(gen, s, d) for s, d in [((100003,), torch.uint8), ((513, 1027), torch.bfloat16), ((3,), torch.int64)]]
    dev = [t.to(DEV) for t in cpu]
    _, _, _, got = _pack_image(dev, tile_bytes=tile_bytes, block_threads=threads)
    assert got == oracle_fmt.data_section(cpu)[0]


@pytest.mark.parametrize("grid_x_log2", [1, 3, 8, 11])
def test_flat_kernel_grid_rows(grid_x_log2):
    """All three span classes (entries shared by 128, 16 and 1 workgroups) go out in one launch whose workgroups are
    numbered row by row over a 2-D grid; with rows of 1, 4, 128 and 1024 workgroups, class boundaries and the padding of the last row fall
    everywhere.  Pack is compared with the oracle, unpack must restore the tensors."""
    from ml_flashpoint.hip import plan as P

    gen = torch.Generator().manual_seed(14)
    shapes = [((3 << 20) + 5,), ((1 << 19) + 1,), (70001,), (4097,), (1500,), (9,)]  # 1 KiB tiles: 128-, 16-, 1-tile spans
    cpu = [_rand_tensor(gen, s, torch.uint8) for s in shapes]
    dev = [t.to(DEV) for t in cpu]
    layout, plan, image, got = _pack_image(dev, tile_bytes=1024, block_threads=64, grid_x_log2=grid_x_log2)
    assert plan.info.n_flat_tiles > 3000
    assert got == oracle_fmt.data_section(cpu)[0]
    targets = [torch.zeros_like(t) for t in dev]
    table = P.ItemTable()
    for t, (off, length) in zip(targets, layout.spans):
        table.add_device(t.data_ptr(), off + length - t.numel(), 1, tuple(t.shape), (1,))
    P.Plan(table.to_array(), b"", layout.image_bytes, tile_bytes=1024, block_threads=64, align_to_tensor=True,
           grid_x_log2=grid_x_log2).unpack(image)
    torch.cuda.synchronize()
    assert all(torch.equal(a, b) for a, b in zip(targets, dev))


def test_pack_misaligned_sources():
    """Views that start at odd element offsets: the source address is not 16-byte aligned."""
    gen = torch.Generator().manual_seed(13)
    base8 = _rand_tensor(gen, (70001,), torch.uint8)
    base16 = _rand_tensor(gen, (50001,), torch.bfloat16)
    cpu = [base8[k : k + 60000] for k in (1, 2, 3, 5, 15)] + [base16[k : k + 40000] for k in (1, 3, 7)]
    dev8, dev16 = base8.to(DEV), base16.to(DEV)
    dev = [dev8[k : k + 60000] for k in (1, 2, 3, 5, 15)] + [dev16[k : k + 40000] for k in (1, 3, 7)]
    _, _, _, got = _pack_image(dev)
    assert got == oracle_fmt.data_section(cpu)[0]


def _views(base):
    """Non-contiguous views of a 3-D base, the kinds the benchmark's strided-views configuration names plus a few more."""
    m = base[0]
    return [
        m.t(),  # transposed
        m[:, ::2],  # every other column
        m[16:48, :],  # row block (contiguous)
        m[:, 8:40],  # column block (row-contiguous pieces)
        base.permute(2, 0, 1),
        base[::2, 1:, ::3],
        base[1].t()[3:, ::2],
        m[5],  # one row
        m[:, 5],  # one column
        base.expand(2, *base.shape)[1],  # stride-0 parent
    ]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float8_e4m3fn, torch.float32, torch.int64, torch.complex128])
def test_pack_strided_views_match_bruteforce_oracle(dtype):
    gen = torch.Generator().manual_seed(14)
    base_cpu = _rand_tensor(gen, (3, 64, 96), dtype)
    base_dev = base_cpu.to(DEV)
    cpu, dev = _views(base_cpu), _views(base_dev)
    layout, plan, _, got = _pack_image(dev)
    want = b"".join(
        oracle_fmt.header_bytes(oracle_fmt.dtype_name(t.dtype), tuple(t.shape)) + oracle_fmt.payload_bytes_bruteforce(t)
        for t in cpu
    )
    assert got == want
    assert got == oracle_fmt.data_section(cpu)[0]
    assert plan.info.n_strided_items > 0


def _broadcast_views(base):
    """Views with stride-0 dimensions (``expand``): every element of the logical tensor is written out, as
    ``copy_`` into a contiguous buffer does."""
    m = base[0]
    return [
        m[5].expand(64, 96),  # one row, repeated: strides (0, 1)
        m[:, 5:6].expand(64, 96),  # one column, repeated along the fast dimension: strides (96, 0)
        m[3, 7].expand(40, 50),  # one element: strides (0, 0)
        base[:, 2:3, ::2].expand(3, 33, 48),  # a broadcast dimension between two real ones, the last one strided
        m.t()[:, None, :].expand(96, 4, 64),  # transposed and broadcast
    ]


@pytest.mark.parametrize("dtype", [torch.float8_e4m3fn, torch.bfloat16, torch.float32, torch.int64])
def test_pack_views_with_broadcast_dimensions(dtype):
    gen = torch.Generator().manual_seed(15)
    base_cpu = _rand_tensor(gen, (3, 64, 96), dtype)
    cpu, dev = _broadcast_views(base_cpu), _broadcast_views(base_cpu.to(DEV))
    assert all(0 in t.stride() for t in dev)
    _, _, _, got = _pack_image(dev)
    assert got == b"".join(
        oracle_fmt.header_bytes(oracle_fmt.dtype_name(t.dtype), tuple(t.shape)) + oracle_fmt.payload_bytes_bruteforce(t)
        for t in cpu
    )
    assert got == oracle_fmt.data_section(cpu)[0]


TRANSPOSE_SHAPES = [(16, 16), (17, 130), (128, 128), (129, 257), (300, 31), (64, 1000), (5, 40, 70)]


@pytest.mark.parametrize("dtype", [torch.float8_e4m3fn, torch.bfloat16, torch.float32, torch.int64, torch.complex128])
def test_transposed_views_pack_and_unpack_through_lds_tiles(dtype):
    """`.t()`-like views (tensor-contiguous dimension != image-contiguous dimension), tile-multiple and ragged
    extents, with and without batch dimensions and storage offsets; both directions."""
    from ml_flashpoint.hip import plan as P

    gen = torch.Generator().manual_seed(31)
    cpu_views, dev_views = [], []
    for shape in TRANSPOSE_SHAPES:
        parent = _rand_tensor(gen, tuple(d + 3 for d in shape), dtype)
        dev_parent = parent.to(DEV)
        sl = tuple(slice(1, 1 + d) for d in shape)
        cpu_views.append(parent[sl].transpose(-1, -2))
        dev_views.append(dev_parent[sl].transpose(-1, -2))
    layout, plan, image, got = _pack_image(dev_views)
    assert plan.info.n_transposed_items == len(TRANSPOSE_SHAPES) and plan.info.n_strided_items == 0
    want, spans = oracle_fmt.data_section(cpu_views)
    assert got == want
    assert got == b"".join(
        oracle_fmt.header_bytes(oracle_fmt.dtype_name(t.dtype), tuple(t.shape)) + oracle_fmt.payload_bytes_bruteforce(t)
        for t in cpu_views[:3]
    ) + want[spans[3][0] :]
    # restore the image into transposed targets embedded in larger zeroed parents
    table = P.ItemTable()
    parents, targets = [], []
    for view, (off, length) in zip(cpu_views, spans):
        tshape = tuple(view.shape[:-2]) + (view.shape[-1] + 2, view.shape[-2] + 5)
        parent = torch.zeros(tshape, dtype=torch.uint8 if dtype == torch.float8_e4m3fn else dtype, device=DEV)
        parent = parent.view(dtype) if dtype == torch.float8_e4m3fn else parent
        target = parent[..., 2:, 5:].transpose(-1, -2)
        assert target.shape == view.shape
        nbytes = view.numel() * view.element_size()
        table.add_device(target.data_ptr(), off + length - nbytes, view.element_size(), tuple(view.shape), tuple(target.stride()))
        parents.append(parent)
        targets.append(target)
    uplan = P.Plan(table.to_array(), b"", layout.image_bytes, align_to_tensor=True)
    assert uplan.info.n_transposed_items == len(TRANSPOSE_SHAPES)
    uplan.unpack(image)
    torch.cuda.synchronize()
    for view, target, parent in zip(cpu_views, targets, parents):
        assert torch.equal(target.cpu().contiguous().reshape(-1).view(torch.uint8), view.contiguous().reshape(-1).view(torch.uint8))
        p8 = parent.cpu().reshape(-1).view(torch.uint8)
        assert int(p8.count_nonzero()) <= view.numel() * view.element_size()  # nothing outside the target was touched
        assert int(parent[..., :2, :].cpu().reshape(-1).view(torch.uint8).count_nonzero()) == 0
        assert int(parent[..., :, :5].cpu().reshape(-1).view(torch.uint8).count_nonzero()) == 0


def test_strided_walk_many_shapes_against_bruteforce():
    """The division-free index walk: inner extents smaller and larger than the block, up to 5 dims, both directions."""
    from ml_flashpoint.hip import plan as P

    gen = torch.Generator().manual_seed(32)
    base = _rand_tensor(gen, (7, 6, 5, 9, 11), torch.int16)
    dev = base.to(DEV)
    pick = lambda t: [  # noqa: E731
        t[::2, :, ::2, :, ::3],
        t[:, 1:4, :, ::4, 2:9:2],
        t.permute(4, 2, 0, 1, 3)[::2],
        t[3, :, :, :, ::5],
        t[..., ::7],
        t[:, :, :, 1, 1],
        t.flatten()[3::13],
    ]
    cpu_views, dev_views = pick(base), pick(dev)
    layout, plan, image, got = _pack_image(dev_views)
    assert plan.info.n_strided_items == len(cpu_views)
    want = b"".join(
        oracle_fmt.header_bytes("int16", tuple(t.shape)) + oracle_fmt.payload_bytes_bruteforce(t) for t in cpu_views
    )
    assert got == want
    back = torch.zeros_like(dev)
    table = P.ItemTable()
    for src, tgt, (off, length) in zip(cpu_views, pick(back), layout.spans):
        table.add_device(tgt.data_ptr(), off + length - src.numel() * 2, 2, tuple(src.shape), tuple(tgt.stride()))
    P.Plan(table.to_array(), b"", layout.image_bytes, align_to_tensor=True).unpack(image)
    torch.cuda.synchronize()
    mask = torch.zeros_like(base, dtype=torch.bool)
    for m in pick(mask):
        m.fill_(True)
    assert torch.equal(back.cpu()[mask], base[mask]) and int(back.cpu()[~mask].abs().sum()) == 0


@pytest.mark.parametrize("dtype", [torch.uint8, torch.bfloat16, torch.float32, torch.int64, torch.complex128])
def test_strided_views_with_long_rows(dtype):
    """Strided views with rows of hundreds to tens of thousands of elements (a workgroup's share of 32 Ki elements
    then covers many rows, or less than one), both directions, against the oracle."""
    from ml_flashpoint.hip import plan as P

    gen = torch.Generator().manual_seed(33)
    base = _rand_tensor(gen, (3, 7, 2100), dtype)
    wide = _rand_tensor(gen, (2, 70001), dtype)
    esz = base.element_size()
    pick = lambda t, w: [  # noqa: E731
        t[:, :, ::2],                      # 1050 per row, 21 rows
        t[:, :, 1::3],
        t[:, ::2, 5:1500:1][:, :, ::1][..., 3:],  # contiguous rows of 1492, too short for the flat kernel at 1 byte
        t[1, :, :997:1][:, ::1][:, 1::2],
        t.permute(1, 0, 2)[:, :, 2:2000:2],
        t[:, :, 40:700],                   # 660 per row
        w[:, ::2],                         # 35001 per row: more than one workgroup's share
        w[1:, 5::1][:, ::3],
    ]
    dev, wide_dev = base.to(DEV), wide.to(DEV)
    cpu_views, dev_views = pick(base, wide), pick(dev, wide_dev)
    layout, plan, image, got = _pack_image(dev_views)
    name = oracle_fmt.dtype_name(dtype)
    want = b"".join(oracle_fmt.header_bytes(name, tuple(t.shape)) + oracle_fmt.payload_bytes(t) for t in cpu_views)
    assert got == want
    small = cpu_views[1]
    assert oracle_fmt.payload_bytes(small) == oracle_fmt.payload_bytes_bruteforce(small)
    back, wide_back = torch.zeros_like(dev), torch.zeros_like(wide_dev)
    table = P.ItemTable()
    for src, tgt, (off, length) in zip(cpu_views, pick(back, wide_back), layout.spans):
        table.add_device(tgt.data_ptr(), off + length - src.numel() * esz, esz, tuple(src.shape), tuple(tgt.stride()))
    P.Plan(table.to_array(), b"", layout.image_bytes, align_to_tensor=True).unpack(image)
    torch.cuda.synchronize()
    mask_base, mask_wide = torch.zeros(base.shape, dtype=torch.bool), torch.zeros(wide.shape, dtype=torch.bool)
    for m in pick(mask_base, mask_wide):
        m.fill_(True)
    for ref, got_dev, mask in ((base, back, mask_base), (wide, wide_back, mask_wide)):
        got_b = got_dev.cpu().contiguous().view(torch.uint8).reshape(*ref.shape, esz)
        want_b = ref.contiguous().view(torch.uint8).reshape(*ref.shape, esz)
        assert torch.equal(got_b[mask], want_b[mask]) and int(got_b[~mask].count_nonzero()) == 0


@pytest.mark.parametrize("dtype", [torch.uint8, torch.bfloat16, torch.float32, torch.complex128])
def test_views_of_the_maximum_rank_and_the_rank_limit(dtype):
    """Eight dimensions is what a descriptor holds.  Views of that rank whose dimensions cannot be merged (reversed
    order, every other element along several axes) pack and unpack like any other; one more dimension is fine as
    long as the tensor is contiguous (it is a run of bytes) and refused otherwise."""
    from ml_flashpoint.hip import plan as P

    gen = torch.Generator().manual_seed(88)
    shape = (3, 2, 4, 2, 3, 2, 2, 5)
    base_cpu = _rand_tensor(gen, shape, dtype)
    base_dev = base_cpu.to(DEV)

    def views(t):
        return [
            t.permute(7, 6, 5, 4, 3, 2, 1, 0),                       # nothing merges
            t[:, :, ::2, :, ::2, :, :, 1::3],                        # steps along three axes
            t.permute(0, 2, 1, 4, 3, 6, 5, 7)[1:, 1:, :, :2],        # pairs swapped, then narrowed
            t[2, 1],                                                 # a contiguous 6-d piece in the middle
        ]

    cpu, dev = views(base_cpu), views(base_dev)
    assert all(v.dim() == 8 for v in cpu[:3]) and not any(v.is_contiguous() for v in cpu[:3])
    layout, plan, image, got = _pack_image(dev)
    assert got == oracle_fmt.data_section(cpu)[0]
    assert got == b"".join(oracle_fmt.header_bytes(oracle_fmt.dtype_name(t.dtype), tuple(t.shape)) +
                           oracle_fmt.payload_bytes_bruteforce(t) for t in cpu)
    # unpack the same image into the same views of a zeroed parent: covered elements come back, the rest stays zero
    zero_dev = torch.zeros_like(base_dev)
    esz = base_cpu.element_size()
    table = P.ItemTable()
    for src, tgt, (off, length) in zip(cpu, views(zero_dev), layout.spans):
        table.add_device(tgt.data_ptr(), off + length - src.numel() * esz, esz, tuple(src.shape), tuple(tgt.stride()))
    P.Plan(table.to_array(), b"", layout.image_bytes, align_to_tensor=True).unpack(image)
    torch.cuda.synchronize()
    mask = torch.zeros(shape, dtype=torch.bool)
    for m in views(mask):
        m.fill_(True)
    got_b = zero_dev.cpu().reshape(-1).view(torch.uint8).reshape(*shape, esz)
    ref_b = base_cpu.reshape(-1).view(torch.uint8).reshape(*shape, esz)
    assert torch.equal(got_b[mask], ref_b[mask]) and int(got_b[~mask].count_nonzero()) == 0

    nine_cpu = _rand_tensor(gen, (2, 2, 2, 2, 2, 2, 2, 2, 3), dtype)
    nine_dev = nine_cpu.to(DEV)
    assert _pack_image([nine_dev])[3] == oracle_fmt.data_section([nine_cpu])[0]
    # a view of nine dimensions that merge into eight goes through the kernels as it is; one that does not is for the
    # saver to stage through a contiguous copy (tests/test_gpu_saver_loader.py)
    merges = nine_dev.transpose(0, 1)
    assert _pack_image([merges])[3] == oracle_fmt.data_section([nine_cpu.transpose(0, 1)])[0]
    with pytest.raises(ValueError, match="contiguous copy"):
        P.build_save_layout([nine_dev.permute(*range(8, -1, -1))])


def test_pack_large_rows_go_through_flat_kernel():
    gen = torch.Generator().manual_seed(15)
    base_cpu = _rand_tensor(gen, (64, 8192), torch.bfloat16)
    base_dev = base_cpu.to(DEV)
    cpu, dev = [base_cpu[:, 1024:5120]], [base_dev[:, 1024:5120]]
    _, plan, _, got = _pack_image(dev)
    assert got == oracle_fmt.data_section(cpu)[0]
    assert plan.info.n_strided_items == 0 and plan.info.n_flat_tiles >= 64


def test_pack_and_unpack_grids_of_more_than_2_to_32_threads():
    """5 GiB through 1 KiB tiles of 1024 threads needs more than 2^32 threads: the grid gets a second dimension.  Checked on the device (payload region of the image == source; round trip restores the source)."""
    from ml_flashpoint.hip import plan as P

    n = 5 * (1 << 30) + 12345
    src = torch.empty(n, dtype=torch.uint8, device=DEV)
    src[: n // 8 * 8].view(torch.int64).random_()
    src[n // 8 * 8 :] = 7
    layout = P.build_save_layout([src])
    hdr = layout.spans[0][1] - n
    image = torch.zeros(layout.image_bytes + 256, dtype=torch.uint8, device=DEV)
    plan = P.Plan(layout.items, layout.blob, layout.image_bytes, tile_bytes=1024, block_threads=1024)
    assert plan.info.n_flat_tiles * 1024 > 1 << 32
    plan.pack(image)
    torch.cuda.synchronize()
    assert torch.equal(image[hdr : hdr + n], src)
    assert bytes(image[:hdr].cpu().numpy()) == oracle_fmt.header_bytes("uint8", (n,)) and int(image[hdr + n :].sum()) == 0
    back = torch.zeros_like(src)
    table = P.ItemTable()
    table.add_device(back.data_ptr(), hdr, 1, (n,), (1,))
    P.Plan(table.to_array(), b"", layout.image_bytes, tile_bytes=1024, block_threads=1024, align_to_tensor=True).unpack(image)
    torch.cuda.synchronize()
    assert torch.equal(back, src)


def test_views_of_a_parent_larger_than_4_gib():
    """Offsets beyond 2^32 bytes on the tensor side and in the image, through the gather, transpose and generic
    kernels.  Checked on the device against torch's own ``contiguous()``; the round trip restores exactly the covered
    elements of a zeroed parent."""
    from ml_flashpoint.hip import plan as P

    rows, cols = 36864, 131072  # 4.5 GiB of uint8
    parent = torch.empty(rows, cols, dtype=torch.uint8, device=DEV)
    parent.view(torch.int64).random_()

    def views(p):
        return [p[:, ::2], p.t(), p[:, 3::7], p[30000:, 5::3]]

    src = views(parent)
    layout = P.build_save_layout(src)
    assert parent.numel() > 1 << 32 and layout.image_bytes > (1 << 32) + (1 << 31)
    image = torch.zeros(layout.image_bytes + 256, dtype=torch.uint8, device=DEV)
    plan = P.Plan(layout.items, layout.blob, layout.image_bytes)
    info = plan.info
    assert info.n_strided_items >= 3
    plan.pack(image)
    torch.cuda.synchronize()
    payload_at = []
    for v, (off, length) in zip(src, layout.spans):
        n = v.numel()
        hdr = length - n
        assert bytes(image[off : off + hdr].cpu().numpy()) == oracle_fmt.header_bytes("uint8", tuple(v.shape))
        assert torch.equal(image[off + hdr : off + length], v.contiguous().reshape(-1))
        payload_at.append(off + hdr)
    assert int(image[layout.image_bytes :].sum()) == 0
    for k, at in enumerate(payload_at):  # one view at a time: p.t() covers everything the others cover
        zero = torch.zeros_like(parent)
        target = views(zero)[k]
        table = P.ItemTable()
        table.add_device(target.data_ptr(), at, 1, tuple(target.shape), tuple(target.stride()))
        P.Plan(table.to_array(), b"", layout.image_bytes, align_to_tensor=True).unpack(image)
        torch.cuda.synchronize()
        assert torch.equal(target, src[k])
        # nothing outside the view was touched: every non-zero byte of the parent lies inside it
        assert int(zero.count_nonzero()) == int(target.count_nonzero())
        del zero


def test_tiny_items_are_copied_one_per_wavefront():
    """Thousands of items of 1..1024 bytes at every alignment: headers and payloads all go through the small-item
    kernel (four items per workgroup); the bytes still match the oracle."""
    gen = torch.Generator().manual_seed(41)
    base = _rand_tensor(gen, (300_000,), torch.uint8)
    dev_base = base.to(DEV)
    cpu, dev, pos = [], [], 0
    for i in range(1500):
        n = 1 + (i * 7) % 1024
        cpu.append(base[pos + (i % 5) : pos + (i % 5) + n])
        dev.append(dev_base[pos + (i % 5) : pos + (i % 5) + n])
        pos += 190
    cpu += [_rand_tensor(gen, (), torch.float64), _rand_tensor(gen, (3,), torch.int64)]
    dev += [t.to(DEV) for t in cpu[-2:]]
    layout, plan, _, got = _pack_image(dev)
    assert got == oracle_fmt.data_section(cpu)[0]
    info = plan.info
    assert info.n_small_items == 2 * len(cpu) and info.n_flat_tiles == 0


def test_pack_host_resident_tensors_travel_in_blob():
    gen = torch.Generator().manual_seed(16)
    cpu = [_rand_tensor(gen, (33, 3), torch.float32), _rand_tensor(gen, (5000,), torch.int64).t(), _rand_tensor(gen, (), torch.int64)]
    mixed = [cpu[0].to(DEV), cpu[1], cpu[2]]
    _, _, _, got = _pack_image(mixed, [b"tail"])
    assert got == oracle_fmt.data_section(cpu, [b"tail"])[0]


def test_unpack_restores_full_tensors_bit_exact():
    from ml_flashpoint.hip import plan as P

    gen = torch.Generator().manual_seed(21)
    cpu = [_rand_tensor(gen, s, d) for s, d in MIXED]
    data, spans = oracle_fmt.data_section(cpu)
    image = torch.frombuffer(bytearray(data), dtype=torch.uint8).to(DEV)
    # (zeroed as bytes: torch has no fill kernel for some of the dtypes, the packed fp4 pairs among them)
    targets = [torch.zeros(t.numel() * t.element_size(), dtype=torch.uint8, device=DEV).view(t.dtype).reshape(t.shape) for t in cpu]
    table = P.ItemTable()
    for t, tgt, (off, length) in zip(cpu, targets, spans):
        nbytes = t.numel() * t.element_size()
        if nbytes:
            table.add_device(tgt.data_ptr(), off + length - nbytes, t.element_size(), tuple(t.shape), tuple(tgt.stride()))
    plan = P.Plan(table.to_array(), b"", len(data), align_to_tensor=True)
    padded = torch.empty(len(data) + 256, dtype=torch.uint8, device=DEV)
    padded[: len(data)] = image
    plan.unpack(padded)
    torch.cuda.synchronize()
    for t, tgt in zip(cpu, targets):
        assert torch.equal(tgt.cpu().contiguous().reshape(-1).view(torch.uint8), t.contiguous().reshape(-1).view(torch.uint8))


def test_unpack_sub_boxes_into_strided_targets():
    """Restore of a narrowed box of the stored tensor into a non-contiguous target (resharding reads)."""
    from ml_flashpoint.hip import plan as P

    gen = torch.Generator().manual_seed(22)
    stored = _rand_tensor(gen, (12, 20, 10), torch.float32)
    data, spans = oracle_fmt.data_section([stored])
    payload_off = spans[0][0] + spans[0][1] - stored.numel() * 4
    image = torch.zeros(len(data) + 256, dtype=torch.uint8, device=DEV)
    image[: len(data)] = torch.frombuffer(bytearray(data), dtype=torch.uint8).to(DEV)
    cases = [((0, 0, 0), (12, 20, 10)), ((1, 0, 3), (2, 2, 2)), ((4, 5, 0), (8, 15, 10)), ((0, 19, 9), (12, 1, 1))]
    for offsets, lengths in cases:
        want = oracle_fmt.read_item(data[spans[0][0] : spans[0][0] + spans[0][1]], offsets, lengths)
        parent = torch.zeros((lengths[0], lengths[1] * 2, lengths[2] + 3), dtype=torch.float32, device=DEV)
        target = parent[:, ::2, 3:]
        src_strides = (200, 10, 1)
        box_off = sum(o * s for o, s in zip(offsets, src_strides)) * 4
        table = P.ItemTable()
        table.add_device(target.data_ptr(), payload_off + box_off, 4, lengths, tuple(target.stride()), image_stride=src_strides)
        plan = P.Plan(table.to_array(), b"", len(data), align_to_tensor=True)
        plan.unpack(image)
        torch.cuda.synchronize()
        assert torch.equal(target.cpu().view(torch.int32), want.contiguous().view(torch.int32))
        assert int(parent[:, 1::2, :].abs().sum()) == 0 and int(parent[:, :, :3].abs().sum()) == 0


def test_plan_rejects_items_outside_image():
    from ml_flashpoint.hip import _lib, plan as P

    t = torch.zeros(100, dtype=torch.float32, device=DEV)
    table = P.ItemTable()
    table.add_device(t.data_ptr(), 10, 4, (100,), (1,))
    with pytest.raises(_lib.HipError, match="does not fit in the image"):
        P.Plan(table.to_array(), b"", 400)
    table = P.ItemTable()
    table.add_blob(0, 0, 16)
    with pytest.raises(_lib.HipError, match="outside the host blob"):
        P.Plan(table.to_array(), b"12345678", 64)


def test_plan_rejects_descriptors_whose_arithmetic_wraps():
    """Shapes whose product wraps 2^64 back onto nbytes, and image-side strides whose reach wraps past the image's
    bounds check, are refused on the host: no kernel is launched with them."""
    from ml_flashpoint.hip import _lib, plan as P

    t = torch.zeros(64, dtype=torch.float32, device=DEV)

    def row(shape, image_stride):
        table = P.ItemTable()
        table.add_device(t.data_ptr(), 0, 4, (8, 8), (8, 1))
        arr = table.to_array()
        arr["ndim"][0] = len(shape)
        arr["shape"][0, : len(shape)] = shape
        arr["stride"][0, : len(shape)] = [1] * len(shape)
        arr["image_stride"][0, : len(shape)] = image_stride
        return arr

    with pytest.raises(_lib.HipError, match="shape does not match nbytes"):
        P.Plan(row((1 << 32, 1 << 32, 64), (0, 0, 1)), b"", 256)  # 2^64 * 64 elements == 64 (mod 2^64)
    with pytest.raises(_lib.HipError, match="reach outside the image"):
        P.Plan(row((2, 32), (1 << 62, 1)), b"", 256)
    with pytest.raises(_lib.HipError, match="reach outside the image"):
        P.Plan(row((2, 2, 16), (1 << 62, 1 << 62, 1)), b"", 256)  # 2^62 + 2^62 wraps a signed 64-bit sum
    with pytest.raises(_lib.HipError, match="not a plausible size"):
        P.Plan(row((8, 8), (8, 1)), b"", 1 << 61)


@pytest.mark.parametrize("nbytes", [1, 15, 1023, 1024, 65535, 65536, 65537, 3 * 65536 + 1024 + 7, (5 << 20) + 13])
def test_crc32c_device_matches_oracle(nbytes, oracle_c):
    from ml_flashpoint.hip import plan as P

    gen = torch.Generator().manual_seed(nbytes)
    host = torch.randint(0, 256, (nbytes,), dtype=torch.uint8, generator=gen)
    dev = host.to(DEV)
    for chunk in (65536, 1 << 20):
        got = P.crc32c_device(dev, nbytes, chunk)
        n_chunks = (nbytes + chunk - 1) // chunk
        want = np.zeros(n_chunks, dtype=np.uint32)
        raw = host.numpy().tobytes()
        oracle_c.oracle_crc32c_chunks(raw, nbytes, chunk, want.ctypes.data)
        assert got.tolist() == want.tolist()
        # checksum of checksums: chaining the chunk CRCs reproduces the CRC of the whole buffer
        whole = int(got[0])
        for k in range(1, n_chunks):
            whole = P.crc32c_combine(whole, int(got[k]), min(chunk, nbytes - k * chunk))
        assert whole == oracle_c.oracle_crc32c(raw, nbytes)


@pytest.mark.parametrize("gib_x2,chunk", [(3, 32 << 20), (17, 32 << 20), (17, 3 << 16)])
def test_crc32c_device_on_buffers_large_enough_for_long_segments(gib_x2, chunk, oracle_c):
    """Buffers of 1.5 and 8.5 GiB are cut into segments of 128 and 512 KiB per wavefront (64 KiB where the chunk size
    allows nothing longer).  Every chunk value, the ragged last one included, is compared with the host routine's
    (SSE4.2, itself held to the oracle by the small cases) and a sample of them with the oracle's byte-table routine;
    the chunk values chain to the checksum of the whole buffer."""
    from ml_flashpoint.hip import plan as P

    gen = torch.Generator().manual_seed(gib_x2)
    block = torch.randint(0, 256, (1 << 29,), dtype=torch.uint8, generator=gen)
    nbytes = gib_x2 * (1 << 29) - 54321
    dev = block.to(DEV).repeat(gib_x2)
    dev[(5 << 28) + 77 :: 1 << 29] ^= 0x5A  # the repeats differ, at places inside segments
    got = P.crc32c_device(dev, nbytes, chunk)
    n_chunks = -(-nbytes // chunk)
    assert len(got) == n_chunks
    sampled = {0, 1, n_chunks // 2, n_chunks - 2, n_chunks - 1}
    step = (1 << 29) // chunk * chunk  # host copies are cut on chunk boundaries
    whole = None
    for start in range(0, nbytes, step):
        raw = dev[start : min(start + step, nbytes)].cpu().numpy()
        for off in range(0, raw.size, chunk):
            k = (start + off) // chunk
            n = min(chunk, raw.size - off)
            assert P.crc32c_host(raw.ctypes.data + off, n) == int(got[k]), f"chunk {k}"
            if k in sampled:
                assert oracle_c.oracle_crc32c(ctypes.cast(ctypes.c_void_p(raw.ctypes.data + off), ctypes.c_char_p), n) == int(got[k]), f"chunk {k}"
        part = P.crc32c_host(raw.ctypes.data, raw.size)
        whole = part if whole is None else P.crc32c_combine(whole, part, raw.size)
    chained = int(got[0])
    for k in range(1, n_chunks):
        chained = P.crc32c_combine(chained, int(got[k]), min(chunk, nbytes - k * chunk))
    assert chained == whole


def test_crc32c_known_vectors_on_device(oracle_c):
    from ml_flashpoint.hip import plan as P

    for data, want in [
        (b"123456789", 0xE3069283),
        (bytes(32), 0x8A9136AA),
        (b"\xff" * 32, 0x62A8AB43),
        (bytes(range(32)), 0x46DD794E),
        (bytes(range(31, -1, -1)), 0x113FDB5C),
    ]:
        dev = torch.frombuffer(bytearray(data), dtype=torch.uint8).to(DEV)
        assert int(P.crc32c_device(dev, len(data), 65536)[0]) == want


@pytest.mark.parametrize("nbytes", [1, 4097, (1 << 20) + 5, (9 << 20) + 12345])
def test_copy_engine_round_trip(nbytes, shm_dir, oracle_c):
    """Device -> mapped tmpfs file -> device through the pinned ring, several chunks, ragged tail."""
    from ml_flashpoint.checkpoint_object_manager.buffer_object.buffer_object_ext import BufferObject
    from ml_flashpoint.hip import plan as P

    gen = torch.Generator().manual_seed(nbytes)
    host = torch.randint(0, 256, (nbytes,), dtype=torch.uint8, generator=gen)
    dev = host.to(DEV)
    engine = P.CopyEngine(slot_bytes=1 << 20, n_slots=3, n_threads=4)
    bo = BufferObject(f"{shm_dir}/obj.bin", 4096 + nbytes, True)
    stream = torch.cuda.current_stream().cuda_stream
    stats = engine.d2h(dev.data_ptr(), bo.get_data_ptr() + 4096, nbytes, stream)
    assert stats.bytes == nbytes and stats.chunks == (nbytes + (1 << 20) - 1) // (1 << 20)
    assert bytes(memoryview(bo)[4096:]) == host.numpy().tobytes()
    back = torch.zeros(nbytes + 64, dtype=torch.uint8, device=DEV)
    engine.h2d(bo.get_data_ptr() + 4096, back.data_ptr(), nbytes, stream)
    torch.cuda.synchronize()
    assert torch.equal(back[:nbytes].cpu(), host) and int(back[nbytes:].sum()) == 0
    # device -> host with the checksum computed beside the copies: same bytes, CRCs equal to the oracle's
    if nbytes >= 65536:
        memoryview(bo)[4096:] = bytes(nbytes)
        stats, crcs = engine.d2h_crc(dev.data_ptr(), bo.get_data_ptr() + 4096, nbytes, stream, 1 << 20)
        assert bytes(memoryview(bo)[4096:]) == host.numpy().tobytes()
        want = np.zeros(len(crcs), dtype=np.uint32)
        oracle_c.oracle_crc32c_chunks(host.numpy().tobytes(), nbytes, 1 << 20, want.ctypes.data)
        assert crcs.tolist() == want.tolist()
    # the same two transfers through the file descriptor (pwrite / pread), at an odd file offset
    memoryview(bo)[:] = bytes(4096 + nbytes)
    bo2 = BufferObject(f"{shm_dir}/obj2.bin", 4096 + 7 + nbytes, True)
    stats = engine.d2h_fd(dev.data_ptr(), bo2.fileno(), 4096 + 7, nbytes, stream)
    assert stats.bytes == nbytes
    assert bytes(memoryview(bo2)[4096 + 7 :]) == host.numpy().tobytes() and bytes(memoryview(bo2)[: 4096 + 7]) == bytes(4096 + 7)
    back.zero_()
    engine.h2d_fd(bo2.fileno(), 4096 + 7, back.data_ptr(), nbytes, stream)
    torch.cuda.synchronize()
    assert torch.equal(back[:nbytes].cpu(), host) and int(back[nbytes:].sum()) == 0
    from ml_flashpoint.hip import _lib

    with pytest.raises(_lib.HipError, match="pread"):  # asking for more than the file holds is an error, not a hang
        engine.h2d_fd(bo2.fileno(), 4096 + 7, back.data_ptr(), nbytes + 64, stream)
    bo.close()
    bo2.close()
    engine.destroy()


@pytest.mark.parametrize("slot_bytes, chunk_bytes", [(1 << 20, 1 << 20), (3 << 20, 1 << 20), (1 << 20, 4 << 20),
                                                     ((1 << 20) + 4096, 3 << 16), (32 << 20, 32 << 20)])
@pytest.mark.parametrize("nbytes", [65536 + 1, (9 << 20) + 12345, (70 << 20) + 7])
@pytest.mark.parametrize("misaligned", [0, 5])
def test_checksums_taken_by_the_host_threads_equal_the_kernels_and_the_oracle(slot_bytes, chunk_bytes, nbytes, misaligned,
                                                                             shm_dir, oracle_c):
    """``mlf_engine_set_host_checksums``: the threads that move the pinned slots into the destination take the
    checksums of what they move - pieces cut at chunk boundaries, three interleaved chains per piece, joined by
    crc(A || B) = crc(A) x^(8 |B|) + crc(B).  Same bytes in the destination, same values as the kernels' and as the
    oracle's, for slots smaller and larger than chunks, sizes that end inside a piece, destinations off the
    32-byte grid (no streaming stores), through the mapping and through the file descriptor."""
    from ml_flashpoint.checkpoint_object_manager.buffer_object.buffer_object_ext import BufferObject
    from ml_flashpoint.hip import plan as P

    gen = torch.Generator().manual_seed(nbytes + slot_bytes)
    host = torch.randint(0, 256, (nbytes,), dtype=torch.uint8, generator=gen)
    raw = host.numpy().tobytes()
    dev = host.to(DEV)
    want = np.zeros(-(-nbytes // chunk_bytes), dtype=np.uint32)
    oracle_c.oracle_crc32c_chunks(raw, nbytes, chunk_bytes, want.ctypes.data)
    engine = P.CopyEngine(slot_bytes=slot_bytes, n_slots=3, n_threads=5)
    bo = BufferObject(f"{shm_dir}/hostcrc.bin", 4096 + misaligned + nbytes, True)
    stream = torch.cuda.current_stream().cuda_stream
    first = 4096 + misaligned
    _, by_kernels = engine.d2h_crc(dev.data_ptr(), bo.get_data_ptr() + first, nbytes, stream, chunk_bytes)
    assert by_kernels.tolist() == want.tolist()
    engine.set_host_checksums(True)
    memoryview(bo)[:] = bytes(first + nbytes)
    stats, by_host = engine.d2h_crc(dev.data_ptr(), bo.get_data_ptr() + first, nbytes, stream, chunk_bytes)
    assert stats.bytes == nbytes and bytes(memoryview(bo)[first:]) == raw and bytes(memoryview(bo)[:first]) == bytes(first)
    assert by_host.tolist() == want.tolist()
    landed = ctypes.c_uint64(0)
    memoryview(bo)[:] = bytes(first + nbytes)
    _, watched = engine.d2h_watched(dev.data_ptr(), bo.get_data_ptr() + first, nbytes, stream, chunk_bytes, landed)
    assert int(landed.value) == nbytes and watched.tolist() == want.tolist() and bytes(memoryview(bo)[first:]) == raw
    engine.set_host_checksums(False)
    _, again = engine.d2h_crc(dev.data_ptr(), bo.get_data_ptr() + first, nbytes, stream, chunk_bytes)
    assert again.tolist() == want.tolist()
    bo.close()
    engine.destroy()


@pytest.mark.parametrize("data_off, nbytes, chunk_bytes", [(0, (5 << 20) + 3, 1 << 20), (777, (5 << 20) + 3, 1 << 20),
                                                           ((3 << 20) - 5, 4, 1 << 20), ((1 << 20) + 4096, 70 << 20, 32 << 20),
                                                           (65536 * 3 + 1, 65536 * 9, 65536)])
def test_pieces_of_a_data_section_are_checksummed_on_the_sections_chunk_grid(data_off, nbytes, chunk_bytes, shm_dir, oracle_c):
    """``mlf_engine_d2h_cut`` / ``mlf_engine_host_copy_cut``: a piece that begins inside a chunk of the section it
    belongs to gets one value for the bytes up to the next boundary, one per whole chunk and one for the rest - the
    parts ``integrity.ChunkChecksums.cuts`` names - each equal to the oracle's CRC-32C of those bytes; joined with
    the neighbours' parts they give the section's chunk values."""
    from ml_flashpoint.checkpoint_object_manager.buffer_object.buffer_object_ext import BufferObject
    from ml_flashpoint.hip import integrity
    from ml_flashpoint.hip import plan as P

    gen = torch.Generator().manual_seed(nbytes + data_off)
    host = torch.randint(0, 256, (nbytes,), dtype=torch.uint8, generator=gen)
    raw = host.numpy().tobytes()
    dev = host.to(DEV)
    parts = integrity.ChunkChecksums.cuts(data_off, nbytes, chunk_bytes)
    want = []
    for first, length in parts:
        one = np.zeros(1, dtype=np.uint32)
        oracle_c.oracle_crc32c_chunks(raw[first - data_off : first - data_off + length], length, 1 << 40, one.ctypes.data)
        want.append(int(one[0]))
    engine = P.CopyEngine(slot_bytes=1 << 20, n_slots=3, n_threads=5)
    bo = BufferObject(f"{shm_dir}/cut.bin", 4096 + nbytes, True)
    stream = torch.cuda.current_stream().cuda_stream
    stats, got = engine.d2h_cut(dev.data_ptr(), bo.get_data_ptr() + 4096, nbytes, data_off, chunk_bytes, producer_stream=stream)
    assert stats.bytes == nbytes and bytes(memoryview(bo)[4096:]) == raw and got == want
    done = torch.cuda.Event()
    done.record()
    landed = ctypes.c_uint64(0)
    memoryview(bo)[4096:] = bytes(nbytes)
    _, got = engine.d2h_cut(dev.data_ptr(), bo.get_data_ptr() + 4096, nbytes, data_off, chunk_bytes,
                            ready_event=done.cuda_event, landed=landed)
    assert int(landed.value) == nbytes and bytes(memoryview(bo)[4096:]) == raw and got == want
    memoryview(bo)[4096:] = bytes(nbytes)
    source = host.clone()
    assert engine.host_copy_cut(bo.get_data_ptr() + 4096, source.data_ptr(), nbytes, data_off, chunk_bytes) == want
    assert bytes(memoryview(bo)[4096:]) == raw
    # the section's chunk values from this piece and a neighbour on either side
    before, after = b"\x5a" * data_off, b"\xa5" * 12345
    whole = before + raw + after
    sums = integrity.ChunkChecksums(chunk_bytes, len(whole))
    for offset, data in ((0, before), (data_off, raw), (data_off + nbytes, after)):
        if not data:
            continue
        values = []
        for first, length in integrity.ChunkChecksums.cuts(offset, len(data), chunk_bytes):
            one = np.zeros(1, dtype=np.uint32)
            oracle_c.oracle_crc32c_chunks(data[first - offset : first - offset + length], length, 1 << 40, one.ctypes.data)
            values.append(int(one[0]))
        sums.add(offset, len(data), got if data is raw else values)
    section = np.zeros(-(-len(whole) // chunk_bytes), dtype=np.uint32)
    oracle_c.oracle_crc32c_chunks(whole, len(whole), chunk_bytes, section.ctypes.data)
    assert sums.result().tolist() == section.tolist()
    lib = __import__("ml_flashpoint.hip._lib", fromlist=["load"]).load()
    out = np.zeros(4, dtype=np.uint32)
    assert lib.mlf_engine_d2h_cut(engine._handle, dev.data_ptr(), bo.get_data_ptr() + 4096, nbytes, stream, None, chunk_bytes,
                                  chunk_bytes, out.ctypes.data, 4, None, None) != 0  # a first part as long as a chunk
    bo.close()
    engine.destroy()


def test_watched_transfer_publishes_only_bytes_that_are_in_place(shm_dir, oracle_c):
    """While a 200 MiB image crosses the link in 1 MiB slots, a second thread follows the progress counter and copies
    whatever prefix it announces out of the mapping: the counter only grows, never runs ahead of the data, ends at the
    full size, and the follower's copy is the image.  Checksums equal those of the unwatched call."""
    import threading

    from ml_flashpoint.checkpoint_object_manager.buffer_object.buffer_object_ext import BufferObject
    from ml_flashpoint.hip import plan as P

    nbytes = (200 << 20) + 4321
    gen = torch.Generator().manual_seed(200)
    host = torch.randint(0, 256, (nbytes,), dtype=torch.uint8, generator=gen)
    want = host.numpy()
    dev = host.to(DEV)
    engine = P.CopyEngine(slot_bytes=1 << 20, n_slots=3, n_threads=4)
    bo = BufferObject(f"{shm_dir}/watched.bin", 4096 + nbytes, True)
    view = np.frombuffer(memoryview(bo), dtype=np.uint8)[4096:]
    landed = ctypes.c_uint64(12345)  # whatever was there before is overwritten with 0 first
    replica = np.zeros(nbytes, dtype=np.uint8)
    seen, done = [], threading.Event()

    def follow():
        have = 0
        while have < nbytes and not done.wait(0.0005):
            now = int(landed.value)
            if now == 12345:
                continue  # the call has not begun
            if now != have:
                seen.append(now)
                replica[have:now] = view[have:now]
                have = now
        now = int(landed.value)
        replica[have:now] = view[have:now]
        seen.append(now)

    follower = threading.Thread(target=follow)
    follower.start()
    stream = torch.cuda.current_stream().cuda_stream
    stats, crcs = engine.d2h_watched(dev.data_ptr(), bo.get_data_ptr() + 4096, nbytes, stream, 1 << 20, landed)
    follower.join(30)
    done.set()
    follower.join()
    assert int(landed.value) == nbytes and stats.bytes == nbytes
    assert seen == sorted(seen) and seen[-1] == nbytes
    assert len(set(seen)) >= 3, "the follower never saw the transfer under way"
    assert all(v % (1 << 20) == 0 for v in seen if v != nbytes)  # whole slots
    assert np.array_equal(replica, want) and np.array_equal(view, want)
    _, plain = engine.d2h_crc(dev.data_ptr(), bo.get_data_ptr() + 4096, nbytes, stream, 1 << 20)
    assert crcs.tolist() == plain.tolist()
    _, none = engine.d2h_watched(dev.data_ptr(), bo.get_data_ptr() + 4096, 4097, stream, 0, landed)
    assert none is None and int(landed.value) == 4097
    del view
    bo.close()
    engine.destroy()


def test_try_allocate_reports_what_the_allocator_cannot_provide():
    """A request the device cannot satisfy comes back as None (after the allocator has returned its unused segments
    and been asked again), not as an exception; an ordinary one as a byte buffer."""
    from ml_flashpoint.hip import plan as P

    assert P.try_allocate(1 << 50, torch.device(DEV)) is None  # a pebibyte
    buf = P.try_allocate(4096, torch.device(DEV))
    assert buf.dtype == torch.uint8 and buf.numel() == 4096 and buf.device == torch.device(DEV)


def test_a_cpp_program_uses_the_two_libraries_without_python_or_torch(shm_dir):
    """tests/cabi/direct_caller.cpp links libmlf_hip.so and libmlf_buffer.so and walks the whole path - plan, pack,
    checksum, watched transfer into a buffer file, reopen, upload through the descriptor, unpack - checking every
    stage against bytes it builds on the host.  Built by ``__graft_entry__.build()``."""
    import os
    import subprocess

    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cabi", "_build", "direct_caller")
    assert os.path.exists(exe), "run __graft_entry__.build() first"
    done = subprocess.run([exe, shm_dir], capture_output=True, text=True, timeout=100)
    assert done.returncode == 0, done.stderr + done.stdout
    assert "direct C-ABI caller ok" in done.stdout
