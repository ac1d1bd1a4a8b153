"""Seeded random differential test of the pack / unpack kernels against the CPU oracle.

Every seed builds a few parent tensors of a random element size and a dozen random views of them (slices with
steps, permutations, transposes, narrow rows, single rows/columns, empty views), packs them in one plan and compares
the whole image with the oracle's data section; then unpacks the image into the same views of zeroed parents and
compares every byte of the parents: covered elements equal the originals, everything else is still zero.
Between them the seeds reach every kernel (flat with its three span classes, small items, vector gather, LDS
transposition, generic walk) at alignments and extents nobody chose by hand.
"""

import random

import numpy as np
import pytest
import torch

from oracle import mlf_format as oracle_fmt

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.uint8, torch.float8_e4m3fn, torch.bfloat16, torch.float16, torch.float32, torch.int64, torch.complex128]


def _random_view(rng: random.Random, t: torch.Tensor) -> torch.Tensor:
    """A random view of ``t`` built from the operations checkpointed tensors go through."""
    v = t
    for _ in range(rng.randint(1, 3)):
        if v.dim() == 0:
            break
        op = rng.choice(["slice", "slice", "step", "permute", "t", "index", "narrow_rows", "empty"])
        d = rng.randrange(v.dim())
        n = v.size(d)
        if op == "slice" and n > 1:
            a = rng.randrange(0, n)
            b = rng.randrange(a + 1, n + 1)
            v = v.narrow(d, a, b - a)
        elif op == "step" and n > 1:
            step = rng.choice([2, 2, 3, 4, 5])
            start = rng.randrange(0, min(step, n))
            v = v[(slice(None),) * d + (slice(start, None, step),)]
        elif op == "permute" and v.dim() > 1:
            perm = list(range(v.dim()))
            rng.shuffle(perm)
            v = v.permute(*perm)
        elif op == "t" and v.dim() >= 2:
            v = v.transpose(-1, -2)
        elif op == "index" and v.dim() > 1 and n > 0:
            v = v.select(d, rng.randrange(n))
        elif op == "narrow_rows" and n > 4:
            v = v.narrow(d, rng.randrange(0, n // 2), max(1, n // 2))
        elif op == "empty" and rng.random() < 0.15:
            v = v.narrow(d, 0, 0)
    return v


def _parents(rng: random.Random, gen: torch.Generator, dtype: torch.dtype):
    esz = torch.empty((), dtype=dtype).element_size()
    shapes = [
        (rng.randint(1, 9), rng.randint(1, 70), rng.randint(1, 300)),
        (rng.randint(16, 400), rng.randint(16, 1500)),
        (rng.randint(1, 3), rng.randint(200, 5000)),
        (rng.randint(1, 200_000),),
        (rng.randint(300_000, 1_500_000),),  # long enough for full groups of tiles in every span class
    ]
    out = []
    for shape in shapes:
        numel = int(np.prod(shape))
        raw = torch.randint(0, 256, (numel * esz,), dtype=torch.uint8, generator=gen)
        out.append(raw.view(dtype).reshape(shape))
    return out


def _bytes_of(t: torch.Tensor) -> torch.Tensor:
    esz = t.element_size()
    flat = t.contiguous().reshape(-1)
    if flat.numel() and flat.stride(0) != 1:  # a one-element tensor keeps whatever stride its view had
        flat = torch.empty(flat.shape, dtype=flat.dtype, device=flat.device).copy_(flat)
    return flat.view(torch.uint8).reshape(*t.shape, esz)


@pytest.mark.parametrize("seed", range(56))
def test_random_views_pack_and_unpack_match_the_oracle(seed):
    from ml_flashpoint.hip import plan as P

    rng = random.Random(1000 + seed)
    gen = torch.Generator().manual_seed(1000 + seed)
    dtype = DTYPES[seed % len(DTYPES)]
    cpu_parents = _parents(rng, gen, dtype)
    dev_parents = [p.to(DEV) for p in cpu_parents]
    picks = []
    for _ in range(12):
        k = rng.randrange(len(cpu_parents))
        state = rng.getstate()
        picks.append((k, state))

    def views_of(parents):
        out = []
        for k, state in picks:
            local = random.Random()
            local.setstate(state)
            out.append(_random_view(local, parents[k]))
        return out

    cpu_views, dev_views = views_of(cpu_parents), views_of(dev_parents)
    assert [tuple(v.shape) for v in cpu_views] == [tuple(v.shape) for v in dev_views]
    assert [v.stride() for v in cpu_views] == [v.stride() for v in dev_views]
    tile_bytes = rng.choice([0, 0, 1024, 2048])
    layout = P.build_save_layout(dev_views)
    plan = P.Plan(layout.items, layout.blob, layout.image_bytes, tile_bytes=tile_bytes)
    image = torch.full((max(layout.image_bytes, 1) + 512,), 0xAB, dtype=torch.uint8, device=DEV)
    plan.pack(image)
    torch.cuda.synchronize()
    host = image.cpu().numpy()
    assert (host[layout.image_bytes :] == 0xAB).all(), "pack wrote past the end of the image"
    want, spans = oracle_fmt.data_section(cpu_views)
    assert layout.spans == spans
    assert host[: layout.image_bytes].tobytes() == want

    esz = cpu_parents[0].element_size()
    zero_parents = [torch.zeros_like(p) for p in dev_parents]
    table = P.ItemTable()
    for src, tgt, (off, length) in zip(cpu_views, views_of(zero_parents), layout.spans):
        nbytes = src.numel() * esz
        if nbytes == 0:
            continue
        table.add_device(tgt.data_ptr(), off + length - nbytes, esz, tuple(src.shape), tuple(tgt.stride()))
    if len(table):
        P.Plan(table.to_array(), b"", layout.image_bytes, tile_bytes=tile_bytes, align_to_tensor=True).unpack(image)
        torch.cuda.synchronize()
    masks = [torch.zeros(p.shape, dtype=torch.bool) for p in cpu_parents]
    for m in views_of(masks):
        m.fill_(True)
    for got_dev, ref, mask in zip(zero_parents, cpu_parents, masks):
        got_b, ref_b = _bytes_of(got_dev.cpu()), _bytes_of(ref)
        assert torch.equal(got_b[mask], ref_b[mask])
        assert int(got_b[~mask].count_nonzero()) == 0
