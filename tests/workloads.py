"""Seeded synthetic state dicts in the shapes of the benchmark's configurations (shared by the tests and bench.py).

Values are generated with ``torch.Generator`` seeds fixed per config, on the requested device; ``scale`` shrinks a
config for quick tests by dividing layer counts / widths, keeping the tensor structure.
"""

from typing import Dict, List, Tuple

import torch


def _gen(device, seed):
    return torch.Generator(device=device).manual_seed(seed)


def gpt2_small(device="cpu", seed=1234, layers=12, d=768, vocab=50257, ctx=1024) -> Dict[str, torch.Tensor]:
    """C1: GPT-2-small, fp32, N(0, 0.02): 148 tensors, 124 439 808 parameters at the default sizes."""
    g = _gen(device, seed)

    def w(*shape):
        return torch.randn(*shape, generator=g, device=device, dtype=torch.float32) * 0.02

    sd = {"transformer.wte.weight": w(vocab, d), "transformer.wpe.weight": w(ctx, d)}
    for i in range(layers):
        p = f"transformer.h.{i}."
        sd[p + "ln_1.weight"], sd[p + "ln_1.bias"] = w(d), w(d)
        sd[p + "attn.c_attn.weight"], sd[p + "attn.c_attn.bias"] = w(d, 3 * d), w(3 * d)
        sd[p + "attn.c_proj.weight"], sd[p + "attn.c_proj.bias"] = w(d, d), w(d)
        sd[p + "ln_2.weight"], sd[p + "ln_2.bias"] = w(d), w(d)
        sd[p + "mlp.c_fc.weight"], sd[p + "mlp.c_fc.bias"] = w(d, 4 * d), w(4 * d)
        sd[p + "mlp.c_proj.weight"], sd[p + "mlp.c_proj.bias"] = w(4 * d, d), w(d)
    sd["transformer.ln_f.weight"], sd["transformer.ln_f.bias"] = w(d), w(d)
    return sd


def llama_shapes(layers=32, d=4096, ffn=14336, kv=1024, vocab=128256) -> List[Tuple[str, Tuple[int, ...]]]:
    shapes = [("model.embed_tokens.weight", (vocab, d))]
    for i in range(layers):
        p = f"model.layers.{i}."
        shapes += [
            (p + "self_attn.q_proj.weight", (d, d)),
            (p + "self_attn.k_proj.weight", (kv, d)),
            (p + "self_attn.v_proj.weight", (kv, d)),
            (p + "self_attn.o_proj.weight", (d, d)),
            (p + "mlp.gate_proj.weight", (ffn, d)),
            (p + "mlp.up_proj.weight", (ffn, d)),
            (p + "mlp.down_proj.weight", (d, ffn)),
            (p + "input_layernorm.weight", (d,)),
            (p + "post_attention_layernorm.weight", (d,)),
        ]
    shapes += [("model.norm.weight", (d,)), ("lm_head.weight", (vocab, d))]
    return shapes


def llama3_8b_shard(device, seed=2024, **dims) -> Dict[str, torch.Tensor]:
    """C2: bf16 weights + fp32 master weights + fp32 Adam m and v.  At the default sizes: 4 x 291 tensors,
    8 030 261 248 parameters, 112 423 657 472 payload bytes.  master ~ N(0, 0.02); bf16 = master.to(bf16);
    m = N(0, 1) * 1e-3; v = |N(0, 1)| * 1e-4."""
    g = _gen(device, seed)
    sd = {}
    for name, shape in llama_shapes(**dims):
        master = torch.randn(*shape, generator=g, device=device, dtype=torch.float32) * 0.02
        sd[f"model.{name}"] = master.to(torch.bfloat16)
        sd[f"optimizer.master.{name}"] = master
        sd[f"optimizer.exp_avg.{name}"] = torch.randn(*shape, generator=g, device=device, dtype=torch.float32) * 1e-3
        sd[f"optimizer.exp_avg_sq.{name}"] = torch.randn(*shape, generator=g, device=device, dtype=torch.float32).abs_() * 1e-4
    return sd


def offloaded_optimizer_shard(device, seed=31, layers=8, d=8192, ffn=16384) -> Dict[str, torch.Tensor]:
    """Weights on the device, optimizer state in host memory (an offloaded optimizer): per layer one bf16 weight of
    ``d`` x ``ffn`` on the device and its fp32 master copy, exp_avg and exp_avg_sq on the host.  At the default
    sizes: 2.1 GB on the device, 12.9 GB on the host."""
    g = _gen(device, seed)
    host = torch.Generator().manual_seed(seed)
    sd = {}
    for i in range(layers):
        master = torch.randn(d, ffn, generator=host, dtype=torch.float32) * 0.02
        sd[f"model.layers.{i}.weight"] = master.to(torch.bfloat16).to(device)
        sd[f"optimizer.master.{i}"] = master
        sd[f"optimizer.exp_avg.{i}"] = torch.randn(d, ffn, generator=host, dtype=torch.float32) * 1e-3
        sd[f"optimizer.exp_avg_sq.{i}"] = torch.randn(d, ffn, generator=host, dtype=torch.float32).abs_() * 1e-4
    _ = g
    return sd


def many_small(device, seed=7, count=20000, min_log2=6, max_log2=22) -> Dict[str, torch.Tensor]:
    """C3: ``count`` tensors, byte sizes log-uniform in [2^min_log2, 2^max_log2], dtypes cycling fp32/bf16/int64."""
    cpu = torch.Generator().manual_seed(seed)
    exps = torch.rand(count, generator=cpu) * (max_log2 - min_log2) + min_log2
    g = _gen(device, seed)
    dtypes = [torch.float32, torch.bfloat16, torch.int64]
    sd = {}
    for i in range(count):
        dtype = dtypes[i % 3]
        esz = torch.empty((), dtype=dtype).element_size()
        numel = max(int(2.0 ** float(exps[i])) // esz, 1)
        if dtype == torch.int64:
            t = torch.randint(-(2**62), 2**62, (numel,), generator=g, device=device, dtype=torch.int64)
        else:
            t = torch.randn(numel, generator=g, device=device, dtype=torch.float32).to(dtype)
        sd[f"small.{i}"] = t
    return sd


def mixtral_expert_shard(device, seed=87, layers=32, experts=8, d=4096, ffn=14336, kv=1024) -> Dict[str, torch.Tensor]:
    """C4: bf16 expert FFN weights (3 per expert per layer) plus attention, router and norms, N(0, 0.02)."""
    g = _gen(device, seed)

    def w(*shape):
        return (torch.randn(*shape, generator=g, device=device, dtype=torch.float32) * 0.02).to(torch.bfloat16)

    sd = {}
    for i in range(layers):
        p = f"model.layers.{i}."
        sd[p + "self_attn.q_proj.weight"], sd[p + "self_attn.o_proj.weight"] = w(d, d), w(d, d)
        sd[p + "self_attn.k_proj.weight"], sd[p + "self_attn.v_proj.weight"] = w(kv, d), w(kv, d)
        sd[p + "block_sparse_moe.gate.weight"] = w(experts, d)
        sd[p + "input_layernorm.weight"], sd[p + "post_attention_layernorm.weight"] = w(d), w(d)
        for e in range(experts):
            q = p + f"block_sparse_moe.experts.{e}."
            sd[q + "w1.weight"], sd[q + "w3.weight"], sd[q + "w2.weight"] = w(ffn, d), w(ffn, d), w(d, ffn)
    return sd


def strided_views(device, seed=5, count=2000, min_dim=1024, max_dim=16384, n_parents=None,
                  mean_view_bytes=10 << 20) -> Tuple[Dict[str, torch.Tensor], list]:
    """C5: ``count`` non-contiguous views - transposed blocks, every-other-column slices and 16-row blocks - of
    bf16 / fp8-e4m3 / fp32 parents with 1k..16k rows and columns (multiples of 16) whose bytes are uniform random.
    Views average ``mean_view_bytes`` of payload (2000 x 10 MB = 20 GB) and share ``n_parents`` parents
    (default count // 32).  Returns (state dict of views, list of parents kept alive)."""
    cpu = torch.Generator().manual_seed(seed)
    g = _gen(device, seed)
    dtypes = [torch.bfloat16, torch.float8_e4m3fn, torch.float32]
    n_parents = n_parents or max(3, count // 32)
    span = (max_dim - min_dim) // 16

    def rnd(lo, hi):  # integer in [lo, hi]
        return lo + int(torch.randint(0, max(hi - lo, 0) + 1, (1,), generator=cpu))

    parents = []
    for p in range(n_parents):
        rows, cols = min_dim + 16 * rnd(0, span), min_dim + 16 * rnd(0, span)
        dtype = dtypes[p % 3]
        esz = torch.empty((), dtype=dtype).element_size()
        raw = torch.randint(0, 256, (rows * cols * esz,), generator=g, device=device, dtype=torch.uint8)
        parents.append(raw.view(dtype).reshape(rows, cols))
    sd = {}
    for i in range(count):
        parent = parents[i % n_parents]
        rows, cols = parent.shape
        esz = parent.element_size()
        want = rnd(mean_view_bytes // 5, 2 * mean_view_bytes - mean_view_bytes // 5) // esz  # elements, mean = target
        kind = (i // n_parents) % 3
        if kind == 0:  # transposed block: h x w of the parent, seen as w x h
            h = 16 * rnd(4, min(rows, 4096) // 16)
            w = max(16, min(cols, (want // h) // 16 * 16))
            r0, c0 = 16 * rnd(0, (rows - h) // 16), 16 * rnd(0, (cols - w) // 16)
            view = parent[r0 : r0 + h, c0 : c0 + w].t()
        elif kind == 1:  # every other column of a band of rows
            h = max(1, min(rows, want // (cols // 2)))
            r0 = rnd(0, rows - h)
            view = parent[r0 : r0 + h, ::2]
        else:  # block of 16-row groups (contiguous in memory, but a view with a storage offset)
            r = max(1, min(rows // 16, want // (16 * cols)))
            k = rnd(0, rows // 16 - r)
            view = parent[16 * k : 16 * (k + r), :]
        sd[f"views.{i}"] = view
    return sd, parents


def payload_bytes(sd) -> int:
    return sum(t.numel() * t.element_size() for t in sd.values() if isinstance(t, torch.Tensor))


def fingerprint(t: torch.Tensor) -> Tuple[int, int]:
    """Order-sensitive 2x63-bit checksum of a tensor's bytes, computed on its device (bit patterns, not values).
    Used to compare restored tensors with the originals at sizes where a second copy does not fit."""
    flat = t.detach().contiguous().reshape(-1)
    if flat.numel() and flat.stride(0) != 1:  # a one-element tensor keeps whatever stride its view had
        flat = torch.empty(flat.shape, dtype=flat.dtype, device=flat.device).copy_(flat)
    flat = flat.view(torch.uint8)
    n = flat.numel()
    pad = (-n) % 8
    if pad:
        flat = torch.cat([flat, torch.zeros(pad, dtype=torch.uint8, device=flat.device)])
    words = flat.view(torch.int64)
    idx = torch.arange(1, words.numel() + 1, device=words.device, dtype=torch.int64)
    a = int(words.sum().item()) & ((1 << 63) - 1)
    b = int((words * (idx * 2 + 1)).sum().item()) & ((1 << 63) - 1)
    return a ^ n, b
