"""Named synthetic workloads of the benchmark / parity harness (the counterpart of the
reference's flash_bias/config.py:12-17 and of the input recipe in flash_bias/benchmark.py:27-43,
:220-228).  Every workload is seeded, generated in fp32 on the CPU and rounded to its dtype
once, so that a CPU checker and the GPU kernels consume identical values."""
import math

import torch

from . import factors

#: B2 H4 d32 r8 sweep of flash_bias/config.py:12,17 (bf16 here)
SWEEP_LENGTHS = (1024, 2048, 4096, 8192, 16384)
HEADLINE = dict(B=2, H=4, L=16384, d=32, r=8)


def _qkv(B, Lq, Lk, H, d, g, dtype):
    q = torch.randn(B, Lq, H, d, generator=g).to(dtype)
    k = torch.randn(B, Lk, H, d, generator=g).to(dtype)
    v = torch.randn(B, Lk, H, d, generator=g).to(dtype)
    do = torch.randn(B, Lq, H, d, generator=g).to(dtype)
    return q, k, v, do


def _pack(q, k, v, do, q_bias, k_bias, causal, scale, **extra):
    out = dict(q=q, k=k, v=v, do=do, q_bias=q_bias, k_bias=k_bias, mask=None, causal=causal,
               softmax_scale=scale)
    out.update(extra)
    return out


def sweep(L, B=2, H=4, d=32, r=8, dtype=torch.bfloat16, seed=0, causal=False):
    """q, k, v ~ N(0,1); q_bias, k_bias ~ N(0,1)/sqrt(r); scale 1/sqrt(d); dO ~ N(0,1)."""
    g = torch.Generator().manual_seed(seed)
    q, k, v, do = _qkv(B, L, L, H, d, g, dtype)
    qb = (torch.randn(B, L, H, r, generator=g) / math.sqrt(r)).to(dtype)
    kb = (torch.randn(B, L, H, r, generator=g) / math.sqrt(r)).to(dtype)
    return _pack(q, k, v, do, qb, kb, causal, 1.0 / math.sqrt(d))


def masked(L, kind, B=2, H=4, dtype=torch.bfloat16, seed=0):
    """The sweep workload plus an additive mask: kind "vector" = (B, 1, 1, L) key-padding style,
    kind "matrix" = (1, H, L, L) per-head matrix broadcast over the batch."""
    w = sweep(L, B=B, H=H, dtype=dtype, seed=seed)
    g = torch.Generator().manual_seed(seed + 1)
    shape = (B, 1, 1, L) if kind == "vector" else (1, H, L, L)
    w["mask"] = torch.randn(*shape, generator=g).to(dtype)
    return w


def plumbing(seed=0):
    """fp32, non-causal, B2 H4 L1024 d32 r8 (CPU-runnable configuration)."""
    return sweep(1024, dtype=torch.float32, seed=seed)


def alibi(L, H=50, d=32, dtype=torch.bfloat16, seed=0, exact=False):
    """Causal LM with ALiBi as a rank-2 bias, B1 H50 d32: q_bias[i] = [-m_h i, 1], k_bias[j] =
    [1, m_h j], computed in fp32 and cast (the checker consumes the cast factors).  exact=True: the
    rank-4 factors that are exact in 16 bits (factors.alibi_factors)."""
    g = torch.Generator().manual_seed(seed)
    q, k, v, do = _qkv(1, L, L, H, d, g, dtype)
    qb, kb = factors.alibi_factors(L, L, H, dtype, exact=exact)
    return _pack(q, k, v, do, qb, kb, True, 1.0 / math.sqrt(d))


def swin(windows=4096, window=16, H=16, d=32, r=16, dtype=torch.bfloat16, seed=0, shifted_types=0):
    """Swin-V2 style windowed attention: `windows` windows of window^2 tokens, per-head bias
    table factored by truncated SVD and shared by all windows (broadcast over batch).
    shifted_types > 0 adds the additive mask of a shifted-window block the way the reference
    hands it to the operator (2_Vision_Transformer/swin_transformer_v2.py:171-173, :190-203):
    one 0 / -100 matrix per window type, repeated over the images into (windows, 1, n, n)."""
    g = torch.Generator().manual_seed(seed)
    n = window * window
    q, k, v, do = _qkv(windows, n, n, H, d, g, dtype)
    table = factors.swin_v2_bias_table(window, H, seed)
    qb, kb, rel = factors.svd_factors(table, r, dtype)
    w = _pack(q, k, v, do, qb, kb, False, 1.0 / math.sqrt(d), bias_table=table, bias_rel_error=rel)
    if shifted_types:
        assert windows % shifted_types == 0
        # tokens of a shifted window fall into up to four regions; pairs from different regions get -100
        region = torch.randint(0, 4, (shifted_types, n), generator=g)
        region[0] = 0  # (the unshifted interior windows see everything)
        m = (region[:, :, None] != region[:, None, :]).to(dtype) * -100.0
        w["mask"] = m.unsqueeze(1).unsqueeze(0).repeat(windows // shifted_types, 1, 1, 1, 1).reshape(windows, 1, n, n)
    return w


def pde(N=32768, H=8, d=32, alpha=10.0, dtype=torch.bfloat16, seed=0, pad_to=8):
    """Spatial-distance bias -alpha |x_i - x_j|^2 over N points in [0,1]^3, exact rank 5.  The factors'
    terms are at most 2 alpha in magnitude, so they are stored with three zero columns (rank 8,
    factors.pad_rank), which selects the rank-8 kernels; pad_to=None leaves them at rank 5."""
    g = torch.Generator().manual_seed(seed)
    q, k, v, do = _qkv(1, N, N, H, d, g, dtype)
    x = torch.rand(1, N, 3, generator=g)
    qb, kb = factors.distance_factors(x, x, alpha, dtype)
    if pad_to:
        qb, kb = factors.pad_rank(qb, kb, pad_to)
    return _pack(q, k, v, do, qb, kb, False, 1.0 / math.sqrt(d), points=x, rank=5)


def pairformer(N=768, H=4, d=32, r=32, dtype=torch.bfloat16, seed=0):
    """Pairformer-shaped triangle attention: N rows (kernel batch) each attending over N
    tokens, factors shared by all rows (broadcast over batch) as in
    4_AlphaFold3/protenix/openfold_local/model/primitives.py:639-640."""
    g = torch.Generator().manual_seed(seed)
    q, k, v, do = _qkv(N, N, N, H, d, g, dtype)
    qb = (torch.randn(1, N, H, r, generator=g) / math.sqrt(r)).to(dtype)
    kb = (torch.randn(1, N, H, r, generator=g) / math.sqrt(r)).to(dtype)
    return _pack(q, k, v, do, qb, kb, False, 1.0 / math.sqrt(d))


def flops(B, H, Lq, Lk, d, r, causal=False):
    """Algorithmic FLOPs (unpadded rank, one recompute of S in the backward, bias add not
    counted): fwd 2 B H P (2d + r), bwd 2 B H P (5d + 3r), P = visible (query, key) pairs."""
    if causal:
        pairs = sum(min(i + 1, Lk) for i in range(Lq)) if Lq != Lk else Lq * (Lq + 1) // 2
    else:
        pairs = Lq * Lk
    fwd = 2.0 * B * H * pairs * (2 * d + r)
    bwd = 2.0 * B * H * pairs * (5 * d + 3 * r)
    return fwd, bwd


def reference_formula_flops(B, H, L, d):
    """The reference's own count (flash_bias/benchmark.py:362-371): 4 B H L^2 d + B H L^2 for the
    forward, three times that for forward + backward; ignores the rank-r products."""
    fwd = 4.0 * B * H * L * L * d + B * H * L * L
    return fwd, 3.0 * fwd
