"""The benchmark configurations at their stated sizes: ALiBi H50 L=8192, Swin-style 4096 windows
of 256 tokens, spatial-distance bias on 32768 points, Pairformer-shaped 768 x 768, and the middle
lengths of the B2 H4 d32 r8 sweep.  The HIP path runs once at full size; it is checked against
the oracle on what the oracle can afford: a subset of query rows against all keys on the CPU
(a query row depends on no other query), or everything, a batch chunk at a time, with the oracle's
own code evaluated in fp32 on the GPU by torch; plus the size-independent identities (rows of P
sum to one, rows of dS sum to zero)."""
import math

import pytest
import torch

from _util import GRAD_TOL, O_TOL, errors
from flashbias_amd import factors, flash_bias_func
from oracle import eager

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16


def _run(dev, q, k, v, qb, kb, mask, causal, scale, do):
    leaves = [t.detach().requires_grad_(True) for t in (q, k, v, qb, kb)]
    o = flash_bias_func(*leaves, mask, causal, scale)
    grads = torch.autograd.grad(o, leaves, do)
    torch.cuda.synchronize()
    return o.detach(), grads


def _checksums(do, grads):
    """sum_j dv_j = sum_i dO_i; sum_j dk_j = 0 (per batch and head), up to the rounding of the
    stored gradients and of the dS that went into them."""
    dv_sum, do_sum = grads[2].float().sum(1), do.float().sum(1)
    assert (dv_sum - do_sum).abs().max() <= 0.02 * do_sum.abs().max()
    gk = grads[1].float()
    bound = 16 * 2.0 ** -9 * gk.abs().sum(1).max() / math.sqrt(gk.shape[1])
    assert gk.sum(1).abs().max() <= bound


def _heads_on_gpu(q, k, v, qb, kb, causal, scale, do, chunk):
    """The eager oracle in fp32 on the GPU, `chunk` heads at a time (batch of one); factors shared by
    the heads get their gradients summed over all chunks."""
    outs = [torch.empty_like(t, dtype=torch.float32) for t in (q, q, k, v)]
    shared = qb.shape[2] == 1
    outs += [torch.zeros_like(t, dtype=torch.float32) for t in (qb, kb)]
    for h0 in range(0, q.shape[2], chunk):
        sl = lambda t: t[:, :, h0:h0 + chunk]
        fs = (lambda t: t) if shared else sl
        res = eager.flashbias_eager_grads(sl(q), sl(k), sl(v), fs(qb), fs(kb), None, causal, scale, sl(do))
        for dst, r in zip(outs[:4], res[:4]):
            dst[:, :, h0:h0 + chunk] = r
        for dst, r in zip(outs[4:], res[4:]):
            fs(dst).add_(r)
    return outs


@pytest.mark.parametrize("exact", [False, True])
def test_alibi_h50_l8192(gpu_device, exact):
    """Configuration 3 at its largest length, every output element against the oracle evaluated in fp32
    on the GPU.  Rank-2 factors as the configuration states them: o, dq, dk, dv, dk_bias (dq_bias of that
    form is ill-conditioned in any backward that consumes the stored 16-bit o, see test_workload_alibi);
    the rank-4 factors that are exact in 16 bits: dq_bias as well."""
    dev, L, H, d = gpu_device, 8192, 50, 32
    g = torch.Generator(device=dev).manual_seed(3)
    q, k, v, do = [torch.randn(1, L, H, d, device=dev, generator=g).to(BF16) for _ in range(4)]
    qb, kb = [t.to(dev) for t in factors.alibi_factors(L, L, H, BF16, exact=exact)]
    scale = 1.0 / math.sqrt(d)
    o, grads = _run(dev, q, k, v, qb, kb, None, True, scale, do)
    ref = _heads_on_gpu(q, k, v, qb, kb, True, scale, do, chunk=5)
    err, _ = errors(o.float(), ref[0])
    assert err <= O_TOL[BF16], err
    for name, got, want in zip(("dq", "dk", "dv", "dq_bias", "dk_bias"), grads, ref[1:]):
        _, rel = errors(got.float(), want)
        if name == "dq_bias" and not exact:
            continue
        assert rel <= GRAD_TOL, (name, rel)
    _checksums(do, grads)
    assert torch.equal(o[:, 0], v[:, 0])  # the first query sees one key
    ones = flash_bias_func(q, k, torch.ones_like(v), qb, kb, None, True, scale)
    assert (ones.float() - 1).abs().max() <= 2.0 ** -7


def _chunked_on_gpu(q, k, v, qb, kb, scale, do, chunk):
    """The eager oracle in fp32 on the GPU, `chunk` batch entries at a time; factors broadcast over
    the batch get their gradients summed over all chunks."""
    B = q.shape[0]
    o = torch.empty_like(q, dtype=torch.float32)
    dq, dk, dv = (torch.empty_like(t, dtype=torch.float32) for t in (q, k, v))
    shared = qb.shape[0] == 1
    dqb = torch.zeros_like(qb, dtype=torch.float32) if shared else torch.empty_like(qb, dtype=torch.float32)
    dkb = torch.zeros_like(kb, dtype=torch.float32) if shared else torch.empty_like(kb, dtype=torch.float32)
    for b0 in range(0, B, chunk):
        sl = slice(b0, min(b0 + chunk, B))
        fs = lambda t: t if t.shape[0] == 1 else t[sl]
        res = eager.flashbias_eager_grads(q[sl], k[sl], v[sl], fs(qb), fs(kb), None, False, scale, do[sl])
        o[sl], dq[sl], dk[sl], dv[sl] = res[0], res[1], res[2], res[3]
        if shared:
            dqb += res[4]
            dkb += res[5]
        else:
            dqb[sl], dkb[sl] = res[4], res[5]
    return o, dq, dk, dv, dqb, dkb


def _compare_all(o, grads, ref):
    err, _ = errors(o.float(), ref[0])
    assert err <= O_TOL[BF16], err
    for name, got, want in zip(("dq", "dk", "dv", "dq_bias", "dk_bias"), grads, ref[1:]):
        _, rel = errors(got.float(), want)
        assert rel <= GRAD_TOL, (name, rel)


def test_swin_4096_windows(gpu_device):
    """Configuration 4: 4096 windows of 16 x 16 tokens, H16 d32, rank-16 SVD factors of a relative
    position bias table shared by all windows; every output against the oracle."""
    dev, W, n, H, d, r = gpu_device, 4096, 256, 16, 32, 16
    g = torch.Generator(device=dev).manual_seed(4)
    q, k, v, do = [torch.randn(W, n, H, d, device=dev, generator=g).to(BF16) for _ in range(4)]
    table = factors.swin_v2_bias_table(16, H, seed=0)
    qb, kb, rel = factors.svd_factors(table, r, BF16)
    assert rel.max() < 0.05
    qb, kb = qb.to(dev), kb.to(dev)
    scale = 1.0 / math.sqrt(d)
    o, grads = _run(dev, q, k, v, qb, kb, None, False, scale, do)
    assert grads[3].shape == qb.shape and grads[4].shape == kb.shape
    ref = _chunked_on_gpu(q, k, v, qb, kb, scale, do, chunk=256)
    _compare_all(o, grads, ref)
    _checksums(do, grads)


@pytest.mark.parametrize("pad_to", [None, 8])
def test_pde_32768_points(gpu_device, pad_to):
    """Configuration 5a: -alpha |x_i - x_j|^2 on 32768 points as exact rank-5 factors shared by
    the 8 heads, as they are (the operator pads rank 5 to 16: general kernels) and padded to rank 8 by
    the caller (factors.pad_rank: the streamlined kernels); every output against the oracle."""
    dev, N, H, d = gpu_device, 32768, 8, 32
    g = torch.Generator(device=dev).manual_seed(5)
    q, k, v, do = [torch.randn(1, N, H, d, device=dev, generator=g).to(BF16) for _ in range(4)]
    x = torch.rand(1, N, 3, device=dev, generator=g)
    qb, kb = factors.distance_factors(x, x, 10.0, BF16)
    if pad_to:
        qb, kb = factors.pad_rank(qb, kb, pad_to)
    scale = 1.0 / math.sqrt(d)
    o, grads = _run(dev, q, k, v, qb, kb, None, False, scale, do)
    assert grads[3].shape == qb.shape
    ref = _heads_on_gpu(q, k, v, qb, kb, False, scale, do, chunk=1)
    _compare_all(o, grads, ref)
    _checksums(do, grads)


def test_pairformer_768(gpu_device):
    """Configuration 5b: 768 rows (the kernel's batch) attending over 768 tokens, H4 d32, rank-32
    factors shared by all rows; every output against the oracle."""
    dev, N, H, d, r = gpu_device, 768, 4, 32, 32
    g = torch.Generator(device=dev).manual_seed(6)
    q, k, v, do = [torch.randn(N, N, H, d, device=dev, generator=g).to(BF16) for _ in range(4)]
    qb, kb = [(torch.randn(1, N, H, r, device=dev, generator=g) / math.sqrt(r)).to(BF16) for _ in range(2)]
    scale = 1.0 / math.sqrt(d)
    o, grads = _run(dev, q, k, v, qb, kb, None, False, scale, do)
    ref = _chunked_on_gpu(q, k, v, qb, kb, scale, do, chunk=64)
    _compare_all(o, grads, ref)
    _checksums(do, grads)


@pytest.mark.parametrize("L", [2048, 4096, 8192, 16384])
def test_sweep_middle_lengths(gpu_device, L):
    """Configuration 2 from L=2048 up to the headline length (L=1024 is covered by the parity cases):
    every element of o and of the five gradients against the oracle."""
    dev, B, H, d, r = gpu_device, 2, 4, 32, 8
    g = torch.Generator(device=dev).manual_seed(L)
    q, k, v, do = [torch.randn(B, L, H, d, device=dev, generator=g).to(BF16) for _ in range(4)]
    qb, kb = [(torch.randn(B, L, H, r, device=dev, generator=g) / math.sqrt(r)).to(BF16) for _ in range(2)]
    scale = 1.0 / math.sqrt(d)
    o, grads = _run(dev, q, k, v, qb, kb, None, False, scale, do)
    ref = _chunked_on_gpu(q, k, v, qb, kb, scale, do, chunk=1)
    _compare_all(o, grads, ref)
    _checksums(do, grads)
