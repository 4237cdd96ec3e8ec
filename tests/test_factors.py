"""CPU tests of the factor builders and workload generators (closed forms and invariants)."""
import math

import pytest

import torch

from flashbias_amd import factors, workloads


def _dense(q_bias, k_bias):
    return q_bias.permute(0, 2, 1, 3).double() @ k_bias.permute(0, 2, 3, 1).double()


def test_alibi_slopes_and_factors_closed_form():
    """m_h = 2^(-8 (h+1) / H) (attention_with_alibi_bias.py:8-15); bias_ij = -m_h (i - j)."""
    for H in (4, 8, 50):
        m = factors.alibi_slopes(H).double()
        ref = torch.tensor([(2.0 ** 8) ** (-(h + 1) / H) for h in range(H)], dtype=torch.float64)
        assert torch.allclose(m, ref, rtol=1e-6)
    qb, kb = factors.alibi_factors(33, 47, 8)
    assert qb.shape == (1, 33, 8, 2) and kb.shape == (1, 47, 8, 2)
    i, j = torch.arange(33.0).double(), torch.arange(47.0).double()
    want = -factors.alibi_slopes(8).double()[:, None, None] * (i[:, None] - j[None, :])
    assert torch.allclose(_dense(qb, kb)[0], want, atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("reference_sign", [False, True])
def test_alibi_factors_exact_in_16_bits(dtype, reference_sign):
    """The rank-4 factors: the product of the 16-bit factors equals -m (i - j) exactly, with m the
    slope rounded to the dtype, at positions up to 8192 and beyond; the rank-2 closed form cast
    to 16 bits is off by units there (which is why the module does not use it)."""
    H, L = 8, 8192 + 300
    qb, kb = factors.alibi_factors(L, L, H, dtype, exact=True, reference_sign=reference_sign)
    assert qb.shape == (1, L, H, 4) and kb.shape == (1, L, H, 4) and qb.dtype == dtype
    m = factors.alibi_slopes(H).to(dtype).double()
    rows = torch.tensor([0, 1, 255, 256, 257, 1000, 4095, 4096, 8191, 8192, L - 1])
    got = torch.einsum("ihr,jhr->hij", qb[0, rows].double(), kb[0].double())
    sgn = 1.0 if reference_sign else -1.0
    want = sgn * m[:, None, None] * (rows.double()[None, :, None] - torch.arange(L).double()[None, None, :])
    assert torch.equal(got, want)
    # and in fp32 accumulation, which is what the kernels do
    got32 = torch.einsum("ihr,jhr->hij", qb[0, rows].float(), kb[0].float())
    assert torch.equal(got32.double(), want)
    true = sgn * factors.alibi_slopes(H).double()[:, None, None] * (rows.double()[None, :, None] - torch.arange(L).double()[None, None, :])
    ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    assert ((got - true).abs() <= ulp * true.abs() + 1e-12).all()
    # the cast rank-2 form, for comparison
    q2, k2 = factors.alibi_factors(L, L, H, dtype, reference_sign=reference_sign)
    err2 = (torch.einsum("ihr,jhr->hij", q2[0, rows].double(), k2[0].double()) - true).abs().max()
    assert err2 > 0.4


def test_distance_factors_identity():
    """-alpha |x_i - x_j|^2 = [-alpha|x_i|^2, -alpha, 2 alpha x_i] . [1, |x_j|^2, x_j], exact rank D+2."""
    g = torch.Generator().manual_seed(0)
    xq = torch.rand(2, 40, 3, generator=g, dtype=torch.float64)
    xk = torch.rand(2, 50, 3, generator=g, dtype=torch.float64)
    qb, kb = factors.distance_factors(xq, xk, 10.0, torch.float64)
    assert qb.shape == (2, 40, 1, 5) and kb.shape == (2, 50, 1, 5)
    want = -10.0 * torch.cdist(xq, xk) ** 2
    assert torch.allclose(_dense(qb, kb)[:, 0], want, atol=1e-12)


def test_svd_factors_are_eckart_young_optimal():
    g = torch.Generator().manual_seed(1)
    bias = torch.randn(3, 24, 24, generator=g, dtype=torch.float64)
    qb, kb, rel = factors.svd_factors(bias, 6, torch.float64)
    rec = _dense(qb, kb)[0]
    s = torch.linalg.svdvals(bias)
    tail = (s[:, 6:] ** 2).sum(-1).sqrt()
    assert torch.allclose((rec - bias).flatten(1).norm(dim=1), tail, rtol=1e-9)
    assert torch.allclose(rel.double(), tail / bias.flatten(1).norm(dim=1), rtol=1e-5)
    full_q, full_k, rel0 = factors.svd_factors(bias, 24, torch.float64)
    assert torch.allclose(_dense(full_q, full_k)[0], bias, atol=1e-10) and rel0.max() < 1e-6


def test_swin_table_structure():
    """Relative-position bias: depends on (dy, dx) only, lies in (0, 16), low effective rank."""
    t = factors.swin_v2_bias_table(8, 4, seed=3)
    assert t.shape == (4, 64, 64) and t.min() > 0 and t.max() < 16
    idx = lambda y, x: y * 8 + x
    assert torch.equal(t[:, idx(2, 3), idx(1, 1)], t[:, idx(5, 6), idx(4, 4)])  # same (dy, dx) = (1, 2)
    _, _, rel = factors.svd_factors(t, 16)
    assert rel.max() < 0.05


def test_workloads_are_seeded_and_shaped():
    a, b = workloads.sweep(256, seed=5), workloads.sweep(256, seed=5)
    assert all(torch.equal(a[n], b[n]) for n in ("q", "k", "v", "q_bias", "k_bias", "do"))
    assert a["q"].shape == (2, 256, 4, 32) and a["q_bias"].shape == (2, 256, 4, 8) and a["q"].dtype == torch.bfloat16
    assert abs(a["q_bias"].float().std().item() - 1 / math.sqrt(8)) < 0.02
    w = workloads.alibi(128, H=6)
    assert w["causal"] and w["q_bias"].shape == (1, 128, 6, 2)
    w = workloads.swin(windows=3, window=4, H=2, r=4)
    assert w["q"].shape == (3, 16, 2, 32) and w["q_bias"].shape == (1, 16, 2, 4)
    w = workloads.pde(N=64, H=2)  # rank 5, stored with three zero columns
    assert w["q_bias"].shape == (1, 64, 1, 8) and not w["q_bias"][..., 5:].any() and not w["k_bias"][..., 5:].any()
    w5 = workloads.pde(N=64, H=2, pad_to=None)
    assert w5["q_bias"].shape == (1, 64, 1, 5) and torch.equal(w5["q_bias"], w["q_bias"][..., :5])
    assert factors.pad_rank(w["q_bias"], w["k_bias"], 8)[0] is w["q_bias"]
    w = workloads.pairformer(N=16, H=2, r=8)
    assert w["q"].shape == (16, 16, 2, 32) and w["k_bias"].shape == (1, 16, 2, 8)


def test_flop_formulas():
    fwd, bwd = workloads.flops(2, 4, 16384, 16384, 32, 8)
    assert fwd == 2 * 2 * 4 * 16384 ** 2 * 72 and bwd == 2 * 2 * 4 * 16384 ** 2 * 184
    assert abs(fwd + bwd - 1.0995e12) < 1e9
    cf, _ = workloads.flops(1, 1, 100, 100, 32, 8, causal=True)
    assert cf == 2 * 5050 * 72
    rect, _ = workloads.flops(1, 1, 5, 3, 4, 0, causal=True)
    assert rect == 2 * (1 + 2 + 3 + 3 + 3) * 8
    rf, rfb = workloads.reference_formula_flops(2, 4, 16384, 32)
    assert abs(rf - 2.770e11) < 1e8 and rfb == 3 * rf


@pytest.mark.parametrize("r,bmask,hmask,bk,hk", [(8, True, False, False, False), (5, False, True, True, False),
                                                 (0, True, True, False, False), (16, False, False, True, True)])
def test_vector_mask_as_factor_column(r, bmask, hmask, bk, hk):
    """The wrapper's folding of a vector mask into the factors (1_i * mask_j as one more rank) is
    an identity of the oracle, -inf entries and all broadcast combinations included."""
    from _util import make_inputs, oracle
    from flashbias_amd.interface import _fold_vector_mask
    B, Lq, Lk, H = 2, 37, 53, 3
    q, k, v, qb, kb, do = make_inputs(B, Lq, Lk, H, 16, r, torch.float32, seed=5, bk=(bk, hk))
    g = torch.Generator().manual_seed(6)
    mask = torch.randn(B if bmask else 1, H if hmask else 1, 1, Lk, generator=g)
    mask[..., Lk - 9:] = float("-inf")
    mask[0, 0, 0, 3] = float("-inf")
    want = oracle(q, k, v, qb, kb, mask, False, None, do)
    qn, kn = _fold_vector_mask(q, qb, kb, mask)
    assert qn.shape[-1] == kn.shape[-1] == r + 1
    got = oracle(q, k, v, qn, kn, None, False, None, do)
    names = ("o", "lse", "dq", "dk", "dv")
    for name, a, b in zip(names, got[:5], want[:5]):
        assert torch.allclose(a, b, rtol=1e-5, atol=1e-5), name
    if r:
        # gradients of the original columns; broadcast dims of the folded key factor are summed
        dqb, dkb = got[5][..., :r], got[6][..., :r]
        assert torch.allclose(dqb, want[5], rtol=1e-4, atol=1e-5)
        red = [i for i in (0, 2) if kb.shape[i] == 1 and dkb.shape[i] != 1]
        if red:
            dkb = dkb.sum(dim=red, keepdim=True)
        assert torch.allclose(dkb, want[6], rtol=1e-4, atol=1e-5)
