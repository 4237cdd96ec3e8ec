"""Pins the CPU oracle (oracle/eager.py, oracle/blocked.c) without the reference:
brute force on tiny shapes, library routines on special cases, closed forms and
invariants, each chosen so that a dropped term, a wrong sign/index or a transposed
operand fails at least one check."""
import math

import pytest
import torch

from oracle import blocked, eager

torch.set_num_threads(4)


def _inputs(B, Lq, Lk, H, d, r, seed=0, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Lq, H, d, generator=g, dtype=dtype)
    k = torch.randn(B, Lk, H, d, generator=g, dtype=dtype)
    v = torch.randn(B, Lk, H, d, generator=g, dtype=dtype)
    qb = torch.randn(B, Lq, H, r, generator=g, dtype=dtype) / math.sqrt(r) if r else None
    kb = torch.randn(B, Lk, H, r, generator=g, dtype=dtype) / math.sqrt(r) if r else None
    do = torch.randn(B, Lq, H, d, generator=g, dtype=dtype)
    return q, k, v, qb, kb, do


def _brute(q, k, v, qb, kb, mask, causal, scale):
    """Pure-Python loops: o[b,i,h,:] and lse[b,h,i]."""
    B, Lq, H, d = q.shape
    Lk = k.shape[1]
    o = torch.zeros(B, Lq, H, d, dtype=torch.float64)
    lse = torch.zeros(B, H, Lq, dtype=torch.float64)
    for b in range(B):
        for h in range(H):
            for i in range(Lq):
                logit = []
                for j in range(Lk):
                    if causal and j > i:
                        logit.append(-math.inf)
                        continue
                    s = scale * sum(float(q[b, i, h, c]) * float(k[b, j, h, c]) for c in range(d))
                    if qb is not None:
                        s += sum(float(qb[b, i, h, c]) * float(kb[b, j, h, c])
                                 for c in range(qb.shape[-1]))
                    if mask is not None:
                        s += float(mask.expand(B, H, Lq, Lk)[b, h, i, j])
                    logit.append(s)
                mx = max(logit)
                w = [math.exp(x - mx) for x in logit]
                z = sum(w)
                lse[b, h, i] = mx + math.log(z)
                for j in range(Lk):
                    o[b, i, h] += (w[j] / z) * v[b, j, h].double()
    return o, lse


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("Lq,Lk", [(5, 5), (4, 7), (7, 4)])
def test_eager_vs_brute_force(Lq, Lk, causal):
    if causal and Lq > Lk:
        pytest.skip("rows with no visible key are NaN in both (softmax of all -inf)")
    q, k, v, qb, kb, _ = _inputs(2, Lq, Lk, 2, 3, 2, seed=Lq * 10 + Lk)
    mask = torch.randn(2, 1, Lq, Lk, dtype=torch.float64)
    o, lse = eager.flashbias_eager(q, k, v, qb, kb, mask, causal, 0.7, dtype=torch.float64,
                                   return_lse=True)
    ob, lb = _brute(q, k, v, qb, kb, mask, causal, 0.7)
    assert torch.allclose(o, ob, atol=1e-12)
    assert torch.allclose(lse, lb, atol=1e-12)


def test_eager_zero_factors_is_sdpa():
    q, k, v, qb, kb, _ = _inputs(2, 33, 47, 3, 16, 4)
    o = eager.flashbias_eager(q, k, v, qb * 0, kb, None, False, None, dtype=torch.float64)
    ref = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2)).transpose(1, 2)
    assert torch.allclose(o, ref, atol=1e-12)
    o_none = eager.flashbias_eager(q, k, v, None, None, None, False, None, dtype=torch.float64)
    assert torch.allclose(o_none, ref, atol=1e-12)


@pytest.mark.parametrize("causal", [False, True])
def test_eager_concat_identity(causal):
    """attention_func.py:188-237: SDPA over [q*scale, q_bias] / [k, k_bias] with scale 1."""
    q, k, v, qb, kb, _ = _inputs(2, 40, 40, 3, 8, 5, seed=3)
    o = eager.flashbias_eager(q, k, v, qb, kb, None, causal, 0.3, dtype=torch.float64)
    ref = eager.flashbias_concat_sdpa(q, k, v, qb, kb, 0.3, causal)
    assert torch.allclose(o, ref, atol=1e-12)


def test_eager_ones_and_shift_invariance():
    q, k, v, qb, kb, _ = _inputs(1, 19, 23, 2, 8, 3, seed=5)
    o = eager.flashbias_eager(q, k, torch.ones_like(v), qb, kb, None, False, None,
                              dtype=torch.float64)
    assert torch.allclose(o, torch.ones_like(o), atol=1e-13)
    # bias_ij -> bias_ij + c_i leaves softmax rows unchanged, shifts lse by c_i
    c = torch.randn(1, 19, 2, 1, dtype=torch.float64)
    qb2 = torch.cat([qb, c], -1)
    kb2 = torch.cat([kb, torch.ones(1, 23, 2, 1, dtype=torch.float64)], -1)
    o1, l1 = eager.flashbias_eager(q, k, v, qb, kb, None, False, None, dtype=torch.float64,
                                   return_lse=True)
    o2, l2 = eager.flashbias_eager(q, k, v, qb2, kb2, None, False, None, dtype=torch.float64,
                                   return_lse=True)
    assert torch.allclose(o1, o2, atol=1e-12)
    assert torch.allclose(l2 - l1, c[..., 0].permute(0, 2, 1), atol=1e-12)


def test_eager_causal_structure():
    q, k, v, qb, kb, _ = _inputs(2, 12, 12, 2, 4, 2, seed=7, dtype=torch.float32)
    o = eager.flashbias_eager(q, k, v, qb, kb, None, True, None)
    assert torch.equal(o[:, 0], v[:, 0])  # a single visible key: softmax weight exactly 1
    k2, v2 = k.clone(), v.clone()
    k2[:, 7:] += 3.0
    v2[:, 7:] -= 5.0
    o2 = eager.flashbias_eager(q, k2, v2, qb, kb, None, True, None)
    assert torch.equal(o[:, :7], o2[:, :7])
    assert not torch.equal(o[:, 7:], o2[:, 7:])


def test_eager_broadcast_factors_and_mask_types():
    q, k, v, qb, kb, _ = _inputs(2, 9, 11, 3, 4, 2, seed=9)
    qb1, kb1 = qb[:1, :, :1], kb[:1]
    full = eager.flashbias_eager(q, k, v, qb1.expand(2, -1, 3, -1), kb1.expand(2, -1, -1, -1),
                                 None, False, None, dtype=torch.float64)
    bc = eager.flashbias_eager(q, k, v, qb1, kb1, None, False, None, dtype=torch.float64)
    assert torch.equal(full, bc)
    vec = torch.randn(2, 1, 1, 11, dtype=torch.float64)
    a = eager.flashbias_eager(q, k, v, qb, kb, vec, False, None, dtype=torch.float64)
    b = eager.flashbias_eager(q, k, v, qb, kb, vec.expand(2, 3, 9, 11), False, None,
                              dtype=torch.float64)
    assert torch.equal(a, b)
    ob, _ = _brute(q, k, v, qb, kb, vec, False, 0.5)
    assert torch.allclose(a, ob, atol=1e-12)


def _closed_form_grads(q, k, v, qb, kb, causal, scale, do):
    """dV = P^T dO, dP = dO V^T, dS = P*(dP - delta), dQ = scale dS K, dK = scale dS^T Q
    (flash_bias_triton.py:696-732); dq_bias = dS k_bias, dk_bias = dS^T q_bias
    (benchmark.py:76-77 with dBias = dS)."""
    B, Lq, H, d = q.shape
    bias = eager.materialize_bias(qb, kb, B, H)
    s = eager.logits(q, k, scale, bias, causal).permute(0, 2, 1, 3)  # (B,H,Lq,Lk)
    p = torch.softmax(s, -1)
    qh, kh, vh, doh = (t.permute(0, 2, 1, 3) for t in (q, k, v, do))
    dv = p.transpose(-1, -2) @ doh
    dp = doh @ vh.transpose(-1, -2)
    delta = (p * dp).sum(-1, keepdim=True)
    ds = p * (dp - delta)
    dq = scale * ds @ kh
    dk = scale * ds.transpose(-1, -2) @ qh
    dqb = ds @ kb.permute(0, 2, 1, 3)
    dkb = ds.transpose(-1, -2) @ qb.permute(0, 2, 1, 3)
    return [t.permute(0, 2, 1, 3) for t in (dq, dk, dv, dqb, dkb)], ds, delta


@pytest.mark.parametrize("causal", [False, True])
def test_eager_grads_closed_form(causal):
    q, k, v, qb, kb, do = _inputs(2, 14, 14, 2, 6, 3, seed=11)
    res = eager.flashbias_eager_grads(q, k, v, qb, kb, None, causal, 0.4, do,
                                      dtype=torch.float64)
    cf, ds, delta = _closed_form_grads(q, k, v, qb, kb, causal, 0.4, do)
    for got, want in zip(res[1:], cf):
        assert torch.allclose(got, want, atol=1e-11)
    assert ds.sum(-1).abs().max() < 1e-12  # rows of dS sum to zero
    o = res[0]
    assert torch.allclose(delta[..., 0], (o * do).sum(-1).permute(0, 2, 1), atol=1e-12)


def test_eager_grads_finite_differences():
    q, k, v, qb, kb, do = _inputs(1, 5, 6, 2, 3, 2, seed=13)
    res = eager.flashbias_eager_grads(q, k, v, qb, kb, None, False, 0.6, do,
                                      dtype=torch.float64)
    args = [q, k, v, qb, kb]
    eps = 1e-6
    for idx, g in enumerate(res[1:]):
        num = torch.zeros(g.numel(), dtype=g.dtype)
        flat = args[idx].reshape(-1)
        for e in range(flat.numel()):
            old = flat[e].item()
            flat[e] = old + eps
            fp = (eager.flashbias_eager(*args, None, False, 0.6, dtype=torch.float64) * do).sum()
            flat[e] = old - eps
            fm = (eager.flashbias_eager(*args, None, False, 0.6, dtype=torch.float64) * do).sum()
            flat[e] = old
            num[e] = (fp - fm) / (2 * eps)
        assert torch.allclose(g, num.view(g.shape), atol=1e-7), idx


def test_eager_grads_reduce_over_broadcast_dims():
    q, k, v, qb, kb, do = _inputs(2, 8, 8, 3, 4, 2, seed=15)
    qb1, kb1 = qb[:1], kb[:, :, :1]
    full = eager.flashbias_eager_grads(q, k, v, qb1.expand(2, -1, -1, -1).contiguous(),
                                       kb1.expand(-1, -1, 3, -1).contiguous(), None, False, None,
                                       do, dtype=torch.float64)
    bc = eager.flashbias_eager_grads(q, k, v, qb1, kb1, None, False, None, do,
                                     dtype=torch.float64)
    assert bc[4].shape == qb1.shape and bc[5].shape == kb1.shape
    assert torch.allclose(bc[4], full[4].sum(0, keepdim=True), atol=1e-12)
    assert torch.allclose(bc[5], full[5].sum(2, keepdim=True), atol=1e-12)


def test_eager_sliced_equals_full():
    q, k, v, qb, kb, do = _inputs(2, 10, 13, 2, 4, 3, seed=17, dtype=torch.float32)
    full = eager.flashbias_eager_grads(q, k, v, qb, kb, None, False, None, do)
    sl = eager.flashbias_eager_sliced(q, k, v, qb, kb, None, False, None, do)
    for a, b in zip(full, sl):
        assert torch.allclose(a, b, atol=1e-6)


@pytest.mark.parametrize("causal", [False, True])
def test_backward_from_stored_results(causal):
    """The closed-form backward from stored (o, lse): without rounding it is autograd through
    the eager path (also with broadcast factors and a mask); with the reference's two bf16
    roundings it stays within the usual gradient tolerance on well-conditioned inputs."""
    q, k, v, qb, kb, do = _inputs(2, 21, 21, 3, 8, 4, seed=31)
    qb, kb = qb[:1], kb[:, :, :1]
    mask = torch.randn(2, 1, 1, 21, dtype=torch.float64)
    auto = eager.flashbias_eager_grads(q, k, v, qb, kb, mask, causal, 0.35, do, dtype=torch.float64)
    o, lse = eager.flashbias_eager(q, k, v, qb, kb, mask, causal, 0.35, dtype=torch.float64,
                                   return_lse=True)
    exact = eager.flashbias_backward_stored(q, k, v, qb, kb, mask, causal, 0.35, o, lse, do,
                                            dtype=torch.float64)
    for a, b in zip(exact, auto[1:]):
        assert a.shape == b.shape and torch.allclose(a, b, atol=1e-11)
    rounded = eager.flashbias_backward_stored(q, k, v, qb, kb, mask, causal, 0.35, o, lse, do,
                                              round_dtype=torch.bfloat16, dtype=torch.float64)
    for a, b in zip(rounded, auto[1:]):
        assert not torch.equal(a, b)
        assert (a - b).abs().max() <= 2e-2 * b.abs().max()


# --------------------------------------------------------------------------- blocked C
def _check_blocked(B, Lq, Lk, H, d, r, causal, mask_kind, bm, bn, seed, bq=False, bk=False):
    q, k, v, qb, kb, do = _inputs(B, Lq, Lk, H, d, r, seed=seed, dtype=torch.float32)
    if bq:
        qb = qb[:1]
    if bk:
        kb = kb[:, :, :1]
    mask = None
    if mask_kind == "vector":
        mask = torch.randn(B, 1, 1, Lk)
    elif mask_kind == "matrix":
        mask = torch.randn(1, H, Lq, Lk)
    o, lse = blocked.blocked_fwd(q, k, v, qb, kb, mask, causal, None, bm, bn)
    ref = eager.flashbias_eager_grads(q, k, v, qb, kb, mask, causal, None, do,
                                      dtype=torch.float64)
    _, lse_ref = eager.flashbias_eager(q, k, v, qb, kb, mask, causal, None, dtype=torch.float64,
                                       return_lse=True)
    assert (o - ref[0]).abs().max() < 2e-5
    assert (lse - lse_ref).abs().max() < 2e-5
    grads = blocked.blocked_bwd(q, k, v, qb, kb, mask, causal, None, o, lse, do, bm, bn)
    for got, want in zip(grads, ref[1:]):
        if want is None:
            assert got is None
            continue
        assert got.shape == want.shape
        assert (got - want).abs().max() <= 5e-5 * max(1.0, want.abs().max().item())


def test_blocked_plumbing_config():
    """The CPU-runnable configuration of the benchmark: fp32, non-causal, B2 H4 L1024 d32 r8."""
    _check_blocked(2, 1024, 1024, 4, 32, 8, False, None, 128, 128, seed=0)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("mask_kind", [None, "vector", "matrix"])
def test_blocked_ragged(causal, mask_kind):
    _check_blocked(2, 75, 117, 3, 40, 5, causal, mask_kind, 32, 64, seed=21)


def test_blocked_broadcast_factors_and_no_bias():
    _check_blocked(2, 50, 50, 3, 16, 4, True, None, 16, 16, seed=23, bq=True, bk=True)
    _check_blocked(1, 33, 65, 2, 24, 0, False, None, 64, 32, seed=25)


def test_c_oracle_is_clean_under_sanitizers():
    """oracle/blocked.c rebuilt with -fsanitize=address,undefined and run on ragged, rectangular,
    causal, masked and broadcast shapes with exactly sized buffers (oracle/sanitize_check.c)."""
    import os
    import subprocess
    odir = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle")
    subprocess.check_call(["make", "-C", odir, "sanitize"], stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:verify_asan_link_order=0")
    res = subprocess.run([os.path.join(odir, "_sanitize", "sanitize_check")], capture_output=True, text=True, env=env)
    assert res.returncode == 0, res.stderr[-2000:]
    assert "clean" in res.stdout
