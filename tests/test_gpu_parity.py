"""GPU parity tests: the HIP path, called through the C ABI by ``flash_bias_func``, against
the CPU oracle on the same seeded, dtype-rounded inputs.

Tolerances (the gate of the headline metric): max-abs error of o <= 1e-2 (fp16) / 2e-2 (bf16);
for each of dq, dk, dv, dq_bias, dk_bias: max|err| / max|ref| <= 5e-2; causal structure exact.
"""
import math
import os

import pytest
import torch

from _util import GRAD_TOL, O_TOL, errors, make_inputs, oracle, run_gpu
from flashbias_amd import flash_bias_func, workloads

pytestmark = pytest.mark.gpu
NAMES = ("o", "dq", "dk", "dv", "dq_bias", "dk_bias")


def _gate(got, ref, dtype, skip=(), o_by_magnitude=False):
    """o_by_magnitude: the tolerance on o (an absolute one, stated for benchmark-like inputs whose outputs stay
    below 2) grows with max|o| beyond 2: under a peaked softmax o is close to single rows of v, |o| reaches 4-5,
    and rounding the output to bf16 alone costs up to 2^-6 there."""
    refs = [ref[0]] + list(ref[2:])
    for name, g, w in zip(NAMES, got, refs):
        if w is None:
            assert g is None
            continue
        assert g.shape == w.shape, name
        assert torch.isfinite(g).all(), name
        err, rel = errors(g, w)
        if name == "o":
            tol = O_TOL[dtype] * (max(1.0, float(w.abs().max()) / 2.0) if o_by_magnitude else 1.0)
            assert err <= tol, (name, err, tol)
        elif w.abs().max() == 0:  # e.g. a single visible key: dS is identically zero in exact arithmetic; here it is
            # dP - delta, two fp32 sums of the same products in different orders, summed over the queries
            assert err <= 1e-4, (name, err)
        elif name not in skip:
            assert rel <= GRAD_TOL, (name, err, rel)


def _case(gpu_device, B, Lq, Lk, H, d, r, dtype, causal, mask=None, scale=None, seed=1, o_by_magnitude=False, **bc):
    q, k, v, qb, kb, do = make_inputs(B, Lq, Lk, H, d, r, dtype, seed=seed, **bc)
    ref = oracle(q, k, v, qb, kb, mask, causal, scale, do)
    got = run_gpu(flash_bias_func, q, k, v, qb, kb, mask, causal, scale, do, gpu_device)
    _gate(got, ref, dtype, o_by_magnitude=o_by_magnitude)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("causal", [False, True])
def test_benchmark_shape_family(gpu_device, dtype, causal):
    """B2 H4 d32 r8 of flash_bias/config.py:12 at L=1024 (also the reference's own
    correctness shape family, flash_bias/benchmark.py:31)."""
    _case(gpu_device, 2, 1024, 1024, 4, 32, 8, dtype, causal)


def test_reference_correctness_script_shape(gpu_device):
    """flash_bias/benchmark.py:27-47,65: B1 L1024 H2 d32 r8 fp16, factors ~ N(0,1) (not scaled),
    upstream gradient of loss = -o.sum()."""
    g = torch.Generator().manual_seed(0)
    q, k, v = [torch.randn(1, 1024, 2, 32, generator=g).half() for _ in range(3)]
    qb, kb = [torch.randn(1, 1024, 2, 8, generator=g).half() for _ in range(2)]
    do = -torch.ones(1, 1024, 2, 32).half()
    ref = oracle(q, k, v, qb, kb, None, False, 1 / math.sqrt(32), do)
    got = run_gpu(flash_bias_func, q, k, v, qb, kb, None, False, 1 / math.sqrt(32), do, gpu_device)
    _gate(got, ref, torch.float16)


@pytest.mark.parametrize("d", [16, 32, 40, 64, 128])
@pytest.mark.parametrize("causal", [False, True])
def test_head_dims(gpu_device, d, causal):
    _case(gpu_device, 1, 200, 200, 2, d, 8, torch.bfloat16, causal)


@pytest.mark.parametrize("r", [0, 2, 5, 8, 16, 32, 96])
def test_ranks(gpu_device, r):
    _case(gpu_device, 1, 160, 224, 2, 32, r, torch.bfloat16, False)


@pytest.mark.parametrize("d,r", [(64, 64), (128, 64), (64, 128), (16, 128), (128, 128), (72, 24), (128, 8), (96, 32),
                                 (128, 0)])
@pytest.mark.parametrize("causal", [False, True])
def test_large_head_dim_and_rank_together(gpu_device, d, r, causal):
    """Instantiations with many contraction steps: their register budget, LDS footprint, (head dim
    128) multi-pass dk/dv and (head dims above 64, rank <= 32) 32-key tiles in the dq kernel differ
    from the small configurations."""
    _case(gpu_device, 2, 333, 401, 2, d, r, torch.bfloat16, causal, seed=17)


@pytest.mark.parametrize("d,r,scale", [(32, 8, None), (32, 8, 0.25), (32, 8, 0.29), (32, 8, 3.0), (64, 16, None),
                                       (64, 32, 0.5), (64, 24, 0.3), (128, 8, None), (32, 0, None), (32, 0, 0.7),
                                       (32, 8, -0.2), (64, 0, -0.125), (32, 8, 1.0), (32, 16, 1.0), (64, 32, 1.0),
                                       (128, 8, 1.0)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_scale_folded_into_the_contraction(gpu_device, d, r, scale, dtype):
    """Where it is exact (no factors; a scale of exactly 1, which leaves the factors as they are,
    for both element types; bf16 factors with a power-of-two scale or r <= 8) the kernels
    compute scale * (q k^T + (q_b / scale) k_b^T) in one MFMA chain; elsewhere (fp16 factors, other
    scales at larger ranks, scales <= 0, and loops shorter than 512 with factors) they scale the
    fp32 q k^T product.  Both against the oracle, with factors large enough (bias entries
    ~ N(0, 10^2)) that the bias dominates."""
    B, Lq, Lk, H = 2, 530, 600, 2
    q, k, v, qb, kb, do = make_inputs(B, Lq, Lk, H, d, r, dtype, seed=23)
    if r:
        qb = (qb.float() * 10.0 * math.sqrt(r)).to(dtype)  # entries of q_b k_b^T: std 1 / sqrt(r) before
    for causal in (False, True):
        ref = oracle(q, k, v, qb, kb, None, causal, scale, do)
        got = run_gpu(flash_bias_func, q, k, v, qb, kb, None, causal, scale, do, gpu_device)
        _gate(got, ref, dtype)


@pytest.mark.parametrize("scale", [None, 0.25, 0.29, 0.3, 1.0])
def test_infinite_factor_column(gpu_device, scale):
    """A key-padding column in the factors themselves (q_b column of ones against a k_b column of
    0 / -inf): with the scale folded into q_b or k_b as high and low parts, both parts must give
    the same infinity (scales whose reciprocal rounds up, rounds down, and is exact in bf16)."""
    B, Lq, Lk, H, d, r = 2, 520, 584, 2, 32, 8
    q, k, v, qb, kb, do = make_inputs(B, Lq, Lk, H, d, r, torch.bfloat16, seed=29)
    qb[..., r - 1] = 1.0
    kb[..., r - 1] = 0.0
    kb[:, Lk - 70:, :, r - 1] = float("-inf")
    kb[0, 3, :, r - 1] = float("-inf")
    ref = oracle(q, k, v, qb, kb, None, False, scale, do)
    got = run_gpu(flash_bias_func, q, k, v, qb, kb, None, False, scale, do, gpu_device)
    # the gradient of that q_b column is a sum with 0 * inf terms in any arithmetic: compare the rest
    for name, g, w in zip(NAMES, got, [ref[0]] + list(ref[2:])):
        if name == "dq_bias":
            g, w = g[..., :r - 1], w[..., :r - 1]
        assert torch.isfinite(g).all(), name
        err, rel = errors(g, w)
        assert (err <= O_TOL[torch.bfloat16]) if name == "o" else (rel <= GRAD_TOL), (name, err, rel)


@pytest.mark.parametrize("Lq,Lk", [(1, 1), (1, 257), (75, 117), (117, 75), (129, 64), (64, 129), (255, 255)])
@pytest.mark.parametrize("causal", [False, True])
def test_ragged_lengths(gpu_device, Lq, Lk, causal):
    _case(gpu_device, 2, Lq, Lk, 3, 40, 5, torch.float16, causal)


def test_odd_head_dim_and_unaligned_rank(gpu_device):
    """d and r that are not multiples of 8: rows are not 16-byte aligned, the element-wise
    load path is used."""
    _case(gpu_device, 2, 90, 70, 2, 20, 3, torch.bfloat16, True)
    _case(gpu_device, 1, 130, 130, 3, 100, 7, torch.float16, False)


@pytest.mark.parametrize("bq,bk", [((True, False), (True, False)), ((True, True), (False, True)),
                                   ((False, True), (True, True))])
def test_broadcast_factors(gpu_device, bq, bk):
    """Factors shared over batch and/or heads (stride 0); their gradients are summed over the
    shared dims, which is what autograd through the eager path gives."""
    _case(gpu_device, 3, 100, 140, 4, 32, 16, torch.bfloat16, False, bq=bq, bk=bk)


@pytest.mark.parametrize("kind", ["vector", "matrix", "matrix_bcast", "vector_f32"])
@pytest.mark.parametrize("causal", [False, True])
def test_additive_mask(gpu_device, kind, causal):
    B, Lq, Lk, H = 2, 96, 150, 3
    g = torch.Generator().manual_seed(5)
    if kind == "vector":
        mask = torch.randn(B, 1, 1, Lk, generator=g).bfloat16()
    elif kind == "vector_f32":
        mask = torch.randn(B, H, 1, Lk, generator=g)
    elif kind == "matrix":
        mask = torch.randn(B, H, Lq, Lk, generator=g).bfloat16()
    else:  # the Swin shifted-window form: 0 / -100 per (window, 1, N, N)
        mask = (torch.rand(B, 1, Lq, Lk, generator=g) < 0.3).float() * -100.0
    _case(gpu_device, B, Lq, Lk, H, 32, 8, torch.bfloat16, causal, mask=mask)


@pytest.mark.parametrize("r,bmask,hmask,bk", [(8, True, False, (False, False)), (16, False, True, (True, False)),
                                              (0, True, True, (False, False)), (8, False, False, (True, True))])
def test_vector_mask_folded_into_factors(gpu_device, monkeypatch, r, bmask, hmask, bk):
    """On large problems the wrapper passes a vector mask of the input dtype to the kernels as
    one more factor column (forced here at a small size); key-padding style -inf entries, all
    broadcast combinations of mask and key factor, and no factors at all."""
    from flashbias_amd import interface
    monkeypatch.setattr(interface, "_FOLD_MIN_PAIRS", 0)
    B, Lq, Lk, H = 2, 300, 520, 4
    q, k, v, qb, kb, do = make_inputs(B, Lq, Lk, H, 32, r, torch.bfloat16, seed=31, bk=bk)
    g = torch.Generator().manual_seed(32)
    mask = torch.randn(B if bmask else 1, H if hmask else 1, 1, Lk, generator=g).bfloat16()
    mask[..., Lk - 100:] = float("-inf")
    mask[0, 0, 0, 5] = float("-inf")
    ref = oracle(q, k, v, qb, kb, mask, False, None, do)
    got = run_gpu(flash_bias_func, q, k, v, qb, kb, mask, False, None, do, gpu_device)
    _gate(got, ref, torch.bfloat16)
    # the same call through the kernels' own mask path
    monkeypatch.setattr(interface, "_FOLD_MIN_PAIRS", 1 << 62)
    got2 = run_gpu(flash_bias_func, q, k, v, qb, kb, mask, False, None, do, gpu_device)
    _gate(got2, ref, torch.bfloat16)


def test_very_long_sequence_properties(gpu_device):
    """L = 65536 (too long for the dense oracle): the first 1024 rows of a causal problem do not
    depend on anything behind them, so they must equal the L = 1024 result of the same inputs
    (forward and all gradients restricted to that prefix when dO is zero elsewhere); with v = 1
    every output is 1."""
    B, L, H, d, r, P = 1, 65536, 2, 32, 8, 1024
    q, k, v, qb, kb, do = make_inputs(B, L, L, H, d, r, torch.bfloat16, seed=41)
    do[:, P:] = 0
    full = run_gpu(flash_bias_func, q, k, v, qb, kb, None, True, None, do, gpu_device)
    head = run_gpu(flash_bias_func, q[:, :P], k[:, :P], v[:, :P], qb[:, :P], kb[:, :P], None, True, None, do[:, :P],
                   gpu_device)
    for name, a, b in zip(NAMES, full, head):
        a = a[:, :P]
        assert torch.isfinite(a).all(), name
        err, rel = errors(a, b)
        assert rel <= 2e-2, (name, err, rel)  # same arithmetic, different tile sizes and summation order
    for name, a in zip(NAMES[2:], full[2:]):  # keys past the prefix receive no gradient
        if name in ("dk", "dv", "dk_bias"):
            assert a[:, P:].abs().max() == 0, name
    dev = gpu_device
    o = flash_bias_func(q.to(dev), k.to(dev), torch.ones_like(v).to(dev), qb.to(dev), kb.to(dev), None, False, None)
    assert (o.float() - 1).abs().max().item() <= 1e-2


def test_noncontiguous_inputs_and_scale(gpu_device):
    """q, k, v as strided views of a packed qkv projection, as the application modules create
    them; non-default softmax scale."""
    B, L, H, d, r = 2, 130, 4, 32, 8
    g = torch.Generator().manual_seed(9)
    qkv = torch.randn(B, L, 3, H, d, generator=g).bfloat16()
    q, k, v = qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2]
    qb = (torch.randn(B, H, L, r, generator=g) / math.sqrt(r)).bfloat16().permute(0, 2, 1, 3)
    kb = (torch.randn(B, H, L, r, generator=g) / math.sqrt(r)).bfloat16().permute(0, 2, 1, 3)
    do = torch.randn(B, L, H, d, generator=g).bfloat16()
    ref = oracle(q, k, v, qb, kb, None, False, 0.3, do)
    dev = gpu_device
    qkv_d = qkv.to(dev).requires_grad_(True)
    qb_d = qb.to(dev).requires_grad_(True)  # keeps the permuted strides
    kb_d = kb.to(dev).requires_grad_(True)
    assert qb_d.stride(-1) == 1 and not qb_d.is_contiguous()
    o = flash_bias_func(qkv_d[:, :, 0], qkv_d[:, :, 1], qkv_d[:, :, 2], qb_d, kb_d, None, False, 0.3)
    gqkv, gqb, gkb = torch.autograd.grad(o, [qkv_d, qb_d, kb_d], do.to(dev))
    got = [o.detach().float().cpu(), gqkv[:, :, 0].float().cpu(), gqkv[:, :, 1].float().cpu(),
           gqkv[:, :, 2].float().cpu(), gqb.float().cpu(), gkb.float().cpu()]
    _gate(got, ref, torch.bfloat16)


@pytest.mark.parametrize("stride", [(1 << 24) - 8, 1 << 24])
def test_huge_row_strides(gpu_device, stride):
    """Rows 32 MB apart: just below the limit the tile loaders keep their 32-bit offsets, at the
    limit the kernels must take the element-wise path (64-bit addresses)."""
    B, L, H, d, r = 1, 5, 1, 32, 8
    q, k, v, qb, kb, do = make_inputs(B, L, L, H, d, r, torch.bfloat16, seed=21)
    ref = oracle(q, k, v, qb, kb, None, False, None, do)
    dev = gpu_device

    def spread(t):  # the same values in rows `stride` elements apart
        buf = torch.zeros(L * stride, dtype=t.dtype, device=dev)
        view = buf.as_strided(t.shape, (L * stride, stride, t.shape[-1], 1))
        view.copy_(t.to(dev))
        return view.detach().requires_grad_(True)

    leaves = [spread(t) for t in (q, k, v, qb, kb)]
    assert leaves[0].stride(1) == stride
    o = flash_bias_func(*leaves, None, False, None)
    grads = torch.autograd.grad(o, leaves, spread(do).detach())
    got = [o.detach().float().cpu()] + [g.float().cpu() for g in grads]
    _gate(got, ref, torch.bfloat16)


def test_lse_and_default_scale(gpu_device):
    from flashbias_amd.interface import _flash_bias_forward
    q, k, v, qb, kb, do = make_inputs(2, 300, 260, 2, 64, 8, torch.bfloat16, seed=3)
    ref = oracle(q, k, v, qb, kb, None, True, None, do)
    dev = gpu_device
    o, lse, scale = _flash_bias_forward(q.to(dev), k.to(dev), v.to(dev), qb.to(dev), kb.to(dev), None, True, None)
    assert scale == pytest.approx(1 / 8)
    assert lse.shape == (2, 2, 300) and lse.dtype == torch.float32
    assert (lse.cpu() - ref[1]).abs().max() < 2e-3
    o0, _, scale0 = _flash_bias_forward(q.to(dev), k.to(dev), v.to(dev), qb.to(dev), kb.to(dev), None, True, 0)
    assert scale0 == scale and torch.equal(o0, o)  # 0 falls back to the default like `or` does


@pytest.mark.parametrize("B,L,H,d,r", [
    (2, 333, 3, 32, 8),     # small grid: the streamlined causal forward (one query block per wave)
    (8, 700, 16, 32, 8),    # the same on a grid that fills the chip, several key tiles
    (4, 1100, 8, 32, 0),    # ... without factors
    (2, 333, 3, 32, 16),    # the general forward
    (2, 400, 2, 64, 8)])
def test_causal_structure_is_exact(gpu_device, B, L, H, d, r):
    """o[:, 0] == v[:, 0] bit for bit, and changing k / v / k_bias at keys j > i leaves o[i]
    bit-identical (top-left aligned causal mask, flash_bias_triton.py:262)."""
    dev = gpu_device
    q, k, v, qb, kb, _ = [t.to(dev) if t is not None else None
                          for t in make_inputs(B, L, L, H, d, r, torch.bfloat16, seed=4)]
    o = flash_bias_func(q, k, v, qb, kb, None, True, None)
    assert torch.equal(o[:, 0], v[:, 0])
    for cut in (1, 64, 65, 200, L - 1):
        k2, v2 = k.clone(), v.clone()
        kb2 = kb.clone() if r else None
        k2[:, cut:] += 3
        v2[:, cut:] -= 5
        if r:
            kb2[:, cut:] *= -2
        o2 = flash_bias_func(q, k2, v2, qb, kb2, None, True, None)
        assert torch.equal(o[:, :cut], o2[:, :cut]), cut
        assert not torch.equal(o[:, cut:], o2[:, cut:]), cut


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,n,pitch", [(1, 8, 8), (37, 200, 200), (300, 64 * 5, 64 * 5 + 24), (4096, 1024, 1024)])
def test_sum_over_batch_entry_point(gpu_device, dtype, B, n, pitch):
    """fb_sum_over_batch against a float64 sum of the same 16-bit values: fp32 output to fp32
    accuracy, 16-bit output to its rounding; the same bits on a second run."""
    from flashbias_amd import _lib
    from flashbias_amd.interface import _dtype_code, _stream
    lib = _lib.load()
    g = torch.Generator(device=gpu_device).manual_seed(B)
    store = torch.randn(B, pitch, device=gpu_device, generator=g).to(dtype)
    want = store[:, :n].double().sum(0)
    code = _dtype_code(dtype)
    outs = []
    for out_dtype in (torch.float32, dtype, dtype):
        out = torch.full((n + 8,), 7.0, device=gpu_device, dtype=out_dtype)
        _lib.check_status(lib.fb_sum_over_batch(store.data_ptr(), out.data_ptr(), code, _dtype_code(out_dtype), B, n,
                                                pitch, _stream()))
        torch.cuda.synchronize()
        assert (out[n:] == 7).all()  # nothing written past the row
        outs.append(out[:n])
    scale = max(want.abs().max().item(), 1.0)
    assert (outs[0].double() - want).abs().max() <= 1e-5 * scale
    assert (outs[1].double() - want).abs().max() <= 2.0 ** -8 * scale
    assert torch.equal(outs[1], outs[2])


@pytest.mark.parametrize("case", ["plain", "rank5_shared_by_heads", "shared_by_batch_vector_mask", "matrix_mask_no_factors",
                                  "constant_factors", "constant_factors_streamlined", "grouped_gradients",
                                  "factors_expanded_by_the_caller"])
def test_cpp_and_python_autograd_functions_agree(gpu_device, case):
    """flash_bias_func runs the autograd function in C++ (flashbias_amd/_fb_torch.so) when that is
    built; FlashBiasFunc is the same in Python.  Same library calls, so the same bits, for the output
    and every gradient: also when the factors ask for no gradient (the library then skips them), when the
    kernels sum the factor gradients over groups of batch entries, and when a caller expands shared factors
    over the batch itself (batch stride 0 in a full-shape tensor: no groups, autograd sums the expansion)."""
    from flashbias_amd import FlashBiasFunc, interface
    assert interface._extension() is not None, "flashbias_amd/_fb_torch.so is not built"
    dev, dt = gpu_device, torch.bfloat16
    B, L, H, d = 3, 200, 4, 32
    if case in ("grouped_gradients", "factors_expanded_by_the_caller"):
        B, L, H = 48, 256, 16
    if case == "constant_factors_streamlined":
        B, L, H = 2, 1024, 4
    g = torch.Generator().manual_seed(21)
    q, k, v, do = [torch.randn(B, L, H, d, generator=g).to(dt).to(dev) for _ in range(4)]
    qb = kb = mask = None
    expand = lambda t: t
    if case in ("plain", "constant_factors", "constant_factors_streamlined"):
        qb, kb = [(torch.randn(B, L, H, 8, generator=g) / 3).to(dt).to(dev) for _ in range(2)]
    elif case == "rank5_shared_by_heads":
        qb, kb = [(torch.randn(B, L, 1, 5, generator=g) / 2).to(dt).to(dev) for _ in range(2)]
    elif case in ("shared_by_batch_vector_mask", "grouped_gradients", "factors_expanded_by_the_caller"):
        qb, kb = [(torch.randn(1, L, H, 16, generator=g) / 4).to(dt).to(dev) for _ in range(2)]
        if case == "shared_by_batch_vector_mask":
            mask = torch.zeros(B, 1, 1, L, dtype=dt).masked_fill(torch.rand(B, 1, 1, L, generator=g) < 0.2, float("-inf")).to(dev)
        if case == "factors_expanded_by_the_caller":
            expand = lambda t: t.expand(B, -1, -1, -1)
    else:
        mask = torch.randn(1, H, L, L, generator=g).to(dt).to(dev)
    wants_factor_grads = not case.startswith("constant_factors")
    outs = []
    for fn in (flash_bias_func, FlashBiasFunc.apply):
        leaves = [t.clone().requires_grad_(True) for t in (q, k, v)]
        bias = [None, None]
        if qb is not None:
            bias = [t.clone().requires_grad_(wants_factor_grads) for t in (qb, kb)]
            if wants_factor_grads:
                leaves += bias
        o = fn(leaves[0], leaves[1], leaves[2], expand(bias[0]), expand(bias[1]), mask, case == "plain", None)
        outs.append([o.detach()] + list(torch.autograd.grad(o, leaves, do)))
    for a, b in zip(*outs):
        assert a.shape == b.shape and torch.equal(a, b)
    if case == "factors_expanded_by_the_caller":
        # the gradient of the un-expanded factors is the same sum over the batch whoever forms it (the kernels in
        # groups plus the library's reduction, or autograd's expand backward over the full-shape gradient)
        assert outs[0][4].shape == qb.shape and outs[0][5].shape == kb.shape
        leaves = [t.clone().requires_grad_(True) for t in (q, k, v, qb, kb)]
        o = flash_bias_func(*leaves, None, False, None)
        for a, b in zip(outs[0][4:], torch.autograd.grad(o, leaves, do)[3:]):
            assert (a.float() - b.float()).abs().max() <= 2.0 ** -6 * b.float().abs().max()


def test_mask_gradient_is_refused_in_backward_only(gpu_device):
    """As the reference (flash_bias_triton.py:1371): a mask that requires a gradient is accepted by the forward
    (inference, no_grad) and refused when the backward is asked for it; the same in the C++ and the Python
    autograd function."""
    from flashbias_amd import FlashBiasFunc
    dev, dt = gpu_device, torch.bfloat16
    q, k, v, qb, kb, do = [t.to(dev) for t in make_inputs(1, 64, 64, 2, 32, 8, dt, seed=3)]
    mask = torch.zeros(1, 2, 64, 64, device=dev, dtype=dt, requires_grad=True)
    for fn in (flash_bias_func, FlashBiasFunc.apply):
        for fa, fb_ in ((qb, kb), (None, None)):
            with torch.no_grad():
                want = fn(q, k, v, fa, fb_, mask.detach(), False, None)
                assert torch.equal(fn(q, k, v, fa, fb_, mask, False, None), want)
            o = fn(q.clone().requires_grad_(True), k, v, fa, fb_, mask, False, None)
            with pytest.raises((AssertionError, RuntimeError), match="mask gradient"):
                o.backward(do)
            # a mask that asks for nothing: the backward runs
            o = fn(q.clone().requires_grad_(True), k, v, fa, fb_, mask.detach(), False, None)
            o.backward(do)


def test_backward_reproducibility(gpu_device):
    """All five gradients are accumulated in registers in a fixed order (no atomics):
    bit-identical from run to run."""
    dev = gpu_device
    ins = [t.to(dev).requires_grad_(True) for t in make_inputs(2, 700, 700, 4, 32, 8, torch.bfloat16, seed=6)[:5]]
    do = torch.randn(2, 700, 4, 32, device=dev, dtype=torch.bfloat16)
    runs = []
    for _ in range(3):
        o = flash_bias_func(*ins, None, True, None)
        runs.append(torch.autograd.grad(o, ins, do))
    for other in runs[1:]:
        for idx in range(5):
            assert torch.equal(runs[0][idx], other[idx])


def test_backward_phases_through_the_c_abi(gpu_device):
    """fb_bwd_preprocess / fb_bwd_dkv / fb_bwd_dq called one by one give what fb_bwd gives, and
    the preprocess leaves -rowsum(o * dO) and lse * log2(e) in the scratch buffer (the delta of
    flash_bias_triton.py:358-400 with the sign and the scaling that the main kernels consume)."""
    from flashbias_amd import _lib
    from flashbias_amd.interface import _params, _stream, _tensor
    dev = gpu_device
    B, L, H, d, r = 2, 333, 3, 32, 8
    q, k, v, qb, kb, do = [t.to(dev) for t in make_inputs(B, L, L, H, d, r, torch.bfloat16, seed=11)]
    lib = _lib.load()

    def params():
        p, keep = _params(q, k, v, qb, kb, None, True, None)
        bufs = dict(o=torch.empty_like(q), lse=torch.empty((B, H, L), device=dev, dtype=torch.float32),
                    dq=torch.empty_like(q), dk=torch.empty_like(k), dv=torch.empty_like(v),
                    dqb=torch.empty((B, L, H, r), device=dev, dtype=q.dtype),
                    dkb=torch.empty((B, L, H, r), device=dev, dtype=q.dtype),
                    scratch=torch.full((lib.fb_bwd_workspace_bytes(p) // 4,), float("nan"), device=dev,
                                       dtype=torch.float32))
        p.o, p.lse, p.dout = _tensor(bufs["o"]), bufs["lse"].data_ptr(), _tensor(do)
        p.dq, p.dk, p.dv = _tensor(bufs["dq"]), _tensor(bufs["dk"]), _tensor(bufs["dv"])
        p.dq_bias, p.dk_bias, p.delta = _tensor(bufs["dqb"]), _tensor(bufs["dkb"]), bufs["scratch"].data_ptr()
        return p, keep, bufs

    p1, keep1, whole = params()
    _lib.check_status(lib.fb_fwd(p1, _stream()))
    _lib.check_status(lib.fb_bwd(p1, _stream()))
    p2, keep2, parts = params()
    _lib.check_status(lib.fb_fwd(p2, _stream()))
    for name in ("fb_bwd_preprocess", "fb_bwd_dkv", "fb_bwd_dq"):
        _lib.check_status(getattr(lib, name)(p2, _stream()))
    torch.cuda.synchronize()
    for name in ("o", "lse", "dq", "dk", "dv", "dqb", "dkb", "scratch"):
        assert torch.equal(whole[name], parts[name]), name
    o, lse = whole["o"].float(), whole["lse"]
    delta = (o * do.float()).sum(-1).permute(0, 2, 1)  # (B, H, L)
    n = B * H * L
    stats = whole["scratch"][:2 * n].view(2, B, H, L)
    assert torch.allclose(stats[0], -delta, rtol=1e-5, atol=1e-5)
    assert torch.allclose(stats[1], lse * math.log2(math.e), rtol=1e-6, atol=1e-6)
    # the same two values once more per query, as three 16-bit parts each (what the streamlined dk/dv
    # kernel feeds to its MFMAs): -lse * log2(e) in elements 0..2, -delta in 3..5, zeros in 6, 7
    off = (2 * n + 3) // 4 * 4
    parts = whole["scratch"][off:off + 4 * n].view(torch.bfloat16).view(B, H, L, 8).float()
    assert torch.allclose(parts[..., 0:3].sum(-1), -stats[1], rtol=1e-6, atol=1e-6)
    assert torch.allclose(parts[..., 3:6].sum(-1), stats[0], rtol=1e-6, atol=1e-6)
    assert (parts[..., 6:] == 0).all()


@pytest.mark.parametrize("dtype,B,H,Lq,Lk,r,causal", [
    (torch.bfloat16, 2, 4, 1024, 1024, 8, False), (torch.float16, 2, 4, 2048, 2048, 8, True),
    (torch.bfloat16, 2, 4, 4096, 4096, 0, False), (torch.bfloat16, 1, 8, 1000, 3000, 8, False),
    (torch.bfloat16, 4, 2, 2500, 1111, 8, True), (torch.float16, 2, 4, 1100, 1100, 8, False),
    (torch.bfloat16, 1, 4, 640, 700, 0, False),
    # the general kernels (ranks 16 ... 32): small grids, and causal grids of up to 1.5 workgroups per slot and kind
    (torch.bfloat16, 1, 48, 2048, 2048, 16, True), (torch.float16, 2, 4, 1024, 1024, 16, False),
    (torch.bfloat16, 2, 8, 700, 1500, 32, True), (torch.float16, 1, 8, 1024, 1000, 24, False)])
def test_small_grid_backward_in_one_launch(gpu_device, dtype, B, H, Lq, Lk, r, causal):
    """On grids that give neither backward kernel more than one workgroup per compute unit (with factors of rank 16
    and more under a causal mask: up to one and a half per workgroup slot) fb_bwd runs
    the preprocess step and one launch that holds the dq and the dk/dv workgroups side by side: the
    gradients and the scratch buffer are bit for bit those of the three phases launched one by one,
    and the gradients pass the gate against the oracle (ragged and rectangular shapes, even and odd
    tile counts included)."""
    from flashbias_amd import _lib
    from flashbias_amd.interface import _params, _stream, _tensor
    dev = gpu_device
    q, k, v, qb, kb, do = [None if t is None else t.to(dev) for t in make_inputs(B, Lq, Lk, H, 32, r, dtype, seed=41)]
    do = do * 0.25
    lib = _lib.load()

    def params():
        p, keep = _params(q, k, v, qb, kb, None, causal, None)
        bufs = dict(o=torch.empty_like(q), lse=torch.empty((B, H, Lq), device=dev, dtype=torch.float32),
                    dq=torch.empty_like(q), dk=torch.empty_like(k), dv=torch.empty_like(v),
                    scratch=torch.full((lib.fb_bwd_workspace_bytes(p) // 4,), float("nan"), device=dev,
                                       dtype=torch.float32))
        p.o, p.lse, p.dout = _tensor(bufs["o"]), bufs["lse"].data_ptr(), _tensor(do)
        p.dq, p.dk, p.dv = _tensor(bufs["dq"]), _tensor(bufs["dk"]), _tensor(bufs["dv"])
        if r:
            bufs["dqb"] = torch.empty((B, Lq, H, r), device=dev, dtype=dtype)
            bufs["dkb"] = torch.empty((B, Lk, H, r), device=dev, dtype=dtype)
            p.dq_bias, p.dk_bias = _tensor(bufs["dqb"]), _tensor(bufs["dkb"])
        p.delta = bufs["scratch"].data_ptr()
        return p, keep, bufs

    p1, keep1, whole = params()
    _lib.check_status(lib.fb_fwd(p1, _stream()))
    _lib.check_status(lib.fb_bwd(p1, _stream()))
    p2, keep2, parts = params()
    _lib.check_status(lib.fb_fwd(p2, _stream()))
    for name in ("fb_bwd_preprocess", "fb_bwd_dkv", "fb_bwd_dq"):
        _lib.check_status(getattr(lib, name)(p2, _stream()))
    torch.cuda.synchronize()
    for name in whole:
        if name == "scratch":  # (bit patterns: what neither path writes is still the NaN it was filled with)
            assert torch.equal(whole[name].view(torch.int32), parts[name].view(torch.int32)), name
        else:
            assert torch.equal(whole[name], parts[name]), name
    ref = oracle(q, k, v, qb, kb, None, causal, None, do)
    cpu = lambda t: t.detach().float().cpu()
    assert (cpu(whole["o"]) - ref[0]).abs().max() <= O_TOL[dtype]
    names = ("dq", "dk", "dv") + (("dqb", "dkb") if r else ())
    for name, want in zip(names, ref[2:]):
        assert (cpu(whole[name]) - want).abs().max() <= GRAD_TOL * want.abs().max(), name


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,Lq,Lk,H,d,r,group,causal,mask", [
    (11, 200, 200, 3, 32, 16, 4, False, False),   # ragged last group, window-sized sequences
    (8, 256, 256, 2, 32, 8, 8, False, False),     # one group: a single row of factor gradients
    (6, 130, 70, 2, 16, 16, 2, False, False),     # head dim 16: dq and dq_bias share an accumulator block
    (5, 96, 96, 2, 64, 32, 3, True, False),
    (4, 100, 100, 2, 24, 5, 2, False, False),     # unaligned rank: element-wise loaders and stores
    (6, 64, 64, 4, 32, 16, 3, False, True)])      # additive matrix mask (the shifted windows of Swin)
def test_factor_gradients_summed_over_batch_groups(gpu_device, dtype, B, Lq, Lk, H, d, r, group, causal, mask):
    """fb_params.bias_grad_group = g: dq, dk, dv are those of the ungrouped call (bit for bit where both
    run the same kernels), and row
    i of dq_bias / dk_bias is the sum over batch entries [i g, (i + 1) g) of the ungrouped call's rows
    (up to their 16-bit rounding: the grouped call rounds the fp32 sum once)."""
    from flashbias_amd import _lib
    from flashbias_amd.interface import _params, _stream, _tensor
    dev = gpu_device
    q, k, v, qb, kb, do = [t.to(dev) for t in make_inputs(B, Lq, Lk, H, d, r, dtype, seed=31)]
    qb, kb = qb[:1], kb[:1]  # shared by the batch
    m = None
    if mask:
        m = torch.where(torch.rand(1, 1, Lq, Lk, device=dev) < 0.2, -100.0, 0.0).to(dtype)
    lib = _lib.load()

    def run(g):
        p, keep = _params(q, k, v, qb, kb, m, causal, None)
        rows = -(-B // g)
        bufs = dict(o=torch.empty_like(q), lse=torch.empty((B, H, Lq), device=dev, dtype=torch.float32),
                    dq=torch.empty_like(q), dk=torch.empty_like(k), dv=torch.empty_like(v),
                    dqb=torch.full((rows, Lq, H, p.r), float("nan"), device=dev, dtype=dtype),
                    dkb=torch.full((rows, Lk, H, p.r), float("nan"), device=dev, dtype=dtype),
                    scratch=torch.empty(lib.fb_bwd_workspace_bytes(p) // 4, device=dev, dtype=torch.float32))
        p.o, p.lse, p.dout = _tensor(bufs["o"]), bufs["lse"].data_ptr(), _tensor(do)
        p.dq, p.dk, p.dv = _tensor(bufs["dq"]), _tensor(bufs["dk"]), _tensor(bufs["dv"])
        p.dq_bias, p.dk_bias, p.delta = _tensor(bufs["dqb"]), _tensor(bufs["dkb"]), bufs["scratch"].data_ptr()
        p.bias_grad_group = g
        _lib.check_status(lib.fb_fwd(p, _stream()))
        _lib.check_status(lib.fb_bwd(p, _stream()))
        torch.cuda.synchronize()
        del keep
        return bufs

    one, grouped = run(1), run(group)
    # head dim 32 with rank 8 runs the streamlined kernels ungrouped and the general ones grouped: equal
    # up to rounding there, bit for bit everywhere else
    same_kernels = not (d == 32 and r == 8)
    for name in ("o", "lse", "dq", "dk", "dv"):
        if same_kernels or name in ("o", "lse"):
            assert torch.equal(one[name], grouped[name]), name
        else:
            a, b = one[name].float(), grouped[name].float()
            assert (a - b).abs().max() <= 2e-2 * a.abs().max(), name
    for name in ("dqb", "dkb"):
        full = one[name].float()
        pad = (-B) % group
        if pad:
            full = torch.cat([full, torch.zeros((pad,) + full.shape[1:], device=dev)])
        want = full.view(-1, group, *full.shape[1:]).sum(1)
        got = grouped[name].float()
        assert torch.isfinite(got).all(), name
        # the ungrouped rows carry one 16-bit rounding each, the grouped sum carries one in all
        eps = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
        tol = eps * (one[name].float().abs().view(-1, *full.shape[1:]).max() * group + want.abs().max())
        assert (got - want).abs().max() <= tol, (name, float((got - want).abs().max()), float(tol))


@pytest.mark.parametrize("dtype,B,H,Lq,Lk,r,scale,group,grads", [
    (torch.bfloat16, 40, 8, 256, 256, 16, None, 1, True),    # the Swin shape: full windows, rank 16
    (torch.bfloat16, 70, 4, 256, 256, 16, None, 4, True),    # factors shared by the batch, groups of 4 (last group ragged)
    (torch.float16, 33, 8, 200, 130, 8, None, 1, True),      # ragged lengths, three key waves empty
    (torch.bfloat16, 64, 4, 100, 256, 32, 1.0, 2, True),     # one query step, rank 32, scale 1 (no multiply per score)
    (torch.bfloat16, 32, 8, 256, 72, 24, 0.3, 1, True),      # rank 24, explicit scale
    (torch.float16, 256, 1, 129, 255, 0, None, 1, True),     # no factors
    (torch.bfloat16, 36, 8, 250, 250, 16, None, 1, False),   # constant factors: no dq_bias / dk_bias
    (torch.bfloat16, 64, 4, 256, 256, 8, None, 8, False),    # constant shared factors, groups
    # enough (batch, head) pairs for a workgroup to walk several entries without summing their factor gradients
    (torch.bfloat16, 1101, 4, 200, 256, 16, None, 1, True),  # four per workgroup, the last workgroup ragged
    (torch.float16, 2100, 1, 129, 255, 0, None, 1, True),    # no factors, two per workgroup
    (torch.bfloat16, 4100, 2, 64, 64, 8, 1.0, 1, False),     # constant factors, eight per workgroup
])
def test_window_backward(gpu_device, dtype, B, H, Lq, Lk, r, scale, group, grads):
    """Whole sequences of at most 256 positions at head dim 32 on grids that fill the chip: fb_bwd runs the
    preprocess step and one kernel that forms all five gradients per (batch, head), dq summed inside the
    workgroup.  Checked through the C ABI against the oracle, against the three phases called one by one (other
    kernels, other summation orders: equal up to rounding) and against itself (bit-reproducible)."""
    from flashbias_amd import _lib
    from flashbias_amd.interface import _params, _stream, _tensor
    dev = gpu_device
    shared = group > 1
    q, k, v, qb, kb, do = make_inputs(B, Lq, Lk, H, 32, r, dtype, seed=41, bq=(shared, False), bk=(shared, False))
    ref = oracle(q, k, v, qb, kb, None, False, scale, do)
    q, k, v, do = [t.to(dev) for t in (q, k, v, do)]
    if r:
        qb, kb = qb.to(dev), kb.to(dev)
    lib = _lib.load()

    def run(fused):
        p, keep = _params(q, k, v, qb, kb, None, False, scale)
        rows = -(-B // group)
        bufs = dict(o=torch.empty_like(q), lse=torch.empty((B, H, Lq), device=dev, dtype=torch.float32),
                    dq=torch.full_like(q, float("nan")), dk=torch.full_like(k, float("nan")), dv=torch.full_like(v, float("nan")),
                    scratch=torch.empty(lib.fb_bwd_workspace_bytes(p) // 4, device=dev, dtype=torch.float32))
        p.o, p.lse, p.dout = _tensor(bufs["o"]), bufs["lse"].data_ptr(), _tensor(do)
        p.dq, p.dk, p.dv, p.delta = _tensor(bufs["dq"]), _tensor(bufs["dk"]), _tensor(bufs["dv"]), bufs["scratch"].data_ptr()
        if r and grads:
            bufs["dqb"] = torch.full((rows, Lq, H, r), float("nan"), device=dev, dtype=dtype)
            bufs["dkb"] = torch.full((rows, Lk, H, r), float("nan"), device=dev, dtype=dtype)
            p.dq_bias, p.dk_bias = _tensor(bufs["dqb"]), _tensor(bufs["dkb"])
        p.bias_grad_group = group
        _lib.check_status(lib.fb_fwd(p, _stream()))
        if fused:
            _lib.check_status(lib.fb_bwd(p, _stream()))
        else:
            for fn in (lib.fb_bwd_preprocess, lib.fb_bwd_dkv, lib.fb_bwd_dq):
                _lib.check_status(fn(p, _stream()))
        torch.cuda.synchronize()
        del keep
        return bufs

    one, two, phases = run(True), run(True), run(False)
    f = lambda t: t.float().cpu()
    names = ["dq", "dk", "dv"] + (["dqb", "dkb"] if r and grads else [])
    for name in names:
        assert not torch.isnan(one[name].float()).any(), name
        assert torch.equal(one[name], two[name]), name
        err = (f(one[name]) - f(phases[name])).abs().max()
        assert err <= 2.0 ** -6 * f(phases[name]).abs().max(), (name, err)
    for name, want in zip(("dq", "dk", "dv"), ref[2:5]):
        assert errors(f(one[name]), want)[1] <= GRAD_TOL, name
    if r and grads:
        for name, want in (("dqb", ref[5]), ("dkb", ref[6])):
            got = f(one[name]).sum(0, keepdim=True) if shared else f(one[name])
            tol = GRAD_TOL if not shared else 2e-2  # (summed rows: the rounding of each stored row adds up)
            assert errors(got, want)[1] <= max(tol, GRAD_TOL), name


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,r_in,r_out", [(1000, 2, 16), (777, 5, 8), (300, 7, 16), (513, 16, 2), (129, 8, 5), (64, 20, 24),
                                             (50, 3, 6), (1, 1, 8)])
def test_resize_rank(gpu_device, dtype, rows, r_in, r_out):
    """fb_resize_rank through the C ABI: zero columns appended, or the first columns taken, bit for bit; also
    into an output that is not 16-byte aligned."""
    from flashbias_amd import _lib
    from flashbias_amd.interface import _stream
    lib = _lib.load()
    g = torch.Generator().manual_seed(5)
    x = torch.randn(rows, r_in, generator=g).to(dtype).to(gpu_device)
    keep = min(r_in, r_out)
    want = torch.zeros(rows, r_out, dtype=dtype, device=gpu_device)
    want[:, :keep] = x[:, :keep]
    for offset in (0, 1):
        buf = torch.full((rows * r_out + 8,), float("nan"), dtype=dtype, device=gpu_device)
        out = buf[offset:offset + rows * r_out].view(rows, r_out)
        _lib.check_status(lib.fb_resize_rank(x.data_ptr(), out.data_ptr(), rows, r_in, r_out, _stream()))
        torch.cuda.synchronize()
        assert torch.equal(out, want)
        assert torch.isnan(buf[offset + rows * r_out:].float()).all() and torch.isnan(buf[:offset].float()).all()


def test_rank_padding_inside_the_operator(gpu_device):
    """Factors of rank 5 through flash_bias_func (padded per call by the library's kernel, their gradients cut
    back by it) against the same factors padded by the tensor library beforehand: same bits."""
    B, L, H, d, r = 2, 300, 3, 32, 5
    q, k, v, qb, kb, do = [t.to(gpu_device) for t in make_inputs(B, L, L, H, d, r, torch.bfloat16, seed=51)]
    leaves = [t.clone().requires_grad_(True) for t in (q, k, v, qb, kb)]
    got = torch.autograd.grad(flash_bias_func(*leaves, None, True, None), leaves, do)
    leaves2 = [t.clone().requires_grad_(True) for t in (q, k, v, qb, kb)]
    pad = lambda t: torch.nn.functional.pad(t, (0, 16 - r))  # (ranks below 8 go to 16)
    want = torch.autograd.grad(flash_bias_func(*leaves2[:3], pad(leaves2[3]), pad(leaves2[4]), None, True, None), leaves2, do)
    for a, b in zip(got, want):
        assert a.shape == b.shape and torch.equal(a, b)
    # a permuted view (what the reference's harness passes, benchmark.py:233-235) takes the tensor library's pad
    qbp = qb.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3).requires_grad_(True)
    got2 = torch.autograd.grad(flash_bias_func(leaves[0], leaves[1], leaves[2], qbp, leaves[4], None, True, None), [qbp], do)
    assert torch.equal(got2[0], got[3])


def _random_windows(count, seed):
    """Reproducible draws from what the window backward accepts: any lengths up to 256, ranks 0 ... 32 in steps of
    8, both element types, factors per entry or shared with groups of any size, with or without factor gradients,
    on grids of at least one workgroup per compute unit."""
    import random
    rnd = random.Random(seed)
    out = []
    for idx in range(count):
        r = rnd.choice([0, 8, 16, 16, 24, 32])
        group = rnd.choice([1, 1, 2, 3, 5, 8, 32]) if r else 1
        H = rnd.choice([1, 2, 4, 8])
        B = -(-rnd.choice([256, 300, 512]) // H) * group + rnd.choice([0, 0, 1, group - 1])
        lens = [rnd.choice([1, 31, 32, 33, 64, 100, 127, 128, 129, 160, 200, 255, 256]) for _ in range(2)]
        if rnd.random() < 0.4:
            lens[1] = lens[0]
        out.append((rnd.choice([torch.bfloat16, torch.float16]), B, H, lens[0], lens[1], r,
                    rnd.choice([None, None, 1.0, 0.3]), group, rnd.random() < 0.7, idx))
    return out


@pytest.mark.parametrize("dtype,B,H,Lq,Lk,r,scale,group,grads,idx",
                         _random_windows(int(os.environ.get("FB_RANDOM_WINDOWS", "10")),
                                         int(os.environ.get("FB_RANDOM_SEED", "20240"))))
def test_random_windows(gpu_device, dtype, B, H, Lq, Lk, r, scale, group, grads, idx):
    """The window backward on shapes nobody picked by hand, against the three phases launched one by one (whose
    kernels the rest of this file holds against the oracle) and against itself."""
    from flashbias_amd import _lib
    from flashbias_amd.interface import _params, _stream, _tensor
    dev = gpu_device
    g = torch.Generator(device="cpu").manual_seed(3000 + idx)
    mk = lambda *shape: torch.randn(*shape, generator=g).to(dtype).to(dev)
    q, k, v, do = mk(B, Lq, H, 32), mk(B, Lk, H, 32), mk(B, Lk, H, 32), mk(B, Lq, H, 32)
    qb = kb = None
    if r:
        fb = 1 if group > 1 else B
        qb, kb = mk(fb, Lq, H, r) / r ** 0.5, mk(fb, Lk, H, r) / r ** 0.5
    lib = _lib.load()

    def run(fused):
        p, keep = _params(q, k, v, qb, kb, None, False, scale)
        bufs = dict(o=torch.empty_like(q), lse=torch.empty((B, H, Lq), device=dev, dtype=torch.float32),
                    dq=torch.full_like(q, float("nan")), dk=torch.full_like(k, float("nan")), dv=torch.full_like(v, float("nan")),
                    scratch=torch.empty(lib.fb_bwd_workspace_bytes(p) // 4, device=dev, dtype=torch.float32))
        p.o, p.lse, p.dout = _tensor(bufs["o"]), bufs["lse"].data_ptr(), _tensor(do)
        p.dq, p.dk, p.dv, p.delta = _tensor(bufs["dq"]), _tensor(bufs["dk"]), _tensor(bufs["dv"]), bufs["scratch"].data_ptr()
        if r and grads:
            rows = -(-B // group)
            bufs["dqb"] = torch.full((rows, Lq, H, r), float("nan"), device=dev, dtype=dtype)
            bufs["dkb"] = torch.full((rows, Lk, H, r), float("nan"), device=dev, dtype=dtype)
            p.dq_bias, p.dk_bias = _tensor(bufs["dqb"]), _tensor(bufs["dkb"])
        p.bias_grad_group = group if r else 0
        _lib.check_status(lib.fb_fwd(p, _stream()))
        for fn in ((lib.fb_bwd,) if fused else (lib.fb_bwd_preprocess, lib.fb_bwd_dkv, lib.fb_bwd_dq)):
            _lib.check_status(fn(p, _stream()))
        torch.cuda.synchronize()
        del keep
        return bufs

    one, two, phases = run(True), run(True), run(False)
    for name in ["dq", "dk", "dv"] + (["dqb", "dkb"] if r and grads else []):
        a, b = one[name].float(), phases[name].float()
        assert torch.isfinite(a).all(), name
        assert torch.equal(one[name], two[name]), name
        # (other kernels, other summation orders; grouped rows are sums of up to `group` entries rounded once; with a
        # single key dq and dk are zero up to the rounding of the stored o, hence the floor)
        scale_of = max(float(b.abs().max()), 0.05)
        assert (a - b).abs().max() <= 2.0 ** -6 * scale_of, (name, float((a - b).abs().max()), float(b.abs().max()))


def test_shared_factors_large_batch_of_windows(gpu_device):
    """A batch large enough for the library to suggest groups (64 windows x 16 heads of 256 tokens,
    factors shared by the windows, as in swin_transformer_v2.py:178-203): all five gradients through
    autograd against the oracle."""
    from flashbias_amd import _lib
    from flashbias_amd.interface import _params
    dev = gpu_device
    B, L, H, d, r = 512, 256, 16, 32, 16
    q, k, v, qb, kb, do = [t.to(dev) for t in make_inputs(B, L, L, H, d, r, torch.bfloat16, seed=32)]
    qb, kb = qb[:1].contiguous(), kb[:1].contiguous()
    p, keep = _params(q, k, v, qb, kb, None, False, None)
    assert _lib.load().fb_suggest_bias_grad_group(p) > 1
    del keep
    leaves = [t.clone().requires_grad_(True) for t in (q, k, v, qb, kb)]
    o = flash_bias_func(*leaves, None, False, None)
    grads = torch.autograd.grad(o, leaves, do)
    sub = slice(0, 8)  # o, dq, dk, dv of eight windows against the oracle
    ref = oracle(q[sub], k[sub], v[sub], qb, kb, None, False, None, do[sub])
    cpu = lambda t: t.detach().float().cpu()
    assert (cpu(o[sub]) - ref[0]).abs().max() <= O_TOL[torch.bfloat16]
    for name, got, want in zip(("dq", "dk", "dv"), grads[:3], ref[2:5]):
        assert (cpu(got[sub]) - want).abs().max() <= GRAD_TOL * want.abs().max(), name
    # the factor gradients: the sum over all windows, against the ungrouped path of the C ABI summed in fp64
    from flashbias_amd.interface import _stream, _tensor
    lib = _lib.load()
    p, keep = _params(q, k, v, qb, kb, None, False, None)
    lse = torch.empty((B, H, L), device=dev, dtype=torch.float32)
    bufs = [torch.empty_like(q) for _ in range(4)]
    full = [torch.empty((B, L, H, r), device=dev, dtype=q.dtype) for _ in range(2)]
    scratch = torch.empty(lib.fb_bwd_workspace_bytes(p) // 4, device=dev, dtype=torch.float32)
    p.o, p.lse, p.dout = _tensor(bufs[0]), lse.data_ptr(), _tensor(do)
    p.dq, p.dk, p.dv = _tensor(bufs[1]), _tensor(bufs[2]), _tensor(bufs[3])
    p.dq_bias, p.dk_bias, p.delta = _tensor(full[0]), _tensor(full[1]), scratch.data_ptr()
    _lib.check_status(lib.fb_fwd(p, _stream()))
    _lib.check_status(lib.fb_bwd(p, _stream()))
    torch.cuda.synchronize()
    for name, got, f in zip(("dq_bias", "dk_bias"), grads[3:], full):
        want = f.double().sum(0, keepdim=True)
        assert got.shape == want.shape
        assert (got.double() - want).abs().max() <= 2e-2 * want.abs().max(), name


@pytest.mark.parametrize("Lq,Lk", [(1000, 1000), (777, 1300), (1300, 777)])
@pytest.mark.parametrize("causal", [False, True])
def test_long_ragged_sequences(gpu_device, Lq, Lk, causal):
    """Many steps through the three-stage LDS ring of the dk/dv kernel, last step ragged."""
    _case(gpu_device, 1, Lq, Lk, 2, 32, 8, torch.bfloat16, causal, seed=12)


@pytest.mark.parametrize("B,H,Lq,Lk,r,causal", [(8, 16, 1000, 1000, 8, False), (8, 32, 700, 700, 8, True),
                                                 (4, 64, 777, 1300, 16, False), (8, 32, 1300, 777, 0, True),
                                                 (64, 16, 256, 256, 8, False), (64, 16, 128, 128, 16, False),
                                                 (48, 16, 380, 300, 16, True),
                                                 (16, 16, 700, 520, 32, False), (40, 16, 520, 700, 24, True)])
def test_large_grids_ragged(gpu_device, B, H, Lq, Lk, r, causal):
    """Grids of at least two (causal: three) 256-query workgroups per compute unit of an MI355X
    (256 CUs): the launchers then pick the two-query-blocks-per-wave kernels, which the small
    cases above never reach; ragged last tiles, rectangular and causal shapes.  The last two are
    windows whose last 256-query workgroup would be half empty: they take 128-query workgroups on a
    grid that would otherwise get the large ones.  Ranks 32 and 24: four operand steps per score, the
    widest forward that keeps two query blocks per wave."""
    assert B * H * ((Lq + 255) // 256) >= (3 if causal else 2) * 256
    _case(gpu_device, B, Lq, Lk, H, 32, r, torch.bfloat16, causal, seed=13)


@pytest.mark.parametrize("B,H,Lq,Lk,d,r,causal,dtype", [
    (2, 4, 1024, 1024, 32, 8, False, torch.bfloat16),    # streamlined kernels, one mixed backward launch
    (8, 16, 1000, 1000, 32, 8, True, torch.float16),     # streamlined dq and dk/dv kernels on a grid that fills the chip
    (1, 8, 2048, 2048, 32, 5, False, torch.bfloat16),    # rank 5: padded to 16 by the operator, general kernels
    (3, 4, 300, 520, 32, 16, False, torch.bfloat16),     # general kernels
    (2, 2, 200, 333, 64, 32, True, torch.bfloat16),
    (40, 16, 256, 256, 32, 16, False, torch.bfloat16),   # factors shared by a large batch (groups of batch entries)
])
def test_constant_factors_skip_their_gradients(gpu_device, B, H, Lq, Lk, d, r, causal, dtype):
    """Factors that do not require a gradient (ALiBi slopes, tables loaded from a file, coordinates): the library
    is given no dq_bias / dk_bias; o, dq, dk, dv are bit for bit those of the call that computes all five."""
    shared = B >= 32
    q, k, v, qb, kb, do = make_inputs(B, Lq, Lk, H, d, r, dtype, seed=77, bq=(shared, False), bk=(shared, False))
    dev = gpu_device

    def run(factor_grads):
        leaves = [t.to(dev).requires_grad_(True) for t in (q, k, v)]
        fac = [t.to(dev).requires_grad_(factor_grads) for t in (qb, kb)]
        o = flash_bias_func(leaves[0], leaves[1], leaves[2], fac[0], fac[1], None, causal, None)
        grads = torch.autograd.grad(o, leaves + (fac if factor_grads else []), do.to(dev))
        return [o.detach()] + list(grads)

    full, part = run(True), run(False)
    assert len(full) == 6 and len(part) == 4
    for name, a, b in zip(("o", "dq", "dk", "dv"), full, part):
        assert torch.equal(a, b), name
    # and through the C ABI: null outputs are accepted, one of two is not
    from flashbias_amd import _lib
    from flashbias_amd.interface import _params, _stream, _tensor
    lib = _lib.load()
    qd, kd, vd, qbd, kbd, dod = [t.to(dev) for t in (q, k, v, qb, kb, do)]
    p, keep = _params(qd, kd, vd, qbd, kbd, None, causal, None)
    o = torch.empty_like(qd)
    lse = torch.empty((B, H, Lq), device=dev, dtype=torch.float32)
    p.o, p.lse = _tensor(o), lse.data_ptr()
    _lib.check_status(lib.fb_fwd(p, _stream()))
    outs = [torch.empty_like(t) for t in (qd, kd, vd)]
    p.dout, p.dq, p.dk, p.dv = _tensor(dod), _tensor(outs[0]), _tensor(outs[1]), _tensor(outs[2])
    scratch = torch.empty(lib.fb_bwd_workspace_bytes(p) // 4, device=dev, dtype=torch.float32)
    p.delta = scratch.data_ptr()
    for name in ("fb_bwd", "fb_bwd_static"):
        for t in outs:
            t.zero_()
        _lib.check_status(getattr(lib, name)(p, _stream()))
        torch.cuda.synchronize()
        for nm, a, b in zip(("dq", "dk", "dv"), full[1:4], outs):
            assert torch.equal(a, b), (name, nm)
    _lib.check_status(lib.fb_bwd_preprocess(p, _stream()))
    _lib.check_status(lib.fb_bwd_dkv(p, _stream()))
    _lib.check_status(lib.fb_bwd_dq(p, _stream()))
    torch.cuda.synchronize()
    # (whole sequences of at most 256 positions on a grid that fills the chip: fb_bwd runs the window kernel, the
    # phases the two general ones: other summation orders, equal up to rounding)
    window = d == 32 and max(Lq, Lk) <= 256 and not causal and B * H >= 256
    for nm, a, b in zip(("dq", "dk", "dv"), full[1:4], outs):
        if window:
            assert (a.float() - b.float()).abs().max() <= 2.0 ** -6 * a.float().abs().max(), ("phases", nm)
        else:
            assert torch.equal(a, b), ("phases", nm)


def _random_configurations(n, seed):
    """n configurations drawn with a fixed seed from everything the operator accepts: head dims 8 ... 128
    (not only multiples of 8), ranks 0 ... 64, lengths 1 ... 900 on either side, either element type,
    causal or not, broadcast factors, the three mask forms, explicit scales.  Sizes are chosen so that
    some grids fill the chip (the launchers then pick their large-workgroup kernels) and most do not."""
    import numpy as np
    rng = np.random.RandomState(seed)
    out = []
    for i in range(n):
        d = int(rng.choice([8, 16, 24, 32, 32, 32, 40, 64, 64, 96, 128]))
        r = int(rng.choice([0, 2, 5, 8, 8, 16, 16, 24, 32, 64]))
        big = rng.rand() < 0.25  # a grid of several workgroups per compute unit
        B, H = (int(rng.randint(8, 25)), int(rng.choice([8, 16]))) if big else (int(rng.randint(1, 4)), int(rng.randint(1, 6)))
        hi = 420 if big else 900
        Lq, Lk = int(rng.randint(1, hi)), int(rng.randint(1, hi))
        if d > 64 and big:
            B = max(B // 4, 1)
        causal = bool(rng.rand() < 0.4)
        dtype = "bf16" if rng.rand() < 0.6 else "f16"
        mask = str(rng.choice(["none", "none", "none", "vector", "matrix", "vector_f32"]))
        bq = (bool(rng.rand() < 0.2), bool(rng.rand() < 0.2))
        bk = (bool(rng.rand() < 0.2), bool(rng.rand() < 0.2))
        scale = None if rng.rand() < 0.7 else float(rng.choice([1.0, 0.5, 0.05]))
        out.append(pytest.param(B, H, Lq, Lk, d, r, causal, dtype, mask, bq, bk, scale, i,
                                id="%d-B%dH%d-%dx%d-d%dr%d-%s%s-%s" % (i, B, H, Lq, Lk, d, r, dtype, "-causal" if causal else "", mask)))
    return out


# (FB_RANDOM_CASES / FB_RANDOM_SEED in the environment draw a longer or a different list for a soak run)
@pytest.mark.parametrize("B,H,Lq,Lk,d,r,causal,dtype,mask_kind,bq,bk,scale,idx",
                         _random_configurations(int(os.environ.get("FB_RANDOM_CASES", "36")),
                                                int(os.environ.get("FB_RANDOM_SEED", "20240"))))
def test_random_configurations(gpu_device, B, H, Lq, Lk, d, r, causal, dtype, mask_kind, bq, bk, scale, idx):
    """Whatever the launchers choose for a configuration nobody picked by hand must meet the same gate."""
    dt = torch.bfloat16 if dtype == "bf16" else torch.float16
    g = torch.Generator().manual_seed(1000 + idx)
    mask = None
    if mask_kind == "vector":
        mask = torch.randn(B, 1, 1, Lk, generator=g).to(dt)
    elif mask_kind == "vector_f32":
        mask = torch.randn(1, H, 1, Lk, generator=g)
    elif mask_kind == "matrix":
        mask = torch.randn(B, 1, Lq, Lk, generator=g).to(dt)
    # (explicit scales of 0.5 and 1 give logits with a spread of 4-11: peaked rows, outputs as large as v itself)
    _case(gpu_device, B, Lq, Lk, H, d, r, dt, causal, mask=mask, scale=scale, seed=2000 + idx, o_by_magnitude=True, bq=bq, bk=bk)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("r", [0, 8])
@pytest.mark.parametrize("causal", [False, True])
def test_streamlined_kernels(gpu_device, dtype, r, causal):
    """Head dim 32, rank 8 or no factors, aligned, unmasked, on grids that fill an MI355X: the shapes
    that take the streamlined forward kernel (two query blocks per wave, at least two 256-query workgroups per
    compute unit; under a causal mask its one-block instantiation) and the streamlined dk/dv kernel (at least two 128-key workgroups per compute
    unit), with ragged last tiles on both sides, in both element types."""
    B, H, Lq, Lk = (8, 32, 1800, 600) if causal else (8, 16, 1000, 1000)
    assert B * H * ((Lq + 255) // 256) >= 2 * 256 and B * H * ((Lk + 127) // 128) >= 2 * 256
    _case(gpu_device, B, Lq, Lk, H, 32, r, dtype, causal, seed=14)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("which", ["q_bias", "k_bias", "logits"])
def test_streamlined_kernels_fall_back(gpu_device, which, causal):
    """Inputs the streamlined kernels cannot take make their workgroups run the general algorithm
    instead: an fp16 factor entry that overflows once log2(e) is folded into it (60000, facing a zero
    column of the other factor, so the bias itself is unchanged: q_bias for the forward and dq
    kernels, k_bias for dk/dv), and logits so peaked that P = 2^(s - m) with the fixed reference
    point leaves fp16's range (unscaled N(0,1) factors of rank 8, as in the reference's own
    correctness script, at a length where some row sums exceed the limit)."""
    B, L, H, d, r = 2, 640, 2, 32, 8
    q, k, v, qb, kb, do = make_inputs(B, L, L, H, d, r, torch.float16, seed=15)
    if which == "logits":
        g = torch.Generator().manual_seed(16)
        qb, kb = [torch.randn(B, L, H, r, generator=g).half() * 1.5 for _ in range(2)]
    else:
        big, zero = (qb, kb) if which == "q_bias" else (kb, qb)
        zero[..., 3] = 0
        big[:, ::7, :, 3] = 60000.0
        do = (do.float() * 0.03).half()  # (keeps the gradient of the zero column, ~ 60000 dS, inside fp16)
    ref = oracle(q, k, v, qb, kb, None, causal, None, do)
    got = run_gpu(flash_bias_func, q, k, v, qb, kb, None, causal, None, do, gpu_device)
    _gate(got, ref, torch.float16)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("offset", [0, 1])
def test_matrix_mask_alignment(gpu_device, dtype, offset):
    """Matrix masks that allow aligned 4-key loads, and views of them that do not."""
    B, L, H = 1, 200, 2
    g = torch.Generator().manual_seed(13)
    big = torch.randn(1, H, L, L + 8, generator=g).to(dtype)
    mask = big[..., offset:offset + L]  # row stride L + 8; offset 1 breaks the alignment of every row
    _case(gpu_device, B, L, L, H, 32, 8, torch.bfloat16, False, mask=mask, seed=14)


def _random_case(idx):
    """A reproducible draw from the space of supported shapes: lengths, head dim, rank, dtype,
    causal flag, factor broadcasting and mask kind / dtype / alignment."""
    import random
    rnd = random.Random(1000 + idx)
    d = rnd.choice([8, 16, 24, 32, 32, 32, 40, 64, 64, 72, 128])
    r = rnd.choice([0, 8, 8, 8, 16, 24, 32, 64])
    lens = [rnd.choice([1, 17, 63, 64, 65, 127, 128, 129, 200, 256, 333, 512, 640, 701]) for _ in range(2)]
    if rnd.random() < 0.5:
        lens[1] = lens[0]
    dtype = rnd.choice([torch.bfloat16, torch.float16])
    causal = rnd.random() < 0.4
    bq = (rnd.random() < 0.25, rnd.random() < 0.25)
    bk = (rnd.random() < 0.25, rnd.random() < 0.25)
    mask_kind = rnd.choice([None, None, "vector", "matrix", "matrix", "matrix_f32", "matrix_shifted"])
    return dict(B=rnd.choice([1, 2]), H=rnd.choice([1, 3]), Lq=lens[0], Lk=lens[1], d=d, r=r, dtype=dtype, causal=causal,
                bq=bq, bk=bk, mask_kind=mask_kind, scale=rnd.choice([None, 0.3]))


@pytest.mark.parametrize("idx", range(40))
def test_random_shapes(gpu_device, idx):
    c = _random_case(idx)
    g = torch.Generator().manual_seed(2000 + idx)
    B, H, Lq, Lk = c["B"], c["H"], c["Lq"], c["Lk"]
    mask = None
    if c["mask_kind"] == "vector":
        mask = torch.randn(B, 1, 1, Lk, generator=g).to(c["dtype"])
    elif c["mask_kind"] == "matrix":
        mask = torch.randn(1, H, Lq, Lk, generator=g).to(c["dtype"])
    elif c["mask_kind"] == "matrix_f32":
        mask = torch.randn(B, 1, Lq, Lk, generator=g)
    elif c["mask_kind"] == "matrix_shifted":  # rows that are not 16-byte aligned
        mask = torch.randn(1, H, Lq, Lk + 3, generator=g).to(c["dtype"])[..., 3:]
    _case(gpu_device, B, Lq, Lk, H, c["d"], c["r"], c["dtype"], c["causal"], mask=mask, scale=c["scale"], seed=3000 + idx,
          bq=c["bq"], bk=c["bk"])


# ------------------------------------------------------------------ named workloads (reduced)
def _run_workload(gpu_device, w, dtype, skip=()):
    mask = w.get("mask")
    ref = oracle(w["q"], w["k"], w["v"], w["q_bias"], w["k_bias"], mask, w["causal"], w["softmax_scale"], w["do"])
    got = run_gpu(flash_bias_func, w["q"], w["k"], w["v"], w["q_bias"], w["k_bias"], mask, w["causal"],
                  w["softmax_scale"], w["do"], gpu_device)
    _gate(got, ref, dtype, skip)
    return got, ref


def _stored_backward_gate(gpu_device, w, dtype, report=None):
    """The principled gate for a backward that consumes *stored* forward results: the kernels'
    own o and lse go to oracle.eager.flashbias_backward_stored, the restatement of the reference's
    backward contract including its two 16-bit roundings (P and dS, flash_bias_triton.py:696,
    :714; delta from the stored o, :398), and all five gradients are held to the usual
    max|err| / max|ref| <= 5e-2 against that."""
    from flashbias_amd.interface import _flash_bias_backward, _flash_bias_forward
    from oracle import eager
    dev = gpu_device
    t = {n: (None if w[n] is None else w[n].to(dev)) for n in ("q", "k", "v", "q_bias", "k_bias", "do")}
    o, lse, scale = _flash_bias_forward(t["q"], t["k"], t["v"], t["q_bias"], t["k_bias"], None, w["causal"],
                                        w["softmax_scale"])
    got = _flash_bias_backward(t["do"], t["q"], t["k"], t["v"], o, t["q_bias"], t["k_bias"], lse, None, w["causal"],
                               scale)
    torch.cuda.synchronize()
    f = lambda x: x.detach().float().cpu()
    want = eager.flashbias_backward_stored(f(w["q"]), f(w["k"]), f(w["v"]), f(w["q_bias"]), f(w["k_bias"]), None,
                                           w["causal"], scale, f(o), f(lse), f(w["do"]), round_dtype=dtype)
    for name, g, r in zip(NAMES[1:], got, want):
        _, rel = errors(f(g), r)
        if report is not None:
            report[name] = rel
        assert rel <= GRAD_TOL, (name, rel)


def test_workload_alibi(gpu_device, capsys):
    """Causal ALiBi as the rank-2 bias of the benchmark configuration, H=50 (reduced L).
    o, dq, dk, dv and dk_bias pass the usual gate against the fp32 oracle.  dq_bias does not, and cannot in any
    backward that follows the reference's contract of consuming the stored 16-bit o
    (delta = rowsum(o * dO), flash_bias_triton.py:398): dq_bias[i, 1] = sum_j dS_ij m j with rows of dS that sum
    to zero, so an error eps in delta_i comes back multiplied by m sum_j P_ij j (about m i, hundreds), and the
    rounding of the stored o alone, with everything else exact, already leaves 0.8 of max|dq_bias| (the oracle
    run that way on the CPU).  So dq_bias is held (a) to the bound that this conditioning argument gives from the
    oracle's own P, dS and the 2^-8 unit roundoff of the stored o, of dS and of the result, and (b), like all five gradients, to the usual 5e-2
    against the oracle that applies the reference's two roundings to the kernels' stored o and lse.  With factors
    that are exact in 16 bits (next test) the plain gate holds for dq_bias too."""
    w = workloads.alibi(L=1024, H=50)
    got, ref = _run_workload(gpu_device, w, torch.bfloat16, skip=("dq_bias",))
    raw = {n: errors(g, r)[1] for n, g, r in zip(NAMES[4:], got[4:], ref[5:])}
    assert raw["dk_bias"] <= GRAD_TOL
    # the conditioning bound: |err dq_bias_i| <= 2^-8 (sum_j |dS_ij| |k_bias_j| + |o_i| . |dO_i| |sum_j P_ij k_bias_j| + |dq_bias_i|)
    from oracle import eager
    f = lambda t: t.float()
    q, k, v, qb, kb, do = [f(w[n]) for n in ("q", "k", "v", "q_bias", "k_bias", "do")]
    s = eager.logits(q, k, w["softmax_scale"], eager.materialize_bias(qb, kb, 1, 50), True).permute(0, 2, 1, 3)
    p = torch.softmax(s, dim=-1)                                  # (1, H, Lq, Lk)
    doh, oh = do.permute(0, 2, 1, 3), ref[0].permute(0, 2, 1, 3)
    dp = doh @ v.permute(0, 2, 3, 1)
    ds = p * (dp - (oh * doh).sum(-1, keepdim=True))
    kbh = kb.expand(1, -1, 50, -1).permute(0, 2, 1, 3)
    bound = 2.0 ** -8 * (ds.abs() @ kbh.abs() + (oh.abs() * doh.abs()).sum(-1, keepdim=True) * (p @ kbh).abs()
                         + ref[5].abs().permute(0, 2, 1, 3))
    err = (got[4] - ref[5]).abs().permute(0, 2, 1, 3)
    assert (err <= bound + 1e-3 * ref[5].abs().max()).all(), (err / bound.clamp_min(1e-30)).max()
    stored = {}
    _stored_backward_gate(gpu_device, w, torch.bfloat16, report=stored)
    with capsys.disabled():
        print(f"\n[alibi L=1024 H=50 rank-2] max|err|/max|ref| against the fp32 oracle: {raw}; conditioning bound "
              f"/ max|ref|: {(bound.max() / ref[5].abs().max()).item():.2f}; against the stored-rounding oracle: {stored}")


def test_workload_alibi_exact_factors(gpu_device):
    """The same workload with the rank-4 factors that are exact in 16 bits (every column below
    256 in magnitude): all five gradients pass the plain gate against the fp32 oracle."""
    w = workloads.alibi(L=1024, H=50, exact=True)
    _run_workload(gpu_device, w, torch.bfloat16)
    _stored_backward_gate(gpu_device, w, torch.bfloat16)


def test_workload_swin(gpu_device):
    """Swin-V2 windows (reduced count), SVD factors shared by all windows; also reports how
    close the rank-16 factors are to the exact table."""
    w = workloads.swin(windows=8)
    got, _ = _run_workload(gpu_device, w, torch.bfloat16)
    assert w["bias_rel_error"].max() < 0.05
    from oracle import eager
    exact = eager.attention_eager(w["q"].float(), w["k"].float(), w["v"].float(), w["softmax_scale"],
                                  w["bias_table"][None].expand(8, -1, -1, -1))
    assert (got[0] - exact).abs().max() < 0.1


def test_workload_swin_shifted_windows(gpu_device):
    """The same windows with the 0 / -100 matrix mask of a shifted-window block, one matrix per
    window type repeated over the images and broadcast over the heads."""
    w = workloads.swin(windows=8, shifted_types=4)
    assert w["mask"].shape == (8, 1, 256, 256)
    _run_workload(gpu_device, w, torch.bfloat16)


def test_workload_pde(gpu_device):
    """Exact rank-5 spatial-distance bias (reduced N); bias magnitudes up to ~30."""
    _run_workload(gpu_device, workloads.pde(N=2048), torch.bfloat16)


def test_small_constant_factors_take_rank_8(gpu_device):
    """Factors of rank below 8 are padded to 16 by the operator whatever their values; a caller whose
    factors have small entries pads them to rank 8 itself (factors.pad_rank) and then gets the
    streamlined kernels.  The choice depends on shapes only: no look at the data, no
    synchronisation, the same kernels eagerly and under graph capture."""
    from flashbias_amd import factors
    from flashbias_amd import interface as I
    dev = gpu_device
    w = workloads.pde(N=2048, pad_to=None)
    q, k = w["q"].to(dev), w["k"].to(dev)
    qb, kb = w["q_bias"].to(dev), w["k_bias"].to(dev)
    assert qb.shape[-1] == 5
    assert I._prepare_factors(q, k, qb, kb, None)[0].shape[-1] == 16
    q8, k8 = factors.pad_rank(qb, kb, 8)
    assert q8.shape[-1] == k8.shape[-1] == 8 and torch.equal(q8[..., :5], qb) and not q8[..., 5:].any()
    assert I._prepare_factors(q, k, q8, k8, None)[0] is q8
    a = workloads.alibi(1024)
    assert I._prepare_factors(a["q"].to(dev), a["k"].to(dev), a["q_bias"].to(dev), a["k_bias"].to(dev), None)[0].shape[-1] == 16
    # the PDE workload both ways against the oracle: rank 8 (streamlined kernels) and rank 5 -> 16 (general)
    got8, _ = _run_workload(gpu_device, workloads.pde(N=4096), torch.bfloat16)
    got16, _ = _run_workload(gpu_device, workloads.pde(N=4096, pad_to=None), torch.bfloat16)
    assert got8[4].shape[-1] == 8 and got16[4].shape[-1] == 5
    assert not got8[4][..., 5:].any()  # (zero columns of k_bias: zero gradient columns of q_bias)


def test_workload_pairformer(gpu_device):
    """Pairformer-shaped: rows as batch, rank-32 factors shared over rows (reduced N)."""
    _run_workload(gpu_device, workloads.pairformer(N=192), torch.bfloat16)


def test_modules(gpu_device):
    """Module-level drop-ins (ALiBi attention block, Swin-V2 window attention core) against the
    same modules evaluated with the eager oracle in place of the kernel."""
    from flashbias_amd import modules
    from oracle import eager
    dev = gpu_device
    torch.manual_seed(0)
    import flashbias_amd.modules as M
    real = M.flash_bias_func

    def oracle_func(q, k, v, qb, kb, mask, causal, scale):
        return eager.flashbias_eager(q.float(), k.float(), v.float(), qb.float(), kb.float(),
                                     None if mask is None else mask.float(), causal, scale).to(q.dtype)

    blocks = [(modules.AttentionWithALiBiBias(64, 4, 32).to(dev), torch.randn(2, 200, 64, device=dev), {}),
              (modules.WindowAttentionCore(64, 8, 2, rank=8).to(dev), torch.randn(6, 64, 64, device=dev),
               {"mask": (torch.rand(3, 64, 64, device=dev) < 0.2).float() * -100.0})]
    for mod, x, kw in blocks:
        x.requires_grad_(True)
        y = mod(x, **kw)
        gx, = torch.autograd.grad(y.sum(), x)
        M.flash_bias_func = oracle_func
        try:
            y_ref = mod(x, **kw)
            gx_ref, = torch.autograd.grad(y_ref.sum(), x)
        finally:
            M.flash_bias_func = real
        assert (y - y_ref).abs().max() <= 2e-2 * max(1.0, y_ref.abs().max().item())
        assert (gx - gx_ref).abs().max() <= 5e-2 * gx_ref.abs().max()


# ---------------------------------------------------------------- headline size: properties
@pytest.fixture(scope="module")
def headline(gpu_device):
    w = workloads.sweep(workloads.HEADLINE["L"])
    dev = gpu_device
    t = {n: w[n].to(dev) for n in ("q", "k", "v", "q_bias", "k_bias", "do")}
    leaves = [t[n].requires_grad_(True) for n in ("q", "k", "v", "q_bias", "k_bias")]
    o = flash_bias_func(*leaves, None, False, w["softmax_scale"])
    grads = torch.autograd.grad(o, leaves, t["do"])
    torch.cuda.synchronize()
    return w, t, o.detach(), grads


def test_headline_rows_against_oracle(gpu_device, headline):
    """At B2 H4 L16384 d32 r8 a query row depends on all keys but on no other query: o, dq,
    dq_bias of a subset of rows are checked against the oracle run on (those rows, all keys)."""
    w, t, o, grads = headline
    rows = torch.cat([torch.arange(0, 64), torch.arange(8000, 8064), torch.arange(16320, 16384)])
    sub = lambda x: x[:, rows]
    ref = oracle(sub(w["q"]), w["k"], w["v"], sub(w["q_bias"]), w["k_bias"], None, False, w["softmax_scale"],
                 sub(w["do"]))
    err, _ = errors(o[:, rows].float().cpu(), ref[0])
    assert err <= O_TOL[torch.bfloat16]
    for got, want in ((grads[0], ref[2]), (grads[3], ref[5])):
        _, rel = errors(got[:, rows].float().cpu(), want)
        assert rel <= GRAD_TOL


def test_headline_checksums(gpu_device, headline):
    """Size-independent identities: rows of P sum to 1, so sum_j dv_j = sum_i dO_i; rows of dS
    sum to 0, so sum_j dk_j = 0 and sum_j dk_bias_j = 0 (up to the rounding of the stored
    gradients)."""
    w, t, o, grads = headline
    dv_sum = grads[2].float().sum(1)
    do_sum = t["do"].float().sum(1)
    assert (dv_sum - do_sum).abs().max() <= 0.02 * do_sum.abs().max()
    for gk in (grads[1], grads[4]):
        # every stored element, and every dS that went into it, carries a rounding error of 2^-9
        bound = 16 * 2.0 ** -9 * gk.float().abs().sum(1).max() / math.sqrt(gk.shape[1])
        assert gk.float().sum(1).abs().max() <= bound


def test_headline_ones_value(gpu_device, headline):
    w, t, _, _ = headline
    o = flash_bias_func(t["q"], t["k"], torch.ones_like(t["v"]), t["q_bias"], t["k_bias"], None, False, None)
    assert (o.float() - 1).abs().max() <= 2.0 ** -7


def test_headline_matches_concat_sdpa(gpu_device, headline):
    """Library cross-check at full size: the concat identity of
    flash_bias/attention_func.py:188-237 evaluated by torch's fused attention on the GPU."""
    w, t, o, grads = headline
    q, k, v, qb, kb = [t[n].detach().requires_grad_(True) for n in ("q", "k", "v", "q_bias", "k_bias")]
    s = w["softmax_scale"]
    qc = torch.cat([q * s, qb], -1).transpose(1, 2)
    kc = torch.cat([k, kb], -1).transpose(1, 2)
    ref = torch.nn.functional.scaled_dot_product_attention(qc, kc, v.transpose(1, 2), scale=1.0).transpose(1, 2)
    rgrads = torch.autograd.grad(ref, [q, k, v, qb, kb], t["do"])
    assert (o.float() - ref.float()).abs().max() <= O_TOL[torch.bfloat16]
    for got, want in zip(grads, rgrads):
        _, rel = errors(got.float(), want.float())
        assert rel <= GRAD_TOL


# ---------------------------------------------------------------- the harness's comparison providers
def test_comparison_providers_compute_the_same_attention(gpu_device):
    """bench.py times two PyTorch formulations next to the kernels: fused SDPA on the concatenated
    features (flash_bias/attention_func.py:188-237) and SDPA with the materialised dense bias as
    attn_mask (:150-185).  Both must be the computation of the oracle at L=1024 (o, and the
    gradients each of them has: five for the concat form, dq, dk, dv for the dense-bias form),
    otherwise the comparison lines would time something else."""
    import bench
    dev = gpu_device
    w = workloads.sweep(1024)
    ref = oracle(w["q"], w["k"], w["v"], w["q_bias"], w["k_bias"], None, False, w["softmax_scale"], w["do"])
    wd = {n: (t.to(dev) if isinstance(t, torch.Tensor) else t) for n, t in w.items()}
    leaves = [wd[n].requires_grad_(True) for n in ("q", "k", "v", "q_bias", "k_bias")]
    o = bench._sdpa_concat(wd)
    grads = torch.autograd.grad(o, leaves, wd["do"])
    _gate([o.detach().float().cpu()] + [g.float().cpu() for g in grads], ref, torch.bfloat16)
    with torch.no_grad():
        bias = (wd["q_bias"].permute(0, 2, 1, 3) @ wd["k_bias"].permute(0, 2, 3, 1)).contiguous()
    o = bench._sdpa_dense(wd, bias)
    grads = torch.autograd.grad(o, leaves[:3], wd["do"])
    assert errors(o.detach().float().cpu(), ref[0])[0] <= 3e-2  # (the bias itself is rounded to bf16 here)
    for g, want in zip(grads, ref[2:5]):
        assert errors(g.float().cpu(), want)[1] <= GRAD_TOL
