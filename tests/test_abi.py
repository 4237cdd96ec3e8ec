"""CPU-only checks of the C ABI: the in-tree library loads, exports every symbol that
include/flashbias.h declares, and rejects bad arguments with the documented status codes
before anything touches a GPU."""
import ctypes
import os
import re

import pytest
import torch

from flashbias_amd import _lib, flash_bias_func

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "flashbias.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return set(re.findall(r"\b(fb_[a-z_]+)\s*\(", text))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    declared = _declared_symbols()
    assert declared == set(_lib.EXPORTS)
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.fb_version() == 3


def test_workspace_size_query():
    lib = _lib.load()
    p = _lib.new_params()
    p.B, p.H, p.Lq = 2, 4, 1000
    # per query row: -delta and lse * log2(e) as floats, then one 16-byte chunk of 16-bit parts
    assert lib.fb_bwd_workspace_bytes(p) == 2 * 4 * 1000 * (2 * 4 + 16)
    p.Lq = 1001  # the chunks start 16-byte aligned
    assert lib.fb_bwd_workspace_bytes(p) == (2 * 8008 + 3) // 4 * 4 * 4 + 8008 * 16
    p.Lq = 0
    assert lib.fb_bwd_workspace_bytes(p) == 0
    assert lib.fb_bwd_workspace_bytes(None) == 0


def _good(pass_=0):
    p = _lib.new_params()
    p.dtype = _lib.FB_BF16
    p.B, p.H, p.Lq, p.Lk, p.d, p.r = 2, 4, 128, 128, 32, 8
    p.scale = 0.25
    fake = 0x10000  # never dereferenced: fb_check does not touch the GPU
    t = lambda c: _lib.FbTensor(fake, 128 * 4 * c, c, 4 * c)
    p.q, p.k, p.v, p.o = t(32), t(32), t(32), t(32)
    p.q_bias, p.k_bias = t(8), t(8)
    p.lse = fake
    if pass_ == 1:
        p.dout, p.dq, p.dk, p.dv = t(32), t(32), t(32), t(32)
        p.dq_bias, p.dk_bias = t(8), t(8)
        p.delta = fake
    return p


def test_check_accepts_good_params():
    lib = _lib.load()
    assert lib.fb_check(_good(0), 0) == 0
    assert lib.fb_check(_good(1), 1) == 0
    assert lib.fb_last_error() == b""


@pytest.mark.parametrize("mutate,code", [
    (lambda p: setattr(p, "size", 8), -7),
    (lambda p: setattr(p, "dtype", 2), -3),
    (lambda p: setattr(p, "d", 129), -2),
    (lambda p: setattr(p, "d", 0), -2),
    (lambda p: setattr(p, "r", 129), -2),
    (lambda p: setattr(p, "Lk", 0), -2),
    (lambda p: setattr(p, "scale", 0.0), -9),
    (lambda p: setattr(p, "scale", float("nan")), -9),
    (lambda p: setattr(p.q, "ptr", None), -1),
    (lambda p: setattr(p.k_bias, "ptr", None), -1),
    (lambda p: setattr(p, "lse", None), -1),
    (lambda p: setattr(p.v, "stride_s", -32), -4),
    (lambda p: setattr(p.k, "stride_s", 16), -4),  # rows of an input would overlap
    (lambda p: setattr(p, "B", 1 << 20) or setattr(p, "H", 1 << 10), -2),  # grid beyond 2^31 - 1 workgroups
    (lambda p: setattr(p.o, "stride_b", 0), -4),
    (lambda p: setattr(p.o, "stride_s", 16), -4),
    (lambda p: setattr(p, "mask_type", 3), -5),
    (lambda p: (setattr(p, "mask_type", 1), setattr(p, "mask_dtype", 0), setattr(p.mask, "ptr", 0x10000)), -5),
    (lambda p: (setattr(p, "mask_type", 2), setattr(p, "mask_dtype", 2)), -1),
])
def test_check_rejects_forward(mutate, code):
    p = _good(0)
    mutate(p)
    lib = _lib.load()
    assert lib.fb_check(p, 0) == code
    assert lib.fb_last_error() != b""
    assert lib.fb_fwd(p, None) == code  # rejected before any launch


@pytest.mark.parametrize("mutate,code", [
    (lambda p: setattr(p.dout, "ptr", None), -1),
    (lambda p: setattr(p.dq_bias, "ptr", None), -1),
    (lambda p: setattr(p, "delta", None), -1),
    (lambda p: setattr(p.dk, "stride_h", 0), -4),
    (lambda p: setattr(p.dk_bias, "stride_b", 0), -4),
    (lambda p: setattr(p, "bias_grad_group", -1), -2),
])
def test_check_rejects_backward(mutate, code):
    p = _good(1)
    mutate(p)
    lib = _lib.load()
    assert lib.fb_check(p, 1) == code
    for fn in (lib.fb_bwd, lib.fb_bwd_preprocess, lib.fb_bwd_dkv, lib.fb_bwd_dq):
        assert fn(p, None) == code


def test_factor_gradients_may_be_left_out():
    """Both of dq_bias and dk_bias null: the caller does not want them; one of them null: an error."""
    lib = _lib.load()
    p = _good(1)
    p.dq_bias.ptr = p.dk_bias.ptr = None
    assert lib.fb_check(p, 1) == 0
    p = _good(1)
    p.dk_bias.ptr = None
    assert lib.fb_check(p, 1) == -1


def test_grouped_factor_gradients_checks_and_suggestion():
    """bias_grad_group = g: the factor gradients have ceil(B / g) batch rows, so a single group may
    use a zero batch stride; the library suggests groups only for factors shared by a large batch of
    short sequences."""
    lib = _lib.load()
    p = _good(1)
    p.dq_bias.stride_b = p.dk_bias.stride_b = 0
    assert lib.fb_check(p, 1) == -4          # two batch rows would alias
    p.bias_grad_group = 2                    # one group of two: a single row
    assert lib.fb_check(p, 1) == 0
    assert lib.fb_suggest_bias_grad_group(p) == 1      # B = 2
    p.B, p.H, p.Lq, p.Lk, p.r = 4096, 16, 256, 256, 16
    assert lib.fb_suggest_bias_grad_group(p) == 1      # the factors are not shared by the batch
    p.q_bias.stride_b = p.k_bias.stride_b = 0
    assert lib.fb_suggest_bias_grad_group(p) == 32     # whole windows at head dim 32: one workgroup per (batch, head)
    p.causal = 1
    assert lib.fb_suggest_bias_grad_group(p) == 8      # ... which causal calls are not
    p.causal, p.d = 0, 64
    assert lib.fb_suggest_bias_grad_group(p) == 8
    p.d = 32
    p.B = 256
    assert lib.fb_suggest_bias_grad_group(p) == 4      # still 1024 workgroups of 256 queries
    p.B = 64
    assert lib.fb_suggest_bias_grad_group(p) == 1
    p.B, p.Lq = 4096, 1024
    assert lib.fb_suggest_bias_grad_group(p) == 1      # long sequences keep one batch entry per workgroup
    p.Lq, p.r = 256, 0
    assert lib.fb_suggest_bias_grad_group(p) == 1
    assert lib.fb_suggest_bias_grad_group(None) == 1


@pytest.mark.parametrize("args,code", [
    ((None, 0x1000, 1, 1, 4, 64, 64), -1),
    ((0x1000, None, 1, 1, 4, 64, 64), -1),
    ((0x1000, 0x2000, 2, 2, 4, 64, 64), -3),   # fp32 in
    ((0x1000, 0x2000, 1, 0, 4, 64, 64), -3),   # bf16 in, fp16 out
    ((0x1000, 0x2000, 1, 1, 0, 64, 64), -2),
    ((0x1000, 0x2000, 1, 1, 4, 60, 64), -4),   # rows of 60 elements: not whole 16-byte chunks
    ((0x1000, 0x2000, 1, 1, 4, 64, 32), -4),   # rows would overlap
    ((0x1008, 0x2000, 1, 1, 4, 64, 64), -4),   # not 16-byte aligned
])
def test_sum_over_batch_rejects(args, code):
    lib = _lib.load()
    assert lib.fb_sum_over_batch(*args, None) == code  # rejected before any launch
    assert lib.fb_last_error() != b""


@pytest.mark.parametrize("args,code", [
    ((None, 0x2000, 10, 2, 16), -1), ((0x1000, None, 10, 2, 16), -1),
    ((0x1000, 0x2000, 0, 2, 16), -2), ((0x1000, 0x2000, 10, 0, 16), -2), ((0x1000, 0x2000, 10, 2, 5000), -2),
])
def test_resize_rank_rejects(args, code):
    lib = _lib.load()
    assert lib.fb_resize_rank(*args, None) == code  # rejected before any launch
    assert lib.fb_last_error() != b""


def test_null_params():
    lib = _lib.load()
    assert lib.fb_check(None, 0) == -1
    assert lib.fb_bwd(None, None) == -1


def test_params_struct_matches_header_size():
    # a wrong field order or type would change the size the library checks against
    p = _lib.new_params()
    assert p.size == ctypes.sizeof(_lib.FbParams)
    p.B = p.H = p.Lq = p.Lk = p.d = 1
    p.scale = 1.0
    assert _lib.load().fb_check(p, 0) == -1  # got past the ABI check, stopped at "q: null"
    assert b"q:" in _lib.load().fb_last_error()


def test_operator_rejects_cpu_and_fp32_inputs():
    """No CPU or fallback path: the host wrapper asserts like the reference's launcher
    (flash_bias/flash_bias_triton.py:1107-1109)."""
    q = torch.randn(1, 8, 1, 16, dtype=torch.bfloat16)
    with pytest.raises(AssertionError):
        flash_bias_func(q, q, q)
    with pytest.raises(AssertionError):
        flash_bias_func(q.float(), q.float(), q.float())
    with pytest.raises(AssertionError):
        flash_bias_func(q, q[:, :4], q)


def test_vector_mask_fold_respects_the_rank_limit():
    """Folding a key-padding mask into the factors adds a column before the rank is padded to a
    multiple of 8: rank 127 becomes 128, rank 128 would become 136, beyond what the library takes,
    and keeps the kernels' own mask path."""
    from flashbias_amd.interface import _fold_keeps_rank_in_range
    assert _fold_keeps_rank_in_range(None) and _fold_keeps_rank_in_range(8) and _fold_keeps_rank_in_range(120)
    assert _fold_keeps_rank_in_range(121) and _fold_keeps_rank_in_range(127)
    assert not _fold_keeps_rank_in_range(128)


def test_argument_checks_are_clean_under_sanitizers():
    """fb_checks.cpp (fb_check, the size queries) rebuilt with -fsanitize=address,undefined and driven
    with well-formed and malformed parameter blocks (flashbias_amd/csrc/sanitize_check.cpp)."""
    import os
    import subprocess
    csrc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "flashbias_amd", "csrc")
    subprocess.check_call(["make", "-C", csrc, "sanitize"], stdout=subprocess.DEVNULL)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:verify_asan_link_order=0")
    res = subprocess.run([os.path.join(csrc, "build", "sanitize_check")], capture_output=True, text=True, env=env)
    assert res.returncode == 0, res.stderr[-2000:]
    assert "clean" in res.stdout
