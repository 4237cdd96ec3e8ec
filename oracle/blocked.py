"""ctypes binding of ``oracle/blocked.c`` (test infrastructure, never shipped).

Runs the plain-C fp32 restatement of the reference's tiled forward / backward
(flash_bias/flash_bias_triton.py:128-355, :358-400, :450-869) on CPU tensors.
"""
import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


class _T(ctypes.Structure):
    _fields_ = [("p", ctypes.c_void_p), ("sb", ctypes.c_int64), ("sh", ctypes.c_int64),
                ("ss", ctypes.c_int64)]


class _Params(ctypes.Structure):
    _fields_ = ([(n, ctypes.c_int32) for n in
                 ("B", "H", "Lq", "Lk", "d", "r", "causal", "mask_type", "block_m", "block_n")]
                + [("scale", ctypes.c_float)]
                + [(n, _T) for n in ("q", "k", "v", "qb", "kb", "o", "dO", "dq", "dk", "dv",
                                     "dqb", "dkb", "mask")]
                + [("lse", ctypes.c_void_p), ("delta", ctypes.c_void_p)])


def build():
    subprocess.check_call(["make", "-s", "-C", _HERE, "libfb_oracle.so"])


def _lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "libfb_oracle.so")
        if not os.path.exists(path):
            build()
        _LIB = ctypes.CDLL(path)
        assert _LIB.fbo_params_size() == ctypes.sizeof(_Params)
    return _LIB


def _t(x, batch=None, nheads=None):
    """(B|1, L, H|1, c) fp32 tensor -> pointer + (batch, head, seq) strides, 0 where broadcast."""
    if x is None:
        return _T(None, 0, 0, 0)
    assert x.dtype == torch.float32 and x.stride(-1) == 1 and not x.is_cuda
    sb = x.stride(0) if (batch is None or x.shape[0] == batch) and x.shape[0] > 1 else 0
    sh = x.stride(2) if (nheads is None or x.shape[2] == nheads) and x.shape[2] > 1 else 0
    return _T(x.data_ptr(), sb, sh, x.stride(1))


def _mask(mask, batch, nheads, lq, lk):
    if mask is None:
        return None, 0, _T(None, 0, 0, 0)
    assert mask.dim() == 4 and mask.shape[3] == lk
    m = mask.float().contiguous()
    mtype = 1 if m.shape[2] == 1 and lq != 1 else 2
    sb = m.stride(0) if m.shape[0] > 1 else 0
    sh = m.stride(1) if m.shape[1] > 1 else 0
    return m, mtype, _T(m.data_ptr(), sb, sh, m.stride(2) if mtype == 2 else 0)


def _common(q, k, v, q_bias, k_bias, mask, causal, softmax_scale, block_m, block_n):
    batch, lq, nheads, d = q.shape
    lk = k.shape[1]
    P = _Params()
    P.B, P.H, P.Lq, P.Lk, P.d = batch, nheads, lq, lk, d
    P.r = 0 if q_bias is None else q_bias.shape[-1]
    P.causal = int(bool(causal))
    P.block_m, P.block_n = block_m, block_n
    P.scale = softmax_scale or d ** -0.5
    keep = [t.float().contiguous() if t is not None else None for t in (q, k, v, q_bias, k_bias)]
    P.q, P.k, P.v = _t(keep[0]), _t(keep[1]), _t(keep[2])
    P.qb, P.kb = _t(keep[3], batch, nheads), _t(keep[4], batch, nheads)
    m, P.mask_type, P.mask = _mask(mask, batch, nheads, lq, lk)
    keep.append(m)
    return P, keep


def blocked_fwd(q, k, v, q_bias=None, k_bias=None, mask=None, causal=False, softmax_scale=None,
                block_m=64, block_n=64):
    """Returns (o fp32 (B, Lq, H, d), lse fp32 (B, H, Lq))."""
    P, keep = _common(q, k, v, q_bias, k_bias, mask, causal, softmax_scale, block_m, block_n)
    o = torch.empty_like(keep[0])
    lse = torch.empty(P.B, P.H, P.Lq, dtype=torch.float32)
    P.o, P.lse = _t(o), lse.data_ptr()
    rc = _lib().fbo_fwd(ctypes.byref(P))
    assert rc == 0
    return o, lse


def blocked_bwd(q, k, v, q_bias, k_bias, mask, causal, softmax_scale, o, lse, do,
                block_m=64, block_n=64):
    """Returns (dq, dk, dv, dq_bias, dk_bias) fp32; factor grads have the factors' own
    (possibly broadcast) shapes."""
    P, keep = _common(q, k, v, q_bias, k_bias, mask, causal, softmax_scale, block_m, block_n)
    o32, do32, lse32 = o.float().contiguous(), do.float().contiguous(), lse.float().contiguous()
    delta = torch.empty_like(lse32)
    grads = [torch.zeros_like(t) if t is not None else None for t in keep[:5]]
    P.o, P.dO, P.lse, P.delta = _t(o32), _t(do32), lse32.data_ptr(), delta.data_ptr()
    P.dq, P.dk, P.dv = _t(grads[0]), _t(grads[1]), _t(grads[2])
    P.dqb, P.dkb = _t(grads[3], P.B, P.H), _t(grads[4], P.B, P.H)
    lib = _lib()
    assert lib.fbo_delta(ctypes.byref(P)) == 0
    assert lib.fbo_bwd(ctypes.byref(P)) == 0
    return tuple(grads)
