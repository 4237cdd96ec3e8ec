"""Shared helpers of the GPU parity tests: seeded inputs (generated in fp32 on the CPU, rounded
to the test dtype once, so that the CPU oracle and the GPU kernels see identical values) and
the tolerance gate."""
import math

import torch

from oracle import eager

# max-abs error allowed on o (fp16 / bf16) and max|err| / max|ref| allowed on every gradient
O_TOL = {torch.float16: 1e-2, torch.bfloat16: 2e-2}
GRAD_TOL = 5e-2


def make_inputs(B, Lq, Lk, H, d, r, dtype, seed=0, bq=(False, False), bk=(False, False)):
    """q, k, v ~ N(0,1); q_bias, k_bias ~ N(0,1)/sqrt(r); dO ~ N(0,1).  bq / bk = (broadcast
    over batch, broadcast over heads) for the two factors."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Lq, H, d, generator=g).to(dtype)
    k = torch.randn(B, Lk, H, d, generator=g).to(dtype)
    v = torch.randn(B, Lk, H, d, generator=g).to(dtype)
    do = torch.randn(B, Lq, H, d, generator=g).to(dtype)
    qb = kb = None
    if r:
        qb = (torch.randn(1 if bq[0] else B, Lq, 1 if bq[1] else H, r, generator=g) / math.sqrt(r)).to(dtype)
        kb = (torch.randn(1 if bk[0] else B, Lk, 1 if bk[1] else H, r, generator=g) / math.sqrt(r)).to(dtype)
    return q, k, v, qb, kb, do


def oracle(q, k, v, qb, kb, mask, causal, scale, do):
    """(o, lse, dq, dk, dv, dq_bias, dk_bias) in fp32 on the CPU from the rounded inputs."""
    f = lambda t: None if t is None else t.detach().float().cpu()
    args = (f(q), f(k), f(v), f(qb), f(kb), f(mask), causal, scale)
    res = eager.flashbias_eager_grads(*args, f(do), dtype=torch.float32)
    _, lse = eager.flashbias_eager(*args, dtype=torch.float32, return_lse=True)
    return (res[0], lse) + tuple(res[1:])


def run_gpu(fn, q, k, v, qb, kb, mask, causal, scale, do, device):
    """o and the five gradients from the operator under test, as fp32 CPU tensors."""
    leaves = [t.to(device).requires_grad_(True) for t in (q, k, v)]
    if qb is not None:
        leaves += [t.to(device).requires_grad_(True) for t in (qb, kb)]
    qq, kk, vv = leaves[:3]
    bb = leaves[3:] if qb is not None else [None, None]
    m = None if mask is None else mask.to(device)
    o = fn(qq, kk, vv, bb[0], bb[1], m, causal, scale)
    grads = torch.autograd.grad(o, leaves, do.to(device))
    torch.cuda.synchronize()
    out = [o.detach().float().cpu()] + [g_.float().cpu() for g_ in grads]
    while len(out) < 6:
        out.append(None)
    return out


def errors(got, want):
    """max-abs error and error relative to max|want|."""
    err = (got - want).abs().max().item()
    return err, err / max(want.abs().max().item(), 1e-30)
