"""Writes the golden vectors of tests/golden/*.npz.

The reference holds no golden vectors for flash_bias_func (its only check,
flash_bias/benchmark.py:22-215, prints differences), and its Triton kernels cannot run without a
GPU, so the vectors come from the mathematics: numpy float64, dense, the closed forms of
softmax attention with an additive bias written out with einsum, no autograd and no code shared
with `oracle/`:

    S  = scale q k^T + q_bias k_bias^T (+ mask) (+ causal -inf)     flash_bias_triton.py:243-282
    P  = softmax(S), lse = logsumexp(S), o = P v                    :283-329
    dv = P^T dO, dP = dO v^T, delta = rowsum(o * dO)                :696-705, :398
    dS = P * (dP - delta)                                           :711
    dq = scale dS k, dk = scale dS^T q                              :717, :725
    dq_bias = dS k_bias, dk_bias = dS^T q_bias                      :718-719, :725-790
    (a factor broadcast over batch or heads gets the sum over that dimension)

Inputs are seeded, generated in fp32, rounded once to bf16 (so that a 16-bit kernel sees exactly
the stored values) and stored as fp32.  Run from the repository root:

    python tests/golden/make_fixtures.py
"""
import math
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))

# name: B, Lq, Lk, H, d, r, causal, mask kind, (factor broadcast over batch, over heads), scale
CASES = {
    "square_d32_r8": (2, 48, 48, 2, 32, 8, False, None, (False, False), None),
    "causal_rect_d32_r8": (1, 40, 72, 3, 32, 8, True, None, (False, False), None),
    "ragged_d40_r5_scale": (2, 33, 19, 1, 40, 5, False, None, (False, False), 0.21),
    "vector_mask_d16_r2": (2, 24, 56, 2, 16, 2, False, "vec", (False, False), None),
    "matrix_mask_causal_d64_r16": (1, 36, 36, 2, 64, 16, True, "mat", (False, False), None),
    "broadcast_factors_d32_r16": (3, 32, 32, 2, 32, 16, False, None, (True, False), None),
    "shared_heads_d128_r32": (2, 20, 28, 3, 128, 32, False, None, (False, True), None),
    "no_factors_d32": (1, 50, 50, 2, 32, 0, True, None, (False, False), None),
}


def _round(x):
    return x.to(torch.bfloat16).to(torch.float64).numpy()


def inputs(name):
    B, Lq, Lk, H, d, r, causal, mkind, bc, scale = CASES[name]
    g = torch.Generator().manual_seed(1000 + sorted(CASES).index(name))
    out = {
        "q": _round(torch.randn(B, Lq, H, d, generator=g)),
        "k": _round(torch.randn(B, Lk, H, d, generator=g)),
        "v": _round(torch.randn(B, Lk, H, d, generator=g)),
        "do": _round(torch.randn(B, Lq, H, d, generator=g)),
    }
    if r:
        fb, fh = (1 if bc[0] else B), (1 if bc[1] else H)
        out["q_bias"] = _round(torch.randn(fb, Lq, fh, r, generator=g) / math.sqrt(r))
        out["k_bias"] = _round(torch.randn(fb, Lk, fh, r, generator=g) / math.sqrt(r))
    if mkind == "vec":
        m = torch.randn(B, 1, 1, Lk, generator=g)
        m[:, :, :, Lk - 5:] = -30000.0  # key padding, finite so that every row keeps some weight
        out["mask"] = _round(m)
    elif mkind == "mat":
        out["mask"] = _round(torch.randn(1, H, Lq, Lk, generator=g))
    return out, causal, (scale if scale is not None else 1.0 / math.sqrt(d))


def closed_forms(x, causal, scale):
    q, k, v, do = x["q"], x["k"], x["v"], x["do"]
    B, Lq, H, _ = q.shape
    Lk = k.shape[1]
    s = scale * np.einsum("bihc,bjhc->bhij", q, k)
    if "q_bias" in x:
        qb = np.broadcast_to(x["q_bias"], (B, Lq, H, x["q_bias"].shape[-1]))
        kb = np.broadcast_to(x["k_bias"], (B, Lk, H, x["k_bias"].shape[-1]))
        s = s + np.einsum("bihc,bjhc->bhij", qb, kb)
    if "mask" in x:
        s = s + x["mask"]
    if causal:
        s = np.where(np.arange(Lq)[:, None] >= np.arange(Lk)[None, :], s, -np.inf)
    mx = s.max(-1, keepdims=True)
    e = np.exp(s - mx)
    den = e.sum(-1, keepdims=True)
    p = e / den
    res = {"lse": (mx + np.log(den))[..., 0], "o": np.einsum("bhij,bjhc->bihc", p, v)}
    res["dv"] = np.einsum("bhij,bihc->bjhc", p, do)
    dp = np.einsum("bihc,bjhc->bhij", do, v)
    delta = np.einsum("bihc,bihc->bhi", res["o"], do)
    ds = p * (dp - delta[..., None])
    res["dq"] = scale * np.einsum("bhij,bjhc->bihc", ds, k)
    res["dk"] = scale * np.einsum("bhij,bihc->bjhc", ds, q)
    if "q_bias" in x:
        dqb = np.einsum("bhij,bjhc->bihc", ds, kb)
        dkb = np.einsum("bhij,bihc->bjhc", ds, qb)
        for name, full in (("dq_bias", dqb), ("dk_bias", dkb)):
            shape = x[name[1:]].shape
            if shape[0] == 1 and B > 1:
                full = full.sum(0, keepdims=True)
            if shape[2] == 1 and H > 1:
                full = full.sum(2, keepdims=True)
            res[name] = full
    return res


def main():
    for name in sorted(CASES):
        x, causal, scale = inputs(name)
        want = closed_forms(x, causal, scale)
        arrays = {"in_" + n: a.astype(np.float32) for n, a in x.items()}
        arrays.update({"out_" + n: a.astype(np.float32) for n, a in want.items()})
        arrays["causal"] = np.array(int(causal))
        arrays["scale"] = np.array(scale, dtype=np.float64)
        path = os.path.join(HERE, name + ".npz")
        np.savez_compressed(path, **arrays)
        print(name, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
