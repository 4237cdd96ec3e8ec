"""The committed golden vectors (tests/golden/*.npz, written by tests/golden/make_fixtures.py from
numpy float64 closed forms that share no code with `oracle/`) against the two CPU oracles and,
on the GPU, against the HIP kernels through flash_bias_func."""
import glob
import os

import numpy as np
import pytest
import torch

from oracle import blocked, eager

from _util import GRAD_TOL, O_TOL, errors

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "*.npz")))
NAMES = [os.path.splitext(os.path.basename(p))[0] for p in GOLDEN]
OUTS = ("o", "lse", "dq", "dk", "dv", "dq_bias", "dk_bias")


def _load(path):
    with np.load(path, allow_pickle=False) as z:
        ins = {n[3:]: torch.from_numpy(z[n]) for n in z.files if n.startswith("in_")}
        want = {n[4:]: torch.from_numpy(z[n]) for n in z.files if n.startswith("out_")}
        return ins, want, bool(int(z["causal"])), float(z["scale"])


def test_fixtures_are_present():
    assert len(GOLDEN) >= 8


@pytest.mark.parametrize("path", GOLDEN, ids=NAMES)
def test_eager_oracle_reproduces_the_golden_vectors(path):
    x, want, causal, scale = _load(path)
    args = (x["q"], x["k"], x["v"], x.get("q_bias"), x.get("k_bias"), x.get("mask"), causal, scale)
    o, dq, dk, dv, dqb, dkb = eager.flashbias_eager_grads(*args, x["do"], dtype=torch.float64)
    _, lse = eager.flashbias_eager(*args, dtype=torch.float64, return_lse=True)
    got = dict(o=o, lse=lse, dq=dq, dk=dk, dv=dv, dq_bias=dqb, dk_bias=dkb)
    for name in OUTS:
        if name in want:
            assert got[name].shape == want[name].shape, name
            assert torch.allclose(got[name].float(), want[name], rtol=2e-5, atol=2e-5), name
        else:
            assert got[name] is None, name


@pytest.mark.parametrize("path", GOLDEN, ids=NAMES)
def test_blocked_c_oracle_reproduces_the_golden_vectors(path):
    """The tile-by-tile recurrences (online softmax, P recomputed from the stored lse) in fp32,
    with tiles smaller than the sequences so that several are chained."""
    x, want, causal, scale = _load(path)
    args = (x["q"], x["k"], x["v"], x.get("q_bias"), x.get("k_bias"), x.get("mask"), causal, scale)
    o, lse = blocked.blocked_fwd(*args, block_m=16, block_n=16)
    dq, dk, dv, dqb, dkb = blocked.blocked_bwd(*args, o, lse, x["do"], block_m=16, block_n=16)
    got = dict(o=o, lse=lse, dq=dq, dk=dk, dv=dv, dq_bias=dqb, dk_bias=dkb)
    for name in OUTS:
        if name in want:
            err, rel = errors(got[name].float(), want[name])
            assert got[name].shape == want[name].shape and rel < 1e-4, (name, err, rel)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("path", GOLDEN, ids=NAMES)
def test_hip_kernels_reproduce_the_golden_vectors(gpu_device, path, dtype):
    """Tolerance of the metric: max-abs error on o 1e-2 (fp16) / 2e-2 (bf16), every gradient
    within 5e-2 of its largest entry.  The stored inputs are bf16-representable; fp16 cannot hold
    the -30000 of the key-padding mask's neighbours exactly but holds the values themselves."""
    from flashbias_amd import flash_bias_func
    x, want, causal, scale = _load(path)
    if dtype == torch.float16 and any((t.to(dtype).float() != t).any() for t in x.values()):
        pytest.skip("inputs of this case are not representable in fp16")
    dev = gpu_device
    names = [n for n in ("q", "k", "v", "q_bias", "k_bias") if n in x]
    leaves = {n: x[n].to(dtype).to(dev).requires_grad_(True) for n in names}
    mask = x["mask"].to(dtype).to(dev) if "mask" in x else None
    o = flash_bias_func(leaves["q"], leaves["k"], leaves["v"], leaves.get("q_bias"), leaves.get("k_bias"),
                        mask, causal, scale)
    grads = torch.autograd.grad(o, [leaves[n] for n in names], x["do"].to(dtype).to(dev))
    torch.cuda.synchronize()
    err, _ = errors(o.float().cpu(), want["o"])
    assert err <= O_TOL[dtype], ("o", err)
    for n, g in zip(names, grads):
        ref = want["d" + n]
        assert g.shape == ref.shape, n
        err, rel = errors(g.float().cpu(), ref)
        assert rel <= GRAD_TOL, ("d" + n, err, rel)
