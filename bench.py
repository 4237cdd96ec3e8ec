#!/usr/bin/env python3
"""Benchmark of the FlashBias hot path on one MI355X.

A step is one forward + backward of ``flash_bias_func`` on the headline workload of the
reference's benchmark (flash_bias/config.py:12, flash_bias/benchmark.py:218-374): B2 H4 L16384
d32 r8, non-causal, bf16, synthetic seeded inputs already resident in HBM.  Prints ONE JSON
line:

  value        whole-step throughput in TFLOP/s, algorithmic FLOPs 2 B H L^2 (7d + 4r)
  ms_per_step  forward + backward wall time per step
  roofline     the dominant kernel (backward dk/dv) timed alone with events on its stream,
               against the dense bf16 MFMA peak
  cpu_baseline the eager oracle (restated reference eager attention) on the host cores, on a
               bounded sample of the same workload

``--report`` instead prints a table over the other named workloads (not part of the contract).
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 / fp16 MFMA
# HBM bytes of one dk/dv launch at the headline shape: rocprofv3 FETCH_SIZE (x2.0, calibrated on a copy of
# known size) + WRITE_SIZE, see profiles/headline_fwd_bwd_kernels.md; a counter figure, not measured live
DKV_HBM_BYTES = 1.71e8
PEAK_HBM_GBS = 8000.0


def _to_dev(w, dev):
    import torch
    return {n: (t.to(dev) if isinstance(t, torch.Tensor) else t) for n, t in w.items()}


def _time_events(fn, steps, warmup, isolated=False):
    """Average milliseconds of fn() measured with events on the current stream.  isolated: one
    event pair per call, so that the tail of one launch cannot overlap the head of the next (what
    a kernel trace reports as a launch's duration); otherwise one pair around all the calls
    (throughput of back-to-back launches)."""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    if isolated:
        pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
        for start, end in pairs:
            start.record()
            fn()
            end.record()
        torch.cuda.synchronize()
        return sum(start.elapsed_time(end) for start, end in pairs) / steps
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        fn()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / steps


def _phase_timers(w, dev):
    """Callables that launch the forward, the whole backward (fb_bwd: the dq kernel, which also
    forms delta, then the dk/dv kernel) and the three backward phases alone through the C ABI
    (buffers allocated once, outside the timed region)."""
    import torch
    from flashbias_amd import _lib
    from flashbias_amd.interface import _prepare, _stream, _tensor
    lib = _lib.load()
    q, k, v, qb, kb, do = (w[n] for n in ("q", "k", "v", "q_bias", "k_bias", "do"))
    p, keep = _prepare(q, k, v, qb, kb, w.get("mask"), w["causal"], w["softmax_scale"])
    o = torch.empty_like(q)
    lse = torch.empty((p.B, p.H, p.Lq), device=dev, dtype=torch.float32)
    p.o, p.lse = _tensor(o), lse.data_ptr()
    grads = [torch.empty_like(t) for t in (q, k, v)]
    p.dout, p.dq, p.dk, p.dv = _tensor(do), _tensor(grads[0]), _tensor(grads[1]), _tensor(grads[2])
    if qb is not None:
        full = [torch.empty((p.B, L, p.H, p.r), device=dev, dtype=q.dtype) for L in (p.Lq, p.Lk)]
        p.dq_bias, p.dk_bias = _tensor(full[0]), _tensor(full[1])
        keep += full
    delta = torch.empty((2,) + tuple(lse.shape), device=lse.device, dtype=torch.float32)  # -delta, lse*log2(e)
    p.delta = delta.data_ptr()
    keep += [o, lse, grads, delta]

    def call(fn):
        def run():
            _lib.check_status(fn(p, _stream()))
        return run
    return {name: call(getattr(lib, name)) for name in
            ("fb_fwd", "fb_bwd", "fb_bwd_preprocess", "fb_bwd_dkv", "fb_bwd_dq")}, keep


def _cpu_baseline(w, flops_per_slice):
    """Eager oracle, fp32, all host cores, on ONE (batch, head) slice of the workload at full
    sequence length (the (L, L) fp32 intermediates are 1 GiB each at L=16384)."""
    import torch
    from oracle import eager
    cores = os.cpu_count() or 1
    try:
        cores = len(os.sched_getaffinity(0))
    except AttributeError:
        pass
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    nslices = 2  # of the workload's B*H (batch, head) slices: about 13 s on 16 cores at L=16384
    dt = 0.0
    for h in range(nslices):
        sl = lambda t: t[:1, :, h:h + 1].float().cpu()
        args = (sl(w["q"]), sl(w["k"]), sl(w["v"]), sl(w["q_bias"]), sl(w["k_bias"]), None, w["causal"],
                w["softmax_scale"])
        do = sl(w["do"])
        t0 = time.perf_counter()
        eager.flashbias_eager_grads(*args, do)
        dt += time.perf_counter() - t0
    return {"value": round(nslices * flops_per_slice / dt / 1e12, 5), "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "seconds": round(dt, 2),
            "sample": "%d of B*H (batch, head) slices at full L, one fwd+bwd of the eager oracle in fp32 each" % nslices}


def headline(args):
    import torch
    from flashbias_amd import flash_bias_func, workloads
    dev = torch.device("cuda:0")
    hl = workloads.HEADLINE
    w = _to_dev(workloads.sweep(hl["L"], hl["B"], hl["H"], hl["d"], hl["r"], torch.bfloat16, seed=0), dev)
    leaves = [w[n].requires_grad_(True) for n in ("q", "k", "v", "q_bias", "k_bias")]

    def step():
        o = flash_bias_func(*leaves, None, False, w["softmax_scale"])
        return torch.autograd.grad(o, leaves, w["do"])

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / args.steps

    f_fwd, f_bwd = workloads.flops(hl["B"], hl["H"], hl["L"], hl["L"], hl["d"], hl["r"])
    phases, keep = _phase_timers({n: (t.detach() if isinstance(t, torch.Tensor) else t) for n, t in w.items()}, dev)
    ms = {name: _time_events(fn, args.steps, max(1, args.warmup), isolated=True) for name, fn in phases.items()}
    # dominant kernel: dk/dv/dk_bias.  Its algorithmic share of the backward: S recompute
    # (d + r), dP (d), dV (d), dK|dK_b (d + r) of the 2 B H L^2 (5d + 3r); the dq kernel carries
    # the dQ|dQ_b product (d + r) and, beyond the algorithmic count, a second S / dP recompute.
    f_dkv = 2.0 * hl["B"] * hl["H"] * hl["L"] * hl["L"] * (4 * hl["d"] + 2 * hl["r"])
    tflops_main = f_dkv / (ms["fb_bwd_dkv"] * 1e-3) / 1e12
    value = (f_fwd + f_bwd) / (ms_step * 1e-3) / 1e12
    ref_fwd, ref_fb = workloads.reference_formula_flops(hl["B"], hl["H"], hl["L"], hl["d"])
    out = {
        "metric": "fwd+bwd ms & TFLOP/s (% bf16 MFMA peak) at B2 H4 L16384 d32 r8, 1 GPU",
        "value": round(value, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "flash_bias_func fwd+bwd, B2 H4 L16384 d32 r8, non-causal, bf16 "
                               "(flash_bias/config.py:12 at len=16384)"},
        "pct_of_bf16_mfma_peak": round(100 * value / PEAK_BF16_TFLOPS, 2),
        "fwd_ms": round(ms["fb_fwd"], 4),
        "fwd_tflops": round(f_fwd / (ms["fb_fwd"] * 1e-3) / 1e12, 2),
        "bwd_ms": round(ms["fb_bwd"], 4),
        "kernel_ms": {k: round(v, 4) for k, v in ms.items()},
        "reference_formula_tflops": round(ref_fb / (ms_step * 1e-3) / 1e12, 2),
        "roofline": {"kernel": "bwd_dkv_kernel (fb_bwd_dkv)", "bound": "mfma", "achieved": round(tflops_main, 2),
                     "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": round(tflops_main / PEAK_BF16_TFLOPS, 4),
                     "traffic": DKV_HBM_BYTES},
    }
    del keep
    if not args.no_cpu:
        out["cpu_baseline"] = _cpu_baseline(w, (f_fwd + f_bwd) / (hl["B"] * hl["H"]))
    print(json.dumps(out))


def _sdpa_concat(w):
    """The reference's pure-PyTorch FlashBias (flash_bias/attention_func.py:188-237): fused SDPA
    over the concatenated features [q * scale, q_bias] / [k, k_bias] with scale 1."""
    import torch
    B, _, H, _ = w["q"].shape
    qb = w["q_bias"].expand(B, -1, H, -1)
    kb = w["k_bias"].expand(B, -1, H, -1)
    qc = torch.cat([w["q"] * w["softmax_scale"], qb], -1)
    kc = torch.cat([w["k"], kb], -1)
    pad = (-qc.shape[-1]) % 8
    if pad:
        qc = torch.nn.functional.pad(qc, (0, pad))
        kc = torch.nn.functional.pad(kc, (0, pad))
    return torch.nn.functional.scaled_dot_product_attention(
        qc.transpose(1, 2), kc.transpose(1, 2), w["v"].transpose(1, 2), is_causal=w["causal"], scale=1.0).transpose(1, 2)


def _sdpa_dense(w, bias):
    """SDPA with the materialised (B, H, Lq, Lk) bias as attn_mask (attention_func.py:150-185)."""
    import torch
    return torch.nn.functional.scaled_dot_product_attention(
        w["q"].transpose(1, 2), w["k"].transpose(1, 2), w["v"].transpose(1, 2), attn_mask=bias,
        scale=w["softmax_scale"]).transpose(1, 2)


def _time_torch(make_out, leaves, do, steps, warmup):
    """fwd and fwd+bwd milliseconds of a torch provider."""
    import torch
    fwd = _time_events(lambda: make_out(), steps, warmup)

    def fb():
        torch.autograd.grad(make_out(), leaves, do)
    return fwd, _time_events(fb, steps, warmup)


def report(args):
    """fwd / fwd+bwd milliseconds and TFLOP/s over the named workloads, next to what PyTorch-ROCm
    offers for the same math (SDPA on concatenated features; SDPA with a dense bias where the
    N x N bias fits comfortably).  Informational, not part of the one-line contract."""
    import torch
    from flashbias_amd import workloads
    dev = torch.device("cuda:0")
    rows = []
    cases = [(f"sweep L={L}", lambda L=L: workloads.sweep(L), True) for L in workloads.SWEEP_LENGTHS]
    cases += [(f"alibi causal L={L}", lambda L=L: workloads.alibi(L), False) for L in (2048, 4096, 8192)]
    cases += [("swin 4096x256 r16", lambda: workloads.swin(), False), ("pde N=32768 r5", lambda: workloads.pde(), False),
              ("pairformer 768 r32", lambda: workloads.pairformer(), False),
              ("swin 4096x256 r16 + shifted-window mask", lambda: workloads.swin(shifted_types=64), None),
              ("sweep L=4096 + vector mask", lambda: workloads.masked(4096, "vector"), None),
              ("sweep L=4096 + matrix mask", lambda: workloads.masked(4096, "matrix"), None)]
    # other head dims and ranks at L=8192, and a causal language-model-like shape
    cases += [(f"sweep L=8192 d={d} r={r}", lambda d=d, r=r: workloads.sweep(8192, d=d, r=r), None)
              for d, r in ((64, 8), (64, 32), (64, 64), (128, 8), (128, 64))]
    cases += [("causal B4 H32 L=4096 d=128 r8", lambda: workloads.sweep(4096, B=4, H=32, d=128, causal=True), None)]
    for name, make, dense in cases:
        w = _to_dev(make(), dev)
        B, Lq, H, d = w["q"].shape
        r = w["q_bias"].shape[-1]
        f_fwd, f_bwd = workloads.flops(B, H, Lq, w["k"].shape[1], d, r, w["causal"])
        phases, keep = _phase_timers(w, dev)
        ms = {n: _time_events(fn, args.steps, args.warmup) for n, fn in phases.items()}
        ours_fwd = ms["fb_fwd"]
        ours_fb = ours_fwd + ms["fb_bwd"]
        del keep
        leaves = [w[n].requires_grad_(True) for n in ("q", "k", "v", "q_bias", "k_bias")]
        cat_fwd = cat_fb = den_fwd = den_fb = float("nan")
        if dense is not None:  # the comparison providers are timed on the unmasked workloads only
            cat_fwd, cat_fb = _time_torch(lambda: _sdpa_concat(w), leaves, w["do"], args.steps, args.warmup)
        if dense:
            with torch.no_grad():
                bias = (w["q_bias"].permute(0, 2, 1, 3) @ w["k_bias"].permute(0, 2, 3, 1)).contiguous()
            den_fwd, den_fb = _time_torch(lambda: _sdpa_dense(w, bias), leaves[:3], w["do"], args.steps, args.warmup)
            del bias
        rows.append((name, ours_fwd, f_fwd / ours_fwd / 1e9, ours_fb, (f_fwd + f_bwd) / ours_fb / 1e9, cat_fwd, cat_fb,
                     den_fwd, den_fb))
        del w, leaves
        torch.cuda.empty_cache()
    print("| workload | fwd ms | fwd TFLOP/s | fwd+bwd ms | fwd+bwd TFLOP/s | % bf16 peak | SDPA-concat fwd / fwd+bwd ms "
          "| SDPA dense-bias fwd / fwd+bwd ms |")
    print("|---|---|---|---|---|---|---|---|")
    for name, a, b, c, d_, e, f, g, h in rows:
        print(f"| {name} | {a:.3f} | {b:.1f} | {c:.3f} | {d_:.1f} | {100 * d_ / PEAK_BF16_TFLOPS:.1f} | {e:.3f} / {f:.3f} "
              f"| {g:.3f} / {h:.3f} |")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--report", action="store_true", help="table over all named workloads")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="before the run, copy a 256 MiB buffer 3 times (a plain copy kernel of known size, "
                         "used to scale the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the path has no collective; (batch, head) pairs are "
                 "independent and would be split across GPUs with no exchange. Run with --gpus 1.")
    from flashbias_amd import _lib
    _lib.load()  # fail loudly if the HIP library is not built
    if args.calibrate_copy:
        import torch
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda:0").fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if args.report:
        report(args)
    else:
        headline(args)


if __name__ == "__main__":
    main()
