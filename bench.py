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

The same line carries, beyond the contract's fields: ``gate`` (the tolerance gate of the metric
evaluated on the very tensors of the timed steps: a subset of query rows against the CPU oracle
plus the size-independent checksums), ``sweep`` (forward and forward + backward milliseconds of
every benchmark configuration at its stated size, timed through ``flash_bias_func`` and autograd,
so that gradient reduction over broadcast factors, rank padding and mask folding are inside),
``modules`` (forward and forward + backward milliseconds of the two module drop-ins, projections included),
``fp16`` (the headline step in fp16, the dtype of the reference's published numbers),
``factors_permuted_inside`` (the headline step with the (B, H, L, r) -> (B, L, H, r)
``permute().contiguous()`` of the factors inside the timed region, as flash_bias/benchmark.py:233-235
times it) and ``providers`` (what PyTorch-ROCm offers for the same math at the headline shape).

``--report`` instead prints a table over more workloads (not part of the contract).
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
PEAK_HBM_GBS = 8000.0
MIN_WARM_SECONDS = 0.1  # of untimed calls before every event-timed measurement (_time_events)
PROFILE_SUMMARY = os.path.join(ROOT, "profiles", "headline_fwd_bwd_kernels.md")


def _profiled(key, kernel):
    """A figure of `kernel` at the headline shape as the tracked rocprofv3 summary states it, a line
    `<key> <kernel> <value>`: `hbm_bytes_per_launch` (FETCH_SIZE and WRITE_SIZE counters scaled by a copy
    of known size) or `avg_launch_ns` (the kernel trace's average duration); None when the summary has no
    such line.  Figures of the profiled run, not measured live."""
    try:
        with open(PROFILE_SUMMARY) as f:
            for line in f:
                parts = line.split()
                if len(parts) >= 3 and parts[0] == key and parts[1] == kernel:
                    return float(parts[2])
    except OSError:
        pass
    return None


def _to_dev(w, dev):
    import torch
    return {n: (t.to(dev) if isinstance(t, torch.Tensor) else t) for n, t in w.items()}


def _time_events(fn, steps, warmup, isolated=False):
    """Average milliseconds of fn() measured with events on the current stream.  isolated: one
    event pair per call, so that the tail of one launch cannot overlap the head of the next (what
    a kernel trace reports as a launch's duration); otherwise one pair around all the calls
    (throughput of back-to-back launches)."""
    import torch
    t0 = time.perf_counter()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    # (whatever ran before may have left the GPU idle for a while, building inputs on the host for instance: at
    # least a tenth of a second of calls before anything is timed)
    while time.perf_counter() - t0 < MIN_WARM_SECONDS:
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
    from flashbias_amd.interface import _params, _stream, _tensor
    lib = _lib.load()
    q, k, v, qb, kb, do = (w[n] for n in ("q", "k", "v", "q_bias", "k_bias", "do"))
    p, keep = _params(q, k, v, qb, kb, w.get("mask"), w["causal"], w["softmax_scale"])
    o = torch.empty_like(q)
    lse = torch.empty((p.B, p.H, p.Lq), device=dev, dtype=torch.float32)
    p.o, p.lse = _tensor(o), lse.data_ptr()
    grads = [torch.empty_like(t) for t in (q, k, v)]
    p.dout, p.dq, p.dk, p.dv = _tensor(do), _tensor(grads[0]), _tensor(grads[1]), _tensor(grads[2])
    if qb is not None:
        full = [torch.empty((p.B, L, p.H, p.r), device=dev, dtype=q.dtype) for L in (p.Lq, p.Lk)]
        p.dq_bias, p.dk_bias = _tensor(full[0]), _tensor(full[1])
        keep += full
    delta = torch.empty(lib.fb_bwd_workspace_bytes(p) // 4, device=lse.device, dtype=torch.float32)  # backward scratch
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


def _autograd_ms(leaves, extra, do, steps, warmup, prepare=None):
    """fwd and fwd+bwd milliseconds of flash_bias_func through autograd (events on the current
    stream around all the steps).  prepare: work done inside the timed region before the call
    (returns the factor pair to use)."""
    import torch
    from flashbias_amd import flash_bias_func
    mask, causal, scale = extra

    def fwd():
        fac = prepare() if prepare else leaves[3:5]
        return flash_bias_func(leaves[0], leaves[1], leaves[2], fac[0], fac[1], mask, causal, scale)

    def fb():
        return torch.autograd.grad(fwd(), leaves, do)

    with torch.no_grad():
        t_fwd = _time_events(fwd, steps, warmup)
    return t_fwd, _time_events(fb, steps, warmup)


def _constant_factors_ms(leaves, extra, do, steps, warmup):
    """fwd+bwd milliseconds of the same step when the factors are constants (no gradient asked of them,
    as in the reference's own applications: ALiBi slopes, attention_with_alibi_bias.py:44-52; tables
    loaded from a file, swin_transformer_v2.py:147-152): the operator then computes dq, dk, dv only."""
    import torch
    from flashbias_amd import flash_bias_func
    mask, causal, scale = extra
    fac = [t.detach() for t in leaves[3:5]]

    def fb():
        o = flash_bias_func(leaves[0], leaves[1], leaves[2], fac[0], fac[1], mask, causal, scale)
        return torch.autograd.grad(o, leaves[:3], do)

    return _time_events(fb, steps, warmup)


def _graph_ms(leaves, extra, do, steps, warmup):
    """fwd+bwd milliseconds of the same autograd step captured once in a HIP graph and replayed: what
    a training loop that captures its step pays, without the host's per-call work (which bounds the
    eager figure when the kernels of a step take less than about 0.1 ms).  Every replay's gradients
    are compared with the eager step's bit for bit; returns None if they differ or capture fails."""
    import torch
    from flashbias_amd import flash_bias_func
    mask, causal, scale = extra

    def step():
        o = flash_bias_func(leaves[0], leaves[1], leaves[2], leaves[3], leaves[4], mask, causal, scale)
        return torch.autograd.grad(o, leaves, do)

    eager = [g.clone() for g in step()]
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                step()
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            grads = step()
        for _ in range(max(1, warmup)):
            graph.replay()
            torch.cuda.synchronize()
            if not all(torch.equal(a, b) for a, b in zip(grads, eager)):
                return None
        ms = _time_events(graph.replay, steps, 0)
        torch.cuda.synchronize()
        if not all(torch.equal(a, b) for a, b in zip(grads, eager)):
            return None
        return ms
    except RuntimeError:
        return None


def _device_configs(dev):
    """(name, builder) of every benchmark configuration at its stated size; q, k, v, dO are drawn on
    the device (timing does not depend on the values), the factors come from the builders."""
    import torch
    from flashbias_amd import factors

    def base(B, L, H, d, dtype=torch.bfloat16):
        return [torch.randn(B, L, H, d, device=dev).to(dtype) for _ in range(4)]

    def sweep(L):
        q, k, v, do = base(2, L, 4, 32)
        qb, kb = [(torch.randn(2, L, 4, 8, device=dev) / math.sqrt(8)).bfloat16() for _ in range(2)]
        return q, k, v, qb, kb, do, False, 8

    def alibi(L):
        q, k, v, do = base(1, L, 50, 32)
        qb, kb = factors.alibi_factors(L, L, 50, torch.bfloat16, device=dev)
        return q, k, v, qb, kb, do, True, 2

    def swin():
        q, k, v, do = base(4096, 256, 16, 32)
        qb, kb, _ = factors.svd_factors(factors.swin_v2_bias_table(16, 16, 0), 16, torch.bfloat16)
        return q, k, v, qb.to(dev), kb.to(dev), do, False, 16

    def pde():
        q, k, v, do = base(1, 32768, 8, 32)
        x = torch.rand(1, 32768, 3, device=dev)
        # (terms of at most 2 alpha: the caller pads its constant factors to rank 8 once, which selects the rank-8 kernels)
        qb, kb = factors.pad_rank(*factors.distance_factors(x, x, 10.0, torch.bfloat16), 8)
        return q, k, v, qb, kb, do, False, 5

    def pairformer():
        q, k, v, do = base(768, 768, 4, 32)
        qb, kb = [(torch.randn(1, 768, 4, 32, device=dev) / math.sqrt(32)).bfloat16() for _ in range(2)]
        return q, k, v, qb, kb, do, False, 32

    # (the reference's own sweep starts at 2^8, flash_bias/config.py:17)
    cfgs = [(f"sweep B2 H4 d32 r8 L={L}", lambda L=L: sweep(L)) for L in (256, 512, 1024, 2048, 4096, 8192, 16384)]
    cfgs += [(f"alibi causal B1 H50 d32 r2 L={L}", lambda L=L: alibi(L)) for L in (2048, 4096, 8192)]
    cfgs += [("swin 4096 windows x 256 H16 d32 r16 (factors shared by the windows)", swin),
             ("pde N=32768 H8 d32 r5 (factors shared by the heads)", pde),
             ("pairformer 768 x 768 H4 d32 r32 (factors shared by the rows)", pairformer)]
    return cfgs


def _swin_accuracy(dev):
    """What configuration 4 asks to be reported beside its timings: how well the rank-16 factors reproduce the
    bias table (relative Frobenius error, worst head) and how far the operator's output is from the attention
    with the dense table and from the oracle on the same factors (eight windows, fp32 oracle on the CPU)."""
    import torch
    from flashbias_amd import flash_bias_func, workloads
    from oracle import eager
    w = workloads.swin(windows=8)
    with torch.no_grad():
        o = flash_bias_func(*(w[n].to(dev) for n in ("q", "k", "v", "q_bias", "k_bias")), None, False,
                            w["softmax_scale"]).float().cpu()
    f = lambda n: w[n].float()
    dense = eager.attention_eager(f("q"), f("k"), f("v"), w["softmax_scale"], w["bias_table"][None].expand(8, -1, -1, -1))
    same = eager.flashbias_eager(f("q"), f("k"), f("v"), f("q_bias"), f("k_bias"), None, False, w["softmax_scale"])
    return {"bias_reconstruction_rel_error": round(float(w["bias_rel_error"].max()), 5),
            "o_max_abs_err_vs_dense_table": round(float((o - dense).abs().max()), 5),
            "o_max_abs_err_vs_oracle_on_the_factors": round(float((o - same).abs().max()), 5)}


def _sweep(dev, steps, warmup, only=None):
    import torch
    from flashbias_amd import workloads
    out = []
    for name, build in _device_configs(dev):
        if only is not None and only not in name:
            continue
        q, k, v, qb, kb, do, causal, r = build()
        B, L, H, d = q.shape
        leaves = [t.requires_grad_(True) for t in (q, k, v, qb, kb)]
        t_fwd, t_fb = _autograd_ms(leaves, (None, causal, 1.0 / math.sqrt(d)), do, steps, warmup)
        t_graph = _graph_ms(leaves, (None, causal, 1.0 / math.sqrt(d)), do, steps, warmup)
        t_const = _constant_factors_ms(leaves, (None, causal, 1.0 / math.sqrt(d)), do, steps, warmup)
        f_fwd, f_bwd = workloads.flops(B, H, L, L, d, r, causal)
        # algorithmic HBM bytes of a step: every input read once per pass, every output written once
        # (forward: q k v factors -> o, lse; backward: q k v o dO factors lse -> dq dk dv and the factor
        # gradients in the factors' own shapes)
        size = lambda *ts: sum(t.numel() * t.element_size() for t in ts)
        lse_bytes = 4 * B * H * L
        hbm = (size(q, k, v, qb, kb) + size(q) + lse_bytes) + (size(q, k, v, q, do, qb, kb) + lse_bytes + size(q, k, v, qb, kb))
        out.append({"workload": name, "fwd_ms": round(t_fwd, 4), "fwd_bwd_ms": round(t_fb, 4),
                    "fwd_tflops": round(f_fwd / t_fwd / 1e9, 1), "fwd_bwd_tflops": round((f_fwd + f_bwd) / t_fb / 1e9, 1),
                    "pct_of_bf16_mfma_peak": round(100 * (f_fwd + f_bwd) / t_fb / 1e9 / PEAK_BF16_TFLOPS, 2),
                    "fwd_bwd_graph_ms": None if t_graph is None else round(t_graph, 4),
                    "graph_pct_of_bf16_mfma_peak": None if t_graph is None else
                    round(100 * (f_fwd + f_bwd) / t_graph / 1e9 / PEAK_BF16_TFLOPS, 2),
                    # (not comparable with fwd_bwd_ms: two of the five gradients are not computed)
                    "fwd_bwd_ms_constant_factors": round(t_const, 4),
                    "hbm_algorithmic_gb": round(hbm / 1e9, 3), "hbm_gbs": round(hbm / t_fb / 1e6, 1),
                    "pct_of_hbm_peak": round(100 * hbm / t_fb / 1e6 / PEAK_HBM_GBS, 2)})
        del q, k, v, qb, kb, do, leaves
        torch.cuda.empty_cache()
        if name.startswith("swin"):
            out[-1].update(_swin_accuracy(dev))
    return out


def _modules(dev, steps, warmup):
    """Layer-level timing of the two module drop-ins (flashbias_amd/modules.py) at the sizes of the benchmark
    configurations they belong to: the ALiBi causal self-attention block
    (1_Language_Model/attention_with_alibi_bias.py:18-64) at B1 L=4096 H50 x 32 and the Swin-V2 window attention
    core (2_Vision_Transformer/swin_transformer_v2.py:155-207) on 4096 windows of 256 tokens, H16 x 32, rank 16.
    bf16 parameters and activations, forward and forward + backward (gradient of the input and of every
    parameter), the projections of the layer included."""
    import torch
    from flashbias_amd import modules
    out = {}
    cases = [("AttentionWithALiBiBias B1 L=4096 dim=1600 (H50 x 32), causal, exact rank-4 factors",
              lambda: modules.AttentionWithALiBiBias(1600, 50, 32), (1, 4096, 1600)),
             ("WindowAttentionCore 4096 windows x 256 tokens dim=512 (H16 x 32), rank 16",
              lambda: modules.WindowAttentionCore(512, 16, 16, rank=16), (4096, 256, 512))]
    for name, make, shape in cases:
        torch.manual_seed(0)
        mod = make().to(dev).to(torch.bfloat16)
        x = torch.randn(*shape, device=dev, dtype=torch.bfloat16, requires_grad=True)
        dy = torch.randn(*shape, device=dev, dtype=torch.bfloat16)
        params = [x] + [p for p in mod.parameters() if p.requires_grad]
        with torch.no_grad():
            t_fwd = _time_events(lambda: mod(x), steps, warmup)
        t_fb = _time_events(lambda: torch.autograd.grad(mod(x), params, dy), steps, warmup)
        out[name] = {"fwd_ms": round(t_fwd, 4), "fwd_bwd_ms": round(t_fb, 4)}
        del mod, x, dy, params
        torch.cuda.empty_cache()
    return out


def _gate(w, o, grads):
    """The tolerance gate of the metric on the tensors of a timed step: o, dq, dq_bias of 192 query
    rows against the CPU oracle run on (those rows, all keys); dk, dv, dk_bias through the
    identities sum_j dv_j = sum_i dO_i and sum_j dk_j = 0 = sum_j dk_bias_j."""
    import torch
    from oracle import eager
    L = w["q"].shape[1]
    rows = torch.cat([torch.arange(0, 64), torch.arange(L // 2 - 32, L // 2 + 32), torch.arange(L - 64, L)])
    f = lambda t: t.detach().float().cpu()
    sub = lambda t: f(t[:, rows])
    ref = eager.flashbias_eager_grads(sub(w["q"]), f(w["k"]), f(w["v"]), sub(w["q_bias"]), f(w["k_bias"]), None, False,
                                      w["softmax_scale"], sub(w["do"]))
    rel = lambda got, want: ((f(got) - want).abs().max() / want.abs().max()).item()
    o_err = (f(o[:, rows]) - ref[0]).abs().max().item()
    ratios = {"dq": rel(grads[0][:, rows], ref[1]), "dq_bias": rel(grads[3][:, rows], ref[4])}
    do_sum = w["do"].float().sum(1)
    ratios["dv (column sums)"] = ((grads[2].float().sum(1) - do_sum).abs().max() / do_sum.abs().max()).item()
    for name, gk in (("dk (column sums)", grads[1]), ("dk_bias (column sums)", grads[4])):
        gk = gk.float()
        ratios[name] = (gk.sum(1).abs().max() / (gk.abs().sum(1).max() / math.sqrt(gk.shape[1]))).item()
    ok = (o_err <= 2e-2 and ratios["dq"] <= 5e-2 and ratios["dq_bias"] <= 5e-2 and ratios["dv (column sums)"] <= 2e-2
          and ratios["dk (column sums)"] <= 16 * 2.0 ** -9 and ratios["dk_bias (column sums)"] <= 16 * 2.0 ** -9)
    return {"pass": bool(ok), "o_max_abs_err": round(o_err, 5), "o_tol": 2e-2, "grad_tol": 5e-2,
            "ratios": {k: round(v, 5) for k, v in ratios.items()},
            "checked": "192 query rows x all keys of o, dq, dq_bias against the fp32 CPU oracle; column sums of dv, dk, dk_bias"}


PRIME_SECONDS = 1.0  # untimed steps before the warm-up steps of the headline measurement (see headline())


def headline(args):
    import torch
    from flashbias_amd import flash_bias_func, workloads
    dev = torch.device("cuda:0")
    hl = workloads.HEADLINE
    w = _to_dev(workloads.sweep(hl["L"], hl["B"], hl["H"], hl["d"], hl["r"], torch.bfloat16, seed=0), dev)
    leaves = [w[n].requires_grad_(True) for n in ("q", "k", "v", "q_bias", "k_bias")]

    def step():
        o = flash_bias_func(*leaves, None, False, w["softmax_scale"])
        return o, torch.autograd.grad(o, leaves, w["do"])

    # A GPU that has been idle (this process has only generated the inputs so far) takes tens of milliseconds under
    # load to reach the state it then holds, longer than W warm-up steps of 1.7 ms last (same box, 20 timed steps
    # after 5 warm-up steps: 1.71-1.73 ms per step from idle, 1.67 after a quarter of a second of steps, 1.66
    # after one second): the first second of steps is not part of the measurement (stated in the line as
    # `primed_s`); the W warm-up steps and the K timed steps follow it directly.
    t_prime = time.perf_counter()
    while time.perf_counter() - t_prime < PRIME_SECONDS:
        step()
        torch.cuda.synchronize()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        last = step()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / args.steps
    gate = _gate(w, last[0].detach(), last[1])
    del last

    f_fwd, f_bwd = workloads.flops(hl["B"], hl["H"], hl["L"], hl["L"], hl["d"], hl["r"])
    phases, keep = _phase_timers({n: (t.detach() if isinstance(t, torch.Tensor) else t) for n, t in w.items()}, dev)
    # (the gate above kept the host busy and the GPU idle for seconds: as before the timed steps, half a second of
    # steps first, so that the first phase timed is not the one that finds the GPU cold)
    t_prime = time.perf_counter()
    while time.perf_counter() - t_prime < 0.5 * PRIME_SECONDS:
        step()
        torch.cuda.synchronize()
    ms = {name: _time_events(fn, args.steps, max(1, args.warmup), isolated=True) for name, fn in phases.items()}
    fwd_row = _time_events(phases["fb_fwd"], args.steps, max(1, args.warmup))
    # dominant kernel: dk/dv/dk_bias.  Its algorithmic share of the backward: S recompute
    # (d + r), dP (d), dV (d), dK|dK_b (d + r) of the 2 B H L^2 (5d + 3r); the dq kernel carries
    # the dQ|dQ_b product (d + r) and, beyond the algorithmic count, a second S / dP recompute.
    f_dkv = 2.0 * hl["B"] * hl["H"] * hl["L"] * hl["L"] * (4 * hl["d"] + 2 * hl["r"])
    tflops_main = f_dkv / (ms["fb_bwd_dkv"] * 1e-3) / 1e12
    prof_ns = _profiled("avg_launch_ns", "bwd_dkv_lean_kernel")
    prof_ms = None if prof_ns is None else round(prof_ns * 1e-6, 4)
    prof_frac = None if prof_ns is None else round(f_dkv / (prof_ns * 1e-9) / 1e12 / PEAK_BF16_TFLOPS, 4)
    value = (f_fwd + f_bwd) / (ms_step * 1e-3) / 1e12
    ref_fwd, ref_fb = workloads.reference_formula_flops(hl["B"], hl["H"], hl["L"], hl["d"])
    out = {
        "metric": "fwd+bwd ms & TFLOP/s (% bf16 MFMA peak) at B2 H4 L16384 d32 r8, 1 GPU",
        "value": round(value, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "primed_s": PRIME_SECONDS,
        "ms_per_step": round(ms_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "flash_bias_func fwd+bwd, B2 H4 L16384 d32 r8, non-causal, bf16 "
                               "(flash_bias/config.py:12 at len=16384)"},
        "pct_of_bf16_mfma_peak": round(100 * value / PEAK_BF16_TFLOPS, 2),
        # fwd_ms, bwd_ms, kernel_ms: one launch at a time between a pair of events (as the reference's harness
        # times a provider: triton.testing.do_bench, benchmark.py:354); fwd_ms_in_a_row: the same launches back to back between one pair
        "fwd_ms": round(ms["fb_fwd"], 4),
        "fwd_tflops": round(f_fwd / (ms["fb_fwd"] * 1e-3) / 1e12, 2),
        "fwd_ms_in_a_row": round(fwd_row, 4),
        "bwd_ms": round(ms["fb_bwd"], 4),
        "kernel_ms": {k: round(v, 4) for k, v in ms.items()},
        "reference_formula_tflops": round(ref_fb / (ms_step * 1e-3) / 1e12, 2),
        # achieved / frac: this run's own launches (one event pair per launch on the launch stream).  The tracked
        # profile's average for the same kernel (another box, under the profiler) is stated beside them.
        "roofline": {"kernel": "bwd_dkv_lean_kernel (fb_bwd_dkv)", "bound": "mfma", "achieved": round(tflops_main, 2),
                     "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": round(tflops_main / PEAK_BF16_TFLOPS, 4),
                     "traffic": _profiled("hbm_bytes_per_launch", "bwd_dkv_lean_kernel"),
                     "flop_per_launch": f_dkv, "launch_ms": round(ms["fb_bwd_dkv"], 4),
                     "profile_launch_ms": prof_ms, "frac_from_profile": prof_frac},
        "gate": gate,
    }
    del keep
    if not args.no_extras:
        steps, warm = max(5, args.steps // 2), max(2, args.warmup // 2)
        extra = (None, False, w["softmax_scale"])
        # the factors as flash_bias/benchmark.py:220-235 creates them, permuted inside the timed step
        stored = [w[n].detach().permute(0, 2, 1, 3).contiguous() for n in ("q_bias", "k_bias")]  # (B, H, L, r)
        fac_leaves = leaves[:3] + [t.requires_grad_(True) for t in stored]
        inside = _autograd_ms(fac_leaves, extra, w["do"], steps, warm,
                              prepare=lambda: [t.permute(0, 2, 1, 3).contiguous() for t in fac_leaves[3:]])
        out["factors_permuted_inside"] = {"fwd_ms": round(inside[0], 4), "fwd_bwd_ms": round(inside[1], 4)}
        del stored, fac_leaves
        half = [w[n].detach().half().requires_grad_(True) for n in ("q", "k", "v", "q_bias", "k_bias")]
        t16 = _autograd_ms(half, extra, w["do"].half(), steps, warm)
        out["fp16"] = {"fwd_ms": round(t16[0], 4), "fwd_bwd_ms": round(t16[1], 4),
                       "fwd_bwd_tflops": round((f_fwd + f_bwd) / t16[1] / 1e9, 1),
                       "pct_of_fp16_mfma_peak": round(100 * (f_fwd + f_bwd) / t16[1] / 1e9 / PEAK_BF16_TFLOPS, 2)}
        del half
        cat = _time_torch(lambda: _sdpa_concat(w), leaves, w["do"], 3, 1)
        with torch.no_grad():
            bias = (w["q_bias"].permute(0, 2, 1, 3) @ w["k_bias"].permute(0, 2, 3, 1)).contiguous()
        den = _time_torch(lambda: _sdpa_dense(w, bias), leaves[:3], w["do"], 3, 1)
        del bias
        out["providers"] = {"torch SDPA on concatenated [q*scale, q_bias] / [k, k_bias] (attention_func.py:188-237)":
                            {"fwd_ms": round(cat[0], 3), "fwd_bwd_ms": round(cat[1], 3)},
                            "torch SDPA with the materialised dense bias (attention_func.py:150-185; no factor gradients)":
                            {"fwd_ms": round(den[0], 3), "fwd_bwd_ms": round(den[1], 3)}}
        torch.cuda.empty_cache()
        out["sweep"] = _sweep(dev, steps, warm)
        out["modules"] = _modules(dev, steps, warm)
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
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the sweep, fp16, permuted-factors and provider timings (profiling runs)")
    ap.add_argument("--report", action="store_true", help="table over all named workloads")
    ap.add_argument("--only", metavar="TEXT", help="time only the benchmark configurations whose name contains TEXT "
                                                   "(as in the line's `sweep`; for profiling runs), print them as JSON")
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
    if args.only == "modules":
        import torch
        print(json.dumps({"modules": _modules(torch.device("cuda:0"), args.steps, args.warmup)}))
    elif args.only:
        import torch
        print(json.dumps({"sweep": _sweep(torch.device("cuda:0"), args.steps, args.warmup, args.only)}))
    elif args.report:
        report(args)
    else:
        headline(args)


if __name__ == "__main__":
    main()
