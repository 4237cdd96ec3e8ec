"""fb_bwd_static (the backward entry point that allocates nothing) against fb_bwd, through the C ABI."""
import pytest
import torch

from _util import make_inputs


@pytest.mark.gpu
def test_static_scratch_backward_matches_fb_bwd(gpu_device):
    """Two calls in a row, the second on a smaller input: every gradient and nothing else differs
    from what fb_bwd writes with a caller-owned scratch buffer (bit-exact: same kernels)."""
    from flashbias_amd import _lib
    from flashbias_amd.interface import _params, _stream, _tensor
    dev = gpu_device
    lib = _lib.load()

    def run(B, L, H, d, r, causal, seed):
        q, k, v, qb, kb, do = [t.to(dev) for t in make_inputs(B, L, L, H, d, r, torch.bfloat16, seed=seed)]

        def params(with_scratch):
            p, keep = _params(q, k, v, qb, kb, None, causal, None)
            bufs = dict(o=torch.empty_like(q), lse=torch.empty((B, H, L), device=dev, dtype=torch.float32),
                        dq=torch.full_like(q, float("nan")), dk=torch.full_like(k, float("nan")),
                        dv=torch.full_like(v, float("nan")),
                        dqb=torch.full((B, L, H, r), float("nan"), device=dev, dtype=q.dtype),
                        dkb=torch.full((B, L, H, r), float("nan"), device=dev, dtype=q.dtype))
            p.o, p.lse, p.dout = _tensor(bufs["o"]), bufs["lse"].data_ptr(), _tensor(do)
            p.dq, p.dk, p.dv = _tensor(bufs["dq"]), _tensor(bufs["dk"]), _tensor(bufs["dv"])
            p.dq_bias, p.dk_bias = _tensor(bufs["dqb"]), _tensor(bufs["dkb"])
            if with_scratch:
                bufs["scratch"] = torch.empty(lib.fb_bwd_workspace_bytes(p) // 4, device=dev, dtype=torch.float32)
                p.delta = bufs["scratch"].data_ptr()
            return p, keep, bufs

        p1, keep1, want = params(True)
        _lib.check_status(lib.fb_fwd(p1, _stream()))
        _lib.check_status(lib.fb_bwd(p1, _stream()))
        p2, keep2, got = params(False)  # delta stays null: the static entry point must not need it
        _lib.check_status(lib.fb_fwd(p2, _stream()))
        _lib.check_status(lib.fb_bwd_static(p2, _stream()))
        torch.cuda.synchronize()
        for name in ("dq", "dk", "dv", "dqb", "dkb"):
            assert not torch.isnan(want[name].float()).any(), name
            assert torch.equal(want[name], got[name]), name

    run(2, 777, 3, 32, 8, True, seed=21)
    run(1, 130, 2, 32, 8, False, seed=22)  # smaller: the array still holds the first call's values
    run(40, 200, 8, 32, 16, False, seed=24)  # whole sequences in one workgroup: a single launch that needs no scratch


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,B,L,H,causal,r", [(torch.float16, 2, 1024, 4, False, 8),   # small grid: preprocess + one mixed launch
                                                  (torch.bfloat16, 3, 520, 8, True, 8),
                                                  (torch.bfloat16, 2, 640, 8, True, 16)])   # ... of the general kernels
def test_static_scratch_backward_in_a_graph(gpu_device, dtype, B, L, H, causal, r):
    """fb_bwd_static captured in a HIP graph after fb_init() (the address of the static array is looked up outside
    the capture) and replayed three times with the program's own eager work between the replays: every replay's
    gradients are bit for bit those of fb_bwd."""
    from flashbias_amd import _lib
    from flashbias_amd.interface import _params, _tensor
    dev = gpu_device
    lib = _lib.load()
    assert lib.fb_init() == 0
    q, k, v, qb, kb, do = [t.to(dev) for t in make_inputs(B, L, L, H, 32, r, dtype, seed=23)]
    p, keep = _params(q, k, v, qb, kb, None, causal, None)
    o, lse = torch.empty_like(q), torch.empty((B, H, L), device=dev, dtype=torch.float32)
    names = ("dq", "dk", "dv", "dqb", "dkb")
    shapes = dict(dq=q.shape, dk=k.shape, dv=v.shape, dqb=qb.shape, dkb=kb.shape)
    bufs = {n: torch.zeros(shapes[n], device=dev, dtype=dtype) for n in names}
    p.o, p.lse, p.dout = _tensor(o), lse.data_ptr(), _tensor(do)
    p.dq, p.dk, p.dv = _tensor(bufs["dq"]), _tensor(bufs["dk"]), _tensor(bufs["dv"])
    p.dq_bias, p.dk_bias = _tensor(bufs["dqb"]), _tensor(bufs["dkb"])
    scratch = torch.empty(lib.fb_bwd_workspace_bytes(p) // 4, device=dev, dtype=torch.float32)
    p.delta = scratch.data_ptr()
    raw = lambda: torch._C._cuda_getCurrentRawStream(torch.cuda.current_device())
    _lib.check_status(lib.fb_fwd(p, raw()))
    _lib.check_status(lib.fb_bwd(p, raw()))
    torch.cuda.synchronize()
    want = {n: bufs[n].clone() for n in names}
    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        _lib.check_status(lib.fb_bwd_static(p, raw()))  # (warm-up: occupancy caches)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _lib.check_status(lib.fb_bwd_static(p, raw()))
    for _ in range(3):
        for n in names:
            bufs[n].fill_(float("nan"))  # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for n in names:
            assert torch.equal(bufs[n], want[n]), n


def test_static_scratch_rejects_sizes_beyond_its_array():
    """The size check comes before anything touches the GPU, so this runs on the CPU."""
    from flashbias_amd import _lib
    lib = _lib.load()
    p = _lib.new_params()
    p.dtype, p.B, p.H, p.Lq, p.Lk, p.d, p.r, p.scale = _lib.FB_BF16, 64, 64, 2048, 2048, 32, 0, 1.0
    assert lib.fb_bwd_workspace_bytes(p) > (32 << 20)
    assert lib.fb_bwd_static(p, None) == -2
    assert b"static scratch" in lib.fb_last_error()
