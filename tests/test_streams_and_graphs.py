"""Stream and graph use of the operator."""
import pytest
import torch

from _util import make_inputs
from flashbias_amd import flash_bias_func

pytestmark = pytest.mark.gpu


def _leaves(dev, seed):
    q, k, v, qb, kb, do = make_inputs(2, 300, 300, 4, 32, 8, torch.bfloat16, seed=seed)
    return [t.to(dev) for t in (q, k, v, qb, kb)], do.to(dev)


def _fwd_bwd(leaves, do):
    xs = [t.detach().requires_grad_(True) for t in leaves]
    o = flash_bias_func(*xs, None, True, None)
    return [o.detach()] + list(torch.autograd.grad(o, xs, do))


def test_side_stream_matches_default_stream(gpu_device):
    leaves, do = _leaves(gpu_device, 3)
    want = _fwd_bwd(leaves, do)
    torch.cuda.synchronize()
    s = torch.cuda.Stream(device=gpu_device)
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        got = _fwd_bwd(leaves, do)
    s.synchronize()
    for g, w in zip(got, want):
        assert torch.equal(g, w)


def test_graph_replays_match_eager(gpu_device):
    """Forward and backward captured in one graph: every replay, with new values in the static
    inputs, is bit-identical to the eager result (the library allocates nothing and keeps no
    state between calls)."""
    static, static_do = _leaves(gpu_device, 4)
    s = torch.cuda.Stream(device=gpu_device)
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for _ in range(2):
            _fwd_bwd(static, static_do)
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = _fwd_bwd(static, static_do)
    for seed in (5, 6, 7):
        fresh, fresh_do = _leaves(gpu_device, seed)
        for dst, src in zip(static + [static_do], fresh + [fresh_do]):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in outs]
        want = _fwd_bwd(fresh, fresh_do)
        torch.cuda.synchronize()
        for g, w in zip(got, want):
            assert torch.equal(g, w)
