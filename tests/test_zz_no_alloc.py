"""The layer norm backward entry point that allocates nothing, through the C-ABI, against the
ordinary entry point (same kernels, same geometry: every output bit for bit) and the oracle."""
import numpy as np
import pytest

from oracle import haste_oracle as O
from util import TOL, dev, host, relerr

pytestmark = pytest.mark.gpu


def _run(name, x, gamma, dy, dg0, db0):
    import torch
    from haste_amd import lib as hlib
    rows, D = x.shape
    dx = torch.full_like(x, float("nan"))
    dgamma, dbeta = dg0.clone(), db0.clone()
    hlib.call(name, rows, D, gamma, x, dy, dx, dgamma, dbeta, None)
    return dx, dgamma, dbeta


def _case(rows, D, seed):
    r = np.random.default_rng(seed)
    f32 = lambda a: a.astype(np.float32).astype(np.float64)
    return (f32(r.standard_normal((rows, D)) * 2.0 + 0.7), f32(r.uniform(0.5, 1.5, D)),
            f32(r.standard_normal((rows, D))), f32(r.standard_normal(D)), f32(r.standard_normal(D)))


def test_no_alloc_layer_norm_backward_matches_the_allocating_entry_point():
    import torch
    # two calls in a row on the same device array, the second with a smaller input (fewer
    # workgroups and narrower rows), then an unaligned width and a single row
    for i, (rows, D) in enumerate([(16000, 1024), (777, 768), (37, 1001), (1, 4)]):
        print("no_alloc layer_norm_backward", rows, D, flush=True)
        x, gamma, dy, dg0, db0 = _case(rows, D, 100 + i)
        args = [dev(a) for a in (x, gamma, dy, dg0, db0)]
        got = _run("haste_hip_layer_norm_backward_noalloc_f32", *args)
        want = _run("haste_hip_layer_norm_backward_f32", *args)
        torch.cuda.synchronize()
        for g, w in zip(got, want):
            assert torch.equal(g, w)
        _, co = O.layer_norm_forward(x, gamma, None)
        dxo, dgo, dbo = O.layer_norm_backward(x, gamma, dy, co)
        assert relerr(host(got[0]), dxo) < TOL
        assert relerr(host(got[1]), dgo + dg0) < TOL
        assert relerr(host(got[2]), dbo + db0) < TOL


def test_no_alloc_layer_norm_backward_rejects_sizes_beyond_its_array():
    import torch
    from haste_amd import lib as hlib
    x = torch.zeros(8, 5000, device="cuda")
    g = torch.ones(5000, device="cuda")
    with pytest.raises(hlib.HasteHipError) as e:
        hlib.call("haste_hip_layer_norm_backward_noalloc_f32", 8, 5000, g, x, x, x.clone(), g.clone(),
                  None, None)
    assert e.value.code == 2 and "4096" in str(e.value)


def test_no_alloc_layer_norm_backward_in_a_graph():
    """What the entry point is for: two calls of different sizes recorded into a HIP graph on a
    side stream (after one eager call, which looks up the array's address) and replayed twice,
    with eager work between the replays; every replay gives the eager results' bits."""
    import torch
    from haste_amd import lib as hlib
    name = "haste_hip_layer_norm_backward_noalloc_f32"
    cases = [[dev(a) for a in _case(rows, D, 200 + i)] for i, (rows, D) in enumerate([(4000, 512), (333, 260)])]
    eager = [_run(name, *args) for args in cases]
    torch.cuda.synchronize()
    s = torch.cuda.Stream()
    outs = []
    with torch.cuda.stream(s):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=s):
            for x, gamma, dy, dg0, db0 in cases:
                rows, D = x.shape
                dx, dgamma, dbeta = torch.empty_like(x), torch.empty_like(dg0), torch.empty_like(db0)
                dgamma.copy_(dg0)
                dbeta.copy_(db0)
                hlib.call(name, rows, D, gamma, x, dy, dx, dgamma, dbeta, None, stream=s.cuda_stream)
                outs.append((dx, dgamma, dbeta))
        for replay in range(2):
            print("no_alloc replay", replay, flush=True)
            for o in outs:
                o[0].fill_(float("nan"))
            s.synchronize()
            between = _run(name, *cases[1])  # eager, on the current (side) stream
            s.synchronize()
            graph.replay()
            s.synchronize()
            for got, want in zip(outs, eager):
                for g, w in zip(got, want):
                    assert torch.equal(g, w), replay
            for g, w in zip(between, eager[1]):
                assert torch.equal(g, w)
        del graph
