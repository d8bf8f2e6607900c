"""Stand-alone layer norm kernels on the GPU vs the fp64 oracle."""
import numpy as np
import pytest

from oracle import haste_oracle as O
from util import TOL, dev, host, relerr

pytestmark = pytest.mark.gpu

SHAPES = [(1, 1), (3, 5), (7, 33), (64, 64), (100, 256), (37, 1000), (3200, 1024), (500, 2048),
          (33, 4096), (9, 1023),
          # wider than a wavefront keeps in registers: the row-per-workgroup kernels
          (5, 5000), (3, 4101), (40, 8192)]


@pytest.mark.parametrize("with_beta", [False, True])
@pytest.mark.parametrize("rows,D", SHAPES)
def test_layer_norm_forward_backward(rows, D, with_beta):
    from haste_amd import ops
    import torch
    print("layer_norm", rows, D, with_beta, flush=True)
    r = np.random.default_rng(rows * 31 + D)
    f32 = lambda a: a.astype(np.float32).astype(np.float64)
    x = f32(r.standard_normal((rows, D)) * 2.0 + 0.7)
    gamma = f32(r.uniform(0.5, 1.5, D))
    beta = f32(r.standard_normal(D)) if with_beta else None
    dy = f32(r.standard_normal((rows, D)))
    y, cache = ops.layer_norm_forward(dev(x), dev(gamma), dev(beta) if with_beta else None)
    dx, dgamma, dbeta = ops.layer_norm_backward(dev(x), dev(gamma), dev(dy), cache, with_beta)
    torch.cuda.synchronize()
    yo, co = O.layer_norm_forward(x, gamma, beta)
    dxo, dgo, dbo = O.layer_norm_backward(x, gamma, dy, co)
    assert relerr(host(y), yo) < TOL
    assert relerr(host(cache), co) < TOL
    assert relerr(host(dx), dxo) < TOL
    assert relerr(host(dgamma), dgo) < TOL
    if with_beta:
        assert relerr(host(dbeta), dbo) < TOL


def test_layer_norm_backward_in_place_and_deterministic():
    from haste_amd import ops
    import torch
    r = np.random.default_rng(1)
    x, gamma, dy = dev(r.standard_normal((777, 768))), dev(r.uniform(0.5, 1.5, 768)), r.standard_normal((777, 768))
    a = ops.layer_norm_backward(x, gamma, dev(dy))
    b = ops.layer_norm_backward(x, gamma, dev(dy), in_place=True)
    torch.cuda.synchronize()
    for u, v in zip(a, b):
        assert torch.equal(u, v)
