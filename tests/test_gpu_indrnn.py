"""IndRNN and LayerNormIndRNN on the GPU (through the C-ABI) vs the fp64 oracle."""
import numpy as np
import pytest

from oracle import haste_oracle as O
from util import TOL, dev, host, problem, relerr

pytestmark = pytest.mark.gpu

# T on both sides of the kernels' batches of 16 steps: no whole batch, whole batches only, a tail
SHAPES = [(1, 1, 1, 1), (3, 2, 3, 4), (9, 3, 7, 5), (15, 2, 3, 6), (16, 3, 5, 70), (17, 5, 20, 70),
          (30, 16, 32, 256), (32, 2, 4, 33), (33, 2, 4, 33), (50, 64, 64, 512),
          # the width of the reference's IndRNN speed script (validation/pytorch_speed.py:7-20)
          (20, 64, 256, 4096)]


@pytest.mark.parametrize("layer_norm", [False, True])
@pytest.mark.parametrize("zoneout", [0.0, 0.3])
@pytest.mark.parametrize("T,N,C,H", SHAPES)
def test_indrnn_training_forward_backward(T, N, C, H, zoneout, layer_norm):
    from haste_amd import ops
    import torch
    print("indrnn", T, N, C, H, zoneout, layer_norm, flush=True)
    p = problem(300 + T + N + C + H, T, N, C, H, 1, zoneout)
    gam = p["gamma"] if layer_norm else None
    mask = dev(p["mask"])
    x_t = dev(p["x"]).permute(2, 0, 1).contiguous()
    W_t = dev(p["W"]).t().contiguous()
    if layer_norm:
        h, act_Wx, cache = ops.layer_norm_indrnn_forward(True, zoneout, dev(p["x"]), dev(p["h0"]),
                                                         dev(p["W"]), dev(p["u"]), dev(p["b"]),
                                                         dev(gam), mask)
        outs = ops.layer_norm_indrnn_backward(x_t, W_t, dev(p["u"]), dev(p["b"]), dev(gam), mask, h,
                                              act_Wx, cache, dev(p["dh_new"]))
    else:
        h = ops.indrnn_forward(True, zoneout, dev(p["x"]), dev(p["h0"]), dev(p["W"]), dev(p["u"]),
                               dev(p["b"]), mask)
        outs = ops.indrnn_backward(x_t, W_t, dev(p["u"]), dev(p["b"]), mask, h, dev(p["dh_new"]))
    torch.cuda.synchronize()
    fwd = O.indrnn_forward(p["W"], p["u"], p["b"], p["x"], p["h0"], True, zoneout, p["mask"], gam)
    g = O.indrnn_backward(p["W"], p["u"], p["b"], p["x"], fwd, p["dh_new"], p["mask"], gam)
    assert relerr(host(h), fwd["h"]) < TOL
    names = ("dx", "dh0", "dW", "du", "db") + (("dgamma",) if layer_norm else ())
    for name, ours in zip(names, outs):
        assert relerr(host(ours), g[name]) < TOL, name


def test_indrnn_inference_zoneout_blend():
    from haste_amd import ops
    import torch
    T, N, C, H = 12, 4, 8, 96
    p = problem(5, T, N, C, H, 1, 0.2)
    h = ops.indrnn_forward(False, 0.2, dev(p["x"]), dev(p["h0"]), dev(p["W"]), dev(p["u"]),
                           dev(p["b"]), dev(p["mask"]))
    torch.cuda.synchronize()
    fwd = O.indrnn_forward(p["W"], p["u"], p["b"], p["x"], p["h0"], False, 0.2, p["mask"])
    assert relerr(host(h), fwd["h"]) < TOL
