"""LayerNormLSTM and LayerNormGRU on the GPU (through the C-ABI) vs the fp64 oracle."""
import numpy as np
import pytest

from oracle import haste_oracle as O
from util import TOL, dev, host, problem, relerr

pytestmark = pytest.mark.gpu

# The smallest case keeps H >= 4 and C >= 2: a layer norm over one or two elements has a
# constant output, and with C == 1 the norm of x*W does not depend on the scale of x, so
# those input gradients are pure rounding noise to which no relative tolerance applies.
SHAPES = [(1, 1, 3, 4), (3, 2, 3, 4), (5, 3, 7, 5), (6, 17, 20, 36), (4, 16, 32, 64),
          (10, 33, 48, 128), (8, 32, 64, 256), (6, 64, 96, 512),
          (3, 200, 16, 64), (2, 300, 8, 48), (2, 520, 8, 32),
          # hidden sizes beyond what stays on chip: the backward pass, then both passes, run
          # step by step (GEMM + row-wise norms + pointwise kernels)
          (3, 5, 24, 640), (2, 6, 16, 1536), (2, 130, 8, 1100),
          # resident forward whose norm of x*W is wider than 4096 columns
          (2, 3, 8, 1028),
          # hidden sizes whose backward recurrence keeps part of its slice of R in registers
          # (LSTM: 592 < H <= 1104, GRU: 784 < H <= 1472), tiles of 16, 32 and 64 rows
          (3, 20, 16, 768), (3, 64, 24, 1024), (2, 100, 8, 900), (2, 40, 8, 1300), (3, 130, 8, 1000),
          # ... and whose forward recurrence does (512 < H <= 2048 at small batches)
          (4, 16, 8, 640), (3, 7, 8, 2048), (2, 33, 8, 1600)]


@pytest.mark.parametrize("zoneout", [0.0, 0.3])
@pytest.mark.parametrize("T,N,C,H", SHAPES)
def test_layer_norm_lstm_training_forward_backward(T, N, C, H, zoneout):
    from haste_amd import ops
    import torch
    print("ln_lstm", T, N, C, H, zoneout, flush=True)
    p = problem(400 + T + N + C + H, T, N, C, H, 4, zoneout)
    mask = dev(p["mask"])
    gam, gh, bh = dev(p["gamma"]), dev(p["gamma_h"]), dev(p["beta_h"])
    outs = ops.layer_norm_lstm_forward(True, zoneout, dev(p["x"]), dev(p["h0"]), dev(p["c0"]),
                                       dev(p["W"]), dev(p["R"]), dev(p["b"]), gam, gh, bh, mask)
    torch.cuda.synchronize()
    h, c, act_Wx, act_Wx_norm, cache1, act_Rh, cache2, act_c_norm, cache3 = outs
    fwd = O.layer_norm_lstm_forward(p["W"], p["R"], p["b"], p["gamma"], p["gamma_h"], p["beta_h"],
                                    p["x"], p["h0"], p["c0"], True, zoneout, p["mask"])
    assert relerr(host(h), fwd["h"]) < TOL
    assert relerr(host(c), fwd["c"]) < TOL
    assert relerr(host(act_Wx_norm), fwd["v"]) < TOL
    assert relerr(host(act_Rh), fwd["act_Rh"]) < TOL
    assert relerr(host(act_c_norm), fwd["act_c_norm"]) < TOL
    assert relerr(host(cache2), fwd["cache2"]) < TOL
    assert relerr(host(cache3), fwd["cache3"]) < TOL
    x_t = dev(p["x"]).permute(2, 0, 1).contiguous()
    grads = ops.layer_norm_lstm_backward(
        x_t, dev(p["W"]).t().contiguous(), dev(p["R"]).t().contiguous(), dev(p["b"]), gam, gh, bh,
        mask, h, c, act_Wx, act_Wx_norm, cache1, act_Rh, cache2, act_c_norm, cache3,
        dev(p["dh_new"]), dev(p["dc_new"]))
    torch.cuda.synchronize()
    g = O.layer_norm_lstm_backward(p["W"], p["R"], p["b"], p["gamma"], p["gamma_h"], p["beta_h"],
                                   p["x"], fwd, p["dh_new"], p["dc_new"], p["mask"])
    names = ("dx", "dh0", "dc0", "dW", "dR", "db", "dgamma", "dgamma_h", "dbeta_h")
    for name, ours in zip(names, grads):
        assert relerr(host(ours), g[name]) < TOL, name


@pytest.mark.parametrize("zoneout", [0.0, 0.3])
@pytest.mark.parametrize("T,N,C,H", SHAPES)
def test_layer_norm_gru_training_forward_backward(T, N, C, H, zoneout):
    from haste_amd import ops
    import torch
    print("ln_gru", T, N, C, H, zoneout, flush=True)
    p = problem(500 + T + N + C + H, T, N, C, H, 3, zoneout)
    mask = dev(p["mask"])
    gam = dev(p["gamma"])
    h, cache, act_Wx, cache1, act_Rh, cache2 = ops.layer_norm_gru_forward(
        True, zoneout, dev(p["x"]), dev(p["h0"]), dev(p["W"]), dev(p["R"]), dev(p["b"]),
        dev(p["b2"]), gam, mask)
    torch.cuda.synchronize()
    fwd = O.layer_norm_gru_forward(p["W"], p["R"], p["b"], p["b2"], p["gamma"], p["x"], p["h0"],
                                   True, zoneout, p["mask"])
    assert relerr(host(h), fwd["h"]) < TOL
    assert relerr(host(cache), fwd["v"]) < TOL
    assert relerr(host(act_Rh), fwd["act_Rh"]) < TOL
    x_t = dev(p["x"]).permute(2, 0, 1).contiguous()
    grads = ops.layer_norm_gru_backward(
        x_t, dev(p["W"]).t().contiguous(), dev(p["R"]).t().contiguous(), dev(p["b"]), dev(p["b2"]),
        gam, mask, h, cache, act_Wx, cache1, act_Rh, cache2, dev(p["dh_new"]))
    torch.cuda.synchronize()
    g = O.layer_norm_gru_backward(p["W"], p["R"], p["b"], p["b2"], p["gamma"], p["x"], fwd,
                                  p["dh_new"], p["mask"])
    for name, ours in zip(("dx", "dh0", "dW", "dR", "dbx", "dbr", "dgamma"), grads):
        assert relerr(host(ours), g[name]) < TOL, name


def test_layer_norm_lstm_inference_forward():
    from haste_amd import ops
    import torch
    T, N, C, H = 15, 8, 32, 128
    p = problem(6, T, N, C, H, 4, 0.25)  # a probability float represents exactly (it crosses the ABI as float)
    outs = ops.layer_norm_lstm_forward(False, 0.25, dev(p["x"]), dev(p["h0"]), dev(p["c0"]),
                                       dev(p["W"]), dev(p["R"]), dev(p["b"]), dev(p["gamma"]),
                                       dev(p["gamma_h"]), dev(p["beta_h"]), dev(p["mask"]))
    torch.cuda.synchronize()
    fwd = O.layer_norm_lstm_forward(p["W"], p["R"], p["b"], p["gamma"], p["gamma_h"], p["beta_h"],
                                    p["x"], p["h0"], p["c0"], False, 0.25, p["mask"])
    assert relerr(host(outs[0]), fwd["h"]) < TOL
    assert relerr(host(outs[1]), fwd["c"]) < TOL


@pytest.mark.parametrize("T,N,C,H", [(6, 5, 12, 40), (5, 32, 16, 256), (4, 9, 8, 1100)])
def test_layer_norm_lstm_backward_with_badly_scaled_sums(T, N, C, H):
    """The backward step sends the row sums of the h*R norm as coefficients of the cell-state
    norm's dsigma and dmu (one exchange for both norms).  Inputs that make those terms large
    against their total -- norm scales of both signs and sizes, a cell state with a large
    common offset, upstream cell gradients with one -- must still give the oracle's gradients."""
    from haste_amd import ops
    import torch
    print("ln_lstm scaled", T, N, C, H, flush=True)
    p = problem(900 + T + N + C + H, T, N, C, H, 4, 0.2)
    r = np.random.default_rng(7 + H)
    f32 = lambda a: a.astype(np.float32).astype(np.float64)
    p["gamma"] = f32(r.uniform(-3.0, 3.0, p["gamma"].shape))
    p["gamma_h"] = f32(r.uniform(-2.0, 2.0, p["gamma_h"].shape))
    p["c0"] = f32(p["c0"] * 4.0 + 10.0)
    p["dc_new"] = f32(p["dc_new"] + 5.0)
    p["R"] = f32(p["R"] * 4.0)
    mask = dev(p["mask"])
    gam, gh, bh = dev(p["gamma"]), dev(p["gamma_h"]), dev(p["beta_h"])
    outs = ops.layer_norm_lstm_forward(True, 0.2, dev(p["x"]), dev(p["h0"]), dev(p["c0"]),
                                       dev(p["W"]), dev(p["R"]), dev(p["b"]), gam, gh, bh, mask)
    h, c, act_Wx, act_Wx_norm, cache1, act_Rh, cache2, act_c_norm, cache3 = outs
    fwd = O.layer_norm_lstm_forward(p["W"], p["R"], p["b"], p["gamma"], p["gamma_h"], p["beta_h"],
                                    p["x"], p["h0"], p["c0"], True, 0.2, p["mask"])
    assert relerr(host(h), fwd["h"]) < TOL
    assert relerr(host(c), fwd["c"]) < TOL
    grads = ops.layer_norm_lstm_backward(
        dev(p["x"]).permute(2, 0, 1).contiguous(), dev(p["W"]).t().contiguous(),
        dev(p["R"]).t().contiguous(), dev(p["b"]), gam, gh, bh, mask, h, c, act_Wx, act_Wx_norm,
        cache1, act_Rh, cache2, act_c_norm, cache3, dev(p["dh_new"]), dev(p["dc_new"]))
    torch.cuda.synchronize()
    g = O.layer_norm_lstm_backward(p["W"], p["R"], p["b"], p["gamma"], p["gamma_h"], p["beta_h"],
                                   p["x"], fwd, p["dh_new"], p["dc_new"], p["mask"])
    names = ("dx", "dh0", "dc0", "dW", "dR", "db", "dgamma", "dgamma_h", "dbeta_h")
    for name, ours in zip(names, grads):
        assert relerr(host(ours), g[name]) < TOL, name
