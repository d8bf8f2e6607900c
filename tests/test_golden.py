"""The committed vectors under tests/golden/ (made by tests/golden/make_fixtures.py).

CPU: the oracle must reproduce every file: the `*_torchnn` ones were made by
torch.nn.LSTM / torch.nn.GRU / F.layer_norm + autograd without the oracle, the
`*_oracle` ones freeze the oracle's own answers.  GPU: the C-ABI must reproduce every
file to 1e-4 (max|a-b| / max|b| per tensor).
"""
import os

import numpy as np
import pytest

from oracle import haste_oracle as O
from util import TOL, dev, host, relerr

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
ORACLE_TOL = 1e-11


def load(name):
    with np.load(os.path.join(GOLDEN, name), allow_pickle=False) as f:
        return {k: f[k] for k in f.files}


def close(a, b, tol, what):
    assert np.shape(a) == np.shape(b), what
    assert relerr(a, b) < tol, what


# ---- the oracle against the files ------------------------------------------------------
def test_oracle_lstm_torchnn():
    g = load("lstm_torchnn.npz")
    h, c, v = O.lstm_forward(g["W"], g["R"], g["b"], g["x"], g["h0"], g["c0"])
    close(h[1:], g["y"], ORACLE_TOL, "y")
    close(h[-1], g["h_T"], ORACLE_TOL, "h_T")
    close(c[-1], g["c_T"], ORACLE_TOL, "c_T")
    out = O.lstm_backward(g["W"], g["R"], g["b"], g["x"], h, c, v, g["dh_new"], g["dc_new"])
    for name, a in zip(("dx", "dW", "dR", "db", "dh0", "dc0"), out):
        close(a, g[name], ORACLE_TOL, name)


def test_oracle_gru_torchnn():
    g = load("gru_torchnn.npz")
    h, v = O.gru_forward(g["W"], g["R"], g["bx"], g["br"], g["x"], g["h0"])
    close(h[1:], g["y"], ORACLE_TOL, "y")
    out = O.gru_backward(g["W"], g["R"], g["bx"], g["br"], g["x"], h, v, g["dh_new"])
    for name, a in zip(("dx", "dW", "dR", "dbx", "dbr", "dh0"), out):
        close(a, g[name], ORACLE_TOL, name)


def test_oracle_layer_norm_torchnn():
    g = load("layer_norm_torchnn.npz")
    y, cache = O.layer_norm_forward(g["x"], g["gamma"], g["beta"])
    close(y, g["y"], ORACLE_TOL, "y")
    dx, dgamma, dbeta = O.layer_norm_backward(g["x"], g["gamma"], g["dy"], cache)
    close(dx, g["dx"], 1e-10, "dx")
    close(dgamma, g["dgamma"], ORACLE_TOL, "dgamma")
    close(dbeta, g["dbeta"], ORACLE_TOL, "dbeta")


def test_oracle_reproduces_frozen_answers():
    g = load("lstm_zoneout_oracle.npz")
    zo = float(g["zoneout"])
    h, c, v = O.lstm_forward(g["W"], g["R"], g["b"], g["x"], g["h0"], g["c0"], True, zo, g["mask"])
    out = O.lstm_backward(g["W"], g["R"], g["b"], g["x"], h, c, v, g["dh_new"], g["dc_new"], g["mask"])
    for name, a in zip(("h", "c", "v", "dx", "dW", "dR", "db", "dh0", "dc0", "dv"), (h, c, v) + tuple(out)):
        close(a, g[name], 1e-13, name)
    hi, ci, _ = O.lstm_forward(g["W"], g["R"], g["b"], g["x"], g["h0"], g["c0"], False, zo, g["mask"])
    close(hi, g["h_inference"], 1e-13, "h_inference")

    g = load("gru_zoneout_oracle.npz")
    h, v = O.gru_forward(g["W"], g["R"], g["b"], g["b2"], g["x"], g["h0"], True, zo, g["mask"])
    out = O.gru_backward(g["W"], g["R"], g["b"], g["b2"], g["x"], h, v, g["dh_new"], g["mask"])
    for name, a in zip(("h", "v", "dx", "dW", "dR", "dbx", "dbr", "dh0"), (h, v) + tuple(out)):
        close(a, g[name], 1e-13, name)

    g = load("layer_norm_lstm_oracle.npz")
    fwd = O.layer_norm_lstm_forward(g["W"], g["R"], g["b"], g["gamma"], g["gamma_h"], g["beta_h"],
                                    g["x"], g["h0"], g["c0"], True, zo, g["mask"])
    bwd = O.layer_norm_lstm_backward(g["W"], g["R"], g["b"], g["gamma"], g["gamma_h"], g["beta_h"],
                                     g["x"], fwd, g["dh_new"], g["dc_new"], g["mask"])
    for k, a in fwd.items():
        close(a, g["fwd_" + k], 1e-13, k)
    for k, a in bwd.items():
        close(a, g["bwd_" + k], 1e-13, k)

    g = load("layer_norm_gru_oracle.npz")
    fwd = O.layer_norm_gru_forward(g["W"], g["R"], g["b"], g["b2"], g["gamma"], g["x"], g["h0"],
                                   True, zo, g["mask"])
    bwd = O.layer_norm_gru_backward(g["W"], g["R"], g["b"], g["b2"], g["gamma"], g["x"], fwd,
                                    g["dh_new"], g["mask"])
    for k, a in fwd.items():
        close(a, g["fwd_" + k], 1e-13, k)
    for k, a in bwd.items():
        close(a, g["bwd_" + k], 1e-13, k)

    for name, use_gamma in (("indrnn_oracle.npz", False), ("layer_norm_indrnn_oracle.npz", True)):
        g = load(name)
        gamma = g["gamma"] if use_gamma else None
        fwd = O.indrnn_forward(g["W"], g["u"], g["b"], g["x"], g["h0"], True, zo, g["mask"], gamma)
        bwd = O.indrnn_backward(g["W"], g["u"], g["b"], g["x"], fwd, g["dh_new"], g["mask"], gamma)
        for k, a in fwd.items():
            if a is not None:
                close(a, g["fwd_" + k], 1e-13, k)
        for k, a in bwd.items():
            close(a, g["bwd_" + k], 1e-13, k)


# ---- the GPU library against the files ---------------------------------------------------
def _t(a):
    """[T,N,C] device tensor -> the [C,T,N] layout the backward passes take."""
    return a.permute(2, 0, 1).contiguous()


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["lstm_torchnn.npz", "lstm_zoneout_oracle.npz"])
def test_gpu_lstm_golden(name):
    from haste_amd import ops
    import torch
    g = load(name)
    zo = float(g["zoneout"]) if "zoneout" in g else 0.0
    mask = dev(g.get("mask"))
    x, W, R, b = dev(g["x"]), dev(g["W"]), dev(g["R"]), dev(g["b"])
    h, c, cache = ops.lstm_forward(True, zo, x, dev(g["h0"]), dev(g["c0"]), W, R, b, mask)
    if "y" in g:
        close(host(h[1:]), g["y"], TOL, "y")
        close(host(c[-1]), g["c_T"], TOL, "c_T")
    else:
        close(host(h), g["h"], TOL, "h")
        close(host(c), g["c"], TOL, "c")
        close(host(cache), g["v"], TOL, "v")
    out = ops.lstm_backward(_t(x), W.t().contiguous(), R.t().contiguous(), b, mask, h, c, cache,
                            dev(g["dh_new"]), dev(g["dc_new"]))
    torch.cuda.synchronize()
    for k, a in zip(("dx", "dh0", "dc0", "dW", "dR", "db"), out):
        close(host(a), g[k], TOL, k)
    if "h_inference" in g:
        hi, ci, _ = ops.lstm_forward(False, zo, x, dev(g["h0"]), dev(g["c0"]), W, R, b, mask)
        close(host(hi), g["h_inference"], TOL, "h_inference")
        close(host(ci), g["c_inference"], TOL, "c_inference")


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["gru_torchnn.npz", "gru_zoneout_oracle.npz"])
def test_gpu_gru_golden(name):
    from haste_amd import ops
    import torch
    g = load(name)
    zo = float(g["zoneout"]) if "zoneout" in g else 0.0
    mask = dev(g.get("mask"))
    bx, br = (g["bx"], g["br"]) if "bx" in g else (g["b"], g["b2"])
    x, W, R, bx, br = dev(g["x"]), dev(g["W"]), dev(g["R"]), dev(bx), dev(br)
    h, cache = ops.gru_forward(True, zo, x, dev(g["h0"]), W, R, bx, br, mask)
    if "y" in g:
        close(host(h[1:]), g["y"], TOL, "y")
    else:
        close(host(h), g["h"], TOL, "h")
        close(host(cache), g["v"], TOL, "v")
    out = ops.gru_backward(_t(x), W.t().contiguous(), R.t().contiguous(), bx, br, mask, h, cache,
                           dev(g["dh_new"]))
    torch.cuda.synchronize()
    for k, a in zip(("dx", "dh0", "dW", "dR", "dbx", "dbr"), out):
        close(host(a), g[k], TOL, k)


@pytest.mark.gpu
def test_gpu_layer_norm_golden():
    from haste_amd import ops
    g = load("layer_norm_torchnn.npz")
    x, gamma, beta = dev(g["x"]), dev(g["gamma"]), dev(g["beta"])
    y, cache = ops.layer_norm_forward(x, gamma, beta)
    close(host(y), g["y"], TOL, "y")
    dx, dgamma, dbeta = ops.layer_norm_backward(x, gamma, dev(g["dy"]), cache)
    close(host(dx), g["dx"], TOL, "dx")
    close(host(dgamma), g["dgamma"], TOL, "dgamma")
    close(host(dbeta), g["dbeta"], TOL, "dbeta")


@pytest.mark.gpu
def test_gpu_layer_norm_lstm_golden():
    from haste_amd import ops
    g = load("layer_norm_lstm_oracle.npz")
    zo, mask = float(g["zoneout"]), dev(g["mask"])
    x, W, R, b = dev(g["x"]), dev(g["W"]), dev(g["R"]), dev(g["b"])
    gamma, gamma_h, beta_h = dev(g["gamma"]), dev(g["gamma_h"]), dev(g["beta_h"])
    fwd = ops.layer_norm_lstm_forward(True, zo, x, dev(g["h0"]), dev(g["c0"]), W, R, b, gamma,
                                      gamma_h, beta_h, mask)
    h, c, act_Wx, act_Wx_norm, _, act_Rh, _, act_c_norm, _ = fwd
    for k, a in (("h", h), ("c", c), ("act_Wx", act_Wx), ("v", act_Wx_norm), ("act_Rh", act_Rh),
                 ("act_c_norm", act_c_norm)):
        close(host(a), g["fwd_" + k], TOL, k)
    out = ops.layer_norm_lstm_backward(_t(x), W.t().contiguous(), R.t().contiguous(), b, gamma,
                                       gamma_h, beta_h, mask, *fwd, dev(g["dh_new"]), dev(g["dc_new"]))
    for k, a in zip(("dx", "dh0", "dc0", "dW", "dR", "db", "dgamma", "dgamma_h", "dbeta_h"), out):
        close(host(a), g["bwd_" + k], TOL, k)


@pytest.mark.gpu
def test_gpu_layer_norm_gru_golden():
    from haste_amd import ops
    g = load("layer_norm_gru_oracle.npz")
    zo, mask = float(g["zoneout"]), dev(g["mask"])
    x, W, R, bx, br = dev(g["x"]), dev(g["W"]), dev(g["R"]), dev(g["b"]), dev(g["b2"])
    gamma = dev(g["gamma"])
    fwd = ops.layer_norm_gru_forward(True, zo, x, dev(g["h0"]), W, R, bx, br, gamma, mask)
    h, cache, act_Wx, _, act_Rh, _ = fwd
    for k, a in (("h", h), ("v", cache), ("act_Wx", act_Wx), ("act_Rh", act_Rh)):
        close(host(a), g["fwd_" + k], TOL, k)
    out = ops.layer_norm_gru_backward(_t(x), W.t().contiguous(), R.t().contiguous(), bx, br, gamma,
                                      mask, *fwd, dev(g["dh_new"]))
    for k, a in zip(("dx", "dh0", "dW", "dR", "dbx", "dbr", "dgamma"), out):
        close(host(a), g["bwd_" + k], TOL, k)


@pytest.mark.gpu
def test_gpu_indrnn_golden():
    from haste_amd import ops
    g = load("indrnn_oracle.npz")
    zo, mask = float(g["zoneout"]), dev(g["mask"])
    x, W, u, b = dev(g["x"]), dev(g["W"]), dev(g["u"]), dev(g["b"])
    h = ops.indrnn_forward(True, zo, x, dev(g["h0"]), W, u, b, mask)
    close(host(h), g["fwd_h"], TOL, "h")
    out = ops.indrnn_backward(_t(x), W.t().contiguous(), u, b, mask, h, dev(g["dh_new"]))
    for k, a in zip(("dx", "dh0", "dW", "du", "db"), out):
        close(host(a), g["bwd_" + k], TOL, k)

    g = load("layer_norm_indrnn_oracle.npz")
    mask = dev(g["mask"])
    x, W, u, b, gamma = dev(g["x"]), dev(g["W"]), dev(g["u"]), dev(g["b"]), dev(g["gamma"])
    h, act_Wx, cache = ops.layer_norm_indrnn_forward(True, zo, x, dev(g["h0"]), W, u, b, gamma, mask)
    close(host(h), g["fwd_h"], TOL, "h")
    out = ops.layer_norm_indrnn_backward(_t(x), W.t().contiguous(), u, b, gamma, mask, h, act_Wx,
                                         cache, dev(g["dh_new"]))
    for k, a in zip(("dx", "dh0", "dW", "du", "db", "dgamma"), out):
        close(host(a), g["bwd_" + k], TOL, k)
