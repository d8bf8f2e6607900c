"""Pins the oracle's hand-derived backward passes (all cells, with and without
zoneout) against torch autograd of a forward assembled from library pieces
(matmul, torch.sigmoid/tanh, F.layer_norm), against fp64 central finite
differences, and against invariants the mathematics fixes.

The forward assemblies follow the reference's CPU definitions, read as text:
frameworks/pytorch/lstm.py:33-66, gru.py:33-66, indrnn.py:33-54,
layer_norm_lstm.py:33-69, layer_norm_gru.py:33-67, layer_norm_indrnn.py:33-56.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import haste_oracle as O

torch.set_num_threads(4)
TD = torch.float64


def _relerr(a, b):
    return np.max(np.abs(a - b)) / max(np.max(np.abs(b)), 1e-30)


def _t(a, grad=True):
    t = torch.from_numpy(np.array(a, dtype=np.float64))
    return t.requires_grad_() if grad else t


def _zone(hn, hp, mask_t):
    return (hn - hp) * mask_t + hp if mask_t is not None else hn


# ---- torch forwards (library pieces only) ---------------------------------
def torch_lstm(W, R, b, x, h0, c0, mask):
    H = R.shape[0]
    h, c = [h0], [c0]
    Wx = x @ W
    for t in range(x.shape[0]):
        a = Wx[t] + h[t] @ R + b
        i, g, f, o = torch.chunk(a, 4, 1)
        c.append(torch.sigmoid(f) * c[t] + torch.sigmoid(i) * torch.tanh(g))
        hn = torch.sigmoid(o) * torch.tanh(c[-1])
        h.append(_zone(hn, h[t], mask[t] if mask is not None else None))
    return torch.stack(h), torch.stack(c)


def torch_gru(W, R, bx, br, x, h0, mask):
    h = [h0]
    Wx = x @ W + bx
    for t in range(x.shape[0]):
        Rh = h[t] @ R + br
        vx, vh = torch.chunk(Wx[t], 3, 1), torch.chunk(Rh, 3, 1)
        z = torch.sigmoid(vx[0] + vh[0])
        r = torch.sigmoid(vx[1] + vh[1])
        g = torch.tanh(vx[2] + r * vh[2])
        h.append(_zone(z * h[t] + (1 - z) * g, h[t], mask[t] if mask is not None else None))
    return torch.stack(h)


def torch_ln_lstm(W, R, b, gamma, gamma_h, beta_h, x, h0, c0, mask):
    H = R.shape[0]
    h, c = [h0], [c0]
    Wx = F.layer_norm(x @ W, (4 * H,), weight=gamma[0])
    for t in range(x.shape[0]):
        a = F.layer_norm(h[t] @ R, (4 * H,), weight=gamma[1]) + Wx[t] + b
        i, g, f, o = torch.chunk(a, 4, 1)
        c.append(torch.sigmoid(f) * c[t] + torch.sigmoid(i) * torch.tanh(g))
        hn = torch.sigmoid(o) * torch.tanh(F.layer_norm(c[-1], (H,), weight=gamma_h, bias=beta_h))
        h.append(_zone(hn, h[t], mask[t] if mask is not None else None))
    return torch.stack(h), torch.stack(c)


def torch_ln_gru(W, R, bx, br, gamma, x, h0, mask):
    H = R.shape[0]
    h = [h0]
    Wx = F.layer_norm(x @ W, (3 * H,), weight=gamma[0]) + bx
    for t in range(x.shape[0]):
        Rh = F.layer_norm(h[t] @ R, (3 * H,), weight=gamma[1]) + br
        vx, vh = torch.chunk(Wx[t], 3, 1), torch.chunk(Rh, 3, 1)
        z = torch.sigmoid(vx[0] + vh[0])
        r = torch.sigmoid(vx[1] + vh[1])
        g = torch.tanh(vx[2] + r * vh[2])
        h.append(_zone(z * h[t] + (1 - z) * g, h[t], mask[t] if mask is not None else None))
    return torch.stack(h)


def torch_indrnn(W, u, b, x, h0, mask, gamma=None):
    H = u.shape[0]
    h = [h0]
    Wx = x @ W
    if gamma is not None:
        Wx = F.layer_norm(Wx, (H,), weight=gamma[0])
    Wx = Wx + b
    for t in range(x.shape[0]):
        hn = torch.tanh(Wx[t] + h[t] * u)
        h.append(_zone(hn, h[t], mask[t] if mask is not None else None))
    return torch.stack(h)


# ---- problem builders -----------------------------------------------------
def _problem(seed, T, N, C, H, G, zoneout):
    r = np.random.default_rng(seed)
    k = 1.0 / np.sqrt(H)
    p = dict(
        W=r.uniform(-k, k, (C, G * H)), R=r.uniform(-k, k, (H, G * H)),
        b=r.uniform(-k, k, G * H), b2=r.uniform(-k, k, G * H),
        x=r.standard_normal((T, N, C)), h0=r.standard_normal((N, H)) * 0.5,
        c0=r.standard_normal((N, H)) * 0.5,
        dh_new=r.standard_normal((T + 1, N, H)), dc_new=r.standard_normal((T + 1, N, H)),
        gamma=r.uniform(0.5, 1.5, (2, G * H)), gamma_h=r.uniform(0.5, 1.5, H),
        beta_h=r.uniform(-0.5, 0.5, H), u=r.uniform(-1, 1, H),
        mask=(r.uniform(size=(T, N, H)) < 0.6).astype(np.float64) if zoneout else None)
    return p


SHAPES = [(4, 3, 4, 5), (7, 2, 3, 6)]


@pytest.mark.parametrize("zoneout", [False, True])
@pytest.mark.parametrize("T,N,C,H", SHAPES)
def test_lstm_zoneout_autograd(T, N, C, H, zoneout):
    p = _problem(10, T, N, C, H, 4, zoneout)
    h, c, v = O.lstm_forward(p["W"], p["R"], p["b"], p["x"], p["h0"], p["c0"], True,
                             0.4 if zoneout else 0.0, p["mask"])
    dx, dW, dR, db, dh0, dc0, _ = O.lstm_backward(
        p["W"], p["R"], p["b"], p["x"], h, c, v, p["dh_new"], p["dc_new"], p["mask"])
    W, R, b, x, h0, c0 = (_t(p[k]) for k in ("W", "R", "b", "x", "h0", "c0"))
    mk = _t(p["mask"], False) if zoneout else None
    ht, ct = torch_lstm(W, R, b, x, h0, c0, mk)
    ((ht[1:] * _t(p["dh_new"][1:], False)).sum() + (ct[1:] * _t(p["dc_new"][1:], False)).sum()).backward()
    assert _relerr(h, ht.detach().numpy()) < 1e-12
    assert _relerr(c, ct.detach().numpy()) < 1e-12
    for ours, theirs in ((dx, x), (dW, W), (dR, R), (db, b), (dh0, h0), (dc0, c0)):
        assert _relerr(ours, theirs.grad.numpy()) < 1e-10


@pytest.mark.parametrize("zoneout", [False, True])
@pytest.mark.parametrize("T,N,C,H", SHAPES)
def test_gru_zoneout_autograd(T, N, C, H, zoneout):
    p = _problem(11, T, N, C, H, 3, zoneout)
    h, v = O.gru_forward(p["W"], p["R"], p["b"], p["b2"], p["x"], p["h0"], True,
                         0.4 if zoneout else 0.0, p["mask"])
    dx, dW, dR, dbx, dbr, dh0, _, _ = O.gru_backward(
        p["W"], p["R"], p["b"], p["b2"], p["x"], h, v, p["dh_new"], p["mask"])
    W, R, bx, br, x, h0 = (_t(p[k]) for k in ("W", "R", "b", "b2", "x", "h0"))
    mk = _t(p["mask"], False) if zoneout else None
    ht = torch_gru(W, R, bx, br, x, h0, mk)
    (ht[1:] * _t(p["dh_new"][1:], False)).sum().backward()
    assert _relerr(h, ht.detach().numpy()) < 1e-12
    for ours, theirs in ((dx, x), (dW, W), (dR, R), (dbx, bx), (dbr, br), (dh0, h0)):
        assert _relerr(ours, theirs.grad.numpy()) < 1e-10


@pytest.mark.parametrize("zoneout", [False, True])
@pytest.mark.parametrize("T,N,C,H", SHAPES)
def test_layer_norm_lstm_autograd(T, N, C, H, zoneout):
    p = _problem(12, T, N, C, H, 4, zoneout)
    fwd = O.layer_norm_lstm_forward(p["W"], p["R"], p["b"], p["gamma"], p["gamma_h"], p["beta_h"],
                                    p["x"], p["h0"], p["c0"], True, 0.4 if zoneout else 0.0, p["mask"])
    g = O.layer_norm_lstm_backward(p["W"], p["R"], p["b"], p["gamma"], p["gamma_h"], p["beta_h"],
                                   p["x"], fwd, p["dh_new"], p["dc_new"], p["mask"])
    W, R, b, gamma, gamma_h, beta_h, x, h0, c0 = (
        _t(p[k]) for k in ("W", "R", "b", "gamma", "gamma_h", "beta_h", "x", "h0", "c0"))
    mk = _t(p["mask"], False) if zoneout else None
    ht, ct = torch_ln_lstm(W, R, b, gamma, gamma_h, beta_h, x, h0, c0, mk)
    ((ht[1:] * _t(p["dh_new"][1:], False)).sum() + (ct[1:] * _t(p["dc_new"][1:], False)).sum()).backward()
    assert _relerr(fwd["h"], ht.detach().numpy()) < 1e-12
    assert _relerr(fwd["c"], ct.detach().numpy()) < 1e-12
    for name, theirs in (("dx", x), ("dW", W), ("dR", R), ("db", b), ("dh0", h0), ("dc0", c0),
                         ("dgamma", gamma), ("dgamma_h", gamma_h), ("dbeta_h", beta_h)):
        assert _relerr(g[name], theirs.grad.numpy()) < 1e-9, name


@pytest.mark.parametrize("zoneout", [False, True])
@pytest.mark.parametrize("T,N,C,H", SHAPES)
def test_layer_norm_gru_autograd(T, N, C, H, zoneout):
    p = _problem(13, T, N, C, H, 3, zoneout)
    fwd = O.layer_norm_gru_forward(p["W"], p["R"], p["b"], p["b2"], p["gamma"], p["x"], p["h0"],
                                   True, 0.4 if zoneout else 0.0, p["mask"])
    g = O.layer_norm_gru_backward(p["W"], p["R"], p["b"], p["b2"], p["gamma"], p["x"], fwd,
                                  p["dh_new"], p["mask"])
    W, R, bx, br, gamma, x, h0 = (_t(p[k]) for k in ("W", "R", "b", "b2", "gamma", "x", "h0"))
    mk = _t(p["mask"], False) if zoneout else None
    ht = torch_ln_gru(W, R, bx, br, gamma, x, h0, mk)
    (ht[1:] * _t(p["dh_new"][1:], False)).sum().backward()
    assert _relerr(fwd["h"], ht.detach().numpy()) < 1e-12
    for name, theirs in (("dx", x), ("dW", W), ("dR", R), ("dbx", bx), ("dbr", br), ("dh0", h0),
                         ("dgamma", gamma)):
        assert _relerr(g[name], theirs.grad.numpy()) < 1e-9, name


@pytest.mark.parametrize("layer_norm", [False, True])
@pytest.mark.parametrize("zoneout", [False, True])
@pytest.mark.parametrize("T,N,C,H", SHAPES)
def test_indrnn_autograd(T, N, C, H, zoneout, layer_norm):
    p = _problem(14, T, N, C, H, 1, zoneout)
    gam = p["gamma"] if layer_norm else None
    bias = p["b"]
    fwd = O.indrnn_forward(p["W"], p["u"], bias, p["x"], p["h0"], True,
                           0.4 if zoneout else 0.0, p["mask"], gam)
    g = O.indrnn_backward(p["W"], p["u"], bias, p["x"], fwd, p["dh_new"], p["mask"], gam)
    W, u, b, x, h0 = (_t(p[k]) for k in ("W", "u", "b", "x", "h0"))
    gamma = _t(p["gamma"]) if layer_norm else None
    mk = _t(p["mask"], False) if zoneout else None
    ht = torch_indrnn(W, u, b, x, h0, mk, gamma)
    (ht[1:] * _t(p["dh_new"][1:], False)).sum().backward()
    assert _relerr(fwd["h"], ht.detach().numpy()) < 1e-12
    for name, theirs in (("dx", x), ("dW", W), ("du", u), ("db", b), ("dh0", h0)):
        assert _relerr(g[name], theirs.grad.numpy()) < 1e-10, name
    if layer_norm:
        assert _relerr(g["dgamma"][0], gamma.grad.numpy()[0]) < 1e-10
        assert np.all(g["dgamma"][1] == 0)


# ---- finite differences (brute force on tiny shapes) ----------------------
def _fd(fun, arr, eps=1e-6):
    g = np.zeros_like(arr)
    it = np.nditer(arr, flags=["multi_index"])
    for _ in it:
        i = it.multi_index
        old = arr[i]
        arr[i] = old + eps
        fp = fun()
        arr[i] = old - eps
        fm = fun()
        arr[i] = old
        g[i] = (fp - fm) / (2 * eps)
    return g


def test_finite_differences_all_cells():
    T, N, C, H = 3, 2, 3, 4
    # LSTM with zoneout
    p = _problem(20, T, N, C, H, 4, True)

    def loss_lstm():
        h, c, _ = O.lstm_forward(p["W"], p["R"], p["b"], p["x"], p["h0"], p["c0"], True, 0.4, p["mask"])
        return (h[1:] * p["dh_new"][1:]).sum() + (c[1:] * p["dc_new"][1:]).sum()
    h, c, v = O.lstm_forward(p["W"], p["R"], p["b"], p["x"], p["h0"], p["c0"], True, 0.4, p["mask"])
    dx, dW, dR, db, dh0, dc0, _ = O.lstm_backward(
        p["W"], p["R"], p["b"], p["x"], h, c, v, p["dh_new"], p["dc_new"], p["mask"])
    for ours, key in ((dx, "x"), (dW, "W"), (dR, "R"), (db, "b"), (dh0, "h0"), (dc0, "c0")):
        assert _relerr(ours, _fd(loss_lstm, p[key])) < 1e-6, key

    # GRU with zoneout
    p = _problem(21, T, N, C, H, 3, True)

    def loss_gru():
        h, _ = O.gru_forward(p["W"], p["R"], p["b"], p["b2"], p["x"], p["h0"], True, 0.4, p["mask"])
        return (h[1:] * p["dh_new"][1:]).sum()
    h, v = O.gru_forward(p["W"], p["R"], p["b"], p["b2"], p["x"], p["h0"], True, 0.4, p["mask"])
    dx, dW, dR, dbx, dbr, dh0, _, _ = O.gru_backward(
        p["W"], p["R"], p["b"], p["b2"], p["x"], h, v, p["dh_new"], p["mask"])
    for ours, key in ((dx, "x"), (dW, "W"), (dR, "R"), (dbx, "b"), (dbr, "b2"), (dh0, "h0")):
        assert _relerr(ours, _fd(loss_gru, p[key])) < 1e-6, key

    # LayerNorm LSTM with zoneout
    p = _problem(22, T, N, C, H, 4, True)

    def fwd_lnl():
        return O.layer_norm_lstm_forward(p["W"], p["R"], p["b"], p["gamma"], p["gamma_h"], p["beta_h"],
                                         p["x"], p["h0"], p["c0"], True, 0.4, p["mask"])

    def loss_lnl():
        f = fwd_lnl()
        return (f["h"][1:] * p["dh_new"][1:]).sum() + (f["c"][1:] * p["dc_new"][1:]).sum()
    g = O.layer_norm_lstm_backward(p["W"], p["R"], p["b"], p["gamma"], p["gamma_h"], p["beta_h"],
                                   p["x"], fwd_lnl(), p["dh_new"], p["dc_new"], p["mask"])
    for name, key in (("dx", "x"), ("dW", "W"), ("dR", "R"), ("db", "b"), ("dh0", "h0"), ("dc0", "c0"),
                      ("dgamma", "gamma"), ("dgamma_h", "gamma_h"), ("dbeta_h", "beta_h")):
        assert _relerr(g[name], _fd(loss_lnl, p[key])) < 2e-6, name

    # LayerNorm GRU with zoneout
    p = _problem(23, T, N, C, H, 3, True)

    def fwd_lng():
        return O.layer_norm_gru_forward(p["W"], p["R"], p["b"], p["b2"], p["gamma"], p["x"], p["h0"],
                                        True, 0.4, p["mask"])

    def loss_lng():
        return (fwd_lng()["h"][1:] * p["dh_new"][1:]).sum()
    g = O.layer_norm_gru_backward(p["W"], p["R"], p["b"], p["b2"], p["gamma"], p["x"], fwd_lng(),
                                  p["dh_new"], p["mask"])
    for name, key in (("dx", "x"), ("dW", "W"), ("dR", "R"), ("dbx", "b"), ("dbr", "b2"), ("dh0", "h0"),
                      ("dgamma", "gamma")):
        assert _relerr(g[name], _fd(loss_lng, p[key])) < 2e-6, name

    # IndRNN with zoneout
    p = _problem(24, T, N, C, H, 1, True)

    def fwd_ind():
        return O.indrnn_forward(p["W"], p["u"], p["b"], p["x"], p["h0"], True, 0.4, p["mask"])

    def loss_ind():
        return (fwd_ind()["h"][1:] * p["dh_new"][1:]).sum()
    g = O.indrnn_backward(p["W"], p["u"], p["b"], p["x"], fwd_ind(), p["dh_new"], p["mask"])
    for name, key in (("dx", "x"), ("dW", "W"), ("du", "u"), ("db", "b"), ("dh0", "h0")):
        assert _relerr(g[name], _fd(loss_ind, p[key])) < 1e-6, name


# ---- invariants -----------------------------------------------------------
def test_zoneout_invariants():
    T, N, C, H = 5, 3, 4, 6
    p = _problem(30, T, N, C, H, 4, False)
    ones = np.ones((T, N, H))
    zeros = np.zeros((T, N, H))
    h_ref, c_ref, v_ref = O.lstm_forward(p["W"], p["R"], p["b"], p["x"], p["h0"], p["c0"])
    # mask == 1 everywhere: same as no zoneout, bit for bit
    h1, c1, _ = O.lstm_forward(p["W"], p["R"], p["b"], p["x"], p["h0"], p["c0"], True, 0.3, ones)
    assert np.array_equal(h1, h_ref) or _relerr(h1, h_ref) < 1e-15
    # mask == 0 everywhere: h never changes; dh0 = sum of upstream grads; dx == 0 when dc_new == 0
    h0s, c0s, v0s = O.lstm_forward(p["W"], p["R"], p["b"], p["x"], p["h0"], p["c0"], True, 0.3, zeros)
    assert all(np.array_equal(h0s[t], p["h0"]) for t in range(T + 1))
    dcz = np.zeros_like(p["dc_new"])
    dx, dW, dR, db, dh0, dc0, _ = O.lstm_backward(p["W"], p["R"], p["b"], p["x"], h0s, c0s, v0s,
                                                  p["dh_new"], dcz, zeros)
    assert np.allclose(dh0, p["dh_new"][1:].sum(0))
    assert np.all(dx == 0)
    # inference zoneout is the convex blend p*h_old + (1-p)*h_new (mask only enables it)
    hi, _, _ = O.lstm_forward(p["W"], p["R"], p["b"], p["x"][:1], p["h0"], p["c0"], False, 0.25, ones[:1])
    hn, _, _ = O.lstm_forward(p["W"], p["R"], p["b"], p["x"][:1], p["h0"], p["c0"], False)
    assert np.allclose(hi[1], 0.25 * p["h0"] + 0.75 * hn[1])
    # GRU, mask == 0: dx == 0 and dh0 == sum of upstream grads
    q = _problem(31, T, N, C, H, 3, False)
    hg, vg = O.gru_forward(q["W"], q["R"], q["b"], q["b2"], q["x"], q["h0"], True, 0.3, zeros)
    dx, *_rest = O.gru_backward(q["W"], q["R"], q["b"], q["b2"], q["x"], hg, vg, q["dh_new"], zeros)
    assert np.all(dx == 0)
    assert np.allclose(_rest[4], q["dh_new"][1:].sum(0))


def test_batch_permutation_and_accumulation_linearity():
    T, N, C, H = 4, 5, 3, 4
    p = _problem(32, T, N, C, H, 4, True)
    perm = np.array([3, 0, 4, 1, 2])
    h, c, v = O.lstm_forward(p["W"], p["R"], p["b"], p["x"], p["h0"], p["c0"], True, 0.4, p["mask"])
    hp, cp, vp = O.lstm_forward(p["W"], p["R"], p["b"], p["x"][:, perm], p["h0"][perm], p["c0"][perm],
                                True, 0.4, p["mask"][:, perm])
    assert np.allclose(hp, h[:, perm], rtol=0, atol=1e-14)
    # backward is linear in (dh_new, dc_new)
    a = O.lstm_backward(p["W"], p["R"], p["b"], p["x"], h, c, v, p["dh_new"], p["dc_new"], p["mask"])
    b2 = O.lstm_backward(p["W"], p["R"], p["b"], p["x"], h, c, v, 2 * p["dh_new"], 2 * p["dc_new"], p["mask"])
    for u1, u2 in zip(a, b2):
        assert np.allclose(2 * u1, u2, rtol=1e-12, atol=1e-12)
    assert np.all(np.abs(h) < 1.0 + np.abs(p["h0"]).max())
