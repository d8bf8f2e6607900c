"""Pins the oracle's LSTM, GRU and LayerNorm against library routines
(torch.nn.LSTM, torch.nn.GRU, torch.nn.functional.layer_norm) and their autograd.

The method is the reference's own `native_consistency` check
(reference validation/pytorch.py:65-89), extended to every gradient output.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import haste_oracle as O

torch.set_num_threads(4)


def _rng(seed):
    return np.random.default_rng(seed)


def _relerr(a, b):
    return np.max(np.abs(a - b)) / max(np.max(np.abs(b)), 1e-30)


@pytest.mark.parametrize("T,N,C,H", [(5, 3, 4, 6), (12, 4, 7, 5), (1, 2, 3, 4)])
def test_lstm_matches_torch_nn_lstm(T, N, C, H):
    r = _rng(1)
    k = 1.0 / np.sqrt(H)
    W = r.uniform(-k, k, (C, 4 * H))
    R = r.uniform(-k, k, (H, 4 * H))
    b = r.uniform(-k, k, 4 * H)
    x = r.standard_normal((T, N, C))
    h0 = r.standard_normal((N, H)) * 0.5
    c0 = r.standard_normal((N, H)) * 0.5
    dy = r.standard_normal((T, N, H))
    dhT = r.standard_normal((N, H))
    dcT = r.standard_normal((N, H))

    h, c, v = O.lstm_forward(W, R, b, x, h0, c0)
    dh_new = np.zeros((T + 1, N, H))
    dh_new[1:] = dy
    dh_new[T] += dhT
    dc_new = np.zeros((T + 1, N, H))
    dc_new[T] = dcT
    dx, dW, dR, db, dh0, dc0, _ = O.lstm_backward(W, R, b, x, h, c, v, dh_new, dc_new)

    w_ih, w_hh, b_ih, b_hh = O.lstm_to_native(W, R, b)
    m = torch.nn.LSTM(C, H).double()
    with torch.no_grad():
        m.weight_ih_l0.copy_(torch.from_numpy(w_ih))
        m.weight_hh_l0.copy_(torch.from_numpy(w_hh))
        m.bias_ih_l0.copy_(torch.from_numpy(b_ih))
        m.bias_hh_l0.copy_(torch.from_numpy(b_hh))
    xt = torch.from_numpy(x).requires_grad_()
    h0t = torch.from_numpy(h0).requires_grad_()
    c0t = torch.from_numpy(c0).requires_grad_()
    y, (hT, cT) = m(xt, (h0t[None], c0t[None]))
    loss = (y * torch.from_numpy(dy)).sum() + (hT[0] * torch.from_numpy(dhT)).sum() \
        + (cT[0] * torch.from_numpy(dcT)).sum()
    loss.backward()

    assert _relerr(h[1:], y.detach().numpy()) < 1e-12
    assert _relerr(c[T], cT[0].detach().numpy()) < 1e-12
    assert _relerr(dx, xt.grad.numpy()) < 1e-11
    assert _relerr(dh0, h0t.grad.numpy()) < 1e-11
    assert _relerr(dc0, c0t.grad.numpy()) < 1e-11
    # native grads come back in native layout: map ours into it
    gW, gR, gb, _ = O.lstm_to_native(dW, dR, db)
    assert _relerr(gW, m.weight_ih_l0.grad.numpy()) < 1e-11
    assert _relerr(gR, m.weight_hh_l0.grad.numpy()) < 1e-11
    assert _relerr(gb * 2.0, m.bias_ih_l0.grad.numpy()) < 1e-11
    assert _relerr(gb * 2.0, m.bias_hh_l0.grad.numpy()) < 1e-11


@pytest.mark.parametrize("T,N,C,H", [(5, 3, 4, 6), (9, 2, 5, 7), (1, 2, 3, 4)])
def test_gru_matches_torch_nn_gru(T, N, C, H):
    r = _rng(2)
    k = 1.0 / np.sqrt(H)
    W = r.uniform(-k, k, (C, 3 * H))
    R = r.uniform(-k, k, (H, 3 * H))
    bx = r.uniform(-k, k, 3 * H)
    br = r.uniform(-k, k, 3 * H)
    x = r.standard_normal((T, N, C))
    h0 = r.standard_normal((N, H)) * 0.5
    dy = r.standard_normal((T, N, H))

    h, v = O.gru_forward(W, R, bx, br, x, h0)
    dh_new = np.zeros((T + 1, N, H))
    dh_new[1:] = dy
    dx, dW, dR, dbx, dbr, dh0, _, _ = O.gru_backward(W, R, bx, br, x, h, v, dh_new)

    w_ih, w_hh, b_ih, b_hh = O.gru_to_native(W, R, bx, br)
    m = torch.nn.GRU(C, H).double()
    with torch.no_grad():
        m.weight_ih_l0.copy_(torch.from_numpy(w_ih))
        m.weight_hh_l0.copy_(torch.from_numpy(w_hh))
        m.bias_ih_l0.copy_(torch.from_numpy(b_ih))
        m.bias_hh_l0.copy_(torch.from_numpy(b_hh))
    xt = torch.from_numpy(x).requires_grad_()
    h0t = torch.from_numpy(h0).requires_grad_()
    y, _ = m(xt, h0t[None])
    (y * torch.from_numpy(dy)).sum().backward()

    assert _relerr(h[1:], y.detach().numpy()) < 1e-12
    assert _relerr(dx, xt.grad.numpy()) < 1e-11
    assert _relerr(dh0, h0t.grad.numpy()) < 1e-11
    gW, gR, gbx, gbr = O.gru_to_native(dW, dR, dbx, dbr)
    assert _relerr(gW, m.weight_ih_l0.grad.numpy()) < 1e-11
    assert _relerr(gR, m.weight_hh_l0.grad.numpy()) < 1e-11
    assert _relerr(gbx, m.bias_ih_l0.grad.numpy()) < 1e-11
    assert _relerr(gbr, m.bias_hh_l0.grad.numpy()) < 1e-11


@pytest.mark.parametrize("rows,D,with_beta", [(7, 16, True), (5, 33, False), (1, 4, True)])
def test_layer_norm_matches_functional(rows, D, with_beta):
    r = _rng(3)
    x = r.standard_normal((rows, D)) * 2.0 + 0.7
    gamma = r.standard_normal(D)
    beta = r.standard_normal(D) if with_beta else None
    dy = r.standard_normal((rows, D))

    y, cache = O.layer_norm_forward(x, gamma, beta)
    dx, dgamma, dbeta = O.layer_norm_backward(x, gamma, dy, cache)

    xt = torch.from_numpy(x).requires_grad_()
    gt = torch.from_numpy(gamma).requires_grad_()
    bt = torch.from_numpy(beta).requires_grad_() if with_beta else None
    yt = F.layer_norm(xt, (D,), gt, bt, eps=1e-5)
    (yt * torch.from_numpy(dy)).sum().backward()

    assert _relerr(y, yt.detach().numpy()) < 1e-12
    assert _relerr(dx, xt.grad.numpy()) < 1e-10
    assert _relerr(dgamma, gt.grad.numpy()) < 1e-11
    if with_beta:
        assert _relerr(dbeta, bt.grad.numpy()) < 1e-11
    # cache holds (mean, 1/sqrt(biased var + eps))
    assert np.allclose(cache[:, 0], x.mean(-1))
    assert np.allclose(cache[:, 1], 1.0 / np.sqrt(x.var(-1) + 1e-5))
