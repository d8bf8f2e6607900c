"""Writes the committed golden vectors under tests/golden/.

Usage: python tests/golden/make_fixtures.py

The reference (lmnt-com/haste) ships no golden vectors, known-answer tests or fixtures
for its fused-RNN path, so these files are produced here from two independent sources:

* `*_torchnn.npz` — inputs in the haste weight layout and the outputs/gradients that
  `torch.nn.LSTM` / `torch.nn.GRU` / `torch.nn.functional.layer_norm` (float64, CPU,
  autograd) give for them after the native-weight map of the reference
  (frameworks/pytorch/lstm.py:169-180, gru.py:171-178).  Nothing under oracle/ is used
  to make them, so they pin the oracle from outside.
* `*_oracle.npz` — inputs and the outputs of oracle/haste_oracle.py for the cells and
  options torch.nn cannot express (zoneout, layer-norm cells, IndRNN).  The oracle is
  pinned separately (autograd of forwards assembled from library pieces, finite
  differences); these files freeze its answers so that a later change to it, or to the
  GPU kernels, shows up against a constant.

Only inputs and expected outputs are stored (float64 arrays, a few KB per file).
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from oracle import haste_oracle as O  # noqa: E402


def f32(a):
    return np.asarray(a).astype(np.float32).astype(np.float64)


def inputs(seed, T, N, C, H, G, zoneout=0.0):
    r = np.random.default_rng(seed)
    k = 1.0 / np.sqrt(H)
    d = dict(
        W=f32(r.uniform(-k, k, (C, G * H))), R=f32(r.uniform(-k, k, (H, G * H))),
        b=f32(r.uniform(-k, k, G * H)), b2=f32(r.uniform(-k, k, G * H)),
        x=f32(r.standard_normal((T, N, C))), h0=f32(r.standard_normal((N, H)) * 0.5),
        c0=f32(r.standard_normal((N, H)) * 0.5),
        dh_new=f32(r.standard_normal((T + 1, N, H))), dc_new=f32(r.standard_normal((T + 1, N, H))),
        gamma=f32(r.uniform(0.5, 1.5, (2, G * H))), gamma_h=f32(r.uniform(0.5, 1.5, H)),
        beta_h=f32(r.uniform(-0.5, 0.5, H)), u=f32(r.uniform(-1, 1, H)))
    if zoneout:
        d["mask"] = (r.uniform(size=(T, N, H)) >= zoneout).astype(np.float64)
        d["zoneout"] = np.float64(zoneout)
    return d


def t64(a, grad=False):
    return torch.tensor(np.asarray(a), dtype=torch.float64, requires_grad=grad)


def lstm_native(W, R, b):
    # frameworks/pytorch/lstm.py:169-180: gate blocks i,g,f,o -> i,f,g,o, transposed,
    # the bias split evenly over b_ih and b_hh.
    def reorder(w):
        i, g, f, o = torch.chunk(w, 4, dim=-1)
        return torch.cat([i, f, g, o], dim=-1)
    return reorder(W).t(), reorder(R).t(), reorder(b) / 2, reorder(b) / 2


def gru_native(W, R, bx, br):
    # frameworks/pytorch/gru.py:171-178: gate blocks z,r,g -> r,z,g.
    def reorder(w):
        z, r, g = torch.chunk(w, 3, dim=-1)
        return torch.cat([r, z, g], dim=-1)
    return reorder(W).t(), reorder(R).t(), reorder(bx), reorder(br)


def make_lstm_torchnn():
    T, N, C, H = 6, 3, 5, 8
    d = inputs(11, T, N, C, H, 4)
    W, R, b, x = t64(d["W"], True), t64(d["R"], True), t64(d["b"], True), t64(d["x"], True)
    h0, c0 = t64(d["h0"], True), t64(d["c0"], True)
    w_ih, w_hh, b_ih, b_hh = lstm_native(W, R, b)
    y, hT, cT = torch._VF.lstm(x, (h0[None], c0[None]), [w_ih, w_hh, b_ih, b_hh], True, 1, 0.0,
                               False, False, False)
    # upstream gradients on every output step, and extra ones on the final h and c
    dy, dhT, dcT = t64(d["dh_new"][1:]), t64(d["dh_new"][0]), t64(d["dc_new"][T])
    loss = (y * dy).sum() + (hT[0] * dhT).sum() + (cT[0] * dcT).sum()
    dx, dW, dR, db, dh0, dc0 = torch.autograd.grad(loss, [x, W, R, b, h0, c0])
    keep = {k: d[k] for k in ("W", "R", "b", "x", "h0", "c0")}
    dh_new = np.concatenate([np.zeros((1, N, H)), dy.numpy()], 0)
    dh_new[T] += dhT.numpy()
    dc_new = np.zeros((T + 1, N, H))
    dc_new[T] = dcT.numpy()
    keep.update(dh_new=dh_new, dc_new=dc_new, y=y.detach().numpy(), h_T=hT[0].detach().numpy(),
                c_T=cT[0].detach().numpy(), dx=dx.numpy(), dW=dW.numpy(), dR=dR.numpy(), db=db.numpy(),
                dh0=dh0.numpy(), dc0=dc0.numpy())
    np.savez(os.path.join(HERE, "lstm_torchnn.npz"), **keep)


def make_gru_torchnn():
    T, N, C, H = 6, 3, 5, 8
    d = inputs(12, T, N, C, H, 3)
    W, R, bx, br = t64(d["W"], True), t64(d["R"], True), t64(d["b"], True), t64(d["b2"], True)
    x, h0 = t64(d["x"], True), t64(d["h0"], True)
    w_ih, w_hh, b_ih, b_hh = gru_native(W, R, bx, br)
    y, hT = torch._VF.gru(x, h0[None], [w_ih, w_hh, b_ih, b_hh], True, 1, 0.0, False, False, False)
    dy = t64(d["dh_new"][1:])
    dx, dW, dR, dbx, dbr, dh0 = torch.autograd.grad((y * dy).sum(), [x, W, R, bx, br, h0])
    keep = dict(W=d["W"], R=d["R"], bx=d["b"], br=d["b2"], x=d["x"], h0=d["h0"],
                dh_new=np.concatenate([np.zeros((1, N, H)), dy.numpy()], 0),
                y=y.detach().numpy(), dx=dx.numpy(), dW=dW.numpy(), dR=dR.numpy(), dbx=dbx.numpy(),
                dbr=dbr.numpy(), dh0=dh0.numpy())
    np.savez(os.path.join(HERE, "gru_torchnn.npz"), **keep)


def make_layer_norm_torchnn():
    rows, D = 7, 24
    r = np.random.default_rng(13)
    x, gamma, beta = f32(r.standard_normal((rows, D)) * 2 + 0.3), f32(r.uniform(0.5, 1.5, D)), f32(r.uniform(-1, 1, D))
    dy = f32(r.standard_normal((rows, D)))
    xt, gt, bt = t64(x, True), t64(gamma, True), t64(beta, True)
    y = torch.nn.functional.layer_norm(xt, (D,), gt, bt, eps=1e-5)
    dx, dgamma, dbeta = torch.autograd.grad((y * t64(dy)).sum(), [xt, gt, bt])
    np.savez(os.path.join(HERE, "layer_norm_torchnn.npz"), x=x, gamma=gamma, beta=beta, dy=dy,
             y=y.detach().numpy(), dx=dx.numpy(), dgamma=dgamma.numpy(), dbeta=dbeta.numpy())


def make_oracle_fixtures():
    T, N, C, H = 5, 3, 6, 8
    zo = 0.3

    d = inputs(21, T, N, C, H, 4, zo)
    h, c, v = O.lstm_forward(d["W"], d["R"], d["b"], d["x"], d["h0"], d["c0"], True, zo, d["mask"])
    dx, dW, dR, db, dh0, dc0, dv = O.lstm_backward(d["W"], d["R"], d["b"], d["x"], h, c, v,
                                                   d["dh_new"], d["dc_new"], d["mask"])
    hi, ci, _ = O.lstm_forward(d["W"], d["R"], d["b"], d["x"], d["h0"], d["c0"], False, zo, d["mask"])
    np.savez(os.path.join(HERE, "lstm_zoneout_oracle.npz"), **d, h=h, c=c, v=v, dx=dx, dW=dW, dR=dR,
             db=db, dh0=dh0, dc0=dc0, dv=dv, h_inference=hi, c_inference=ci)

    d = inputs(22, T, N, C, H, 3, zo)
    h, v = O.gru_forward(d["W"], d["R"], d["b"], d["b2"], d["x"], d["h0"], True, zo, d["mask"])
    out = O.gru_backward(d["W"], d["R"], d["b"], d["b2"], d["x"], h, v, d["dh_new"], d["mask"])
    names = ("dx", "dW", "dR", "dbx", "dbr", "dh0")
    np.savez(os.path.join(HERE, "gru_zoneout_oracle.npz"), **d, h=h, v=v,
             **{k: out[k] if isinstance(out, dict) else out[i] for i, k in enumerate(names)})

    d = inputs(23, T, N, C, H, 4, zo)
    fwd = O.layer_norm_lstm_forward(d["W"], d["R"], d["b"], d["gamma"], d["gamma_h"], d["beta_h"],
                                    d["x"], d["h0"], d["c0"], True, zo, d["mask"])
    bwd = O.layer_norm_lstm_backward(d["W"], d["R"], d["b"], d["gamma"], d["gamma_h"], d["beta_h"],
                                     d["x"], fwd, d["dh_new"], d["dc_new"], d["mask"])
    np.savez(os.path.join(HERE, "layer_norm_lstm_oracle.npz"), **d,
             **{"fwd_" + k: a for k, a in fwd.items()}, **{"bwd_" + k: a for k, a in bwd.items()})

    d = inputs(24, T, N, C, H, 3, zo)
    fwd = O.layer_norm_gru_forward(d["W"], d["R"], d["b"], d["b2"], d["gamma"], d["x"], d["h0"],
                                   True, zo, d["mask"])
    bwd = O.layer_norm_gru_backward(d["W"], d["R"], d["b"], d["b2"], d["gamma"], d["x"], fwd,
                                    d["dh_new"], d["mask"])
    np.savez(os.path.join(HERE, "layer_norm_gru_oracle.npz"), **d,
             **{"fwd_" + k: a for k, a in fwd.items()}, **{"bwd_" + k: a for k, a in bwd.items()})

    for name, use_gamma in (("indrnn_oracle.npz", False), ("layer_norm_indrnn_oracle.npz", True)):
        d = inputs(25 + use_gamma, T, N, C, H, 1, zo)
        gamma = d["gamma"] if use_gamma else None
        fwd = O.indrnn_forward(d["W"], d["u"], d["b"], d["x"], d["h0"], True, zo, d["mask"], gamma)
        bwd = O.indrnn_backward(d["W"], d["u"], d["b"], d["x"], fwd, d["dh_new"], d["mask"], gamma)
        np.savez(os.path.join(HERE, name), **d,
                 **{"fwd_" + k: a for k, a in fwd.items() if a is not None},
                 **{"bwd_" + k: a for k, a in bwd.items()})


if __name__ == "__main__":
    make_lstm_torchnn()
    make_gru_torchnn()
    make_layer_norm_torchnn()
    make_oracle_fixtures()
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
