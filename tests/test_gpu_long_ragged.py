"""Long sequences at ragged shapes: LSTM and GRU forward + backward on the GPU vs the fp64 oracle.

The short ragged cases of test_gpu_lstm.py / test_gpu_gru.py have T <= 12 and the long ones
round shapes.  What the persistent kernels do between workgroups -- rotating polled tiles,
partial tiles polled in LDS, pieces of partial sums that are reset two steps after they were
read, a last workgroup that owns the padding, a set without rows, slice rows in registers on
groups that span XCDs -- depends on both at once: skew between workgroups builds up over the
steps and a ragged geometry decides who resets what.  Every case also runs twice and must
give the same bits.
"""
import numpy as np
import pytest

from oracle import haste_oracle as O
from util import TOL, dev, host, problem, relerr

pytestmark = pytest.mark.gpu

# (T, N, C, H); nothing a multiple of a tile
SHAPES = [
    (257, 37, 50, 300),   # two 4-row sets per workgroup, a ragged last set, a ragged last workgroup
    (64, 41, 24, 500),    # the same at H just under 512: 32 column workgroups, the last one ragged
    (257, 1, 16, 300),    # one batch row: weights in registers (forward), one 4-row tile (backward)
    (100, 5, 12, 200),    # 4-row tiles, two of them, one ragged
    (100, 13, 12, 390),   # 4-row tiles with the backward recurrence in scattered form (one set)
    (64, 130, 16, 200),   # tiles of 16 / 32 rows
    (64, 20, 16, 700),    # slice rows in registers, groups that span XCDs
    (64, 70, 8, 1000),    # the same with 16-row tiles of five groups
    (64, 9, 8, 1300),     # forward resident with slice rows in registers, backward step by step
]


def _lstm_once(p, zoneout):
    from haste_amd import ops
    import torch
    mask = dev(p["mask"])
    h, c, cache = ops.lstm_forward(True, zoneout, dev(p["x"]), dev(p["h0"]), dev(p["c0"]),
                                   dev(p["W"]), dev(p["R"]), dev(p["b"]), mask)
    torch.cuda.synchronize()
    fwd = (h.clone(), c.clone(), cache.clone())
    x_t = dev(p["x"]).permute(2, 0, 1).contiguous()
    dx, dh, dc, dW, dR, db = ops.lstm_backward(
        x_t, dev(p["W"]).t().contiguous(), dev(p["R"]).t().contiguous(), dev(p["b"]), mask, h, c, cache,
        dev(p["dh_new"]), dev(p["dc_new"]))
    torch.cuda.synchronize()
    return fwd, (dx, dW, dR, db, dh, dc, cache)  # the cache now holds the gate gradients


@pytest.mark.parametrize("zoneout", [0.0, 0.3])
@pytest.mark.parametrize("T,N,C,H", SHAPES)
def test_lstm_long_ragged(T, N, C, H, zoneout):
    import torch
    print("lstm long ragged", T, N, C, H, zoneout, flush=True)
    p = problem(1100 + T + N + C + H, T, N, C, H, 4, zoneout)
    fwd, grads = _lstm_once(p, zoneout)
    ho, co, vo = O.lstm_forward(p["W"], p["R"], p["b"], p["x"], p["h0"], p["c0"], True, zoneout, p["mask"])
    for name, ours, theirs in zip(("h", "c", "v"), fwd, (ho, co, vo)):
        assert relerr(host(ours), theirs) < TOL, name
    ref = O.lstm_backward(p["W"], p["R"], p["b"], p["x"], ho, co, vo, p["dh_new"], p["dc_new"], p["mask"])
    for name, ours, theirs in zip(("dx", "dW", "dR", "db", "dh0", "dc0", "dv"), grads, ref):
        assert relerr(host(ours), theirs) < TOL, name
    fwd2, grads2 = _lstm_once(p, zoneout)
    for a, b in zip(fwd + grads, fwd2 + grads2):
        assert torch.equal(a, b)


def _gru_once(p, zoneout):
    from haste_amd import ops
    import torch
    mask = dev(p["mask"])
    h, cache = ops.gru_forward(True, zoneout, dev(p["x"]), dev(p["h0"]), dev(p["W"]), dev(p["R"]),
                               dev(p["b"]), dev(p["b2"]), mask)
    torch.cuda.synchronize()
    x_t = dev(p["x"]).permute(2, 0, 1).contiguous()
    grads = ops.gru_backward(x_t, dev(p["W"]).t().contiguous(), dev(p["R"]).t().contiguous(),
                             dev(p["b"]), dev(p["b2"]), mask, h, cache, dev(p["dh_new"]))
    torch.cuda.synchronize()
    return (h, cache), tuple(grads)


@pytest.mark.parametrize("zoneout", [0.0, 0.3])
@pytest.mark.parametrize("T,N,C,H", SHAPES)
def test_gru_long_ragged(T, N, C, H, zoneout):
    import torch
    print("gru long ragged", T, N, C, H, zoneout, flush=True)
    p = problem(1200 + T + N + C + H, T, N, C, H, 3, zoneout)
    fwd, grads = _gru_once(p, zoneout)
    ho, vo = O.gru_forward(p["W"], p["R"], p["b"], p["b2"], p["x"], p["h0"], True, zoneout, p["mask"])
    assert relerr(host(fwd[0]), ho) < TOL
    assert relerr(host(fwd[1]), vo) < TOL
    dx, dW, dR, dbx, dbr, dh0, _, _ = O.gru_backward(p["W"], p["R"], p["b"], p["b2"], p["x"], ho, vo,
                                                     p["dh_new"], p["mask"])
    for name, ours, theirs in zip(("dx", "dh0", "dW", "dR", "dbx", "dbr"), grads,
                                  (dx, dh0, dW, dR, dbx, dbr)):
        assert relerr(host(ours), theirs) < TOL, name
    fwd2, grads2 = _gru_once(p, zoneout)
    for a, b in zip(fwd + grads, fwd2 + grads2):
        assert torch.equal(a, b)


# The layer-norm cells at the same geometries.  Their recurrences are chaotic for such weights (a
# float32 run of the oracle itself leaves its float64 self over a few dozen steps), so, as at
# BASELINE configuration 4, the check is: the free-running trajectory over the first steps,
# every step taken on its own from the GPU's state (the new state and everything the step
# saves for the backward pass), the backward pass on what the GPU's forward pass saved, and a
# second run with the same bits.
LN_SHAPES = [(257, 37, 50, 300), (64, 41, 24, 500), (100, 5, 12, 200), (64, 130, 16, 200),
             (64, 20, 16, 700), (64, 70, 8, 1000), (64, 9, 8, 1300)]
FREE_STEPS = 12


def _ln_lstm_once(p, zoneout):
    from haste_amd import ops
    import torch
    mask = dev(p["mask"])
    gam, gh, bh = dev(p["gamma"]), dev(p["gamma_h"]), dev(p["beta_h"])
    outs = ops.layer_norm_lstm_forward(True, zoneout, dev(p["x"]), dev(p["h0"]), dev(p["c0"]),
                                       dev(p["W"]), dev(p["R"]), dev(p["b"]), gam, gh, bh, mask)
    torch.cuda.synchronize()
    fwd = tuple(o.clone() for o in outs)  # the backward pass works in the saved buffers
    h, c, act_Wx, act_Wx_norm, cache1, act_Rh, cache2, act_c_norm, cache3 = outs
    grads = ops.layer_norm_lstm_backward(
        dev(p["x"]).permute(2, 0, 1).contiguous(), dev(p["W"]).t().contiguous(),
        dev(p["R"]).t().contiguous(), dev(p["b"]), gam, gh, bh, mask, h, c, act_Wx, act_Wx_norm,
        cache1, act_Rh, cache2, act_c_norm, cache3, dev(p["dh_new"]), dev(p["dc_new"]))
    torch.cuda.synchronize()
    return fwd, tuple(grads)


@pytest.mark.parametrize("zoneout", [0.0, 0.3])
@pytest.mark.parametrize("T,N,C,H", LN_SHAPES)
def test_layer_norm_lstm_long_ragged(T, N, C, H, zoneout):
    import torch
    print("ln_lstm long ragged", T, N, C, H, zoneout, flush=True)
    p = problem(1300 + T + N + C + H, T, N, C, H, 4, zoneout)
    fwd, grads = _ln_lstm_once(p, zoneout)
    h, c, act_Wx, act_Wx_norm, cache1, act_Rh, cache2, act_c_norm, cache3 = (host(o) for o in fwd)
    cache1, cache2, cache3 = (a.reshape(T, N, 2) for a in (cache1, cache2, cache3))
    args = (p["W"], p["R"], p["b"], p["gamma"], p["gamma_h"], p["beta_h"])
    mk = lambda a, b: None if p["mask"] is None else p["mask"][a:b]
    F = FREE_STEPS
    free = O.layer_norm_lstm_forward(*args, p["x"][:F], p["h0"], p["c0"], True, zoneout, mk(0, F))
    assert relerr(h[:F + 1], free["h"]) < TOL and relerr(c[:F + 1], free["c"]) < TOL
    worst = {}
    for t in range(T):
        one = O.layer_norm_lstm_forward(*args, p["x"][t:t + 1], h[t], c[t], True, zoneout, mk(t, t + 1))
        for name, ours, theirs in (("h", h[t + 1], one["h"][1]), ("c", c[t + 1], one["c"][1]),
                                   ("v", act_Wx_norm[t], one["v"][0]), ("act_Rh", act_Rh[t], one["act_Rh"][0]),
                                   ("act_c_norm", act_c_norm[t], one["act_c_norm"][0]),
                                   ("cache2", cache2[t], one["cache2"][0]), ("cache3", cache3[t], one["cache3"][0])):
            worst[name] = max(worst.get(name, 0.0), relerr(ours, theirs))
    assert max(worst.values()) < TOL, worst
    saved = dict(h=h, c=c, v=act_Wx_norm, act_Wx=act_Wx, act_Rh=act_Rh, act_c_norm=act_c_norm,
                 cache1=cache1, cache2=cache2, cache3=cache3)
    g = O.layer_norm_lstm_backward(*args, p["x"], saved, p["dh_new"], p["dc_new"], p["mask"])
    for name, ours in zip(("dx", "dh0", "dc0", "dW", "dR", "db", "dgamma", "dgamma_h", "dbeta_h"), grads):
        assert relerr(host(ours), g[name]) < TOL, name
    fwd2, grads2 = _ln_lstm_once(p, zoneout)
    for a, b in zip(fwd + grads, fwd2 + grads2):
        assert torch.equal(a, b)


def _ln_gru_once(p, zoneout):
    from haste_amd import ops
    import torch
    mask = dev(p["mask"])
    gam = dev(p["gamma"])
    outs = ops.layer_norm_gru_forward(True, zoneout, dev(p["x"]), dev(p["h0"]), dev(p["W"]), dev(p["R"]),
                                      dev(p["b"]), dev(p["b2"]), gam, mask)
    torch.cuda.synchronize()
    fwd = tuple(o.clone() for o in outs)
    h, cache, act_Wx, cache1, act_Rh, cache2 = outs
    grads = ops.layer_norm_gru_backward(
        dev(p["x"]).permute(2, 0, 1).contiguous(), dev(p["W"]).t().contiguous(),
        dev(p["R"]).t().contiguous(), dev(p["b"]), dev(p["b2"]), gam, mask, h, cache, act_Wx, cache1,
        act_Rh, cache2, dev(p["dh_new"]))
    torch.cuda.synchronize()
    return fwd, tuple(grads)


@pytest.mark.parametrize("zoneout", [0.0, 0.3])
@pytest.mark.parametrize("T,N,C,H", LN_SHAPES)
def test_layer_norm_gru_long_ragged(T, N, C, H, zoneout):
    import torch
    print("ln_gru long ragged", T, N, C, H, zoneout, flush=True)
    p = problem(1400 + T + N + C + H, T, N, C, H, 3, zoneout)
    fwd, grads = _ln_gru_once(p, zoneout)
    h, v, act_Wx, cache1, act_Rh, cache2 = (host(o) for o in fwd)
    cache1, cache2 = cache1.reshape(T, N, 2), cache2.reshape(T, N, 2)
    args = (p["W"], p["R"], p["b"], p["b2"], p["gamma"])
    mk = lambda a, b: None if p["mask"] is None else p["mask"][a:b]
    F = FREE_STEPS
    free = O.layer_norm_gru_forward(*args, p["x"][:F], p["h0"], True, zoneout, mk(0, F))
    assert relerr(h[:F + 1], free["h"]) < TOL
    worst = {}
    for t in range(T):
        one = O.layer_norm_gru_forward(*args, p["x"][t:t + 1], h[t], True, zoneout, mk(t, t + 1))
        for name, ours, theirs in (("h", h[t + 1], one["h"][1]), ("v", v[t], one["v"][0]),
                                   ("act_Rh", act_Rh[t], one["act_Rh"][0]),
                                   ("cache2", cache2[t], one["cache2"][0])):
            worst[name] = max(worst.get(name, 0.0), relerr(ours, theirs))
    assert max(worst.values()) < TOL, worst
    saved = dict(h=h, v=v, act_Wx=act_Wx, act_Rh=act_Rh, cache1=cache1, cache2=cache2)
    g = O.layer_norm_gru_backward(*args, p["x"], saved, p["dh_new"], p["mask"])
    for name, ours in zip(("dx", "dh0", "dW", "dR", "dbx", "dbr", "dgamma"), grads):
        assert relerr(host(ours), g[name]) < TOL, name
    fwd2, grads2 = _ln_gru_once(p, zoneout)
    for a, b in zip(fwd + grads, fwd2 + grads2):
        assert torch.equal(a, b)
