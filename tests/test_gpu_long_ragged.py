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
