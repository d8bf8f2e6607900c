"""Single-step Iterate entry points (LSTM, GRU; forward and backward) on the GPU: a
sequence of steps must reproduce the fp64 oracle's all-steps results, like Run does."""
import numpy as np
import pytest

from oracle import haste_oracle as O
from util import TOL, dev, host, problem, relerr

pytestmark = pytest.mark.gpu

SHAPES = [(3, 2, 3, 4), (4, 5, 7, 20), (5, 16, 32, 64), (3, 64, 48, 128), (4, 1, 128, 512),
          (2, 3, 16, 1536)]  # the last one streams R


@pytest.mark.parametrize("zoneout", [0.0, 0.3])
@pytest.mark.parametrize("T,N,C,H", SHAPES)
def test_lstm_iterate(T, N, C, H, zoneout):
    from haste_amd import ops
    import torch
    print("lstm iterate", T, N, C, H, zoneout, flush=True)
    p = problem(300 + T + N + C + H, T, N, C, H, 4, zoneout)
    W, R, b, x = dev(p["W"]), dev(p["R"]), dev(p["b"]), dev(p["x"])
    mask = dev(p["mask"]) if zoneout else None
    hs, cs, vs = [dev(p["h0"])], [dev(p["c0"])], []
    for t in range(T):
        h1, c1, v = ops.lstm_forward_iterate(True, zoneout, x[t].contiguous(), hs[t], cs[t], W, R, b,
                                             mask[t].contiguous() if zoneout else None)
        hs.append(h1), cs.append(c1), vs.append(v)
    ho, co, vo = O.lstm_forward(p["W"], p["R"], p["b"], p["x"], p["h0"], p["c0"], True, zoneout, p["mask"])
    assert relerr(host(torch.stack(hs)), ho) < TOL
    assert relerr(host(torch.stack(cs)), co) < TOL
    assert relerr(host(torch.stack(vs)), vo) < TOL

    # in-place state update (h_out aliases h), inference mode
    hi, ci = dev(p["h0"]).clone(), dev(p["c0"]).clone()
    for t in range(T):
        ops.lstm_forward_iterate(False, zoneout, x[t].contiguous(), hi, ci, W, R, b,
                                 mask[t].contiguous() if zoneout else None, h_out=hi, c_out=ci)
    hio, cio, _ = O.lstm_forward(p["W"], p["R"], p["b"], p["x"], p["h0"], p["c0"], False, zoneout, p["mask"])
    assert relerr(host(hi), hio[-1]) < TOL
    assert relerr(host(ci), cio[-1]) < TOL

    W_t, R_t = W.t().contiguous(), R.t().contiguous()
    opts = dict(device="cuda", dtype=W.dtype)
    dW, dR, db = torch.zeros(C, 4 * H, **opts), torch.zeros(H, 4 * H, **opts), torch.zeros(4 * H, **opts)
    dh, dc = torch.zeros(N, H, **opts), torch.zeros(N, H, **opts)
    dh_new, dc_new = dev(p["dh_new"]), dev(p["dc_new"])
    dxs = [None] * T
    for t in range(T - 1, -1, -1):
        dxs[t] = ops.lstm_backward_iterate(x[t].t().contiguous(), W_t, R_t, b, hs[t], cs[t], cs[t + 1],
                                           dh_new[t + 1].contiguous(), dc_new[t + 1].contiguous(),
                                           vs[t], dW, dR, db, dh, dc,
                                           mask[t].contiguous() if zoneout else None)
    torch.cuda.synchronize()
    ref = O.lstm_backward(p["W"], p["R"], p["b"], p["x"], ho, co, vo, p["dh_new"], p["dc_new"], p["mask"])
    for name, ours, theirs in zip(("dx", "dW", "dR", "db", "dh0", "dc0", "dv"),
                                  (torch.stack(dxs), dW, dR, db, dh, dc, torch.stack(vs)), ref):
        assert relerr(host(ours), theirs) < TOL, name


@pytest.mark.parametrize("zoneout", [0.0, 0.3])
@pytest.mark.parametrize("T,N,C,H", SHAPES)
def test_gru_iterate(T, N, C, H, zoneout):
    from haste_amd import ops
    import torch
    print("gru iterate", T, N, C, H, zoneout, flush=True)
    p = problem(400 + T + N + C + H, T, N, C, H, 3, zoneout)
    W, R, bx, br, x = dev(p["W"]), dev(p["R"]), dev(p["b"]), dev(p["b2"]), dev(p["x"])
    mask = dev(p["mask"]) if zoneout else None
    hs, vs = [dev(p["h0"])], []
    for t in range(T):
        h1, v = ops.gru_forward_iterate(True, zoneout, x[t].contiguous(), hs[t], W, R, bx, br,
                                        mask[t].contiguous() if zoneout else None)
        hs.append(h1), vs.append(v)
    ho, vo = O.gru_forward(p["W"], p["R"], p["b"], p["b2"], p["x"], p["h0"], True, zoneout, p["mask"])
    assert relerr(host(torch.stack(hs)), ho) < TOL
    assert relerr(host(torch.stack(vs)), vo) < TOL

    W_t, R_t = W.t().contiguous(), R.t().contiguous()
    opts = dict(device="cuda", dtype=W.dtype)
    dW, dR = torch.zeros(C, 3 * H, **opts), torch.zeros(H, 3 * H, **opts)
    dbx, dbr, dh = torch.zeros(3 * H, **opts), torch.zeros(3 * H, **opts), torch.zeros(N, H, **opts)
    dh_new = dev(p["dh_new"])
    dxs = [None] * T
    for t in range(T - 1, -1, -1):
        dxs[t] = ops.gru_backward_iterate(x[t].t().contiguous(), W_t, R_t, bx, br, hs[t], vs[t],
                                          dh_new[t + 1].contiguous(), dW, dR, dbx, dbr, dh,
                                          mask[t].contiguous() if zoneout else None)
    torch.cuda.synchronize()
    ref = O.gru_backward(p["W"], p["R"], p["b"], p["b2"], p["x"], ho, vo, p["dh_new"], p["mask"])
    for name, ours, theirs in zip(("dx", "dW", "dR", "dbx", "dbr", "dh0"),
                                  (torch.stack(dxs), dW, dR, dbx, dbr, dh), ref):
        assert relerr(host(ours), theirs) < TOL, name


# ---- the one-kernel single step (up to 8 rows): ragged and large sizes, both cells ----------
STEP_SHAPES = [(1, 1, 1), (8, 7, 5), (3, 100, 333), (8, 513, 1025), (2, 64, 4096), (5, 1030, 260), (7, 16, 16),
               (1, 2048, 512)]


@pytest.mark.parametrize("N,C,H", STEP_SHAPES)
@pytest.mark.parametrize("training,zoneout", [(True, 0.0), (True, 0.3), (False, 0.3)])
def test_single_step_kernel(N, C, H, training, zoneout):
    from haste_amd import ops
    import torch
    print("single step", N, C, H, training, zoneout, flush=True)
    p = problem(500 + N + C + H, 1, N, C, H, 4, zoneout)
    mask = dev(p["mask"][0]) if zoneout else None
    x, h0, c0 = dev(p["x"][0]), dev(p["h0"]), dev(p["c0"])
    h1, c1, v = ops.lstm_forward_iterate(training, zoneout, x, h0, c0, dev(p["W"]), dev(p["R"]), dev(p["b"]), mask)
    ho, co, vo = O.lstm_forward(p["W"], p["R"], p["b"], p["x"], p["h0"], p["c0"], training, zoneout, p["mask"])
    assert relerr(host(h1), ho[1]) < TOL and relerr(host(c1), co[1]) < TOL
    if training:
        assert relerr(host(v), vo[0]) < TOL
    # the state updated in place gives the same bits
    hi, ci = h0.clone(), c0.clone()
    ops.lstm_forward_iterate(training, zoneout, x, hi, ci, dev(p["W"]), dev(p["R"]), dev(p["b"]), mask,
                             h_out=hi, c_out=ci)
    torch.cuda.synchronize()
    assert torch.equal(hi, h1) and torch.equal(ci, c1)

    W3, R3 = dev(p["W"][:, :3 * H]), dev(p["R"][:, :3 * H])
    bx, br = dev(p["b"][:3 * H]), dev(p["b2"][:3 * H])
    g1, gv = ops.gru_forward_iterate(training, zoneout, x, h0, W3, R3, bx, br, mask)
    go, gvo = O.gru_forward(p["W"][:, :3 * H], p["R"][:, :3 * H], p["b"][:3 * H], p["b2"][:3 * H], p["x"], p["h0"],
                            training, zoneout, p["mask"])
    assert relerr(host(g1), go[1]) < TOL
    if training:
        assert relerr(host(gv), gvo[0]) < TOL
    gi = h0.clone()
    ops.gru_forward_iterate(training, zoneout, x, gi, W3, R3, bx, br, mask, h_out=gi)
    torch.cuda.synchronize()
    assert torch.equal(gi, g1)


@pytest.mark.parametrize("N,C,H", [(4, 48, 200), (8, 512, 512)])
def test_single_step_dropconnect_equals_premasked_weights(N, C, H):
    from haste_amd import ops
    import torch
    p = problem(77, 1, N, C, H, 4)
    r = np.random.default_rng(5)
    m = (r.uniform(size=p["R"].shape) >= 0.05).astype(np.float64)
    scale = 1.0 / 0.95
    args = (True, 0.0, dev(p["x"]), dev(p["h0"]), dev(p["c0"]), dev(p["W"]))
    h1, c1, v1 = ops.lstm_forward(*args, dev(p["R"]), dev(p["b"]), dev(None), dropconnect_mask=dev(m),
                                  dropconnect_scale=scale)
    R_eff = (dev(p["R"]) * dev(m)) * np.float32(scale)
    h2, c2, v2 = ops.lstm_forward(*args, R_eff.contiguous(), dev(p["b"]), dev(None))
    torch.cuda.synchronize()
    assert torch.equal(h1, h2) and torch.equal(c1, c2) and torch.equal(v1, v2)
