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
