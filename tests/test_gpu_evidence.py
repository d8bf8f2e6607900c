"""Evidence beyond the per-shape parity tests: the zoneout keep path bit for bit, saturated
gate pre-activations and the tanh series / rational switch, the drift of the chaotic
LayerNormLSTM configuration against the float32 oracle's own, many launches in a row
bit-equal to the first, and two host threads on two streams.

Zoneout semantics: reference lib/lstm_forward_gpu.cu.cc:77-83 (h = (h_new - h_old) * mask +
h_old, so with a 0/1 mask h[t+1] == h[t] exactly where the mask is 0)."""
import threading

import numpy as np
import pytest

from oracle import haste_oracle as O
from util import TOL, dev, host, problem, relerr

pytestmark = pytest.mark.gpu


def _kept_exactly(h, mask):
    """h[T+1,N,H], mask[T,N,H] of 0/1: every kept element equals its predecessor bit for bit."""
    import torch
    keep = mask == 0
    assert int(keep.sum()) > 0
    a = h[1:][keep].view(torch.int32)
    b = h[:-1][keep].view(torch.int32)
    return torch.equal(a, b)


# tiny / ragged, the GRU + LSTM training configurations (N=64, T=100, H=512), the single-row
# kernel, the LayerNormLSTM configuration (N=32, T=500, H=256) and a streamed-R size
ZONEOUT_SHAPES = [(5, 3, 7, 5), (6, 17, 20, 36), (100, 64, 512, 512), (9, 1, 16, 300),
                  (500, 32, 256, 256), (3, 5, 24, 640)]


@pytest.mark.parametrize("T,N,C,H", ZONEOUT_SHAPES)
def test_zoneout_keeps_the_previous_state_bit_for_bit(T, N, C, H):
    import torch
    from haste_amd import ops
    print("zoneout keep path", T, N, C, H, flush=True)
    p = problem(900 + T + N, T, N, C, H, 4, 0.1)
    mask = dev(p["mask"])
    x, h0, c0 = dev(p["x"]), dev(p["h0"]), dev(p["c0"])
    # LSTM
    h, _, _ = ops.lstm_forward(True, 0.1, x, h0, c0, dev(p["W"]), dev(p["R"]), dev(p["b"]), mask)
    assert _kept_exactly(h, mask), "lstm"
    # GRU
    W3, R3 = dev(p["W"][:, :3 * H]), dev(p["R"][:, :3 * H])
    h, _ = ops.gru_forward(True, 0.1, x, h0, W3, R3, dev(p["b"][:3 * H]), dev(p["b2"][:3 * H]), mask)
    assert _kept_exactly(h, mask), "gru"
    # IndRNN, LayerNormIndRNN
    W1 = dev(p["W"][:, :H])
    h = ops.indrnn_forward(True, 0.1, x, h0, W1, dev(p["u"]), dev(p["b"][:H]), mask)
    assert _kept_exactly(h, mask), "indrnn"
    h = ops.layer_norm_indrnn_forward(True, 0.1, x, h0, W1, dev(p["u"]), dev(p["b"][:H]),
                                      dev(p["gamma"][:1, :H]), mask)[0]
    assert _kept_exactly(h, mask), "layer_norm_indrnn"
    if H >= 4:
        # LayerNormLSTM, LayerNormGRU
        h = ops.layer_norm_lstm_forward(True, 0.1, x, h0, c0, dev(p["W"]), dev(p["R"]), dev(p["b"]),
                                        dev(p["gamma"]), dev(p["gamma_h"]), dev(p["beta_h"]), mask)[0]
        assert _kept_exactly(h, mask), "layer_norm_lstm"
        h = ops.layer_norm_gru_forward(True, 0.1, x, h0, W3, R3, dev(p["b"][:3 * H]),
                                       dev(p["b2"][:3 * H]), dev(p["gamma"][:, :3 * H]), mask)[0]
        assert _kept_exactly(h, mask), "layer_norm_gru"
    torch.cuda.synchronize()


@pytest.mark.parametrize("scale", [30.0, 90.0, 1e4, 1e30])
@pytest.mark.parametrize("T,N,C,H", [(6, 5, 8, 36), (5, 1, 8, 64), (4, 40, 16, 128)])
def test_saturated_gate_pre_activations(T, N, C, H, scale):
    """|pre-activation| of 30 .. 1e30 (and, through the bias, both signs in every gate): sigma
    and tanh must saturate to exactly representable neighbours of 0 / 1 / -1, never NaN."""
    import torch
    from haste_amd import ops
    p = problem(77, T, N, C, H, 4)
    r = np.random.default_rng(int(scale) % 1000 + T)
    f32 = lambda a: a.astype(np.float32).astype(np.float64)
    p["x"] = f32(p["x"] * scale)
    p["b"] = f32(r.choice([-1.0, 1.0], size=4 * H) * scale * r.uniform(0.5, 1.0, 4 * H))
    h, c, v = ops.lstm_forward(True, 0.0, dev(p["x"]), dev(p["h0"]), dev(p["c0"]), dev(p["W"]),
                               dev(p["R"]), dev(p["b"]), dev(None))
    torch.cuda.synchronize()
    assert bool(torch.isfinite(h).all()) and bool(torch.isfinite(c).all()) and bool(torch.isfinite(v).all())
    with np.errstate(over="ignore"):
        ho, co, vo = O.lstm_forward(p["W"], p["R"], p["b"], p["x"], p["h0"], p["c0"])
    assert relerr(host(v), vo) < TOL and relerr(host(h), ho) < TOL and relerr(host(c), co) < TOL
    # GRU through the same inputs
    W3, R3 = dev(p["W"][:, :3 * H]), dev(p["R"][:, :3 * H])
    hg, vg = ops.gru_forward(True, 0.0, dev(p["x"]), dev(p["h0"]), W3, R3, dev(p["b"][:3 * H]),
                             dev(p["b2"][:3 * H]), dev(None))
    torch.cuda.synchronize()
    assert bool(torch.isfinite(hg).all())
    with np.errstate(over="ignore"):
        hgo, vgo = O.gru_forward(p["W"][:, :3 * H], p["R"][:, :3 * H], p["b"][:3 * H], p["b2"][:3 * H],
                                 p["x"], p["h0"])
    assert relerr(host(hg), hgo) < TOL
    # z, r, g saturate; the fourth cached block (Rh_g + br_g) is a plain product
    assert relerr(host(vg)[..., :3 * H], vgo[..., :3 * H]) < TOL


def test_tanh_across_the_series_switch():
    """IndRNN with W = I, u = 0, b = 0 is h[t+1] = tanh(x[t]) element by element: a sweep of x
    that straddles |x| = 0.25 (where the device tanh changes from its odd series to the
    exponential form) and runs out to saturation, against numpy's tanh.  Relative error per
    element, so the small arguments count as much as the large ones."""
    import torch
    from haste_amd import ops
    H = 256
    xs = np.concatenate([
        np.linspace(0.2499, 0.2501, 2048), -np.linspace(0.2499, 0.2501, 2048),
        np.geomspace(1e-30, 0.25, 4096), -np.geomspace(1e-30, 0.25, 4096),
        np.linspace(0.25, 20.0, 4096), -np.linspace(0.25, 20.0, 4096),
        np.array([0.0, 0.25, -0.25, np.nextafter(np.float32(0.25), np.float32(0)),
                  np.nextafter(np.float32(0.25), np.float32(1)), 88.0, -88.0, 1e10, -1e10] + [0.0] * 247)])
    xs = xs.astype(np.float32).astype(np.float64)
    assert xs.size % H == 0
    T = xs.size // H
    x = xs.reshape(T, 1, H)
    h = ops.indrnn_forward(False, 0.0, dev(x), dev(np.zeros((1, H))), dev(np.eye(H)), dev(np.zeros(H)),
                           dev(np.zeros(H)), dev(None))
    torch.cuda.synchronize()
    got = host(h)[1:].reshape(-1)
    want = np.tanh(xs)
    nz = want != 0
    rel = np.abs(got[nz] - want[nz]) / np.abs(want[nz])
    print("tanh: max relative error %.3e at x = %r" % (rel.max(), xs[nz][rel.argmax()]), flush=True)
    assert rel.max() < 2e-6, (rel.max(), xs[nz][rel.argmax()])
    assert np.all(got[~nz] == 0)
    assert np.all(np.abs(got) <= 1.0)


def test_config4_drift_stays_within_the_float32_noise_floor():
    """LayerNormLSTM N=32 T=500 C=H=256 is chaotic: any float32 evaluation drifts from the
    float64 trajectory.  The oracle itself run in float32 gives the size of that drift; the
    GPU's free-running trajectory must stay within 3x of it at t = 50, 100 and 200 (and
    within the plain tolerance where the floor is below it)."""
    import torch
    from haste_amd import ops
    T, N, C, H = 200, 32, 256, 256
    p = problem(4, 500, N, C, H, 4, 0.1, forget_bias=1.0)
    p["gamma"][:] = 1.0
    p["gamma_h"][:] = 1.0
    p["beta_h"][:] = 0.0
    names = ("W", "R", "b", "gamma", "gamma_h", "beta_h")
    x, mask = p["x"][:T], p["mask"][:T]
    f64 = O.layer_norm_lstm_forward(*[p[k] for k in names], x, p["h0"], p["c0"], True, 0.1, mask)
    f32 = O.layer_norm_lstm_forward(*[p[k].astype(np.float32) for k in names], x.astype(np.float32),
                                    p["h0"].astype(np.float32), p["c0"].astype(np.float32), True,
                                    np.float32(0.1), mask.astype(np.float32))
    outs = ops.layer_norm_lstm_forward(True, 0.1, dev(x), dev(p["h0"]), dev(p["c0"]), dev(p["W"]),
                                       dev(p["R"]), dev(p["b"]), dev(p["gamma"]), dev(p["gamma_h"]),
                                       dev(p["beta_h"]), dev(mask))
    torch.cuda.synchronize()
    hg, cg = host(outs[0]), host(outs[1])
    for t in (50, 100, 200):
        for name, g, a, b in (("h", hg, f32["h"], f64["h"]), ("c", cg, f32["c"], f64["c"])):
            floor = relerr(a[t], b[t])
            drift = relerr(g[t], b[t])
            print("t=%d %s: gpu drift %.3e, float32 oracle drift %.3e" % (t, name, drift, floor), flush=True)
            assert drift <= max(3.0 * floor, TOL), (t, name, drift, floor)


def _metric_problem():
    T, N, C, H = 100, 64, 512, 512
    p = problem(31, T, N, C, H, 4, forget_bias=1.0)
    d = {k: dev(p[k]) for k in ("x", "h0", "c0", "W", "R", "b", "dh_new", "dc_new")}
    d["x_t"] = d["x"].permute(2, 0, 1).contiguous()
    d["W_t"] = d["W"].t().contiguous()
    d["R_t"] = d["R"].t().contiguous()
    return d


def _fwd_bwd(ops, d, none):
    h, c, v = ops.lstm_forward(True, 0.0, d["x"], d["h0"], d["c0"], d["W"], d["R"], d["b"], none)
    g = ops.lstm_backward(d["x_t"], d["W_t"], d["R_t"], d["b"], none, h, c, v, d["dh_new"], d["dc_new"])
    return (h, c) + tuple(g)


def test_many_launches_in_a_row_are_bit_equal_to_the_first():
    """3000 forward + backward passes at the metric shape and 200 passes of the streaming
    inference shape (N=1, T=2000): the lock-free exchanges (polled tiles, polled partial tiles,
    epochs and tickets that only ever grow) must give the first launch's bits every time.
    Stops at the first mismatch."""
    import torch
    from haste_amd import ops
    none = dev(None)
    d = _metric_problem()
    first = _fwd_bwd(ops, d, none)
    torch.cuda.synchronize()
    for i in range(3000):
        outs = _fwd_bwd(ops, d, none)
        if i % 100 == 99:
            torch.cuda.synchronize()
            print("metric shape: %d launches" % (i + 1), flush=True)
        same = all(torch.equal(a, b) for a, b in zip(first, outs))  # synchronizes
        assert same, "launch %d differs from the first" % (i + 1)
    T, C, H = 2000, 512, 512
    p = problem(32, T, 1, C, H, 4)
    args = (False, 0.0, dev(p["x"]), dev(p["h0"]), dev(p["c0"]), dev(p["W"]), dev(p["R"]), dev(p["b"]), none)
    h1, c1, _ = ops.lstm_forward(*args)
    for i in range(200):
        h2, c2, _ = ops.lstm_forward(*args)
        assert torch.equal(h1, h2) and torch.equal(c1, c2), "streaming launch %d differs" % (i + 1)
    print("streaming shape: 200 launches", flush=True)


@pytest.mark.parametrize("T,N,C,H,launches", [(50, 32, 32, 256, 400), (20, 64, 16, 768, 150), (30, 8, 16, 128, 200)])
def test_many_layer_norm_launches_in_a_row_are_bit_equal_to_the_first(T, N, C, H, launches):
    """The layer-norm cells add tagged row exchanges, gathers inside a wavefront and inputs parked
    in LDS by a helper wavefront to the lock-free machinery: repeated LayerNormLSTM and LayerNormGRU
    forward + backward passes (4-row tiles with parked inputs; tall tiles across XCDs; a tile that
    leaves wavefronts idle) must give the first launch's bits every time.  Stops at the first
    mismatch."""
    import torch
    from haste_amd import ops
    print("ln soak", T, N, C, H, launches, flush=True)
    p = problem(77 + H, T, N, C, H, 4, 0.2)
    mask = dev(p["mask"])
    x, h0, c0 = dev(p["x"]), dev(p["h0"]), dev(p["c0"])
    W, R, b = dev(p["W"]), dev(p["R"]), dev(p["b"])
    gam, gh, bh = dev(p["gamma"]), dev(p["gamma_h"]), dev(p["beta_h"])
    x_t, W_t, R_t = ops.transpose3(x, W, R)
    dh_new, dc_new = dev(p["dh_new"]), dev(p["dc_new"])

    def lstm_pass():
        outs = ops.layer_norm_lstm_forward(True, 0.2, x, h0, c0, W, R, b, gam, gh, bh, mask)
        h, c, act_Wx, act_Wx_norm, cache1, act_Rh, cache2, act_c_norm, cache3 = outs
        keep = (h.clone(), c.clone(), act_Rh.clone(), act_c_norm.clone())
        g = ops.layer_norm_lstm_backward(x_t, W_t, R_t, b, gam, gh, bh, mask, h, c, act_Wx, act_Wx_norm,
                                         cache1, act_Rh, cache2, act_c_norm, cache3, dh_new, dc_new)
        return keep + tuple(g)

    W3, R3, b3 = W[:, :3 * H].contiguous(), R[:, :3 * H].contiguous(), b[:3 * H].contiguous()
    gam3 = gam[:, :3 * H].contiguous()
    x_t3, W3_t, R3_t = ops.transpose3(x, W3, R3)

    def gru_pass():
        h, cache, act_Wx, cache1, act_Rh, cache2 = ops.layer_norm_gru_forward(
            True, 0.2, x, h0, W3, R3, b3, b3, gam3, mask)
        keep = (h.clone(), act_Rh.clone())
        g = ops.layer_norm_gru_backward(x_t3, W3_t, R3_t, b3, b3, gam3, mask, h, cache, act_Wx, cache1,
                                        act_Rh, cache2, dh_new)
        return keep + tuple(g)

    for name, one_pass in (("LayerNormLSTM", lstm_pass), ("LayerNormGRU", gru_pass)):
        first = one_pass()
        torch.cuda.synchronize()
        for i in range(launches):
            outs = one_pass()
            same = all(torch.equal(a, b) for a, b in zip(first, outs))  # synchronizes
            assert same, "%s launch %d differs from the first" % (name, i + 1)
        print("%s: %d launches" % (name, launches), flush=True)


def test_two_host_threads_on_two_streams_match_the_serial_results():
    """Each thread runs forward + backward passes of its own problem on its own stream; the
    persistent kernels of the two streams are chained by the library.  Results must equal the
    serial ones bit for bit."""
    import torch
    from haste_amd import ops
    shapes = [(40, 64, 128, 512), (60, 16, 64, 256)]
    probs = []
    for i, (T, N, C, H) in enumerate(shapes):
        p = problem(40 + i, T, N, C, H, 4, 0.1)
        d = {k: dev(p[k]) for k in ("x", "h0", "c0", "W", "R", "b", "dh_new", "dc_new", "mask")}
        d["x_t"] = d["x"].permute(2, 0, 1).contiguous()
        d["W_t"] = d["W"].t().contiguous()
        d["R_t"] = d["R"].t().contiguous()
        probs.append(d)

    def run(d):
        h, c, v = ops.lstm_forward(True, 0.1, d["x"], d["h0"], d["c0"], d["W"], d["R"], d["b"], d["mask"])
        g = ops.lstm_backward(d["x_t"], d["W_t"], d["R_t"], d["b"], d["mask"], h, c, v, d["dh_new"],
                              d["dc_new"])
        return (h, c) + tuple(g)

    serial = [run(d) for d in probs]
    torch.cuda.synchronize()
    results = [None, None]
    errors = []

    def worker(i):
        try:
            s = torch.cuda.Stream()
            with torch.cuda.stream(s):
                outs = []
                for _ in range(20):
                    outs.append(run(probs[i]))
                s.synchronize()
                results[i] = outs
        except Exception as e:  # surfaced below
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not errors, errors
    assert all(not t.is_alive() for t in threads)
    torch.cuda.synchronize()
    for i in range(2):
        for outs in results[i]:
            for a, b in zip(serial[i], outs):
                assert torch.equal(a, b)
