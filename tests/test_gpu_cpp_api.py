"""Drives tests/cpp/api_check (a C++ caller of include/haste.h, the libhaste-compatible
class API) with seeded inputs and checks everything it writes against the fp64 oracle."""
import os
import subprocess
import tempfile

import numpy as np
import pytest

from oracle import haste_oracle as O
from util import TOL, problem, relerr

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "cpp", "api_check")
DTYPE = np.float32  # np.float64 runs the classes instantiated for double ("f64:<cell>")
LENT_WORKSPACE = "0"  # "1": api_check lends the library its scratch memory (haste_hip_set_workspace)


def _run(cell, T, N, C, H, zoneout, inputs, out_shapes):
    if not os.path.exists(BIN):
        pytest.fail("tests/cpp/api_check is not built (python -c 'import __graft_entry__ as g; g.build()')")
    with tempfile.TemporaryDirectory() as d:
        fin, fout = os.path.join(d, "in.bin"), os.path.join(d, "out.bin")
        with open(fin, "wb") as f:
            for a in inputs:
                f.write(np.ascontiguousarray(a, dtype=DTYPE).tobytes())
        print("api_check", cell, T, N, C, H, zoneout, flush=True)
        res = subprocess.run([BIN, ("f64:" if DTYPE is np.float64 else "") + cell, str(T), str(N), str(C), str(H), str(zoneout), fin, fout],
                             capture_output=True, text=True, timeout=100,
                             env=dict(os.environ, HASTE_API_CHECK_LENT_WORKSPACE=LENT_WORKSPACE))
        assert res.returncode == 0, res.stdout + res.stderr
        raw = np.fromfile(fout, dtype=DTYPE).astype(np.float64)
    outs, off = [], 0
    for shp in out_shapes:
        n = int(np.prod(shp))
        outs.append(raw[off:off + n].reshape(shp))
        off += n
    assert off == raw.size
    return outs


CASES = [(5, 3, 7, 12, 0.0), (9, 20, 24, 64, 0.3)]


@pytest.mark.parametrize("T,N,C,H,zoneout", CASES)
@pytest.mark.parametrize("ln", [False, True, "iterate"])
def test_cpp_lstm(T, N, C, H, zoneout, ln):
    p = problem(700 + T + H, T, N, C, H, 4, zoneout)
    mask = [p["mask"]] if zoneout else []
    base = [p["W"], p["R"], p["b"], p["x"], p["h0"], p["c0"], p["dh_new"], p["dc_new"]]
    shapes = [(T + 1, N, H), (T + 1, N, H), (T, N, C), (C, 4 * H), (H, 4 * H), (4 * H,), (N, H), (N, H)]
    if ln is True:
        outs = _run("layer_norm_lstm", T, N, C, H, zoneout,
                    base + [p["gamma"], p["gamma_h"], p["beta_h"]] + mask,
                    shapes + [(2, 4 * H), (H,), (H,)])
        fwd = O.layer_norm_lstm_forward(p["W"], p["R"], p["b"], p["gamma"], p["gamma_h"], p["beta_h"],
                                        p["x"], p["h0"], p["c0"], True, zoneout, p["mask"])
        g = O.layer_norm_lstm_backward(p["W"], p["R"], p["b"], p["gamma"], p["gamma_h"], p["beta_h"],
                                       p["x"], fwd, p["dh_new"], p["dc_new"], p["mask"])
        ref = [fwd["h"], fwd["c"], g["dx"], g["dW"], g["dR"], g["db"], g["dh0"], g["dc0"],
               g["dgamma"], g["dgamma_h"], g["dbeta_h"]]
    else:
        # "iterate": the same problem one step at a time through Iterate()
        outs = _run("lstm_iterate" if ln else "lstm", T, N, C, H, zoneout, base + mask, shapes)
        h, c, v = O.lstm_forward(p["W"], p["R"], p["b"], p["x"], p["h0"], p["c0"], True, zoneout, p["mask"])
        dx, dW, dR, db, dh0, dc0, _ = O.lstm_backward(p["W"], p["R"], p["b"], p["x"], h, c, v,
                                                      p["dh_new"], p["dc_new"], p["mask"])
        ref = [h, c, dx, dW, dR, db, dh0, dc0]
    for i, (a, b) in enumerate(zip(outs, ref)):
        assert relerr(a, b) < TOL, i


@pytest.mark.parametrize("T,N,C,H,zoneout", CASES)
@pytest.mark.parametrize("ln", [False, True, "iterate"])
def test_cpp_gru(T, N, C, H, zoneout, ln):
    p = problem(710 + T + H, T, N, C, H, 3, zoneout)
    mask = [p["mask"]] if zoneout else []
    base = [p["W"], p["R"], p["b"], p["b2"], p["x"], p["h0"], p["dh_new"]]
    shapes = [(T + 1, N, H), (T, N, C), (C, 3 * H), (H, 3 * H), (3 * H,), (3 * H,), (N, H)]
    if ln is True:
        outs = _run("layer_norm_gru", T, N, C, H, zoneout, base + [p["gamma"]] + mask,
                    shapes + [(2, 3 * H)])
        fwd = O.layer_norm_gru_forward(p["W"], p["R"], p["b"], p["b2"], p["gamma"], p["x"], p["h0"],
                                       True, zoneout, p["mask"])
        g = O.layer_norm_gru_backward(p["W"], p["R"], p["b"], p["b2"], p["gamma"], p["x"], fwd,
                                      p["dh_new"], p["mask"])
        ref = [fwd["h"], g["dx"], g["dW"], g["dR"], g["dbx"], g["dbr"], g["dh0"], g["dgamma"]]
    else:
        outs = _run("gru_iterate" if ln else "gru", T, N, C, H, zoneout, base + mask, shapes)
        h, v = O.gru_forward(p["W"], p["R"], p["b"], p["b2"], p["x"], p["h0"], True, zoneout, p["mask"])
        dx, dW, dR, dbx, dbr, dh0, _, _ = O.gru_backward(p["W"], p["R"], p["b"], p["b2"], p["x"], h, v,
                                                         p["dh_new"], p["mask"])
        ref = [h, dx, dW, dR, dbx, dbr, dh0]
    for i, (a, b) in enumerate(zip(outs, ref)):
        assert relerr(a, b) < TOL, i


@pytest.mark.parametrize("T,N,C,H,zoneout", CASES)
@pytest.mark.parametrize("ln", [False, True])
def test_cpp_indrnn(T, N, C, H, zoneout, ln):
    p = problem(720 + T + H, T, N, C, H, 1, zoneout)
    mask = [p["mask"]] if zoneout else []
    gam = p["gamma"] if ln else None
    base = [p["W"], p["u"], p["b"], p["x"], p["h0"], p["dh_new"]]
    shapes = [(T + 1, N, H), (T, N, C), (C, H), (H,), (H,), (N, H)]
    outs = _run("layer_norm_indrnn" if ln else "indrnn", T, N, C, H, zoneout,
                base + ([gam] if ln else []) + mask, shapes + ([(2, H)] if ln else []))
    fwd = O.indrnn_forward(p["W"], p["u"], p["b"], p["x"], p["h0"], True, zoneout, p["mask"], gam)
    g = O.indrnn_backward(p["W"], p["u"], p["b"], p["x"], fwd, p["dh_new"], p["mask"], gam)
    ref = [fwd["h"], g["dx"], g["dW"], g["du"], g["db"], g["dh0"]] + ([g["dgamma"]] if ln else [])
    for i, (a, b) in enumerate(zip(outs, ref)):
        assert relerr(a, b) < TOL, i


def test_cpp_layer_norm_partial_cursor():
    rows_t, rows_n, D = 5, 7, 96
    rows = rows_t * rows_n
    r = np.random.default_rng(3)
    f32 = lambda a: a.astype(np.float32).astype(np.float64)
    x, gamma, beta, dy = (f32(r.standard_normal((rows, D))), f32(r.uniform(0.5, 1.5, D)),
                          f32(r.standard_normal(D)), f32(r.standard_normal((rows, D))))
    outs = _run("layer_norm", rows_t, rows_n, 1, D, 0.0, [x, gamma, beta, dy],
                [(rows, D), (rows, 2), (rows, D), (D,), (D,)])
    y, cache = O.layer_norm_forward(x, gamma, beta)
    dx, dgamma, dbeta = O.layer_norm_backward(x, gamma, dy, cache)
    for i, (a, b) in enumerate(zip(outs, [y, cache, dx, dgamma, dbeta])):
        assert relerr(a, b) < TOL, i


def test_cpp_classes_with_a_workspace_lent_by_the_caller(monkeypatch):
    """The same C++ callers with the library's scratch memory lent through haste_hip_set_workspace
    (sized by haste_hip_workspace_bytes) and haste_hip_stream_status asked at the end."""
    import sys
    monkeypatch.setattr(sys.modules[__name__], "LENT_WORKSPACE", "1")
    test_cpp_lstm(9, 20, 24, 64, 0.3, False)
    test_cpp_lstm(9, 20, 24, 64, 0.3, True)
    test_cpp_lstm(5, 3, 7, 12, 0.0, "iterate")
