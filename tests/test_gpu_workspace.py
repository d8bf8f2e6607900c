"""Caller-owned scratch memory (haste_hip_set_workspace / haste_hip_workspace_bytes), calls
recorded into a HIP graph, and the status of a stream's persistent kernels
(haste_hip_stream_status).  The reference hands every buffer in from the caller
(lib/haste/lstm.h:98-117) and has no error reporting; these are this library's counterparts.
"""
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _inputs(T, N, C, H, dev, seed=0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    k = H ** -0.5
    u = lambda *s: ((torch.rand(*s, generator=g, dtype=torch.float64) * 2 - 1) * k).to(dtype).to(dev)
    n = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64).to(dtype).to(dev)
    return dict(x=n(T, N, C), W=u(C, 4 * H), R=u(H, 4 * H), b=u(4 * H), h0=torch.zeros(N, H, device=dev, dtype=dtype),
                dh=n(T + 1, N, H), dc=n(T + 1, N, H),
                mask=(torch.rand(T, N, H, generator=g) >= 0.1).to(dtype).to(dev))


def _lstm_step(ops, a):
    """Forward + backward as the reference's benchmark loop does it."""
    h, c, cache = ops.lstm_forward(True, 0.1, a["x"], a["h0"], a["h0"], a["W"], a["R"], a["b"], a["mask"])
    x_t = ops.transpose(a["x"])
    W_t = ops.transpose(a["W"])
    R_t = ops.transpose(a["R"])
    dx, dh, dc, dW, dR, db = ops.lstm_backward(x_t, W_t, R_t, a["b"], a["mask"], h, c, cache, a["dh"], a["dc"])
    return dict(h=h, c=c, dx=dx, dh=dh, dc=dc, dW=dW, dR=dR, db=db)


@pytest.mark.parametrize("shape", [(12, 64, 512, 512), (9, 5, 40, 72), (3, 2, 64, 1536)])
def test_graph_replays_with_a_lent_workspace_match_eager(shape):
    """Forward + backward recorded into a graph on a stream whose scratch memory the caller
    lent: every replay -- with eager library work of another shape and synchronizations in
    between -- gives the eager results bit for bit.  (12, 64, 512, 512): two-set kernels with
    the fused input projection, split GEMMs; (3, 2, 64, 1536): the step-wise regime.)"""
    from haste_amd import ops
    T, N, C, H = shape
    dev = torch.device("cuda:0")
    a = _inputs(T, N, C, H, dev)
    other = _inputs(5, 7, 24, 48, dev, seed=1)
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        need = max(ops.workspace_bytes(T, N, C, H), ops.workspace_bytes(5, 7, 24, 48))
        lent = torch.empty(need, dtype=torch.uint8, device=dev)
        ops.set_workspace(lent)
        try:
            eager = {k: v.clone() for k, v in _lstm_step(ops, a).items()}
            other_eager = {k: v.clone() for k, v in _lstm_step(ops, other).items()}
            s.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=s):
                out = _lstm_step(ops, a)
            for replay in range(4):
                print("replay", replay, shape, flush=True)
                for v in out.values():
                    v.fill_(float("nan"))
                between = _lstm_step(ops, other)      # eager launches between the replays
                s.synchronize()
                graph.replay()
                s.synchronize()
                ops.stream_status()
                for k in eager:
                    assert torch.equal(out[k], eager[k]), (replay, k)
                    assert torch.equal(between[k], other_eager[k]), (replay, "eager between", k)
            del graph
        finally:
            s.synchronize()
            ops.set_workspace(None)


def test_lent_workspace_too_small_is_refused_before_anything_runs():
    from haste_amd import lib, ops
    dev = torch.device("cuda:0")
    a = _inputs(6, 64, 512, 512, dev)
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        lent = torch.empty(128 * 1024, dtype=torch.uint8, device=dev)
        ops.set_workspace(lent)
        try:
            with pytest.raises(lib.HasteHipError) as e:
                ops.lstm_forward(True, 0.0, a["x"], a["h0"], a["h0"], a["W"], a["R"], a["b"], a["mask"])
            assert e.value.code == 2 and "too small" in str(e.value)
        finally:
            s.synchronize()
            ops.set_workspace(None)
        # and the stream works again with a workspace of the library's own
        h, _, _ = ops.lstm_forward(True, 0.0, a["x"], a["h0"], a["h0"], a["W"], a["R"], a["b"], a["mask"])
        s.synchronize()
        assert torch.isfinite(h).all()


def test_set_workspace_checks_its_arguments():
    import ctypes
    from haste_amd import lib
    handle = lib.load()
    handle.haste_hip_set_workspace.restype = ctypes.c_int
    handle.haste_hip_set_workspace.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]
    buf = torch.empty(1 << 20, dtype=torch.uint8, device="cuda:0")
    s = torch.cuda.Stream()
    assert handle.haste_hip_set_workspace(s.cuda_stream, buf.data_ptr() + 4, 1 << 19) == 1   # unaligned
    assert handle.haste_hip_set_workspace(s.cuda_stream, buf.data_ptr(), 1024) == 1          # no room for the control block
    assert handle.haste_hip_set_workspace(s.cuda_stream, None, 0) == 0


CELLS = ["lstm", "gru", "layer_norm_lstm", "layer_norm_gru", "indrnn", "layer_norm_indrnn"]


@pytest.mark.parametrize("shape", [(7, 3, 20, 36), (20, 64, 512, 512), (5, 128, 256, 1024), (4, 33, 96, 1536),
                                   (3, 1, 64, 2048), (50, 32, 256, 256)])
def test_workspace_bytes_bounds_what_every_cell_needs(shape):
    """Every layer, forward and backward, float and double, on a fresh stream: what the library
    asked of its own workspace stays below haste_hip_workspace_bytes for that shape."""
    from haste_amd import layers, ops
    T, N, C, H = shape
    dev = torch.device("cuda:0")
    bound = ops.workspace_bytes(T, N, C, H)
    for dtype in (torch.float32, torch.float64):
        if dtype == torch.float64 and T * N * H > 1 << 19:
            continue
        s = torch.cuda.Stream()
        with torch.cuda.stream(s):
            for name in ["LSTM", "GRU", "LayerNormLSTM", "LayerNormGRU", "IndRNN", "LayerNormIndRNN"]:
                torch.manual_seed(0)
                kw = {"zoneout": 0.1}
                if name in ("LSTM", "GRU"):
                    kw["dropout"] = 0.05
                layer = getattr(layers, name)(C, H, **kw).to(dev).to(dtype)
                x = torch.randn(T, N, C, device=dev, dtype=dtype, requires_grad=True)
                y, _ = layer(x)
                y.sum().backward()
                s.synchronize()
                used = ops.workspace_high_water()
                print(shape, dtype, name, "high water", used, "bound", bound, flush=True)
                assert used <= bound, (name, dtype, used, bound)


def test_stream_status_is_ok_on_a_healthy_stream():
    from haste_amd import ops
    dev = torch.device("cuda:0")
    a = _inputs(5, 8, 32, 64, dev)
    ops.lstm_forward(True, 0.0, a["x"], a["h0"], a["h0"], a["W"], a["R"], a["b"], a["mask"])
    torch.cuda.synchronize()
    ops.stream_status()


def child_timeout():
    """Runs in a process whose environment makes every group barrier wait for a workgroup that
    does not exist, with a small spin limit: the kernel gives up, reports it and still ends."""
    sys.path.insert(0, ROOT)
    from haste_amd import lib, ops
    dev = torch.device("cuda:0")
    a = _inputs(4, 4, 32, 64, dev)
    print("launch with an absent workgroup", flush=True)
    h, c, _ = ops.lstm_forward(True, 0.0, a["x"], a["h0"], a["h0"], a["W"], a["R"], a["b"], a["mask"])  # returns OK
    torch.cuda.synchronize()
    try:
        ops.stream_status()
    except lib.HasteHipError as e:
        assert e.code == 4, e.code
        assert "gave up waiting" in str(e), str(e)
    else:
        raise AssertionError("the time-out was not reported")
    ops.stream_status()  # reported once, then clear
    print("timeout reported", flush=True)


def test_a_wait_that_runs_out_is_reported_by_stream_status():
    env = dict(os.environ, HASTE_HIP_TEST_HOOKS="1", HASTE_HIP_SPIN_LIMIT="512", HASTE_HIP_TEST_ABSENT_WORKGROUP="1",
               PYTHONPATH=os.pathsep.join([ROOT, os.path.join(ROOT, "tests")]))
    res = subprocess.run([sys.executable, os.path.abspath(__file__), "timeout"], env=env,
                         capture_output=True, text=True, timeout=110)
    assert res.returncode == 0, res.stdout + res.stderr
    assert "timeout reported" in res.stdout


if __name__ == "__main__":
    if sys.argv[1:] == ["timeout"]:
        child_timeout()
