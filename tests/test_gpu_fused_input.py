"""LSTM and GRU forward recurrences: x*W computed inside the recurrence (4-row tiles) gives, to rounding,
what the recurrence gives on x*W from a GEMM launched before it.

The variant with the separate GEMM is selected by an environment variable that the library reads
once, so it runs in a child process.  The shapes have 8-row tiles run as two 4-row sets per
workgroup: a ragged last set, a set without rows, full sets."""
import os
import subprocess
import sys
import tempfile

import numpy as np
import pytest

from util import dev, host, problem, relerr

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# (T, N, C, H)
SHAPES = [(6, 41, 24, 512), (5, 64, 32, 256), (4, 36, 8, 72), (5, 40, 300, 320), (4, 13, 512, 400)]


def run_cells(T, N, C, H):
    """LSTM and GRU forward + backward with zoneout; every output as float64 arrays."""
    import torch
    from haste_amd import ops
    out = {}
    p = problem(900 + T + N + C + H, T, N, C, H, 4, 0.2)
    mask = dev(p["mask"])
    h, c, cache = ops.lstm_forward(True, 0.2, dev(p["x"]), dev(p["h0"]), dev(p["c0"]),
                                   dev(p["W"]), dev(p["R"]), dev(p["b"]), mask)
    x_t = dev(p["x"]).permute(2, 0, 1).contiguous()
    grads = ops.lstm_backward(x_t, dev(p["W"]).t().contiguous(), dev(p["R"]).t().contiguous(),
                              dev(p["b"]), mask, h, c, cache, dev(p["dh_new"]), dev(p["dc_new"]))
    for name, t in zip(("h", "c", "dx", "dh", "dc", "dW", "dR", "db", "dv"), (h, c) + tuple(grads) + (cache,)):
        out["lstm_" + name] = host(t)

    p = problem(901 + T + N + C + H, T, N, C, H, 3, 0.2)
    mask = dev(p["mask"])
    W, R, bx, br = dev(p["W"]), dev(p["R"]), dev(p["b"]), dev(p["b2"])
    h, cache = ops.gru_forward(True, 0.2, dev(p["x"]), dev(p["h0"]), W, R, bx, br, mask)
    x_t = dev(p["x"]).permute(2, 0, 1).contiguous()
    grads = ops.gru_backward(x_t, W.t().contiguous(), R.t().contiguous(), bx, br, mask, h, cache,
                             dev(p["dh_new"]))
    for i, t in enumerate((h,) + tuple(grads)):
        out["gru_%d" % i] = host(t)
    torch.cuda.synchronize()
    return out


def child(path):
    arrays = {}
    for shape in SHAPES:
        for k, v in run_cells(*shape).items():
            arrays["%d_%d_%d_%d_%s" % (shape + (k,))] = v
    np.savez(path, **arrays)


def _child_outputs(d, name, **env_vars):
    path = os.path.join(d, name + ".npz")
    env = dict(os.environ, PYTHONPATH=os.pathsep.join([ROOT, os.path.join(ROOT, "tests")]), **env_vars)
    res = subprocess.run([sys.executable, os.path.abspath(__file__), path], env=env,
                         capture_output=True, text=True, timeout=110)
    assert res.returncode == 0, res.stdout + res.stderr
    return np.load(path)


def test_input_projection_inside_the_recurrence_matches_the_separate_gemm():
    """x*W computed by the forward recurrence beside its waits (this process) against x*W from
    the GEMM launched before it (child process): the same sums in another order, so equal to
    rounding, forward and -- through the saved activations -- backward."""
    with tempfile.TemporaryDirectory() as d:
        separate = _child_outputs(d, "separate", HASTE_HIP_FUSED_INPUT="0")
        for shape in SHAPES:
            print("fused input projection vs separate GEMM", shape, flush=True)
            for k, v in run_cells(*shape).items():
                ref = separate["%d_%d_%d_%d_%s" % (shape + (k,))]
                assert relerr(v, ref) < 5e-6, (shape, k)


if __name__ == "__main__":
    child(sys.argv[1])
