"""LSTM forward/backward on the GPU (through the C-ABI) vs the fp64 oracle."""
import numpy as np
import pytest

from oracle import haste_oracle as O
from util import TOL, dev, host, problem, relerr

pytestmark = pytest.mark.gpu

# (T, N, C, H): tiny, ragged (sizes that are not multiples of any tile), and config-like
SHAPES = [(1, 1, 1, 1), (3, 2, 3, 4), (5, 3, 7, 5), (6, 17, 20, 36), (4, 16, 32, 64),
          (10, 33, 48, 128), (8, 64, 64, 256), (12, 16, 128, 256), (6, 128, 96, 512),
          (3, 200, 16, 64), (2, 300, 8, 48), (2, 520, 8, 32),
          # 8-row tiles run as two 4-row sets per workgroup: ragged last set, a set without rows,
          # hidden sizes that are not multiples of the 16 units of a workgroup
          (7, 41, 24, 512), (5, 57, 16, 200), (4, 36, 8, 72),
          (1, 40, 8, 128), (2, 64, 8, 64), (3, 50, 8, 16),
          # one batch row: the forward pass keeps the recurrent weights in registers (H <= 512)
          (9, 1, 7, 100), (6, 1, 16, 512), (5, 1, 8, 300), (4, 1, 8, 48), (7, 1, 5, 17),
          # hidden sizes beyond what stays on chip: the backward pass, then both passes, stream R
          (3, 5, 40, 640), (3, 4, 32, 1536), (2, 70, 24, 1300), (2, 128, 16, 1024),
          # 608 < H <= 1120: the backward recurrence keeps part of its slice of R in registers
          # (8, 16, 24 or 32 k-groups per wavefront; tiles of 16, 32 and 64 rows; hidden sizes
          # that leave single k-groups and a ragged last workgroup)
          (4, 64, 32, 1024), (3, 17, 24, 768), (3, 100, 16, 896), (2, 200, 16, 1000),
          (3, 9, 8, 700), (2, 256, 8, 1024), (3, 30, 8, 1120), (5, 16, 8, 1023),
          # 1024 < H <= 2048 with up to 64 rows: the forward recurrence keeps part of its slice
          # of R in registers as well (8 hidden units per workgroup, tiles of 16, 32 and 64 rows)
          (3, 20, 16, 2048), (2, 64, 8, 2048), (3, 9, 24, 1536), (2, 50, 8, 1800), (3, 16, 8, 1290)]


def run_lstm(p, training, zoneout_prob, T, N, C, H):
    from haste_amd import ops
    import torch
    mask = dev(p["mask"])
    h, c, cache = ops.lstm_forward(training, zoneout_prob, dev(p["x"]), dev(p["h0"]), dev(p["c0"]),
                                   dev(p["W"]), dev(p["R"]), dev(p["b"]), mask)
    torch.cuda.synchronize()
    return h, c, cache, mask


@pytest.mark.parametrize("zoneout", [0.0, 0.3])
@pytest.mark.parametrize("T,N,C,H", SHAPES)
def test_lstm_training_forward_backward(T, N, C, H, zoneout):
    from haste_amd import ops
    import torch
    print("lstm fwd+bwd", T, N, C, H, zoneout, flush=True)
    p = problem(100 + T + N + C + H, T, N, C, H, 4, zoneout)
    h, c, cache, mask = run_lstm(p, True, zoneout, T, N, C, H)
    ho, co, vo = O.lstm_forward(p["W"], p["R"], p["b"], p["x"], p["h0"], p["c0"], True, zoneout, p["mask"])
    assert relerr(host(h), ho) < TOL
    assert relerr(host(c), co) < TOL
    assert relerr(host(cache), vo) < TOL

    x_t = dev(p["x"]).permute(2, 0, 1).contiguous()
    W_t = dev(p["W"]).t().contiguous()
    R_t = dev(p["R"]).t().contiguous()
    dx, dh, dc, dW, dR, db = ops.lstm_backward(x_t, W_t, R_t, dev(p["b"]), mask, h, c, cache,
                                               dev(p["dh_new"]), dev(p["dc_new"]))
    torch.cuda.synchronize()
    ref = O.lstm_backward(p["W"], p["R"], p["b"], p["x"], ho, co, vo, p["dh_new"], p["dc_new"], p["mask"])
    for name, ours, theirs in zip(("dx", "dW", "dR", "db", "dh0", "dc0", "dv"),
                                  (dx, dW, dR, db, dh, dc, cache), ref):
        assert relerr(host(ours), theirs) < TOL, name


@pytest.mark.parametrize("zoneout", [0.0, 0.25])
@pytest.mark.parametrize("T,N,C,H", [(20, 16, 128, 256), (12, 1, 32, 512), (9, 1, 8, 130), (8, 50, 16, 512)])
def test_lstm_inference_forward(zoneout, T, N, C, H):
    """Inference (zoneout as the convex blend) through the tile, single-row and two-set kernels."""
    p = problem(7, T, N, C, H, 4, zoneout)
    h, c, _, _ = run_lstm(p, False, zoneout, T, N, C, H)
    ho, co, _ = O.lstm_forward(p["W"], p["R"], p["b"], p["x"], p["h0"], p["c0"], False, zoneout, p["mask"])
    assert relerr(host(h), ho) < TOL
    assert relerr(host(c), co) < TOL


@pytest.mark.parametrize("T,N,C,H", [(6, 8, 16, 64), (5, 48, 16, 128), (6, 1, 16, 200), (3, 20, 16, 1536)])
def test_lstm_dropconnect_fused_equals_premasked_weights(T, N, C, H):
    """Bit for bit, in the 4-row tile kernel, the two-set kernel and the single-row kernel."""
    from haste_amd import ops
    import torch
    p = problem(9, T, N, C, H, 4)
    r = np.random.default_rng(3)
    m = (r.uniform(size=p["R"].shape) >= 0.05).astype(np.float64)
    scale = 1.0 / 0.95
    args = (True, 0.0, dev(p["x"]), dev(p["h0"]), dev(p["c0"]), dev(p["W"]))
    h1, c1, v1 = ops.lstm_forward(*args, dev(p["R"]), dev(p["b"]), dev(None),
                                  dropconnect_mask=dev(m), dropconnect_scale=scale)
    R_eff = (dev(p["R"]) * dev(m)) * np.float32(scale)
    h2, c2, v2 = ops.lstm_forward(*args, R_eff.contiguous(), dev(p["b"]), dev(None))
    torch.cuda.synchronize()
    assert torch.equal(h1, h2) and torch.equal(c1, c2) and torch.equal(v1, v2)


def test_lstm_accumulates_into_weight_gradients_and_is_deterministic():
    from haste_amd import ops
    import torch
    T, N, C, H = 7, 32, 24, 64
    p = problem(11, T, N, C, H, 4, 0.2)
    outs = []
    for _ in range(2):
        h, c, cache, mask = run_lstm(p, True, 0.2, T, N, C, H)
        x_t = dev(p["x"]).permute(2, 0, 1).contiguous()
        outs.append(ops.lstm_backward(x_t, dev(p["W"]).t().contiguous(), dev(p["R"]).t().contiguous(),
                                      dev(p["b"]), mask, h, c, cache, dev(p["dh_new"]), dev(p["dc_new"])))
    torch.cuda.synchronize()
    for a, b in zip(*outs):
        assert torch.equal(a, b)


def test_lstm_streamed_dropconnect_and_inference():
    """DropConnect and the inference-mode zoneout blend on the path that streams R (H = 1536)."""
    from haste_amd import ops
    import torch
    T, N, C, H = 3, 6, 16, 1536
    p = problem(12, T, N, C, H, 4, 0.25)
    m = (np.random.default_rng(4).uniform(size=p["R"].shape) >= 0.1).astype(np.float64)
    scale = np.float64(np.float32(1.0 / 0.9))
    h, c, v = ops.lstm_forward(False, 0.25, dev(p["x"]), dev(p["h0"]), dev(p["c0"]), dev(p["W"]),
                               dev(p["R"]), dev(p["b"]), dev(p["mask"]), dropconnect_mask=dev(m),
                               dropconnect_scale=float(scale))
    torch.cuda.synchronize()
    ho, co, _ = O.lstm_forward(p["W"], p["R"] * m * scale, p["b"], p["x"], p["h0"], p["c0"], False, 0.25,
                               p["mask"])
    assert relerr(host(h), ho) < TOL
    assert relerr(host(c), co) < TOL


# The forward recurrence computes x*W itself for 4-row tiles (N <= 32: one set; 33..64: two sets)
# when C <= 512 is a multiple of 4 and H > 192: input sizes below, at and between the 64-feature
# groups a wavefront takes, one and two groups per wavefront, batches that leave rows of the last
# tile empty, a single step with more than 8 rows.
FUSED_INPUT_SHAPES = [(3, 4, 4, 196), (5, 7, 36, 200), (2, 31, 64, 256), (4, 32, 100, 300), (3, 33, 128, 260),
                      (6, 64, 256, 512), (2, 50, 260, 512), (3, 9, 512, 208), (1, 40, 384, 512), (4, 61, 508, 448)]


@pytest.mark.parametrize("zoneout", [0.0, 0.3])
@pytest.mark.parametrize("T,N,C,H", FUSED_INPUT_SHAPES)
def test_lstm_input_projection_inside_the_recurrence(T, N, C, H, zoneout):
    test_lstm_training_forward_backward(T, N, C, H, zoneout)


@pytest.mark.parametrize("T,N,C,H", [(4, 24, 96, 256), (3, 64, 512, 512)])
def test_lstm_dropconnect_with_input_projection_inside(T, N, C, H):
    test_lstm_dropconnect_fused_equals_premasked_weights(T, N, C, H)
    test_lstm_inference_forward(0.25, T, N, C, H)


def _launch_counts(lib, names):
    import ctypes
    out = {}
    for name in names:
        total, count = ctypes.c_double(0.0), ctypes.c_int(0)
        assert lib.haste_hip_profile_read(name.encode(), ctypes.byref(total), ctypes.byref(count)) == 0
        out[name] = count.value
    return out


@pytest.mark.parametrize("cell", ["lstm", "gru"])
@pytest.mark.parametrize("N,H", [(5, 640), (64, 768), (64, 1024), (128, 1024)])
def test_backward_of_mid_sized_hidden_states_is_one_persistent_launch(cell, N, H):
    """608 < H <= 1024 (GRU: above 816): the backward pass is one launch of the persistent
    recurrence, not one product and one pointwise launch per step."""
    from haste_amd import lib as hlib, ops
    import torch
    T, C = 3, 16
    gates = 4 if cell == "lstm" else 3
    p = problem(7, T, N, C, H, 4, 0.0)
    lib = hlib.load()
    none = torch.empty(0, 0, 0, device="cuda:0")
    x, h0 = dev(p["x"]), dev(p["h0"])
    W, R, b = dev(p["W"][:, :gates * H]), dev(p["R"][:, :gates * H]), dev(p["b"][:gates * H])
    x_t, W_t, R_t = ops.transpose(x), ops.transpose(W), ops.transpose(R)
    lib.haste_hip_profile_reset()
    lib.haste_hip_profile_enable(1)
    try:
        if cell == "lstm":
            h, c, cache = ops.lstm_forward(True, 0.0, x, h0, dev(p["c0"]), W, R, b, none)
            ops.lstm_backward(x_t, W_t, R_t, b, none, h, c, cache, dev(p["dh_new"]), dev(p["dc_new"]))
        else:
            b2 = dev(p["b2"][:3 * H])
            h, cache = ops.gru_forward(True, 0.0, x, h0, W, R, b, b2, none)
            ops.gru_backward(x_t, W_t, R_t, b, b2, none, h, cache, dev(p["dh_new"]))
        torch.cuda.synchronize()
    finally:
        lib.haste_hip_profile_enable(0)
    n = _launch_counts(lib, [cell + "_backward_recurrence", cell + "_backward_steps"])
    lib.haste_hip_profile_reset()
    assert n[cell + "_backward_recurrence"] == 1 and n[cell + "_backward_steps"] == 0, n


@pytest.mark.parametrize("cell", ["lstm", "gru"])
@pytest.mark.parametrize("N,H", [(1, 1536), (32, 2048), (64, 2048)])
def test_forward_of_large_hidden_states_is_one_persistent_launch(cell, N, H):
    """1024 < H <= 2048 with up to 64 rows: the forward pass is one launch of the persistent
    recurrence (part of the slice of R in registers), not one product per step."""
    from haste_amd import lib as hlib, ops
    import torch
    T, C = 3, 16
    gates = 4 if cell == "lstm" else 3
    p = problem(9, T, N, C, H, 4, 0.0)
    lib = hlib.load()
    none = torch.empty(0, 0, 0, device="cuda:0")
    x, h0 = dev(p["x"]), dev(p["h0"])
    W, R, b = dev(p["W"][:, :gates * H]), dev(p["R"][:, :gates * H]), dev(p["b"][:gates * H])
    lib.haste_hip_profile_reset()
    lib.haste_hip_profile_enable(1)
    try:
        if cell == "lstm":
            ops.lstm_forward(False, 0.0, x, h0, dev(p["c0"]), W, R, b, none)
        else:
            ops.gru_forward(False, 0.0, x, h0, W, R, b, dev(p["b2"][:3 * H]), none)
        torch.cuda.synchronize()
    finally:
        lib.haste_hip_profile_enable(0)
    n = _launch_counts(lib, [cell + "_forward_recurrence", cell + "_forward_steps"])
    lib.haste_hip_profile_reset()
    assert n[cell + "_forward_recurrence"] == 1 and n[cell + "_forward_steps"] == 0, n
