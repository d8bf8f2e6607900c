"""GRU forward/backward on the GPU (through the C-ABI) vs the fp64 oracle."""
import numpy as np
import pytest

from oracle import haste_oracle as O
from util import TOL, dev, host, problem, relerr

pytestmark = pytest.mark.gpu

SHAPES = [(1, 1, 1, 1), (3, 2, 3, 4), (5, 3, 7, 5), (6, 17, 20, 36), (4, 16, 32, 64),
          (10, 33, 48, 128), (8, 64, 64, 256), (6, 128, 96, 512),
          (3, 200, 16, 64), (2, 300, 8, 48), (2, 520, 8, 32),
          # 8-row tiles run as two 4-row sets per workgroup: ragged last set, a set without rows,
          # hidden sizes that are not multiples of the 16 units of a workgroup
          (7, 41, 24, 512), (5, 57, 16, 200), (4, 36, 8, 72),
          (1, 40, 8, 128), (2, 64, 8, 64), (3, 50, 8, 16),
          # one batch row: the forward pass keeps the recurrent weights in registers (H <= 512)
          (9, 1, 7, 100), (6, 1, 16, 512), (5, 1, 8, 300), (4, 1, 8, 48), (7, 1, 5, 17),
          # hidden sizes beyond what stays on chip: the backward pass, then both passes, stream R
          (3, 5, 40, 704), (3, 4, 32, 1536), (2, 70, 24, 1700), (2, 128, 16, 1024),
          # 816 < H <= 1488: the backward recurrence keeps part of its slice of R in registers
          # (8, 16, 24 or 32 k-groups per wavefront; tiles of 16, 32 and 64 rows; hidden sizes
          # that leave single k-groups and a ragged last workgroup)
          (4, 64, 32, 1024), (3, 17, 24, 900), (3, 100, 16, 1200), (2, 60, 16, 1400),
          (5, 16, 8, 1023), (2, 256, 8, 1024), (3, 9, 8, 1488),
          # 1024 < H <= 2048 with up to 64 rows: the forward recurrence keeps part of its slice
          # of R in registers as well (8 hidden units per workgroup, tiles of 16, 32 and 64 rows)
          (3, 20, 16, 2048), (2, 64, 8, 2048), (3, 9, 24, 1536), (2, 50, 8, 1800), (3, 16, 8, 1290), (2, 256, 8, 1024)]


@pytest.mark.parametrize("zoneout", [0.0, 0.3])
@pytest.mark.parametrize("T,N,C,H", SHAPES)
def test_gru_training_forward_backward(T, N, C, H, zoneout):
    from haste_amd import ops
    import torch
    print("gru fwd+bwd", T, N, C, H, zoneout, flush=True)
    p = problem(200 + T + N + C + H, T, N, C, H, 3, zoneout)
    mask = dev(p["mask"])
    h, cache = ops.gru_forward(True, zoneout, dev(p["x"]), dev(p["h0"]), dev(p["W"]), dev(p["R"]),
                               dev(p["b"]), dev(p["b2"]), mask)
    torch.cuda.synchronize()
    ho, vo = O.gru_forward(p["W"], p["R"], p["b"], p["b2"], p["x"], p["h0"], True, zoneout, p["mask"])
    assert relerr(host(h), ho) < TOL
    assert relerr(host(cache), vo) < TOL
    x_t = dev(p["x"]).permute(2, 0, 1).contiguous()
    outs = ops.gru_backward(x_t, dev(p["W"]).t().contiguous(), dev(p["R"]).t().contiguous(),
                            dev(p["b"]), dev(p["b2"]), mask, h, cache, dev(p["dh_new"]))
    torch.cuda.synchronize()
    dx, dW, dR, dbx, dbr, dh0, _, _ = O.gru_backward(p["W"], p["R"], p["b"], p["b2"], p["x"], ho, vo,
                                                     p["dh_new"], p["mask"])
    for name, ours, theirs in zip(("dx", "dh0", "dW", "dR", "dbx", "dbr"), outs,
                                  (dx, dh0, dW, dR, dbx, dbr)):
        assert relerr(host(ours), theirs) < TOL, name


@pytest.mark.parametrize("zoneout", [0.0, 0.25])
@pytest.mark.parametrize("T,N,C,H", [(20, 16, 128, 256), (8, 50, 16, 512), (12, 1, 32, 512), (9, 1, 8, 130)])
def test_gru_inference_forward(zoneout, T, N, C, H):
    """Inference (zoneout as the convex blend) through the tile, two-set and single-row kernels."""
    from haste_amd import ops
    import torch
    p = problem(8, T, N, C, H, 3, zoneout)
    h, _ = ops.gru_forward(False, zoneout, dev(p["x"]), dev(p["h0"]), dev(p["W"]), dev(p["R"]),
                           dev(p["b"]), dev(p["b2"]), dev(p["mask"]))
    torch.cuda.synchronize()
    ho, _ = O.gru_forward(p["W"], p["R"], p["b"], p["b2"], p["x"], p["h0"], False, zoneout, p["mask"])
    assert relerr(host(h), ho) < TOL


@pytest.mark.parametrize("T,N,C,H", [(6, 8, 16, 64), (5, 48, 16, 128), (6, 1, 16, 200)])
def test_gru_dropconnect_fused_equals_premasked_weights(T, N, C, H):
    """Bit for bit, in the 4-row tile kernel, the two-set kernel and the single-row kernel."""
    from haste_amd import ops
    import torch
    p = problem(9, T, N, C, H, 3)
    m = (np.random.default_rng(3).uniform(size=p["R"].shape) >= 0.05).astype(np.float64)
    scale = 1.0 / 0.95
    args = (True, 0.0, dev(p["x"]), dev(p["h0"]), dev(p["W"]))
    h1, v1 = ops.gru_forward(*args, dev(p["R"]), dev(p["b"]), dev(p["b2"]), dev(None),
                             dropconnect_mask=dev(m), dropconnect_scale=scale)
    R_eff = ((dev(p["R"]) * dev(m)) * np.float32(scale)).contiguous()
    h2, v2 = ops.gru_forward(*args, R_eff, dev(p["b"]), dev(p["b2"]), dev(None))
    torch.cuda.synchronize()
    assert torch.equal(h1, h2) and torch.equal(v1, v2)
