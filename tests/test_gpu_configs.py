"""Parity at the benchmark configurations (full sizes) against the fp64 oracle, plus
size-independent properties: run-to-run bit stability, batch-permutation equivariance,
linearity of the backward pass in the upstream gradients."""
import numpy as np
import pytest

from oracle import haste_oracle as O
from util import TOL, dev, host, problem, relerr

pytestmark = pytest.mark.gpu


def _lstm_grads(ops, p, h, c, cache, mask):
    x_t = dev(p["x"]).permute(2, 0, 1).contiguous()
    return ops.lstm_backward(x_t, dev(p["W"]).t().contiguous(), dev(p["R"]).t().contiguous(),
                             dev(p["b"]), mask, h, c, cache, dev(p["dh_new"]), dev(p["dc_new"]))


def test_config1_lstm_inference_matches_torch_nn_lstm():
    """LSTM forward inference N=16 T=100 C=128 H=256, b=0, h0=c0=0, vs torch.nn.LSTM on CPU."""
    import torch
    from haste_amd import ops
    from oracle import cpu_baseline
    T, N, C, H = 100, 16, 128, 256
    p = problem(1, T, N, C, H, 4)
    p["b"][:] = 0
    p["h0"][:] = 0
    p["c0"][:] = 0
    h, c, _ = ops.lstm_forward(False, 0.0, dev(p["x"]), dev(p["h0"]), dev(p["c0"]), dev(p["W"]),
                               dev(p["R"]), dev(p["b"]), dev(None))
    torch.cuda.synchronize()
    m = cpu_baseline.native_lstm(p["W"], p["R"], p["b"]).double()
    with torch.no_grad():
        y, (hT, cT) = m(torch.from_numpy(p["x"]))
    assert relerr(host(h)[1:], y.numpy()) < TOL
    assert relerr(host(c)[T], cT[0].numpy()) < TOL
    ho, co, _ = O.lstm_forward(p["W"], p["R"], p["b"], p["x"], p["h0"], p["c0"], False)
    assert relerr(host(h), ho) < TOL and relerr(host(c), co) < TOL


def test_config2_gru_training_zoneout_dropconnect():
    """GRU fwd+bwd N=64 T=100 C=H=512, zoneout 0.1, DropConnect 0.05 fused into the R load."""
    import torch
    from haste_amd import ops
    T, N, C, H = 100, 64, 512, 512
    p = problem(2, T, N, C, H, 3, 0.1)
    r = np.random.default_rng(22)
    dmask = (r.uniform(size=p["R"].shape) >= 0.05).astype(np.float64)
    scale = np.float64(np.float32(1.0 / 0.95))
    mask = dev(p["mask"])
    h, cache = ops.gru_forward(True, 0.1, dev(p["x"]), dev(p["h0"]), dev(p["W"]), dev(p["R"]),
                               dev(p["b"]), dev(p["b2"]), mask, dropconnect_mask=dev(dmask),
                               dropconnect_scale=float(scale))
    # R_eff in fp32 exactly as the kernel forms it
    R_eff32 = ((dev(p["R"]) * dev(dmask)) * np.float32(scale)).contiguous()
    outs = ops.gru_backward(dev(p["x"]).permute(2, 0, 1).contiguous(), dev(p["W"]).t().contiguous(),
                            R_eff32.t().contiguous(), dev(p["b"]), dev(p["b2"]), mask, h, cache,
                            dev(p["dh_new"]))
    torch.cuda.synchronize()
    R_eff = host(R_eff32)
    ho, vo = O.gru_forward(p["W"], R_eff, p["b"], p["b2"], p["x"], p["h0"], True, 0.1, p["mask"])
    dx, dW, dR, dbx, dbr, dh0, _, _ = O.gru_backward(p["W"], R_eff, p["b"], p["b2"], p["x"], ho, vo,
                                                     p["dh_new"], p["mask"])
    assert relerr(host(h), ho) < TOL
    assert relerr(host(cache), vo) < TOL
    for name, ours, theirs in zip(("dx", "dh0", "dW", "dR", "dbx", "dbr"), outs,
                                  (dx, dh0, dW, dR, dbx, dbr)):
        assert relerr(host(ours), theirs) < TOL, name


@pytest.mark.parametrize("N", [128, 64])
def test_config3_and_metric_lstm_training(N):
    """LSTM fwd+bwd N=128 (config 3) and N=64 (metric), T=100 C=H=512, forget bias 1,
    upstream gradients on every output step plus the final h and c."""
    import torch
    from haste_amd import ops
    T, C, H = 100, 512, 512
    p = problem(3, T, N, C, H, 4, forget_bias=1.0)
    p["dc_new"][:T] = 0.0  # only the final cell state receives an upstream gradient
    h, c, cache = ops.lstm_forward(True, 0.0, dev(p["x"]), dev(p["h0"]), dev(p["c0"]), dev(p["W"]),
                                   dev(p["R"]), dev(p["b"]), dev(None))
    torch.cuda.synchronize()
    ho, co, vo = O.lstm_forward(p["W"], p["R"], p["b"], p["x"], p["h0"], p["c0"])
    assert relerr(host(h), ho) < TOL and relerr(host(c), co) < TOL and relerr(host(cache), vo) < TOL
    grads = _lstm_grads(ops, p, h, c, cache, dev(None))
    torch.cuda.synchronize()
    ref = O.lstm_backward(p["W"], p["R"], p["b"], p["x"], ho, co, vo, p["dh_new"], p["dc_new"])
    for name, ours, theirs in zip(("dx", "dh0", "dc0", "dW", "dR", "db"), grads,
                                  (ref[0], ref[4], ref[5], ref[1], ref[2], ref[3])):
        assert relerr(host(ours), theirs) < TOL, name


def test_config4_layer_norm_lstm_training():
    """LayerNormLSTM fwd+bwd N=32 T=500 C=H=256, gamma=1 beta=0, forget bias 1, zoneout 0.1.

    With these weights the normalised recurrence is chaotic: the same oracle run in float32
    drifts from its float64 self by 4e-6 at t=20, 2e-4 at t=100, 8e-3 at t=200 and O(1) at
    t=500, so no float32 implementation can track the float64 trajectory to 1e-4 over 500
    free-running steps.  The check is therefore (1) the free-running trajectory over the
    first 20 steps, (2) every one of the 500 steps taken one at a time from the GPU's own
    state (the step map itself), and (3) the backward pass against the oracle's backward
    pass on the activations the GPU forward pass saved."""
    import torch
    from haste_amd import ops
    T, N, C, H = 500, 32, 256, 256
    p = problem(4, T, N, C, H, 4, 0.1, forget_bias=1.0)
    p["gamma"][:] = 1.0
    p["gamma_h"][:] = 1.0
    p["beta_h"][:] = 0.0
    mask = dev(p["mask"])
    gam, gh, bh = dev(p["gamma"]), dev(p["gamma_h"]), dev(p["beta_h"])
    outs = ops.layer_norm_lstm_forward(True, 0.1, dev(p["x"]), dev(p["h0"]), dev(p["c0"]),
                                       dev(p["W"]), dev(p["R"]), dev(p["b"]), gam, gh, bh, mask)
    torch.cuda.synchronize()
    h, c, act_Wx, act_Wx_norm, cache1, act_Rh, cache2, act_c_norm, cache3 = outs
    hg, cg = host(h), host(c)
    args = (p["W"], p["R"], p["b"], p["gamma"], p["gamma_h"], p["beta_h"])
    # (1) free-running, first 20 steps
    f20 = O.layer_norm_lstm_forward(*args, p["x"][:20], p["h0"], p["c0"], True, 0.1, p["mask"][:20])
    assert relerr(hg[:21], f20["h"]) < TOL and relerr(cg[:21], f20["c"]) < TOL
    # (2) each step from the GPU's own state
    # ... the new state and everything the step saves for the backward pass
    sv = dict(v=host(act_Wx_norm), act_Rh=host(act_Rh), act_c_norm=host(act_c_norm),
              cache2=host(cache2).reshape(T, N, 2), cache3=host(cache3).reshape(T, N, 2))
    worst = {}
    for t in range(T):
        one = O.layer_norm_lstm_forward(*args, p["x"][t:t + 1], hg[t], cg[t], True, 0.1,
                                        p["mask"][t:t + 1])
        errs = dict(h=relerr(hg[t + 1], one["h"][1]), c=relerr(cg[t + 1], one["c"][1]))
        errs.update({k: relerr(a[t], one[k][0]) for k, a in sv.items()})
        worst = {k: max(worst.get(k, 0.0), e) for k, e in errs.items()}
    assert max(worst.values()) < TOL, worst
    # (3) backward on the saved activations
    saved = dict(h=hg, c=cg, v=host(act_Wx_norm), act_Wx=host(act_Wx), act_Rh=host(act_Rh),
                 act_c_norm=host(act_c_norm), cache1=host(cache1).reshape(T, N, 2),
                 cache2=host(cache2).reshape(T, N, 2), cache3=host(cache3).reshape(T, N, 2))
    grads = ops.layer_norm_lstm_backward(
        dev(p["x"]).permute(2, 0, 1).contiguous(), dev(p["W"]).t().contiguous(),
        dev(p["R"]).t().contiguous(), dev(p["b"]), gam, gh, bh, mask, h, c, act_Wx, act_Wx_norm,
        cache1, act_Rh, cache2, act_c_norm, cache3, dev(p["dh_new"]), dev(p["dc_new"]))
    torch.cuda.synchronize()
    g = O.layer_norm_lstm_backward(*args, p["x"], saved, p["dh_new"], p["dc_new"], p["mask"])
    for name, ours in zip(("dx", "dh0", "dc0", "dW", "dR", "db", "dgamma", "dgamma_h", "dbeta_h"), grads):
        assert relerr(host(ours), g[name]) < TOL, name


def test_config5_lstm_streaming_inference():
    """LSTM inference N=1 T=2000 C=H=512."""
    import torch
    from haste_amd import ops
    T, N, C, H = 2000, 1, 512, 512
    p = problem(5, T, N, C, H, 4)
    p["b"][:] = 0
    p["h0"][:] = 0
    p["c0"][:] = 0
    h, c, _ = ops.lstm_forward(False, 0.0, dev(p["x"]), dev(p["h0"]), dev(p["c0"]), dev(p["W"]),
                               dev(p["R"]), dev(p["b"]), dev(None))
    torch.cuda.synchronize()
    ho, co, _ = O.lstm_forward(p["W"], p["R"], p["b"], p["x"], p["h0"], p["c0"], False)
    assert relerr(host(h), ho) < TOL and relerr(host(c), co) < TOL


def test_full_size_properties():
    """At the metric size: bit-stable across runs, equivariant under batch permutation,
    backward linear in the upstream gradients, weight gradients accumulate."""
    import torch
    from haste_amd import ops
    T, N, C, H = 100, 64, 512, 512
    p = problem(6, T, N, C, H, 4, 0.1)
    mask = dev(p["mask"])

    def fwd(perm=None):
        sel = (lambda a: a) if perm is None else (lambda a: np.ascontiguousarray(a[:, perm]))
        sel0 = (lambda a: a) if perm is None else (lambda a: np.ascontiguousarray(a[perm]))
        return ops.lstm_forward(True, 0.1, dev(sel(p["x"])), dev(sel0(p["h0"])), dev(sel0(p["c0"])),
                                dev(p["W"]), dev(p["R"]), dev(p["b"]), dev(sel(p["mask"])))
    h1, c1, v1 = fwd()
    h2, c2, v2 = fwd()
    torch.cuda.synchronize()
    assert torch.equal(h1, h2) and torch.equal(c1, c2) and torch.equal(v1, v2)
    perm = np.random.default_rng(0).permutation(N)
    hp, cp, _ = fwd(perm)
    torch.cuda.synchronize()
    assert torch.equal(hp, h1[:, torch.from_numpy(perm).cuda()])

    g1 = _lstm_grads(ops, p, h1, c1, v1.clone(), mask)
    g1b = _lstm_grads(ops, p, h1, c1, v1.clone(), mask)
    torch.cuda.synchronize()
    for a, b in zip(g1, g1b):
        assert torch.equal(a, b)
    q = dict(p)
    q["dh_new"] = 2.0 * p["dh_new"]
    q["dc_new"] = 2.0 * p["dc_new"]
    g2 = _lstm_grads(ops, q, h1, c1, v1.clone(), mask)
    torch.cuda.synchronize()
    for a, b in zip(g1, g2):
        assert torch.equal(2.0 * a, b)  # scaling by two is exact in binary floating point
