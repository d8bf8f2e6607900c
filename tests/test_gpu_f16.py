"""The half-precision GRU (haste_hip_gru_*_f16, what gru::ForwardPass<__half> /
BackwardPass<__half> bind to) against the fp64 oracle on half-representable inputs.

Tolerance 2e-2 (max-norm relative, per tensor): every stored tensor is rounded to half
(2^-11 relative) and the states / carried gradients are rounded once per step; products are
accumulated in fp32.  The reference's own half instantiation computes in half throughout."""
import numpy as np
import pytest

from oracle import haste_oracle as O
from util import host, problem, relerr

pytestmark = pytest.mark.gpu

TOL16 = 2e-2
# the last two: the persistent kernels' two-set and 16-row tiles; BASELINE configuration 2's shape
# (shortened) with an unaligned batch
SHAPES = [(3, 2, 3, 4), (4, 5, 7, 20), (6, 16, 32, 64), (8, 33, 48, 128), (3, 70, 24, 300),
          (1, 5, 12, 40), (20, 63, 512, 512),
          # sizes that are multiples of 8: the products run on the half matrix cores
          (20, 64, 512, 512), (50, 8, 64, 264), (40, 1, 16, 64),
          # long sequences: on the half matrix cores, and ragged (fp32 on widened tensors)
          (100, 16, 32, 128), (101, 7, 24, 100)]


def dev16(a):
    import torch
    if a is None:
        return torch.empty(0, 0, 0, dtype=torch.float16, device="cuda")
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float16)).cuda()


def half_problem(seed, T, N, C, H, zoneout):
    p = problem(seed, T, N, C, H, 3, zoneout)
    return {k: (v.astype(np.float16).astype(np.float64) if v is not None else None) for k, v in p.items()}


@pytest.mark.parametrize("zoneout", [0.0, 0.3])
@pytest.mark.parametrize("T,N,C,H", SHAPES)
def test_f16_gru_training_forward_backward(T, N, C, H, zoneout):
    from haste_amd import ops
    import torch
    print("gru f16", T, N, C, H, zoneout, flush=True)
    p = half_problem(900 + T + N + C + H, T, N, C, H, zoneout)
    mask = dev16(p["mask"])
    h, cache = ops.gru_forward(True, zoneout, dev16(p["x"]), dev16(p["h0"]), dev16(p["W"]), dev16(p["R"]),
                               dev16(p["b"]), dev16(p["b2"]), mask)
    torch.cuda.synchronize()
    assert h.dtype == torch.float16 and cache.dtype == torch.float16
    ho, vo = O.gru_forward(p["W"], p["R"], p["b"], p["b2"], p["x"], p["h0"], True, zoneout, p["mask"])
    assert relerr(host(h), ho) < TOL16
    assert relerr(host(cache), vo) < TOL16
    grads = ops.gru_backward(ops.transpose(dev16(p["x"])), ops.transpose(dev16(p["W"])),
                             ops.transpose(dev16(p["R"])), dev16(p["b"]), dev16(p["b2"]), mask, h, cache,
                             dev16(p["dh_new"]))
    torch.cuda.synchronize()
    # the oracle's backward from the GPU's own (half) activations: what the kernels were given
    ref = O.gru_backward(p["W"], p["R"], p["b"], p["b2"], p["x"], host(h), host(cache), p["dh_new"], p["mask"])
    for name, ours, theirs in zip(("dx", "dh0", "dW", "dR", "dbx", "dbr"), grads,
                                  (ref[0], ref[5], ref[1], ref[2], ref[3], ref[4])):
        assert ours.dtype == torch.float16
        assert relerr(host(ours), theirs) < TOL16, name


def test_f16_gru_inference_and_iterate():
    from haste_amd import ops
    import torch
    T, N, C, H = 6, 9, 16, 40
    p = half_problem(17, T, N, C, H, 0.25)
    W, R, bx, br, x = (dev16(p[k]) for k in ("W", "R", "b", "b2", "x"))
    h, _ = ops.gru_forward(False, 0.25, x, dev16(p["h0"]), W, R, bx, br, dev16(p["mask"]))
    ho, _ = O.gru_forward(p["W"], p["R"], p["b"], p["b2"], p["x"], p["h0"], False, 0.25, p["mask"])
    assert relerr(host(h), ho) < TOL16
    # One step at a time: the state passes through the caller's half tensor between the calls,
    # while a pass over all steps keeps it in fp32 and rounds what it hands back, so the two
    # agree to half's rounding, not bit for bit.
    hs = [dev16(p["h0"])]
    for t in range(T):
        h1, _ = ops.gru_forward_iterate(False, 0.25, x[t].contiguous(), hs[t], W, R, bx, br,
                                        dev16(p["mask"])[t].contiguous())
        hs.append(h1)
    torch.cuda.synchronize()
    assert relerr(host(torch.stack(hs)), ho) < TOL16
    assert relerr(host(torch.stack(hs)), host(h)) < 4e-3


@pytest.mark.parametrize("N,C,H", [(1, 512, 512), (3, 40, 100), (8, 24, 36), (5, 700, 16)])
def test_f16_gru_single_step_of_a_small_batch(N, C, H):
    """A step of at most 8 rows is one kernel on the half tensors: Iterate for training (gates
    stored, zoneout by mask) and inference (zoneout by expectation), the state updated in place,
    and a one-step Run under DropConnect, each against the oracle's step."""
    from haste_amd import ops
    import torch
    print("gru f16 single step", N, C, H, flush=True)
    T = 3
    p = half_problem(50 + N + C + H, T, N, C, H, 0.3)
    W, R, bx, br, x, mask = (dev16(p[k]) for k in ("W", "R", "b", "b2", "x", "mask"))
    for training in (True, False):
        ho, vo = O.gru_forward(p["W"], p["R"], p["b"], p["b2"], p["x"], p["h0"], training, 0.3, p["mask"])
        state = dev16(p["h0"])
        for t in range(T):
            h1, v1 = ops.gru_forward_iterate(training, 0.3, x[t].contiguous(), state, W, R, bx, br,
                                             mask[t].contiguous(), h_out=state)
            assert h1.data_ptr() == state.data_ptr()
            torch.cuda.synchronize()
            assert relerr(host(state), ho[t + 1]) < TOL16, (training, t)
            if training:
                assert relerr(host(v1), vo[t]) < TOL16, t
    r = np.random.default_rng(N)
    m = (r.uniform(size=(H, 3 * H)) > 0.25).astype(np.float64)
    h, cache = ops.gru_forward(True, 0.3, x[:1].contiguous(), dev16(p["h0"]), W, R, bx, br,
                               mask[:1].contiguous(), dropconnect_mask=dev16(m), dropconnect_scale=2.0)
    ho, vo = O.gru_forward(p["W"], p["R"] * m * 2.0, p["b"], p["b2"], p["x"][:1], p["h0"], True, 0.3,
                           p["mask"][:1])
    assert relerr(host(h), ho) < TOL16
    assert relerr(host(cache), vo) < TOL16


def test_f16_gru_dropconnect_and_accumulated_gradients():
    """DropConnect on the half GRU against the oracle on pre-masked recurrent weights (the mask's
    scale chosen so that the masked weights are exact in half), and the backward pass adding
    to what dW, dR, dbx, dbr already hold (the C-ABI's contract; ops.gru_backward starts them at
    zero, so the entry point is called directly)."""
    from haste_amd import ops, lib as hlib
    import torch
    T, N, C, H = 5, 9, 16, 48
    p = half_problem(31, T, N, C, H, 0.2)
    r = np.random.default_rng(5)
    m = (r.uniform(size=(H, 3 * H)) > 0.25).astype(np.float64)
    scale = 2.0
    mask = dev16(p["mask"])
    h, cache = ops.gru_forward(True, 0.2, dev16(p["x"]), dev16(p["h0"]), dev16(p["W"]), dev16(p["R"]),
                               dev16(p["b"]), dev16(p["b2"]), mask, dropconnect_mask=dev16(m),
                               dropconnect_scale=scale)
    ho, vo = O.gru_forward(p["W"], p["R"] * m * scale, p["b"], p["b2"], p["x"], p["h0"], True, 0.2, p["mask"])
    assert relerr(host(h), ho) < TOL16
    assert relerr(host(cache), vo) < TOL16

    Rm = (p["R"] * m * scale).astype(np.float16).astype(np.float64)
    ref = O.gru_backward(p["W"], Rm, p["b"], p["b2"], p["x"], host(h), host(cache), p["dh_new"], p["mask"])
    start = {k: r.standard_normal(s).astype(np.float16).astype(np.float64)
             for k, s in (("dW", (C, 3 * H)), ("dR", (H, 3 * H)), ("dbx", (3 * H,)), ("dbr", (3 * H,)))}
    start["dh"] = np.zeros((N, H))  # the gradient carried into the last step: none
    out = {k: dev16(a) for k, a in start.items()}
    dx = torch.empty(T, N, C, dtype=torch.float16, device="cuda")
    dp = torch.empty(T, N, 3 * H, dtype=torch.float16, device="cuda")
    dq = torch.empty(T, N, 3 * H, dtype=torch.float16, device="cuda")
    hlib.call("haste_hip_gru_backward_f16", T, N, C, H, ops.transpose(dev16(p["W"])), ops.transpose(dev16(Rm)),
              dev16(p["b"]), dev16(p["b2"]), ops.transpose(dev16(p["x"])), h, cache, dev16(p["dh_new"]), dx,
              out["dW"], out["dR"], out["dbx"], out["dbr"], out["dh"], dp, dq, mask)
    torch.cuda.synchronize()
    assert relerr(host(dx), ref[0]) < TOL16
    for name, theirs in (("dW", ref[1]), ("dR", ref[2]), ("dbx", ref[3]), ("dbr", ref[4]), ("dh", ref[5])):
        assert relerr(host(out[name]), theirs + start[name]) < TOL16, name


def test_f16_gru_with_a_lent_workspace():
    """The staging area of the half GRU lives in the stream's workspace: a lent buffer that is too
    small is refused with the size in the error text; one of haste_hip_gru_half_workspace_bytes
    gives the bits of the library-owned run."""
    from haste_amd import ops, lib as hlib
    import torch
    T, N, C, H = 7, 10, 24, 64
    p = half_problem(77, T, N, C, H, 0.2)
    args = [dev16(p[k]) for k in ("x", "h0", "W", "R", "b", "b2", "mask")]

    def run():
        h, cache = ops.gru_forward(True, 0.2, *args)
        grads = ops.gru_backward(ops.transpose(args[0]), ops.transpose(args[2]), ops.transpose(args[3]), args[4],
                                 args[5], args[6], h, cache, dev16(p["dh_new"]))
        torch.cuda.synchronize()
        return (h, cache) + tuple(grads)

    want = run()
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        small = torch.empty(ops.workspace_bytes(T, N, C, H) // 4 // 64, dtype=torch.float32, device="cuda")
        ops.set_workspace(small)
        try:
            with pytest.raises(hlib.HasteHipError) as e:
                ops.gru_forward(True, 0.2, *args)
            assert e.value.code == 2 and "too small" in str(e.value)
            lent = torch.empty(ops.workspace_bytes(T, N, C, H, half_gru=True) // 4 + 64, dtype=torch.float32,
                               device="cuda")
            ops.set_workspace(lent)
            got = run()
        finally:
            torch.cuda.synchronize()
            ops.set_workspace(None)
    for g, w in zip(got, want):
        assert torch.equal(g, w)


@pytest.mark.parametrize("a_float", [False, True])
@pytest.mark.parametrize("accumulate", [False, True])
@pytest.mark.parametrize("M,N,K", [(1, 1, 8), (37, 53, 24), (128, 128, 64), (130, 257, 200), (300, 100, 1000),
                                   (64, 1536, 512), (512, 200, 6400), (1000, 512, 1536)])
def test_f16_gemm_nt(M, N, K, accumulate, a_float):
    """The half GRU's product kernel, C (+)= A * Bt^T in fp32 from half operands (A also from
    fp32, rounded as it is read), against numpy on the same half values: whole and ragged tiles,
    tails of K, products cut along K."""
    from haste_amd import lib as hlib
    import torch
    r = np.random.default_rng(M + 3 * N + 7 * K)
    a = r.standard_normal((M, K))
    bt = r.standard_normal((N, K))
    c0 = r.standard_normal((M, N)).astype(np.float32)
    # an fp32 A reaches half through float, as in the kernel
    a16, bt16 = a.astype(np.float32).astype(np.float16), bt.astype(np.float16)
    A = torch.from_numpy(a.astype(np.float32)).cuda() if a_float else torch.from_numpy(a16).cuda()
    Bt = torch.from_numpy(bt16).cuda()
    C = torch.from_numpy(c0).cuda()
    hlib.call("haste_hip_gemm_half_nt", int(a_float), M, N, K, A, K, Bt, K, C, N, int(accumulate))
    torch.cuda.synchronize()
    ref = a16.astype(np.float64) @ bt16.astype(np.float64).T + (c0 if accumulate else 0.0)
    assert relerr(host(C), ref) < 1e-5  # fp32 accumulation over up to 6400 terms


def test_f16_gemm_nt_refuses_what_it_cannot_address():
    from haste_amd import lib as hlib
    import torch
    A = torch.zeros(4, 12, dtype=torch.float16, device="cuda")
    C = torch.zeros(4, 4, device="cuda")
    with pytest.raises(hlib.HasteHipError) as e:
        hlib.call("haste_hip_gemm_half_nt", 0, 4, 4, 12, A, 12, A, 12, C, 4, 0)  # K not a multiple of 8
    assert e.value.code == 2


def test_f16_lstm_is_refused():
    """As in the reference, half exists for the GRU only."""
    from haste_amd import ops
    p = {k: v for k, v in problem(1, 2, 2, 3, 4, 4).items()}
    with pytest.raises(ValueError):
        ops.lstm_forward(True, 0.0, dev16(p["x"]), dev16(p["h0"]), dev16(p["c0"]), dev16(p["W"]),
                         dev16(p["R"]), dev16(p["b"]), dev16(None))


@pytest.mark.parametrize("trans_a,M,N,K", [(False, 1, 1, 1), (False, 37, 53, 29), (False, 128, 192, 64),
                                           (True, 70, 130, 45), (True, 5, 20, 33), (False, 300, 100, 1000)])
@pytest.mark.parametrize("accumulate", [False, True])
def test_f16_gemm_and_transpose(trans_a, M, N, K, accumulate):
    from haste_amd import ops
    import torch
    r = np.random.default_rng(M * 7 + N * 3 + K)
    h16 = lambda a: a.astype(np.float16).astype(np.float64)
    a = h16(r.standard_normal((K, M) if trans_a else (M, K)))
    b = h16(r.standard_normal((K, N)))
    c0 = h16(r.standard_normal((M, N)))
    out = dev16(c0)
    ops.gemm(dev16(a), dev16(b), out=out, trans_a=trans_a, accumulate=accumulate)
    ref = (a.T if trans_a else a) @ b + (c0 if accumulate else 0.0)
    assert relerr(host(out), ref) < 2e-3  # one rounding to half of an fp32-accumulated product
    t = ops.transpose(dev16(a))
    assert torch.equal(t, dev16(a).t().contiguous())
