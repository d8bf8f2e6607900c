"""Benchmark of the hot path on one MI355X.

Metric (BASELINE.json): LSTM forward + backward, ms per batch, at N=64, T=100,
C=H=512, fp32; plus microseconds per timestep of streaming inference at N=1, T=2000.

One step = ForwardPass::Run (training) + the caller-side transposes of x, W, R +
BackwardPass::Run, as the reference's benchmark times it
(benchmarks/benchmark_lstm.cc:399-465).  Inputs are synthetic, seeded, and resident in
HBM before the timed region.  Prints one JSON line.
"""
import argparse
import ctypes
import json
import os
import sys

import numpy as np

PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_FP64_MFMA_TFLOPS = 78.6
PEAK_HBM_GBS = 8000.0

# HBM bytes per launch at the metric workload, from two rocprofv3 --pmc runs (FETCH_SIZE, then
# WRITE_SIZE) scaled by what the same counters read for a 1 GiB device copy (--workload copy):
# one FETCH_SIZE unit = 2.000 KiB, one WRITE_SIZE unit = 1.000 KiB.  A GEMM "launch" is the mean
# of the step's three products (dx; dW and dR, which share a launch that counts as two), each with
# its split reduce; the forward recurrence includes the input projection it computes itself.
TRAFFIC_SOURCE = "profiles/lstm_fwd_bwd_N64_T100_H512_hbm_traffic_pmc.txt (a constant from that profile, not measured in this run)"
MEASURED_TRAFFIC_BYTES = {"gemm_f32": 143.2e6, "lstm_forward_recurrence": 161.3e6,
                          "lstm_backward_recurrence": 196.1e6,
                          # at N=1 C=512 H=4096 (--workload stepwise): 131558.5 FETCH_SIZE units
                          # + 192 WRITE_SIZE units per launch of the streaming kernel
                          "gemm_f32_skinny": 269.6e6}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-budget", type=float, default=15.0)
    ap.add_argument("--workload", choices=["all", "metric", "streaming", "stepwise", "hbm_kernels", "copy", "configs",
                                           "peak", "iterate"],
                    default="all",
                    help="restrict the run to one workload (for profiling); the JSON line is "
                         "only complete with 'all'.  'copy' runs a plain device copy of known "
                         "size, the yardstick for the FETCH_SIZE / WRITE_SIZE counters")
    return ap.parse_args()


def make_inputs(T, N, C, H, seed=0, forget_bias=1.0):
    r = np.random.default_rng(seed)
    k = 1.0 / np.sqrt(H)
    W = r.uniform(-k, k, (C, 4 * H)).astype(np.float32)
    R = r.uniform(-k, k, (H, 4 * H)).astype(np.float32)
    b = np.zeros(4 * H, np.float32)
    b[2 * H:3 * H] = forget_bias
    x = r.standard_normal((T, N, C)).astype(np.float32)
    dy = r.standard_normal((T, N, H)).astype(np.float32)
    dhT = r.standard_normal((N, H)).astype(np.float32)
    dcT = r.standard_normal((N, H)).astype(np.float32)
    return W, R, b, x, dy, dhT, dcT


def profile_read(lib, name):
    total = ctypes.c_double(0.0)
    count = ctypes.c_int(0)
    rc = lib.haste_hip_profile_read(name.encode(), ctypes.byref(total), ctypes.byref(count))
    if rc != 0:
        raise RuntimeError("haste_hip_profile_read failed: %d" % rc)
    return total.value, count.value


def run_metric(args, torch, lib, ops, dev):
    """LSTM fwd+bwd N=64 T=100 C=H=512: ms per batch and the per-kernel breakdown."""
    T, N, C, H = 100, 64, 512, 512
    W, R, b, x, dy, dhT, dcT = make_inputs(T, N, C, H)
    Wd, Rd, bd, xd = (torch.from_numpy(a).to(dev) for a in (W, R, b, x))
    h0 = torch.zeros(N, H, device=dev)
    c0 = torch.zeros(N, H, device=dev)
    dh_new = torch.zeros(T + 1, N, H, device=dev)
    dh_new[1:] = torch.from_numpy(dy).to(dev)
    dh_new[T] += torch.from_numpy(dhT).to(dev)
    dc_new = torch.zeros(T + 1, N, H, device=dev)
    dc_new[T] = torch.from_numpy(dcT).to(dev)
    no_mask = torch.empty(0, 0, 0, device=dev)

    # The timed step is the loop body of the reference's benchmark (benchmarks/benchmark_lstm.cc:
    # 399-463): ForwardPass::Run, the three caller-side transposes the backward API asks for
    # (cublasSgeam there, the library's helper here), BackwardPass::Run -- through the C-ABI, on
    # buffers allocated once.  As there, dW, dR, db accumulate over the iterations and dh, dc
    # carry over; nothing is zeroed or copied inside the loop.
    from haste_amd import lib as hlib
    f32 = dict(device=dev, dtype=torch.float32)
    h = torch.zeros(T + 1, N, H, **f32)
    c = torch.zeros(T + 1, N, H, **f32)
    h[0], c[0] = h0, c0
    v = torch.empty(T, N, 4 * H, **f32)
    x_t = torch.empty(C, T, N, **f32)
    W_t = torch.empty(4 * H, C, **f32)
    R_t = torch.empty(4 * H, H, **f32)
    dx = torch.empty(T, N, C, **f32)
    dW, dR, db = torch.zeros(C, 4 * H, **f32), torch.zeros(H, 4 * H, **f32), torch.zeros(4 * H, **f32)
    dh, dc = torch.zeros(N, H, **f32), torch.zeros(N, H, **f32)

    def step():
        hlib.call("haste_hip_lstm_forward_f32", True, T, N, C, H, Wd, Rd, bd, xd, h, c, v, None, 0.0, None)
        hlib.call("haste_hip_transpose3_f32", T * N, C, xd, x_t, C, 4 * H, Wd, W_t, H, 4 * H, Rd, R_t)
        hlib.call("haste_hip_lstm_backward_f32", T, N, C, H, W_t, R_t, bd, x_t, h, c, dh_new, dc_new,
                  dx, dW, dR, db, dh, dc, v, None)

    # The same work as a caller of the PyTorch-level ops sees it: outputs allocated per call,
    # h0 / c0 copied into slot 0, the accumulated gradients zero-filled (reported beside it).
    def ops_step():
        hh, cc, cache = ops.lstm_forward(True, 0.0, xd, h0, c0, Wd, Rd, bd, no_mask)
        return ops.lstm_backward(*ops.transpose3(xd, Wd, Rd), bd, no_mask,
                                 hh, cc, cache, dh_new, dc_new)

    for _ in range(args.warmup):
        ops_step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(args.steps):
        ops_step()
    e1.record()
    torch.cuda.synchronize()
    ms_per_ops_step = e0.elapsed_time(e1) / args.steps

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    ev0 = torch.cuda.Event(enable_timing=True)
    ev1 = torch.cuda.Event(enable_timing=True)
    ev0.record()
    for _ in range(args.steps):
        step()
    ev1.record()
    torch.cuda.synchronize()
    ms_per_step = ev0.elapsed_time(ev1) / args.steps

    # The same K steps again with per-kernel event timing switched on in the library
    # (events on the stream the kernels run on).
    lib.haste_hip_profile_reset()
    lib.haste_hip_profile_enable(1)
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    lib.haste_hip_profile_enable(0)
    f_gemm = 2.0 * T * N * C * 4 * H  # each of the 4 products x*W, dx, dW, dR (C == H)
    f_rec = 2.0 * T * N * H * 4 * H   # h*R over all steps, forward or backward
    gemm_ms, gemm_count = profile_read(lib, "gemm_f32")
    # With 4-row batch tiles the forward recurrence computes x*W itself: the step then has
    # three GEMM products instead of four and the forward kernel does the flops of two.
    fused_input = round(gemm_count / args.steps) == 3
    kernels = {}
    for name, flops in (("gemm_f32", f_gemm),
                        ("lstm_forward_recurrence", f_rec + (f_gemm if fused_input else 0.0)),
                        ("lstm_backward_recurrence", f_rec)):
        total_ms, count = profile_read(lib, name)
        avg_ms = total_ms / max(count, 1)
        tf = flops / (avg_ms * 1e-3) / 1e12 if avg_ms > 0 else 0.0
        kernels[name] = {"launches_per_step": count / args.steps, "avg_ms": round(avg_ms, 5),
                         "ms_per_step": round(total_ms / args.steps, 5),
                         "flops_per_launch": flops, "tflops": round(tf, 3),
                         "frac_of_fp32_mfma_peak": round(tf / PEAK_FP32_MFMA_TFLOPS, 4)}
    if fused_input:
        kernels["lstm_forward_recurrence"]["computes_input_projection"] = True
    lib.haste_hip_profile_reset()
    # The roofline entry is the kernel with the longest single launch (a recurrence), with the
    # whole step beside it: all six products of the step, 2*T*N*4H*(3C + 3H) flops, over the
    # step's wall time.
    total_flops = 3.0 * (f_gemm + f_rec)
    tflops_whole = total_flops / (ms_per_step * 1e-3) / 1e12
    dominant = max(kernels, key=lambda k: kernels[k]["avg_ms"])
    dom = kernels[dominant]
    roofline = {"kernel": dominant, "bound": "mfma", "achieved": dom["tflops"],
                "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
                "frac": round(dom["tflops"] / PEAK_FP32_MFMA_TFLOPS, 4),
                "traffic": MEASURED_TRAFFIC_BYTES.get(dominant),
                "traffic_source": TRAFFIC_SOURCE,
                "us_per_launch": round(dom["avg_ms"] * 1e3, 2),
                "whole_step_tflops": round(tflops_whole, 3),
                "whole_step_frac": round(tflops_whole / PEAK_FP32_MFMA_TFLOPS, 4)}
    return dict(ms_per_step=ms_per_step, ms_per_ops_step=ms_per_ops_step, kernels=kernels, roofline=roofline,
                tflops_whole_step=tflops_whole, host=(W, R, b, x, dy))


def run_measured_peak(args, torch, lib, ops, dev):
    """What the fp32 matrix cores deliver on this box on a long, square product (the library's
    own GEMM at 8192^3), beside the nominal 157.3 TFLOP/s the fractions are quoted against."""
    n = 8192
    a = torch.randn(n, n, device=dev)
    b = torch.randn(n, n, device=dev)
    out = torch.empty(n, n, device=dev)
    for _ in range(2):
        ops.gemm(a, b, out=out)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    reps = 5
    e0.record()
    for _ in range(reps):
        ops.gemm(a, b, out=out)
    e1.record()
    torch.cuda.synchronize()
    tf = 2.0 * n ** 3 / (e0.elapsed_time(e1) / reps * 1e-3) / 1e12
    return {"workload": "gemm_f32 8192 x 8192 x 8192", "tflops": round(tf, 2),
            "frac_of_nominal": round(tf / PEAK_FP32_MFMA_TFLOPS, 4)}


def run_iterate(args, torch, lib, ops, dev):
    """Single steps through the Iterate entry points (the reference's autoregressive API,
    lib/haste/lstm.h:73-86): microseconds per call, N=1, C=H=512, inference, end to end on
    preallocated buffers (the state ping-pongs between two pairs)."""
    from haste_amd import lib as hlib
    N, C, H = 1, 512, 512
    g = torch.Generator(device="cpu").manual_seed(3)
    k = H ** -0.5
    W = ((torch.rand(C, 4 * H, generator=g) * 2 - 1) * k).to(dev)
    R = ((torch.rand(H, 4 * H, generator=g) * 2 - 1) * k).to(dev)
    b = torch.zeros(4 * H, device=dev)
    x = torch.randn(N, C, generator=g).to(dev)
    hs = [torch.zeros(N, H, device=dev), torch.zeros(N, H, device=dev)]
    cs = [torch.zeros(N, H, device=dev), torch.zeros(N, H, device=dev)]
    v = torch.empty(N, 4 * H, device=dev)

    def call(i):
        hlib.call("haste_hip_lstm_forward_iterate_f32", False, N, C, H, W, R, b, x, hs[i & 1], cs[i & 1],
                  hs[(i + 1) & 1], cs[(i + 1) & 1], v, None, 0.0, None)
    for i in range(20):
        call(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    reps = 400
    e0.record()
    for i in range(reps):
        call(i)
    e1.record()
    torch.cuda.synchronize()
    out = {"workload": "LSTM Iterate N=1 C=H=512 fp32 inference, %d calls back to back" % reps,
           "us_per_call": round(e0.elapsed_time(e1) * 1e3 / reps, 3)}

    # The same calls recorded into a HIP graph (the stream's scratch memory lent by the caller,
    # so that nothing allocates under capture) and replayed: what a decoding loop that replays a
    # captured chunk of steps pays per step.
    chunk = 100
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        lent = torch.empty(ops.workspace_bytes(1, N, C, H), dtype=torch.uint8, device=dev)
        ops.set_workspace(lent)
        try:
            for i in range(4):
                call(i)
            side.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                for i in range(chunk):
                    call(i)
            graph.replay()
            side.synchronize()
            g0, g1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            g0.record()
            for _ in range(10):
                graph.replay()
            g1.record()
            side.synchronize()
            out["us_per_call_graph_replay"] = round(g0.elapsed_time(g1) * 1e3 / (10 * chunk), 3)
            out["graph"] = "%d calls per graph, 10 replays" % chunk
            del graph
        finally:
            side.synchronize()
            ops.set_workspace(None)
    return out


def run_streaming(args, torch, lib, ops, dev):
    """LSTM inference N=1 T=2000 C=H=512: microseconds per timestep."""
    T1, N1, C, H = 2000, 1, 512, 512
    W1, R1, b1, x1, *_ = make_inputs(T1, N1, C, H, seed=1, forget_bias=0.0)
    W1d, R1d, b1d, x1d = (torch.from_numpy(a).to(dev) for a in (W1, R1, b1, x1))
    h01 = torch.zeros(N1, H, device=dev)
    c01 = torch.zeros(N1, H, device=dev)
    no_mask = torch.empty(0, 0, 0, device=dev)

    def stream_step():
        return ops.lstm_forward(False, 0.0, x1d, h01, c01, W1d, R1d, b1d, no_mask)

    for _ in range(3):
        stream_step()
    torch.cuda.synchronize()
    ev0 = torch.cuda.Event(enable_timing=True)
    ev1 = torch.cuda.Event(enable_timing=True)
    lib.haste_hip_profile_reset()
    lib.haste_hip_profile_enable(1)
    reps = 10
    ev0.record()
    for _ in range(reps):
        stream_step()
    ev1.record()
    torch.cuda.synchronize()
    lib.haste_hip_profile_enable(0)
    us_total = ev0.elapsed_time(ev1) * 1e3 / reps / T1
    rec_ms, rec_n = profile_read(lib, "lstm_forward_recurrence")
    lib.haste_hip_profile_reset()
    us_rec = rec_ms * 1e3 / max(rec_n, 1) / T1
    b_step = 4.0 * (4 * H * H + 2 * 4 * H + 4 * H)  # R + Wx_t + b + h,c in + h,c out
    gbs = b_step / (us_rec * 1e-6) / 1e9
    out = {"workload": "LSTM inference N=1 T=2000 C=H=512 fp32",
           "us_per_timestep": round(us_total, 4),
           "us_per_timestep_recurrence_kernel": round(us_rec, 4),
           "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS,
                        "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4),
                        "bytes_per_step_model": b_step,
                        "note": "streamed-R byte model; R is kept on chip, so this is an "
                                "equivalent bandwidth, not HBM traffic"}}
    return out, (W1, R1, b1, x1)


def run_stepwise(args, torch, lib, ops, dev):
    """LSTM inference N=1 T=50 C=512 H=4096 (the largest hidden size of the reference's
    benchmark grid): R does not fit on chip and is streamed from HBM by every step's product."""
    T, N, C, H = 50, 1, 512, 4096
    g = torch.Generator(device="cpu").manual_seed(2)
    k = H ** -0.5
    W = ((torch.rand(C, 4 * H, generator=g) * 2 - 1) * k).to(dev)
    R = ((torch.rand(H, 4 * H, generator=g) * 2 - 1) * k).to(dev)
    b = torch.zeros(4 * H, device=dev)
    x = torch.randn(T, N, C, generator=g).to(dev)
    h0, c0 = torch.zeros(N, H, device=dev), torch.zeros(N, H, device=dev)
    no_mask = torch.empty(0, 0, 0, device=dev)

    def step():
        return ops.lstm_forward(False, 0.0, x, h0, c0, W, R, b, no_mask)

    for _ in range(3):
        step()
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    reps = 10
    ev0.record()
    for _ in range(reps):
        step()
    ev1.record()
    torch.cuda.synchronize()
    us_total = ev0.elapsed_time(ev1) * 1e3 / reps / T
    # again with per-kernel event timing switched on in the library
    lib.haste_hip_profile_reset()
    lib.haste_hip_profile_enable(1)
    for _ in range(reps):
        step()
    torch.cuda.synchronize()
    lib.haste_hip_profile_enable(0)
    ms, n = profile_read(lib, "gemm_f32_skinny")
    lib.haste_hip_profile_reset()
    us_product = ms * 1e3 / max(n, 1)
    b_product = 4.0 * H * 4 * H  # R, read once per step
    gbs = b_product / (us_product * 1e-6) / 1e9
    return {"workload": "LSTM inference N=1 T=50 C=512 H=4096 fp32",
            "us_per_timestep": round(us_total, 3),
            "roofline": {"kernel": "gemm_f32_skinny", "bound": "hbm", "achieved": round(gbs, 1),
                         "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4),
                         "us_per_launch": round(us_product, 2), "bytes_per_launch": b_product,
                         "traffic": MEASURED_TRAFFIC_BYTES.get("gemm_f32_skinny")}}


def run_hbm_kernels(args, torch, lib, ops, dev):
    """The HBM-bound kernels of the path against the 8 TB/s roof: stand-alone layer norm
    (rows = T*N of BASELINE configuration 4, D = 4H), IndRNN recurrences and the transpose
    helper.  Algorithmic bytes: each distinct tensor element read or written once."""
    out = {}

    def timed(names, fn, reps=20):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        lib.haste_hip_profile_reset()
        lib.haste_hip_profile_enable(1)
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        lib.haste_hip_profile_enable(0)
        res = {}
        for name in names:
            ms, n = profile_read(lib, name)
            res[name] = ms / max(n, 1)
        lib.haste_hip_profile_reset()
        return res

    def entry(ms, nbytes):
        gbs = nbytes / (ms * 1e-3) / 1e9
        return {"us": round(ms * 1e3, 2), "bytes": nbytes, "bound": "hbm", "achieved": round(gbs, 1),
                "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4)}

    rows, D = 500 * 32, 1024
    x = torch.randn(rows, D, device=dev)
    dy = torch.randn(rows, D, device=dev)
    gamma = torch.rand(D, device=dev) + 0.5
    cache = [None]

    def ln():
        y, cache[0] = ops.layer_norm_forward(x, gamma, None)
        ops.layer_norm_backward(x, gamma, dy, cache[0], False)
    t = timed(("layer_norm_forward", "layer_norm_backward"), ln)
    out["layer_norm_forward_16000x1024"] = entry(t["layer_norm_forward"], 4.0 * (2 * rows * D + 2 * rows))
    out["layer_norm_backward_16000x1024"] = entry(t["layer_norm_backward"], 4.0 * 3 * rows * D)

    T, N, C, H = 100, 64, 512, 512
    xs = torch.randn(T, N, C, device=dev)
    W = (torch.rand(C, H, device=dev) - 0.5) * H ** -0.5
    u = torch.rand(H, device=dev) - 0.5
    b = torch.zeros(H, device=dev)
    h0 = torch.zeros(N, H, device=dev)
    dh_new = torch.randn(T + 1, N, H, device=dev)
    no_mask = torch.empty(0, 0, 0, device=dev)
    x_t, W_t = ops.transpose(xs), ops.transpose(W)

    def ind():
        h = ops.indrnn_forward(True, 0.0, xs, h0, W, u, b, no_mask)
        ops.indrnn_backward(x_t, W_t, u, b, no_mask, h, dh_new)
    t = timed(("indrnn_forward_recurrence", "indrnn_backward_recurrence"), ind)
    # forward: x*W in, h out; backward: h (twice: h_t, h_{t+1} are the same tensor) and
    # dh_new in, the gradient w.r.t. x*W out
    out["indrnn_forward_N64_T100_H512"] = entry(t["indrnn_forward_recurrence"], 4.0 * 2 * T * N * H)
    out["indrnn_backward_N64_T100_H512"] = entry(t["indrnn_backward_recurrence"], 4.0 * 3 * T * N * H)

    t = timed(("transpose_f32",), lambda: ops.transpose(xs))
    out["transpose_6400x512"] = entry(t["transpose_f32"], 4.0 * 2 * T * N * C)
    del xs, x_t, dh_new

    # The reference's IndRNN speed script (validation/pytorch_speed.py:7-20): T=2500, N=64,
    # C=256, H=4096, where the recurrences move 5 / 8 GB and are bound by HBM.
    T, N, C, H = 2500, 64, 256, 4096
    xs = torch.randn(T, N, C, device=dev)
    W = (torch.rand(C, H, device=dev) - 0.5) * H ** -0.5
    u = torch.rand(H, device=dev) - 0.5
    b = torch.zeros(H, device=dev)
    h0 = torch.zeros(N, H, device=dev)
    dh_new = torch.randn(T + 1, N, H, device=dev)
    x_t, W_t = ops.transpose(xs), ops.transpose(W)
    total = {}

    def ind_speed():
        e = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
        e[0].record()
        h = ops.indrnn_forward(True, 0.0, xs, h0, W, u, b, no_mask)
        e[1].record()
        ops.indrnn_backward(x_t, W_t, u, b, no_mask, h, dh_new)
        e[2].record()
        torch.cuda.synchronize()
        total["fwd"], total["bwd"] = e[0].elapsed_time(e[1]), e[1].elapsed_time(e[2])
    t = timed(("indrnn_forward_recurrence", "indrnn_backward_recurrence"), ind_speed, reps=3)
    out["indrnn_forward_N64_T2500_C256_H4096"] = entry(t["indrnn_forward_recurrence"], 4.0 * 2 * T * N * H)
    out["indrnn_backward_N64_T2500_C256_H4096"] = entry(t["indrnn_backward_recurrence"], 4.0 * 3 * T * N * H)
    del xs, x_t, dh_new

    # Yardstick: what a plain device copy of 1 GiB (read once, written once: the same mix of
    # traffic as the IndRNN recurrences) reaches on this box.
    src = torch.empty(256 * 1024 * 1024, device=dev)
    dst = torch.empty_like(src)
    for _ in range(2):
        dst.copy_(src)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(5):
        dst.copy_(src)
    e1.record()
    torch.cuda.synchronize()
    out["device_copy_1GiB"] = entry(e0.elapsed_time(e1) / 5.0, 2.0 * 4 * src.numel())
    del src, dst
    out["indrnn_speed_script_shape"] = {"forward_pass_ms": round(total["fwd"], 3), "backward_pass_ms": round(total["bwd"], 3),
                                        "note": "whole passes (x*W, recurrence; recurrence, dW, dx) at the shape of "
                                                "the reference's validation/pytorch_speed.py"}
    return out


def run_configs(args, torch, lib, ops, dev):
    """The other BASELINE.json configurations (parity-test cases; timed here for the record):
    forward (+ backward with the caller-side transposes) in ms per call, with the algorithmic
    flops of the matrix products (2*T*N*G*H*(C + H) forward, three times that forward +
    backward) and the fraction of the matrix cores' peak for the arithmetic type.  Also the
    other instantiations of the reference at the metric shape: the double LSTM (step-wise regime:
    one product and one pointwise launch per step) and the half GRU (fp32 recurrences on widened
    tensors, products on the half matrix cores)."""
    details = {}

    def note(key, ms, flops, peak=PEAK_FP32_MFMA_TFLOPS, dtype="f32"):
        tf = flops / (ms * 1e-3) / 1e12
        details[key] = {"ms": ms, "flops": flops, "tflops": round(tf, 3), "dtype": dtype,
                        "peak_tflops": peak, "frac_of_mfma_peak": round(tf / peak, 4)}

    def timed(fn, reps):
        # untimed calls first: the allocator's pools, the library's scratch buffer and the clocks
        # settle within the first dozen calls of a shape (GRU configuration: 0.83 -> 0.79 ms)
        for _ in range(12):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return round(e0.elapsed_time(e1) / reps, 4)

    g = torch.Generator(device="cpu").manual_seed(0)

    def rnd(*shape, scale=1.0):
        return (torch.randn(*shape, generator=g) * scale).to(dev)

    def uni(k, *shape):
        return ((torch.rand(*shape, generator=g) * 2 - 1) * k).to(dev)
    no_mask = torch.empty(0, 0, 0, device=dev)
    out = {}

    T, N, C, H = 100, 16, 128, 256  # config 1: LSTM forward inference
    k = H ** -0.5
    x, W, R, b = rnd(T, N, C), uni(k, C, 4 * H), uni(k, H, 4 * H), torch.zeros(4 * H, device=dev)
    z = torch.zeros(N, H, device=dev)
    out["lstm_inference_N16_T100_C128_H256_ms"] = timed(
        lambda: ops.lstm_forward(False, 0.0, x, z, z, W, R, b, no_mask), 50)
    note("lstm_inference_N16_T100_C128_H256", out["lstm_inference_N16_T100_C128_H256_ms"],
         2.0 * T * N * 4 * H * (C + H))

    T, N, C, H = 100, 64, 512, 512  # config 2: GRU training, zoneout 0.1, DropConnect 0.05
    k = H ** -0.5
    x, W, R = rnd(T, N, C), uni(k, C, 3 * H), uni(k, H, 3 * H)
    bx, br, z = uni(k, 3 * H), uni(k, 3 * H), torch.zeros(N, H, device=dev)
    zm = (torch.rand(T, N, H, generator=g) >= 0.1).float().to(dev)
    dm = (torch.rand(H, 3 * H, generator=g) >= 0.05).float().to(dev)
    dh_new = rnd(T + 1, N, H)

    def gru_step():
        h, cache = ops.gru_forward(True, 0.1, x, z, W, R, bx, br, zm, dm, 1.0 / 0.95)
        Reff_t = ops.transpose(R * dm * (1.0 / 0.95))
        return ops.gru_backward(ops.transpose(x), ops.transpose(W), Reff_t, bx, br, zm, h, cache, dh_new)
    out["gru_fwd_bwd_N64_T100_H512_zoneout_dropconnect_ms"] = timed(gru_step, 30)
    note("gru_fwd_bwd_N64_T100_H512_zoneout_dropconnect", out["gru_fwd_bwd_N64_T100_H512_zoneout_dropconnect_ms"],
         3 * 2.0 * T * N * 3 * H * (C + H))

    # the half GRU of the reference (lib/gru_forward_gpu.cu.cc:373) at the same shape
    xh, Wh, Rh, bxh, brh, zh, zmh, dhh = (a.half() for a in (x, W, R, bx, br, z, zm, dh_new))

    def gru_half_step():
        h, cache = ops.gru_forward(True, 0.1, xh, zh, Wh, Rh, bxh, brh, zmh)
        return ops.gru_backward(ops.transpose(xh), ops.transpose(Wh), ops.transpose(Rh), bxh, brh, zmh, h, cache, dhh)
    ms = timed(gru_half_step, 20)
    out["gru_f16_fwd_bwd_N64_T100_H512_zoneout_ms"] = ms
    # half tensors; the recurrences (half of the flops) run in fp32 on widened copies, the
    # products around them on the half matrix cores: quoted against the fp32 peak, like the rest
    note("gru_f16_fwd_bwd_N64_T100_H512_zoneout", ms, 3 * 2.0 * T * N * 3 * H * (C + H), PEAK_FP32_MFMA_TFLOPS,
         "f16 tensors, f32 recurrences, f16 products with f32 accumulation")

    T, N, C, H = 100, 128, 512, 512  # config 3: LSTM training, N=128
    x, W, R = rnd(T, N, C), uni(k, C, 4 * H), uni(k, H, 4 * H)
    b = torch.zeros(4 * H, device=dev)
    b[2 * H:3 * H] = 1.0
    z = torch.zeros(N, H, device=dev)
    dh_new, dc_new = rnd(T + 1, N, H), rnd(T + 1, N, H)

    def lstm_step():
        h, c, cache = ops.lstm_forward(True, 0.0, x, z, z, W, R, b, no_mask)
        return ops.lstm_backward(*ops.transpose3(x, W, R), b, no_mask, h, c,
                                 cache, dh_new, dc_new)
    out["lstm_fwd_bwd_N128_T100_H512_ms"] = timed(lstm_step, 30)
    note("lstm_fwd_bwd_N128_T100_H512", out["lstm_fwd_bwd_N128_T100_H512_ms"], 3 * 2.0 * T * N * 4 * H * (C + H))

    # the double LSTM of the reference (lib/lstm_forward_gpu.cu.cc:368-369) at the metric shape
    Nd = 64
    xd_, Wd_, Rd_, bd_, zd_ = x[:, :Nd].double().contiguous(), W.double(), R.double(), b.double(), z[:Nd].double()
    dhd_, dcd_ = dh_new[:, :Nd].double().contiguous(), dc_new[:, :Nd].double().contiguous()
    no_mask64 = torch.empty(0, 0, 0, device=dev, dtype=torch.float64)

    def lstm_double_step():
        h, c, cache = ops.lstm_forward(True, 0.0, xd_, zd_, zd_, Wd_, Rd_, bd_, no_mask64)
        return ops.lstm_backward(*ops.transpose3(xd_, Wd_, Rd_), bd_, no_mask64, h, c, cache, dhd_, dcd_)
    ms = timed(lstm_double_step, 10)
    out["lstm_f64_fwd_bwd_N64_T100_H512_ms"] = ms
    note("lstm_f64_fwd_bwd_N64_T100_H512", ms, 3 * 2.0 * T * Nd * 4 * H * (C + H), PEAK_FP64_MFMA_TFLOPS, "f64")

    T, N, C, H = 500, 32, 256, 256  # config 4: LayerNormLSTM training, zoneout 0.1
    k = H ** -0.5
    x, W, R = rnd(T, N, C), uni(k, C, 4 * H), uni(k, H, 4 * H)
    b = torch.zeros(4 * H, device=dev)
    b[2 * H:3 * H] = 1.0
    gamma, gamma_h, beta_h = torch.ones(2, 4 * H, device=dev), torch.ones(H, device=dev), torch.zeros(H, device=dev)
    z = torch.zeros(N, H, device=dev)
    zm = (torch.rand(T, N, H, generator=g) >= 0.1).float().to(dev)
    dh_new, dc_new = rnd(T + 1, N, H), rnd(T + 1, N, H)

    def ln_lstm_step():
        fwd = ops.layer_norm_lstm_forward(True, 0.1, x, z, z, W, R, b, gamma, gamma_h, beta_h, zm)
        return ops.layer_norm_lstm_backward(*ops.transpose3(x, W, R), b, gamma,
                                            gamma_h, beta_h, zm, *fwd, dh_new, dc_new)
    out["layer_norm_lstm_fwd_bwd_N32_T500_H256_zoneout_ms"] = timed(ln_lstm_step, 10)
    note("layer_norm_lstm_fwd_bwd_N32_T500_H256_zoneout", out["layer_norm_lstm_fwd_bwd_N32_T500_H256_zoneout_ms"],
         3 * 2.0 * T * N * 4 * H * (C + H))
    return out, details


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: the path has no multi-GPU component "
              "(got --gpus %d)" % args.gpus, file=sys.stderr)
        sys.exit(2)
    import torch
    from haste_amd import lib as hlib, ops
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    lib = hlib.load()
    torch.cuda.set_device(0)
    dev = torch.device("cuda:0")

    if args.workload == "copy":
        n = 256 * 1024 * 1024  # floats: 1 GiB read + 1 GiB written per copy
        src = torch.ones(n, device=dev)
        dst = torch.empty_like(src)
        for _ in range(args.steps):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"workload": "copy", "bytes_read_per_copy": 4 * n,
                          "bytes_written_per_copy": 4 * n, "copies": args.steps}))
        return
    if args.workload == "metric":
        m = run_metric(args, torch, lib, ops, dev)
        print(json.dumps({"workload": "metric", "ms_per_step": round(m["ms_per_step"], 4),
                          "ms_per_step_pytorch_ops": round(m["ms_per_ops_step"], 4),
                          "kernels": m["kernels"]}))
        return
    if args.workload == "configs":
        configs, details = run_configs(args, torch, lib, ops, dev)
        print(json.dumps({"other_configs_ms": configs, "other_configs": details}))
        return
    if args.workload == "streaming":
        s, _ = run_streaming(args, torch, lib, ops, dev)
        print(json.dumps(s))
        return
    if args.workload == "stepwise":
        print(json.dumps(run_stepwise(args, torch, lib, ops, dev)))
        return
    if args.workload == "peak":
        print(json.dumps(run_measured_peak(args, torch, lib, ops, dev)))
        return
    if args.workload == "iterate":
        print(json.dumps(run_iterate(args, torch, lib, ops, dev)))
        return
    if args.workload == "hbm_kernels":
        print(json.dumps(run_hbm_kernels(args, torch, lib, ops, dev)))
        return

    m = run_metric(args, torch, lib, ops, dev)
    streaming, host1 = run_streaming(args, torch, lib, ops, dev)
    stepwise = run_stepwise(args, torch, lib, ops, dev)
    hbm_kernels = run_hbm_kernels(args, torch, lib, ops, dev)
    configs, config_details = run_configs(args, torch, lib, ops, dev)
    measured_peak = run_measured_peak(args, torch, lib, ops, dev)
    iterate = run_iterate(args, torch, lib, ops, dev)
    m["roofline"]["measured_peak"] = measured_peak["tflops"]
    m["roofline"]["frac_of_measured_peak"] = round(m["roofline"]["achieved"] / measured_peak["tflops"], 4)

    # CPU baseline: torch.nn.LSTM fwd+bwd on the host cores (bounded sample).
    cpu = None
    if not args.no_cpu_baseline:
        from oracle import cpu_baseline
        W, R, b, x, dy = m["host"]
        W1, R1, b1, x1 = host1
        threads = torch.get_num_threads()
        t = cpu_baseline.time_lstm_fwd_bwd(W, R, b, x, dy, budget_s=args.cpu_budget)
        t1 = cpu_baseline.time_lstm_inference(W1, R1, b1, x1[:500], budget_s=4.0)
        torch.set_num_threads(1)
        t1_single = cpu_baseline.time_lstm_inference(W1, R1, b1, x1[:500], budget_s=4.0)
        torch.set_num_threads(threads)
        cpu = {"value": round(t["median"] * 1e3, 3), "min": round(t["min"] * 1e3, 3), "unit": "ms/batch",
               "cores": threads, "kind": "port", "cpu_model": cpu_baseline.cpu_model(),
               "sample": "torch.nn.LSTM fwd+bwd fp32 on host CPU, same weights via the native "
                         "weight map, N=64 T=100 C=H=512, median (and minimum) of %d iterations; "
                         "os.cpu_count=%d" % (t["iterations"], os.cpu_count()),
               "n1_us_per_timestep": round(t1["median"] * 1e6 / 500, 3),
               "n1_us_per_timestep_min": round(t1["min"] * 1e6 / 500, 3),
               "n1_us_per_timestep_one_thread": round(t1_single["median"] * 1e6 / 500, 3),
               "n1_us_per_timestep_one_thread_min": round(t1_single["min"] * 1e6 / 500, 3),
               "n1_sample": "torch.nn.LSTM inference N=1, first 500 of 2000 steps, %d threads: median "
                            "of %d; one thread: median of %d" % (threads, t1["iterations"], t1_single["iterations"])}

    out = {
        "metric": "LSTM fwd+bwd ms/batch (N=64,T=100,H=512 fp32)",
        "value": round(m["ms_per_step"], 4), "unit": "ms/batch",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(m["ms_per_step"], 4), "higher_is_better": False, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "LSTM training fwd+bwd N=64 T=100 C=H=512 fp32, forget bias 1: the loop "
                               "body of the reference's benchmark_lstm.cc (ForwardPass::Run, the "
                               "three caller-side transposes, BackwardPass::Run) through the C-ABI"},
        "ms_per_step_pytorch_ops": round(m["ms_per_ops_step"], 4),
        "achieved_tflops_whole_step": round(m["tflops_whole_step"], 3),
        "roofline": m["roofline"],
        "kernels": m["kernels"],
        "streaming_n1": streaming,
        "stepwise_n1_h4096": stepwise,
        "hbm_kernels": hbm_kernels,
        "other_configs_ms": configs,
        "other_configs": config_details,
        "measured_fp32_mfma_peak": measured_peak,
        "iterate_n1": iterate,
        "cpu_baseline": cpu,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
