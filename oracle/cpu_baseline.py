"""CPU baseline for the benchmark (TEST/BENCH INFRASTRUCTURE, not product code).

Runs the same LSTM weights through torch.nn.LSTM on the host CPU, using the
Haste -> native weight map (reference frameworks/pytorch/lstm.py:159-180), the
way the reference's own validation does (validation/pytorch.py:65-89).
"""
import time

import numpy as np
import torch

from . import haste_oracle as O


def native_lstm(W, R, b):
    C, H = W.shape[0], R.shape[0]
    w_ih, w_hh, b_ih, b_hh = O.lstm_to_native(W.astype(np.float64), R.astype(np.float64),
                                              b.astype(np.float64))
    m = torch.nn.LSTM(C, H)
    with torch.no_grad():
        m.weight_ih_l0.copy_(torch.from_numpy(w_ih).float())
        m.weight_hh_l0.copy_(torch.from_numpy(w_hh).float())
        m.bias_ih_l0.copy_(torch.from_numpy(b_ih).float())
        m.bias_hh_l0.copy_(torch.from_numpy(b_hh).float())
    return m


def time_lstm_fwd_bwd(W, R, b, x, dy, budget_s=15.0, warmup=2, min_iters=3):
    """Median and minimum seconds of torch.nn.LSTM forward + backward on CPU, fp32."""
    m = native_lstm(W, R, b)
    xt = torch.from_numpy(x.astype(np.float32)).requires_grad_()
    dyt = torch.from_numpy(dy.astype(np.float32))
    times = []
    t_start = time.perf_counter()
    it = 0
    while True:
        m.zero_grad(set_to_none=True)
        xt.grad = None
        t0 = time.perf_counter()
        y, _ = m(xt)
        y.backward(dyt)
        dt = time.perf_counter() - t0
        it += 1
        if it > warmup:
            times.append(dt)
        if len(times) >= min_iters and time.perf_counter() - t_start > budget_s:
            break
        if len(times) >= 50:
            break
    return {"median": float(np.median(times)), "min": float(np.min(times)), "iterations": len(times)}


def time_lstm_inference(W, R, b, x, budget_s=10.0, warmup=1, min_iters=3):
    """Median and minimum seconds of torch.nn.LSTM forward (no grad) on CPU, fp32."""
    m = native_lstm(W, R, b)
    xt = torch.from_numpy(x.astype(np.float32))
    times = []
    t_start = time.perf_counter()
    it = 0
    with torch.no_grad():
        while True:
            t0 = time.perf_counter()
            m(xt)
            dt = time.perf_counter() - t0
            it += 1
            if it > warmup:
                times.append(dt)
            if len(times) >= min_iters and time.perf_counter() - t_start > budget_s:
                break
            if len(times) >= 50:
                break
    return {"median": float(np.median(times)), "min": float(np.min(times)), "iterations": len(times)}


def cpu_model():
    """Model name of the host CPU (/proc/cpuinfo), or the platform's processor string."""
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    import platform
    return platform.processor() or "unknown"
