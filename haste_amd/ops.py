"""Op-level interface: the functions the reference exposes from its PyTorch binding
(`haste_pytorch_lib.<cell>_forward / <cell>_backward`, reference
frameworks/pytorch/{lstm,gru,indrnn,layer_norm_lstm,layer_norm_gru,layer_norm_indrnn}.cc),
with the same argument order, allocation protocol and return tuples, implemented by
calls into libhaste_hip.so.  Tensors are float32 or float64, for the GRU also float16 (all tensors of a call alike),
contiguous, on the GPU; torch is used only to allocate device memory and to name the
current stream.
"""
import torch

from . import lib


def _check(*tensors):
    # reference frameworks/pytorch/support.h:20-22 (CHECK_INPUT)
    for t in tensors:
        if not t.is_cuda:
            raise ValueError("tensor must be a GPU tensor")
        if not t.is_contiguous():
            raise ValueError("tensor must be contiguous")
        if t.numel() and t.dtype not in _SUFFIX:
            raise ValueError("only float32, float64 and (GRU) float16 are implemented")


_SUFFIX = {torch.float32: "_f32", torch.float64: "_f64", torch.float16: "_f16"}


def _call(entry, *args):
    """Calls `entry` + "_f32" / "_f64" according to the tensors among `args`, which must all
    have one dtype (the reference's bindings dispatch the same way, AT_DISPATCH_FLOATING_TYPES,
    frameworks/pytorch/lstm.cc:65)."""
    dtypes = {a.dtype for a in args if isinstance(a, torch.Tensor) and a.numel()}
    if len(dtypes) != 1:
        raise ValueError("all tensors of a call must have the same dtype, got %s" % sorted(map(str, dtypes)))
    name = entry + _SUFFIX[dtypes.pop()]
    if not hasattr(lib.load(), name):
        # as in the reference, half exists for the GRU only (lib/gru_forward_gpu.cu.cc:373)
        raise ValueError("%s is not implemented" % name)
    lib.call(name, *args)


def stream_status(stream=None):
    """After the caller has synchronized `stream` (default: the current stream): raises
    lib.HasteHipError when a persistent kernel launched on it gave up a bounded wait (its
    outputs, and those of library kernels queued behind it, are invalid); see
    haste_hip_stream_status in include/haste_hip.h."""
    import ctypes
    handle = lib.load()
    if stream is None:
        stream = torch.cuda.current_stream().cuda_stream
    handle.haste_hip_stream_status.restype = ctypes.c_int
    rc = handle.haste_hip_stream_status(ctypes.c_void_p(stream))
    if rc != 0:
        raise lib.HasteHipError(rc, "haste_hip_stream_status")


def workspace_bytes(time_steps, batch_size, input_size, hidden_size, half_gru=False):
    """Upper bound of the scratch memory any cell needs for these sizes on the current device
    (half_gru: the GRU on half tensors, which also stages fp32 copies of its tensors there)."""
    import ctypes
    handle = lib.load()
    fn = handle.haste_hip_gru_half_workspace_bytes if half_gru else handle.haste_hip_workspace_bytes
    fn.restype = ctypes.c_size_t
    fn.argtypes = [ctypes.c_int] * 4
    return int(fn(time_steps, batch_size, input_size, hidden_size))


def set_workspace(buffer, stream=None):
    """Lends the library `buffer` (a contiguous GPU tensor from torch's allocator, which the
    caller keeps alive and leaves alone) as the scratch memory of `stream` (default: the current
    stream); None takes it back.  With a lent buffer the ops allocate, free and synchronize
    nothing themselves, so they can be recorded into a HIP graph."""
    import ctypes
    handle = lib.load()
    if stream is None:
        stream = torch.cuda.current_stream().cuda_stream
    handle.haste_hip_set_workspace.restype = ctypes.c_int
    handle.haste_hip_set_workspace.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]
    if buffer is None:
        rc = handle.haste_hip_set_workspace(ctypes.c_void_p(stream), None, 0)
    else:
        if not (buffer.is_cuda and buffer.is_contiguous()):
            raise ValueError("the workspace must be a contiguous GPU tensor")
        rc = handle.haste_hip_set_workspace(ctypes.c_void_p(stream), ctypes.c_void_p(buffer.data_ptr()),
                                            buffer.numel() * buffer.element_size())
    if rc != 0:
        raise lib.HasteHipError(rc, "haste_hip_set_workspace")


def workspace_high_water(stream=None):
    """Bytes of scratch memory the calls made on `stream` so far have needed (what to lend for
    a replay of the same calls)."""
    import ctypes
    handle = lib.load()
    if stream is None:
        stream = torch.cuda.current_stream().cuda_stream
    out = ctypes.c_size_t(0)
    handle.haste_hip_workspace_high_water.restype = ctypes.c_int
    rc = handle.haste_hip_workspace_high_water(ctypes.c_void_p(stream), ctypes.byref(out))
    if rc != 0:
        raise lib.HasteHipError(rc, "haste_hip_workspace_high_water")
    return int(out.value)


def _zeros(opts, *shapes):
    """Zero tensors of the given shapes carved out of one allocation: one fill kernel for all
    the accumulated outputs of a backward pass (each starts on a 256-byte boundary)."""
    sizes = [int(torch.Size(shp).numel()) for shp in shapes]
    starts, total = [], 0
    for n in sizes:
        starts.append(total)
        total += (n + 63) // 64 * 64
    flat = torch.zeros(total, **opts)
    return [flat[a:a + n].view(shp) for a, n, shp in zip(starts, sizes, shapes)]


def _mask_or_none(has_zoneout, zoneout_mask):
    return zoneout_mask if has_zoneout else None


def gemm(a, b, out=None, trans_a=False, accumulate=False):
    """out[M,N] = op(a) @ b (+ out). a is [M,K], or [K,M] when trans_a."""
    _check(a, b)
    K, M = (a.shape if trans_a else (a.shape[1], a.shape[0]))
    N = b.shape[1]
    assert b.shape[0] == K
    if out is None:
        assert not accumulate
        out = torch.empty(M, N, device=a.device, dtype=a.dtype)
    _call("haste_hip_gemm", int(trans_a), M, N, K, a, a.stride(0), b, b.stride(0),
             out, out.stride(0), int(accumulate))
    return out


def transpose(a, out=None):
    """[rows, cols] -> [cols, rows] (a contiguous copy); leading dimensions of `a` beyond
    the last are folded into rows, so x[T,N,C] gives x_t[C,T,N]."""
    _check(a)
    cols = a.shape[-1]
    rows = a.numel() // cols
    if out is None:
        out = torch.empty((cols,) + tuple(a.shape[:-1]), device=a.device, dtype=a.dtype)
    _call("haste_hip_transpose", rows, cols, a, out)
    return out


def transpose3(a, b, c):
    """transpose() of three float32 tensors in one launch: the x_t, W_t, R_t a backward pass asks
    its caller for (reference frameworks/pytorch/lstm.py:84-86)."""
    outs = []
    args = []
    for m in (a, b, c):
        _check(m)
        if m.dtype != torch.float32:
            return transpose(a), transpose(b), transpose(c)
        cols = m.shape[-1]
        rows = m.numel() // cols
        out = torch.empty((cols,) + tuple(m.shape[:-1]), device=m.device, dtype=m.dtype)
        outs.append(out)
        args += [rows, cols, m, out]
    lib.call("haste_hip_transpose3_f32", *args)
    return tuple(outs)


# ---- LSTM (reference frameworks/pytorch/lstm.cc:31-157) ---------------------
def lstm_forward(training, zoneout_prob, x, h0, c0, kernel, recurrent_kernel, bias, zoneout_mask,
                 dropconnect_mask=None, dropconnect_scale=1.0):
    T, N, C = x.shape
    H = recurrent_kernel.shape[0]
    has_zoneout = bool(zoneout_prob) and zoneout_mask.numel() > 0
    _check(x, h0, c0, kernel, recurrent_kernel, bias, zoneout_mask)
    opts = dict(device=x.device, dtype=x.dtype)
    output = torch.empty(T + 1, N, H, **opts)
    output_state = torch.empty(T + 1, N, H, **opts)
    cache = torch.empty(T, N, 4 * H, **opts)
    torch._foreach_copy_([output[0], output_state[0]], [h0, c0])  # one kernel for both
    zp = float(zoneout_prob) if has_zoneout else 0.0
    mask = _mask_or_none(has_zoneout, zoneout_mask)
    if dropconnect_mask is None:
        _call("haste_hip_lstm_forward", bool(training), T, N, C, H, kernel, recurrent_kernel,
                 bias, x, output, output_state, cache, None, zp, mask)
    else:
        _check(dropconnect_mask)
        _call("haste_hip_lstm_forward_dropconnect", bool(training), T, N, C, H, kernel,
                 recurrent_kernel, bias, x, output, output_state, cache, zp, mask,
                 dropconnect_mask, float(dropconnect_scale))
    return output, output_state, cache


def lstm_backward(x_t, kernel_t, recurrent_kernel_t, bias, zoneout_mask, h, c, cache, dh_new, dc_new):
    C, T, N = x_t.shape
    H = recurrent_kernel_t.shape[1]
    has_zoneout = zoneout_mask.numel() > 0
    _check(x_t, kernel_t, recurrent_kernel_t, bias, zoneout_mask, h, c, cache, dh_new, dc_new)
    opts = dict(device=x_t.device, dtype=x_t.dtype)
    dx = torch.empty(T, N, C, **opts)
    dW, dR, db, dh, dc = _zeros(opts, (C, 4 * H), (H, 4 * H), (4 * H,), (N, H), (N, H))
    _call("haste_hip_lstm_backward", T, N, C, H, kernel_t, recurrent_kernel_t, bias, x_t,
             h, c, dh_new, dc_new, dx, dW, dR, db, dh, dc, cache,
             _mask_or_none(has_zoneout, zoneout_mask))
    return dx, dh, dc, dW, dR, db


# ---- single LSTM steps (reference lib/haste/lstm.h:73-86,201-219; no binding of the
# reference exposes them, examples/lstm.cc:252,309 calls them from C++) ------------------
def lstm_forward_iterate(training, zoneout_prob, x, h, c, kernel, recurrent_kernel, bias,
                         zoneout_mask=None, h_out=None, c_out=None):
    """One step: x[N,C], h,c[N,H] -> h_out,c_out[N,H], v[N,4H] (activations when training)."""
    N, C = x.shape
    H = recurrent_kernel.shape[0]
    _check(x, h, c, kernel, recurrent_kernel, bias)
    h_out = torch.empty_like(h) if h_out is None else h_out
    c_out = torch.empty_like(c) if c_out is None else c_out
    v = torch.empty(N, 4 * H, device=x.device, dtype=x.dtype)
    has_zoneout = bool(zoneout_prob) and zoneout_mask is not None and zoneout_mask.numel() > 0
    _call("haste_hip_lstm_forward_iterate", bool(training), N, C, H, kernel, recurrent_kernel,
             bias, x, h, c, h_out, c_out, v, None, float(zoneout_prob) if has_zoneout else 0.0,
             zoneout_mask if has_zoneout else None)
    return h_out, c_out, v


def lstm_backward_iterate(x_t, kernel_t, recurrent_kernel_t, bias, h, c, c_new, dh_new, dc_new, v,
                          dW, dR, db, dh, dc, zoneout_mask=None):
    """One reverse step: x_t[C,N]; h,c = states before the step, c_new = cell state after it;
    dW, dR, db are accumulated into, dh, dc updated in place, v consumed.  Returns dx[N,C]."""
    C, N = x_t.shape
    H = recurrent_kernel_t.shape[1]
    _check(x_t, kernel_t, recurrent_kernel_t, bias, h, c, c_new, dh_new, dc_new, v, dW, dR, db, dh, dc)
    dx = torch.empty(N, C, device=x_t.device, dtype=x_t.dtype)
    has_zoneout = zoneout_mask is not None and zoneout_mask.numel() > 0
    _call("haste_hip_lstm_backward_iterate", N, C, H, kernel_t, recurrent_kernel_t, bias, x_t,
             h, c, c_new, dh_new, dc_new, dx, dW, dR, db, dh, dc, v,
             zoneout_mask if has_zoneout else None)
    return dx


# ---- single GRU steps (reference lib/haste/gru.h:72-84,172-189) -------------------------
def gru_forward_iterate(training, zoneout_prob, x, h, kernel, recurrent_kernel, bias,
                        recurrent_bias, zoneout_mask=None, h_out=None):
    N, C = x.shape
    H = recurrent_kernel.shape[0]
    _check(x, h, kernel, recurrent_kernel, bias, recurrent_bias)
    h_out = torch.empty_like(h) if h_out is None else h_out
    v = torch.empty(N, 4 * H, device=x.device, dtype=x.dtype)
    tmp_Wx = torch.empty(N, 3 * H, device=x.device, dtype=x.dtype)
    has_zoneout = bool(zoneout_prob) and zoneout_mask is not None and zoneout_mask.numel() > 0
    _call("haste_hip_gru_forward_iterate", bool(training), N, C, H, kernel, recurrent_kernel,
             bias, recurrent_bias, x, h, h_out, v, tmp_Wx, None,
             float(zoneout_prob) if has_zoneout else 0.0, zoneout_mask if has_zoneout else None)
    return h_out, v


def gru_backward_iterate(x_t, kernel_t, recurrent_kernel_t, bias, recurrent_bias, h, v, dh_new,
                         dW, dR, dbx, dbr, dh, zoneout_mask=None):
    C, N = x_t.shape
    H = recurrent_kernel_t.shape[1]
    _check(x_t, kernel_t, recurrent_kernel_t, bias, recurrent_bias, h, v, dh_new, dW, dR, dbx, dbr, dh)
    opts = dict(device=x_t.device, dtype=x_t.dtype)
    dx = torch.empty(N, C, **opts)
    dp = torch.empty(N, 3 * H, **opts)
    dq = torch.empty(N, 3 * H, **opts)
    has_zoneout = zoneout_mask is not None and zoneout_mask.numel() > 0
    _call("haste_hip_gru_backward_iterate", N, C, H, kernel_t, recurrent_kernel_t, bias,
             recurrent_bias, x_t, h, v, dh_new, dx, dW, dR, dbx, dbr, dh, dp, dq,
             zoneout_mask if has_zoneout else None)
    return dx


# ---- GRU (reference frameworks/pytorch/gru.cc:30-163) -----------------------
def gru_forward(training, zoneout_prob, x, h0, kernel, recurrent_kernel, bias, recurrent_bias,
                zoneout_mask, dropconnect_mask=None, dropconnect_scale=1.0):
    T, N, C = x.shape
    H = recurrent_kernel.shape[0]
    has_zoneout = bool(zoneout_prob) and zoneout_mask.numel() > 0
    _check(x, h0, kernel, recurrent_kernel, bias, recurrent_bias, zoneout_mask)
    opts = dict(device=x.device, dtype=x.dtype)
    output = torch.empty(T + 1, N, H, **opts)
    cache = torch.empty(T, N, 4 * H, **opts)
    tmp_Wx = torch.empty(T, N, 3 * H, **opts)
    output[0] = h0
    zp = float(zoneout_prob) if has_zoneout else 0.0
    mask = _mask_or_none(has_zoneout, zoneout_mask)
    if dropconnect_mask is None:
        _call("haste_hip_gru_forward", bool(training), T, N, C, H, kernel, recurrent_kernel,
                 bias, recurrent_bias, x, output, cache if training else None, tmp_Wx, None, zp, mask)
    else:
        _check(dropconnect_mask)
        _call("haste_hip_gru_forward_dropconnect", bool(training), T, N, C, H, kernel,
                 recurrent_kernel, bias, recurrent_bias, x, output, cache if training else None,
                 tmp_Wx, zp, mask, dropconnect_mask, float(dropconnect_scale))
    return output, cache


def gru_backward(x_t, kernel_t, recurrent_kernel_t, bias, recurrent_bias, zoneout_mask, h, cache,
                 dh_new):
    C, T, N = x_t.shape
    H = recurrent_kernel_t.shape[1]
    has_zoneout = zoneout_mask.numel() > 0
    _check(x_t, kernel_t, recurrent_kernel_t, bias, recurrent_bias, zoneout_mask, h, cache, dh_new)
    opts = dict(device=x_t.device, dtype=x_t.dtype)
    dx = torch.empty(T, N, C, **opts)
    dW, dR, dbx, dbr, dh = _zeros(opts, (C, 3 * H), (H, 3 * H), (3 * H,), (3 * H,), (N, H))
    dp = torch.empty(T, N, 3 * H, **opts)
    dq = torch.empty(T, N, 3 * H, **opts)
    _call("haste_hip_gru_backward", T, N, C, H, kernel_t, recurrent_kernel_t, bias,
             recurrent_bias, x_t, h, cache, dh_new, dx, dW, dR, dbx, dbr, dh, dp, dq,
             _mask_or_none(has_zoneout, zoneout_mask))
    return dx, dh, dW, dR, dbx, dbr


# ---- Layer norm (reference lib/haste/layer_norm.h) ---------------------------
def layer_norm_forward(x, gamma, beta=None):
    _check(x, gamma)
    rows, dim = x.numel() // x.shape[-1], x.shape[-1]
    y = torch.empty_like(x)
    cache = torch.empty(rows, 2, device=x.device, dtype=x.dtype)
    _call("haste_hip_layer_norm_forward", rows, dim, gamma, beta, x, y, cache)
    return y, cache


def layer_norm_backward(x, gamma, dy, cache=None, with_beta=True, in_place=False):
    _check(x, gamma, dy)
    rows, dim = x.numel() // x.shape[-1], x.shape[-1]
    dx = dy if in_place else torch.empty_like(x)
    dgamma = torch.zeros_like(gamma)
    dbeta = torch.zeros_like(gamma) if with_beta else None
    _call("haste_hip_layer_norm_backward", rows, dim, gamma, x, dy, dx, dgamma, dbeta, cache)
    return dx, dgamma, dbeta


# ---- IndRNN (reference frameworks/pytorch/indrnn.cc:30-140) -------------------
def indrnn_forward(training, zoneout_prob, x, h0, kernel, recurrent_scale, bias, zoneout_mask):
    T, N, C = x.shape
    H = recurrent_scale.shape[0]
    has_zoneout = bool(zoneout_prob) and zoneout_mask.numel() > 0
    _check(x, h0, kernel, recurrent_scale, bias, zoneout_mask)
    opts = dict(device=x.device, dtype=x.dtype)
    output = torch.empty(T + 1, N, H, **opts)
    workspace = torch.empty(T, N, H, **opts)
    output[0] = h0
    _call("haste_hip_indrnn_forward", bool(training), T, N, C, H, kernel, recurrent_scale,
             bias, x, output, workspace, float(zoneout_prob) if has_zoneout else 0.0,
             _mask_or_none(has_zoneout, zoneout_mask))
    return output


def indrnn_backward(x_t, kernel_t, recurrent_scale, bias, zoneout_mask, h, dh_new):
    C, T, N = x_t.shape
    H = recurrent_scale.shape[0]
    has_zoneout = zoneout_mask.numel() > 0
    _check(x_t, kernel_t, recurrent_scale, bias, zoneout_mask, h, dh_new)
    opts = dict(device=x_t.device, dtype=x_t.dtype)
    dx = torch.empty(T, N, C, **opts)
    dW, du, db, dh = _zeros(opts, (C, H), (H,), (H,), (N, H))
    workspace = torch.empty(T, N, H, **opts)
    _call("haste_hip_indrnn_backward", T, N, C, H, kernel_t, recurrent_scale, bias, x_t, h,
             dh_new, dx, dW, du, db, dh, workspace, _mask_or_none(has_zoneout, zoneout_mask))
    return dx, dh, dW, du, db


# ---- LayerNorm IndRNN (reference frameworks/pytorch/layer_norm_indrnn.cc:31-174) ----
def layer_norm_indrnn_forward(training, zoneout_prob, x, h0, kernel, recurrent_scale, bias, gamma,
                              zoneout_mask):
    T, N, C = x.shape
    H = recurrent_scale.shape[0]
    has_zoneout = bool(zoneout_prob) and zoneout_mask.numel() > 0
    _check(x, h0, kernel, recurrent_scale, bias, gamma, zoneout_mask)
    opts = dict(device=x.device, dtype=x.dtype)
    output = torch.empty(T + 1, N, H, **opts)
    workspace = torch.empty(T, N, H, **opts)
    act_Wx = torch.empty(T, N, H, **opts)
    act_Wx_norm_cache = torch.empty(T, N, 2, **opts)
    output[0] = h0
    _call("haste_hip_layer_norm_indrnn_forward", bool(training), T, N, C, H, kernel,
             recurrent_scale, bias, x, output, workspace, act_Wx, gamma[0], act_Wx_norm_cache,
             float(zoneout_prob) if has_zoneout else 0.0, _mask_or_none(has_zoneout, zoneout_mask))
    return output, act_Wx, act_Wx_norm_cache


def layer_norm_indrnn_backward(x_t, kernel_t, recurrent_scale, bias, gamma, zoneout_mask, h, act_Wx,
                               act_Wx_norm_cache, dh_new):
    C, T, N = x_t.shape
    H = recurrent_scale.shape[0]
    has_zoneout = zoneout_mask.numel() > 0
    _check(x_t, kernel_t, recurrent_scale, bias, gamma, zoneout_mask, h, act_Wx, dh_new)
    opts = dict(device=x_t.device, dtype=x_t.dtype)
    dx = torch.empty(T, N, C, **opts)
    dW, du, db, dh = _zeros(opts, (C, H), (H,), (H,), (N, H))
    workspace = torch.empty(T, N, H, **opts)
    dgamma = torch.zeros_like(gamma)
    _call("haste_hip_layer_norm_indrnn_backward", T, N, C, H, kernel_t, recurrent_scale, bias,
             x_t, h, dh_new, dx, dW, du, db, dh, workspace, act_Wx, gamma[0], dgamma[0],
             _mask_or_none(has_zoneout, zoneout_mask))
    return dx, dh, dW, du, db, dgamma


# ---- LayerNorm LSTM (reference frameworks/pytorch/layer_norm_lstm.cc:31-297) ---------
def layer_norm_lstm_forward(training, zoneout_prob, x, h0, c0, kernel, recurrent_kernel, bias,
                            gamma, gamma_h, beta_h, zoneout_mask):
    T, N, C = x.shape
    H = recurrent_kernel.shape[0]
    has_zoneout = bool(zoneout_prob) and zoneout_mask.numel() > 0
    _check(x, h0, c0, kernel, recurrent_kernel, bias, gamma, gamma_h, beta_h, zoneout_mask)
    opts = dict(device=x.device, dtype=x.dtype)
    output = torch.empty(T + 1, N, H, **opts)
    output_state = torch.empty(T + 1, N, H, **opts)
    act_Wx = torch.empty(T, N, 4 * H, **opts)
    act_Wx_norm = torch.empty(T, N, 4 * H, **opts)
    act_Wx_norm_cache = torch.empty(T, N, 2, **opts)
    act_Rh = torch.empty(T, N, 4 * H, **opts)
    act_Rh_norm_cache = torch.empty(T, N, 2, **opts)
    act_c_norm = torch.empty(T, N, H, **opts)
    act_c_norm_cache = torch.empty(T, N, 2, **opts)
    output[0] = h0
    output_state[0] = c0
    _call("haste_hip_layer_norm_lstm_forward", bool(training), T, N, C, H, kernel,
             recurrent_kernel, bias, x, output, output_state, act_Wx, None,
             gamma[0], act_Wx_norm_cache, act_Wx_norm, act_Rh, gamma[1], act_Rh_norm_cache,
             gamma_h, beta_h, act_c_norm_cache, act_c_norm,
             float(zoneout_prob) if has_zoneout else 0.0, _mask_or_none(has_zoneout, zoneout_mask))
    return (output, output_state, act_Wx, act_Wx_norm, act_Wx_norm_cache, act_Rh, act_Rh_norm_cache,
            act_c_norm, act_c_norm_cache)


def layer_norm_lstm_backward(x_t, kernel_t, recurrent_kernel_t, bias, gamma, gamma_h, beta_h,
                             zoneout_mask, h, c, act_Wx, act_Wx_norm, act_Wx_norm_cache, act_Rh,
                             act_Rh_norm_cache, act_c_norm, act_c_norm_cache, dh_new, dc_new):
    C, T, N = x_t.shape
    H = recurrent_kernel_t.shape[1]
    has_zoneout = zoneout_mask.numel() > 0
    _check(x_t, kernel_t, recurrent_kernel_t, bias, gamma, gamma_h, beta_h, zoneout_mask, h, c,
           act_Wx, act_Wx_norm, act_Wx_norm_cache, act_Rh, act_Rh_norm_cache, act_c_norm,
           act_c_norm_cache, dh_new, dc_new)
    opts = dict(device=x_t.device, dtype=x_t.dtype)
    dx = torch.empty(T, N, C, **opts)
    dW, dR, db, dgamma, dgamma_h, dbeta_h, dh, dc = _zeros(
        opts, (C, 4 * H), (H, 4 * H), (4 * H,), tuple(gamma.shape), (H,), (H,), (N, H), (N, H))
    _call("haste_hip_layer_norm_lstm_backward", T, N, C, H, kernel_t, recurrent_kernel_t,
             bias, x_t, h, c, dh_new, dc_new, dx, dW, dR, db, dh, dc,
             act_Wx, gamma[0], dgamma[0], act_Wx_norm, act_Rh, gamma[1], dgamma[1],
             act_Rh_norm_cache, gamma_h, beta_h, dgamma_h, dbeta_h, act_c_norm_cache, act_c_norm,
             _mask_or_none(has_zoneout, zoneout_mask))
    return dx, dh, dc, dW, dR, db, dgamma, dgamma_h, dbeta_h


# ---- LayerNorm GRU (reference frameworks/pytorch/layer_norm_gru.cc:30-230) -----------
def layer_norm_gru_forward(training, zoneout_prob, x, h0, kernel, recurrent_kernel, bias,
                           recurrent_bias, gamma, zoneout_mask):
    T, N, C = x.shape
    H = recurrent_kernel.shape[0]
    has_zoneout = bool(zoneout_prob) and zoneout_mask.numel() > 0
    _check(x, h0, kernel, recurrent_kernel, bias, recurrent_bias, gamma, zoneout_mask)
    opts = dict(device=x.device, dtype=x.dtype)
    output = torch.empty(T + 1, N, H, **opts)
    cache = torch.empty(T, N, 4 * H, **opts)
    act_Wx = torch.empty(T, N, 3 * H, **opts)
    tmp_Wx_norm = torch.empty(T, N, 3 * H, **opts)
    act_Wx_norm_cache = torch.empty(T, N, 2, **opts)
    act_Rh = torch.empty(T, N, 3 * H, **opts)
    act_Rh_norm_cache = torch.empty(T, N, 2, **opts)
    output[0] = h0
    _call("haste_hip_layer_norm_gru_forward", bool(training), T, N, C, H, kernel,
             recurrent_kernel, bias, recurrent_bias, x, output, cache if training else None,
             act_Wx, gamma[0], act_Wx_norm_cache, tmp_Wx_norm, act_Rh, gamma[1], act_Rh_norm_cache,
             None, float(zoneout_prob) if has_zoneout else 0.0,
             _mask_or_none(has_zoneout, zoneout_mask))
    return output, cache, act_Wx, act_Wx_norm_cache, act_Rh, act_Rh_norm_cache


def layer_norm_gru_backward(x_t, kernel_t, recurrent_kernel_t, bias, recurrent_bias, gamma,
                            zoneout_mask, h, cache, act_Wx, act_Wx_norm_cache, act_Rh,
                            act_Rh_norm_cache, dh_new):
    C, T, N = x_t.shape
    H = recurrent_kernel_t.shape[1]
    has_zoneout = zoneout_mask.numel() > 0
    _check(x_t, kernel_t, recurrent_kernel_t, bias, recurrent_bias, gamma, zoneout_mask, h, cache,
           act_Wx, act_Wx_norm_cache, act_Rh, act_Rh_norm_cache, dh_new)
    opts = dict(device=x_t.device, dtype=x_t.dtype)
    dx = torch.empty(T, N, C, **opts)
    dW, dR, dbx, dbr, dh, dgamma = _zeros(opts, (C, 3 * H), (H, 3 * H), (3 * H,), (3 * H,), (N, H),
                                          tuple(gamma.shape))
    dp = torch.empty(T, N, 3 * H, **opts)
    dq = torch.empty(T, N, 3 * H, **opts)
    _call("haste_hip_layer_norm_gru_backward", T, N, C, H, kernel_t, recurrent_kernel_t, bias,
             recurrent_bias, x_t, h, cache, dh_new, dx, dW, dR, dbx, dbr, dh, dp, dq,
             act_Wx, gamma[0], dgamma[0], act_Rh, gamma[1], dgamma[1], act_Rh_norm_cache,
             _mask_or_none(has_zoneout, zoneout_mask))
    return dx, dh, dW, dR, dbx, dbr, dgamma
