"""CPU oracle for the fused-RNN hot path (TEST INFRASTRUCTURE, not product code).

A NumPy restatement, in float64 by default, of the arithmetic that the
reference's `ForwardPass<T>::Run` / `BackwardPass<T>::Run` perform for the
lstm, gru, layer_norm, layer_norm_lstm, layer_norm_gru, indrnn and
layer_norm_indrnn cells.  Only tests, the smoke check and the CPU-baseline leg
of the benchmark may import this module; the shipped library never does.

Conventions (reference `lib/haste.h:18-26`): T steps, N batch, C input size,
H hidden size; arrays are row-major with the rightmost index fastest.  Gate
blocks are contiguous column ranges of width H: LSTM `i,g,f,o`, GRU `z,r,g`.
The backward functions take the *untransposed* x, W, R (the reference takes
caller-made transposes; the transposition is layout, not arithmetic).

How each function is pinned (see tests/test_oracle_*.py):
  lstm_forward/backward      torch.nn.LSTM + autograd via the native-weight map
                             (reference frameworks/pytorch/lstm.py:159-201)
  gru_forward/backward       torch.nn.GRU + autograd (frameworks/pytorch/gru.py:161-208)
  layer_norm_forward/backward  torch.nn.functional.layer_norm + autograd
  layer_norm_lstm_*, layer_norm_gru_*, indrnn_*, layer_norm_indrnn_*, zoneout
                             autograd of a forward assembled from library
                             pieces (F.layer_norm, torch.sigmoid/tanh, matmul),
                             fp64 central finite differences on tiny shapes,
                             and the mask==1 / mask==0 / T==1 invariants.
"""
import numpy as np

LN_EPS = 1e-5  # reference lib/layer_norm_forward_gpu.cu.cc:77


def sigmoid(x):
    # reference lib/inline_ops.h:22-24
    return 1.0 / (1.0 + np.exp(-x))


def d_sigmoid(y):
    # reference lib/inline_ops.h:34-36 (derivative expressed in the output)
    return y * (1.0 - y)


def d_tanh(y):
    # reference lib/inline_ops.h:40-42
    return 1.0 - y * y


def _zoneout_forward(h_new, h_old, training, zoneout_prob, mask_t):
    # reference lib/lstm_forward_gpu.cu.cc:77-83 (identical in every cell)
    if zoneout_prob and mask_t is not None:
        if training:
            return (h_new - h_old) * mask_t + h_old
        return zoneout_prob * h_old + (1.0 - zoneout_prob) * h_new
    return h_new


# --------------------------------------------------------------------------
# Layer norm
# --------------------------------------------------------------------------
def layer_norm_forward(x, gamma, beta=None):
    """Row-wise layer norm over the last dim, biased variance, eps 1e-5.

    reference lib/layer_norm_forward_gpu.cu.cc:45-87.
    Returns (y, cache) with cache[..., 0] = mean, cache[..., 1] = invstd.
    """
    mean = x.mean(axis=-1, keepdims=True)
    xc = x - mean
    var = (xc * xc).mean(axis=-1, keepdims=True)
    invstd = 1.0 / np.sqrt(var + LN_EPS)
    y = xc * invstd * gamma
    if beta is not None:
        y = y + beta
    cache = np.concatenate([mean, invstd], axis=-1)
    return y, cache


def layer_norm_backward(x, gamma, dy, cache=None):
    """reference lib/layer_norm_backward_gpu.cu.cc:46-92.

    Returns (dx, dgamma, dbeta); dgamma/dbeta are the sums over all rows.
    """
    D = x.shape[-1]
    if cache is None:
        _, cache = layer_norm_forward(x, gamma)
    mean = cache[..., 0:1]
    invstd = cache[..., 1:2]
    xc = x - mean
    z = xc * invstd
    red = tuple(range(x.ndim - 1))
    dgamma = (z * dy).sum(axis=red)
    dbeta = dy.sum(axis=red)
    db = gamma * dy
    s0 = (xc * db).sum(axis=-1, keepdims=True)
    s1 = xc.sum(axis=-1, keepdims=True)
    s2 = db.sum(axis=-1, keepdims=True)
    dsigma = -0.5 * s0 * invstd * invstd * invstd
    dmu = (-2.0 * s1 * dsigma / D) - (s2 * invstd)
    dx = (2.0 * xc * dsigma / D) + (invstd * db) + (dmu / D)
    return dx, dgamma, dbeta


# --------------------------------------------------------------------------
# LSTM
# --------------------------------------------------------------------------
def lstm_forward(W, R, b, x, h0, c0, training=True, zoneout_prob=0.0, zoneout_mask=None):
    """reference lib/lstm_forward_gpu.cu.cc:55-86 (pointwise) and :313-366 (Run).

    Returns h[T+1,N,H], c[T+1,N,H], v[T,N,4H] (post-activation i,g,f,o).
    """
    T, N, _ = x.shape
    H = R.shape[0]
    dt = x.dtype
    h = np.zeros((T + 1, N, H), dt)
    c = np.zeros((T + 1, N, H), dt)
    v = np.zeros((T, N, 4 * H), dt)
    h[0], c[0] = h0, c0
    Wx = x.reshape(T * N, -1) @ W
    Wx = Wx.reshape(T, N, 4 * H)
    for t in range(T):
        a = Wx[t] + h[t] @ R + b
        i = sigmoid(a[:, 0 * H:1 * H])
        g = np.tanh(a[:, 1 * H:2 * H])
        f = sigmoid(a[:, 2 * H:3 * H])
        o = sigmoid(a[:, 3 * H:4 * H])
        v[t] = np.concatenate([i, g, f, o], axis=1)
        c[t + 1] = f * c[t] + i * g
        hn = o * np.tanh(c[t + 1])
        mt = zoneout_mask[t] if zoneout_mask is not None else None
        h[t + 1] = _zoneout_forward(hn, h[t], training, zoneout_prob, mt)
    return h, c, v


def lstm_backward(W, R, b, x, h, c, v, dh_new, dc_new, zoneout_mask=None):
    """reference lib/lstm_backward_gpu.cu.cc:47-95 (pointwise) and :319-405 (Run).

    dh_new, dc_new: [T+1,N,H]; slot 0 is never read (reference :362-363).
    Returns dx, dW, dR, db, dh0, dc0 and dv[T,N,4H] (what the reference leaves in `v`).
    """
    T, N, _ = x.shape
    H = R.shape[0]
    dt = x.dtype
    dh = np.zeros((N, H), dt)
    dc = np.zeros((N, H), dt)
    dv = np.zeros((T, N, 4 * H), dt)
    for t in range(T - 1, -1, -1):
        i = v[t][:, 0 * H:1 * H]
        g = v[t][:, 1 * H:2 * H]
        f = v[t][:, 2 * H:3 * H]
        o = v[t][:, 3 * H:4 * H]
        dc_total = dc_new[t + 1] + dc
        dh_total = dh_new[t + 1] + dh
        c_tanh = np.tanh(c[t + 1])
        if zoneout_mask is not None:
            m = zoneout_mask[t]
            dh = (1.0 - m) * dh_total
            dh_total = m * dh_total
        else:
            dh = np.zeros((N, H), dt)
        do_ = c_tanh * dh_total
        dc_tanh = o * dh_total
        dc_total = dc_total + d_tanh(c_tanh) * dc_tanh
        df = c[t] * dc_total
        dc = f * dc_total
        di = g * dc_total
        dg = i * dc_total
        dv[t] = np.concatenate(
            [d_sigmoid(i) * di, d_tanh(g) * dg, d_sigmoid(f) * df, d_sigmoid(o) * do_], axis=1)
        dh = dh + dv[t] @ R.T
    dvf = dv.reshape(T * N, 4 * H)
    db = dvf.sum(axis=0)
    dW = x.reshape(T * N, -1).T @ dvf
    dR = h[:T].reshape(T * N, H).T @ dvf
    dx = (dvf @ W.T).reshape(x.shape)
    return dx, dW, dR, db, dh, dc, dv


# --------------------------------------------------------------------------
# GRU
# --------------------------------------------------------------------------
def gru_forward(W, R, bx, br, x, h0, training=True, zoneout_prob=0.0, zoneout_mask=None):
    """reference lib/gru_forward_gpu.cu.cc:46-84 and :314-371.

    Returns h[T+1,N,H], v[T,N,4H] = (z, r, g, Rh_g + br_g).
    """
    T, N, _ = x.shape
    H = R.shape[0]
    dt = x.dtype
    h = np.zeros((T + 1, N, H), dt)
    v = np.zeros((T, N, 4 * H), dt)
    h[0] = h0
    Wx = (x.reshape(T * N, -1) @ W).reshape(T, N, 3 * H)
    for t in range(T):
        Rh = h[t] @ R
        z = sigmoid(Wx[t][:, 0:H] + Rh[:, 0:H] + bx[0:H] + br[0:H])
        r = sigmoid(Wx[t][:, H:2 * H] + Rh[:, H:2 * H] + bx[H:2 * H] + br[H:2 * H])
        qg = Rh[:, 2 * H:] + br[2 * H:]
        g = np.tanh(Wx[t][:, 2 * H:] + r * qg + bx[2 * H:])
        v[t] = np.concatenate([z, r, g, qg], axis=1)
        hn = z * h[t] + (1.0 - z) * g
        mt = zoneout_mask[t] if zoneout_mask is not None else None
        h[t + 1] = _zoneout_forward(hn, h[t], training, zoneout_prob, mt)
    return h, v


def _gru_pointwise_backward(h_t, v_t, dh_total, m, H):
    # reference lib/gru_backward_gpu.cu.cc:45-95
    z = v_t[:, 0:H]
    r = v_t[:, H:2 * H]
    g = v_t[:, 2 * H:3 * H]
    qg = v_t[:, 3 * H:4 * H]
    if m is not None:
        dh = (1.0 - m) * dh_total
        dh_total = m * dh_total
        dh = dh + z * dh_total
    else:
        dh = z * dh_total
    dg = (1.0 - z) * dh_total
    dz = (h_t - g) * dh_total
    dp_g = d_tanh(g) * dg
    dq_g = dp_g * r
    dr = dp_g * qg
    dp_r = d_sigmoid(r) * dr
    dp_z = d_sigmoid(z) * dz
    dp = np.concatenate([dp_z, dp_r, dp_g], axis=1)
    dq = np.concatenate([dp_z, dp_r, dq_g], axis=1)
    return dp, dq, dh


def gru_backward(W, R, bx, br, x, h, v, dh_new, zoneout_mask=None):
    """reference lib/gru_backward_gpu.cu.cc:45-95 and :321-409.

    Returns dx, dW, dR, dbx, dbr, dh0, dp[T,N,3H], dq[T,N,3H].
    """
    T, N, _ = x.shape
    H = R.shape[0]
    dt = x.dtype
    dh = np.zeros((N, H), dt)
    dp = np.zeros((T, N, 3 * H), dt)
    dq = np.zeros((T, N, 3 * H), dt)
    for t in range(T - 1, -1, -1):
        m = zoneout_mask[t] if zoneout_mask is not None else None
        dp[t], dq[t], dh = _gru_pointwise_backward(h[t], v[t], dh_new[t + 1] + dh, m, H)
        dh = dh + dq[t] @ R.T
    dpf = dp.reshape(T * N, 3 * H)
    dqf = dq.reshape(T * N, 3 * H)
    dbx = dpf.sum(axis=0)
    dbr = dqf.sum(axis=0)
    dx = (dpf @ W.T).reshape(x.shape)
    dW = x.reshape(T * N, -1).T @ dpf
    dR = h[:T].reshape(T * N, H).T @ dqf
    return dx, dW, dR, dbx, dbr, dh, dp, dq


# --------------------------------------------------------------------------
# LayerNorm LSTM
# --------------------------------------------------------------------------
def layer_norm_lstm_forward(W, R, b, gamma, gamma_h, beta_h, x, h0, c0,
                            training=True, zoneout_prob=0.0, zoneout_mask=None):
    """reference lib/layer_norm_lstm_forward_gpu.cu.cc:50-71,95-108 and :276-340.

    gamma: [2,4H] (row 0 scales LN(xW), row 1 scales LN(hR)); gamma_h, beta_h: [H].
    Returns a dict with h, c, act_Wx, act_Wx_norm_out (post-activation gates in
    training), act_Rh (pre-norm hR for every step), act_c_norm, and the three
    (mean, invstd) caches.
    """
    T, N, _ = x.shape
    H = R.shape[0]
    dt = x.dtype
    h = np.zeros((T + 1, N, H), dt)
    c = np.zeros((T + 1, N, H), dt)
    h[0], c[0] = h0, c0
    act_Wx = (x.reshape(T * N, -1) @ W).reshape(T, N, 4 * H)
    act_Wx_norm, cache1 = layer_norm_forward(act_Wx, gamma[0])
    act_Rh = np.zeros((T, N, 4 * H), dt)
    cache2 = np.zeros((T, N, 2), dt)
    act_c_norm = np.zeros((T, N, H), dt)
    cache3 = np.zeros((T, N, 2), dt)
    v = np.zeros((T, N, 4 * H), dt)
    for t in range(T):
        act_Rh[t] = h[t] @ R
        rh_norm, cache2[t] = layer_norm_forward(act_Rh[t], gamma[1])
        a = act_Wx_norm[t] + rh_norm + b
        i = sigmoid(a[:, 0 * H:1 * H])
        g = np.tanh(a[:, 1 * H:2 * H])
        f = sigmoid(a[:, 2 * H:3 * H])
        o = sigmoid(a[:, 3 * H:4 * H])
        v[t] = np.concatenate([i, g, f, o], axis=1)
        c[t + 1] = f * c[t] + i * g
        act_c_norm[t], cache3[t] = layer_norm_forward(c[t + 1], gamma_h, beta_h)
        hn = o * np.tanh(act_c_norm[t])
        mt = zoneout_mask[t] if zoneout_mask is not None else None
        h[t + 1] = _zoneout_forward(hn, h[t], training, zoneout_prob, mt)
    return dict(h=h, c=c, act_Wx=act_Wx, v=v, act_Rh=act_Rh, act_c_norm=act_c_norm,
                cache1=cache1, cache2=cache2, cache3=cache3)


def layer_norm_lstm_backward(W, R, b, gamma, gamma_h, beta_h, x, fwd, dh_new, dc_new,
                             zoneout_mask=None):
    """reference lib/layer_norm_lstm_backward_gpu.cu.cc:44-64,84-117 and :255-352.

    `fwd` is the dict returned by layer_norm_lstm_forward.
    Returns dict(dx,dW,dR,db,dh0,dc0,dgamma[2,4H],dgamma_h,dbeta_h).
    """
    T, N, _ = x.shape
    H = R.shape[0]
    dt = x.dtype
    h, c, v = fwd["h"], fwd["c"], fwd["v"]
    act_Wx, act_Rh, act_c_norm = fwd["act_Wx"], fwd["act_Rh"], fwd["act_c_norm"]
    dh = np.zeros((N, H), dt)
    dc = np.zeros((N, H), dt)
    dv = np.zeros((T, N, 4 * H), dt)
    dRh = np.zeros((T, N, 4 * H), dt)
    dgamma = np.zeros((2, 4 * H), dt)
    dgamma_h = np.zeros(H, dt)
    dbeta_h = np.zeros(H, dt)
    for t in range(T - 1, -1, -1):
        i = v[t][:, 0 * H:1 * H]
        g = v[t][:, 1 * H:2 * H]
        f = v[t][:, 2 * H:3 * H]
        o = v[t][:, 3 * H:4 * H]
        dh_total = dh_new[t + 1] + dh
        if zoneout_mask is not None:
            m = zoneout_mask[t]
            dh = (1.0 - m) * dh_total
            dh_total = m * dh_total
        else:
            dh = np.zeros((N, H), dt)
        c_tanh = np.tanh(act_c_norm[t])
        do_ = c_tanh * dh_total
        dln3 = d_tanh(c_tanh) * (o * dh_total)
        dv_o = d_sigmoid(o) * do_
        dc_ln, dgh, dbh = layer_norm_backward(c[t + 1], gamma_h, dln3, fwd["cache3"][t])
        dgamma_h += dgh
        dbeta_h += dbh
        dc_total = dc_new[t + 1] + dc + dc_ln
        df = c[t] * dc_total
        dc = f * dc_total
        di = g * dc_total
        dg = i * dc_total
        dv[t] = np.concatenate(
            [d_sigmoid(i) * di, d_tanh(g) * dg, d_sigmoid(f) * df, dv_o], axis=1)
        dRh[t], dg1, _ = layer_norm_backward(act_Rh[t], gamma[1], dv[t], fwd["cache2"][t])
        dgamma[1] += dg1
        dh = dh + dRh[t] @ R.T
    dWx, dg0, _ = layer_norm_backward(act_Wx, gamma[0], dv, fwd["cache1"])
    dgamma[0] += dg0
    dvf = dv.reshape(T * N, 4 * H)
    dWxf = dWx.reshape(T * N, 4 * H)
    dRhf = dRh.reshape(T * N, 4 * H)
    db = dvf.sum(axis=0)
    dW = x.reshape(T * N, -1).T @ dWxf
    dR = h[:T].reshape(T * N, H).T @ dRhf
    dx = (dWxf @ W.T).reshape(x.shape)
    return dict(dx=dx, dW=dW, dR=dR, db=db, dh0=dh, dc0=dc, dgamma=dgamma,
                dgamma_h=dgamma_h, dbeta_h=dbeta_h, dv=dv, dRh=dRh, dWx=dWx)


# --------------------------------------------------------------------------
# LayerNorm GRU
# --------------------------------------------------------------------------
def layer_norm_gru_forward(W, R, bx, br, gamma, x, h0,
                           training=True, zoneout_prob=0.0, zoneout_mask=None):
    """reference lib/layer_norm_gru_forward_gpu.cu.cc:25-83 and :242-305.

    gamma: [2,3H]. Biases are added after the norms.
    """
    T, N, _ = x.shape
    H = R.shape[0]
    dt = x.dtype
    h = np.zeros((T + 1, N, H), dt)
    v = np.zeros((T, N, 4 * H), dt)
    h[0] = h0
    act_Wx = (x.reshape(T * N, -1) @ W).reshape(T, N, 3 * H)
    Wx_norm, cache1 = layer_norm_forward(act_Wx, gamma[0])
    act_Rh = np.zeros((T, N, 3 * H), dt)
    cache2 = np.zeros((T, N, 2), dt)
    for t in range(T):
        act_Rh[t] = h[t] @ R
        Rh, cache2[t] = layer_norm_forward(act_Rh[t], gamma[1])
        Wxt = Wx_norm[t]
        z = sigmoid(Wxt[:, 0:H] + Rh[:, 0:H] + bx[0:H] + br[0:H])
        r = sigmoid(Wxt[:, H:2 * H] + Rh[:, H:2 * H] + bx[H:2 * H] + br[H:2 * H])
        qg = Rh[:, 2 * H:] + br[2 * H:]
        g = np.tanh(Wxt[:, 2 * H:] + r * qg + bx[2 * H:])
        v[t] = np.concatenate([z, r, g, qg], axis=1)
        hn = z * h[t] + (1.0 - z) * g
        mt = zoneout_mask[t] if zoneout_mask is not None else None
        h[t + 1] = _zoneout_forward(hn, h[t], training, zoneout_prob, mt)
    return dict(h=h, v=v, act_Wx=act_Wx, act_Rh=act_Rh, cache1=cache1, cache2=cache2)


def layer_norm_gru_backward(W, R, bx, br, gamma, x, fwd, dh_new, zoneout_mask=None):
    """reference lib/layer_norm_gru_backward_gpu.cu.cc:25-95 and :219-310."""
    T, N, _ = x.shape
    H = R.shape[0]
    dt = x.dtype
    h, v = fwd["h"], fwd["v"]
    dh = np.zeros((N, H), dt)
    dp = np.zeros((T, N, 3 * H), dt)
    dq = np.zeros((T, N, 3 * H), dt)
    dRh = np.zeros((T, N, 3 * H), dt)
    dgamma = np.zeros((2, 3 * H), dt)
    for t in range(T - 1, -1, -1):
        m = zoneout_mask[t] if zoneout_mask is not None else None
        dp[t], dq[t], dh = _gru_pointwise_backward(h[t], v[t], dh_new[t + 1] + dh, m, H)
        dRh[t], dg1, _ = layer_norm_backward(fwd["act_Rh"][t], gamma[1], dq[t], fwd["cache2"][t])
        dgamma[1] += dg1
        dh = dh + dRh[t] @ R.T
    dWx, dg0, _ = layer_norm_backward(fwd["act_Wx"], gamma[0], dp, fwd["cache1"])
    dgamma[0] += dg0
    dpf = dp.reshape(T * N, 3 * H)
    dqf = dq.reshape(T * N, 3 * H)
    dWxf = dWx.reshape(T * N, 3 * H)
    dRhf = dRh.reshape(T * N, 3 * H)
    dbx = dpf.sum(axis=0)
    dbr = dqf.sum(axis=0)
    dx = (dWxf @ W.T).reshape(x.shape)
    dW = x.reshape(T * N, -1).T @ dWxf
    dR = h[:T].reshape(T * N, H).T @ dRhf
    return dict(dx=dx, dW=dW, dR=dR, dbx=dbx, dbr=dbr, dh0=dh, dgamma=dgamma,
                dp=dp, dq=dq, dWx=dWx, dRh=dRh)


# --------------------------------------------------------------------------
# IndRNN and LayerNorm IndRNN
# --------------------------------------------------------------------------
def indrnn_forward(W, u, b, x, h0, training=True, zoneout_prob=0.0, zoneout_mask=None,
                   gamma=None):
    """reference lib/indrnn_forward_gpu.cu.cc:44-62,114-210; with `gamma` ([2,H],
    only row 0 used) it is lib/layer_norm_indrnn_forward_gpu.cu.cc:114-213."""
    T, N, _ = x.shape
    H = u.shape[0]
    dt = x.dtype
    h = np.zeros((T + 1, N, H), dt)
    h[0] = h0
    act_Wx = (x.reshape(T * N, -1) @ W).reshape(T, N, H)
    cache1 = None
    Wx = act_Wx
    if gamma is not None:
        Wx, cache1 = layer_norm_forward(act_Wx, gamma[0])
    for t in range(T):
        hn = np.tanh(Wx[t] + u * h[t] + b)
        mt = zoneout_mask[t] if zoneout_mask is not None else None
        h[t + 1] = _zoneout_forward(hn, h[t], training, zoneout_prob, mt)
    return dict(h=h, act_Wx=act_Wx, cache1=cache1)


def indrnn_backward(W, u, b, x, fwd, dh_new, zoneout_mask=None, gamma=None):
    """reference lib/indrnn_backward_gpu.cu.cc:46-73,122-207 (dW is assigned, not
    accumulated); with `gamma`, lib/layer_norm_indrnn_backward_gpu.cu.cc:122-209."""
    T, N, _ = x.shape
    H = u.shape[0]
    dt = x.dtype
    h = fwd["h"]
    dh = np.zeros((N, H), dt)
    dk = np.zeros((T, N, H), dt)
    du = np.zeros(H, dt)
    db = np.zeros(H, dt)
    for t in range(T - 1, -1, -1):
        dh_total = dh_new[t + 1] + dh
        d0 = np.zeros((N, H), dt)
        if zoneout_mask is not None:
            m = zoneout_mask[t]
            d0 = (1.0 - m) * dh_total
            dh_total = m * dh_total
        dk[t] = d_tanh(h[t + 1]) * dh_total
        dh = d0 + u * dk[t]
        du += (h[t] * dk[t]).sum(axis=0)
        db += dk[t].sum(axis=0)
    out = dict(du=du, db=db, dh0=dh, dk=dk)
    dWx = dk
    if gamma is not None:
        dWx, dg0, _ = layer_norm_backward(fwd["act_Wx"], gamma[0], dk, fwd["cache1"])
        dgamma = np.zeros_like(gamma)
        dgamma[0] = dg0
        out["dgamma"] = dgamma
    dWxf = dWx.reshape(T * N, H)
    out["dW"] = x.reshape(T * N, -1).T @ dWxf
    out["dx"] = (dWxf @ W.T).reshape(x.shape)
    return out


# --------------------------------------------------------------------------
# Weight-layout maps to torch.nn (reference frameworks/pytorch/lstm.py:159-201,
# gru.py:161-208); used by the tests and by the CPU baseline.
# --------------------------------------------------------------------------
def lstm_to_native(W, R, b):
    def reorder(w):
        i, g, f, o = np.split(w, 4, axis=-1)
        return np.concatenate([i, f, g, o], axis=-1)
    half = reorder(b) / 2.0
    return (np.ascontiguousarray(reorder(W).T), np.ascontiguousarray(reorder(R).T),
            half, half.copy())


def gru_to_native(W, R, bx, br):
    def reorder(w):
        z, r, g = np.split(w, 3, axis=-1)
        return np.concatenate([r, z, g], axis=-1)
    return (np.ascontiguousarray(reorder(W).T), np.ascontiguousarray(reorder(R).T),
            reorder(bx), reorder(br))
