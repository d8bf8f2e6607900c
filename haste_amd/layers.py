"""torch.nn layers over the fused GPU ops: the user-facing counterpart of the reference's
`haste_pytorch` package (frameworks/pytorch/{lstm,gru,indrnn,layer_norm_lstm,layer_norm_gru,
layer_norm_indrnn,base_rnn}.py) with the same class names, constructor arguments, parameter
names, shapes, gate orders and initialisers, the same `forward(input, state=None,
lengths=None)` contract and the same `to_native_weights` / `from_native_weights` maps.

As in the reference (frameworks/pytorch/lstm.py:244-266, base_rnn.py:72-76), `_is_cuda()`
decides per call between the fused GPU op and a plain torch loop over the time steps written
here (`_eager_*`): layers whose parameters live on the CPU run that loop, and patching
`_is_cuda` to return False (what the reference's validation/pytorch.py:42-62 does to compare
its two paths) runs it on GPU tensors too.  The loop is differentiated by autograd and is
never taken for GPU parameters unless patched in.

Differences, on purpose:
  * DropConnect of LSTM and GRU is applied inside the recurrence kernel while it loads the
    recurrent matrix (the mask is drawn here and handed over), instead of materialising a
    dropped-out copy of the matrix first (frameworks/pytorch/lstm.py:252).
"""
import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops

__all__ = ["LSTM", "GRU", "IndRNN", "LayerNormLSTM", "LayerNormGRU", "LayerNormIndRNN"]


def _time_major_t(x):
    """[T,N,C] -> [C,T,N], the layout the backward passes take x in."""
    return ops.transpose(x) if x.is_cuda else x.permute(2, 0, 1).contiguous()


def _t(w):
    return ops.transpose(w) if w.is_cuda and w.is_contiguous() else w.t().contiguous()


def _single_shot(ctx, name):
    """The fused backward passes overwrite the activations the forward pass saved (as the
    reference's do, lib/lstm_backward_gpu.cu.cc:92-95), so a graph can be walked once."""
    if getattr(ctx, "consumed", False):
        raise RuntimeError("%s: backward through the same forward pass twice is not supported "
                           "(the saved activations were consumed by the first)" % name)
    ctx.consumed = True


def _no_training_backward(name):
    return RuntimeError("%s backward can only be called in training mode" % name)


# ---- autograd glue (reference frameworks/pytorch/lstm.py:69-88 and siblings) -------------
class _LSTMFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, training, zoneout_prob, x, h0, c0, kernel, recurrent_kernel, bias, zoneout_mask,
                dropconnect_mask, dropconnect_scale):
        h, c, cache = ops.lstm_forward(training, zoneout_prob, x, h0, c0, kernel, recurrent_kernel,
                                       bias, zoneout_mask, dropconnect_mask, dropconnect_scale)
        ctx.save_for_backward(x, kernel, recurrent_kernel, bias, zoneout_mask, h, c, cache,
                              dropconnect_mask if dropconnect_mask is not None else x.new_empty(0))
        ctx.training = training
        ctx.dropconnect_scale = dropconnect_scale
        ctx.mark_non_differentiable(zoneout_mask)
        return h, c

    @staticmethod
    def backward(ctx, grad_h, grad_c):
        if not ctx.training:
            raise _no_training_backward("LSTM")
        x, kernel, recurrent_kernel, bias, zoneout_mask, h, c, cache, dmask = ctx.saved_tensors
        if dmask.numel():
            recurrent_kernel = recurrent_kernel * dmask * ctx.dropconnect_scale
        _single_shot(ctx, "LSTM")  # the backward pass overwrites the activation cache
        dx, dh, dc, dW, dR, db = ops.lstm_backward(
            _time_major_t(x), _t(kernel), _t(recurrent_kernel), bias, zoneout_mask, h, c,
            cache, grad_h.contiguous(), grad_c.contiguous())
        if dmask.numel():
            dR = dR * dmask * ctx.dropconnect_scale
        return None, None, dx, dh, dc, dW, dR, db, None, None, None


class _GRUFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, training, zoneout_prob, x, h0, kernel, recurrent_kernel, bias, recurrent_bias,
                zoneout_mask, dropconnect_mask, dropconnect_scale):
        h, cache = ops.gru_forward(training, zoneout_prob, x, h0, kernel, recurrent_kernel, bias,
                                   recurrent_bias, zoneout_mask, dropconnect_mask, dropconnect_scale)
        ctx.save_for_backward(x, kernel, recurrent_kernel, bias, recurrent_bias, zoneout_mask, h, cache,
                              dropconnect_mask if dropconnect_mask is not None else x.new_empty(0))
        ctx.training = training
        ctx.dropconnect_scale = dropconnect_scale
        ctx.mark_non_differentiable(zoneout_mask)
        return h

    @staticmethod
    def backward(ctx, grad_h):
        if not ctx.training:
            raise _no_training_backward("GRU")
        x, kernel, recurrent_kernel, bias, recurrent_bias, zoneout_mask, h, cache, dmask = ctx.saved_tensors
        if dmask.numel():
            recurrent_kernel = recurrent_kernel * dmask * ctx.dropconnect_scale
        dx, dh, dW, dR, dbx, dbr = ops.gru_backward(
            _time_major_t(x), _t(kernel), _t(recurrent_kernel), bias, recurrent_bias, zoneout_mask, h,
            cache, grad_h.contiguous())
        if dmask.numel():
            dR = dR * dmask * ctx.dropconnect_scale
        return None, None, dx, dh, dW, dR, dbx, dbr, None, None, None


class _IndRNNFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, training, zoneout_prob, x, h0, kernel, recurrent_scale, bias, zoneout_mask):
        h = ops.indrnn_forward(training, zoneout_prob, x, h0, kernel, recurrent_scale, bias, zoneout_mask)
        ctx.save_for_backward(x, kernel, recurrent_scale, bias, zoneout_mask, h)
        ctx.training = training
        ctx.mark_non_differentiable(zoneout_mask)
        return h

    @staticmethod
    def backward(ctx, grad_h):
        if not ctx.training:
            raise _no_training_backward("IndRNN")
        x, kernel, recurrent_scale, bias, zoneout_mask, h = ctx.saved_tensors
        dx, dh, dW, du, db = ops.indrnn_backward(_time_major_t(x), _t(kernel), recurrent_scale, bias,
                                                 zoneout_mask, h, grad_h.contiguous())
        return None, None, dx, dh, dW, du, db, None


class _LayerNormIndRNNFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, training, zoneout_prob, x, h0, kernel, recurrent_scale, bias, gamma, zoneout_mask):
        h, act_Wx, cache = ops.layer_norm_indrnn_forward(training, zoneout_prob, x, h0, kernel,
                                                         recurrent_scale, bias, gamma, zoneout_mask)
        ctx.save_for_backward(x, kernel, recurrent_scale, bias, gamma, zoneout_mask, h, act_Wx, cache)
        ctx.training = training
        ctx.mark_non_differentiable(zoneout_mask)
        return h

    @staticmethod
    def backward(ctx, grad_h):
        if not ctx.training:
            raise _no_training_backward("LayerNormIndRNN")
        x, kernel, recurrent_scale, bias, gamma, zoneout_mask, h, act_Wx, cache = ctx.saved_tensors
        dx, dh, dW, du, db, dgamma = ops.layer_norm_indrnn_backward(
            _time_major_t(x), _t(kernel), recurrent_scale, bias, gamma, zoneout_mask, h, act_Wx, cache,
            grad_h.contiguous())
        return None, None, dx, dh, dW, du, db, dgamma, None


class _LayerNormLSTMFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, training, zoneout_prob, x, h0, c0, kernel, recurrent_kernel, bias, gamma, gamma_h,
                beta_h, zoneout_mask):
        outs = ops.layer_norm_lstm_forward(training, zoneout_prob, x, h0, c0, kernel, recurrent_kernel,
                                           bias, gamma, gamma_h, beta_h, zoneout_mask)
        ctx.save_for_backward(x, kernel, recurrent_kernel, bias, gamma, gamma_h, beta_h, zoneout_mask,
                              *outs)
        ctx.training = training
        ctx.mark_non_differentiable(zoneout_mask)
        return outs[0], outs[1]

    @staticmethod
    def backward(ctx, grad_h, grad_c):
        if not ctx.training:
            raise _no_training_backward("LayerNormLSTM")
        (x, kernel, recurrent_kernel, bias, gamma, gamma_h, beta_h, zoneout_mask, h, c, act_Wx,
         act_Wx_norm, cache1, act_Rh, cache2, act_c_norm, cache3) = ctx.saved_tensors
        _single_shot(ctx, "LayerNormLSTM")  # the saved activations are overwritten below
        grads = ops.layer_norm_lstm_backward(
            _time_major_t(x), _t(kernel), _t(recurrent_kernel), bias, gamma, gamma_h, beta_h,
            zoneout_mask, h, c, act_Wx, act_Wx_norm, cache1, act_Rh, cache2, act_c_norm, cache3,
            grad_h.contiguous(), grad_c.contiguous())
        return (None, None) + tuple(grads) + (None,)


class _LayerNormGRUFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, training, zoneout_prob, x, h0, kernel, recurrent_kernel, bias, recurrent_bias,
                gamma, zoneout_mask):
        outs = ops.layer_norm_gru_forward(training, zoneout_prob, x, h0, kernel, recurrent_kernel, bias,
                                          recurrent_bias, gamma, zoneout_mask)
        ctx.save_for_backward(x, kernel, recurrent_kernel, bias, recurrent_bias, gamma, zoneout_mask,
                              *outs)
        ctx.training = training
        ctx.mark_non_differentiable(zoneout_mask)
        return outs[0]

    @staticmethod
    def backward(ctx, grad_h):
        if not ctx.training:
            raise _no_training_backward("LayerNormGRU")
        (x, kernel, recurrent_kernel, bias, recurrent_bias, gamma, zoneout_mask, h, cache, act_Wx,
         cache1, act_Rh, cache2) = ctx.saved_tensors
        grads = ops.layer_norm_gru_backward(
            _time_major_t(x), _t(kernel), _t(recurrent_kernel), bias, recurrent_bias, gamma,
            zoneout_mask, h, cache, act_Wx, cache1, act_Rh, cache2, grad_h.contiguous())
        return (None, None) + tuple(grads) + (None,)


# ---- the time loop in plain torch (reference *Script functions, e.g. frameworks/pytorch/
# lstm.py:33-66, gru.py:33-66, layer_norm_lstm.py:31-66, layer_norm_gru.py:31-64,
# indrnn.py:32-51, layer_norm_indrnn.py:32-53) -------------------------------------------------
def _eager_recurrence(step, first, steps, training, zoneout_prob, zoneout_mask):
    """Runs `step(t, states) -> states` for t = 0 .. steps-1 from the states `first` (a tuple,
    hidden state first) and returns each state's sequence stacked to [steps+1, N, H].  Zoneout
    acts on the hidden state only: the mask picks new or old during training, inference blends
    (reference frameworks/pytorch/lstm.py:58-62)."""
    history = [[s] for s in first]
    for t in range(steps):
        new = list(step(t, tuple(seq[-1] for seq in history)))
        if zoneout_prob:
            old_h = history[0][-1]
            if training:
                new[0] = (new[0] - old_h) * zoneout_mask[t] + old_h
            else:
                new[0] = zoneout_prob * old_h + (1 - zoneout_prob) * new[0]
        for seq, value in zip(history, new):
            seq.append(value)
    return tuple(torch.stack(seq) for seq in history)


def _norm(v, gamma, beta=None):
    return F.layer_norm(v, (v.shape[-1],), weight=gamma, bias=beta)


def _eager_lstm(training, zoneout_prob, x, h0, c0, kernel, recurrent_kernel, bias, zoneout_mask,
                gamma=None, gamma_h=None, beta_h=None):
    """LSTM (gamma None) or LayerNormLSTM: returns (h, c), each [T+1, N, H]."""
    wx = x @ kernel if gamma is None else _norm(x @ kernel, gamma[0])

    def step(t, state):
        h, c = state
        rh = h @ recurrent_kernel if gamma is None else _norm(h @ recurrent_kernel, gamma[1])
        i, g, f, o = torch.chunk(rh + wx[t] + bias, 4, dim=1)
        c_new = torch.sigmoid(f) * c + torch.sigmoid(i) * torch.tanh(g)
        seen = c_new if gamma is None else _norm(c_new, gamma_h, beta_h)
        return torch.sigmoid(o) * torch.tanh(seen), c_new

    return _eager_recurrence(step, (h0, c0), x.shape[0], training, zoneout_prob, zoneout_mask)


def _eager_gru(training, zoneout_prob, x, h0, kernel, recurrent_kernel, bias, recurrent_bias,
               zoneout_mask, gamma=None):
    """GRU (gamma None) or LayerNormGRU, reset gate applied after the recurrent product."""
    wx = (x @ kernel if gamma is None else _norm(x @ kernel, gamma[0])) + bias

    def step(t, state):
        (h,) = state
        rh = (h @ recurrent_kernel if gamma is None else _norm(h @ recurrent_kernel, gamma[1])) + recurrent_bias
        xz, xr, xg = torch.chunk(wx[t], 3, dim=1)
        hz, hr, hg = torch.chunk(rh, 3, dim=1)
        z = torch.sigmoid(xz + hz)
        r = torch.sigmoid(xr + hr)
        return (z * h + (1 - z) * torch.tanh(xg + r * hg),)

    return _eager_recurrence(step, (h0,), x.shape[0], training, zoneout_prob, zoneout_mask)[0]


def _eager_indrnn(training, zoneout_prob, x, h0, kernel, recurrent_scale, bias, zoneout_mask, gamma=None):
    """IndRNN (gamma None) or LayerNormIndRNN."""
    wx = (x @ kernel if gamma is None else _norm(x @ kernel, gamma[0])) + bias

    def step(t, state):
        return (torch.tanh(wx[t] + state[0] * recurrent_scale),)

    return _eager_recurrence(step, (h0,), x.shape[0], training, zoneout_prob, zoneout_mask)[0]


def _dropped(weight, mask, scale):
    """The recurrent matrix under DropConnect (what F.dropout gives the reference's loop,
    frameworks/pytorch/lstm.py:263), differentiable with respect to `weight`."""
    return weight if mask is None else weight * mask * scale


# ---- shared layer behaviour (reference frameworks/pytorch/base_rnn.py:25-100) ------------
class _RNNBase(nn.Module):
    _name = "RNN"

    def __init__(self, input_size, hidden_size, batch_first, zoneout, return_state_sequence,
                 dropout=0.0):
        super().__init__()
        if not 0.0 <= dropout <= 1.0:
            raise ValueError("%s: dropout must be in [0.0, 1.0]" % self._name)
        if not 0.0 <= zoneout <= 1.0:
            raise ValueError("%s: zoneout must be in [0.0, 1.0]" % self._name)
        self.input_size = input_size
        self.hidden_size = hidden_size
        self.batch_first = batch_first
        self.zoneout = zoneout
        self.dropout = dropout
        self.return_state_sequence = return_state_sequence

    def _time_major(self, x):
        return x.permute(1, 0, 2) if self.batch_first else x

    def _initial_state(self, x, state, count):
        """`count` tensors of shape [N,H]: zeros, or the caller's [1,N,H] states checked."""
        shape = [1, x.shape[1], self.hidden_size]
        if state is None:
            return tuple(x.new_zeros(shape[1:]) for _ in range(count))
        states = (state,) if count == 1 else state
        if count > 1 and (not isinstance(states, (tuple, list)) or len(states) != count):
            raise ValueError("RNN state must be a tuple of %d tensors" % count)
        for s in states:
            if not torch.is_tensor(s) or list(s.shape) != shape:
                raise ValueError("RNN state has invalid shape; expected %s, got %s"
                                 % (shape, list(s.shape) if torch.is_tensor(s) else type(s)))
        return tuple(s[0].contiguous() for s in states)

    def _final_state(self, seq, lengths):
        """seq: [T+1,N,H] state after every step (slot 0 = initial state)."""
        if self.return_state_sequence:
            return self._time_major(seq[1:]).unsqueeze(0)
        if lengths is not None:
            cols = torch.arange(seq.size(1), device=seq.device)
            rows = torch.as_tensor(lengths, device=seq.device, dtype=torch.long)
            return seq[rows, cols].unsqueeze(0)
        return seq[-1].unsqueeze(0)

    def _zoneout_mask(self, x):
        # 1 = take the new value (reference frameworks/pytorch/base_rnn.py:64-70)
        if self.zoneout:
            return x.new_empty(x.shape[0], x.shape[1], self.hidden_size).bernoulli_(1.0 - self.zoneout)
        return x.new_empty(0, 0, 0)

    def _dropconnect_mask(self, weight):
        """(mask, scale) for inverted dropout on the recurrent matrix, or (None, 1.0)."""
        if not self.training or not self.dropout:
            return None, 1.0
        if self.dropout >= 1.0:
            return torch.zeros_like(weight), 0.0
        keep = 1.0 - self.dropout
        return torch.empty_like(weight).bernoulli_(keep), 1.0 / keep

    def _is_cuda(self):
        """True: the fused GPU ops run; False: the plain torch loop (reference
        frameworks/pytorch/base_rnn.py:72-76)."""
        on_gpu = [t.is_cuda for t in self.parameters()]
        if any(on_gpu) and not all(on_gpu):
            raise ValueError("RNN tensors should all be CUDA tensors or none should be CUDA tensors")
        return any(on_gpu)

    def _check_fused(self, x):
        """What the fused ops need beyond the reference's checks: the input on the GPU and one
        of the dtypes the library is built for, shared by the input and every parameter."""
        tensors = list(self.parameters()) + [x]
        if not x.is_cuda:
            raise RuntimeError("%s: the parameters are GPU tensors, the input must be one too" % self._name)
        if x.dtype not in (torch.float32, torch.float64, torch.float16) or any(t.dtype != x.dtype for t in tensors):
            raise RuntimeError(
                "%s: parameters and input must all have one dtype: float32, float64 or (GRU) float16" % self._name)


def _init_gates(kernel, recurrent_kernel, hidden_size, gates):
    for g in range(gates):
        nn.init.xavier_uniform_(kernel[:, g * hidden_size:(g + 1) * hidden_size])
        nn.init.orthogonal_(recurrent_kernel[:, g * hidden_size:(g + 1) * hidden_size])


def _regroup(w, order_in, order_out):
    """Reorders the gate blocks along the last dimension, e.g. 'igfo' -> 'ifgo'."""
    blocks = dict(zip(order_in, torch.chunk(w, len(order_in), dim=-1)))
    return torch.cat([blocks[g] for g in order_out], dim=-1)


class LSTM(_RNNBase):
    """Long short-term memory layer; gate order i,g,f,o (reference frameworks/pytorch/lstm.py:91-265).

    Parameters: kernel [input_size, 4H] (Xavier uniform per gate), recurrent_kernel [H, 4H]
    (orthogonal per gate), bias [4H] (zeros, forget block = forget_bias).
    """
    _name = "LSTM"

    def __init__(self, input_size, hidden_size, batch_first=False, forget_bias=1.0, dropout=0.0,
                 zoneout=0.0, return_state_sequence=False):
        super().__init__(input_size, hidden_size, batch_first, zoneout, return_state_sequence, dropout)
        self.forget_bias = forget_bias
        self.kernel = nn.Parameter(torch.empty(input_size, hidden_size * 4))
        self.recurrent_kernel = nn.Parameter(torch.empty(hidden_size, hidden_size * 4))
        self.bias = nn.Parameter(torch.empty(hidden_size * 4))
        self.reset_parameters()

    def reset_parameters(self):
        H = self.hidden_size
        with torch.no_grad():
            _init_gates(self.kernel, self.recurrent_kernel, H, 4)
            self.bias.zero_()
            self.bias[2 * H:3 * H].fill_(self.forget_bias)

    def to_native_weights(self):
        """(weight_ih_l0, weight_hh_l0, bias_ih_l0, bias_hh_l0) of an equivalent torch.nn.LSTM."""
        half = _regroup(self.bias.detach(), "igfo", "ifgo") / 2.0
        return (nn.Parameter(_t(_regroup(self.kernel.detach(), "igfo", "ifgo"))),
                nn.Parameter(_t(_regroup(self.recurrent_kernel.detach(), "igfo", "ifgo"))),
                nn.Parameter(half), nn.Parameter(half.clone()))

    def from_native_weights(self, weight_ih_l0, weight_hh_l0, bias_ih_l0, bias_hh_l0):
        """Loads the weights of a torch.nn.LSTM layer."""
        self.kernel = nn.Parameter(_regroup(weight_ih_l0.detach().t(), "ifgo", "igfo").contiguous())
        self.recurrent_kernel = nn.Parameter(_regroup(weight_hh_l0.detach().t(), "ifgo", "igfo").contiguous())
        self.bias = nn.Parameter(_regroup((bias_ih_l0 + bias_hh_l0).detach(), "ifgo", "igfo").contiguous())

    def forward(self, input, state=None, lengths=None):
        """input [T,N,C] ([N,T,C] if batch_first) -> (output, (h_n, c_n)); h_n, c_n are [1,N,H],
        taken at `lengths` when given (the output itself is not masked)."""
        x = self._time_major(input)
        h0, c0 = self._initial_state(x, state, 2)
        dmask, dscale = self._dropconnect_mask(self.recurrent_kernel)
        zmask = self._zoneout_mask(x)
        if self._is_cuda():
            self._check_fused(x)
            h, c = _LSTMFunction.apply(self.training, self.zoneout, x.contiguous(), h0, c0,
                                       self.kernel.contiguous(), self.recurrent_kernel.contiguous(),
                                       self.bias.contiguous(), zmask, dmask, dscale)
        else:
            h, c = _eager_lstm(self.training, self.zoneout, x, h0, c0, self.kernel,
                               _dropped(self.recurrent_kernel, dmask, dscale), self.bias, zmask)
        return self._time_major(h[1:]), (self._final_state(h, lengths), self._final_state(c, lengths))


class GRU(_RNNBase):
    """Gated recurrent unit layer, "reset-after" form, gate order z,r,g (reference
    frameworks/pytorch/gru.py:91-272).  Parameters: kernel [C,3H], recurrent_kernel [H,3H],
    bias [3H], recurrent_bias [3H]."""
    _name = "GRU"

    def __init__(self, input_size, hidden_size, batch_first=False, dropout=0.0, zoneout=0.0,
                 return_state_sequence=False):
        super().__init__(input_size, hidden_size, batch_first, zoneout, return_state_sequence, dropout)
        self.kernel = nn.Parameter(torch.empty(input_size, hidden_size * 3))
        self.recurrent_kernel = nn.Parameter(torch.empty(hidden_size, hidden_size * 3))
        self.bias = nn.Parameter(torch.empty(hidden_size * 3))
        self.recurrent_bias = nn.Parameter(torch.empty(hidden_size * 3))
        self.reset_parameters()

    def reset_parameters(self):
        with torch.no_grad():
            _init_gates(self.kernel, self.recurrent_kernel, self.hidden_size, 3)
            self.bias.zero_()
            self.recurrent_bias.zero_()

    def to_native_weights(self):
        """(weight_ih_l0, weight_hh_l0, bias_ih_l0, bias_hh_l0) of an equivalent torch.nn.GRU."""
        return (nn.Parameter(_t(_regroup(self.kernel.detach(), "zrg", "rzg"))),
                nn.Parameter(_t(_regroup(self.recurrent_kernel.detach(), "zrg", "rzg"))),
                nn.Parameter(_regroup(self.bias.detach(), "zrg", "rzg").contiguous()),
                nn.Parameter(_regroup(self.recurrent_bias.detach(), "zrg", "rzg").contiguous()))

    def from_native_weights(self, weight_ih_l0, weight_hh_l0, bias_ih_l0, bias_hh_l0):
        self.kernel = nn.Parameter(_regroup(weight_ih_l0.detach().t(), "rzg", "zrg").contiguous())
        self.recurrent_kernel = nn.Parameter(_regroup(weight_hh_l0.detach().t(), "rzg", "zrg").contiguous())
        self.bias = nn.Parameter(_regroup(bias_ih_l0.detach(), "rzg", "zrg").contiguous())
        self.recurrent_bias = nn.Parameter(_regroup(bias_hh_l0.detach(), "rzg", "zrg").contiguous())

    def forward(self, input, state=None, lengths=None):
        x = self._time_major(input)
        (h0,) = self._initial_state(x, state, 1)
        dmask, dscale = self._dropconnect_mask(self.recurrent_kernel)
        zmask = self._zoneout_mask(x)
        if self._is_cuda():
            self._check_fused(x)
            h = _GRUFunction.apply(self.training, self.zoneout, x.contiguous(), h0,
                                   self.kernel.contiguous(), self.recurrent_kernel.contiguous(),
                                   self.bias.contiguous(), self.recurrent_bias.contiguous(),
                                   zmask, dmask, dscale)
        else:
            h = _eager_gru(self.training, self.zoneout, x, h0, self.kernel,
                           _dropped(self.recurrent_kernel, dmask, dscale), self.bias,
                           self.recurrent_bias, zmask)
        return self._time_major(h[1:]), self._final_state(h, lengths)


class IndRNN(_RNNBase):
    """Independently recurrent layer h' = tanh(xW + u*h + b) (reference
    frameworks/pytorch/indrnn.py:78-190).  Parameters: kernel [C,H], recurrent_scale [H]
    (uniform in [-0.5, 0.5]), bias [H]."""
    _name = "IndRNN"

    def __init__(self, input_size, hidden_size, batch_first=False, zoneout=0.0,
                 return_state_sequence=False):
        super().__init__(input_size, hidden_size, batch_first, zoneout, return_state_sequence)
        self.kernel = nn.Parameter(torch.empty(input_size, hidden_size))
        self.recurrent_scale = nn.Parameter(torch.empty(hidden_size))
        self.bias = nn.Parameter(torch.empty(hidden_size))
        self.reset_parameters()

    def reset_parameters(self):
        with torch.no_grad():
            nn.init.xavier_uniform_(self.kernel)
            nn.init.uniform_(self.recurrent_scale, -0.5, 0.5)
            self.bias.zero_()

    def forward(self, input, state=None, lengths=None):
        x = self._time_major(input)
        (h0,) = self._initial_state(x, state, 1)
        zmask = self._zoneout_mask(x)
        if self._is_cuda():
            self._check_fused(x)
            h = _IndRNNFunction.apply(self.training, self.zoneout, x.contiguous(), h0,
                                      self.kernel.contiguous(), self.recurrent_scale.contiguous(),
                                      self.bias.contiguous(), zmask)
        else:
            h = _eager_indrnn(self.training, self.zoneout, x, h0, self.kernel, self.recurrent_scale,
                              self.bias, zmask)
        return self._time_major(h[1:]), self._final_state(h, lengths)


class LayerNormIndRNN(_RNNBase):
    """IndRNN with layer norm on the input projection (reference
    frameworks/pytorch/layer_norm_indrnn.py:83-203); gamma is [2,H], only row 0 is used."""
    _name = "LayerNormIndRNN"

    def __init__(self, input_size, hidden_size, batch_first=False, zoneout=0.0,
                 return_state_sequence=False):
        super().__init__(input_size, hidden_size, batch_first, zoneout, return_state_sequence)
        self.kernel = nn.Parameter(torch.empty(input_size, hidden_size))
        self.recurrent_scale = nn.Parameter(torch.empty(hidden_size))
        self.bias = nn.Parameter(torch.empty(hidden_size))
        self.gamma = nn.Parameter(torch.empty(2, hidden_size))
        self.reset_parameters()

    def reset_parameters(self):
        with torch.no_grad():
            nn.init.xavier_uniform_(self.kernel)
            nn.init.uniform_(self.recurrent_scale, -0.5, 0.5)
            self.bias.zero_()
            self.gamma.fill_(1.0)

    def forward(self, input, state=None, lengths=None):
        x = self._time_major(input)
        (h0,) = self._initial_state(x, state, 1)
        zmask = self._zoneout_mask(x)
        if self._is_cuda():
            self._check_fused(x)
            h = _LayerNormIndRNNFunction.apply(self.training, self.zoneout, x.contiguous(), h0,
                                               self.kernel.contiguous(), self.recurrent_scale.contiguous(),
                                               self.bias.contiguous(), self.gamma.contiguous(), zmask)
        else:
            h = _eager_indrnn(self.training, self.zoneout, x, h0, self.kernel, self.recurrent_scale,
                              self.bias, zmask, gamma=self.gamma)
        return self._time_major(h[1:]), self._final_state(h, lengths)


class LayerNormLSTM(_RNNBase):
    """LSTM with layer norm on xW, on hR and on the cell state (reference
    frameworks/pytorch/layer_norm_lstm.py:94-245).  Extra parameters: gamma [2,4H] (ones),
    gamma_h [H] (ones), beta_h [H] (zeros)."""
    _name = "LayerNormLSTM"

    def __init__(self, input_size, hidden_size, batch_first=False, forget_bias=1.0, dropout=0.0,
                 zoneout=0.0, return_state_sequence=False):
        super().__init__(input_size, hidden_size, batch_first, zoneout, return_state_sequence, dropout)
        self.forget_bias = forget_bias
        self.kernel = nn.Parameter(torch.empty(input_size, hidden_size * 4))
        self.recurrent_kernel = nn.Parameter(torch.empty(hidden_size, hidden_size * 4))
        self.bias = nn.Parameter(torch.empty(hidden_size * 4))
        self.gamma = nn.Parameter(torch.empty(2, hidden_size * 4))
        self.gamma_h = nn.Parameter(torch.empty(hidden_size))
        self.beta_h = nn.Parameter(torch.empty(hidden_size))
        self.reset_parameters()

    def reset_parameters(self):
        H = self.hidden_size
        with torch.no_grad():
            _init_gates(self.kernel, self.recurrent_kernel, H, 4)
            self.bias.zero_()
            self.bias[2 * H:3 * H].fill_(self.forget_bias)
            self.gamma.fill_(1.0)
            self.gamma_h.fill_(1.0)
            self.beta_h.zero_()

    def forward(self, input, state=None, lengths=None):
        x = self._time_major(input)
        h0, c0 = self._initial_state(x, state, 2)
        dmask, dscale = self._dropconnect_mask(self.recurrent_kernel)
        R = _dropped(self.recurrent_kernel, dmask, dscale)
        zmask = self._zoneout_mask(x)
        if self._is_cuda():
            self._check_fused(x)
            h, c = _LayerNormLSTMFunction.apply(self.training, self.zoneout, x.contiguous(), h0, c0,
                                                self.kernel.contiguous(), R.contiguous(),
                                                self.bias.contiguous(), self.gamma.contiguous(),
                                                self.gamma_h.contiguous(), self.beta_h.contiguous(), zmask)
        else:
            h, c = _eager_lstm(self.training, self.zoneout, x, h0, c0, self.kernel, R, self.bias, zmask,
                               gamma=self.gamma, gamma_h=self.gamma_h, beta_h=self.beta_h)
        return self._time_major(h[1:]), (self._final_state(h, lengths), self._final_state(c, lengths))


class LayerNormGRU(_RNNBase):
    """GRU with layer norm on xW and on hR (reference frameworks/pytorch/layer_norm_gru.py:94-233);
    gamma is [2,3H] (ones)."""
    _name = "LayerNormGRU"

    def __init__(self, input_size, hidden_size, batch_first=False, dropout=0.0, zoneout=0.0,
                 return_state_sequence=False):
        super().__init__(input_size, hidden_size, batch_first, zoneout, return_state_sequence, dropout)
        self.kernel = nn.Parameter(torch.empty(input_size, hidden_size * 3))
        self.recurrent_kernel = nn.Parameter(torch.empty(hidden_size, hidden_size * 3))
        self.bias = nn.Parameter(torch.empty(hidden_size * 3))
        self.recurrent_bias = nn.Parameter(torch.empty(hidden_size * 3))
        self.gamma = nn.Parameter(torch.empty(2, hidden_size * 3))
        self.reset_parameters()

    def reset_parameters(self):
        with torch.no_grad():
            _init_gates(self.kernel, self.recurrent_kernel, self.hidden_size, 3)
            self.bias.zero_()
            self.recurrent_bias.zero_()
            self.gamma.fill_(1.0)

    def forward(self, input, state=None, lengths=None):
        x = self._time_major(input)
        (h0,) = self._initial_state(x, state, 1)
        dmask, dscale = self._dropconnect_mask(self.recurrent_kernel)
        R = _dropped(self.recurrent_kernel, dmask, dscale)
        zmask = self._zoneout_mask(x)
        if self._is_cuda():
            self._check_fused(x)
            h = _LayerNormGRUFunction.apply(self.training, self.zoneout, x.contiguous(), h0,
                                            self.kernel.contiguous(), R.contiguous(),
                                            self.bias.contiguous(), self.recurrent_bias.contiguous(),
                                            self.gamma.contiguous(), zmask)
        else:
            h = _eager_gru(self.training, self.zoneout, x, h0, self.kernel, R, self.bias,
                           self.recurrent_bias, zmask, gamma=self.gamma)
        return self._time_major(h[1:]), self._final_state(h, lengths)
