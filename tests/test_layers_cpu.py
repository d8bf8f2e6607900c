"""Host-side behaviour of the torch.nn layers (no GPU needed): parameter names, shapes and
initial values as in the reference's haste_pytorch layers, the native-weight maps checked
against torch.nn.LSTM / torch.nn.GRU through the oracle, argument validation, and the plain
torch loop that layers with CPU parameters run (the reference's *Script path), against the
oracle's forward and backward passes."""
import numpy as np
import pytest
import torch

import haste_amd
from oracle import haste_oracle as O


def test_parameter_names_shapes_and_init():
    C, H = 6, 8
    lstm = haste_amd.LSTM(C, H, forget_bias=1.5)
    assert {k: tuple(v.shape) for k, v in lstm.named_parameters()} == {
        "kernel": (C, 4 * H), "recurrent_kernel": (H, 4 * H), "bias": (4 * H,)}
    b = lstm.bias.detach().numpy()
    assert np.all(b[2 * H:3 * H] == 1.5) and np.all(np.delete(b, np.s_[2 * H:3 * H]) == 0)
    # orthogonal per gate block (reference frameworks/pytorch/lstm.py:203-210)
    for g in range(4):
        blk = lstm.recurrent_kernel.detach()[:, g * H:(g + 1) * H]
        assert torch.allclose(blk.t() @ blk, torch.eye(H), atol=1e-5)
    gru = haste_amd.GRU(C, H)
    assert {k: tuple(v.shape) for k, v in gru.named_parameters()} == {
        "kernel": (C, 3 * H), "recurrent_kernel": (H, 3 * H), "bias": (3 * H,), "recurrent_bias": (3 * H,)}
    ind = haste_amd.IndRNN(C, H)
    assert {k: tuple(v.shape) for k, v in ind.named_parameters()} == {
        "kernel": (C, H), "recurrent_scale": (H,), "bias": (H,)}
    assert float(ind.recurrent_scale.detach().abs().max()) <= 0.5
    lnl = haste_amd.LayerNormLSTM(C, H)
    assert tuple(lnl.gamma.shape) == (2, 4 * H) and tuple(lnl.gamma_h.shape) == (H,)
    assert torch.all(lnl.gamma == 1) and torch.all(lnl.gamma_h == 1) and torch.all(lnl.beta_h == 0)
    assert torch.all(lnl.bias[2 * H:3 * H] == 1.0)
    lng = haste_amd.LayerNormGRU(C, H)
    assert tuple(lng.gamma.shape) == (2, 3 * H)
    lni = haste_amd.LayerNormIndRNN(C, H)
    assert tuple(lni.gamma.shape) == (2, H)


def test_lstm_native_weight_maps():
    C, H, T, N = 5, 7, 4, 3
    torch.manual_seed(0)
    layer = haste_amd.LSTM(C, H).double()
    with torch.no_grad():
        layer.bias.normal_()
    ref = torch.nn.LSTM(C, H).double()
    for name, w in zip(("weight_ih_l0", "weight_hh_l0", "bias_ih_l0", "bias_hh_l0"), layer.to_native_weights()):
        setattr(ref, name, w)
    x = torch.randn(T, N, C, dtype=torch.float64)
    y, _ = ref(x)
    h, _, _ = O.lstm_forward(layer.kernel.detach().numpy(), layer.recurrent_kernel.detach().numpy(),
                             layer.bias.detach().numpy(), x.numpy(), np.zeros((N, H)), np.zeros((N, H)))
    assert np.max(np.abs(h[1:] - y.detach().numpy())) < 1e-12
    # and back
    other = haste_amd.LSTM(C, H).double()
    other.from_native_weights(ref.weight_ih_l0, ref.weight_hh_l0, ref.bias_ih_l0, ref.bias_hh_l0)
    assert torch.allclose(other.kernel, layer.kernel) and torch.allclose(other.recurrent_kernel, layer.recurrent_kernel)
    assert torch.allclose(other.bias, layer.bias)


def test_gru_native_weight_maps():
    C, H, T, N = 5, 7, 4, 3
    torch.manual_seed(1)
    layer = haste_amd.GRU(C, H).double()
    with torch.no_grad():
        layer.bias.normal_()
        layer.recurrent_bias.normal_()
    ref = torch.nn.GRU(C, H).double()
    for name, w in zip(("weight_ih_l0", "weight_hh_l0", "bias_ih_l0", "bias_hh_l0"), layer.to_native_weights()):
        setattr(ref, name, w)
    x = torch.randn(T, N, C, dtype=torch.float64)
    y, _ = ref(x)
    h, _ = O.gru_forward(layer.kernel.detach().numpy(), layer.recurrent_kernel.detach().numpy(),
                         layer.bias.detach().numpy(), layer.recurrent_bias.detach().numpy(), x.numpy(),
                         np.zeros((N, H)))
    assert np.max(np.abs(h[1:] - y.detach().numpy())) < 1e-12
    other = haste_amd.GRU(C, H).double()
    other.from_native_weights(ref.weight_ih_l0, ref.weight_hh_l0, ref.bias_ih_l0, ref.bias_hh_l0)
    for a, b in zip(other.parameters(), layer.parameters()):
        assert torch.allclose(a, b)


def test_argument_validation():
    with pytest.raises(ValueError):
        haste_amd.LSTM(4, 4, dropout=1.5)
    with pytest.raises(ValueError):
        haste_amd.GRU(4, 4, zoneout=-0.1)
    layer = haste_amd.LSTM(4, 4)
    assert layer._is_cuda() is False
    # state shape is checked before anything runs (reference base_rnn.py:81-100)
    x = torch.zeros(2, 3, 4)
    with pytest.raises(ValueError):
        layer._initial_state(x, (torch.zeros(1, 3, 4),), 2)
    with pytest.raises(ValueError):
        layer._initial_state(x, (torch.zeros(1, 3, 5), torch.zeros(1, 3, 4)), 2)
    h0, c0 = layer._initial_state(x, None, 2)
    assert tuple(h0.shape) == (3, 4) and float(h0.abs().sum()) == 0


def test_final_state_selection():
    layer = haste_amd.GRU(4, 5)
    seq = torch.arange(6 * 3 * 5, dtype=torch.float32).reshape(6, 3, 5)  # T=5 plus the initial slot
    assert torch.equal(layer._final_state(seq, None), seq[-1][None])
    got = layer._final_state(seq, torch.tensor([5, 2, 1]))
    assert torch.equal(got[0, 0], seq[5, 0]) and torch.equal(got[0, 1], seq[2, 1]) and torch.equal(got[0, 2], seq[1, 2])
    layer.return_state_sequence = True
    assert tuple(layer._final_state(seq, None).shape) == (1, 5, 3, 5)
    layer.batch_first = True
    assert tuple(layer._final_state(seq, None).shape) == (1, 3, 5, 5)


# ---- the plain torch loop of CPU layers (reference frameworks/pytorch/lstm.py:33-66 and
# siblings) against the oracle: outputs, final states and every gradient, float64 ------------
def _np(t):
    return t.detach().numpy().astype(np.float64)


def _cpu_masks(layer, T, N, seed):
    """What the layer draws after torch.manual_seed(seed): DropConnect first, then zoneout."""
    torch.manual_seed(seed)
    dmask, dscale = None, 1.0
    if getattr(layer, "dropout", 0.0) and layer.training:
        dmask = torch.empty_like(layer.recurrent_kernel).bernoulli_(1.0 - layer.dropout)
        dscale = 1.0 / (1.0 - layer.dropout)
    zmask = torch.empty(T, N, layer.hidden_size, dtype=layer.kernel.dtype).bernoulli_(1.0 - layer.zoneout)
    return dmask, dscale, zmask


def _close(a, b, what):
    err = np.max(np.abs(_np(a) - b)) / max(np.max(np.abs(b)), 1e-30)
    assert err < 1e-10, (what, err)


@pytest.mark.parametrize("name", ["LSTM", "LayerNormLSTM"])
def test_cpu_lstm_layers_match_the_oracle(name):
    T, N, C, H = 6, 4, 5, 7
    torch.manual_seed(1)
    layer = getattr(haste_amd, name)(C, H, dropout=0.2, zoneout=0.3).double()
    with torch.no_grad():
        for p_ in layer.parameters():
            p_.add_(0.1 * torch.randn_like(p_))
    x = torch.randn(T, N, C, dtype=torch.float64, requires_grad=True)
    h0, c0 = torch.randn(1, N, H, dtype=torch.float64), torch.randn(1, N, H, dtype=torch.float64)
    dmask, dscale, zmask = _cpu_masks(layer, T, N, 11)
    torch.manual_seed(11)
    y, (hn, cn) = layer(x, (h0, c0), lengths=[6, 2, 1, 4])
    dy = torch.randn(T, N, H, dtype=torch.float64)
    (y * dy).sum().backward()
    W, R, b, m = _np(layer.kernel), _np(layer.recurrent_kernel), _np(layer.bias), _np(zmask)
    Reff = R * _np(dmask) * dscale
    dh_new = np.concatenate([np.zeros((1, N, H)), _np(dy)], 0)
    if name == "LSTM":
        h, c, v = O.lstm_forward(W, Reff, b, _np(x), _np(h0[0]), _np(c0[0]), True, 0.3, m)
        dx, dW, dR, db = O.lstm_backward(W, Reff, b, _np(x), h, c, v, dh_new, np.zeros_like(dh_new), m)[:4]
        extra = {}
    else:
        g, gh, bh = _np(layer.gamma), _np(layer.gamma_h), _np(layer.beta_h)
        fwd = O.layer_norm_lstm_forward(W, Reff, b, g, gh, bh, _np(x), _np(h0[0]), _np(c0[0]), True, 0.3, m)
        h, c = fwd["h"], fwd["c"]
        back = O.layer_norm_lstm_backward(W, Reff, b, g, gh, bh, _np(x), fwd, dh_new, np.zeros_like(dh_new), m)
        dx, dW, dR, db = back["dx"], back["dW"], back["dR"], back["db"]
        extra = {"gamma": back["dgamma"], "gamma_h": back["dgamma_h"], "beta_h": back["dbeta_h"]}
    _close(y, h[1:], "output")
    for n_, length in enumerate([6, 2, 1, 4]):
        _close(hn[0, n_], h[length, n_], "h_n at lengths")
        _close(cn[0, n_], c[length, n_], "c_n at lengths")
    _close(x.grad, dx, "dx"); _close(layer.kernel.grad, dW, "dW"); _close(layer.bias.grad, db, "db")
    _close(layer.recurrent_kernel.grad, dR * _np(dmask) * dscale, "dR through the DropConnect mask")
    for k, ref in extra.items():
        _close(getattr(layer, k).grad, ref, k)
    # inference: no DropConnect, zoneout is the deterministic blend
    layer.eval()
    with torch.no_grad():
        ye, _ = layer(x, (h0, c0))
    if name == "LSTM":
        he = O.lstm_forward(W, R, b, _np(x), _np(h0[0]), _np(c0[0]), False, 0.3, m)[0]
    else:
        he = O.layer_norm_lstm_forward(W, R, b, g, gh, bh, _np(x), _np(h0[0]), _np(c0[0]), False, 0.3, m)["h"]
    _close(ye, he[1:], "inference output")


@pytest.mark.parametrize("name", ["GRU", "LayerNormGRU"])
def test_cpu_gru_layers_match_the_oracle(name):
    T, N, C, H = 5, 3, 6, 8
    torch.manual_seed(2)
    layer = getattr(haste_amd, name)(C, H, dropout=0.25, zoneout=0.2, batch_first=True).double()
    with torch.no_grad():
        for p_ in layer.parameters():
            p_.add_(0.1 * torch.randn_like(p_))
    xb = torch.randn(N, T, C, dtype=torch.float64, requires_grad=True)   # batch first
    dmask, dscale, zmask = _cpu_masks(layer, T, N, 12)
    torch.manual_seed(12)
    y, hn = layer(xb)
    dy = torch.randn(N, T, H, dtype=torch.float64)
    (y * dy).sum().backward()
    x = _np(xb).transpose(1, 0, 2)
    W, R, bx, br, m = (_np(layer.kernel), _np(layer.recurrent_kernel), _np(layer.bias),
                       _np(layer.recurrent_bias), _np(zmask))
    Reff = R * _np(dmask) * dscale
    dh_new = np.concatenate([np.zeros((1, N, H)), _np(dy).transpose(1, 0, 2)], 0)
    if name == "GRU":
        h, v = O.gru_forward(W, Reff, bx, br, x, np.zeros((N, H)), True, 0.2, m)
        dx, dW, dR, dbx, dbr = O.gru_backward(W, Reff, bx, br, x, h, v, dh_new, m)[:5]
        extra = {}
    else:
        g = _np(layer.gamma)
        fwd = O.layer_norm_gru_forward(W, Reff, bx, br, g, x, np.zeros((N, H)), True, 0.2, m)
        h = fwd["h"]
        back = O.layer_norm_gru_backward(W, Reff, bx, br, g, x, fwd, dh_new, m)
        dx, dW, dR, dbx, dbr = back["dx"], back["dW"], back["dR"], back["dbx"], back["dbr"]
        extra = {"gamma": back["dgamma"]}
    _close(y, h[1:].transpose(1, 0, 2), "output")
    _close(hn[0], h[-1], "h_n")
    _close(xb.grad, dx.transpose(1, 0, 2), "dx"); _close(layer.kernel.grad, dW, "dW")
    _close(layer.bias.grad, dbx, "dbx"); _close(layer.recurrent_bias.grad, dbr, "dbr")
    _close(layer.recurrent_kernel.grad, dR * _np(dmask) * dscale, "dR through the DropConnect mask")
    for k, ref in extra.items():
        _close(getattr(layer, k).grad, ref, k)


@pytest.mark.parametrize("name", ["IndRNN", "LayerNormIndRNN"])
def test_cpu_indrnn_layers_match_the_oracle(name):
    T, N, C, H = 7, 3, 4, 6
    torch.manual_seed(3)
    layer = getattr(haste_amd, name)(C, H, zoneout=0.25, return_state_sequence=True).double()
    with torch.no_grad():
        for p_ in layer.parameters():
            p_.add_(0.1 * torch.randn_like(p_))
    x = torch.randn(T, N, C, dtype=torch.float64, requires_grad=True)
    _, _, zmask = _cpu_masks(layer, T, N, 13)
    torch.manual_seed(13)
    y, states = layer(x)
    assert tuple(states.shape) == (1, T, N, H) and torch.equal(states[0], y)
    dy = torch.randn(T, N, H, dtype=torch.float64)
    (y * dy).sum().backward()
    W, u, b, m = _np(layer.kernel), _np(layer.recurrent_scale), _np(layer.bias), _np(zmask)
    gamma = _np(layer.gamma) if name == "LayerNormIndRNN" else None
    fwd = O.indrnn_forward(W, u, b, _np(x), np.zeros((N, H)), True, 0.25, m, gamma=gamma)
    dh_new = np.concatenate([np.zeros((1, N, H)), _np(dy)], 0)
    back = O.indrnn_backward(W, u, b, _np(x), fwd, dh_new, m, gamma=gamma)
    _close(y, fwd["h"][1:], "output")
    _close(x.grad, back["dx"], "dx"); _close(layer.kernel.grad, back["dW"], "dW")
    _close(layer.recurrent_scale.grad, back["du"], "du"); _close(layer.bias.grad, back["db"], "db")
    if gamma is not None:
        _close(layer.gamma.grad[0], back["dgamma"][0] if np.ndim(back["dgamma"]) == 2 else back["dgamma"], "dgamma")


def test_mixed_cpu_and_gpu_parameters_are_refused():
    layer = haste_amd.GRU(3, 4)

    class Fake:
        def __init__(self, is_cuda):
            self.is_cuda = is_cuda
    layer.parameters = lambda: [Fake(f) for f in (True, False, False, False)]
    with pytest.raises(ValueError, match="all be CUDA tensors or none"):
        layer._is_cuda()
