"""Host-side behaviour of the torch.nn layers (no GPU needed): parameter names, shapes and
initial values as in the reference's haste_pytorch layers, the native-weight maps checked
against torch.nn.LSTM / torch.nn.GRU through the oracle, argument validation, and the
refusal to run on CPU tensors."""
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


def test_argument_validation_and_cpu_refusal():
    with pytest.raises(ValueError):
        haste_amd.LSTM(4, 4, dropout=1.5)
    with pytest.raises(ValueError):
        haste_amd.GRU(4, 4, zoneout=-0.1)
    layer = haste_amd.LSTM(4, 4)
    with pytest.raises(RuntimeError, match="no CPU path"):
        layer(torch.zeros(2, 3, 4))
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
