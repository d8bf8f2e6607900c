"""The double-precision entry points (haste_hip_*_f64, what ForwardPass<double> /
BackwardPass<double> bind to) against the fp64 oracle: the float parity tests of every cell
are run again with float64 tensors and a tolerance of 1e-10."""
import numpy as np
import pytest

import test_gpu_cpp_api
import test_gpu_gru
import test_gpu_indrnn
import test_gpu_iterate
import test_gpu_layer_norm
import test_gpu_layer_norm_cells
import test_gpu_lstm
from util import host, relerr

pytestmark = pytest.mark.gpu

TOL64 = 1e-10
MODULES = (test_gpu_lstm, test_gpu_gru, test_gpu_layer_norm_cells, test_gpu_indrnn,
           test_gpu_layer_norm, test_gpu_iterate)
# (T, N, C, H): tiny, ragged, a few tiles, and one with more rows than a column-sum chunk
SHAPES = [(1, 1, 3, 4), (3, 2, 3, 4), (5, 3, 7, 5), (6, 17, 20, 36), (4, 16, 32, 64),
          (7, 33, 48, 128), (3, 70, 24, 300)]


def dev64(a):
    import torch
    if a is None:
        return torch.empty(0, 0, 0, dtype=torch.float64, device="cuda")
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float64)).cuda()


@pytest.fixture
def double_precision(monkeypatch):
    for mod in MODULES:
        monkeypatch.setattr(mod, "dev", dev64)
        if hasattr(mod, "TOL"):
            monkeypatch.setattr(mod, "TOL", TOL64)


@pytest.mark.parametrize("zoneout", [0.0, 0.3])
@pytest.mark.parametrize("T,N,C,H", SHAPES)
def test_f64_lstm_gru(double_precision, T, N, C, H, zoneout):
    test_gpu_lstm.test_lstm_training_forward_backward(T, N, C, H, zoneout)
    test_gpu_gru.test_gru_training_forward_backward(T, N, C, H, zoneout)


@pytest.mark.parametrize("zoneout", [0.0, 0.3])
@pytest.mark.parametrize("T,N,C,H", SHAPES)
def test_f64_layer_norm_cells(double_precision, T, N, C, H, zoneout):
    test_gpu_layer_norm_cells.test_layer_norm_lstm_training_forward_backward(T, N, C, H, zoneout)
    test_gpu_layer_norm_cells.test_layer_norm_gru_training_forward_backward(T, N, C, H, zoneout)


@pytest.mark.parametrize("layer_norm", [False, True])
@pytest.mark.parametrize("zoneout", [0.0, 0.3])
@pytest.mark.parametrize("T,N,C,H", SHAPES[1:])
def test_f64_indrnn(double_precision, T, N, C, H, zoneout, layer_norm):
    test_gpu_indrnn.test_indrnn_training_forward_backward(T, N, C, H, zoneout, layer_norm)


def test_f64_inference_dropconnect_determinism(double_precision):
    for zoneout in (0.0, 0.25):
        test_gpu_lstm.test_lstm_inference_forward(zoneout, 20, 16, 128, 256)
        test_gpu_gru.test_gru_inference_forward(zoneout, 20, 16, 128, 256)
    test_gpu_layer_norm_cells.test_layer_norm_lstm_inference_forward()
    test_gpu_lstm.test_lstm_dropconnect_fused_equals_premasked_weights(6, 8, 16, 64)
    test_gpu_gru.test_gru_dropconnect_fused_equals_premasked_weights(6, 8, 16, 64)
    test_gpu_lstm.test_lstm_accumulates_into_weight_gradients_and_is_deterministic()


@pytest.mark.parametrize("with_beta", [False, True])
@pytest.mark.parametrize("rows,D", [(1, 1), (3, 5), (7, 33), (100, 256), (37, 1000), (300, 2048), (5, 5000)])
def test_f64_layer_norm(double_precision, rows, D, with_beta):
    test_gpu_layer_norm.test_layer_norm_forward_backward(rows, D, with_beta)


# 0.25: the inference-mode blend takes the probability as float, as the reference's signatures
# do, so only a probability float represents exactly matches the oracle to 1e-10
@pytest.mark.parametrize("zoneout", [0.0, 0.25])
@pytest.mark.parametrize("T,N,C,H", [(3, 2, 3, 4), (4, 5, 7, 20), (3, 64, 48, 128)])
def test_f64_iterate(double_precision, T, N, C, H, zoneout):
    test_gpu_iterate.test_lstm_iterate(T, N, C, H, zoneout)
    test_gpu_iterate.test_gru_iterate(T, N, C, H, zoneout)


@pytest.mark.parametrize("trans_a,M,N,K", [(False, 1, 1, 1), (False, 37, 53, 29), (False, 128, 192, 64),
                                           (True, 70, 130, 45), (True, 5, 20, 33), (False, 300, 100, 1000),
                                           # few tiles, long contractions: cut along K into pieces
                                           (False, 64, 512, 2048), (True, 33, 70, 3001),
                                           # whole panels and columns inside the problem: the loads without
                                           # bounds checks (rows beyond M beyond the buffer's range)
                                           (True, 128, 256, 640), (False, 100, 128, 96), (True, 192, 128, 2080)])
@pytest.mark.parametrize("accumulate", [False, True])
def test_f64_gemm_and_transpose(trans_a, M, N, K, accumulate):
    from haste_amd import ops
    import torch
    r = np.random.default_rng(M * 7 + N * 3 + K)
    a = r.standard_normal((K, M) if trans_a else (M, K))
    b = r.standard_normal((K, N))
    c0 = r.standard_normal((M, N))
    out = dev64(c0)
    ops.gemm(dev64(a), dev64(b), out=out, trans_a=trans_a, accumulate=accumulate)
    ref = (a.T if trans_a else a) @ b + (c0 if accumulate else 0.0)
    assert relerr(host(out), ref) < 1e-13
    t = ops.transpose(dev64(a))
    assert torch.equal(t, dev64(a).t().contiguous())


def test_f64_layers_match_torch_nn():
    """haste_amd.LSTM / GRU in double against torch.nn.LSTM / GRU in double on the CPU."""
    import torch
    import haste_amd
    torch.manual_seed(3)
    T, N, C, H = 9, 5, 12, 20
    x = torch.randn(T, N, C, dtype=torch.float64)
    for ours_cls, theirs_cls in ((haste_amd.LSTM, torch.nn.LSTM), (haste_amd.GRU, torch.nn.GRU)):
        ours = ours_cls(C, H).double().cuda()
        theirs = theirs_cls(C, H).double()
        with torch.no_grad():
            for name, value in zip(("weight_ih_l0", "weight_hh_l0", "bias_ih_l0", "bias_hh_l0"),
                                   ours.to_native_weights()):
                getattr(theirs, name).copy_(value.cpu())
        xg = x.cuda().requires_grad_(True)
        xc = x.clone().requires_grad_(True)
        yo, _ = ours(xg)
        yt, _ = theirs(xc)
        assert relerr(host(yo), yt.detach().numpy()) < TOL64
        dy = torch.randn(T, N, H, dtype=torch.float64)
        yo.backward(dy.cuda())
        yt.backward(dy)
        assert relerr(host(xg.grad), xc.grad.numpy()) < TOL64


@pytest.mark.parametrize("cell", ["lstm", "layer_norm_lstm", "lstm_iterate", "gru", "layer_norm_gru",
                                  "gru_iterate", "indrnn", "layer_norm_indrnn"])
def test_f64_cpp_classes(monkeypatch, cell):
    """ForwardPass<double> / BackwardPass<double> of every namespace of include/haste.h."""
    monkeypatch.setattr(test_gpu_cpp_api, "DTYPE", np.float64)
    monkeypatch.setattr(test_gpu_cpp_api, "TOL", TOL64)
    T, N, C, H, zoneout = 9, 20, 24, 64, 0.3
    ln = "iterate" if cell.endswith("_iterate") else cell.startswith("layer_norm")
    if "lstm" in cell:
        test_gpu_cpp_api.test_cpp_lstm(T, N, C, H, zoneout, ln)
    elif "gru" in cell:
        test_gpu_cpp_api.test_cpp_gru(T, N, C, H, zoneout, ln)
    else:
        test_gpu_cpp_api.test_cpp_indrnn(T, N, C, H, zoneout, ln)
