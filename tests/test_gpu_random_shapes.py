"""Seeded random problem sizes through every cell (resident and step-wise regimes) against
the fp64 oracle: sizes nobody picked by hand, so that a geometry the fixed lists miss
(a tile height, a K chunking, a row too wide for one kernel) still gets exercised."""
import numpy as np
import pytest

import test_gpu_gru
import test_gpu_indrnn
import test_gpu_layer_norm_cells
import test_gpu_lstm

pytestmark = pytest.mark.gpu


def _shapes(seed, count, hidden):
    r = np.random.default_rng(seed)
    out = []
    for i in range(count):
        T = int(r.integers(1, 6))
        N = int(r.integers(1, 300)) if i % 2 else int(r.integers(1, 70))
        C = int(r.integers(2, 60))
        H = int(hidden(r))
        out.append((T, N, C, H, float(r.choice([0.0, 0.3]))))
    return out


RESIDENT = _shapes(11, 10, lambda r: r.integers(4, 560))
# beyond what LDS alone holds: backward only (577..1000), both passes (1028 and up), widths
# that are and are not multiples of 4 (part of the slice in registers, or step by step)
STEPWISE = [(T, min(N, 140), C, H, z) for T, N, C, H, z in
            _shapes(12, 8, lambda r: r.choice([577, 580, 644, 700, 801, 1028, 1100, 1301, 1537]))]
# any hidden size from the first that needs registers beside LDS to past the last that fits
# them, at batch sizes that take tiles of 16, 32 and 64 rows or fall back to single steps
REGISTER_ROWS = [(min(T, 3), min(N, 260), C, H, z) for T, N, C, H, z in
                 _shapes(13, 14, lambda r: r.integers(580, 2150))]


@pytest.mark.parametrize("T,N,C,H,zoneout", RESIDENT + STEPWISE + REGISTER_ROWS)
def test_random_sizes_lstm_gru(T, N, C, H, zoneout):
    test_gpu_lstm.test_lstm_training_forward_backward(T, N, C, H, zoneout)
    test_gpu_gru.test_gru_training_forward_backward(T, N, C, H, zoneout)


@pytest.mark.parametrize("T,N,C,H,zoneout", RESIDENT + STEPWISE[:4] + REGISTER_ROWS[:6])
def test_random_sizes_layer_norm_cells(T, N, C, H, zoneout):
    test_gpu_layer_norm_cells.test_layer_norm_lstm_training_forward_backward(T, N, C, H, zoneout)
    test_gpu_layer_norm_cells.test_layer_norm_gru_training_forward_backward(T, N, C, H, zoneout)


@pytest.mark.parametrize("T,N,C,H,zoneout", RESIDENT)
def test_random_sizes_indrnn(T, N, C, H, zoneout):
    test_gpu_indrnn.test_indrnn_training_forward_backward(T, N, C, H, zoneout, False)
    test_gpu_indrnn.test_indrnn_training_forward_backward(T, N, C, H, zoneout, True)
