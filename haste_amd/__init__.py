"""haste_amd: MI355X (gfx950) implementation of Haste's fused-RNN hot path.

`haste_amd.ops` mirrors the op interface of the reference's PyTorch binding
(`haste_pytorch_lib.*_forward / *_backward`) on top of the C-ABI library
`libhaste_hip.so`; `haste_amd.lib` is the ctypes loader; `haste_amd.layers` holds the
torch.nn layers (LSTM, GRU, IndRNN, LayerNormLSTM, LayerNormGRU, LayerNormIndRNN) with the
class names and arguments of the reference's `haste_pytorch` package.
"""
from . import lib  # noqa: F401
from .layers import GRU, LSTM, IndRNN, LayerNormGRU, LayerNormIndRNN, LayerNormLSTM  # noqa: F401

__version__ = "0.1.0"
