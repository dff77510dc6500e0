"""Python-level quantized-tensor helpers.

Reference: ``src/tpp_pytorch_extension/qtypes.py``.  (The reference file also
imports ``remap_and_quantize_qint4`` whose native registration is commented out,
``src/csrc/qtypes.cpp:1090``; that name is not re-exported here.)
"""
import torch

from ._C import _qtype as qtype
from ._C._qtype import (  # noqa: F401
    q_per_block_scales,
    q_per_block_block_size,
    q_per_block_axis,
    q_per_block_pack_size,
    remap_and_quantize_mxfp4,
    remap_and_quantize_qint8,
    quantize_mxfp4,
    quantize_int8sym,
    quantize_int4sym,
    create_qtensor_int8sym,
)
from ._ops import q_per_block_qval as _qval


def q_per_block_qval(qtensor: torch.Tensor):
    """Raw storage of the quantized tensor in the reference layout.  For qint8
    this is the int8 tensor of the logical shape (qtypes.py:27-29 of the
    reference); for quint4x2 the logical shape counts nibbles, so the packed
    uint8 bytes ``[N/32, K/64, 32, 32]`` are returned."""
    return _qval(qtensor)


def get_qval(qtensor: torch.Tensor):
    return q_per_block_qval(qtensor)


def get_scales(qtensor: torch.Tensor):
    return q_per_block_scales(qtensor)


def get_axis(qtensor: torch.Tensor):
    return q_per_block_axis(qtensor)


def get_block_size(qtensor: torch.Tensor):
    return q_per_block_block_size(qtensor)
