"""MI355X-native build of the weight-quantized LLM linear path, behind the
import paths and operator names of tpp_pytorch_extension.

    import tpp_pytorch_extension
    from tpp_pytorch_extension._C import _qtype
    w = _qtype.remap_and_quantize_mxfp4(blocked_weight)
    y = torch.ops.tpp_llm.fc_plain(x, w, bias, -1, [])
"""
import torch

from . import _lib
from . import _C
from .utils.xsmm import get_vnni_blocking, manual_seed
from .utils import blocked_layout
from .utils import float8
from . import qtypes
from . import nn

__all__ = ["_C", "qtypes", "nn", "blocked_layout", "get_vnni_blocking", "manual_seed"]


def reset_debug_timers():
    """The reference resets its per-scope CPU timers here (src/csrc/init.cpp:42);
    GPU work is profiled with rocprofv3 / torch.profiler instead, so this is a no-op."""


def print_debug_timers(tid=0, detailed=True):
    """See reset_debug_timers."""
