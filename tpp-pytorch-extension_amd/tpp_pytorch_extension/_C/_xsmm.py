"""Reference: the _xsmm submodule (src/csrc/xsmm.cpp): libxsmm init, RNG seed
and the VNNI packing factor per dtype.  Only the packing factor has meaning on
the GPU; the weight layouts keep the reference's VNNI2 (bf16) / VNNI4 (int8)."""
import torch


def get_vnni_blocking(dtype):
    if dtype in (torch.bfloat16, torch.float16):
        return 2
    if dtype in (torch.int8, torch.uint8, torch.qint8):
        return 4
    return 1


def manual_seed(seed):
    torch.manual_seed(seed)


def init_libxsmm():
    return None
