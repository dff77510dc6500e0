"""Reference: src/tpp_pytorch_extension/utils/xsmm.py."""
from .._C import _xsmm as xsmm_cpp


def manual_seed(seed):
    xsmm_cpp.manual_seed(seed)


def get_vnni_blocking(dtype):
    return xsmm_cpp.get_vnni_blocking(dtype)
