"""Reference: src/tpp_pytorch_extension/utils/float8.py:25-32 -- the
``Tensor.cvt_to`` helper the blocked-layout classes rely on."""
import torch


def cvt_to(self, dtype):
    return self if self.dtype == dtype else self.to(dtype)


torch.Tensor.cvt_to = cvt_to
