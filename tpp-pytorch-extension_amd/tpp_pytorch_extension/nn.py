"""``tpp_pytorch_extension.nn``: the module-level linear.

Reference: ``src/tpp_pytorch_extension/nn.py`` (fc_plain :5, TppLinear :9,
BlockedWeight :27, FixLinear :47, OptimizeForLinear :72).  ``FixLinear`` gains
the ``weight_dtype`` values ``"mxfp4"`` / ``"qint8"`` the LLM front-end uses;
unquantized blocked weights are not a GPU path here and raise in fc_plain.
"""
import torch

from .utils.xsmm import get_vnni_blocking
from ._C import _qtype as qtype


def fc_plain(input, weight, bias=torch.Tensor(), parallel_dim=-1, split_sizes=[]):
    return torch.ops.tpp_llm.fc_plain(input, weight, bias, parallel_dim, split_sizes)


class TppLinear(torch.nn.Linear):
    def forward(self, input):
        weight = self.weight
        if hasattr(self, "weight_2"):
            weight = self.weight_2
            rows = input.numel() // input.shape[-1]
            if hasattr(self, "weight_1") and rows > 192:
                weight = self.weight_1
        if self.bias is not None:
            bias = self.bias
        else:
            bias = torch.Tensor().to(torch.bfloat16 if weight.is_quantized else weight.dtype)
        input = input.to(torch.bfloat16 if weight.is_quantized else weight.dtype)
        return fc_plain(input, weight, bias)


def BlockedWeight(weight, bk, bc, dtype):
    """W[N, K] -> [N/bk, K/bc, bc, bk] (fp32) or [N/bk, K/bc, bc/v, bk, v] (VNNI-v)."""
    N, K = weight.shape
    if dtype == torch.float32:
        return weight.view(N // bk, bk, K // bc, bc).permute(0, 2, 3, 1).to(dtype).contiguous()
    v = get_vnni_blocking(dtype)
    return weight.view(N // bk, bk, K // bc, bc // v, v).permute(0, 2, 3, 1, 4).to(dtype).contiguous()


def _quantize_blocked(blocked, weight_dtype):
    if weight_dtype == "mxfp4":
        return qtype.remap_and_quantize_mxfp4(blocked)
    if weight_dtype == "qint8":
        return qtype.remap_and_quantize_qint8(blocked)
    if weight_dtype == "qint2":
        return qtype.remap_and_quantize_qint2_intlv(blocked)
    raise ValueError(f"Unknown weight_dtype {weight_dtype}")


def FixLinear(self, bkbc_2, bkbc_1=None, layer_dtype=None, weight_dtype=None):
    if not isinstance(self, torch.nn.Linear) or isinstance(self, TppLinear):
        return
    self.__class__ = TppLinear
    if layer_dtype is None:
        layer_dtype = self.weight.dtype
    if weight_dtype is None:
        weight_dtype = layer_dtype
    bk, bc = bkbc_2
    w2 = BlockedWeight(self.weight.data, bk, bc, layer_dtype)
    if isinstance(weight_dtype, str):
        with torch.no_grad():
            w2 = torch.nn.Parameter(_quantize_blocked(w2, weight_dtype), requires_grad=False)
    self.weight_2 = w2
    if bkbc_1 is not None and not isinstance(weight_dtype, str):
        bk, bc = bkbc_1
        self.weight_1 = BlockedWeight(self.weight.data, bk, bc, layer_dtype)
    if self.bias is not None:
        self.bias.data = self.bias.data.to(torch.bfloat16 if isinstance(weight_dtype, str) else layer_dtype)


def OptimizeForLinear(model, weight_dtype="mxfp4"):
    for m in model.modules():
        if isinstance(m, torch.nn.Linear):
            ofm, ifm = m.weight.shape
            if ofm % 64 == 0 and ifm % 64 == 0:
                FixLinear(m, (16, 64), (64, 64), torch.bfloat16, weight_dtype)
