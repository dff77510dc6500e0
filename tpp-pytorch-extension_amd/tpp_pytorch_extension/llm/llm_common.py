"""LLM-side module API of the quantized linear.

Reference: ``src/tpp_pytorch_extension/llm/llm_common.py`` -- ``fc_plain``
(:379), ``BlockedLinear`` (:383-434), ``FixLinear`` (:437-515) and the
``TppCache`` wrapper handed around as ``past_key_values`` (:80-182), and the
small helpers callers of that module import next to them (``compare``,
``print_line_info``, ``BlockedLayerNorm``, and the process-group helpers in
their one-process form: ``get_rank`` / ``get_size`` / ``set_pg`` /
``all_reduce`` / ``ShardLinear``, :47-77, :429-434, :517-578).  The torch.jit
tracing wrapper of that file has no counterpart: decode steps are replayed
as HIP graphs instead.
"""
import inspect

import torch

from ..utils.blocked_layout import BlockedParameter, BlockedModule
from ..utils.xsmm import get_vnni_blocking
from .._C import _fused_llm_infer as fused_llm_cpp  # noqa: F401
from .._C import _qtype as qtype

USE_LOW_PREC_PARAMS = True
global_layer_dtype = torch.float32


def block(model):
    for m in model.modules():
        if hasattr(m, "maybe_block_params"):
            m.maybe_block_params()


def fc_plain(input, weight, bias=torch.Tensor(), parallel_dim=-1, split_sizes=[]):
    return torch.ops.tpp_llm.fc_plain(input, weight, bias, parallel_dim, split_sizes)


class BlockedLinear(BlockedModule, torch.nn.Linear):
    def maybe_block_params(self):
        if hasattr(self.weight, "block"):
            self.weight.block()
        if self.bias is not None and hasattr(self.bias, "block"):
            self.bias.block()

    def parallelize(self, dim, rank, size, block_size=1):
        if size <= 1:
            return
        raise NotImplementedError("tensor-parallel sharding is not part of the single-GPU path")

    def _io_dtype(self):
        return torch.bfloat16 if self.weight.is_quantized else self.weight.dtype

    def forward(self, input):
        self.maybe_block_params()
        bias = self.bias if self.bias is not None else torch.Tensor().to(self._io_dtype())
        input = input.to(self._io_dtype())
        parallel_dim = self.parallel_dim if self.model_parallel else -1
        split_sizes = self.split_sizes if hasattr(self, "split_sizes") else []
        return fc_plain(input, self.weight, bias, parallel_dim, split_sizes)

    # post-op variants used by the decoder layer
    # (src/csrc/llm/fused_llm_infer.cpp:1261-1273)
    def forward_add(self, input, residual, scale=1.0):
        bias = self.bias if self.bias is not None else torch.Tensor()
        return torch.ops.tpp_llm.fc_add(input.to(self._io_dtype()), self.weight, bias, residual, scale)

    def forward_silu(self, input):
        bias = self.bias if self.bias is not None else torch.Tensor()
        return torch.ops.tpp_llm.fc_silu(input.to(self._io_dtype()), self.weight, bias)

    def forward_mul(self, input, mul_in):
        bias = self.bias if self.bias is not None else torch.Tensor()
        return torch.ops.tpp_llm.fc_mul(input.to(self._io_dtype()), self.weight, bias, mul_in)


class BlockedLayerNorm(BlockedModule, torch.nn.LayerNorm):
    """llm_common.py:429-434: a LayerNorm whose parameters may be blocked.  bf16 inputs on the GPU run the
    lyr_norm kernel of the decoder blocks; anything else takes torch's own."""

    def maybe_block_params(self):
        if self.elementwise_affine:
            if hasattr(self.weight, "block"):
                self.weight.block()
            if self.bias is not None and hasattr(self.bias, "block"):
                self.bias.block()

    def forward(self, input):
        from .. import _ops
        if (input.is_cuda and input.dtype == torch.bfloat16 and self.elementwise_affine and self.bias is not None
                and len(self.normalized_shape) == 1 and self.normalized_shape[0] % 8 == 0
                and self.weight.dtype in (torch.float32, torch.bfloat16) and self.bias.dtype == self.weight.dtype):
            return _ops.layer_norm(input, self.weight.data, self.bias.data, self.eps)
        return super().forward(input)


def compare(ref, opt, name=""):
    """llm_common.py:47-63: print where `opt` leaves `ref` (relative to the mean magnitude), worst first."""
    ref, opt = ref.detach().float().cpu(), opt.detach().float().cpu()
    if ref.allclose(opt, atol=1e-6, rtol=1e-6):
        return True
    print(f"{name}: ref = {ref.reshape(-1)[:8]}, opt = {opt.reshape(-1)[:8]}")
    adiff = (ref - opt).abs()
    rdiff = adiff / ref.abs().mean()
    worst = torch.argsort(rdiff.reshape(-1), descending=True)[:8]
    for i in worst.tolist():
        print(f"{i}: ref: {ref.reshape(-1)[i].item():.7g} opt: {opt.reshape(-1)[i].item():.7g} "
              f"diff: {adiff.reshape(-1)[i].item():.7g}  rdiff: {rdiff.reshape(-1)[i].item():.7g}")
    return False


def print_line_info():
    """llm_common.py:70-77: where the caller is running and who called it."""
    cf = inspect.currentframe().f_back
    up = cf.f_back
    where = f"{up.f_code.co_filename}:{up.f_lineno}:{up.f_code.co_name}()" if up is not None else "<top>"
    print(f"Running At {cf.f_code.co_name}():{cf.f_lineno}  from {where}")


# Process-group helpers (llm_common.py:517-578).  This build runs one process on one GPU: rank 0 of 1, collectives
# are the identity; with an initialised torch.distributed group of more than one rank they refuse, because the
# tensor-parallel exchange steps of the decoder blocks are not built.
def get_rank():
    if torch.distributed.is_available() and torch.distributed.is_initialized():
        return torch.distributed.get_rank()
    return 0


def get_size():
    if torch.distributed.is_available() and torch.distributed.is_initialized():
        return torch.distributed.get_world_size()
    return 1


def _one_process(what):
    if get_size() > 1:
        raise NotImplementedError(f"{what}: tensor parallelism over {get_size()} ranks is not built (one GPU per model)")


def set_pg():
    _one_process("set_pg")


def all_reduce(t):
    _one_process("all_reduce")
    return t


def shm_allreduce(t):
    _one_process("shm_allreduce")
    return t


def ShardLinear(m, dim, rank, size, block_size=1):
    """llm_common.py:517-546: keep rank's share of an nn.Linear, split along the output (dim 0) or input (dim 1)
    features in whole blocks of block_size, and record every rank's share in m.split_sizes.  Pure slicing: it is
    what a tensor-parallel caller does before FixLinear; the exchange steps it implies are not built."""
    total = m.weight.shape[dim]
    if total % block_size:
        raise ValueError(f"dim_size ({total}) is not multiple of block_size ({block_size})")
    blocks = total // block_size
    cuts = [0] + [((blocks * (i + 1)) // size) * block_size for i in range(size)]
    lo, hi = cuts[rank], cuts[rank + 1]
    m.split_sizes = [cuts[i + 1] - cuts[i] for i in range(size)]
    with torch.no_grad():
        if dim == 0:
            m.weight.data = m.weight.data[lo:hi, :].contiguous()
            if m.bias is not None:
                m.bias.data = m.bias.data[lo:hi].contiguous()
        else:
            m.weight.data = m.weight.data[:, lo:hi].contiguous()
            if m.bias is not None:
                m.bias.data = m.bias.data / size


def _resolve_weight_dtype(weight_dtype, layer_dtype):
    if weight_dtype is None:
        return layer_dtype
    if isinstance(weight_dtype, str):
        if weight_dtype in ("mxfp4", "qint8", "qint2"):
            return weight_dtype
        try:
            return getattr(torch, weight_dtype)
        except AttributeError:
            raise ValueError(f"Unknown weight_dtype {weight_dtype}")
    if not isinstance(weight_dtype, torch.dtype):
        raise ValueError(f"weight_dtype must be either str or torch.dtype but is {type(weight_dtype)}")
    return weight_dtype


def FixLinear(self, bk=None, bc=None, layer_dtype=global_layer_dtype, parallel_dim=None, block_size=1,
              weight_dtype=None):
    """Turn an nn.Linear into a BlockedLinear: block the weight ([bk, bc] tiles,
    VNNI-packed for low precision) and quantize it when weight_dtype names a
    quantized format."""
    if not isinstance(self, torch.nn.Linear) or isinstance(self, BlockedLinear):
        return
    self.__class__ = BlockedLinear
    self.model_parallel = False
    if parallel_dim is not None:
        self.parallelize(parallel_dim, 0, 1, block_size=block_size)
    weight_dtype = _resolve_weight_dtype(weight_dtype, layer_dtype)

    self.weight = BlockedParameter(self.weight.data)
    if layer_dtype != torch.float32 and USE_LOW_PREC_PARAMS:
        v = get_vnni_blocking(layer_dtype)
        self.weight.set_blocking_param(([bk, [bc // v, v]], [0, 2, 3, 1, 4], layer_dtype))
    else:
        self.weight.set_blocking_param(([bk, bc], [0, 2, 3, 1]))
    if self.bias is not None:
        self.bias = BlockedParameter(self.bias.data)
        self.bias.set_blocking_param((None, None, layer_dtype))
    block(self)
    with torch.no_grad():
        if weight_dtype == "mxfp4":
            self.weight = torch.nn.Parameter(qtype.remap_and_quantize_mxfp4(self.weight), requires_grad=False)
        elif weight_dtype == "qint8":
            self.weight = torch.nn.Parameter(qtype.remap_and_quantize_qint8(self.weight), requires_grad=False)
        elif weight_dtype == "qint2":
            self.weight = torch.nn.Parameter(qtype.remap_and_quantize_qint2_intlv(self.weight), requires_grad=False)
        else:
            self.weight = torch.nn.Parameter(self.weight.data.to(weight_dtype), requires_grad=False)
        if self.bias is not None and isinstance(weight_dtype, str):
            self.bias = torch.nn.Parameter(self.bias.data.to(torch.bfloat16), requires_grad=False)


class TppCache:
    """past_key_values object of the optimized models (llm_common.py:80-182): a thin wrapper around the cache the
    fused decoder layers append to (`get_cpp()`).  The fused layers append keys inside their attention launch;
    `update` serves callers that hold key / value tensors themselves."""

    # what transformers' generate() asks of a cache object it did not create
    is_compileable = False
    is_sliding = False

    def __init__(self, capacity=0, **kwargs):
        from .fused_llama_infer import TppCache as _CoreCache
        self.tpp_cache = _CoreCache(capacity)
        self.static_mask = None  # an additive mask over the whole capacity that replaces the aligned one (graph replay)

    def __len__(self):
        return self.tpp_cache.size()

    def __getitem__(self, layer_idx):
        raise NotImplementedError

    def __iter__(self):
        raise NotImplementedError

    def update(self, key_states, value_states, layer_idx, cache_kwargs=None):
        """llm_common.py:113-124 of the reference: append to the layer and return [keys, values]."""
        return self.tpp_cache.update(key_states, value_states, layer_idx)

    def get_seq_length(self, layer_idx=0):
        return self.tpp_cache.get_seq_length(layer_idx)

    def get_max_length(self):
        return self.tpp_cache.get_capacity()

    def crop(self, max_length):
        seq_len = self.get_seq_length()
        if max_length < 0:
            max_length = seq_len - abs(max_length)
        if seq_len > max_length:
            self.tpp_cache.crop(max_length)

    def align_and_invert_mask(self, mask, inputs_embeds):
        if self.static_mask is not None:
            return self.static_mask
        if mask is None:
            mask = torch.ones((inputs_embeds.shape[0], inputs_embeds.shape[1]), device=inputs_embeds.device,
                              dtype=torch.bfloat16)
        return self.tpp_cache.align_and_invert_mask(mask.to(torch.bfloat16), torch.finfo(torch.bfloat16).min)

    def reorder_cache(self, beam_idx):
        self.tpp_cache.reorder_cache(beam_idx)

    def get_cpp(self):
        return self.tpp_cache


def generate_past_key_values(model, batch_size, seq_len, num_beams=1):
    return TppCache(capacity=seq_len)
