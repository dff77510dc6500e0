"""Qwen2 decoder front-end on the fused linears: what the reference's
``tpp_pytorch_extension.llm.fused_qwen2_infer`` offers (Qwen2DecoderLayer /
FixQwen2DecoderLayer / OptimizeModelForQwen2, src/tpp_pytorch_extension/llm/fused_qwen2_infer.py:45-238)
on top of ``torch.classes.tpp_llm.Qwen2DecoderLayer`` (src/csrc/llm/fused_llm_infer.cpp:1289-1510).

A Qwen2 layer is the Llama layer with biases on the q, k and v projections: the
same RMSNorm, rotate-half rotary, KV cache, attention, SwiGLU and residual adds,
so everything but the parameter list is shared with fused_llama_infer.
"""
import os
import types

import torch

from .. import _lib
from .._lib import TppxError
from . import fused_llama_infer as _llama
from .fused_llama_infer import (LlamaDecoderLayer, LlamaDecoderLayerModule, LlamaModel_forward, TppCache,  # noqa: F401
                                generate_greedy, generate_greedy_graph)

__all__ = ["Qwen2DecoderLayer", "FixQwen2DecoderLayer", "OptimizeModelForQwen2", "Qwen2Model_forward", "TppCache",
           "generate_greedy", "generate_greedy_graph"]


class Qwen2DecoderLayer(LlamaDecoderLayer):
    """torch.classes.tpp_llm.Qwen2DecoderLayer(params, layer_idx, eps, H, max_positions, rotary_dim) with
    params = [ln_in gamma, Wq, Wk, Wv, Wo, ln_post gamma, Wg, Wu, Wd, bq, bk, bv, embed_positions]
    (fused_llm_infer.cpp:1304-1334).  forward is LlamaDecoderLayer's with the three biases on the fused q/k/v GEMM
    (fused_llm_infer.cpp:1462-1480); weight-format flags and the first-token copies behave as for Llama
    (fused_llm_infer.cpp:1336-1386, 1432-1447)."""

    def _take_params(self, params):
        if len(params) != 13:
            raise TppxError(_lib.EINVAL, f"Qwen2DecoderLayer takes 13 parameters, got {len(params)}")
        (self.t_Gi, self.t_Wq, self.t_Wk, self.t_Wv, self.t_Wp, self.t_Gpa, self.t_Wg, self.t_Wu, self.t_Wd,
         self.t_Bq, self.t_Bk, self.t_Bv, self.t_EP) = params


class Qwen2DecoderLayerModule(LlamaDecoderLayerModule):
    """What a transformers Qwen2DecoderLayer becomes (fused_qwen2_infer.py:45-101)."""


def FixQwen2DecoderLayer(self, bk=None, bc=None, layer_dtype=torch.bfloat16, weight_dtype="mxfp4",
                         embed_positions=None):
    """fused_qwen2_infer.py:104-177: quantize the seven linears of a transformers Qwen2DecoderLayer in place
    (FixLinear with [bk, bc] blocking) and attach the fused block; the q/k/v biases ride along as bf16."""
    import transformers
    from .llm_common import FixLinear
    if not isinstance(self, transformers.models.qwen2.modeling_qwen2.Qwen2DecoderLayer):
        return
    self.__class__ = Qwen2DecoderLayerModule
    self.features_block_size = bc
    self.layer_dtype = layer_dtype
    self.model_parallel = False
    for m in self.modules():
        if isinstance(m, torch.nn.Linear):
            FixLinear(m, bk, bc, layer_dtype, weight_dtype=weight_dtype)
    if not hasattr(self, "cpp_block"):
        at, mlp = self.self_attn, self.mlp
        for name in ("o_proj",):
            if getattr(at, name).bias is not None:
                raise NotImplementedError("a bias on the attention output projection is not part of Qwen2DecoderLayer")
        for lin in (mlp.gate_proj, mlp.up_proj, mlp.down_proj):
            if lin.bias is not None:
                raise NotImplementedError("mlp biases are not part of Qwen2DecoderLayer")

        def bias_of(lin):
            return None if lin.bias is None else lin.bias.data.to(torch.bfloat16).contiguous()

        params = [self.input_layernorm.weight.data.float(), at.q_proj.weight, at.k_proj.weight, at.v_proj.weight,
                  at.o_proj.weight, self.post_attention_layernorm.weight.data.float(), mlp.gate_proj.weight,
                  mlp.up_proj.weight, mlp.down_proj.weight, bias_of(at.q_proj), bias_of(at.k_proj), bias_of(at.v_proj),
                  embed_positions]
        self.cpp_block = Qwen2DecoderLayer(params, at.layer_idx, self.input_layernorm.variance_epsilon, at.head_dim,
                                           embed_positions.shape[1], at.head_dim)


Qwen2Model_forward = LlamaModel_forward  # fused_qwen2_infer.py:240-340: the same walk over the layers on a TppCache


def OptimizeModelForQwen2(model, dtype=torch.bfloat16, device="cuda", weight_dtype=None, quantize_lm_head=False):
    """fused_qwen2_infer.py:180-238 for one GPU: the rotary table from the model's own rotary_emb, every
    Qwen2DecoderLayer fused, the remaining nn.Linear (the lm_head) turned into a BlockedLinear, Qwen2Model.forward of
    this instance replaced.  Sliding-window attention is refused as in the reference (:184-187).  weight_dtype as for
    Llama (None = bf16 weights, "mxfp4", "qint8", "qint2"); the KV cache holds TPPX_KV_CAPACITY keys per sequence
    (default: the model's max_position_embeddings)."""
    import transformers
    from .llm_common import FixLinear
    q2 = transformers.models.qwen2.modeling_qwen2
    from .fused_llama_infer import layer_weight_dtype
    weight_dtype = layer_weight_dtype("OptimizeModelForQwen2", weight_dtype, dtype)
    if getattr(model.config, "use_sliding_window", False):
        raise NotImplementedError("use_sliding_window is not supported for Qwen2 yet!")
    model.config._attn_implementation = "tpp"
    embed_positions = None
    for m in model.modules():
        if isinstance(m, q2.Qwen2PreTrainedModel) and hasattr(m, "rotary_emb"):
            mp = m.rotary_emb.config.max_position_embeddings
            where = m.rotary_emb.inv_freq.device
            cs = m.rotary_emb(torch.empty([1], dtype=torch.float, device=where), torch.arange(mp, device=where).unsqueeze(0))
            embed_positions = torch.cat(cs, dim=0).view([2, mp, -1]).to(torch.float).to(device).contiguous()
            break
    if embed_positions is None:
        raise NotImplementedError("Unable to create embed_positions")
    model.to(device=device, dtype=dtype)
    with torch.no_grad():
        for m in list(model.modules()):
            if isinstance(m, q2.Qwen2DecoderLayer):
                FixQwen2DecoderLayer(m, 16, 64, dtype, weight_dtype, embed_positions)
        head_dtype = None if not quantize_lm_head else ("qint8" if quantize_lm_head is True else quantize_lm_head)
        for m in list(model.modules()):  # FixLinear is a no-op for the ones fixed above
            if not isinstance(m, torch.nn.Linear) or m.weight.shape[1] % 64:
                continue
            if head_dtype is not None:
                if m.weight.shape[0] % 32 == 0:
                    FixLinear(m, 16, 64, dtype, weight_dtype=head_dtype)
            elif m.weight.shape[0] % 100 == 0:
                FixLinear(m, 100, 64, dtype)
            elif m.weight.shape[0] % 64 == 0:
                FixLinear(m, 64, 64, dtype)
    for m in model.modules():
        if isinstance(m, q2.Qwen2Model):
            m._tpp_kv_capacity = int(os.environ.get("TPPX_KV_CAPACITY", embed_positions.shape[1]))
            m._tpp_norm_weight = m.norm.weight.data.float().contiguous()
            m._tpp_norm_eps = m.norm.variance_epsilon
            m.forward = types.MethodType(Qwen2Model_forward, m)
            m._tpp_core_model = True
    return model
