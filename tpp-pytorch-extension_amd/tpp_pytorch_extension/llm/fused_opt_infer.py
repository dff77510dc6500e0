"""OPT decoder front-end on the fused linears: what the reference's
``tpp_pytorch_extension.llm.fused_opt_infer`` offers (OPTDecoderLayer / FixOPTDecoderLayer / OptimizeModelForOPT,
src/tpp_pytorch_extension/llm/fused_opt_infer.py:45-300) on top of ``torch.classes.tpp_llm.OPTDecoderLayer``
(src/csrc/llm/fused_llm_infer.cpp:850-1069).

An OPT layer has biases on all six linears, LayerNorm (with bias) before or after each half
(do_layer_norm_before), a ReLU MLP and no rotary embedding: positions are a learned embedding added to the token
embeddings in front of the first layer.
"""
import os
import types

import torch

from .. import _lib, _ops
from .._lib import TppxError
from .fused_llama_infer import (FormatSwitches, TppCache, check_layer_inputs, generate_greedy,  # noqa: F401
                                generate_greedy_graph, rotate_append_attend)

__all__ = ["OPTDecoderLayer", "FixOPTDecoderLayer", "OptimizeModelForOPT", "OPTDecoder_forward", "lyr_norm",
           "TppCache", "generate_greedy", "generate_greedy_graph"]

lyr_norm = _ops.layer_norm  # lyr_norm (fused_llm_infer.cpp:254-306)


class OPTDecoderLayer(FormatSwitches):
    """torch.classes.tpp_llm.OPTDecoderLayer(params, layer_idx, eps1, eps2, H, do_layer_norm_before) with
    params = [ln1 gamma, ln1 beta, ln2 gamma, ln2 beta, Wq, bq, Wk, bk, Wv, bv, Wo, bo, W fc1, b fc1, W fc2, b fc2]
    (fused_llm_infer.cpp:878-897); forward as fused_llm_infer.cpp:985-1067.  inputs = [hidden, mask] (no position
    ids: the layer does not rotate)."""

    _weight_names = ("t_Wq", "t_Wk", "t_Wv", "t_Wp", "t_Wi", "t_Wo")

    def __init__(self, params, layer_idx, eps1, eps2, H, do_layer_norm_before):
        if len(params) != 16:
            raise TppxError(_lib.EINVAL, f"OPTDecoderLayer takes 16 parameters, got {len(params)}")
        (self.t_G1, self.t_B1, self.t_G2, self.t_B2, self.t_Wq, self.t_Bq, self.t_Wk, self.t_Bk, self.t_Wv, self.t_Bv,
         self.t_Wp, self.t_Bp, self.t_Wi, self.t_Bi, self.t_Wo, self.t_Bo) = params
        self.layer_idx, self.eps1, self.eps2, self.H = int(layer_idx), float(eps1), float(eps2), int(H)
        self.do_layer_norm_before = bool(do_layer_norm_before)
        self._pos = {}
        self._setup_formats()
        self.N = _ops.weight_nk(self.t_Wq)[0] // self.H

    def forward(self, inputs, cache, use_cache=True):
        t_HS = inputs[0]
        t_am = inputs[1] if len(inputs) > 1 else None
        B, S, _ = t_HS.shape
        pos = self._pos.get((t_HS.device, S))  # never read (nothing is rotated), but the append launch takes one
        if pos is None:
            pos = self._pos[(t_HS.device, S)] = torch.zeros((1, S), dtype=torch.int64, device=t_HS.device)
        check_layer_inputs("OPTDecoderLayer", t_HS, pos, cache)
        Wq, Wk, Wv, Wp, Wi, Wo = self._weights_for(B * S)
        t_res = t_HS
        if self.do_layer_norm_before:
            t_HS = lyr_norm(t_HS, self.t_G1, self.t_B1, self.eps1)
        q, k, v = _ops.qkv_gemm(t_HS, [Wq, Wk, Wv], [self.t_Bq, self.t_Bk, self.t_Bv])
        ctx = rotate_append_attend(q, k, v, t_am, pos, cache, self.layer_idx, B, S, self.N, self.N, self.H, None, None)
        t_HS = _ops.fc_add(ctx, Wp, self.t_Bp, t_res, 1.0)
        if not self.do_layer_norm_before:
            t_HS = lyr_norm(t_HS, self.t_G1, self.t_B1, self.eps1)
        t_res = t_HS
        if self.do_layer_norm_before:
            t_HS = lyr_norm(t_HS, self.t_G2, self.t_B2, self.eps2)
        t_HS = _ops.fc_relu(t_HS, Wi, self.t_Bi)
        t_HS = _ops.fc_add(t_HS, Wo, self.t_Bo, t_res, 1.0)
        if not self.do_layer_norm_before:
            t_HS = lyr_norm(t_HS, self.t_G2, self.t_B2, self.eps2)
        return [t_HS]


# ---------------------------------------------------------------------------
# Hugging Face front-end (src/tpp_pytorch_extension/llm/fused_opt_infer.py:45-300)
# ---------------------------------------------------------------------------
class OPTDecoderLayerModule(torch.nn.Module):
    """What a transformers OPTDecoderLayer becomes (fused_opt_infer.py:45-106)."""

    def forward(self, hidden_states, attention_mask=None, past_key_values=None, use_cache=False, position_ids=None,
                past_key_value=None, **kwargs):
        if not hasattr(self, "cpp_block"):
            raise ValueError("cpp_block is not initialized")
        cache = past_key_values if past_key_values is not None else past_key_value
        if cache is None:
            raise ValueError("the optimized decoder layer needs a TppCache (past_key_values)")
        core = cache.get_cpp() if hasattr(cache, "get_cpp") else cache
        hs = hidden_states.to(torch.bfloat16).contiguous()
        mask = attention_mask.to(torch.bfloat16).contiguous() if attention_mask is not None else None
        return self.cpp_block.forward([hs, mask], core, use_cache)[0]


def FixOPTDecoderLayer(self, bk=None, bc=None, layer_dtype=torch.bfloat16, weight_dtype="mxfp4"):
    """fused_opt_infer.py:109-172: quantize the six linears of a transformers OPTDecoderLayer in place and attach
    the fused block; LayerNorm parameters and the six biases ride along as bf16."""
    import transformers
    from .llm_common import FixLinear
    if not isinstance(self, transformers.models.opt.modeling_opt.OPTDecoderLayer):
        return
    self.__class__ = OPTDecoderLayerModule
    self.features_block_size = bc
    self.layer_dtype = layer_dtype
    self.model_parallel = False
    for m in self.modules():
        if isinstance(m, torch.nn.Linear):
            FixLinear(m, bk, bc, layer_dtype, weight_dtype=weight_dtype)
    if not hasattr(self, "cpp_block"):
        at = self.self_attn
        dev = at.q_proj.weight.device

        def vec(t):
            return None if t is None else t.data.to(device=dev, dtype=torch.bfloat16).contiguous()

        params = [vec(self.self_attn_layer_norm.weight), vec(self.self_attn_layer_norm.bias),
                  vec(self.final_layer_norm.weight), vec(self.final_layer_norm.bias),
                  at.q_proj.weight, vec(at.q_proj.bias), at.k_proj.weight, vec(at.k_proj.bias),
                  at.v_proj.weight, vec(at.v_proj.bias), at.out_proj.weight, vec(at.out_proj.bias),
                  self.fc1.weight, vec(self.fc1.bias), self.fc2.weight, vec(self.fc2.bias)]
        self.cpp_block = OPTDecoderLayer(params, at.layer_idx, self.self_attn_layer_norm.eps,
                                         self.final_layer_norm.eps, at.head_dim, self.do_layer_norm_before)


def OPTDecoder_forward(self, input_ids=None, attention_mask=None, past_key_values=None, inputs_embeds=None,
                       use_cache=None, position_ids=None, **kwargs):
    """fused_opt_infer.py:205-300: token embeddings + learned position embeddings (positions counted over the 0/1
    attention mask), the additive key mask, the layers on a TppCache, final LayerNorm and output projection."""
    from transformers.modeling_outputs import BaseModelOutputWithPast
    from .llm_common import TppCache as HFTppCache
    if (input_ids is None) == (inputs_embeds is None):
        raise ValueError("You must specify exactly one of input_ids or inputs_embeds")
    if input_ids is not None:
        input_ids = input_ids.view(-1, input_ids.shape[-1])
    if inputs_embeds is None:
        inputs_embeds = self.embed_tokens(input_ids)
    if not isinstance(past_key_values, HFTppCache):
        if past_key_values is None or past_key_values.get_seq_length() == 0:
            past_key_values = HFTppCache(capacity=self._tpp_kv_capacity)
        else:
            raise ValueError("past_key_values must be of TppCache type")
    past_seen = past_key_values.get_seq_length()
    S = inputs_embeds.shape[1]
    if attention_mask is None:
        attention_mask = torch.ones(inputs_embeds.shape[0], past_seen + S, device=inputs_embeds.device)
    mask = past_key_values.align_and_invert_mask(attention_mask, inputs_embeds)
    if position_ids is None:
        position_ids = torch.cumsum(attention_mask, dim=1)
        position_ids = (position_ids * attention_mask - 1).long()
        position_ids = position_ids[:, past_seen:]  # cut positions if there are cached keys
    pos_embeds = self.embed_positions(attention_mask, past_seen, position_ids=position_ids)
    if self.project_in is not None:
        inputs_embeds = self.project_in(inputs_embeds)
    hidden_states = (inputs_embeds + pos_embeds.to(inputs_embeds.device)).to(torch.bfloat16)
    for layer in self.layers:
        hidden_states = layer(hidden_states, attention_mask=mask, past_key_values=past_key_values, use_cache=True)
    past_key_values.get_cpp().advance(S)
    if self.final_layer_norm is not None:
        hidden_states = lyr_norm(hidden_states, self._tpp_ln_f[0], self._tpp_ln_f[1], self._tpp_ln_f[2])
    if self.project_out is not None:
        hidden_states = self.project_out(hidden_states)
    return BaseModelOutputWithPast(last_hidden_state=hidden_states, past_key_values=past_key_values)


def OptimizeModelForOPT(model, dtype=torch.bfloat16, device="cuda", weight_dtype=None):
    """fused_opt_infer.py:175-203 for one GPU: every OPTDecoderLayer fused, every remaining nn.Linear (lm_head,
    project_in / project_out) turned into a bf16 BlockedLinear with 16 x 64 blocking as the reference does,
    OPTDecoder.forward of this instance replaced.  weight_dtype as for Llama (None = bf16 weights, "mxfp4", "qint8",
    "qint2"); the KV cache holds TPPX_KV_CAPACITY keys per sequence (default: max_position_embeddings)."""
    import transformers
    from .llm_common import FixLinear
    op = transformers.models.opt.modeling_opt
    from .fused_llama_infer import layer_weight_dtype
    weight_dtype = layer_weight_dtype("OptimizeModelForOPT", weight_dtype, dtype)
    for i, l in enumerate(model.model.decoder.layers):
        if not hasattr(l.self_attn, "layer_idx") or l.self_attn.layer_idx is None:
            l.self_attn.layer_idx = i
    model.to(device=device, dtype=dtype)
    with torch.no_grad():
        for m in list(model.modules()):
            if isinstance(m, op.OPTDecoderLayer):
                FixOPTDecoderLayer(m, 16, 64, dtype, weight_dtype)
        for m in list(model.modules()):  # FixLinear is a no-op for the ones fixed above
            if isinstance(m, torch.nn.Linear) and m.weight.shape[1] % 64 == 0 and m.weight.shape[0] % 16 == 0:
                FixLinear(m, 16, 64, dtype)
    for m in model.modules():
        if isinstance(m, op.OPTDecoder):
            m._tpp_kv_capacity = int(os.environ.get("TPPX_KV_CAPACITY", model.config.max_position_embeddings))
            if m.final_layer_norm is not None:
                m._tpp_ln_f = (m.final_layer_norm.weight.data.to(torch.bfloat16).contiguous(),
                               m.final_layer_norm.bias.data.to(torch.bfloat16).contiguous(), m.final_layer_norm.eps)
            m.forward = types.MethodType(OPTDecoder_forward, m)
            m._tpp_core_model = True
    return model
