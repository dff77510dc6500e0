"""GPT-J decoder front-end on the fused linears: what the reference's
``tpp_pytorch_extension.llm.fused_gptj_infer`` offers (GPTJBlock / FixGPTJBlock / OptimizeModelForGPTJ,
src/tpp_pytorch_extension/llm/fused_gptj_infer.py:46-304) on top of ``torch.classes.tpp_llm.GPTJBlock``
(src/csrc/llm/fused_llm_infer.cpp:607-848).

A GPT-J block normalises once (LayerNorm with bias), runs attention and the MLP side by side on the normalised
input and adds both to the residual:  out = fc_out(gelu(fc_in(h))) + out_proj(attn(h)) + x,  h = ln_1(x).  Rotary
embedding is on adjacent pairs of the first rotary_dim dims of every head, from a sin | cos table.
"""
import os
import types

import torch

from .. import _lib, _ops
from .._lib import TppxError
from .fused_llama_infer import (FormatSwitches, TppCache, check_layer_inputs, generate_greedy,  # noqa: F401
                                generate_greedy_graph, rotate_append_attend)

__all__ = ["GPTJBlock", "FixGPTJBlock", "OptimizeModelForGPTJ", "GPTJModel_forward", "create_sinusoidal_positions",
           "apply_rotary_pos_emb_gptj", "lyr_norm", "TppCache", "generate_greedy", "generate_greedy_graph"]

lyr_norm = _ops.layer_norm  # lyr_norm (fused_llm_infer.cpp:254-306)


def create_sinusoidal_positions(num_pos, dim):
    """fused_gptj_infer.py:46-51: f32 [num_pos][dim] = sin | cos of position * 10000^(-2i/dim)."""
    inv_freq = 1.0 / (10000 ** (torch.arange(0, dim, 2) / dim))
    sinusoid_inp = torch.einsum("i , j -> i j", torch.arange(num_pos, dtype=torch.float), inv_freq).float()
    return torch.cat((torch.sin(sinusoid_inp), torch.cos(sinusoid_inp)), dim=1)


def apply_rotary_pos_emb_gptj(t_in, t_emb_pos, t_pos, N, H):
    """In place on t_in [B][S][N*H] (fused_llm_infer.cpp:150-205); t_emb_pos f32 [MP][HR]; t_pos i64 [B_pos][S]."""
    L = _lib.lib()
    if not t_in.is_cuda or t_in.dtype != torch.bfloat16 or not t_in.is_contiguous():
        raise TppxError(_lib.EINVAL, "rotary: input must be a contiguous bfloat16 tensor on the GPU")
    B, S = t_in.shape[0], t_in.shape[1]
    _lib.check(L.tppx_rotary_gptj(t_in.data_ptr(), t_emb_pos.data_ptr(), t_pos.data_ptr(), B, S, N, H,
                                  t_emb_pos.shape[0], t_emb_pos.shape[1], t_pos.shape[0], _lib.stream_of(t_in)))
    return t_in


class GPTJBlock(FormatSwitches):
    """torch.classes.tpp_llm.GPTJBlock(params, layer_idx, eps, H, max_positions, rotary_dim) with
    params = [ln gamma, ln beta, Wq, Wk, Wv, Wo, W fc_in, b fc_in, W fc_out, b fc_out, embed_positions]
    (fused_llm_infer.cpp:622-648); forward as fused_llm_infer.cpp:740-846 with the q, k, v and fc_in GEMMs in one
    launch (the reference's default FUSED_QKV_GEMM = 2; GELU on the fourth)."""

    _weight_names = ("t_Wq", "t_Wk", "t_Wv", "t_Wp", "t_Wi", "t_Wo")

    def __init__(self, params, layer_idx, eps, H, max_positions, rotary_dim):
        if len(params) != 11:
            raise TppxError(_lib.EINVAL, f"GPTJBlock takes 11 parameters, got {len(params)}")
        (self.t_G, self.t_B, self.t_Wq, self.t_Wk, self.t_Wv, self.t_Wp, self.t_Wi, self.t_Bi, self.t_Wo, self.t_Bo,
         self.t_EP) = params
        self.layer_idx, self.eps, self.H = int(layer_idx), float(eps), int(H)
        self.max_positions, self.rotary_dim = int(max_positions), int(rotary_dim)
        if self.t_EP.dim() != 2 or self.t_EP.shape[1] % 16 or self.t_EP.shape[1] > self.H:
            raise TppxError(_lib.ESHAPE, f"GPTJBlock: embed_positions must be [max_positions][rotary_dim] with rotary_dim a "
                                         f"multiple of 16 and at most H = {self.H}, got {tuple(self.t_EP.shape)}")
        self.t_EP = self.t_EP.to(torch.float32).contiguous()  # the kernel reads an fp32 sin | cos table
        self._setup_formats()
        self.N = _ops.weight_nk(self.t_Wq)[0] // self.H

    def forward(self, inputs, cache, use_cache=True):
        """inputs = [hidden [B][S][hidden], additive mask [B][keys] or empty, position_ids i64 [B or 1][S]]; the S new
        keys go to cache positions get_seq_length() .. +S-1 and the caller advances the cache after the last block."""
        t_HS, t_am, t_pid = inputs[0], inputs[1], inputs[2]
        B, S, _ = t_HS.shape
        check_layer_inputs("GPTJBlock", t_HS, t_pid, cache)
        Wq, Wk, Wv, Wp, Wi, Wo = self._weights_for(B * S)
        t_res = t_HS
        h = lyr_norm(t_HS, self.t_G, self.t_B, self.eps)
        q, k, v, t_I = _ops.qkv_gemm(h, [Wq, Wk, Wv, Wi], [None, None, None, self.t_Bi])
        ctx = rotate_append_attend(q, k, v, t_am, t_pid, cache, self.layer_idx, B, S, self.N, self.N, self.H,
                                   self.t_EP, "gptj")
        t_SO = _ops.fc_plain(ctx, Wp, None)
        return [_ops.fc_add2(t_I, Wo, self.t_Bo, t_SO, t_res, 1.0)]


# ---------------------------------------------------------------------------
# Hugging Face front-end (src/tpp_pytorch_extension/llm/fused_gptj_infer.py:54-304)
# ---------------------------------------------------------------------------
class GPTJBlockModule(torch.nn.Module):
    """What a transformers GPTJBlock becomes (fused_gptj_infer.py:54-103)."""

    def forward(self, hidden_states, layer_past=None, attention_mask=None, position_ids=None, use_cache=False, **kwargs):
        if not hasattr(self, "cpp_block"):
            raise ValueError("cpp_block is not initialized")
        if position_ids is None:
            raise ValueError("position_ids is required")
        if layer_past is None:
            raise ValueError("the optimized block needs a TppCache (layer_past)")
        core = layer_past.get_cpp() if hasattr(layer_past, "get_cpp") else layer_past
        hs = hidden_states.to(torch.bfloat16).contiguous()
        mask = attention_mask.to(torch.bfloat16).contiguous() if attention_mask is not None else None
        return (self.cpp_block.forward([hs, mask, position_ids.contiguous()], core, use_cache)[0],)


def FixGPTJBlock(self, bk=None, bc=None, layer_dtype=torch.bfloat16, weight_dtype="mxfp4"):
    """fused_gptj_infer.py:106-172: quantize the six linears of a transformers GPTJBlock in place and attach the
    fused block; LayerNorm parameters and the two MLP biases ride along as bf16, the block's own sin | cos table
    (attn.embed_positions) as fp32."""
    import transformers
    from .llm_common import FixLinear
    if not isinstance(self, transformers.models.gptj.modeling_gptj.GPTJBlock):
        return
    self.__class__ = GPTJBlockModule
    self.features_block_size = bc
    self.layer_dtype = layer_dtype
    self.model_parallel = False
    for m in self.modules():
        if isinstance(m, torch.nn.Linear):
            FixLinear(m, bk, bc, layer_dtype, weight_dtype=weight_dtype)
    if not hasattr(self, "cpp_block"):
        at, mlp = self.attn, self.mlp
        if not hasattr(at, "embed_positions"):
            raise ValueError("embed_positions not created")
        dev = at.q_proj.weight.device

        def vec(t):
            return t.data.to(device=dev, dtype=torch.bfloat16).contiguous()

        params = [vec(self.ln_1.weight), vec(self.ln_1.bias), at.q_proj.weight, at.k_proj.weight, at.v_proj.weight,
                  at.out_proj.weight, mlp.fc_in.weight, vec(mlp.fc_in.bias), mlp.fc_out.weight, vec(mlp.fc_out.bias),
                  at.embed_positions.to(device=dev, dtype=torch.float32).contiguous()]
        self.cpp_block = GPTJBlock(params, at.layer_idx, self.ln_1.eps, at.head_dim, at.embed_positions.size(0),
                                   at.rotary_dim)


def GPTJModel_forward(self, input_ids=None, past_key_values=None, attention_mask=None, token_type_ids=None,
                      position_ids=None, inputs_embeds=None, use_cache=None, cache_position=None, **kwargs):
    """fused_gptj_infer.py:196-304: embeddings, position ids from the cache length, additive key mask from the 0/1
    attention mask, the blocks on a TppCache, final LayerNorm."""
    from transformers.modeling_outputs import BaseModelOutputWithPast
    from .llm_common import TppCache as HFTppCache
    if (input_ids is None) == (inputs_embeds is None):
        raise ValueError("You must specify exactly one of input_ids or inputs_embeds")
    if inputs_embeds is None:
        inputs_embeds = self.wte(input_ids)
    if not isinstance(past_key_values, HFTppCache):
        if past_key_values is None or past_key_values.get_seq_length() == 0:
            past_key_values = HFTppCache(capacity=self._tpp_kv_capacity)
        else:
            raise ValueError("past_key_values must be of TppCache type")
    past_seen = past_key_values.get_seq_length()
    S = inputs_embeds.shape[1]
    if cache_position is None:
        cache_position = torch.arange(past_seen, past_seen + S, device=inputs_embeds.device)
    if position_ids is None:
        position_ids = cache_position.unsqueeze(0)
    mask = None if attention_mask is None else past_key_values.align_and_invert_mask(attention_mask, inputs_embeds)
    hidden_states = inputs_embeds
    if token_type_ids is not None:
        hidden_states = hidden_states + self.wte(token_type_ids.view(-1, S))
    hidden_states = hidden_states.to(torch.bfloat16)
    for block in self.h:
        hidden_states = block(hidden_states, layer_past=past_key_values, attention_mask=mask,
                              position_ids=position_ids, use_cache=True)[0]
    past_key_values.get_cpp().advance(S)
    hidden_states = lyr_norm(hidden_states, self._tpp_ln_f[0], self._tpp_ln_f[1], self._tpp_ln_f[2])
    return BaseModelOutputWithPast(last_hidden_state=hidden_states, past_key_values=past_key_values)


def OptimizeModelForGPTJ(model, dtype=torch.bfloat16, device="cuda", weight_dtype=None):
    """fused_gptj_infer.py:175-193 for one GPU: every GPTJBlock fused, the lm_head turned into a BlockedLinear with
    the reference's 100 x 64 blocking (64 x 64 when the vocabulary does not divide), GPTJModel.forward of this
    instance replaced.  weight_dtype as for Llama (None = bf16 weights, "mxfp4", "qint8", "qint2"); the KV cache
    holds TPPX_KV_CAPACITY keys per sequence (default: the model's n_positions)."""
    import transformers
    from .llm_common import FixLinear
    gj = transformers.models.gptj.modeling_gptj
    from .fused_llama_infer import layer_weight_dtype
    weight_dtype = layer_weight_dtype("OptimizeModelForGPTJ", weight_dtype, dtype)
    tables = {}
    for name, m in model.named_modules():  # before the cast: the sin | cos tables are fp32 buffers
        if isinstance(m, gj.GPTJAttention):
            tables[name] = m.embed_positions.detach().to(torch.float32).clone()
    model.to(device=device, dtype=dtype)
    for name, m in model.named_modules():
        if name in tables:
            m.embed_positions = tables[name].to(device)
    with torch.no_grad():
        for m in list(model.modules()):
            if isinstance(m, gj.GPTJBlock):
                FixGPTJBlock(m, 16, 64, dtype, weight_dtype)
        for m in list(model.modules()):  # FixLinear is a no-op for the ones fixed above
            if not isinstance(m, torch.nn.Linear) or m.weight.shape[1] % 64:
                continue
            if m.weight.shape[0] % 100 == 0:
                FixLinear(m, 100, 64, dtype)
            elif m.weight.shape[0] % 64 == 0:
                FixLinear(m, 64, 64, dtype)
    for m in model.modules():
        if isinstance(m, gj.GPTJModel):
            m._tpp_kv_capacity = int(os.environ.get("TPPX_KV_CAPACITY", model.config.n_positions))
            m._tpp_ln_f = (m.ln_f.weight.data.to(torch.bfloat16).contiguous(),
                           m.ln_f.bias.data.to(torch.bfloat16).contiguous(), m.ln_f.eps)
            m.forward = types.MethodType(GPTJModel_forward, m)
            m._tpp_core_model = True
    return model
