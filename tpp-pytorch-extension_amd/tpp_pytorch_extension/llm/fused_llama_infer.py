"""Llama decoder layer on the GPU: the reference's fused decoder block
(`LlamaDecoderLayer::_forward`, src/csrc/llm/fused_llm_infer.cpp:1195-1286) and
its KV cache (`TppCache` / `LayerCache`, src/csrc/llm/attn.h:164-404) for the
decode step (one new token per sequence) and for prompt processing, built from
the quantized linears and the decoder-side kernels of libtppx_hip.so.

`LlamaDecoderLayer` keeps the constructor and `forward` signature of
`torch.classes.tpp_llm.LlamaDecoderLayer` (fused_llm_infer.cpp:1084-1110,
1186-1192, 1603-1606); `TppCache` keeps the reference's method names.

`OptimizeModelForLlama` / `FixLlamaDecoderLayer` / `LlamaModel_forward` are the
front-end of src/tpp_pytorch_extension/llm/fused_llama_infer.py:104-336 for a
Hugging Face `LlamaForCausalLM`: every decoder layer is replaced by one
`LlamaDecoderLayer` call, the model's forward runs on a `TppCache`.
"""
import math
import os
import types

import torch

from .. import _lib, _ops
from .._lib import TppxError


# ---------------------------------------------------------------------------
# operator wrappers
# ---------------------------------------------------------------------------
def _bf16_cuda(t, name):
    if not t.is_cuda or t.dtype != torch.bfloat16:
        raise TppxError(_lib.EINVAL, f"{name} must be a bfloat16 tensor on the GPU")
    return t.contiguous()


rms_norm = _ops.rms_norm  # llama_rms_norm (fused_llm_infer.cpp:337-363)

# decode steps: rotary embedding + cache append inside the attention launch (TPPX_FUSE_ROTARY=0: separate launch)
FUSE_ROTARY = os.environ.get("TPPX_FUSE_ROTARY", "1") == "1"
# Greedy decoding: argmax, the counters and the next token's embedding row in one launch at the end of a decode step
# (tppx_greedy_next) instead of torch's argmax / copy / add / index_select kernels.  TPPX_FUSE_GREEDY=0 keeps those.
FUSE_GREEDY = os.environ.get("TPPX_FUSE_GREEDY", "1") == "1"


# Weight-format switches of the decoder layers, read once at import like the reference's file-statics
# (src/csrc/llm/fused_llm_infer.cpp:35-45).  A layer built from UNQUANTIZED blocked weights quantizes them itself
# under USE_MXFP4 / USE_QINT8 / USE_QINT2 (the decode-step copy); passes of FT_OPT_SIZE or more tokens run on the
# first-token copy instead, which stays unquantized unless USE_*_FT picks a format for it, and is only used when
# TPP_CACHE_REMAPPED_WEIGHTS is on.
def _env_int(name, default):
    v = os.environ.get(name, "")
    return int(v) if v.strip() else default


SUMS_GATE_UP_ROWS = _env_int("TPPX_SUMS_GATE_UP_ROWS", 4)  # decode steps of up to this many rows normalise inside gate/up
TPP_CACHE_REMAPPED_WEIGHTS = _env_int("TPP_CACHE_REMAPPED_WEIGHTS", 1)
FT_OPT_SIZE = _env_int("FT_OPT_SIZE", 256)
USE_MXFP4 = _env_int("USE_MXFP4", 0)
USE_MXFP4_FT = _env_int("USE_MXFP4_FT", 0)
USE_QINT8 = _env_int("USE_QINT8", 0)
USE_QINT8_FT = _env_int("USE_QINT8_FT", 0)
USE_QINT2 = _env_int("USE_QINT2", 0)
USE_QINT2_FT = _env_int("USE_QINT2_FT", 0)


def wt_tensor_for_first_token(t):
    """wt_tensor_for_first_token (fused_llm_infer.cpp:365-420): the copy of an unquantized weight that passes of
    FT_OPT_SIZE or more tokens run on.  The reference re-blocks it to 64 output channels per block for its CPU
    GEMM; the kernels here read any blocking through the native tiles made on first use, so unquantized stays as
    it is -- and USE_QINT8_FT / USE_MXFP4_FT / USE_QINT2_FT (in the reference's order) quantize it."""
    if USE_QINT8_FT == 1:
        return _ops.remap_and_quantize_qint8(t)
    if USE_MXFP4_FT == 1:
        return _ops.remap_and_quantize_mxfp4(t)
    if USE_QINT2_FT == 1:
        return _ops.remap_and_quantize_qint2_intlv(t)
    return t


def apply_rotary_pos_emb_llama(t_in, t_emb_pos, t_pos, N, H):
    """In place on t_in [B][S][N*H] (fused_llm_infer.cpp:207-253); t_emb_pos f32 [2][MP][HR]; t_pos i64 [B_pos][S]."""
    L = _lib.lib()
    if not t_in.is_cuda or t_in.dtype != torch.bfloat16 or not t_in.is_contiguous():
        raise TppxError(_lib.EINVAL, "rotary: input must be a contiguous bfloat16 tensor on the GPU")
    B, S = t_in.shape[0], t_in.shape[1]
    _lib.check(L.tppx_rotary_llama(t_in.data_ptr(), t_emb_pos.data_ptr(), t_pos.data_ptr(), B, S, N, H,
                                   t_emb_pos.shape[1], t_emb_pos.shape[2], t_pos.shape[0], _lib.stream_of(t_in)))
    return t_in


class TppCache:
    """KV cache of all layers (TppCache, src/csrc/llm/attn.h:229-404).  Storage per layer is
    `[B][Nkv][capacity][H]` bf16 for keys and for values (the reference's blocked
    `[S1][B][N][32][H]` layouts are internal to its CPU kernels; nothing outside the class sees them).
    The sequence length lives in a device int32 so that a decode step can be replayed as a graph."""

    block_size = 32  # LayerCache::block_size, used by align_and_invert_mask
    SLAB_BYTES = 64 << 20  # layers are allocated together while a group stays under this

    def __init__(self, capacity=0):
        self.capacity = int(capacity)
        self.layers = {}          # layer_idx -> (k, v)
        self._spare = {}          # layer_idx -> [2][B][Nkv][capacity][H], zeroed storage waiting for that layer
        self.seq_len_dev = None   # int32 [1]: keys in the cache (same for every layer)
        self._host_len = 0
        self._sync_len = 0        # length every layer had when the fused layers last advanced the cache
        self._layer_len = {}      # layers that update() has moved since then
        # decode steps: row sums of squares of the residual stream, handed from the GEMM that writes it to the
        # GEMM behind the next RMSNorm (two tables: after attention, after the MLP) + the tensor the second belongs to
        self._sums = None
        self._sums_of = None

    # -- reference method names -------------------------------------------------
    def get_seq_length(self, layer_idx=0):
        return self._layer_len.get(layer_idx, self._host_len if layer_idx == 0 else self._sync_len)

    def get_capacity(self):
        return self.capacity

    def size(self):
        return len(self.layers)

    def get(self, layer_idx):
        k, v = self.layers[layer_idx]
        return [k[:, :, :self._host_len], v[:, :, :self._host_len]]

    def crop(self, max_length):
        if self._host_len > max_length:
            self._host_len = int(max_length)
            self.seq_len_dev.fill_(self._host_len)
        self._sync_len = min(self._sync_len, int(max_length))
        self._layer_len = {i: min(n, int(max_length)) for i, n in self._layer_len.items()}

    def reorder_cache(self, beam_idx):
        """attn.h:327-366 (beam search): afterwards sequence b continues the keys and values sequence beam_idx[b]
        held.  The reference records the indices and gathers inside attention; here the rows move once per step."""
        beam_idx = beam_idx.to(torch.int64)
        for i, (k, v) in self.layers.items():
            if beam_idx.numel() != k.shape[0]:
                raise TppxError(_lib.ESHAPE, f"TppCache.reorder_cache: {beam_idx.numel()} indices for {k.shape[0]} sequences")
            n = self._host_len
            k[:, :, :n].copy_(k[:, :, :n].index_select(0, beam_idx.to(k.device)))
            v[:, :, :n].copy_(v[:, :, :n].index_select(0, beam_idx.to(v.device)))
        self._sums_of = None

    def align_and_invert_mask(self, t_mask, pad_value=-10000.0):
        """attn.h:310-322: [B][S] 0/1 mask -> additive mask padded to a multiple of 32 keys."""
        B, S = t_mask.shape
        S_pad = (S + self.block_size - 1) // self.block_size * self.block_size
        mask_pad = t_mask.new_full((B, S_pad), pad_value)
        mask_pad[:, :S].masked_fill_(t_mask == 1, 0.0)
        return mask_pad

    # -- storage ------------------------------------------------------------------
    def _ensure(self, layer_idx, B, Nkv, H, device):
        if self.capacity <= 0:
            raise TppxError(_lib.EINVAL, "TppCache: give the cache a capacity (keys per sequence) before use")
        if layer_idx not in self.layers:
            # Small caches come several layers to an allocation (the layers of a pass ask in ascending order): one
            # allocator call and one fill for up to eight layers' keys and values instead of two per layer, which
            # at prompts of a hundred tokens were a device allocation per layer on every fresh cache.
            shape = (B, Nkv, self.capacity, H)
            spare = self._spare.pop(layer_idx, None)
            if spare is None or tuple(spare.shape[1:]) != shape or spare.device != torch.device(device):
                per_layer = 4 * B * Nkv * self.capacity * H
                group = max(1, min(8, self.SLAB_BYTES // max(per_layer, 1)))
                slab = torch.zeros((group, 2) + shape, dtype=torch.bfloat16, device=device)
                self._spare = {layer_idx + j: slab[j] for j in range(1, group) if layer_idx + j not in self.layers}
                spare = slab[0]
            self.layers[layer_idx] = (spare[0], spare[1])
        if self.seq_len_dev is None:
            self.seq_len_dev = torch.zeros(1, dtype=torch.int32, device=device)
        return self.layers[layer_idx]

    def fill_(self, layer_idx, keys, values):
        """Load a context: keys / values bf16 [B][Nkv][S][H] become positions 0..S-1."""
        B, Nkv, S, H = keys.shape
        k, v = self._ensure(layer_idx, B, Nkv, H, keys.device)
        k[:, :, :S].copy_(keys)
        v[:, :, :S].copy_(values)
        self._host_len = self._sync_len = S
        self._layer_len = {}
        self.seq_len_dev.fill_(S)
        return self

    def advance(self, n=1):
        """One decode step appended n keys to every layer (host-side bookkeeping + device counter)."""
        self._host_len += n
        self.seq_len_dev.add_(n)
        self._sync_len = self._host_len
        self._layer_len = {}

    def _advance_host(self, n=1):
        """Host-side bookkeeping alone, for steps whose device counter moved inside a replayed graph: every layer
        holds n more keys."""
        self._host_len += n
        self._sync_len = self._host_len
        self._layer_len = {}

    def update(self, key_states, value_states, layer_idx):
        """TppCache::update / LayerCache::update (src/csrc/llm/attn.h:198-222,258-274): append key_states /
        value_states [B][Nkv][S][H] (bf16, already rotated) to layer `layer_idx` at that layer's length and return
        the layer's [keys, values] up to the new length.  A cache that is too small grows by KV_CACHE_INC_SIZE
        positions beyond what is needed, as the reference's does.  The fused decoder layers do not come through
        here (they append inside their attention launch); this is the way in for callers that hold k / v tensors.
        Lengths are tracked per layer like the reference's offsets; the shared counter follows layer 0."""
        B, Nkv, S, H = key_states.shape
        if value_states.shape != key_states.shape:
            raise TppxError(_lib.ESHAPE, "TppCache.update: keys and values differ in shape")
        base = self._layer_len.get(layer_idx, self._sync_len)
        if self.capacity < base + S:
            self._grow(base + S + int(os.environ.get("KV_CACHE_INC_SIZE", "128")))
        k, v = self._ensure(layer_idx, B, Nkv, H, key_states.device)
        if k.shape[0] != B or k.shape[1] != Nkv or k.shape[3] != H:
            raise TppxError(_lib.ESHAPE, f"TppCache.update: states {tuple(key_states.shape)} do not fit the cache "
                                         f"{tuple(k.shape)}")
        k[:, :, base:base + S].copy_(key_states)
        v[:, :, base:base + S].copy_(value_states)
        self._layer_len[layer_idx] = base + S
        if layer_idx == 0:
            self._host_len = base + S
            self.seq_len_dev.fill_(self._host_len)
        self._sums_of = None
        return [k[:, :, :base + S], v[:, :, :base + S]]

    def _grow(self, new_capacity):
        """Reallocate every layer for `new_capacity` positions, rounded up to whole blocks of 32 like the
        reference's storage (attn.h:186-194)."""
        new_capacity = (new_capacity + self.block_size - 1) // self.block_size * self.block_size
        for i, (k, v) in list(self.layers.items()):
            nk = torch.zeros((k.shape[0], k.shape[1], new_capacity, k.shape[3]), dtype=k.dtype, device=k.device)
            nv = torch.zeros_like(nk)
            nk[:, :, :k.shape[2]].copy_(k)
            nv[:, :, :v.shape[2]].copy_(v)
            self.layers[i] = (nk, nv)
        self.capacity = new_capacity


def rotate_append_attend(q, k, v, t_am, t_pid, cache, layer_idx, B, S, Nq, Nkv, H, t_EP, style):
    """What every decoder block of the reference does between its q/k/v GEMMs and its output projection
    (fused_llm_infer.cpp:784-789, 1025-1027, 1252-1257): rotary embedding on q and k in place (style "llama":
    rotate-half with a [2][MP][HR] cos / sin table; "gptj": adjacent pairs with a [MP][HR] sin | cos table; None:
    no rotation, OPT), append of the S new keys and values at the cache length (LayerCache::update, attn.h:198-222),
    attention over the cached and the new keys (attn<T>, attn.cpp:781-955).  Returns the context [B][S][Nq*H]."""
    L = _lib.lib()
    st = _lib.stream_of(q)
    kc, vc = cache._ensure(layer_idx, B, Nkv, H, q.device)
    ws = _lib.workspace(q)
    mask_ptr = t_am.data_ptr() if t_am is not None and t_am.numel() else None
    mask_ld = t_am.shape[-1] if mask_ptr else 0
    if style == "gptj":
        _lib.check(L.tppx_rotary_kv_append_gptj(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), t_EP.data_ptr(), t_pid.data_ptr(), kc.data_ptr(), vc.data_ptr(),
            cache.seq_len_dev.data_ptr(), B, S, Nq, Nkv, H, t_EP.shape[0], t_EP.shape[1], t_pid.shape[0],
            cache.capacity, st))
    else:
        emb = t_EP.data_ptr() if style == "llama" else None  # no table: append only, q is not touched
        _lib.check(L.tppx_rotary_kv_append_llama(
            q.data_ptr() if emb else None, k.data_ptr(), v.data_ptr(), emb, t_pid.data_ptr(), kc.data_ptr(), vc.data_ptr(),
            cache.seq_len_dev.data_ptr(), B, S, Nq, Nkv, H, t_EP.shape[1] if emb else 1, t_EP.shape[2] if emb else H,
            t_pid.shape[0], cache.capacity, st))
    ctx = torch.empty_like(q)
    if S == 1:
        _lib.check(L.tppx_attn_decode(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), mask_ptr, mask_ld,
                                      cache.seq_len_dev.data_ptr(), 1, ctx.data_ptr(), B, Nq, Nkv, H, cache.capacity,
                                      ws.data_ptr(), ws.numel(), st))
    else:
        _lib.check(L.tppx_attn_prefill(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), mask_ptr, mask_ld,
                                       cache.get_seq_length(), ctx.data_ptr(), B, S, Nq, Nkv, H, cache.capacity, st))
    return ctx


def attn(t_QL, t_KL, t_VL, t_AM, cache, layer_idx, isCausal=True):
    """_C._tpp_attn.attn (attn_wrapper, src/csrc/llm/attn.cpp:957-1043): append t_KL / t_VL [B][Nkv][Sq][H] to layer
    `layer_idx` of the cache, then attention of t_QL [B][Nkv][Sq][R][H] (R = query heads per key head) over all
    cached keys; additive mask t_AM [B][keys] or empty; returns the context in t_QL's layout.  The new tokens see
    the older keys and, causally, each other; isCausal = False is only taken for one query token per sequence,
    where it means the same (the prompt kernel here is causal)."""
    L = _lib.lib()
    if t_QL.dim() != 5 or not t_QL.is_cuda or t_QL.dtype != torch.bfloat16:
        raise TppxError(_lib.EINVAL, "attn: t_QL must be a bfloat16 tensor [B][Nkv][Sq][R][H] on the GPU")
    B, Nkv, Sq, R, H = t_QL.shape
    if not isCausal and Sq != 1:
        raise TppxError(_lib.EUNSUPPORTED, "attn: non-causal attention over several query tokens is not built")
    if tuple(t_KL.shape) != (B, Nkv, Sq, H) or tuple(t_VL.shape) != (B, Nkv, Sq, H):
        raise TppxError(_lib.ESHAPE, f"attn: keys / values must be [B][Nkv][Sq][H] = {(B, Nkv, Sq, H)}")
    core = cache.get_cpp() if hasattr(cache, "get_cpp") else cache
    core.update(_bf16_cuda(t_KL, "t_KL"), _bf16_cuda(t_VL, "t_VL"), layer_idx)
    key_len = core.get_seq_length(layer_idx)
    kc, vc = core.layers[layer_idx]
    q = t_QL.permute(0, 2, 1, 3, 4).reshape(B, Sq, Nkv * R, H).contiguous()  # head index = key head * R + r
    out = torch.empty_like(q)
    st = _lib.stream_of(q)
    ws = _lib.workspace(q)
    mask = t_AM.to(torch.bfloat16).contiguous() if t_AM is not None and t_AM.numel() else None
    mask_ptr, mask_ld = (mask.data_ptr(), mask.shape[-1]) if mask is not None else (None, 0)
    klen = torch.full((1,), key_len, dtype=torch.int32, device=q.device)
    if Sq == 1:
        _lib.check(L.tppx_attn_decode(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), mask_ptr, mask_ld, klen.data_ptr(), 0,
                                      out.data_ptr(), B, Nkv * R, Nkv, H, core.capacity, ws.data_ptr(), ws.numel(), st))
    else:
        _lib.check(L.tppx_attn_prefill(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), mask_ptr, mask_ld, key_len - Sq,
                                       out.data_ptr(), B, Sq, Nkv * R, Nkv, H, core.capacity, st))
    return out.view(B, Sq, Nkv, R, H).permute(0, 2, 1, 3, 4).contiguous()


def check_layer_inputs(who, t_HS, t_pid, cache):
    """Shape checks shared by the decoder blocks: room in the cache for the S new keys, int64 positions [B or 1][S]."""
    B, S, _ = t_HS.shape
    if cache.get_seq_length() + S > cache.capacity:
        raise TppxError(_lib.ESHAPE, f"{who}: {cache.get_seq_length()} cached + {S} new keys exceed "
                                     f"the cache capacity {cache.capacity}")
    if t_pid.dim() != 2 or t_pid.shape[1] != S or t_pid.shape[0] not in (1, B) or t_pid.dtype != torch.int64:
        raise TppxError(_lib.ESHAPE, f"{who}: position_ids must be int64 [B or 1][S={S}], got "
                                     f"{tuple(t_pid.shape)} {t_pid.dtype}")


class FormatSwitches:
    """The weight-format handling every decoder block of the reference repeats in its constructor and at the top of
    its forward (e.g. fused_llm_infer.cpp:650-738, 741-758 for GPT-J): quantized weights serve every pass;
    unquantized ones are quantized for the decode steps under USE_MXFP4 / USE_QINT8 / USE_QINT2 after the
    first-token copies were taken; passes of FT_OPT_SIZE or more tokens run on those copies when
    TPP_CACHE_REMAPPED_WEIGHTS is on.  `_weight_names` lists the attributes holding the linears' weights."""

    _weight_names = ()

    def _setup_formats(self):
        self.first_token_remapped = False
        self._first = None
        names = self._weight_names
        if isinstance(getattr(self, names[0]), _ops.QTensor):
            self._first = tuple(getattr(self, n) for n in names)
            self.first_token_remapped = True
        else:
            quant = (_ops.remap_and_quantize_mxfp4 if USE_MXFP4 else _ops.remap_and_quantize_qint8 if USE_QINT8
                     else _ops.remap_and_quantize_qint2_intlv if USE_QINT2 else None)
            if quant is not None:
                self.remap_for_first_token()
                for n in names:
                    setattr(self, n, quant(getattr(self, n)))

    def remap_for_first_token(self):
        """remap_for_first_token of the reference's blocks (fused_llm_infer.cpp:726-738, 972-983, 1164-1175)."""
        self._first = tuple(wt_tensor_for_first_token(getattr(self, n)) for n in self._weight_names)
        self.first_token_remapped = True

    def _weights_for(self, rows):
        """check_weight_reuse + the switch to the first-token copies (fused_llm_infer.cpp:518-524, 1216-1227)."""
        if rows >= FT_OPT_SIZE and TPP_CACHE_REMAPPED_WEIGHTS:
            if not self.first_token_remapped:
                self.remap_for_first_token()
            return self._first
        return tuple(getattr(self, n) for n in self._weight_names)


class LlamaDecoderLayer(FormatSwitches):
    """torch.classes.tpp_llm.LlamaDecoderLayer(params, layer_idx, eps, H, max_positions, rotary_dim)
    with params = [ln_in gamma, Wq, Wk, Wv, Wo, ln_post gamma, Wg, Wu, Wd, embed_positions]
    (fused_llm_infer.cpp:1096-1110); the linears are quantized tensors of this package or blocked bf16 weights."""

    _weight_names = ("t_Wq", "t_Wk", "t_Wv", "t_Wp", "t_Wg", "t_Wu", "t_Wd")

    def _take_params(self, params):
        (self.t_Gi, self.t_Wq, self.t_Wk, self.t_Wv, self.t_Wp, self.t_Gpa,
         self.t_Wg, self.t_Wu, self.t_Wd, self.t_EP) = params
        self.t_Bq = self.t_Bk = self.t_Bv = None

    def __init__(self, params, layer_idx, eps, H, max_positions, rotary_dim):
        self._take_params(params)
        self.layer_idx, self.eps, self.H = int(layer_idx), float(eps), int(H)
        self.max_positions, self.rotary_dim = int(max_positions), int(rotary_dim)
        # fused_llm_infer.cpp:1112-1162: quantized weights serve every pass; unquantized ones are quantized here
        # for the decode steps under USE_MXFP4 / USE_QINT8 / USE_QINT2, after the first-token copies were taken
        self._setup_formats()
        self.Nq = _ops.weight_nk(self.t_Wq)[0] // self.H
        self.Nkv = _ops.weight_nk(self.t_Wk)[0] // self.H

    def forward(self, inputs, cache, use_cache=True):
        """inputs = [hidden [B][S][hidden], additive mask [B][keys] or empty, position_ids i64 [B or 1][S]].
        S = 1 is the decode step (cache length read from the device counter, so the call can be replayed in a
        graph); S > 1 processes a prompt or several new tokens causally on top of the cached keys.  The S new keys
        go to cache positions get_seq_length() .. +S-1; the caller advances the cache once all layers have run."""
        L = _lib.lib()
        t_HS, t_am, t_pid = inputs[0], inputs[1], inputs[2]
        B, S, hidden = t_HS.shape
        check_layer_inputs(type(self).__name__, t_HS, t_pid, cache)
        st = _lib.stream_of(t_HS)
        empty = torch.empty(0, dtype=torch.bfloat16, device=t_HS.device)
        Wq, Wk, Wv, Wp, Wg, Wu, Wd = self._weights_for(B * S)
        t_res = t_HS
        # Decode steps on MXFP4 weights: the o- and down-projection launches leave the row sums of squares of the
        # residual stream, so the RMSNorm behind them is a scale applied while the next GEMM stages its input.
        M = B * S
        if cache._sums is None:
            cache._sums = (_ops.sums_table(t_HS.device), _ops.sums_table(t_HS.device))
        # Above four rows the gate/up launch is better off behind the separate normalisation kernel: every workgroup
        # repeats the M x K conversion while its weight stream waits (measured +4.4 us at 8..16 rows against +0.6 up
        # to 4, a launch costs about 3); the q/k/v launch breaks even there and keeps the sums.
        sums_attn = cache._sums[0] if (M <= SUMS_GATE_UP_ROWS and _ops.takes_row_sums(Wp, M)) else None
        sums_out = cache._sums[1] if _ops.takes_row_sums(Wd, M) else None
        sums_in = cache._sums[1] if cache._sums_of is t_HS else None
        # input RMSNorm + q/k/v GEMMs
        q, k, v = _ops.qkv_gemm(t_HS, [Wq, Wk, Wv], [self.t_Bq, self.t_Bk, self.t_Bv],
                                norm=(self.t_Gi, self.eps, sums_in))
        kc, vc = cache._ensure(self.layer_idx, B, self.Nkv, self.H, t_HS.device)
        ws = _lib.workspace(t_HS)
        mask_ptr = t_am.data_ptr() if t_am is not None and t_am.numel() else None
        mask_ld = t_am.shape[-1] if mask_ptr else 0
        if S == 1 and FUSE_ROTARY and self.H == 128 and self.t_EP.shape[2] == 128:
            # decode step: rotary, cache append and attention in one launch
            ctx = torch.empty_like(q)
            _lib.check(L.tppx_attn_decode_rotary(
                q.data_ptr(), k.data_ptr(), v.data_ptr(), self.t_EP.data_ptr(), t_pid.data_ptr(), t_pid.shape[0],
                self.t_EP.shape[1], self.t_EP.shape[2], kc.data_ptr(), vc.data_ptr(), mask_ptr, mask_ld,
                cache.seq_len_dev.data_ptr(), ctx.data_ptr(), B, self.Nq, self.Nkv, self.H, cache.capacity,
                ws.data_ptr(), ws.numel(), st))
            return self._after_attention(ctx, t_res, empty, cache, sums_attn, sums_out, Wp, Wg, Wu, Wd)
        ctx = rotate_append_attend(q, k, v, t_am, t_pid, cache, self.layer_idx, B, S, self.Nq, self.Nkv, self.H,
                                   self.t_EP, "llama")
        return self._after_attention(ctx, t_res, empty, cache, sums_attn, sums_out, Wp, Wg, Wu, Wd)

    def _after_attention(self, ctx, t_res, empty, cache, sums_attn, sums_out, Wp, Wg, Wu, Wd):
        t_SO = _ops.fc_add(ctx, Wp, empty, t_res, 1.0, row_sumsq=sums_attn)
        # post-attention RMSNorm + gate/up GEMMs + silu*mul
        t_I = _ops.swiglu_gate_up(t_SO, Wg, Wu, norm=(self.t_Gpa, self.eps, sums_attn))
        t_Out = _ops.fc_add(t_I, Wd, empty, t_SO, 1.0, row_sumsq=sums_out)
        cache._sums_of = t_Out if sums_out is not None else None
        return [t_Out]


def llama_rotary_table(max_positions, head_dim, base=10000.0, device="cuda"):
    """embed_positions as OptimizeModelForLlama builds it (fused_llama_infer.py:188-201): f32 [2][MP][head_dim]
    = cos / sin of position * inv_freq, frequencies repeated over the two halves."""
    inv_freq = 1.0 / (base ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
    freqs = torch.outer(torch.arange(max_positions, dtype=torch.float32), inv_freq)
    emb = torch.cat((freqs, freqs), dim=-1)
    return torch.stack((emb.cos(), emb.sin())).to(device)


class LlamaDecoder:
    """Self-contained Llama-shape decoder for greedy decoding with random-initialised, quantized weights:
    embedding, `n_layers` LlamaDecoderLayer, final RMSNorm, quantized lm_head, argmax.  One decode step is
    captured once as a HIP graph (positions, sequence length and the current token live in device memory)
    and replayed per token."""

    def __init__(self, hidden=4096, inter=11008, n_layers=32, n_heads=32, n_kv_heads=32, vocab=32000,
                 max_positions=4096, eps=1e-5, weight_dtype="mxfp4", seed=0, device="cuda"):
        self.hidden, self.n_layers, self.vocab = hidden, n_layers, vocab
        self.H = hidden // n_heads
        self.eps, self.device = eps, torch.device(device)
        g = torch.Generator(device=self.device).manual_seed(seed)
        quant = _ops.remap_and_quantize_mxfp4 if weight_dtype == "mxfp4" else _ops.remap_and_quantize_qint8

        def lin(N, K):
            W = (torch.randn((N, K), generator=g, device=self.device) * 0.02).to(torch.bfloat16)
            q = quant(W.view(N // 16, 16, K // 64, 32, 2).permute(0, 2, 3, 1, 4).contiguous())
            q.native()
            return q

        self.embed = (torch.randn((vocab, hidden), generator=g, device=self.device) * 0.02).to(torch.bfloat16)
        self.EP = llama_rotary_table(max_positions, self.H, device=self.device)
        ones = torch.ones(hidden, dtype=torch.float32, device=self.device)
        self.layers = []
        for i in range(n_layers):
            params = [ones, lin(n_heads * self.H, hidden), lin(n_kv_heads * self.H, hidden), lin(n_kv_heads * self.H, hidden),
                      lin(hidden, n_heads * self.H), ones, lin(inter, hidden), lin(inter, hidden), lin(hidden, inter), self.EP]
            self.layers.append(LlamaDecoderLayer(params, i, eps, self.H, max_positions, self.H))
        self.norm_w = ones
        self.lm_head = lin(vocab, hidden)
        self.n_kv_heads = n_kv_heads
        self._graph = None

    def new_cache(self, B, context, capacity, seed=1):
        """Cache pre-filled with `context` positions of N(0,1) keys / values in every layer."""
        cache = TppCache(capacity)
        g = torch.Generator(device=self.device).manual_seed(seed)
        for i in range(self.n_layers):
            shape = (B, self.n_kv_heads, context, self.H)
            cache.fill_(i, torch.randn(shape, generator=g, device=self.device).to(torch.bfloat16),
                        torch.randn(shape, generator=g, device=self.device).to(torch.bfloat16))
        return cache

    def step(self, tokens, pos, cache):
        """tokens i64 [B] (device), pos i64 [B][1] (device) -> next tokens i64 [B]; appends to the cache storage
        (the caller advances the counters)."""
        h = self.embed.index_select(0, tokens).unsqueeze(1)
        for layer in self.layers:
            h = layer.forward([h, None, pos], cache)[0]
        h = rms_norm(h, self.norm_w, self.eps)
        logits = _ops.fc_plain(h, self.lm_head, None)
        return logits.view(logits.shape[0], -1).argmax(dim=-1)

    def _step_greedy(self, h, cur, pos, cache, advance=True):
        """One decode step that ends in tppx_greedy_next: h bf16 [B][1][hidden] holds the embeddings of the current
        tokens; afterwards cur (i64 [B]) holds the next tokens and, with advance, pos (i64 [B][1]) and the cache's
        device counter have moved on by one and h holds the next tokens' embeddings -- everything a replayed graph
        needs for its next step.  Without advance nothing but cur changes (the warm-up in front of a capture)."""
        x = h
        for layer in self.layers:
            x = layer.forward([x, None, pos], cache)[0]
        x = rms_norm(x, self.norm_w, self.eps)
        logits = _ops.fc_plain(x, self.lm_head, None)
        B = logits.shape[0]
        logits = logits.view(B, -1)
        _lib.check(_lib.lib().tppx_greedy_next(
            logits.data_ptr(), B, logits.shape[1], self.embed.data_ptr(), self.hidden, cur.data_ptr(),
            pos.data_ptr() if advance else None, cache.seq_len_dev.data_ptr() if advance else None,
            h.data_ptr() if advance else None, _lib.stream_of(logits)))
        return cur

    def _greedy_fusable(self, B):
        return (FUSE_GREEDY and self.vocab % 8 == 0 and self.hidden % 8 == 0 and self.embed.is_contiguous()
                and self.embed.dtype == torch.bfloat16 and B < 65536)

    def prefill(self, prompt, cache, mask=None):
        """prompt i64 [B][S] (device) on top of whatever the cache holds -> next tokens i64 [B]; advances the cache
        by S.  mask: additive bf16 [B][keys] over cache positions (TppCache.align_and_invert_mask) or None."""
        B, S = prompt.shape
        past = cache.get_seq_length()
        pos = torch.arange(past, past + S, dtype=torch.int64, device=self.device).unsqueeze(0)
        h = self.embed.index_select(0, prompt.reshape(-1)).view(B, S, self.hidden)
        for layer in self.layers:
            h = layer.forward([h, mask, pos], cache)[0]
        cache.advance(S)
        h = rms_norm(h[:, -1:].contiguous(), self.norm_w, self.eps)  # only the last position feeds the lm_head
        logits = _ops.fc_plain(h, self.lm_head, None)
        return logits.view(B, -1).argmax(dim=-1)

    def generate(self, prompt, n_new, capacity=None, use_graph=True):
        """Greedy generation as run_generation.py drives it: the prompt in one pass, then one token per step.
        Returns i64 [B][n_new]."""
        B, S = prompt.shape
        cache = TppCache(capacity or S + n_new + 32)
        first = self.prefill(prompt, cache)
        if n_new == 1:
            return first.view(B, 1)
        rest = self.greedy_decode(first, cache, n_new - 1, use_graph=use_graph)
        return torch.cat([first.view(B, 1), rest], dim=1)

    def _check_room(self, cache, n_new):
        """A replayed decode step checks nothing on the host: past the cache's capacity the kernels drop the new
        key / value, past the rotary table they skip the rotation.  Refuse such a run up front."""
        start = cache.get_seq_length()
        if start + n_new > cache.get_capacity():
            raise TppxError(_lib.ESHAPE, f"decoding {n_new} tokens from position {start} overruns the cache "
                                         f"capacity {cache.get_capacity()}")
        if start + n_new > self.EP.shape[1]:
            raise TppxError(_lib.ESHAPE, f"decoding {n_new} tokens from position {start} overruns the rotary table "
                                         f"({self.EP.shape[1]} positions)")

    def time_decode_steps(self, tokens, cache, n_new):
        """Seconds spent in n_new replays of the captured decode step (capture excluded)."""
        import time
        self._check_room(cache, n_new + 1)  # one untimed eager step precedes the replays
        B = tokens.shape[0]
        cur = tokens.clone()
        pos = torch.full((B, 1), cache.get_seq_length(), dtype=torch.int64, device=self.device)
        fused = self._greedy_fusable(B)
        if fused:
            h = self.embed.index_select(0, cur).unsqueeze(1).contiguous()
            self._step_greedy(h, cur.clone(), pos, cache, advance=False)
        else:
            self.step(cur, pos, cache)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            if fused:
                self._step_greedy(h, cur, pos, cache)
            else:
                nxt = self.step(cur, pos, cache)
                cur.copy_(nxt)
                pos.add_(1)
                cache.seq_len_dev.add_(1)
        graph.replay()  # one untimed replay
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n_new - 1):
            graph.replay()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        cache._advance_host(n_new)  # every replay moved the device counter
        return dt * n_new / (n_new - 1)

    def greedy_decode(self, tokens, cache, n_new, use_graph=True):
        """Greedy decode of n_new tokens per sequence from the [B] start tokens; returns i64 [B][n_new]."""
        self._check_room(cache, n_new)
        B = tokens.shape[0]
        cur = tokens.clone()
        pos = torch.full((B, 1), cache.get_seq_length(), dtype=torch.int64, device=self.device)
        out = torch.empty((B, n_new), dtype=torch.int64, device=self.device)
        if use_graph:
            fused = self._greedy_fusable(B)
            # warm-up outside capture (allocations, lazy module loads); it leaves the counters where they are
            if fused:
                h = self.embed.index_select(0, cur).unsqueeze(1).contiguous()
                self._step_greedy(h, cur.clone(), pos, cache, advance=False)
            else:
                nxt = self.step(cur, pos, cache)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                if fused:
                    self._step_greedy(h, cur, pos, cache)
                else:
                    nxt = self.step(cur, pos, cache)
                    cur.copy_(nxt)
                    pos.add_(1)
                    cache.seq_len_dev.add_(1)
            for t in range(n_new):
                graph.replay()
                out[:, t].copy_(cur)
                cache._advance_host(1)
        else:
            for t in range(n_new):
                nxt = self.step(cur, pos, cache)
                cur.copy_(nxt)
                out[:, t].copy_(cur)
                pos.add_(1)
                cache.advance(1)
        return out


# ---------------------------------------------------------------------------
# Hugging Face front-end (src/tpp_pytorch_extension/llm/fused_llama_infer.py:45-336)
# ---------------------------------------------------------------------------
class LlamaDecoderLayerModule(torch.nn.Module):
    """What a transformers LlamaDecoderLayer becomes (fused_llama_infer.py:45-101): the module keeps its
    sub-modules (quantized in place) and forwards through `cpp_block`, one LlamaDecoderLayer of this file."""

    def forward(self, hidden_states, attention_mask=None, position_ids=None, past_key_values=None, use_cache=False,
                past_key_value=None, **kwargs):
        if not hasattr(self, "cpp_block"):
            raise ValueError("cpp_block is not initialized")
        if position_ids is None:
            raise ValueError("position_ids is required")
        cache = past_key_values if past_key_values is not None else past_key_value
        if cache is None:
            raise ValueError("the optimized decoder layer needs a TppCache (past_key_values)")
        core = cache.get_cpp() if hasattr(cache, "get_cpp") else cache
        hs = hidden_states.to(torch.bfloat16).contiguous()
        mask = attention_mask.to(torch.bfloat16).contiguous() if attention_mask is not None else None
        return self.cpp_block.forward([hs, mask, position_ids.contiguous()], core, use_cache)[0]


def FixLlamaDecoderLayer(self, bk=None, bc=None, layer_dtype=torch.bfloat16, weight_dtype="mxfp4",
                         embed_positions=None):
    """fused_llama_infer.py:104-173: quantize the seven linears of a transformers LlamaDecoderLayer in place
    (FixLinear with [bk, bc] blocking) and attach the fused block."""
    import transformers
    from .llm_common import FixLinear
    if not isinstance(self, transformers.models.llama.modeling_llama.LlamaDecoderLayer):
        return
    self.__class__ = LlamaDecoderLayerModule
    self.features_block_size = bc
    self.layer_dtype = layer_dtype
    self.model_parallel = False
    for m in self.modules():
        if isinstance(m, torch.nn.Linear):
            if m.bias is not None:
                raise NotImplementedError("attention_bias / mlp_bias are not supported for Llama")
            FixLinear(m, bk, bc, layer_dtype, weight_dtype=weight_dtype)
    if not hasattr(self, "cpp_block"):
        at, mlp = self.self_attn, self.mlp
        params = [self.input_layernorm.weight.data.float(), at.q_proj.weight, at.k_proj.weight, at.v_proj.weight,
                  at.o_proj.weight, self.post_attention_layernorm.weight.data.float(), mlp.gate_proj.weight,
                  mlp.up_proj.weight, mlp.down_proj.weight, embed_positions]
        self.cpp_block = LlamaDecoderLayer(params, at.layer_idx, self.input_layernorm.variance_epsilon, at.head_dim,
                                           embed_positions.shape[1], at.head_dim)


def LlamaModel_forward(self, input_ids=None, attention_mask=None, position_ids=None, past_key_values=None,
                       inputs_embeds=None, use_cache=None, cache_position=None, **kwargs):
    """fused_llama_infer.py:228-336: embeddings, position ids from the cache length, additive key mask from the
    0/1 attention mask, the decoder layers on a TppCache, final norm."""
    from transformers.modeling_outputs import BaseModelOutputWithPast
    from .llm_common import TppCache as HFTppCache
    if (input_ids is None) == (inputs_embeds is None):
        raise ValueError("You cannot specify both input_ids and inputs_embeds at the same time, and must specify either one")
    if inputs_embeds is None:
        inputs_embeds = self.embed_tokens(input_ids)
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
    hidden_states = inputs_embeds.to(torch.bfloat16)
    for layer in self.layers[: self.config.num_hidden_layers]:
        hidden_states = layer(hidden_states, attention_mask=mask, position_ids=position_ids,
                              past_key_values=past_key_values, use_cache=True)
    past_key_values.get_cpp().advance(S)
    hidden_states = rms_norm(hidden_states, self._tpp_norm_weight, self._tpp_norm_eps)
    return BaseModelOutputWithPast(last_hidden_state=hidden_states, past_key_values=past_key_values)


def layer_weight_dtype(who, weight_dtype, dtype):
    """The weight_dtype argument of the reference's OptimizeModelFor* (None = the layer dtype; a torch dtype or its
    name; "mxfp4" / "qint8" / "qint2", run_generation.py:68-75) as FixLinear takes it.  The fused blocks compute in
    bf16, so an unquantized format other than bf16 is refused."""
    if weight_dtype is None:
        weight_dtype = dtype
    if isinstance(weight_dtype, str) and weight_dtype not in ("mxfp4", "qint8", "qint2"):
        weight_dtype = getattr(torch, weight_dtype, weight_dtype)
    if weight_dtype in ("mxfp4", "qint8", "qint2") or weight_dtype == torch.bfloat16:
        return weight_dtype
    raise TppxError(_lib.EUNSUPPORTED, f"{who}: weight_dtype {weight_dtype!r} (bfloat16, mxfp4, qint8 or qint2)")


def OptimizeModelForLlama(model, dtype=torch.bfloat16, device="cuda", weight_dtype=None, quantize_lm_head=False):
    """fused_llama_infer.py:176-226 for one GPU: the rotary table from the model's own rotary_emb, every
    LlamaDecoderLayer fused, every remaining nn.Linear (the lm_head) turned into a BlockedLinear with the
    reference's blocking (100 x 64 where the vocabulary allows, else 64 x 64) and bf16 weights, LlamaModel.forward
    of this instance replaced.  quantize_lm_head: True / "qint8" / "mxfp4" quantizes the lm_head as well
    (run_generation.py:277-282 does it with remap_and_quantize_qint8 after the call; that works here too).
    weight_dtype as in the reference: None = the layers keep bf16 weights (and quantize them themselves under
    USE_MXFP4 / USE_QINT8 / USE_QINT2), or "mxfp4" / "qint8" / "qint2".  Difference: the KV cache is allocated for
    TPPX_KV_CAPACITY keys per sequence (default: the model's max_position_embeddings)."""
    import transformers
    from .llm_common import FixLinear
    weight_dtype = layer_weight_dtype("OptimizeModelForLlama", weight_dtype, dtype)
    if getattr(model.config, "attention_bias", False):
        raise NotImplementedError("attention_bias is not supported for Llama yet!")
    model.config._attn_implementation = "tpp"
    embed_positions = None
    for m in model.modules():
        if isinstance(m, transformers.models.llama.modeling_llama.LlamaPreTrainedModel) and hasattr(m, "rotary_emb"):
            # before the model is cast: the rotary module's frequencies are still fp32
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
            if isinstance(m, transformers.models.llama.modeling_llama.LlamaDecoderLayer):
                FixLlamaDecoderLayer(m, 16, 64, dtype, weight_dtype, embed_positions)
        head_dtype = None if not quantize_lm_head else ("qint8" if quantize_lm_head is True else quantize_lm_head)
        for m in list(model.modules()):  # FixLinear is a no-op for the ones fixed above
            if not isinstance(m, torch.nn.Linear) or m.weight.shape[1] % 64:
                continue
            if head_dtype is not None:  # quantized tiles are 16 output channels high
                if m.weight.shape[0] % 32 == 0:
                    FixLinear(m, 16, 64, dtype, weight_dtype=head_dtype)
            elif m.weight.shape[0] % 100 == 0:
                FixLinear(m, 100, 64, dtype)
            elif m.weight.shape[0] % 64 == 0:
                FixLinear(m, 64, 64, dtype)
    for m in model.modules():
        if isinstance(m, transformers.models.llama.modeling_llama.LlamaModel):
            m._tpp_kv_capacity = int(os.environ.get("TPPX_KV_CAPACITY", embed_positions.shape[1]))
            m._tpp_norm_weight = m.norm.weight.data.float().contiguous()
            m._tpp_norm_eps = m.norm.variance_epsilon
            m.forward = types.MethodType(LlamaModel_forward, m)
            m._tpp_core_model = True
    return model


def generate_greedy(model, input_ids, max_new_tokens, attention_mask=None):
    """Greedy loop over an optimized LlamaForCausalLM as run_generation.py drives generate(): the prompt in one
    forward, then one token per forward on the same TppCache.  Returns i64 [B][S + max_new_tokens]."""
    ids = input_ids
    cache = None
    cur = input_ids
    for _ in range(max_new_tokens):
        pos = None
        if attention_mask is not None:
            # positions count the real tokens, as generate() derives them from the mask (padding gets position 1)
            pos = attention_mask.long().cumsum(-1) - 1
            pos = pos.masked_fill(attention_mask == 0, 1)[:, -cur.shape[1]:]
        out = model(input_ids=cur, attention_mask=attention_mask, position_ids=pos, past_key_values=cache,
                    use_cache=True, logits_to_keep=1)
        cache = out.past_key_values
        cur = out.logits[:, -1].argmax(dim=-1, keepdim=True)
        ids = torch.cat([ids, cur], dim=1)
        if attention_mask is not None:
            attention_mask = torch.cat([attention_mask, attention_mask.new_ones((ids.shape[0], 1))], dim=1)
    return ids


def generate_greedy_graph(model, input_ids, max_new_tokens, attention_mask=None):
    """generate_greedy with the decode steps replayed from one HIP graph: the prompt runs as usual, then a single
    step of the patched inner model (embedding, layers, final norm), the lm_head and the argmax is captured and
    replayed max_new_tokens - 1 times.  What changes from step to step lives on the device: the current tokens, their
    positions (counted over real tokens, as generate() derives them from the mask), the cache length, and an additive
    key mask over the cache's whole capacity (0 everywhere but at the prompt's padding), so that no kernel argument
    depends on the step.  Works on every model an OptimizeModelFor* of this package has patched; returns i64
    [B][S + max_new_tokens], the same tokens as generate_greedy."""
    from .llm_common import TppCache as HFTppCache
    core = next((m for m in model.modules() if getattr(m, "_tpp_core_model", False)), None)
    if core is None:
        raise TppxError(_lib.EINVAL, "generate_greedy_graph: the model was not optimized by this package")
    B, S = input_ids.shape
    dev = input_ids.device
    if attention_mask is None:
        attention_mask = torch.ones_like(input_ids)
    cap = core._tpp_kv_capacity
    if S + max_new_tokens > cap:
        raise TppxError(_lib.ESHAPE, f"generate_greedy_graph: {S} prompt + {max_new_tokens} new tokens exceed the "
                                     f"cache capacity {cap}")
    cache = HFTppCache(capacity=cap)
    pos0 = attention_mask.long().cumsum(-1) - 1
    pos0 = pos0.masked_fill(attention_mask == 0, 1)
    out = model(input_ids=input_ids, attention_mask=attention_mask, position_ids=pos0, past_key_values=cache,
                use_cache=True, logits_to_keep=1)
    cur = out.logits[:, -1].argmax(dim=-1, keepdim=True)
    ids = [input_ids, cur]
    if max_new_tokens <= 1:
        return torch.cat(ids[:1 + max_new_tokens], dim=1)
    inner = cache.get_cpp()
    # additive mask over the whole capacity: the lowest bf16 at the prompt's padding, 0 elsewhere (keys past the
    # cache length are never read)
    width = (inner.capacity + inner.block_size - 1) // inner.block_size * inner.block_size
    smask = torch.zeros((B, width), dtype=torch.bfloat16, device=dev)
    smask[:, :S].masked_fill_(attention_mask == 0, torch.finfo(torch.bfloat16).min)
    cache.static_mask = smask
    cur = cur.clone()
    pos = (pos0[:, -1:] + 1).contiguous()
    ones = torch.ones((B, 1), dtype=attention_mask.dtype, device=dev)

    def step():
        h = core(input_ids=cur, attention_mask=ones, position_ids=pos, past_key_values=cache, use_cache=True)
        logits = model.lm_head(h.last_hidden_state[:, -1:])
        return logits[:, -1].argmax(dim=-1, keepdim=True)

    try:
        # warm-up outside capture (allocations, lazy module loads), then the counters go back: the key it wrote at the
        # cache's end is written again by the first replay
        host_len = inner.get_seq_length()
        step()
        inner.seq_len_dev.sub_(1)
        inner._advance_host(host_len - inner.get_seq_length())
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            nxt = step()  # (the patched forward moves the device counter itself)
            cur.copy_(nxt)
            pos.add_(1)
        inner._advance_host(host_len - inner.get_seq_length())  # capture ran the host bookkeeping once, no kernels
        for _ in range(max_new_tokens - 1):
            graph.replay()
            inner._advance_host(1)
            ids.append(cur.clone())
    finally:
        cache.static_mask = None
    return torch.cat(ids, dim=1)
