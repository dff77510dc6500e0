"""Qwen2DecoderLayer (the Llama layer with q/k/v biases) against the composition of the oracle functions, and
OptimizeModelForQwen2 against the stock transformers model holding the dequantized weights.

Tolerances as for the Llama layer: a whole layer rel-L2 <= 2e-2 against the oracle composition; logits of the
optimized model rel-L2 <= 3e-2 (MXFP4) / 6e-2 (QINT8: int8 activations) against fp32 transformers.
"""
import numpy as np
import pytest
import torch

import oracle as O
from util import t2bits, randn_bf16, block_bf16, bits2f, assert_close_bf16

pytestmark = pytest.mark.gpu


def _q2():
    import tpp_pytorch_extension  # noqa: F401
    from tpp_pytorch_extension.llm import fused_qwen2_infer as F
    return F


def _layer(F, fmt, seed):
    from tpp_pytorch_extension import _ops
    from tpp_pytorch_extension.llm import fused_llama_infer as FL
    hidden, inter, Nq, Nkv, H, MP = 512, 1024, 4, 2, 128, 256
    rng = torch.Generator().manual_seed(seed)

    def lin(N, K, s):
        W = randn_bf16((N, K), 0.05, s)
        if fmt == "mxfp4":
            return W, _ops.remap_and_quantize_mxfp4(block_bf16(W).cuda()), O.remap_quantize_mxfp4(W.float().numpy())
        return W, _ops.remap_and_quantize_qint8(block_bf16(W).cuda()), O.remap_quantize_qint8(W.float().numpy())

    Ws = [lin(Nq * H, hidden, seed + 1), lin(Nkv * H, hidden, seed + 2), lin(Nkv * H, hidden, seed + 3),
          lin(hidden, Nq * H, seed + 4), lin(inter, hidden, seed + 5), lin(inter, hidden, seed + 6),
          lin(hidden, inter, seed + 7)]
    Bs = [randn_bf16((Nq * H,), 0.5, seed + 8), randn_bf16((Nkv * H,), 0.5, seed + 9), randn_bf16((Nkv * H,), 0.5, seed + 10)]
    g1 = torch.rand(hidden, generator=rng) + 0.5
    g2 = torch.rand(hidden, generator=rng) + 0.5
    EP = FL.llama_rotary_table(MP, H, device="cpu")
    layer = F.Qwen2DecoderLayer([g1.cuda(), Ws[0][1], Ws[1][1], Ws[2][1], Ws[3][1], g2.cuda(), Ws[4][1], Ws[5][1],
                                 Ws[6][1], Bs[0].cuda(), Bs[1].cuda(), Bs[2].cuda(), EP.cuda()], 0, 1e-5, H, MP, H)

    def mm(a_bits, w, bias=None, post=O.POST_NONE, post_in=None):
        b = None if bias is None else t2bits(bias)
        if fmt == "mxfp4":
            return O.linear_mxfp4(a_bits, w[2][0], w[2][1], b, post, post_in, None, 1.0, O.MODE_IDEAL)
        return O.linear_qint8(a_bits, w[2][0], w[2][1], b, post, post_in, None, 1.0, O.MODE_IDEAL)

    return layer, Ws, Bs, g1, g2, EP, mm, (hidden, inter, Nq, Nkv, H, MP)


@pytest.mark.parametrize("fmt", ["mxfp4", "qint8"])
@pytest.mark.parametrize("past,S", [(37, 1), (0, 70), (21, 9)])
def test_qwen2_decoder_layer_against_oracle(fmt, past, S):
    """Qwen2DecoderLayer.forward (decode step and prompt passes) against the oracle composition
    (fused_llm_infer.cpp:1455-1502): biases enter the q, k and v GEMMs before the rotary."""
    F = _q2()
    layer, Ws, Bs, g1, g2, EP, mm, (hidden, inter, Nq, Nkv, H, MP) = _layer(F, fmt, 300)
    B, cap = 2, 128
    cache = F.TppCache(cap)
    k0, v0 = randn_bf16((B, Nkv, past, H), 1.0, 361), randn_bf16((B, Nkv, past, H), 1.0, 362)
    if past:
        cache.fill_(0, k0.cuda(), v0.cuda())
    x = randn_bf16((B, S, hidden), 1.0, 363)
    pos = torch.arange(past, past + S, dtype=torch.int64).unsqueeze(0).repeat(B if S == 1 else 1, 1)
    out = layer.forward([x.cuda(), None, pos.cuda()], cache, True)[0]
    cache.advance(S)
    assert out.shape == (B, S, hidden) and cache.get_seq_length() == past + S

    xb = t2bits(x).reshape(B * S, hidden)
    h = O.rms_norm(xb, g1.numpy(), 1e-5)
    q, k, v = mm(h, Ws[0], Bs[0]), mm(h, Ws[1], Bs[1]), mm(h, Ws[2], Bs[2])
    q = O.rotary_llama(q.reshape(B, S, -1), EP.numpy(), pos.numpy(), Nq, H).reshape(B, S, Nq, H)
    k = O.rotary_llama(k.reshape(B, S, -1), EP.numpy(), pos.numpy(), Nkv, H).reshape(B, S, Nkv, H).transpose(0, 2, 1, 3)
    v = v.reshape(B, S, Nkv, H).transpose(0, 2, 1, 3)
    kall = np.concatenate([t2bits(k0), k], axis=2)
    vall = np.concatenate([t2bits(v0), v], axis=2)
    if S == 1:
        ctxv = O.attn_decode(q.reshape(B, Nq, H), kall, vall).reshape(B, Nq * H)
    else:
        ctxv = O.attn_prefill(q, kall, vall).reshape(B * S, Nq * H)
    so = mm(ctxv, Ws[3], None, O.POST_ADD_SCALE, xb)
    h2 = O.rms_norm(so, g2.numpy(), 1e-5)
    gate = mm(h2, Ws[4], None, O.POST_SILU)
    ref = mm(mm(h2, Ws[5], None, O.POST_MUL, gate), Ws[6], None, O.POST_ADD_SCALE, so)
    g, r = bits2f(t2bits(out)).reshape(B * S, hidden).astype(np.float64), bits2f(ref).astype(np.float64)
    rel = np.sqrt(((g - r) ** 2).sum() / (r ** 2).sum())
    assert rel <= 2e-2, rel
    # the biased, rotated keys and the biased values are what the cache holds
    kc, vc = cache.get(0)
    assert_close_bf16(t2bits(kc[:, :, past:]), np.ascontiguousarray(k), ulps=2 if fmt == "qint8" else 1, what="cached keys")
    assert_close_bf16(t2bits(vc[:, :, past:]), np.ascontiguousarray(v), ulps=2 if fmt == "qint8" else 1, what="cached values")
    # the biases matter: the same layer without them gives something else
    from tpp_pytorch_extension.llm import fused_llama_infer as FL
    plain = FL.LlamaDecoderLayer([layer.t_Gi, layer.t_Wq, layer.t_Wk, layer.t_Wv, layer.t_Wp, layer.t_Gpa, layer.t_Wg,
                                  layer.t_Wu, layer.t_Wd, layer.t_EP], 0, 1e-5, H, MP, H)
    cache2 = F.TppCache(cap)
    if past:
        cache2.fill_(0, k0.cuda(), v0.cuda())
    out2 = plain.forward([x.cuda(), None, pos.cuda()], cache2, True)[0]
    assert not torch.equal(out2, out)


def test_qwen2_decoder_layer_parameter_list():
    F = _q2()
    from tpp_pytorch_extension._lib import TppxError
    with pytest.raises(TppxError):
        F.Qwen2DecoderLayer([None] * 10, 0, 1e-5, 128, 256, 128)


@pytest.mark.parametrize("weight_dtype", ["mxfp4", "qint8", "bf16"])
def test_optimize_model_for_qwen2_against_transformers(weight_dtype):
    """OptimizeModelForQwen2 on a random-initialised transformers Qwen2ForCausalLM (2 layers, GQA 4/2 heads of 128,
    q/k/v biases drawn at N(0, 0.5) so that they matter): logits of the prompt pass and of two decode steps against
    the stock model in fp32 on the CPU holding the dequantized weights and the bf16-rounded biases."""
    transformers = pytest.importorskip("transformers")
    import copy
    F = _q2()
    cfg = transformers.Qwen2Config(hidden_size=512, intermediate_size=1024, num_hidden_layers=2, num_attention_heads=4,
                                   num_key_value_heads=2, vocab_size=1024, max_position_embeddings=256,
                                   rms_norm_eps=1e-5, attn_implementation="eager", use_sliding_window=False,
                                   tie_word_embeddings=False)
    torch.manual_seed(31)
    ref_model = transformers.Qwen2ForCausalLM(cfg).eval()
    with torch.no_grad():
        for m in ref_model.modules():
            if isinstance(m, torch.nn.Linear):
                w = m.weight.data.to(torch.bfloat16).float()
                if weight_dtype == "mxfp4":
                    q, sc = O.remap_quantize_mxfp4(w.numpy())
                    m.weight.data.copy_(torch.from_numpy(O.dequantize_mxfp4_plain(q, sc)))
                elif weight_dtype == "qint8":
                    q, sc, _ = O.remap_quantize_qint8(w.numpy())
                    m.weight.data.copy_(torch.from_numpy(O.dequantize_qint8_plain(q, sc)))
                else:
                    m.weight.data.copy_(w)
                if m.bias is not None:
                    m.bias.data.copy_((torch.randn_like(m.bias) * 0.5).to(torch.bfloat16).float())
            elif isinstance(m, torch.nn.Embedding):
                m.weight.data.copy_(m.weight.data.to(torch.bfloat16).float())
    assert ref_model.model.layers[0].self_attn.q_proj.bias is not None
    opt_model = F.OptimizeModelForQwen2(copy.deepcopy(ref_model), torch.bfloat16, "cuda",
                                        None if weight_dtype == "bf16" else weight_dtype).eval()
    assert type(opt_model.model.layers[0].cpp_block).__name__ == "Qwen2DecoderLayer"
    tol = 3e-2 if weight_dtype == "mxfp4" else 6e-2

    ids = torch.randint(0, 1024, (2, 19), generator=torch.Generator().manual_seed(32))
    am = torch.ones_like(ids)
    am[1, :4] = 0  # left padding of sequence 1
    pos = (am.cumsum(-1) - 1).clamp(min=0)

    def rel(a, b):
        a, b = a.double(), b.double()
        return float(((a - b).norm() / b.norm()))

    with torch.no_grad():
        r = ref_model(input_ids=ids, attention_mask=am, position_ids=pos, use_cache=True)
        o = opt_model(input_ids=ids.cuda(), attention_mask=am.cuda(), position_ids=pos.cuda(), use_cache=True)
        assert o.logits.shape == r.logits.shape
        assert rel(o.logits[0].float().cpu(), r.logits[0]) <= tol
        assert rel(o.logits[1, 4:].float().cpu(), r.logits[1, 4:]) <= tol
        cache_o, cache_r = o.past_key_values, r.past_key_values
        assert cache_o.get_seq_length() == 19 and len(cache_o) == 2
        for step in range(2):
            nxt = r.logits[:, -1].argmax(-1, keepdim=True)
            am = torch.cat([am, torch.ones(2, 1, dtype=am.dtype)], 1)
            pos = pos[:, -1:] + 1
            r = ref_model(input_ids=nxt, attention_mask=am, position_ids=pos, past_key_values=cache_r, use_cache=True)
            o = opt_model(input_ids=nxt.cuda(), attention_mask=am.cuda(), position_ids=pos.cuda(),
                          past_key_values=cache_o, use_cache=True)
            assert rel(o.logits.float().cpu(), r.logits) <= tol
        assert cache_o.get_seq_length() == 21
    out = F.generate_greedy(opt_model, ids[:1].cuda(), 5)
    assert out.shape == (1, 24) and torch.equal(out[:, :19].cpu(), ids[:1])
    # sliding-window attention is refused, as in the reference
    cfg_sw = copy.deepcopy(cfg)
    cfg_sw.use_sliding_window = True
    with pytest.raises(NotImplementedError):
        F.OptimizeModelForQwen2(transformers.Qwen2ForCausalLM(cfg_sw), torch.bfloat16, "cuda",
                                "bfloat16" if weight_dtype == "bf16" else weight_dtype)
    # an unquantized format that the bf16 blocks cannot hold is refused by name
    from tpp_pytorch_extension._lib import TppxError
    with pytest.raises(TppxError):
        F.OptimizeModelForQwen2(transformers.Qwen2ForCausalLM(cfg), torch.bfloat16, "cuda", "float32")
