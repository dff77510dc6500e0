"""GPTJBlock and OPTDecoderLayer: their LayerNorm and GPT-J rotary kernels against the oracle and plain PyTorch,
one block against the composition of the oracle functions, and the optimized transformers models against the stock
ones holding the dequantized weights.

Tolerances: LayerNorm and rotary within 1 bf16 ulp of the fp32 recipe; a whole block rel-L2 <= 2e-2 against the
oracle composition; logits of the optimized models rel-L2 <= 3e-2 (MXFP4) / 6e-2 (QINT8) against fp32 transformers.
"""
import copy

import numpy as np
import pytest
import torch

import oracle as O
from util import t2bits, randn_bf16, block_bf16, bits2f, assert_close_bf16

pytestmark = pytest.mark.gpu


def _gj():
    import tpp_pytorch_extension  # noqa: F401
    from tpp_pytorch_extension.llm import fused_gptj_infer as F
    return F


def _opt():
    import tpp_pytorch_extension  # noqa: F401
    from tpp_pytorch_extension.llm import fused_opt_infer as F
    return F


@pytest.mark.parametrize("K", [4096, 1000, 8])
@pytest.mark.parametrize("pdt", [torch.float32, torch.bfloat16])
def test_layer_norm(K, pdt):
    F = _gj()
    x = randn_bf16((7, 3, K), 1.5, 11) + 0.75
    x = x.to(torch.bfloat16)
    rng = torch.Generator().manual_seed(12)
    g = (torch.randn(K, generator=rng) * 0.5 + 1.0).to(pdt)
    b = (torch.randn(K, generator=rng) * 0.3).to(pdt)
    y = F.lyr_norm(x.cuda(), g.cuda(), b.cuda(), 1e-5)
    ref = O.layer_norm(t2bits(x).reshape(-1, K), g.float().numpy(), b.float().numpy(), 1e-5)
    assert_close_bf16(t2bits(y).reshape(-1, K), ref, what=f"layer_norm K={K}")
    # torch's own layer_norm in fp32 on the same values
    t = torch.nn.functional.layer_norm(x.float(), (K,), g.float(), b.float(), 1e-5)
    assert_close_bf16(t2bits(y).reshape(-1, K), t2bits(t.to(torch.bfloat16)).reshape(-1, K), what="layer_norm vs torch")
    from tpp_pytorch_extension._lib import TppxError
    with pytest.raises(TppxError):
        F.lyr_norm(x.cuda(), g.cuda(), b.float().cuda() if pdt == torch.bfloat16 else b.bfloat16().cuda(), 1e-5)


@pytest.mark.parametrize("H,HR", [(128, 64), (256, 64), (64, 64), (32, 16), (80, 32), (200, 64)])
def test_rotary_gptj(H, HR):
    F = _gj()
    B, S, N, MP = 2, 5, 3, 64
    t = randn_bf16((B, S, N * H), 1.0, 21)
    emb = F.create_sinusoidal_positions(MP, HR)
    pos = torch.tensor([[3, 9, 63, 64, 0], [1, 2, 3, 4, 70]], dtype=torch.int64)  # 64 and 70 are out of range: untouched
    got = F.apply_rotary_pos_emb_gptj(t.clone().cuda(), emb.cuda(), pos.cuda(), N, H)
    ref = O.rotary_gptj(t2bits(t), emb.numpy(), pos.numpy(), N, H)
    assert_close_bf16(t2bits(got), ref, what=f"rotary gptj H={H} HR={HR}")
    assert torch.equal(got.cpu()[0, 3], t[0, 3]) and torch.equal(got.cpu()[1, 4], t[1, 4])
    assert torch.equal(got.cpu().view(B, S, N, H)[..., HR:], t.view(B, S, N, H)[..., HR:])
    got1 = F.apply_rotary_pos_emb_gptj(t.clone().cuda(), emb.cuda(), pos[:1].cuda(), N, H)
    ref1 = O.rotary_gptj(t2bits(t), emb.numpy(), pos[:1].numpy(), N, H)
    assert_close_bf16(t2bits(got1), ref1, what="rotary gptj broadcast positions")


def _lin(fmt, N, K, s):
    from tpp_pytorch_extension import _ops
    W = randn_bf16((N, K), 0.05, s)
    if fmt == "mxfp4":
        return _ops.remap_and_quantize_mxfp4(block_bf16(W).cuda()), O.remap_quantize_mxfp4(W.float().numpy())
    return _ops.remap_and_quantize_qint8(block_bf16(W).cuda()), O.remap_quantize_qint8(W.float().numpy())


def _mm(fmt, a_bits, w, bias=None, post=O.POST_NONE, post_in=None, post_in2=None):
    b = None if bias is None else t2bits(bias)
    f = O.linear_mxfp4 if fmt == "mxfp4" else O.linear_qint8
    return f(a_bits, w[1][0], w[1][1], b, post, post_in, post_in2, 1.0, O.MODE_IDEAL)


def _rel(out, ref_bits):
    g, r = bits2f(t2bits(out)).reshape(ref_bits.shape).astype(np.float64), bits2f(ref_bits).astype(np.float64)
    return np.sqrt(((g - r) ** 2).sum() / (r ** 2).sum())


@pytest.mark.parametrize("fmt", ["mxfp4", "qint8"])
@pytest.mark.parametrize("past,S", [(37, 1), (0, 70), (21, 9)])
def test_gptj_block_against_oracle(fmt, past, S):
    """GPTJBlock.forward against the oracle composition (fused_llm_infer.cpp:760-846, FUSED_QKV_GEMM = 2):
    one LayerNorm, q/k/v and GELU(fc_in) on it, GPT-J rotary, attention, out_proj, fc_out + both residuals."""
    F = _gj()
    hidden, inter, N, H, HR, MP = 512, 2048, 4, 128, 64, 256
    B, cap = 2, 128
    rng = torch.Generator().manual_seed(400)
    Ws = [_lin(fmt, hidden, hidden, 401 + i) for i in range(4)] + [_lin(fmt, inter, hidden, 405), _lin(fmt, hidden, inter, 406)]
    Bi, Bo = randn_bf16((inter,), 0.3, 407), randn_bf16((hidden,), 0.3, 408)
    g = (torch.rand(hidden, generator=rng) + 0.5).to(torch.bfloat16)
    bt = (torch.randn(hidden, generator=rng) * 0.2).to(torch.bfloat16)
    EP = F.create_sinusoidal_positions(MP, HR)
    blk = F.GPTJBlock([g.cuda(), bt.cuda(), Ws[0][0], Ws[1][0], Ws[2][0], Ws[3][0], Ws[4][0], Bi.cuda(), Ws[5][0],
                       Bo.cuda(), EP.cuda()], 0, 1e-5, H, MP, HR)
    cache = F.TppCache(cap)
    k0, v0 = randn_bf16((B, N, past, H), 1.0, 461), randn_bf16((B, N, past, H), 1.0, 462)
    if past:
        cache.fill_(0, k0.cuda(), v0.cuda())
    x = randn_bf16((B, S, hidden), 1.0, 463)
    pos = torch.arange(past, past + S, dtype=torch.int64).unsqueeze(0)
    out = blk.forward([x.cuda(), None, pos.cuda()], cache, True)[0]
    cache.advance(S)
    assert out.shape == (B, S, hidden) and cache.get_seq_length() == past + S

    xb = t2bits(x).reshape(B * S, hidden)
    h = O.layer_norm(xb, g.float().numpy(), bt.float().numpy(), 1e-5)
    q, k, v = _mm(fmt, h, Ws[0]), _mm(fmt, h, Ws[1]), _mm(fmt, h, Ws[2])
    q = O.rotary_gptj(q.reshape(B, S, -1), EP.numpy(), pos.numpy(), N, H).reshape(B, S, N, H)
    k = O.rotary_gptj(k.reshape(B, S, -1), EP.numpy(), pos.numpy(), N, H).reshape(B, S, N, H).transpose(0, 2, 1, 3)
    v = v.reshape(B, S, N, H).transpose(0, 2, 1, 3)
    kall, vall = np.concatenate([t2bits(k0), k], axis=2), np.concatenate([t2bits(v0), v], axis=2)
    if S == 1:
        ctxv = O.attn_decode(q.reshape(B, N, H), kall, vall).reshape(B, N * H)
    else:
        ctxv = O.attn_prefill(q, kall, vall).reshape(B * S, N * H)
    so = _mm(fmt, ctxv, Ws[3])
    inter_v = _mm(fmt, h, Ws[4], Bi, O.POST_GELU)
    ref = _mm(fmt, inter_v, Ws[5], Bo, O.POST_ADD2_SCALE, so, xb)
    assert _rel(out, ref) <= 2e-2
    kc, vc = cache.get(0)
    # Three chained operators (LayerNorm, GEMM, rotary) separate the cache from the input.  One normalised element
    # that lands on the other side of a bf16 rounding boundary (about one in a thousand does: fp32 summation order)
    # moves every key of its row by a few hundredths of an ulp, which flips the rounding of a few percent of them:
    # every element must be within one ulp (two for int8 activations), but their number is not bounded here.
    u = 2 if fmt == "qint8" else 1
    assert_close_bf16(t2bits(kc[:, :, past:]), np.ascontiguousarray(k), ulps=u, max_mismatch=None, what="cached keys")
    assert_close_bf16(t2bits(vc[:, :, past:]), np.ascontiguousarray(v), ulps=u, max_mismatch=None, what="cached values")
    from tpp_pytorch_extension._lib import TppxError
    with pytest.raises(TppxError):
        F.GPTJBlock([None] * 10, 0, 1e-5, H, MP, HR)


@pytest.mark.parametrize("fmt", ["mxfp4", "qint8"])
@pytest.mark.parametrize("before", [True, False])
@pytest.mark.parametrize("past,S", [(37, 1), (0, 70)])
def test_opt_decoder_layer_against_oracle(fmt, before, past, S):
    """OPTDecoderLayer.forward against the oracle composition (fused_llm_infer.cpp:1005-1060) for both placements
    of the LayerNorms: biases on every linear, no rotary, ReLU MLP."""
    F = _opt()
    hidden, inter, N, H = 512, 1024, 8, 64
    B, cap = 2, 128
    rng = torch.Generator().manual_seed(500)
    Ws = [_lin(fmt, hidden, hidden, 501 + i) for i in range(4)] + [_lin(fmt, inter, hidden, 505), _lin(fmt, hidden, inter, 506)]
    Bs = [randn_bf16((hidden,), 0.3, 507 + i) for i in range(4)] + [randn_bf16((inter,), 0.3, 511), randn_bf16((hidden,), 0.3, 512)]
    ln = [(torch.rand(hidden, generator=rng) + 0.5).to(torch.bfloat16), (torch.randn(hidden, generator=rng) * 0.2).to(torch.bfloat16),
          (torch.rand(hidden, generator=rng) + 0.5).to(torch.bfloat16), (torch.randn(hidden, generator=rng) * 0.2).to(torch.bfloat16)]
    params = [t.cuda() for t in ln]
    for i in range(6):
        params += [Ws[i][0], Bs[i].cuda()]
    layer = F.OPTDecoderLayer(params, 0, 1e-5, 1e-5, H, before)
    cache = F.TppCache(cap)
    k0, v0 = randn_bf16((B, N, past, H), 1.0, 561), randn_bf16((B, N, past, H), 1.0, 562)
    if past:
        cache.fill_(0, k0.cuda(), v0.cuda())
    x = randn_bf16((B, S, hidden), 1.0, 563)
    out = layer.forward([x.cuda(), None], cache, True)[0]
    cache.advance(S)
    assert out.shape == (B, S, hidden) and cache.get_seq_length() == past + S

    def lnorm(bits, i):
        return O.layer_norm(bits, ln[2 * i].float().numpy(), ln[2 * i + 1].float().numpy(), 1e-5)

    xb = t2bits(x).reshape(B * S, hidden)
    h = lnorm(xb, 0) if before else xb
    q, k, v = _mm(fmt, h, Ws[0], Bs[0]), _mm(fmt, h, Ws[1], Bs[1]), _mm(fmt, h, Ws[2], Bs[2])
    q = q.reshape(B, S, N, H)
    k = k.reshape(B, S, N, H).transpose(0, 2, 1, 3)
    v = v.reshape(B, S, N, H).transpose(0, 2, 1, 3)
    kall, vall = np.concatenate([t2bits(k0), k], axis=2), np.concatenate([t2bits(v0), v], axis=2)
    if S == 1:
        ctxv = O.attn_decode(q.reshape(B, N, H), kall, vall).reshape(B, N * H)
    else:
        ctxv = O.attn_prefill(q, kall, vall).reshape(B * S, N * H)
    hs = _mm(fmt, ctxv, Ws[3], Bs[3], O.POST_ADD_SCALE, xb)
    if not before:
        hs = lnorm(hs, 0)
    res = hs
    if before:
        hs = lnorm(hs, 1)
    hs = _mm(fmt, hs, Ws[4], Bs[4], O.POST_RELU)
    ref = _mm(fmt, hs, Ws[5], Bs[5], O.POST_ADD_SCALE, res)
    if not before:
        ref = lnorm(ref, 1)
    assert _rel(out, ref) <= 2e-2
    kc, vc = cache.get(0)
    u = 2 if fmt == "qint8" else 1
    assert_close_bf16(t2bits(kc[:, :, past:]), np.ascontiguousarray(k), ulps=u, max_mismatch=None, what="cached keys (not rotated)")
    assert_close_bf16(t2bits(vc[:, :, past:]), np.ascontiguousarray(v), ulps=u, max_mismatch=None, what="cached values")


def _dequantized_copy(ref_model, weight_dtype):
    """Weights := dequantize(quantize(weights)) and bf16-rounded embeddings / vectors, as the fused model sees them."""
    with torch.no_grad():
        for m in ref_model.modules():
            if isinstance(m, torch.nn.Linear):
                w = m.weight.data.to(torch.bfloat16).float()
                if w.shape[0] % 32 == 0 and w.shape[1] % 128 == 0 and getattr(m, "_quantize_me", True) and weight_dtype != "bf16":
                    if weight_dtype == "mxfp4":
                        q, sc = O.remap_quantize_mxfp4(w.numpy())
                        w = torch.from_numpy(O.dequantize_mxfp4_plain(q, sc))
                    else:
                        q, sc, _ = O.remap_quantize_qint8(w.numpy())
                        w = torch.from_numpy(O.dequantize_qint8_plain(q, sc))
                m.weight.data.copy_(w)
                if m.bias is not None:
                    m.bias.data.copy_((torch.randn_like(m.bias) * 0.3).to(torch.bfloat16).float())
            elif isinstance(m, torch.nn.Embedding):
                m.weight.data.copy_(m.weight.data.to(torch.bfloat16).float())
            elif isinstance(m, torch.nn.LayerNorm):
                m.weight.data.copy_((torch.rand_like(m.weight) + 0.5).to(torch.bfloat16).float())
                m.bias.data.copy_((torch.randn_like(m.bias) * 0.2).to(torch.bfloat16).float())


def _compare_with_stock(ref_model, opt_model, tol, vocab, generate):
    ids = torch.randint(0, vocab, (2, 19), generator=torch.Generator().manual_seed(32))
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
        assert cache_o.get_seq_length() == 19
        for step in range(2):
            nxt = r.logits[:, -1].argmax(-1, keepdim=True)
            am = torch.cat([am, torch.ones(2, 1, dtype=am.dtype)], 1)
            pos = pos[:, -1:] + 1
            r = ref_model(input_ids=nxt, attention_mask=am, position_ids=pos, past_key_values=cache_r, use_cache=True)
            o = opt_model(input_ids=nxt.cuda(), attention_mask=am.cuda(), position_ids=pos.cuda(),
                          past_key_values=cache_o, use_cache=True)
            assert rel(o.logits.float().cpu(), r.logits) <= tol
        assert cache_o.get_seq_length() == 21
    out = generate(opt_model, ids[:1].cuda(), 5)
    assert out.shape == (1, 24) and torch.equal(out[:, :19].cpu(), ids[:1])


@pytest.mark.parametrize("weight_dtype", ["mxfp4", "qint8", "bf16"])
def test_optimize_model_for_gptj_against_transformers(weight_dtype):
    """OptimizeModelForGPTJ on a random-initialised transformers GPTJForCausalLM (2 blocks, 4 heads of 128, rotary
    on 64 dims) against the stock model in fp32 on the CPU holding the dequantized weights.  The stock model is
    configured with the erf GELU, which is what GeluPostOp computes (fused_gemm.h:1349, xsmm_functors.h:2794)."""
    transformers = pytest.importorskip("transformers")
    F = _gj()
    cfg = transformers.GPTJConfig(n_embd=512, n_head=4, n_layer=2, n_positions=256, rotary_dim=64, vocab_size=1600,
                                  activation_function="gelu", bos_token_id=1, eos_token_id=2,
                                  attn_implementation="eager", resid_pdrop=0.0, embd_pdrop=0.0, attn_pdrop=0.0)
    torch.manual_seed(41)
    ref_model = transformers.GPTJForCausalLM(cfg).eval()
    ref_model.lm_head._quantize_me = False
    _dequantized_copy(ref_model, weight_dtype)
    opt_model = F.OptimizeModelForGPTJ(copy.deepcopy(ref_model), torch.bfloat16, "cuda",
                                       None if weight_dtype == "bf16" else weight_dtype).eval()
    assert type(opt_model.transformer.h[0].cpp_block).__name__ == "GPTJBlock"
    _compare_with_stock(ref_model, opt_model, 3e-2 if weight_dtype == "mxfp4" else 6e-2, 1600, F.generate_greedy)


@pytest.mark.parametrize("weight_dtype", ["mxfp4", "qint8", "bf16"])
@pytest.mark.parametrize("before,proj,hidden", [(True, 512, 512), (False, 512, 512), (True, 256, 512), (True, 640, 640)])
def test_optimize_model_for_opt_against_transformers(weight_dtype, before, proj, hidden):
    """OptimizeModelForOPT on a random-initialised transformers OPTForCausalLM (2 layers, 8 heads of 64 -- or of 80,
    a head size that is no power of two, as OPT-2.7B has; LayerNorm before or after each half; with and without the
    project_in / project_out linears) against the stock model in fp32 on the CPU holding the dequantized weights."""
    transformers = pytest.importorskip("transformers")
    F = _opt()
    cfg = transformers.OPTConfig(hidden_size=hidden, ffn_dim=2 * hidden, num_hidden_layers=2, num_attention_heads=8,
                                 vocab_size=1024, max_position_embeddings=256, do_layer_norm_before=before,
                                 word_embed_proj_dim=proj, dropout=0.0, attention_dropout=0.0, layerdrop=0.0,
                                 bos_token_id=1, eos_token_id=2, pad_token_id=0, attn_implementation="eager",
                                 tie_word_embeddings=False)
    torch.manual_seed(51)
    ref_model = transformers.OPTForCausalLM(cfg).eval()
    ref_model.lm_head._quantize_me = False
    if ref_model.model.decoder.project_in is not None:
        ref_model.model.decoder.project_in._quantize_me = False
        ref_model.model.decoder.project_out._quantize_me = False
    _dequantized_copy(ref_model, weight_dtype)
    opt_model = F.OptimizeModelForOPT(copy.deepcopy(ref_model), torch.bfloat16, "cuda",
                                      None if weight_dtype == "bf16" else weight_dtype).eval()
    assert type(opt_model.model.decoder.layers[0].cpp_block).__name__ == "OPTDecoderLayer"
    _compare_with_stock(ref_model, opt_model, 3e-2 if weight_dtype == "mxfp4" else 6e-2, 1024, F.generate_greedy)


@pytest.mark.parametrize("family", ["llama", "qwen2", "gptj", "opt"])
def test_transformers_generate_on_optimized_models(family):
    """transformers' own generate() (greedy, left-padded batch) runs on the optimized model of every family and
    returns the tokens of this package's plain greedy loop."""
    T = pytest.importorskip("transformers")
    import tpp_pytorch_extension  # noqa: F401
    from tpp_pytorch_extension.llm import fused_llama_infer as FL, fused_qwen2_infer as FQ
    torch.manual_seed(7)
    if family == "llama":
        model = T.LlamaForCausalLM(T.LlamaConfig(hidden_size=512, intermediate_size=1024, num_hidden_layers=2,
                                                 num_attention_heads=4, num_key_value_heads=2, vocab_size=1024,
                                                 max_position_embeddings=256, head_dim=128))
        opt, F = FL.OptimizeModelForLlama(model.eval(), torch.bfloat16, "cuda", "mxfp4"), FL
    elif family == "qwen2":
        model = T.Qwen2ForCausalLM(T.Qwen2Config(hidden_size=512, intermediate_size=1024, num_hidden_layers=2,
                                                 num_attention_heads=4, num_key_value_heads=2, vocab_size=1024,
                                                 max_position_embeddings=256, use_sliding_window=False,
                                                 tie_word_embeddings=False))
        opt, F = FQ.OptimizeModelForQwen2(model.eval(), torch.bfloat16, "cuda", "mxfp4"), FQ
    elif family == "gptj":
        model = T.GPTJForCausalLM(T.GPTJConfig(n_embd=512, n_head=4, n_layer=2, n_positions=256, rotary_dim=64,
                                               vocab_size=1600, bos_token_id=1, eos_token_id=2))
        opt, F = _gj().OptimizeModelForGPTJ(model.eval(), torch.bfloat16, "cuda", "mxfp4"), _gj()
    else:
        model = T.OPTForCausalLM(T.OPTConfig(hidden_size=512, ffn_dim=1024, num_hidden_layers=2, num_attention_heads=8,
                                             vocab_size=1024, max_position_embeddings=256, bos_token_id=1,
                                             eos_token_id=2, pad_token_id=0))
        opt, F = _opt().OptimizeModelForOPT(model.eval(), torch.bfloat16, "cuda", "mxfp4"), _opt()
    opt = opt.eval()
    ids = torch.randint(3, 1000, (2, 11), generator=torch.Generator().manual_seed(8)).cuda()
    am = torch.ones_like(ids)
    am[1, :3] = 0
    out = opt.generate(input_ids=ids, attention_mask=am, max_new_tokens=4, do_sample=False, pad_token_id=0)
    assert out.shape == (2, 15) and torch.equal(out[:, :11], ids)
    ref = F.generate_greedy(opt, ids, 4, attention_mask=am)
    assert torch.equal(out, ref)
    # the same tokens with the decode steps replayed from one graph (longer, so that the cache crosses a block of 32)
    long_ref = F.generate_greedy(opt, ids, 30, attention_mask=am)
    long_graph = F.generate_greedy_graph(opt, ids, 30, attention_mask=am)
    assert long_graph.shape == (2, 41) and torch.equal(long_graph, long_ref)
    assert torch.equal(F.generate_greedy_graph(opt, ids[:1], 1), F.generate_greedy(opt, ids[:1], 1))
    from tpp_pytorch_extension._lib import TppxError
    with pytest.raises(TppxError):
        F.generate_greedy_graph(opt, ids, 400, attention_mask=am)  # 11 + 400 keys do not fit the cache of 256
