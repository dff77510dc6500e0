"""Every BASELINE configuration against the CPU oracle at its REAL shape, through the same op calls (and therefore
the same launch plans: kernel, grid, K split) that bench.py times.

Tolerances are those of test_gpu_linear.py: every output within 1 bf16 ulp of the ideal oracle (2 through SiLU),
rel-L2 <= 4e-3; against the reference's chunked bf16 re-rounding (faithful mode) rel-L2 <= 2^-9 * sqrt(#chunks);
a whole decoder-layer step rel-L2 <= 2e-2 against the composition of the oracle functions.
"""
import ctypes

import numpy as np
import pytest
import torch

import oracle as O
from util import t2bits, randn_bf16, block_bf16, bits2f, assert_close_bf16, err_stats

pytestmark = pytest.mark.gpu

_CACHE = {}


def _ops():
    import tpp_pytorch_extension  # noqa: F401
    from tpp_pytorch_extension import _ops
    return _ops


def _weight(fmt, N, K, seed):
    """(GPU quantized tensor, oracle qdata, oracle scales), quantized once per (format, shape, seed); the GPU bytes
    must equal the oracle's before any GEMM is compared."""
    key = (fmt, N, K, seed)
    if key not in _CACHE:
        ops = _ops()
        W = randn_bf16((N, K), 0.02, seed)
        Wb = block_bf16(W).cuda()
        if fmt == "mxfp4":
            qw = ops.remap_and_quantize_mxfp4(Wb)
            q_or, s_or = O.remap_quantize_mxfp4(W.float().numpy())
        else:
            qw = ops.remap_and_quantize_qint8(Wb)
            q_or, s_or, _ = O.remap_quantize_qint8(W.float().numpy())
        assert np.array_equal(qw.qdata.cpu().numpy(), q_or), "quantized values differ from the oracle"
        assert np.array_equal(qw.scales.cpu().numpy().reshape(s_or.shape), s_or), "scales differ from the oracle"
        del W, Wb
        _CACHE[key] = (qw, q_or, s_or)
    return _CACHE[key]


def _plan(fmt, M, N, K, qbs=256):
    """Kernel names the library launches for this call with the package's workspace (what bench.py reports)."""
    from tpp_pytorch_extension import _lib
    L = _lib.lib()
    buf = ctypes.create_string_buffer(4096)
    if fmt == "qint8":
        _lib.check(L.tppx_plan_linear_qint8(M, N, K, qbs, 1, 0, _lib.WORKSPACE_BYTES, buf, len(buf)))
    else:
        _lib.check(L.tppx_plan_linear_mxfp4(M, N, K, 0, _lib.WORKSPACE_BYTES, buf, len(buf)))
    return [ln.split(" grid=")[0].replace("void ", "") for ln in buf.value.decode().strip().splitlines()]


# ---------------------------------------------------------------------------------------------------------------
# config 1 is covered at full size by test_gpu_linear.py::test_cfg1_mxfp4_fc_plain
# config 2: QINT8 fc_add, up 4096 -> 11008 (test_gpu_linear.py::test_cfg2_qint8_up_projection_full_size) and
#           down 11008 -> 4096 (here)
# ---------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("M", [1, 8, 32, 64])
def test_cfg2_qint8_down_projection_full_size(M):
    """N = 4096, K = 11008: 256 channel tiles (one per workgroup, or K split across workgroups at 64 rows), 43 scale
    blocks over the waves; also the reference's own re-rounding schedule (64-wide groups below 64 rows, 256-wide
    at 64 rows)."""
    import bench
    assert (4096, 11008) in bench.CFG2_SHAPES.values() and M in bench.CFG2_MS
    qw, q_or, s_or = _weight("qint8", 4096, 11008, 2242)
    x = randn_bf16((M, 11008), 1.0, 2300 + M)
    r = randn_bf16((M, 4096), 1.0, 2400 + M)
    y = torch.ops.tpp_llm.fc_add(x.cuda(), qw, torch.Tensor(), r.cuda(), 1.0)
    ref = O.linear_qint8(t2bits(x), q_or, s_or, None, O.POST_ADD_SCALE, t2bits(r), None, 1.0, O.MODE_IDEAL)
    pre = O.linear_qint8(t2bits(x), q_or, s_or)
    assert_close_bf16(t2bits(y), ref, what=f"cfg2 down M={M}", pre_bits=pre)
    faithful = O.linear_qint8(t2bits(x), q_or, s_or, None, O.POST_ADD_SCALE, t2bits(r), None, 1.0, O.MODE_FAITHFUL)
    groups = 11008 // (256 if M == 64 else 64)
    assert err_stats(t2bits(y), faithful)["rel_l2"] <= 2.0 ** -9 * np.sqrt(groups)
    names = _plan("qint8", M, 4096, 11008)
    assert names and names[-1].startswith("tppx::skinny_qint8"), names
    # the same bits on a second call (K-split arrival counters back at zero)
    assert torch.equal(y, torch.ops.tpp_llm.fc_add(x.cuda(), qw, torch.Tensor(), r.cuda(), 1.0))


# ---------------------------------------------------------------------------------------------------------------
# config 3: MXFP4 SwiGLU MLP block 4096 -> 11008 -> 4096 through torch.ops.tpp_llm.swiglu_mlp
# ---------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("M", [1, 4, 16, 64])
def test_cfg3_mxfp4_swiglu_mlp_full_size(M):
    ops = _ops()
    wg, qg, sg = _weight("mxfp4", 11008, 4096, 3301)
    wu, qu, su = _weight("mxfp4", 11008, 4096, 3302)
    wd, qd, sd = _weight("mxfp4", 4096, 11008, 3303)
    x = randn_bf16((M, 4096), 1.0, 3310 + M)
    xg = x.cuda()
    out = torch.ops.tpp_llm.swiglu_mlp(xg, wg, wu, wd, xg, 1.0)  # residual = the block's input
    xb = t2bits(x)
    gate = O.linear_mxfp4(xb, qg, sg, None, O.POST_SILU)
    inter = O.linear_mxfp4(xb, qu, su, None, O.POST_MUL, gate)
    # the gate/up launch against the oracle, then the down projection on the GPU's own intermediate (so that its
    # 1-ulp bound is not blurred by the intermediate's), then the whole block
    got_inter = ops.swiglu_gate_up(xg, wg, wu)
    assert_close_bf16(t2bits(got_inter), inter, ulps=2, what=f"cfg3 gate/up M={M}")
    gi = t2bits(got_inter)
    ref = O.linear_mxfp4(gi, qd, sd, None, O.POST_ADD_SCALE, xb, None, 1.0)
    pre = O.linear_mxfp4(gi, qd, sd)
    assert_close_bf16(t2bits(out), ref, what=f"cfg3 block M={M}", pre_bits=pre)
    whole = O.linear_mxfp4(inter, qd, sd, None, O.POST_ADD_SCALE, xb, None, 1.0)
    assert err_stats(t2bits(out), whole)["rel_l2"] <= 4e-3
    # fused == composition of the three reference ops, bit for bit
    g = ops.fc_silu(xg, wg, None)
    u = ops.fc_mul(xg, wu, None, g)
    assert torch.equal(got_inter, u)
    assert torch.equal(out, ops.fc_add(u, wd, None, xg, 1.0))
    for n, k in ((11008, 4096), (4096, 11008)):
        names = _plan("mxfp4", M, n, k)
        assert names and names[-1].startswith("tppx::skinny_mxfp4"), names


# ---------------------------------------------------------------------------------------------------------------
# config 4: M = 2048 prefill GEMMs at the 70B layer dims
# ---------------------------------------------------------------------------------------------------------------
def test_cfg4_down_projection_k28672_slice():
    """K = 28672 (224 K steps of the large-M kernel, 7 of the reference's 4096-wide chunks) on a 256-channel slice,
    all 2048 rows, with bias and the residual: ideal oracle (1 ulp) and the reference's chunked re-rounding."""
    ops = _ops()
    M, N, K = 2048, 256, 28672
    qw, q_or, s_or = _weight("mxfp4", N, K, 4401)
    x = randn_bf16((M, K), 1.0, 4402)
    bias = randn_bf16((N,), 0.01, 4403)
    r = randn_bf16((M, N), 1.0, 4404)
    y = ops.fc_add(x.cuda(), qw, bias.cuda(), r.cuda(), 1.0)
    ref = O.linear_mxfp4(t2bits(x), q_or, s_or, t2bits(bias), O.POST_ADD_SCALE, t2bits(r), None, 1.0, O.MODE_IDEAL)
    pre = O.linear_mxfp4(t2bits(x), q_or, s_or, t2bits(bias))
    assert_close_bf16(t2bits(y), ref, what="cfg4 down slice", pre_bits=pre)
    faithful = O.linear_mxfp4(t2bits(x), q_or, s_or, t2bits(bias), O.POST_ADD_SCALE, t2bits(r), None, 1.0,
                              O.MODE_FAITHFUL)
    assert err_stats(t2bits(y), faithful)["rel_l2"] <= 2.0 ** -9 * np.sqrt(7)
    assert _plan("mxfp4", M, 8192, K)[-1].startswith("tppx::big_mxfp4_kernel")


_ROWS = np.array(sorted(set([0, 1, 15, 16, 127, 128, 255, 256, 257, 1023, 1024, 2046, 2047] +
                            list(np.random.default_rng(44).choice(2048, 64, replace=False)))))


def _sampled(y, rows):
    return t2bits(y[torch.from_numpy(rows).cuda()])


def test_cfg4_full_n_qkv_and_o():
    """The fused q/k/v launch (N = 8192 + 1024 + 1024 = 640 workgroups of 128 rows) and the o-projection (8192,
    with the residual) at M = 2048, K = 8192: 77 sampled rows (block edges + 64 random) of every output against the
    oracle, all 2048 rows fused == separate bit for bit."""
    ops = _ops()
    M, K = 2048, 8192
    ws = [_weight("mxfp4", n, K, 4410 + i) for i, n in enumerate((8192, 1024, 1024))]
    x = randn_bf16((M, K), 1.0, 4420)
    xg = x.cuda()
    outs = torch.ops.tpp_llm.qkv_gemm(xg, [w[0] for w in ws], [torch.Tensor()] * 3)
    xs = t2bits(x)[_ROWS]
    for (qw, q_or, s_or), o in zip(ws, outs):
        assert torch.equal(o, ops.fc_plain(xg, qw, None))
        ref = O.linear_mxfp4(xs, q_or, s_or)
        assert_close_bf16(_sampled(o, _ROWS), ref, what=f"cfg4 qkv N={o.shape[-1]}")
    # o-projection on the q output, residual = x
    qw, q_or, s_or = _weight("mxfp4", 8192, K, 4413)
    h = ops.fc_add(outs[0], qw, None, xg, 1.0)
    qs = t2bits(outs[0])[_ROWS]
    ref = O.linear_mxfp4(qs, q_or, s_or, None, O.POST_ADD_SCALE, xs, None, 1.0)
    assert_close_bf16(_sampled(h, _ROWS), ref, what="cfg4 o-projection", pre_bits=O.linear_mxfp4(qs, q_or, s_or))
    assert _plan("mxfp4", M, 10240, K)[-1].startswith("tppx::big_mxfp4_kernel")


def test_cfg4_full_n_gate_up_and_down():
    """gate / up (N = 28672 each, ONE grid of 1792 workgroups with the gate tile parked in the workspace, then the
    elementwise pass) and the down projection (K = 28672, N = 8192) at M = 2048: sampled rows against the oracle,
    all rows fused == fc_silu then fc_mul bit for bit."""
    ops = _ops()
    M, H, I = 2048, 8192, 28672
    wg, qg, sg = _weight("mxfp4", I, H, 4431)
    wu, qu, su = _weight("mxfp4", I, H, 4432)
    x = randn_bf16((M, H), 1.0, 4433)
    xg = x.cuda()
    inter = ops.swiglu_gate_up(xg, wg, wu)
    g = ops.fc_silu(xg, wg, None)
    assert torch.equal(inter, ops.fc_mul(xg, wu, None, g))
    del g
    xs = t2bits(x)[_ROWS]
    gate = O.linear_mxfp4(xs, qg, sg, None, O.POST_SILU)
    ref = O.linear_mxfp4(xs, qu, su, None, O.POST_MUL, gate)
    assert_close_bf16(_sampled(inter, _ROWS), ref, ulps=2, what="cfg4 gate/up")
    del _CACHE[("mxfp4", I, H, 4431)], _CACHE[("mxfp4", I, H, 4432)]
    wd, qd, sd = _weight("mxfp4", H, I, 4434)
    out = ops.fc_add(inter, wd, None, xg, 1.0)
    its = t2bits(inter)[_ROWS]
    ref = O.linear_mxfp4(its, qd, sd, None, O.POST_ADD_SCALE, xs, None, 1.0)
    assert_close_bf16(_sampled(out, _ROWS), ref, what="cfg4 down", pre_bits=O.linear_mxfp4(its, qd, sd))
    # the MLP op = the same three calls
    assert torch.equal(out, torch.ops.tpp_llm.swiglu_mlp(xg, wg, wu, wd, xg, 1.0))
    del _CACHE[("mxfp4", H, I, 4434)]


# ---------------------------------------------------------------------------------------------------------------
# config 5: one decoder layer of the 7B-shape model at full size, one decode step on a 2048-token cache
# ---------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("B", [1, 16])
def test_cfg5_full_size_layer_step(B):
    """hidden 4096, 32 heads x 128, intermediate 11008, cache of 2048 positions of N(0,1): LlamaDecoderLayer.forward
    for one new token per sequence against the composition of the oracle functions (fused_llm_infer.cpp:1229-1275),
    and the key / value it appends."""
    import tpp_pytorch_extension  # noqa: F401
    from tpp_pytorch_extension.llm import fused_llama_infer as F
    hidden, inter, Nh, H, MP = 4096, 11008, 32, 128, 4096
    ctx, cap = 2048, 2048 + 160
    Ws = [_weight("mxfp4", n, k, 5500 + i) for i, (n, k) in enumerate(
        [(hidden, hidden)] * 4 + [(inter, hidden)] * 2 + [(hidden, inter)])]
    rng = torch.Generator().manual_seed(55)
    g1 = torch.rand(hidden, generator=rng) + 0.5
    g2 = torch.rand(hidden, generator=rng) + 0.5
    EP = F.llama_rotary_table(MP, H, device="cpu")
    layer = F.LlamaDecoderLayer([g1.cuda(), Ws[0][0], Ws[1][0], Ws[2][0], Ws[3][0], g2.cuda(), Ws[4][0], Ws[5][0],
                                 Ws[6][0], EP.cuda()], 0, 1e-5, H, MP, H)
    cache = F.TppCache(cap)
    k0, v0 = randn_bf16((B, Nh, ctx, H), 1.0, 5561), randn_bf16((B, Nh, ctx, H), 1.0, 5562)
    cache.fill_(0, k0.cuda(), v0.cuda())
    x = randn_bf16((B, 1, hidden), 1.0, 5563)
    pos = torch.full((B, 1), ctx, dtype=torch.int64)
    out = layer.forward([x.cuda(), None, pos.cuda()], cache, True)[0]
    cache.advance(1)

    def mm(a_bits, w, post=O.POST_NONE, post_in=None):
        return O.linear_mxfp4(a_bits, w[1], w[2], None, post, post_in, None, 1.0, O.MODE_IDEAL)

    xb = t2bits(x).reshape(B, hidden)
    h = O.rms_norm(xb, g1.numpy(), 1e-5)
    q, k, v = mm(h, Ws[0]), mm(h, Ws[1]), mm(h, Ws[2])
    q = O.rotary_llama(q.reshape(B, 1, -1), EP.numpy(), pos.numpy(), Nh, H).reshape(B, Nh, H)
    k = O.rotary_llama(k.reshape(B, 1, -1), EP.numpy(), pos.numpy(), Nh, H).reshape(B, Nh, 1, H)
    kall = np.concatenate([t2bits(k0), k], axis=2)
    vall = np.concatenate([t2bits(v0), v.reshape(B, Nh, 1, H)], axis=2)
    ctxv = O.attn_decode(q, kall, vall).reshape(B, Nh * H)
    so = mm(ctxv, Ws[3], O.POST_ADD_SCALE, xb)
    h2 = O.rms_norm(so, g2.numpy(), 1e-5)
    gate = mm(h2, Ws[4], O.POST_SILU)
    ref = mm(mm(h2, Ws[5], O.POST_MUL, gate), Ws[6], O.POST_ADD_SCALE, so)
    g, r = bits2f(t2bits(out)).reshape(B, hidden).astype(np.float64), bits2f(ref).astype(np.float64)
    rel = np.sqrt(((g - r) ** 2).sum() / (r ** 2).sum())
    assert rel <= 2e-2, rel
    kc, vc = cache.get(0)
    assert kc.shape[2] == ctx + 1
    assert_close_bf16(t2bits(kc[:, :, ctx]), k.reshape(B, Nh, H), what="cached key")
    assert_close_bf16(t2bits(vc[:, :, ctx]), v.reshape(B, Nh, H), what="cached value")
    assert torch.equal(kc[:, :, :ctx].cpu(), k0)


# ---------------------------------------------------------------------------------------------------------------
# config 5 as bench.py runs it: the 32-layer 7B-shape decoder, 2048-token context, 128 greedy tokens from one
# replayed graph.  No oracle finishes 32 layers x 128 steps in seconds, so the chain is held by properties: the
# replayed steps give the tokens of eager launches of the same kernels (first 8 steps), every token is a vocabulary
# id, the counters end at 2048 + 128 in every layer, and the appended keys are there (non-zero) and nothing beyond.
# ---------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("B", [1, 16])
def test_cfg5_full_size_greedy_chain(B):
    import bench
    model = bench.cfg5_model(torch)
    assert model.n_layers == 32 and model.hidden == 4096 and model.vocab == 32000
    ctx, new = 2048, 128
    tok = torch.randint(0, 32000, (B,), generator=torch.Generator().manual_seed(5), dtype=torch.int64).cuda()
    cache = model.new_cache(B, ctx, ctx + new + 32)
    out = model.greedy_decode(tok, cache, new)  # one graph, 128 replays
    torch.cuda.synchronize()
    assert out.shape == (B, new) and int(out.min()) >= 0 and int(out.max()) < 32000
    assert int(cache.seq_len_dev.item()) == ctx + new
    assert [cache.get_seq_length(i) for i in (0, 15, 31)] == [ctx + new] * 3
    for i in (0, 31):
        k, v = cache.layers[i]
        assert bool((k[:, :, ctx:ctx + new].float().abs().amax(dim=-1) > 0).all()), "a replayed step left no key"
        assert float(k[:, :, ctx + new:].float().abs().max()) == 0.0 and float(v[:, :, ctx + new:].float().abs().max()) == 0.0
    del cache
    eager_cache = model.new_cache(B, ctx, ctx + new + 32)  # same seed: the same context
    eager = model.greedy_decode(tok, eager_cache, 8, use_graph=False)
    assert torch.equal(out[:, :8], eager), "replayed steps and eager steps give different tokens"
    del eager_cache
    bench._MODEL.clear()
    torch.cuda.empty_cache()
