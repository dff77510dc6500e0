"""Parity of the decode-side operators (RMSNorm, rotary, KV append, decode
attention) and of one decoder-layer step against the numpy restatements in
oracle/ and against plain PyTorch fp32 references.

Stated tolerances (floating-point kernels): RMSNorm and rotary within 1 bf16 ulp
of the fp32 recipe; attention rel-L2 <= 5e-3 and every element within
2^-7 * max|out| of the fp64 answer (probabilities rounded to bf16 as the
reference stores them); a whole layer step rel-L2 <= 2e-2 against the
composition of the oracle functions.
"""
import numpy as np
import pytest
import torch

import oracle as O
from util import t2bits, randn_bf16, block_bf16, bits2f, assert_close_bf16

pytestmark = pytest.mark.gpu


def _llm():
    import tpp_pytorch_extension  # noqa: F401
    from tpp_pytorch_extension.llm import fused_llama_infer as F
    return F


@pytest.mark.parametrize("K", [4096, 1000, 8])
@pytest.mark.parametrize("gdt", [torch.float32, torch.bfloat16])
def test_rms_norm(K, gdt):
    F = _llm()
    x = randn_bf16((7, 3, K), 1.5, 11)
    g = (torch.randn(K, generator=torch.Generator().manual_seed(12)) * 0.5 + 1.0).to(gdt)
    y = F.rms_norm(x.cuda(), g.cuda(), 1e-5)
    ref = O.rms_norm(t2bits(x).reshape(-1, K), g.float().numpy(), 1e-5)
    assert_close_bf16(t2bits(y).reshape(-1, K), ref, what=f"rms_norm K={K}")
    # independent torch fp32 statement of the same formula
    xf = x.float()
    t = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-5)) * g.float()
    assert_close_bf16(t2bits(y).reshape(-1, K), t2bits(t.to(torch.bfloat16)).reshape(-1, K), what="rms_norm vs torch")


@pytest.mark.parametrize("H,HR", [(128, 128), (128, 64), (96, 96), (80, 32), (200, 80)])
def test_rotary_llama(H, HR):
    F = _llm()
    B, S, N, MP = 2, 5, 6, 64
    t = randn_bf16((B, S, N * H), 1.0, 21)
    emb = F.llama_rotary_table(MP, HR, device="cpu")
    pos = torch.tensor([[3, 9, 63, 64, 0], [1, 2, 3, 4, 70]], dtype=torch.int64)  # 64 and 70 are out of range: untouched
    got = F.apply_rotary_pos_emb_llama(t.clone().cuda(), emb.cuda(), pos.cuda(), N, H)
    ref = O.rotary_llama(t2bits(t), emb.numpy(), pos.numpy(), N, H)
    assert_close_bf16(t2bits(got), ref, what=f"rotary HR={HR}")
    # untouched positions are bit-identical to the input
    assert torch.equal(got.cpu()[0, 3], t[0, 3]) and torch.equal(got.cpu()[1, 4], t[1, 4])
    # broadcast positions ([1][S])
    got1 = F.apply_rotary_pos_emb_llama(t.clone().cuda(), emb.cuda(), pos[:1].cuda(), N, H)
    ref1 = O.rotary_llama(t2bits(t), emb.numpy(), pos[:1].numpy(), N, H)
    assert_close_bf16(t2bits(got1), ref1, what="rotary broadcast positions")


def _attn(F, q, kc, vc, L, mask=None, ws=True):
    from tpp_pytorch_extension import _lib
    Lb = _lib.lib()
    B, Nq, H = q.shape
    Nkv, Smax = kc.shape[1], kc.shape[2]
    out = torch.empty_like(q)
    ln = torch.tensor([L - 1], dtype=torch.int32, device="cuda")  # counter before the append, +1 in the call
    w = _lib.workspace(q)
    _lib.check(Lb.tppx_attn_decode(q.data_ptr(), kc.data_ptr(), vc.data_ptr(),
                                   None if mask is None else mask.data_ptr(), 0 if mask is None else mask.shape[1],
                                   ln.data_ptr(), 1, out.data_ptr(), B, Nq, Nkv, H, Smax,
                                   w.data_ptr() if ws else None, w.numel() if ws else 0, _lib.stream_of(q)))
    return out


@pytest.mark.parametrize("kernel", ["auto", "rows", "wide"])
@pytest.mark.parametrize("B,Nq,Nkv,L,Smax", [(1, 32, 32, 2048, 2304), (3, 8, 2, 77, 128), (2, 4, 4, 1, 64),
                                             (16, 32, 32, 300, 512), (1, 32, 32, 129, 4096), (2, 8, 8, 1000, 1000)])
def test_attn_decode(B, Nq, Nkv, L, Smax, kernel, monkeypatch):
    """Both single-query kernels (64 keys per trip on scalar arithmetic; 128 keys per trip on the packed bf16 dot
    instruction) on every shape, and the launch planner's own choice."""
    if kernel != "auto":
        monkeypatch.setenv("TPPX_ATTN_WIDE", "1" if kernel == "wide" else "0")
    F = _llm()
    q = randn_bf16((B, Nq, 128), 1.0, 31)
    k = randn_bf16((B, Nkv, Smax, 128), 1.0, 32)
    v = randn_bf16((B, Nkv, Smax, 128), 1.0, 33)
    got = _attn(F, q.cuda(), k.cuda(), v.cuda(), L)
    ref = O.attn_decode(t2bits(q), t2bits(k[:, :, :L]), t2bits(v[:, :, :L]))
    g, r = bits2f(t2bits(got)).astype(np.float64), bits2f(ref).astype(np.float64)
    rel = np.sqrt(((g - r) ** 2).sum() / (r ** 2).sum())
    assert rel <= 5e-3, rel
    assert np.abs(g - r).max() <= 2.0 ** -7 * np.abs(r).max()
    # one workgroup per head (no workspace) gives the same answer within the same bound
    got1 = _attn(F, q.cuda(), k.cuda(), v.cuda(), L, ws=False)
    g1 = bits2f(t2bits(got1)).astype(np.float64)
    assert np.sqrt(((g1 - r) ** 2).sum() / (r ** 2).sum()) <= 5e-3
    # plain PyTorch fp32 softmax attention
    kk = k[:, :, :L].float().repeat_interleave(Nq // Nkv, dim=1)
    vv = v[:, :, :L].float().repeat_interleave(Nq // Nkv, dim=1)
    s = torch.einsum("bnh,bnlh->bnl", q.float(), kk) / np.sqrt(128.0)
    t = torch.einsum("bnl,bnlh->bnh", torch.softmax(s, -1), vv).numpy().astype(np.float64)
    assert np.sqrt(((g - t) ** 2).sum() / (t ** 2).sum()) <= 1e-2


def test_attn_decode_split_merge_in_launch_equals_second_kernel(monkeypatch):
    """With a workspace the keys are split over several workgroups per head; the split that arrives last merges
    them inside the launch.  Twenty launches in a row (the arrival counters must return to zero) give the bits of
    the two-kernel path (TPPX_ATTN_ONE_LAUNCH=0), which merges in the same order."""
    F = _llm()
    B, Nq, Nkv, L, Smax = 2, 8, 4, 1500, 1536
    q = randn_bf16((B, Nq, 128), 1.0, 81).cuda()
    k = randn_bf16((B, Nkv, Smax, 128), 1.0, 82).cuda()
    v = randn_bf16((B, Nkv, Smax, 128), 1.0, 83).cuda()
    outs = [_attn(F, q, k, v, L) for _ in range(20)]
    monkeypatch.setenv("TPPX_ATTN_ONE_LAUNCH", "0")
    two = _attn(F, q, k, v, L)
    for o in outs:
        assert torch.equal(o, two)


@pytest.mark.parametrize("kernel", ["rows", "wide"])
@pytest.mark.parametrize("B,Nq,Nkv,L0,Smax,B_pos", [(1, 32, 32, 2048, 2304, 1), (3, 8, 2, 300, 512, 3), (2, 4, 4, 0, 64, 1),
                                                     (16, 32, 32, 77, 128, 16), (1, 8, 8, 255, 256, 1), (2, 4, 2, 128, 512, 2)])
def test_attn_decode_with_rotary_and_append_in_the_launch(B, Nq, Nkv, L0, Smax, B_pos, kernel, monkeypatch):
    monkeypatch.setenv("TPPX_ATTN_WIDE", "1" if kernel == "wide" else "0")
    """tppx_attn_decode_rotary = tppx_rotary_kv_append_llama + tppx_attn_decode(kv_len_add = 1) in one launch: same
    attention output (the rotation may contract its multiply-adds differently: bf16 tolerance), the same key / value
    row appended at position L0, nothing else in the cache touched, q / k / v inputs left as they were."""
    F = _llm()
    from tpp_pytorch_extension import _lib
    Lb = _lib.lib()
    MP = 4096
    EP = F.llama_rotary_table(MP, 128)
    q = randn_bf16((B, 1, Nq * 128), 1.0, 91).cuda()
    k = randn_bf16((B, 1, Nkv * 128), 1.0, 92).cuda()
    v = randn_bf16((B, 1, Nkv * 128), 1.0, 93).cuda()
    kc0 = randn_bf16((B, Nkv, Smax, 128), 1.0, 94).cuda()
    vc0 = randn_bf16((B, Nkv, Smax, 128), 1.0, 95).cuda()
    pos = (torch.arange(B_pos, dtype=torch.int64) * 3 + L0).view(B_pos, 1).cuda()
    ln = torch.tensor([L0], dtype=torch.int32, device="cuda")
    st = _lib.stream_of(q)
    w = _lib.workspace(q)
    # two launches
    qa, ka, kca, vca = q.clone(), k.clone(), kc0.clone(), vc0.clone()
    _lib.check(Lb.tppx_rotary_kv_append_llama(qa.data_ptr(), ka.data_ptr(), v.data_ptr(), EP.data_ptr(), pos.data_ptr(),
                                              kca.data_ptr(), vca.data_ptr(), ln.data_ptr(), B, 1, Nq, Nkv, 128, MP, 128,
                                              B_pos, Smax, st))
    outa = torch.empty((B, Nq, 128), dtype=torch.bfloat16, device="cuda")
    _lib.check(Lb.tppx_attn_decode(qa.data_ptr(), kca.data_ptr(), vca.data_ptr(), None, 0, ln.data_ptr(), 1,
                                   outa.data_ptr(), B, Nq, Nkv, 128, Smax, w.data_ptr(), w.numel(), st))
    # one launch
    qb, kb, vb, kcb, vcb = q.clone(), k.clone(), v.clone(), kc0.clone(), vc0.clone()
    outb = torch.empty_like(outa)
    _lib.check(Lb.tppx_attn_decode_rotary(qb.data_ptr(), kb.data_ptr(), vb.data_ptr(), EP.data_ptr(), pos.data_ptr(), B_pos,
                                          MP, 128, kcb.data_ptr(), vcb.data_ptr(), None, 0, ln.data_ptr(), outb.data_ptr(),
                                          B, Nq, Nkv, 128, Smax, w.data_ptr(), w.numel(), st))
    torch.cuda.synchronize()
    assert torch.equal(qb, q) and torch.equal(kb, k) and torch.equal(vb, v)
    assert_close_bf16(t2bits(kcb[:, :, L0]), t2bits(kca[:, :, L0]), what="appended key")
    assert torch.equal(vcb[:, :, L0], vca[:, :, L0])
    keep = torch.ones(Smax, dtype=torch.bool)
    keep[L0] = False
    assert torch.equal(kcb[:, :, keep], kc0[:, :, keep]) and torch.equal(vcb[:, :, keep], vc0[:, :, keep])
    a, b = outa.double(), outb.double()
    assert float((a - b).norm() / a.norm()) <= 5e-3
    assert float((a - b).abs().max()) <= 2.0 ** -7 * float(a.abs().max())
    # a full cache: nothing is written, the cached keys are attended to
    full = torch.tensor([Smax], dtype=torch.int32, device="cuda")
    _lib.check(Lb.tppx_attn_decode_rotary(qb.data_ptr(), kb.data_ptr(), vb.data_ptr(), EP.data_ptr(), pos.data_ptr(), B_pos,
                                          MP, 128, kcb.data_ptr(), vcb.data_ptr(), None, 0, full.data_ptr(), outb.data_ptr(),
                                          B, Nq, Nkv, 128, Smax, w.data_ptr(), w.numel(), st))
    torch.cuda.synchronize()
    assert torch.equal(kcb[:, :, keep], kc0[:, :, keep]) and torch.isfinite(outb.float()).all()


@pytest.mark.parametrize("kernel", ["rows", "wide"])
def test_attn_decode_mask(kernel, monkeypatch):
    """Additive mask over key positions; cache rows past the valid length hold NaN and must not reach the output
    (the kernels read whole trips, clamped to the cache, and drop what lies past the length)."""
    monkeypatch.setenv("TPPX_ATTN_WIDE", "1" if kernel == "wide" else "0")
    F = _llm()
    B, Nq, L, Smax = 2, 4, 100, 128
    q = randn_bf16((B, Nq, 128), 1.0, 41)
    k = randn_bf16((B, Nq, Smax, 128), 1.0, 42)
    v = randn_bf16((B, Nq, Smax, 128), 1.0, 43)
    k[:, :, L:] = float("nan")
    v[:, :, L:] = float("nan")
    keep = torch.ones(B, L, dtype=torch.int64)
    keep[0, :17] = 0  # left padding of sequence 0
    mask = F.TppCache(Smax).align_and_invert_mask(keep.to(torch.bfloat16))
    assert mask.shape == (B, 128) and float(mask[0, 0]) == -9984.0 and float(mask[0, 17]) == 0.0  # bf16(-10000)
    got = _attn(F, q.cuda(), k.cuda(), v.cuda(), L, mask=mask.cuda())
    ref = O.attn_decode(t2bits(q), t2bits(k[:, :, :L]), t2bits(v[:, :, :L]), mask.float().numpy())
    g, r = bits2f(t2bits(got)).astype(np.float64), bits2f(ref).astype(np.float64)
    assert np.isfinite(g).all()
    assert np.sqrt(((g - r) ** 2).sum() / (r ** 2).sum()) <= 5e-3


def _attn_prefill(q, kc, vc, past, mask=None):
    from tpp_pytorch_extension import _lib
    Lb = _lib.lib()
    B, S, Nq, H = q.shape
    Nkv, Smax = kc.shape[1], kc.shape[2]
    out = torch.empty_like(q)
    _lib.check(Lb.tppx_attn_prefill(q.data_ptr(), kc.data_ptr(), vc.data_ptr(),
                                    None if mask is None else mask.data_ptr(), 0 if mask is None else mask.shape[1],
                                    past, out.data_ptr(), B, S, Nq, Nkv, H, Smax, _lib.stream_of(q)))
    return out


@pytest.mark.parametrize("B,S,Nq,Nkv,past,Smax", [(1, 256, 4, 4, 0, 256), (2, 77, 8, 2, 0, 128), (2, 5, 4, 4, 100, 128),
                                                  (1, 130, 2, 1, 63, 256), (3, 1, 4, 2, 40, 64)])
@pytest.mark.parametrize("queries_per_wave", [16, 32])
def test_attn_prefill(B, S, Nq, Nkv, past, Smax, queries_per_wave, monkeypatch):
    """Causal attention for S query tokens against the oracle (tolerance as for the single-query kernel: rel-L2
    5e-3, max-abs 2^-7 of the largest output) and against plain PyTorch fp32 causal softmax attention (1e-2), with
    both of the kernel's shapes (the library picks by launch size; the knob forces one)."""
    _llm()
    monkeypatch.setenv("TPPX_ATTN_QG", str(queries_per_wave // 16))
    L = past + S
    q = randn_bf16((B, S, Nq, 128), 1.0, 51)
    k = randn_bf16((B, Nkv, Smax, 128), 1.0, 52)
    v = randn_bf16((B, Nkv, Smax, 128), 1.0, 53)
    got = _attn_prefill(q.cuda(), k.cuda(), v.cuda(), past)
    ref = O.attn_prefill(t2bits(q), t2bits(k[:, :, :L]), t2bits(v[:, :, :L]))
    g, r = bits2f(t2bits(got)).astype(np.float64), bits2f(ref).astype(np.float64)
    assert np.sqrt(((g - r) ** 2).sum() / (r ** 2).sum()) <= 5e-3
    assert np.abs(g - r).max() <= 2.0 ** -7 * np.abs(r).max()
    kk = k[:, :, :L].float().repeat_interleave(Nq // Nkv, dim=1)
    vv = v[:, :, :L].float().repeat_interleave(Nq // Nkv, dim=1)
    s = torch.einsum("bsnh,bnlh->bnsl", q.float(), kk) / np.sqrt(128.0)
    causal = torch.arange(L)[None, :] > (past + torch.arange(S))[:, None]
    s = s.masked_fill(causal[None, None], float("-inf"))
    t = torch.einsum("bnsl,bnlh->bsnh", torch.softmax(s, -1), vv).numpy().astype(np.float64)
    assert np.sqrt(((g - t) ** 2).sum() / (t ** 2).sum()) <= 1e-2
    if S == 1:  # one query: the single-query kernel's problem
        F = _llm()
        dec = _attn(F, q[:, 0].contiguous().cuda(), k.cuda(), v.cuda(), L)
        d = bits2f(t2bits(dec)).astype(np.float64).reshape(g.shape)
        assert np.sqrt(((g - d) ** 2).sum() / (d ** 2).sum()) <= 5e-3


def test_attn_prefill_full_size_rows_equal_single_query_problem():
    """The 7B prompt shape (2048 tokens, 32 heads): every sampled query row must solve the single-query problem on
    the keys it sees -- checked against the oracle's single-query function, which the multi-query restatement is
    pinned to row by row (the full multi-query oracle would take minutes at this size)."""
    _llm()
    B, S, Nq = 1, 2048, 32
    q = randn_bf16((B, S, Nq, 128), 1.0, 71)
    k = randn_bf16((B, Nq, S, 128), 1.0, 72)
    v = randn_bf16((B, Nq, S, 128), 1.0, 73)
    got = _attn_prefill(q.cuda(), k.cuda(), v.cuda(), 0).cpu()
    for i in (0, 1, 63, 64, 65, 1023, 1024, 2046, 2047):
        ref = O.attn_decode(t2bits(q[:, i]), t2bits(k[:, :, :i + 1]), t2bits(v[:, :, :i + 1]))
        g, r = bits2f(t2bits(got[:, i])).astype(np.float64), bits2f(ref).astype(np.float64)
        assert np.sqrt(((g - r) ** 2).sum() / (r ** 2).sum()) <= 5e-3, i
        assert np.abs(g - r).max() <= 2.0 ** -7 * np.abs(r).max(), i


@pytest.mark.parametrize("S,Nq,queries_per_wave", [(600, 32, 16), (1100, 32, 32), (700, 48, 16)])
def test_attn_prefill_more_than_256_workgroups(S, Nq, queries_per_wave, monkeypatch):
    """Launches of more than 256 workgroups whose query blocks per head do not divide 256 (the heads of every other
    run of 256 workgroups walk their blocks in the other order; a run boundary inside a head must not change that
    head's order): EVERY row against plain PyTorch fp32 causal attention."""
    _llm()
    monkeypatch.setenv("TPPX_ATTN_QG", str(queries_per_wave // 16))
    q = randn_bf16((1, S, Nq, 128), 1.0, 61)
    k = randn_bf16((1, Nq, S, 128), 1.0, 62)
    v = randn_bf16((1, Nq, S, 128), 1.0, 63)
    got = _attn_prefill(q.cuda(), k.cuda(), v.cuda(), 0).float()
    s = torch.einsum("bsnh,bnlh->bnsl", q.cuda().float(), k.cuda().float()) / np.sqrt(128.0)
    causal = torch.arange(S, device="cuda")[None, :] > torch.arange(S, device="cuda")[:, None]
    s = s.masked_fill(causal[None, None], float("-inf"))
    ref = torch.einsum("bnsl,bnlh->bsnh", torch.softmax(s, -1), v.cuda().float())
    err = (got - ref).flatten(2).norm(dim=-1) / ref.flatten(2).norm(dim=-1)  # per (batch, row)
    assert float(err.max()) <= 2e-2, (int(err.argmax()), float(err.max()))


@pytest.mark.parametrize("queries_per_wave", [16, 32])
def test_attn_prefill_mask_and_errors(queries_per_wave, monkeypatch):
    F = _llm()
    monkeypatch.setenv("TPPX_ATTN_QG", str(queries_per_wave // 16))
    from tpp_pytorch_extension._lib import TppxError
    B, S, Nq, Smax = 2, 70, 4, 128
    q = randn_bf16((B, S, Nq, 128), 1.0, 61)
    k = randn_bf16((B, Nq, Smax, 128), 1.0, 62)
    v = randn_bf16((B, Nq, Smax, 128), 1.0, 63)
    keep = torch.ones(B, S, dtype=torch.int64)
    keep[0, :9] = 0  # left padding of sequence 0
    mask = F.TppCache(Smax).align_and_invert_mask(keep.to(torch.bfloat16))
    got = _attn_prefill(q.cuda(), k.cuda(), v.cuda(), 0, mask=mask.cuda())
    ref = O.attn_prefill(t2bits(q), t2bits(k[:, :, :S]), t2bits(v[:, :, :S]), mask.float().numpy())
    g, r = bits2f(t2bits(got)).astype(np.float64), bits2f(ref).astype(np.float64)
    # rows of sequence 0 that see only padded keys are the plain average the reference also produces; compare all
    assert np.sqrt(((g - r) ** 2).sum() / (r ** 2).sum()) <= 5e-3
    with pytest.raises(TppxError):
        _attn_prefill(q.cuda(), k.cuda(), v.cuda(), Smax - S + 1)  # does not fit the cache


def test_decoder_layer_step_and_cache():
    """One LlamaDecoderLayer.forward on a small shape against the composition of the oracle functions, plus the
    cache bookkeeping (append position, rotated keys in the cache, reference method names)."""
    F = _llm()
    from tpp_pytorch_extension import _ops
    hidden, inter, Nq, Nkv, H, MP = 512, 1024, 4, 2, 128, 256
    B, ctx, cap = 2, 37, 64
    rng = torch.Generator().manual_seed(5)

    def lin(N, K, seed):
        W = randn_bf16((N, K), 0.05, seed)
        return W, _ops.remap_and_quantize_mxfp4(block_bf16(W).cuda()), O.remap_quantize_mxfp4(W.float().numpy())

    Ws = [lin(Nq * H, hidden, 51), lin(Nkv * H, hidden, 52), lin(Nkv * H, hidden, 53), lin(hidden, Nq * H, 54),
          lin(inter, hidden, 55), lin(inter, hidden, 56), lin(hidden, inter, 57)]
    g1 = torch.rand(hidden, generator=rng) + 0.5
    g2 = torch.rand(hidden, generator=rng) + 0.5
    EP = F.llama_rotary_table(MP, H, device="cpu")
    layer = F.LlamaDecoderLayer([g1.cuda(), Ws[0][1], Ws[1][1], Ws[2][1], Ws[3][1], g2.cuda(), Ws[4][1], Ws[5][1],
                                 Ws[6][1], EP.cuda()], 0, 1e-5, H, MP, H)
    cache = F.TppCache(cap)
    k0, v0 = randn_bf16((B, Nkv, ctx, H), 1.0, 61), randn_bf16((B, Nkv, ctx, H), 1.0, 62)
    cache.fill_(0, k0.cuda(), v0.cuda())
    assert cache.get_seq_length() == ctx and cache.get_capacity() == cap and cache.size() == 1
    x = randn_bf16((B, 1, hidden), 1.0, 63)
    pos = torch.full((B, 1), ctx, dtype=torch.int64)
    out = layer.forward([x.cuda(), None, pos.cuda()], cache, True)[0]
    cache.advance(1)
    assert cache.get_seq_length() == ctx + 1

    # oracle composition (fused_llm_infer.cpp:1229-1275)
    def mm(a_bits, w, post=O.POST_NONE, post_in=None):
        return O.linear_mxfp4(a_bits, w[2][0], w[2][1], None, post, post_in, None, 1.0, O.MODE_IDEAL)

    xb = t2bits(x).reshape(B, hidden)
    h = O.rms_norm(xb, g1.numpy(), 1e-5)
    q, k, v = mm(h, Ws[0]), mm(h, Ws[1]), mm(h, Ws[2])
    q = O.rotary_llama(q.reshape(B, 1, -1), EP.numpy(), pos.numpy(), Nq, H).reshape(B, Nq, H)
    k = O.rotary_llama(k.reshape(B, 1, -1), EP.numpy(), pos.numpy(), Nkv, H).reshape(B, Nkv, 1, H)
    kall = np.concatenate([t2bits(k0), k], axis=2)
    vall = np.concatenate([t2bits(v0), v.reshape(B, Nkv, 1, H)], axis=2)
    ctxv = O.attn_decode(q, kall, vall).reshape(B, Nq * H)
    so = mm(ctxv, Ws[3], O.POST_ADD_SCALE, xb)
    h2 = O.rms_norm(so, g2.numpy(), 1e-5)
    gate = mm(h2, Ws[4], O.POST_SILU)
    inter_v = mm(h2, Ws[5], O.POST_MUL, gate)
    ref = mm(inter_v, Ws[6], O.POST_ADD_SCALE, so)
    g, r = bits2f(t2bits(out)).reshape(B, hidden).astype(np.float64), bits2f(ref).astype(np.float64)
    rel = np.sqrt(((g - r) ** 2).sum() / (r ** 2).sum())
    assert rel <= 2e-2, rel
    # the cache got the rotated key and the value at position ctx, earlier positions untouched
    kc, vc = cache.get(0)
    assert kc.shape[2] == ctx + 1
    assert_close_bf16(t2bits(kc[:, :, ctx]), k.reshape(B, Nkv, H), what="cached key")
    assert_close_bf16(t2bits(vc[:, :, ctx]), v.reshape(B, Nkv, H), what="cached value")
    assert torch.equal(kc[:, :, :ctx].cpu(), k0)
    with pytest.raises(Exception):
        layer.forward([x.repeat(1, 2, 1).cuda(), None, pos.cuda()], cache, True)  # two tokens, one position each


@pytest.mark.parametrize("past,S", [(0, 70), (37, 9)])
def test_decoder_layer_prompt(past, S):
    """LlamaDecoderLayer.forward on S tokens per sequence (prompt processing, with and without cached keys)
    against the composition of the oracle functions; the S rotated keys and the values land in the cache."""
    F = _llm()
    from tpp_pytorch_extension import _ops
    hidden, inter, Nq, Nkv, H, MP = 512, 1024, 4, 2, 128, 256
    B, cap = 2, 128
    rng = torch.Generator().manual_seed(15)

    def lin(N, K, seed):
        W = randn_bf16((N, K), 0.05, seed)
        return W, _ops.remap_and_quantize_mxfp4(block_bf16(W).cuda()), O.remap_quantize_mxfp4(W.float().numpy())

    Ws = [lin(Nq * H, hidden, 151), lin(Nkv * H, hidden, 152), lin(Nkv * H, hidden, 153), lin(hidden, Nq * H, 154),
          lin(inter, hidden, 155), lin(inter, hidden, 156), lin(hidden, inter, 157)]
    g1 = torch.rand(hidden, generator=rng) + 0.5
    g2 = torch.rand(hidden, generator=rng) + 0.5
    EP = F.llama_rotary_table(MP, H, device="cpu")
    layer = F.LlamaDecoderLayer([g1.cuda(), Ws[0][1], Ws[1][1], Ws[2][1], Ws[3][1], g2.cuda(), Ws[4][1], Ws[5][1],
                                 Ws[6][1], EP.cuda()], 0, 1e-5, H, MP, H)
    cache = F.TppCache(cap)
    k0, v0 = randn_bf16((B, Nkv, past, H), 1.0, 161), randn_bf16((B, Nkv, past, H), 1.0, 162)
    if past:
        cache.fill_(0, k0.cuda(), v0.cuda())
    x = randn_bf16((B, S, hidden), 1.0, 163)
    pos = torch.arange(past, past + S, dtype=torch.int64).unsqueeze(0)
    out = layer.forward([x.cuda(), None, pos.cuda()], cache, True)[0]
    cache.advance(S)
    assert out.shape == (B, S, hidden) and cache.get_seq_length() == past + S

    def mm(a_bits, w, post=O.POST_NONE, post_in=None):
        return O.linear_mxfp4(a_bits, w[2][0], w[2][1], None, post, post_in, None, 1.0, O.MODE_IDEAL)

    xb = t2bits(x).reshape(B * S, hidden)
    h = O.rms_norm(xb, g1.numpy(), 1e-5)
    q, k, v = mm(h, Ws[0]), mm(h, Ws[1]), mm(h, Ws[2])
    q = O.rotary_llama(q.reshape(B, S, -1), EP.numpy(), pos.numpy(), Nq, H).reshape(B, S, Nq, H)
    k = O.rotary_llama(k.reshape(B, S, -1), EP.numpy(), pos.numpy(), Nkv, H).reshape(B, S, Nkv, H).transpose(0, 2, 1, 3)
    v = v.reshape(B, S, Nkv, H).transpose(0, 2, 1, 3)
    kall = np.concatenate([t2bits(k0), k], axis=2)
    vall = np.concatenate([t2bits(v0), v], axis=2)
    ctxv = O.attn_prefill(q, kall, vall).reshape(B * S, Nq * H)
    so = mm(ctxv, Ws[3], O.POST_ADD_SCALE, xb)
    h2 = O.rms_norm(so, g2.numpy(), 1e-5)
    gate = mm(h2, Ws[4], O.POST_SILU)
    ref = mm(mm(h2, Ws[5], O.POST_MUL, gate), Ws[6], O.POST_ADD_SCALE, so)
    g, r = bits2f(t2bits(out)).reshape(B * S, hidden).astype(np.float64), bits2f(ref).astype(np.float64)
    rel = np.sqrt(((g - r) ** 2).sum() / (r ** 2).sum())
    assert rel <= 2e-2, rel
    kc, vc = cache.get(0)
    assert_close_bf16(t2bits(kc[:, :, past:]), np.ascontiguousarray(k), what="cached keys")
    assert_close_bf16(t2bits(vc[:, :, past:]), np.ascontiguousarray(v), what="cached values")
    if past:
        assert torch.equal(kc[:, :, :past].cpu(), k0)


def test_generate_prompt_then_decode():
    """Prompt in one pass + decode steps: the first generated token equals the one obtained by feeding the prompt
    token by token through the decode step (same keys in the cache up to rounding, same argmax on this seed), and
    the graph and eager decode loops agree after a prompt."""
    F = _llm()
    model = F.LlamaDecoder(hidden=512, inter=1024, n_layers=2, n_heads=4, n_kv_heads=2, vocab=1024,
                           max_positions=256, seed=4)
    prompt = torch.randint(0, 1024, (3, 21), generator=torch.Generator().manual_seed(9)).cuda()
    a = model.generate(prompt, 6, use_graph=True)
    b = model.generate(prompt, 6, use_graph=False)
    assert a.shape == (3, 6) and torch.equal(a, b)
    # token by token
    cache = F.TppCache(64)
    for t in range(prompt.shape[1]):
        pos = torch.full((3, 1), t, dtype=torch.int64, device="cuda")
        nxt = model.step(prompt[:, t].contiguous(), pos, cache)
        cache.advance(1)
    c2 = F.TppCache(64)
    model.prefill(prompt, c2)
    k1, k2 = cache.get(1)[0].float(), c2.get(1)[0].float()
    assert ((k1 - k2).norm() / k1.norm()).item() <= 2e-2
    assert torch.equal(nxt, a[:, 0])


def test_greedy_decode_graph_equals_eager():
    """The replayed decode-step graph produces the tokens of the eager loop (same kernels, same order)."""
    F = _llm()
    model = F.LlamaDecoder(hidden=512, inter=1024, n_layers=2, n_heads=4, n_kv_heads=4, vocab=1024,
                           max_positions=256, seed=3)
    tok = torch.tensor([5, 77, 300], dtype=torch.int64, device="cuda")
    a = model.greedy_decode(tok, model.new_cache(3, 40, 64), 8, use_graph=False)
    b = model.greedy_decode(tok, model.new_cache(3, 40, 64), 8, use_graph=True)
    assert a.shape == (3, 8) and torch.equal(a, b)
    # a replayed step checks nothing on the host: runs that would overrun the cache or the rotary table are refused
    from tpp_pytorch_extension._lib import TppxError
    with pytest.raises(TppxError):
        model.greedy_decode(tok, model.new_cache(3, 40, 44), 8)
    with pytest.raises(TppxError):
        model.greedy_decode(tok, model.new_cache(3, 250, 300), 8)


@pytest.mark.parametrize("B,V,hidden", [(1, 32000, 4096), (3, 1024, 512), (16, 32000, 4096), (2, 8, 8)])
def test_greedy_next_token_step(B, V, hidden):
    """tppx_greedy_next against torch: argmax (first maximal index, ties and a NaN row included), the embedding row of
    the chosen token, position and cache-length counters moved on by one."""
    _llm()
    from tpp_pytorch_extension import _lib
    g = torch.Generator().manual_seed(40 + B)
    logits = torch.randn((B, V), generator=g).to(torch.bfloat16)
    logits[0, V // 2] = logits[0].max()          # a tie: the earlier index wins
    logits[0, 3] = logits[0].max()
    if B > 1:
        logits[1, V - 1] = float("nan")          # torch.argmax takes a NaN for the maximum
    embed = torch.randn((V, hidden), generator=g).to(torch.bfloat16).cuda()
    lg = logits.cuda()
    tokens = torch.full((B,), -1, dtype=torch.int64, device="cuda")
    pos = torch.arange(B, dtype=torch.int64, device="cuda").view(B, 1) + 7
    seq = torch.tensor([41], dtype=torch.int32, device="cuda")
    h = torch.zeros((B, 1, hidden), dtype=torch.bfloat16, device="cuda")
    L = _lib.lib()
    _lib.check(L.tppx_greedy_next(lg.data_ptr(), B, V, embed.data_ptr(), hidden, tokens.data_ptr(), pos.data_ptr(),
                                  seq.data_ptr(), h.data_ptr(), _lib.stream_of(lg)))
    want = lg.argmax(dim=-1)
    assert torch.equal(tokens, want), (tokens, want)
    assert torch.equal(h.view(B, hidden), embed.index_select(0, want))
    assert torch.equal(pos.view(-1).cpu(), torch.arange(B) + 8) and seq.item() == 42
    # only the tokens when the other outputs are not asked for
    t2 = torch.empty_like(tokens)
    _lib.check(L.tppx_greedy_next(lg.data_ptr(), B, V, None, 0, t2.data_ptr(), None, None, None, _lib.stream_of(lg)))
    assert torch.equal(t2, want) and seq.item() == 42
    assert L.tppx_greedy_next(lg.data_ptr(), B, V + 1, None, 0, t2.data_ptr(), None, None, None, None) == _lib.ESHAPE


@pytest.mark.parametrize("M", [1, 5, 16])
@pytest.mark.parametrize("K", [512, 4096])
def test_rms_norm_fused_into_gemms(M, K, monkeypatch):
    """llama_rms_norm inside the q/k/v launch and inside the gate/up launch gives the bits of the separate
    normalisation kernel followed by the plain GEMM launches, except where the row scale differs in its last bit
    (sum order) and flips a bf16 rounding of a normalised activation: compared with the GEMM tolerance."""
    F = _llm()
    from tpp_pytorch_extension import _ops
    monkeypatch.setattr(_ops, "FUSE_NORM", True)
    Ns = (1536, 512, 512) if K == 4096 else (12288, 256, 256)   # 768+ channel tiles exercise 3 tiles per workgroup
    ws = []
    for i, n in enumerate(Ns):
        W = randn_bf16((n, K), 0.03, 400 + i)
        ws.append(_ops.remap_and_quantize_mxfp4(block_bf16(W).cuda()))
    x = randn_bf16((M, K), 1.3, 410).cuda()
    gamma = (torch.rand(K, generator=torch.Generator().manual_seed(411)) + 0.5).cuda()
    fused = _ops.qkv_gemm(x, ws, [None] * 3, norm=(gamma, 1e-5))
    h = F.rms_norm(x, gamma, 1e-5)
    sep = _ops.qkv_gemm(h, ws, [None] * 3)
    for a, b in zip(fused, sep):
        assert_close_bf16(t2bits(a), t2bits(b), what=f"fused norm qkv M={M} K={K}")
        assert (a != b).float().mean() < 0.01
    wg, wu = ws[1], ws[2]
    fz = _ops.swiglu_gate_up(x, wg, wu, norm=(gamma, 1e-5))
    sp = _ops.swiglu_gate_up(h, wg, wu)
    assert_close_bf16(t2bits(fz), t2bits(sp), ulps=2, what=f"fused norm swiglu M={M} K={K}")
    # without a norm the same entry point is a plain GEMM
    from tpp_pytorch_extension import _lib
    L = _lib.lib()
    qn, sn = ws[0].native()
    y = torch.empty((M, Ns[0]), dtype=torch.bfloat16, device="cuda")
    seg = (_lib.Seg * 1)()
    seg[0].qw, seg[0].sw, seg[0].y, seg[0].N, seg[0].post_op, seg[0].post_scale = qn.data_ptr(), sn.data_ptr(), y.data_ptr(), Ns[0], 0, 1.0
    _lib.check(L.tppx_norm_multi_linear_mxfp4(h.data_ptr(), None, 0.0, seg, 1, M, K, 0, _lib.stream_of(h)))
    assert_close_bf16(t2bits(y), t2bits(sep[0]), what="LDS-staged plain GEMM")


@pytest.mark.parametrize("M", [1, 3, 16])
@pytest.mark.parametrize("Kprod,N", [(512, 4096), (11008, 4096), (1024, 2048)])
def test_rms_norm_from_row_sums(M, Kprod, N):
    """The residual-add GEMM leaves the row sums of squares of its output in a [16][256] table (every producing
    kernel: all rows in LDS, 4 rows for a long K, one row group); the table equals the sums computed from the output
    bits, and the q/k/v and gate/up launches that take their RMSNorm scale from it match the normalisation kernel
    followed by the plain launches within the GEMM tolerance (the row scale can differ in its last bit)."""
    F = _llm()
    from tpp_pytorch_extension import _ops
    Wp = _ops.remap_and_quantize_mxfp4(block_bf16(randn_bf16((N, Kprod), 0.03, 500)).cuda())
    xin = randn_bf16((M, Kprod), 1.0, 501).cuda()
    res = randn_bf16((M, N), 1.0, 502).cuda()
    tab = torch.full((16, 256), 7.0, dtype=torch.float32, device="cuda")  # stale contents must not survive
    h = _ops.fc_add(xin, Wp, None, res, 1.0, row_sumsq=tab)
    assert torch.equal(h, _ops.fc_add(xin, Wp, None, res, 1.0))
    want = (h.double() ** 2).sum(-1).cpu().numpy()
    got = tab[:M].double().sum(-1).cpu().numpy()
    assert np.allclose(got, want, rtol=1e-5), (got, want)
    gamma = (torch.rand(N, generator=torch.Generator().manual_seed(503)) + 0.5).cuda()
    ws = [_ops.remap_and_quantize_mxfp4(block_bf16(randn_bf16((n, N), 0.03, 510 + i)).cuda())
          for i, n in enumerate((1536, 512, 512))]
    hn = F.rms_norm(h, gamma, 1e-5)
    fused = _ops.qkv_gemm(h, ws, [None] * 3, norm=(gamma, 1e-5, tab))
    for a, b in zip(fused, _ops.qkv_gemm(hn, ws, [None] * 3)):
        assert_close_bf16(t2bits(a), t2bits(b), what=f"norm from row sums, qkv M={M}")
        assert (a != b).float().mean() < 0.01
    fz = _ops.swiglu_gate_up(h, ws[1], ws[2], norm=(gamma, 1e-5, tab))
    assert_close_bf16(t2bits(fz), t2bits(_ops.swiglu_gate_up(hn, ws[1], ws[2])), ulps=2, what=f"norm from row sums, swiglu M={M}")


@pytest.mark.parametrize("weight_dtype", ["mxfp4", "qint8", "bf16"])
def test_optimize_model_for_llama_against_transformers(weight_dtype):
    """OptimizeModelForLlama on a random-initialised transformers LlamaForCausalLM (2 layers, GQA 4/2 heads of
    128): the logits of the prompt pass and of two decode steps against the stock transformers model in fp32 on
    the CPU holding the *dequantized* weights (exactly representable), i.e. the same function up to the bf16
    roundings of the fused path (and, for QINT8, the int8 rounding of the activations: looser bound).  Left
    padding goes through the additive key mask."""
    transformers = pytest.importorskip("transformers")
    import copy
    F = _llm()
    cfg = transformers.LlamaConfig(hidden_size=512, intermediate_size=1024, num_hidden_layers=2, num_attention_heads=4,
                                   num_key_value_heads=2, vocab_size=1024, max_position_embeddings=256, head_dim=128,
                                   rms_norm_eps=1e-5, attn_implementation="eager")
    torch.manual_seed(11)
    ref_model = transformers.LlamaForCausalLM(cfg).eval()
    with torch.no_grad():
        for m in ref_model.modules():
            if isinstance(m, torch.nn.Linear):  # weights := dequantize(quantize(weights)), as the fused model sees them
                w = m.weight.data.to(torch.bfloat16).float()
                if weight_dtype == "mxfp4":
                    q, sc = O.remap_quantize_mxfp4(w.numpy())
                    m.weight.data.copy_(torch.from_numpy(O.dequantize_mxfp4_plain(q, sc)))
                elif weight_dtype == "qint8":
                    q, sc, _ = O.remap_quantize_qint8(w.numpy())
                    m.weight.data.copy_(torch.from_numpy(O.dequantize_qint8_plain(q, sc)))
                else:
                    m.weight.data.copy_(w)
            elif isinstance(m, torch.nn.Embedding):
                m.weight.data.copy_(m.weight.data.to(torch.bfloat16).float())
    opt_model = F.OptimizeModelForLlama(copy.deepcopy(ref_model), torch.bfloat16, "cuda",
                                        None if weight_dtype == "bf16" else weight_dtype).eval()
    assert not opt_model.lm_head.weight.is_quantized and opt_model.lm_head.weight.dim() == 5  # bf16, as the reference's
    tol = 3e-2 if weight_dtype == "mxfp4" else 6e-2

    ids = torch.randint(0, 1024, (2, 19), generator=torch.Generator().manual_seed(12))
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
        # padded positions of sequence 1 are arbitrary in both models; compare the real ones
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


def _tiny_optimized_llama(weight_dtype="mxfp4", seed=21):
    transformers = pytest.importorskip("transformers")
    F = _llm()
    cfg = transformers.LlamaConfig(hidden_size=512, intermediate_size=1024, num_hidden_layers=2, num_attention_heads=4,
                                   num_key_value_heads=2, vocab_size=1024, max_position_embeddings=256, head_dim=128,
                                   rms_norm_eps=1e-5, attn_implementation="eager")
    torch.manual_seed(seed)
    return F, F.OptimizeModelForLlama(transformers.LlamaForCausalLM(cfg).eval(), torch.bfloat16, "cuda", weight_dtype).eval()


def _assert_greedy(opt, out, am, n_prompt):
    """Every generated token is a maximiser of the logits a teacher-forced pass over the finished sequence gives at
    the position before it, up to the bf16 noise between the kernels of the two passes (3 % of the largest logit:
    a random token of the 1024 passes with probability < 1 %)."""
    n_new = out.shape[1] - n_prompt
    am = torch.cat([am, am.new_ones((am.shape[0], n_new))], dim=1)
    with torch.no_grad():
        logits = opt(input_ids=out[:, :-1], attention_mask=am[:, :-1]).logits.float()
    for t in range(n_prompt - 1, out.shape[1] - 1):
        lt = logits[:, t]
        gap = lt.max(-1).values - lt.gather(1, out[:, t + 1:t + 2])[:, 0]
        assert bool((gap <= 0.03 * lt.abs().max(-1).values).all()), (t, gap.tolist())


def test_transformers_generate_on_optimized_model():
    """run_generation.py:420 calls model.generate(): greedy generate() of the installed transformers on the optimized
    model gives the same tokens on the cache the patched forward creates and on a TppCache handed in, and those
    tokens, like the package's own greedy loop's, are the argmax of the model's logits (the two loops put
    different numbers of rows through the lm_head in the prompt pass, so near-ties of a random model may break
    differently between them); beam search runs on the same cache through reorder_cache."""
    F, opt = _tiny_optimized_llama()
    from tpp_pytorch_extension.llm.llm_common import TppCache
    ids = torch.randint(0, 1024, (2, 19), generator=torch.Generator().manual_seed(12)).cuda()
    am = torch.ones_like(ids)
    am[1, :4] = 0
    want = F.generate_greedy(opt, ids, 6, attention_mask=am)
    assert want.shape == (2, 25) and torch.equal(want[:, :19], ids)
    _assert_greedy(opt, want, am, 19)
    got = opt.generate(input_ids=ids, attention_mask=am, max_new_tokens=6, do_sample=False)
    assert got.shape == (2, 25) and torch.equal(got[:, :19], ids)
    _assert_greedy(opt, got, am, 19)
    got2 = opt.generate(input_ids=ids, attention_mask=am, max_new_tokens=6, do_sample=False,
                        past_key_values=TppCache(capacity=64))
    assert torch.equal(got2, got)
    beams = opt.generate(input_ids=ids, attention_mask=am, max_new_tokens=6, do_sample=False, num_beams=3)
    assert beams.shape == want.shape and torch.equal(beams[:, :19], ids)


def test_cache_reorder_moves_sequences():
    """TppCache.reorder_cache (attn.h:327-366): after reordering with [1, 0] a decode step on swapped tokens gives
    the swapped logits of the same step on the untouched cache, bit for bit (rows of a decode step do not mix)."""
    F, opt = _tiny_optimized_llama()
    ids = torch.randint(0, 1024, (2, 23), generator=torch.Generator().manual_seed(13)).cuda()
    nxt = torch.tensor([[5], [9]], device="cuda")
    with torch.no_grad():
        a = opt(input_ids=ids, use_cache=True)
        la = opt(input_ids=nxt, past_key_values=a.past_key_values, use_cache=True).logits
        b = opt(input_ids=ids, use_cache=True)
        b.past_key_values.reorder_cache(torch.tensor([1, 0], device="cuda"))
        lb = opt(input_ids=nxt.flip(0), past_key_values=b.past_key_values, use_cache=True).logits
    assert torch.equal(lb, la.flip(0))
    from tpp_pytorch_extension._lib import TppxError
    with pytest.raises(TppxError):
        b.past_key_values.reorder_cache(torch.tensor([0, 1, 0], device="cuda"))


def test_lm_head_quantized_on_request():
    """The lm_head stays bf16 by default; quantize_lm_head=True and run_generation.py:277-282's own way
    (remap_and_quantize_qint8 on the blocked bf16 weight after the call) both give a QINT8 head whose logits stay
    within the int8 rounding of the bf16 head's."""
    transformers = pytest.importorskip("transformers")
    import copy
    F = _llm()
    from tpp_pytorch_extension import _ops
    cfg = transformers.LlamaConfig(hidden_size=512, intermediate_size=1024, num_hidden_layers=1, num_attention_heads=4,
                                   num_key_value_heads=2, vocab_size=1600, max_position_embeddings=128, head_dim=128,
                                   rms_norm_eps=1e-5, attn_implementation="eager")
    torch.manual_seed(31)
    base = transformers.LlamaForCausalLM(cfg).eval()
    a = F.OptimizeModelForLlama(copy.deepcopy(base), torch.bfloat16, "cuda", "mxfp4").eval()
    assert tuple(a.lm_head.weight.shape) == (16, 8, 32, 100, 2)  # FixLinear(m, 100, 64, bf16)
    b = F.OptimizeModelForLlama(copy.deepcopy(base), torch.bfloat16, "cuda", "mxfp4", quantize_lm_head=True).eval()
    assert b.lm_head.weight.is_quantized and b.lm_head.weight.dtype == torch.qint8
    c = F.OptimizeModelForLlama(copy.deepcopy(base), torch.bfloat16, "cuda", "mxfp4").eval()
    with torch.no_grad():
        c.lm_head.weight = torch.nn.Parameter(_ops.remap_and_quantize_qint8(c.lm_head.weight), requires_grad=False)
    ids = torch.randint(0, 1600, (2, 9), generator=torch.Generator().manual_seed(32)).cuda()
    with torch.no_grad():
        la, lb, lc = (m(input_ids=ids).logits.float() for m in (a, b, c))
    assert torch.equal(lb, lc)
    assert float((lb - la).norm() / la.norm()) <= 2e-2


def test_cache_update_appends_and_grows():
    """TppCache.update (attn.h:198-222,258-274): append [B][Nkv][S][H] states layer by layer, per-layer lengths,
    growth past the capacity, and attention over the updated cache equals attention over the concatenated keys."""
    F = _llm()
    from tpp_pytorch_extension.llm.llm_common import TppCache as HFCache
    B, Nkv, H = 2, 2, 128
    cache = HFCache(capacity=0)
    k1, v1 = randn_bf16((B, Nkv, 40, H), 1.0, 901).cuda(), randn_bf16((B, Nkv, 40, H), 1.0, 902).cuda()
    k2, v2 = randn_bf16((B, Nkv, 3, H), 1.0, 903).cuda(), randn_bf16((B, Nkv, 3, H), 1.0, 904).cuda()
    for layer in (0, 1):
        ks, vs = cache.update(k1, v1, layer)
        assert ks.shape == (B, Nkv, 40, H) and torch.equal(ks, k1) and torch.equal(vs, v1)
    assert cache.get_seq_length() == 40 and len(cache) == 2
    cap0 = cache.get_max_length()
    assert cap0 >= 40 + 128 and cap0 % 32 == 0          # grew by KV_CACHE_INC_SIZE beyond the need, whole blocks
    ks, vs = cache.update(k2, v2, 0)
    assert cache.get_seq_length(0) == 43 and cache.get_seq_length(1) == 40
    ks1, _ = cache.update(k2, v2, 1)
    assert torch.equal(ks, torch.cat([k1, k2], 2)) and torch.equal(ks1, ks)
    big = randn_bf16((B, Nkv, cap0, H), 1.0, 905).cuda()
    ks, _ = cache.update(big, big, 0)                    # past the capacity: storage is reallocated, contents kept
    assert cache.get_max_length() >= 43 + cap0 and torch.equal(ks[:, :, :43], torch.cat([k1, k2], 2))
    core = cache.get_cpp()
    q = randn_bf16((B, 4, H), 1.0, 906)
    kc, vc = core.layers[1]
    got = _attn(F, q.cuda(), kc, vc, 43)
    ref = O.attn_decode(t2bits(q), t2bits(torch.cat([k1, k2], 2)), t2bits(torch.cat([v1, v2], 2)))
    g, r = bits2f(t2bits(got)).astype(np.float64), bits2f(ref).astype(np.float64)
    assert np.sqrt(((g - r) ** 2).sum() / (r ** 2).sum()) <= 5e-3


@pytest.mark.parametrize("Sq,past", [(1, 37), (9, 21), (40, 0)])
def test_attn_entry_point_of_the_cache_module(Sq, past):
    """_C._tpp_attn.attn (attn_wrapper, attn.cpp:957-1043): keys / values appended to a layer of the cache, then
    attention of q [B][Nkv][Sq][R][H] over everything cached, against the oracle's functions on the same tensors."""
    _llm()
    from tpp_pytorch_extension._C import _tpp_attn
    from tpp_pytorch_extension._lib import TppxError
    B, Nkv, R, H = 2, 2, 2, 128
    cache = _tpp_attn.TppCache(64)
    k0, v0 = randn_bf16((B, Nkv, past, H), 1.0, 81), randn_bf16((B, Nkv, past, H), 1.0, 82)
    if past:
        cache.update(k0.cuda(), v0.cuda(), 3)
    q = randn_bf16((B, Nkv, Sq, R, H), 1.0, 83)
    k, v = randn_bf16((B, Nkv, Sq, H), 1.0, 84), randn_bf16((B, Nkv, Sq, H), 1.0, 85)
    got = _tpp_attn.attn(q.cuda(), k.cuda(), v.cuda(), torch.Tensor(), cache, 3, True).cpu()
    assert got.shape == q.shape and cache.get_seq_length(3) == past + Sq
    kall = np.concatenate([t2bits(k0), t2bits(k)], axis=2)
    vall = np.concatenate([t2bits(v0), t2bits(v)], axis=2)
    qo = q.permute(0, 2, 1, 3, 4).reshape(B, Sq, Nkv * R, H)  # the oracle's head order: key head * R + r
    if Sq == 1:
        ref = O.attn_decode(t2bits(qo[:, 0]), kall, vall).reshape(B, 1, Nkv, R, H)
    else:
        ref = O.attn_prefill(t2bits(qo), kall, vall).reshape(B, Sq, Nkv, R, H)
    ref = ref.transpose(0, 2, 1, 3, 4)
    g, r = bits2f(t2bits(got)).astype(np.float64), bits2f(np.ascontiguousarray(ref)).astype(np.float64)
    assert np.sqrt(((g - r) ** 2).sum() / (r ** 2).sum()) <= 5e-3
    assert np.abs(g - r).max() <= 2.0 ** -7 * np.abs(r).max()
    if Sq > 1:
        with pytest.raises(TppxError):
            _tpp_attn.attn(q.cuda(), k.cuda(), v.cuda(), torch.Tensor(), cache, 3, False)
