"""Attention for head sizes other than 128 (attn<T>, src/csrc/llm/attn.cpp:781-955, is generic in the head size):
the kernels behind tppx_attn_decode / tppx_attn_prefill for those sizes, against the oracle (tolerance as for the 128-wide
kernels: rel-L2 5e-3, max-abs 2^-7 of the largest output) and plain PyTorch fp32 softmax attention (1e-2), and a
decoder layer with 64-wide heads against the oracle composition."""
import numpy as np
import pytest
import torch

import oracle as O
from util import t2bits, randn_bf16, block_bf16, bits2f, assert_close_bf16
from test_gpu_decoder import _attn, _attn_prefill, _llm

pytestmark = pytest.mark.gpu


def _close(got, ref, torch_ref):
    g, r = bits2f(t2bits(got)).astype(np.float64), bits2f(ref).astype(np.float64)
    assert np.isfinite(g).all()
    assert np.sqrt(((g - r) ** 2).sum() / (r ** 2).sum()) <= 5e-3
    assert np.abs(g - r).max() <= 2.0 ** -7 * np.abs(r).max()
    assert np.sqrt(((g - torch_ref) ** 2).sum() / (torch_ref ** 2).sum()) <= 1e-2


@pytest.mark.parametrize("H", [64, 96, 256, 8, 200])
@pytest.mark.parametrize("B,Nq,Nkv,L,Smax", [(3, 8, 2, 77, 128), (2, 4, 4, 1, 64), (1, 8, 8, 300, 320), (2, 2, 1, 64, 64)])
def test_attn_decode_other_head_sizes(H, B, Nq, Nkv, L, Smax):
    F = _llm()
    q = randn_bf16((B, Nq, H), 1.0, 31 + H)
    k = randn_bf16((B, Nkv, Smax, H), 1.0, 32 + H)
    v = randn_bf16((B, Nkv, Smax, H), 1.0, 33 + H)
    k[:, :, L:] = float("nan")  # rows past the valid length must not reach the output
    v[:, :, L:] = float("nan")
    got = _attn(F, q.cuda(), k.cuda(), v.cuda(), L)
    ref = O.attn_decode(t2bits(q), t2bits(k[:, :, :L]), t2bits(v[:, :, :L]))
    kk = k[:, :, :L].float().repeat_interleave(Nq // Nkv, dim=1)
    vv = v[:, :, :L].float().repeat_interleave(Nq // Nkv, dim=1)
    s = torch.einsum("bnh,bnlh->bnl", q.float(), kk) / np.sqrt(float(H))
    t = torch.einsum("bnl,bnlh->bnh", torch.softmax(s, -1), vv).numpy().astype(np.float64)
    _close(got, ref, t)


def test_attn_decode_other_head_size_with_mask():
    F = _llm()
    B, Nq, L, Smax, H = 2, 4, 100, 128, 64
    q = randn_bf16((B, Nq, H), 1.0, 41)
    k = randn_bf16((B, Nq, Smax, H), 1.0, 42)
    v = randn_bf16((B, Nq, Smax, H), 1.0, 43)
    keep = torch.ones(B, L, dtype=torch.int64)
    keep[0, :17] = 0  # left padding of sequence 0
    mask = F.TppCache(Smax).align_and_invert_mask(keep.to(torch.bfloat16))
    got = _attn(F, q.cuda(), k.cuda(), v.cuda(), L, mask=mask.cuda())
    ref = O.attn_decode(t2bits(q), t2bits(k[:, :, :L]), t2bits(v[:, :, :L]), mask.float().numpy())
    g, r = bits2f(t2bits(got)).astype(np.float64), bits2f(ref).astype(np.float64)
    assert np.isfinite(g).all()
    assert np.sqrt(((g - r) ** 2).sum() / (r ** 2).sum()) <= 5e-3


@pytest.mark.parametrize("H", [64, 80, 256, 8, 200])
@pytest.mark.parametrize("B,Nq,Nkv,L,Smax", [(1, 4, 2, 700, 1024), (2, 8, 8, 100, 1024), (1, 2, 1, 1000, 1000)])
def test_attn_decode_other_head_sizes_split_key_range(H, B, Nq, Nkv, L, Smax, monkeypatch):
    """Caches of 512 keys and more: the key range is dealt to several workgroups per query (some of them past the
    valid length, leaving empty states) and merged by a second launch; one split gives the same answer up to the
    order of the sums."""
    F = _llm()
    q = randn_bf16((B, Nq, H), 1.0, 131 + H)
    k = randn_bf16((B, Nkv, Smax, H), 1.0, 132 + H)
    v = randn_bf16((B, Nkv, Smax, H), 1.0, 133 + H)
    k[:, :, L:] = float("nan")
    v[:, :, L:] = float("nan")
    got = _attn(F, q.cuda(), k.cuda(), v.cuda(), L)
    ref = O.attn_decode(t2bits(q), t2bits(k[:, :, :L]), t2bits(v[:, :, :L]))
    kk = k[:, :, :L].float().repeat_interleave(Nq // Nkv, dim=1)
    vv = v[:, :, :L].float().repeat_interleave(Nq // Nkv, dim=1)
    s = torch.einsum("bnh,bnlh->bnl", q.float(), kk) / np.sqrt(float(H))
    t = torch.einsum("bnl,bnlh->bnh", torch.softmax(s, -1), vv).numpy().astype(np.float64)
    _close(got, ref, t)
    monkeypatch.setenv("TPPX_ATTN_GENERIC_SPLITS", "1")
    one = _attn(F, q.cuda(), k.cuda(), v.cuda(), L)
    _close(one, ref, t)
    monkeypatch.setenv("TPPX_ATTN_GENERIC_SPLITS", "5")
    five = _attn(F, q.cuda(), k.cuda(), v.cuda(), L)
    _close(five, ref, t)
    none = _attn(F, q.cuda(), k.cuda(), v.cuda(), L, ws=False)  # no workspace: one split
    assert torch.equal(none, one)


@pytest.mark.parametrize("H", [64, 80, 96, 256, 8, 200])
@pytest.mark.parametrize("B,S,Nq,Nkv,past,Smax", [(1, 130, 4, 4, 0, 256), (2, 77, 8, 2, 0, 128), (2, 5, 4, 4, 100, 128), (3, 1, 4, 2, 40, 64)])
def test_attn_prefill_other_head_sizes(H, B, S, Nq, Nkv, past, Smax):
    _llm()
    L = past + S
    q = randn_bf16((B, S, Nq, H), 1.0, 51 + H)
    k = randn_bf16((B, Nkv, Smax, H), 1.0, 52 + H)
    v = randn_bf16((B, Nkv, Smax, H), 1.0, 53 + H)
    got = _attn_prefill(q.cuda(), k.cuda(), v.cuda(), past)
    ref = O.attn_prefill(t2bits(q), t2bits(k[:, :, :L]), t2bits(v[:, :, :L]))
    kk = k[:, :, :L].float().repeat_interleave(Nq // Nkv, dim=1)
    vv = v[:, :, :L].float().repeat_interleave(Nq // Nkv, dim=1)
    s = torch.einsum("bsnh,bnlh->bnsl", q.float(), kk) / np.sqrt(float(H))
    causal = torch.arange(L)[None, :] > (past + torch.arange(S))[:, None]
    s = s.masked_fill(causal[None, None], float("-inf"))
    t = torch.einsum("bnsl,bnlh->bsnh", torch.softmax(s, -1), vv).numpy().astype(np.float64)
    _close(got, ref, t)


def test_unsupported_head_sizes_are_rejected():
    from tpp_pytorch_extension import _lib
    _llm()
    L = _lib.lib()
    A = 1 << 20
    for H in (4, 12, 264, 512):
        assert L.tppx_attn_decode(A, A, A, None, 0, A, 0, A, 1, 4, 4, H, 64, None, 0, None) == _lib.EUNSUPPORTED
        assert L.tppx_attn_prefill(A, A, A, None, 0, 0, A, 1, 8, 4, 4, H, 64, None) == _lib.EUNSUPPORTED


@pytest.mark.parametrize("H", [64, 96])
@pytest.mark.parametrize("S,past", [(1, 21), (40, 0), (7, 30)])
def test_decoder_layer_with_64_wide_heads(S, past, H):
    """LlamaDecoderLayer (src/csrc/llm/fused_llm_infer.cpp:1229-1275) with head size 64, and 96 (no power of two: the
    rotate-half pairs of a head can straddle two waves of the rotary launch): rotary + cache append as their own
    launch, attention on the kernels for other head sizes, MXFP4 linears; against the composition of the oracle
    functions (rel-L2 <= 2e-2 for the layer output, cached keys / values within 1 bf16 ulp)."""
    import tpp_pytorch_extension  # noqa: F401
    from tpp_pytorch_extension import _ops
    F = _llm()
    HID, INTER, NQ, NKV, MP = 256, 512, 4, 2, 256
    shapes = [(NQ * H, HID), (NKV * H, HID), (NKV * H, HID), (HID, NQ * H), (INTER, HID), (INTER, HID), (HID, INTER)]
    Ws = [randn_bf16(s, 0.05, 910 + i) for i, s in enumerate(shapes)]
    rng = torch.Generator().manual_seed(91)
    g1, g2 = torch.rand(HID, generator=rng) + 0.5, torch.rand(HID, generator=rng) + 0.5
    EP = F.llama_rotary_table(MP, H, device="cpu")
    qws = [_ops.remap_and_quantize_mxfp4(block_bf16(W).cuda()) for W in Ws]
    layer = F.LlamaDecoderLayer([g1.cuda()] + qws[:4] + [g2.cuda()] + qws[4:] + [EP.cuda()], 0, 1e-5, H, MP, H)
    assert (layer.Nq, layer.Nkv, layer.H) == (NQ, NKV, H)
    B, cap = 2, 128
    cache = F.TppCache(cap)
    k0, v0 = randn_bf16((B, NKV, past, H), 1.0, 961), randn_bf16((B, NKV, past, H), 1.0, 962)
    if past:
        cache.fill_(0, k0.cuda(), v0.cuda())
    x = randn_bf16((B, S, HID), 1.0, 963 + S)
    pos = torch.arange(past, past + S, dtype=torch.int64).unsqueeze(0).repeat(B, 1)
    out = layer.forward([x.cuda(), None, pos.cuda()], cache, True)[0]
    cache.advance(S)
    qo = [O.remap_quantize_mxfp4(W.float().numpy()) for W in Ws]
    mm = [(lambda a, post=O.POST_NONE, pin=None, q=q, s=s: O.linear_mxfp4(a, q, s, None, post, pin, None, 1.0, O.MODE_IDEAL)) for q, s in qo]
    xb = t2bits(x).reshape(B * S, HID)
    h = O.rms_norm(xb, g1.numpy(), 1e-5)
    q, k, v = mm[0](h), mm[1](h), mm[2](h)
    q = O.rotary_llama(q.reshape(B, S, -1), EP.numpy(), pos.numpy(), NQ, H).reshape(B, S, NQ, H)
    k = O.rotary_llama(k.reshape(B, S, -1), EP.numpy(), pos.numpy(), NKV, H).reshape(B, S, NKV, H).transpose(0, 2, 1, 3)
    v = v.reshape(B, S, NKV, H).transpose(0, 2, 1, 3)
    kall = np.concatenate([t2bits(k0), k], axis=2)
    vall = np.concatenate([t2bits(v0), v], axis=2)
    if S == 1:
        ctx = O.attn_decode(q.reshape(B, NQ, H), kall, vall).reshape(B, NQ * H)
    else:
        ctx = O.attn_prefill(q, kall, vall).reshape(B * S, NQ * H)
    so = mm[3](ctx, O.POST_ADD_SCALE, xb)
    h2 = O.rms_norm(so, g2.numpy(), 1e-5)
    gate = mm[4](h2, O.POST_SILU)
    ref = mm[6](mm[5](h2, O.POST_MUL, gate), O.POST_ADD_SCALE, so)
    g, r = bits2f(t2bits(out)).reshape(B * S, HID).astype(np.float64), bits2f(ref).astype(np.float64)
    rel = np.sqrt(((g - r) ** 2).sum() / (r ** 2).sum())
    assert rel <= 2e-2, rel
    kc, vc = cache.get(0)
    assert_close_bf16(t2bits(kc[:, :, past:]), np.ascontiguousarray(k), what="cached keys")
    assert_close_bf16(t2bits(vc[:, :, past:]), np.ascontiguousarray(v), what="cached values")


@pytest.mark.parametrize("H", [64, 256])
def test_attn_prefill_other_head_sizes_full_prompt_and_plain_kernel(H, monkeypatch):
    """A prompt long enough for many key tiles and for more than 256 workgroups (the ones past 256 walk their query
    blocks in the other order): sampled rows against the oracle's single-query function, and the MFMA kernel
    against the plain one-wave-per-query kernel it replaced, over every row."""
    _llm()
    B, S, Nq = 2, 600, 16
    q = randn_bf16((B, S, Nq, H), 1.0, 171 + H)
    k = randn_bf16((B, Nq, S, H), 1.0, 172 + H)
    v = randn_bf16((B, Nq, S, H), 1.0, 173 + H)
    got = _attn_prefill(q.cuda(), k.cuda(), v.cuda(), 0).cpu()
    for i in (0, 1, 63, 64, 65, 511, 599):
        ref = O.attn_decode(t2bits(q[:, i]), t2bits(k[:, :, :i + 1]), t2bits(v[:, :, :i + 1]))
        g, r = bits2f(t2bits(got[:, i])).astype(np.float64), bits2f(ref).astype(np.float64)
        assert np.sqrt(((g - r) ** 2).sum() / (r ** 2).sum()) <= 5e-3, i
        assert np.abs(g - r).max() <= 2.0 ** -7 * np.abs(r).max(), i
    monkeypatch.setenv("TPPX_ATTN_PREFILL_MFMA", "0")
    plain = _attn_prefill(q.cuda(), k.cuda(), v.cuda(), 0).cpu()
    d = (plain.float() - got.float()).double()
    assert float(d.norm() / plain.double().norm()) <= 5e-3


@pytest.mark.parametrize("H", [64, 200])
def test_attn_prefill_other_head_size_with_mask(H):
    F = _llm()
    B, S, Nq, Smax = 2, 70, 4, 128
    q = randn_bf16((B, S, Nq, H), 1.0, 181 + H)
    k = randn_bf16((B, Nq, Smax, H), 1.0, 182 + H)
    v = randn_bf16((B, Nq, Smax, H), 1.0, 183 + H)
    keep = torch.ones(B, S, dtype=torch.int64)
    keep[0, :9] = 0  # left padding of sequence 0
    mask = F.TppCache(Smax).align_and_invert_mask(keep.to(torch.bfloat16))
    got = _attn_prefill(q.cuda(), k.cuda(), v.cuda(), 0, mask=mask.cuda())
    ref = O.attn_prefill(t2bits(q), t2bits(k[:, :, :S]), t2bits(v[:, :, :S]), mask.float().numpy())
    g, r = bits2f(t2bits(got)).astype(np.float64), bits2f(ref).astype(np.float64)
    assert np.isfinite(g).all()
    assert np.sqrt(((g - r) ** 2).sum() / (r ** 2).sum()) <= 5e-3
