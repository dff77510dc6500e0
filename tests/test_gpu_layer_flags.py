"""Weight-format switches of the decoder layer (src/csrc/llm/fused_llm_infer.cpp:35-45, 365-420, 1112-1175,
1216-1227): a LlamaDecoderLayer built from UNQUANTIZED blocked bf16 weights quantizes them itself under USE_MXFP4 /
USE_QINT8 / USE_QINT2 for the decode steps, keeps a first-token copy that stays unquantized unless USE_*_FT names a
format, and runs passes of FT_OPT_SIZE or more tokens on that copy when TPP_CACHE_REMAPPED_WEIGHTS is on.

Every case runs one decode step (1 token per sequence) and one prompt pass (FT_OPT_SIZE or more tokens) and compares
both with the composition of the oracle functions (fused_llm_infer.cpp:1229-1275) on the format the reference would
use for that pass: rel-L2 <= 2e-2 for the layer output (the GEMM tolerance compounded through seven linears, two
norms and the attention), cached keys / values within 1 bf16 ulp.  Also the unquantized-weight GEMM at prompt shapes
(the LDS-tiled bf16 kernel) against the oracle by itself.
"""
import numpy as np
import pytest
import torch

import oracle as O
from util import t2bits, randn_bf16, block_bf16, bits2f, assert_close_bf16

pytestmark = pytest.mark.gpu

HID, INTER, NQ, NKV, H, MP = 512, 1024, 4, 2, 128, 512
SHAPES = [(NQ * H, HID), (NKV * H, HID), (NKV * H, HID), (HID, NQ * H), (INTER, HID), (INTER, HID), (HID, INTER)]


def _oracle_linear(fmt, W):
    """fmt in {bf16, mxfp4, qint8, qint2} -> f(a_bits, post, post_in) on the plain weight W (bf16 tensor [N][K])."""
    Wf = W.float().numpy()
    if fmt == "bf16":
        wb = t2bits(W)
        return lambda a, post=O.POST_NONE, pin=None: O.linear_bf16(a, wb, None, post, pin, None, 1.0)
    if fmt == "mxfp4":
        q, s = O.remap_quantize_mxfp4(Wf)
        return lambda a, post=O.POST_NONE, pin=None: O.linear_mxfp4(a, q, s, None, post, pin, None, 1.0, O.MODE_IDEAL)
    if fmt == "qint8":
        q, s, _ = O.remap_quantize_qint8(Wf)
    else:
        q2, s2, _ = O.remap_quantize_qint2_intlv(Wf)
        q, s = O.qint2_to_qint8_layout(q2, s2)
    return lambda a, post=O.POST_NONE, pin=None: O.linear_qint8(a, q, s, None, post, pin, None, 1.0, O.MODE_IDEAL)


def _oracle_layer(mm, g1, g2, EP, xb, pos, B, S, k0, v0):
    """The layer on B x S tokens with `mm[i]` as the i-th linear; returns (out bits [B*S][HID], keys, values)."""
    h = O.rms_norm(xb, g1, 1e-5)
    q, k, v = mm[0](h), mm[1](h), mm[2](h)
    q = O.rotary_llama(q.reshape(B, S, -1), EP, pos, NQ, H).reshape(B, S, NQ, H)
    k = O.rotary_llama(k.reshape(B, S, -1), EP, pos, NKV, H).reshape(B, S, NKV, H).transpose(0, 2, 1, 3)
    v = v.reshape(B, S, NKV, H).transpose(0, 2, 1, 3)
    kall = np.concatenate([k0, k], axis=2)
    vall = np.concatenate([v0, v], axis=2)
    if S == 1:
        ctx = O.attn_decode(q.reshape(B, NQ, H), kall, vall).reshape(B, NQ * H)
    else:
        ctx = O.attn_prefill(q, kall, vall).reshape(B * S, NQ * H)
    so = mm[3](ctx, O.POST_ADD_SCALE, xb)
    h2 = O.rms_norm(so, g2, 1e-5)
    gate = mm[4](h2, O.POST_SILU)
    out = mm[6](mm[5](h2, O.POST_MUL, gate), O.POST_ADD_SCALE, so)
    return out, np.ascontiguousarray(k), np.ascontiguousarray(v)


CASES = [
    # flags set to 1, TPP_CACHE_REMAPPED_WEIGHTS, (format of the decode step, format of the prompt pass)
    ({}, 1, ("bf16", "bf16")),
    ({"USE_MXFP4": 1}, 1, ("mxfp4", "bf16")),
    ({"USE_MXFP4": 1, "USE_MXFP4_FT": 1}, 1, ("mxfp4", "mxfp4")),
    ({"USE_QINT8": 1}, 1, ("qint8", "bf16")),
    ({"USE_QINT8": 1, "USE_QINT8_FT": 1}, 1, ("qint8", "qint8")),
    ({"USE_QINT2": 1}, 1, ("qint2", "bf16")),
    ({"USE_QINT2": 1, "USE_QINT2_FT": 1}, 1, ("qint2", "qint2")),
    ({"USE_MXFP4": 1, "USE_QINT8_FT": 1}, 1, ("mxfp4", "qint8")),   # the _FT switches are independent of the decode format
    ({"USE_MXFP4": 1}, 0, ("mxfp4", "mxfp4")),                      # no cached first-token copy: every pass on the decode weights
    ({"USE_MXFP4": 1, "USE_QINT8": 1}, 1, ("mxfp4", "bf16")),       # USE_MXFP4 wins (the reference's if / else-if order)
]


@pytest.mark.parametrize("flags,cache_remapped,fmts", CASES)
def test_layer_weight_format_flags(flags, cache_remapped, fmts, monkeypatch):
    import tpp_pytorch_extension  # noqa: F401
    from tpp_pytorch_extension import _ops
    from tpp_pytorch_extension.llm import fused_llama_infer as F
    for name in ("USE_MXFP4", "USE_MXFP4_FT", "USE_QINT8", "USE_QINT8_FT", "USE_QINT2", "USE_QINT2_FT"):
        monkeypatch.setattr(F, name, flags.get(name, 0))
    monkeypatch.setattr(F, "TPP_CACHE_REMAPPED_WEIGHTS", cache_remapped)
    monkeypatch.setattr(F, "FT_OPT_SIZE", 32)
    Ws = [randn_bf16(s, 0.05, 810 + i) for i, s in enumerate(SHAPES)]
    rng = torch.Generator().manual_seed(81)
    g1, g2 = torch.rand(HID, generator=rng) + 0.5, torch.rand(HID, generator=rng) + 0.5
    EP = F.llama_rotary_table(MP, H, device="cpu")
    blocked = [block_bf16(W).cuda() for W in Ws]
    layer = F.LlamaDecoderLayer([g1.cuda()] + blocked[:4] + [g2.cuda()] + blocked[4:] + [EP.cuda()], 0, 1e-5, H, MP, H)
    assert (layer.Nq, layer.Nkv) == (NQ, NKV)
    # what the constructor left: decode weights quantized under USE_*, the first-token copies taken before that
    quantized = fmts[0] != "bf16"
    assert isinstance(layer.t_Wq, _ops.QTensor) == quantized and isinstance(layer.t_Wd, _ops.QTensor) == quantized
    assert layer.first_token_remapped == quantized  # otherwise taken lazily by the first long pass

    for S, fmt in ((1, fmts[0]), (40, fmts[1])):
        B, past, cap = 2, 21, 128
        cache = F.TppCache(cap)
        k0, v0 = randn_bf16((B, NKV, past, H), 1.0, 861), randn_bf16((B, NKV, past, H), 1.0, 862)
        cache.fill_(0, k0.cuda(), v0.cuda())
        x = randn_bf16((B, S, HID), 1.0, 863 + S)
        pos = torch.arange(past, past + S, dtype=torch.int64).unsqueeze(0).repeat(B, 1)
        out = layer.forward([x.cuda(), None, pos.cuda()], cache, True)[0]
        cache.advance(S)
        mm = [_oracle_linear(fmt, W) for W in Ws]
        ref, k, v = _oracle_layer(mm, g1.numpy(), g2.numpy(), EP.numpy(), t2bits(x).reshape(B * S, HID), pos.numpy(),
                                  B, S, t2bits(k0), t2bits(v0))
        g, r = bits2f(t2bits(out)).reshape(B * S, HID).astype(np.float64), bits2f(ref).astype(np.float64)
        rel = np.sqrt(((g - r) ** 2).sum() / (r ** 2).sum())
        assert rel <= 2e-2, (S, fmt, rel)
        kc, vc = cache.get(0)
        assert_close_bf16(t2bits(kc[:, :, past:]), k, what=f"cached keys S={S} {fmt}")
        assert_close_bf16(t2bits(vc[:, :, past:]), v, what=f"cached values S={S} {fmt}")
        if fmt != fmts[1 - (S > 1)]:
            # the two passes use different formats: the other format's oracle must NOT match as closely, i.e. the
            # pass really ran on the copy the flags name
            other = [_oracle_linear(fmts[1 - (S > 1)], W) for W in Ws]
            ref2 = _oracle_layer(other, g1.numpy(), g2.numpy(), EP.numpy(), t2bits(x).reshape(B * S, HID), pos.numpy(),
                                 B, S, t2bits(k0), t2bits(v0))[0]
            r2 = bits2f(ref2).astype(np.float64)
            assert np.sqrt(((g - r2) ** 2).sum() / (r2 ** 2).sum()) > rel
    if cache_remapped:
        assert layer.first_token_remapped
        assert isinstance(layer._first[0], _ops.QTensor) == (fmts[1] != "bf16")


@pytest.mark.parametrize("M,N,K,post", [(128, 256, 512, "none"), (300, 1056, 1024, "add"), (2048, 4096, 4096, "silu"),
                                        (65, 48, 128, "mul"), (1000, 11008, 4096, "none"), (193, 16, 128, "add"),
                                        (257, 4112, 256, "mul")])
def test_unquantized_bf16_weight_gemm_at_prompt_shapes(M, N, K, post, monkeypatch):
    """TppBlockedLinearW<bf16, bf16> (src/csrc/fused_gemm.h:785-1073, non-quantized branch) above 64 rows: the
    LDS-tiled bf16 kernels (ragged rows, ragged channel tiles: from 192 rows the 128 x 256 form of the large prefill
    kernel with hand-counted weight loads, below that and under TPPX_BF16_BIG=0 the 128 x 128 one) and the
    row-group kernel give the oracle's tile."""
    import ctypes
    import tpp_pytorch_extension  # noqa: F401
    from tpp_pytorch_extension import _ops, _lib
    posts = {"none": O.POST_NONE, "add": O.POST_ADD_SCALE, "silu": O.POST_SILU, "mul": O.POST_MUL}
    W = randn_bf16((N, K), 0.05, 9000 + N)
    x = randn_bf16((M, K), 1.0, 9001 + M)
    b = randn_bf16((N,), 0.01, 9002)
    pin = randn_bf16((M, N), 1.0, 9003)
    ref = O.linear_bf16(t2bits(x), t2bits(W), t2bits(b), posts[post], t2bits(pin), None, 0.5)
    pre = O.linear_bf16(t2bits(x), t2bits(W), t2bits(b)) if post == "add" else None
    wb = block_bf16(W).cuda()
    for flags in (_lib.FLAG_FORCE_TILED, _lib.FLAG_FORCE_SKINNY, 0):
        y = _ops.linear(x.cuda(), wb, b.cuda(), posts[post], pin.cuda(), None, 0.5, flags=flags)
        assert_close_bf16(t2bits(y), ref, ulps=2 if post == "silu" else 1, what=f"bf16 weight M={M} N={N} K={K} {post} flags={flags}",
                          pre_bits=pre)
    monkeypatch.setenv("TPPX_BF16_BIG", "0")
    y = _ops.linear(x.cuda(), wb, b.cuda(), posts[post], pin.cuda(), None, 0.5, flags=_lib.FLAG_FORCE_TILED)
    assert_close_bf16(t2bits(y), ref, ulps=2 if post == "silu" else 1, what=f"bf16 weight M={M} N={N} K={K} {post} 128 x 128 kernel",
                      pre_bits=pre)
