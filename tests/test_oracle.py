"""Pins the CPU oracle (oracle/tppx_oracle.c) before anything is compared with it.

Evidence used, per function:
  * MX element / scale math: golden vectors written from the reference's own
    src/csrc/mxfp_quant.h (tests/golden/mxfp4_golden.npz), the live shim
    around that header where it was built, OCP-MX known answers, and an
    independent nearest / ties-to-even table search over all bf16 patterns.
  * INT8: invariants (|w - q*s| <= s/2, the block maximum maps to +-127, an
    all-zero block has scale 0) and an fp64 restatement.
  * Layouts: the closed-form index maps coded in C against the view/permute
    chain restated with numpy, and against a brute-force loop on a tiny case.
  * Linears: fp64 matmul over the exactly de-quantized weight; exact int32
    block sums; agreement of the faithful and ideal modes where the reference
    rounds only once.
  * Post-ops: torch CPU ops with the same bf16 rounding points.
"""
import os

import numpy as np
import pytest
import torch

import oracle as O
from util import bits2f, t2bits, randn_bf16

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "mxfp4_golden.npz")
GRID = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0], np.float64)


def _encode_all(vals):
    return O.e2m1_encode_array(vals)


def _ref_value_to_code(ref):
    """The value -> code chain of the reference (qtypes.cpp:99-131): +-0 -> 0,
    a NaN matches nothing and leaves 0."""
    codes = np.zeros(ref.shape, np.int64)
    for i, r in enumerate(ref):
        if r != r or r == 0.0:
            continue
        idx = int(np.where(GRID == abs(float(r)))[0][0])
        codes[i] = idx | (8 if r < 0 else 0)
    return codes


def test_e2m1_against_golden_all_bf16():
    g = np.load(GOLD)
    vals = (np.arange(65536, dtype=np.uint32) << 16).view(np.float32)
    want = _ref_value_to_code(g["e2m1_bf16_out"].view(np.float32))
    got = _encode_all(vals)
    assert np.array_equal(got, want)


def test_e2m1_against_golden_ties_and_random_fp32():
    g = np.load(GOLD)
    vals = g["tie_in"].view(np.float32)
    want = _ref_value_to_code(g["tie_out"].view(np.float32))
    assert np.array_equal(_encode_all(vals), want)


def test_scale_against_golden():
    g = np.load(GOLD)
    a = (np.arange(32768, dtype=np.uint32) << 16).view(np.float32)
    assert np.array_equal(O.mx_quant_scale_of_amax_array(a).view(np.uint32), g["scale_bf16_out"])
    a = g["scale_in"].view(np.float32)
    assert np.array_equal(O.mx_quant_scale_of_amax_array(a).view(np.uint32), g["scale_out"])


def test_against_live_reference_shim():
    R = O.ref_lib()
    if R is None:
        pytest.skip("oracle/_ref not built (reference tree not mounted)")
    rng = np.random.default_rng(3)
    for v in (rng.standard_normal(3000) * 4).astype(np.float32):
        r = R.ref_e2m1_round(float(v))
        want = 0.0 if (r != r) else r
        assert O.e2m1_decode(O.e2m1_encode(float(v))) == want
    for v in np.abs(rng.standard_normal(3000)).astype(np.float32) * np.float32(2.0) ** rng.integers(-130, 127, 3000):
        v = np.float32(v)
        a = np.float32(R.ref_mx_shared_scale(float(v))).view(np.uint32)
        b = np.float32(O.mx_quant_scale(O.mx_scale_byte(float(v)))).view(np.uint32)
        assert a == b


def test_ocp_mx_known_answers():
    # value/scale -> E2M1 value (ties to even mantissa, saturation at 6)
    for v, want in [(1.25, 1.0), (1.75, 2.0), (2.5, 2.0), (3.5, 4.0), (5.0, 4.0), (0.25, 0.0), (0.75, 1.0),
                    (7.0, 6.0), (6.5, 6.0), (-5.0, -4.0), (0.2499, 0.0), (0.2501, 0.5), (100.0, 6.0),
                    (-0.08, 0.0)]:
        assert O.e2m1_decode(O.e2m1_encode(v)) == want, v
    assert O.e2m1_encode(-0.08) == 0  # never the negative-zero code
    assert O.e2m1_encode(-0.0) == 0
    # block maximum -> E8M0 byte: floor(log2 max) - 2 + 127
    for a, want in [(1.0, 125), (0.078, 121), (6.0, 127), (7.9, 127), (0.0, 0), (1e-40, 0), (3e38, 252)]:
        assert O.mx_scale_byte(a) == want, a
    assert O.mx_dequant_scale(0) == 0.0 and O.mx_dequant_scale(127) == 1.0


def test_e2m1_independent_table_search():
    """Nearest grid point, ties to the even code, computed in fp64 without the
    oracle's threshold chain."""
    vals = (np.arange(65536, dtype=np.uint32) << 16).view(np.float32)
    finite = np.isfinite(vals)
    a = np.minimum(np.abs(vals[finite].astype(np.float64)), 8.0)  # everything from 8 up saturates
    grid9 = np.append(GRID, 8.0)  # 8 = first value beyond the format; rounds there, then saturates
    d = np.abs(a[:, None] - grid9[None, :])
    best = d.min(axis=1)
    cand = d == best[:, None]
    idx = np.empty(a.shape, np.int64)
    for i in range(a.size):
        c = np.flatnonzero(cand[i])
        idx[i] = c[0] if len(c) == 1 else [k for k in c if k % 2 == 0][0]
    idx = np.minimum(idx, 7)
    want = np.where((idx > 0) & (np.signbit(vals[finite])), idx | 8, idx)
    assert np.array_equal(_encode_all(vals[finite]), want)


def test_int8_invariants():
    rng = np.random.default_rng(5)
    t = (rng.standard_normal((6, 4, 64, 16, 4)) * 0.02).astype(np.float32)
    t[0, 0] = 0.0  # an all-zero block
    q, s = O.quantize_int8sym(t, 256, 2, True)
    assert s.shape == (6, 4, 1, 16) and q.shape == t.shape
    assert np.all(s[0, 0] == 0.0) and np.all(q[0, 0] == 0)
    sb = np.broadcast_to(s[:, :, :, :, None], (6, 4, 1, 16, 1))
    assert np.all(np.abs(t - q * sb) <= sb * 0.5 * (1 + 1e-6) + 1e-12)
    amax = np.abs(t).max(axis=(2, 4))
    assert np.array_equal(s[:, :, 0, :], (amax.astype(np.float64) / 127.0).astype(np.float32))
    assert np.array_equal(np.abs(q).max(axis=(2, 4))[1:], np.full((5, 4, 16), 127))
    d = O.dequantize_int8sym(q, s, 256, 2, True)
    assert np.array_equal(d, q.astype(np.float32) * sb)


def test_act_quant_matches_generic_quantizer():
    x = randn_bf16((5, 768), 1.0, 11)
    xq, sa = O.quant_act_int8(t2bits(x), 256)
    q2, s2 = O.quantize_int8sym(x.float().numpy(), 256, -1, False)
    assert np.array_equal(xq, q2) and np.array_equal(sa, s2)


@pytest.mark.parametrize("shape", [(64, 128), (96, 320)])
def test_layout_closed_form_equals_view_permute_chain(shape):
    N, K = shape
    rng = np.random.default_rng(N)
    W = O.bf16_round((rng.standard_normal((N, K)) * 0.02).astype(np.float32))
    for vnni in (2, 1):  # 5-D bf16-style and 4-D fp32-style blocked inputs
        Wb = O.block_weight(W, 16, 64, vnni)
        assert np.array_equal(O.unblock_weight(Wb), W)
        q1, s1 = O.remap_and_quantize_mxfp4_blocked(Wb)
        q2, s2 = O.remap_quantize_mxfp4(W)
        assert np.array_equal(q1, q2) and np.array_equal(s1, s2)
        qa, sa, qbs = O.remap_and_quantize_qint8_blocked(Wb)
        qb, sb, qbs2 = O.remap_quantize_qint8(W)
        assert qbs == qbs2 and np.array_equal(qa, qb) and np.array_equal(sa, sb)
    # a 64-wide output block (K2 > 32) is split instead of paired
    q3, s3 = O.remap_and_quantize_mxfp4_blocked(O.block_weight(W[:64], 64, 64, 2))
    q4, s4 = O.remap_quantize_mxfp4(W[:64])
    assert np.array_equal(q3, q4) and np.array_equal(s3, s4)


def test_mx_block_maximum_nan_rule():
    """PerBlockQuantizer::quantize_symetric (qtypes.h:156-162) starts its maximum at |first element| and updates with
    std::max(max, |v|): a NaN in the first slot of a block stays (shared exponent 255 -> scale byte 255, every
    code 0), a NaN in any other slot never wins the comparison (the block keeps the scale of its finite maximum;
    the NaN element itself encodes as 0).  The closed-form restatement must agree with the restatement of the
    reference's own view / permute / generic-quantizer chain on both, and Inf always wins."""
    W = np.full((32, 64), 0.5, np.float32)
    W[3, 0] = np.nan        # first slot of block (row 3, half 0)
    W[4, 33] = np.nan       # second slot of block (row 4, half 1)
    W[5, 32 + 7] = np.inf
    W[6, 0] = -np.inf
    q1, s1 = O.remap_and_quantize_mxfp4_blocked(O.block_weight(W, 16, 64, 1))
    q2, s2 = O.remap_quantize_mxfp4(W)
    assert np.array_equal(q1, q2) and np.array_equal(s1, s2)
    sc = s2[0, 0]  # [h][k2]
    assert sc[0, 3] == 255 and sc[1, 4] == 124 and sc[1, 5] == 255 and sc[0, 6] == 255 and sc[0, 0] == 124
    deq = O.dequantize_mxfp4_plain(q2, s2)
    assert deq[4, 33] == 0.0 and deq[4, 34] == 0.5 and deq[0, 0] == 0.5


def test_int4_quantizer_closed_form_and_invariants():
    """Int4SymQuant (qtypes.cpp:199-246): scale = max/7 (double division), codes clamp(rne(w/scale), -8, 7) as two's
    complement nibbles, low nibble = even element; dequantize = table[code] * scale.  Known answers, the error bound
    |w - q*s| <= s/2 and brute force against an independent numpy statement."""
    t = np.array([[7.0, -7.0, 3.5, 2.5, 1.49, -0.5, 0.5, 0.0]], np.float32)          # max 7 -> scale 1
    q, s = O.quantize_int4sym(t, 8, -1, False)
    assert s.shape == (1, 1) and s[0, 0] == 1.0
    codes = np.stack([q[0] & 0xF, q[0] >> 4], -1).reshape(-1)
    assert codes.tolist() == [7, 9, 4, 2, 1, 0, 0, 0]                               # -7 -> 9, 3.5 -> 4, 2.5 -> 2, -0.5 -> -0
    rng = np.random.default_rng(4)
    x = (rng.standard_normal((5, 3, 64, 6, 2)) * 0.3).astype(np.float32)
    q, s = O.quantize_int4sym(x, 32, 2, True)
    d = O.dequantize_int4sym(q, s, 32, 2, True)
    # independent statement: blocks of 16 x 2 elements along axis 2 sharing (.., k2)
    xb = x.reshape(5, 3, 4, 16, 6, 2)
    amax = np.abs(xb).max(axis=(3, 5), keepdims=True)
    sc = (amax.astype(np.float64) / 7.0).astype(np.float32)
    inv = np.where(sc != 0, np.float32(1.0) / sc, np.float32(0.0)).astype(np.float32)
    qq = np.clip(np.rint((xb * inv).astype(np.float32)), -8, 7)
    assert np.array_equal(s.reshape(5, 3, 4, 6), sc.reshape(5, 3, 4, 6))
    assert np.array_equal(d.reshape(xb.shape), (qq * sc).astype(np.float32))
    assert (np.abs(d.reshape(xb.shape) - xb) <= sc / 2 + 1e-12).all()


@pytest.mark.parametrize("N,K", [(32, 256), (96, 768), (64, 192)])
def test_qint2_closed_form_equals_view_permute_chain(N, K):
    """remap_and_quantize_qint2_intlv (qtypes.cpp:1004-1073): the closed-form C restatement against a numpy
    restatement of the reference's own view / permute / bit-pack chain; ternary codes, ties to even, zero blocks."""
    rng = np.random.default_rng(N + K)
    W = O.bf16_round((rng.standard_normal((N, K)) * 0.02).astype(np.float32))
    W[1, :64] = 0.0
    q, sc, bs = O.remap_quantize_qint2_intlv(W)
    assert bs == O.qint2_block_size(K) and K % bs == 0
    q2, sc2 = O.remap_quantize_qint2_intlv_chain(W, bs)
    assert np.array_equal(q, q2) and np.array_equal(sc, sc2)
    # brute force one element: channel n, input k
    for n, k in ((0, 0), (13, 77), (31, K - 1), (N - 1, 5)):
        b, c = divmod(k, bs)
        s = max(np.abs(W[n, b * bs:(b + 1) * bs]).max(), np.float32(1e-8))
        t = np.rint(np.float32(W[n, k]) / np.float32(s))
        code = 1 if t >= 1 else (2 if t <= -1 else 0)
        n1, r = divmod(n, 32)
        byte = q[n1, b, c // 4, r % 8, c % 4]
        assert (byte >> (2 * (r // 8))) & 3 == code and sc[n1, b, r, 0] == s
    v8, s8 = O.qint2_to_qint8_layout(q, sc)
    assert set(np.unique(v8).tolist()) <= {-1, 0, 1}


def test_layout_brute_force_index_formula():
    N, K = 32, 64
    W = np.arange(N * K, dtype=np.float32).reshape(N, K) % 13 - 6.0
    q, s = O.remap_quantize_mxfp4(W)
    Wd = O.dequantize_mxfp4_plain(q, s)
    t5 = O.dequantize_mxfp4(q.reshape(1, 1, 32, 32, 1), s)  # generic blocked-shape dequantizer
    for n in range(N):
        for k in range(K):
            b = int(q[0, 0, k // 2, n])
            code = (b >> 4) if (k & 1) else (b & 15)
            x = int(s[0, 0, k // 32, n])
            assert Wd[n, k] == O.E2M1_TABLE[code] * O.mx_dequant_scale(x)
            assert t5[0, 0, k // 2, n, k & 1] == Wd[n, k]
    qi, si, qbs = O.remap_quantize_qint8(W)
    assert qbs == 64
    Wi = O.dequantize_qint8_plain(qi, si)
    for n in range(N):
        for k in range(K):
            assert Wi[n, k] == np.float32(qi[n // 16, 0, k // 4, n % 16, k % 4]) * si[n // 16, 0, 0, n % 16]


def test_qint8_block_size_rule():
    assert O.qint8_block_size(4096) == 256 and O.qint8_block_size(11008) == 256
    assert O.qint8_block_size(192) == 64 and O.qint8_block_size(384) == 128
    assert O.qint8_block_size(4096, 4096) == 4096


def test_mx_roundtrip_error_bound():
    rng = np.random.default_rng(9)
    W = (rng.standard_normal((64, 256)) * 0.02).astype(np.float32)
    q, s = O.remap_quantize_mxfp4(W)
    Wd = O.dequantize_mxfp4_plain(q, s)
    scale = np.array([[O.mx_dequant_scale(int(s[n // 32, k // 64, (k % 64) // 32, n % 32])) for k in range(256)]
                      for n in range(64)], np.float32)
    # the block maximum lies in [4, 8) scale units: rounding costs at most half
    # the largest step (1.0) and saturation at 6 at most 2.0
    assert np.all(np.abs(W - Wd) <= scale * 2.0 + 1e-12)
    assert np.all(np.abs(W - Wd)[np.abs(W) <= 6 * scale] <= scale[np.abs(W) <= 6 * scale] * 1.0 + 1e-12)


@pytest.mark.parametrize("fmt", ["mxfp4", "qint8"])
def test_linear_reduces_to_fp64_matmul(fmt):
    M, N, K = 7, 96, 512
    W = randn_bf16((N, K), 0.02, 21).float().numpy()
    x = randn_bf16((M, K), 1.0, 22)
    bias = randn_bf16((N,), 0.01, 23)
    xb, bb = t2bits(x), t2bits(bias)
    if fmt == "mxfp4":
        q, s = O.remap_quantize_mxfp4(W)
        Wd = O.dequantize_mxfp4_plain(q, s).astype(np.float64)
        want = x.float().numpy().astype(np.float64) @ Wd.T + bits2f(bb)
        y = O.linear_mxfp4(xb, q, s, bb)
        y64 = O.linear_mxfp4(xb, q, s, bb, mode=O.MODE_F64)
        assert np.array_equal(y, O.linear_mxfp4(xb, q, s, bb, mode=O.MODE_FAITHFUL))  # one chunk when M/64 <= 4
    else:
        q, s, qbs = O.remap_quantize_qint8(W)
        xq, sa = O.quant_act_int8(xb, qbs)
        acc = O.qint8_block_sums(xq, q)
        Wq = np.round(O.dequantize_qint8_plain(q, np.ones_like(s))).astype(np.int64)
        want_acc = np.einsum("mbk,nbk->mnb", xq.astype(np.int64).reshape(M, K // qbs, qbs), Wq.reshape(N, K // qbs, qbs))
        assert np.array_equal(acc, want_acc)  # exact int32 block sums
        sw = s.reshape(N // 16, K // qbs, 16).transpose(0, 2, 1).reshape(N, K // qbs)
        want = (acc.astype(np.float64) * sa[:, None, :].astype(np.float64) * sw[None].astype(np.float64)).sum(-1) + bits2f(bb)
        y = O.linear_qint8(xb, q, s, bb)
        y64 = O.linear_qint8(xb, q, s, bb, mode=O.MODE_F64)
    want_bf16 = O.f32_to_bf16(want.astype(np.float32))
    # fp64 mode is the exact sum rounded once (up to the double->float->bf16 double rounding)
    assert np.mean(y64 != want_bf16) < 2e-3
    # fp32 accumulation stays within one bf16 ulp of the exact result
    d = np.abs(bits2f(y).astype(np.float64) - want)
    assert np.all(d <= 2.0 ** -7 * np.abs(want) + 2.0 ** -8 * np.sqrt(np.mean(want * want)))


def test_faithful_chunking_differs_only_within_tolerance():
    M, N, K = 384, 32, 8192  # M/64 > 4 -> the reference re-rounds every 4096 input channels
    W = randn_bf16((N, K), 0.02, 31).float().numpy()
    x = t2bits(randn_bf16((M, K), 1.0, 32))
    q, s = O.remap_quantize_mxfp4(W)
    a = bits2f(O.linear_mxfp4(x, q, s, mode=O.MODE_IDEAL)).astype(np.float64)
    b = bits2f(O.linear_mxfp4(x, q, s, mode=O.MODE_FAITHFUL)).astype(np.float64)
    assert np.any(a != b)
    assert np.sqrt(((a - b) ** 2).sum() / (a ** 2).sum()) < 2.0 ** -9 * np.sqrt(2)


def test_post_ops_against_torch_rounding_points():
    y = randn_bf16((4096,), 2.0, 41)
    in1 = randn_bf16((4096,), 1.0, 42)
    in2 = randn_bf16((4096,), 1.0, 43)
    bf = torch.bfloat16
    yf, a, b = y.float(), in1.float(), in2.float()
    cases = {
        O.POST_MUL: (a * yf).to(bf),
        O.POST_ADD_SCALE: (yf + a * 0.5).to(bf),
        O.POST_ADD2_SCALE: ((yf + a).to(bf).float() + b * 0.5).to(bf),
        O.POST_RELU: torch.clamp_min(y, 0),
    }
    for post, want in cases.items():
        got = O.post_op(t2bits(y), post, t2bits(in1), t2bits(in2), 0.5)
        assert np.array_equal(got, t2bits(want)), post
    # transcendental post-ops: libm vs torch may differ in the last fp32 bit
    silu = (yf * torch.sigmoid(yf).to(bf).float()).to(bf)
    gelu = torch.nn.functional.gelu(yf).to(bf)
    for post, want in ((O.POST_SILU, silu), (O.POST_GELU, gelu)):
        got = bits2f(O.post_op(t2bits(y), post)).astype(np.float64)
        w = want.float().numpy().astype(np.float64)
        assert np.all(np.abs(got - w) <= 2.0 ** -7 * np.abs(w) + 1e-30)
        assert np.mean(got != w) < 0.01


# ---------------------------------------------------------------------------
# decode-side operators: the numpy restatements against independent statements
# ---------------------------------------------------------------------------
def test_oracle_rms_norm_against_torch_and_closed_form():
    import torch
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(5, 384, generator=g) * 2).to(torch.bfloat16)
    w = torch.rand(384, generator=g) + 0.5
    got = O.bf16_to_f32(O.rms_norm(x.view(torch.int16).numpy().view(np.uint16), w.numpy(), 1e-6))
    xf = x.float()
    ref = ((xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-6)) * w).to(torch.bfloat16).float().numpy()
    assert np.abs(got - ref).max() <= 2.0 ** -7 * np.abs(ref).max()
    assert (got != ref).mean() < 0.02  # at most a last-bit difference from the order of the fp32 operations
    # closed form: a constant row c with unit weight normalises to sign(c) (eps negligible)
    c = np.full((1, 64), 3.0, np.float32)
    one = O.bf16_to_f32(O.rms_norm(O.f32_to_bf16(c), np.ones(64, np.float32), 1e-12))
    assert np.allclose(one, 1.0, atol=2.0 ** -8)


def test_oracle_rotary_is_a_rotation_and_matches_rotate_half():
    import torch
    B, S, N, H, MP = 2, 3, 2, 32, 16
    g = torch.Generator().manual_seed(4)
    t = torch.randn(B, S, N * H, generator=g).to(torch.bfloat16)
    inv = 1.0 / (10000.0 ** (torch.arange(0, H, 2).float() / H))
    fr = torch.outer(torch.arange(MP).float(), inv)
    emb = torch.stack((torch.cat((fr, fr), -1).cos(), torch.cat((fr, fr), -1).sin()))
    pos = torch.tensor([[0, 5, 15], [7, 16, 2]])  # 16 is out of range
    got = O.bf16_to_f32(O.rotary_llama(t.view(torch.int16).numpy().view(np.uint16), emb.numpy(), pos.numpy(), N, H))
    # the Hugging Face formulation: x*cos + rotate_half(x)*sin with rotate_half(x) = cat(-x2, x1)
    x = t.float().view(B, S, N, H)
    p = pos.clamp(max=MP - 1)
    cos, sin = emb[0][p][:, :, None, :], emb[1][p][:, :, None, :]
    rh = torch.cat((-x[..., H // 2:], x[..., :H // 2]), -1)
    ref = (x * cos + rh * sin)
    ref[1, 1] = x[1, 1]  # position 16 >= MP stays untouched
    ref = ref.to(torch.bfloat16).float().view(B, S, N * H).numpy()
    assert np.abs(got - ref).max() <= 2.0 ** -7 * np.abs(ref).max()
    # position 0 is the identity, and a rotation keeps the norm of every (h2, H/2+h2) pair
    assert np.array_equal(got[0, 0], t.float().numpy()[0, 0])
    a = t.float().view(B, S, N, 2, H // 2).numpy()
    b = got.reshape(B, S, N, 2, H // 2)
    assert np.allclose((a ** 2).sum(3), (b ** 2).sum(3), rtol=2e-2, atol=1e-3)


def test_oracle_layer_norm_against_torch_and_closed_forms():
    """The LayerNorm restatement against torch's own layer_norm (an independent library routine, evaluated in
    fp64) and against what the formula fixes: a constant row gives beta exactly (v = 0, x*s + b = 0), a row of
    +-a has mean 0 and variance a^2, and swapping gamma with beta or dropping the mean changes the result."""
    import torch
    g = torch.Generator().manual_seed(13)
    x = (torch.randn(5, 384, generator=g) * 2 + 0.7).to(torch.bfloat16)
    w = torch.rand(384, generator=g) + 0.5
    b = torch.randn(384, generator=g) * 0.3
    got = O.bf16_to_f32(O.layer_norm(x.view(torch.int16).numpy().view(np.uint16), w.numpy(), b.numpy(), 1e-5))
    ref64 = torch.nn.functional.layer_norm(x.double(), (384,), w.double(), b.double(), 1e-5)
    ref = ref64.float().to(torch.bfloat16).float().numpy()
    assert np.abs(got - ref).max() <= 2.0 ** -7 * np.abs(ref).max()
    assert (got != ref).mean() < 0.02  # E[x^2] - m^2 in fp32 against the two-pass fp64 variance: last-bit differences
    # without the mean (RMSNorm) or with gamma and beta swapped the answer is far off
    nomean = ((x.double() * torch.rsqrt(x.double().pow(2).mean(-1, keepdim=True) + 1e-5)) * w + b).float().numpy()
    assert np.abs(got - nomean).max() > 0.1
    swapped = torch.nn.functional.layer_norm(x.double(), (384,), b.double(), w.double(), 1e-5).float().numpy()
    assert np.abs(got - swapped).max() > 0.1
    # closed forms
    c = np.full((1, 64), 3.0, np.float32)
    beta = np.linspace(-1, 1, 64).astype(np.float32)
    const = O.bf16_to_f32(O.layer_norm(O.f32_to_bf16(c), np.full(64, 7.0, np.float32), beta, 1e-5))
    assert np.array_equal(const[0], O.bf16_to_f32(O.f32_to_bf16(beta)))
    pm = np.tile(np.array([2.0, -2.0], np.float32), 32)[None]
    out = O.bf16_to_f32(O.layer_norm(O.f32_to_bf16(pm), np.ones(64, np.float32), np.zeros(64, np.float32), 1e-12))
    assert np.allclose(out, np.sign(pm), atol=2.0 ** -8)


def test_oracle_rotary_gptj_is_a_rotation_of_adjacent_pairs():
    """The GPT-J rotary restatement against the Hugging Face formulation (x*cos + rotate_every_two(x)*sin with the
    sin | cos table of create_sinusoidal_positions, written out here in torch) and against closed forms: position 0
    is the identity, dims >= rotary_dim are untouched, adjacent pairs keep their norm, and (x, 0) at angle theta
    becomes (x cos theta, x sin theta) -- a swapped table half or a wrong sign fails one of them."""
    import torch
    B, S, N, H, HR, MP = 2, 3, 2, 32, 16, 16
    g = torch.Generator().manual_seed(14)
    t = torch.randn(B, S, N * H, generator=g).to(torch.bfloat16)
    inv = 1.0 / (10000.0 ** (torch.arange(0, HR, 2).float() / HR))
    fr = torch.outer(torch.arange(MP).float(), inv)
    emb = torch.cat((fr.sin(), fr.cos()), dim=1)  # [MP][HR]
    pos = torch.tensor([[0, 5, 15], [7, 16, 2]])  # 16 is out of range
    got = O.bf16_to_f32(O.rotary_gptj(t.view(torch.int16).numpy().view(np.uint16), emb.numpy(), pos.numpy(), N, H))
    x = t.float().view(B, S, N, H)
    p = pos.clamp(max=MP - 1)
    sin = torch.repeat_interleave(emb[p][:, :, None, :HR // 2], 2, dim=-1)
    cos = torch.repeat_interleave(emb[p][:, :, None, HR // 2:], 2, dim=-1)
    xr = x[..., :HR]
    r2 = torch.stack((-xr[..., 1::2], xr[..., ::2]), dim=-1).flatten(-2)  # rotate_every_two
    ref = x.clone()
    ref[..., :HR] = xr * cos + r2 * sin
    ref[1, 1] = x[1, 1]
    ref = ref.to(torch.bfloat16).float().view(B, S, N * H).numpy()
    assert np.abs(got - ref).max() <= 2.0 ** -7 * np.abs(ref).max()
    tf = t.float().numpy()
    assert np.array_equal(got[0, 0], tf[0, 0])                                     # position 0
    assert np.array_equal(got.reshape(B, S, N, H)[..., HR:], tf.reshape(B, S, N, H)[..., HR:])  # pass-through dims
    a = tf.reshape(B, S, N, H)[..., :HR].reshape(B, S, N, HR // 2, 2)
    b = got.reshape(B, S, N, H)[..., :HR].reshape(B, S, N, HR // 2, 2)
    assert np.allclose((a ** 2).sum(-1), (b ** 2).sum(-1), rtol=2e-2, atol=1e-3)
    one = np.zeros((1, 1, H), np.float32)
    one[0, 0, 0] = 1.0                                                             # pair 0 = (1, 0)
    e = O.bf16_to_f32(O.rotary_gptj(O.f32_to_bf16(one), emb.numpy(), np.array([[3]]), 1, H))
    theta = 3.0 * float(inv[0])
    assert abs(e[0, 0, 0] - np.cos(theta)) < 2.0 ** -8 and abs(e[0, 0, 1] - np.sin(theta)) < 2.0 ** -8


def test_oracle_attn_decode_against_softmax_and_special_cases():
    import torch
    B, Nq, Nkv, L, H = 2, 4, 2, 19, 16
    g = torch.Generator().manual_seed(6)
    q = torch.randn(B, Nq, H, generator=g).to(torch.bfloat16)
    k = torch.randn(B, Nkv, L, H, generator=g).to(torch.bfloat16)
    v = torch.randn(B, Nkv, L, H, generator=g).to(torch.bfloat16)
    bits = lambda t: t.contiguous().view(torch.int16).numpy().view(np.uint16)
    got = O.bf16_to_f32(O.attn_decode(bits(q), bits(k), bits(v), None, round_probs=False))
    kk, vv = k.double().repeat_interleave(2, 1), v.double().repeat_interleave(2, 1)
    s = torch.einsum("bnh,bnlh->bnl", q.double(), kk) / np.sqrt(H)
    ref = torch.einsum("bnl,bnlh->bnh", torch.softmax(s, -1), vv).numpy()
    assert np.abs(got - ref).max() <= 2.0 ** -8 * np.abs(ref).max() + 1e-6
    # bf16 probabilities change the answer by well under a percent
    gotb = O.bf16_to_f32(O.attn_decode(bits(q), bits(k), bits(v)))
    assert np.sqrt(((gotb - ref) ** 2).sum() / (ref ** 2).sum()) < 5e-3
    # one key: the output is that key's value; identical values: the output is that value whatever the scores
    one = O.bf16_to_f32(O.attn_decode(bits(q), bits(k[:, :, :1]), bits(v[:, :, :1])))
    assert np.array_equal(one, v[:, :, 0].float().repeat_interleave(2, 1).numpy())
    vc = v[:, :, :1].expand(-1, -1, L, -1)
    same = O.bf16_to_f32(O.attn_decode(bits(q), bits(k), bits(vc), None, round_probs=False))
    assert np.abs(same - vc[:, :, 0].float().repeat_interleave(2, 1).numpy()).max() <= 2.0 ** -7 * 4
    # a -10000 mask entry removes the key
    m = np.zeros((B, L), np.float32); m[:, 3] = -10000.0
    masked = O.bf16_to_f32(O.attn_decode(bits(q), bits(k), bits(v), m, round_probs=False))
    keep = [i for i in range(L) if i != 3]
    dropped = O.bf16_to_f32(O.attn_decode(bits(q), bits(k[:, :, keep]), bits(v[:, :, keep]), None, round_probs=False))
    assert np.array_equal(masked, dropped)


def test_oracle_attn_prefill_against_causal_softmax_and_decode():
    """Pins the multi-query restatement: (i) the textbook causal softmax attention in fp64 (library routine),
    (ii) row i equals the single-query function on the first off+i+1 keys (bit for bit: same arithmetic),
    (iii) the first query of an empty-past prompt returns the first value row exactly."""
    import torch
    B, S, Nq, Nkv, past, H = 2, 7, 4, 2, 5, 16
    L = past + S
    g = torch.Generator().manual_seed(8)
    q = torch.randn(B, S, Nq, H, generator=g).to(torch.bfloat16)
    k = torch.randn(B, Nkv, L, H, generator=g).to(torch.bfloat16)
    v = torch.randn(B, Nkv, L, H, generator=g).to(torch.bfloat16)
    bits = lambda t: t.contiguous().view(torch.int16).numpy().view(np.uint16)
    got = O.bf16_to_f32(O.attn_prefill(bits(q), bits(k), bits(v), None, round_probs=False))
    kk, vv = k.double().repeat_interleave(2, 1), v.double().repeat_interleave(2, 1)
    s = torch.einsum("bsnh,bnlh->bnsl", q.double(), kk) / np.sqrt(H)
    causal = torch.arange(L)[None, :] > (past + torch.arange(S))[:, None]
    s = s.masked_fill(causal[None, None], float("-inf"))
    ref = torch.einsum("bnsl,bnlh->bsnh", torch.softmax(s, -1), vv).numpy()
    assert np.abs(got - ref).max() <= 2.0 ** -8 * np.abs(ref).max() + 1e-6
    m = np.zeros((B, L), np.float32); m[0, :3] = -10000.0
    full = O.attn_prefill(bits(q), bits(k), bits(v), m)
    for i in range(S):
        n_keys = past + i + 1
        one = O.attn_decode(bits(q[:, i]), bits(k[:, :, :n_keys]), bits(v[:, :, :n_keys]), m)
        assert np.array_equal(full[:, i], one), i
    first = O.bf16_to_f32(O.attn_prefill(bits(q), bits(k[:, :, :S]), bits(v[:, :, :S])))
    assert np.array_equal(first[:, 0], v[:, :, 0].float().repeat_interleave(2, 1).numpy())


def test_oracle_linear_bf16_against_mxfp4_restatement_and_closed_forms():
    """The bf16-weight linear is pinned three ways: (1) on weights MXFP4 represents exactly it must give what the
    MXFP4 restatement gives on their quantized form (same sums, one rounding each; a transposed operand, a missing
    bias or a second rounding breaks it); (2) small-integer operands make every product and sum exact, so the result
    is the integer matrix product; (3) the post-op is the shared one."""
    rng = np.random.default_rng(5)
    M, N, K = 7, 64, 256
    W = randn_bf16((N, K), 0.02, 41)
    q, sc = O.remap_quantize_mxfp4(W.float().numpy())
    Wd = torch.from_numpy(O.dequantize_mxfp4_plain(q, sc)).to(torch.bfloat16)
    assert torch.equal(Wd.float(), torch.from_numpy(O.dequantize_mxfp4_plain(q, sc)))  # exactly representable
    x = randn_bf16((M, K), 1.0, 42)
    bias = randn_bf16((N,), 0.01, 43)
    res = randn_bf16((M, N), 1.0, 44)
    for post, kw in ((O.POST_NONE, {}), (O.POST_ADD_SCALE, dict(post_in=t2bits(res), post_scale=0.5)), (O.POST_SILU, {})):
        a = O.linear_bf16(t2bits(x), t2bits(Wd), t2bits(bias), post, **kw)
        b = O.linear_mxfp4(t2bits(x), q, sc, t2bits(bias), post, mode=O.MODE_F64, **kw)
        assert np.array_equal(a, b), post
    xi = torch.from_numpy(rng.integers(-4, 5, (M, K)).astype(np.float32)).to(torch.bfloat16)
    wi = torch.from_numpy(rng.integers(-3, 4, (N, K)).astype(np.float32)).to(torch.bfloat16)
    want = (xi.double() @ wi.double().T)  # |sum| <= 256 * 12: exact in fp32, not always in bf16
    got = bits2f(O.linear_bf16(t2bits(xi), t2bits(wi)))
    assert np.array_equal(got, want.float().to(torch.bfloat16).float().numpy())


def test_oracle_mxfp8_activation_quantizer_known_answers():
    """OCP E4M3 / MX block scale: known codes (1.0 = 0x38, 448 = 0x7E = the largest finite, saturation above it,
    2^-9 = the smallest subnormal, ties to even on both sides of the normal boundary), decode(encode) over all 254
    finite codes, and the block rule on hand-made blocks (max 1.0 -> scale 2^-8, so 1.0 is stored as 256 = 0x78)."""
    c = np.arange(256, dtype=np.uint8)
    fin = c[(c & 0x7F) != 0x7F]
    assert np.array_equal(O.e4m3_encode(O.e4m3_decode(fin)), fin)
    assert O.e4m3_decode([0x7E])[0] == 448.0 and O.e4m3_decode([0x01])[0] == 2.0 ** -9 and O.e4m3_decode([0x08])[0] == 2.0 ** -6
    vals = [1.0, 448, 500, 2 ** -9, 2 ** -10, 3 * 2 ** -10, 1.0625, 1.1875, -1.0, 0.9 * 2 ** -6, 17.0, 19.0]
    want = [0x38, 0x7E, 0x7E, 0x01, 0x00, 0x02, 0x38, 0x3A, 0xB8, 0x07, 0x58, 0x5A]  # 17 -> 16 (tie, even), 19 -> 20
    assert O.e4m3_encode(vals).tolist() == want
    x = np.zeros((1, 64), np.float32)
    x[0, :4] = [1.0, -0.5, 0.75, 2.0 ** -12]          # block 0: max 1.0
    x[0, 32:36] = [1.9, 0.001, -1.9, 100.0 * 2 ** -8]  # block 1: max 1.9 (bf16 1.8984375): 1.898 * 256 = 486 saturates
    xb = t2bits(torch.from_numpy(x).to(torch.bfloat16))
    codes, sc = O.quant_act_mxfp8(xb)
    assert sc.tolist() == [[119, 119]]
    assert codes[0, :4].tolist() == [0x78, 0xF0, 0x74, 0x18]  # 256, -128, 192, 2^-12 * 256 = 2^-4
    assert codes[0, 32] == 0x7E and codes[0, 34] == 0xFE and codes[0, 35] == O.e4m3_encode([100.0])[0]
    d = O.dequant_act_mxfp8(codes, sc)
    assert d[0, 0] == 1.0 and d[0, 1] == -0.5 and d[0, 32] == 448.0 / 256


def test_oracle_linear_qint8_f32_against_bf16_path_and_fp64():
    """orc_linear_qint8_f32 (pre-quantized activations, everything after the integer sums in fp32):
    * on bf16 activations and a bf16 bias, rounding its result to bf16 gives orc_linear_qint8 (mode ideal) bit for bit
      (the same multiply-add chain, rounded once at the end);
    * against the formula in fp64 from independently formed integer block sums (relative error of an fp32 chain);
    * float activations quantize from their own values: the scale of a block is max|x| / 127 of the fp32 values."""
    rng = np.random.default_rng(21)
    M, N, K = 5, 48, 768
    W = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    q, sw, qbs = O.remap_quantize_qint8(W)
    x = randn_bf16((M, K), 1.0, 22)
    bias = randn_bf16((N,), 0.1, 23)
    xq, sa = O.quantize_int8sym(x.float().numpy(), qbs, -1, False)
    y32 = O.linear_qint8_f32(xq, sa, q, sw, bias.float().numpy())
    ybf = O.linear_qint8(t2bits(x), q, sw, t2bits(bias), O.POST_NONE, None, None, 1.0, O.MODE_IDEAL)
    assert np.array_equal(t2bits(torch.from_numpy(y32).to(torch.bfloat16)), ybf)
    # fp64 formula, weight un-blocked by hand: element [n1][b][a][k2][v] = Wq[n1*16 + k2][b*qbs + a*4 + v]
    Wq = q.transpose(0, 3, 1, 2, 4).reshape(N, K).astype(np.int64)
    swn = sw.reshape(N // 16, K // qbs, 16).transpose(0, 2, 1).reshape(N, K // qbs).astype(np.float64)
    isum = np.einsum("mbk,nbk->mnb", xq.astype(np.int64).reshape(M, K // qbs, qbs), Wq.reshape(N, K // qbs, qbs))
    ref = (isum * sa.astype(np.float64)[:, None, :] * swn[None, :, :]).sum(-1) + bias.float().numpy().astype(np.float64)
    assert np.abs(y32 - ref).max() <= 1e-5 * np.abs(ref).max()
    # fp32 activations that bf16 cannot hold
    xf = (rng.standard_normal((M, K)) * 3.0).astype(np.float32)
    xq2, sa2 = O.quantize_int8sym(xf, qbs, -1, False)
    amax = np.abs(xf.reshape(M, K // qbs, qbs)).max(-1)
    assert np.array_equal(sa2, (amax.astype(np.float64) / 127.0).astype(np.float32))
    assert np.abs(xq2).max() == 127 and np.abs(xq2.astype(np.float64) * np.repeat(sa2, qbs, 1) - xf).max() <= sa2.max() * 0.5 * 1.0001


def test_oracle_w4a8_layout_table_and_linear():
    """The W4A8 restatement (USE_MXFP4_INT8):
    * layout: the one-step index map equals the reference's sequence of views and permutes, for source channel
      blocks below, at and above 8, and each element sits where the documented formula says;
    * packed bytes: byte j of a group holds K value j in its low and K value 4 + j in its high nibble, and the
      codes / scales are those of the default-layout MXFP4 quantizer on the same weight (same 32-value blocks);
    * integer table: |w_i * 6/127 - e2m1| <= 0.5 * 6/127 for all 16 codes, sign symmetric, exact at 0 and 6;
    * linear: equals an fp64 evaluation of its formula within fp32 chain error, and the exact-MXFP4 product on the
      dequantized activations within the table's rounding (0.5/127 of full scale per weight)."""
    rng = np.random.default_rng(31)
    for N, K, bk, bc in [(32, 128, 16, 64), (64, 256, 32, 64), (16, 64, 8, 32), (64, 128, 64, 128), (32, 64, 4, 64)]:
        W = rng.standard_normal((N, K)).astype(np.float32)
        t = W.reshape(N // bk, bk, K // bc, bc // 2, 2).transpose(0, 2, 3, 1, 4).copy()
        if bk >= 8:
            a = O.mxfp4_int8_layout(t)
            assert np.array_equal(a, O.mxfp4_int8_layout_chain(t))
        else:
            a = O.mxfp4_int8_layout_chain(t)
        nb, c1, g, n8, j = N // 8 - 1, K // bc - 1, bc // 8 - 1, 5, 3
        assert a[nb, c1, g, n8, j] == W[nb * 8 + n8, c1 * bc + g * 8 + (j % 2) * 4 + j // 2]
    N, K, bk, bc = 64, 256, 16, 64
    W = (rng.standard_normal((N, K)) * 0.05).astype(np.float32)
    t = W.reshape(N // bk, bk, K // bc, bc // 2, 2).transpose(0, 2, 3, 1, 4).copy()
    q, sc = O.remap_quantize_mxfp4_int8(t)
    assert q.shape == (N // 8, K // bc, bc // 8, 8, 4) and sc.shape == (N // 8, K // bc, bc // 32, 8)
    q0, sc0 = O.remap_quantize_mxfp4(W)            # default layout [N/32][K/64][32][32] + [N/32][K/64][2][32]
    Wd = O.dequantize_mxfp4_plain(q0, sc0)
    codes = np.stack([q & 15, q >> 4], axis=-1)    # [..][n8][j][lo/hi] -> K value j + 4*hi
    e2m1 = np.array([O.lib().orc_e2m1_decode(c) for c in range(16)], np.float32)
    vals = e2m1[codes].transpose(0, 3, 1, 2, 5, 4).reshape(N, K // bc, bc // 8, 8)  # [n][c1][g][k = hi*4 + j]
    scale = np.array([O.lib().orc_mx_dequant_scale(int(b)) for b in range(256)], np.float32)[sc]  # [nb][c1][sb][n8]
    scale = np.repeat(scale.transpose(0, 3, 1, 2).reshape(N, K // 32), 32, axis=1)
    assert np.array_equal(vals.reshape(N, K) * scale, Wd)
    tbl = np.array([O.lib().orc_w4a8_weight_int(c) for c in range(16)], np.float64)
    assert np.abs(tbl * 6.0 / 127.0 - e2m1.astype(np.float64)).max() <= 0.5 * 6.0 / 127.0 + 1e-12
    assert np.array_equal(tbl[8:], -tbl[:8]) and tbl[0] == 0 and tbl[7] == 127
    # linear
    M = 7
    x = randn_bf16((M, K), 1.0, 32)
    bias = randn_bf16((N,), 0.1, 33)
    y = bits2f(O.linear_w4a8(t2bits(x), q, sc, bc, t2bits(bias))).astype(np.float64)
    xq, sa = O.quantize_act_w4a8(x.float().numpy())
    wi = tbl[np.stack([q & 15, q >> 4], axis=-1)].transpose(0, 3, 1, 2, 5, 4).reshape(N, K)
    isum = np.einsum("mbk,nbk->mnb", xq.astype(np.float64).reshape(M, K // 32, 32), wi.reshape(N, K // 32, 32))
    wsc = scale[:, ::32].astype(np.float64)
    ref = (isum * sa.astype(np.float64)[:, None, :] * wsc[None, :, :]).sum(-1) + bias.float().numpy().astype(np.float64)
    assert np.abs(y - ref).max() <= 2.0 ** -8 * np.abs(ref).max()
    exact = (xq.astype(np.float64) * np.repeat(sa / O.W4A8_ACT_SCALE, 32, axis=1)) @ Wd.astype(np.float64).T \
        + bias.float().numpy().astype(np.float64)
    assert np.sqrt(((ref - exact) ** 2).sum() / (exact ** 2).sum()) <= 1.5e-2


def test_wide_activation_linears_pinned_on_bf16_inputs():
    """linear_mxfp4_wide / linear_bf16_wide (float / half activations, fp64 dot product) against the pinned bf16
    restatements: on activations that ARE bf16 values the float tile, rounded to bf16, is the ideal-mode tile of
    linear_mxfp4 / linear_bf16 except where the fp32 summation order crosses a rounding boundary (a few elements per
    thousand at K = 512, one bf16 ulp each); the post-ops on float match the bf16 ones within bf16 resolution."""
    rng = np.random.default_rng(5)
    M, N, K = 24, 64, 512
    W = (rng.standard_normal((N, K)) * 0.05).astype(np.float32)
    wb = O.f32_to_bf16(W)
    xb = O.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    xf = O.bf16_to_f32(xb)
    bias_b = O.f32_to_bf16((rng.standard_normal(N) * 0.1).astype(np.float32))
    q, sc = O.remap_quantize_mxfp4(O.bf16_to_f32(wb))
    for wide, narrow in ((O.linear_mxfp4_wide(xf, q, sc, O.bf16_to_f32(bias_b)), O.linear_mxfp4(xb, q, sc, bias_b)),
                         (O.linear_bf16_wide(xf, wb, O.bf16_to_f32(bias_b)), O.linear_bf16(xb, wb, bias_b))):
        assert wide.dtype == np.float32
        as_bf16 = O.f32_to_bf16(wide)
        diff = as_bf16 != narrow
        assert diff.mean() <= 5e-3
        assert np.abs(O.bf16_to_f32(as_bf16) - O.bf16_to_f32(narrow)).max() <= 2.0 ** -7 * np.abs(O.bf16_to_f32(narrow)).max()
    # half: one rounding of the same exact sum
    xh = xf.astype(np.float16)
    wide_h = O.linear_mxfp4_wide(xh, q, sc, None)
    exact = xh.astype(np.float64) @ O.dequantize_mxfp4_plain(q, sc).astype(np.float64).T
    assert wide_h.dtype == np.float16 and np.array_equal(wide_h, exact.astype(np.float32).astype(np.float16))
    # post-ops on float: the textbook formulas
    y = (rng.standard_normal((M, N))).astype(np.float32)
    a = (rng.standard_normal((M, N))).astype(np.float32)
    b = (rng.standard_normal((M, N))).astype(np.float32)
    assert np.allclose(O.post_op_wide(y, O.POST_SILU), y / (1 + np.exp(-y.astype(np.float64))), rtol=1e-6, atol=1e-7)
    assert np.array_equal(O.post_op_wide(y, O.POST_MUL, a), a * y)
    assert np.allclose(O.post_op_wide(y, O.POST_ADD_SCALE, a, None, 0.25), y + 0.25 * a.astype(np.float64), rtol=1e-7, atol=1e-7)
    assert np.allclose(O.post_op_wide(y, O.POST_ADD2_SCALE, a, b, 0.25), y.astype(np.float64) + a + 0.25 * b, rtol=1e-6, atol=1e-6)
    assert np.array_equal(O.post_op_wide(y, O.POST_RELU), np.maximum(y, 0))
    import math
    assert np.allclose(O.post_op_wide(y[:2], O.POST_GELU), [[0.5 * v * (1 + math.erf(v / math.sqrt(2))) for v in r] for r in y[:2]], rtol=1e-6, atol=1e-7)
    # half post-ops store half after every step
    yh, ah = y.astype(np.float16), a.astype(np.float16)
    assert np.array_equal(O.post_op_wide(yh, O.POST_MUL, ah), (ah.astype(np.float32) * yh.astype(np.float32)).astype(np.float16))


def test_w4a8_integer_table_is_bounded_the_reference_table_is_unreadable_here():
    """The integers the reference multiplies for MXFP4 weights in the W4A8 mode (USE_MXFP4_INT8,
    src/csrc/fused_gemm.h:965-978) come out of its JIT library, whose sources are not in the tree: the table cannot be
    read here, so it is restated as round-to-nearest of E2M1 x 127/6 and BOUNDED instead of pinned -- for every one of
    the 16 codes table[c] x 6/127 lies within half an int8 step (0.5 x 6/127) of the E2M1 value, the table is odd,
    monotone in the code's magnitude, exact at 0 and at the format's maximum 6 (= 127), and no other integer is closer
    to any code.  Parity of this one table stays unpinned."""
    e2m1 = np.array([O.lib().orc_e2m1_decode(c) for c in range(16)], np.float64)
    tbl = np.array([O.lib().orc_w4a8_weight_int(c) for c in range(16)], np.float64)
    step = 6.0 / 127.0
    assert np.abs(tbl * step - e2m1).max() <= 0.5 * step + 1e-12
    assert np.array_equal(tbl[8:], -tbl[:8]) and tbl[0] == 0 and tbl[7] == 127 and tbl[15] == -127
    assert np.all(np.diff(tbl[:8]) > 0) and np.all(np.abs(tbl) <= 127) and np.array_equal(tbl, np.rint(tbl))
    for c in range(16):
        for other in (tbl[c] - 1, tbl[c] + 1):
            assert abs(other * step - e2m1[c]) >= abs(tbl[c] * step - e2m1[c])
