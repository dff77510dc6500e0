"""The helper set on arbitrary layouts and the low-bit affine weight formats.

* quantize_mxfp4 / quantize_int8sym / quantize_int4sym(t, block_size, axis, is_vnni) on layouts other than the two
  linear-layer weight layouts, and dequantize() of every such tensor (quantized activations included): bytes, scales
  and fp32 values equal the oracle's generic per-block functions (PerBlockQuantizer, src/csrc/qtypes.h:30-243).
* remap_and_quantize_qint2_intlv (src/csrc/qtypes.cpp:1004-1073, the "qint2" choice of FixLinear): packed bytes and
  scales equal the oracle (itself pinned against a restatement of the reference's view / permute / pack chain), and
  the W2A8 linear on it equals the W8A8 oracle on the ternary weight (exact int32 block sums, same scales).
* quantize_int4sym on the VNNI2 weight layout feeds the linears the same way.
"""
import numpy as np
import pytest
import torch

import oracle as O
from util import t2bits, randn_bf16, block_bf16, assert_close_bf16

pytestmark = pytest.mark.gpu


def _ops():
    import tpp_pytorch_extension  # noqa: F401
    from tpp_pytorch_extension import _ops
    return _ops


GEOMS = [
    # shape, block_size, axis, is_vnni
    ((6, 96), 32, -1, False),            # plain rows, blocks along the last axis
    ((3, 5, 128), 64, 2, False),
    ((4, 2, 16, 8, 2), 32, 2, True),     # VNNI2 weight-like with 8-channel blocks
    ((2, 3, 64, 10, 4), 128, 2, True),   # VNNI4, odd channel count
    ((2, 64, 3, 2), 64, 1, True),        # blocks along axis 1, two trailing dims
]


@pytest.mark.parametrize("shape,bs,axis,vnni", GEOMS)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("fmt", ["mxfp4", "int8", "int4"])
def test_generic_quantize_and_dequantize(shape, bs, axis, vnni, dtype, fmt):
    ops = _ops()
    g = torch.Generator().manual_seed(hash((shape, bs, fmt)) % 1000)
    t = (torch.randn(shape, generator=g) * 0.7).to(dtype)
    t.view(-1)[::17] = 0.0
    t.view(-1)[3] = 5.0
    ref_in = t.float().numpy()
    if fmt == "mxfp4":
        qt = ops.quantize_mxfp4(t.cuda(), bs, axis, vnni)
        q_or, s_or = O.quantize_mxfp4(ref_in, bs, axis, vnni)
        d_or = O.dequantize_mxfp4(q_or, s_or, bs, axis, vnni)
        assert qt.dtype == torch.quint4x2 and ops.q_per_block_pack_size(qt) == 2
    elif fmt == "int8":
        qt = ops.quantize_int8sym(t.cuda(), bs, axis, vnni)
        q_or, s_or = O.quantize_int8sym(ref_in, bs, axis, vnni)
        d_or = O.dequantize_int8sym(q_or, s_or, bs, axis, vnni)
        assert qt.dtype == torch.qint8 and ops.q_per_block_pack_size(qt) == 1
    else:
        qt = ops.quantize_int4sym(t.cuda(), bs, axis, vnni)
        q_or, s_or = O.quantize_int4sym(ref_in, bs, axis, vnni)
        d_or = O.dequantize_int4sym(q_or, s_or, bs, axis, vnni)
        assert qt.dtype == torch.quint4x2
    assert qt.is_quantized and tuple(qt.shape) == tuple(shape)
    assert ops.q_per_block_block_size(qt) == bs and ops.q_per_block_axis(qt) == (axis % len(shape))
    assert np.array_equal(ops.q_per_block_scales(qt).cpu().numpy().reshape(s_or.shape), s_or)
    assert np.array_equal(qt.qdata.cpu().numpy().reshape(q_or.shape), q_or)
    d = qt.dequantize()
    assert d.dtype == torch.float32 and tuple(d.shape) == tuple(shape)
    assert np.array_equal(d.cpu().numpy().view(np.uint32), d_or.view(np.uint32))


def test_activation_qtensor_dequantizes():
    """quantize_int8sym(x, QBS, -1, False) on bf16 activations (the call the W8A8 linear makes, fused_gemm.h:1249)
    gives a tensor whose dequantize() is q * scale per (row, block)."""
    ops = _ops()
    x = randn_bf16((3, 7, 512), 1.0, 77)
    qt = ops.quantize_int8sym(x.cuda(), 256, -1, False)
    xq, sa = O.quant_act_int8(t2bits(x).reshape(21, 512), 256)
    assert np.array_equal(qt.qdata.cpu().numpy().reshape(21, 512), xq)
    want = O.dequantize_int8sym(xq, sa, 256, 1, False)
    assert np.array_equal(qt.dequantize().cpu().numpy().reshape(21, 512), want)


@pytest.mark.parametrize("N,K", [(64, 256), (4096, 1024), (96, 11008)])
@pytest.mark.parametrize("src", ["bf16_5d", "f32_4d"])
def test_qint2_quantizer_bit_exact(N, K, src):
    ops = _ops()
    W = randn_bf16((N, K), 0.02, 31 + N)
    W[5, :128] = 0.0
    W[7] = 0.0          # an all-zero (channel, block): scale clamps to 1e-8, codes 0
    W[9, 3] = 0.5 * W[9, :256].abs().max()  # an exact tie at 0.5: rounds to even (0)
    if src == "bf16_5d":
        qt = ops.remap_and_quantize_qint2_intlv(block_bf16(W).cuda())
    else:
        Wf = W.float()
        qt = ops.remap_and_quantize_qint2_intlv(Wf.view(N // 16, 16, K // 64, 64).permute(0, 2, 3, 1).contiguous().cuda())
    q_or, s_or, bs = O.remap_quantize_qint2_intlv(W.float().numpy())
    assert ops.q_per_block_block_size(qt) == bs and qt.dtype == torch.quint2x4 and ops.q_per_block_pack_size(qt) == 4
    assert tuple(qt.shape) == (N // 32, K // bs, bs // 4, 32, 4)
    assert np.array_equal(qt.scales.cpu().numpy(), s_or)
    assert np.array_equal(qt.qdata.cpu().numpy(), q_or)
    # dequantize = ternary value * scale in the logical blocked shape
    v8, s8 = O.qint2_to_qint8_layout(q_or, s_or)
    Wd = O.dequantize_qint8_plain(v8, s8)                                    # plain [N][K]
    want = Wd.reshape(N // 32, 32, K // bs, bs // 4, 4).transpose(0, 2, 3, 1, 4)
    assert np.array_equal(qt.dequantize().cpu().numpy(), want)


@pytest.mark.parametrize("M", [1, 8, 40, 200])
def test_qint2_linear(M):
    """W2A8: int8 activations per 256-block x ternary weights, exact int32 block sums, fp32 scales -- the W8A8
    oracle on the expanded weight.  fc_add through the module API (FixLinear weight_dtype="qint2")."""
    ops = _ops()
    from tpp_pytorch_extension.llm.llm_common import FixLinear, BlockedLinear
    N, K = 1024, 2048
    torch.manual_seed(5)
    lin = torch.nn.Linear(K, N, bias=True)
    W = lin.weight.data.clone().to(torch.bfloat16)
    b = lin.bias.data.clone().to(torch.bfloat16)
    FixLinear(lin, 16, 64, torch.bfloat16, weight_dtype="qint2")
    assert isinstance(lin, BlockedLinear) and lin.weight.is_quantized and lin.weight.dtype == torch.quint2x4
    q_or, s_or, bs = O.remap_quantize_qint2_intlv(W.float().numpy())
    assert np.array_equal(lin.weight.qdata.cpu().numpy(), q_or)
    v8, s8 = O.qint2_to_qint8_layout(q_or, s_or)
    x = randn_bf16((M, K), 1.0, 41)
    r = randn_bf16((M, N), 1.0, 42)
    y = torch.ops.tpp_llm.fc_add(x.cuda(), lin.weight, b.cuda(), r.cuda(), 1.0)
    ref = O.linear_qint8(t2bits(x), v8, s8, t2bits(b), O.POST_ADD_SCALE, t2bits(r), None, 1.0)
    assert_close_bf16(t2bits(y), ref, what=f"qint2 fc_add M={M}", pre_bits=O.linear_qint8(t2bits(x), v8, s8, t2bits(b)))
    y2 = lin.cuda()(x.cuda())
    assert_close_bf16(t2bits(y2), O.linear_qint8(t2bits(x), v8, s8, t2bits(b)), what=f"qint2 module M={M}")


@pytest.mark.parametrize("M", [3, 64, 130])
def test_qint4_vnni2_weight_linear(M):
    """quantize_int4sym on a weight in the VNNI2 layout [N/16, K/QBS, QBS/2, 16, 2] gives a tensor the linears accept
    (kQUInt4x2 + per-block affine -> TppBlockedQInt8LinearW, fused_gemm.h:1530-1534): W4A8 with exact int32 sums."""
    ops = _ops()
    N, K, qbs = 512, 1024, 256
    W = randn_bf16((N, K), 0.02, 51)
    t = W.view(N // 16, 16, K // qbs, qbs // 2, 2).permute(0, 2, 3, 1, 4).contiguous()
    qt = ops.quantize_int4sym(t.cuda(), qbs, 2, True)
    q_or, s_or = O.quantize_int4sym(t.float().numpy(), qbs, 2, True)
    assert np.array_equal(qt.qdata.cpu().numpy().reshape(q_or.shape), q_or) and np.array_equal(qt.scales.cpu().numpy(), s_or)
    assert qt.is_weight()
    # the int8 weight with the same values, in the QINT8 reference layout
    codes = np.stack([q_or[..., 0] & 0xF, q_or[..., 0] >> 4], axis=-1).astype(np.int16)
    vals = np.where(codes >= 8, codes - 16, codes).astype(np.int8)            # [N/16][K/qbs][qbs/2][16][2]
    v8 = vals.reshape(N // 16, K // qbs, qbs // 4, 2, 16, 2).transpose(0, 1, 2, 4, 3, 5).reshape(N // 16, K // qbs, qbs // 4, 16, 4)
    x = randn_bf16((M, K), 1.0, 52)
    y = ops.fc_plain(x.cuda(), qt, None)
    ref = O.linear_qint8(t2bits(x), np.ascontiguousarray(v8), s_or)
    assert_close_bf16(t2bits(y), ref, what=f"qint4 fc_plain M={M}")


@pytest.mark.parametrize("M", [1, 5, 70])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_fc_plain_float_and_half_activations(M, dtype):
    """fc_plain's element-type switch (fused_llm_infer.cpp:1526-1545) on a QINT8 weight: float / half activations are
    quantized from their own values, the GEMM accumulates and adds the bias in fp32, the output has the activations'
    type.  Bit-exact against the oracle's fp32 chain (half: its single rounding to half)."""
    ops = _ops()
    N, K = 96, 1024
    W = randn_bf16((N, K), 0.02, 61)
    qw = ops.remap_and_quantize_qint8(block_bf16(W).cuda())
    q_or, s_or, qbs = O.remap_quantize_qint8(W.float().numpy())
    g = torch.Generator().manual_seed(62 + M)
    x = (torch.randn((M, K), generator=g) * 1.7).to(dtype)
    bias = (torch.randn((N,), generator=g) * 0.1).to(dtype)
    y = ops.fc_plain(x.cuda(), qw, bias.cuda())
    assert y.dtype == dtype and tuple(y.shape) == (M, N)
    xq, sa = O.quantize_int8sym(x.float().numpy(), qbs, -1, False)
    ref = torch.from_numpy(O.linear_qint8_f32(xq, sa, q_or, s_or, bias.float().numpy())).to(dtype)
    assert torch.equal(y.cpu(), ref)
    # leading dimensions are kept, no bias
    y3 = ops.fc_plain(x.cuda().view(1, M, K), qw, None)
    ref3 = torch.from_numpy(O.linear_qint8_f32(xq, sa, q_or, s_or, None)).to(dtype)
    assert tuple(y3.shape) == (1, M, N) and torch.equal(y3.cpu().view(M, N), ref3)
    # post-ops work on the output type (fused_gemm.h:1343-1488 with Tout = float / half)
    acc = torch.from_numpy(O.linear_qint8_f32(xq, sa, q_or, s_or, None)).to(dtype)
    res = (torch.randn((M, N), generator=g) * 0.5).to(dtype)
    for post, fn, args in ((O.POST_SILU, ops.fc_silu, ()), (O.POST_ADD_SCALE, ops.fc_add, (res.cuda(), 0.5)),
                           (O.POST_MUL, ops.fc_mul, (res.cuda(),))):
        got = fn(x.cuda(), qw, None, *args)
        want = O.post_op_wide(acc.numpy(), post, res.numpy(), None, 0.5)
        assert got.dtype == dtype
        tol = 2e-3 if dtype == torch.float16 else 2e-6
        assert np.allclose(got.cpu().float().numpy(), want.astype(np.float32), rtol=tol, atol=tol), post


@pytest.mark.parametrize("M", [1, 7, 70])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("wkind", ["mxfp4", "bf16"])
def test_float_and_half_activations_on_mxfp4_and_bf16_weights(M, dtype, wkind):
    """TppBlockedLinearW<Tin, uint8_t, Tout> / <Tin, bfloat16, Tout> with Tin = float or half
    (src/csrc/fused_gemm.h:1519-1523, 1541-1550): the activations keep their own precision (a bf16-rounded input would
    miss the bound below by two orders of magnitude), fp32 sums, output and post-ops in the activations' type.
    Against the oracle's exact (fp64) dot product: float within 4 fp32 ulps of sum |x||w| (the fp32 accumulation over
    K), half within one half ulp of it; then every post-op."""
    ops = _ops()
    N, K = 96, 1024
    W = randn_bf16((N, K), 0.05, 161)
    g = torch.Generator().manual_seed(162 + M)
    x = (torch.randn((M, K), generator=g) * 1.3).to(dtype)
    bias = (torch.randn((N,), generator=g) * 0.1).to(dtype)
    if wkind == "mxfp4":
        w = ops.remap_and_quantize_mxfp4(block_bf16(W).cuda())
        q_or, s_or = O.remap_quantize_mxfp4(W.float().numpy())
        Wd = O.dequantize_mxfp4_plain(q_or, s_or)
        lin = lambda *a: O.linear_mxfp4_wide(x.numpy(), q_or, s_or, *a)  # noqa: E731
    else:
        w = block_bf16(W).cuda()
        Wd = W.float().numpy()
        lin = lambda *a: O.linear_bf16_wide(x.numpy(), t2bits(W), *a)  # noqa: E731
    y = ops.fc_plain(x.cuda(), w, bias.cuda())
    assert y.dtype == dtype and tuple(y.shape) == (M, N)
    ref = lin(bias.numpy())
    mag = np.abs(x.float().numpy()).astype(np.float64) @ np.abs(Wd).astype(np.float64).T + np.abs(bias.float().numpy())
    d = np.abs(y.cpu().float().numpy().astype(np.float64) - ref.astype(np.float64))
    if dtype == torch.float32:
        assert (d <= 4 * 2.0 ** -23 * mag).all(), float((d / mag).max())
        # the input was NOT rounded to bf16 on the way in
        y_bf = ops.fc_plain(x.to(torch.bfloat16).float().cuda(), w, bias.cuda()).cpu().numpy().astype(np.float64)
        assert np.abs(y_bf - ref).max() > 50 * d.max()
    else:
        ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(ref.astype(np.float64)), 2.0 ** -14))) - 10)
        assert (d <= ulp + 4 * 2.0 ** -23 * mag).all()
        assert np.mean(y.cpu().numpy() != ref) <= 1e-2  # fp32 sums of 1024 products land across a half rounding boundary now and then
    # leading dimensions kept, no bias
    y3 = ops.fc_plain(x.cuda().view(1, M, K), w, None)
    assert tuple(y3.shape) == (1, M, N)
    # post-ops on the output type
    res = (torch.randn((M, N), generator=g) * 0.5).to(dtype)
    res2 = (torch.randn((M, N), generator=g) * 0.5).to(dtype)
    tol = 2e-3 if dtype == torch.float16 else 1e-5
    for post, call in ((O.POST_SILU, lambda: ops.fc_silu(x.cuda(), w, bias.cuda())),
                       (O.POST_MUL, lambda: ops.fc_mul(x.cuda(), w, bias.cuda(), res.cuda())),
                       (O.POST_ADD_SCALE, lambda: ops.fc_add(x.cuda(), w, bias.cuda(), res.cuda(), 0.5)),
                       (O.POST_ADD2_SCALE, lambda: ops.fc_add2(x.cuda(), w, bias.cuda(), res.cuda(), res2.cuda(), 0.5)),
                       (O.POST_GELU, lambda: ops.fc_gelu(x.cuda(), w, bias.cuda())),
                       (O.POST_RELU, lambda: ops.fc_relu(x.cuda(), w, bias.cuda()))):
        got = call()
        want = lin(bias.numpy(), post, res.numpy(), res2.numpy(), 0.5)
        assert got.dtype == dtype
        assert np.allclose(got.cpu().float().numpy(), want.astype(np.float32), rtol=tol, atol=tol * 4), post


@pytest.mark.parametrize("M", [3, 40])
def test_fc_plain_prequantized_input(M):
    """A qint8 activation tensor (quantize_int8sym over the last axis with the weight's block size) is used as it is
    (fused_gemm.h:1244-1246); the compute type is the bias's, float without one (fused_llm_infer.cpp:1529-1535)."""
    ops = _ops()
    N, K = 64, 768
    W = randn_bf16((N, K), 0.02, 71)
    qw = ops.remap_and_quantize_qint8(block_bf16(W).cuda())
    q_or, s_or, qbs = O.remap_quantize_qint8(W.float().numpy())
    x = randn_bf16((M, K), 1.0, 72)
    bias = randn_bf16((N,), 0.1, 73)
    xq = ops.quantize_int8sym(x.cuda(), qbs, -1, False)
    # bfloat16 bias: the bf16 kernels on the caller's quantized rows = the call that quantizes by itself
    yb = ops.fc_plain(xq, qw, bias.cuda())
    assert yb.dtype == torch.bfloat16 and torch.equal(yb, ops.fc_plain(x.cuda(), qw, bias.cuda()))
    # no bias: float
    yf = ops.fc_plain(xq, qw, None)
    xq_or, sa_or = O.quantize_int8sym(x.float().numpy(), qbs, -1, False)
    assert yf.dtype == torch.float32
    assert np.array_equal(yf.cpu().numpy(), O.linear_qint8_f32(xq_or, sa_or, q_or, s_or, None))
    # float bias: float
    yfb = ops.fc_plain(xq, qw, bias.float().cuda())
    assert np.array_equal(yfb.cpu().numpy(), O.linear_qint8_f32(xq_or, sa_or, q_or, s_or, bias.float().numpy()))
    from tpp_pytorch_extension._lib import TppxError
    with pytest.raises(TppxError):  # quantized with another block size
        ops.fc_plain(ops.quantize_int8sym(x.cuda(), 64, -1, False), qw, None)


@pytest.mark.parametrize("bk,bc", [(16, 64), (32, 64), (64, 128)])
def test_w4a8_layout_and_quantizer(bk, bc):
    """remap_and_quantize_mxfp4(t, int8_layout=True) = the reference's USE_MXFP4_INT8 branch: packed bytes and E8M0
    scales equal the oracle's (whose layout is pinned against the reference's view / permute chain)."""
    ops = _ops()
    N, K = 128, 256
    W = randn_bf16((N, K), 0.05, 81)
    t = W.view(N // bk, bk, K // bc, bc // 2, 2).permute(0, 2, 3, 1, 4).contiguous()
    qt = ops.remap_and_quantize_mxfp4(t.cuda(), int8_layout=True)
    q_or, s_or = O.remap_quantize_mxfp4_int8(t.float().numpy())
    assert tuple(qt.shape) == (N // 8, K // bc, bc // 8, 8, 8) and qt.weight_kind() == "mxfp4_int8"
    assert qt.weight_nk() == (N, K)
    assert np.array_equal(qt.qdata.cpu().numpy().reshape(q_or.shape), q_or)
    assert np.array_equal(qt.scales.cpu().numpy().reshape(s_or.shape), s_or)
    # dequantize() gives the fp32 values in the blocked shape (the generic per-block path)
    d = qt.dequantize().cpu().numpy()
    v = O.mxfp4_int8_layout(t.float().numpy())
    assert d.shape == v.shape and np.abs(d - v).max() <= 0.25 * np.abs(v).max()


@pytest.mark.parametrize("M", [1, 16, 70])
@pytest.mark.parametrize("post", ["none", "silu", "add"])
def test_w4a8_linear(M, post):
    """The W4A8 GEMM (int8 activations over blocks of 32, scales times 6/127, MXFP4 weights as integers, K = 32
    int8 MFMA) against the oracle's restatement: same integer sums, same fp32 chain -> bf16 equality up to the
    post-op's tolerance."""
    ops = _ops()
    N, K, bk, bc = 96, 512, 16, 64
    W = randn_bf16((N, K), 0.05, 82)
    t = W.view(N // bk, bk, K // bc, bc // 2, 2).permute(0, 2, 3, 1, 4).contiguous()
    qt = ops.remap_and_quantize_mxfp4(t.cuda(), int8_layout=True)
    q_or, s_or = O.remap_quantize_mxfp4_int8(t.float().numpy())
    x = randn_bf16((M, K), 1.0, 83 + M)
    bias = randn_bf16((N,), 0.1, 84)
    in1 = randn_bf16((M, N), 1.0, 85)
    POSTS = {"none": O.POST_NONE, "silu": O.POST_SILU, "add": O.POST_ADD_SCALE}
    y = ops.linear(x.cuda(), qt, bias.cuda(), POSTS[post], in1.cuda() if post == "add" else None, None, 0.5)
    ref = O.linear_w4a8(t2bits(x), q_or, s_or, bc, t2bits(bias), POSTS[post], t2bits(in1) if post == "add" else None,
                        None, 0.5)
    assert_close_bf16(t2bits(y), ref, ulps=2 if post == "silu" else 1, what=f"w4a8 M={M} post={post}")
    if post == "none":
        # and close to the exact MXFP4 GEMM on bf16 activations (two quantization errors apart)
        exact = ops.linear(x.cuda(), ops.remap_and_quantize_mxfp4(block_bf16(W).cuda(), int8_layout=False), bias.cuda())
        a, b = y.double(), exact.double()
        assert float((a - b).norm() / b.norm()) <= 3e-2
        # the group operators fall back to one GEMM per weight
        q1, q2 = ops.qkv_gemm(x.cuda(), [qt, qt], [bias.cuda(), None])
        assert torch.equal(q1, y) and torch.equal(q2, ops.linear(x.cuda(), qt, None))
        sw = ops.swiglu_gate_up(x.cuda(), qt, qt)
        assert torch.equal(sw, ops.fc_mul(x.cuda(), qt, None, ops.fc_silu(x.cuda(), qt, None)))


@pytest.mark.parametrize("kind", ["qint4", "qint2"])
@pytest.mark.parametrize("M", [100, 130])
def test_packed_code_kernel_block_rows(kind, M):
    """tppx_linear_qintx beyond 64 rows (the Python op keeps such calls on the expanded tiles): block rows of 64 on the
    grid's second axis, the last one ragged; against the op on the expanded int8 tiles (another kernel family, so
    another fp32 summation order: one ulp, plus the pre-op tile's ulp through the residual add)."""
    ops = _ops()
    from tpp_pytorch_extension import _lib
    N, K = 1056 if kind == "qint4" else 1088, 2048
    W = randn_bf16((N, K), 0.02, 2800 + M)
    if kind == "qint4":
        qt = ops.quantize_int4sym(W.view(N // 16, 16, K // 256, 128, 2).permute(0, 2, 3, 1, 4).contiguous().cuda(), 256, 2, True)
    else:
        qt = ops.remap_and_quantize_qint2_intlv(block_bf16(W).cuda())
    x = randn_bf16((M, K), 1.0, 2810 + M).cuda()
    r = randn_bf16((M, N), 1.0, 2830).cuda()
    packed, sn, bits = qt.native_packed()
    xq, sa = ops._qint8_scratch(x, M, K, 256)
    y = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    _lib.check(_lib.lib().tppx_linear_qintx(x.data_ptr(), xq.data_ptr(), sa.data_ptr(), packed.data_ptr(), sn.data_ptr(), None,
                                            r.data_ptr(), None, y.data_ptr(), M, N, K, bits, O.POST_ADD_SCALE, 1.0, 0,
                                            _lib.stream_of(x)))
    assert M > 64  # the op itself does not take the packed kernel here
    ref = ops.linear(x, qt, None, O.POST_ADD_SCALE, r, None, 1.0)
    pre = ops.linear(x, qt, None)
    assert_close_bf16(t2bits(y), t2bits(ref), what=f"{kind} packed block rows M={M}", pre_bits=t2bits(pre))


@pytest.mark.parametrize("M,N,K,bc,post", [(64, 96, 512, 64, "none"), (200, 272, 1024, 128, "add"), (129, 128, 256, 32, "silu"),
                                           (300, 1040, 1280, 64, "mul"), (257, 16, 128, 32, "add2"), (640, 512, 2048, 64, "relu")])
def test_w4a8_wide_kernel(M, N, K, bc, post, monkeypatch):
    """W4A8 passes of many rows (tppx_linear_mxfp4_int8_wide): the int8 rows and the weight integers times their
    block's power of two as bf16 MFMA operands, one K = 32 MFMA per MX block, one fp32 multiply-add with
    sa[row][block] per output and block in ascending order from the bias -- the oracle's loop
    (src/csrc/fused_gemm.h:965-978 restated) term for term, so the GEMM result is EQUAL to the oracle's, bit for
    bit; post-ops keep their usual bound.  Ragged row and channel counts, blocks of all-zero rows, every post-op
    family, and the row threshold that picks the kernel."""
    ops = _ops()
    from tpp_pytorch_extension import _lib
    posts = {"none": O.POST_NONE, "add": O.POST_ADD_SCALE, "silu": O.POST_SILU, "mul": O.POST_MUL,
             "add2": O.POST_ADD2_SCALE, "relu": O.POST_RELU}
    W = randn_bf16((N, K), 0.05, 2800 + M)
    t = W.view(N // 16, 16, K // bc, bc // 2, 2).permute(0, 2, 3, 1, 4).contiguous()
    qt = ops.remap_and_quantize_mxfp4(t.cuda(), int8_layout=True)
    q_or, s_or = O.remap_quantize_mxfp4_int8(t.float().numpy())
    x = randn_bf16((M, K), 1.0, 2810 + M)
    x[0, 5] = 0.0
    x[2, :64] = 0.0  # two all-zero blocks: scale 0, codes 0
    x[M - 1] = 0.0
    b = randn_bf16((N,), 0.01, 2820)
    r = randn_bf16((M, N), 1.0, 2830)
    r2 = randn_bf16((M, N), 1.0, 2840) if post == "add2" else None
    assert M >= ops.W4A8_WIDE_ROWS and qt.native_w4a8_wide() is not None
    # the GEMM alone: equal to the oracle
    y0 = ops.linear(x.cuda(), qt, b.cuda(), O.POST_NONE, None, None, 1.0)
    pre = O.linear_w4a8(t2bits(x), q_or, s_or, bc, t2bits(b))
    assert np.array_equal(t2bits(y0), pre), f"w4a8 wide M={M} N={N} K={K}: {(t2bits(y0) != pre).sum()} of {pre.size} differ"
    y = ops.linear(x.cuda(), qt, b.cuda(), posts[post], r.cuda(), None if r2 is None else r2.cuda(), 0.5)
    ref = O.linear_w4a8(t2bits(x), q_or, s_or, bc, t2bits(b), posts[post], t2bits(r), None if r2 is None else t2bits(r2), 0.5)
    assert_close_bf16(t2bits(y), ref, ulps=2 if post == "silu" else 1, what=f"w4a8 wide M={M} N={N} K={K} {post}")
    # without a bias, and against the simple kernel below the threshold (the same sums in another order)
    y1 = ops.linear(x.cuda(), qt, None, O.POST_NONE, None, None, 1.0)
    assert np.array_equal(t2bits(y1), O.linear_w4a8(t2bits(x), q_or, s_or, bc, None))
    monkeypatch.setattr(ops, "W4A8_WIDE_ROWS", 1 << 30)
    y2 = ops.linear(x.cuda(), qt, b.cuda(), O.POST_NONE, None, None, 1.0)
    assert_close_bf16(t2bits(y2), pre, ulps=1, what="simple kernel")
    # the entry point rejects a workspace that is too small, and misaligned outputs
    L = _lib.lib()
    out = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    small = torch.empty(1024, dtype=torch.uint8, device="cuda")
    rc = L.tppx_linear_mxfp4_int8_wide(x.cuda().data_ptr(), qt.native_w4a8_wide().data_ptr(), None, None, None, out.data_ptr(),
                                       M, N, K, 0, 1.0, small.data_ptr(), small.numel(), None)
    assert rc == _lib.EINVAL and b"workspace" in L.tppx_last_error()


def test_w4a8_wide_kernel_at_a_layer_shape():
    """One 7B-shape projection (11008 x 4096) at 512 rows: the many-row W4A8 kernel equal to the oracle."""
    ops = _ops()
    M, N, K, bc = 512, 11008, 4096, 64
    W = randn_bf16((N, K), 0.02, 2900)
    t = W.view(N // 16, 16, K // bc, bc // 2, 2).permute(0, 2, 3, 1, 4).contiguous()
    qt = ops.remap_and_quantize_mxfp4(t.cuda(), int8_layout=True)
    q_or, s_or = O.remap_quantize_mxfp4_int8(t.float().numpy())
    x = randn_bf16((M, K), 1.0, 2901)
    y = ops.linear(x.cuda(), qt, None, O.POST_NONE, None, None, 1.0)
    ref = O.linear_w4a8(t2bits(x), q_or, s_or, bc, None)
    assert np.array_equal(t2bits(y), ref)


@pytest.mark.parametrize("M,N,K,bc,post", [(1, 4096, 4096, 64, "none"), (8, 11008, 4096, 64, "add"), (16, 512, 2048, 128, "silu"),
                                           (5, 96, 1280, 32, "mul"), (8, 4096, 11008, 64, "add"), (3, 8448, 1536, 64, "none"),
                                           (16, 4096, 11008, 64, "add")])
def test_w4a8_decode_kernel(M, N, K, bc, post, monkeypatch):
    """W4A8 decode calls (TppBlockedLinearW<int8_t, uint8_t, Tout>, src/csrc/fused_gemm.h:965-978, at most 16 rows) in
    one launch: rows quantized to int8 over blocks of 32 inside the kernel, K split over the waves of a workgroup,
    weights from tiles made once by tppx_prepack_mxfp4_int8.  Within 1 bf16 ulp (2 through SiLU) of the oracle's
    restatement and of the two-step path (the same integer sums and per-block fp32 multiply-adds in another order);
    16 rows x 11008 do not fit the kernel's LDS and take the two-step path by themselves."""
    ops = _ops()
    from tpp_pytorch_extension import _lib
    posts = {"none": O.POST_NONE, "add": O.POST_ADD_SCALE, "silu": O.POST_SILU, "mul": O.POST_MUL}
    W = randn_bf16((N, K), 0.05, 2700 + M)
    t = W.view(N // 16, 16, K // bc, bc // 2, 2).permute(0, 2, 3, 1, 4).contiguous()
    qt = ops.remap_and_quantize_mxfp4(t.cuda(), int8_layout=True)
    q_or, s_or = O.remap_quantize_mxfp4_int8(t.float().numpy())
    assert np.array_equal(qt.qdata.cpu().numpy().reshape(q_or.shape), q_or)
    x = randn_bf16((M, K), 1.0, 2710 + M)
    x[0, 5] = 0.0
    if M > 2:
        x[2, :64] = 0.0  # two all-zero blocks: scale 0, codes 0
    b = randn_bf16((N,), 0.01, 2720)
    r = randn_bf16((M, N), 1.0, 2730)
    y = ops.linear(x.cuda(), qt, b.cuda(), posts[post], r.cuda(), None, 0.5)
    fits = not (M == 16 and K == 11008)
    rc = _lib.lib().tppx_linear_mxfp4_int8_rows(x.cuda().data_ptr(), *[a.data_ptr() for a in qt.native_w4a8()], None, None, None,
                                                torch.empty((M, N), dtype=torch.bfloat16, device="cuda").data_ptr(), M, N, K,
                                                0, 1.0, None)
    assert (rc == _lib.OK) == fits and (fits or rc == _lib.EUNSUPPORTED)
    ref = O.linear_w4a8(t2bits(x), q_or, s_or, bc, t2bits(b), posts[post], t2bits(r), None, 0.5)
    # (the GEMM tile before an additive / multiplicative post-op may itself be one ulp from the oracle's: its ulp
    # is added to the bound)
    pre = O.linear_w4a8(t2bits(x), q_or, s_or, bc, t2bits(b)) if post in ("add", "mul") else None
    assert_close_bf16(t2bits(y), ref, ulps=2 if post == "silu" else 1, what=f"w4a8 decode M={M} N={N} K={K} {post}", pre_bits=pre)
    monkeypatch.setattr(ops, "W4A8_DECODE", False)
    y2 = ops.linear(x.cuda(), qt, b.cuda(), posts[post], r.cuda(), None, 0.5)
    assert_close_bf16(t2bits(y), t2bits(y2), ulps=2 if post == "silu" else 1, what="one launch vs quantizer + GEMM", pre_bits=pre)
    if not fits:
        assert torch.equal(y, y2)


@pytest.mark.parametrize("kind", ["qint4", "qint2"])
@pytest.mark.parametrize("M,N,K,post", [(1, 11008, 4096, "none"), (8, 4096, 11008, "add"), (16, 4096, 4096, "silu"),
                                        (5, 96, 1024, "mul"), (3, 8448, 14336, "add"),
                                        (32, 11008, 4096, "add"), (64, 4096, 11008, "add"), (40, 96, 1024, "mul"),
                                        (17, 544, 2048, "silu"), (64, 8448, 1536, "none"), (33, 4064, 2816, "add")])
def test_packed_code_decode_kernel_equals_expanded_weight(kind, M, N, K, post, monkeypatch):
    """QINT4 / ternary QINT2 weights at their own width (src/csrc/fused_gemm.h:1110-1126 multiplies the packed codes as
    they lie): up to 64 rows the decode kernels stream N*K/2 or N*K/4 bytes of codes and expand them in registers in
    front of the int8 MFMA.  Same integer sums, scales and rounding as the expanded int8 tiles: within 1 ulp (2 through
    SiLU) of the oracle on the expanded weight, and the SAME BITS as the int8-tile kernel that sums K in the same order
    (TPPX_PACKED_CODES=0; above 16 rows that is the eight-wave kernel without a K split across workgroups)."""
    ops = _ops()
    from tpp_pytorch_extension import _lib
    posts = {"none": O.POST_NONE, "add": O.POST_ADD_SCALE, "silu": O.POST_SILU, "mul": O.POST_MUL}
    W = randn_bf16((N, K), 0.02, 2600 + M)
    if kind == "qint4":
        t = W.view(N // 16, 16, K // 256, 128, 2).permute(0, 2, 3, 1, 4).contiguous()  # VNNI2 [N/16][K/256][128][16][2]
        qt = ops.quantize_int4sym(t.cuda(), 256, 2, True)
    else:
        qt = ops.remap_and_quantize_qint2_intlv(block_bf16(W).cuda())
    assert qt.weight_kind() == kind and qt.block_size == 256
    x = randn_bf16((M, K), 1.0, 2610 + M).cuda()
    b = randn_bf16((N,), 0.01, 2620).cuda()
    r = randn_bf16((M, N), 1.0, 2630).cuda()
    y = ops.linear(x, qt, b, posts[post], r, None, 0.5)
    packed, sn, bits = qt.native_packed()
    assert packed.numel() == N * K * bits // 8
    # the packed path really ran: the entry point accepts the call (no fall-through) and gives the op's bits
    y2 = torch.empty_like(y)
    xq, sa = ops._qint8_scratch(x, M, K, 256)
    _lib.check(_lib.lib().tppx_linear_qintx(x.data_ptr(), xq.data_ptr(), sa.data_ptr(), packed.data_ptr(), sn.data_ptr(),
                                            b.data_ptr(), r.data_ptr(), None, y2.data_ptr(), M, N, K, bits, posts[post], 0.5,
                                            0, _lib.stream_of(x)))
    assert torch.equal(y2, y)
    if M > 16:  # the quantised rows are still in xq / sa: the GEMM alone
        y3 = torch.empty_like(y)
        _lib.check(_lib.lib().tppx_linear_qintx(x.data_ptr(), xq.data_ptr(), sa.data_ptr(), packed.data_ptr(), sn.data_ptr(),
                                                b.data_ptr(), r.data_ptr(), None, y3.data_ptr(), M, N, K, bits, posts[post],
                                                0.5, _lib.FLAG_XQ_REUSE, _lib.stream_of(x)))
        assert torch.equal(y3, y)
    # against the default path on the expanded int8 tiles (itself tested against the oracle above): another fp32
    # summation order above 16 rows, so one ulp apart at most
    monkeypatch.setattr(ops, "PACKED_CODES", False)
    y_default = ops.linear(x, qt, b, posts[post], r, None, 0.5)
    assert_close_bf16(t2bits(y), t2bits(y_default), ulps=2 if post == "silu" else 1, what=f"{kind} packed vs expanded tiles M={M}")
    # eight waves, no K split across workgroups: the packed kernels' summation order
    monkeypatch.setenv("TPPX_QINT8_NK", "0")
    monkeypatch.setenv("TPPX_SKINNY_SPLITK", "0")
    if M > 16:
        monkeypatch.setenv("TPPX_SKINNY_WAVES", "8")
    _lib.lib().tppx_reload_env()
    y_expanded = ops.linear(x, qt, b, posts[post], r, None, 0.5)
    assert torch.equal(y, y_expanded), "packed codes and expanded int8 tiles give different bits"

