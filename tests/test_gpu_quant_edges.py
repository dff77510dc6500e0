"""GPU quantizers / dequantizers on the inputs the reference's own MX header was run on (tests/golden/) and on the
edge blocks of the format (all-zero, fp32 subnormal, smallest exponents, saturation, exact ties, Inf / NaN, -0),
bit for bit against the oracle and against the golden outputs themselves; the fp32 4-D blocked input path of both
weight quantizers; the helper set around them (dequantize, quantize_int8sym, create_qtensor_int8sym -> fc_plain).

Reference: src/csrc/qtypes.cpp:36-197 (MxFP4Quant, Int8SymQuant), :69-77,87-131 (flush / scale / element rules),
src/csrc/mxfp_quant.h:127-161,240-300, src/csrc/qtypes.cpp:438-473,521-577 (dequantize), :654-668.
"""
import os

import numpy as np
import pytest
import torch

import oracle as O
from util import t2bits, randn_bf16, block_bf16, assert_close_bf16

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "mxfp4_golden.npz")


def _ops():
    import tpp_pytorch_extension  # noqa: F401
    from tpp_pytorch_extension import _ops
    return _ops


def _block_f32(W, bk=16, bc=64):
    """fp32 4-D blocked layout [N/bk][K/bc][bc][bk] (blocked_layout.py:75-80 without the VNNI pairing)."""
    N, K = W.shape
    return W.view(N // bk, bk, K // bc, bc).permute(0, 2, 3, 1).contiguous()


def _rows_of_blocks(vals, setter):
    """fp32 matrix [N][K] (N % 32 == 0, K = 64) whose 32-wide K blocks hold 31 of `vals` each plus `setter`, the
    element that fixes the block's shared exponent; returns (W, index of every value inside W.view(-1))."""
    vals = np.asarray(vals, np.float32)
    nblk = (vals.size + 30) // 31
    nblk = (nblk + 63) // 64 * 64  # 2 blocks per row, 32 rows per weight tile
    buf = np.zeros((nblk, 32), np.float32)
    buf[:, 31] = setter
    flat_idx = np.arange(vals.size)
    b, j = flat_idx // 31, flat_idx % 31
    buf[b, j] = vals
    W = buf.reshape(nblk // 2, 64)
    return torch.from_numpy(W.copy()), (b * 32 + j)


def _quantize_both(W):
    """GPU (fp32 4-D blocked input) and oracle quantization of the same fp32 matrix."""
    ops = _ops()
    qw = ops.remap_and_quantize_mxfp4(_block_f32(W).cuda())
    q_or, s_or = O.remap_quantize_mxfp4(W.numpy())
    return qw, q_or, s_or


def _plain(deq_blocked):
    """[N/32][K/64][32 c2][32 k2][2] -> [N][K]"""
    n1, c1 = deq_blocked.shape[:2]
    return deq_blocked.permute(0, 3, 1, 2, 4).reshape(n1 * 32, c1 * 64)


def test_mxfp4_elements_against_golden_all_bf16_and_ties():
    """Every bf16 pattern below 8 in magnitude and the fp32 tie neighbourhoods of the golden file, in blocks whose
    shared scale is 2^0 (a 7.5 in the block): the GPU's codes must decode to what the reference header returned."""
    z = np.load(GOLD)
    bf_all = (np.arange(65536, dtype=np.uint32) << 16).view(np.float32)
    tie_in = z["tie_in"].view(np.float32)
    vin = np.concatenate([bf_all, tie_in])
    vout = np.concatenate([z["e2m1_bf16_out"].view(np.float32), z["tie_out"].view(np.float32)])
    keep = np.isfinite(vin) & (np.abs(vin) < 8.0)
    vin, vout = vin[keep], vout[keep]
    W, idx = _rows_of_blocks(vin, 7.5)
    qw, q_or, s_or = _quantize_both(W)
    assert np.array_equal(qw.qdata.cpu().numpy(), q_or)
    assert np.array_equal(qw.scales.cpu().numpy(), s_or)
    assert (s_or == 127).all()
    got = _plain(qw.dequantize()).cpu().numpy().reshape(-1)[idx]
    assert np.array_equal(got, vout + 0.0), "GPU codes decode to something else than the reference header's result"


def test_mxfp4_scales_against_golden():
    """Block maxima from the golden file (random positive fp32 over the whole exponent range, subnormals included)
    and every non-negative bf16 pattern: the E8M0 byte on the GPU equals the one derived from the reference header's
    scale (its fp32 exponent field; 2^-127 and flushed blocks are byte 0)."""
    z = np.load(GOLD)
    amax = np.concatenate([z["scale_in"].view(np.float32), (np.arange(32768, dtype=np.uint32) << 16).view(np.float32)])
    scale = np.concatenate([z["scale_out"], z["scale_bf16_out"]])
    keep = np.isfinite(amax)
    amax, scale = amax[keep], scale[keep]
    nblk = (amax.size + 63) // 64 * 64
    buf = np.zeros((nblk, 32), np.float32)
    buf[:amax.size, 5] = amax
    buf[:amax.size, 9] = -0.5 * amax
    buf[:amax.size, 17] = 0.3 * amax
    W = torch.from_numpy(buf.reshape(nblk // 2, 64).copy())
    qw, q_or, s_or = _quantize_both(W)
    assert np.array_equal(qw.qdata.cpu().numpy(), q_or)
    assert np.array_equal(qw.scales.cpu().numpy(), s_or)
    # scales [N/32][1][2 h][32 k2] -> per (row, half) = per block in buffer order
    got = qw.scales.cpu().numpy()[:, 0].transpose(0, 2, 1).reshape(-1)[:amax.size]
    want = ((scale >> 23) & 0xFF).astype(np.uint8)  # exponent field of the header's fp32 scale
    assert np.array_equal(got, want)


def test_mxfp4_edge_blocks():
    """All-zero block, -0 everywhere, fp32 subnormal maximum (block flushed), biased exponents 1 and 2 (scale byte
    0 = 2^-127), values saturating at 6, exact ties, Inf blocks and a NaN in the first slot (scale byte 255), a NaN
    in another slot (ignored by the maximum, qtypes.h:156-162), a huge finite maximum."""
    sub = np.float32(1e-40)
    tiny1 = np.array([0x00800000], np.uint32).view(np.float32)[0]  # biased exponent 1
    tiny2 = np.array([0x01000000], np.uint32).view(np.float32)[0]  # biased exponent 2
    blocks = []

    def blk(vals):
        b = np.zeros(32, np.float32)
        b[:len(vals)] = vals
        blocks.append(b)

    blk([])
    blk([-0.0] * 32)
    blk([sub, -sub, sub * 3])
    blk([tiny1, -tiny1 * 0.5, tiny1 * 0.75])
    blk([tiny2, tiny2 * 0.5, -tiny2 * 0.26])
    blk([1.0, 0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 7.0, 6.5, -5.0, 0.2499, 0.2501, -0.08])  # max 7 -> scale 1
    blk([7.9, 7.99, -7.9, 6.0, 6.01])
    blk([np.inf, 1.0, -2.0])
    blk([-np.inf, 0.0, 3.0])
    blk([np.nan, 1.0, -1.0])          # NaN in the first slot: max = NaN -> byte 255
    blk([1.0, np.nan, -1.0, 0.5])     # NaN elsewhere: std::max never picks it, the element itself gets code 0
    blk([3.0e38, -1.0e38, 2.0e38, 1.0])
    blk([-3.4e38, 3.4e38])
    while len(blocks) % 64:
        blocks.append(np.full(32, np.float32(0.01 * len(blocks))))
    W = torch.from_numpy(np.stack(blocks).reshape(-1, 64).copy())
    qw, q_or, s_or = _quantize_both(W)
    assert np.array_equal(qw.scales.cpu().numpy(), s_or), "scale bytes differ on edge blocks"
    assert np.array_equal(qw.qdata.cpu().numpy(), q_or), "element codes differ on edge blocks"
    sc = qw.scales.cpu().numpy()[:, 0].transpose(0, 2, 1).reshape(-1)
    assert sc[0] == 0 and sc[1] == 0 and sc[2] == 0 and sc[3] == 0 and sc[4] == 0
    assert sc[5] == 127 and sc[7] == 255 and sc[8] == 255 and sc[9] == 255 and sc[10] == 125 and sc[11] == 252
    # the same blocks as bf16 5-D input where they are representable
    Wb = W.to(torch.bfloat16)
    ops = _ops()
    qb = ops.remap_and_quantize_mxfp4(block_bf16(Wb).cuda())
    qb_or, sb_or = O.remap_quantize_mxfp4(Wb.float().numpy())
    assert np.array_equal(qb.qdata.cpu().numpy(), qb_or) and np.array_equal(qb.scales.cpu().numpy(), sb_or)


@pytest.mark.parametrize("N,K", [(64, 128), (4096, 1024)])
def test_dequantize_mxfp4_bit_exact(N, K):
    """QTensor.dequantize() / aten.dequantize of an MXFP4 weight == the oracle's dequantize in the blocked shape
    [N/32][K/64][32][32][2], bit for bit, including flushed (scale byte 0) blocks."""
    ops = _ops()
    W = randn_bf16((N, K), 0.02, 901)
    W[3, 32:64] = 0.0
    W[5, :32] = 1e-39
    qw = ops.remap_and_quantize_mxfp4(block_bf16(W).cuda())
    q_or, s_or = O.remap_quantize_mxfp4(W.float().numpy())
    assert np.array_equal(qw.qdata.cpu().numpy(), q_or)
    want = O.dequantize_mxfp4(q_or.reshape(q_or.shape + (1,)), s_or, 32, 2, True)
    got = qw.dequantize()
    assert got.dtype == torch.float32 and tuple(got.shape) == (N // 32, K // 64, 32, 32, 2)
    assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
    assert torch.equal(torch.dequantize(qw), got)
    # and it is the plain-layout dequantize re-blocked
    assert np.array_equal(_plain(got).cpu().numpy(), O.dequantize_mxfp4_plain(q_or, s_or))


@pytest.mark.parametrize("N,K", [(64, 192), (64, 384), (4096, 1024)])
def test_dequantize_qint8_bit_exact(N, K):
    ops = _ops()
    W = randn_bf16((N, K), 0.02, 902)
    W[7] = 0.0
    qw = ops.remap_and_quantize_qint8(block_bf16(W).cuda())
    q_or, s_or, qbs = O.remap_quantize_qint8(W.float().numpy())
    assert qw.block_size == qbs
    want = O.dequantize_int8sym(q_or, s_or, qbs, 2, True)
    got = qw.dequantize()
    assert tuple(got.shape) == tuple(q_or.shape)
    assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
    assert torch.equal(torch.dequantize(qw), got)


@pytest.mark.parametrize("fmt", ["mxfp4", "qint8"])
def test_weight_quantizers_take_fp32_4d_blocked_input(fmt):
    """The 4-D fp32 layout [N/bk][K/bc][bc][bk] (qtypes.cpp:813-838 builds the VNNI pairs itself) with values that
    are NOT bf16-representable: bytes and scales equal the oracle's on the same fp32 values, and equal the 5-D bf16
    path on bf16-representable values."""
    ops = _ops()
    N, K = 256, 512
    g = torch.Generator().manual_seed(903)
    W = torch.randn((N, K), generator=g) * 0.02
    W[9, 64:96] = 0.0
    if fmt == "mxfp4":
        qw = ops.remap_and_quantize_mxfp4(_block_f32(W).cuda())
        q_or, s_or = O.remap_quantize_mxfp4(W.numpy())
    else:
        qw = ops.remap_and_quantize_qint8(_block_f32(W).cuda())
        q_or, s_or, _ = O.remap_quantize_qint8(W.numpy())
    assert np.array_equal(qw.qdata.cpu().numpy(), q_or)
    assert np.array_equal(qw.scales.cpu().numpy().reshape(s_or.shape), s_or)
    Wb = W.to(torch.bfloat16)
    f = ops.remap_and_quantize_mxfp4 if fmt == "mxfp4" else ops.remap_and_quantize_qint8
    a, b = f(_block_f32(Wb.float()).cuda()), f(block_bf16(Wb).cuda())
    assert torch.equal(a.qdata, b.qdata) and torch.equal(a.scales, b.scales)
    # the linear on the fp32-made weight
    x = randn_bf16((5, K), 1.0, 904)
    y = ops.fc_plain(x.cuda(), qw, None)
    lin = O.linear_mxfp4 if fmt == "mxfp4" else O.linear_qint8
    assert_close_bf16(t2bits(y), lin(t2bits(x), q_or, s_or), what=f"{fmt} weight from fp32 4-D input")


def test_quantize_int8sym_vnni_weight_and_create_qtensor():
    """quantize_int8sym(t, QBS, 2, True) on the VNNI4 weight layout == the oracle's generic per-block quantizer;
    create_qtensor_int8sym on caller-made int8 values + fp32 scales gives a weight that fc_plain runs on, with the
    oracle's result for those very values (qtypes.cpp:613-624,654-668)."""
    ops = _ops()
    N, K, qbs = 128, 512, 256
    g = torch.Generator().manual_seed(905)
    t = (torch.randn((N // 16, K // qbs, qbs // 4, 16, 4), generator=g) * 0.02).to(torch.bfloat16)
    t[2, 1, :, 3] = 0.0  # a zero (channel, block): scale 0, all codes 0
    qt = ops.quantize_int8sym(t.cuda(), qbs, 2, True)
    q_or, s_or = O.quantize_int8sym(t.float().numpy(), qbs, 2, True)
    assert np.array_equal(qt.qdata.cpu().numpy(), q_or)
    assert np.array_equal(qt.scales.cpu().numpy(), s_or)
    assert ops.q_per_block_block_size(qt) == qbs and ops.q_per_block_axis(qt) == 2 and ops.q_per_block_pack_size(qt) == 1
    # caller-made values: not the output of any quantizer
    val = torch.randint(-127, 128, (N // 16, K // qbs, qbs // 4, 16, 4), generator=g, dtype=torch.int8)
    scl = (torch.rand((N // 16, K // qbs, 1, 16), generator=g) * 1e-3 + 1e-4).float()
    w = ops.create_qtensor_int8sym(val.cuda(), scl.cuda(), qbs, 2, True)
    assert w.is_quantized and w.dtype == torch.qint8 and tuple(w.shape) == tuple(val.shape)
    x = randn_bf16((9, K), 1.0, 906)
    bias = randn_bf16((N,), 0.01, 907)
    y = ops.fc_plain(x.cuda(), w, bias.cuda())
    ref = O.linear_qint8(t2bits(x), val.numpy(), scl.numpy(), t2bits(bias))
    assert_close_bf16(t2bits(y), ref, what="fc_plain on create_qtensor_int8sym")
    want = O.dequantize_int8sym(val.numpy(), scl.numpy(), qbs, 2, True)
    assert np.array_equal(w.dequantize().cpu().numpy(), want)
