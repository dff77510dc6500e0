"""Parity of the HIP linears against the CPU oracle (ideal mode: fp32
accumulate, one bf16 rounding, reference rounding points in the post-ops).

Stated tolerance: every output within 1 bf16 ulp of the oracle (2 ulp where a
sigmoid is involved, because libm's and the GPU's expf differ in the last
bit), relative L2 error <= 4e-3; against the reference's own bf16 re-rounding
schedule (faithful mode) rel-L2 <= 2^-9 * sqrt(#K-groups) for QINT8.
"""
import numpy as np
import pytest
import torch

import oracle as O
from util import t2bits, randn_bf16, block_bf16, assert_close_bf16, err_stats

pytestmark = pytest.mark.gpu

POSTS = {"none": O.POST_NONE, "silu": O.POST_SILU, "mul": O.POST_MUL, "add": O.POST_ADD_SCALE,
         "add2": O.POST_ADD2_SCALE, "gelu": O.POST_GELU, "relu": O.POST_RELU}


def _lib_mod():
    import tpp_pytorch_extension  # noqa: F401
    from tpp_pytorch_extension import _lib
    return _lib


def _ops():
    import tpp_pytorch_extension  # noqa: F401
    from tpp_pytorch_extension import _ops
    return _ops


def _make(fmt, N, K, seed):
    ops = _ops()
    W = randn_bf16((N, K), 0.02, seed)
    Wb = block_bf16(W).cuda()
    if fmt == "mxfp4":
        qw = ops.remap_and_quantize_mxfp4(Wb)
        q_or, s_or = O.remap_quantize_mxfp4(W.float().numpy())
    else:
        qw = ops.remap_and_quantize_qint8(Wb)
        q_or, s_or, _ = O.remap_quantize_qint8(W.float().numpy())
    # the quantized bytes must be identical before the GEMM is compared
    assert np.array_equal(qw.qdata.cpu().numpy(), q_or), "quantized values differ from the oracle"
    assert np.array_equal(qw.scales.cpu().numpy().reshape(s_or.shape), s_or), "scales differ from the oracle"
    return qw, q_or, s_or


def _run(fmt, M, N, K, post, with_bias, seed, ulps=1, flags=0):
    ops = _ops()
    qw, q_or, s_or = _make(fmt, N, K, seed)
    x = randn_bf16((M, K), 1.0, seed + 1)
    bias = randn_bf16((N,), 0.01, seed + 2) if with_bias else None
    in1 = randn_bf16((M, N), 1.0, seed + 3)
    in2 = randn_bf16((M, N), 1.0, seed + 4)
    scale = 0.5 if post in ("add", "add2") else 1.0
    y = ops.linear(x.cuda(), qw, None if bias is None else bias.cuda(), POSTS[post],
                   in1.cuda(), in2.cuda(), scale, flags=flags)
    torch.cuda.synchronize()
    lin = O.linear_mxfp4 if fmt == "mxfp4" else O.linear_qint8
    ref = lin(t2bits(x), q_or, s_or, None if bias is None else t2bits(bias), POSTS[post],
              t2bits(in1), t2bits(in2), scale, O.MODE_IDEAL)
    s = assert_close_bf16(t2bits(y), ref, ulps=ulps, what=f"{fmt} M={M} N={N} K={K} post={post}")
    return y, ref, s, (qw, q_or, s_or, x, bias, in1, in2, scale)


@pytest.mark.parametrize("fmt", ["mxfp4", "qint8"])
@pytest.mark.parametrize("M", [1, 3, 16, 17, 33, 64])
def test_fc_plain_small(fmt, M):
    _run(fmt, M, 256, 512, "none", True, 100 + M)


@pytest.mark.parametrize("fmt", ["mxfp4", "qint8"])
@pytest.mark.parametrize("post", ["silu", "mul", "add", "add2", "gelu", "relu"])
def test_post_ops(fmt, post):
    _run(fmt, 5, 128, 768, post, post != "mul", 200, ulps=2 if post in ("silu", "gelu") else 1)


@pytest.mark.parametrize("fmt", ["mxfp4", "qint8"])
def test_no_bias_ragged_k(fmt):
    # K = 11008 = 86*128 = 43*256: an odd number of K units, waves get uneven ranges
    _run(fmt, 8, 64, 11008, "none", False, 300)


@pytest.mark.parametrize("M,N,K", [(12, 64, 11008), (13, 64, 11008), (9, 64, 14336), (4, 32, 16384), (1, 64, 4096)])
def test_qint8_few_rows_quantised_in_the_gemm_ring_forms(M, N, K):
    """QINT8 with the activation quantisation inside the GEMM kernel, one channel tile per workgroup: up to three
    K blocks per wave run a ring of four weight tiles (six quantisation passes in flight once a wave has more than 16
    (row, block) items: 36 and 39 items here, two rounds), four blocks per wave (K >= 14336) the ring of eight."""
    _run("qint8", M, N, K, "add", True, 9100 + M + K)


def test_cfg1_mxfp4_fc_plain():
    """BASELINE config 1: M=16, K=N=4096, MXFP4, bias."""
    _run("mxfp4", 16, 4096, 4096, "none", True, 1235)


@pytest.mark.parametrize("M", [1, 8, 32, 64])
def test_cfg2_qint8_fc_add(M):
    """BASELINE config 2 (down-projection shape scaled in N to keep the CPU oracle fast)."""
    y, ref, s, ctx = _run("qint8", M, 512, 11008, "add", False, 1236 + M)
    qw, q_or, s_or, x, bias, in1, in2, scale = ctx
    faithful = O.linear_qint8(t2bits(x), q_or, s_or, None, O.POST_ADD_SCALE, t2bits(in1), None, scale,
                              O.MODE_FAITHFUL)
    st = err_stats(t2bits(y), faithful)
    groups = 11008 // (256 if M == 64 else 64)
    assert st["rel_l2"] <= 2.0 ** -9 * np.sqrt(groups), st["rel_l2"]


def test_qint8_block_64_and_128():
    ops = _ops()
    for K in (192, 384):  # -> QBS 64 and 128 by the reference's rule
        W = randn_bf16((64, K), 0.02, 7)
        qw = ops.remap_and_quantize_qint8(block_bf16(W).cuda())
        q_or, s_or, qbs = O.remap_quantize_qint8(W.float().numpy())
        assert qw.block_size == qbs
        assert np.array_equal(qw.qdata.cpu().numpy(), q_or)
        x = randn_bf16((4, K), 1.0, 8)
        y = ops.fc_plain(x.cuda(), qw, torch.Tensor())
        ref = O.linear_qint8(t2bits(x), q_or, s_or)
        assert_close_bf16(t2bits(y), ref, what=f"qbs={qbs}")


@pytest.mark.parametrize("fmt", ["mxfp4", "qint8"])
def test_qkv_gemm_equals_separate(fmt):
    ops = _ops()
    K, M = 1024, 7
    ws = [_make(fmt, n, K, 40 + i)[0] for i, n in enumerate((512, 128, 128))]
    bs = [randn_bf16((n,), 0.01, 50 + i).cuda() for i, n in enumerate((512, 128, 128))]
    x = randn_bf16((2, M, K), 1.0, 60).cuda()
    outs = torch.ops.tpp_llm.qkv_gemm(x, ws, bs)
    for w, b, o in zip(ws, bs, outs):
        sep = torch.ops.tpp_llm.fc_plain(x, w, b, -1, [])
        assert o.shape == sep.shape == (2, M, w.weight_nk()[0])
        assert torch.equal(o, sep)


def test_swiglu_fused_equals_composition():
    ops = _ops()
    K, N, M = 512, 1024, 9
    wg, wu = _make("mxfp4", N, K, 70)[0], _make("mxfp4", N, K, 71)[0]
    wd = _make("mxfp4", K, N, 72)[0]
    x = randn_bf16((M, K), 1.0, 73).cuda()
    fused = ops.swiglu_gate_up(x, wg, wu)
    g = ops.fc_silu(x, wg, None)
    u = ops.fc_mul(x, wu, None, g)
    assert torch.equal(fused, u)
    out = torch.ops.tpp_llm.swiglu_mlp(x, wg, wu, wd, x, 1.0)
    assert torch.equal(out, ops.fc_add(u, wd, None, x, 1.0))


def test_module_api_and_errors():
    import tpp_pytorch_extension  # noqa: F401
    from tpp_pytorch_extension.llm.llm_common import FixLinear, BlockedLinear
    from tpp_pytorch_extension._lib import TppxError

    torch.manual_seed(0)
    lin = torch.nn.Linear(256, 128, bias=True)
    W, b = lin.weight.data.clone(), lin.bias.data.clone()
    FixLinear(lin, 16, 64, torch.bfloat16, weight_dtype="mxfp4")
    assert isinstance(lin, BlockedLinear) and lin.weight.is_quantized
    assert lin.weight.dtype == torch.quint4x2 and lin.weight.size(-1) == 2
    x = torch.randn(3, 5, 256).cuda()
    y = lin(x)  # fp32 input is cast to bf16 by the module, as in the reference
    q_or, s_or = O.remap_quantize_mxfp4(W.to(torch.bfloat16).float().numpy())
    ref = O.linear_mxfp4(t2bits(x.to(torch.bfloat16).view(15, 256)), q_or, s_or, t2bits(b.to(torch.bfloat16)))
    assert y.shape == (3, 5, 128) and y.dtype == torch.bfloat16
    assert_close_bf16(t2bits(y).reshape(15, 128), ref, what="BlockedLinear")
    with pytest.raises(TppxError):
        torch.ops.tpp_llm.fc_plain(x.to(torch.bfloat16)[..., :128].contiguous(), lin.weight, torch.Tensor(), -1, [])
    yf = torch.ops.tpp_llm.fc_plain(x, lin.weight, torch.Tensor(), -1, [])  # fp32 activations: fp32 result
    assert yf.dtype == torch.float32 and yf.shape == (3, 5, 128)
    with pytest.raises(TppxError):
        torch.ops.tpp_llm.fc_plain(x.to(torch.float64), lin.weight, torch.Tensor(), -1, [])
    e = torch.ops.tpp_llm.fc_plain(torch.empty(0, 256, dtype=torch.bfloat16).cuda(), lin.weight, torch.Tensor(), -1, [])
    assert e.shape == (0, 128)


@pytest.mark.parametrize("fmt", ["mxfp4", "qint8"])
@pytest.mark.parametrize("M", [65, 200, 256])
@pytest.mark.parametrize("family", ["tiled", "skinny", "auto"])
def test_prefill_tiled_small(fmt, M, family):
    """More than 64 rows: the LDS-tiled kernels (N = 384 leaves the last 128-wide block half empty, M = 65 / 200
    leave the last row block ragged) or the decode kernels over several block rows of 64 (the library picks by a
    cost estimate; both families forced here)."""
    from tpp_pytorch_extension import _lib
    flags = {"tiled": _lib.FLAG_FORCE_TILED, "skinny": _lib.FLAG_FORCE_SKINNY, "auto": 0}[family]
    _run(fmt, M, 384, 1024, "add", True, 500 + M, flags=flags)


@pytest.mark.parametrize("fmt", ["mxfp4", "qint8"])
@pytest.mark.parametrize("M,N,K", [(128, 11008, 1024), (192, 4096, 2048), (130, 512, 11008)])
def test_mid_size_m_block_rows(fmt, M, N, K):
    """65..256 rows at 7B-like widths: few output tiles, so the decode kernels run block rows of 64 over the full
    grid (ragged last block row, three channel tiles per workgroup, K split over the waves)."""
    _run(fmt, M, N, K, "add", True, 8800 + M)


@pytest.mark.parametrize("post", ["none", "silu", "mul", "add2", "gelu"])
def test_prefill_mxfp4_ragged_blocks_and_post_ops(post):
    """Large-M MXFP4 kernel (256 x 256 workgroup tiles): two row blocks with a
    ragged second one, three channel blocks with two tiles in the last, an odd
    number of K steps, every fused epilogue through the coalesced store path."""
    _run("mxfp4", 300, 544, 384, post, post != "mul", 700, ulps=2 if post in ("silu", "gelu") else 1)


@pytest.mark.parametrize("tile", [1, 2, 3])
@pytest.mark.parametrize("post", ["none", "silu", "add2"])
def test_prefill_mxfp4_every_workgroup_tile_ragged(tile, post, monkeypatch):
    """The three workgroup tiles of the large-M MXFP4 kernel (256 x 256, 128 x 256 two per CU, 128 x 512), each
    forced, on the ragged case above (rows, channel blocks and K steps all uneven) against the oracle."""
    monkeypatch.setenv("TPPX_TILED_BIG_TILE", str(tile))
    _run("mxfp4", 300, 544, 384, post, True, 705, ulps=2 if post == "silu" else 1)


def test_prefill_mxfp4_workgroup_tiles_and_xcd_splits_agree(monkeypatch):
    """Every workgroup tile and every split of the tile space over the XCDs computes the same sums in the same order:
    identical bits, single GEMM, fused q/k/v and the gate/up pair."""
    ops = _ops()
    M, K = 1024, 512
    w = _make("mxfp4", 4096, K, 710)[0]
    ws = [_make("mxfp4", n, K, 711 + i)[0] for i, n in enumerate((2048, 1024, 1024))]
    wg, wu = _make("mxfp4", 4096, K, 715)[0], _make("mxfp4", 4096, K, 716)[0]
    x = randn_bf16((M, K), 1.0, 717).cuda()

    def run():
        return [ops.fc_plain(x, w, None)] + list(ops.qkv_gemm(x, ws, [None] * 3)) + [ops.swiglu_gate_up(x, wg, wu)]

    monkeypatch.setenv("TPPX_TILED_BIG_TILE", "1")
    monkeypatch.setenv("TPPX_TILED_XCD_M", "1")
    want = run()
    assert torch.equal(want[4], ops.fc_mul(x, wu, None, ops.fc_silu(x, wg, None)))
    for tile in (1, 2, 3):
        for xm in (1, 2, 4):
            monkeypatch.setenv("TPPX_TILED_BIG_TILE", str(tile))
            monkeypatch.setenv("TPPX_TILED_XCD_M", str(xm))
            for i, (a, b) in enumerate(zip(run(), want)):
                assert torch.equal(a, b), (tile, xm, i)


@pytest.mark.parametrize("M", [70, 150, 200, 500])
def test_prefill_forms_for_small_launches_agree(M, monkeypatch):
    """Launches that leave CUs empty run other forms of the large-M kernel's body -- 64 x 128 workgroups of four waves
    up to 128 workgroups of 128 x 256, eight waves per 128 x 256 workgroup up to 256 -- with the same sums in the
    same order: identical bits to the four-wave 128 x 256 form, for a single GEMM (ragged rows and channel blocks),
    fused q/k/v, the gate/up pair and unquantized bf16 weights; the same for the QINT8 kernel's 64 x 256 form (single
    GEMM and fused q/k/v); and the single MXFP4 GEMM against the oracle."""
    ops = _ops()
    K = 640
    w, q_or, s_or = _make("mxfp4", 1056, K, 720)[:3]
    ws = [_make("mxfp4", n, K, 721 + i)[0] for i, n in enumerate((1024, 256, 256))]
    wg, wu = _make("mxfp4", 1120, K, 725)[0], _make("mxfp4", 1120, K, 726)[0]
    Wb = randn_bf16((1056, K), 0.05, 727)
    wb = block_bf16(Wb).cuda()
    w8 = _make("qint8", 1056, 768, 729)[0]
    w8s = [_make("qint8", n, 768, 730 + i)[0] for i, n in enumerate((1024, 256, 256))]
    x8 = randn_bf16((M, 768), 1.0, 733).cuda()
    x = randn_bf16((M, K), 1.0, 728)
    xg = x.cuda()

    def run():
        return [ops.fc_plain(xg, w, None)] + list(ops.qkv_gemm(xg, ws, [None] * 3)) + [ops.swiglu_gate_up(xg, wg, wu)] + \
            [ops.linear(xg, wb, None, O.POST_NONE, None, None, 1.0, flags=_lib_mod().FLAG_FORCE_TILED)] + \
            [ops.fc_plain(x8, w8, None)] + list(ops.qkv_gemm(x8, w8s, [None] * 3))

    monkeypatch.setenv("TPPX_TILED_MIN_M", "0")  # the LDS-tiled family whatever the cost estimate says
    got = run()
    ref = O.linear_mxfp4(t2bits(x), q_or, s_or, None, O.POST_NONE, None, None, 1.0, O.MODE_IDEAL)
    assert_close_bf16(t2bits(got[0]), ref, ulps=1, what=f"64 x 128 workgroups M={M}")
    monkeypatch.setenv("TPPX_TILED_SMALL", "0")
    mid = run()
    monkeypatch.setenv("TPPX_TILED_W8", "0")
    base = run()
    for i, (a, b, c) in enumerate(zip(got, mid, base)):
        assert torch.equal(a, c) and torch.equal(b, c), i


@pytest.mark.parametrize("fmt", ["mxfp4", "qint8"])
def test_prefill_tiled_m2048(fmt):
    """Prefill row count of BASELINE config 4 (M = 2048) on a layer slice the
    CPU oracle finishes in seconds; also compared with the reference's chunked
    bf16 re-rounding schedule (K = 8192 > 4096 -> two chunks for MXFP4)."""
    y, ref, s, ctx = _run(fmt, 2048, 256, 8192, "none", True, 600)
    qw, q_or, s_or, x, bias, in1, in2, scale = ctx
    lin = O.linear_mxfp4 if fmt == "mxfp4" else O.linear_qint8
    faithful = lin(t2bits(x), q_or, s_or, t2bits(bias), O.POST_NONE, None, None, 1.0, O.MODE_FAITHFUL)
    st = err_stats(t2bits(y), faithful)
    bound = 2.0 ** -9 * np.sqrt(2 if fmt == "mxfp4" else 8192 // 256)
    assert st["rel_l2"] <= bound, st["rel_l2"]


def test_prefill_qkv_and_swiglu_equal_composition():
    ops = _ops()
    K, M = 1024, 130
    ws = [_make("mxfp4", n, K, 80 + i)[0] for i, n in enumerate((256, 128, 128))]
    x = randn_bf16((M, K), 1.0, 90).cuda()
    outs = torch.ops.tpp_llm.qkv_gemm(x, ws, [torch.Tensor()] * 3)
    for w, o in zip(ws, outs):
        assert torch.equal(o, ops.fc_plain(x, w, None))
    wg, wu = _make("mxfp4", 512, K, 91)[0], _make("mxfp4", 512, K, 92)[0]
    fused = ops.swiglu_gate_up(x, wg, wu)
    assert torch.equal(fused, ops.fc_mul(x, wu, None, ops.fc_silu(x, wg, None)))


@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("bias", [False, True])
def test_prefill_swiglu_one_grid_equals_composition(bias, fused, monkeypatch):
    """Prefill rows: gate and up run as ONE launch of the large-M kernel.  fused: every workgroup computes both
    projections of its 128 output channels and forms silu(gate) * up in its epilogue; otherwise (TPPX_TILED_DUAL_FUSED=0)
    the gate tile is parked in the workspace and an elementwise pass forms the product.  Either way the bits of
    fc_silu followed by fc_mul, ragged last row block and ragged last channel block included."""
    monkeypatch.setenv("TPPX_TILED_DUAL_FUSED", "1" if fused else "0")
    ops = _ops()
    K, M, N = 512, 300, 1056
    wg, qg, sg_ = _make("mxfp4", N, K, 191)
    wu, qu, su = _make("mxfp4", N, K, 192)
    x = randn_bf16((M, K), 1.0, 193).cuda()
    bg = randn_bf16((N,), 0.05, 194).cuda() if bias else None
    bu = randn_bf16((N,), 0.05, 195).cuda() if bias else None
    fused = ops.swiglu_gate_up(x, wg, wu, bg, bu)
    assert torch.equal(fused, ops.fc_mul(x, wu, bu, ops.fc_silu(x, wg, bg)))
    gate = O.linear_mxfp4(t2bits(x.cpu()), qg, sg_, None if bg is None else t2bits(bg.cpu()), O.POST_SILU)
    ref = O.linear_mxfp4(t2bits(x.cpu()), qu, su, None if bu is None else t2bits(bu.cpu()), O.POST_MUL, gate)
    assert_close_bf16(t2bits(fused), ref, ulps=2, what="prefill swiglu gate/up")


@pytest.mark.parametrize("M", [2, 12])
def test_swiglu_long_k_few_rows(M):
    """Gate/up pair with K = 8192 (beyond the 16-row LDS image): the 4-row staged kernel (M = 2) and the tile-by-tile
    kernel with one row group (M = 12) with two accumulator sets; bits of silu-then-mul, and the oracle."""
    ops = _ops()
    K, N = 8192, 1056
    wg, qg, sg_ = _make("mxfp4", N, K, 311)
    wu, qu, su = _make("mxfp4", N, K, 312)
    x = randn_bf16((M, K), 1.0, 313)
    fused = ops.swiglu_gate_up(x.cuda(), wg, wu)
    assert torch.equal(fused, ops.fc_mul(x.cuda(), wu, None, ops.fc_silu(x.cuda(), wg, None)))
    gate = O.linear_mxfp4(t2bits(x), qg, sg_, None, O.POST_SILU)
    ref = O.linear_mxfp4(t2bits(x), qu, su, None, O.POST_MUL, gate)
    assert_close_bf16(t2bits(fused), ref, ulps=2, what=f"swiglu gate/up K=8192 M={M}")


@pytest.mark.parametrize("M", [2, 12])
def test_swiglu_full_size_gate_up_equals_composition(M):
    """Llama-7B gate/up shape (688 channel tiles): the fused kernel takes one
    (M <= 4) or two channel tiles of each GEMM per workgroup; both must give the
    bits of silu-then-mul through the single-GEMM kernels, and match the oracle."""
    ops = _ops()
    wg, qg, sg_ = _make("mxfp4", 11008, 512, 301)
    wu, qu, su = _make("mxfp4", 11008, 512, 302)
    x = randn_bf16((M, 512), 1.0, 303)
    fused = ops.swiglu_gate_up(x.cuda(), wg, wu)
    assert torch.equal(fused, ops.fc_mul(x.cuda(), wu, None, ops.fc_silu(x.cuda(), wg, None)))
    gate = O.linear_mxfp4(t2bits(x), qg, sg_, None, O.POST_SILU)
    ref = O.linear_mxfp4(t2bits(x), qu, su, None, O.POST_MUL, gate)
    assert_close_bf16(t2bits(fused), ref, ulps=2, what=f"swiglu gate/up M={M}")


@pytest.mark.parametrize("M", [17, 32, 40, 64])
def test_mxfp4_row_group_kernel_full_size(M):
    """17..64 rows at the Llama-7B up-projection shape (688 channel tiles: three per workgroup, ragged last group,
    M = 40: a partly filled row group) with bias and the residual post-op."""
    y, ref, s, ctx = _run("mxfp4", M, 11008, 1024, "add", True, 7100 + M)


@pytest.mark.parametrize("M", [24, 64])
def test_mxfp4_row_group_kernel_uneven_k_split_and_swiglu(M):
    """K = 11008 (86 K tiles over 8 waves: 10 or 11 each); q/k/v segments in one launch; the gate/up pair as
    silu(gate) then up * gate in place: all equal to the single-GEMM calls bit for bit, which match the oracle."""
    ops = _ops()
    y, ref, s, ctx = _run("mxfp4", M, 256, 11008, "none", False, 7200 + M)
    K = 1024
    ws = [_make("mxfp4", n, K, 7300 + i)[0] for i, n in enumerate((4096, 512, 512))]
    x = randn_bf16((M, K), 1.0, 7310).cuda()
    outs = torch.ops.tpp_llm.qkv_gemm(x, ws, [torch.Tensor()] * 3)
    for w, o in zip(ws, outs):
        assert torch.equal(o, ops.fc_plain(x, w, None))
    wg, qg, sg_ = _make("mxfp4", 11008, K, 7320)
    wu, qu, su = _make("mxfp4", 11008, K, 7321)
    fused = ops.swiglu_gate_up(x, wg, wu)
    assert torch.equal(fused, ops.fc_mul(x, wu, None, ops.fc_silu(x, wg, None)))
    gate = O.linear_mxfp4(t2bits(x.cpu()), qg, sg_, None, O.POST_SILU)
    ref2 = O.linear_mxfp4(t2bits(x.cpu()), qu, su, None, O.POST_MUL, gate)
    assert_close_bf16(t2bits(fused), ref2, ulps=2, what=f"swiglu gate/up M={M}")


@pytest.mark.parametrize("fmt,M,N", [("mxfp4", 40, 4096), ("mxfp4", 64, 4064), ("qint8", 40, 4096), ("qint8", 64, 4080)])
def test_k_split_across_workgroups(fmt, M, N):
    """33..64 rows, at most 256 channel tiles and K = 11008: K is split across workgroups (4 parts of 21/22/21/22
    K tiles for MXFP4, 2 parts of 21/22 blocks for QINT8), the partial sums go through the workspace and the
    workgroup that finishes last adds them.  N = 4064 (254 tiles) or 4080 (255): a ragged last group; M = 40: a partly filled row
    group.  Forty launches in a row must give the same bits (the arrival counters return to zero, no launch sees
    another's partial sums)."""
    ops = _ops()
    y, ref, s, ctx = _run(fmt, M, N, 11008, "add", True, 7400 + M)
    qw, q_or, s_or, x, bias, in1, in2, scale = ctx
    xs, b, r = x.cuda(), bias.cuda(), in1.cuda()
    first = torch.ops.tpp_llm.fc_add(xs, qw, b, r, scale)
    outs = [torch.ops.tpp_llm.fc_add(xs, qw, b, r, scale) for _ in range(40)]
    torch.cuda.synchronize()
    assert torch.equal(first, y)
    for o in outs:
        assert torch.equal(o, first)


@pytest.mark.parametrize("M,N,K,post", [(64, 4096, 8192, "add"), (33, 4080, 14336, "add2"), (50, 2048, 16384, "none"),
                                        (17, 4096, 11008, "mul"), (32, 4064, 14336, "silu"), (64, 1600, 32768, "add"),
                                        (20, 4096, 12288, "gelu")])
def test_qint8_tile_by_k_part_kernel(M, N, K, post, monkeypatch):
    """QINT8, 17..64 rows, up to 256 channel tiles and a long K: four channel tiles x four K parts per workgroup with
    the activation operands shared through LDS, K in four slices across workgroups, partial tiles exchanged as
    128-bit device-scope stores / loads (2..8 steps per wave, ragged last channel group, partly filled row groups,
    every post-op).  Against the oracle; twenty launches give the same bits; the kernel it replaces
    (TPPX_QINT8_NK=0) is within one ulp of it as well (another summation order, so not bit-identical)."""
    import ctypes
    from tpp_pytorch_extension import _lib
    buf = ctypes.create_string_buffer(2048)
    _lib.check(_lib.lib().tppx_plan_linear_qint8(M, N, K, 256, 1, 0, _lib.WORKSPACE_BYTES, buf, len(buf)))
    assert "skinny_qint8_nk_kernel" in buf.value.decode(), buf.value.decode()
    y, ref, st, ctx = _run("qint8", M, N, K, post, True, 7700 + M, ulps=2 if post in ("silu", "gelu") else 1)
    qw, q_or, s_or, x, bias, in1, in2, scale = ctx
    ops = _ops()
    again = [ops.linear(x.cuda(), qw, bias.cuda(), POSTS[post], in1.cuda(), in2.cuda(), scale) for _ in range(20)]
    torch.cuda.synchronize()
    for o in again:
        assert torch.equal(o, y)
    monkeypatch.setenv("TPPX_QINT8_NK", "0")
    old = ops.linear(x.cuda(), qw, bias.cuda(), POSTS[post], in1.cuda(), in2.cuda(), scale)
    assert_close_bf16(t2bits(old), ref, ulps=2 if post in ("silu", "gelu") else 1, what="kernel without the tile x K-part grid")


@pytest.mark.parametrize("form", [0, 1])
@pytest.mark.parametrize("M,N,K,post", [(64, 4096, 8192, "add"), (33, 4064, 14336, "add2"), (50, 2048, 16384, "none"),
                                        (64, 1632, 12288, "silu"), (47, 4096, 11008, "mul")])
def test_mxfp4_tile_by_k_part_kernel(M, N, K, post, form, monkeypatch):
    """MXFP4, 33..64 rows, up to 256 channel tiles and a long K: four channel tiles x four K parts per workgroup (two
    tiles per wave and eight waves, or one and sixteen: TPPX_MXFP4_NK_FORM), a K tile's activations staged once per
    workgroup, K in four slices across workgroups, workgroups walking their K part from rotated starting tiles.
    Against the oracle; twenty launches give the same bits; the kernel it replaces (TPPX_MXFP4_NK=0) meets the oracle
    too."""
    import ctypes
    from tpp_pytorch_extension import _lib
    monkeypatch.setenv("TPPX_MXFP4_NK_FORM", str(form))
    buf = ctypes.create_string_buffer(2048)
    _lib.check(_lib.lib().tppx_plan_linear_mxfp4(M, N, K, 0, _lib.WORKSPACE_BYTES, buf, len(buf)))
    assert "skinny_mxfp4_nk_kernel<4, 4, %d," % (2 - form) in buf.value.decode(), buf.value.decode()
    y, ref, st, ctx = _run("mxfp4", M, N, K, post, True, 7800 + M, ulps=2 if post == "silu" else 1)
    qw, q_or, s_or, x, bias, in1, in2, scale = ctx
    ops = _ops()
    again = [ops.linear(x.cuda(), qw, bias.cuda(), POSTS[post], in1.cuda(), in2.cuda(), scale) for _ in range(20)]
    torch.cuda.synchronize()
    for o in again:
        assert torch.equal(o, y)
    if form == 0:
        monkeypatch.setenv("TPPX_MXFP4_NK", "0")
        old = ops.linear(x.cuda(), qw, bias.cuda(), POSTS[post], in1.cuda(), in2.cuda(), scale)
        assert_close_bf16(t2bits(old), ref, ulps=2 if post == "silu" else 1, what="kernel without the tile x K-part grid")


@pytest.mark.parametrize("split", [True, False])
@pytest.mark.parametrize("M,N,K", [(5, 4096, 11008), (16, 4096, 11008), (9, 2048, 16384), (16, 4096, 8192)])
def test_mxfp4_few_rows_long_k_split_across_workgroups(M, N, K, split, monkeypatch):
    """5..16 rows, at most 256 channel tiles and a K too long for one workgroup's staging: the LDS-staged kernel with
    K in 4 parts across workgroups of 4 channel tiles (21/22 K tiles per part at K = 11008, 1 or 2 per wave), partial
    sums through the workspace, the last workgroup to arrive finishes -- or (TPPX_MXFP4_XL_SPLIT=0) the tile-by-tile
    kernel.  Against the oracle; the row sums of squares the finishing workgroup leaves equal the sums over the output
    bits; repeated launches give the same bits."""
    monkeypatch.setenv("TPPX_MXFP4_XL_SPLIT", "1" if split else "0")
    ops = _ops()
    y, ref, s, ctx = _run("mxfp4", M, N, K, "add", True, 7500 + M)
    qw, q_or, s_or, x, bias, in1, in2, scale = ctx
    xs, b, r = x.cuda(), bias.cuda(), in1.cuda()
    tab = torch.full((16, 256), 3.0, dtype=torch.float32, device="cuda")  # stale contents must not survive
    outs = [ops.fc_add(xs, qw, b, r, scale, row_sumsq=tab) for _ in range(20)]
    torch.cuda.synchronize()
    for o in outs:
        assert torch.equal(o, y)
    want = (y.double() ** 2).sum(-1).cpu().numpy()
    got = tab[:M].double().sum(-1).cpu().numpy()
    assert np.allclose(got, want, rtol=1e-5), (got, want)


def test_prefill_qint8_qkv_one_launch_equals_separate():
    """QINT8, enough rows for the large-M kernel: fused q/k/v share one launch (ragged channel blocks: 544, 128 and
    256 channels) and give the bits of the single-GEMM calls, which match the oracle."""
    ops = _ops()
    K, M = 1024, 300
    made = [_make("qint8", n, K, 280 + i) for i, n in enumerate((544, 128, 256))]
    ws = [m[0] for m in made]
    x = randn_bf16((M, K), 1.0, 290)
    bs = [randn_bf16((n,), 0.01, 295 + i).cuda() for i, n in enumerate((544, 128, 256))]
    outs = torch.ops.tpp_llm.qkv_gemm(x.cuda(), ws, bs)
    for (w, q_or, s_or), b, o in zip(made, bs, outs):
        assert torch.equal(o, ops.fc_plain(x.cuda(), w, b))
        ref = O.linear_qint8(t2bits(x), q_or, s_or, t2bits(b.cpu()))
        assert_close_bf16(t2bits(o), ref, what="qint8 fused qkv, large M")


def test_prefill_qkv_one_launch_equals_separate():
    """With enough rows the fused q/k/v GEMMs share one launch of the large-M
    kernel (one grid over the channel blocks of all three)."""
    ops = _ops()
    K, M = 512, 300
    ws = [_make("mxfp4", n, K, 180 + i)[0] for i, n in enumerate((544, 128, 256))]
    x = randn_bf16((M, K), 1.0, 190).cuda()
    bs = [randn_bf16((n,), 0.01, 195 + i).cuda() for i, n in enumerate((544, 128, 256))]
    outs = torch.ops.tpp_llm.qkv_gemm(x, ws, bs)
    for w, b, o in zip(ws, bs, outs):
        assert torch.equal(o, ops.fc_plain(x, w, b))


_FULL_UP = {}


def _full_up():
    """One Llama-7B up-projection weight (N=11008, K=4096), quantized once."""
    if not _FULL_UP:
        _FULL_UP["w"] = _make("qint8", 11008, 4096, 4242)
    return _FULL_UP["w"]


@pytest.mark.parametrize("M", [1, 4, 8, 16, 32, 40, 64])
def test_cfg2_qint8_up_projection_full_size(M):
    """The kernel variants that only large N selects (two and three channel
    tiles per wave, ragged last workgroup: 688 tiles), at BASELINE's real shape."""
    ops = _ops()
    qw, q_or, s_or = _full_up()
    x = randn_bf16((M, 4096), 1.0, 500 + M)
    r = randn_bf16((M, 11008), 1.0, 600 + M)
    y = torch.ops.tpp_llm.fc_add(x.cuda(), qw, torch.Tensor(), r.cuda(), 1.0)
    ref = O.linear_qint8(t2bits(x), q_or, s_or, None, O.POST_ADD_SCALE, t2bits(r), None, 1.0, O.MODE_IDEAL)
    pre = O.linear_qint8(t2bits(x), q_or, s_or)
    assert_close_bf16(t2bits(y), ref, what=f"qint8 up-projection M={M}", pre_bits=pre)


def test_qint8_fused_quant_shared_lds():
    """16 rows x K=8192 with three channel tiles per workgroup: the quantised activations and the cross-wave
    reduction do not fit the LDS side by side, so the reduction reuses the activations' region."""
    y, ref, s, ctx = _run("qint8", 16, 8448, 8192, "add", True, 4242)
    assert_close_bf16(t2bits(y), ref, what="qint8 M=16 K=8192 N=8448")


@pytest.mark.parametrize("M,K", [(128, 512), (200, 11008), (2048, 4096)])
def test_qint8_activation_quantizer_many_rows_bit_exact(M, K):
    """From 128 rows on, 256-wide blocks take the quantizer that gives 16 lanes to a (row, block); with zero rows, a
    row of one value and a huge value in the input, bytes and scales must equal the oracle's."""
    from tpp_pytorch_extension import _lib
    L = _lib.lib()
    x = randn_bf16((M, K), 1.0, 41)
    x[5] = 0.0
    x[7] = -0.375
    x[9, 300] = 3.0e38
    x = x.cuda()
    xq = torch.empty((M, K), dtype=torch.int8, device="cuda")
    sa = torch.empty((M, K // 256), dtype=torch.float32, device="cuda")
    _lib.check(L.tppx_quant_act_int8(x.data_ptr(), M, K, 256, xq.data_ptr(), sa.data_ptr(), _lib.stream_of(x)))
    xq_or, sa_or = O.quant_act_int8(t2bits(x.cpu()), 256)
    assert np.array_equal(sa.cpu().numpy(), sa_or)
    assert np.array_equal(xq.cpu().numpy(), xq_or)


@pytest.mark.parametrize("M", [3, 24, 64])
def test_qint8_prequantized_and_reused_activations(M):
    """x == NULL takes row-major int8 activations + scales (the reference's
    pre-quantized input); TPPX_FLAG_XQ_REUSE skips the re-quantization when a
    second GEMM runs on the same input.  Both must give the bits of the plain
    call, and the activation quantization itself must match the oracle."""
    from tpp_pytorch_extension import _lib
    L = _lib.lib()
    N, K, qbs = 512, 1024, 256
    qw, q_or, s_or = _make("qint8", N, K, 31)
    qw2, q_or2, s_or2 = _make("qint8", N, K, 32)
    x = randn_bf16((M, K), 1.0, 33).cuda()
    st = _lib.stream_of(x)
    ws = _lib.workspace(x)
    xq_rm = torch.empty((M, K), dtype=torch.int8, device="cuda")
    sa_rm = torch.empty((M, K // qbs), dtype=torch.float32, device="cuda")
    _lib.check(L.tppx_quant_act_int8(x.data_ptr(), M, K, qbs, xq_rm.data_ptr(), sa_rm.data_ptr(), st))
    xq_or, sa_or = O.quant_act_int8(t2bits(x.cpu()), qbs)
    assert np.array_equal(xq_rm.cpu().numpy(), xq_or) and np.array_equal(sa_rm.cpu().numpy(), sa_or)

    def call(xptr, xq, sa, w, flags):
        qn, sn = w.native()
        y = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
        _lib.check(L.tppx_linear_qint8(xptr, xq.data_ptr(), sa.data_ptr(), qn.data_ptr(), sn.data_ptr(), None, None,
                                       None, y.data_ptr(), M, N, K, qbs, 0, 1.0, flags, ws.data_ptr(), ws.numel(), st))
        return y

    xq = torch.empty(((M + 63) // 64 * 64, K), dtype=torch.int8, device="cuda")
    sa = torch.empty(((M + 63) // 64 * 64, K // qbs), dtype=torch.float32, device="cuda")
    y_plain = call(x.data_ptr(), xq, sa, qw, 0)
    y2_reuse = call(x.data_ptr(), xq, sa, qw2, _lib.FLAG_XQ_REUSE)
    y2_plain = call(x.data_ptr(), xq.clone().zero_(), sa.clone().zero_(), qw2, 0)
    y_pre = call(None, xq_rm, sa_rm, qw, 0)
    torch.cuda.synchronize()
    ref = O.linear_qint8(t2bits(x.cpu()), q_or, s_or)
    assert_close_bf16(t2bits(y_plain), ref, what=f"plain M={M}")
    assert torch.equal(y_pre, y_plain), "pre-quantized input gives different bits"
    assert torch.equal(y2_reuse, y2_plain), "reused activation quantization gives different bits"


def _shape_sweep():
    """48 seeded (format, M, N, K, post-op, bias) cases across the kernel selection boundaries: 1..64 rows, channel
    counts that leave ragged workgroups, K from one native tile to the Llama intermediate size."""
    import random
    rnd = random.Random(20240)
    cases = []
    for i in range(48):
        fmt = rnd.choice(["mxfp4", "qint8"])
        M = rnd.choice([1, 2, 3, 4, 5, 7, 8, 9, 15, 16, 17, 20, 31, 32, 33, 47, 48, 63, 64])
        N = rnd.choice([32, 64, 96, 160, 512, 1056, 4128, 8224])
        K = rnd.choice([128, 256, 384, 512, 1024, 2048, 2304, 4096, 5120, 8192, 11008])
        if fmt == "qint8" and K % 256:
            K = (K // 256 + 1) * 256
        cases.append((fmt, M, N, K, rnd.choice(["none", "silu", "mul", "add", "add2", "gelu", "relu"]), rnd.random() < 0.5, 9100 + i))
    return cases


@pytest.mark.parametrize("fmt,M,N,K,post,bias,seed", _shape_sweep())
def test_shape_sweep(fmt, M, N, K, post, bias, seed):
    ops = _ops()
    qw, q_or, s_or = _make(fmt, N, K, seed)
    x = randn_bf16((M, K), 1.0, seed + 1)
    b = randn_bf16((N,), 0.01, seed + 2) if bias else None
    in1, in2 = randn_bf16((M, N), 1.0, seed + 3), randn_bf16((M, N), 1.0, seed + 4)
    scale = 0.5 if post in ("add", "add2") else 1.0
    y = ops.linear(x.cuda(), qw, None if b is None else b.cuda(), POSTS[post], in1.cuda(), in2.cuda(), scale)
    lin = O.linear_mxfp4 if fmt == "mxfp4" else O.linear_qint8
    bb = None if b is None else t2bits(b)
    ref = lin(t2bits(x), q_or, s_or, bb, POSTS[post], t2bits(in1), t2bits(in2), scale, O.MODE_IDEAL)
    pre = lin(t2bits(x), q_or, s_or, bb) if post in ("add", "add2") else None  # the tile a residual can cancel
    assert_close_bf16(t2bits(y), ref, ulps=2 if post in ("silu", "gelu") else 1,
                      what=f"{fmt} M={M} N={N} K={K} post={post}", pre_bits=pre)


def test_launch_plan_names_the_kernels():
    import ctypes
    from tpp_pytorch_extension import _lib
    L = _lib.lib()
    buf = ctypes.create_string_buffer(2048)
    _lib.check(L.tppx_plan_linear_qint8(64, 11008, 4096, 256, 1, 0, 1 << 25, buf, len(buf)))
    lines = buf.value.decode().strip().splitlines()
    assert len(lines) == 2 and "quant_act_int8_rows_kernel" in lines[0] and "skinny_qint8_kernel<" in lines[1]
    _lib.check(L.tppx_plan_linear_qint8(1, 11008, 4096, 256, 1, 0, 1 << 25, buf, len(buf)))
    assert buf.value.decode().count("\n") == 1 and "skinny_qint8_fq_kernel<" in buf.value.decode()
    _lib.check(L.tppx_plan_linear_mxfp4(2048, 8192, 8192, 0, 0, buf, len(buf)))
    assert "big_mxfp4_kernel" in buf.value.decode()
    _lib.check(L.tppx_plan_linear_mxfp4(100, 8192, 8192, _lib.FLAG_FORCE_TILED, 0, buf, len(buf)))
    assert "big_mxfp4_kernel<2, false, 2, 2>" in buf.value.decode()  # 64 x 128 workgroups from 65 rows on
    _lib.check(L.tppx_plan_linear_mxfp4(128, 11008, 4096, 0, 0, buf, len(buf)))  # few tiles: block rows of 64
    assert "skinny_mxfp4_mg_kernel" in buf.value.decode() and "x2x" in buf.value.decode()


@pytest.mark.parametrize("M,N,K,post,layout", [
    (1, 2000, 512, "none", "vnni2"), (5, 272, 1024, "add", "vnni2"), (16, 4096, 4096, "none", "vnni2"),
    (17, 1008, 384, "silu", "plain"), (33, 528, 640, "mul", "vnni2"), (64, 1024, 11008, "add", "vnni2"),
    (100, 304, 256, "add2", "plain"), (200, 1040, 512, "none", "blocked100")])
def test_bf16_weight_linear(M, N, K, post, layout):
    """Unquantized bf16 weights (the reference's default lm_head class, TppBlockedLinearW<bf16,bf16>) through
    fc_plain / the post-op GEMMs: 1 ulp of the oracle's single-rounding result, for the blocked VNNI2 layout
    BlockedLinear makes, a plain [N][K] matrix, and the lm_head's own blocking (bk = N/10-style odd block
    heights: here 104 = 1040/10 rows per block)."""
    ops = _ops()
    W = randn_bf16((N, K), 0.02, 81)
    x = randn_bf16((M, K), 1.0, 82)
    bias = randn_bf16((N,), 0.01, 83)
    in1, in2 = randn_bf16((M, N), 1.0, 84), randn_bf16((M, N), 1.0, 85)
    scale = 0.5 if post in ("add", "add2") else 1.0
    if layout == "vnni2":
        Wg = block_bf16(W).cuda()
    elif layout == "plain":
        Wg = W.cuda()
    else:
        Wg = block_bf16(W, bk=104, bc=64).cuda()
    y = ops.linear(x.cuda(), Wg, bias.cuda(), POSTS[post], in1.cuda(), in2.cuda(), scale)
    ref = O.linear_bf16(t2bits(x), t2bits(W), t2bits(bias), POSTS[post], t2bits(in1), t2bits(in2), scale)
    assert_close_bf16(t2bits(y), ref, ulps=1, what=f"bf16 weight M={M} N={N} K={K} post={post} {layout}",
                      pre_bits=O.linear_bf16(t2bits(x), t2bits(W), t2bits(bias)) if post in ("add", "add2") else None)
    y2 = ops.linear(x.cuda(), Wg, bias.cuda(), POSTS[post], in1.cuda(), in2.cuda(), scale)  # cached native tiles
    assert torch.equal(y, y2)


def test_bf16_weight_module_and_errors():
    import tpp_pytorch_extension  # noqa: F401
    from tpp_pytorch_extension.llm.llm_common import FixLinear, BlockedLinear
    from tpp_pytorch_extension._lib import TppxError
    torch.manual_seed(3)
    lin = torch.nn.Linear(256, 1000, bias=False)  # lm_head-like: FixLinear(m, 100, 64, bf16) keeps bf16 weights
    W = lin.weight.data.clone().to(torch.bfloat16)
    FixLinear(lin, 100, 64, torch.bfloat16)
    assert isinstance(lin, BlockedLinear) and not lin.weight.is_quantized and lin.weight.dim() == 5
    lin = lin.cuda()
    x = randn_bf16((2, 3, 256), 1.0, 86)
    with pytest.raises(TppxError):  # N = 1000 is not a multiple of 16
        lin(x.cuda())
    lin = torch.nn.Linear(256, 1600, bias=True)
    W, b = lin.weight.data.clone().to(torch.bfloat16), lin.bias.data.clone().to(torch.bfloat16)
    FixLinear(lin, 100, 64, torch.bfloat16)
    lin = lin.cuda()
    y = lin(x.cuda())
    ref = O.linear_bf16(t2bits(x.view(6, 256)), t2bits(W), t2bits(b))
    assert y.shape == (2, 3, 1600)
    assert_close_bf16(t2bits(y).reshape(6, 1600), ref, what="bf16 BlockedLinear")
    with pytest.raises(TppxError):
        _ops().linear(x.cuda()[..., :128].contiguous(), lin.weight, None)


def _mxfp8_from_operand_order(xq, xs, M, K):
    """GPU layout [Mp/16][K/128][2][64][16] / [Mp/64][K/128][64][4] (Mp = M rounded up to 64) -> codes [Mp][K],
    scale bytes [Mp][K/32]."""
    Mt, Kt = (M + 63) // 64 * 4, K // 128
    q = xq.view(Mt, Kt, 2, 4, 16, 16).permute(0, 4, 1, 2, 3, 5).reshape(Mt * 16, K)  # [mt][m][kt][h][g][16]
    s = xs.view(Mt // 4, Kt, 4, 16, 4).permute(0, 4, 3, 1, 2).reshape(Mt * 16, K // 32)  # [q][t][m][kt][b]
    return q.cpu().numpy(), s.cpu().numpy()


@pytest.mark.parametrize("M,K", [(1, 128), (37, 384), (128, 4096)])
def test_mxfp8_activation_quantizer_bit_exact(M, K):
    from tpp_pytorch_extension import _lib
    _ops()
    x = randn_bf16((M, K), 1.0, 91)
    x[0, :32] = 0.0                      # an all-zero block
    x.view(-1)[5::97] *= 37.0            # outliers that set block maxima
    Mp = (M + 63) // 64 * 64
    xq = torch.empty(Mp * K, dtype=torch.uint8, device="cuda")
    xs = torch.empty(Mp * K // 32, dtype=torch.uint8, device="cuda")
    xg = x.cuda()
    _lib.check(_lib.lib().tppx_quant_act_mxfp8(xg.data_ptr(), M, K, xq.data_ptr(), xs.data_ptr(), _lib.stream_of(xg)))
    q, s = _mxfp8_from_operand_order(xq, xs, M, K)
    q_or, s_or = O.quant_act_mxfp8(t2bits(x))
    assert np.array_equal(q[:M], q_or) and np.array_equal(s[:M], s_or)
    assert not q[M:].any() and not s[M:].any()  # padded rows are zeros


@pytest.mark.parametrize("M,N,K,post", [(128, 256, 256, "none"), (1, 32, 128, "none"), (200, 544, 384, "add"),
                                         (333, 4096, 1024, "silu"), (2048, 512, 4096, "none")])
def test_mxfp4_linear_on_fp8_activations(M, N, K, post):
    """TPPX_FLAG_ACT_FP8: MXFP4 weights on the block-scaled MFMA with MXFP8 activations.  Against the oracle of the
    same arithmetic (exact products, fp32 sums: 1 ulp, 2 through SiLU as for the other kernels), and against the reference-arithmetic oracle (bf16
    activations) within the rounding of E4M3: rel-L2 <= 5e-2."""
    from tpp_pytorch_extension import _lib
    ops = _ops()
    qw, q_or, s_or = _make("mxfp4", N, K, 95)
    x = randn_bf16((M, K), 1.0, 96)
    bias = randn_bf16((N,), 0.01, 97)
    in1 = randn_bf16((M, N), 1.0, 98)
    scale = 0.5 if post == "add" else 1.0
    y = ops.linear(x.cuda(), qw, bias.cuda(), POSTS[post], in1.cuda(), None, scale, flags=_lib.FLAG_ACT_FP8)
    ref = O.linear_mxfp4_fp8act(t2bits(x), q_or, s_or, t2bits(bias), POSTS[post], t2bits(in1), None, scale)
    pre = O.linear_mxfp4_fp8act(t2bits(x), q_or, s_or, t2bits(bias)) if post == "add" else None
    # the block-scaled MFMA adds the 128 products of an instruction with the hardware's own internal alignment, not
    # as exact fp64 sums: more elements land one ulp off than with another fp32 order (2-3 per thousand seen)
    assert_close_bf16(t2bits(y), ref, ulps=2 if post == "silu" else 1, what=f"fp8-act M={M} N={N} K={K} {post}",
                      pre_bits=pre, max_mismatch=None if post == "silu" else 1e-2)
    exact = O.linear_mxfp4(t2bits(x), q_or, s_or, t2bits(bias), POSTS[post], t2bits(in1), None, scale, O.MODE_IDEAL)
    assert err_stats(t2bits(y), exact)["rel_l2"] <= 5e-2


@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("M,K,widths", [(160, 512, (512, 256, 256)), (300, 384, (544, 288, 288))])
def test_fp8_activation_qkv_and_swiglu_equal_separate_calls(M, K, widths, fused, monkeypatch):
    """fused: the gate/up pair with both projections per workgroup and silu(gate) * up in the epilogue; otherwise
    (TPPX_TILED_DUAL_FUSED=0) the parked gate tile and the elementwise pass.  The second shape has ragged row, channel
    and K blocks."""
    from tpp_pytorch_extension import _lib, _ops as ops
    _ops()
    monkeypatch.setenv("TPPX_TILED_DUAL_FUSED", "1" if fused else "0")
    x = randn_bf16((M, K), 1.0, 99).cuda()
    ws = [_make("mxfp4", n, K, 100 + i)[0] for i, n in enumerate(widths)]
    old = ops.ACT_FP8
    ops.ACT_FP8 = True
    try:
        q, k, v = ops.qkv_gemm(x, ws, [None, None, None])
        sw = ops.swiglu_gate_up(x, ws[1], ws[2])
    finally:
        ops.ACT_FP8 = old
    for got, w in zip((q, k, v), ws):
        assert torch.equal(got, ops.linear(x, w, None, flags=_lib.FLAG_ACT_FP8))
    g = ops.linear(x, ws[1], None, POSTS["silu"], flags=_lib.FLAG_ACT_FP8)
    assert torch.equal(sw, ops.linear(x, ws[2], None, POSTS["mul"], g, flags=_lib.FLAG_ACT_FP8))
    from tpp_pytorch_extension._lib import TppxError
    Lb = _lib.lib()
    y = torch.empty(M, widths[0], dtype=torch.bfloat16, device="cuda")
    qn, sn = ws[0].native()
    with pytest.raises(TppxError):  # no workspace for the quantised activations
        _lib.check(Lb.tppx_linear_mxfp4(x.data_ptr(), qn.data_ptr(), sn.data_ptr(), None, None, None, y.data_ptr(),
                                        M, widths[0], K, 0, 1.0, _lib.FLAG_ACT_FP8, None, 0, _lib.stream_of(x)))


def test_split_launches_from_two_threads_on_two_streams():
    """Launches that split K over workgroups (partial sums in the workspace, an arrival counter per output group, the
    last arrival merges) and split-KV attention launches, issued by two Python threads, each on a stream of its own, so
    that they overlap on the card.  The ops take their workspace per (device, stream) and the library hands the
    arrival counters out in rotation, so the threads need no ordering between them.  Every output must carry the bits
    of the same call made alone on one stream; the comparison stops at the first mismatch."""
    import threading
    from tpp_pytorch_extension import _lib, _ops as ops
    _ops()
    Lb = _lib.lib()
    dev = torch.device("cuda:0")
    cases = []
    for fmt, M, N, K, seed in (("qint8", 64, 4096, 11008, 701), ("mxfp4", 64, 512, 4096, 702), ("mxfp4", 33, 256, 8192, 703)):
        qw = _make(fmt, N, K, seed)[0]
        x = randn_bf16((M, K), 1.0, seed + 1).cuda()
        r = randn_bf16((M, N), 1.0, seed + 2).cuda()
        cases.append(("linear", qw, x, r))
    B, Nq, Smax, Lk = 1, 32, 2304, 2000
    q = randn_bf16((B, Nq, 128), 1.0, 711).cuda()
    kc = randn_bf16((B, Nq, Smax, 128), 1.0, 712).cuda()
    vc = randn_bf16((B, Nq, Smax, 128), 1.0, 713).cuda()
    ln = torch.tensor([Lk - 1], dtype=torch.int32, device=dev)
    cases.append(("attn", q, kc, vc))

    def call(case):
        if case[0] == "linear":
            _, qw, x, r = case
            return ops.linear(x, qw, None, POSTS["add"], r, None, 0.5)
        _, q, kc, vc = case
        ws = _lib.workspace(q)
        out = torch.empty_like(q)
        _lib.check(Lb.tppx_attn_decode(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), None, 0, ln.data_ptr(), 1,
                                       out.data_ptr(), B, Nq, Nq, 128, Smax, ws.data_ptr(), ws.numel(), _lib.stream_of(q)))
        return out

    alone = [call(c) for c in cases]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = [[], []]
    seen_ws = [None, None]
    errors = []

    def worker(si):
        try:
            with torch.cuda.stream(streams[si]):
                seen_ws[si] = _lib.workspace(q).data_ptr()
                for it in range(24):
                    ci = (it + 2 * si) % len(cases)  # the two threads run different cases side by side
                    outs[si].append((ci, call(cases[ci])))
        except Exception as e:  # reported by the main thread
            errors.append((si, repr(e)))

    threads = [threading.Thread(target=worker, args=(si,)) for si in (0, 1)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors
    assert len({seen_ws[0], seen_ws[1], _lib.workspace(q).data_ptr()}) == 3, "each stream works in a workspace of its own"
    for si in (0, 1):
        assert len(outs[si]) == 24
        for it, (ci, y) in enumerate(outs[si]):
            assert torch.equal(y, alone[ci]), f"thread {si}, launch {it}, case {ci}: differs from the single-stream result"


@pytest.mark.parametrize("M", [1, 5, 16])
@pytest.mark.parametrize("widths", [(512, 512, 512), (768, 256, 256), (512, 128)])
def test_qkv_one_gemm_over_concatenated_weights(M, widths, monkeypatch):
    """Decode steps run q/k/v as ONE GEMM over the concatenated native weights with three output matrices
    (tppx_qkv_linear_mxfp4): the same bits as the segment-table launch and as separate calls, with and without the
    RMSNorm in the launch (from handed row sums, or formed in the launch), with some biases missing; the projections'
    own native copies become views into the concatenation and keep working on their own."""
    from tpp_pytorch_extension import _ops as ops
    _ops()
    K = 2048
    ws = [_make("mxfp4", n, K, 140 + i)[0] for i, n in enumerate(widths)]
    bs = [randn_bf16((widths[0],), 0.01, 150).cuda()] + [None] * (len(widths) - 1)
    x = randn_bf16((M, K), 1.0, 160 + M).cuda()
    gamma = (torch.rand(K) + 0.5).cuda()
    monkeypatch.setattr(ops, "QKV_ONE_GEMM", False)
    seg = ops.qkv_gemm(x, ws, bs)
    monkeypatch.setattr(ops, "QKV_ONE_GEMM", True)
    one = ops.qkv_gemm(x, ws, bs)
    assert getattr(ws[0], "_tppx_qkv_cat", None) is not None  # the one-GEMM path ran
    for a, b, w, bias in zip(one, seg, ws, bs):
        assert a.shape == b.shape and a.is_contiguous() and torch.equal(a, b)
        assert torch.equal(a, ops.fc_plain(x, w, bias))  # native views into the concatenation
    # RMSNorm inside the launch, sums formed there
    monkeypatch.setattr(ops, "FUSE_NORM", True)
    monkeypatch.setattr(ops, "QKV_ONE_GEMM", False)
    seg_n = ops.qkv_gemm(x, ws, bs, norm=(gamma, 1e-5))
    monkeypatch.setattr(ops, "QKV_ONE_GEMM", True)
    one_n = ops.qkv_gemm(x, ws, bs, norm=(gamma, 1e-5))
    for a, b in zip(one_n, seg_n):
        assert torch.equal(a, b)
    # RMSNorm from the row sums a producing GEMM left (here: formed by hand in the table's layout, slot 0 of 256)
    table = ops.sums_table(x.device)
    table[:M, 0] = (x.float() ** 2).sum(-1)
    monkeypatch.setattr(ops, "QKV_ONE_GEMM", False)
    seg_s = ops.qkv_gemm(x, ws, bs, norm=(gamma, 1e-5, table))
    monkeypatch.setattr(ops, "QKV_ONE_GEMM", True)
    one_s = ops.qkv_gemm(x, ws, bs, norm=(gamma, 1e-5, table))
    for a, b in zip(one_s, seg_s):
        assert torch.equal(a, b)
