"""QINT8 scale blocks other than the default 256 input channels, up to per-output-channel scales (one block = all of
K: QINT8_BLOCK_SIZE=4096 on the Llama-7B up-projection, the literal "fp32 per-channel scales" of the QINT8
configuration; QINT8_BLOCK_SIZE=11008 on the down-projection), against the CPU oracle through the same op calls.

Block-size rule: remap_and_quantize_qint8 (src/csrc/qtypes.cpp:866-932); the GEMM that consumes such blocks:
TppBlockedQInt8LinearW (src/csrc/fused_gemm.h:1103-1110 n_Hc_blocks, 1183-1233 one dequant per block).

Tolerances as everywhere: weight bytes / scales and int8 activations bit-exact; outputs within 1 bf16 ulp of the ideal
oracle, at most 1e-3 of them different at all, rel-L2 <= 4e-3; against the reference's chunked re-rounding (faithful
mode) rel-L2 <= 2^-9 * sqrt(#chunks).
"""
import ctypes

import numpy as np
import pytest
import torch

import oracle as O
from util import t2bits, randn_bf16, block_bf16, assert_close_bf16, err_stats

pytestmark = pytest.mark.gpu

_CACHE = {}


def _weight(N, K, qbs, seed):
    """(GPU quantized tensor, oracle values, oracle scales) for QINT8_BLOCK_SIZE = qbs; GPU bytes == oracle bytes."""
    key = (N, K, qbs, seed)
    if key not in _CACHE:
        import tpp_pytorch_extension  # noqa: F401
        from tpp_pytorch_extension import _ops
        W = randn_bf16((N, K), 0.02, seed)
        old = _ops.QINT8_BLOCK_SIZE
        _ops.QINT8_BLOCK_SIZE = qbs
        try:
            qw = _ops.remap_and_quantize_qint8(block_bf16(W).cuda())
        finally:
            _ops.QINT8_BLOCK_SIZE = old
        q_or, s_or, got_qbs = O.remap_quantize_qint8(W.float().numpy(), env_block=qbs)
        assert got_qbs == qbs and qw.block_size == qbs
        assert np.array_equal(qw.qdata.cpu().numpy(), q_or), "quantized values differ from the oracle"
        assert np.array_equal(qw.scales.cpu().numpy().reshape(s_or.shape), s_or), "scales differ from the oracle"
        _CACHE[key] = (qw, q_or, s_or)
    return _CACHE[key]


def _plan(M, N, K, qbs):
    from tpp_pytorch_extension import _lib
    buf = ctypes.create_string_buffer(4096)
    _lib.check(_lib.lib().tppx_plan_linear_qint8(M, N, K, qbs, 1, 0, _lib.WORKSPACE_BYTES, buf, len(buf)))
    return [ln.split(" grid=")[0].replace("void ", "") for ln in buf.value.decode().strip().splitlines()]


def _noalloc(qw, x, res, M, N, K, qbs):
    from tpp_pytorch_extension import _lib
    qn, sn = qw.native()
    y = torch.full((M, N), 7.0, dtype=torch.bfloat16, device="cuda")
    _lib.check(_lib.lib().tppx_linear_qint8_noalloc(x.data_ptr(), qn.data_ptr(), sn.data_ptr(), None, res.data_ptr(), None,
                                                    y.data_ptr(), M, N, K, qbs, _lib.POST_ADD_SCALE, 1.0, 0,
                                                    _lib.stream_of(x)))
    return y


def _check_fc_add(M, N, K, qbs, seed, what, noalloc=True):
    qw, q_or, s_or = _weight(N, K, qbs, seed)
    x = randn_bf16((M, K), 1.0, seed + 10 + M)
    r = randn_bf16((M, N), 1.0, seed + 100 + M)
    xg, rg = x.cuda(), r.cuda()
    y = torch.ops.tpp_llm.fc_add(xg, qw, torch.Tensor(), rg, 1.0)
    ref = O.linear_qint8(t2bits(x), q_or, s_or, None, O.POST_ADD_SCALE, t2bits(r), None, 1.0, O.MODE_IDEAL)
    pre = O.linear_qint8(t2bits(x), q_or, s_or)
    assert_close_bf16(t2bits(y), ref, what=what, pre_bits=pre)
    faithful = O.linear_qint8(t2bits(x), q_or, s_or, None, O.POST_ADD_SCALE, t2bits(r), None, 1.0, O.MODE_FAITHFUL)
    chunks = K // (qbs if M % 64 == 0 else 64)  # remainder rows are re-rounded every 64 input channels
    assert err_stats(t2bits(y), faithful)["rel_l2"] <= 2.0 ** -9 * np.sqrt(chunks)
    # the GEMM tile without a post-op: one ulp at most, and almost every element equal
    y0 = torch.ops.tpp_llm.fc_plain(xg, qw, torch.Tensor(), -1, [])
    assert_close_bf16(t2bits(y0), pre, what=what + " (no post-op)", max_mismatch=1e-3)
    assert torch.equal(y, torch.ops.tpp_llm.fc_add(xg, qw, torch.Tensor(), rg, 1.0)), "second call gives other bits"
    if noalloc and M <= 64:
        assert torch.equal(y, _noalloc(qw, xg, rg, M, N, K, qbs)), "static-scratch entry point gives other bits"
    return y


@pytest.mark.parametrize("qbs", [512, 1024, 4096])
@pytest.mark.parametrize("M", [1, 8, 32, 64])
def test_cfg2_up_projection_large_blocks(M, qbs):
    """4096 -> 11008 with blocks of 512, 1024 and 4096 = K (per-output-channel scales): K is dealt to the waves in
    256-wide runs inside a block, so all waves of a workgroup stay busy; up to 16 rows the activation quantisation
    stays inside the GEMM launch (the waves exchange their row maxima through LDS)."""
    _check_fc_add(M, 11008, 4096, qbs, 7100 + qbs, f"up-projection qbs={qbs} M={M}")
    names = _plan(M, 11008, 4096, qbs)
    assert names[-1].startswith("tppx::skinny_qint8"), names
    assert (len(names) == 1) == (M <= 16), names  # one launch with the quantisation fused, else quantizer + GEMM


@pytest.mark.parametrize("M", [1, 8, 16, 64])
def test_cfg2_down_projection_per_output_channel(M):
    """11008 -> 4096 with one block = all 11008 input channels (43 runs of 256): row maxima across all 16 waves, 24
    (row, run) items per wave at 8 rows, the K split across two workgroups at 64 rows."""
    _check_fc_add(M, 4096, 11008, 11008, 7300, f"down-projection qbs=K M={M}")


@pytest.mark.parametrize("M,N,K,qbs", [(5, 512, 1280, 320), (40, 96, 1920, 640), (3, 256, 768, 384), (64, 1024, 2048, 128),
                                       (17, 528, 4096, 2048), (16, 8448, 8192, 8192), (9, 11008, 4096, 4096)])
def test_other_block_sizes(M, N, K, qbs):
    """Blocks that are not a whole number of 256-wide runs (K dealt tile by tile, folds at block ends and at the end
    of a wave's range), below 256, and large blocks where the fused quantisation does not fit (more than 8 rows
    with three channel tiles per workgroup; the shared LDS region at 16 rows x 8192)."""
    _check_fc_add(M, N, K, qbs, 7500 + qbs, f"M={M} N={N} K={K} qbs={qbs}")


@pytest.mark.parametrize("M,K,qbs", [(1, 4096, 4096), (33, 11008, 11008), (64, 4096, 1024), (130, 32768, 32768), (7, 2048, 512)])
def test_activation_quantizer_large_blocks_bit_exact(M, K, qbs):
    """The stand-alone quantizer on blocks of several runs (one workgroup per (row, block), maxima through LDS; a
    second pass over the row beyond 16 Ki channels), with a zero row, a constant row and a huge value."""
    from tpp_pytorch_extension import _lib
    x = randn_bf16((M, K), 1.0, 77)
    if M > 5:
        x[5] = 0.0
        x[3] = -0.375
    x[0, K - 1] = 3.0e38
    x = x.cuda()
    xq = torch.empty((M, K), dtype=torch.int8, device="cuda")
    sa = torch.empty((M, K // qbs), dtype=torch.float32, device="cuda")
    _lib.check(_lib.lib().tppx_quant_act_int8(x.data_ptr(), M, K, qbs, xq.data_ptr(), sa.data_ptr(), _lib.stream_of(x)))
    xq_or, sa_or = O.quant_act_int8(t2bits(x.cpu()), qbs)
    assert np.array_equal(sa.cpu().numpy(), sa_or)
    assert np.array_equal(xq.cpu().numpy(), xq_or)


@pytest.mark.parametrize("M,qbs", [(128, 1024), (300, 4096)])
def test_large_blocks_many_rows(M, qbs):
    """More than 64 rows: block rows of the decode kernels or the LDS-tiled kernel, whichever the planner takes."""
    _check_fc_add(M, 1024, 4096, qbs, 7700 + qbs, f"M={M} qbs={qbs}", noalloc=False)
