"""tppx_linear_qint8_noalloc (scratch in a static device array of the library) against tppx_linear_qint8 (scratch
from the caller) through the C ABI: the same kernels, so the same bits -- on two calls in a row on one GPU, the
second with a smaller input (the array keeps the first call's contents), then on a third shape that splits K
across workgroups; sizes beyond the array are rejected before any launch."""
import numpy as np
import pytest
import torch

import oracle as O
from util import t2bits, randn_bf16, block_bf16, assert_close_bf16

pytestmark = pytest.mark.gpu


def _both(L, _lib, qw, x, res, M, N, K, qbs, post, ws_bytes=4 * 256 * 4 * 256 * 4):
    qn, sn = qw.native()
    st = _lib.stream_of(x)
    y0 = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    y1 = torch.full((M, N), 7.0, dtype=torch.bfloat16, device="cuda")
    xq = torch.empty(((M + 63) // 64 * 64, K), dtype=torch.int8, device="cuda")
    sa = torch.empty(((M + 63) // 64 * 64, K // qbs), dtype=torch.float32, device="cuda")
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
    _lib.check(L.tppx_linear_qint8(x.data_ptr(), xq.data_ptr(), sa.data_ptr(), qn.data_ptr(), sn.data_ptr(), None,
                                   _lib.ptr(res), None, y0.data_ptr(), M, N, K, qbs, post, 1.0, 0, ws.data_ptr(),
                                   ws.numel(), st))
    _lib.check(L.tppx_linear_qint8_noalloc(x.data_ptr(), qn.data_ptr(), sn.data_ptr(), None, _lib.ptr(res), None,
                                           y1.data_ptr(), M, N, K, qbs, post, 1.0, 0, st))
    torch.cuda.synchronize()
    return y0, y1


def test_noalloc_entry_point_equals_caller_scratch_entry_point():
    import tpp_pytorch_extension  # noqa: F401
    from tpp_pytorch_extension import _lib, _ops
    L = _lib.lib()
    cases = [(64, 4096, 11008), (8, 512, 1024), (33, 4080, 11008), (1, 11008, 4096)]  # (M, N, K): 1st and 3rd split K
    for i, (M, N, K) in enumerate(cases):
        W = randn_bf16((N, K), 0.02, 9900 + i)
        qw = _ops.remap_and_quantize_qint8(block_bf16(W).cuda())
        q_or, s_or, qbs = O.remap_quantize_qint8(W.float().numpy())
        x = randn_bf16((M, K), 1.0, 9910 + i)
        r = randn_bf16((M, N), 1.0, 9920 + i)
        y0, y1 = _both(L, _lib, qw, x.cuda(), r.cuda(), M, N, K, qbs, _lib.POST_ADD_SCALE)
        assert torch.equal(y0, y1), f"case {i}: static-scratch entry point gives different bits"
        ref = O.linear_qint8(t2bits(x), q_or, s_or, None, O.POST_ADD_SCALE, t2bits(r), None, 1.0)
        assert_close_bf16(t2bits(y1), ref, what=f"noalloc M={M} N={N} K={K}", pre_bits=O.linear_qint8(t2bits(x), q_or, s_or))
    # beyond the static array: rejected with a clear error, nothing launched
    A = 1 << 20
    assert L.tppx_linear_qint8_noalloc(A, A, A, None, None, None, A, 65, 16, 256, 256, 0, 1.0, 0, None) == _lib.ESHAPE
    assert "static scratch" in L.tppx_last_error().decode()
    assert L.tppx_linear_qint8_noalloc(A, A, A, None, None, None, A, 1, 16, 32768 + 256, 256, 0, 1.0, 0, None) == _lib.ESHAPE
    assert L.tppx_linear_qint8_noalloc(None, A, A, None, None, None, A, 1, 16, 256, 256, 0, 1.0, 0, None) == _lib.EINVAL
    assert L.tppx_linear_qint8_noalloc(A, A, A, None, None, None, A, 1, 16, 256, 256, 0, 1.0, _lib.FLAG_XQ_REUSE, None) == _lib.EINVAL


def test_noalloc_entry_point_inside_graph_capture():
    """After one eager call on the device (which takes the static array's address), the entry point can be recorded
    into a HIP graph -- it allocates nothing -- and every replay gives the bits of the eager call, on the fused-
    quantisation path (8 rows), the quantizer + GEMM path (40 rows) and the K-split path (64 rows, long K)."""
    import tpp_pytorch_extension  # noqa: F401
    from tpp_pytorch_extension import _lib, _ops
    L = _lib.lib()
    for i, (M, N, K) in enumerate([(8, 512, 1024), (40, 256, 2048), (64, 4096, 11008)]):
        W = randn_bf16((N, K), 0.02, 9950 + i)
        qw = _ops.remap_and_quantize_qint8(block_bf16(W).cuda())
        qn, sn = qw.native()
        x = randn_bf16((M, K), 1.0, 9960 + i).cuda()
        r = randn_bf16((M, N), 1.0, 9970 + i).cuda()
        y_eager = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
        y_graph = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")

        def call(y):
            _lib.check(L.tppx_linear_qint8_noalloc(x.data_ptr(), qn.data_ptr(), sn.data_ptr(), None, r.data_ptr(), None,
                                                   y.data_ptr(), M, N, K, 256, _lib.POST_ADD_SCALE, 1.0, 0,
                                                   _lib.stream_of(x)))

        call(y_eager)
        torch.cuda.synchronize()
        # capture_error_mode="global" (torch's default, spelled out): a hipMalloc / hipFree or any other call that is
        # illegal under capture, from any thread, fails the capture -- so a capture that succeeds allocated nothing
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, capture_error_mode="global"):
            call(y_graph)
        for rep in range(3):
            y_graph.zero_()
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(y_graph, y_eager), f"case {i}: replay {rep} differs from the eager call"
            call(y_eager)  # eager work of the same entry point between the replays
            torch.cuda.synchronize()
