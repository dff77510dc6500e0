"""Host-side checks that need no GPU: the C-ABI library loads and exports every
entry point include/tppx.h declares, arguments are validated before any HIP
call (error codes, never a crash or exit), and the Python drop-in layer
(blocked layouts, module classes, helper names) behaves like the reference's.
"""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _lib():
    import tpp_pytorch_extension  # noqa: F401
    from tpp_pytorch_extension import _lib
    return _lib


def test_header_symbols_are_exported_and_bound():
    L = _lib()
    hdr = open(os.path.join(ROOT, "include", "tppx.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    declared = set(re.findall(r"\b(tppx_[a-z0-9_]+)\s*\(", hdr))
    assert len(declared) >= 14
    lib = L.lib()
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in tppx.h but not exported"
    assert declared == set(L.SIGNATURES), "ctypes signatures and tppx.h disagree"
    assert lib.tppx_version() == 100


def test_seg_struct_matches_header_layout():
    L = _lib()
    # 6 pointers, int64, int32, float
    assert ctypes.sizeof(L.Seg) == 6 * 8 + 8 + 4 + 4
    assert L.Seg.N.offset == 48 and L.Seg.post_op.offset == 56 and L.Seg.post_scale.offset == 60


def test_argument_validation_without_gpu():
    L = _lib()
    lib = L.lib()
    A = 1 << 20  # a fake, 16-byte aligned "device pointer": validation must reject before touching it

    def err():
        return lib.tppx_last_error().decode()

    # null pointers
    assert lib.tppx_linear_mxfp4(None, A, A, None, None, None, A, 1, 32, 128, 0, 1.0, 0, None, 0, None) == L.EINVAL
    assert "null" in err()
    assert lib.tppx_linear_qint8(A, None, A, A, A, None, None, None, A, 1, 16, 256, 256, 0, 1.0, 0, None, 0, None) == L.EINVAL
    # misaligned
    assert lib.tppx_linear_mxfp4(A + 2, A, A, None, None, None, A, 1, 32, 128, 0, 1.0, 0, None, 0, None) == L.EINVAL
    assert "aligned" in err()
    # shapes: M = 0, K not a multiple of 64, N not a multiple of 32 / 16, block size mismatch
    assert lib.tppx_linear_mxfp4(A, A, A, None, None, None, A, 0, 32, 128, 0, 1.0, 0, None, 0, None) == L.ESHAPE
    assert lib.tppx_linear_mxfp4(A, A, A, None, None, None, A, 1, 32, 100, 0, 1.0, 0, None, 0, None) == L.ESHAPE
    assert lib.tppx_linear_mxfp4(A, A, A, None, None, None, A, 1, 48, 128, 0, 1.0, 0, None, 0, None) == L.ESHAPE
    assert lib.tppx_linear_mxfp4(A, A, A, None, None, None, A, 1, 32, 192, 0, 1.0, 0, None, 0, None) == L.EUNSUPPORTED
    assert lib.tppx_linear_qint8(A, A, A, A, A, None, None, None, A, 1, 24, 256, 256, 0, 1.0, 0, None, 0, None) == L.ESHAPE
    assert lib.tppx_linear_qint8(A, A, A, A, A, None, None, None, A, 1, 16, 256, 192, 0, 1.0, 0, None, 0, None) == L.ESHAPE
    assert "block size" in err()
    # unquantized bf16 weights: K in whole 128-channel tiles, N in 16s, blocking must divide the matrix
    assert lib.tppx_linear_bf16(A, A, None, None, None, A, 1, 16, 192, 0, 1.0, 0, None) == L.ESHAPE
    assert lib.tppx_linear_bf16(A, A, None, None, None, A, 1, 24, 128, 0, 1.0, 0, None) == L.ESHAPE
    assert lib.tppx_linear_bf16(A, None, None, None, None, A, 1, 16, 128, 0, 1.0, 0, None) == L.EINVAL
    assert lib.tppx_prepack_bf16(A, 32, 256, 16, 48, 2, A, None) == L.ESHAPE
    assert lib.tppx_prepack_bf16(A, 32, 256, 16, 64, 3, A, None) == L.ESHAPE
    # post-op id and its inputs
    assert lib.tppx_linear_mxfp4(A, A, A, None, None, None, A, 1, 32, 128, 9, 1.0, 0, None, 0, None) == L.EINVAL
    assert lib.tppx_linear_mxfp4(A, A, A, None, None, None, A, 1, 32, 128, L.POST_MUL, 1.0, 0, None, 0, None) == L.EINVAL
    assert "post_in" in err()
    assert lib.tppx_linear_mxfp4(A, A, A, None, A, None, A, 1, 32, 128, L.POST_ADD2_SCALE, 1.0, 0, None, 0, None) == L.EINVAL
    # flags and workspace
    assert lib.tppx_linear_mxfp4(A, A, A, None, None, None, A, 1, 32, 128, 0, 1.0, 64, None, 0, None) == L.EINVAL
    assert lib.tppx_linear_mxfp4(A, A, A, None, None, None, A, 1, 32, 128, 0, 1.0, 3, None, 0, None) == L.EINVAL
    assert lib.tppx_linear_mxfp4(A, A, A, None, None, None, A, 1, 32, 128, 0, 1.0, 0, None, 4096, None) == L.EINVAL
    # fused groups
    segs = (L.Seg * 5)()
    assert lib.tppx_multi_linear_mxfp4(A, segs, 5, 1, 128, 0, None, 0, None) == L.EINVAL
    assert lib.tppx_multi_linear_mxfp4(A, segs, 0, 1, 128, 0, None, 0, None) == L.EINVAL
    # quantizers
    assert lib.tppx_quantize_mxfp4(A, 0, 48, 128, 16, 64, 2, A, A, None) == L.ESHAPE
    assert lib.tppx_quantize_mxfp4(A, 7, 64, 128, 16, 64, 2, A, A, None) == L.EINVAL
    assert lib.tppx_quantize_qint8(A, 1, 64, 128, 16, 64, 2, 96, A, A, None) == L.ESHAPE
    assert lib.tppx_quant_act_int8(A, 1, 100, 256, A, A, None) == L.ESHAPE
    assert lib.tppx_prepack_mxfp4(A, A, 64, 192, A, A, None) == L.ESHAPE
    assert lib.tppx_dequantize_qint8(None, A, 16, 256, 256, A, None) == L.EINVAL


def test_python_layer_fails_loudly_without_gpu():
    L = _lib()
    from tpp_pytorch_extension._C import _qtype
    if torch.cuda.is_available():
        pytest.skip("checks the no-GPU behaviour")
    w = torch.randn(64, 128).to(torch.bfloat16).view(4, 16, 2, 32, 2).permute(0, 2, 3, 1, 4).contiguous()
    with pytest.raises(L.TppxError):
        _qtype.remap_and_quantize_mxfp4(w)
    with pytest.raises(L.TppxError):
        torch.ops.tpp_llm.fc_plain(torch.randn(2, 128), torch.randn(64, 128), torch.Tensor(), -1, [])


def test_reference_names_are_importable():
    import tpp_pytorch_extension as tpx
    from tpp_pytorch_extension import qtypes, nn
    from tpp_pytorch_extension._C import _qtype, _fused_llm_infer
    from tpp_pytorch_extension.llm import llm_common
    from tpp_pytorch_extension.utils import blocked_layout
    for n in ("quantize_mxfp", "quantize_mxfp4", "quantize_int8sym", "quantize_int4sym", "create_qtensor_int8sym",
              "create_qtensor_int2sym", "q_per_block_scales", "q_per_block_pack_size", "q_per_block_block_size",
              "q_per_block_axis", "remap_and_quantize_mxfp4", "remap_and_quantize_qint8",
              "remap_and_quantize_qint2_intlv", "fix_vnni"):
        assert callable(getattr(_qtype, n)), n
    for n in ("get_qval", "get_scales", "get_axis", "get_block_size", "q_per_block_qval"):
        assert callable(getattr(qtypes, n)), n
    assert callable(_fused_llm_infer.fc_plain) and callable(nn.fc_plain) and callable(llm_common.fc_plain)
    for n in ("BlockedLinear", "FixLinear"):
        assert hasattr(llm_common, n)
    for n in ("TppLinear", "BlockedWeight", "FixLinear", "OptimizeForLinear"):
        assert hasattr(nn, n)
    for n in ("BlockingManager", "BlockedParameter", "BlockedModule"):
        assert hasattr(blocked_layout, n)
    assert tpx.get_vnni_blocking(torch.bfloat16) == 2 and tpx.get_vnni_blocking(torch.float32) == 1
    for op in ("fc_plain", "fc_add", "fc_silu", "fc_mul", "qkv_gemm", "swiglu_mlp"):
        assert hasattr(torch.ops.tpp_llm, op)


def test_blocking_manager_matches_index_formula():
    from tpp_pytorch_extension.utils.blocked_layout import BlockingManager
    from tpp_pytorch_extension.nn import BlockedWeight
    N, K = 48, 128
    W = torch.arange(N * K, dtype=torch.float32).view(N, K)
    bm = BlockingManager(W.shape, blocking_factors=[16, [32, 2]], permute=[0, 2, 3, 1, 4])
    Wb = bm.block(W)
    assert list(Wb.shape) == [3, 2, 32, 16, 2] == bm.blocked_shape
    for (n1, c1, c2, k2, c3) in [(0, 0, 0, 0, 0), (2, 1, 31, 15, 1), (1, 0, 7, 3, 1)]:
        assert Wb[n1, c1, c2, k2, c3] == W[n1 * 16 + k2, c1 * 64 + c2 * 2 + c3]
    assert torch.equal(bm.unblock(Wb), W)
    assert torch.equal(BlockedWeight(W, 16, 64, torch.bfloat16), Wb.to(torch.bfloat16))
    assert torch.equal(BlockedWeight(W, 16, 64, torch.float32), W.view(3, 16, 2, 64).permute(0, 2, 3, 1))
    with pytest.raises(AssertionError):
        BlockingManager((50, 128), blocking_factors=[16, 64], permute=[0, 2, 3, 1])


def test_blocked_module_state_dict_round_trip():
    """BlockedModule saves BlockedParameters in the plain layout and re-blocks
    them on load (reference: blocked_layout.py:309-364)."""
    from tpp_pytorch_extension.utils.blocked_layout import BlockedModule, BlockedParameter

    class Mod(BlockedModule):
        def __init__(self):
            super().__init__()
            self.w = BlockedParameter(torch.arange(64 * 128, dtype=torch.float32).view(64, 128))
            self.w.set_blocking_param(([16, 64], [0, 2, 3, 1]))

    m = Mod()
    plain = m.w.data.clone()
    m.w.block()
    assert list(m.w.shape) == [4, 2, 64, 16] and m.w.is_blocked()
    sd = m.state_dict()
    assert list(sd["w"].shape) == [64, 128] and torch.equal(sd["w"], plain)
    assert m.w.is_blocked()
    m2 = Mod()
    m2.w.block()
    m2.load_state_dict({"w": plain * 2})
    assert m2.w.is_blocked() and list(m2.w.shape) == [4, 2, 64, 16]
    m2.w.unblock()
    assert torch.equal(m2.w.data, plain * 2)


def test_fix_linear_unquantized_keeps_blocked_weight():
    from tpp_pytorch_extension.llm.llm_common import FixLinear, BlockedLinear
    torch.manual_seed(1)
    lin = torch.nn.Linear(128, 64, bias=True)
    W = lin.weight.data.clone()
    FixLinear(lin, 16, 64, torch.float32)
    assert isinstance(lin, BlockedLinear) and list(lin.weight.shape) == [4, 2, 64, 16]
    assert torch.equal(lin.weight.data, W.view(4, 16, 2, 64).permute(0, 2, 3, 1))
    with pytest.raises(ValueError):
        FixLinear(torch.nn.Linear(64, 64), 16, 64, torch.bfloat16, weight_dtype="nf4")


def test_fix_vnni_and_block_size_rule():
    from tpp_pytorch_extension import _ops
    t = torch.arange(2 * 2 * 8 * 4 * 4, dtype=torch.float32).view(2, 2, 8, 4, 4).to(torch.bfloat16)
    v2 = _ops.fix_vnni(t)
    assert list(v2.shape) == [2, 2, 16, 4, 2]
    assert v2[1, 0, 5, 2, 1] == t[1, 0, 2, 2, 3]  # c2'=5 -> c2=2, half 1 -> c3 = 2 + 1
    assert _ops.qint8_block_size_for(4096) == 256 and _ops.qint8_block_size_for(11008) == 256
    assert _ops.qint8_block_size_for(192) == 64 and _ops.qint8_block_size_for(384) == 128


def test_launch_plans_of_the_baseline_shapes():
    """Host-side planning (no GPU work): which kernel and grid the library would launch for the BASELINE shapes --
    decode GEMMs fill one round of 256 workgroups, the prefill GEMMs get the workgroup tile whose rounds are full, the
    q/k/v GEMM the half-size workgroups that shorten its last round."""
    import ctypes
    from tpp_pytorch_extension import _lib
    L = _lib.lib()
    buf = ctypes.create_string_buffer(4096)

    def plan(fn, *args):
        _lib.check(fn(*args, buf, len(buf)))
        return buf.value.decode().strip().splitlines()

    ws = 1 << 25
    # config 2: QINT8 MLP linears
    assert "skinny_qint8_fq_kernel<3," in plan(L.tppx_plan_linear_qint8, 1, 11008, 4096, 256, 1, 0, ws)[0]
    lines = plan(L.tppx_plan_linear_qint8, 64, 4096, 11008, 256, 1, 0, ws)
    assert len(lines) == 2 and "quant_act_int8_rows_kernel" in lines[0]
    # four channel tiles x four K parts per workgroup, K in four slices across workgroups (64 groups x 4)
    assert "skinny_qint8_nk_kernel<4, 4, 4, 3, 1, 8> grid=256x1x1 block=1024" in lines[1], lines
    lines = plan(L.tppx_plan_linear_qint8, 32, 4096, 11008, 256, 1, 0, ws)
    assert "skinny_qint8_nk_kernel<2, 4, 4, 3, 1, 8> grid=256x1x1" in lines[1], lines
    lines = plan(L.tppx_plan_linear_qint8, 64, 4096, 11008, 256, 1, 0, 0)  # no workspace: no K split
    assert "skinny_qint8_kernel<4, 1, 4, 8, 8, true> grid=256x1x1" in lines[1], lines
    assert len(plan(L.tppx_plan_linear_qint8, 64, 4096, 11008, 256, 0, 0, ws)) == 1             # pre-quantized input
    # config 3 / 5: MXFP4 decode
    assert "skinny_mxfp4_x4_kernel<1, 4, false> grid=256x1x1" in plan(L.tppx_plan_linear_mxfp4, 1, 4096, 11008, 0, ws)[0]
    assert "skinny_mxfp4_xl_kernel<4, 2, false, 0, 8> grid=64x1x4" in plan(L.tppx_plan_linear_mxfp4, 16, 4096, 11008, 0, ws)[0]
    assert "skinny_mxfp4_mg_kernel<1, 1, false, 4, 16, false>" in plan(L.tppx_plan_linear_mxfp4, 16, 4096, 11008, 0, 0)[0]  # no workspace
    assert "skinny_mxfp4_xl_kernel<1, 2, false, 0, 8> grid=256x1x1" in plan(L.tppx_plan_linear_mxfp4, 16, 4096, 4096, 0, ws)[0]
    gate_up = (ctypes.c_int64 * 2)(11008, 11008)
    assert "skinny_mxfp4_xl_kernel<3, 2, true, 0, 2> grid=230x1x1" in plan(L.tppx_plan_multi_linear_mxfp4, gate_up, 2, 1, 4096, 1, 0, ws)[0]
    assert "skinny_mxfp4_mg_kernel<4, 3, true, 2, 8, true> grid=230x1x1" in plan(L.tppx_plan_multi_linear_mxfp4, gate_up, 2, 64, 4096, 1, 0, ws)[0]
    # config 4: prefill at 2048 rows
    assert "big_mxfp4_kernel<8, false, 1, 8> grid=256x1x1 block=512" in plan(L.tppx_plan_linear_mxfp4, 2048, 8192, 8192, 0, 0)[0]
    assert "big_mxfp4_kernel<8, false, 1, 8> grid=256x1x1" in plan(L.tppx_plan_linear_mxfp4, 2048, 8192, 28672, 0, 0)[0]
    qkv = (ctypes.c_int64 * 3)(8192, 1024, 1024)
    assert "big_mxfp4_kernel<8, false, 1, 4> grid=640x1x1 block=256" in plan(L.tppx_plan_multi_linear_mxfp4, qkv, 3, 2048, 8192, 0, 0, 0)[0]
    pair = (ctypes.c_int64 * 2)(28672, 28672)
    lines = plan(L.tppx_plan_multi_linear_mxfp4, pair, 2, 2048, 8192, 1, 0, 0)
    assert len(lines) == 1 and "big_mxfp4_kernel<8, true, 1, 8> grid=1792x1x1" in lines[0]       # silu*mul in the epilogue
    lines = plan(L.tppx_plan_multi_linear_mxfp4, pair, 2, 2048, 8192, 1, _lib.FLAG_ACT_FP8, 1 << 28)
    assert any("big_fp8_kernel<8, true> grid=1792x1x1" in l for l in lines), lines
    # prompts of a few hundred tokens: launches of at most 128 workgroups of 128 x 256 run as four times as many of
    # 64 x 128; up to 256 of them, as eight waves per workgroup
    assert "big_mxfp4_kernel<2, false, 2, 2> grid=256x1x1 block=256" in plan(L.tppx_plan_linear_mxfp4, 512, 4096, 4096,
                                                                             _lib.FLAG_FORCE_TILED, 0)[0]
    assert "big_mxfp4_kernel<2, false, 2, 2>" in plan(L.tppx_plan_linear_mxfp4, 512, 4096, 4096, 0, 0)[0]   # and it is the choice
    assert "big_mxfp4_kernel<4, false, 2, 4> grid=172x1x1 block=512" in plan(L.tppx_plan_linear_mxfp4, 512, 11008, 4096,
                                                                             _lib.FLAG_FORCE_TILED, 0)[0]
    pair7 = (ctypes.c_int64 * 2)(11008, 11008)
    assert "big_mxfp4_kernel<4, true, 2, 4> grid=172x1x1 block=512" in plan(L.tppx_plan_multi_linear_mxfp4, pair7, 2, 256, 4096, 1,
                                                                           _lib.FLAG_FORCE_TILED, 0)[0]
    assert "big_qint8_small_kernel grid=128x1x1 block=512" in plan(L.tppx_plan_linear_qint8, 512, 4096, 4096, 256, 1,
                                                                    _lib.FLAG_FORCE_TILED, 1 << 25)[-1]
    assert "big_qint8_kernel grid=172x1x1 block=512" in plan(L.tppx_plan_linear_qint8, 512, 11008, 4096, 256, 1,
                                                              _lib.FLAG_FORCE_TILED, 1 << 25)[-1]
    pair1 = (ctypes.c_int64 * 2)(4096, 4096)
    assert "big_mxfp4_kernel<2, true, 2, 2> grid=256x1x1 block=256" in plan(L.tppx_plan_multi_linear_mxfp4, pair1, 2, 256, 4096, 1,
                                                                           _lib.FLAG_FORCE_TILED, 0)[0]
    assert "big_mxfp4_kernel<8, false, 1, 8> grid=176x1x1 block=512" in plan(L.tppx_plan_linear_mxfp4, 1024, 11008, 4096,
                                                                             _lib.FLAG_FORCE_TILED, 0)[0]  # 128 x 512: eight waves anyway
    # from 65 rows on the 64-row forms take what the planner hands to a tiled kernel
    assert "big_mxfp4_kernel<2, false, 2, 2> grid=96x1x1 block=256" in plan(L.tppx_plan_linear_mxfp4, 160, 4096, 4096, 0, 0)[0]
    assert "skinny_mxfp4" in plan(L.tppx_plan_linear_mxfp4, 128, 4096, 4096, 0, ws)[0]
    assert "big_qint8_small_kernel grid=129x1x1 block=512" in plan(L.tppx_plan_linear_qint8, 160, 11008, 4096, 256, 1, 0, ws)[-1]
    assert "big_mxfp4_kernel<2, false, 2, 2>" in plan(L.tppx_plan_linear_mxfp4, 100, 4096, 4096, _lib.FLAG_FORCE_TILED, 0)[0]


def test_launch_plans_of_per_output_channel_qint8():
    """QINT8 with one scale block = all of K (and other multiples of 256): up to 16 rows the quantisation stays inside
    the GEMM launch (maxima exchanged between the waves), above that the big-block quantizer runs in front; all 8 or
    16 waves of a workgroup get a share of K (the grid and block are those of the 256-wide default)."""
    import ctypes
    from tpp_pytorch_extension import _lib
    L = _lib.lib()
    buf = ctypes.create_string_buffer(4096)

    def plan(*args):
        _lib.check(L.tppx_plan_linear_qint8(*args, buf, len(buf)))
        return buf.value.decode().strip().splitlines()

    ws = 1 << 25
    for M in (1, 8):
        one = plan(M, 11008, 4096, 4096, 1, 0, ws)
        assert len(one) == 1 and "skinny_qint8_fq_kernel<3, 4, 16, 16, 4, true, 8> grid=230x1x1 block=1024" in one[0], one
        one = plan(M, 4096, 11008, 11008, 1, 0, ws)
        assert len(one) == 1 and "skinny_qint8_fq_kernel<1, 4, 16, 16, 6, true, 8> grid=256x1x1 block=1024" in one[0], one
    two = plan(64, 11008, 4096, 4096, 1, 0, ws)
    assert len(two) == 2 and "quant_act_int8_bigblk_kernel grid=64x1x1 block=256" in two[0], two
    assert "skinny_qint8_kernel<4, 3, 2, 8, 8, true> grid=230x1x1 block=512" in two[1], two
    two = plan(64, 4096, 11008, 11008, 1, 0, ws)
    assert "quant_act_int8_bigblk_kernel grid=64x1x1 block=704" in two[0] and "skinny_qint8_nk_kernel<4," in two[1], two
    # a block that is not a whole number of 256-wide runs is dealt tile by tile: still one GEMM launch, quantizer in front
    odd = plan(5, 512, 1280, 320, 1, 0, ws)
    assert len(odd) == 2 and "quant_act_int8_kernel" in odd[0] and "skinny_qint8_kernel<1, 1, 4, 16, 4, true>" in odd[1], odd


def test_environment_switches_are_read_once(monkeypatch):
    """The library keeps a TPPX_* switch after its first read (no getenv per launch, and a captured graph's kernel
    choice cannot drift); tppx_reload_env() makes it read again."""
    import ctypes
    from tpp_pytorch_extension import _lib
    L = _lib.lib()
    buf = ctypes.create_string_buffer(4096)

    def plan():
        _lib.check(L.tppx_plan_linear_qint8(1, 4096, 4096, 256, 1, 0, 0, buf, len(buf)))
        return buf.value.decode()

    L.tppx_reload_env()
    assert "skinny_qint8_fq_kernel" in plan()
    os.environ["TPPX_SKINNY_FUSEDQ"] = "0"
    try:
        assert "skinny_qint8_fq_kernel" in plan(), "the switch was read again without a reload"
        L.tppx_reload_env()
        assert "skinny_qint8_fq_kernel" not in plan() and "quant_act_int8" in plan()
    finally:
        del os.environ["TPPX_SKINNY_FUSEDQ"]
        L.tppx_reload_env()
    assert "skinny_qint8_fq_kernel" in plan()


def test_cache_lengths_after_graph_replayed_steps():
    """Steps replayed from a graph move the device counter themselves; the host bookkeeping that follows them must
    move every layer's length, so that get_seq_length(layer) and a later update() on any layer see the new keys."""
    from tpp_pytorch_extension.llm.fused_llama_infer import TppCache
    cache = TppCache(64)
    kv = torch.zeros((1, 2, 5, 8), dtype=torch.bfloat16)
    for i in range(3):
        cache.fill_(i, kv, kv)
    cache._advance_host(4)  # what greedy_decode / time_decode_steps do per replay
    assert [cache.get_seq_length(i) for i in range(3)] == [9, 9, 9]
    one = torch.ones((1, 2, 1, 8), dtype=torch.bfloat16)
    k, v = cache.update(one, one, 2)
    assert k.shape[2] == 10 and cache.get_seq_length(2) == 10 and cache.get_seq_length(1) == 9
    assert float(k[0, 0, 9, 0]) == 1.0 and float(k[0, 0, 8, 0]) == 0.0


def test_qwen2_front_end_surface():
    """The Qwen2 front-end mirrors the reference module's names (fused_qwen2_infer.py:45-238) and checks its
    parameter list without touching a GPU."""
    from tpp_pytorch_extension.llm import fused_qwen2_infer as Q
    from tpp_pytorch_extension.llm import fused_llama_infer as F
    from tpp_pytorch_extension._lib import TppxError
    for name in ("Qwen2DecoderLayer", "FixQwen2DecoderLayer", "OptimizeModelForQwen2", "Qwen2Model_forward", "TppCache"):
        assert hasattr(Q, name), name
    assert issubclass(Q.Qwen2DecoderLayer, F.LlamaDecoderLayer)
    with pytest.raises(TppxError):
        Q.Qwen2DecoderLayer([None] * 10, 0, 1e-6, 128, 64, 128)  # the Llama list: three biases short


def test_gptj_and_opt_front_end_surface():
    """The GPT-J and OPT front-ends mirror the reference modules' names (fused_gptj_infer.py:46-193,
    fused_opt_infer.py:45-203) and check their parameter lists without touching a GPU."""
    from tpp_pytorch_extension.llm import fused_gptj_infer as G
    from tpp_pytorch_extension.llm import fused_opt_infer as P
    from tpp_pytorch_extension._lib import TppxError
    for name in ("GPTJBlock", "FixGPTJBlock", "OptimizeModelForGPTJ", "GPTJModel_forward", "create_sinusoidal_positions"):
        assert hasattr(G, name), name
    for name in ("OPTDecoderLayer", "FixOPTDecoderLayer", "OptimizeModelForOPT", "OPTDecoder_forward"):
        assert hasattr(P, name), name
    with pytest.raises(TppxError):
        G.GPTJBlock([None] * 10, 0, 1e-5, 256, 2048, 64)
    with pytest.raises(TppxError):
        P.OPTDecoderLayer([None] * 11, 0, 1e-5, 1e-5, 64, True)
    t = G.create_sinusoidal_positions(8, 4)  # sin | cos of position * 10000^(-2i/dim)
    assert t.shape == (8, 4) and torch.allclose(t[0], torch.tensor([0.0, 0.0, 1.0, 1.0]))
    assert torch.allclose(t[3, :2], torch.sin(torch.tensor([3.0, 0.03]))) and torch.allclose(t[3, 2:], torch.cos(torch.tensor([3.0, 0.03])))


def test_common_module_helpers_one_process():
    """llm_common's process-group helpers in their one-process form, ShardLinear as pure slicing (the shards of all
    ranks tile the weight; a row-parallel split sums back to the whole linear), BlockedLayerNorm on the CPU."""
    import copy
    from tpp_pytorch_extension.llm import llm_common as C
    assert C.get_rank() == 0 and C.get_size() == 1
    C.set_pg()
    t = torch.arange(4.0)
    assert C.all_reduce(t) is t and C.shm_allreduce(t) is t
    torch.manual_seed(3)
    lin = torch.nn.Linear(96, 160)
    x = torch.randn(5, 96)
    full = lin(x)
    def shard(dim, r, size, bs):
        m = copy.deepcopy(lin)
        C.ShardLinear(m, dim, r, size, bs)  # in place, like the reference's
        return m

    cols = [shard(0, r, 3, 32) for r in range(3)]
    assert cols[0].split_sizes == [32, 64, 64] and [c.weight.shape[0] for c in cols] == [32, 64, 64]
    assert torch.equal(torch.cat([c.weight.data for c in cols]), lin.weight.data)
    assert torch.allclose(torch.cat([torch.nn.functional.linear(x, c.weight, c.bias) for c in cols], -1), full, atol=1e-6)
    rows = [shard(1, r, 3, 32) for r in range(3)]
    assert rows[0].split_sizes == [32, 32, 32]
    parts = [torch.nn.functional.linear(x[:, 32 * r:32 * r + 32], m.weight, m.bias) for r, m in enumerate(rows)]
    assert torch.allclose(sum(parts), full, atol=1e-5)  # the bias was divided by the number of ranks
    with pytest.raises(ValueError):
        shard(0, 0, 2, 64)  # 160 is not a multiple of 64
    ln = C.BlockedLayerNorm(64)
    y = ln(torch.randn(3, 64))
    assert torch.allclose(y.mean(-1), torch.zeros(3), atol=1e-5)
    assert C.compare(t, t.clone(), "same") is True and C.compare(t, t + 1, "shifted") is False


def test_cache_allocates_small_layers_together():
    """Layers of a small KV cache share one zeroed allocation (up to eight layers, keys and values), handed out as
    the layers ask for storage; a layer of another shape, or a cache whose layers are large, allocates on its own."""
    import torch
    from tpp_pytorch_extension.llm.fused_llama_infer import TppCache
    c = TppCache(48)
    got = [c._ensure(i, 2, 4, 16, "cpu") for i in range(10)]
    base = got[0][0].untyped_storage().data_ptr()
    assert all(k.untyped_storage().data_ptr() == base and v.untyped_storage().data_ptr() == base for k, v in got[:8])
    assert got[8][0].untyped_storage().data_ptr() != base           # ninth layer: the next group
    ptrs = {t.data_ptr() for kv in got for t in kv}
    assert len(ptrs) == 20                                          # no two layers share memory
    for k, v in got:
        assert k.shape == (2, 4, 48, 16) and k.is_contiguous() and v.is_contiguous()
        assert not k.any() and not v.any()
    assert c._ensure(3, 2, 4, 16, "cpu")[0].data_ptr() == got[3][0].data_ptr()   # a layer keeps its storage
    k, _ = c._ensure(10, 1, 4, 16, "cpu")                            # another shape: not the waiting storage
    assert k.shape == (1, 4, 48, 16) and not k.any()
    big = TppCache(48)
    big.SLAB_BYTES = 4 * 2 * 4 * 48 * 16                            # room for one layer only
    a, b = big._ensure(0, 2, 4, 16, "cpu"), big._ensure(1, 2, 4, 16, "cpu")
    assert a[0].untyped_storage().data_ptr() != b[0].untyped_storage().data_ptr() and not big._spare
