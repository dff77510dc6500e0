"""Operator layer: the reference's ``torch.ops.tpp_llm`` entry point plus the
post-op variants the decoder layer uses, and the ``_C._qtype`` helper set.

Every function here validates, allocates the output with torch and enqueues
HIP kernels through the C ABI on the current stream.  Nothing computes on the
host.
"""
import ctypes
import os

import torch

from . import _lib
from ._lib import (POST_NONE, POST_SILU, POST_MUL, POST_ADD_SCALE, POST_ADD2_SCALE, POST_GELU,
                   POST_RELU, TppxError)
from ._qtensor import QTensor, QSCHEME_MXFP, QSCHEME_AFFINE

# QINT8_BLOCK_SIZE is read once at import like the reference's file-static
# (src/csrc/qtypes.cpp:28).
QINT8_BLOCK_SIZE = int(os.environ.get("QINT8_BLOCK_SIZE", "256"))


# ----------------------------------------------------------------------------
# quantize / remap helpers  (reference: pybind submodule _qtype, qtypes.cpp:1075-1093)
# ----------------------------------------------------------------------------
def _blocked_geometry(t):
    """(N, K, bk, bc, vnni) of a blocked weight [N/bk, K/bc, bc/v, bk, v] or [N/bk, K/bc, bc, bk]."""
    if t.dim() == 5:
        n1, c1, c2, k2, c3 = t.shape
        return n1 * k2, c1 * c2 * c3, k2, c2 * c3, c3
    if t.dim() == 4:
        n1, c1, c2, k2 = t.shape
        return n1 * k2, c1 * c2, k2, c2, 1
    if t.dim() == 2:
        return t.shape[0], t.shape[1], 1, t.shape[1], 1
    raise TppxError(_lib.ESHAPE, f"expected a 4-D or 5-D blocked weight, got shape {tuple(t.shape)}")


def _float_weight_on_gpu(t):
    if isinstance(t, QTensor):
        raise TppxError(_lib.EINVAL, "weight is already quantized")
    t = t.detach()
    if t.dtype == torch.bfloat16:
        dt = _lib.DT_BF16
    elif t.dtype == torch.float32:
        dt = _lib.DT_F32
    else:
        raise TppxError(_lib.EUNSUPPORTED, f"Unknown dtype for quantization: {t.dtype}")
    if not t.is_cuda:
        if not torch.cuda.is_available():
            _lib.require_gpu(t, "weight to quantize")
        t = t.cuda()
    return t.contiguous(), dt


# USE_MXFP4_INT8 (qtypes.cpp:31): remap_and_quantize_mxfp4 produces the VNNI8-interleaved layout whose GEMM runs on
# int8 activations (W4A8)
USE_MXFP4_INT8 = os.environ.get("USE_MXFP4_INT8", "0") not in ("0", "")


def _remap_mxfp4_int8(t):
    """The USE_MXFP4_INT8 branch of remap_and_quantize_mxfp4 (qtypes.cpp:787-790, 792-861): N blocks of 8 channels,
    K in groups of 8 ordered 0,4,1,5,2,6,3,7 (a packed byte holds values i and 4 + i), then quantize_mxfp4(t, 32,
    2, true) -> quint4x2 [N/8, K/bc, bc/8, 8, 8] with E8M0 scales [N/8, K/bc, bc/32, 8]."""
    t, _ = _float_weight_on_gpu(t)
    N, K, bk, bc, vnni = _blocked_geometry(t)
    if t.dim() == 4 and bc % 8:
        raise TppxError(_lib.ESHAPE, "Shape not compatible for VNNI2")
    if (bk < 8 and (8 % bk or (N // bk) % (8 // bk))) or (bk > 8 and bk % 8):
        raise TppxError(_lib.ESHAPE, "Shape not compatible for MXFP4")
    if bc % 32 or N % 16:
        raise TppxError(_lib.ESHAPE, "Shape not compatible for VNNI8")
    C1 = K // bc
    if t.dim() == 5:
        W = t.permute(0, 3, 1, 2, 4).reshape(N, K)   # [N/bk][K/bc][bc/vnni][bk][vnni] -> plain rows
    else:
        W = t.permute(0, 3, 1, 2).reshape(N, K)      # [N/bk][K/bc][bc][bk]
    g = W.reshape(N // 8, 8, C1, bc // 8, 2, 4).permute(0, 2, 3, 1, 5, 4).reshape(N // 8, C1, bc // 8, 8, 8).contiguous()
    return _quantize_generic(g, 32, 2, True, _lib.Q_MXFP4)


def remap_and_quantize_mxfp4(t, int8_layout=None):
    """Reference: remap_and_quantize_mxfp4 (src/csrc/qtypes.cpp:783-864).
    Blocked bf16 5-D / fp32 4-D weight -> quint4x2 tensor [N/32, K/64, 32, 32, 2]; with int8_layout (default: the
    USE_MXFP4_INT8 environment flag) the W4A8 layout [N/8, K/bc, bc/8, 8, 8]."""
    if USE_MXFP4_INT8 if int8_layout is None else int8_layout:
        return _remap_mxfp4_int8(t)
    L = _lib.lib()
    t, dt = _float_weight_on_gpu(t)
    N, K, bk, bc, vnni = _blocked_geometry(t)
    if t.dim() == 4 and bc % 2:
        raise TppxError(_lib.ESHAPE, "Shape not compatible for VNNI2")
    if bk < 32 and (32 % bk or (N // bk) % (32 // bk)):
        raise TppxError(_lib.ESHAPE, "Shape not compatible for MXFP4")
    if bc != 64:
        raise TppxError(_lib.EUNSUPPORTED, f"MXFP4 weights are built for input-channel blocks of 64 (got {bc})")
    if N % 32 or K % 64:
        raise TppxError(_lib.ESHAPE, "Shape not compatible for MXFP4")
    q = torch.empty((N // 32, K // 64, 32, 32), dtype=torch.uint8, device=t.device)
    sc = torch.empty((N // 32, K // 64, 2, 32), dtype=torch.uint8, device=t.device)
    _lib.check(L.tppx_quantize_mxfp4(t.data_ptr(), dt, N, K, bk, bc, vnni, q.data_ptr(), sc.data_ptr(),
                                     _lib.stream_of(t)))
    return QTensor(q, sc, (N // 32, K // 64, 32, 32, 2), torch.quint4x2, QSCHEME_MXFP, 32, 2, True, 2)


def qint8_block_size_for(K):
    """Block-size rule of remap_and_quantize_qint8 (qtypes.cpp:878-889)."""
    if K % QINT8_BLOCK_SIZE == 0:
        return QINT8_BLOCK_SIZE
    q = 4096
    while q >= 64:
        if QINT8_BLOCK_SIZE > q and K % q == 0:
            return q
        q //= 2
    raise TppxError(_lib.ESHAPE, f"no QINT8 block size divides K={K}")


def remap_and_quantize_qint8(t):
    """Reference: remap_and_quantize_qint8 (src/csrc/qtypes.cpp:866-932).
    -> qint8 tensor [N/16, K/QBS, QBS/4, 16, 4] with fp32 scales [N/16, K/QBS, 1, 16]."""
    L = _lib.lib()
    t, dt = _float_weight_on_gpu(t)
    N, K, bk, bc, vnni = _blocked_geometry(t)
    # any blocking of the source is read; the quantized tensor always has 16-channel blocks (the reference keeps
    # the source's: quantizing the 100-channel-blocked lm_head gives [N/100, K/QBS, QBS/4, 100, 4] there), with the
    # same values and per-(channel, K block) scales
    if N % 16:
        raise TppxError(_lib.ESHAPE, f"QINT8 weights need a multiple of 16 output channels (got {N})")
    if 4 % vnni:
        raise TppxError(_lib.ESHAPE, "Shape not compatible for VNNI4")
    qbs = qint8_block_size_for(K)
    q = torch.empty((N // 16, K // qbs, qbs // 4, 16, 4), dtype=torch.int8, device=t.device)
    sc = torch.empty((N // 16, K // qbs, 1, 16), dtype=torch.float32, device=t.device)
    _lib.check(L.tppx_quantize_qint8(t.data_ptr(), dt, N, K, bk, bc, vnni, qbs, q.data_ptr(),
                                     sc.data_ptr(), _lib.stream_of(t)))
    return QTensor(q, sc, tuple(q.shape), torch.qint8, QSCHEME_AFFINE, qbs, 2, True, 1)


def _per_block_geometry(shape, block_size, axis, is_vnni, pack):
    """(pre, bs, post, vnni, scale_sizes) as PerBlockQuantizer derives them (src/csrc/qtypes.h:30-68)."""
    sizes = list(shape)
    if axis < 0:
        axis += len(sizes)
    if is_vnni:
        vnni = sizes.pop()
    else:
        if axis != len(sizes) - 1:
            raise TppxError(_lib.EINVAL, f"Invalid axis {axis}")
        if sizes[axis] % pack:
            raise TppxError(_lib.ESHAPE, "Invalid dim size")
        vnni = pack
        sizes[axis] //= pack
    if block_size % vnni:
        raise TppxError(_lib.ESHAPE, "Block size must be multiple of VNNI pack size")
    bsi = block_size // vnni
    if not (0 <= axis < len(sizes)):
        raise TppxError(_lib.EINVAL, "Invalid axis")
    if sizes[axis] % bsi:
        raise TppxError(_lib.ESHAPE, "Axis size must be multiple of block_size")
    sizes[axis] //= bsi
    pre = 1
    for d in sizes[: axis + 1]:
        pre *= d
    post = 1
    for d in sizes[axis + 1:]:
        post *= d
    return pre, bsi, post, vnni, sizes, axis


def _quantize_generic(t, block_size, axis, is_vnni, fmt):
    """quantize_mxfp4 / quantize_int8sym / quantize_int4sym on any layout (PerBlockQuantizer::quantize_symetric,
    src/csrc/qtypes.h:133-193): the generic per-block kernel."""
    L = _lib.lib()
    if isinstance(t, QTensor):
        raise TppxError(_lib.EINVAL, "tensor is already quantized")
    if t.dtype not in (torch.bfloat16, torch.float32):
        raise TppxError(_lib.EUNSUPPORTED, f"Unsupported input type for quantization: {t.dtype}")
    _lib.require_gpu(t, "tensor to quantize")
    t = t.detach().contiguous()
    pack = 1 if fmt == _lib.Q_INT8 else 2
    pre, bs, post, vnni, ssz, axis = _per_block_geometry(t.shape, block_size, axis, is_vnni, pack)
    if pack == 2 and vnni % 2:
        raise TppxError(_lib.ESHAPE, "4-bit formats pack two codes per byte: the packed dimension must be even")
    qshape = tuple(t.shape[:-1]) + (t.shape[-1] // pack,)
    q = torch.empty(qshape, dtype=torch.int8 if fmt == _lib.Q_INT8 else torch.uint8, device=t.device)
    sc = torch.empty(tuple(ssz), dtype=torch.uint8 if fmt == _lib.Q_MXFP4 else torch.float32, device=t.device)
    if t.numel():
        dt = _lib.DT_BF16 if t.dtype == torch.bfloat16 else _lib.DT_F32
        _lib.check(L.tppx_quantize_per_block(t.data_ptr(), dt, fmt, pre, bs, post, vnni, q.data_ptr(), sc.data_ptr(),
                                             _lib.stream_of(t)))
    if fmt == _lib.Q_MXFP4:
        return QTensor(q, sc, tuple(t.shape), torch.quint4x2, QSCHEME_MXFP, block_size, axis, is_vnni, 2)
    if fmt == _lib.Q_INT8:
        return QTensor(q, sc, tuple(t.shape), torch.qint8, QSCHEME_AFFINE, block_size, axis, is_vnni, 1)
    return QTensor(q, sc, tuple(t.shape), torch.quint4x2, QSCHEME_AFFINE, block_size, axis, is_vnni, 2)


def quantize_mxfp4(t, block_size, axis, is_vnni):
    """Reference: quantize_mxfp4 (qtypes.cpp:602-611).  The layout remap_and_quantize_mxfp4 feeds it
    ([N/32, K/64, 32, 32, 2], block 32, axis 2, VNNI) takes the weight kernel; any other layout the generic
    per-block kernel (same bytes)."""
    if axis < 0:
        axis += t.dim()
    if t.dim() == 5 and tuple(t.shape[2:]) == (32, 32, 2) and block_size == 32 and axis == 2 and is_vnni and t.shape[1] > 0:
        L = _lib.lib()
        t, dt = _float_weight_on_gpu(t)
        N, K = t.shape[0] * 32, t.shape[1] * 64
        q = torch.empty((N // 32, K // 64, 32, 32), dtype=torch.uint8, device=t.device)
        sc = torch.empty((N // 32, K // 64, 2, 32), dtype=torch.uint8, device=t.device)
        # the input is already [N/32][K/64][32][32][2]: bk=32, bc=64, vnni=2
        _lib.check(L.tppx_quantize_mxfp4(t.data_ptr(), dt, N, K, 32, 64, 2, q.data_ptr(), sc.data_ptr(), _lib.stream_of(t)))
        return QTensor(q, sc, (N // 32, K // 64, 32, 32, 2), torch.quint4x2, QSCHEME_MXFP, 32, 2, True, 2)
    qt = _quantize_generic(t, block_size, axis, is_vnni, _lib.Q_MXFP4)
    return qt


def quantize_mxfp(t, block_size, axis, is_vnni, dtype):
    """Reference: quantize_mxfp (qtypes.cpp:592-600); only the E2M1 element type exists there too
    (PerBlockMxFPQuantizer::quantize asserts on anything but kQUInt4x2, qtypes.cpp:430-432)."""
    if dtype != torch.quint4x2:
        raise TppxError(_lib.EUNSUPPORTED, "Unsupported MXFP datatype")
    return quantize_mxfp4(t, block_size, axis, is_vnni)


def quantize_int8sym(t, block_size, axis, is_vnni):
    """Reference: quantize_int8sym (qtypes.cpp:613-624).  The VNNI4 weight [N/16, K/QBS, QBS/4, 16, 4] (axis 2) and
    row-major bf16 activations quantized along the last axis take their own kernels; every other layout the generic
    per-block kernel (same bytes)."""
    L = _lib.lib()
    if axis < 0:
        axis += t.dim()
    if is_vnni and t.dim() == 5 and tuple(t.shape[3:]) == (16, 4) and axis == 2 and t.shape[2] * 4 == block_size \
            and block_size % 64 == 0:
        t, dt = _float_weight_on_gpu(t)
        N, K = t.shape[0] * 16, t.shape[1] * block_size
        q = torch.empty(tuple(t.shape), dtype=torch.int8, device=t.device)
        sc = torch.empty((t.shape[0], t.shape[1], 1, 16), dtype=torch.float32, device=t.device)
        # the input is already [N/16][K/QBS][QBS/4][16][4]: bk=16, bc=QBS, vnni=4
        _lib.check(L.tppx_quantize_qint8(t.data_ptr(), dt, N, K, 16, block_size, 4, block_size,
                                         q.data_ptr(), sc.data_ptr(), _lib.stream_of(t)))
        return QTensor(q, sc, tuple(q.shape), torch.qint8, QSCHEME_AFFINE, block_size, 2, True, 1)
    if (not is_vnni) and axis == t.dim() - 1 and t.dtype == torch.bfloat16 and t.is_cuda and block_size % 64 == 0 \
            and t.shape[-1] % block_size == 0 and t.numel() > 0:
        K = t.shape[-1]
        t = t.contiguous()
        M = t.numel() // K
        xq = torch.empty(tuple(t.shape), dtype=torch.int8, device=t.device)
        sa = torch.empty(tuple(t.shape[:-1]) + (K // block_size,), dtype=torch.float32, device=t.device)
        _lib.check(L.tppx_quant_act_int8(t.data_ptr(), M, K, block_size, xq.data_ptr(), sa.data_ptr(),
                                         _lib.stream_of(t)))
        return QTensor(xq, sa, tuple(t.shape), torch.qint8, QSCHEME_AFFINE, block_size, axis, False, 1)
    return _quantize_generic(t, block_size, axis, is_vnni, _lib.Q_INT8)


def quantize_int4sym(t, block_size, axis, is_vnni):
    """Reference: quantize_int4sym (qtypes.cpp:626-637; Int4SymQuant :199-246): scale = max/7, codes in [-8, 7],
    two per byte.  A weight in the VNNI2 layout [N/16, K/QBS, QBS/2, 16, 2] (axis 2) is accepted by the linears."""
    return _quantize_generic(t, block_size, axis, is_vnni, _lib.Q_INT4)


def create_qtensor_int8sym(val, scales, block_size, axis, is_vnni):
    """Reference: create_qtensor_int8sym (qtypes.cpp:654-668): wrap caller-supplied int8 values + fp32 scales."""
    if val.dtype != torch.int8 or scales.dtype != torch.float32:
        raise TppxError(_lib.EINVAL, "create_qtensor_int8sym expects int8 values and float32 scales")
    if axis < 0:
        axis += val.dim()
    return QTensor(val.contiguous(), scales.contiguous(), tuple(val.shape), torch.qint8, QSCHEME_AFFINE,
                   block_size, axis, is_vnni, 1)


def create_qtensor_int2sym(sizes, val, scales, block_size, axis, is_vnni):
    """Reference: create_qtensor_int2sym (qtypes.cpp:686-702): wrap caller-supplied packed 2-bit codes (uint8, four
    per byte) + fp32 scales as a kQUInt2x4 tensor of logical shape `sizes`."""
    if val.dtype != torch.uint8 or scales.dtype != torch.float32:
        raise TppxError(_lib.EINVAL, "create_qtensor_int2sym expects uint8 values and float32 scales")
    sizes = tuple(int(d) for d in sizes)
    if axis < 0:
        axis += len(sizes)
    return QTensor(val.contiguous(), scales.contiguous(), sizes, torch.quint2x4, QSCHEME_AFFINE, block_size, axis,
                   is_vnni, 4)


QINT2_BLOCK_SIZE = int(os.environ.get("QINT2_BLOCK_SIZE", "256"))


def qint2_block_size_for(K):
    """Block-size rule of remap_and_quantize_qint2_intlv (qtypes.cpp:1031-1043)."""
    if K % QINT2_BLOCK_SIZE == 0:
        return QINT2_BLOCK_SIZE
    q = 4096
    while q >= 64:
        if QINT2_BLOCK_SIZE > q and K % q == 0:
            return q
        q //= 2
    raise TppxError(_lib.ESHAPE, f"no QINT2 block size divides K={K}")


def remap_and_quantize_qint2_intlv(t):
    """Reference: remap_and_quantize_qint2_intlv (src/csrc/qtypes.cpp:1004-1073), the "qint2" choice of FixLinear:
    ternary weights, four codes per byte interleaved over output channels.
    -> quint2x4 tensor of logical shape [N/32, K/QBS, QBS/4, 32, 4]; packed bytes [N/32, K/QBS, QBS/4, 8, 4];
    fp32 scales [N/32, K/QBS, 32, 1].  (TPP_QINT2_AS_QINT1 is not built.)"""
    L = _lib.lib()
    if os.environ.get("TPP_QINT2_AS_QINT1", "0") not in ("0", ""):
        raise TppxError(_lib.EUNSUPPORTED, "TPP_QINT2_AS_QINT1 (1-bit weights) is not built")
    t, dt = _float_weight_on_gpu(t)
    N, K, bk, bc, vnni = _blocked_geometry(t)
    if N % 32:
        raise TppxError(_lib.EUNSUPPORTED, f"QINT2 weights are built for a multiple of 32 output channels (got {N})")
    if K % 4:
        raise TppxError(_lib.ESHAPE, "C must be multiple of 4")
    bs = qint2_block_size_for(K)
    q = torch.empty((N // 32, K // bs, bs // 4, 8, 4), dtype=torch.uint8, device=t.device)
    sc = torch.empty((N // 32, K // bs, 32, 1), dtype=torch.float32, device=t.device)
    _lib.check(L.tppx_quantize_qint2_intlv(t.data_ptr(), dt, N, K, bk, bc, vnni, bs, q.data_ptr(), sc.data_ptr(),
                                           _lib.stream_of(t)))
    return create_qtensor_int2sym((N // 32, K // bs, bs // 4, 32, 4), q, sc, bs, 2, True)


def _as_q(t):
    if not isinstance(t, QTensor):
        raise TppxError(_lib.EINVAL, "expected a per-block quantized tensor")
    return t


def q_per_block_scales(t):
    return _as_q(t).scales


def q_per_block_pack_size(t):
    return _as_q(t).pack_size


def q_per_block_block_size(t):
    return _as_q(t).block_size


def q_per_block_axis(t):
    return _as_q(t).axis


def q_per_block_qval(t):
    """Packed storage in the reference layout: int8 values for qint8, the
    packed uint8 bytes [N/32, K/64, 32, 32] for quint4x2."""
    return _as_q(t).qdata


def fix_vnni(t):
    """Reference: fix_vnni (qtypes.cpp:740-781): pure re-layout of an unquantized blocked weight."""
    dims = t.dim()
    if dims < 4:
        raise TppxError(_lib.ESHAPE, f"Invalid shape, dims = {dims}")
    K1, C1, C2, K2 = t.shape[:4]
    C3 = t.shape[4] if dims == 5 else 1
    if t.dtype == torch.bfloat16:
        if C3 == 2:
            return t
        if C3 == 4:
            return (t.view(K1, C1, C2, K2, 2, 2).permute(0, 1, 2, 4, 3, 5).contiguous()
                    .view(K1, C1, C2 * 2, K2, 2))
        if C3 == 1:
            if C2 % 2:
                raise TppxError(_lib.ESHAPE, f"Shape incompatible for VNNI2 layout, C2 = {C2}")
            return t.view(K1, C1, C2 // 2, 2, K2).permute(0, 1, 2, 4, 3).contiguous()
        raise TppxError(_lib.ESHAPE, "Shape incompatible for VNNI2 layout")
    if t.dtype == torch.float32:
        if C3 == 1 and dims == 4:
            return t
        if C3 == 1:
            return t.view(K1, C1, C2, K2)
        return t.permute(0, 1, 2, 4, 3).contiguous().view(K1, C1, C2 * C3, K2)
    raise TppxError(_lib.EUNSUPPORTED, "Unknown dtype for FIX_VNNI layout")


# ----------------------------------------------------------------------------
# linears
# ----------------------------------------------------------------------------
def _prep_input(input, weight):
    if not isinstance(weight, QTensor):
        raise TppxError(
            _lib.EUNSUPPORTED,
            "only MXFP4 / QINT8 quantized and bfloat16 weights are built on this path "
            "(quantize the weight with remap_and_quantize_mxfp4 / remap_and_quantize_qint8)",
        )
    if not weight.is_weight():
        raise TppxError(_lib.EUNSUPPORTED, f"Unsupported qscheme / layout for a linear weight: {weight!r}")
    _lib.require_gpu(weight.qdata, "weight")
    if isinstance(input, QTensor):
        raise TppxError(_lib.EUNSUPPORTED, "pre-quantized activations go through linear() / fc_plain() only")
    _lib.require_gpu(input, "input")
    if input.dtype != torch.bfloat16:
        raise TppxError(_lib.EUNSUPPORTED,
                        f"this operator takes bfloat16 activations (got {input.dtype}); float / half activations and "
                        f"pre-quantized qint8 activations are built for fc_plain / linear without a post-op on "
                        f"QINT8-family weights")
    N, K = weight.weight_nk()
    if input.shape[-1] != K:
        raise TppxError(_lib.ESHAPE, f"input has {input.shape[-1]} features, weight expects {K}")
    x = input.contiguous()
    M = x.numel() // K
    return x, M, N, K


def _bf16_native(weight):
    """Native tiles of an unquantized bf16 weight (blocked 5-D / 4-D or plain 2-D), made on first use and kept on
    the tensor (the role of the reference's cached first-token remap)."""
    key = (weight.data_ptr(), weight._version)
    have = getattr(weight, "_tppx_native_bf16", None)
    if have is not None and have[0] == key:
        return have[1]
    N, K, bk, bc, v = _blocked_geometry(weight)
    _lib.require_gpu(weight, "weight")
    w = weight.detach().contiguous()
    nat = torch.empty(N * K, dtype=torch.bfloat16, device=w.device)
    _lib.check(_lib.lib().tppx_prepack_bf16(w.data_ptr(), N, K, bk, bc, v, nat.data_ptr(), _lib.stream_of(w)))
    weight._tppx_native_bf16 = (key, nat)
    return nat


def _linear_bf16(input, weight, bias, post, post_in, post_in2, post_scale, flags):
    """TppBlockedLinearW<bf16,bf16> (src/csrc/fused_gemm.h:785-1073): unquantized bf16 weight."""
    if isinstance(input, QTensor):
        raise TppxError(_lib.EUNSUPPORTED, "pre-quantized activations are not built; pass bfloat16")
    _lib.require_gpu(input, "input")
    if input.dtype != torch.bfloat16:
        raise TppxError(_lib.EUNSUPPORTED, f"bfloat16 weights take bfloat16 activations (got {input.dtype})")
    N, K = _blocked_geometry(weight)[:2]
    if input.shape[-1] != K:
        raise TppxError(_lib.ESHAPE, f"input has {input.shape[-1]} features, weight expects {K}")
    x = input.contiguous()
    M = x.numel() // K
    y = torch.empty(tuple(input.shape[:-1]) + (N,), dtype=torch.bfloat16, device=x.device)
    if M == 0:
        return y
    bias = _prep_bias(bias, N, x.device)
    post_in = _prep_post(post_in, M, N, "post-op input", x.device)
    post_in2 = _prep_post(post_in2, M, N, "second post-op input", x.device)
    nat = _bf16_native(weight)
    _lib.check(_lib.lib().tppx_linear_bf16(x.data_ptr(), nat.data_ptr(), _lib.ptr(bias), _lib.ptr(post_in),
                                           _lib.ptr(post_in2), y.data_ptr(), M, N, K, post, post_scale, flags,
                                           _lib.stream_of(x)))
    return y


def _prep_bias(bias, N, dev):
    if bias is None or bias.numel() == 0:
        return None
    if bias.numel() != N:
        raise TppxError(_lib.ESHAPE, f"bias has {bias.numel()} elements, expected {N}")
    if bias.dtype != torch.bfloat16 or bias.device != dev:
        bias = bias.to(device=dev, dtype=torch.bfloat16)
    return bias.contiguous()


def _prep_post(t, M, N, name, dev):
    if t is None:
        return None
    if t.numel() != M * N or t.shape[-1] != N:
        raise TppxError(_lib.ESHAPE, f"{name} must have the output's shape [..., {N}] with {M} rows, got {tuple(t.shape)}")
    if t.dtype != torch.bfloat16 or t.device != dev:
        raise TppxError(_lib.EINVAL, f"{name} must be a bfloat16 tensor on {dev}")
    return t.contiguous()


def _qint8_scratch(x, M, K, qbs):
    # the library may lay the quantized rows out in 64-row operand tiles
    xq = torch.empty(((M + 63) // 64 * 64, K), dtype=torch.int8, device=x.device)
    sa = torch.empty(((M + 63) // 64 * 64, K // qbs), dtype=torch.float32, device=x.device)
    return xq, sa


# Opt-in (TPPX_ACT_FP8=1, or flags=FLAG_ACT_FP8 on linear()): MXFP4 GEMMs with more than 64 rows quantize their
# activations to MXFP8 and run on the block-scaled MFMA.  Not the reference's arithmetic (its activations stay bf16).
ACT_FP8 = os.environ.get("TPPX_ACT_FP8", "0") == "1"


def _mxfp4_flags_ws(x, M, K, flags=0):
    """(flags, workspace) of an MXFP4 call: the FP8-activation path keeps the quantised activations in the workspace."""
    if ACT_FP8 and M > 64:
        flags |= _lib.FLAG_ACT_FP8
    ws = _lib.workspace(x)
    if flags & _lib.FLAG_ACT_FP8:
        Mp = (M + 63) // 64 * 64
        need = Mp * K + Mp * (K // 32)
        if need > ws.numel():
            ws = torch.empty(need, dtype=torch.uint8, device=x.device)
    return flags, ws


def _wide_post(acc, ctype, post, post_in, post_in2, post_scale, shape):
    """fp32 GEMM tile (bias + dot) -> the activations' type with the post-op applied there (tppx_post_op_wide)."""
    L = _lib.lib()
    if ctype == torch.float32 and post == POST_NONE:
        return acc.view(shape)
    out = torch.empty(shape, dtype=ctype, device=acc.device)
    ins = []
    for t, need in ((post_in, post in (POST_MUL, POST_ADD_SCALE, POST_ADD2_SCALE)), (post_in2, post == POST_ADD2_SCALE)):
        if not need:
            ins.append(None)
            continue
        if t is None or tuple(t.shape) != tuple(shape) or t.device != acc.device:
            raise TppxError(_lib.ESHAPE, f"post-op {post} needs an input of the output's shape {tuple(shape)} on {acc.device}")
        ins.append(t.to(ctype).contiguous())
    if out.numel():
        _lib.check(L.tppx_post_op_wide(acc.data_ptr(), _lib.DT_F16 if ctype == torch.float16 else _lib.DT_F32, post,
                                       _lib.ptr(ins[0]), _lib.ptr(ins[1]), float(post_scale), out.data_ptr(),
                                       out.numel(), _lib.stream_of(acc)))
    return out


def _linear_wide(input, weight, bias, post, post_in, post_in2, post_scale):
    """float / half activations on an MXFP4 or an unquantized bf16 weight: TppBlockedLinearW<Tin, uint8_t, Tout> /
    <Tin, bfloat16, Tout> with Tin = float or half (src/csrc/fused_gemm.h:1519-1523, 1541-1550).  The activations are
    NOT rounded to bf16: fp32 products and sums (every weight value is exact in fp32), output and post-op in the
    activations' type."""
    L = _lib.lib()
    _lib.require_gpu(input, "input")
    ctype = input.dtype
    if isinstance(weight, QTensor):
        N, K = weight.weight_nk()
        qn, sn = weight.native()
        kind = _lib.W_MXFP4
    else:
        N, K = _blocked_geometry(weight)[:2]
        qn, sn, kind = _bf16_native(weight), None, _lib.W_BF16
    if input.shape[-1] != K:
        raise TppxError(_lib.ESHAPE, f"input has {input.shape[-1]} features, weight expects {K}")
    x = input.contiguous()
    M = x.numel() // K
    shape = tuple(input.shape[:-1]) + (N,)
    acc = torch.empty((M, N), dtype=torch.float32, device=x.device)
    if M:
        b = None
        if bias is not None and bias.numel():
            if bias.numel() != N:
                raise TppxError(_lib.ESHAPE, f"bias has {bias.numel()} elements, the weight {N} channels")
            b = bias.to(device=x.device, dtype=torch.float32).contiguous()
        _lib.check(L.tppx_linear_wide(x.data_ptr(), _lib.DT_F16 if ctype == torch.float16 else _lib.DT_F32, qn.data_ptr(),
                                      _lib.ptr(sn), kind, _lib.ptr(b), acc.data_ptr(), M, N, K, _lib.stream_of(x)))
    return _wide_post(acc, ctype, post, post_in, post_in2, post_scale, shape)


def _linear_other_types(input, weight, bias, post, flags, post_in=None, post_in2=None, post_scale=1.0):
    """The element-type switch of fc_plain_wrap (src/csrc/llm/fused_llm_infer.cpp:1526-1545) beyond bfloat16.
    QINT8-family weights (TppBlockedQInt8LinearW, src/csrc/fused_gemm.h:1236-1249):
      float / half activations    quantized from their own values (quantize_int8sym over the last axis with the
                                  weight's block size), fp32 accumulation and bias, output in the activations' type;
      pre-quantized qint8 input   used as it is; the compute type is the bias's, float without a bias (:1529-1535).
    A bfloat16 compute type runs the bf16 kernels on the quantized rows; float / half the fp32-output kernel.
    MXFP4 and unquantized bf16 weights take float / half activations as they are (_linear_wide)."""
    L = _lib.lib()
    wide_weight = (isinstance(weight, QTensor) and weight.is_weight() and weight.weight_kind() == "mxfp4") or \
        (_is_plain(weight) and weight.dtype == torch.bfloat16)
    if wide_weight and not isinstance(input, QTensor):
        return _linear_wide(input, weight, bias, post, post_in, post_in2, post_scale)
    if not isinstance(weight, QTensor) or not weight.is_weight() or weight.weight_kind() in ("mxfp4", "mxfp4_int8"):
        raise TppxError(_lib.EUNSUPPORTED, "pre-quantized activations need a QINT8, QINT4 or QINT2 weight; float / half "
                                           "activations any weight but the W4A8 layout")
    _lib.require_gpu(weight.qdata, "weight")
    N, K = weight.weight_nk()
    qbs = weight.block_size
    if isinstance(input, QTensor):
        if input._qscheme != QSCHEME_AFFINE or input.qdata.dtype != torch.int8 or input.is_weight() \
                or input.block_size != qbs or input.axis != len(input.shape) - 1:
            raise TppxError(_lib.EUNSUPPORTED, f"a pre-quantized input must be qint8, quantized over its last axis with "
                                               f"the weight's block size {qbs}: {input!r}")
        act = input
        ctype = bias.dtype if bias is not None and bias.numel() else torch.float32
    else:
        _lib.require_gpu(input, "input")
        ctype = input.dtype
        if input.shape[-1] != K:
            raise TppxError(_lib.ESHAPE, f"input has {input.shape[-1]} features, weight expects {K}")
        act = quantize_int8sym(input.float().contiguous(), qbs, -1, False)
    shape = tuple(act.shape)
    if shape[-1] != K:
        raise TppxError(_lib.ESHAPE, f"input has {shape[-1]} features, weight expects {K}")
    xq, sa = act.qdata.contiguous(), act.scales.contiguous()
    M = xq.numel() // K
    qn, sn = weight.native()
    st = _lib.stream_of(xq)
    if ctype == torch.bfloat16:
        y = torch.empty(shape[:-1] + (N,), dtype=torch.bfloat16, device=xq.device)
        if M:
            b = _prep_bias(bias, N, xq.device)
            p1 = _prep_post(post_in, M, N, "post-op input", xq.device) if post in (POST_MUL, POST_ADD_SCALE, POST_ADD2_SCALE) else None
            p2 = _prep_post(post_in2, M, N, "second post-op input", xq.device) if post == POST_ADD2_SCALE else None
            ws = _lib.workspace(xq)
            _lib.check(L.tppx_linear_qint8(None, xq.data_ptr(), sa.data_ptr(), qn.data_ptr(), sn.data_ptr(), _lib.ptr(b),
                                           _lib.ptr(p1), _lib.ptr(p2), y.data_ptr(), M, N, K, qbs, post, float(post_scale),
                                           flags, ws.data_ptr(), ws.numel(), st))
        return y
    if ctype not in (torch.float32, torch.float16):
        raise TppxError(_lib.EUNSUPPORTED, f"compute type {ctype} is not built")
    y = torch.empty((M, N), dtype=torch.float32, device=xq.device)
    if M:
        b = None
        if bias is not None and bias.numel():
            if bias.numel() != N:
                raise TppxError(_lib.ESHAPE, f"bias has {bias.numel()} elements, the weight {N} channels")
            b = bias.to(device=xq.device, dtype=torch.float32).contiguous()
        _lib.check(L.tppx_linear_qint8_f32(xq.data_ptr(), sa.data_ptr(), qn.data_ptr(), sn.data_ptr(), _lib.ptr(b),
                                           y.data_ptr(), M, N, K, qbs, st))
    return _wide_post(y, ctype, post, post_in, post_in2, post_scale, shape[:-1] + (N,))


PACKED_CODES = os.environ.get("TPPX_PACKED_CODES", "1") == "1"
W4A8_ACT_SCALE = 6.0 / 127.0
W4A8_DECODE = os.environ.get("TPPX_W4A8_DECODE", "1") == "1"
W4A8_WIDE_ROWS = int(os.environ.get("TPPX_W4A8_WIDE_ROWS", "64"))


def _linear_w4a8(input, weight, bias, post, post_in, post_in2, post_scale):
    """TppBlockedLinearW<int8_t, uint8_t, Tout> (src/csrc/fused_gemm.h:965-978, 1523-1526): bf16 activations are
    quantized to int8 over blocks of 32 (quantize_int8sym with the weight's block size), the scales multiplied by
    6/127, and the GEMM runs on int8 against the MXFP4 weight in its VNNI8 layout."""
    L = _lib.lib()
    _lib.require_gpu(input, "input")
    if input.dtype != torch.bfloat16:
        raise TppxError(_lib.EUNSUPPORTED, f"the W4A8 path takes bfloat16 activations (got {input.dtype})")
    N, K = weight.weight_nk()
    if input.shape[-1] != K:
        raise TppxError(_lib.ESHAPE, f"input has {input.shape[-1]} features, weight expects {K}")
    x = input.contiguous()
    M = x.numel() // K
    y = torch.empty(tuple(input.shape[:-1]) + (N,), dtype=torch.bfloat16, device=x.device)
    if M == 0:
        return y
    bias = _prep_bias(bias, N, x.device)
    post_in = _prep_post(post_in, M, N, "post-op input", x.device)
    post_in2 = _prep_post(post_in2, M, N, "second post-op input", x.device)
    # decode steps: one launch that quantizes its rows itself and splits K over the waves of a workgroup
    # (TPPX_W4A8_DECODE=0 keeps the two-step path)
    nat = weight.native_w4a8() if (M <= 16 and W4A8_DECODE) else None
    if nat is not None:
        rc = L.tppx_linear_mxfp4_int8_rows(x.data_ptr(), nat[0].data_ptr(), nat[1].data_ptr(), _lib.ptr(bias),
                                           _lib.ptr(post_in), _lib.ptr(post_in2), y.data_ptr(), M, N, K, post, post_scale,
                                           _lib.stream_of(x))
        if rc != _lib.EUNSUPPORTED:  # rows that do not fit the kernel's LDS take the two-step path
            _lib.check(rc)
            return y
    # prompt passes: rows and weights as bf16-coded integers on the bf16 MFMA, one fp32 multiply-add per block
    # (TPPX_W4A8_WIDE_ROWS: from how many rows; the weight keeps a second, 2-byte-per-value copy for it)
    wide = weight.native_w4a8_wide() if M >= W4A8_WIDE_ROWS else None
    if wide is not None:
        mp = (M + 127) // 128 * 128
        ws = torch.empty(mp * K * 2 + mp * (K // 32) * 4, dtype=torch.uint8, device=x.device)
        _lib.check(L.tppx_linear_mxfp4_int8_wide(x.data_ptr(), wide.data_ptr(), _lib.ptr(bias), _lib.ptr(post_in),
                                                 _lib.ptr(post_in2), y.data_ptr(), M, N, K, post, post_scale,
                                                 ws.data_ptr(), ws.numel(), _lib.stream_of(x)))
        return y
    act = quantize_int8sym(x.view(M, K), 32, -1, False)
    sa = act.scales.mul_(W4A8_ACT_SCALE)
    _lib.check(L.tppx_linear_mxfp4_int8(act.qdata.data_ptr(), sa.data_ptr(), weight.qdata.data_ptr(),
                                        weight.scales.data_ptr(), _lib.ptr(bias), _lib.ptr(post_in), _lib.ptr(post_in2),
                                        y.data_ptr(), M, N, K, weight.shape[2] * 8, post, post_scale, _lib.stream_of(x)))
    return y


def _is_w4a8(w):
    return isinstance(w, QTensor) and w.weight_kind() == "mxfp4_int8"


def _is_plain(w):
    """An unquantized (bf16 / fp32, blocked or flat) weight tensor."""
    return isinstance(w, torch.Tensor) and not isinstance(w, QTensor)


def weight_nk(w):
    """(output channels, input channels) of a quantized or an unquantized blocked weight."""
    return tuple(w.weight_nk()) if isinstance(w, QTensor) else tuple(_blocked_geometry(w)[:2])


def _one_launch_group(weights):
    """Do these weights share a fused launch (one quantized format in the default layout)?  Unquantized weights,
    the W4A8 layout and mixed formats run one GEMM per weight."""
    if any(_is_plain(w) or _is_w4a8(w) for w in weights):
        return False
    return all(w._qscheme == weights[0]._qscheme and w.block_size == weights[0].block_size and
               w.weight_kind() == weights[0].weight_kind() for w in weights)


def linear(input, weight, bias=None, post=POST_NONE, post_in=None, post_in2=None, post_scale=1.0, flags=0,
           row_sumsq=None):
    """One quantized GEMM with a fused post-op
    (call_gemm_with_post_op, src/csrc/fused_gemm.h:1510-1597).
    row_sumsq: f32 [16][256] table that receives the row sums of squares of the output (see sums_table());
    only honoured where takes_row_sums() says so."""
    L = _lib.lib()
    other_type = isinstance(input, QTensor) or (isinstance(input, torch.Tensor) and input.dtype in (torch.float32, torch.float16))
    if other_type and not _is_w4a8(weight):
        if row_sumsq is not None:
            raise TppxError(_lib.EUNSUPPORTED, "row sums of squares need bfloat16 activations")
        return _linear_other_types(input, weight, bias, post, flags, post_in, post_in2, post_scale)
    if not isinstance(weight, QTensor) and isinstance(weight, torch.Tensor) and weight.dtype == torch.bfloat16:
        if row_sumsq is not None:
            raise TppxError(_lib.EUNSUPPORTED, "row sums of squares need an MXFP4 weight and at most 16 rows")
        return _linear_bf16(input, weight, bias, post, post_in, post_in2, post_scale, flags)
    if _is_w4a8(weight):
        if row_sumsq is not None:
            raise TppxError(_lib.EUNSUPPORTED, "row sums of squares need an MXFP4 weight in the default layout")
        return _linear_w4a8(input, weight, bias, post, post_in, post_in2, post_scale)
    x, M, N, K = _prep_input(input, weight)
    out_shape = tuple(input.shape[:-1]) + (N,)
    y = torch.empty(out_shape, dtype=torch.bfloat16, device=x.device)
    if M == 0:
        return y
    bias = _prep_bias(bias, N, x.device)
    post_in = _prep_post(post_in, M, N, "post-op input", x.device)
    post_in2 = _prep_post(post_in2, M, N, "second post-op input", x.device)
    # QINT4 / QINT2 decode steps (up to 64 rows): the codes streamed at their own width and expanded in registers
    # (same bits as the expanded int8 tiles).  TPPX_PACKED_CODES=0 keeps the expanded tiles.
    if PACKED_CODES and M <= 64 and weight.weight_kind() in ("qint4", "qint2") and weight.block_size == 256 \
            and row_sumsq is None and not (flags & ~_lib.FLAG_XQ_REUSE):
        qp, sp, bits = weight.native_packed()
        xq, sa = _qint8_scratch(x, M, K, 256) if M > 16 else (None, None)
        rc = L.tppx_linear_qintx(x.data_ptr(), _lib.ptr(xq), _lib.ptr(sa), qp.data_ptr(), sp.data_ptr(), _lib.ptr(bias),
                                 _lib.ptr(post_in), _lib.ptr(post_in2), y.data_ptr(), M, N, K, bits, post, post_scale,
                                 flags, _lib.stream_of(x))
        if rc != _lib.EUNSUPPORTED:  # rows that do not fit the in-kernel quantisation fall through to the int8 tiles
            _lib.check(rc)
            return y
    qn, sn = weight.native()
    st = _lib.stream_of(x)
    ws = _lib.workspace(x)
    if row_sumsq is not None:
        if not takes_row_sums(weight, M):
            raise TppxError(_lib.EUNSUPPORTED, "row sums of squares need an MXFP4 weight and at most 16 rows")
        _lib.check(L.tppx_linear_mxfp4_rowsq(x.data_ptr(), qn.data_ptr(), sn.data_ptr(), _lib.ptr(bias),
                                             _lib.ptr(post_in), _lib.ptr(post_in2), y.data_ptr(), M, N, K,
                                             post, post_scale, flags, ws.data_ptr(), ws.numel(),
                                             row_sumsq.data_ptr(), st))
    elif weight._qscheme == QSCHEME_MXFP:
        flags, ws = _mxfp4_flags_ws(x, M, K, flags)
        _lib.check(L.tppx_linear_mxfp4(x.data_ptr(), qn.data_ptr(), sn.data_ptr(), _lib.ptr(bias),
                                       _lib.ptr(post_in), _lib.ptr(post_in2), y.data_ptr(), M, N, K,
                                       post, post_scale, flags, ws.data_ptr(), ws.numel(), st))
    else:
        qbs = weight.block_size
        xq, sa = _qint8_scratch(x, M, K, qbs)
        _lib.check(L.tppx_linear_qint8(x.data_ptr(), xq.data_ptr(), sa.data_ptr(), qn.data_ptr(),
                                       sn.data_ptr(), _lib.ptr(bias), _lib.ptr(post_in),
                                       _lib.ptr(post_in2), y.data_ptr(), M, N, K, qbs, post,
                                       post_scale, flags, ws.data_ptr(), ws.numel(), st))
    return y


def fc_plain(input, weight, bias, parallel_dim=-1, split_sizes=()):
    """torch.ops.tpp_llm.fc_plain (fc_plain_wrap, src/csrc/llm/fused_llm_infer.cpp:1514-1566)."""
    if parallel_dim not in (-1, None):
        raise TppxError(_lib.EUNSUPPORTED,
                        "tensor-parallel fc_plain (parallel_dim 0/1) needs a process group; this build runs one GPU")
    return linear(input, weight, bias, POST_NONE)


def fc_add(input, weight, bias, residual, scale=1.0, row_sumsq=None):
    """GEMM + AddScalePostOp(residual, scale) (fused_llm_infer.cpp:1261,1273)."""
    return linear(input, weight, bias, POST_ADD_SCALE, residual, None, scale, row_sumsq=row_sumsq)


def fc_add2(input, weight, bias, residual1, residual2, scale=1.0):
    """GEMM + Add2ScalePostOp (src/csrc/fused_gemm.h:1460)."""
    return linear(input, weight, bias, POST_ADD2_SCALE, residual1, residual2, scale)


def fc_silu(input, weight, bias):
    """GEMM + SiluPostOp (fused_llm_infer.cpp:1271)."""
    return linear(input, weight, bias, POST_SILU)


def fc_gelu(input, weight, bias):
    return linear(input, weight, bias, POST_GELU)


def fc_relu(input, weight, bias):
    return linear(input, weight, bias, POST_RELU)


def fc_mul(input, weight, bias, mul_in):
    """GEMM + MulPostOp(mul_in) (fused_llm_infer.cpp:1272)."""
    return linear(input, weight, bias, POST_MUL, mul_in)


def rms_norm(t_in, t_wt, eps):
    """llama_rms_norm (src/csrc/llm/fused_llm_infer.cpp:337-363): bf16 in/out, fp32 or bf16 weight."""
    L = _lib.lib()
    if not t_in.is_cuda or t_in.dtype != torch.bfloat16:
        raise TppxError(_lib.EINVAL, "llama_rms_norm: input must be a bfloat16 tensor on the GPU")
    x = t_in.contiguous()
    K = x.shape[-1]
    if t_wt.dtype not in (torch.float32, torch.bfloat16) or t_wt.numel() != K or not t_wt.is_cuda:
        raise TppxError(_lib.EINVAL, "llama_rms_norm: weight must be fp32 or bf16 [K] on the GPU")
    y = torch.empty_like(x)
    rows = x.numel() // K
    if rows:
        _lib.check(L.tppx_rms_norm(x.data_ptr(), t_wt.contiguous().data_ptr(), 0 if t_wt.dtype == torch.float32 else 1,
                                   y.data_ptr(), rows, K, float(eps), _lib.stream_of(x)))
    return y


def layer_norm(t_in, t_gamma, t_beta, eps):
    """lyr_norm (src/csrc/llm/fused_llm_infer.cpp:254-306): bf16 in/out, gamma and beta both fp32 or both bf16."""
    L = _lib.lib()
    if not t_in.is_cuda or t_in.dtype != torch.bfloat16:
        raise TppxError(_lib.EINVAL, "lyr_norm: input must be a bfloat16 tensor on the GPU")
    x = t_in.contiguous()
    K = x.shape[-1]
    if t_gamma.dtype not in (torch.float32, torch.bfloat16) or t_gamma.numel() != K or not t_gamma.is_cuda:
        raise TppxError(_lib.EINVAL, "lyr_norm: gamma must be fp32 or bf16 [K] on the GPU")
    if t_beta.dtype != t_gamma.dtype or t_beta.numel() != K or not t_beta.is_cuda:
        raise TppxError(_lib.EINVAL, "lyr_norm: beta must have gamma's dtype and size")
    y = torch.empty_like(x)
    rows = x.numel() // K
    if rows:
        _lib.check(L.tppx_layer_norm(x.data_ptr(), t_gamma.contiguous().data_ptr(), t_beta.contiguous().data_ptr(),
                                     0 if t_gamma.dtype == torch.float32 else 1, y.data_ptr(), rows, K, float(eps),
                                     _lib.stream_of(x)))
    return y


# RMSNorm inside the GEMM launch (tppx_norm_multi_linear_mxfp4 / tppx_norm_swiglu_mxfp4).  Off by default: on MI355X
# the fused launch measured slower than the normalisation kernel followed by the plain launch (every workgroup
# repeats the row reduction behind a barrier, and the extra registers spill); TPPX_FUSE_NORM=1 turns it on.
FUSE_NORM = os.environ.get("TPPX_FUSE_NORM", "0") == "1"


# RMSNorm scale from row sums of squares that the GEMM which wrote the activations left behind
# (tppx_linear_mxfp4_rowsq -> tppx_normsq_*): no normalisation launch and no pass over the row.  On by default;
# TPPX_NORM_FROM_SUMS=0 goes back to the separate normalisation kernel.
NORM_FROM_SUMS = os.environ.get("TPPX_NORM_FROM_SUMS", "1") == "1"


def sums_table(device):
    """A table for the row sums of squares of one activation tensor: f32 [16][256]."""
    return torch.zeros((16, 256), dtype=torch.float32, device=device)


def takes_row_sums(weight, M):
    """Can the GEMM with this weight leave row sums of squares of its output (MXFP4 decode kernels, <= 16 rows,
    at most 256 workgroups of up to three channel tiles: 12288 output channels)?"""
    if not isinstance(weight, QTensor):
        return False
    w = weight
    return (NORM_FROM_SUMS and w._qscheme == QSCHEME_MXFP and w.weight_kind() == "mxfp4" and 0 < M <= 16
            and w.weight_nk()[0] <= 12288)


def _norm_fits(norm, scheme, M, K):
    gamma = norm[0]
    return (scheme == QSCHEME_MXFP and 0 < M <= 16 and K % 128 == 0 and (K == 4096 or K == 2048 or K <= 2048)
            and gamma.dtype == torch.float32 and gamma.is_cuda and gamma.is_contiguous())


def _norm_fusable(norm, scheme, M, K):
    """RMSNorm can ride inside the GEMM launch for MXFP4 decode steps (<= 16 rows, the LDS staging fits): always
    when the row sums of squares are handed over (norm = (gamma, eps, table)), otherwise only with TPPX_FUSE_NORM."""
    if norm is None:
        return False
    handed = len(norm) > 2 and norm[2] is not None
    if not (handed and NORM_FROM_SUMS) and not FUSE_NORM:
        return False
    return _norm_fits(norm, scheme, M, K)


def _norm_table(norm):
    return norm[2] if (len(norm) > 2 and norm[2] is not None and NORM_FROM_SUMS) else None


# Decode steps (<= 16 rows) on MXFP4 weights: q/k/v as ONE GEMM over the concatenated native weights, so that every
# workgroup gets the same number of channel tiles (three segments of 256 tiles do not divide into 256 groups of 3:
# 192 workgroups of 4 on 256 CUs).  TPPX_QKV_ONE_GEMM=0 keeps the segment table.
QKV_ONE_GEMM = os.environ.get("TPPX_QKV_ONE_GEMM", "1") == "1"


def _qkv_cat(weights):
    """Concatenated native tiles / scales of the projections, built once and kept on the first weight; the
    projections' own native copies become views into it (no second copy in memory)."""
    key = tuple(id(w) for w in weights) + tuple(w.qdata.data_ptr() for w in weights)
    have = getattr(weights[0], "_tppx_qkv_cat", None)
    if have is not None and have[0] == key:
        return have[1], have[2]
    nats = [w.native() for w in weights]
    qn = torch.cat([a.reshape(-1) for a, _ in nats])
    sn = torch.cat([b.reshape(-1) for _, b in nats])
    qo = so = 0
    for w, (a, b) in zip(weights, nats):
        w._native = (qn[qo:qo + a.numel()].view(a.shape), sn[so:so + b.numel()].view(b.shape))
        qo += a.numel()
        so += b.numel()
    weights[0]._tppx_qkv_cat = (key, qn, sn)
    return qn, sn


def _qkv_one_gemm(L, input, x, M, K, weights, biases, norm):
    """The fused q/k/v launch as one GEMM with three output matrices (tppx_qkv_linear_mxfp4); None when the case is
    not its (other formats, more than 16 rows, a 4th GEMM with its GELU, a shape the LDS-staged kernel does not take)."""
    n = len(weights)
    if n not in (2, 3) or not (0 < M <= 16) or any(_as_q(w).weight_kind() != "mxfp4" for w in weights):
        return None
    widths = [w.weight_nk()[0] for w in weights]
    if any(w.weight_nk()[1] != K for w in weights):
        raise TppxError(_lib.ESHAPE, "Fused QKV weight block mismatch")
    N = sum(widths)
    qn, sn = _qkv_cat(weights)
    bias = None
    if any(b is not None and b.numel() for b in biases[:n]):
        # the projections' biases side by side, built once per set of bias tensors and kept on the first weight
        key = tuple((id(b), b.data_ptr(), b._version) if b is not None and b.numel() else None for b in biases[:n])
        have = getattr(weights[0], "_tppx_qkv_bias", None)
        if have is None or have[0] != key:
            have = (key, torch.cat([(_prep_bias(b, w, x.device) if b is not None and b.numel()
                                     else torch.zeros(w, dtype=torch.bfloat16, device=x.device))
                                    for b, w in zip(biases, widths)]))
            weights[0]._tppx_qkv_bias = have
        bias = have[1]
    buf = torch.empty(M * N, dtype=torch.bfloat16, device=x.device)
    gamma = sums = None
    eps = 0.0
    if norm is not None:  # fusable, or qkv_gemm() has applied it already
        gamma, eps, sums = norm[0], float(norm[1]), _norm_table(norm)
    n1 = widths[0]
    n2 = widths[0] + widths[1]
    rc = L.tppx_qkv_linear_mxfp4(x.data_ptr(), _lib.ptr(sums), _lib.ptr(gamma), eps, qn.data_ptr(), sn.data_ptr(),
                                 _lib.ptr(bias), buf.data_ptr(), M, N, K, n1, n2, 0, _lib.stream_of(x))
    if rc == _lib.EUNSUPPORTED:
        return None
    _lib.check(rc)
    outs, o = [], 0
    for w in widths:
        outs.append(buf[o:o + M * w].view(tuple(input.shape[:-1]) + (w,)))
        o += M * w
    return outs


def qkv_gemm(input, weights, biases, norm=None):
    """fused_qkv_gemm (src/csrc/llm/fused_llm_infer.cpp:423-505): several GEMMs
    over one activation in one launch; a 4th GEMM gets GELU (GPT-J fc_in).
    norm = (gamma, eps): llama_rms_norm is applied to the input first (inside
    the same launch for MXFP4 decode steps, as a separate launch otherwise)."""
    L = _lib.lib()
    weights = list(weights)
    if not _one_launch_group(weights):  # unquantized weights, the W4A8 layout, mixed formats: one GEMM per weight
        if norm is not None:
            input = rms_norm(input, norm[0], norm[1])
        biases = list(biases) if biases is not None else []
        biases += [None] * (len(weights) - len(biases))
        return [linear(input, w, b, POST_GELU if (len(weights) == 4 and i == 3) else POST_NONE)
                for i, (w, b) in enumerate(zip(weights, biases))]
    if norm is not None:
        xin, Min, _, Kin = _prep_input(input, list(weights)[0])
        if not _norm_fusable(norm, list(weights)[0]._qscheme, Min, Kin):
            input, norm = rms_norm(input, norm[0], norm[1]), None
    weights = list(weights)
    biases = list(biases) if biases is not None else []
    n = len(weights)
    if n < 1 or n > 4:
        raise TppxError(_lib.EINVAL, f"qkv_gemm takes 1..4 weights, got {n}")
    while len(biases) < n:
        biases.append(None)
    x, M, N0, K = _prep_input(input, weights[0])
    scheme = weights[0]._qscheme
    outs = _qkv_one_gemm(L, input, x, M, K, weights, biases, norm) if QKV_ONE_GEMM else None
    if outs is not None:
        return outs
    segs = (_lib.Seg * n)()
    outs, keep = [], []
    for i, w in enumerate(weights):
        xi, Mi, Ni, Ki = _prep_input(input, w)
        if w._qscheme != scheme or Ki != K or w.block_size != weights[0].block_size:
            raise TppxError(_lib.ESHAPE, "Fused QKV weight block mismatch")
        y = torch.empty(tuple(input.shape[:-1]) + (Ni,), dtype=torch.bfloat16, device=x.device)
        b = _prep_bias(biases[i], Ni, x.device)
        qn, sn = w.native()
        keep.append((b, qn, sn))
        segs[i].qw = qn.data_ptr()
        segs[i].sw = sn.data_ptr()
        segs[i].bias = _lib.ptr(b)
        segs[i].post_in = None
        segs[i].post_in2 = None
        segs[i].y = y.data_ptr()
        segs[i].N = Ni
        segs[i].post_op = POST_GELU if (n == 4 and i == 3) else POST_NONE
        segs[i].post_scale = 1.0
        outs.append(y)
    if M == 0:
        return outs
    st = _lib.stream_of(x)
    ws = _lib.workspace(x)
    if scheme == QSCHEME_MXFP and norm is not None and _norm_table(norm) is not None:
        _lib.check(L.tppx_normsq_multi_linear_mxfp4(x.data_ptr(), _norm_table(norm).data_ptr(), norm[0].data_ptr(),
                                                    float(norm[1]), segs, n, M, K, 0, st))
    elif scheme == QSCHEME_MXFP and norm is not None:
        _lib.check(L.tppx_norm_multi_linear_mxfp4(x.data_ptr(), norm[0].data_ptr(), float(norm[1]), segs, n, M, K, 0, st))
    elif scheme == QSCHEME_MXFP:
        fl, ws = _mxfp4_flags_ws(x, M, K)
        _lib.check(L.tppx_multi_linear_mxfp4(x.data_ptr(), segs, n, M, K, fl, ws.data_ptr(), ws.numel(), st))
    else:
        qbs = weights[0].block_size
        xq, sa = _qint8_scratch(x, M, K, qbs)
        _lib.check(L.tppx_multi_linear_qint8(x.data_ptr(), xq.data_ptr(), sa.data_ptr(), segs, n, M, K,
                                             qbs, 0, ws.data_ptr(), ws.numel(), st))
    return outs


def swiglu_gate_up(input, w_gate, w_up, b_gate=None, b_up=None, norm=None):
    """silu(x Wg^T) * (x Wu^T) in one launch with the reference's bf16 rounding
    points (fused_llm_infer.cpp:1271-1272).  norm = (gamma, eps): llama_rms_norm
    on the input first (fused_llm_infer.cpp:1269), inside the launch when possible."""
    L = _lib.lib()
    if not _one_launch_group([w_gate, w_up]):
        if norm is not None:
            input = rms_norm(input, norm[0], norm[1])
        return fc_mul(input, w_up, b_up, fc_silu(input, w_gate, b_gate))
    if norm is not None:
        _, M0, _, K0 = _prep_input(input, w_gate)
        if not _norm_fusable(norm, w_gate._qscheme, M0, K0):
            input, norm = rms_norm(input, norm[0], norm[1]), None
    x, M, N, K = _prep_input(input, w_gate)
    x2, M2, N2, K2 = _prep_input(input, w_up)
    if N2 != N or w_gate._qscheme != w_up._qscheme:
        raise TppxError(_lib.ESHAPE, "gate and up projections must have the same shape and format")
    if w_gate._qscheme != QSCHEME_MXFP:
        g = fc_silu(input, w_gate, b_gate)
        return fc_mul(input, w_up, b_up, g)
    y = torch.empty(tuple(input.shape[:-1]) + (N,), dtype=torch.bfloat16, device=x.device)
    if M == 0:
        return y
    bg = _prep_bias(b_gate, N, x.device)
    bu = _prep_bias(b_up, N, x.device)
    qg, sg = w_gate.native()
    qu, su = w_up.native()
    if norm is not None and _norm_table(norm) is not None:
        _lib.check(L.tppx_normsq_swiglu_mxfp4(x.data_ptr(), _norm_table(norm).data_ptr(), norm[0].data_ptr(),
                                              float(norm[1]), qg.data_ptr(), sg.data_ptr(), _lib.ptr(bg),
                                              qu.data_ptr(), su.data_ptr(), _lib.ptr(bu), y.data_ptr(), M, N, K, 0,
                                              _lib.stream_of(x)))
        return y
    if norm is not None:
        _lib.check(L.tppx_norm_swiglu_mxfp4(x.data_ptr(), norm[0].data_ptr(), float(norm[1]), qg.data_ptr(), sg.data_ptr(),
                                            _lib.ptr(bg), qu.data_ptr(), su.data_ptr(), _lib.ptr(bu), y.data_ptr(),
                                            M, N, K, 0, _lib.stream_of(x)))
        return y
    fl, ws = _mxfp4_flags_ws(x, M, K)
    if not fl and M > 64 and M * N * 2 > ws.numel():
        # prefill: room for the gate tile lets the library run gate and up as one grid (fuller last round)
        ws = torch.empty(M * N * 2, dtype=torch.uint8, device=x.device)
    elif fl & _lib.FLAG_ACT_FP8:
        # the same behind the quantised activations
        Mp = (M + 63) // 64 * 64
        need = (Mp * K + Mp * (K // 32) + 255) // 256 * 256 + M * N * 2
        if need > ws.numel():
            ws = torch.empty(need, dtype=torch.uint8, device=x.device)
    _lib.check(L.tppx_swiglu_mxfp4(x.data_ptr(), qg.data_ptr(), sg.data_ptr(), _lib.ptr(bg), qu.data_ptr(),
                                   su.data_ptr(), _lib.ptr(bu), y.data_ptr(), M, N, K, fl, ws.data_ptr(),
                                   ws.numel(), _lib.stream_of(x)))
    return y


def swiglu_mlp(input, w_gate, w_up, w_down, residual, scale=1.0):
    """The Llama MLP block (fused_llm_infer.cpp:1271-1273):
    down( silu(gate(x)) * up(x) ) + residual*scale."""
    inter = swiglu_gate_up(input, w_gate, w_up)
    return fc_add(inter, w_down, None, residual, scale)


# ----------------------------------------------------------------------------
# torch.library registration (namespace tpp_llm, like TORCH_LIBRARY(tpp_llm, m),
# fused_llm_infer.cpp:1588-1611)
# ----------------------------------------------------------------------------
_libdef = torch.library.Library("tpp_llm", "DEF")
_libdef.define("fc_plain(Tensor input, Tensor weight, Tensor bias, int parallel_dim, int[] split_sizes) -> Tensor")
_libdef.define("fc_add(Tensor input, Tensor weight, Tensor bias, Tensor residual, float scale=1.0) -> Tensor")
_libdef.define("fc_silu(Tensor input, Tensor weight, Tensor bias) -> Tensor")
_libdef.define("fc_mul(Tensor input, Tensor weight, Tensor bias, Tensor mul_in) -> Tensor")
_libdef.define("qkv_gemm(Tensor input, Tensor[] weights, Tensor[] biases) -> Tensor[]")
_libdef.define("swiglu_mlp(Tensor input, Tensor w_gate, Tensor w_up, Tensor w_down, Tensor residual, float scale=1.0) -> Tensor")

_IMPLS = {
    "fc_plain": fc_plain,
    "fc_add": fc_add,
    "fc_silu": fc_silu,
    "fc_mul": fc_mul,
    "qkv_gemm": qkv_gemm,
    "swiglu_mlp": swiglu_mlp,
}
for _name, _fn in _IMPLS.items():
    # plain (non-subclass) tensors land here: the weight is then not quantized,
    # which this build rejects with a clear error inside the implementation
    _libdef.impl(_name, _fn, "CompositeExplicitAutograd")

# QTensor.__torch_dispatch__ routes the ops here
DISPATCH = {getattr(torch.ops.tpp_llm, n).default: f for n, f in _IMPLS.items()}
