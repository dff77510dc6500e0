"""CPU oracle for the weight-quantized linear path -- TEST INFRASTRUCTURE ONLY.

numpy + ctypes front-end of ``libtppx_oracle.so`` (``oracle/tppx_oracle.c``).
Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module; the product package never does.

bf16 tensors are carried as ``numpy.uint16`` bit patterns.

The layout helpers restate the reference's ``view``/``permute`` chains
(``src/tpp_pytorch_extension/utils/blocked_layout.py:28-80``,
``src/csrc/qtypes.cpp:783-932``) with numpy ``reshape``/``transpose`` so that
they can be compared, byte for byte, with the closed-form index maps coded in
C (``orc_remap_quantize_*``).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libtppx_oracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libmxref.so")

POST_NONE, POST_SILU, POST_MUL, POST_ADD_SCALE, POST_ADD2_SCALE, POST_GELU, POST_RELU = range(7)
MODE_IDEAL, MODE_FAITHFUL, MODE_F64 = range(3)

_c_i64 = ctypes.c_int64
_c_p = ctypes.c_void_p


def build(force=False):
    """Compile the C restatement (and the reference shim when the reference
    tree is present)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libtppx_oracle.so"])
    if os.path.isdir("/root/reference/src/csrc"):
        subprocess.check_call(["make", "-C", _HERE, "ref"])


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(
                "oracle library not built: run `make -C oracle` (or __graft_entry__.build())"
            )
        L = ctypes.CDLL(_LIB_PATH)
        L.orc_mx_scale_byte.argtypes = [ctypes.c_float]
        L.orc_mx_scale_byte.restype = ctypes.c_int
        L.orc_mx_quant_scale.argtypes = [ctypes.c_int]
        L.orc_mx_quant_scale.restype = ctypes.c_float
        L.orc_mx_dequant_scale.argtypes = [ctypes.c_int]
        L.orc_mx_dequant_scale.restype = ctypes.c_float
        L.orc_e2m1_encode.argtypes = [ctypes.c_float]
        L.orc_e2m1_encode.restype = ctypes.c_int
        L.orc_e2m1_decode.argtypes = [ctypes.c_int]
        L.orc_e2m1_decode.restype = ctypes.c_float
        L.orc_num_threads.restype = ctypes.c_int
        _lib = L
    return _lib


def ref_lib():
    """The shim around the reference's own mxfp_quant.h, or None when it was
    not built (it only builds where the reference tree is mounted)."""
    if not os.path.exists(_REF_PATH):
        return None
    R = ctypes.CDLL(_REF_PATH)
    R.ref_mx_shared_scale.argtypes = [ctypes.c_float]
    R.ref_mx_shared_scale.restype = ctypes.c_float
    R.ref_e2m1_round.argtypes = [ctypes.c_float]
    R.ref_e2m1_round.restype = ctypes.c_float
    return R


def _p(a):
    return None if a is None else a.ctypes.data_as(_c_p)


def _c(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


# ----------------------------------------------------------------------------
# bf16 helpers
# ----------------------------------------------------------------------------
def f32_to_bf16(a):
    a = _c(a, np.float32)
    out = np.empty(a.shape, np.uint16)
    lib().orc_f32_to_bf16(_p(a), _p(out), _c_i64(a.size))
    return out


def bf16_to_f32(a):
    a = _c(a, np.uint16)
    return (a.astype(np.uint32) << 16).view(np.float32)


def bf16_round(a):
    """fp32 -> nearest bf16 -> fp32."""
    return bf16_to_f32(f32_to_bf16(a))


# ----------------------------------------------------------------------------
# element math (scalar)
# ----------------------------------------------------------------------------
def mx_scale_byte(amax):
    return lib().orc_mx_scale_byte(float(amax))


def mx_quant_scale(x):
    return lib().orc_mx_quant_scale(int(x))


def mx_dequant_scale(x):
    return lib().orc_mx_dequant_scale(int(x))


def e2m1_encode(v):
    return lib().orc_e2m1_encode(float(v))


def e2m1_decode(c):
    return lib().orc_e2m1_decode(int(c))


def e2m1_encode_array(v):
    v = _c(v, np.float32)
    out = np.empty(v.shape, np.int32)
    lib().orc_e2m1_encode_n(_p(v), _p(out), _c_i64(v.size))
    return out.astype(np.int64)


def mx_quant_scale_of_amax_array(a):
    a = _c(a, np.float32)
    out = np.empty(a.shape, np.float32)
    lib().orc_mx_quant_scale_of_amax_n(_p(a), _p(out), _c_i64(a.size))
    return out


E2M1_TABLE = np.array(
    [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0],
    np.float32,
)


# ----------------------------------------------------------------------------
# blocked layout  (blocked_layout.py:28-80 ; llm_common.py:468-490 ; nn.py:27-44)
# ----------------------------------------------------------------------------
def block_weight(W, bk=16, bc=64, vnni=2):
    """W[N,K] -> [N/bk, K/bc, bc/vnni, bk, vnni] (vnni > 1) or
    [N/bk, K/bc, bc, bk] (vnni == 1): view + permute(0,2,3,1[,4])."""
    N, K = W.shape
    assert N % bk == 0 and K % bc == 0
    if vnni == 1:
        return np.ascontiguousarray(W.reshape(N // bk, bk, K // bc, bc).transpose(0, 2, 3, 1))
    assert bc % vnni == 0
    return np.ascontiguousarray(
        W.reshape(N // bk, bk, K // bc, bc // vnni, vnni).transpose(0, 2, 3, 1, 4)
    )


def unblock_weight(Wb):
    if Wb.ndim == 4:
        n1, c1, c2, k2 = Wb.shape
        return np.ascontiguousarray(Wb.transpose(0, 3, 1, 2)).reshape(n1 * k2, c1 * c2)
    n1, c1, c2, k2, c3 = Wb.shape
    return np.ascontiguousarray(Wb.transpose(0, 3, 1, 2, 4)).reshape(n1 * k2, c1 * c2 * c3)


def remap_mxfp4(t):
    """The re-layout half of remap_and_quantize_mxfp4 (qtypes.cpp:783-839,
    default USE_MXFP4_INT8=0): bring a blocked weight to [N/32,K/.,.,32,2]."""
    want = 32
    if t.ndim == 5:
        K1, C1, C2, K2, C3 = t.shape
        if K2 < want and want % K2 == 0:
            r = want // K2
            if K1 % r:
                raise ValueError("Shape not compatible for MXFP4")
            t = t.reshape(K1 // r, r, C1, C2, K2, C3).transpose(0, 2, 3, 1, 4, 5)
            t = np.ascontiguousarray(t).reshape(K1 // r, C1, C2, r * K2, C3)
        elif K2 > want and K2 % want == 0:
            r = K2 // want
            t = t.reshape(K1, C1, C2, r, want, C3).transpose(0, 3, 1, 2, 4, 5)
            t = np.ascontiguousarray(t).reshape(K1 * r, C1, C2, want, C3)
    elif t.ndim == 4:
        K1, C1, C2, K2 = t.shape
        if C2 % 2:
            raise ValueError("Shape not compatible for VNNI2")
        if K2 < want and want % K2 == 0:
            r = want // K2
            if K1 % r:
                raise ValueError("Shape not compatible for MXFP4")
            t = t.reshape(K1 // r, r, C1, C2 // 2, 2, K2).transpose(0, 2, 3, 1, 5, 4)
            t = np.ascontiguousarray(t).reshape(K1 // r, C1, C2 // 2, r * K2, 2)
        elif K2 > want and K2 % want == 0:
            r = K2 // want
            t = t.reshape(K1, C1, C2 // 2, 2, r, want).transpose(0, 4, 1, 2, 5, 3)
            t = np.ascontiguousarray(t).reshape(K1 * r, C1, C2 // 2, want, 2)
        else:
            t = t.reshape(K1, C1, C2 // 2, 2, K2).transpose(0, 1, 2, 4, 3)
            t = np.ascontiguousarray(t)
    else:
        raise ValueError("expected a 4-D or 5-D blocked weight")
    return np.ascontiguousarray(t)


def qint8_block_size(K, env_block=256):
    """Block-size choice of remap_and_quantize_qint8 (qtypes.cpp:878-889)."""
    if K % env_block == 0:
        return env_block
    q = 4096
    while q >= 64:
        if env_block > q and K % q == 0:
            return q
        q //= 2
    return None


def remap_qint8(t, env_block=256):
    """The re-layout half of remap_and_quantize_qint8 (qtypes.cpp:866-924):
    -> ([N/bk, K/QBS, QBS/4, bk, 4], QBS)."""
    if t.ndim == 5:
        K1, C1, C2, K2, C3 = t.shape
        C = C1 * C2 * C3
        qbs = qint8_block_size(C, env_block)
        if qbs is not None:
            C2, C1 = qbs // C3, C // qbs
        if C3 != 4:
            r = 4 // C3
            if C2 % r:
                raise ValueError("Shape not compatible for VNNI4")
            t = t.reshape(K1, C1, C2 // r, r, K2, C3).transpose(0, 1, 2, 4, 3, 5)
            t = np.ascontiguousarray(t).reshape(K1, C1, C2 // r, K2, r * C3)
        else:
            t = t.reshape(K1, C1, C2, K2, C3)
        return np.ascontiguousarray(t), C2 * C3
    if t.ndim == 4:
        K1, C1, C2, K2 = t.shape
        C = C1 * C2
        qbs = qint8_block_size(C, env_block)
        if qbs is not None:
            C2, C1 = qbs, C // qbs
        if C2 % 4:
            raise ValueError("Shape not compatible for VNNI4")
        t = t.reshape(K1, C1, C2 // 4, 4, K2).transpose(0, 1, 2, 4, 3)
        return np.ascontiguousarray(t), C2
    raise ValueError("expected a 4-D or 5-D blocked weight")


def _per_block_geometry(shape, block_size, axis, is_vnni, pack):
    """(pre, bs, post, vnni, scale_shape) of PerBlockQuantizer (qtypes.h:30-68)."""
    sizes = list(shape)
    if axis < 0:
        axis += len(sizes)
    if is_vnni:
        vnni = sizes.pop()
    else:
        assert axis == len(sizes) - 1, "Invalid axis"
        assert sizes[axis] % pack == 0
        vnni = pack
        sizes[axis] //= pack
    assert block_size % vnni == 0
    bsi = block_size // vnni
    assert len(sizes) > axis and sizes[axis] % bsi == 0
    sizes[axis] //= bsi
    pre = int(np.prod(sizes[: axis + 1], dtype=np.int64))
    post = int(np.prod(sizes[axis + 1 :], dtype=np.int64))
    return pre, bsi, post, vnni, sizes


def quantize_mxfp4(t, block_size=32, axis=2, is_vnni=True):
    """quantize_mxfp4 (qtypes.cpp:602-611) on an fp32 array.
    Returns (packed uint8 with last dim halved, E8M0 scale bytes)."""
    t = _c(t, np.float32)
    pre, bs, post, vnni, ssz = _per_block_geometry(t.shape, block_size, axis, is_vnni, 2)
    out = np.empty(t.shape[:-1] + (t.shape[-1] // 2,), np.uint8)
    sc = np.empty(ssz, np.uint8)
    lib().orc_mxfp4_quantize_generic(
        _p(t), _c_i64(pre), _c_i64(bs), _c_i64(post), _c_i64(vnni), _p(out), _p(sc)
    )
    return out, sc


def dequantize_mxfp4(q, sc, block_size=32, axis=2, is_vnni=True):
    q = _c(q, np.uint8)
    sc = _c(sc, np.uint8)
    shape = q.shape[:-1] + (q.shape[-1] * 2,)
    pre, bs, post, vnni, _ = _per_block_geometry(shape, block_size, axis, is_vnni, 2)
    out = np.empty(shape, np.float32)
    lib().orc_mxfp4_dequantize_generic(
        _p(q), _p(sc), _c_i64(pre), _c_i64(bs), _c_i64(post), _c_i64(vnni), _p(out)
    )
    return out


def quantize_int8sym(t, block_size, axis, is_vnni):
    """quantize_int8sym (qtypes.cpp:613-624) on an fp32 array."""
    t = _c(t, np.float32)
    pre, bs, post, vnni, ssz = _per_block_geometry(t.shape, block_size, axis, is_vnni, 1)
    out = np.empty(t.shape, np.int8)
    sc = np.empty(ssz, np.float32)
    lib().orc_int8_quantize_generic(
        _p(t), _c_i64(pre), _c_i64(bs), _c_i64(post), _c_i64(vnni), _p(out), _p(sc)
    )
    return out, sc


def dequantize_int8sym(q, sc, block_size, axis, is_vnni):
    q = _c(q, np.int8)
    sc = _c(sc, np.float32)
    pre, bs, post, vnni, _ = _per_block_geometry(q.shape, block_size, axis, is_vnni, 1)
    out = np.empty(q.shape, np.float32)
    lib().orc_int8_dequantize_generic(
        _p(q), _p(sc), _c_i64(pre), _c_i64(bs), _c_i64(post), _c_i64(vnni), _p(out)
    )
    return out


def quantize_int4sym(t, block_size, axis, is_vnni):
    """quantize_int4sym (qtypes.cpp:626-637, Int4SymQuant :199-246) on an fp32 array.
    Returns (packed uint8 with the last dim halved, fp32 scales)."""
    t = _c(t, np.float32)
    pre, bs, post, vnni, ssz = _per_block_geometry(t.shape, block_size, axis, is_vnni, 2)
    out = np.empty(t.shape[:-1] + (t.shape[-1] // 2,), np.uint8)
    sc = np.empty(ssz, np.float32)
    lib().orc_int4_quantize_generic(_p(t), _c_i64(pre), _c_i64(bs), _c_i64(post), _c_i64(vnni), _p(out), _p(sc))
    return out, sc


def dequantize_int4sym(q, sc, block_size, axis, is_vnni):
    q = _c(q, np.uint8)
    sc = _c(sc, np.float32)
    shape = q.shape[:-1] + (q.shape[-1] * 2,)
    pre, bs, post, vnni, _ = _per_block_geometry(shape, block_size, axis, is_vnni, 2)
    out = np.empty(shape, np.float32)
    lib().orc_int4_dequantize_generic(_p(q), _p(sc), _c_i64(pre), _c_i64(bs), _c_i64(post), _c_i64(vnni), _p(out))
    return out


def qint2_block_size(K, env_block=256):
    """Block rule of remap_and_quantize_qint2_intlv (qtypes.cpp:1031-1043): QINT2_BLOCK_SIZE if it divides the
    input channels, else the largest smaller power of two >= 64 that does."""
    return qint8_block_size(K, env_block)


def remap_quantize_qint2_intlv(W, bs=None, env_block=256):
    """remap_and_quantize_qint2_intlv (qtypes.cpp:1004-1073) on a plain fp32 W[N][K], N % 32 == 0:
    -> (packed uint8 [N/32][K/bs][bs/4][8][4], fp32 scales [N/32][K/bs][32][1], bs).
    The logical (unpacked) tensor is [N/32][K/bs][bs/4][32][4]."""
    W = _c(W, np.float32)
    N, K = W.shape
    if bs is None:
        bs = qint2_block_size(K, env_block)
    assert N % 32 == 0 and K % bs == 0 and bs % 4 == 0
    q = np.empty((N // 32, K // bs, bs // 4, 8, 4), np.uint8)
    sc = np.empty((N // 32, K // bs, 32, 1), np.float32)
    lib().orc_remap_quantize_qint2_intlv(_p(W), _c_i64(N), _c_i64(K), _c_i64(bs), _p(q), _p(sc))
    return q, sc, bs


def remap_quantize_qint2_intlv_chain(W, bs):
    """The same through a restatement of the reference's own view / permute / pack chain (numpy), the check of
    the closed form above.  W plain [N][K] fp32 (the reference first flattens its blocked input to this)."""
    W = np.ascontiguousarray(W, np.float32)
    N, K = W.shape
    K1, K2, K3, C3 = N // 32, 8, 4, 4
    C1, C2 = K // bs, bs // C3
    t = W.reshape(K1, K2 * K3, C1, bs).transpose(0, 2, 1, 3)
    amax = np.abs(t).max(-1, keepdims=True)
    scales = np.maximum(amax.astype(np.float32), np.float32(1.0e-8))
    qv = np.clip(np.rint((t / scales).astype(np.float32)), -1.0, 1.0).astype(np.int32).astype(np.uint8) & 0x3
    qv[qv == 3] = 2
    qv = np.ascontiguousarray(qv).reshape(K1, C1, K3, K2, C2, C3).transpose(2, 0, 1, 4, 3, 5)
    packed = qv[0] | (qv[1] << 2) | (qv[2] << 4) | (qv[3] << 6)
    return np.ascontiguousarray(packed).astype(np.uint8), np.ascontiguousarray(scales)


def qint2_to_qint8_layout(q2, sc2):
    """Ternary codes {0: 0, 1: +1, 2: -1} and scales of the interleaved 2-bit layout as an int8 weight in the QINT8
    reference layout (q [N/16][K/bs][bs/4][16][4] i8, scales [N/16][K/bs][1][16]): the operand the W2A8 GEMM
    (TppBlockedQInt8LinearW on a kQUInt2x4 weight, src/csrc/fused_gemm.h:1112-1128) multiplies."""
    q2 = _c(q2, np.uint8)
    n1, nb, c2, _, _ = q2.shape
    codes = np.stack([(q2 >> (2 * k3)) & 3 for k3 in range(4)], axis=3)        # [n1][nb][c2][k3][k2][c3]
    val = np.where(codes == 1, 1, np.where(codes == 2, -1, 0)).astype(np.int8)
    val = val.reshape(n1, nb, c2, 32, 4)                                        # row r = k3*8 + k2
    val = val.reshape(n1, nb, c2, 2, 16, 4).transpose(0, 3, 1, 2, 4, 5).reshape(n1 * 2, nb, c2, 16, 4)
    sc = _c(sc2, np.float32).reshape(n1, nb, 2, 16).transpose(0, 2, 1, 3).reshape(n1 * 2, nb, 1, 16)
    return np.ascontiguousarray(val), np.ascontiguousarray(sc)


def remap_and_quantize_mxfp4_blocked(Wb):
    """Full reference entry point on a blocked fp32 array (view/permute chain
    + generic quantiser).  -> (qdata [N/32,K/64,32,32] u8, scales [N/32,K/64,2,32] u8)"""
    t = remap_mxfp4(_c(Wb, np.float32))
    q, sc = quantize_mxfp4(t, 32, 2, True)
    return q.reshape(q.shape[:-1]), sc


def remap_and_quantize_qint8_blocked(Wb, env_block=256):
    """-> (q [N/bk,K/QBS,QBS/4,bk,4] i8, scales [N/bk,K/QBS,1,bk] f32, QBS)"""
    t, qbs = remap_qint8(_c(Wb, np.float32), env_block)
    q, sc = quantize_int8sym(t, qbs, 2, True)
    return q, sc, qbs


# closed-form (plain W[N,K]) versions coded in C -----------------------------
def remap_quantize_mxfp4(W):
    W = _c(W, np.float32)
    N, K = W.shape
    assert N % 32 == 0 and K % 64 == 0
    q = np.empty((N // 32, K // 64, 32, 32), np.uint8)
    sc = np.empty((N // 32, K // 64, 2, 32), np.uint8)
    lib().orc_remap_quantize_mxfp4(_p(W), _c_i64(N), _c_i64(K), _p(q), _p(sc))
    return q, sc


def dequantize_mxfp4_plain(q, sc):
    q = _c(q, np.uint8)
    sc = _c(sc, np.uint8)
    N, K = q.shape[0] * 32, q.shape[1] * 64
    W = np.empty((N, K), np.float32)
    lib().orc_dequantize_mxfp4(_p(q), _p(sc), _c_i64(N), _c_i64(K), _p(W))
    return W


def mxfp4_int8_layout(t):
    """The VNNI8-interleaved weight layout of remap_and_quantize_mxfp4 under USE_MXFP4_INT8 (qtypes.cpp:787-790,
    792-861) as ONE index map: blocked VNNI2 input [N/bk][K/bc][bc/2][bk][2] (bk, bc multiples of 8) ->
    [N/8][K/bc][bc/8][8][8], element [nb][c1][g][n8][j] = W[nb*8 + n8][c1*bc + g*8 + (j % 2)*4 + j // 2]
    (K values 0,4,1,5,2,6,3,7 of the group: a packed byte holds values i and 4 + i)."""
    t = _c(t, np.float32)
    K1, C1, C2, K2, C3 = t.shape
    assert C3 == 2 and K2 % 8 == 0 and C2 % 4 == 0
    N, bc = K1 * K2, C2 * 2
    W = t.transpose(0, 3, 1, 2, 4).reshape(N, C1 * bc)          # plain [N][K]
    g = W.reshape(N // 8, 8, C1, bc // 8, 2, 4)                 # [nb][n8][c1][g][i2][i4], k = i2*4 + i4
    return np.ascontiguousarray(g.transpose(0, 2, 3, 1, 5, 4).reshape(N // 8, C1, bc // 8, 8, 8))  # j = i4*2 + i2


def mxfp4_int8_layout_chain(t):
    """The same layout by the reference's own sequence of views and permutes (qtypes.cpp:792-811 with desired_K2 = 8,
    then :840-861), restated step by step: the pin of mxfp4_int8_layout()."""
    t = _c(t, np.float32)
    K1, C1, C2, K2, C3 = t.shape
    if K2 < 8 and 8 % K2 == 0:
        R = 8 // K2
        t = t.reshape(K1 // R, R, C1, C2, K2, C3).transpose(0, 2, 3, 1, 4, 5).reshape(K1 // R, C1, C2, R * K2, C3)
    elif K2 > 8 and K2 % 8 == 0:
        R = K2 // 8
        t = t.reshape(K1, C1, C2, R, 8, C3).transpose(0, 3, 1, 2, 4, 5).reshape(K1 * R, C1, C2, 8, C3)
    K1, C1, C2, K2, C3 = t.shape
    if C3 < 8:
        R = 8 // C3
        t = t.reshape(K1, C1, C2 // R, R, K2, C3).transpose(0, 1, 2, 4, 3, 5).reshape(K1, C1, C2 // R, K2, R * C3)
    sh = t.shape
    t = t.reshape(sh[:4] + (2, 4)).transpose(0, 1, 2, 3, 5, 4).reshape(sh)
    return np.ascontiguousarray(t)


def remap_quantize_mxfp4_int8(t):
    """remap_and_quantize_mxfp4 with USE_MXFP4_INT8 = 1 on a blocked VNNI2 weight: the layout above, then
    quantize_mxfp4(t, 32, 2, true) (qtypes.cpp:862).  -> (u8 [N/8][K/bc][bc/8][8][4], E8M0 u8 [N/8][K/bc][bc/32][8])."""
    v = mxfp4_int8_layout(t)
    return quantize_mxfp4(v, 32, 2, True)


W4A8_ACT_SCALE = np.float32(6.0 / 127.0)


def quantize_act_w4a8(x_f32):
    """Activations of the W4A8 GEMM (fused_gemm.h:970-977): quantize_int8sym over blocks of 32 of the last axis, the
    scales then multiplied in place by 6/127 (a float tensor times a scalar: fp32 product)."""
    xq, sa = quantize_int8sym(_c(x_f32, np.float32), 32, -1, False)
    return xq, (sa * W4A8_ACT_SCALE).astype(np.float32)


def linear_w4a8(x_bf16, q, sc, bc, bias=None, post=POST_NONE, post_in=None, post_in2=None, post_scale=1.0):
    x = bf16_to_f32(_c(x_bf16, np.uint16))
    xq, sa = quantize_act_w4a8(x)
    q = _c(q, np.uint8)
    sc = _c(sc, np.uint8)
    M, K = xq.shape
    N = q.shape[0] * 8
    assert q.shape[1] * bc == K and q.shape[2] * 8 == bc
    bias = None if bias is None else _c(bias, np.uint16)
    post_in = None if post_in is None else _c(post_in, np.uint16)
    post_in2 = None if post_in2 is None else _c(post_in2, np.uint16)
    y = np.empty((M, N), np.uint16)
    lib().orc_linear_w4a8(_p(xq), _p(sa), _c_i64(M), _c_i64(K), _p(q), _p(sc), _c_i64(N), _c_i64(bc), _p(bias),
                          ctypes.c_int(post), _p(post_in), _p(post_in2), ctypes.c_float(post_scale), _p(y))
    return y


def remap_quantize_qint8(W, qbs=None, env_block=256):
    W = _c(W, np.float32)
    N, K = W.shape
    if qbs is None:
        qbs = qint8_block_size(K, env_block)
    assert N % 16 == 0 and K % qbs == 0 and qbs % 64 == 0
    q = np.empty((N // 16, K // qbs, qbs // 4, 16, 4), np.int8)
    sc = np.empty((N // 16, K // qbs, 1, 16), np.float32)
    lib().orc_remap_quantize_qint8(_p(W), _c_i64(N), _c_i64(K), _c_i64(qbs), _p(q), _p(sc))
    return q, sc, qbs


def dequantize_qint8_plain(q, sc):
    q = _c(q, np.int8)
    sc = _c(sc, np.float32)
    n1, nb, a, bk, v = q.shape
    assert bk == 16 and v == 4
    qbs = a * 4
    N, K = n1 * 16, nb * qbs
    W = np.empty((N, K), np.float32)
    lib().orc_dequantize_qint8(_p(q), _p(sc), _c_i64(N), _c_i64(K), _c_i64(qbs), _p(W))
    return W


def quant_act_int8(x_bf16, qbs):
    x = _c(x_bf16, np.uint16)
    M, K = x.shape
    xq = np.empty((M, K), np.int8)
    sa = np.empty((M, K // qbs), np.float32)
    lib().orc_quant_act_int8(_p(x), _c_i64(M), _c_i64(K), _c_i64(qbs), _p(xq), _p(sa))
    return xq, sa


def qint8_block_sums(xq, q):
    xq = _c(xq, np.int8)
    q = _c(q, np.int8)
    M, K = xq.shape
    n1, nb, a, bk, v = q.shape
    N, qbs = n1 * 16, a * 4
    acc = np.empty((M, N, nb), np.int32)
    lib().orc_qint8_block_sums(_p(xq), _c_i64(M), _c_i64(K), _p(q), _c_i64(N), _c_i64(qbs), _p(acc))
    return acc


# ----------------------------------------------------------------------------
# post-ops and linears
# ----------------------------------------------------------------------------
def post_op(y_bf16, post, in1=None, in2=None, scale=1.0):
    y = _c(y_bf16, np.uint16).copy()
    in1 = None if in1 is None else _c(in1, np.uint16)
    in2 = None if in2 is None else _c(in2, np.uint16)
    lib().orc_post_op(_p(y), _c_i64(y.size), ctypes.c_int(post), _p(in1), _p(in2), ctypes.c_float(scale))
    return y


def linear_mxfp4(x_bf16, q, sc, bias=None, post=POST_NONE, post_in=None, post_in2=None,
                 post_scale=1.0, mode=MODE_IDEAL):
    x = _c(x_bf16, np.uint16)
    q = _c(q, np.uint8)
    sc = _c(sc, np.uint8)
    M, K = x.shape
    N = q.shape[0] * 32
    assert q.shape[1] * 64 == K
    bias = None if bias is None else _c(bias, np.uint16)
    post_in = None if post_in is None else _c(post_in, np.uint16)
    post_in2 = None if post_in2 is None else _c(post_in2, np.uint16)
    y = np.empty((M, N), np.uint16)
    lib().orc_linear_mxfp4(
        _p(x), _c_i64(M), _c_i64(K), _p(q), _p(sc), _c_i64(N), _p(bias), ctypes.c_int(post),
        _p(post_in), _p(post_in2), ctypes.c_float(post_scale), ctypes.c_int(mode), _p(y),
    )
    return y


def linear_qint8(x_bf16, q, sw, bias=None, post=POST_NONE, post_in=None, post_in2=None,
                 post_scale=1.0, mode=MODE_IDEAL):
    x = _c(x_bf16, np.uint16)
    q = _c(q, np.int8)
    sw = _c(sw, np.float32)
    M, K = x.shape
    n1, nb, a, bk, v = q.shape
    N, qbs = n1 * 16, a * 4
    assert nb * qbs == K
    bias = None if bias is None else _c(bias, np.uint16)
    post_in = None if post_in is None else _c(post_in, np.uint16)
    post_in2 = None if post_in2 is None else _c(post_in2, np.uint16)
    y = np.empty((M, N), np.uint16)
    lib().orc_linear_qint8(
        _p(x), _c_i64(M), _c_i64(K), _p(q), _p(sw), _c_i64(N), _c_i64(qbs), _p(bias),
        ctypes.c_int(post), _p(post_in), _p(post_in2), ctypes.c_float(post_scale),
        ctypes.c_int(mode), _p(y),
    )
    return y


def linear_qint8_f32(xq, sa, q, sw, bias=None):
    """TppBlockedQInt8LinearW<float, uint8_t, float> on pre-quantized activations (fused_gemm.h:1236-1249 with a
    quantized t_in, 1076-1341): xq int8 [M][K], sa f32 [M][K/qbs] (quantize_int8sym over the last axis), weight
    q [N/16][K/qbs][qbs/4][16][4] + sw [N/16][K/qbs][1][16]; fp32 bias or None; returns fp32 [M][N]."""
    xq = _c(xq, np.int8)
    sa = _c(sa, np.float32)
    q = _c(q, np.int8)
    sw = _c(sw, np.float32)
    M, K = xq.shape
    n1, nb, a, bk, v = q.shape
    N, qbs = n1 * 16, a * 4
    assert nb * qbs == K and sa.shape == (M, nb)
    bias = None if bias is None else _c(bias, np.float32)
    y = np.empty((M, N), np.float32)
    lib().orc_linear_qint8_f32(_p(xq), _p(sa), _c_i64(M), _c_i64(K), _p(q), _p(sw), _c_i64(N), _c_i64(qbs), _p(bias), _p(y))
    return y


def linear_bf16(x_bf16, w_bf16, bias=None, post=POST_NONE, post_in=None, post_in2=None, post_scale=1.0):
    """Unquantized bf16 weights, TppBlockedLinearW<bf16,bf16> (src/csrc/fused_gemm.h:785-1073, non-quantized branch
    :951-1064 with one K chunk, the M <= 256 case of getBlockingParams :695-721): the bf16 output tile starts as the
    bias, the BRGEMM adds the whole dot product (fp32 inside) and the sum is rounded to bf16 once; then the post-op.
    x bits [M][K], w bits [N][K] (plain layout).  Pinned by the MXFP4 restatement: on weights that MXFP4
    represents exactly both must agree (tests/test_oracle.py)."""
    x = bf16_to_f32(_c(x_bf16, np.uint16)).astype(np.float64)
    w = bf16_to_f32(_c(w_bf16, np.uint16)).astype(np.float64)
    acc = x @ w.T
    if bias is not None:
        acc = acc + bf16_to_f32(_c(bias, np.uint16)).astype(np.float64)[None, :]
    y = f32_to_bf16(acc.astype(np.float32))
    return post_op(y, post, post_in, post_in2, post_scale) if post != POST_NONE else y


# ----------------------------------------------------------------------------
# float / half activations on MXFP4 or unquantized bf16 weights: TppBlockedLinearW<Tin, uint8_t, Tout> and
# <Tin, bfloat16, Tout> with Tin = Tout = float or half (src/csrc/fused_gemm.h:1519-1523, 1541-1550, 785-1073; the
# element-type switch of fc_plain_wrap, src/csrc/llm/fused_llm_infer.cpp:1526-1545).  The activations keep their own
# precision and every weight value is exact in fp32, so the GEMM tile is the exact dot product (evaluated in fp64
# here) plus the bias, rounded once to T; post-ops then work on T, re-rounding to T where the CPU path stores its
# tile (src/csrc/fused_gemm.h:1343-1488).  Pinned by: fp64 matmul of the dequantized weight is the definition; on
# bf16-representable activations the T = float tile rounded to bf16 equals linear_mxfp4 / linear_bf16 (ideal mode)
# up to their fp32 summation order (tests/test_oracle.py).  libxsmm's own summation order and its sigmoid / GELU
# polynomials are not in the tree: parity unpinned for those, covered by the stated tolerance.
# ----------------------------------------------------------------------------
def post_op_wide(y, post, in1=None, in2=None, scale=1.0):
    """y, in1, in2: numpy float32 or float16 arrays of one shape; arithmetic in fp32, stores in y's dtype."""
    T = y.dtype.type
    rt = lambda a: np.asarray(a, np.float32).astype(T).astype(np.float32)  # noqa: E731
    yf = y.astype(np.float32)
    a = None if in1 is None else np.asarray(in1).astype(np.float32)
    b = None if in2 is None else np.asarray(in2).astype(np.float32)
    sc = np.float32(scale)
    if post == POST_SILU:
        out = yf * rt(np.float32(1.0) / (np.float32(1.0) + np.exp(-yf.astype(np.float64)).astype(np.float32)))
    elif post == POST_MUL:
        out = a * yf
    elif post == POST_ADD_SCALE:
        out = (a.astype(np.float64) * np.float64(sc) + yf.astype(np.float64)).astype(np.float32)  # one fused multiply-add
    elif post == POST_ADD2_SCALE:
        t = rt(yf + a)
        out = (b.astype(np.float64) * np.float64(sc) + t.astype(np.float64)).astype(np.float32)
    elif post == POST_GELU:
        from math import erf
        e = np.vectorize(erf)(yf.astype(np.float64) * 0.70710678118654752)
        out = (0.5 * yf.astype(np.float64) * (1.0 + e)).astype(np.float32)
    elif post == POST_RELU:
        out = np.where(yf < 0, np.float32(0), yf)
    else:
        out = yf
    return out.astype(T)


def _linear_wide(x, W_f32, bias, post, post_in, post_in2, post_scale):
    x = np.asarray(x)
    assert x.dtype in (np.float32, np.float16)
    acc = x.astype(np.float64) @ np.asarray(W_f32, np.float64).T
    if bias is not None:
        acc = acc + np.asarray(bias).astype(np.float64)[None, :]
    y = acc.astype(np.float32).astype(x.dtype)
    return post_op_wide(y, post, post_in, post_in2, post_scale)


def linear_mxfp4_wide(x, q, sc, bias=None, post=POST_NONE, post_in=None, post_in2=None, post_scale=1.0):
    """x float32 / float16 [M][K]; q, sc the reference-layout MXFP4 weight; bias / post inputs in x's dtype."""
    return _linear_wide(x, dequantize_mxfp4_plain(q, sc), bias, post, post_in, post_in2, post_scale)


def linear_bf16_wide(x, w_bf16, bias=None, post=POST_NONE, post_in=None, post_in2=None, post_scale=1.0):
    """x float32 / float16 [M][K]; w bits [N][K] (plain layout)."""
    return _linear_wide(x, bf16_to_f32(_c(w_bf16, np.uint16)), bias, post, post_in, post_in2, post_scale)


# ----------------------------------------------------------------------------
# MXFP8 activations of the opt-in FP8-activation GEMM.  No reference code to follow (its activations stay bf16):
# the OCP Microscaling v1.0 recipe -- E4M3 elements (bias 7, subnormals, maximum 448, no infinities), one E8M0
# scale per 32 values with exponent floor(log2 max|x|) - 8, round to nearest even, saturation.
# Pinned by known codes, the decode/encode round trip over all 254 finite codes and tie cases (tests/test_oracle.py).
# ----------------------------------------------------------------------------
def e4m3_decode(c):
    c = np.asarray(c, np.uint8).astype(np.int32)
    e, m = (c >> 3) & 15, c & 7
    mag = np.where(e == 0, m * 2.0 ** -9, (1.0 + m / 8.0) * 2.0 ** (e - 7.0))
    return np.where(c & 0x80, -mag, mag).astype(np.float32)


def e4m3_encode(v):
    v = np.asarray(v, np.float64)
    a = np.minimum(np.abs(v), 448.0)
    _, ex = np.frexp(a)                      # a = f * 2^ex, f in [0.5, 1)
    e = np.maximum(ex - 1, -6)               # exponent of the value's binade, subnormals share 2^-6's
    step = 2.0 ** (e - 3.0)
    r = np.rint(a / step) * step             # RNE at 3 mantissa bits
    _, ex2 = np.frexp(r)
    e2 = ex2 - 1
    normal = r >= 2.0 ** -6
    code = np.where(normal, ((e2 + 7) << 3) | np.rint((r / 2.0 ** e2.astype(np.float64) - 1.0) * 8).astype(np.int64),
                    np.rint(r * 512.0).astype(np.int64))
    return (code | np.where(np.signbit(v), 0x80, 0)).astype(np.uint8)


def quant_act_mxfp8(x_bf16):
    """bf16 bits [M][K] -> (codes u8 [M][K], scale bytes u8 [M][K/32])."""
    x = bf16_to_f32(_c(x_bf16, np.uint16))
    M, K = x.shape
    xb = x.reshape(M, K // 32, 32)
    amax = np.abs(xb).max(-1)
    E = (amax.view(np.uint32) >> 23) & 0xff
    X = np.clip(E.astype(np.int64) - 8, 0, 254)
    codes = e4m3_encode(xb.astype(np.float64) * 2.0 ** (127.0 - X)[..., None])
    return codes.reshape(M, K), X.astype(np.uint8)


def dequant_act_mxfp8(codes, scales):
    M, K = codes.shape
    v = e4m3_decode(codes).reshape(M, K // 32, 32).astype(np.float64) * 2.0 ** (scales.astype(np.float64) - 127.0)[..., None]
    return v.reshape(M, K)


def linear_mxfp4_fp8act(x_bf16, q, sc, bias=None, post=POST_NONE, post_in=None, post_in2=None, post_scale=1.0):
    """The MXFP4 linear on MXFP8-quantised activations: exact products, one rounding of bias + sum to bf16, post-op."""
    xd = dequant_act_mxfp8(*quant_act_mxfp8(x_bf16))
    w = dequantize_mxfp4_plain(q, sc).astype(np.float64)
    acc = xd @ w.T
    if bias is not None:
        acc = acc + bf16_to_f32(_c(bias, np.uint16)).astype(np.float64)[None, :]
    y = f32_to_bf16(acc.astype(np.float32))
    return post_op(y, post, post_in, post_in2, post_scale) if post != POST_NONE else y


def num_threads():
    return lib().orc_num_threads()


def set_num_threads(n):
    lib().orc_set_num_threads(ctypes.c_int(int(n)))


# ---------------------------------------------------------------------------
# Decode-side operators of the decoder layer (numpy restatements; float math,
# compared with a stated tolerance, not bit-exact)
# ---------------------------------------------------------------------------
def _bf16_round_f32(a):
    """fp32 array -> nearest-even bf16, returned as fp32 values."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint32) << 16
    return r.astype(np.uint32).view(np.float32)


def rms_norm(x_bf16, gamma_f32, eps):
    """RMSNormFwdTPP::ref (src/csrc/xsmm_functors.h:4628-4654) on rows of x: v = mean(x^2);
    s = 1/sqrt(v + eps); out = bf16((x*s)*gamma), all in fp32.  Returns bf16 bit patterns."""
    x = bf16_to_f32(_c(x_bf16, np.uint16))
    g = np.asarray(gamma_f32, np.float32)
    v = (x.astype(np.float32) ** 2).sum(-1, dtype=np.float32) * np.float32(1.0 / x.shape[-1])
    s = (np.float32(1.0) / np.sqrt(v + np.float32(eps), dtype=np.float32)).astype(np.float32)
    out = (x * s[..., None]).astype(np.float32) * g
    return f32_to_bf16(out.astype(np.float32))


def layer_norm(x_bf16, gamma_f32, beta_f32, eps):
    """LayerNormFwdTPP::ref (src/csrc/xsmm_functors.h:4786-4819, called per row by lyr_norm,
    src/csrc/llm/fused_llm_infer.cpp:254-282): m = mean(x); v = max(mean(x^2) - m^2, 0); s = 1/sqrt(v + eps);
    b = -s*m; out = bf16((x*s + b)*gamma + beta), all in fp32.  Returns bf16 bit patterns."""
    x = bf16_to_f32(_c(x_bf16, np.uint16)).astype(np.float32)
    g = np.asarray(gamma_f32, np.float32)
    bt = np.asarray(beta_f32, np.float32)
    c = np.float32(1.0 / x.shape[-1])
    m = x.sum(-1, dtype=np.float32) * c
    v = (x * x).sum(-1, dtype=np.float32) * c
    v = np.maximum(v - m * m, np.float32(0.0)).astype(np.float32)
    s = (np.float32(1.0) / np.sqrt(v + np.float32(eps), dtype=np.float32)).astype(np.float32)
    b = (np.float32(-1.0) * s * m).astype(np.float32)
    out = ((x * s[..., None] + b[..., None]).astype(np.float32) * g).astype(np.float32) + bt
    return f32_to_bf16(out.astype(np.float32))


def rotary_gptj(t_bf16, emb_pos, pos, N, H):
    """apply_rotary_pos_emb_gptj (src/csrc/llm/fused_llm_infer.cpp:150-205): t [B][S][N*H] bf16 bits, emb_pos f32
    [MP][HR] = sin | cos, pos i64 [B_pos][S]; pairs (h, h+1) for h < HR with sin = emb[p][h/2], cos = emb[p][HR/2 + h/2];
    out0 = in0*cos - in1*sin, out1 = in1*cos + in0*sin; positions >= MP untouched."""
    t = bf16_to_f32(_c(t_bf16, np.uint16)).copy()
    B, S = t.shape[0], t.shape[1]
    t = t.reshape(B, S, N, H)
    emb_pos = np.asarray(emb_pos, np.float32)
    MP, HR = emb_pos.shape
    coff = HR // 2
    for b in range(B):
        for s in range(S):
            p = int(pos[0 if pos.shape[0] == 1 else b][s])
            if p >= MP:
                continue
            sin, cos = emb_pos[p][:coff], emb_pos[p][coff:HR]
            in0, in1 = t[b, s, :, 0:HR:2].copy(), t[b, s, :, 1:HR:2].copy()
            t[b, s, :, 0:HR:2] = _bf16_round_f32(in0 * cos - in1 * sin)
            t[b, s, :, 1:HR:2] = _bf16_round_f32(in1 * cos + in0 * sin)
    return f32_to_bf16(t.reshape(B, S, N * H))


def rotary_llama(t_bf16, emb_pos, pos, N, H):
    """apply_rotary_pos_emb_llama (src/csrc/llm/fused_llm_infer.cpp:207-253): t [B][S][N*H] bf16 bits,
    emb_pos f32 [2][MP][HR] (cos, sin), pos i64 [B_pos][S]; pairs (h2, HR/2 + h2); positions >= MP untouched."""
    t = bf16_to_f32(_c(t_bf16, np.uint16)).copy()
    B, S = t.shape[0], t.shape[1]
    t = t.reshape(B, S, N, H)
    MP, HR = emb_pos.shape[1], emb_pos.shape[2]
    coff = HR // 2
    for b in range(B):
        for s in range(S):
            p = int(pos[0 if pos.shape[0] == 1 else b][s])
            if p >= MP:
                continue
            cos, sin = emb_pos[0][p][:coff].astype(np.float32), emb_pos[1][p][:coff].astype(np.float32)
            in0, in1 = t[b, s, :, :coff].copy(), t[b, s, :, coff:HR].copy()
            t[b, s, :, :coff] = _bf16_round_f32(in0 * cos - in1 * sin)
            t[b, s, :, coff:HR] = _bf16_round_f32(in1 * cos + in0 * sin)
    return f32_to_bf16(t.reshape(B, S, N * H))


def attn_decode(q_bf16, k_bf16, v_bf16, mask_f32=None, round_probs=True):
    """attn<T> (src/csrc/llm/attn.cpp:781-955) for one query token: q [B][Nq][H], k / v [B][Nkv][L][H] (bf16 bits),
    additive mask f32 [B][L] or None.  scores = q.k / sqrt(H) + mask (fp32); p = exp(s - max); the probabilities that
    multiply V are rounded to bf16 (the reference stores them in bf16, attn.cpp:900-905) while the normaliser sums
    the unrounded ones; output bf16.  Accumulation in fp64 here (the order-independent answer)."""
    q = bf16_to_f32(_c(q_bf16, np.uint16)).astype(np.float64)
    k = bf16_to_f32(_c(k_bf16, np.uint16)).astype(np.float64)
    v = bf16_to_f32(_c(v_bf16, np.uint16)).astype(np.float64)
    B, Nq, H = q.shape
    Nkv = k.shape[1]
    R = Nq // Nkv
    out = np.empty((B, Nq, H), np.float32)
    for b in range(B):
        for n in range(Nq):
            s = (k[b, n // R] @ q[b, n]) / np.sqrt(np.float64(H))
            if mask_f32 is not None:
                s = s + mask_f32[b][: s.shape[0]].astype(np.float64)
            p = np.exp(s - s.max())
            pb = _bf16_round_f32(p.astype(np.float32)).astype(np.float64) if round_probs else p
            out[b, n] = (pb @ v[b, n // R] / p.sum()).astype(np.float32)
    return f32_to_bf16(out)


def attn_prefill(q_bf16, k_bf16, v_bf16, mask_f32=None, round_probs=True):
    """attn<T> (src/csrc/llm/attn.cpp:781-955) with isCausal for S query tokens: q [B][S][Nq][H], k / v
    [B][Nkv][L][H] (bf16 bits; the last S keys belong to the S queries, attn.cpp:797 offset = key_len - Sq), additive
    mask f32 [B][L] or None.  Query i sees keys 0 .. L-S+i (the reference overwrites the later scores with -1e9,
    attn.cpp:884-900, whose exponential is exactly 0 in fp32); the rest as attn_decode: probabilities rounded to bf16
    before they multiply V, the normaliser sums the unrounded ones, fp64 accumulation, bf16 output [B][S][Nq][H]."""
    q = bf16_to_f32(_c(q_bf16, np.uint16)).astype(np.float64)
    k = bf16_to_f32(_c(k_bf16, np.uint16)).astype(np.float64)
    v = bf16_to_f32(_c(v_bf16, np.uint16)).astype(np.float64)
    B, S, Nq, H = q.shape
    Nkv, L = k.shape[1], k.shape[2]
    R = Nq // Nkv
    off = L - S
    out = np.empty((B, S, Nq, H), np.float32)
    for b in range(B):
        for n in range(Nq):
            sc = (q[b, :, n] @ k[b, n // R].T) / np.sqrt(np.float64(H))  # [S][L]
            if mask_f32 is not None:
                sc = sc + mask_f32[b][None, :L].astype(np.float64)
            for i in range(S):
                s = sc[i, : off + i + 1]
                p_ = np.exp(s - s.max())
                pb = _bf16_round_f32(p_.astype(np.float32)).astype(np.float64) if round_probs else p_
                out[b, i, n] = (pb @ v[b, n // R][: off + i + 1] / p_.sum()).astype(np.float32)
    return f32_to_bf16(out)
