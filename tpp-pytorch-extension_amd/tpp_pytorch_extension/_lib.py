"""ctypes binding of libtppx_hip.so (the C ABI declared in include/tppx.h).

The HIP library is the only compute backend of this package: if it is missing
the import of any op fails loudly; there is no CPU or eager fallback.
"""
import ctypes
import threading
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libtppx_hip.so")

OK, EINVAL, ESHAPE, EUNSUPPORTED, EHIP = 0, -1, -2, -3, -4
POST_NONE, POST_SILU, POST_MUL, POST_ADD_SCALE, POST_ADD2_SCALE, POST_GELU, POST_RELU = range(7)
DT_F32, DT_BF16, DT_F16 = 0, 1, 2
W_MXFP4, W_BF16 = 0, 1
Q_MXFP4, Q_INT8, Q_INT4 = 0, 1, 2
FLAG_NONE, FLAG_FORCE_SKINNY, FLAG_FORCE_TILED, FLAG_ACT_FP8, FLAG_XQ_REUSE = 0, 1, 2, 4, 8


class TppxError(RuntimeError):
    """Raised where the reference would TPP_ASSERT (printf + exit) or TORCH_CHECK."""

    def __init__(self, code, msg):
        super().__init__(f"tppx error {code}: {msg}")
        self.code = code


class Seg(ctypes.Structure):
    _fields_ = [
        ("qw", ctypes.c_void_p),
        ("sw", ctypes.c_void_p),
        ("bias", ctypes.c_void_p),
        ("post_in", ctypes.c_void_p),
        ("post_in2", ctypes.c_void_p),
        ("y", ctypes.c_void_p),
        ("N", ctypes.c_int64),
        ("post_op", ctypes.c_int32),
        ("post_scale", ctypes.c_float),
    ]


_vp, _i64, _i32, _f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float

# name -> argtypes; every entry point declared in include/tppx.h
SIGNATURES = {
    "tppx_version": [],
    "tppx_last_error": [],
    "tppx_reload_env": [],
    "tppx_quantize_mxfp4": [_vp, _i32, _i64, _i64, _i64, _i64, _i64, _vp, _vp, _vp],
    "tppx_quantize_qint8": [_vp, _i32, _i64, _i64, _i64, _i64, _i64, _i64, _vp, _vp, _vp],
    "tppx_dequantize_mxfp4": [_vp, _vp, _i64, _i64, _vp, _vp],
    "tppx_dequantize_qint8": [_vp, _vp, _i64, _i64, _i64, _vp, _vp],
    "tppx_quantize_per_block": [_vp, _i32, _i32, _i64, _i64, _i64, _i64, _vp, _vp, _vp],
    "tppx_dequantize_per_block": [_vp, _vp, _i32, _i64, _i64, _i64, _i64, _vp, _vp],
    "tppx_quantize_qint2_intlv": [_vp, _i32, _i64, _i64, _i64, _i64, _i64, _i64, _vp, _vp, _vp],
    "tppx_dequantize_qint2_intlv": [_vp, _vp, _i64, _i64, _i64, _vp, _vp],
    "tppx_prepack_qint2": [_vp, _vp, _i64, _i64, _i64, _vp, _vp, _vp],
    "tppx_prepack_qint4": [_vp, _i64, _i64, _i64, _vp, _vp],
    "tppx_prepack_mxfp4": [_vp, _vp, _i64, _i64, _vp, _vp, _vp],
    "tppx_prepack_qint8": [_vp, _i64, _i64, _i64, _vp, _vp],
    "tppx_quant_act_int8": [_vp, _i64, _i64, _i64, _vp, _vp, _vp],
    "tppx_quant_act_mxfp8": [_vp, _i64, _i64, _vp, _vp, _vp],
    "tppx_prepack_bf16": [_vp, _i64, _i64, _i64, _i64, _i32, _vp, _vp],
    "tppx_linear_bf16": [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _f32, _i32, _vp],
    "tppx_linear_mxfp4": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _f32, _i32, _vp, _i64, _vp],
    "tppx_linear_qint8": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i32, _f32, _i32,
                          _vp, _i64, _vp],
    "tppx_linear_qint8_noalloc": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i32, _f32, _i32, _vp],
    "tppx_multi_linear_mxfp4": [_vp, ctypes.POINTER(Seg), _i32, _i64, _i64, _i32, _vp, _i64, _vp],
    "tppx_multi_linear_qint8": [_vp, _vp, _vp, ctypes.POINTER(Seg), _i32, _i64, _i64, _i64, _i32, _vp, _i64, _vp],
    "tppx_swiglu_mxfp4": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _vp, _i64, _vp],
    "tppx_norm_multi_linear_mxfp4": [_vp, _vp, ctypes.c_float, ctypes.POINTER(Seg), _i32, _i64, _i64, _i32, _vp],
    "tppx_norm_swiglu_mxfp4": [_vp, _vp, ctypes.c_float, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _vp],
    "tppx_linear_mxfp4_rowsq": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, ctypes.c_float, _i32, _vp, _i64, _vp, _vp],
    "tppx_normsq_multi_linear_mxfp4": [_vp, _vp, _vp, ctypes.c_float, ctypes.POINTER(Seg), _i32, _i64, _i64, _i32, _vp],
    "tppx_normsq_swiglu_mxfp4": [_vp, _vp, _vp, ctypes.c_float, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _vp],
    "tppx_rms_norm": [_vp, _vp, _i32, _vp, _i64, _i64, ctypes.c_float, _vp],
    "tppx_layer_norm": [_vp, _vp, _vp, _i32, _vp, _i64, _i64, ctypes.c_float, _vp],
    "tppx_rotary_gptj": [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _vp],
    "tppx_rotary_kv_append_gptj": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64,
                                   _i64, _i64, _vp],
    "tppx_rotary_llama": [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _vp],
    "tppx_rotary_kv_append_llama": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64,
                                    _i64, _i64, _vp],
    "tppx_linear_qint8_f32": [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp],
    "tppx_pack_qint_tiles": [_vp, _i64, _i64, _i32, _vp, _vp],
    "tppx_prepack_mxfp4_int8": [_vp, _vp, _i64, _i64, _i64, _vp, _vp, _vp],
    "tppx_linear_mxfp4_int8_rows": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _f32, _vp],
    "tppx_prepack_mxfp4_int8_wide": [_vp, _vp, _i64, _i64, _i64, _vp, _vp],
    "tppx_linear_mxfp4_int8_wide": [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _f32, _vp, _i64, _vp],
    "tppx_linear_qintx": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _i32, _f32, _i32, _vp],
    "tppx_linear_wide": [_vp, _i32, _vp, _vp, _i32, _vp, _vp, _i64, _i64, _i64, _vp],
    "tppx_post_op_wide": [_vp, _i32, _i32, _vp, _vp, _f32, _vp, _i64, _vp],
    "tppx_linear_mxfp4_int8": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i32, _f32, _vp],
    "tppx_greedy_next": [_vp, _i64, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _vp],
    "tppx_qkv_linear_mxfp4": [_vp, _vp, _vp, _f32, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i32, _vp],
    "tppx_attn_decode": [_vp, _vp, _vp, _vp, _i64, _vp, _i64, _vp, _i64, _i64, _i64, _i64, _i64, _vp, _i64, _vp],
    "tppx_attn_decode_rotary": [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _vp, _vp, _i64, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp, _i64, _vp],
    "tppx_attn_prefill": [_vp, _vp, _vp, _vp, _i64, _i64, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _vp],
    "tppx_plan_linear_mxfp4": [_i64, _i64, _i64, _i32, _i64, ctypes.c_char_p, _i64],
    "tppx_plan_linear_qint8": [_i64, _i64, _i64, _i64, _i32, _i32, _i64, ctypes.c_char_p, _i64],
    "tppx_plan_multi_linear_mxfp4": [ctypes.POINTER(_i64), _i32, _i64, _i64, _i32, _i32, _i64, ctypes.c_char_p, _i64],
    "tppx_plan_multi_linear_qint8": [ctypes.POINTER(_i64), _i32, _i64, _i64, _i64, _i32, _i32, _i64, ctypes.c_char_p,
                                     _i64],
}

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: the HIP extension has not been built "
                "(run __graft_entry__.build() or `make -C tpp-pytorch-extension_amd/csrc`). "
                "This package has no fallback path."
            )
        L = ctypes.CDLL(LIB_PATH)
        for name, argtypes in SIGNATURES.items():
            fn = getattr(L, name)
            fn.argtypes = argtypes
            fn.restype = ctypes.c_int
        L.tppx_last_error.restype = ctypes.c_char_p
        _lib = L
    return _lib


def check(rc):
    if rc != OK:
        raise TppxError(rc, lib().tppx_last_error().decode())


def ptr(t):
    """Device pointer of a tensor, or NULL for None / an empty tensor."""
    if t is None or t.numel() == 0:
        return None
    return t.data_ptr()


def stream_of(t):
    return torch.cuda.current_stream(t.device).cuda_stream


WORKSPACE_BYTES = 32 << 20
MAX_STREAM_WORKSPACES = 8  # per device; the least recently used one beyond that is released
_workspaces = {}
_workspaces_lock = threading.Lock()
_workspace_use = {}  # (device, stream) -> tick of its last use
_tick = 0


def workspace(t):
    """Split-K / staging scratch for an op on `t`'s device (see include/tppx.h).
    One zero-initialised buffer per (device, stream): every op orders itself on
    the caller's current stream, so threads that work on streams of their own
    never share scratch and need no ordering between them. Work recorded under
    stream capture uses one more buffer per device, created together with the
    device's first eager one (a capture cannot allocate it): run the op once
    eagerly before capturing, and order replays of different graphs that use
    these ops with respect to each other.  A device keeps at most
    MAX_STREAM_WORKSPACES per-stream buffers: beyond that the least recently
    used one goes back to torch's allocator (it was allocated on its own stream,
    so work still queued there keeps it valid)."""
    global _tick
    dev = t.device.index
    if torch.cuda.is_current_stream_capturing():
        ws = _workspaces.get((dev, "capture"))
        if ws is None:
            raise TppxError(EINVAL, "first call on this device happens inside graph capture: run the op once "
                                    "eagerly before capturing so that its workspace exists")
        return ws
    key = (dev, stream_of(t))
    ws = _workspaces.get(key)
    if ws is None:
        with _workspaces_lock:
            ws = _workspaces.get(key)
            if ws is None:
                if (dev, "capture") not in _workspaces:
                    cap = torch.zeros(WORKSPACE_BYTES, dtype=torch.uint8, device=t.device)
                    torch.cuda.current_stream(t.device).synchronize()  # zeroed before any capture stream sees it
                    _workspaces[(dev, "capture")] = cap
                mine = [k for k in _workspace_use if k[0] == dev]
                if len(mine) >= MAX_STREAM_WORKSPACES:
                    old = min(mine, key=_workspace_use.get)
                    _workspace_use.pop(old)
                    _workspaces.pop(old, None)
                ws = torch.zeros(WORKSPACE_BYTES, dtype=torch.uint8, device=t.device)
                _workspaces[key] = ws
    _tick += 1
    _workspace_use[key] = _tick
    return ws


def require_gpu(t, what):
    if not t.is_cuda:
        raise TppxError(
            EINVAL,
            f"{what} must live on the GPU (got device {t.device}); the quantized-linear "
            "path runs only as HIP kernels and has no CPU fallback",
        )
