"""Stand-in for the reference's custom quantized tensor.

The reference builds an ``at::QTensorImpl`` carrying a ``PerBlockMxFPQuantizer``
/ ``PerBlockAffineQuantizer`` (``src/csrc/qtypes.h:284-389``,
``src/csrc/qtypes.cpp:345-411``).  Such an object cannot be made without a
C++ torch extension, so the same observable surface is provided by a wrapper
tensor subclass: ``is_quantized``, ``dtype`` (``quint4x2`` / ``qint8``), the
blocked logical ``shape`` (``size(-1)`` = 2 / 4), ``qscheme()``,
``dequantize()`` and the per-block accessors.  ``qdata`` / ``scales`` hold the
reference storage layout byte for byte; a GPU-native re-layout is built on
first use and cached next to it (the role the reference's cached first-token
weights play, ``src/csrc/llm/fused_llm_infer.cpp:1216-1227``).
"""
import torch

from . import _lib

QSCHEME_MXFP = "per_block_mxfp"      # reference: kPerBlockMxFP (hijacks kPerChannelSymmetric, qtypes.h:11)
QSCHEME_AFFINE = "per_block_affine"  # reference: kPerBlockAffine (hijacks kPerTensorSymmetric, qtypes.h:12)


class QTensor(torch.Tensor):
    @staticmethod
    def __new__(cls, qdata, scales, shape, qdtype, qscheme, block_size, axis, is_vnni, pack_size):
        r = torch.Tensor._make_wrapper_subclass(
            cls, tuple(shape), dtype=qdtype, device=qdata.device, requires_grad=False
        )
        r.qdata = qdata
        r.scales = scales
        r._qscheme = qscheme
        r.block_size = int(block_size)
        r.axis = int(axis)
        r.is_vnni = bool(is_vnni)
        r.pack_size = int(pack_size)
        r._native = None
        return r

    # -- observable surface of a quantized at::Tensor ------------------------
    @property
    def is_quantized(self):
        return True

    def qscheme(self):
        return torch.per_channel_symmetric if self._qscheme == QSCHEME_MXFP else torch.per_tensor_symmetric

    def __repr__(self):
        return (
            f"QTensor(shape={tuple(self.shape)}, dtype={self.dtype}, qscheme={self._qscheme}, "
            f"block_size={self.block_size}, axis={self.axis}, is_vnni={self.is_vnni}, device={self.device})"
        )

    def _clone_with(self, qdata, scales):
        q = QTensor(qdata, scales, self.shape, self.dtype, self._qscheme, self.block_size,
                    self.axis, self.is_vnni, self.pack_size)
        return q

    # -- per-block geometry (PerBlockQuantizer, src/csrc/qtypes.h:30-68) ------
    def geometry(self):
        """(pre, bs, post, vnni) of the logical tensor viewed as [pre][bs][post][vnni]."""
        sizes = list(self.shape)
        axis = self.axis
        if self.is_vnni:
            vnni = sizes.pop()
        else:
            vnni = self.pack_size
            sizes[axis] //= vnni
        bsi = self.block_size // vnni
        sizes[axis] //= bsi
        pre = 1
        for d in sizes[: axis + 1]:
            pre *= d
        post = 1
        for d in sizes[axis + 1:]:
            post *= d
        return pre, bsi, post, vnni

    # -- weight geometry -----------------------------------------------------
    def weight_kind(self):
        """Which linear-layer weight layout this is: "mxfp4" [N/32, K/64, 32, 32, 2], "mxfp4_int8" (the VNNI8-interleaved
        W4A8 layout) [N/8, K/bc, bc/8, 8, 8], "qint8" [N/16, K/QBS, QBS/4, 16, 4], "qint4" (VNNI2) [N/16, K/QBS, QBS/2,
        16, 2], "qint2" (interleaved ternary) [N/32, K/QBS, QBS/4, 32, 4]; None for any other layout (helper-only
        tensors, quantized activations)."""
        s = tuple(self.shape)
        if len(s) != 5 or not self.is_vnni or self.axis != 2:
            return None
        if self._qscheme == QSCHEME_MXFP:
            if s[2:] == (32, 32, 2) and self.block_size == 32:
                return "mxfp4"
            if s[3:] == (8, 8) and self.block_size == 32 and s[2] % 4 == 0 and (s[0] * 8) % 16 == 0:
                return "mxfp4_int8"
            return None
        if self.dtype == torch.qint8 and s[3:] == (16, 4) and s[2] * 4 == self.block_size:
            return "qint8"
        if self.dtype == torch.quint4x2 and s[3:] == (16, 2) and s[2] * 2 == self.block_size and self.block_size % 64 == 0:
            return "qint4"
        if self.dtype == torch.quint2x4 and s[3:] == (32, 4) and s[2] * 4 == self.block_size and self.block_size % 64 == 0:
            return "qint2"
        return None

    def is_weight(self):
        """True for the weight layouts the linear kernels consume."""
        return self.weight_kind() is not None

    def weight_nk(self):
        s = self.shape
        kind = self.weight_kind()
        if kind == "mxfp4":
            return s[0] * 32, s[1] * 64
        if kind == "mxfp4_int8":
            return s[0] * 8, s[1] * s[2] * 8
        if kind == "qint2":
            return s[0] * 32, s[1] * self.block_size
        return s[0] * 16, s[1] * self.block_size

    def native(self):
        """(qdata_native, scales_for_kernel), built once."""
        if self._native is None:
            L = _lib.lib()
            _lib.require_gpu(self.qdata, "quantized weight")
            if not self.is_weight():
                raise _lib.TppxError(_lib.EUNSUPPORTED, f"not a linear-layer weight layout: {self!r}")
            N, K = self.weight_nk()
            st = _lib.stream_of(self.qdata)
            kind = self.weight_kind()
            if kind == "mxfp4":
                qn = torch.empty_like(self.qdata)
                sn = torch.empty_like(self.scales)
                _lib.check(L.tppx_prepack_mxfp4(self.qdata.data_ptr(), self.scales.data_ptr(), N, K,
                                                qn.data_ptr(), sn.data_ptr(), st))
            elif kind == "mxfp4_int8":
                qn, sn = self.qdata, self.scales  # the W4A8 kernel reads the reference layout as it is
            elif kind == "qint8":
                qn = torch.empty_like(self.qdata)
                sn = self.scales
                _lib.check(L.tppx_prepack_qint8(self.qdata.data_ptr(), N, K, self.block_size,
                                                qn.data_ptr(), st))
            elif kind == "qint4":
                # low-bit affine weights run on the W8A8 kernels: codes expanded once into native int8 tiles
                qn = torch.empty(N * K, dtype=torch.int8, device=self.qdata.device)
                sn = self.scales
                _lib.check(L.tppx_prepack_qint4(self.qdata.data_ptr(), N, K, self.block_size, qn.data_ptr(), st))
            else:
                qn = torch.empty(N * K, dtype=torch.int8, device=self.qdata.device)
                sn = torch.empty((N // 16, K // self.block_size, 1, 16), dtype=torch.float32, device=self.qdata.device)
                _lib.check(L.tppx_prepack_qint2(self.qdata.data_ptr(), self.scales.data_ptr(), N, K, self.block_size,
                                                qn.data_ptr(), sn.data_ptr(), st))
            self._native = (qn, sn)
        return self._native

    def native_packed(self):
        """QINT4 / QINT2 weights: (codes at their own width in the decode kernel's order, scales, bits) --
        N*K*bits/8 bytes made once from the native int8 tiles (tppx_pack_qint_tiles)."""
        have = getattr(self, "_native_packed", None)
        if have is None:
            kind = self.weight_kind()
            if kind not in ("qint4", "qint2"):
                raise _lib.TppxError(_lib.EUNSUPPORTED, f"only QINT4 / QINT2 weights have a packed native form: {self!r}")
            bits = 4 if kind == "qint4" else 2
            qn, sn = self.native()
            N, K = self.weight_nk()
            packed = torch.empty(N * K * bits // 8, dtype=torch.uint8, device=qn.device)
            _lib.check(_lib.lib().tppx_pack_qint_tiles(qn.data_ptr(), N, K, bits, packed.data_ptr(), _lib.stream_of(qn)))
            have = self._native_packed = (packed, sn, bits)
        return have

    def native_w4a8(self):
        """W4A8 (USE_MXFP4_INT8) weights: (codes in MFMA operand order, E8M0 scales per tile and channel) for the
        decode kernel, made once from the reference layout (tppx_prepack_mxfp4_int8); None when K is not a multiple
        of 128 or N of 16."""
        have = getattr(self, "_native_w4a8", None)
        if have is None:
            if self.weight_kind() != "mxfp4_int8":
                raise _lib.TppxError(_lib.EUNSUPPORTED, f"not a W4A8 weight: {self!r}")
            N, K = self.weight_nk()
            if N % 16 or K % 128:
                have = self._native_w4a8 = ()
            else:
                qn = torch.empty(N * K // 2, dtype=torch.uint8, device=self.qdata.device)
                sn = torch.empty(N * K // 32, dtype=torch.uint8, device=self.qdata.device)
                _lib.check(_lib.lib().tppx_prepack_mxfp4_int8(self.qdata.data_ptr(), self.scales.data_ptr(), N, K,
                                                              self.shape[2] * 8, qn.data_ptr(), sn.data_ptr(),
                                                              _lib.stream_of(self.qdata)))
                have = self._native_w4a8 = (qn, sn)
        return have or None

    def native_w4a8_wide(self):
        """W4A8 (USE_MXFP4_INT8) weights for passes of many rows: bf16 operand tiles holding integer * 2^(e - 127),
        2 bytes per weight, made once (tppx_prepack_mxfp4_int8_wide); None when K is not a multiple of 128 or N of
        16."""
        have = getattr(self, "_native_w4a8_wide", None)
        if have is None:
            if self.weight_kind() != "mxfp4_int8":
                raise _lib.TppxError(_lib.EUNSUPPORTED, f"not a W4A8 weight: {self!r}")
            N, K = self.weight_nk()
            if N % 16 or K % 128:
                have = self._native_w4a8_wide = ()
            else:
                wn = torch.empty(N * K, dtype=torch.bfloat16, device=self.qdata.device)
                _lib.check(_lib.lib().tppx_prepack_mxfp4_int8_wide(self.qdata.data_ptr(), self.scales.data_ptr(), N, K,
                                                                   self.shape[2] * 8, wn.data_ptr(),
                                                                   _lib.stream_of(self.qdata)))
                have = self._native_w4a8_wide = (wn,)
        return have[0] if have else None

    def dequantize(self):
        """fp32 tensor in the blocked shape (PerBlock*Quantizer::dequantize,
        src/csrc/qtypes.cpp:438-473,521-577)."""
        L = _lib.lib()
        _lib.require_gpu(self.qdata, "quantized tensor")
        out = torch.empty(tuple(self.shape), dtype=torch.float32, device=self.device)
        if out.numel() == 0:
            return out
        st = _lib.stream_of(self.qdata)
        kind = self.weight_kind()
        if kind == "mxfp4":
            N, K = self.weight_nk()
            _lib.check(L.tppx_dequantize_mxfp4(self.qdata.data_ptr(), self.scales.data_ptr(), N, K,
                                               out.data_ptr(), st))
        elif kind == "qint8":
            N, K = self.weight_nk()
            _lib.check(L.tppx_dequantize_qint8(self.qdata.data_ptr(), self.scales.data_ptr(), N, K,
                                               self.block_size, out.data_ptr(), st))
        elif self.dtype == torch.quint2x4:
            if kind != "qint2":
                raise _lib.TppxError(_lib.EUNSUPPORTED, f"dequantize: only the interleaved ternary weight layout "
                                                        f"is defined for 2-bit tensors, got {self!r}")
            N, K = self.weight_nk()
            _lib.check(L.tppx_dequantize_qint2_intlv(self.qdata.data_ptr(), self.scales.data_ptr(), N, K,
                                                     self.block_size, out.data_ptr(), st))
        else:  # any other layout: the generic per-block kernel (quantized activations, helper-made tensors)
            pre, bs, post, vnni = self.geometry()
            fmt = (_lib.Q_MXFP4 if self._qscheme == QSCHEME_MXFP
                   else (_lib.Q_INT8 if self.dtype == torch.qint8 else _lib.Q_INT4))
            _lib.check(L.tppx_dequantize_per_block(self.qdata.data_ptr(), self.scales.data_ptr(), fmt, pre, bs, post,
                                                   vnni, out.data_ptr(), st))
        return out

    @classmethod
    def __torch_dispatch__(cls, func, types, args=(), kwargs=None):
        kwargs = kwargs or {}
        from . import _ops

        handler = _ops.DISPATCH.get(func)
        if handler is not None:
            return handler(*args, **kwargs)
        if func in (torch.ops.aten.detach.default, torch.ops.aten.alias.default):
            a = args[0]
            q = a._clone_with(a.qdata, a.scales)
            q._native = a._native
            return q
        if func is torch.ops.aten._to_copy.default:
            a = args[0]
            dev = kwargs.get("device", None)
            if kwargs.get("dtype", None) not in (None, a.dtype):
                raise _lib.TppxError(_lib.EUNSUPPORTED, "a quantized tensor cannot change dtype; call dequantize()")
            if dev is None or torch.device(dev) == a.device:
                return a
            return a._clone_with(a.qdata.to(dev), a.scales.to(dev))
        if func is torch.ops.aten.dequantize.self:
            return args[0].dequantize()
        raise _lib.TppxError(
            _lib.EUNSUPPORTED,
            f"{func} is not defined for the per-block quantized tensor; use dequantize() first",
        )
