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

    # -- weight geometry -----------------------------------------------------
    def is_weight(self):
        """True for the two weight layouts the linear kernels consume."""
        s = tuple(self.shape)
        if self._qscheme == QSCHEME_MXFP:
            return len(s) == 5 and s[2:] == (32, 32, 2) and self.block_size == 32 and self.is_vnni
        return (len(s) == 5 and s[3:] == (16, 4) and self.is_vnni and s[2] * 4 == self.block_size)

    def weight_nk(self):
        s = self.shape
        if self._qscheme == QSCHEME_MXFP:
            return s[0] * 32, s[1] * 64
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
            qn = torch.empty_like(self.qdata)
            if self._qscheme == QSCHEME_MXFP:
                sn = torch.empty_like(self.scales)
                _lib.check(L.tppx_prepack_mxfp4(self.qdata.data_ptr(), self.scales.data_ptr(), N, K,
                                                qn.data_ptr(), sn.data_ptr(), st))
            else:
                sn = self.scales
                _lib.check(L.tppx_prepack_qint8(self.qdata.data_ptr(), N, K, self.block_size,
                                                qn.data_ptr(), st))
            self._native = (qn, sn)
        return self._native

    def dequantize(self):
        """fp32 tensor in the blocked shape (PerBlock*Quantizer::dequantize,
        src/csrc/qtypes.cpp:438-473,521-577)."""
        L = _lib.lib()
        _lib.require_gpu(self.qdata, "quantized tensor")
        out = torch.empty(tuple(self.shape), dtype=torch.float32, device=self.device)
        st = _lib.stream_of(self.qdata)
        if self._qscheme == QSCHEME_MXFP:
            if not self.is_weight():
                raise _lib.TppxError(_lib.EUNSUPPORTED, f"dequantize: unsupported MXFP4 layout {self!r}")
            N, K = self.weight_nk()
            _lib.check(L.tppx_dequantize_mxfp4(self.qdata.data_ptr(), self.scales.data_ptr(), N, K,
                                               out.data_ptr(), st))
        elif self.is_weight():
            N, K = self.weight_nk()
            _lib.check(L.tppx_dequantize_qint8(self.qdata.data_ptr(), self.scales.data_ptr(), N, K,
                                               self.block_size, out.data_ptr(), st))
        else:
            raise _lib.TppxError(_lib.EUNSUPPORTED, f"dequantize: unsupported QINT8 layout {self!r}")
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
