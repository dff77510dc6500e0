"""Mirror of the reference's native module ``tpp_pytorch_extension._C``: the
sub-modules of the quantized-linear path (``_qtype``, ``_fused_llm_infer``,
``_xsmm``, ``_tpp_attn``), implemented over the HIP C ABI instead of pybind11."""
from . import _qtype
from . import _fused_llm_infer
from . import _xsmm
from . import _tpp_attn
