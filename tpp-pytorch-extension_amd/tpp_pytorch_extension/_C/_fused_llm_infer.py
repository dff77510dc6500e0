"""Reference: REGISTER_SUBMODULE(_fused_llm_infer, m)
(src/csrc/llm/fused_llm_infer.cpp:1568-1586); only the linear entry point and
its post-op variants are built."""
from .._ops import fc_plain, fc_add, fc_add2, fc_silu, fc_mul, fc_gelu, fc_relu, qkv_gemm, swiglu_gate_up, swiglu_mlp  # noqa: F401
