"""Reference: REGISTER_SUBMODULE(_tpp_attn, m) (src/csrc/llm/attn.cpp:1955-1969): the KV cache class and the
attention entry point over it."""
from ..llm.fused_llama_infer import TppCache, attn  # noqa: F401
