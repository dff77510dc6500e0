"""Reference: REGISTER_SUBMODULE(_qtype, m) (src/csrc/qtypes.cpp:1075-1093)."""
from .._ops import (  # noqa: F401
    quantize_mxfp,
    quantize_mxfp4,
    quantize_int8sym,
    quantize_int4sym,
    create_qtensor_int8sym,
    create_qtensor_int2sym,
    q_per_block_scales,
    q_per_block_pack_size,
    q_per_block_block_size,
    q_per_block_axis,
    remap_and_quantize_mxfp4,
    remap_and_quantize_qint8,
    remap_and_quantize_qint2_intlv,
    fix_vnni,
)
