"""MI355X-native quantized-GEMM path (quant_dot int8/fp8 + fused dequantizelinear,
int4 weight-only GEMM) behind MIGraphX's operator semantics.

The product is the C-ABI shared library ``lib/libmi355_qgemm.so`` declared in
``include/mi355_qgemm.h``; this package only locates, builds and binds it."""
from .capi import (  # noqa: F401
    DT, QP, W4ZP, QuantDotDesc, Mi355Error, lib, lib_path, build_library,
)
