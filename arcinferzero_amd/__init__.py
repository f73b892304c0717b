"""MI355X-native GGUF block-quantized matmul (prefill GEMM, decode GEMV, MoE grouped GEMM) behind a C ABI.

The compute path is the in-tree shared library ``libarcz_hip.so`` (hand-written HIP for gfx950 plus the C++ host
dispatch); this package is a thin ctypes binding over ``include/arcz_hip.h`` and ``include/arcz_engine.h`` with numpy
in and out.  There is no fallback: if the library is missing, importing :mod:`arcinferzero_amd.binding` raises.
"""
from .binding import (  # noqa: F401
    AR4_128, IQ3_S, IQ3_XXS, IQ4_NL, IQ4_XS, MXFP4, Q2_0, Q3_K, Q4_0, Q4_K, Q5_K, Q6_K, Q8_0, ArczError, Buffer, Engine, GgufFile, LaunchList, Runtime, Weight, MoeLayer, gen_normal, gen_weights, gguf_bytes,
    lib, lib_path, planes_bytes, quantize_rows, relayout_q4_0, repack_planes, self_check,
)
