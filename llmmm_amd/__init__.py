"""llmmm_amd: MI355X (gfx950) implementation of LLMMM's matrix-multiplication core.

``llmmm_amd.mm`` mirrors the reference's host entry points on torch CUDA tensors;
``llmmm_amd._lib`` is the raw ctypes view of the C ABI in ``include/llmmm.h``.
"""
from . import _lib  # noqa: F401  (raises if libllmmm.so has not been built)
from .mm import (  # noqa: F401
    construct_mfma_B_layout,
    fp16_gemm,
    fp16_mm,
    fp8_blockwise_symmetric_quantization,
    PlanesRmsnorm,
    fp8_gemm_add_rmsnorm_quant,
    fp8_gemm_planes,
    fp8_gemm_qkv_rope,
    fp8_gemm_blockwise_quant_A_1x128__B_128x128__C_1x128__output_fp8,
    fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_bf16,
    fp8_gemm_blockwise_quant_A_1x128__B_128x128__swiglu__C_1x128__output_fp8,
    fp8_gemm_blockwise_quant_A_1x128__B_128x128__output_fp32,
    make_workspace,
    preshuffle_weight,
    quantize_activation,
    quantize_weight,
    query_config,
    restore_B_layout,
    rmsnorm_quantize_activation,
    transpose_matrix__aligned_128,
    workspace_bytes,
)
