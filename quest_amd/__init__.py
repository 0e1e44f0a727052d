"""quest_amd: the W4A4 linear-layer inference path of QuEST (gemm-quest) on MI355X / gfx950.

`import quest_amd as quest` gives the reference's `quest` call surface; `quest_amd.harness` holds
the counterparts of gemm-quest/benchmarks/utils.py (linear_forward, preprocess_weight, Linear4bit,
the timing helpers).
"""
from .api import (  # noqa: F401
    HADAMARD_ENTRY,
    add_mul_vv,
    find_scale_int4,
    fused_matmul_dequantize_int4_int4t,
    fused_matmul_dequantize_int4_int4t_bf16,
    fused_matmul_dequantize_swiglu_int4_int4t,
    swiglu_interleave_rows,
    generate_random_meta48_int4,
    hadamard128,
    hadamard_quantize_int4,
    matmul_int4_int4t_int32,
    matmul_int4sp_int4t_int32,
    quantize_int4,
    reorder_meta48_int4,
    rmsnorm_hadamard_quantize_int4,
    add_rmsnorm_hadamard_quantize_int4,
    rope_interleaved_,
    silu_mul_hadamard_quantize_int4,
    uncompress_meta48_int4,
    e2m3_tiles_bytes,
    int4_to_e2m3_tiles,
    fused_matmul_dequantize_e2m3,
    rope_gemm_fuses,
    fused_matmul_dequantize_rope_int4_int4t,
    fused_matmul_dequantize_add_int4_int4t,
    gemm_add_fuses,
    hadamard_quantize_e2m3,
    rmsnorm_hadamard_quantize_e2m3,
    add_rmsnorm_hadamard_quantize_e2m3,
    silu_mul_hadamard_quantize_e2m3,
    GEMM_WORKSPACE_MAX_BYTES,
    gemm_workspace,
    gemm_workspace_bytes,
)

__version__ = '0.1.0'
