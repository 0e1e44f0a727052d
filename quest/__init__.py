"""Drop-in name: `import quest` resolves to the MI355X implementation in quest_amd."""
from quest_amd.api import *  # noqa: F401,F403
from quest_amd.api import (  # noqa: F401
    add_mul_vv, find_scale_int4, fused_matmul_dequantize_int4_int4t_bf16, generate_random_meta48_int4,
    matmul_int4_int4t_int32, matmul_int4sp_int4t_int32, quantize_int4, reorder_meta48_int4, uncompress_meta48_int4,
)
