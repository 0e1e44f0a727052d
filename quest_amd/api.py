"""The `quest` call surface of the reference (gemm-quest/quest/__init__.py:6-130) on MI355X.

Same names, argument order, defaults and return values; the work is done by hand-written HIP
kernels reached through the C ABI of libquest_hip.so.  Differences, all additive:
  * float16 is accepted wherever the reference asserts bfloat16;
  * `hadamard128` and `hadamard_quantize_int4` are new (the fused activation kernel);
  * the 4:8-sparse entry points raise NotImplementedError (NVIDIA sparse tensor cores only).
"""
from __future__ import annotations

import ctypes

import torch

from . import _lib
from ._lib import DTYPE_CODE, check, ptr, require_gpu, stream_of

_FLOAT16S = (torch.bfloat16, torch.float16)
HADAMARD_ENTRY = 181. / 2048.        # bf16(2**-3.5) == fp16(2**-3.5): what the reference's matrix holds


def fused_matmul_dequantize_int4_int4t_bf16(
        mat_a: torch.Tensor,
        mat_b: torch.Tensor,
        vec_a_add: torch.Tensor,
        vec_b_add: torch.Tensor,
        vec_a_mul: torch.Tensor,
        vec_b_mul: torch.Tensor,
        out: torch.Tensor = None,
        workspace: torch.Tensor = None,
) -> torch.Tensor:
    """gemm-quest/quest/__init__.py:6-20.  The output dtype follows vec_a_mul (bf16 or fp16).

    `workspace` (not in the reference): a uint8 tensor from `gemm_workspace`, which lets up to 16 tokens split K across
    workgroups; the result is the same bit for bit.  One workspace serves any number of calls on one stream."""
    if out is None:
        out = torch.empty(mat_a.size(0), mat_b.size(0), dtype=vec_a_mul.dtype, device=mat_a.device)
    assert mat_a.dtype == torch.uint8 and mat_b.dtype == torch.uint8 and vec_a_add.dtype == torch.int32 and vec_b_add.dtype == torch.int32
    assert vec_a_mul.dtype in _FLOAT16S and vec_b_mul.dtype == vec_a_mul.dtype and out.dtype == vec_a_mul.dtype
    assert mat_a.is_contiguous() and mat_b.is_contiguous() and vec_a_add.is_contiguous() and vec_b_add.is_contiguous() and vec_a_mul.is_contiguous() and vec_b_mul.is_contiguous() and out.is_contiguous()
    assert mat_a.size(1) == mat_b.size(1) and vec_a_add.numel() == mat_a.size(0) and vec_a_mul.numel() == mat_a.size(0)
    assert vec_b_add.numel() == mat_b.size(0) and vec_b_mul.numel() == mat_b.size(0)
    assert out.size(0) == mat_a.size(0) and out.size(1) == mat_b.size(0)
    dev = require_gpu(mat_a, mat_b, vec_a_add, vec_b_add, vec_a_mul, vec_b_mul, out)
    with torch.cuda.device(dev):
        if workspace is not None:
            assert workspace.dtype == torch.uint8 and workspace.is_contiguous() and workspace.device == out.device
            check(_lib.load().quest_fused_matmul_dequantize_int4_int4t_ws(
                ptr(out), ptr(mat_a), ptr(mat_b), ptr(vec_a_add), ptr(vec_b_add), ptr(vec_a_mul), ptr(vec_b_mul),
                mat_a.size(0), mat_b.size(1) * 2, mat_b.size(0), DTYPE_CODE[out.dtype], ptr(workspace), workspace.numel(),
                stream_of(out)), 'fused_matmul_dequantize_int4_int4t_ws')
        else:
            check(_lib.load().quest_fused_matmul_dequantize_int4_int4t(
                ptr(out), ptr(mat_a), ptr(mat_b), ptr(vec_a_add), ptr(vec_b_add), ptr(vec_a_mul), ptr(vec_b_mul),
                mat_a.size(0), mat_b.size(1) * 2, mat_b.size(0), DTYPE_CODE[out.dtype], stream_of(out)),
                'fused_matmul_dequantize_int4_int4t')
    return out


def fused_matmul_dequantize_rope_int4_int4t(
        mat_a: torch.Tensor,
        mat_b: torch.Tensor,
        vec_a_add: torch.Tensor,
        vec_b_add: torch.Tensor,
        vec_a_mul: torch.Tensor,
        vec_b_mul: torch.Tensor,
        freqs_cis: torch.Tensor,
        rot_cols: int,
        head_dim: int,
        out: torch.Tensor = None,
) -> torch.Tensor:
    """`fused_matmul_dequantize_int4_int4t_bf16` followed by `rope_interleaved_` on the first rot_cols channels (row r is
    position r % T of its sequence, T = freqs_cis.size(0)): in the GEMM's launch where a tiled kernel takes the
    shape, as the two calls otherwise -- the same bits either way."""
    m, n, t = mat_a.size(0), mat_b.size(0), freqs_cis.size(0)
    if out is None:
        out = torch.empty(m, n, dtype=vec_a_mul.dtype, device=mat_a.device)
    assert mat_a.dtype == torch.uint8 and mat_b.dtype == torch.uint8 and vec_a_add.dtype == torch.int32 and vec_b_add.dtype == torch.int32
    assert vec_a_mul.dtype in _FLOAT16S and vec_b_mul.dtype == vec_a_mul.dtype and out.dtype == vec_a_mul.dtype
    assert mat_a.is_contiguous() and mat_b.is_contiguous() and vec_a_add.is_contiguous() and vec_b_add.is_contiguous() and vec_a_mul.is_contiguous() and vec_b_mul.is_contiguous() and out.is_contiguous()
    assert mat_a.size(1) == mat_b.size(1) and vec_a_add.numel() == m and vec_a_mul.numel() == m
    assert vec_b_add.numel() == n and vec_b_mul.numel() == n and out.shape == (m, n)
    assert freqs_cis.dtype == torch.float32 and freqs_cis.is_contiguous() and freqs_cis.shape == (t, head_dim // 2, 2)
    assert m % t == 0 and 0 < rot_cols <= n and rot_cols % head_dim == 0
    dev = require_gpu(mat_a, mat_b, vec_a_add, vec_b_add, vec_a_mul, vec_b_mul, freqs_cis, out)
    with torch.cuda.device(dev):
        rc = _lib.load().quest_fused_matmul_dequantize_rope_int4_int4t(
            ptr(out), ptr(mat_a), ptr(mat_b), ptr(vec_a_add), ptr(vec_b_add), ptr(vec_a_mul), ptr(vec_b_mul),
            m, mat_b.size(1) * 2, n, DTYPE_CODE[out.dtype], ptr(freqs_cis), t, rot_cols, head_dim, stream_of(out))
    if rc in (QUEST_ERR_UNSUPPORTED, QUEST_ERR_BAD_SHAPE):          # nothing was launched: the two calls
        fused_matmul_dequantize_int4_int4t_bf16(mat_a, mat_b, vec_a_add, vec_b_add, vec_a_mul, vec_b_mul, out)
        rope_interleaved_(out.view(m // t, t, n), freqs_cis, rot_cols, head_dim)
        return out
    check(rc, 'fused_matmul_dequantize_rope_int4_int4t')
    return out


def gemm_add_fuses(size_m: int, size_k: int, size_n: int, device=None) -> bool:
    """Whether `fused_matmul_dequantize_add_int4_int4t` runs this size as one launch on `device` (the current one by default)."""
    dev = torch.device('cuda', torch.cuda.current_device()) if device is None else torch.device(device)
    with torch.cuda.device(dev):
        return bool(_lib.load().quest_fused_matmul_dequantize_add_available(
            size_m, size_k, size_n, ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)))


def fused_matmul_dequantize_add_int4_int4t(
        mat_a: torch.Tensor,
        mat_b: torch.Tensor,
        vec_a_add: torch.Tensor,
        vec_b_add: torch.Tensor,
        vec_a_mul: torch.Tensor,
        vec_b_mul: torch.Tensor,
        out: torch.Tensor,
) -> torch.Tensor:
    """out <- dtype(out + dtype(product)) with the product of `fused_matmul_dequantize_int4_int4t_bf16`: the bits of torch's
    `out + product` (the residual addition after a projection), in the GEMM's launch where `gemm_add_fuses` says so and as
    two launches otherwise."""
    m, n = mat_a.size(0), mat_b.size(0)
    assert mat_a.dtype == torch.uint8 and mat_b.dtype == torch.uint8 and vec_a_add.dtype == torch.int32 and vec_b_add.dtype == torch.int32
    assert vec_a_mul.dtype in _FLOAT16S and vec_b_mul.dtype == vec_a_mul.dtype and out.dtype == vec_a_mul.dtype
    assert mat_a.is_contiguous() and mat_b.is_contiguous() and vec_a_add.is_contiguous() and vec_b_add.is_contiguous() and vec_a_mul.is_contiguous() and vec_b_mul.is_contiguous() and out.is_contiguous()
    assert mat_a.size(1) == mat_b.size(1) and vec_a_add.numel() == m and vec_a_mul.numel() == m
    assert vec_b_add.numel() == n and vec_b_mul.numel() == n and out.shape == (m, n)
    dev = require_gpu(mat_a, mat_b, vec_a_add, vec_b_add, vec_a_mul, vec_b_mul, out)
    with torch.cuda.device(dev):
        rc = _lib.load().quest_fused_matmul_dequantize_add_int4_int4t(
            ptr(out), ptr(mat_a), ptr(mat_b), ptr(vec_a_add), ptr(vec_b_add), ptr(vec_a_mul), ptr(vec_b_mul),
            m, mat_b.size(1) * 2, n, DTYPE_CODE[out.dtype], stream_of(out))
    if rc == QUEST_ERR_UNSUPPORTED:                                  # nothing was launched: the two calls
        out += fused_matmul_dequantize_int4_int4t_bf16(mat_a, mat_b, vec_a_add, vec_b_add, vec_a_mul, vec_b_mul)
        return out
    check(rc, 'fused_matmul_dequantize_add_int4_int4t')
    return out


GEMM_WORKSPACE_MAX_BYTES = 16384 + (2 << 20)         # the most quest_gemm_workspace_bytes returns for any shape


def gemm_workspace_bytes(size_m: int, size_k: int, size_n: int) -> int:
    """Bytes of workspace the split-K decode GEMM uses for this shape (0: it does not split)."""
    return int(_lib.load().quest_gemm_workspace_bytes(size_m, size_k, size_n))


def gemm_workspace(device, nbytes: int = GEMM_WORKSPACE_MAX_BYTES) -> torch.Tensor:
    """A zeroed workspace for `fused_matmul_dequantize_int4_int4t(..., workspace=)`; every call leaves it reusable."""
    return torch.zeros(nbytes, dtype=torch.uint8, device=device)


# the same kernel serves both 16-bit float types
fused_matmul_dequantize_int4_int4t = fused_matmul_dequantize_int4_int4t_bf16


def swiglu_interleave_rows(n_out: int, device=None) -> torch.Tensor:
    """Row order `fused_matmul_dequantize_swiglu_int4_int4t` expects of a (2 H, ...) gate-over-up weight stack: the
    index tensor p with stacked[p] = rows in eights, four gate rows followed by the four up rows of the same outputs."""
    assert n_out % 4 == 0
    g = torch.arange(n_out, device=device).view(-1, 1, 4)
    return torch.cat((g, g + n_out), dim=1).reshape(-1)


def fused_matmul_dequantize_swiglu_int4_int4t(
        mat_a: torch.Tensor,
        mat_b: torch.Tensor,
        vec_a_add: torch.Tensor,
        vec_b_add: torch.Tensor,
        vec_a_mul: torch.Tensor,
        vec_b_mul: torch.Tensor,
        out: torch.Tensor = None,
) -> torch.Tensor:
    """The gate/up GEMM of a SwiGLU MLP with `silu(gate) * up` (src/models/llama.py:117-118 of the reference) applied
    in its epilogue: mat_b (2 H, K/2) and the vec_b_* hold the rows in `swiglu_interleave_rows` order; returns (M, H).
    Raises RuntimeError (QUEST_ERR_UNSUPPORTED) for M <= 64 or K % 128 != 0."""
    m, n = mat_a.size(0), mat_b.size(0)
    if out is None:
        out = torch.empty(m, n // 2, dtype=vec_a_mul.dtype, device=mat_a.device)
    assert mat_a.dtype == torch.uint8 and mat_b.dtype == torch.uint8 and vec_a_add.dtype == torch.int32 and vec_b_add.dtype == torch.int32
    assert vec_a_mul.dtype in _FLOAT16S and vec_b_mul.dtype == vec_a_mul.dtype and out.dtype == vec_a_mul.dtype
    for t in (mat_a, mat_b, vec_a_add, vec_b_add, vec_a_mul, vec_b_mul, out):
        assert t.is_contiguous()
    assert mat_a.size(1) == mat_b.size(1) and vec_a_add.numel() == m and vec_a_mul.numel() == m
    assert vec_b_add.numel() == n and vec_b_mul.numel() == n and n % 8 == 0 and out.shape == (m, n // 2)
    dev = require_gpu(mat_a, mat_b, vec_a_add, vec_b_add, vec_a_mul, vec_b_mul, out)
    with torch.cuda.device(dev):
        check(_lib.load().quest_fused_matmul_dequantize_swiglu_int4_int4t(
            ptr(out), ptr(mat_a), ptr(mat_b), ptr(vec_a_add), ptr(vec_b_add), ptr(vec_a_mul), ptr(vec_b_mul),
            m, mat_b.size(1) * 2, n, DTYPE_CODE[out.dtype], stream_of(out)),
            'fused_matmul_dequantize_swiglu_int4_int4t')
    return out


def matmul_int4_int4t_int32(
        mat_a: torch.Tensor,
        mat_b: torch.Tensor,
        out: torch.Tensor = None,
) -> torch.Tensor:
    """gemm-quest/quest/__init__.py:23-33."""
    if out is None:
        out = torch.empty(mat_a.size(0), mat_b.size(0), dtype=torch.int32, device=mat_a.device)
    assert mat_a.dtype == torch.uint8 and mat_b.dtype == torch.uint8 and out.dtype == torch.int32
    assert mat_a.is_contiguous() and mat_b.is_contiguous() and out.is_contiguous()
    assert mat_a.size(1) == mat_b.size(1) and out.size(0) == mat_a.size(0) and out.size(1) == mat_b.size(0)
    dev = require_gpu(mat_a, mat_b, out)
    with torch.cuda.device(dev):
        check(_lib.load().quest_matmul_int4_int4t_int32(
            ptr(out), ptr(mat_a), ptr(mat_b), mat_a.size(0), mat_b.size(1) * 2, mat_b.size(0), stream_of(out)),
            'matmul_int4_int4t_int32')
    return out


def _sparse_unsupported(*_args, **_kwargs):
    raise NotImplementedError(
        'the 4:8-sparse INT4 path of the reference targets NVIDIA sparse tensor cores and is not part of this build')


# gemm-quest/quest/__init__.py:36-84
matmul_int4sp_int4t_int32 = _sparse_unsupported
reorder_meta48_int4 = _sparse_unsupported
uncompress_meta48_int4 = _sparse_unsupported
generate_random_meta48_int4 = _sparse_unsupported


def find_scale_int4(
        x: torch.Tensor,
        scale: torch.Tensor = None,
) -> torch.Tensor:
    """gemm-quest/quest/__init__.py:87-96."""
    if scale is None:
        scale = torch.empty(x.size(0), 1, dtype=x.dtype, device=x.device)
    assert x.dtype in _FLOAT16S and scale.dtype == x.dtype
    assert x.is_contiguous() and scale.is_contiguous()
    assert x.dim() == 2 and scale.numel() == x.size(0)
    dev = require_gpu(x, scale)
    with torch.cuda.device(dev):
        check(_lib.load().quest_find_scale_int4(ptr(scale), ptr(x), x.size(1), x.size(0), DTYPE_CODE[x.dtype],
                                                stream_of(x)), 'find_scale_int4')
    return scale


def quantize_int4(
        x: torch.Tensor,
        scale: torch.Tensor,
        x_int: torch.Tensor = None,
        x_int_packed: torch.Tensor = None,
        x_int_row_sum: torch.Tensor = None,
        do_dequantize: bool = False,
) -> tuple[torch.Tensor, torch.Tensor | None, torch.Tensor | None, torch.Tensor | None]:
    """gemm-quest/quest/__init__.py:99-114.  Outputs passed as None are not produced."""
    assert x.dtype in _FLOAT16S and scale.dtype == x.dtype
    assert x_int is None or x_int.dtype == torch.int8
    assert x_int_packed is None or x_int_packed.dtype == torch.uint8
    assert x_int_row_sum is None or x_int_row_sum.dtype == torch.int32
    assert x.is_contiguous() and scale.is_contiguous()
    assert all(t is None or t.is_contiguous() for t in (x_int, x_int_packed, x_int_row_sum))
    assert x.dim() == 2 and scale.numel() == x.size(0)
    assert x_int is None or x_int.shape == x.shape
    assert x_int_packed is None or (x_int_packed.size(0) == x.size(0) and x_int_packed.size(1) * 2 == x.size(1))
    assert x_int_row_sum is None or x_int_row_sum.numel() == x.size(0)
    dev = require_gpu(x, scale, x_int, x_int_packed, x_int_row_sum)
    with torch.cuda.device(dev):
        check(_lib.load().quest_quantize_int4(ptr(x), ptr(scale), ptr(x_int), ptr(x_int_packed), ptr(x_int_row_sum),
                                              x.size(1), x.size(0), int(bool(do_dequantize)), DTYPE_CODE[x.dtype],
                                              stream_of(x)), 'quantize_int4')
    return x, x_int, x_int_packed, x_int_row_sum


def add_mul_vv(
        vec_a_add: torch.Tensor,
        vec_a_mul: torch.Tensor,
        vec_b_add: torch.Tensor,
        vec_b_mul: torch.Tensor,
        mat_c: torch.Tensor,
        mat_d: torch.Tensor = None,
) -> torch.Tensor:
    """gemm-quest/quest/__init__.py:117-130."""
    if mat_d is None:
        mat_d = torch.empty(mat_c.shape, dtype=vec_a_mul.dtype, device=mat_c.device)
    assert vec_a_add.dtype == torch.int32 and vec_b_add.dtype == torch.int32 and mat_c.dtype == torch.int32
    assert vec_a_mul.dtype in _FLOAT16S and vec_b_mul.dtype == vec_a_mul.dtype and mat_d.dtype == vec_a_mul.dtype
    assert vec_a_add.is_contiguous() and vec_a_mul.is_contiguous() and vec_b_add.is_contiguous() and vec_b_mul.is_contiguous() and mat_c.is_contiguous() and mat_d.is_contiguous()
    assert mat_c.dim() == 2 and mat_d.shape == mat_c.shape
    assert vec_a_add.numel() == mat_c.size(0) and vec_a_mul.numel() == mat_c.size(0)
    assert vec_b_add.numel() == mat_c.size(1) and vec_b_mul.numel() == mat_c.size(1)
    dev = require_gpu(vec_a_add, vec_a_mul, vec_b_add, vec_b_mul, mat_c, mat_d)
    with torch.cuda.device(dev):
        check(_lib.load().quest_add_mul_vv(ptr(mat_d), ptr(vec_a_add), ptr(vec_a_mul), ptr(vec_b_add), ptr(vec_b_mul),
                                           ptr(mat_c), mat_c.size(0), mat_c.size(1), DTYPE_CODE[mat_d.dtype],
                                           stream_of(mat_d)), 'add_mul_vv')
    return mat_d


def hadamard128(x: torch.Tensor, out: torch.Tensor = None, scale: float = HADAMARD_ENTRY) -> torch.Tensor:
    """Block-128 Walsh-Hadamard transform along the last dimension.  scale=181/2048 is the
    activation transform of linear_forward (gemm-quest/benchmarks/utils.py:17,89-90),
    scale=2**-3.5 the weight transform of preprocess_weight (utils.py:38-39).  out may be x."""
    if out is None:
        out = torch.empty_like(x)
    assert x.dtype in _FLOAT16S and out.dtype == x.dtype and out.shape == x.shape
    assert x.is_contiguous() and out.is_contiguous()
    k = x.size(-1)
    dev = require_gpu(x, out)
    with torch.cuda.device(dev):
        check(_lib.load().quest_hadamard128(ptr(out), ptr(x), k, x.numel() // k, float(scale), DTYPE_CODE[x.dtype],
                                            stream_of(x)), 'hadamard128')
    return out


def hadamard_quantize_int4(
        x: torch.Tensor,
        scale: torch.Tensor = None,
        x_int_packed: torch.Tensor = None,
        x_int_row_sum: torch.Tensor = None,
        x_had: torch.Tensor = None,
        hadamard_scale: float = HADAMARD_ENTRY,
        scale_rule: str = 'gaussian',
        from_fp32: bool = False,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """One pass over x: block-128 Hadamard (skipped when hadamard_scale == 0), Gaussian-clip scale,
    INT4 codes packed two per byte, and their row sums -- the three launches of
    gemm-quest/benchmarks/utils.py:89-100 in one.  x_had, if given, receives the transformed
    activations the codes were computed from.  scale_rule: 'gaussian' (the reference's RMS rule) or 'absmax'
    (scale = max|x| / 7.5 + 1e-8).  from_fp32: scale and codes from the transform's fp32 output (the arithmetic of the
    reference's evaluation-side fake quantiser, src/eval_hswag.py:201-214) instead of from the dtype-rounded tensor.
    Returns (scale, x_int_packed, x_int_row_sum)."""
    m, k = x.shape
    rule = {'gaussian': 0, 'absmax': 1}[scale_rule] | (4 if from_fp32 else 0)
    if scale is None:
        scale = torch.empty(m, 1, dtype=x.dtype, device=x.device)
    if x_int_packed is None:
        x_int_packed = torch.empty(m, k // 2, dtype=torch.uint8, device=x.device)
    if x_int_row_sum is None:
        x_int_row_sum = torch.empty(m, 1, dtype=torch.int32, device=x.device)
    assert x.dtype in _FLOAT16S and scale.dtype == x.dtype and x_int_packed.dtype == torch.uint8 and x_int_row_sum.dtype == torch.int32
    assert x.is_contiguous() and scale.is_contiguous() and x_int_packed.is_contiguous() and x_int_row_sum.is_contiguous()
    assert scale.numel() == m and x_int_row_sum.numel() == m and x_int_packed.shape == (m, k // 2)
    assert x_had is None or (x_had.dtype == x.dtype and x_had.shape == x.shape and x_had.is_contiguous())
    dev = require_gpu(x, scale, x_int_packed, x_int_row_sum, x_had)
    with torch.cuda.device(dev):
        check(_lib.load().quest_hadamard_quantize_int4_rule(ptr(x), ptr(scale), ptr(x_int_packed), ptr(x_int_row_sum),
                                                            ptr(x_had), k, m, float(hadamard_scale), rule,
                                                            DTYPE_CODE[x.dtype], stream_of(x)), 'hadamard_quantize_int4')
    return scale, x_int_packed, x_int_row_sum


def _quant_outputs(m, k, dtype, device, scale, x_int_packed, x_int_row_sum):
    if scale is None:
        scale = torch.empty(m, 1, dtype=dtype, device=device)
    if x_int_packed is None:
        x_int_packed = torch.empty(m, k // 2, dtype=torch.uint8, device=device)
    if x_int_row_sum is None:
        x_int_row_sum = torch.empty(m, 1, dtype=torch.int32, device=device)
    assert scale.dtype == dtype and x_int_packed.dtype == torch.uint8 and x_int_row_sum.dtype == torch.int32
    assert scale.is_contiguous() and x_int_packed.is_contiguous() and x_int_row_sum.is_contiguous()
    assert scale.numel() == m and x_int_row_sum.numel() == m and x_int_packed.shape == (m, k // 2)
    return scale, x_int_packed, x_int_row_sum


def rmsnorm_hadamard_quantize_int4(
        x: torch.Tensor,
        norm_weight: torch.Tensor,
        eps: float,
        scale: torch.Tensor = None,
        x_int_packed: torch.Tensor = None,
        x_int_row_sum: torch.Tensor = None,
        x_had: torch.Tensor = None,
        x_norm: torch.Tensor = None,
        hadamard_scale: float = HADAMARD_ENTRY,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """RMSNorm (src/models/llama.py:71-77 of the reference) and `hadamard_quantize_int4` of its output in one pass
    over x (M, K <= 4096): the normalised tensor is not written unless x_norm is given.  Raises RuntimeError with
    status QUEST_ERR_UNSUPPORTED for longer rows.  Returns (scale, x_int_packed, x_int_row_sum)."""
    m, k = x.shape
    assert x.dtype in _FLOAT16S and x.is_contiguous() and norm_weight.dtype == x.dtype and norm_weight.numel() == k
    assert norm_weight.is_contiguous()
    scale, x_int_packed, x_int_row_sum = _quant_outputs(m, k, x.dtype, x.device, scale, x_int_packed, x_int_row_sum)
    for t in (x_had, x_norm):
        assert t is None or (t.dtype == x.dtype and t.shape == x.shape and t.is_contiguous())
    dev = require_gpu(x, norm_weight, scale, x_int_packed, x_int_row_sum, x_had, x_norm)
    with torch.cuda.device(dev):
        check(_lib.load().quest_rmsnorm_hadamard_quantize_int4(
            ptr(x), ptr(norm_weight), float(eps), ptr(scale), ptr(x_int_packed), ptr(x_int_row_sum), ptr(x_had),
            ptr(x_norm), k, m, float(hadamard_scale), DTYPE_CODE[x.dtype], stream_of(x)), 'rmsnorm_hadamard_quantize_int4')
    return scale, x_int_packed, x_int_row_sum


def add_rmsnorm_hadamard_quantize_int4(
        x: torch.Tensor,
        branch: torch.Tensor,
        norm_weight: torch.Tensor,
        eps: float,
        scale: torch.Tensor = None,
        x_int_packed: torch.Tensor = None,
        x_int_row_sum: torch.Tensor = None,
        hadamard_scale: float = HADAMARD_ENTRY,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """`x += branch` (the residual addition of src/models/llama.py:175-176, in place) followed by
    `rmsnorm_hadamard_quantize_int4(x, ...)`, in one pass over the two tensors (M, K <= 4096).
    Returns (scale, x_int_packed, x_int_row_sum); x holds the sum afterwards."""
    m, k = x.shape
    assert x.dtype in _FLOAT16S and x.is_contiguous() and branch.dtype == x.dtype and branch.shape == x.shape
    assert branch.is_contiguous() and branch.data_ptr() != x.data_ptr()
    assert norm_weight.dtype == x.dtype and norm_weight.numel() == k and norm_weight.is_contiguous()
    scale, x_int_packed, x_int_row_sum = _quant_outputs(m, k, x.dtype, x.device, scale, x_int_packed, x_int_row_sum)
    dev = require_gpu(x, branch, norm_weight, scale, x_int_packed, x_int_row_sum)
    with torch.cuda.device(dev):
        check(_lib.load().quest_add_rmsnorm_hadamard_quantize_int4(
            ptr(x), ptr(branch), ptr(norm_weight), float(eps), ptr(scale), ptr(x_int_packed), ptr(x_int_row_sum),
            k, m, float(hadamard_scale), DTYPE_CODE[x.dtype], stream_of(x)), 'add_rmsnorm_hadamard_quantize_int4')
    return scale, x_int_packed, x_int_row_sum


def silu_mul_hadamard_quantize_int4(
        gate_up: torch.Tensor,
        scale: torch.Tensor = None,
        x_int_packed: torch.Tensor = None,
        x_int_row_sum: torch.Tensor = None,
        x_had: torch.Tensor = None,
        x_act: torch.Tensor = None,
        hadamard_scale: float = HADAMARD_ENTRY,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """silu(gate) * up (src/models/llama.py:117-118 of the reference) and `hadamard_quantize_int4` of the product in
    one pass over gate_up (M, 2 K), gate in the first K columns and up in the last K, K <= 4096.  x_act, if given,
    receives the product (M, K).  Returns (scale, x_int_packed, x_int_row_sum)."""
    m, k2 = gate_up.shape
    k = k2 // 2
    assert gate_up.dtype in _FLOAT16S and gate_up.is_contiguous() and k2 == 2 * k
    scale, x_int_packed, x_int_row_sum = _quant_outputs(m, k, gate_up.dtype, gate_up.device, scale, x_int_packed, x_int_row_sum)
    for t in (x_had, x_act):
        assert t is None or (t.dtype == gate_up.dtype and t.shape == (m, k) and t.is_contiguous())
    dev = require_gpu(gate_up, scale, x_int_packed, x_int_row_sum, x_had, x_act)
    with torch.cuda.device(dev):
        check(_lib.load().quest_silu_mul_hadamard_quantize_int4(
            ptr(gate_up), ptr(scale), ptr(x_int_packed), ptr(x_int_row_sum), ptr(x_had), ptr(x_act), k, m,
            float(hadamard_scale), DTYPE_CODE[gate_up.dtype], stream_of(gate_up)), 'silu_mul_hadamard_quantize_int4')
    return scale, x_int_packed, x_int_row_sum


def rope_interleaved_(x: torch.Tensor, freqs_cis: torch.Tensor, rot_cols: int, head_dim: int) -> torch.Tensor:
    """In-place rotary embedding of the first rot_cols columns of x (B, T, C) (src/models/llama.py:43-62 of the
    reference, for q and k at once when x is the fused QKV projection and rot_cols = 2 d).  freqs_cis: fp32
    (T, head_dim / 2, 2)."""
    b, t, c = x.shape
    assert x.dtype in _FLOAT16S and x.is_contiguous()
    assert freqs_cis.dtype == torch.float32 and freqs_cis.is_contiguous() and freqs_cis.shape == (t, head_dim // 2, 2)
    dev = require_gpu(x, freqs_cis)
    with torch.cuda.device(dev):
        check(_lib.load().quest_rope_interleaved(ptr(x), ptr(freqs_cis), b * t, t, c, rot_cols, head_dim,
                                                 DTYPE_CODE[x.dtype], stream_of(x)), 'rope_interleaved')
    return x


# ---- the FP6 matrix-core path: codes kept as "E2M3 tiles" (see include/quest_hip.h) ---------------------------------
def e2m3_tiles_bytes(rows: int, k: int) -> int:
    """Bytes of the E2M3 tiles of a (rows, k) code matrix."""
    n = _lib.load().quest_e2m3_tiles_bytes(rows, k)
    if n == 0:
        raise RuntimeError(f'E2M3 tiles need rows > 0 and K % 64 == 0; got ({rows}, {k})')
    return n


def int4_to_e2m3_tiles(x_int_packed: torch.Tensor, out: torch.Tensor = None) -> torch.Tensor:
    """Packed INT4 codes (rows, K/2) uint8 -> their E2M3 tiles (flat uint8): the operand form of
    `fused_matmul_dequantize_e2m3`, each code q stored as the FP6 E2M3 value q + 1/2."""
    rows, k = x_int_packed.size(0), x_int_packed.size(1) * 2
    if out is None:
        out = torch.empty(e2m3_tiles_bytes(rows, k), dtype=torch.uint8, device=x_int_packed.device)
    assert x_int_packed.dtype == torch.uint8 and x_int_packed.is_contiguous() and x_int_packed.dim() == 2
    assert out.dtype == torch.uint8 and out.is_contiguous() and out.numel() == e2m3_tiles_bytes(rows, k)
    dev = require_gpu(x_int_packed, out)
    with torch.cuda.device(dev):
        check(_lib.load().quest_int4_to_e2m3_tiles(ptr(out), ptr(x_int_packed), rows, k, stream_of(out)), 'int4_to_e2m3_tiles')
    return out


def rope_gemm_fuses(seq_len: int, n: int, rot_cols: int, head_dim: int) -> bool:
    """Whether `fused_matmul_dequantize_e2m3(rope=...)` takes these shapes (otherwise: the GEMM, then `rope_interleaved_`)."""
    return seq_len >= 32 and n % 8 == 0 and head_dim % 32 == 0 and 0 < rot_cols <= n and rot_cols % head_dim == 0


def fused_matmul_dequantize_e2m3(
        a_tiles: torch.Tensor,
        b_tiles: torch.Tensor,
        vec_a_mul: torch.Tensor,
        vec_b_mul: torch.Tensor,
        size_k: int,
        out: torch.Tensor = None,
        swiglu: bool = False,
        add_to_out: bool = False,
        rope: tuple = None,
) -> torch.Tensor:
    """`fused_matmul_dequantize_int4_int4t_bf16` for codes held as E2M3 tiles: (M, N) outputs identical bit for bit,
    from the FP6 matrix instructions; the add vectors are not needed (2 C + a_add + b_add is twice the FP6 sum).
    M and N are the lengths of the scale vectors.  swiglu=True: the epilogue of
    `fused_matmul_dequantize_swiglu_int4_int4t`, b in its interleaved row order, (M, N / 2) outputs.
    add_to_out=True: `out` (required) becomes dtype(out + dtype(product)), the bits of `out + product` in torch -- the
    residual addition after a projection, in the projection's launch.
    rope=(freqs_cis, rot_cols, head_dim): `rope_interleaved_` on the first rot_cols channels of the result, in the same
    launch and with the same bits; row r is position r % T of its sequence, T = freqs_cis.size(0) (see `rope_gemm_fuses`
    for the shapes this takes)."""
    m, n = vec_a_mul.numel(), vec_b_mul.numel()
    assert not (add_to_out and (swiglu or out is None)) and not (rope is not None and (swiglu or add_to_out))
    if out is None:
        out = torch.empty(m, n // 2 if swiglu else n, dtype=vec_a_mul.dtype, device=a_tiles.device)
    assert a_tiles.dtype == torch.uint8 and b_tiles.dtype == torch.uint8 and a_tiles.is_contiguous() and b_tiles.is_contiguous()
    assert a_tiles.numel() == e2m3_tiles_bytes(m, size_k) and b_tiles.numel() == e2m3_tiles_bytes(n, size_k)
    assert vec_a_mul.dtype in _FLOAT16S and vec_b_mul.dtype == vec_a_mul.dtype and out.dtype == vec_a_mul.dtype
    assert vec_a_mul.is_contiguous() and vec_b_mul.is_contiguous() and out.is_contiguous()
    assert out.shape == (m, n // 2 if swiglu else n)
    dev = require_gpu(a_tiles, b_tiles, vec_a_mul, vec_b_mul, out)
    fn = _lib.load().quest_fused_matmul_dequantize_swiglu_e2m3 if swiglu else _lib.load().quest_fused_matmul_dequantize_e2m3
    if add_to_out:
        fn = _lib.load().quest_fused_matmul_dequantize_add_e2m3
    if rope is not None:
        freqs_cis, rot_cols, head_dim = rope
        assert freqs_cis.dtype == torch.float32 and freqs_cis.is_contiguous() and freqs_cis.shape[1:] == (head_dim // 2, 2)
        assert rope_gemm_fuses(freqs_cis.size(0), n, rot_cols, head_dim), 'shape outside the fused rotary epilogue'
        require_gpu(freqs_cis, out)
        with torch.cuda.device(dev):
            check(_lib.load().quest_fused_matmul_dequantize_rope_e2m3(
                ptr(out), ptr(a_tiles), ptr(b_tiles), ptr(vec_a_mul), ptr(vec_b_mul), m, size_k, n, DTYPE_CODE[out.dtype],
                ptr(freqs_cis), freqs_cis.size(0), rot_cols, head_dim, stream_of(out)), 'fused_matmul_dequantize_rope_e2m3')
        return out
    with torch.cuda.device(dev):
        check(fn(ptr(out), ptr(a_tiles), ptr(b_tiles), ptr(vec_a_mul), ptr(vec_b_mul), m, size_k, n,
                 DTYPE_CODE[out.dtype], stream_of(out)), 'fused_matmul_dequantize_e2m3')
    return out


QUEST_ERR_UNSUPPORTED = -5
QUEST_ERR_BAD_SHAPE = -2


def hadamard_quantize_e2m3(
        x: torch.Tensor,
        scale: torch.Tensor = None,
        x_tiles: torch.Tensor = None,
        x_int_packed: torch.Tensor = None,
        x_int_row_sum: torch.Tensor = None,
        x_had: torch.Tensor = None,
        hadamard_scale: float = HADAMARD_ENTRY,
) -> tuple[torch.Tensor, torch.Tensor]:
    """`hadamard_quantize_int4` with the codes written as E2M3 tiles (one pass over x).  x_int_packed / x_int_row_sum,
    if given, receive the packed form of the same codes as well.  Shapes the matrix-core kernel does not take (no
    transform on rows that are not whole blocks of 128, the weight-side factor, rows over 32768) are quantised to packed
    codes first and converted.
    Returns (scale, x_tiles)."""
    m, k = x.shape
    if scale is None:
        scale = torch.empty(m, 1, dtype=x.dtype, device=x.device)
    if x_tiles is None:
        x_tiles = torch.empty(e2m3_tiles_bytes(m, k), dtype=torch.uint8, device=x.device)
    assert x.dtype in _FLOAT16S and x.is_contiguous() and scale.dtype == x.dtype and scale.is_contiguous() and scale.numel() == m
    assert x_tiles.dtype == torch.uint8 and x_tiles.is_contiguous() and x_tiles.numel() == e2m3_tiles_bytes(m, k)
    assert x_int_packed is None or (x_int_packed.dtype == torch.uint8 and x_int_packed.is_contiguous() and x_int_packed.shape == (m, k // 2))
    assert x_int_row_sum is None or (x_int_row_sum.dtype == torch.int32 and x_int_row_sum.is_contiguous() and x_int_row_sum.numel() == m)
    assert x_had is None or (x_had.dtype == x.dtype and x_had.shape == x.shape and x_had.is_contiguous())
    dev = require_gpu(x, scale, x_tiles, x_int_packed, x_int_row_sum, x_had)
    with torch.cuda.device(dev):
        rc = _lib.load().quest_hadamard_quantize_e2m3(ptr(x), ptr(scale), ptr(x_tiles), ptr(x_int_packed), ptr(x_int_row_sum),
                                                      ptr(x_had), k, m, float(hadamard_scale), DTYPE_CODE[x.dtype], stream_of(x))
    if rc == QUEST_ERR_UNSUPPORTED or (rc == QUEST_ERR_BAD_SHAPE and hadamard_scale == 0. and k % 64 == 0):
        _, packed, _ = hadamard_quantize_int4(x, scale, x_int_packed, x_int_row_sum, x_had, hadamard_scale=hadamard_scale)
        int4_to_e2m3_tiles(packed, x_tiles)
    else:
        check(rc, 'hadamard_quantize_e2m3')
    return scale, x_tiles


def _e2m3_outputs(m, k, dtype, device, scale, x_tiles):
    if scale is None:
        scale = torch.empty(m, 1, dtype=dtype, device=device)
    if x_tiles is None:
        x_tiles = torch.empty(e2m3_tiles_bytes(m, k), dtype=torch.uint8, device=device)
    assert scale.dtype == dtype and scale.is_contiguous() and scale.numel() == m
    assert x_tiles.dtype == torch.uint8 and x_tiles.is_contiguous() and x_tiles.numel() == e2m3_tiles_bytes(m, k)
    return scale, x_tiles


def rmsnorm_hadamard_quantize_e2m3(x, norm_weight, eps, scale=None, x_tiles=None, x_norm=None,
                                   hadamard_scale: float = HADAMARD_ENTRY) -> tuple[torch.Tensor, torch.Tensor]:
    """`rmsnorm_hadamard_quantize_int4` with the codes written as E2M3 tiles.  Returns (scale, x_tiles)."""
    m, k = x.shape
    assert x.dtype in _FLOAT16S and x.is_contiguous() and norm_weight.dtype == x.dtype and norm_weight.numel() == k and norm_weight.is_contiguous()
    assert x_norm is None or (x_norm.dtype == x.dtype and x_norm.shape == x.shape and x_norm.is_contiguous())
    scale, x_tiles = _e2m3_outputs(m, k, x.dtype, x.device, scale, x_tiles)
    dev = require_gpu(x, norm_weight, scale, x_tiles, x_norm)
    with torch.cuda.device(dev):
        check(_lib.load().quest_rmsnorm_hadamard_quantize_e2m3(
            ptr(x), ptr(norm_weight), float(eps), ptr(scale), ptr(x_tiles), ptr(x_norm), k, m, float(hadamard_scale),
            DTYPE_CODE[x.dtype], stream_of(x)), 'rmsnorm_hadamard_quantize_e2m3')
    return scale, x_tiles


def add_rmsnorm_hadamard_quantize_e2m3(x, branch, norm_weight, eps, scale=None, x_tiles=None,
                                       hadamard_scale: float = HADAMARD_ENTRY) -> tuple[torch.Tensor, torch.Tensor]:
    """`add_rmsnorm_hadamard_quantize_int4` (x += branch in place, then the norm) with the codes written as E2M3 tiles."""
    m, k = x.shape
    assert x.dtype in _FLOAT16S and x.is_contiguous() and branch.dtype == x.dtype and branch.shape == x.shape
    assert branch.is_contiguous() and branch.data_ptr() != x.data_ptr()
    assert norm_weight.dtype == x.dtype and norm_weight.numel() == k and norm_weight.is_contiguous()
    scale, x_tiles = _e2m3_outputs(m, k, x.dtype, x.device, scale, x_tiles)
    dev = require_gpu(x, branch, norm_weight, scale, x_tiles)
    with torch.cuda.device(dev):
        check(_lib.load().quest_add_rmsnorm_hadamard_quantize_e2m3(
            ptr(x), ptr(branch), ptr(norm_weight), float(eps), ptr(scale), ptr(x_tiles), k, m, float(hadamard_scale),
            DTYPE_CODE[x.dtype], stream_of(x)), 'add_rmsnorm_hadamard_quantize_e2m3')
    return scale, x_tiles


def silu_mul_hadamard_quantize_e2m3(gate_up, scale=None, x_tiles=None, x_act=None,
                                    hadamard_scale: float = HADAMARD_ENTRY) -> tuple[torch.Tensor, torch.Tensor]:
    """`silu_mul_hadamard_quantize_int4` with the codes written as E2M3 tiles.  Returns (scale, x_tiles)."""
    m, k2 = gate_up.shape
    k = k2 // 2
    assert gate_up.dtype in _FLOAT16S and gate_up.is_contiguous() and k2 == 2 * k
    assert x_act is None or (x_act.dtype == gate_up.dtype and x_act.shape == (m, k) and x_act.is_contiguous())
    scale, x_tiles = _e2m3_outputs(m, k, gate_up.dtype, gate_up.device, scale, x_tiles)
    dev = require_gpu(gate_up, scale, x_tiles, x_act)
    with torch.cuda.device(dev):
        check(_lib.load().quest_silu_mul_hadamard_quantize_e2m3(
            ptr(gate_up), ptr(scale), ptr(x_tiles), ptr(x_act), k, m, float(hadamard_scale), DTYPE_CODE[gate_up.dtype],
            stream_of(gate_up)), 'silu_mul_hadamard_quantize_e2m3')
    return scale, x_tiles
