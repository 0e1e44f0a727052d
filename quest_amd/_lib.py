"""ctypes binding of libquest_hip.so (the C ABI declared in include/quest_hip.h).

There is no fallback: if the shared library is missing or an entry point returns an error the
caller gets a RuntimeError.
"""
from __future__ import annotations

import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, 'libquest_hip.so')

QUEST_DTYPE_BF16 = 0
QUEST_DTYPE_FP16 = 1
DTYPE_CODE = {torch.bfloat16: QUEST_DTYPE_BF16, torch.float16: QUEST_DTYPE_FP16}

_vp, _i, _f = ctypes.c_void_p, ctypes.c_int, ctypes.c_float

# name -> argtypes; every function returns an int status unless _RESTYPES says otherwise
SIGNATURES = {
    'quest_version': [],
    'quest_status_string': [_i],
    'quest_find_scale_int4': [_vp, _vp, _i, _i, _i, _vp],
    'quest_quantize_int4': [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    'quest_add_mul_vv': [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp],
    'quest_matmul_int4_int4t_int32': [_vp, _vp, _vp, _i, _i, _i, _vp],
    'quest_fused_matmul_dequantize_int4_int4t': [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    'quest_fused_matmul_dequantize_swiglu_int4_int4t': [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    'quest_hadamard128': [_vp, _vp, _i, _i, _f, _i, _vp],
    'quest_hadamard_quantize_int4': [_vp, _vp, _vp, _vp, _vp, _i, _i, _f, _i, _vp],
    'quest_rmsnorm_hadamard_quantize_int4': [_vp, _vp, _f, _vp, _vp, _vp, _vp, _vp, _i, _i, _f, _i, _vp],
    'quest_add_rmsnorm_hadamard_quantize_int4': [_vp, _vp, _vp, _f, _vp, _vp, _vp, _i, _i, _f, _i, _vp],
    'quest_hadamard_quantize_int4_rule': [_vp, _vp, _vp, _vp, _vp, _i, _i, _f, _i, _i, _vp],
    'quest_rope_interleaved': [_vp, _vp, _i, _i, _i, _i, _i, _i, _vp],
    'quest_silu_mul_hadamard_quantize_int4': [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _f, _i, _vp],
    'quest_gemm_workspace_bytes': [_i, _i, _i],
    'quest_fused_matmul_dequantize_int4_int4t_ws': [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, ctypes.c_size_t, _vp],
    'quest_gemm_noalloc_scratch_bytes': [],
    'quest_fused_matmul_dequantize_int4_int4t_noalloc': [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    'quest_e2m3_tiles_bytes': [_i, _i],
    'quest_int4_to_e2m3_tiles': [_vp, _vp, _i, _i, _vp],
    'quest_fused_matmul_dequantize_e2m3': [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    'quest_fused_matmul_dequantize_add_e2m3': [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    'quest_fused_matmul_dequantize_add_int4_int4t': [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    'quest_fused_matmul_dequantize_add_available': [_i, _i, _i, _vp],
    'quest_fused_matmul_dequantize_rope_int4_int4t': [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _i, _i, _i, _vp],
    'quest_fused_matmul_dequantize_rope_e2m3': [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _i, _i, _i, _vp],
    'quest_fused_matmul_dequantize_swiglu_e2m3': [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    'quest_e2m3_gemm_plan': [_i, _i, _i, _i, _vp],
    'quest_hadamard_quantize_e2m3': [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _f, _i, _vp],
    'quest_rmsnorm_hadamard_quantize_e2m3': [_vp, _vp, _f, _vp, _vp, _vp, _i, _i, _f, _i, _vp],
    'quest_add_rmsnorm_hadamard_quantize_e2m3': [_vp, _vp, _vp, _f, _vp, _vp, _i, _i, _f, _i, _vp],
    'quest_silu_mul_hadamard_quantize_e2m3': [_vp, _vp, _vp, _vp, _i, _i, _f, _i, _vp],
}
# entry points that do not return an int status
_RESTYPES = {'quest_status_string': ctypes.c_char_p, 'quest_e2m3_tiles_bytes': ctypes.c_size_t,
             'quest_gemm_workspace_bytes': ctypes.c_size_t, 'quest_gemm_noalloc_scratch_bytes': ctypes.c_size_t}

_lib = None


def load() -> ctypes.CDLL:
    """Load the library once; raise if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f'{LIB_PATH} is missing: build the HIP kernels first (python -m quest_amd.build). '
                'quest_amd has no fallback path.')
        lib = ctypes.CDLL(LIB_PATH)
        for name, argtypes in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = _RESTYPES.get(name, ctypes.c_int)
        _lib = lib
    return _lib


def check(status: int, what: str) -> None:
    if status != 0:
        msg = load().quest_status_string(status).decode()
        raise RuntimeError(f'{what} failed with status {status}: {msg}')


def ptr(t: torch.Tensor | None) -> ctypes.c_void_p:
    """Device pointer of a tensor; None (an output that is not wanted) becomes NULL."""
    if t is None or t.numel() == 0:
        return ctypes.c_void_p(0)
    return ctypes.c_void_p(t.data_ptr())


def stream_of(t: torch.Tensor) -> ctypes.c_void_p:
    """The HIP stream torch currently launches on for the tensor's device."""
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def require_gpu(*tensors: torch.Tensor) -> torch.device:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if t.device.type != 'cuda':
            raise RuntimeError(f'quest_amd runs on the GPU only; got a tensor on {t.device}')
        if dev is not None and t.device != dev:
            raise RuntimeError(f'tensors on different devices: {dev} and {t.device}')
        dev = t.device
    return dev
