"""ctypes front end of oracle/quest_oracle.c (test infrastructure only; see that file's header).

Every function takes and returns CPU torch tensors; 16-bit floats are passed as their raw
bits.  `build()` compiles the library with the Makefile beside this file.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, 'libquest_oracle.so')
_lib = None

_DT = {torch.bfloat16: 0, torch.float16: 1}


def build() -> str:
    subprocess.run(['make', '-C', _HERE, '-B', 'libquest_oracle.so'], check=True, capture_output=True)
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.qo_bf16_to_f32.restype = ctypes.c_float
        _lib.qo_bf16_to_f32.argtypes = [ctypes.c_uint16]
        _lib.qo_fp16_to_f32.restype = ctypes.c_float
        _lib.qo_fp16_to_f32.argtypes = [ctypes.c_uint16]
        _lib.qo_f32_to_bf16.restype = ctypes.c_uint16
        _lib.qo_f32_to_bf16.argtypes = [ctypes.c_float]
        _lib.qo_f32_to_fp16.restype = ctypes.c_uint16
        _lib.qo_f32_to_fp16.argtypes = [ctypes.c_float]
    return _lib


def _p(t):
    if t is None:
        return ctypes.c_void_p(0)
    assert t.device.type == 'cpu' and t.is_contiguous()
    return ctypes.c_void_p(t.data_ptr())


def _l(v):
    return ctypes.c_long(int(v))


def hadamard128_matmul(x: torch.Tensor, entry: float = 181. / 2048.) -> torch.Tensor:
    y = torch.empty_like(x)
    rows = x.numel() // x.size(-1)
    lib().qo_hadamard128_matmul(_p(y), _p(x), _l(rows), _l(x.size(-1)), ctypes.c_float(entry), _DT[x.dtype])
    return y


def hadamard128_fwht(x: torch.Tensor, scale: float) -> torch.Tensor:
    y = torch.empty_like(x)
    rows = x.numel() // x.size(-1)
    lib().qo_hadamard128_fwht(_p(y), _p(x), _l(rows), _l(x.size(-1)), ctypes.c_float(scale), _DT[x.dtype])
    return y


def find_scale_int4(x: torch.Tensor, order: int = 0) -> torch.Tensor:
    rows = x.numel() // x.size(-1)
    scale = torch.empty(rows, 1, dtype=x.dtype)
    lib().qo_find_scale_int4(_p(scale), _p(x), _l(rows), _l(x.size(-1)), _DT[x.dtype], int(order))
    return scale


def quantize_int4(x: torch.Tensor, scale: torch.Tensor, do_dequantize: bool = False):
    """Returns (x_dq or x, x_int, x_int_packed, x_int_row_sum), all freshly allocated."""
    rows, k = x.numel() // x.size(-1), x.size(-1)
    xc = x.clone()
    x_int = torch.empty(rows, k, dtype=torch.int8)
    packed = torch.empty(rows, k // 2, dtype=torch.uint8)
    row_sum = torch.empty(rows, 1, dtype=torch.int32)
    lib().qo_quantize_int4(_p(xc), _p(scale), _p(x_int), _p(packed), _p(row_sum), _l(rows), _l(k),
                           int(bool(do_dequantize)), _DT[x.dtype])
    return xc, x_int, packed, row_sum


def unpack_int4(packed: torch.Tensor) -> torch.Tensor:
    out = torch.empty(*packed.shape[:-1], packed.size(-1) * 2, dtype=torch.int8)
    lib().qo_unpack_int4(_p(out), _p(packed), _l(packed.numel()))
    return out


def matmul_int4_int4t_int32(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    m, n, k = a.size(0), b.size(0), a.size(1) * 2
    c = torch.empty(m, n, dtype=torch.int32)
    lib().qo_matmul_int4_int4t_int32(_p(c), _p(a), _p(b), _l(m), _l(k), _l(n))
    return c


def add_mul_vv(a_add, a_mul, b_add, b_mul, c) -> torch.Tensor:
    m, n = c.shape
    d = torch.empty(m, n, dtype=a_mul.dtype)
    lib().qo_add_mul_vv(_p(d), _p(a_add), _p(a_mul), _p(b_add), _p(b_mul), _p(c), _l(m), _l(n), _DT[a_mul.dtype])
    return d
