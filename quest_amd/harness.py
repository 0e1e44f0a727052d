"""Host-side counterparts of the reference's inference harness (gemm-quest/benchmarks/utils.py and
bench_e2e.py) on top of the HIP kernels: weight preparation, the W4A4 linear forward, the
`Linear4bit` module and the timing helpers.

Same function names, argument order and defaults as the reference.  The `backend` argument is
kept for call-site compatibility: 'hip' (default) and the reference's 'triton' / 'cuda' all run
the HIP kernels; 'pytorch' (the reference's eager-torch twin) is not part of this build.
"""
from __future__ import annotations

import time

import torch
from torch import nn

from . import api as quest
from .api import HADAMARD_ENTRY

_HIP_BACKENDS = ('hip', 'triton', 'cuda')
WEIGHT_HADAMARD_SCALE = 2. ** -3.5      # utils.py:39


def _check_backend(backend: str) -> None:
    if backend not in _HIP_BACKENDS:
        raise NotImplementedError(
            f"backend {backend!r}: this build runs the HIP kernels only ('hip'; 'triton' and 'cuda' are aliases)")


def find_scale_int4(x: torch.Tensor, scale: torch.Tensor = None, backend: str = 'hip') -> torch.Tensor:
    """utils.py:114-159.  x: (..., K) -> scale (..., 1)."""
    _check_backend(backend)
    if scale is None:
        scale = torch.empty(*x.shape[:-1], 1, dtype=x.dtype, device=x.device)
    quest.find_scale_int4(x.view(-1, x.size(-1)), scale.view(-1, 1))
    return scale


def quantize_int4(x, scale, x_int=None, x_int_packed=None, x_int_row_sum=None, do_dequantize=False, backend='hip'):
    """utils.py:212-270."""
    _check_backend(backend)
    k = x.size(-1)
    quest.quantize_int4(
        x.view(-1, k), scale.view(-1, 1),
        None if x_int is None else x_int.view(-1, k),
        None if x_int_packed is None else x_int_packed.view(-1, k // 2),
        None if x_int_row_sum is None else x_int_row_sum.view(-1, 1),
        do_dequantize)
    return x, x_int, x_int_packed, x_int_row_sum


def add_mul_vv(vec_a_add, vec_a_mul, vec_b_add, vec_b_mul, mat_c, mat_d=None, backend='hip'):
    """utils.py:448-502."""
    _check_backend(backend)
    return quest.add_mul_vv(vec_a_add, vec_a_mul, vec_b_add, vec_b_mul, mat_c, mat_d)


def unpack_int4(x_int_packed: torch.Tensor, meta_e_no_reorder: torch.Tensor = None) -> torch.Tensor:
    """utils.py:420-445 (dense branch): uint8 (..., K/2) -> int8 (..., K), low nibble first."""
    if meta_e_no_reorder is not None:
        raise NotImplementedError('4:8-sparse weights are not part of this build')
    x_int = torch.empty(*x_int_packed.shape[:-1], x_int_packed.size(-1) * 2, dtype=torch.int8, device=x_int_packed.device)
    x_int[..., ::2] = x_int_packed & 0xF
    x_int[..., 1::2] = x_int_packed >> 4
    return torch.where(x_int >= 8, x_int - 16, x_int)


def fused_matmul_dequantize_int4_bf16(mat_a, mat_b, vec_a_add, vec_b_add, vec_a_mul, vec_b_mul, mat_d,
                                      _mat_c=None, debug_mode=True):
    """utils.py:548-587.  debug_mode=True runs the int32 GEMM and the scale epilogue as two
    launches, debug_mode=False the single fused kernel; both give the same bits here."""
    m, n = mat_a.size(0), mat_b.size(0)
    if mat_d is None:
        mat_d = torch.empty(m, n, dtype=vec_a_mul.dtype, device=mat_a.device)
    if debug_mode:
        mat_c = torch.empty(m, n, dtype=torch.int32, device=mat_a.device) if _mat_c is None else _mat_c
        quest.matmul_int4_int4t_int32(mat_a=mat_a, mat_b=mat_b, out=mat_c)
        quest.add_mul_vv(vec_a_add=vec_a_add, vec_a_mul=vec_a_mul, vec_b_add=vec_b_add, vec_b_mul=vec_b_mul,
                         mat_c=mat_c, mat_d=mat_d)
    else:
        quest.fused_matmul_dequantize_int4_int4t_bf16(mat_a=mat_a, mat_b=mat_b, vec_a_add=vec_a_add, vec_b_add=vec_b_add,
                                                      vec_a_mul=vec_a_mul, vec_b_mul=vec_b_mul, out=mat_d)
    return mat_d


def preprocess_weight(weight: torch.Tensor, use_sparse: bool = False, use_hadamard: bool = False, backend: str = 'hip',
                      w_scale_mode: str = 'rms'):
    """utils.py:20-53, dense branch: (N, K) float weight -> (w_int_packed (N, K/2) uint8,
    w_scale (N, 1), w_add (N, 1) int32 = row sum of the codes + K/2, None)."""
    _check_backend(backend)
    if use_sparse:
        raise NotImplementedError('4:8-sparse weights are not part of this build')
    weight = weight.contiguous()
    n, k = weight.shape
    w_scale = torch.empty(n, 1, dtype=weight.dtype, device=weight.device)
    w_int_packed = torch.empty(n, k // 2, dtype=torch.uint8, device=weight.device)
    w_int_row_sum = torch.empty(n, 1, dtype=torch.int32, device=weight.device)
    # one pass: weight-side Hadamard (scale 2^-3.5) when asked, then scale, codes and row sums
    # (w_scale_mode: 'rms' is the reference's rule, 'absmax' puts the row's largest magnitude at the grid's edge)
    quest.hadamard_quantize_int4(weight, w_scale, w_int_packed, w_int_row_sum,
                                 hadamard_scale=WEIGHT_HADAMARD_SCALE if use_hadamard else 0.,
                                 scale_rule={'rms': 'gaussian', 'absmax': 'absmax'}[w_scale_mode])
    w_add = w_int_row_sum + k // 2
    return w_int_packed, w_scale, w_add, None


def linear_forward(activation, w_int_packed, w_scale, w_add, w_meta_e=None, out=None, _a_scale=None,
                   _a_int_packed=None, _a_int_row_sum=None, _c=None, use_hadamard=False, backend='hip'):
    """utils.py:56-111, dense branch: out (M, N) = quantised activation @ quantised weight^T.
    Two launches: the fused Hadamard-scale-quantise-pack kernel, then the GEMM with the scale
    epilogue (the reference uses four)."""
    _check_backend(backend)
    if w_meta_e is not None:
        raise NotImplementedError('4:8-sparse weights are not part of this build')
    m, k, n = activation.size(0), activation.size(1), w_int_packed.size(0)
    dtype, device = activation.dtype, activation.device
    if out is None:
        out = torch.empty(m, n, dtype=dtype, device=device)
    a_scale = torch.empty(m, 1, dtype=dtype, device=device) if _a_scale is None else _a_scale
    a_int_packed = torch.empty(m, k // 2, dtype=torch.uint8, device=device) if _a_int_packed is None else _a_int_packed
    a_int_row_sum = torch.empty(m, 1, dtype=torch.int32, device=device) if _a_int_row_sum is None else _a_int_row_sum
    quest.hadamard_quantize_int4(activation, a_scale, a_int_packed, a_int_row_sum,
                                 hadamard_scale=HADAMARD_ENTRY if use_hadamard else 0.)
    quest.fused_matmul_dequantize_int4_int4t_bf16(mat_a=a_int_packed, mat_b=w_int_packed, vec_a_add=a_int_row_sum,
                                                  vec_b_add=w_add, vec_a_mul=a_scale, vec_b_mul=w_scale, out=out)
    return out


class Linear4bit(nn.Module):
    """bench_e2e.py:41-70: a linear layer holding packed INT4 weights, built from a randomly
    initialised nn.Linear of the same shape (the benchmarks never load trained weights)."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True, device=None, dtype=None,
                 use_sparse: bool = False, use_hadamard: bool = False, use_noop: bool = False):
        super().__init__()
        self.use_hadamard = use_hadamard
        self.use_noop = use_noop
        nn_linear = nn.Linear(in_features, out_features, bias=bias, device=device, dtype=dtype)
        self.bias = nn_linear.bias
        weight = nn_linear.weight.data
        self.weight = torch.empty_like(weight, device=torch.device('meta'))
        w_int_packed, w_scale, w_add, w_meta_e = preprocess_weight(weight=weight, use_sparse=use_sparse,
                                                                   use_hadamard=use_hadamard)
        self.register_buffer('w_int_packed', w_int_packed)
        self.register_buffer('w_scale', w_scale)
        self.register_buffer('w_add', w_add)
        self.register_buffer('w_meta_e', w_meta_e)

    @classmethod
    def from_weight(cls, weight: torch.Tensor, bias: torch.Tensor = None, use_hadamard: bool = False) -> 'Linear4bit':
        """Pack an existing (N, K) weight instead of a random one."""
        self = cls.__new__(cls)
        nn.Module.__init__(self)
        self.use_hadamard, self.use_noop = use_hadamard, False
        self.bias = bias
        self.weight = torch.empty_like(weight, device=torch.device('meta'))
        w_int_packed, w_scale, w_add, _ = preprocess_weight(weight=weight, use_hadamard=use_hadamard)
        self.register_buffer('w_int_packed', w_int_packed)
        self.register_buffer('w_scale', w_scale)
        self.register_buffer('w_add', w_add)
        self.register_buffer('w_meta_e', None)
        return self

    @classmethod
    def empty(cls, in_features: int, out_features: int, bias: bool = False, device=None, dtype=None,
              use_hadamard: bool = False) -> 'Linear4bit':
        """A layer of the given shape with unset buffers, to be filled by `load_state_dict` from a packed checkpoint."""
        self = cls.__new__(cls)
        nn.Module.__init__(self)
        self.use_hadamard, self.use_noop = use_hadamard, False
        self.bias = nn.Parameter(torch.zeros(out_features, dtype=dtype, device=device)) if bias else None
        self.weight = torch.empty(out_features, in_features, dtype=dtype, device=torch.device('meta'))
        self.register_buffer('w_int_packed', torch.zeros(out_features, in_features // 2, dtype=torch.uint8, device=device))
        self.register_buffer('w_scale', torch.zeros(out_features, 1, dtype=dtype, device=device))
        self.register_buffer('w_add', torch.zeros(out_features, 1, dtype=torch.int32, device=device))
        self.register_buffer('w_meta_e', None)
        return self

    def forward_quantized(self, a_scale, a_int_packed, a_int_row_sum, out=None) -> torch.Tensor:
        """The GEMM half of `linear_forward` on activations some fused producer kernel has already quantised:
        (M, 1) scales, (M, K/2) codes, (M, 1) row sums -> (M, N)."""
        y = quest.fused_matmul_dequantize_int4_int4t_bf16(mat_a=a_int_packed, mat_b=self.w_int_packed,
                                                          vec_a_add=a_int_row_sum, vec_b_add=self.w_add,
                                                          vec_a_mul=a_scale, vec_b_mul=self.w_scale, out=out)
        if self.bias is not None:
            y += self.bias
        return y

    def forward(self, x) -> torch.Tensor:
        if not self.use_noop:
            a = x.contiguous().flatten(end_dim=-2)
            y = linear_forward(activation=a, w_int_packed=self.w_int_packed, w_scale=self.w_scale, w_add=self.w_add,
                               w_meta_e=self.w_meta_e, out=None, use_hadamard=self.use_hadamard)
            y = y.unflatten(dim=0, sizes=x.shape[:-1])
        else:
            y = torch.zeros(*x.shape[:-1], self.weight.size(0), dtype=x.dtype, device=x.device)
        if self.bias is not None:
            y += self.bias
        return y


@torch.inference_mode()
def do_bench(f, n_iter: int = 100, n_warmup: int = 10) -> float:
    """utils.py:789-799: seconds per call, wall clock around a device synchronisation."""
    for _ in range(n_warmup):
        f()
    torch.cuda.synchronize()
    ts = time.time()
    for _ in range(n_iter):
        f()
    torch.cuda.synchronize()
    te = time.time()
    return (te - ts) / n_iter


@torch.inference_mode()
def do_bench_network(f, M: int, K: int, N: int, dtype: torch.dtype, device: torch.device, n_layers: int = 20,
                     n_warmup: int = 3) -> float:
    """utils.py:802-835: n_layers back-to-back calls on one aliased workspace, timed eagerly and as a
    replayed HIP graph; the smaller per-layer time is returned."""
    workspace = torch.empty(M * max(K, N), dtype=dtype, device=device)
    activation_in = workspace[:M * K].reshape(M, K)
    activation_out = workspace[:M * N].reshape(M, N)

    def network():
        for _ in range(n_layers):
            f(activation_in, activation_out)

    tf = do_bench(network, n_iter=1, n_warmup=n_warmup)
    graph = torch.cuda.CUDAGraph()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for _ in range(n_warmup):
            network()
    torch.cuda.current_stream().wait_stream(s)
    with torch.cuda.graph(graph):
        network()
    tg = do_bench(graph.replay, n_iter=1, n_warmup=n_warmup)
    return min(tf, tg) / n_layers
