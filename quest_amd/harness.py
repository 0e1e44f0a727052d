"""Host-side counterparts of the reference's inference harness (gemm-quest/benchmarks/utils.py and
bench_e2e.py) on top of the HIP kernels: weight preparation, the W4A4 linear forward, the
`Linear4bit` module and the timing helpers.

Same function names, argument order and defaults as the reference.  The `backend` argument is
kept for call-site compatibility: 'hip' (default) and the reference's 'triton' / 'cuda' all run
the HIP kernels; 'pytorch' (the reference's eager-torch twin) is not part of this build.
"""
from __future__ import annotations

import torch
from torch import nn

from . import api as quest
from .api import HADAMARD_ENTRY

_HIP_BACKENDS = ('hip', 'triton', 'cuda')
WEIGHT_HADAMARD_SCALE = 2. ** -3.5      # utils.py:39

# Which matrix instructions the GEMM of `linear_forward` / `Linear4bit` runs on when the weight's E2M3 tiles are at
# hand: 'fp6' = the FP6 (E2M3) kernel where it is the faster one (a few hundred tokens and more), 'int8' = always the
# INT8 kernels on packed nibbles.  Both give the same bits.
MATRIX_PATH = 'fp6'
E2M3_MIN_TILES = 66                     # 256 x 256 output tiles from which the FP6 kernel is the faster one
E2M3_MIN_K = 2048                       # shortest rows that take it (see prefers_e2m3)
# Whether a producer-fused block lets the FP6 GEMM of an output projection add into the residual stream itself
# (same bits as the addition inside the next norm kernel; one pass over the stream less).
GEMM_ADDS_RESIDUAL = True
GEMM_ADDS_RESIDUAL_PACKED = True       # ... also on packed nibbles, where the INT8 large-tile kernel takes the projection
# ... and the rotary embedding of q and k after the fused QKV projection (the FP6 GEMM's rotary epilogue)
GEMM_ROTATES_QK = True


def prefers_e2m3(m: int, k: int, n: int) -> bool:
    """Whether the FP6 kernel is the faster one for an (m, k) x (n, k) layer.  Its 256 x 256 tiles need about a quarter
    of the chip's 256 compute units busy to beat the INT8 kernels' small tiles: measured over K from 1024 to 11008, N from
    2048 to 13824 and M from 256 to 16384, the FP6 kernel wins from 66 tiles on (M = 1536 at N = 4096, M = 512 at
    N = 11008, M = 3072 at N = 2048) and loses below 64."""
    tiles = ((m + 255) // 256) * ((n + 255) // 256)
    # E2M3_MIN_K: with shorter rows the GEMM is mostly epilogue either way and the tile-writing activation kernels are a
    # little slower than the row-writing ones (12.0 against 10.2 us at [16384, 1024]) -- measured on the 12-layer
    # d = 1024 model at 32 x 512 tokens: 6.01 ms per forward with the FP6 path from K = 1024 on, 5.79 ms from K = 2048 on
    # (its K = 2816 layers), 5.80 ms without it; the 1600M model (K = 2560, 6912) gains 9 %
    return (MATRIX_PATH == 'fp6' and k % 128 == 0 and E2M3_MIN_K <= k <= 65536 and tiles >= E2M3_MIN_TILES and m * n <= (1 << 30))


def weight_tiles(w_int_packed: torch.Tensor) -> torch.Tensor:
    """The E2M3 tiles of packed weight codes (N, K/2): the FP6 kernel's operand form (1.5 x the packed bytes)."""
    return quest.int4_to_e2m3_tiles(w_int_packed)


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
                      w_scale_mode: str = 'rms', quantize_from_fp32: bool = False):
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
                                 scale_rule={'rms': 'gaussian', 'absmax': 'absmax'}[w_scale_mode], from_fp32=quantize_from_fp32)
    w_add = w_int_row_sum + k // 2
    return w_int_packed, w_scale, w_add, None


def linear_forward(activation, w_int_packed, w_scale, w_add, w_meta_e=None, out=None, _a_scale=None,
                   _a_int_packed=None, _a_int_row_sum=None, _c=None, use_hadamard=False, backend='hip', w_tiles=None,
                   _a_tiles=None, quantize_from_fp32=False):
    """utils.py:56-111, dense branch: out (M, N) = quantised activation @ quantised weight^T.
    Two launches: the fused Hadamard-scale-quantise-pack kernel, then the GEMM with the scale
    epilogue (the reference uses four).  With `w_tiles` (`weight_tiles(w_int_packed)`) and enough tokens the codes
    travel as E2M3 tiles and the GEMM runs on the FP6 matrix instructions: the same output bits, faster.
    quantize_from_fp32 (with use_hadamard): the activation codes come from the fp32 transform (factor 2^-3.5, the
    reference's evaluation-side arithmetic, src/eval_hswag.py:201-214) instead of from its 16-bit rounding."""
    _check_backend(backend)
    if w_meta_e is not None:
        raise NotImplementedError('4:8-sparse weights are not part of this build')
    m, k, n = activation.size(0), activation.size(1), w_int_packed.size(0)
    dtype, device = activation.dtype, activation.device
    if out is None:
        out = torch.empty(m, n, dtype=dtype, device=device)
    if quantize_from_fp32 and use_hadamard:
        a_scale, a_int_packed, a_int_row_sum = quest.hadamard_quantize_int4(
            activation, _a_scale, _a_int_packed, _a_int_row_sum, hadamard_scale=WEIGHT_HADAMARD_SCALE, from_fp32=True)
        return quest.fused_matmul_dequantize_int4_int4t_bf16(mat_a=a_int_packed, mat_b=w_int_packed, vec_a_add=a_int_row_sum,
                                                             vec_b_add=w_add, vec_a_mul=a_scale, vec_b_mul=w_scale, out=out)
    if w_tiles is not None and prefers_e2m3(m, k, n):
        a_scale, a_tiles = quest.hadamard_quantize_e2m3(activation, _a_scale, _a_tiles,
                                                        hadamard_scale=HADAMARD_ENTRY if use_hadamard else 0.)
        return quest.fused_matmul_dequantize_e2m3(a_tiles, w_tiles, a_scale, w_scale, k, out)
    a_scale = torch.empty(m, 1, dtype=dtype, device=device) if _a_scale is None else _a_scale
    a_int_packed = torch.empty(m, k // 2, dtype=torch.uint8, device=device) if _a_int_packed is None else _a_int_packed
    a_int_row_sum = torch.empty(m, 1, dtype=torch.int32, device=device) if _a_int_row_sum is None else _a_int_row_sum
    quest.hadamard_quantize_int4(activation, a_scale, a_int_packed, a_int_row_sum,
                                 hadamard_scale=HADAMARD_ENTRY if use_hadamard else 0.)
    quest.fused_matmul_dequantize_int4_int4t_bf16(mat_a=a_int_packed, mat_b=w_int_packed, vec_a_add=a_int_row_sum,
                                                  vec_b_add=w_add, vec_a_mul=a_scale, vec_b_mul=w_scale, out=out)
    return out


class Linear4bit(nn.Module):
    """bench_e2e.py:41-70: a linear layer that holds its weight as packed INT4 codes.

    Buffers, as in the reference: `w_int_packed` (N, K/2) uint8, `w_scale` (N, 1), `w_add` (N, 1) int32 and the
    unused `w_meta_e`; `weight` is a shape-only meta tensor; `bias` is a parameter or None.  The plain constructor
    packs the weight of a freshly initialised `nn.Linear` (the benchmarks never load trained weights),
    `from_weight` packs a given one and `empty` leaves the buffers to `load_state_dict`."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True, device=None, dtype=None,
                 use_sparse: bool = False, use_hadamard: bool = False, use_noop: bool = False):
        super().__init__()
        if use_sparse:
            raise NotImplementedError('4:8-sparse weights are not part of this build')
        dense = nn.Linear(in_features, out_features, bias=bias, device=device, dtype=dtype)
        self._configure(use_hadamard, use_noop)
        self._install(dense.weight.data, dense.bias)

    def _configure(self, use_hadamard: bool, use_noop: bool) -> None:
        self.use_hadamard = use_hadamard
        self.use_noop = use_noop
        # codes from the fp32 transform instead of its 16-bit rounding (see linear_forward); set before packing a weight
        self.quantize_from_fp32 = getattr(self, 'quantize_from_fp32', False)

    def _install(self, weight: torch.Tensor, bias) -> None:
        """Pack `weight` (N, K) and keep `bias` (a tensor, a parameter or None) as a frozen parameter."""
        packed, scale, add, _ = preprocess_weight(weight=weight, use_hadamard=self.use_hadamard,
                                                  quantize_from_fp32=self.quantize_from_fp32)
        self._set_buffers(weight.shape, weight.dtype, packed, scale, add)
        if bias is None:
            self.bias = None
        else:
            self.bias = nn.Parameter(bias.detach().to(weight.dtype), requires_grad=False)

    def _set_buffers(self, shape, dtype, packed, scale, add) -> None:
        self.weight = torch.empty(shape, dtype=dtype, device='meta')
        for name, t in (('w_int_packed', packed), ('w_scale', scale), ('w_add', add), ('w_meta_e', None)):
            self.register_buffer(name, t)
        self._tiles = None               # E2M3 tiles of w_int_packed: derived data, built on first use, not in checkpoints
        self._tiles_of = None

    def w_tiles(self) -> torch.Tensor:
        """The weight codes as E2M3 tiles (built once per content of `w_int_packed`, e.g. again after a checkpoint
        has been loaded into the buffers)."""
        try:
            key = (self.w_int_packed.data_ptr(), self.w_int_packed._version)
        except RuntimeError:              # a tensor created in inference mode keeps no version counter
            key = (self.w_int_packed.data_ptr(), None)
        if self._tiles is None or self._tiles_of != key:
            self._tiles = weight_tiles(self.w_int_packed)
            self._tiles_of = key
        return self._tiles

    @classmethod
    def from_weight(cls, weight: torch.Tensor, bias: torch.Tensor = None, use_hadamard: bool = False,
                    quantize_from_fp32: bool = False) -> 'Linear4bit':
        """Pack an existing (N, K) weight instead of a random one."""
        self = cls.__new__(cls)
        nn.Module.__init__(self)
        self.quantize_from_fp32 = bool(quantize_from_fp32)
        self._configure(use_hadamard, False)
        self._install(weight, bias)
        return self

    @classmethod
    def empty(cls, in_features: int, out_features: int, bias: bool = False, device=None, dtype=None,
              use_hadamard: bool = False) -> 'Linear4bit':
        """A layer of the given shape with unset buffers, to be filled by `load_state_dict` from a packed checkpoint."""
        self = cls.__new__(cls)
        nn.Module.__init__(self)
        self._configure(use_hadamard, False)
        self._set_buffers((out_features, in_features), dtype,
                          torch.zeros(out_features, in_features // 2, dtype=torch.uint8, device=device),
                          torch.zeros(out_features, 1, dtype=dtype, device=device),
                          torch.zeros(out_features, 1, dtype=torch.int32, device=device))
        self.bias = nn.Parameter(torch.zeros(out_features, dtype=dtype, device=device), requires_grad=False) if bias else None
        return self

    def forward_quantized(self, a_scale, a_int_packed, a_int_row_sum, out=None, rope=None, add_to_out=False) -> torch.Tensor:
        """The GEMM half of `linear_forward` on activations some fused producer kernel has already quantised:
        (M, 1) scales, (M, K/2) codes, (M, 1) row sums -> (M, N).  In no-op mode the GEMM is skipped (zeros), which is
        what prices the GEMMs of a producer-fused model: everything else, the quantising producers included, still runs.
        rope = (freqs_cis, rot_cols, head_dim): the first rot_cols channels leave rotated (layers without a bias).
        add_to_out: the result is added to `out` (the residual stream), with the bits of `out + layer(x)` (layers without
        a bias; one launch where `quest.gemm_add_fuses` says so)."""
        if self.use_noop:
            return out if add_to_out else self._noop_output(a_scale)
        if add_to_out:
            assert self.bias is None and rope is None and out is not None
            return quest.fused_matmul_dequantize_add_int4_int4t(a_int_packed, self.w_int_packed, a_int_row_sum, self.w_add,
                                                                a_scale, self.w_scale, out)
        if rope is not None:
            assert self.bias is None
            return quest.fused_matmul_dequantize_rope_int4_int4t(a_int_packed, self.w_int_packed, a_int_row_sum, self.w_add,
                                                                 a_scale, self.w_scale, *rope, out=out)
        y = quest.fused_matmul_dequantize_int4_int4t_bf16(mat_a=a_int_packed, mat_b=self.w_int_packed,
                                                          vec_a_add=a_int_row_sum, vec_b_add=self.w_add,
                                                          vec_a_mul=a_scale, vec_b_mul=self.w_scale, out=out)
        if self.bias is not None:
            y += self.bias
        return y

    def _noop_output(self, a_scale) -> torch.Tensor:
        y = torch.zeros(a_scale.numel(), self.weight.size(0), dtype=a_scale.dtype, device=a_scale.device)
        if self.bias is not None:
            y += self.bias
        return y

    def forward_tiles(self, a_scale, a_tiles, out=None, add_to_out=False, rope=None) -> torch.Tensor:
        """The same for activations quantised to E2M3 tiles: the GEMM on the FP6 matrix instructions.  add_to_out: the
        result is added to `out` (the residual stream) inside the GEMM's launch, with the bits of `out + layer(x)`.
        rope = (freqs_cis, rot_cols, head_dim): the rotary embedding of the first rot_cols channels in the GEMM's launch
        (layers without a bias; the caller checks `quest.rope_gemm_fuses`)."""
        if self.use_noop:
            return out if add_to_out else self._noop_output(a_scale)
        if add_to_out and self.bias is not None:                     # out + (product + bias): the bias first, as torch would
            y = quest.fused_matmul_dequantize_e2m3(a_tiles, self.w_tiles(), a_scale, self.w_scale, self.weight.size(1))
            y += self.bias
            out += y
            return out
        assert rope is None or self.bias is None
        y = quest.fused_matmul_dequantize_e2m3(a_tiles, self.w_tiles(), a_scale, self.w_scale, self.weight.size(1), out,
                                               add_to_out=add_to_out, rope=rope)
        if self.bias is not None:
            y += self.bias
        return y

    def forward(self, x) -> torch.Tensor:
        lead, n = x.shape[:-1], self.weight.size(0)
        rows = x.contiguous().view(-1, x.size(-1))
        if self.use_noop:
            # the reference's no-op layer (bench_e2e.py:62-66) still rotates the activations, so that
            # "int4 minus noop" prices the quantiser and the GEMM only; the rotated tensor is dropped
            if self.use_hadamard:
                quest.hadamard128(rows)
            y = torch.zeros(rows.size(0), n, dtype=x.dtype, device=x.device)
        else:
            m, k = rows.shape
            y = linear_forward(rows, self.w_int_packed, self.w_scale, self.w_add, self.w_meta_e,
                               use_hadamard=self.use_hadamard, quantize_from_fp32=self.quantize_from_fp32,
                               w_tiles=self.w_tiles() if prefers_e2m3(m, k, n) and not self.quantize_from_fp32 else None)
        if self.bias is not None:
            y += self.bias
        return y.view(*lead, n)


def _elapsed_s(fn, n_iter: int) -> float:
    """Seconds per call of `fn`, from a pair of HIP events on the current stream around n_iter calls."""
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(n_iter):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) * 1e-3 / n_iter


@torch.inference_mode()
def do_bench(f, n_iter: int = 100, n_warmup: int = 10) -> float:
    """utils.py:789-799: seconds per call of `f` after `n_warmup` untimed calls.  The reference brackets the timed
    calls with device synchronisations and the host clock; here the bracket is a pair of HIP events on the stream
    the calls go to, which leaves the host's launch jitter before the first call out of the figure."""
    for _ in range(n_warmup):
        f()
    torch.cuda.synchronize()
    return _elapsed_s(f, n_iter)


@torch.inference_mode()
def do_bench_network(f, M: int, K: int, N: int, dtype: torch.dtype, device: torch.device, n_layers: int = 20,
                     n_warmup: int = 3) -> float:
    """utils.py:802-835: `f(activation_in (M, K), activation_out (M, N))` called `n_layers` times back to back on
    two views of one buffer (so that no call finds a fresh output allocation), timed as plain launches and as one
    replayed HIP graph; returns the smaller of the two, in seconds per layer."""
    # Gaussian values, not the reference's uninitialised memory: the kernels' run time depends on the data (degenerate
    # rows take a slower quantiser path, the clock follows the operands' power), and garbage would time something else
    pool = torch.randn(M * max(K, N), dtype=torch.float32, device=device).to(dtype)
    a_in, a_out = pool[:M * K].view(M, K), pool[:M * N].view(M, N)

    def stack():
        for _ in range(n_layers):
            f(a_in, a_out)

    eager_s = do_bench(stack, n_iter=1, n_warmup=n_warmup)
    capture = torch.cuda.Stream(device=device)
    capture.wait_stream(torch.cuda.current_stream(device))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(capture):
        for _ in range(n_warmup):
            stack()
        with torch.cuda.graph(graph, stream=capture):
            stack()
    torch.cuda.current_stream(device).wait_stream(capture)
    graph_s = do_bench(graph.replay, n_iter=1, n_warmup=n_warmup)
    return min(eager_s, graph_s) / n_layers
