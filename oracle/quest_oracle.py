"""CPU oracle for the W4A4 linear path of QuEST's gemm-quest package.

THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only tests/, __graft_entry__.smoke()
and bench.py's cpu_baseline leg may import it; nothing under quest_amd/ does.

It restates, with the same torch CPU ops and in the same order, the reference's
`backend='pytorch'` functions (all paths below are under /root/reference/):

  find_scale_int4      gemm-quest/benchmarks/utils.py:193-209
  quantize_int4        gemm-quest/benchmarks/utils.py:334-365
  unpack_int4          gemm-quest/benchmarks/utils.py:420-445   (dense branch)
  add_mul_vv           gemm-quest/benchmarks/utils.py:535-545
  hadamard128_matmul   gemm-quest/benchmarks/utils.py:17, 89-90 (Hadamard as F.linear)
  matmul_int4_int4t_int32   the integer GEMM as the reference's own check computes it,
                       gemm-quest/benchmarks/utils.py:680, 707-708
  preprocess_weight    gemm-quest/benchmarks/utils.py:20-49     (dense branch)
  linear_forward       gemm-quest/benchmarks/utils.py:56-101    (dense branch)
  linear_fp64          gemm-quest/benchmarks/utils.py:667-678   (fp64 identity)

The reference holds no golden vectors for this path (its only test,
utils.py:626-786, draws inputs from the CUDA RNG and needs the CUDA extension), and
its Python cannot be imported here (fast_hadamard_transform, triton's CUDA backend and a
CUDA device are needed at import time).  The oracle is therefore pinned by what the
mathematics fixes (tests/test_oracle_pins.py): closed forms for constant rows, exact
rational floor division, Sylvester-matrix identities, brute force over every 16-bit input,
integer GEMM against int64 loops, and the independent scalar C restatement in
oracle/quest_oracle.c.

Parity status per function:
  find_scale_int4, quantize_int4, unpack_int4, add_mul_vv, matmul_int4_int4t_int32,
  preprocess_weight(use_hadamard=False), linear_forward(use_hadamard=False): pinned.
  hadamard128_fwht (weights, fast_hadamard_transform's documented definition
  F.linear(x, H)*scale): pinned to tolerance 1e-3 by the Sylvester closed form.
  hadamard128_matmul on activations: parity unpinned at the bit level -- the reference
  runs it as a cuBLAS bf16 GEMM whose accumulation order is unspecified and no reference
  test exercises use_hadamard=True; pinned to <=1e-3 relative by the closed form only.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

# utils.py:208 -- python double, multiplied into an fp32 tensor (so used as fp32)
GAUSS_INT4_STEP = 2.513930578568423 * 2. / ((1 << 4) - 1)
SCALE_EPS = 1e-8
HADAMARD_BLOCK = 128


# ----------------------------------------------------------------------------- Hadamard
def sylvester_signs(n: int = HADAMARD_BLOCK) -> torch.Tensor:
    """(n, n) int8 matrix of +-1, entry (i, j) = (-1)^popcount(i & j)."""
    idx = torch.arange(n, dtype=torch.int64)
    v = idx[:, None] & idx[None, :]
    par = torch.zeros_like(v)
    for b in range(n.bit_length()):
        par ^= (v >> b) & 1
    return (1 - 2 * par).to(torch.int8)


def hadamard_matrix(dtype: torch.dtype) -> torch.Tensor:
    """utils.py:17 -- hadamard_transform(eye(128, dtype), scale=128**-0.5): every entry is
    +-2^-3.5 rounded to `dtype`, which is +-181/2048 = +-0.08837890625 for bf16 and fp16."""
    return (sylvester_signs().to(torch.float32) * (128 ** -0.5)).to(dtype)


def hadamard128_matmul(x: torch.Tensor) -> torch.Tensor:
    """utils.py:89-90 -- F.linear(x.view(-1, 128), HADAMARD_MATRIX).view_as(x)."""
    h = hadamard_matrix(x.dtype)
    return F.linear(x.reshape(-1, HADAMARD_BLOCK), h).view_as(x)


def hadamard128_fwht(x: torch.Tensor, scale: float, out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """Block-128 fast Walsh-Hadamard transform in fp32, butterflies at distance 1, 2, 4, ... 64
    in that order, each `(a, b) -> (a + b, a - b)`, then `* fp32(scale)`, then one rounding
    to `out_dtype`.  This is the definition fast_hadamard_transform documents
    (F.linear(x, sylvester) * scale, fp32 inside), used by utils.py:38-39 on weights with
    scale=2**-3.5.  With scale=181/2048 it is also the order the HIP kernels use on
    activations, so their output is bit-identical to this function."""
    out_dtype = out_dtype or x.dtype
    shape = x.shape
    v = x.to(torch.float32).reshape(-1, HADAMARD_BLOCK).clone()
    h = 1
    while h < HADAMARD_BLOCK:
        w = v.view(-1, HADAMARD_BLOCK // (2 * h), 2, h)
        a = w[:, :, 0, :].clone()
        b = w[:, :, 1, :].clone()
        w[:, :, 0, :] = a + b
        w[:, :, 1, :] = a - b
        h *= 2
    v = v * torch.tensor(scale, dtype=torch.float32)
    return v.to(out_dtype).reshape(shape)


def hadamard_entry(dtype: torch.dtype) -> float:
    """The single magnitude in hadamard_matrix(dtype) (0.08837890625 for bf16/fp16)."""
    return float(torch.tensor(128 ** -0.5, dtype=torch.float32).to(dtype).float())


# ----------------------------------------------------------------------------- S1 / S2
def find_scale_int4(x: torch.Tensor, scale: torch.Tensor | None = None) -> torch.Tensor:
    """utils.py:193-209."""
    if scale is None:
        scale = torch.empty(*x.shape[:-1], 1, dtype=x.dtype)
    xf = x.to(dtype=torch.float32)
    scale_ = (xf * xf).mean(dim=-1, keepdim=True).sqrt() * GAUSS_INT4_STEP + SCALE_EPS
    return scale.copy_(scale_)


def quantize_int4(x, scale, x_int=None, x_int_packed=None, x_int_row_sum=None, do_dequantize=False):
    """utils.py:334-365 (same ops, same order; writes into the buffers it is given)."""
    x_q = (x.to(dtype=torch.float32) / scale.to(dtype=torch.float32)).floor().clamp(16 // -2, 16 // 2 - 1)
    if do_dequantize:
        x_dq = x_q * scale + (scale * .5)
        x.copy_(x_dq)
    if x_int is not None or x_int_packed is not None or x_int_row_sum is not None:
        x_int_ = x_q.to(dtype=torch.int8)
        if x_int is not None:
            x_int.copy_(x_int_)
        if x_int_packed is not None:
            x_int_packed.copy_((x_int_[..., 1::2] << 4) | (x_int_[..., ::2] & 0xF))
        if x_int_row_sum is not None:
            x_int_row_sum.copy_(x_int_.to(dtype=torch.int32).sum(dim=-1, keepdim=True))
    return x, x_int, x_int_packed, x_int_row_sum


def pack_int4(x_int: torch.Tensor) -> torch.Tensor:
    """utils.py:359 -- byte j = (q[2j+1] << 4) | (q[2j] & 0xF), as uint8."""
    return ((x_int[..., 1::2] << 4) | (x_int[..., ::2] & 0xF)).view(torch.uint8)


def unpack_int4(x_int_packed: torch.Tensor) -> torch.Tensor:
    """utils.py:441-445."""
    x_int = torch.empty(*x_int_packed.shape[:-1], x_int_packed.size(-1) * 2, dtype=torch.int8)
    x_int[..., ::2] = x_int_packed & 0xF
    x_int[..., 1::2] = x_int_packed >> 4
    return torch.where(x_int >= 8, x_int - 16, x_int)


# ----------------------------------------------------------------------------- G1 / E1
def matmul_int4_int4t_int32(mat_a: torch.Tensor, mat_b: torch.Tensor, via: str = 'fp64') -> torch.Tensor:
    """C = A @ B.t() on the unpacked codes.  via='fp64' is what the reference's own check
    does (utils.py:680); via='fp32' is exact too while 64*K < 2**24 (every partial sum is an
    integer below 2**24) and is the faster CPU path."""
    a = unpack_int4(mat_a)
    b = unpack_int4(mat_b)
    k = a.size(-1)
    if via == 'fp32':
        assert 64 * k < (1 << 24)
        return (a.to(torch.float32) @ b.to(torch.float32).t()).to(torch.int32)
    return (a.to(torch.float64) @ b.to(torch.float64).t()).to(torch.int32)


def add_mul_vv(vec_a_add, vec_a_mul, vec_b_add, vec_b_mul, mat_c, mat_d=None):
    """utils.py:535-545."""
    if mat_d is None:
        mat_d = torch.empty(mat_c.shape, dtype=vec_a_mul.dtype)
    acc = torch.float32
    mat_d_ = (mat_c * 2 + vec_a_add + vec_b_add.t()).to(dtype=acc) * (.5 * vec_a_mul.to(dtype=acc) * vec_b_mul.t().to(dtype=acc))
    return mat_d.copy_(mat_d_)


def fused_matmul_dequantize_int4_int4t(mat_a, mat_b, vec_a_add, vec_b_add, vec_a_mul, vec_b_mul, via='fp64'):
    """utils.py:581-584 (debug_mode=True composition: integer GEMM, then add_mul_vv)."""
    c = matmul_int4_int4t_int32(mat_a, mat_b, via=via)
    return add_mul_vv(vec_a_add, vec_a_mul, vec_b_add, vec_b_mul, c)


# ----------------------------------------------------------------------------- L1
def find_scale_absmax_int4(x: torch.Tensor, scale: torch.Tensor | None = None) -> torch.Tensor:
    """The other weight-scale rule named for the CPU-runnable benchmark case ("per-row absmax scales"): the step
    that puts the row's largest magnitude at the edge of the INT4 grid, 7.5 steps out (floor(x / s) is then 7 for
    +absmax and -8 for -absmax, both dequantising to +-7.5 s).  Not in the reference's code, which uses the RMS
    rule (utils.py:46); same epsilon as that rule so that an all-zero row is defined."""
    if scale is None:
        scale = torch.empty(*x.shape[:-1], 1, dtype=x.dtype)
    scale_ = x.to(dtype=torch.float32).abs().amax(dim=-1, keepdim=True) / 7.5 + SCALE_EPS
    return scale.copy_(scale_)


def preprocess_weight(weight: torch.Tensor, use_hadamard: bool = False, w_scale_mode: str = 'rms'):
    """utils.py:20-49, dense branch.  Returns (w_int_packed, w_scale, w_add, None).  w_scale_mode='rms' is the
    reference's rule, 'absmax' the one above."""
    if use_hadamard:
        weight = hadamard128_fwht(weight, 2. ** -3.5)
    weight = weight.contiguous()
    n, k = weight.shape
    w_scale = torch.empty(n, 1, dtype=weight.dtype)
    w_int_packed = torch.empty(n, k // 2, dtype=torch.uint8)
    w_int_row_sum = torch.empty(n, 1, dtype=torch.int32)
    {'rms': find_scale_int4, 'absmax': find_scale_absmax_int4}[w_scale_mode](weight, w_scale)
    quantize_int4(weight, w_scale, None, w_int_packed.view(torch.int8), w_int_row_sum, False)
    w_add = w_int_row_sum + k // 2
    return w_int_packed, w_scale, w_add, None


def hadamard_quantize_int4(x: torch.Tensor, hadamard: str = 'fwht'):
    """The activation half of linear_forward (utils.py:89-100): Hadamard, scale, codes,
    row sums.  hadamard='matmul' is the reference's formulation, 'fwht' the fp32 butterfly
    order the HIP kernel uses.  Returns (x_had, scale, packed, row_sum)."""
    if hadamard == 'matmul':
        xh = hadamard128_matmul(x)
    elif hadamard == 'fwht':
        xh = hadamard128_fwht(x, hadamard_entry(x.dtype))
    else:
        raise ValueError(hadamard)
    m, k = xh.shape
    scale = find_scale_int4(xh)
    packed = torch.empty(m, k // 2, dtype=torch.uint8)
    row_sum = torch.empty(m, 1, dtype=torch.int32)
    quantize_int4(xh, scale, None, packed.view(torch.int8), row_sum, False)
    return xh, scale, packed, row_sum


def linear_forward(activation, w_int_packed, w_scale, w_add, use_hadamard=False, hadamard='matmul', via='fp64'):
    """utils.py:56-101, dense branch, with the fused GEMM written as its debug composition
    (integer GEMM + add_mul_vv, utils.py:581-584)."""
    m, k = activation.shape
    if use_hadamard:
        activation = hadamard128_matmul(activation) if hadamard == 'matmul' else \
            hadamard128_fwht(activation, hadamard_entry(activation.dtype))
    a_scale = find_scale_int4(activation)
    a_packed = torch.empty(m, k // 2, dtype=torch.uint8)
    a_row_sum = torch.empty(m, 1, dtype=torch.int32)
    quantize_int4(activation, a_scale, None, a_packed.view(torch.int8), a_row_sum, False)
    return fused_matmul_dequantize_int4_int4t(a_packed, w_int_packed, a_row_sum, w_add, a_scale, w_scale, via=via)


def linear_fp64(a_int, a_scale, w_int, w_scale):
    """utils.py:667-671 -- the fp64 product of the dequantised operands, (q + 1/2) * s."""
    a_dq = (a_int.to(torch.float64) + .5) * a_scale.to(torch.float64)
    w_dq = (w_int.to(torch.float64) + .5) * w_scale.to(torch.float64)
    return a_dq @ w_dq.t()


# ---------------------------------------------------------------------------------------------
# The FP6 (E2M3) operand form of the codes.  No counterpart in the reference: it is this build's storage format for
# the codes of the same GEMM, so what the oracle states is the OCP Microscaling FP6 E2M3 number format itself (1 sign
# bit, 2 exponent bits with bias 1, 3 mantissa bits, subnormals, no Inf/NaN) and the tile layout declared in
# include/quest_hip.h; tests/test_oracle_pins.py pins the decoder by the format's published value table.
# ---------------------------------------------------------------------------------------------
E2M3_FRAGMENT_BYTES = 1536


def e2m3_value(bits: torch.Tensor) -> torch.Tensor:
    """fp64 value of 6-bit E2M3 patterns: (-1)^s * 2^(e-1) * (1 + m/8) for e > 0, (-1)^s * m/8 for e = 0."""
    bits = bits.to(torch.int64)
    sign = 1. - 2. * ((bits >> 5) & 1).to(torch.float64)
    e = (bits >> 3) & 3
    m = (bits & 7).to(torch.float64)
    mag = torch.where(e == 0, m / 8., (1. + m / 8.) * torch.pow(torch.tensor(2., dtype=torch.float64), (e - 1).to(torch.float64)))
    return sign * mag


def e2m3_bits_of_code(q: torch.Tensor) -> torch.Tensor:
    """The E2M3 pattern whose value is q + 1/2, for INT4 codes q in [-8, 7] (found by search over all 64 patterns)."""
    table = e2m3_value(torch.arange(64))
    want = q.to(torch.float64) + .5
    hit = table[None, :] == want.reshape(-1, 1)
    assert bool(hit.any(dim=1).all()), 'a code whose q + 1/2 is not an E2M3 value'
    return hit.to(torch.int64).argmax(dim=1).reshape(q.shape).to(torch.uint8)


def _tile_index(rows: int, k: int):
    """For every (row, k) of a code matrix: byte-independent coordinates (fragment, lane, position in the lane's 32)."""
    r = torch.arange(rows)[:, None].expand(rows, k)
    c = torch.arange(k)[None, :].expand(rows, k)
    frag = (r // 32) * (k // 64) + c // 64
    lane = 32 * ((c % 64) // 32) + r % 32
    return frag, lane, c % 32


def e2m3_tiles_encode(x_int: torch.Tensor) -> torch.Tensor:
    """(rows, K) int8 codes -> flat uint8 E2M3 tiles (layout of include/quest_hip.h; padding rows are zero bytes)."""
    rows, k = x_int.shape
    assert k % 64 == 0
    nfrag = ((rows + 31) // 32) * (k // 64)
    frag, lane, j = _tile_index(rows, k)
    bits = e2m3_bits_of_code(x_int).to(torch.int64)
    # the lane's 24 bytes as a bit string: code j at bits [6 j, 6 j + 6); spread into (nfrag, 64, 192) single bits
    lane_bits = torch.zeros(nfrag, 64, 192, dtype=torch.uint8)
    for b in range(6):
        lane_bits[frag, lane, 6 * j + b] = ((bits >> b) & 1).to(torch.uint8)
    weights = (1 << torch.arange(8)).to(torch.uint8)
    lane_bytes = (lane_bits.view(nfrag, 64, 24, 8) * weights).sum(dim=-1).to(torch.uint8)     # (nfrag, 64, 24)
    out = torch.empty(nfrag, E2M3_FRAGMENT_BYTES, dtype=torch.uint8)
    out[:, :1024] = lane_bytes[:, :, :16].reshape(nfrag, 1024)
    out[:, 1024:] = lane_bytes[:, :, 16:].reshape(nfrag, 512)
    return out.reshape(-1)


def e2m3_tiles_decode(tiles: torch.Tensor, rows: int, k: int) -> torch.Tensor:
    """Flat uint8 E2M3 tiles -> (rows, K) fp64 values (q + 1/2 for tiles that hold codes)."""
    nfrag = ((rows + 31) // 32) * (k // 64)
    t = tiles.reshape(nfrag, E2M3_FRAGMENT_BYTES)
    lane_bytes = torch.cat((t[:, :1024].reshape(nfrag, 64, 16), t[:, 1024:].reshape(nfrag, 64, 8)), dim=2)
    lane_bits = ((lane_bytes[..., None].to(torch.int64) >> torch.arange(8)) & 1).reshape(nfrag, 64, 192)
    frag, lane, j = _tile_index(rows, k)
    bits = torch.zeros(rows, k, dtype=torch.int64)
    for b in range(6):
        bits |= lane_bits[frag, lane, 6 * j + b] << b
    return e2m3_value(bits)


# ---------------------------------------------------------------------------------------------
# The training-side (fake-quantised) statement of the same layer, for judging the packed INT4 path
# against what a QuEST-trained checkpoint was evaluated with.
# ---------------------------------------------------------------------------------------------
OPTIMAL_GAUSSIAN_SCALE_INT4 = 2.513930578568423      # src/models/quantization/base_linear.py:38-48, bits = 4


def fake_quant_hadamard(x: torch.Tensor):
    """src/eval_hswag.py:203-217 (quantize_pack_hadamard_dense, 4 bits, centred): rotate by the block-128 Hadamard
    transform (factor 2^-3.5), clip at 2.5139 rms, round to the 16 levels.  Returns (levels 0..15 in the rotated
    space, scale, step), all fp32."""
    xf = x.to(torch.float32)
    x_had = hadamard128_fwht(xf.reshape(-1, HADAMARD_BLOCK), 2. ** -3.5, out_dtype=torch.float32).reshape(x.shape)
    std = torch.sqrt(torch.mean(x_had ** 2, dim=-1, keepdim=True)) + 1e-8
    scale = OPTIMAL_GAUSSIAN_SCALE_INT4 * std
    step = 2 * scale / 15
    xq = torch.round((torch.clamp(x_had, -scale, scale) + scale) / step)
    return xq, scale, step


def fake_quant_linear(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """src/eval_hswag.py:156-173 (its Linear4bit): both operands fake-quantised in the rotated space, dense fp32
    product.  The rotations cancel in the product, so this is the layer the packed path computes."""
    xq, xs, xstep = fake_quant_hadamard(x)
    wq, ws, wstep = fake_quant_hadamard(weight)
    return F.linear(xq * xstep - xs, wq * wstep - ws, None if bias is None else bias.to(torch.float32))
