"""Seeded random shapes through the C ABI: the dispatch rules meet sizes nobody wrote down.

The fixed lists of tests/test_gpu_parity.py name the boundaries of every kernel; here the shapes are drawn (fixed
seeds, so every run sees the same ones) from the ranges the rules cut up -- token counts from 1 to 9000, K any
multiple of 32 up to 5000 (mostly of 128), ragged channel counts -- and checked against exact integers:

  * the int32 matrix against an fp64 product of the unpacked codes (exact: |C| <= 64 K < 2^53);
  * the fused output against the epilogue formula of `add_mul_vv` (gemm-quest/benchmarks/utils.py:535-545 of the
    reference) applied to that matrix with IEEE fp32 elementwise operations -- bit for bit;
  * the fused activation kernel against its own unfused steps (find_scale_int4, quantize_int4 on its transformed
    tensor) -- codes and row sums bit for bit, scale within the one 16-bit ulp the two fp32 summation orders allow;
  * the kernels with a producer in front against the same producer followed by the plain kernel, bit for bit.
"""
import random

import pytest
import torch

from oracle import quest_oracle as qo

pytestmark = pytest.mark.gpu
DEV = 'cuda:0'


@pytest.fixture(scope='module')
def quest():
    import quest_amd
    from quest_amd import _lib
    _lib.load()
    assert torch.cuda.is_available()
    return quest_amd


def unpack(packed):
    """(rows, K/2) uint8 -> (rows, K) int8 codes, low nibble first (gemm-quest/benchmarks/utils.py:420-445)."""
    lo = (packed & 0xF).to(torch.int8)
    hi = (packed >> 4).to(torch.int8)
    lo = torch.where(lo >= 8, lo - 16, lo)
    hi = torch.where(hi >= 8, hi - 16, hi)
    return torch.stack((lo, hi), dim=-1).flatten(-2)


def bits(t):
    return t.contiguous().view(torch.int16)


def gemm_shapes(seed, count):
    rng = random.Random(seed)
    out = []
    for _ in range(count):
        kind = rng.random()
        if kind < 0.25:
            m = rng.choice([1, 16, 17, 32, 33, 64, 65, 128, 129, 256, 258, 1000, 4096])
        elif kind < 0.5:
            m = rng.randrange(1, 130)
        else:
            m = rng.randrange(1, 9000)
        k = 128 * rng.randrange(1, 24) if rng.random() < 0.8 else 32 * rng.randrange(1, 60)
        n = rng.randrange(1, 6000)
        if rng.random() < 0.6:
            n += n & 1
        while m * n > 3.0e7:                       # keep the fp64 product of a case within a few hundred MB
            n = max(1, n // 2)
        out.append((m, k, n, rng.choice([torch.bfloat16, torch.float16])))
    return out


@pytest.mark.parametrize('seed', [101, 102, 103])
def test_gemm_random_shapes(quest, seed):
    g = torch.Generator(device=DEV).manual_seed(seed)
    for m, k, n, dtype in gemm_shapes(seed, 40):
        a = torch.randint(0, 256, (m, k // 2), dtype=torch.uint8, device=DEV, generator=g)
        b = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device=DEV, generator=g)
        a_add = torch.randint(-300, 300, (m, 1), dtype=torch.int32, device=DEV, generator=g)
        b_add = torch.randint(-300, 300, (n, 1), dtype=torch.int32, device=DEV, generator=g)
        a_mul = (torch.rand(m, 1, device=DEV, generator=g) * 0.09 + 0.01).to(dtype)
        b_mul = (torch.rand(n, 1, device=DEV, generator=g) * 0.09 + 0.01).to(dtype)
        want_c = (unpack(a).double() @ unpack(b).double().T).to(torch.int32)
        got_c = quest.matmul_int4_int4t_int32(a, b)
        assert torch.equal(got_c, want_c), (m, k, n)
        got_d = quest.fused_matmul_dequantize_int4_int4t_bf16(a, b, a_add, b_add, a_mul, b_mul)
        lhs = (want_c * 2 + a_add + b_add.T).float()
        rhs = (0.5 * a_mul.float()) * b_mul.float().T
        assert torch.equal(bits(got_d), bits((lhs * rhs).to(dtype))), (m, k, n, dtype)
        if k % 128 == 0:
            # the FP6 kernel on the same codes as E2M3 tiles: the add vectors are the codes' own sums there
            ua, ub = unpack(a).to(torch.int32), unpack(b).to(torch.int32)
            lhs6 = (want_c * 2 + ua.sum(-1, keepdim=True) + (ub.sum(-1, keepdim=True) + k // 2).T).float()
            got6 = quest.fused_matmul_dequantize_e2m3(quest.int4_to_e2m3_tiles(a), quest.int4_to_e2m3_tiles(b), a_mul, b_mul, k)
            assert torch.equal(bits(got6), bits((lhs6 * rhs).to(dtype))), (m, k, n, dtype)


@pytest.mark.parametrize('seed', [201, 202])
def test_activation_kernel_random_shapes(quest, seed):
    rng = random.Random(seed)
    g = torch.Generator(device=DEV).manual_seed(seed)
    for _ in range(40):
        m = rng.choice([1, 2, 3, 5, 16, 33, 64, 100, 257, 1000, 4097]) if rng.random() < 0.6 else rng.randrange(1, 3000)
        k = 128 * rng.choice([1, 2, 3, 4, 5, 8, 11, 16, 22, 32, 33, 40, 64, 86, 128, 200, 256])
        m = min(m, max(1, int(2.0e7 // k)))
        dtype = rng.choice([torch.bfloat16, torch.float16])
        xf = torch.randn(m, k, device=DEV, generator=g) * (torch.rand(m, 1, device=DEV, generator=g) * 4 + 0.05)
        # rows of small and large magnitude, and one whose values and scale lie in the dtype's subnormals (fp16: below
        # 6.1e-5; the scale stays above zero -- what a zero scale gives is fixed by tests/test_gpu_configs.py)
        if m >= 4:
            xf[0] *= 1e-3
            xf[1] *= 1e3
            xf[2] *= 2e-6 if dtype == torch.float16 else 1e-30
        x = xf.to(dtype)
        x_had = torch.empty_like(x)
        scale, packed, row_sum = quest.hadamard_quantize_int4(x, x_had=x_had)
        s2 = quest.find_scale_int4(x_had)
        assert (bits(scale).int() - bits(s2).int()).abs().max() <= 1, (m, k, dtype)
        _, _, p2, r2 = quest.quantize_int4(x_had.clone(), scale, x_int_packed=torch.empty_like(packed),
                                           x_int_row_sum=torch.empty_like(row_sum))
        assert torch.equal(packed, p2) and torch.equal(row_sum, r2), (m, k, dtype)
        # the two kernels share their quantiser helpers, so a sample of rows also goes through the CPU oracle
        # (IEEE divide, floor, clamp: gemm-quest/benchmarks/utils.py:334-365) with the kernel's transform and scale
        sample = list(range(min(m, 6)))
        o_packed = torch.empty(len(sample), k // 2, dtype=torch.uint8)
        o_sum = torch.empty(len(sample), 1, dtype=torch.int32)
        qo.quantize_int4(x_had[sample].cpu().clone(), scale[sample].cpu(), None, o_packed, o_sum, False)
        assert torch.equal(packed[sample].cpu(), o_packed) and torch.equal(row_sum[sample].cpu(), o_sum), (m, k, dtype)
        # ... and the E2M3 tiles hold the same codes
        _, tiles = quest.hadamard_quantize_e2m3(x)
        assert torch.equal(quest.int4_to_e2m3_tiles(packed).view(-1, 1536)[: (m // 32) * (k // 64)],
                           tiles.view(-1, 1536)[: (m // 32) * (k // 64)]), (m, k, dtype)
        if k > 4096 and rng.random() < 0.5:
            continue
        w = (1 + 0.1 * torch.randn(k, device=DEV, generator=g)).to(dtype)
        x_norm = torch.empty_like(x)
        q1 = quest.rmsnorm_hadamard_quantize_int4(x, w, 1e-5, x_norm=x_norm)
        q2 = quest.hadamard_quantize_int4(x_norm)
        assert torch.equal(bits(q1[0]), bits(q2[0])) and torch.equal(q1[1], q2[1]) and torch.equal(q1[2], q2[2]), (m, k, dtype)
        branch = torch.randn(m, k, device=DEV, generator=g).to(dtype)
        stream, want_sum = x.clone(), x + branch
        q3 = quest.add_rmsnorm_hadamard_quantize_int4(stream, branch, w, 1e-5)
        q4 = quest.rmsnorm_hadamard_quantize_int4(want_sum, w, 1e-5)
        assert torch.equal(bits(stream), bits(want_sum)), (m, k, dtype)
        assert torch.equal(bits(q3[0]), bits(q4[0])) and torch.equal(q3[1], q4[1]) and torch.equal(q3[2], q4[2]), (m, k, dtype)
        gate_up = torch.randn(m, 2 * k, device=DEV, generator=g).to(dtype)
        act = torch.empty(m, k, dtype=dtype, device=DEV)
        q5 = quest.silu_mul_hadamard_quantize_int4(gate_up, x_act=act)
        q6 = quest.hadamard_quantize_int4(act)
        assert torch.equal(bits(q5[0]), bits(q6[0])) and torch.equal(q5[1], q6[1]) and torch.equal(q5[2], q6[2]), (m, k, dtype)
