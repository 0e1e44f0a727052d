"""GPU parity of the FP6 (E2M3) matrix-core path: the operand form of the codes and the GEMM on it, through the C ABI.

Bars: the E2M3 tiles are a re-encoding of the INT4 codes (bit-exact against the oracle's encoder, and decoding them
gives q + 1/2 for exactly the codes that went in); the GEMM's outputs equal the oracle's fused GEMM + scale epilogue
(benchmarks/utils.py:544 on the exact integer matrix) bit for bit -- i.e. the FP6 sums are exact -- and those of the
INT8 kernels on the same codes."""
import pytest
import torch

from oracle import quest_oracle as qo

pytestmark = pytest.mark.gpu

DTYPES = [torch.bfloat16, torch.float16]
DEV = 'cuda:0'


@pytest.fixture(scope='module')
def quest():
    import quest_amd
    from quest_amd import _lib
    _lib.load()
    assert torch.cuda.is_available()
    return quest_amd


def bits(t):
    return t.contiguous().view(torch.int16).to(torch.int32)


def rand_codes(rows, k, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(-8, 8, (rows, k), generator=g).to(torch.int8)


def scales(m, n, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return ((torch.rand(m, 1, generator=g) * 0.09 + 0.01).to(dtype), (torch.rand(n, 1, generator=g) * 0.09 + 0.01).to(dtype))


def oracle_output(qa, qb, a_mul, b_mul):
    """The reference's fused GEMM on packed codes with its add vectors (the oracle's statement of utils.py:544)."""
    k = qa.size(1)
    a_add = qa.to(torch.int32).sum(-1, keepdim=True).to(torch.int32)
    b_add = qb.to(torch.int32).sum(-1, keepdim=True).to(torch.int32) + k // 2
    return qo.fused_matmul_dequantize_int4_int4t(qo.pack_int4(qa), qo.pack_int4(qb), a_add, b_add, a_mul, b_mul, via='fp32')


@pytest.mark.parametrize('shape', [(32, 64), (70, 128), (1, 4096), (257, 384), (4096, 1024), (33, 11008)])
def test_tiles_are_the_oracle_encoding(quest, shape):
    rows, k = shape
    q = rand_codes(rows, k, 11)
    tiles = quest.int4_to_e2m3_tiles(qo.pack_int4(q).to(DEV)).cpu()
    assert tiles.numel() == quest.e2m3_tiles_bytes(rows, k) == ((rows + 31) // 32) * (k // 64) * 1536
    assert torch.equal(tiles, qo.e2m3_tiles_encode(q))
    assert torch.equal(qo.e2m3_tiles_decode(tiles, rows, k), q.double() + .5)


GEMM_SHAPES = [(256, 128, 256), (160, 768, 224), (512, 1024, 1024), (257, 128, 300), (300, 256, 257), (33, 128, 7),
               (1, 4096, 64), (1001, 128, 96), (777, 1152, 4100), (4097, 128, 1031), (1536, 256, 4096),
               (4096, 256, 2048), (2048, 4096, 512), (16390, 256, 1000), (640, 2816, 1024)]


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape', GEMM_SHAPES)
def test_gemm_bit_exact(quest, dtype, shape):
    m, k, n = shape
    qa, qb = rand_codes(m, k, 7), rand_codes(n, k, 8)
    a_mul, b_mul = scales(m, n, dtype, 6)
    want = oracle_output(qa, qb, a_mul, b_mul)
    ta = quest.int4_to_e2m3_tiles(qo.pack_int4(qa).to(DEV))
    tb = quest.int4_to_e2m3_tiles(qo.pack_int4(qb).to(DEV))
    got = quest.fused_matmul_dequantize_e2m3(ta, tb, a_mul.to(DEV), b_mul.to(DEV), k).cpu()
    assert got.dtype == dtype and got.shape == (m, n)
    assert torch.equal(bits(got), bits(want))
    ref = qo.linear_fp64(qa, a_mul, qb, b_mul)
    assert ((got.double() - ref).norm() / ref.norm()) < 1e-2


def test_every_pair_of_codes(quest):
    """Row i of A holds code (i % 16) in every position, row j of B code (j % 16): all 256 products, each summed K times."""
    k = 256
    qa = (torch.arange(32) % 16 - 8).to(torch.int8)[:, None].repeat(1, k)
    qb = (torch.arange(48) % 16 - 8).to(torch.int8)[:, None].repeat(1, k)
    one = torch.ones(32, 1, dtype=torch.float16), torch.ones(48, 1, dtype=torch.float16)
    ta = quest.int4_to_e2m3_tiles(qo.pack_int4(qa).to(DEV))
    tb = quest.int4_to_e2m3_tiles(qo.pack_int4(qb).to(DEV))
    got = quest.fused_matmul_dequantize_e2m3(ta, tb, one[0].to(DEV), one[1].to(DEV), k).cpu().double()
    want = k * (qa[:, :1].double() + .5) @ (qb[:, :1].double() + .5).t()        # |.| <= 256 * 56.25: exact in fp16
    assert torch.equal(got, want)


@pytest.mark.parametrize('k', [11008, 65536])
def test_extreme_sums_are_exact(quest, k):
    """All codes -8 against -8 and against 7: the largest sums the path can see (56.25 K), then half a row of large
    products followed by small random ones (a large accumulator must not swallow the quarter units)."""
    m, n = 64, 96
    qa = torch.full((m, k), -8, dtype=torch.int8)
    qb = torch.full((n, k), -8, dtype=torch.int8)
    qb[1::2] = 7
    qa[32:, k // 2:] = rand_codes(32, k // 2, 3)
    qb[48:, k // 2:] = rand_codes(48, k // 2, 4)
    a_mul, b_mul = scales(m, n, torch.bfloat16, 9)
    ta = quest.int4_to_e2m3_tiles(qo.pack_int4(qa).to(DEV))
    tb = quest.int4_to_e2m3_tiles(qo.pack_int4(qb).to(DEV))
    got = quest.fused_matmul_dequantize_e2m3(ta, tb, a_mul.to(DEV), b_mul.to(DEV), k).cpu()
    assert torch.equal(bits(got), bits(oracle_output(qa, qb, a_mul, b_mul)))


@pytest.mark.parametrize('seed', range(12))
def test_gemm_seeded_fuzz(quest, seed):
    g = torch.Generator().manual_seed(1000 + seed)
    m = int(torch.randint(1, 1200, (1,), generator=g))
    n = int(torch.randint(1, 1500, (1,), generator=g))
    k = 128 * int(torch.randint(1, 24, (1,), generator=g))
    dtype = DTYPES[seed % 2]
    qa, qb = rand_codes(m, k, 2000 + seed), rand_codes(n, k, 3000 + seed)
    a_mul, b_mul = scales(m, n, dtype, 4000 + seed)
    ta = quest.int4_to_e2m3_tiles(qo.pack_int4(qa).to(DEV))
    tb = quest.int4_to_e2m3_tiles(qo.pack_int4(qb).to(DEV))
    got = quest.fused_matmul_dequantize_e2m3(ta, tb, a_mul.to(DEV), b_mul.to(DEV), k).cpu()
    assert torch.equal(bits(got), bits(oracle_output(qa, qb, a_mul, b_mul))), (m, k, n)


@pytest.mark.parametrize('dtype', DTYPES)
def test_gemm_equals_int8_kernels_at_prefill_size(quest, dtype):
    """M = 4096, K = 4096, N = 11008: the whole output against the INT8 kernel on the same codes (itself checked against
    exact integers at this size), bit for bit."""
    m, k, n = 4096, 4096, 11008
    g = torch.Generator(device=DEV).manual_seed(5)
    a = torch.randint(0, 256, (m, k // 2), generator=g, device=DEV, dtype=torch.uint8)
    b = torch.randint(0, 256, (n, k // 2), generator=g, device=DEV, dtype=torch.uint8)
    a_mul = (torch.rand(m, 1, generator=g, device=DEV) * 0.09 + 0.01).to(dtype)
    b_mul = (torch.rand(n, 1, generator=g, device=DEV) * 0.09 + 0.01).to(dtype)
    from quest_amd import harness
    a_add = harness.unpack_int4(a).to(torch.int32).sum(-1, keepdim=True).to(torch.int32)
    b_add = harness.unpack_int4(b).to(torch.int32).sum(-1, keepdim=True).to(torch.int32) + k // 2
    want = quest.fused_matmul_dequantize_int4_int4t_bf16(a, b, a_add, b_add, a_mul, b_mul)
    got = quest.fused_matmul_dequantize_e2m3(quest.int4_to_e2m3_tiles(a), quest.int4_to_e2m3_tiles(b), a_mul, b_mul, k)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    again = quest.fused_matmul_dequantize_e2m3(quest.int4_to_e2m3_tiles(a), quest.int4_to_e2m3_tiles(b), a_mul, b_mul, k)
    assert torch.equal(got.view(torch.int16), again.view(torch.int16))


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape', [(160, 768, 224), (300, 256, 1000), (4096, 128, 4104), (1000, 512, 2048)])
def test_gemm_swiglu_equals_int8_kernel(quest, dtype, shape):
    m, k, n = shape
    h = n // 2
    qa, qb = rand_codes(m, k, 31), rand_codes(n, k, 32)
    a_mul, b_mul = scales(m, n, dtype, 33)
    a, b = qo.pack_int4(qa).to(DEV), qo.pack_int4(qb).to(DEV)
    a_add = qa.to(torch.int32).sum(-1, keepdim=True).to(torch.int32).to(DEV)
    b_add = (qb.to(torch.int32).sum(-1, keepdim=True).to(torch.int32) + k // 2).to(DEV)
    p = quest.swiglu_interleave_rows(h, device=DEV)
    bp, bp_add, bp_mul = b[p].contiguous(), b_add[p].contiguous(), b_mul.to(DEV)[p].contiguous()
    want = quest.fused_matmul_dequantize_swiglu_int4_int4t(a, bp, a_add, bp_add, a_mul.to(DEV), bp_mul)
    got = quest.fused_matmul_dequantize_e2m3(quest.int4_to_e2m3_tiles(a), quest.int4_to_e2m3_tiles(bp), a_mul.to(DEV), bp_mul, k,
                                             swiglu=True)
    assert got.shape == (m, h)
    assert torch.equal(bits(got.cpu()), bits(want.cpu()))


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape', [(300, 256, 1000), (4096, 128, 4104), (1000, 512, 2048), (130, 384, 77), (2048, 2560, 2560), (33, 128, 8)])
def test_gemm_adds_into_the_residual_stream(quest, dtype, shape):
    """add_to_out: out <- dtype(out + dtype(product)), the bits of torch's `out + product` (interior and edge tiles, a
    channel count that is not a multiple of 8, large and tiny residuals, twice in a row on the same buffer)."""
    m, k, n = shape
    g = torch.Generator(device=DEV).manual_seed(41)
    a = torch.randint(0, 256, (m, k // 2), generator=g, device=DEV, dtype=torch.uint8)
    b = torch.randint(0, 256, (n, k // 2), generator=g, device=DEV, dtype=torch.uint8)
    a_mul = (torch.rand(m, 1, generator=g, device=DEV) * 0.09 + 0.01).to(dtype)
    b_mul = (torch.rand(n, 1, generator=g, device=DEV) * 0.09 + 0.01).to(dtype)
    ta, tb = quest.int4_to_e2m3_tiles(a), quest.int4_to_e2m3_tiles(b)
    product = quest.fused_matmul_dequantize_e2m3(ta, tb, a_mul, b_mul, k)
    res = (torch.randn(m, n, generator=g, device=DEV) * torch.rand(m, 1, generator=g, device=DEV) * 50).to(dtype)
    res[0] *= 1e-4
    want = res + product
    got = res.clone()
    ret = quest.fused_matmul_dequantize_e2m3(ta, tb, a_mul, b_mul, k, out=got, add_to_out=True)
    assert ret.data_ptr() == got.data_ptr()
    assert torch.equal(bits(got.cpu()), bits(want.cpu()))
    quest.fused_matmul_dequantize_e2m3(ta, tb, a_mul, b_mul, k, out=got, add_to_out=True)
    assert torch.equal(bits(got.cpu()), bits((want + product).cpu()))


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape', [
    # batch, sequence, K, heads, head_dim, extra channels after q, k, v
    (2, 150, 256, 3, 32, 0), (1, 4096, 128, 2, 64, 0), (3, 100, 512, 5, 96, 0), (2, 512, 2560, 20, 128, 0),
    (5, 33, 128, 1, 128, 8), (1, 32, 128, 2, 32, 0)])
def test_gemm_rotates_q_and_k(quest, dtype, shape):
    """rope=...: the GEMM's output with the first 2 d channels rotated = the plain GEMM followed by the rotary kernel, bit
    for bit (positions wrapping at every sequence, heads narrower and wider than a tile's channel unit, edge tiles, a
    trailing block of channels that is not a head)."""
    bsz, t, k, heads, hd, extra = shape
    m, c = bsz * t, heads * hd
    n = 3 * c + extra
    g = torch.Generator(device=DEV).manual_seed(43)
    a = torch.randint(0, 256, (m, k // 2), generator=g, device=DEV, dtype=torch.uint8)
    b = torch.randint(0, 256, (n, k // 2), generator=g, device=DEV, dtype=torch.uint8)
    a_mul = (torch.rand(m, 1, generator=g, device=DEV) * 0.09 + 0.01).to(dtype)
    b_mul = (torch.rand(n, 1, generator=g, device=DEV) * 0.09 + 0.01).to(dtype)
    ang = torch.rand(t, hd // 2, generator=g, device=DEV) * 6.283
    freqs = torch.stack([torch.cos(ang), torch.sin(ang)], dim=-1).contiguous()
    ta, tb = quest.int4_to_e2m3_tiles(a), quest.int4_to_e2m3_tiles(b)
    want = quest.fused_matmul_dequantize_e2m3(ta, tb, a_mul, b_mul, k)
    plain = want.clone()
    quest.rope_interleaved_(want.view(bsz, t, n), freqs, 2 * c, hd)
    assert quest.rope_gemm_fuses(t, n, 2 * c, hd)
    got = quest.fused_matmul_dequantize_e2m3(ta, tb, a_mul, b_mul, k, rope=(freqs, 2 * c, hd))
    assert torch.equal(bits(got.cpu()), bits(want.cpu()))
    assert torch.equal(bits(got[:, 2 * c:].cpu()), bits(plain[:, 2 * c:].cpu()))           # v (and what follows) untouched
    assert not torch.equal(bits(got[:, :2 * c].cpu()), bits(plain[:, :2 * c].cpu()))


@pytest.mark.parametrize('seed', range(16))
def test_epilogues_seeded_fuzz(quest, seed):
    """Random shapes: the rotary and the residual-add epilogues of the FP6 GEMM and of the packed-nibble GEMM (whichever
    kernel takes the size) against the plain packed-nibble GEMM followed by the rotary kernel / by torch's addition."""
    import random
    rnd = random.Random(5000 + seed)
    dtype = DTYPES[seed % 2]
    hd = rnd.choice([32, 64, 96, 128])
    heads = rnd.randint(1, 12)
    c = heads * hd
    n = 2 * c + 8 * rnd.randint(0, 40)
    t = rnd.choice([32, 33, 64, 100, 128, 512])
    bsz = rnd.choice([1, 2, 3, 5, 8, rnd.randint(1, 16)])
    m, k = bsz * t, 128 * rnd.randint(1, 24)
    g = torch.Generator(device=DEV).manual_seed(6000 + seed)
    a = torch.randint(0, 256, (m, k // 2), generator=g, device=DEV, dtype=torch.uint8)
    b = torch.randint(0, 256, (n, k // 2), generator=g, device=DEV, dtype=torch.uint8)
    a_mul = (torch.rand(m, 1, generator=g, device=DEV) * 0.09 + 0.01).to(dtype)
    b_mul = (torch.rand(n, 1, generator=g, device=DEV) * 0.09 + 0.01).to(dtype)
    from quest_amd import harness
    a_add = harness.unpack_int4(a).to(torch.int32).sum(-1, keepdim=True).to(torch.int32)
    b_add = harness.unpack_int4(b).to(torch.int32).sum(-1, keepdim=True).to(torch.int32) + k // 2
    ang = torch.rand(t, hd // 2, generator=g, device=DEV) * 6.283
    freqs = torch.stack([torch.cos(ang), torch.sin(ang)], dim=-1).contiguous()
    plain = quest.fused_matmul_dequantize_int4_int4t_bf16(a, b, a_add, b_add, a_mul, b_mul)
    want = plain.clone()
    quest.rope_interleaved_(want.view(bsz, t, n), freqs, 2 * c, hd)
    case = (m, t, k, n, heads, hd)
    got = quest.fused_matmul_dequantize_rope_int4_int4t(a, b, a_add, b_add, a_mul, b_mul, freqs, 2 * c, hd)
    assert torch.equal(bits(got.cpu()), bits(want.cpu())), case
    ta, tb = quest.int4_to_e2m3_tiles(a), quest.int4_to_e2m3_tiles(b)
    got = quest.fused_matmul_dequantize_e2m3(ta, tb, a_mul, b_mul, k, rope=(freqs, 2 * c, hd))
    assert torch.equal(bits(got.cpu()), bits(want.cpu())), case
    res = (torch.randn(m, n, generator=g, device=DEV) * 30).to(dtype)
    want = res + plain
    got = res.clone()
    quest.fused_matmul_dequantize_add_int4_int4t(a, b, a_add, b_add, a_mul, b_mul, got)
    assert torch.equal(bits(got.cpu()), bits(want.cpu())), case
    got = res.clone()
    quest.fused_matmul_dequantize_e2m3(ta, tb, a_mul, b_mul, k, out=got, add_to_out=True)
    assert torch.equal(bits(got.cpu()), bits(want.cpu())), case


def test_rope_epilogue_rejects_what_it_does_not_take(quest):
    from quest_amd import _lib
    import ctypes
    lib = _lib.load()
    null, fake = ctypes.c_void_p(0), ctypes.c_void_p(0x1000)
    call = lambda n, seq, rot, hd, f=fake: lib.quest_fused_matmul_dequantize_rope_e2m3(fake, fake, fake, fake, fake, 64, 128, n, 0, f, seq, rot, hd, null)
    assert call(384, 64, 256, 128, null) == -1
    assert call(384, 16, 256, 128) == -2          # sequences shorter than 32
    assert call(384, 64, 256, 48) == -2           # heads that are not whole 32-channel units
    assert call(384, 64, 200, 128) == -2          # rotated channels that are not whole heads
    assert call(384, 64, 512, 128) == -2          # ... or more than there are
    assert call(386, 64, 256, 128) == -2          # channel count not a multiple of 8
    assert not quest.rope_gemm_fuses(16, 384, 256, 128) and not quest.rope_gemm_fuses(64, 384, 256, 48)


def test_error_codes(quest):
    from quest_amd import _lib
    import ctypes
    lib = _lib.load()
    null, fake = ctypes.c_void_p(0), ctypes.c_void_p(0x1000)
    assert lib.quest_fused_matmul_dequantize_e2m3(fake, fake, fake, fake, null, 4, 128, 4, 0, null) == -1
    assert lib.quest_fused_matmul_dequantize_e2m3(fake, fake, fake, fake, fake, 4, 192, 4, 0, null) == -2
    assert lib.quest_fused_matmul_dequantize_e2m3(fake, fake, fake, fake, fake, 4, 1 << 17, 4, 0, null) == -5
    assert lib.quest_fused_matmul_dequantize_e2m3(fake, fake, fake, fake, fake, 4, 128, 4, 7, null) == -3
    assert lib.quest_int4_to_e2m3_tiles(fake, fake, 4, 100, null) == -2
    assert lib.quest_e2m3_tiles_bytes(4, 100) == 0


# --------------------------------------------------------------------------- the activation kernels writing tiles
def rand_act(m, k, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, k, generator=g) * (torch.rand(m, 1, generator=g) * 4 + 0.05)
    return x.to(dtype)


ACT_SHAPES = [(64, 4096), (33, 1024), (70, 128), (5, 2816), (1, 4096), (257, 256), (40, 11008), (9, 8192), (130, 512), (3, 32768)]
# enough rows for workgroups of eight (four) whole rows that stage the tiles in LDS (at least two per compute unit), with a
# ragged last workgroup: rows of one wave's blocks, of fewer, and of two and three waves
STAGED_SHAPES = [(4101, 2560), (4099, 1024), (2051, 6912), (2050, 11008)]


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape', ACT_SHAPES + STAGED_SHAPES)
def test_activation_tiles_hold_the_packed_codes(quest, dtype, shape):
    """The tiles written by the fused activation kernel decode to exactly the codes its packed output holds (which the
    parity tests pin against the oracle), with the same scale, in one launch and in a launch that writes tiles only."""
    m, k = shape
    x = rand_act(m, k, dtype, 21).to(DEV)
    scale, packed, row_sum = quest.hadamard_quantize_int4(x)
    p2 = torch.empty_like(packed)
    r2 = torch.empty_like(row_sum)
    s_both, t_both = quest.hadamard_quantize_e2m3(x, x_int_packed=p2, x_int_row_sum=r2)
    s_only, t_only = quest.hadamard_quantize_e2m3(x)
    assert torch.equal(bits(s_both.cpu()), bits(scale.cpu())) and torch.equal(bits(s_only.cpu()), bits(scale.cpu()))
    assert torch.equal(p2, packed) and torch.equal(r2, row_sum)
    want = qo.unpack_int4(packed.cpu()).double() + .5
    assert torch.equal(qo.e2m3_tiles_decode(t_both.cpu(), m, k), want)
    assert torch.equal(qo.e2m3_tiles_decode(t_only.cpu(), m, k), want)


@pytest.mark.parametrize('dtype', DTYPES)
def test_activation_tiles_degenerate_rows(quest, dtype):
    """Zero rows, a NaN, an Inf and huge / tiny magnitudes: the tiles still hold the packed output's codes."""
    m, k = 8, 512
    x = rand_act(m, k, dtype, 22)
    x[1] = 0
    x[2, 5] = float('nan')
    x[3, 7] = float('inf')
    x[4] *= 1e4 if dtype == torch.float16 else 1e30
    x[5] *= 1e-6 if dtype == torch.float16 else 1e-30
    x = x.to(DEV)
    _, packed, _ = quest.hadamard_quantize_int4(x)
    _, tiles = quest.hadamard_quantize_e2m3(x)
    assert torch.equal(qo.e2m3_tiles_decode(tiles.cpu(), m, k), qo.unpack_int4(packed.cpu()).double() + .5)


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape', [(64, 4096), (33, 1024), (70, 128), (5, 2816), (40, 11008), (130, 512), (3, 32768), (4101, 2560)])
def test_no_transform_on_the_matrix_core_kernel(quest, dtype, shape):
    """hadamard_scale = 0 with rows of whole blocks of 128: the matrix-core kernel without its multiplications (the
    loaded chunks only change lanes).  The scale is the oracle's on x itself (one ulp: summation order), the codes are the
    oracle's given that scale, bit for bit, degenerate elements included, and the tiles hold the same codes."""
    m, k = shape
    x = rand_act(m, k, dtype, 31)
    if m > 4:
        x[1] = 0
        x[2, 5] = float('nan')
        x[3, 7] = float('inf')
        x[4, k - 1] = float('-inf')
    x_had = torch.empty(m, k, dtype=dtype, device=DEV)
    scale, packed, row_sum = quest.hadamard_quantize_int4(x.to(DEV), hadamard_scale=0., x_had=x_had)
    assert torch.equal(bits(x_had.cpu()), bits(x))                           # nothing was multiplied
    want_scale = qo.find_scale_int4(x)
    ok = torch.isfinite(want_scale.float()).flatten() & (want_scale.float().flatten() != 0)
    assert (bits(scale.cpu()) - bits(want_scale)).abs().flatten()[ok].max() <= 1
    want_packed = torch.empty(m, k // 2, dtype=torch.uint8)
    want_sum = torch.empty(m, 1, dtype=torch.int32)
    qo.quantize_int4(x.clone(), scale.cpu(), None, want_packed, want_sum, False)
    clean = torch.ones(m, dtype=torch.bool)
    if m > 4:
        clean[1:5] = False              # scale 0, NaN or Inf: what the codes are is this build's definition, pinned by
                                        # the unfused kernel below (and by the degenerate-row tests of the configurations)
    assert torch.equal(packed.cpu()[clean], want_packed[clean]) and torch.equal(row_sum.cpu()[clean], want_sum[clean])
    unfused = torch.empty(m, k // 2, dtype=torch.uint8, device=DEV)
    quest.quantize_int4(x.to(DEV), scale, None, unfused, None, False)
    assert torch.equal(packed, unfused)
    _, tiles = quest.hadamard_quantize_e2m3(x.to(DEV), hadamard_scale=0.)
    assert torch.equal(qo.e2m3_tiles_decode(tiles.cpu(), m, k), qo.unpack_int4(packed.cpu()).double() + .5)


@pytest.mark.parametrize('dtype', DTYPES)
def test_tiles_fall_back_without_the_matrix_core_transform(quest, dtype):
    """The weight-side factor, and no transform on rows that are not whole blocks of 128: quantised to packed codes by
    the row kernel, then converted."""
    m = 40
    for k, hs in ((384, 2. ** -3.5), (320, 0.), (64, 0.)):
        x = rand_act(m, k, dtype, 23).to(DEV)
        _, packed, _ = quest.hadamard_quantize_int4(x, hadamard_scale=hs)
        _, tiles = quest.hadamard_quantize_e2m3(x, hadamard_scale=hs)
        assert torch.equal(qo.e2m3_tiles_decode(tiles.cpu(), m, k), qo.unpack_int4(packed.cpu()).double() + .5)


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape', [(64, 1024), (33, 4096), (20, 6912), (9, 11008), (4100, 1024), (2052, 6912)])
def test_producer_kernels_write_the_same_tiles(quest, dtype, shape):
    m, k = shape
    g = torch.Generator().manual_seed(24)
    x = rand_act(m, k, dtype, 25).to(DEV)
    w = (1 + 0.1 * torch.randn(k, generator=g)).to(dtype).to(DEV)
    s0, p0, _ = quest.rmsnorm_hadamard_quantize_int4(x, w, 1e-5)
    s1, t1 = quest.rmsnorm_hadamard_quantize_e2m3(x, w, 1e-5)
    assert torch.equal(bits(s0.cpu()), bits(s1.cpu()))
    assert torch.equal(qo.e2m3_tiles_decode(t1.cpu(), m, k), qo.unpack_int4(p0.cpu()).double() + .5)
    br = rand_act(m, k, dtype, 26).to(DEV)
    xa, xb = x.clone(), x.clone()
    s0, p0, _ = quest.add_rmsnorm_hadamard_quantize_int4(xa, br, w, 1e-5)
    s1, t1 = quest.add_rmsnorm_hadamard_quantize_e2m3(xb, br, w, 1e-5)
    assert torch.equal(bits(xa.cpu()), bits(xb.cpu())) and torch.equal(bits(s0.cpu()), bits(s1.cpu()))
    assert torch.equal(qo.e2m3_tiles_decode(t1.cpu(), m, k), qo.unpack_int4(p0.cpu()).double() + .5)
    gu = rand_act(m, 2 * k, dtype, 27).to(DEV)
    s0, p0, _ = quest.silu_mul_hadamard_quantize_int4(gu)
    s1, t1 = quest.silu_mul_hadamard_quantize_e2m3(gu)
    assert torch.equal(bits(s0.cpu()), bits(s1.cpu()))
    assert torch.equal(qo.e2m3_tiles_decode(t1.cpu(), m, k), qo.unpack_int4(p0.cpu()).double() + .5)
