"""GPU parity: every HIP entry point, called through the C ABI (quest_amd.api -> ctypes ->
libquest_hip.so), against the CPU oracle on the same seeded inputs.

Bars: INT4 codes, packed bytes, row sums, int32 accumulators and the scale epilogue are bit-exact;
the Hadamard output agrees with the reference's matmul formulation to <= 1e-3 relative (and is
bit-identical to the fp32-butterfly statement of the oracle); the per-row scale may differ from a
torch-CPU reduction by one 16-bit ulp on a rare row (summation order), which is counted and bounded.
"""
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
    _lib.load()                       # fails loudly if the HIP library is not built
    assert torch.cuda.is_available()
    return quest_amd


def bits(t):
    return t.contiguous().view(torch.int16).to(torch.int32)


def ulp_diff(a, b):
    return (bits(a.cpu()) - bits(b.cpu())).abs()


def rand_act(m, k, dtype, seed, spread=True):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, k, generator=g)
    if spread:
        x = x * (torch.rand(m, 1, generator=g) * 4 + 0.05)
    return x.to(dtype)


# --------------------------------------------------------------------------- S1
@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape', [(160, 768), (37, 4096), (1, 128), (8, 11008), (3, 16384)])
def test_find_scale(quest, dtype, shape):
    x = rand_act(*shape, dtype, seed=1)
    want = qo.find_scale_int4(x)
    got = quest.find_scale_int4(x.to(DEV)).cpu()
    d = ulp_diff(got, want)
    assert d.max() <= 1, 'scale differs from the oracle by more than one ulp'
    assert (d != 0).sum() <= max(1, shape[0] // 100), f'{int((d != 0).sum())} rows differ'


@pytest.mark.parametrize('dtype', DTYPES)
def test_find_scale_constant_rows_exact(quest, dtype):
    vals = torch.tensor([0., 1., -1., 0.5, 3., -7.25, 100., 2. ** -10])
    x = vals.to(dtype)[:, None].repeat(1, 512).contiguous()
    assert torch.equal(quest.find_scale_int4(x.to(DEV)).cpu(), qo.find_scale_int4(x))


# --------------------------------------------------------------------------- S2
@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape', [(160, 768), (5, 4096), (1, 8), (16, 11008)])
def test_quantize_all_outputs_bit_exact(quest, dtype, shape):
    m, k = shape
    x = rand_act(m, k, dtype, seed=2)
    scale = qo.find_scale_int4(x)
    xi = torch.empty(m, k, dtype=torch.int8)
    xp = torch.empty(m, k // 2, dtype=torch.uint8)
    rs = torch.empty(m, 1, dtype=torch.int32)
    xd = x.clone()
    qo.quantize_int4(xd, scale, xi, xp, rs, True)
    gx = x.to(DEV)
    gi = torch.empty(m, k, dtype=torch.int8, device=DEV)
    gp = torch.empty(m, k // 2, dtype=torch.uint8, device=DEV)
    gs = torch.empty(m, 1, dtype=torch.int32, device=DEV)
    out = quest.quantize_int4(gx, scale.to(DEV), gi, gp, gs, True)
    assert out[0] is gx and out[1] is gi and out[2] is gp and out[3] is gs
    assert torch.equal(gi.cpu(), xi)
    assert torch.equal(gp.cpu(), xp)
    assert torch.equal(gs.cpu(), rs)
    assert torch.equal(bits(gx.cpu()), bits(xd))
    # optional outputs left out: x untouched, only what was asked for is written
    gx2 = x.to(DEV)
    gp2 = torch.zeros_like(gp)
    r = quest.quantize_int4(gx2, scale.to(DEV), None, gp2, None, False)
    assert r[1] is None and r[3] is None
    assert torch.equal(gp2.cpu(), xp) and torch.equal(bits(gx2.cpu()), bits(x))


@pytest.mark.parametrize('dtype', DTYPES)
def test_quantize_every_16bit_input(quest, dtype):
    """All 65536 bit patterns as inputs (NaN/Inf rows aside) against a spread of scales."""
    allbits = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16).view(dtype)
    finite = torch.isfinite(allbits.float())
    vals = torch.where(finite, allbits, torch.zeros_like(allbits))
    g = torch.Generator().manual_seed(13)
    scales = torch.cat([torch.tensor([0.3351907, 1.0, 0.007, 3.1, 2. ** -9, 0.0625, 117.0, 0.99, 0.4062, 5e-4,
                                      0.1234, 0.0101, 12.5, 0.75, 1.5, 2.25]),
                        torch.exp(torch.rand(240, generator=g) * 12 - 8)]).to(dtype).view(-1, 1)
    x = vals.view(1, -1).repeat(scales.numel(), 1).contiguous()
    xi = torch.empty(x.shape, dtype=torch.int8)
    rs = torch.empty(x.size(0), 1, dtype=torch.int32)
    qo.quantize_int4(x.clone(), scales, xi, None, rs, False)
    gi = torch.empty(x.shape, dtype=torch.int8, device=DEV)
    gs = torch.empty(x.size(0), 1, dtype=torch.int32, device=DEV)
    quest.quantize_int4(x.to(DEV), scales.to(DEV), gi, None, gs, False)
    assert torch.equal(gi.cpu(), xi)
    assert torch.equal(gs.cpu(), rs)


# --------------------------------------------------------------------------- E1
@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape', [(160, 224), (1, 1), (7, 513), (33, 4096), (300, 2056), (5, 8)])
def test_add_mul_vv(quest, dtype, shape):
    m, n = shape
    g = torch.Generator().manual_seed(3)
    c = torch.randint(-200000, 200000, (m, n), generator=g, dtype=torch.int32)
    a_add = torch.randint(-30000, 30000, (m, 1), generator=g, dtype=torch.int32)
    b_add = torch.randint(-30000, 30000, (n, 1), generator=g, dtype=torch.int32)
    a_mul = (torch.rand(m, 1, generator=g) * 0.09 + 0.01).to(dtype)
    b_mul = (torch.rand(n, 1, generator=g) * 0.09 + 0.01).to(dtype)
    want = qo.add_mul_vv(a_add, a_mul, b_add, b_mul, c)
    got = quest.add_mul_vv(a_add.to(DEV), a_mul.to(DEV), b_add.to(DEV), b_mul.to(DEV), c.to(DEV)).cpu()
    assert torch.equal(bits(got), bits(want))


def test_add_mul_vv_vectors_at_odd_offsets(quest):
    """Rows of whole eights take 16-byte vector accesses; channel vectors that start at an odd element must not."""
    m, n = 37, 264
    g = torch.Generator().manual_seed(4)
    c = torch.randint(-200000, 200000, (m, n), generator=g, dtype=torch.int32)
    a_add = torch.randint(-30000, 30000, (m, 1), generator=g, dtype=torch.int32)
    b_add = torch.randint(-30000, 30000, (n + 1, 1), generator=g, dtype=torch.int32)
    a_mul = (torch.rand(m, 1, generator=g) * 0.09 + 0.01).to(torch.float16)
    b_mul = (torch.rand(n + 1, 1, generator=g) * 0.09 + 0.01).to(torch.float16)
    want = qo.add_mul_vv(a_add, a_mul, b_add[1:], b_mul[1:], c)
    got = quest.add_mul_vv(a_add.to(DEV), a_mul.to(DEV), b_add.to(DEV)[1:], b_mul.to(DEV)[1:], c.to(DEV)).cpu()
    assert torch.equal(bits(got), bits(want))


# --------------------------------------------------------------------------- G1 / G2
def rand_codes(rows, k, seed):
    g = torch.Generator().manual_seed(seed)
    return qo.pack_int4(torch.randint(-8, 8, (rows, k), generator=g).to(torch.int8))


GEMM_SHAPES = [(160, 768, 224), (1, 4096, 4096), (8, 256, 33), (16, 11008, 512), (257, 128, 300),
               (33, 96, 7), (512, 1024, 1024), (300, 160, 257), (256, 2048, 256),
               # a handful of tokens (the weight-streaming kernel): 64-byte row tails, ragged N, each token-tile count
               (3, 384, 18), (16, 128, 16), (17, 1152, 64), (32, 640, 100), (40, 2304, 47), (64, 8192, 32), (5, 28672, 24),
               (12, 160, 40), (65, 256, 48), (100, 1152, 300), (128, 4096, 512), (127, 384, 33),
               # ... 8 to 16 tokens on wide layers: ragged channel counts, the 64-byte row tail
               (16, 256, 8200), (8, 1152, 11008), (13, 128, 8209), (9, 384, 8193), (7, 256, 8200), (16, 256, 8191),
               # enough cells for the two-workgroups-per-CU shape of the large-tile kernel (>= 256 cells of 256 tokens x
               # 32 channels per XCD group): few channels with a ragged last token tile; short K with a channel count
               # that takes the element-wise epilogue
               (16390, 256, 1000), (4096, 128, 4100),
               # the same with fewer than eight channel units (one scheduling group instead of one per XCD)
               (65538, 128, 96),
               # a few hundred tokens with K % 256 == 0 (the small-tile kernel): ragged token and channel tiles, channel
               # counts that take the element-wise epilogue, one and several tiles per CU, a single 256-k stage
               (127, 512, 33), (130, 256, 1000), (448, 768, 4100), (70, 1024, 4097), (1000, 512, 2048), (66, 4096, 8),
               (640, 2816, 1024),
               # ... and a few tens of tokens with thousands of channels
               (40, 256, 8200), (64, 512, 11008), (17, 256, 11010), (33, 256, 8192), (48, 512, 4610), (64, 256, 4096),
               # four 64 x 64 tiles per CU = one round of 128 x 128 tiles (ragged in both directions); one tile per
               # workgroup of the large-tile kernel, cut along single token tiles
               (1000, 512, 4090), (1536, 256, 4096), (768, 128, 8200), (1300, 384, 4100),
               # odd token and channel counts in the large-tile kernel (the 16-bit scale vectors end with half a dword)
               (301, 384, 512), (1001, 128, 96), (4097, 128, 1031), (777, 1152, 4100),
               # the same token counts with K % 256 != 0 (large tiles one or two channel units wide)
               (200, 384, 512), (300, 640, 1000)]


@pytest.mark.parametrize('shape', GEMM_SHAPES)
def test_matmul_int32_bit_exact(quest, shape):
    m, k, n = shape
    a, b = rand_codes(m, k, 4), rand_codes(n, k, 5)
    want = qo.matmul_int4_int4t_int32(a, b, via='fp32')
    got = quest.matmul_int4_int4t_int32(a.to(DEV), b.to(DEV)).cpu()
    assert torch.equal(got, want)


def test_matmul_int32_extreme_codes(quest):
    # every product is (-8)(-8) = +64: the largest accumulator the path can see
    m, k, n = 64, 4096, 96
    a = torch.full((m, k // 2), 0x88, dtype=torch.uint8)
    b = torch.full((n, k // 2), 0x88, dtype=torch.uint8)
    got = quest.matmul_int4_int4t_int32(a.to(DEV), b.to(DEV)).cpu()
    assert (got == 64 * k).all()
    b[:] = 0x77                        # (-8)(7) = -56
    got = quest.matmul_int4_int4t_int32(a.to(DEV), b.to(DEV)).cpu()
    assert (got == -56 * k).all()


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape', [(160, 768, 224), (16, 4096, 4096), (1, 11008, 4096), (257, 256, 301),
                                   (8, 4096, 11008), (3, 384, 18), (33, 1152, 62), (64, 640, 100), (20, 2304, 47),
                                   (65, 256, 48), (100, 1152, 300), (128, 4096, 512),
                                   (16390, 256, 1000), (4096, 128, 4100),
                                   # one or two pipeline stages per tile: the epilogue must wait for its scale vectors itself
                                   (4096, 256, 2048), (16384, 128, 2048),
                                   # a few hundred tokens, K % 256 == 0 (small tiles): ragged tiles, vector and element-wise stores
                                   (127, 512, 33), (130, 256, 1000), (448, 768, 4100), (70, 1024, 4097), (1000, 512, 2048),
                                   (66, 4096, 8), (640, 2816, 1024), (40, 256, 8200), (64, 512, 11008), (17, 256, 11010), (48, 512, 4610),
                                   (1000, 512, 4090), (1536, 256, 4096), (768, 128, 8200), (1300, 384, 4100),
                                   # odd token and channel counts in the large-tile kernel
                                   (301, 384, 512), (1001, 128, 96), (4097, 128, 1031), (777, 1152, 4100),
                                   # ... and K % 256 != 0 (narrow large tiles)
                                   (200, 384, 512), (300, 640, 1000)])
def test_fused_matmul_dequantize_bit_exact(quest, dtype, shape):
    m, k, n = shape
    g = torch.Generator().manual_seed(6)
    a, b = rand_codes(m, k, 7), rand_codes(n, k, 8)
    a_mul = (torch.rand(m, 1, generator=g) * 0.09 + 0.01).to(dtype)
    b_mul = (torch.rand(n, 1, generator=g) * 0.09 + 0.01).to(dtype)
    a_add = qo.unpack_int4(a).to(torch.int32).sum(-1, keepdim=True).to(torch.int32)
    b_add = qo.unpack_int4(b).to(torch.int32).sum(-1, keepdim=True).to(torch.int32) + k // 2
    want = qo.fused_matmul_dequantize_int4_int4t(a, b, a_add, b_add, a_mul, b_mul, via='fp32')
    got = quest.fused_matmul_dequantize_int4_int4t_bf16(
        a.to(DEV), b.to(DEV), a_add.to(DEV), b_add.to(DEV), a_mul.to(DEV), b_mul.to(DEV)).cpu()
    assert got.dtype == dtype
    assert torch.equal(bits(got), bits(want))
    # <= 1e-2 relative against the fp64 value of the dequantised product (the north star's bar)
    ref = qo.linear_fp64(qo.unpack_int4(a), a_mul, qo.unpack_int4(b), b_mul)
    assert ((got.double() - ref).norm() / ref.norm()) < 1e-2


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape', [(160, 768, 224), (66, 128, 8), (200, 256, 512), (300, 256, 1000), (16390, 256, 1000),
                                   (16384, 128, 2048), (4096, 128, 4104), (200, 384, 512), (130, 1024, 4104),
                                   (66, 4096, 8), (1000, 512, 2048), (1000, 512, 4088), (1536, 256, 4096), (768, 128, 8200),
                                   (201, 384, 512), (4099, 128, 1032)])
def test_fused_matmul_dequantize_swiglu(quest, dtype, shape):
    """The gate/up GEMM with silu(gate) * up in its epilogue = the plain fused GEMM on the same (interleaved) weight
    rows followed by the activation kernel's own SwiGLU, bit for bit; and within 2 ulp of torch's CPU expression on the
    plain GEMM's (bit-exact) output."""
    m, k, n = shape                                            # n = 2 H weight rows
    h = n // 2
    g = torch.Generator().manual_seed(30)
    a, b = rand_codes(m, k, 31), rand_codes(n, k, 32)          # b: gate rows 0..H-1, up rows H..2H-1
    a_mul = (torch.rand(m, 1, generator=g) * 0.05 + 0.01).to(dtype)
    b_mul = (torch.rand(n, 1, generator=g) * 0.05 + 0.01).to(dtype)
    a_add = torch.randint(-200, 200, (m, 1), generator=g, dtype=torch.int32)
    b_add = torch.randint(-200, 200, (n, 1), generator=g, dtype=torch.int32)
    ga, gb, ga_add, gb_add, ga_mul, gb_mul = (t.to(DEV) for t in (a, b, a_add, b_add, a_mul, b_mul))
    p = quest.swiglu_interleave_rows(h, device=DEV)
    assert sorted(p.tolist()) == list(range(n)) and p[:8].tolist() == [0, 1, 2, 3, h, h + 1, h + 2, h + 3]
    got = quest.fused_matmul_dequantize_swiglu_int4_int4t(ga, gb[p].contiguous(), ga_add, gb_add[p].contiguous(), ga_mul,
                                                          gb_mul[p].contiguous())
    assert got.shape == (m, h)
    gate_up = quest.fused_matmul_dequantize_int4_int4t_bf16(ga, gb, ga_add, gb_add, ga_mul, gb_mul)     # (M, 2H), halves
    if h % 128 == 0 and h <= 4096:
        act = torch.empty(m, h, dtype=dtype, device=DEV)
        quest.silu_mul_hadamard_quantize_int4(gate_up, x_act=act)
        assert torch.equal(bits(got.cpu()), bits(act.cpu()))
    cpu = gate_up.cpu()
    want = torch.nn.functional.silu(cpu[:, :h]) * cpu[:, h:]
    worst, frac = _ulp_stats(got.cpu(), want)
    assert worst <= 2 and frac < 0.02, (worst, frac)


def test_swiglu_gemm_refuses_small_batches(quest):
    m, k, n = 16, 256, 64
    a, b = rand_codes(m, k, 33).to(DEV), rand_codes(n, k, 34).to(DEV)
    z = torch.zeros(m, 1, dtype=torch.int32, device=DEV)
    zn = torch.zeros(n, 1, dtype=torch.int32, device=DEV)
    with pytest.raises(RuntimeError):
        quest.fused_matmul_dequantize_swiglu_int4_int4t(a, b, z, zn, torch.ones(m, 1, dtype=torch.bfloat16, device=DEV),
                                                        torch.ones(n, 1, dtype=torch.bfloat16, device=DEV))


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape', [(300, 384, 1000), (16384, 128, 1024), (4096, 1024, 3072), (165, 128, 392), (256, 128, 64),
                                   (1000, 128, 4100), (2048, 2560, 2560), (4099, 128, 1031), (48, 256, 128), (256, 256, 192),
                                   (80, 160, 64)])
def test_fused_matmul_dequantize_adds_into_the_residual_stream(quest, dtype, shape):
    """out <- dtype(out + dtype(product)) on packed codes: the bits of torch's `out + product`, in the large-tile kernel's
    epilogue (both its shapes, narrow tiles, edge tiles, a channel count that is not a multiple of 8, large and tiny
    residuals, twice on one buffer) and as two launches where another kernel takes the size -- which
    `gemm_add_fuses` tells beforehand."""
    m, k, n = shape
    g = torch.Generator().manual_seed(47)
    a, b = rand_codes(m, k, 48).to(DEV), rand_codes(n, k, 49).to(DEV)
    a_mul = (torch.rand(m, 1, generator=g) * 0.05 + 0.01).to(dtype).to(DEV)
    b_mul = (torch.rand(n, 1, generator=g) * 0.05 + 0.01).to(dtype).to(DEV)
    a_add = torch.randint(-200, 200, (m, 1), generator=g, dtype=torch.int32).to(DEV)
    b_add = torch.randint(-200, 200, (n, 1), generator=g, dtype=torch.int32).to(DEV)
    product = quest.fused_matmul_dequantize_int4_int4t_bf16(a, b, a_add, b_add, a_mul, b_mul)
    res = (torch.randn(m, n, generator=g) * torch.rand(m, 1, generator=g) * 50).to(dtype)
    res[0] *= 1e-4
    res = res.to(DEV)
    want = res + product
    got = res.clone()
    ret = quest.fused_matmul_dequantize_add_int4_int4t(a, b, a_add, b_add, a_mul, b_mul, got)
    assert ret.data_ptr() == got.data_ptr()
    assert torch.equal(bits(got.cpu()), bits(want.cpu()))
    quest.fused_matmul_dequantize_add_int4_int4t(a, b, a_add, b_add, a_mul, b_mul, got)
    assert torch.equal(bits(got.cpu()), bits((want + product).cpu()))
    from quest_amd import _lib
    rc = _lib.load().quest_fused_matmul_dequantize_add_int4_int4t(
        got.data_ptr(), a.data_ptr(), b.data_ptr(), a_add.data_ptr(), b_add.data_ptr(), a_mul.data_ptr(), b_mul.data_ptr(),
        m, k, n, 0 if dtype == torch.bfloat16 else 1, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert (rc == 0) == quest.gemm_add_fuses(m, k, n) and rc in (0, -5)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    small = k % 256 == 0 and (-(-(-(-m // 64) * -(-n // 64)) // cus) <= 4 or (-(-(-(-m // 64) * -(-n // 64)) // cus) <= 8 and m < 1024 and m % 256))
    assert quest.gemm_add_fuses(m, k, n) == (_tiled_kernel_takes(m, k, n) and not small)


def _tiled_kernel_takes(m, k, n):
    """The dispatch of the fused GEMM (gemm.hip), restated: whether the large-tile or the small-tile kernel gets this size
    (the two with the rotary epilogue) rather than the weight-streaming or the register-staged one."""
    return k % 128 == 0 and m > 64 and not (m <= 128 and n <= 8192)


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape', [
    # batch, sequence, K, heads, head_dim, channels after q and k
    (2, 150, 384, 3, 32, 96), (32, 512, 128, 8, 64, 0), (32, 512, 128, 4, 64, 256), (3, 100, 384, 5, 96, 480),
    (8, 512, 1024, 16, 64, 1024), (5, 33, 128, 1, 128, 136), (4, 64, 128, 1, 32, 0), (1, 48, 256, 2, 64, 128),
    (2, 128, 256, 2, 32, 64), (2, 40, 160, 2, 32, 64), (1, 512, 2560, 20, 128, 2560), (3, 100, 512, 4, 64, 264),
    (4, 512, 256, 16, 128, 2048)])
def test_fused_matmul_dequantize_rope(quest, dtype, shape):
    """The QKV projection whose q and k leave the GEMM rotated = the plain fused GEMM followed by the rotary kernel, bit
    for bit: both shapes of the large-tile kernel, tiles of one or two channel units, both small-tile shapes, edge tiles,
    positions wrapping at every sequence -- and the sizes that another kernel takes (a handful of tokens, K % 128 != 0),
    where the call is the two launches."""
    bsz, t, k, heads, hd, rest = shape
    m, c = bsz * t, heads * hd
    n = 2 * c + rest
    g = torch.Generator().manual_seed(44)
    a, b = rand_codes(m, k, 45).to(DEV), rand_codes(n, k, 46).to(DEV)
    a_mul = (torch.rand(m, 1, generator=g) * 0.05 + 0.01).to(dtype).to(DEV)
    b_mul = (torch.rand(n, 1, generator=g) * 0.05 + 0.01).to(dtype).to(DEV)
    a_add = torch.randint(-200, 200, (m, 1), generator=g, dtype=torch.int32).to(DEV)
    b_add = torch.randint(-200, 200, (n, 1), generator=g, dtype=torch.int32).to(DEV)
    ang = torch.rand(t, hd // 2, generator=g) * 6.283
    freqs = torch.stack([torch.cos(ang), torch.sin(ang)], dim=-1).contiguous().to(DEV)
    plain = quest.fused_matmul_dequantize_int4_int4t_bf16(a, b, a_add, b_add, a_mul, b_mul)
    want = plain.clone()
    quest.rope_interleaved_(want.view(bsz, t, n), freqs, 2 * c, hd)
    got = quest.fused_matmul_dequantize_rope_int4_int4t(a, b, a_add, b_add, a_mul, b_mul, freqs, 2 * c, hd)
    assert torch.equal(bits(got.cpu()), bits(want.cpu()))
    assert not torch.equal(bits(got[:, :2 * c].cpu()), bits(plain[:, :2 * c].cpu()))
    from quest_amd import _lib
    rc = _lib.load().quest_fused_matmul_dequantize_rope_int4_int4t(
        got.data_ptr(), a.data_ptr(), b.data_ptr(), a_add.data_ptr(), b_add.data_ptr(), a_mul.data_ptr(), b_mul.data_ptr(),
        m, k, n, 0 if dtype == torch.bfloat16 else 1, freqs.data_ptr(), t, 2 * c, hd, torch.cuda.current_stream().cuda_stream)
    assert rc == (0 if _tiled_kernel_takes(m, k, n) else -5), rc
    torch.cuda.synchronize()


# --------------------------------------------------------------------------- H1 / H2
@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('scale', [181. / 2048., 2. ** -3.5])
def test_hadamard128(quest, dtype, scale):
    x = rand_act(48, 1024, dtype, seed=9)
    got = quest.hadamard128(x.to(DEV), scale=scale).cpu()
    assert torch.equal(bits(got), bits(qo.hadamard128_fwht(x, scale)))      # same butterfly order
    if scale == 181. / 2048.:
        ref = qo.hadamard128_matmul(x)                                       # the reference's F.linear form
        assert ((got.double() - ref.double()).norm() / ref.double().norm()) < 1e-3
        # element-wise: the two summation orders differ by fp32 noise, i.e. at most one 16-bit ulp of
        # the row's largest output (cancelled-out small outputs may be several of their own ulps apart)
        tol = ref.double().abs().amax(-1, keepdim=True) * 2. ** -8
        assert ((got.double() - ref.double()).abs() <= tol).all()
    # in place
    gx = x.to(DEV)
    quest.hadamard128(gx, out=gx, scale=scale)
    assert torch.equal(bits(gx.cpu()), bits(got))


# --------------------------------------------------------------------------- fused activation kernel
@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape', [(160, 768), (64, 4096), (1, 128), (8, 11008), (16, 2816), (2, 16384), (2, 32768),
                                   (3, 1024), (777, 4096), (5, 3968), (3, 5120), (6, 8192), (2, 28672), (2, 65536),
                                   (50, 256), (50, 512), (37, 2048), (130, 1024), (70, 128)])
def test_hadamard_quantize_fused(quest, dtype, shape):
    """Rows of up to 32768 run the Hadamard on the matrix cores (the reference's matmul formulation, fp32
    accumulation in the hardware's order; rows over 4096 are shared by the waves of a workgroup), longer
    rows run fp32 butterflies."""
    m, k = shape
    x = rand_act(m, k, dtype, seed=10)
    gx = x.to(DEV)
    x_had = torch.empty_like(gx)
    scale, packed, row_sum = quest.hadamard_quantize_int4(gx, x_had=x_had)
    assert torch.equal(bits(gx.cpu()), bits(x)), 'input must not be written'
    had = x_had.cpu()
    # (1) Hadamard: <= 1e-3 relative from the reference's matmul formulation and from the fp32-butterfly oracle,
    # element-wise within one 16-bit ulp of the row's largest output
    for ref in (qo.hadamard128_matmul(x), qo.hadamard128_fwht(x, 181. / 2048.)):
        assert ((had.double() - ref.double()).norm() / ref.double().norm()) < 1e-3
        tol = ref.double().abs().amax(-1, keepdim=True) * 2. ** -8
        assert ((had.double() - ref.double()).abs() <= tol).all()
    if k > 32768:
        assert torch.equal(bits(had), bits(qo.hadamard128_fwht(x, 181. / 2048.)))      # butterfly kernel: same order, same bits
    # (2) scale on the kernel's own transformed tensor: within one ulp of the oracle, rarely different
    want_scale = qo.find_scale_int4(had)
    d = ulp_diff(scale, want_scale)
    assert d.max() <= 1 and (d != 0).sum() <= max(1, m // 100)
    # (3) codes and row sums: bit-exact given the same transformed input and the same scale
    xp = torch.empty(m, k // 2, dtype=torch.uint8)
    rs = torch.empty(m, 1, dtype=torch.int32)
    qo.quantize_int4(had.clone(), scale.cpu(), None, xp, rs, False)
    assert torch.equal(packed.cpu(), xp)
    assert torch.equal(row_sum.cpu(), rs)
    # (4) the unfused kernels on that tensor give the same codes (and the same scale up to the reduction order)
    s2 = quest.find_scale_int4(x_had)
    assert ulp_diff(s2, scale).max() <= 1
    p2 = torch.empty_like(packed)
    r2 = torch.empty_like(row_sum)
    quest.quantize_int4(x_had.clone(), scale, None, p2, r2, False)
    assert torch.equal(p2, packed) and torch.equal(r2, row_sum)
    # (5) outputs that are not asked for are not needed: scale only, and codes without the debug tensor
    s3, p3, r3 = quest.hadamard_quantize_int4(gx)
    assert torch.equal(bits(s3.cpu()), bits(scale.cpu())) and torch.equal(p3, packed) and torch.equal(r3, row_sum)


@pytest.mark.parametrize('dtype', DTYPES)
def test_hadamard_quantize_weight_scale_runs_butterflies(quest, dtype):
    """2^-3.5 (the weight-side factor) is not a 16-bit float, so the fused kernel keeps fp32 butterflies and an
    fp32 factor: same bits as the butterfly oracle, and the fused codes equal the composition of the steps."""
    w = rand_act(96, 2048, dtype, seed=13)
    gw = w.to(DEV)
    w_had = torch.empty_like(gw)
    scale, packed, row_sum = quest.hadamard_quantize_int4(gw, x_had=w_had, hadamard_scale=2. ** -3.5)
    want_had = qo.hadamard128_fwht(w, 2. ** -3.5)
    assert torch.equal(bits(w_had.cpu()), bits(want_had))
    assert ulp_diff(scale, qo.find_scale_int4(want_had)).max() <= 1
    xp = torch.empty(96, 1024, dtype=torch.uint8)
    rs = torch.empty(96, 1, dtype=torch.int32)
    qo.quantize_int4(want_had.clone(), scale.cpu(), None, xp, rs, False)
    assert torch.equal(packed.cpu(), xp) and torch.equal(row_sum.cpu(), rs)


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('use_hadamard', [False, True])
def test_preprocess_weight_absmax_bit_exact(quest, dtype, use_hadamard):
    """The absmax scale rule: a maximum has no summation order, so scale, codes and sums all match bit for bit."""
    from quest_amd import harness
    w = (torch.randn(200, 1152, generator=torch.Generator().manual_seed(14)) * 0.02).to(dtype)
    wp, ws, wa, _ = harness.preprocess_weight(w.to(DEV), use_hadamard=use_hadamard, w_scale_mode='absmax')
    op, os_, oa, _ = qo.preprocess_weight(w, use_hadamard=use_hadamard, w_scale_mode='absmax')
    assert torch.equal(bits(ws.cpu()), bits(os_))
    assert torch.equal(wp.cpu(), op) and torch.equal(wa.cpu(), oa)
    # and the reference's rule through the same entry point is unchanged
    wp2, ws2, wa2, _ = harness.preprocess_weight(w.to(DEV), use_hadamard=use_hadamard)
    op2, os2, oa2, _ = qo.preprocess_weight(w, use_hadamard=use_hadamard)
    assert ulp_diff(ws2, os2).max() <= 1
    if torch.equal(bits(ws2.cpu()), bits(os2)):
        assert torch.equal(wp2.cpu(), op2) and torch.equal(wa2.cpu(), oa2)


@pytest.mark.parametrize('dtype', DTYPES)
def test_packed_linear_against_training_side_fake_quant(quest, dtype):
    """The layer a QuEST-trained checkpoint was evaluated with (fake quantisation in fp32, src/eval_hswag.py of the
    reference) against the packed INT4 layer built from the same dense weight.  The inference path rounds the rotated
    activations to 16 bits before quantising (benchmarks/utils.py:89-90), which moves a per cent or two of the codes
    to the neighbouring level: measured 3.4e-2 relative in bf16 and 1.2e-2 in fp16, for this kernel and for the
    CPU oracle of the reference's inference path alike -- the distance belongs to the path, not to the kernel."""
    from quest_amd import harness
    g = torch.Generator().manual_seed(40)
    x = torch.randn(192, 1024, generator=g).to(dtype)
    w = (torch.randn(320, 1024, generator=g) * 0.02).to(dtype)
    want = qo.fake_quant_linear(x, w).double()
    layer = harness.Linear4bit.from_weight(w.to(DEV), use_hadamard=True)
    got = layer(x.to(DEV)).double().cpu()
    wp, ws, wa, _ = qo.preprocess_weight(w, use_hadamard=True)
    ref = qo.linear_forward(x, wp, ws, wa, use_hadamard=True, hadamard='matmul', via='fp32').double()
    err = (got - want).norm() / want.norm()
    err_ref = (ref - want).norm() / want.norm()
    assert err < (5e-2 if dtype == torch.bfloat16 else 2e-2), float(err)
    assert err < 1.25 * err_ref + 1e-3, (float(err), float(err_ref))


@pytest.mark.parametrize('dtype', DTYPES)
def test_packed_linear_quantised_from_fp32_meets_the_fake_quant_bar(quest, dtype, capsys):
    """With `quantize_from_fp32` weights and activations are quantised from the fp32 transform (factor 2^-3.5) and the
    unrounded scale -- the arithmetic of the evaluation-side fake quantiser (src/eval_hswag.py:201-214) -- and the packed
    layer agrees with the fake-quantised one to <= 1e-2 relative; what is left is the 16-bit rounding of the stored
    scales and of the output."""
    from quest_amd import harness
    g = torch.Generator().manual_seed(40)
    x = torch.randn(192, 1024, generator=g).to(dtype)
    w = (torch.randn(320, 1024, generator=g) * 0.02).to(dtype)
    want = qo.fake_quant_linear(x, w).double()
    layer = harness.Linear4bit.from_weight(w.to(DEV), use_hadamard=True, quantize_from_fp32=True)
    got = layer(x.to(DEV)).double().cpu()
    plain = harness.Linear4bit.from_weight(w.to(DEV), use_hadamard=True)(x.to(DEV)).double().cpu()
    err = float((got - want).norm() / want.norm())
    err_plain = float((plain - want).norm() / want.norm())
    # the codes themselves: the fake quantiser's levels 0..15 are the codes + 8
    wq, _, _ = qo.fake_quant_hadamard(w)
    codes = qo.unpack_int4(layer.w_int_packed.cpu()).to(torch.float32) + 8
    differ = float((codes != wq).float().mean())
    with capsys.disabled():
        print(f'\n[fake-quant bar, {dtype}] from fp32: {err:.2e} (weight codes differing {differ:.2e}); default path: {err_plain:.2e}')
    assert err <= 1e-2, err
    assert differ < 1e-3, differ


# --------------------------------------------------------------------------- producers fused in front
def _ulp_stats(got, want):
    d = ulp_diff(got, want)
    return int(d.max()), float((d != 0).float().mean())


PRODUCER_SHAPES = [(160, 1024), (33, 2816), (5, 128), (64, 4096), (7, 256), (9, 512), (12, 2048), (300, 768),
                   # rows over 4096 (several waves per row): the 1600M model's and Llama-7B's MLP widths among them
                   (40, 5120), (33, 6912), (17, 8192), (20, 11008), (3, 32768)]


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape', PRODUCER_SHAPES)
def test_rmsnorm_hadamard_quantize(quest, dtype, shape):
    """RMSNorm in front of the fused kernel.  The normalised tensor agrees with torch's CPU RMSNorm up to the last
    bit of a few elements (fp32 reduction order and rsqrt), and from that tensor on the kernel is the plain fused
    kernel bit for bit."""
    from oracle import llama_oracle as lo
    m, k = shape
    x = rand_act(m, k, dtype, seed=20)
    w = (1 + 0.1 * torch.randn(k, generator=torch.Generator().manual_seed(21))).to(dtype)
    gx, gw = x.to(DEV), w.to(DEV)
    x_norm = torch.empty_like(gx)
    x_had = torch.empty_like(gx)
    scale, packed, row_sum = quest.rmsnorm_hadamard_quantize_int4(gx, gw, 1e-5, x_had=x_had, x_norm=x_norm)
    assert torch.equal(bits(gx.cpu()), bits(x)), 'input must not be written'
    worst, frac = _ulp_stats(x_norm.cpu(), lo.rmsnorm(x, w, 1e-5))
    assert worst <= 2 and frac < 0.02, (worst, frac)
    had2 = torch.empty_like(gx)
    s2, p2, r2 = quest.hadamard_quantize_int4(x_norm, x_had=had2)
    assert torch.equal(bits(x_had.cpu()), bits(had2.cpu()))
    assert torch.equal(bits(scale.cpu()), bits(s2.cpu())) and torch.equal(packed, p2) and torch.equal(row_sum, r2)
    # outputs that are not asked for
    s3, p3, r3 = quest.rmsnorm_hadamard_quantize_int4(gx, gw, 1e-5)
    assert torch.equal(bits(s3.cpu()), bits(scale.cpu())) and torch.equal(p3, packed) and torch.equal(r3, row_sum)


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape', PRODUCER_SHAPES)
def test_add_rmsnorm_hadamard_quantize(quest, dtype, shape):
    """The residual addition in front of the norm: x becomes dtype(x + branch) -- bit for bit the sum torch's CPU
    addition gives, the oracle's `x + ...` (llama_oracle.forward) -- and everything else is the norm kernel on that
    sum, bit for bit."""
    m, k = shape
    x = rand_act(m, k, dtype, seed=22)
    branch = rand_act(m, k, dtype, seed=23)
    w = (1 + 0.1 * torch.randn(k, generator=torch.Generator().manual_seed(24))).to(dtype)
    want_sum = x + branch                                   # CPU: fp32 sum, one rounding
    gx, gb, gw = x.to(DEV), branch.to(DEV), w.to(DEV)
    scale, packed, row_sum = quest.add_rmsnorm_hadamard_quantize_int4(gx, gb, gw, 1e-5)
    assert torch.equal(bits(gx.cpu()), bits(want_sum)), 'x must hold the rounded sum'
    assert torch.equal(bits(gb.cpu()), bits(branch)), 'the branch must not be written'
    s2, p2, r2 = quest.rmsnorm_hadamard_quantize_int4(want_sum.to(DEV), gw, 1e-5)
    assert torch.equal(bits(scale.cpu()), bits(s2.cpu())) and torch.equal(packed, p2) and torch.equal(row_sum, r2)


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape', PRODUCER_SHAPES)
def test_silu_mul_hadamard_quantize(quest, dtype, shape):
    """SwiGLU product in front of the fused kernel, against torch's CPU silu(gate) * up."""
    m, k = shape
    gu = rand_act(m, 2 * k, dtype, seed=22)
    want = torch.nn.functional.silu(gu[:, :k]) * gu[:, k:]
    ggu = gu.to(DEV)
    x_act = torch.empty(m, k, dtype=dtype, device=DEV)
    x_had = torch.empty_like(x_act)
    scale, packed, row_sum = quest.silu_mul_hadamard_quantize_int4(ggu, x_had=x_had, x_act=x_act)
    assert torch.equal(bits(ggu.cpu()), bits(gu)), 'input must not be written'
    worst, frac = _ulp_stats(x_act.cpu(), want)
    assert worst <= 2 and frac < 0.02, (worst, frac)
    had2 = torch.empty_like(x_act)
    s2, p2, r2 = quest.hadamard_quantize_int4(x_act, x_had=had2)
    assert torch.equal(bits(x_had.cpu()), bits(had2.cpu()))
    assert torch.equal(bits(scale.cpu()), bits(s2.cpu())) and torch.equal(packed, p2) and torch.equal(row_sum, r2)


def test_producers_refuse_rows_over_32768(quest):
    k = 32768 + 128
    x = torch.zeros(2, k, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError):
        quest.rmsnorm_hadamard_quantize_int4(x, torch.ones(k, dtype=torch.bfloat16, device=DEV), 1e-5)
    with pytest.raises(RuntimeError):
        quest.silu_mul_hadamard_quantize_int4(torch.zeros(2, 2 * k, dtype=torch.bfloat16, device=DEV))


def test_llama7b_down_proj_producer(quest):
    """M = 4096, K = 11008 (the SwiGLU product in front of Llama-7B's down projection): the fused producer equals the
    producer's own output run through the plain activation kernel, bit for bit."""
    m, k = 4096, 11008
    g = torch.Generator(device=DEV).manual_seed(7)
    gu = torch.randn(m, 2 * k, generator=g, device=DEV, dtype=torch.float32).to(torch.bfloat16)
    x_act = torch.empty(m, k, dtype=torch.bfloat16, device=DEV)
    scale, packed, row_sum = quest.silu_mul_hadamard_quantize_int4(gu, x_act=x_act)
    s2, p2, r2 = quest.hadamard_quantize_int4(x_act)
    assert torch.equal(scale.view(torch.int16), s2.view(torch.int16)) and torch.equal(packed, p2) and torch.equal(row_sum, r2)


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape', [(2, 48, 4, 64), (3, 17, 2, 32), (1, 512, 16, 64), (2, 5, 1, 8)])
def test_rope_in_place_bit_exact(quest, dtype, shape):
    """q and k rotated inside a fused QKV tensor, against the reference's formulation on the CPU; v untouched."""
    from oracle import llama_oracle as lo
    b, t, nh, hs = shape
    d = nh * hs
    g = torch.Generator().manual_seed(30)
    qkv = torch.randn(b, t, 3 * d, generator=g).to(dtype)
    fc = lo.precompute_freqs_cis(hs, t)
    q, k, v = qkv.split(d, dim=2)
    want_q, want_k = lo.apply_rotary_emb(q.reshape(b, t, nh, hs), k.reshape(b, t, nh, hs), fc)
    got = quest.rope_interleaved_(qkv.to(DEV), fc.to(DEV), 2 * d, hs).cpu()
    gq, gk, gv = got.split(d, dim=2)
    assert torch.equal(bits(gq.reshape(b, t, nh, hs)), bits(want_q))
    assert torch.equal(bits(gk.reshape(b, t, nh, hs)), bits(want_k))
    assert torch.equal(bits(gv.contiguous()), bits(v.contiguous()))


def test_hadamard_quantize_is_deterministic(quest):
    x = rand_act(512, 4096, torch.bfloat16, seed=12).to(DEV)
    a = quest.hadamard_quantize_int4(x)
    b = quest.hadamard_quantize_int4(x)
    assert all(torch.equal(u, v) for u, v in zip(a, b))


@pytest.mark.parametrize('dtype', DTYPES)
def test_hadamard_quantize_without_hadamard(quest, dtype):
    x = rand_act(40, 1024, dtype, seed=11)
    scale, packed, row_sum = quest.hadamard_quantize_int4(x.to(DEV), hadamard_scale=0.)
    want_scale = qo.find_scale_int4(x)
    assert ulp_diff(scale, want_scale).max() <= 1
    xp = torch.empty(40, 512, dtype=torch.uint8)
    rs = torch.empty(40, 1, dtype=torch.int32)
    qo.quantize_int4(x, scale.cpu(), None, xp, rs, False)
    assert torch.equal(packed.cpu(), xp) and torch.equal(row_sum.cpu(), rs)


def test_error_codes_no_launch(quest):
    from quest_amd import _lib
    lib = _lib.load()
    x = torch.zeros(4, 128, dtype=torch.bfloat16, device=DEV)
    s = torch.zeros(4, 1, dtype=torch.bfloat16, device=DEV)
    st = _lib.stream_of(x)
    assert lib.quest_find_scale_int4(None, _lib.ptr(x), 128, 4, 0, st) == -1
    assert lib.quest_find_scale_int4(_lib.ptr(s), _lib.ptr(x), 100, 4, 0, st) == -2
    assert lib.quest_find_scale_int4(_lib.ptr(s), _lib.ptr(x), 128, 4, 7, st) == -3
    assert lib.quest_hadamard_quantize_int4(_lib.ptr(x), _lib.ptr(s), None, None, None, 64, 4, 0.1, 0, st) == -2
    assert lib.quest_matmul_int4_int4t_int32(_lib.ptr(x), _lib.ptr(x), _lib.ptr(x), 4, 48, 4, st) == -2
    with pytest.raises(RuntimeError):
        quest.find_scale_int4(torch.zeros(2, 128, dtype=torch.bfloat16))       # CPU tensor: no fallback
    with pytest.raises(NotImplementedError):
        quest.matmul_int4sp_int4t_int32(None, None, None)
