"""GPU checks at the benchmark's full sizes, where the CPU oracle cannot redo the whole computation in seconds:
size-independent properties over the complete result (checksums of checksums, pack/unpack round trips, the fused
kernel against its own unfused steps, determinism) plus the oracle bit for bit on sampled rows.

  * activation kernel  bf16 [8192, 4096], heavy-tailed data
  * prefill GEMM       M=4096, K=4096, N=11008, uniform codes
  * decode GEMM        M in {1, 8, 16}, (K, N) in {(4096, 4096), (11008, 4096)}
  * 12-layer forward   ids (32, 512), d=1024
"""
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


def bits(t):
    return t.contiguous().view(torch.int16).to(torch.int32)


def unpack_gpu(packed):
    """(rows, K/2) uint8 -> (rows, K) int8 codes, low nibble first (gemm-quest/benchmarks/utils.py:420-445)."""
    lo = (packed & 0xF).to(torch.int8)
    hi = (packed >> 4).to(torch.int8)
    lo = torch.where(lo >= 8, lo - 16, lo)
    hi = torch.where(hi >= 8, hi - 16, hi)
    return torch.stack((lo, hi), dim=-1).flatten(-2)


def heavy_tailed(m, k, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, k, generator=g) / torch.sqrt(torch.randn(m, k, 3, generator=g).pow(2).mean(-1))   # Student-t(3)
    cols = torch.randperm(k, generator=g)[: max(1, k // 100)]
    x[:, cols] *= 20
    return x.to(dtype)


def test_activation_kernel_8192x4096(quest):
    m, k = 8192, 4096
    x = heavy_tailed(m, k, torch.bfloat16, seed=0)
    gx = x.to(DEV)
    x_had = torch.empty_like(gx)
    scale, packed, row_sum = quest.hadamard_quantize_int4(gx, x_had=x_had)
    assert torch.equal(bits(gx.cpu()), bits(x)), 'input must not be written'

    # the whole result: codes in range by construction of the nibbles, row sums = sum of the unpacked codes
    codes = unpack_gpu(packed)
    assert torch.equal(codes.to(torch.int32).sum(-1, keepdim=True), row_sum.to(torch.int32))
    assert (scale.float() > 0).all()

    # the fused kernel = its unfused steps on its own transformed tensor, everywhere
    s2 = quest.find_scale_int4(x_had)
    d = (bits(scale.cpu()) - bits(s2.cpu())).abs()               # two fp32 summation orders: one 16-bit ulp on a rare row
    assert d.max() <= 1 and (d != 0).sum() <= m // 1000
    _, _, p2, r2 = quest.quantize_int4(x_had.clone(), scale, x_int_packed=torch.empty_like(packed),
                                       x_int_row_sum=torch.empty_like(row_sum))
    assert torch.equal(packed, p2) and torch.equal(row_sum, r2)

    # deterministic
    s3, p3, r3 = quest.hadamard_quantize_int4(gx)
    assert torch.equal(bits(scale.cpu()), bits(s3.cpu())) and torch.equal(packed, p3) and torch.equal(row_sum, r3)

    # the oracle on sampled rows: transform within tolerance, codes bit for bit given the kernel's transform and scale
    rows = torch.randperm(m, generator=torch.Generator().manual_seed(1))[:96]
    xs = x[rows]
    want_had = qo.hadamard128_matmul(xs)
    got_had = x_had[rows.to(DEV)].cpu()
    rel = (got_had.double() - want_had.double()).norm() / want_had.double().norm()
    assert rel <= 1e-3, rel                                     # the bar stated for the Hadamard transform
    want_scale = qo.find_scale_int4(got_had)
    got_scale = scale[rows.to(DEV)].cpu()
    assert (bits(got_scale) - bits(want_scale)).abs().max() <= 1          # fp32 summation order: one 16-bit ulp at most
    _, _, want_packed, want_sum = qo.quantize_int4(got_had.clone(), got_scale,
                                                   x_int_packed=torch.empty(len(rows), k // 2, dtype=torch.uint8),
                                                   x_int_row_sum=torch.empty(len(rows), 1, dtype=torch.int32))
    assert torch.equal(packed[rows.to(DEV)].cpu(), want_packed)
    assert torch.equal(row_sum[rows.to(DEV)].cpu(), want_sum)


def test_activation_tensor_of_2_gib_and_more(quest):
    """An input of 2 GiB and more goes to the kernel as several launches of whole rows (32-bit offsets inside one):
    the rows either side of the cut, the first and the last ones must equal what the same rows give as a tensor of
    their own, bit for bit, and every row sum must match its codes."""
    k = 4096
    cut = ((1 << 31) - 1) // (2 * k)                 # rows in the first launch: 262143
    m = cut + 300
    g = torch.Generator(device=DEV).manual_seed(5)
    x = torch.randn(m, k, generator=g, device=DEV, dtype=torch.float32).to(torch.bfloat16)
    assert x.numel() * 2 >= 1 << 31
    scale, packed, row_sum = quest.hadamard_quantize_int4(x)
    for lo, hi in ((0, 128), (cut - 160, cut + 160), (m - 128, m)):
        s2, p2, r2 = quest.hadamard_quantize_int4(x[lo:hi])
        assert torch.equal(bits(scale[lo:hi].cpu()), bits(s2.cpu())), (lo, hi)
        assert torch.equal(packed[lo:hi], p2) and torch.equal(row_sum[lo:hi], r2), (lo, hi)
    step = 32768
    for lo in range(0, m, step):                      # in pieces: the unpacked codes of everything would be 2 GiB more
        codes = unpack_gpu(packed[lo:lo + step])
        assert torch.equal(codes.to(torch.int32).sum(-1, keepdim=True), row_sum[lo:lo + step].to(torch.int32)), lo
    assert (scale.float() > 0).all()


def _gemm_inputs(m, k, n, seed, dtype=torch.float16):
    g = torch.Generator().manual_seed(seed)
    a = torch.randint(-8, 8, (m, k), generator=g, dtype=torch.int8)
    b = torch.randint(-8, 8, (n, k), generator=g, dtype=torch.int8)
    pack = lambda q: ((q[:, 1::2] << 4) | (q[:, ::2] & 0xF)).view(torch.uint8)       # noqa: E731
    a_mul = (torch.rand(m, 1, generator=g) * 0.09 + 0.01).to(dtype)
    b_mul = (torch.rand(n, 1, generator=g) * 0.09 + 0.01).to(dtype)
    a_add = a.to(torch.int32).sum(-1, keepdim=True).to(torch.int32)
    b_add = (b.to(torch.int32).sum(-1, keepdim=True) + k // 2).to(torch.int32)
    return a, b, pack(a), pack(b), a_add, b_add, a_mul, b_mul


# the prefill shape of the benchmark (the XCD groups divide the channels); the model's QKV and MLP-output shapes at
# 32 x 512 tokens (more tokens than channels: the groups divide the token tiles), one in each tile shape; a token
# count that leaves the groups unequal shares of token tiles
@pytest.mark.parametrize('shape', [(4096, 4096, 11008), (16384, 1024, 3072), (16384, 2816, 1024), (9000, 512, 4104)])
def test_prefill_gemm_full_size(quest, shape):
    m, k, n = shape
    a, b, ap, bp, a_add, b_add, a_mul, b_mul = _gemm_inputs(m, k, n, seed=0)
    gap, gbp = ap.to(DEV), bp.to(DEV)
    c = quest.matmul_int4_int4t_int32(gap, gbp)

    # checksum of checksums, exact in fp64 (|sum| < 2^53): sum_n C[m, n] = a[m, :] . colsum(b), sum_m C[m, n] = b[n, :] . colsum(a)
    ga, gb = a.to(DEV).double(), b.to(DEV).double()
    assert torch.equal(c.double().sum(1), ga @ gb.sum(0))
    assert torch.equal(c.double().sum(0), gb @ ga.sum(0))

    # sampled rows and columns against exact integer arithmetic on the CPU
    gen = torch.Generator().manual_seed(2)
    rows = torch.randperm(m, generator=gen)[:48]
    cols = torch.randperm(n, generator=gen)[:48]
    want_rows = (a[rows].double() @ b.double().T).to(torch.int32)
    want_cols = (a.double() @ b[cols].double().T).to(torch.int32)
    assert torch.equal(c[rows.to(DEV)].cpu(), want_rows)
    assert torch.equal(c[:, cols.to(DEV)].cpu(), want_cols)

    # the fused epilogue = the epilogue formula on that int32 matrix (gemm-quest/benchmarks/utils.py:535-545), everywhere
    dev = lambda *ts: [t.to(DEV) for t in ts]                                           # noqa: E731
    g_a_add, g_b_add, g_a_mul, g_b_mul = dev(a_add, b_add, a_mul, b_mul)
    d = quest.fused_matmul_dequantize_int4_int4t_bf16(gap, gbp, g_a_add, g_b_add, g_a_mul, g_b_mul)
    lhs = (c * 2 + g_a_add + g_b_add.T).float()
    rhs = (0.5 * g_a_mul.float()) * g_b_mul.float().T
    assert torch.equal(bits(d), bits((lhs * rhs).to(d.dtype)))
    d2 = quest.add_mul_vv(g_a_add, g_a_mul, g_b_add, g_b_mul, c)
    assert torch.equal(bits(d), bits(d2))
    # against the real-valued product: <= 1e-2 relative
    rows64 = rows[:16]
    real = ((a[rows64].double() + 0.5) * a_mul[rows64].double()) @ ((b.double() + 0.5) * b_mul.double()).T
    rel = (d[rows64.to(DEV)].cpu().double() - real).norm() / real.norm()
    assert rel <= 1e-2, rel


@pytest.mark.parametrize('m', [1, 8, 16])
@pytest.mark.parametrize('kn', [(4096, 4096), (11008, 4096), (4096, 11008)])
def test_decode_gemm_full_shapes(quest, m, kn):
    k, n = kn
    a, b, ap, bp, a_add, b_add, a_mul, b_mul = _gemm_inputs(m, k, n, seed=3 + m)
    want_c = (a.double() @ b.double().T).to(torch.int32)
    c = quest.matmul_int4_int4t_int32(ap.to(DEV), bp.to(DEV))
    assert torch.equal(c.cpu(), want_c)
    d = quest.fused_matmul_dequantize_int4_int4t_bf16(ap.to(DEV), bp.to(DEV), a_add.to(DEV), b_add.to(DEV), a_mul.to(DEV), b_mul.to(DEV))
    want_d = qo.add_mul_vv(a_add, a_mul, b_add, b_mul, want_c)
    assert torch.equal(bits(d.cpu()), bits(want_d))


def test_forward_full_config():
    """The 12-layer model at ids (32, 512): the producer-fused forward is deterministic, replays from a HIP graph bit
    for bit, and stays within INT4 noise of the forward whose glue is plain torch (a per cent or two of the codes of
    every layer sit within bf16 rounding of a quantisation step and flip between the two)."""
    from quest_amd import llama
    cfg = llama.LlamaConfig()
    ids = torch.randint(0, cfg.vocab_size, (32, cfg.sequence_length), generator=torch.Generator().manual_seed(0)).to(DEV)
    out = {}
    for fused in (False, True):
        torch.manual_seed(0)
        model = llama.Llama(cfg).to(torch.bfloat16).to(DEV).eval()
        llama.quantize_model(model, 'int4', use_hadamard=True, fuse_gate_up=True, fuse_producers=fused)
        with torch.inference_mode():
            out[fused] = model(ids)['logits'].float()
            again = model(ids)['logits'].float()
        assert torch.equal(out[fused], again)
        assert torch.isfinite(out[fused]).all()
        if fused:
            r = llama.bench_forward(model, 32, cfg.sequence_length, n_warmup=2, n_iter=2)
            assert r['graph_matches_eager']
        del model
    rel = (out[True] - out[False]).norm() / out[False].norm()
    assert rel < 0.2, rel
