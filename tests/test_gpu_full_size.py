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

    # the same codes as E2M3 tiles, over the whole tensor: byte for byte the conversion of the packed output (which
    # tests/test_gpu_e2m3.py holds against the oracle's encoding); m is whole row blocks, so there is no padding
    s4, tiles = quest.hadamard_quantize_e2m3(gx)
    assert torch.equal(bits(s4.cpu()), bits(scale.cpu()))
    assert torch.equal(tiles, quest.int4_to_e2m3_tiles(packed))
    assert torch.equal(qo.e2m3_tiles_decode(tiles[:2 * (k // 64) * 1536].cpu(), 64, k), qo.unpack_int4(packed[:64].cpu()).double() + .5)

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
    # the tiles of the same tensor (the second launch continues in the row block after the cut): byte for byte the
    # conversion of the packed codes, over every whole row block
    s6, tiles = quest.hadamard_quantize_e2m3(x)
    assert torch.equal(bits(s6.cpu()), bits(scale.cpu()))
    whole = (m // 32) * (k // 64) * 1536
    assert torch.equal(tiles[:whole], quest.int4_to_e2m3_tiles(packed)[:whole])
    del tiles
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


@pytest.mark.parametrize('shape', [(4096, 4096, 11008), (16384, 1024, 3072), (16384, 2816, 1024), (9000, 512, 4104)])
def test_prefill_gemm_e2m3_full_size(quest, shape):
    """The FP6 kernel at the same sizes, by the same method: its output is the epilogue formula on the exact integer
    matrix -- 2 C + a_add + b_add recovered from checksums and sampled rows as above -- everywhere, bit for bit."""
    m, k, n = shape
    a, b, ap, bp, a_add, b_add, a_mul, b_mul = _gemm_inputs(m, k, n, seed=0)
    gap, gbp = ap.to(DEV), bp.to(DEV)
    g_a_add, g_b_add, g_a_mul, g_b_mul = (t.to(DEV) for t in (a_add, b_add, a_mul, b_mul))
    d = quest.fused_matmul_dequantize_e2m3(quest.int4_to_e2m3_tiles(gap), quest.int4_to_e2m3_tiles(gbp), g_a_mul, g_b_mul, k)
    # exact integers on the GPU in fp64 (|values| < 2^53), independent of either GEMM kernel
    ga, gb = a.to(DEV).double(), b.to(DEV).double()
    gen = torch.Generator().manual_seed(2)
    rows = torch.randperm(m, generator=gen)[:64].to(DEV)
    c_rows = (ga[rows] @ gb.T).to(torch.int32)
    lhs = (c_rows * 2 + g_a_add[rows] + g_b_add.T).float()
    rhs = (0.5 * g_a_mul[rows].float()) * g_b_mul.float().T
    assert torch.equal(bits(d[rows]), bits((lhs * rhs).to(d.dtype)))
    # everywhere: against the INT8 kernel, whose int32 matrix the test above pins by checksums
    want = quest.fused_matmul_dequantize_int4_int4t_bf16(gap, gbp, g_a_add, g_b_add, g_a_mul, g_b_mul)
    assert torch.equal(bits(d), bits(want))


def test_swiglu_gemm_full_size(quest):
    """The gate/up GEMM of Llama-7B with the gated unit in its epilogue, M = 4096, K = 4096, 2 H = 22016: equal to the
    plain fused GEMM (pinned above) on the same rows followed by torch's silu(gate) * up -- within 2 ulp on under 2 % of
    the elements (the fast exponential) everywhere against torch on the GPU and on 64 sampled rows against torch on the
    CPU; the INT8 and the FP6 kernel agree bit for bit."""
    m, k, n = 4096, 4096, 22016
    h = n // 2
    a, b, ap, bp, a_add, b_add, a_mul, b_mul = _gemm_inputs(m, k, n, seed=5, dtype=torch.bfloat16)
    gap, gbp = ap.to(DEV), bp.to(DEV)
    g_a_add, g_b_add, g_a_mul, g_b_mul = (t.to(DEV) for t in (a_add, b_add, a_mul * 0.1, b_mul * 0.1))
    p = quest.swiglu_interleave_rows(h, device=DEV)
    bpi, bai, bmi = gbp[p].contiguous(), g_b_add[p].contiguous(), g_b_mul[p].contiguous()
    got = quest.fused_matmul_dequantize_swiglu_int4_int4t(gap, bpi, g_a_add, bai, g_a_mul, bmi)
    assert got.shape == (m, h)
    got6 = quest.fused_matmul_dequantize_e2m3(quest.int4_to_e2m3_tiles(gap), quest.int4_to_e2m3_tiles(bpi), g_a_mul, bmi, k, swiglu=True)
    assert torch.equal(bits(got), bits(got6))
    gate_up = quest.fused_matmul_dequantize_int4_int4t_bf16(gap, gbp, g_a_add, g_b_add, g_a_mul, g_b_mul)     # (M, 2 H): gates, then ups
    want = torch.nn.functional.silu(gate_up[:, :h].float()).to(gate_up.dtype).float() * gate_up[:, h:].float()
    want = want.to(gate_up.dtype)
    d = (bits(got) - bits(want)).abs()
    assert int(d.max()) <= 2 and float((d != 0).float().mean()) < 0.02, (int(d.max()), float((d != 0).float().mean()))
    gen = torch.Generator().manual_seed(6)
    rows = torch.randperm(m, generator=gen)[:64]
    cpu = gate_up[rows.to(DEV)].cpu()
    want_cpu = torch.nn.functional.silu(cpu[:, :h]) * cpu[:, h:]
    dc = (bits(got[rows.to(DEV)].cpu()) - bits(want_cpu)).abs()
    assert int(dc.max()) <= 2 and float((dc != 0).float().mean()) < 0.02


@pytest.mark.parametrize('m', [1, 8, 16])
@pytest.mark.parametrize('kn', [(4096, 4096), (11008, 4096)])
def test_decode_layer_as_one_workload(quest, m, kn, capsys):
    """The decode configuration as the layer it is: fp16 randn activations -> fused Hadamard-quantise -> weight-streaming
    GEMM, through harness.linear_forward.  The output equals the oracle's GEMM + epilogue on the codes the kernel produced,
    bit for bit; those codes against the full oracle pipeline on the same x (F.linear Hadamard, torch-CPU scale,
    quantiser) are counted and bounded."""
    from quest_amd import harness
    k, n = kn
    g = torch.Generator().manual_seed(100 + m)
    x = torch.randn(m, k, generator=g).half()
    b = torch.randint(-8, 8, (n, k), generator=g, dtype=torch.int8)
    w_packed = qo.pack_int4(b)
    w_scale = (torch.rand(n, 1, generator=g) * 0.09 + 0.01).half()
    w_add = (b.to(torch.int32).sum(-1, keepdim=True) + k // 2).to(torch.int32)
    a_scale = torch.empty(m, 1, dtype=torch.float16, device=DEV)
    a_packed = torch.empty(m, k // 2, dtype=torch.uint8, device=DEV)
    a_row_sum = torch.empty(m, 1, dtype=torch.int32, device=DEV)
    y = harness.linear_forward(x.to(DEV), w_packed.to(DEV), w_scale.to(DEV), w_add.to(DEV), use_hadamard=True,
                               _a_scale=a_scale, _a_int_packed=a_packed, _a_int_row_sum=a_row_sum)
    want = qo.fused_matmul_dequantize_int4_int4t(a_packed.cpu(), w_packed, a_row_sum.cpu(), w_add, a_scale.cpu(), w_scale, via='fp32')
    assert torch.equal(bits(y.cpu()), bits(want))
    _, o_scale, o_packed, _ = qo.hadamard_quantize_int4(x, hadamard='matmul')
    differ = float((qo.unpack_int4(a_packed.cpu()) != qo.unpack_int4(o_packed)).float().mean())
    scale_ulps = int((bits(a_scale.cpu()) - bits(o_scale)).abs().max())
    with capsys.disabled():
        print(f'\n[decode layer M={m} K={k} N={n}] activation codes differing from the oracle pipeline: {100 * differ:.3f} %, '
              f'scale within {scale_ulps} ulp')
    assert differ < 0.02 and scale_ulps <= 1
    ref = qo.linear_forward(x, w_packed, w_scale, w_add, use_hadamard=True, hadamard='matmul', via='fp32').double()
    assert float((y.cpu().double() - ref).norm() / ref.norm()) < 1e-2


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


@pytest.mark.parametrize('m', [1, 5, 16])
@pytest.mark.parametrize('kn', [(32768, 512), (32768, 1000), (32768, 2048), (16384, 1024), (65536, 250), (16384, 1022), (4096, 4096), (11008, 4096)])
def test_decode_gemm_split_k(quest, m, kn):
    """K split across workgroups through a caller-owned workspace (long rows, few channels; the last two shapes do not
    split and take the plain kernel): bit-exact against the oracle, the same workspace reused across shapes and calls
    without clearing it (every call leaves its counters at zero), also from a HIP graph."""
    k, n = kn
    a, b, ap, bp, a_add, b_add, a_mul, b_mul = _gemm_inputs(m, k, n, seed=11 + m)
    want_d = qo.add_mul_vv(a_add, a_mul, b_add, b_mul, (a.double() @ b.double().T).to(torch.int32))
    if 'work' not in _SPLIT_K_STATE:
        _SPLIT_K_STATE['work'] = quest.gemm_workspace(DEV)
    work = _SPLIT_K_STATE['work']
    assert quest.gemm_workspace_bytes(m, k, n) <= work.numel()
    assert (quest.gemm_workspace_bytes(m, k, n) > 0) == (k >= 16384)
    args = [t.to(DEV) for t in (ap, bp, a_add, b_add, a_mul, b_mul)]
    for _ in range(3):
        d = quest.fused_matmul_dequantize_int4_int4t_bf16(*args, workspace=work)
        assert torch.equal(bits(d.cpu()), bits(want_d))
    assert int(work[:16384].view(torch.int32).abs().max()) == 0
    out = torch.empty_like(d)
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        quest.fused_matmul_dequantize_int4_int4t_bf16(*args, out=out, workspace=work)
    torch.cuda.current_stream().wait_stream(side)
    with torch.cuda.graph(graph):
        quest.fused_matmul_dequantize_int4_int4t_bf16(*args, out=out, workspace=work)
    for _ in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(bits(out.cpu()), bits(want_d))


_SPLIT_K_STATE = {}


def test_decode_gemm_split_k_falls_back(quest):
    """No workspace, one too small, or a shape that does not split: the plain kernel runs, same result."""
    m, k, n = 4, 32768, 512
    a, b, ap, bp, a_add, b_add, a_mul, b_mul = _gemm_inputs(m, k, n, seed=2)
    args = [t.to(DEV) for t in (ap, bp, a_add, b_add, a_mul, b_mul)]
    want = quest.fused_matmul_dequantize_int4_int4t_bf16(*args)
    small = torch.zeros(4096, dtype=torch.uint8, device=DEV)
    assert quest.gemm_workspace_bytes(m, k, n) > small.numel()
    assert torch.equal(bits(quest.fused_matmul_dequantize_int4_int4t_bf16(*args, workspace=small)), bits(want))
    assert quest.gemm_workspace_bytes(64, k, n) == 0 and quest.gemm_workspace_bytes(4, 32768 + 64, n) == 0
    assert quest.gemm_workspace_bytes(4, 4096, 4096) == 0
    m = 64
    a, b, ap, bp, a_add, b_add, a_mul, b_mul = _gemm_inputs(m, k, n, seed=3)
    args = [t.to(DEV) for t in (ap, bp, a_add, b_add, a_mul, b_mul)]
    work = quest.gemm_workspace(DEV)
    assert torch.equal(bits(quest.fused_matmul_dequantize_int4_int4t_bf16(*args, workspace=work)),
                       bits(quest.fused_matmul_dequantize_int4_int4t_bf16(*args)))


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
