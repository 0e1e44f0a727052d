"""Pins the CPU oracle (oracle/) before anything is compared with it.

The reference holds no golden vectors for this path, so every function of the oracle is held
against what the mathematics fixes: closed forms, exact rational arithmetic, brute force over
all 16-bit inputs, Sylvester-matrix identities, and the independent scalar C restatement.
Each check is chosen so that a plausible slip (wrong nibble order, round instead of floor,
missing +1/2, transposed operand, dropped K/2, fused multiply-add) fails it.
"""
from fractions import Fraction

import numpy as np
import pytest
import scipy.linalg
import torch

from oracle import quest_oracle as qo

DTYPES = [torch.bfloat16, torch.float16]


def all_finite_16(dtype):
    bits = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16)
    v = bits.view(dtype)
    return v[torch.isfinite(v.float())]


def frac(t):
    """Exact rational value of each element of a float tensor (as python Fractions)."""
    return [Fraction(float(v)) for v in t.double().flatten().tolist()]


def round_to(dtype, value: Fraction) -> float:
    """Correctly rounded (nearest even) `dtype` value of an exact rational, by search over the
    two neighbouring representable numbers found through float64 (exact for our magnitudes)."""
    approx = torch.tensor(float(value), dtype=torch.float64).to(dtype)
    cands = set()
    b = approx.view(torch.int16).item()
    for d in (-1, 0, 1):
        bb = (b + d) & 0xffff
        c = torch.tensor(bb, dtype=torch.int32).to(torch.int16).view(dtype)
        if torch.isfinite(c.float()):
            cands.add(((c.view(torch.int16).item() & 1), float(c)))
    best = min(cands, key=lambda pc: (abs(Fraction(pc[1]) - value), pc[0]))
    return best[1]


# --------------------------------------------------------------------------- conversions in C
@pytest.mark.parametrize('dtype', DTYPES)
def test_c_16bit_to_f32_all_patterns(c_oracle, dtype):
    lib = c_oracle.lib()
    f = lib.qo_fp16_to_f32 if dtype == torch.float16 else lib.qo_bf16_to_f32
    bits = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16)
    want = bits.view(dtype).float()
    got = torch.tensor([f(int(b) & 0xffff) for b in bits.tolist()], dtype=torch.float32)
    assert torch.equal(got.view(torch.int32)[~want.isnan()], want.view(torch.int32)[~want.isnan()])
    assert got[want.isnan()].isnan().all()


@pytest.mark.parametrize('dtype', DTYPES)
def test_c_f32_to_16bit_rne(c_oracle, dtype):
    lib = c_oracle.lib()
    f = lib.qo_f32_to_fp16 if dtype == torch.float16 else lib.qo_f32_to_bf16
    g = torch.Generator().manual_seed(1)
    x = torch.randn(20000, generator=g) * torch.logspace(-9, 5, 20000)
    # exact ties and boundary cases: midpoints between neighbouring 16-bit values
    v = all_finite_16(dtype).float()
    v = v[(v.abs() < 6e4) & (v != 0)][::37]
    mid = ((v.double() + torch.nextafter(v.to(dtype), torch.tensor(float('inf'), dtype=dtype)).double()) / 2).float()
    x = torch.cat([x, mid, torch.tensor([0., -0., 65504., 65519.9, 65520., 1e-8, 5.96e-8, 2.98e-8, 2.9803e-8, 1e38])])
    want = x.to(dtype).view(torch.int16).to(torch.int32) & 0xffff
    got = torch.tensor([f(float(t)) for t in x.tolist()], dtype=torch.int32)
    assert torch.equal(got, want)


# --------------------------------------------------------------------------- Hadamard (H1/H2)
def test_sylvester_is_scipy_hadamard_and_orthogonal():
    s = qo.sylvester_signs().to(torch.int64)
    assert np.array_equal(s.numpy(), scipy.linalg.hadamard(128))
    assert torch.equal(s, s.t())
    assert torch.equal(s @ s, 128 * torch.eye(128, dtype=torch.int64))


@pytest.mark.parametrize('dtype', DTYPES)
def test_hadamard_matrix_entries(dtype):
    h = qo.hadamard_matrix(dtype).float()
    assert torch.equal(h.abs(), torch.full((128, 128), 181. / 2048.))
    assert torch.equal(torch.sign(h).to(torch.int8), qo.sylvester_signs())
    assert qo.hadamard_entry(dtype) == 181. / 2048.


@pytest.mark.parametrize('dtype', DTYPES)
def test_hadamard_unit_vectors_and_exact_integers(c_oracle, dtype):
    # H e_i is row i of the matrix; small-integer inputs make every partial sum exact, so all
    # four implementations must agree bit for bit with the exact closed form.
    eye = torch.eye(128, dtype=dtype)
    for f in (qo.hadamard128_matmul, lambda t: qo.hadamard128_fwht(t, 181. / 2048.),
              c_oracle.hadamard128_matmul, lambda t: c_oracle.hadamard128_fwht(t, 181. / 2048.)):
        assert torch.equal(f(eye), qo.hadamard_matrix(dtype))
    g = torch.Generator().manual_seed(2)
    x = torch.randint(-3, 4, (5, 384), generator=g).to(dtype)
    exact = (x.double().view(-1, 128) @ qo.sylvester_signs().double()) * (181. / 2048.)
    want = exact.to(dtype).view(5, 384)          # exact value -> one rounding
    assert torch.equal(qo.hadamard128_matmul(x), want)
    assert torch.equal(qo.hadamard128_fwht(x, 181. / 2048.), want)
    assert torch.equal(c_oracle.hadamard128_matmul(x), want)
    assert torch.equal(c_oracle.hadamard128_fwht(x, 181. / 2048.), want)


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('scale', [181. / 2048., 2. ** -3.5])
def test_hadamard_random_against_fp64_closed_form(c_oracle, dtype, scale):
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(16, 512, generator=g) * 3).to(dtype)
    exact = ((x.double().view(-1, 128) @ qo.sylvester_signs().double()) * float(np.float32(scale))).view(16, 512)
    y = qo.hadamard128_fwht(x, scale)
    assert torch.equal(y, c_oracle.hadamard128_fwht(x, scale))       # same butterfly order -> same bits
    # against the correctly rounded closed form: the 1e-3 relative bar of the north star
    rel = (y.double() - exact.to(dtype).double()).norm() / exact.norm()
    assert rel < 1e-3
    y32 = qo.hadamard128_fwht(x, scale, out_dtype=torch.float32)
    assert (y32.double() - exact).norm() / exact.norm() < 1e-6         # fp32 inside: error far below 16-bit rounding
    # and never further than one dtype ulp from the correctly rounded value
    ulp = (torch.nextafter(exact.to(dtype).abs(), torch.tensor(float('inf'), dtype=dtype)).double() - exact.to(dtype).abs().double())
    assert ((y.double() - exact).abs() <= ulp).all()
    if scale == 181. / 2048.:
        for ym in (qo.hadamard128_matmul(x), c_oracle.hadamard128_matmul(x)):
            assert (ym.double() - exact.to(dtype).double()).norm() / exact.norm() < 1e-3
            assert (ym.double() - y.double()).norm() / exact.norm() < 1e-3   # the two formulations agree
            assert ((ym.double() - exact).abs() <= ulp).all()


def test_hadamard_norm_and_involution():
    g = torch.Generator().manual_seed(4)
    x = torch.randn(8, 256, generator=g).bfloat16()
    y = qo.hadamard128_fwht(x, 2. ** -3.5, out_dtype=torch.float32)
    assert abs(float(y.norm() / x.float().norm()) - 1) < 1e-5
    back = qo.hadamard128_fwht(y, 2. ** -3.5, out_dtype=torch.float32)
    assert torch.allclose(back, x.float(), atol=1e-5)


# --------------------------------------------------------------------------- S1 scale
def test_scale_constants():
    assert np.float32(qo.GAUSS_INT4_STEP).view(np.uint32) == 0x3eab9e1f
    chain = np.float32(2.513930578568423) * np.float32(2.) / np.float32(15.)     # the CUDA float chain
    assert chain.view(np.uint32) == 0x3eab9e1f
    assert float(np.float32(1e-8)) == 9.99999993922529e-09


@pytest.mark.parametrize('dtype', DTYPES)
def test_scale_constant_rows_closed_form(c_oracle, dtype):
    vals = [0., 1., -1., 0.5, 3., -7.25, 100., 2. ** -10, 1e-3]
    x = torch.tensor(vals).to(dtype)[:, None].repeat(1, 256)
    got = qo.find_scale_int4(x)
    for c, s in zip(x[:, 0].float().tolist(), got[:, 0].tolist()):
        # mean of identical squares is exact when c*c is; sqrt gives |c| back
        prod = Fraction(float(np.float32(abs(c)) * np.float32(qo.GAUSS_INT4_STEP)))
        total = Fraction(float(np.float32(float(prod)) + np.float32(1e-8)))
        assert s == round_to(dtype, total), (c, s)
    for order in (0, 1):
        assert torch.equal(c_oracle.find_scale_int4(x, order), got)
    zero = qo.find_scale_int4(torch.zeros(1, 128, dtype=dtype))
    if dtype == torch.bfloat16:
        assert zero.view(torch.int16).item() == 0x322c      # bf16(1e-8)
    else:
        assert zero.item() == 0.                            # fp16(1e-8) underflows to 0


@pytest.mark.parametrize('dtype', DTYPES)
def test_scale_random_rows_vs_c_and_fp64(c_oracle, dtype):
    g = torch.Generator().manual_seed(5)
    x = (torch.randn(512, 1024, generator=g) * torch.rand(512, 1, generator=g) * 4).to(dtype)
    got = qo.find_scale_int4(x)
    exact = (x.double() ** 2).mean(-1, keepdim=True).sqrt() * float(np.float32(qo.GAUSS_INT4_STEP)) + 1e-8
    assert ((got.double() - exact).abs() / exact).max() < 2 ** -8        # within one 16-bit ulp
    for order in (0, 1):
        c = c_oracle.find_scale_int4(x, order)
        diff = (c.view(torch.int16).int() - got.view(torch.int16).int()).abs()
        assert diff.max() <= 1                        # summation order may move a tie by one ulp
        assert (diff != 0).sum() <= 2                 # and does so on at most a couple of rows in 512


# --------------------------------------------------------------------------- S2 quantise
@pytest.mark.parametrize('dtype', DTYPES)
def test_quantize_all_16bit_inputs_exact_floor(c_oracle, dtype):
    xs = all_finite_16(dtype)
    scales = torch.tensor([0.3351907, 1.0, 0.007, 3.1, 2. ** -9, 0.0625, 117.0, 0.99]).to(dtype)
    for s in scales:
        x = xs.clone().view(1, -1)
        sc = s.view(1, 1)
        x_int = torch.empty(1, x.numel(), dtype=torch.int8)
        packed = torch.empty(1, x.numel() // 2, dtype=torch.uint8)
        rs = torch.empty(1, 1, dtype=torch.int32)
        qo.quantize_int4(x, sc, x_int, packed, rs, False)
        # exact floor: a float64 quotient of two <=11-bit-mantissa numbers is exact when it is an
        # integer and at least 2^-11 (relative) away from one otherwise, so its floor is the true floor
        want = torch.floor(x.double() / sc.double()).clamp(-8, 7).to(torch.int8)
        assert torch.equal(x_int, want)
        _, ci, cp, cs = c_oracle.quantize_int4(x, sc, False)
        assert torch.equal(ci, want) and torch.equal(cp, packed) and torch.equal(cs, rs)
        assert rs.item() == int(want.to(torch.int64).sum())
        assert torch.equal(qo.unpack_int4(packed), want)
        assert torch.equal(c_oracle.unpack_int4(packed), want)


@pytest.mark.parametrize('dtype', DTYPES)
def test_quantize_fraction_spot_checks(dtype):
    g = torch.Generator().manual_seed(6)
    x = (torch.randn(1, 4000, generator=g) * 2).to(dtype)
    # add exact multiples of the scale (ties of floor) on purpose
    s = torch.tensor([[0.40625]]).to(dtype)
    x[0, :200] = (torch.randint(-9, 9, (200,), generator=g).float() * s.float().item()).to(dtype)
    x_int = torch.empty(1, 4000, dtype=torch.int8)
    qo.quantize_int4(x, s, x_int, None, None, False)
    sf = Fraction(float(s))
    for xv, q in zip(frac(x), x_int.flatten().tolist()):
        want = max(-8, min(7, (xv / sf).__floor__()))
        assert q == want


def test_float32_division_floor_is_exact_floor_for_16bit_operands():
    """floor(fl32(x / s)) == floor(x / s) for every pair of bf16/fp16 mantissas whose quotient can
    land in the INT4 range: the property that lets a kernel replace the divide by an exact test."""
    ms = np.arange(1024, 2048, dtype=np.int64)[None, :]
    bad = 0
    total = 0
    for lo in range(1, 2048, 256):
        mx = np.arange(lo, min(lo + 256, 2048), dtype=np.int64)[:, None]
        for e in range(-12, 5):
            exact = (mx << e) // ms if e >= 0 else mx // (ms << -e)          # floor, x > 0
            exact_neg = -((mx << e) // -ms) if False else None
            xf = (mx.astype(np.float32) * np.float32(2.) ** np.float32(e))
            q = np.floor(xf / ms.astype(np.float32))
            keep = exact <= 9
            bad += int((q[keep] != exact[keep]).sum())
            # negative x: floor(-a / s) = -ceil(a / s)
            num = (mx << e) if e >= 0 else mx
            den = ms if e >= 0 else (ms << -e)
            exact_n = -((num + den - 1) // den)
            qn = np.floor(-xf / ms.astype(np.float32))
            keep_n = exact_n >= -10
            bad += int((qn[keep_n] != exact_n[keep_n]).sum())
            total += int(keep.sum() + keep_n.sum())
    assert total > 10_000_000
    assert bad == 0


def test_pack_nibble_order_known_bytes():
    q = torch.tensor([[-8, 7, -1, 3, 0, -1, 5, -6]], dtype=torch.int8)
    # byte j = (q[2j+1] << 4) | (q[2j] & 0xF): low nibble holds the even element
    assert qo.pack_int4(q).tolist() == [[0x78, 0x3f, 0xf0, 0xa5]]
    allb = torch.arange(256, dtype=torch.int32).to(torch.uint8).view(1, 256)
    assert torch.equal(qo.pack_int4(qo.unpack_int4(allb)), allb)
    u = qo.unpack_int4(torch.tensor([[0x78]], dtype=torch.uint8))
    assert u.tolist() == [[-8, 7]]


@pytest.mark.parametrize('dtype', DTYPES)
def test_dequantize_is_q_plus_half_times_scale(c_oracle, dtype):
    g = torch.Generator().manual_seed(7)
    x = (torch.randn(4, 256, generator=g) * 1.5).to(dtype)
    s = qo.find_scale_int4(x)
    x_int = torch.empty(4, 256, dtype=torch.int8)
    xd = x.clone()
    qo.quantize_int4(xd, s, x_int, None, None, True)
    for r in range(4):
        sf = Fraction(float(s[r]))
        for q, d in zip(x_int[r].tolist()[:64], xd[r].tolist()[:64]):
            inner = Fraction(float(np.float32(float(q * sf + sf / 2))))      # one fp32 rounding of the exact sum
            assert d == round_to(dtype, inner)
    cd, ci, _, _ = c_oracle.quantize_int4(x, s, True)
    assert torch.equal(cd, xd) and torch.equal(ci, x_int)


# --------------------------------------------------------------------------- G1 / E1 / L1
def test_int_gemm_tiny_by_hand():
    a = torch.tensor([[1, -2, 3, -8]], dtype=torch.int8)
    b = torch.tensor([[7, 7, -8, -8], [0, 1, 0, -1]], dtype=torch.int8)
    c = qo.matmul_int4_int4t_int32(qo.pack_int4(a), qo.pack_int4(b))
    assert c.tolist() == [[7 - 14 - 24 + 64, -2 + 8]]


@pytest.mark.parametrize('shape', [(5, 64, 7), (33, 256, 17), (16, 1024, 48)])
def test_int_gemm_three_ways(c_oracle, shape):
    m, k, n = shape
    g = torch.Generator().manual_seed(8)
    a = torch.randint(-8, 8, (m, k), generator=g).to(torch.int8)
    b = torch.randint(-8, 8, (n, k), generator=g).to(torch.int8)
    ap, bp = qo.pack_int4(a), qo.pack_int4(b)
    want = (a.to(torch.int64) @ b.to(torch.int64).t()).to(torch.int32)
    assert torch.equal(qo.matmul_int4_int4t_int32(ap, bp, 'fp64'), want)
    assert torch.equal(qo.matmul_int4_int4t_int32(ap, bp, 'fp32'), want)
    assert torch.equal(c_oracle.matmul_int4_int4t_int32(ap, bp), want)
    # extreme codes: every product +64, accumulates to 64*K
    a[:] = -8
    b[:] = -8
    assert (qo.matmul_int4_int4t_int32(qo.pack_int4(a), qo.pack_int4(b), 'fp32') == 64 * k).all()


@pytest.mark.parametrize('dtype', DTYPES)
def test_add_mul_vv_closed_form(c_oracle, dtype):
    g = torch.Generator().manual_seed(9)
    m, n = 12, 20
    c = torch.randint(-60000, 60000, (m, n), generator=g, dtype=torch.int32)
    a_add = torch.randint(-4000, 4000, (m, 1), generator=g, dtype=torch.int32)
    b_add = torch.randint(-4000, 4000, (n, 1), generator=g, dtype=torch.int32)
    a_mul = (torch.rand(m, 1, generator=g) * 0.09 + 0.01).to(dtype)
    b_mul = (torch.rand(n, 1, generator=g) * 0.09 + 0.01).to(dtype)
    d = qo.add_mul_vv(a_add, a_mul, b_add, b_mul, c)
    assert torch.equal(d, c_oracle.add_mul_vv(a_add, a_mul, b_add, b_mul, c))
    for i in range(m):
        for j in range(n):
            lhs = 2 * int(c[i, j]) + int(a_add[i]) + int(b_add[j])
            rhs = Fraction(float(a_mul[i])) * Fraction(float(b_mul[j])) / 2        # exact in fp32 for 16-bit inputs
            assert float(np.float32(float(rhs))) == float(rhs)
            prod = Fraction(float(np.float32(np.float32(lhs) * np.float32(float(rhs)))))
            assert float(d[i, j]) == round_to(dtype, prod)


@pytest.mark.parametrize('dtype', DTYPES)
def test_linear_identity_and_forward(dtype):
    """utils.py:667-678 (fp64 identity) and utils.py:715-716 (linear_forward == fp64 product rounded)."""
    g = torch.Generator().manual_seed(0)
    m, k, n = 160, 768, 224
    w = torch.randn(n, k, generator=g).to(dtype)
    x = torch.randn(m, k, generator=g).to(dtype)
    w_packed, w_scale, w_add, _ = qo.preprocess_weight(w)
    a_scale = qo.find_scale_int4(x)
    a_int = torch.empty(m, k, dtype=torch.int8)
    qo.quantize_int4(x, a_scale, a_int, None, None, False)
    w_int = qo.unpack_int4(w_packed)
    assert torch.equal(w_add, w_int.to(torch.int32).sum(-1, keepdim=True) + k // 2)
    m_ref = qo.linear_fp64(a_int, a_scale, w_int, w_scale)
    ident = a_scale.double() * (2. * a_int.double() @ w_int.double().t() + a_int.double().sum(-1, keepdim=True)
                                + w_int.double().sum(-1, keepdim=True).t() + .5 * k) * (.5 * w_scale.double()).t()
    assert torch.equal(ident, m_ref)
    out = qo.linear_forward(x, w_packed, w_scale, w_add, use_hadamard=False)
    want = m_ref.to(dtype)
    diff = (out.view(torch.int16).int() - want.view(torch.int16).int()).abs()
    # fp32-then-16-bit double rounding may move a rare tie by one ulp
    assert diff.max() <= 1 and (diff != 0).float().mean() < 1e-3
    assert ((out.double() - m_ref).norm() / m_ref.norm()) < 1e-2


def test_linear_forward_hadamard_rotation_preserves_product():
    """With both operands rotated by the same orthogonal block transform the un-quantised product is
    unchanged, so the quantised linear must stay close to the fp product."""
    g = torch.Generator().manual_seed(11)
    m, k, n = 64, 512, 96
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(n, k, generator=g) * 0.02).bfloat16()
    wp, ws, wa, _ = qo.preprocess_weight(w, use_hadamard=True)
    exact = x.double() @ w.double().t()
    for had in ('matmul', 'fwht'):
        out = qo.linear_forward(x, wp, ws, wa, use_hadamard=True, hadamard=had)
        rel = (out.double() - exact).norm() / exact.norm()
        assert rel < 0.2          # 4-bit x 4-bit quantisation noise (~0.1 each), not a numerics bar
    a = qo.linear_forward(x, wp, ws, wa, use_hadamard=True, hadamard='matmul')
    b = qo.linear_forward(x, wp, ws, wa, use_hadamard=True, hadamard='fwht')
    assert ((a.double() - b.double()).norm() / a.double().norm()) < 1e-2


# --------------------------------------------------------------------------- the absmax weight-scale rule
def test_absmax_scale_closed_forms():
    """Row maximum 7.5 -> step exactly 1 (+1e-8 vanishes in 16 bits): +7.5 gets code 7, -7.5 code -8, both
    dequantise to +-7.5; a zero row gets the epsilon alone."""
    for dtype in (torch.bfloat16, torch.float16):
        x = torch.tensor([[7.5, -7.5, 0.4, -0.4, 3.0, 0.0, 6.5, -1.0]], dtype=dtype)
        s = qo.find_scale_absmax_int4(x)
        assert float(s) == 1.0
        q = torch.empty(1, 8, dtype=torch.int8)
        qo.quantize_int4(x.clone(), s, q, None, None, False)
        assert q.tolist() == [[7, -8, 0, -1, 3, 0, 6, -1]]
        z = qo.find_scale_absmax_int4(torch.zeros(2, 128, dtype=dtype))
        assert torch.equal(z, torch.full((2, 1), 1e-8).to(dtype))
    x = torch.randn(64, 256, generator=torch.Generator().manual_seed(3)).bfloat16()
    s = qo.find_scale_absmax_int4(x).float()
    amax = x.float().abs().amax(-1, keepdim=True)
    assert ((s - amax / 7.5).abs() <= amax / 7.5 * 2. ** -8).all()


def test_preprocess_weight_absmax_never_clips_beyond_the_grid():
    w = (torch.randn(32, 256, generator=torch.Generator().manual_seed(4)) * 0.02).bfloat16()
    for had in (False, True):
        packed, scale, add, _ = qo.preprocess_weight(w, use_hadamard=had, w_scale_mode='absmax')
        codes = qo.unpack_int4(packed)
        assert codes.min() >= -8 and codes.max() <= 7
        assert torch.equal(add, codes.to(torch.int32).sum(-1, keepdim=True).to(torch.int32) + 128)
        wt = qo.hadamard128_fwht(w, 2. ** -3.5) if had else w
        deq = (codes.float() + .5) * scale.float()
        # inside the grid the error is at most half a step (plus the rounding of the scale itself)
        assert ((deq - wt.float()).abs() <= scale.float() * 0.51).all()


# --------------------------------------------------------------------------- training-side fake quantisation
def test_fake_quant_grid_is_the_inference_grid():
    """The 16 levels of the training-side quantiser, (k - 7.5) step for k = 0..15, are the inference grid
    (q + 1/2) s with q = k - 8 and s = step; round-to-level and floor-to-code pick the same level except at exact
    ties and where the two scale formulas (epsilon inside or outside the product) differ in the last bits."""
    x = torch.randn(64, 512, generator=torch.Generator().manual_seed(11))
    xq, scale, step = qo.fake_quant_hadamard(x)
    assert xq.min() >= 0 and xq.max() <= 15
    deq = xq * step - scale
    assert torch.allclose(deq, (xq - 7.5) * step, atol=1e-6)
    x_had = qo.hadamard128_fwht(x, 2. ** -3.5)
    s = qo.find_scale_int4(x_had)
    assert torch.allclose(s, step, rtol=1e-6)
    codes = torch.empty(64, 512, dtype=torch.int8)
    qo.quantize_int4(x_had.clone(), s, codes, None, None, False)
    assert ((codes.float() + 8) != xq).float().mean() < 1e-3


def test_fake_quant_linear_equals_packed_linear_in_exact_arithmetic():
    """fp32 end to end on both sides (no 16-bit rounding anywhere): the packed path's integer GEMM and scale
    epilogue reproduce the fake-quantised dense product up to the handful of codes on a rounding tie."""
    g = torch.Generator().manual_seed(12)
    x = torch.randn(32, 256, generator=g)
    w = torch.randn(48, 256, generator=g) * 0.02
    want = qo.fake_quant_linear(x, w)
    xq, xs, xstep = qo.fake_quant_hadamard(x)
    wq, ws, wstep = qo.fake_quant_hadamard(w)
    a, b = (xq - 8).to(torch.int64), (wq - 8).to(torch.int64)
    c = a @ b.t()
    lhs = (2 * c + a.sum(-1, keepdim=True) + (b.sum(-1, keepdim=True) + 128).t()).double()
    got = lhs * (0.5 * xstep.double() * wstep.double().t())
    assert torch.allclose(got, want.double(), rtol=1e-4, atol=1e-6)


# --------------------------------------------------------------------------- E2M3 tiles (the FP6 GEMM's operand form)
def test_e2m3_values_are_the_ocp_fp6_table():
    """OCP Microscaling Formats (MX) v1.0, FP6 E2M3: bias 1, no Inf / NaN; max normal 7.5, min normal 1.0, max
    subnormal 0.875, min subnormal 0.125 -- and the whole table built from exact fractions, not from the oracle's
    formula."""
    v = qo.e2m3_value(torch.arange(64))
    assert float(v[0b011111]) == 7.5 and float(v[0b001000]) == 1.0 and float(v[0b000111]) == 0.875 and float(v[0b000001]) == 0.125
    assert float(v[0b100100]) == -0.5 and float(v[0b111111]) == -7.5 and float(v[0]) == 0.0 and float(v[0b010000]) == 2.0
    for bits in range(64):
        e, m = (bits >> 3) & 3, bits & 7
        mag = Fraction(m, 8) if e == 0 else Fraction(8 + m, 8) * Fraction(2) ** (e - 1)
        assert Fraction(float(v[bits])) == (-mag if bits & 32 else mag)
    pos = v[:32]
    assert bool((pos[1:] > pos[:-1]).all())                       # monotone in the magnitude bits


def test_e2m3_code_patterns_hold_q_plus_half():
    """Every INT4 code has exactly one pattern, its value is q + 1/2, and the patterns are the eight magnitudes
    {0.5, 1.5, ..., 7.5} with the sign bit for negative codes (q and -q - 1 share a magnitude)."""
    q = torch.arange(-8, 8)
    bits = qo.e2m3_bits_of_code(q)
    assert torch.equal(qo.e2m3_value(bits), q.double() + 0.5)
    assert bits[8:].tolist() == [0b000100, 0b001100, 0b010010, 0b010110, 0b011001, 0b011011, 0b011101, 0b011111]
    assert torch.equal(bits[:8].flip(0), bits[8:] | 32)
    table = qo.e2m3_value(torch.arange(64))
    for c in q.tolist():
        assert int((table == c + 0.5).sum()) == 1


def test_e2m3_tiles_layout_bit_by_bit():
    """One nonzero code at a time: its six bits land where the layout says -- fragment (row / 32, k / 64), lane
    32 * ((k % 64) / 32) + row % 32, bit 6 * (k % 32) of the lane's 24 bytes, whose first 16 sit at byte 16 * lane and
    whose last 8 at byte 1024 + 8 * lane of the fragment's 1536.  Everything else holds the pattern of code 0 there."""
    rows, k = 40, 192
    base = qo.e2m3_tiles_encode(torch.zeros(rows, k, dtype=torch.int8))
    assert base.numel() == 2 * 3 * 1536
    zero_pat = 0b000100                                           # 0 + 1/2
    for (r, c, code) in [(0, 0, 7), (0, 5, -8), (31, 63, 3), (33, 64, -1), (39, 191, 6), (17, 100, -5), (5, 21, 2), (6, 26, -3)]:
        x = torch.zeros(rows, k, dtype=torch.int8)
        x[r, c] = code
        t = qo.e2m3_tiles_encode(x)
        diff = (t != base).nonzero().flatten().tolist()
        frag, lane, bit = (r // 32) * (k // 64) + c // 64, 32 * ((c % 64) // 32) + r % 32, 6 * (c % 32)
        pat = {7: 0b011111, -8: 0b111111, 3: 0b010110, -1: 0b100100, 6: 0b011101, -5: 0b111001, 2: 0b010010, -3: 0b110010}[code]
        want = set()
        for b in range(6):
            if ((pat ^ zero_pat) >> b) & 1:
                byte_in_lane = (bit + b) // 8
                want.add(frag * 1536 + (16 * lane + byte_in_lane if byte_in_lane < 16 else 1024 + 8 * lane + byte_in_lane - 16))
        assert set(diff) == want, (r, c, code)
        # and the bits themselves
        lane_bytes = torch.cat((t[frag * 1536 + 16 * lane:frag * 1536 + 16 * lane + 16], t[frag * 1536 + 1024 + 8 * lane:frag * 1536 + 1024 + 8 * lane + 8]))
        word = int.from_bytes(bytes(lane_bytes.tolist()), 'little')
        assert (word >> bit) & 63 == pat


def test_e2m3_tiles_round_trip_and_padding():
    g = torch.Generator().manual_seed(5)
    for rows, k in [(1, 64), (32, 128), (45, 256), (100, 64)]:
        x = torch.randint(-8, 8, (rows, k), generator=g, dtype=torch.int8)
        t = qo.e2m3_tiles_encode(x)
        assert t.numel() == ((rows + 31) // 32) * (k // 64) * 1536
        assert torch.equal(qo.e2m3_tiles_decode(t, rows, k), x.double() + 0.5)
        # a product of decoded tiles is sum (qa + 1/2)(qb + 1/2): twice it is 2 C + sum qa + sum qb + K / 2
        y = torch.randint(-8, 8, (7, k), generator=g, dtype=torch.int8)
        s = qo.e2m3_tiles_decode(t, rows, k) @ qo.e2m3_tiles_decode(qo.e2m3_tiles_encode(y), 7, k).T
        c = x.double() @ y.double().T
        assert torch.equal(2 * s, 2 * c + x.double().sum(1, keepdim=True) + y.double().sum(1)[None, :] + k / 2)
