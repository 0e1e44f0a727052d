/*
 * Scalar C restatement of the W4A4 linear path of QuEST's gemm-quest package.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE: it is the independent second opinion the
 * tests hold the torch oracle (oracle/quest_oracle.py) and the HIP kernels against.  No
 * torch, no vector code, one loop per definition.  Build: `make -C oracle` (needs
 * -ffp-contract=off so that no multiply-add is fused behind the definitions' back).
 *
 * Reference lines followed (paths under /root/reference/gemm-quest/):
 *   qo_find_scale_int4         quest/quantize_kernel.cu:81-92, benchmarks/utils.py:207-208
 *   qo_quantize_int4           quest/quantize_kernel.cu:155-163,199-200, benchmarks/utils.py:342-363
 *   qo_unpack_int4             benchmarks/utils.py:441-445
 *   qo_add_mul_vv              quest/quantize_kernel.cu:299-304, benchmarks/utils.py:544
 *   qo_matmul_int4_int4t_int32 quest/matmul_kernel.cu:8-63 (C = A * B^T on signed nibbles)
 *   qo_hadamard128_matmul      benchmarks/utils.py:17,89-90
 *   qo_hadamard128_fwht        benchmarks/utils.py:38-39 (fast_hadamard_transform's definition)
 *
 * dtype: 0 = bfloat16, 1 = float16 (IEEE binary16).  All 16-bit floats travel as uint16_t.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

float qo_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

uint16_t qo_f32_to_bf16(float f) {          /* round to nearest even; NaN stays NaN */
    uint32_t u = f32_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

float qo_fp16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu, man = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0) return bits_f32(sign);
        float v = (float)man * (1.0f / 16777216.0f);     /* man * 2^-24, exact */
        return sign ? -v : v;
    }
    if (exp == 31) return bits_f32(sign | 0x7f800000u | (man << 13));
    return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

uint16_t qo_f32_to_fp16(float f) {          /* round to nearest even */
    uint32_t u = f32_bits(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
    if (a >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);       /* >= 65520 -> inf */
    if (a < 0x33000001u) return sign;                               /* <= 2^-25 -> 0 */
    int e = (int)(a >> 23) - 127;
    uint32_t man = (a & 0x7fffffu) | 0x800000u;
    int shift = (e < -14) ? (13 + (-14 - e)) : 13;                  /* bits dropped */
    uint32_t kept = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (kept & 1u))) kept++;
    uint32_t out;
    if (e < -14) out = kept;                                        /* subnormal (may carry into normal) */
    else out = ((uint32_t)(e + 15) << 10) + (kept - 0x400u);        /* carry propagates into exponent */
    return (uint16_t)(sign | out);
}

static float load16(const uint16_t *p, int dtype) { return dtype ? qo_fp16_to_f32(*p) : qo_bf16_to_f32(*p); }
static uint16_t store16(float f, int dtype) { return dtype ? qo_f32_to_fp16(f) : qo_f32_to_bf16(f); }

/* ---- Hadamard ---------------------------------------------------------------------- */
static int parity7(int v) { v ^= v >> 4; v ^= v >> 2; v ^= v >> 1; return v & 1; }

/* y[r, blk*128 + j] = dtype( sum_i x[r, blk*128 + i] * h(i, j) ), h = +-entry, fp32 running sum
 * over i = 0..127 in index order.  `entry` is 181/2048 for the reference's bf16 matrix. */
void qo_hadamard128_matmul(uint16_t *y, const uint16_t *x, long rows, long k, float entry, int dtype) {
    for (long r = 0; r < rows; r++)
        for (long b = 0; b < k; b += 128)
            for (int j = 0; j < 128; j++) {
                float acc = 0.f;
                for (int i = 0; i < 128; i++) {
                    float h = parity7(i & j) ? -entry : entry;
                    acc = acc + load16(&x[r * k + b + i], dtype) * h;
                }
                y[r * k + b + j] = store16(acc, dtype);
            }
}

/* In-place radix-2 butterflies at distance 1, 2, 4, ... 64, then * scale, then one rounding. */
void qo_hadamard128_fwht(uint16_t *y, const uint16_t *x, long rows, long k, float scale, int dtype) {
    float v[128];
    for (long r = 0; r < rows; r++)
        for (long b = 0; b < k; b += 128) {
            for (int i = 0; i < 128; i++) v[i] = load16(&x[r * k + b + i], dtype);
            for (int h = 1; h < 128; h <<= 1)
                for (int i = 0; i < 128; i += 2 * h)
                    for (int j = i; j < i + h; j++) {
                        float a = v[j], c = v[j + h];
                        v[j] = a + c;
                        v[j + h] = a - c;
                    }
            for (int i = 0; i < 128; i++) y[r * k + b + i] = store16(v[i] * scale, dtype);
        }
}

/* ---- scale ------------------------------------------------------------------------- */
/* order: 0 = fp32 running sum in index order; 1 = double accumulation rounded once to fp32
 * (what an order-free exact reduction would give, up to 1 fp32 ulp). */
void qo_find_scale_int4(uint16_t *scale, const uint16_t *x, long rows, long k, int dtype, int order) {
    const float factor = (float)(2.513930578568423 * 2. / 15.);
    for (long r = 0; r < rows; r++) {
        float sum;
        if (order == 0) {
            float s = 0.f;
            for (long i = 0; i < k; i++) { float v = load16(&x[r * k + i], dtype); s = s + v * v; }
            sum = s;
        } else {
            double s = 0.;
            for (long i = 0; i < k; i++) { double v = load16(&x[r * k + i], dtype); s += v * v; }
            sum = (float)s;
        }
        float mean_sq = sum / (float)k;
        float sd = sqrtf(mean_sq);
        float prod = sd * factor;
        scale[r] = store16(prod + 1e-8f, dtype);
    }
}

/* ---- quantise / pack / row sum ----------------------------------------------------- */
void qo_quantize_int4(uint16_t *x, const uint16_t *scale, int8_t *x_int, uint8_t *x_packed,
                      int32_t *row_sum, long rows, long k, int do_dequantize, int dtype) {
    for (long r = 0; r < rows; r++) {
        float s = load16(&scale[r], dtype);
        int32_t sum = 0;
        for (long i = 0; i < k; i += 2) {
            int8_t q[2];
            for (int e = 0; e < 2; e++) {
                float xf = load16(&x[r * k + i + e], dtype);
                float qf = floorf(xf / s);
                qf = fmaxf(qf, -8.f);
                qf = fminf(qf, 7.f);
                q[e] = (int8_t)(int)qf;
                if (do_dequantize) {
                    float a = qf * s, h = s * 0.5f;
                    x[r * k + i + e] = store16(a + h, dtype);
                }
                if (x_int) x_int[r * k + i + e] = q[e];
                sum += q[e];
            }
            if (x_packed) x_packed[r * (k / 2) + i / 2] = (uint8_t)(((uint8_t)q[1] << 4) | ((uint8_t)q[0] & 0x0f));
        }
        if (row_sum) row_sum[r] = sum;
    }
}

void qo_unpack_int4(int8_t *x_int, const uint8_t *x_packed, long n_bytes) {
    for (long i = 0; i < n_bytes; i++) {
        int lo = x_packed[i] & 0xf, hi = x_packed[i] >> 4;
        x_int[2 * i] = (int8_t)(lo >= 8 ? lo - 16 : lo);
        x_int[2 * i + 1] = (int8_t)(hi >= 8 ? hi - 16 : hi);
    }
}

/* ---- integer GEMM and the scale epilogue ------------------------------------------- */
void qo_matmul_int4_int4t_int32(int32_t *c, const uint8_t *a, const uint8_t *b, long m, long k, long n) {
    int8_t *au = (int8_t *)malloc((size_t)m * k), *bu = (int8_t *)malloc((size_t)n * k);
    qo_unpack_int4(au, a, m * k / 2);
    qo_unpack_int4(bu, b, n * k / 2);
    for (long i = 0; i < m; i++)
        for (long j = 0; j < n; j++) {
            int32_t acc = 0;
            for (long t = 0; t < k; t++) acc += (int32_t)au[i * k + t] * (int32_t)bu[j * k + t];
            c[i * n + j] = acc;
        }
    free(au);
    free(bu);
}

void qo_add_mul_vv(uint16_t *d, const int32_t *a_add, const uint16_t *a_mul, const int32_t *b_add,
                   const uint16_t *b_mul, const int32_t *c, long m, long n, int dtype) {
    for (long i = 0; i < m; i++)
        for (long j = 0; j < n; j++) {
            float lhs = (float)(c[i * n + j] * 2 + a_add[i] + b_add[j]);
            float half_a = 0.5f * load16(&a_mul[i], dtype);
            float rhs = half_a * load16(&b_mul[j], dtype);
            d[i * n + j] = store16(lhs * rhs, dtype);
        }
}
