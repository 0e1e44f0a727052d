// Row-wise kernels of the W4A4 linear path for gfx950: the Gaussian-clip scale, the INT4
// quantiser with nibble packing and row sums, the scale epilogue on an int32 matrix, the
// block-128 Walsh-Hadamard transform, and the single-pass fusion of Hadamard + scale +
// quantise + pack that the linear layer uses.  All are HBM-bound: every row is read once with
// 16-byte loads per lane and kept in registers until its outputs are written.
//
// Reference statements of the same arithmetic (file:line under gemm-quest/ of the reference):
//   scale      quest/quantize_kernel.cu:38-94,   benchmarks/utils.py:193-209
//   quantise   quest/quantize_kernel.cu:120-229, benchmarks/utils.py:334-365
//   epilogue   quest/quantize_kernel.cu:264-306, benchmarks/utils.py:535-545
//   Hadamard   benchmarks/utils.py:17,38-39,89-90
#include "common.h"

namespace quest {

// ---------------------------------------------------------------------------------------------
// Walsh-Hadamard butterflies on one 16-byte chunk per lane.  A 128-element block is spread over
// 16 consecutive lanes x 8 registers: distances 1, 2, 4 are inside the lane, 8, 16, 32, 64 are
// lane xor 1, 2, 4, 8.  Each butterfly is (a, b) -> (a + b, a - b) with `a` the element at the
// lower index, so the result is the same bit pattern as the textbook in-place loop.
// ---------------------------------------------------------------------------------------------
template <int M>
__device__ __forceinline__ void fwht_lane_stage(float (&v)[8], uint32_t sign) {
#pragma unroll
    for (int e = 0; e < 8; e++) {
        float other = lane_xor_f<M>(v[e]);
        float self = __uint_as_float(__float_as_uint(v[e]) ^ sign);   // -own on the upper lane
        v[e] = self + other;                                            // lower: a + b, upper: a - b
    }
}

__device__ __forceinline__ void fwht128_chunk(float (&v)[8], int lane) {
#pragma unroll
    for (int h = 1; h < 8; h <<= 1) {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            if ((j & h) == 0) {
                float a = v[j], b = v[j + h];
                v[j] = a + b;
                v[j + h] = a - b;
            }
        }
    }
    fwht_lane_stage<1>(v, (lane & 1) ? 0x80000000u : 0u);
    fwht_lane_stage<2>(v, (lane & 2) ? 0x80000000u : 0u);
    fwht_lane_stage<4>(v, (lane & 4) ? 0x80000000u : 0u);
    fwht_lane_stage<8>(v, (lane & 8) ? 0x80000000u : 0u);
}

template <int DT>
__device__ __forceinline__ void unpack8(const uint4 &raw, float (&v)[8]) {
    v[0] = lo_f32<DT>(raw.x); v[1] = hi_f32<DT>(raw.x);
    v[2] = lo_f32<DT>(raw.y); v[3] = hi_f32<DT>(raw.y);
    v[4] = lo_f32<DT>(raw.z); v[5] = hi_f32<DT>(raw.z);
    v[6] = lo_f32<DT>(raw.w); v[7] = hi_f32<DT>(raw.w);
}

template <int DT>
__device__ __forceinline__ uint4 pack8(const float (&v)[8]) {
    uint4 r;
    r.x = pack2_from_f32<DT>(v[0], v[1]);
    r.y = pack2_from_f32<DT>(v[2], v[3]);
    r.z = pack2_from_f32<DT>(v[4], v[5]);
    r.w = pack2_from_f32<DT>(v[6], v[7]);
    return r;
}

// eight codes (as floats in [-8, 7]) -> one dword, element 0 in the lowest nibble
__device__ __forceinline__ uint32_t pack_nibbles8(const float (&q)[8], int &sum) {
    uint32_t w = 0;
#pragma unroll
    for (int e = 0; e < 8; e++) {
        int c = (int)q[e];
        sum += c;
        w |= ((uint32_t)c & 0xFu) << (4 * e);
    }
    return w;
}

// ---------------------------------------------------------------------------------------------
// Fused Hadamard + scale + quantise + pack: one workgroup per row, NCHUNK 16-byte chunks per
// thread, the row lives in registers between its single read and its writes.
// ---------------------------------------------------------------------------------------------
template <int DT, int NCHUNK, int BLOCK>
__global__ void __launch_bounds__(BLOCK)
hadamard_quantize_kernel(const uint16_t *__restrict__ x, uint16_t *__restrict__ scale,
                         uint32_t *__restrict__ packed, int32_t *__restrict__ row_sum,
                         uint16_t *__restrict__ x_had, int K, float had_scale, int scale_rule) {
    __shared__ float slots_f[BLOCK / 64];
    __shared__ int slots_i[BLOCK / 64];
    const int row = blockIdx.x;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int nchunks = K >> 3;
    const uint4 *xr = reinterpret_cast<const uint4 *>(x + (size_t)row * K);
    // QUEST_QUANT_FROM_FP32: scale and codes come from the transform's fp32 output and the unrounded scale -- the
    // arithmetic of the reference's evaluation-side fake quantiser (src/eval_hswag.py:201-214), which never holds the
    // rotated tensor in 16 bits -- instead of from the dtype-rounded tensor the inference path materialises
    const bool from_fp32 = (scale_rule & QUEST_QUANT_FROM_FP32) != 0;
    scale_rule &= ~QUEST_QUANT_FROM_FP32;

    uint4 raw[NCHUNK];
#pragma unroll
    for (int i = 0; i < NCHUNK; i++) {
        const int c = i * BLOCK + tid;
        raw[i] = (c < nchunks) ? xr[c] : make_uint4(0, 0, 0, 0);
    }

    float y[NCHUNK][8];
    float sumsq = 0.f, amax = 0.f;
#pragma unroll
    for (int i = 0; i < NCHUNK; i++) {
        unpack8<DT>(raw[i], y[i]);
        if (had_scale != 0.f) {
            fwht128_chunk(y[i], lane);
#pragma unroll
            for (int e = 0; e < 8; e++) y[i][e] *= had_scale;
            raw[i] = pack8<DT>(y[i]);           // the transform's output exists only in dtype ...
            if (!from_fp32) unpack8<DT>(raw[i], y[i]);     // ... unless the caller asks for the fp32 one to be quantised
        }
#pragma unroll
        for (int e = 0; e < 8; e++) {
            sumsq += y[i][e] * y[i][e];         // squares of 16-bit floats are exact in fp32
            amax = fmaxf(amax, fabsf(y[i][e]));
        }
    }
    if (x_had != nullptr) {
        uint4 *hr = reinterpret_cast<uint4 *>(x_had + (size_t)row * K);
#pragma unroll
        for (int i = 0; i < NCHUNK; i++) {
            const int c = i * BLOCK + tid;
            if (c < nchunks) hr[c] = raw[i];
        }
    }

    // QUEST_SCALE_GAUSSIAN: the reference's rule from the row's mean square; QUEST_SCALE_ABSMAX: the row's largest
    // magnitude sits 7.5 steps out (a maximum is exact whatever the order, so this scale has no rounding slack)
    float s32;
    if (scale_rule == QUEST_SCALE_ABSMAX) {
        const float m = block_max_f<BLOCK>(amax, slots_f);
        s32 = __fadd_rn(__fdiv_rn(m, 7.5f), kScaleEps);
    } else {
        const float total = block_sum_f<BLOCK>(sumsq, slots_f);
        s32 = scale_from_sumsq(total, K);
    }
    const uint32_t s16 = from_f32<DT>(s32);
    if (tid == 0) scale[row] = (uint16_t)s16;
    const float s = from_fp32 ? s32 : to_f32<DT>(s16);

    if (packed == nullptr && row_sum == nullptr) return;
    const float inv = quant_inv(s);
    int isum = 0;
#pragma unroll
    for (int i = 0; i < NCHUNK; i++) {
        float q[8];
#pragma unroll
        for (int e = 0; e < 8; e++) q[e] = quant_code_inv(y[i][e], inv);
        int csum = 0;
        const uint32_t w = pack_nibbles8(q, csum);
        const int c = i * BLOCK + tid;
        if (c < nchunks) {                      // chunks past the row's end are padding
            isum += csum;
            if (packed != nullptr) packed[(size_t)row * nchunks + c] = w;
        }
    }
    if (row_sum != nullptr) {
        const int t = block_sum_i<BLOCK>(isum, slots_i);
        if (tid == 0) row_sum[row] = t;
    }
}

// ---------------------------------------------------------------------------------------------
// Stand-alone Hadamard (weights offline; activations when the caller wants the unfused steps)
// ---------------------------------------------------------------------------------------------
template <int DT>
__global__ void __launch_bounds__(256)
hadamard128_kernel(uint16_t *__restrict__ y, const uint16_t *__restrict__ x, long nchunks_total, float had_scale) {
    const int lane = threadIdx.x & 63;
    // 16 consecutive chunks (= threads) make one block; the grid strides in multiples of 256 threads
    for (long c = (long)blockIdx.x * 256 + threadIdx.x; c < nchunks_total; c += (long)gridDim.x * 256) {
        uint4 raw = reinterpret_cast<const uint4 *>(x)[c];
        float v[8];
        unpack8<DT>(raw, v);
        fwht128_chunk(v, lane);
#pragma unroll
        for (int e = 0; e < 8; e++) v[e] *= had_scale;
        reinterpret_cast<uint4 *>(y)[c] = pack8<DT>(v);
    }
}

// ---------------------------------------------------------------------------------------------
// Scale only
// ---------------------------------------------------------------------------------------------
template <int DT>
__global__ void __launch_bounds__(256)
find_scale_kernel(uint16_t *__restrict__ scale, const uint16_t *__restrict__ x, int K) {
    __shared__ float slots_f[4];
    const int row = blockIdx.x;
    const int nchunks = K >> 3;
    const uint4 *xr = reinterpret_cast<const uint4 *>(x + (size_t)row * K);
    float sumsq = 0.f;
    for (int c = threadIdx.x; c < nchunks; c += 256) {
        float v[8];
        unpack8<DT>(xr[c], v);
#pragma unroll
        for (int e = 0; e < 8; e++) sumsq += v[e] * v[e];
    }
    const float total = block_sum_f<256>(sumsq, slots_f);
    if (threadIdx.x == 0) scale[row] = (uint16_t)from_f32<DT>(scale_from_sumsq(total, K));
}

// ---------------------------------------------------------------------------------------------
// Quantise with a given scale; every output optional
// ---------------------------------------------------------------------------------------------
template <int DT>
__global__ void __launch_bounds__(256)
quantize_kernel(uint16_t *__restrict__ x, const uint16_t *__restrict__ scale, int8_t *__restrict__ x_int,
                uint32_t *__restrict__ packed, int32_t *__restrict__ row_sum, int K, int do_dequantize) {
    __shared__ int slots_i[4];
    const int row = blockIdx.x;
    const int nchunks = K >> 3;
    uint4 *xr = reinterpret_cast<uint4 *>(x + (size_t)row * K);
    const float s = to_f32<DT>(scale[row]);
    const float half_s = __fmul_rn(s, 0.5f);
    const float inv = quant_inv(s);
    // scales in the fast range take the clamp-free form of the quantiser (in its variant for arbitrary inputs: this
    // entry point pairs any x with any scale), the others the med3 form; both equal the IEEE-divide statement
    const bool fast = quant_fast_ok(s);
    const float inv28 = quant_inv28(s);
    int isum = 0;
    // two chunks per thread and pass, both loads issued before either is used (a row of 4096 is exactly one pass)
    for (int c0 = threadIdx.x; c0 < nchunks; c0 += 512) {
        const int c1 = c0 + 256;
        const bool two = c1 < nchunks;
        uint4 raw[2];
        raw[0] = xr[c0];
        raw[1] = two ? xr[c1] : make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int u = 0; u < 2; u++) {
            if (u == 1 && !two) break;
            const int c = u == 0 ? c0 : c1;
            float v[8], q[8];
            unpack8<DT>(raw[u], v);
            if (fast) {
#pragma unroll
                for (int e = 0; e < 8; e++) q[e] = (float)(quant_top_nibble_any(v[e], inv28) >> 28);
            } else {
#pragma unroll
                for (int e = 0; e < 8; e++) q[e] = quant_code_inv(v[e], inv);
            }
            if (do_dequantize) {
#pragma unroll
                for (int e = 0; e < 8; e++) v[e] = __fadd_rn(__fmul_rn(q[e], s), half_s);
                xr[c] = pack8<DT>(v);
            }
            const uint32_t w = pack_nibbles8(q, isum);
            if (packed != nullptr) packed[(size_t)row * nchunks + c] = w;
            if (x_int != nullptr) {
                uint2 b;
                b.x = ((uint32_t)(int)q[0] & 0xFFu) | (((uint32_t)(int)q[1] & 0xFFu) << 8) |
                      (((uint32_t)(int)q[2] & 0xFFu) << 16) | (((uint32_t)(int)q[3] & 0xFFu) << 24);
                b.y = ((uint32_t)(int)q[4] & 0xFFu) | (((uint32_t)(int)q[5] & 0xFFu) << 8) |
                      (((uint32_t)(int)q[6] & 0xFFu) << 16) | (((uint32_t)(int)q[7] & 0xFFu) << 24);
                reinterpret_cast<uint2 *>(x_int + (size_t)row * K)[c] = b;
            }
        }
    }
    if (row_sum != nullptr) {
        const int t = block_sum_i<256>(isum, slots_i);
        if (threadIdx.x == 0) row_sum[row] = t;
    }
}

// ---------------------------------------------------------------------------------------------
// Scale epilogue on an int32 matrix (the unfused debug path)
// ---------------------------------------------------------------------------------------------
template <int DT>
__global__ void __launch_bounds__(256)
add_mul_vv_kernel(uint16_t *__restrict__ d, const int32_t *__restrict__ a_add, const uint16_t *__restrict__ a_mul,
                  const int32_t *__restrict__ b_add, const uint16_t *__restrict__ b_mul,
                  const int32_t *__restrict__ c, int size_a, int size_b) {
    const int col_blocks = (size_b + 255) / 256;
    const int row = blockIdx.x / col_blocks;
    const int col = (blockIdx.x % col_blocks) * 256 + threadIdx.x;
    if (row >= size_a || col >= size_b) return;
    const size_t idx = (size_t)row * size_b + col;
    const float lhs = (float)(c[idx] * 2 + a_add[row] + b_add[col]);
    const float rhs = __fmul_rn(__fmul_rn(0.5f, to_f32<DT>(a_mul[row])), to_f32<DT>(b_mul[col]));
    d[idx] = (uint16_t)from_f32<DT>(__fmul_rn(lhs, rhs));
}

// ---------------------------------------------------------------------------------------------
// launchers
// ---------------------------------------------------------------------------------------------
template <int DT>
static int launch_hadamard_quantize(const void *x, void *scale, uint8_t *packed, int32_t *row_sum, void *x_had,
                                    int K, int M, float had_scale, int scale_rule, hipStream_t st) {
    const int nchunks = K >> 3;
#define QUEST_HQ(NCH, BLK)                                                                              \
    hadamard_quantize_kernel<DT, NCH, BLK><<<dim3(M), dim3(BLK), 0, st>>>(                              \
        (const uint16_t *)x, (uint16_t *)scale, (uint32_t *)packed, row_sum, (uint16_t *)x_had, K, had_scale, scale_rule)
    if (nchunks <= 256) QUEST_HQ(1, 256);
    else if (nchunks <= 512) QUEST_HQ(2, 256);
    else if (nchunks <= 1024) QUEST_HQ(4, 256);
    else if (nchunks <= 2048) QUEST_HQ(8, 256);
    else if (nchunks <= 8192) QUEST_HQ(8, 1024);
    else return QUEST_ERR_UNSUPPORTED;
#undef QUEST_HQ
    return launch_status();
}

// Rotary position embedding on interleaved pairs, in place (src/models/llama.py:43-62 of the reference): the first
// n_heads * head_dim elements of every row are heads of (re, im) pairs; pair i of a head at position t turns by the
// angle whose (cos, sin) is freqs[t][i].  fp32 products and sums in the reference's order, one rounding to dtype.
template <int DT>
__global__ void __launch_bounds__(256)
rope_kernel(uint16_t *__restrict__ x, const float *__restrict__ freqs, int n_rows, int seq_len, int row_stride,
            int rot_cols, int head_dim) {
    const int chunks = rot_cols >> 3;                        // 16-byte chunks (4 pairs) to rotate per row
    const long idx = (long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (long)n_rows * chunks) return;
    const int row = (int)(idx / chunks);
    const int col = (int)(idx % chunks) * 8;
    const int t = row % seq_len;
    const int pair0 = (col % head_dim) >> 1;
    uint4 *p = reinterpret_cast<uint4 *>(x + (size_t)row * row_stride + col);
    const float4 *f = reinterpret_cast<const float4 *>(freqs + ((size_t)t * (head_dim >> 1) + pair0) * 2);
    const uint4 v = *p;
    const float4 f01 = f[0], f23 = f[1];
    const uint32_t in[4] = {v.x, v.y, v.z, v.w};
    const float cs[4][2] = {{f01.x, f01.y}, {f01.z, f01.w}, {f23.x, f23.y}, {f23.z, f23.w}};
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float re = lo_f32<DT>(in[i]), im = hi_f32<DT>(in[i]);
        const float c = cs[i][0], sn = cs[i][1];
        const float out_re = __fsub_rn(__fmul_rn(re, c), __fmul_rn(im, sn));
        const float out_im = __fadd_rn(__fmul_rn(re, sn), __fmul_rn(im, c));
        o[i] = from_f32<DT>(out_re) | (from_f32<DT>(out_im) << 16);
    }
    *p = make_uint4(o[0], o[1], o[2], o[3]);
}

}  // namespace quest

using namespace quest;

extern "C" int quest_find_scale_int4(void *scale, const void *x, int group_size, int batch_size, int dtype, void *stream) {
    forget_stale_error();
    if (!scale || !x) return QUEST_ERR_NULL_POINTER;
    if (!check_dtype(dtype)) return QUEST_ERR_BAD_DTYPE;
    if (group_size <= 0 || batch_size <= 0 || (group_size & 7)) return QUEST_ERR_BAD_SHAPE;
    if (!aligned(x, 16)) return QUEST_ERR_ALIGNMENT;
    hipStream_t st = (hipStream_t)stream;
    if (dtype == QUEST_DTYPE_BF16)
        find_scale_kernel<0><<<dim3(batch_size), dim3(256), 0, st>>>((uint16_t *)scale, (const uint16_t *)x, group_size);
    else
        find_scale_kernel<1><<<dim3(batch_size), dim3(256), 0, st>>>((uint16_t *)scale, (const uint16_t *)x, group_size);
    return launch_status();
}

extern "C" int quest_quantize_int4(void *x, const void *scale, int8_t *x_int, uint8_t *x_int_packed,
                                   int32_t *x_int_row_sum, int group_size, int batch_size, int do_dequantize,
                                   int dtype, void *stream) {
    forget_stale_error();
    if (!x || !scale) return QUEST_ERR_NULL_POINTER;
    if (!check_dtype(dtype)) return QUEST_ERR_BAD_DTYPE;
    if (group_size <= 0 || batch_size <= 0 || (group_size & 7)) return QUEST_ERR_BAD_SHAPE;
    if (!aligned(x, 16) || !aligned(x_int, 8) || !aligned(x_int_packed, 4)) return QUEST_ERR_ALIGNMENT;
    hipStream_t st = (hipStream_t)stream;
    if (dtype == QUEST_DTYPE_BF16)
        quantize_kernel<0><<<dim3(batch_size), dim3(256), 0, st>>>((uint16_t *)x, (const uint16_t *)scale, x_int,
                                                                    (uint32_t *)x_int_packed, x_int_row_sum, group_size, do_dequantize);
    else
        quantize_kernel<1><<<dim3(batch_size), dim3(256), 0, st>>>((uint16_t *)x, (const uint16_t *)scale, x_int,
                                                                    (uint32_t *)x_int_packed, x_int_row_sum, group_size, do_dequantize);
    return launch_status();
}

// Eight consecutive columns per thread (32 + 32 + 16 bytes in, 16 out, all as 16-byte vectors): for matrices whose rows are
// whole eights and 16-byte aligned.  Same arithmetic per element as the kernel above.
template <int DT>
__global__ void __launch_bounds__(256)
add_mul_vv_x8_kernel(uint16_t *__restrict__ d, const int32_t *__restrict__ a_add, const uint16_t *__restrict__ a_mul,
                     const int32_t *__restrict__ b_add, const uint16_t *__restrict__ b_mul,
                     const int32_t *__restrict__ c, int size_a, int size_b) {
    const int chunks = size_b >> 3;                                   // per row
    const int col_blocks = (chunks + 255) / 256;
    const int row = blockIdx.x / col_blocks;
    const int chunk = (blockIdx.x % col_blocks) * 256 + threadIdx.x;
    if (row >= size_a || chunk >= chunks) return;
    const int col = chunk * 8;
    const size_t idx = (size_t)row * size_b + col;
    const int4 c0 = *reinterpret_cast<const int4 *>(c + idx), c1 = *reinterpret_cast<const int4 *>(c + idx + 4);
    const int4 b0 = *reinterpret_cast<const int4 *>(b_add + col), b1 = *reinterpret_cast<const int4 *>(b_add + col + 4);
    const uint4 bm = *reinterpret_cast<const uint4 *>(b_mul + col);
    const int ra = a_add[row];
    const float half_am = __fmul_rn(0.5f, to_f32<DT>(a_mul[row]));
    const int cs[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
    const int bs[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
    const uint32_t ms[4] = {bm.x, bm.y, bm.z, bm.w};
    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const float l0 = (float)(cs[2 * j] * 2 + ra + bs[2 * j]), l1 = (float)(cs[2 * j + 1] * 2 + ra + bs[2 * j + 1]);
        const float r0 = __fmul_rn(half_am, lo_f32<DT>(ms[j])), r1 = __fmul_rn(half_am, hi_f32<DT>(ms[j]));
        o[j] = (uint32_t)from_f32<DT>(__fmul_rn(l0, r0)) | ((uint32_t)from_f32<DT>(__fmul_rn(l1, r1)) << 16);
    }
    *reinterpret_cast<uint4 *>(d + idx) = make_uint4(o[0], o[1], o[2], o[3]);
}

extern "C" int quest_add_mul_vv(void *mat_d, const int32_t *vec_a_add, const void *vec_a_mul, const int32_t *vec_b_add,
                                const void *vec_b_mul, const int32_t *mat_c, int size_a, int size_b, int dtype,
                                void *stream) {
    forget_stale_error();
    if (!mat_d || !vec_a_add || !vec_a_mul || !vec_b_add || !vec_b_mul || !mat_c) return QUEST_ERR_NULL_POINTER;
    if (!check_dtype(dtype)) return QUEST_ERR_BAD_DTYPE;
    if (size_a <= 0 || size_b <= 0) return QUEST_ERR_BAD_SHAPE;
    hipStream_t st = (hipStream_t)stream;
    if ((size_b & 7) == 0 && aligned(mat_d, 16) && aligned(mat_c, 16) && aligned(vec_b_add, 16) && aligned(vec_b_mul, 16)) {
        const long nb8 = (long)((size_b / 8 + 255) / 256) * size_a;
        if (nb8 > 0x7fffffffL) return QUEST_ERR_UNSUPPORTED;
        if (dtype == QUEST_DTYPE_BF16)
            add_mul_vv_x8_kernel<0><<<dim3((unsigned)nb8), dim3(256), 0, st>>>(
                (uint16_t *)mat_d, vec_a_add, (const uint16_t *)vec_a_mul, vec_b_add, (const uint16_t *)vec_b_mul, mat_c, size_a, size_b);
        else
            add_mul_vv_x8_kernel<1><<<dim3((unsigned)nb8), dim3(256), 0, st>>>(
                (uint16_t *)mat_d, vec_a_add, (const uint16_t *)vec_a_mul, vec_b_add, (const uint16_t *)vec_b_mul, mat_c, size_a, size_b);
        return launch_status();
    }
    const long nblocks = (long)((size_b + 255) / 256) * size_a;
    if (nblocks > 0x7fffffffL) return QUEST_ERR_UNSUPPORTED;
    dim3 grid((unsigned)nblocks);
    if (dtype == QUEST_DTYPE_BF16)
        add_mul_vv_kernel<0><<<grid, dim3(256), 0, st>>>((uint16_t *)mat_d, vec_a_add, (const uint16_t *)vec_a_mul, vec_b_add,
                                                         (const uint16_t *)vec_b_mul, mat_c, size_a, size_b);
    else
        add_mul_vv_kernel<1><<<grid, dim3(256), 0, st>>>((uint16_t *)mat_d, vec_a_add, (const uint16_t *)vec_a_mul, vec_b_add,
                                                         (const uint16_t *)vec_b_mul, mat_c, size_a, size_b);
    return launch_status();
}

extern "C" int quest_hadamard128(void *y, const void *x, int group_size, int batch_size, float had_scale, int dtype,
                                 void *stream) {
    forget_stale_error();
    if (!y || !x) return QUEST_ERR_NULL_POINTER;
    if (!check_dtype(dtype)) return QUEST_ERR_BAD_DTYPE;
    if (group_size <= 0 || batch_size <= 0 || (group_size & 127)) return QUEST_ERR_BAD_SHAPE;
    if (!aligned(x, 16) || !aligned(y, 16)) return QUEST_ERR_ALIGNMENT;
    hipStream_t st = (hipStream_t)stream;
    const long nchunks = (long)batch_size * (group_size >> 3);
    long blocks = (nchunks + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    if (dtype == QUEST_DTYPE_BF16)
        hadamard128_kernel<0><<<dim3((unsigned)blocks), dim3(256), 0, st>>>((uint16_t *)y, (const uint16_t *)x, nchunks, had_scale);
    else
        hadamard128_kernel<1><<<dim3((unsigned)blocks), dim3(256), 0, st>>>((uint16_t *)y, (const uint16_t *)x, nchunks, had_scale);
    return launch_status();
}

extern "C" int quest_hadamard_quantize_int4(const void *x, void *scale, uint8_t *x_int_packed, int32_t *x_int_row_sum,
                                            void *x_had, int group_size, int batch_size, float had_scale, int dtype,
                                            void *stream) {
    forget_stale_error();
    if (!x || !scale) return QUEST_ERR_NULL_POINTER;
    if (!check_dtype(dtype)) return QUEST_ERR_BAD_DTYPE;
    // the transform works on blocks of 128; without it (had_scale == 0) a row only has to be whole 16-byte chunks
    if (group_size <= 0 || batch_size <= 0 || (group_size & (had_scale != 0.f ? 127 : 7))) return QUEST_ERR_BAD_SHAPE;
    if (!aligned(x, 16) || !aligned(x_had, 16) || !aligned(x_int_packed, 4)) return QUEST_ERR_ALIGNMENT;
    hipStream_t st = (hipStream_t)stream;
    // rows of up to 32768 with a Hadamard entry the dtype holds exactly: matrix cores; anything else: butterflies
    const int rc = launch_hadamard_quantize_mfma(0, x, nullptr, 0.f, scale, x_int_packed, x_int_row_sum, x_had, nullptr,
                                                 group_size, batch_size, had_scale, dtype, st);
    if (rc != QUEST_ERR_UNSUPPORTED) return rc;
    if (dtype == QUEST_DTYPE_BF16)
        return launch_hadamard_quantize<0>(x, scale, x_int_packed, x_int_row_sum, x_had, group_size, batch_size, had_scale,
                                           QUEST_SCALE_GAUSSIAN, st);
    return launch_hadamard_quantize<1>(x, scale, x_int_packed, x_int_row_sum, x_had, group_size, batch_size, had_scale,
                                       QUEST_SCALE_GAUSSIAN, st);
}

extern "C" int quest_hadamard_quantize_int4_rule(const void *x, void *scale, uint8_t *x_int_packed, int32_t *x_int_row_sum,
                                                 void *x_had, int group_size, int batch_size, float had_scale,
                                                 int scale_rule, int dtype, void *stream) {
    forget_stale_error();
    if (scale_rule == QUEST_SCALE_GAUSSIAN)
        return quest_hadamard_quantize_int4(x, scale, x_int_packed, x_int_row_sum, x_had, group_size, batch_size, had_scale,
                                            dtype, stream);
    if ((scale_rule & ~QUEST_QUANT_FROM_FP32) != QUEST_SCALE_ABSMAX && (scale_rule & ~QUEST_QUANT_FROM_FP32) != QUEST_SCALE_GAUSSIAN)
        return QUEST_ERR_BAD_SHAPE;
    if (!x || !scale) return QUEST_ERR_NULL_POINTER;
    if (!check_dtype(dtype)) return QUEST_ERR_BAD_DTYPE;
    // the transform works on blocks of 128; without it (had_scale == 0) a row only has to be whole 16-byte chunks
    if (group_size <= 0 || batch_size <= 0 || (group_size & (had_scale != 0.f ? 127 : 7))) return QUEST_ERR_BAD_SHAPE;
    if (!aligned(x, 16) || !aligned(x_had, 16) || !aligned(x_int_packed, 4)) return QUEST_ERR_ALIGNMENT;
    hipStream_t st = (hipStream_t)stream;
    if (dtype == QUEST_DTYPE_BF16)
        return launch_hadamard_quantize<0>(x, scale, x_int_packed, x_int_row_sum, x_had, group_size, batch_size, had_scale,
                                           scale_rule, st);
    return launch_hadamard_quantize<1>(x, scale, x_int_packed, x_int_row_sum, x_had, group_size, batch_size, had_scale,
                                       scale_rule, st);
}

extern "C" int quest_rmsnorm_hadamard_quantize_int4(const void *x, const void *norm_weight, float eps, void *scale,
                                                    uint8_t *x_int_packed, int32_t *x_int_row_sum, void *x_had,
                                                    void *x_norm, int group_size, int batch_size, float had_scale,
                                                    int dtype, void *stream) {
    forget_stale_error();
    if (!x || !norm_weight || !scale) return QUEST_ERR_NULL_POINTER;
    if (!check_dtype(dtype)) return QUEST_ERR_BAD_DTYPE;
    if (group_size <= 0 || batch_size <= 0 || (group_size & 127)) return QUEST_ERR_BAD_SHAPE;
    if (!aligned(x, 16) || !aligned(norm_weight, 16) || !aligned(x_had, 16) || !aligned(x_norm, 16) || !aligned(x_int_packed, 16))
        return QUEST_ERR_ALIGNMENT;
    return launch_hadamard_quantize_mfma(1, x, norm_weight, eps, scale, x_int_packed, x_int_row_sum, x_had, x_norm,
                                         group_size, batch_size, had_scale, dtype, (hipStream_t)stream);
}

extern "C" int quest_add_rmsnorm_hadamard_quantize_int4(void *x, const void *branch, const void *norm_weight, float eps,
                                                        void *scale, uint8_t *x_int_packed, int32_t *x_int_row_sum,
                                                        int group_size, int batch_size, float had_scale, int dtype,
                                                        void *stream) {
    forget_stale_error();
    if (!x || !branch || !norm_weight || !scale) return QUEST_ERR_NULL_POINTER;
    if (!check_dtype(dtype)) return QUEST_ERR_BAD_DTYPE;
    if (group_size <= 0 || batch_size <= 0 || (group_size & 127)) return QUEST_ERR_BAD_SHAPE;
    if (!aligned(x, 16) || !aligned(branch, 16) || !aligned(norm_weight, 16) || !aligned(x_int_packed, 16))
        return QUEST_ERR_ALIGNMENT;
    return launch_hadamard_quantize_mfma(1, x, norm_weight, eps, scale, x_int_packed, x_int_row_sum, nullptr, nullptr,
                                         group_size, batch_size, had_scale, dtype, (hipStream_t)stream, branch, x);
}

extern "C" int quest_silu_mul_hadamard_quantize_int4(const void *gate_up, void *scale, uint8_t *x_int_packed,
                                                     int32_t *x_int_row_sum, void *x_had, void *x_act, int group_size,
                                                     int batch_size, float had_scale, int dtype, void *stream) {
    forget_stale_error();
    if (!gate_up || !scale) return QUEST_ERR_NULL_POINTER;
    if (!check_dtype(dtype)) return QUEST_ERR_BAD_DTYPE;
    if (group_size <= 0 || batch_size <= 0 || (group_size & 127)) return QUEST_ERR_BAD_SHAPE;
    if (!aligned(gate_up, 16) || !aligned(x_had, 16) || !aligned(x_act, 16) || !aligned(x_int_packed, 16)) return QUEST_ERR_ALIGNMENT;
    return launch_hadamard_quantize_mfma(2, gate_up, nullptr, 0.f, scale, x_int_packed, x_int_row_sum, x_had, x_act,
                                         group_size, batch_size, had_scale, dtype, (hipStream_t)stream);
}

// ---- the same kernels writing the codes as E2M3 tiles (the operand form of gemm_e2m3.hip) -------------------------------
static int e2m3_rows_check(const void *x, const void *scale, const void *tiles, int group_size, int batch_size, int dtype) {
    if (!x || !scale || !tiles) return QUEST_ERR_NULL_POINTER;
    if (!check_dtype(dtype)) return QUEST_ERR_BAD_DTYPE;
    if (group_size <= 0 || batch_size <= 0 || (group_size & 127)) return QUEST_ERR_BAD_SHAPE;
    if (!aligned(x, 16) || !aligned(tiles, 16)) return QUEST_ERR_ALIGNMENT;
    return QUEST_OK;
}

extern "C" int quest_hadamard_quantize_e2m3(const void *x, void *scale, void *x_tiles, uint8_t *x_int_packed,
                                            int32_t *x_int_row_sum, void *x_had, int group_size, int batch_size,
                                            float had_scale, int dtype, void *stream) {
    forget_stale_error();
    const int rc = e2m3_rows_check(x, scale, x_tiles, group_size, batch_size, dtype);
    if (rc != QUEST_OK) return rc;
    if (!aligned(x_had, 16) || !aligned(x_int_packed, 4)) return QUEST_ERR_ALIGNMENT;
    return launch_hadamard_quantize_mfma(0, x, nullptr, 0.f, scale, x_int_packed, x_int_row_sum, x_had, nullptr, group_size,
                                         batch_size, had_scale, dtype, (hipStream_t)stream, nullptr, nullptr, (uint8_t *)x_tiles);
}

extern "C" int quest_rmsnorm_hadamard_quantize_e2m3(const void *x, const void *norm_weight, float eps, void *scale,
                                                    void *x_tiles, void *x_norm, int group_size, int batch_size,
                                                    float had_scale, int dtype, void *stream) {
    forget_stale_error();
    const int rc = e2m3_rows_check(x, scale, x_tiles, group_size, batch_size, dtype);
    if (rc != QUEST_OK) return rc;
    if (!norm_weight) return QUEST_ERR_NULL_POINTER;
    if (!aligned(norm_weight, 16) || !aligned(x_norm, 16)) return QUEST_ERR_ALIGNMENT;
    return launch_hadamard_quantize_mfma(1, x, norm_weight, eps, scale, nullptr, nullptr, nullptr, x_norm, group_size, batch_size,
                                         had_scale, dtype, (hipStream_t)stream, nullptr, nullptr, (uint8_t *)x_tiles);
}

extern "C" int quest_add_rmsnorm_hadamard_quantize_e2m3(void *x, const void *branch, const void *norm_weight, float eps,
                                                        void *scale, void *x_tiles, int group_size, int batch_size,
                                                        float had_scale, int dtype, void *stream) {
    forget_stale_error();
    const int rc = e2m3_rows_check(x, scale, x_tiles, group_size, batch_size, dtype);
    if (rc != QUEST_OK) return rc;
    if (!branch || !norm_weight) return QUEST_ERR_NULL_POINTER;
    if (!aligned(branch, 16) || !aligned(norm_weight, 16)) return QUEST_ERR_ALIGNMENT;
    return launch_hadamard_quantize_mfma(1, x, norm_weight, eps, scale, nullptr, nullptr, nullptr, nullptr, group_size, batch_size,
                                         had_scale, dtype, (hipStream_t)stream, branch, x, (uint8_t *)x_tiles);
}

extern "C" int quest_silu_mul_hadamard_quantize_e2m3(const void *gate_up, void *scale, void *x_tiles, void *x_act,
                                                     int group_size, int batch_size, float had_scale, int dtype,
                                                     void *stream) {
    forget_stale_error();
    const int rc = e2m3_rows_check(gate_up, scale, x_tiles, group_size, batch_size, dtype);
    if (rc != QUEST_OK) return rc;
    if (!aligned(x_act, 16)) return QUEST_ERR_ALIGNMENT;
    return launch_hadamard_quantize_mfma(2, gate_up, nullptr, 0.f, scale, nullptr, nullptr, nullptr, x_act, group_size, batch_size,
                                         had_scale, dtype, (hipStream_t)stream, nullptr, nullptr, (uint8_t *)x_tiles);
}

extern "C" int quest_rope_interleaved(void *x, const float *freqs_cis, int n_rows, int seq_len, int row_stride,
                                      int rot_cols, int head_dim, int dtype, void *stream) {
    forget_stale_error();
    if (!x || !freqs_cis) return QUEST_ERR_NULL_POINTER;
    if (!check_dtype(dtype)) return QUEST_ERR_BAD_DTYPE;
    if (n_rows <= 0 || seq_len <= 0 || rot_cols <= 0 || head_dim <= 0 || (head_dim & 7) || (rot_cols % head_dim) ||
        rot_cols > row_stride || (row_stride & 7))
        return QUEST_ERR_BAD_SHAPE;
    if (!aligned(x, 16) || !aligned(freqs_cis, 16)) return QUEST_ERR_ALIGNMENT;
    const long work = (long)n_rows * (rot_cols >> 3);
    const unsigned blocks = (unsigned)((work + 255) / 256);
    hipStream_t st = (hipStream_t)stream;
    if (dtype == QUEST_DTYPE_BF16)
        rope_kernel<0><<<dim3(blocks), dim3(256), 0, st>>>((uint16_t *)x, freqs_cis, n_rows, seq_len, row_stride, rot_cols, head_dim);
    else
        rope_kernel<1><<<dim3(blocks), dim3(256), 0, st>>>((uint16_t *)x, freqs_cis, n_rows, seq_len, row_stride, rot_cols, head_dim);
    return launch_status();
}
