// Shared device helpers for the gfx950 kernels of libquest_hip.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/quest_hip.h"

namespace quest {

// ---- 16-bit float <-> fp32 ------------------------------------------------------------------
// DT = QUEST_DTYPE_BF16 (0) or QUEST_DTYPE_FP16 (1); values travel as raw uint16_t bits.
template <int DT>
__device__ __forceinline__ float to_f32(uint32_t h16) {
    if constexpr (DT == QUEST_DTYPE_BF16) {
        return __uint_as_float(h16 << 16);
    } else {
        return (float)__builtin_bit_cast(_Float16, (uint16_t)h16);
    }
}

// low / high half of a dword holding two 16-bit floats
template <int DT>
__device__ __forceinline__ float lo_f32(uint32_t w) {
    if constexpr (DT == QUEST_DTYPE_BF16) return __uint_as_float(w << 16);
    else return to_f32<DT>(w & 0xffffu);
}
template <int DT>
__device__ __forceinline__ float hi_f32(uint32_t w) {
    if constexpr (DT == QUEST_DTYPE_BF16) return __uint_as_float(w & 0xffff0000u);
    else return to_f32<DT>(w >> 16);
}

// Round an fp32 value to nearest even.  The empty asm pins `f` as an fp32 register first: without
// it the compiler folds a preceding fp32 multiply into v_fma_mixlo_f16, which rounds the exact
// product once to fp16 instead of first to fp32 and then to fp16 as the reference arithmetic does.
template <int DT>
__device__ __forceinline__ uint32_t from_f32(float f) {
    asm volatile("" : "+v"(f));
    if constexpr (DT == QUEST_DTYPE_BF16) {
        return (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)f);
    } else {
        return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)f);
    }
}
template <int DT>
__device__ __forceinline__ uint32_t pack2_from_f32(float lo, float hi) {
    return from_f32<DT>(lo) | (from_f32<DT>(hi) << 16);
}
// The same pair as one two-element conversion (v_cvt_pk_bf16_f32 / v_cvt_pk_f16_f32, both round to
// nearest even).  Only for values that do not come out of an fp32 multiply (see from_f32).
template <int DT>
__device__ __forceinline__ uint32_t pack2_rne(float lo, float hi) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    const f32x2 v = {lo, hi};
    if constexpr (DT == QUEST_DTYPE_BF16) {
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
    } else {
        typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
    }
}

// Two fp32 products rounded to the dtype and packed.  The empty asm pins both as fp32 registers (see from_f32), then
// one two-element conversion rounds each to nearest even.
template <int DT>
__device__ __forceinline__ uint32_t pack2_rounded_products(float lo, float hi) {
    asm volatile("" : "+v"(lo), "+v"(hi));
    return pack2_rne<DT>(lo, hi);
}

// SwiGLU on two packed 16-bit pairs: dtype(dtype(silu(gate)) * up), silu(g) = g / (1 + exp(-g)) in fp32 (fast
// exponential and reciprocal), as src/models/llama.py:117-118 of the reference rounds it.  One definition for the
// activation kernel and the GEMM epilogue, so that the two agree bit for bit.
template <int DT>
__device__ __forceinline__ uint32_t silu_mul_pair(uint32_t gate2, uint32_t up2) {
    auto silu = [](float g) { return __fdividef(g, 1.0f + __expf(-g)); };
    const uint32_t a = pack2_rounded_products<DT>(silu(lo_f32<DT>(gate2)), silu(hi_f32<DT>(gate2)));
    return pack2_rounded_products<DT>(__fmul_rn(lo_f32<DT>(a), lo_f32<DT>(up2)), __fmul_rn(hi_f32<DT>(a), hi_f32<DT>(up2)));
}

// ---- cross-lane moves -----------------------------------------------------------------------
// value of lane (lane ^ M); M = 1, 2, 8 are single DPP moves, 4 and 16 LDS-crossbar swizzles.
template <int M>
__device__ __forceinline__ int lane_xor_i(int v) {
    if constexpr (M == 1) return __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true);        // quad_perm [1,0,3,2]
    else if constexpr (M == 2) return __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true);   // quad_perm [2,3,0,1]
    else if constexpr (M == 4) return __builtin_amdgcn_ds_swizzle(v, (4 << 10) | 0x1F);
    else if constexpr (M == 8) return __builtin_amdgcn_update_dpp(0, v, 0x128, 0xF, 0xF, true);  // row_ror:8
    else if constexpr (M == 16) return __builtin_amdgcn_ds_swizzle(v, (16 << 10) | 0x1F);
    else return __shfl_xor(v, 32, 64);
}
template <int M>
__device__ __forceinline__ float lane_xor_f(float v) {
    return __int_as_float(lane_xor_i<M>(__float_as_int(v)));
}

// Butterfly all-reduce over the 64 lanes; every lane ends with the same bits (fixed order).
__device__ __forceinline__ float wave_sum_f(float v) {
    v += lane_xor_f<1>(v);
    v += lane_xor_f<2>(v);
    v += lane_xor_f<4>(v);
    v += lane_xor_f<8>(v);
    v += lane_xor_f<16>(v);
    v += lane_xor_f<32>(v);
    return v;
}
__device__ __forceinline__ int wave_sum_i(int v) {
    v += lane_xor_i<1>(v);
    v += lane_xor_i<2>(v);
    v += lane_xor_i<4>(v);
    v += lane_xor_i<8>(v);
    v += lane_xor_i<16>(v);
    v += lane_xor_i<32>(v);
    return v;
}

// Sum over the 64 lanes with DPP moves only (no LDS crossbar traffic); lane 0..63 all get the total.
// Pairing inside 16 lanes: xor 1, xor 2, mirror of 8 (any pairing serves a symmetric sum), rotate by 8;
// then the four 16-lane totals are read as scalars and added in lane order.
__device__ __forceinline__ float wave_sum_dpp_f(float v) {
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));   // row_half_mirror
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xF, 0xF, true));   // row_ror:8
    const float a = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    const float b = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    const float c = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    const float d = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return ((a + b) + c) + d;
}
__device__ __forceinline__ int wave_sum_dpp_i(int v) {
    v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true);
    v += __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true);
    v += __builtin_amdgcn_update_dpp(0, v, 0x141, 0xF, 0xF, true);
    v += __builtin_amdgcn_update_dpp(0, v, 0x128, 0xF, 0xF, true);
    return __builtin_amdgcn_readlane(v, 0) + __builtin_amdgcn_readlane(v, 16) + __builtin_amdgcn_readlane(v, 32) +
           __builtin_amdgcn_readlane(v, 48);
}

// Block all-reduce through LDS: per-wave totals are added in wave order by every thread.
// `slots` must hold BLOCK / 64 entries; two barriers, so it can be reused right after.
template <int BLOCK>
__device__ __forceinline__ float block_sum_f(float v, float *slots) {
    v = wave_sum_f(v);
    if constexpr (BLOCK == 64) return v;
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) slots[wave] = v;
    __syncthreads();
    float t = slots[0];
#pragma unroll
    for (int w = 1; w < BLOCK / 64; w++) t += slots[w];
    __syncthreads();
    return t;
}
// The same for a maximum of non-negative values.
template <int BLOCK>
__device__ __forceinline__ float block_max_f(float v, float *slots) {
    v = fmaxf(v, lane_xor_f<1>(v));
    v = fmaxf(v, lane_xor_f<2>(v));
    v = fmaxf(v, lane_xor_f<4>(v));
    v = fmaxf(v, lane_xor_f<8>(v));
    v = fmaxf(v, lane_xor_f<16>(v));
    v = fmaxf(v, lane_xor_f<32>(v));
    if constexpr (BLOCK == 64) return v;
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) slots[wave] = v;
    __syncthreads();
    float t = slots[0];
#pragma unroll
    for (int w = 1; w < BLOCK / 64; w++) t = fmaxf(t, slots[w]);
    __syncthreads();
    return t;
}
template <int BLOCK>
__device__ __forceinline__ int block_sum_i(int v, int *slots) {
    v = wave_sum_i(v);
    if constexpr (BLOCK == 64) return v;
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) slots[wave] = v;
    __syncthreads();
    int t = slots[0];
#pragma unroll
    for (int w = 1; w < BLOCK / 64; w++) t += slots[w];
    __syncthreads();
    return t;
}

// ---- the quantiser ---------------------------------------------------------------------------
// fp32(2.513930578568423 * 2 / 15): the Gaussian-MSE-optimal INT4 clip over 7.5 steps.
__device__ constexpr float kGaussInt4Step = 0.3351907438091231f;
__device__ constexpr float kScaleEps = 1e-8f;

// scale from a row's sum of squares; separate multiply and add (no fused multiply-add), as the
// PyTorch statement of the rule evaluates it.
__device__ __forceinline__ float scale_from_sumsq(float sumsq, int k) {
    float mean_sq = __fdiv_rn(sumsq, (float)k);
    float sd = __fsqrt_rn(mean_sq);
    return __fadd_rn(__fmul_rn(sd, kGaussInt4Step), kScaleEps);
}

// clamp(floor(x / s), -8, 7), bit-identical to the IEEE-divide form for 16-bit-float x and s.
// With inv = fl(1 / s) the product t = fl(x * inv) is within 2^-23 (relative) of x / s.  A quotient of
// two such numbers that is not an integer lies at least 2^-14 (relative) away from the next one, so
// only exact-integer quotients can land on the wrong side of their floor; nudging t by 2^-21 |t|
// towards +inf puts those back (and moves nothing else across an integer).  NaN (0 / 0) comes out
// of v_med3_f32 as -8, like fmaxf / fminf in the CUDA kernel this replaces.
__device__ __forceinline__ float quant_inv(float s) { return __fdiv_rn(1.0f, s); }
__device__ __forceinline__ float quant_code_inv(float x, float inv) {
    const float t = __fmul_rn(x, inv);
    const float tn = __builtin_fmaf(__builtin_fabsf(t), 4.76837158203125e-07f, t);      // 2^-21
    return __builtin_floorf(__builtin_amdgcn_fmed3f(tn, -8.f, 7.5f));
}
// the same code as an integer: the clamp makes the floor-and-convert instruction safe
__device__ __forceinline__ int quant_code_inv_i(float x, float inv) {
    const float t = __fmul_rn(x, inv);
    const float tn = __builtin_fmaf(__builtin_fabsf(t), 4.76837158203125e-07f, t);
    const float m = __builtin_amdgcn_fmed3f(tn, -8.f, 7.5f);
    int q;
    asm("v_cvt_flr_i32_f32 %0, %1" : "=v"(q) : "v"(m));
    return q;
}
// The same code without a clamp instruction, for scales in [2^-99, 2^15] (kQuantFastMin/Max; the caller takes the
// med3 form above for any other scale, NaN and zero included): t = x * (inv * 2^28), the same nudge, and the
// floor-and-convert instruction, which saturates at +-2^31; the top four bits of the resulting integer are then the
// two's-complement nibble of clamp(floor(x / s), -8, 7): floor(floor(2^28 y) / 2^28) = floor(y), and the
// saturation at +-2^31 is the clamp at -8 and 8 - 2^-28.  (Above 2^15 a quotient of 16-bit floats can underflow
// fp32 where the product with 2^28 does not; below 2^-99 inv * 2^28 overflows.)
// `x` must be finite and |x / s| < 2^99, which holds when s is the Gaussian or absmax scale of x's own row.
__device__ constexpr float kQuantFastMin = 0x1p-99f, kQuantFastMax = 0x1p15f;
__device__ __forceinline__ bool quant_fast_ok(float s) { return s >= kQuantFastMin && s <= kQuantFastMax; }
__device__ __forceinline__ float quant_inv28(float s) { return __fmul_rn(__fdiv_rn(1.0f, s), 0x1p28f); }
__device__ __forceinline__ int quant_top_nibble(float x, float inv28) {
    const float t = __fmul_rn(x, inv28);
    const float tn = __builtin_fmaf(__builtin_fabsf(t), 4.76837158203125e-07f, t);
    int q;
    asm("v_cvt_flr_i32_f32 %0, %1" : "=v"(q) : "v"(tn));
    return q;
}
// The same on the low / high half of a dword of two 16-bit floats.  fp16 halves go into the multiplication as they
// are (v_fma_mix_f32 converts its selected half on the way in; its addend +0 only turns a product of -0 into +0,
// which the nudge does anyway); bf16 halves are fp32 bit patterns once shifted or masked.
template <int DT, int HI>
__device__ __forceinline__ int quant_top_nibble_half(uint32_t w, float inv28) {
    if constexpr (DT == QUEST_DTYPE_BF16) {
        return quant_top_nibble(HI ? hi_f32<DT>(w) : lo_f32<DT>(w), inv28);
    } else {
        float t;
        if constexpr (HI) asm("v_fma_mix_f32 %0, %1, %2, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(t) : "v"(w), "v"(inv28));
        else asm("v_fma_mix_f32 %0, %1, %2, 0 op_sel_hi:[1,0,0]" : "=v"(t) : "v"(w), "v"(inv28));
        const float tn = __builtin_fmaf(__builtin_fabsf(t), 4.76837158203125e-07f, t);
        int q;
        asm("v_cvt_flr_i32_f32 %0, %1" : "=v"(q) : "v"(tn));
        return q;
    }
}
// ... for any finite or infinite x (a product that overflows to -inf turns the nudge into inf - inf = NaN, which
// the maximum replaces by the most negative float: code -8, as the clamp of the reference gives)
__device__ __forceinline__ int quant_top_nibble_any(float x, float inv28) {
    const float t = __fmul_rn(x, inv28);
    float tn = __builtin_fmaf(__builtin_fabsf(t), 4.76837158203125e-07f, t);
    tn = __builtin_fmaxf(tn, -3.4028234663852886e38f);
    int q;
    asm("v_cvt_flr_i32_f32 %0, %1" : "=v"(q) : "v"(tn));
    return q;
}
// floor of the same nudged quotient as a float, unclamped, on the low / high half of a dword of two 16-bit floats: for
// consumers whose next conversion saturates (the FP6 operand form).  x finite and s in the fast range, as above.
template <int DT, int HI>
__device__ __forceinline__ float quant_floor_half(uint32_t w, float inv) {
    float t;
    if constexpr (DT == QUEST_DTYPE_BF16) {
        t = __fmul_rn(HI ? hi_f32<DT>(w) : lo_f32<DT>(w), inv);
    } else {
        if constexpr (HI) asm("v_fma_mix_f32 %0, %1, %2, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(t) : "v"(w), "v"(inv));
        else asm("v_fma_mix_f32 %0, %1, %2, 0 op_sel_hi:[1,0,0]" : "=v"(t) : "v"(w), "v"(inv));
    }
    return __builtin_floorf(__builtin_fmaf(__builtin_fabsf(t), 4.76837158203125e-07f, t));
}
// appends the nibble in the top four bits of `n` below the nibbles already in `packed` (which move up by four bits)
__device__ __forceinline__ uint32_t push_top_nibble(uint32_t packed, int n) {
    return __builtin_amdgcn_alignbit(packed, (uint32_t)n, 28);
}
// reference form with the correctly rounded divide (kept for the exhaustive equivalence test)
__device__ __forceinline__ float quant_code(float x, float s) {
    float q = __builtin_floorf(__fdiv_rn(x, s));
    q = fmaxf(q, -8.f);
    q = fminf(q, 7.f);
    return q;
}

// what a GEMM writes: the two 16-bit float types share their codes with QUEST_DTYPE_*
enum { OUT_BF16 = 0, OUT_FP16 = 1, OUT_INT32 = 2 };

// gemm_decode.hip: the weight-streaming GEMM for M <= 64; QUEST_ERR_UNSUPPORTED when it does not apply
int launch_gemm_decode(int out_kind, void *out, const uint8_t *a, const uint8_t *b, const int32_t *a_add,
                       const int32_t *b_add, const void *a_mul, const void *b_mul, int M, int K, int N, hipStream_t st);

// ... and its split-K form for M <= 16 with a workspace (see gemm_decode.hip); gemm_decode_workspace_bytes is what it needs
int launch_gemm_decode_splitk(int out_kind, void *out, const uint8_t *a, const uint8_t *b, const int32_t *a_add,
                              const int32_t *b_add, const void *a_mul, const void *b_mul, int M, int K, int N, void *workspace,
                              size_t workspace_bytes, hipStream_t st);
size_t gemm_decode_workspace_bytes(int K, int N);

// hadamard_mfma.hip: the matrix-core fused activation kernel, optionally with the producer of the activation in
// front (pre: 0 none, 1 RMSNorm, 2 SiLU(gate) * up); QUEST_ERR_UNSUPPORTED when it does not apply
int launch_hadamard_quantize_mfma(int pre, const void *x, const void *norm_w, float eps, void *scale, uint8_t *packed,
                                  int32_t *row_sum, void *x_had, void *pre_out, int K, int M, float had_scale, int dtype,
                                  hipStream_t st, const void *add_in = nullptr, void *sum_out = nullptr, uint8_t *tiles = nullptr);

inline int check_dtype(int dtype) { return dtype == QUEST_DTYPE_BF16 || dtype == QUEST_DTYPE_FP16; }
inline int aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }
// HIP keeps the last error until someone reads it.  An entry point judges its own launches by that error, so whatever an
// earlier call left behind (a failed call of the caller's in this thread, a failed device query in here) is read and
// dropped first: forget_stale_error() before the first launch of an entry point, launch_status() after the last.
inline void forget_stale_error() { (void)hipGetLastError(); }

// Compute units of the device the stream belongs to.  Asked for once per call that needs it (two host-side queries,
// no stream operation, nothing cached): the library keeps no state and a process may drive several devices.
inline int device_cu_count(hipStream_t st) {
    int dev = 0, cus = 0;
    const bool found = hipStreamGetDevice(st, &dev) == hipSuccess || hipGetDevice(&dev) == hipSuccess;
    const bool counted = found && hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && cus > 0;
    forget_stale_error();                      // a failed query must not be taken for the launch that follows
    return counted ? cus : 256;
}
inline int launch_status() { return hipGetLastError() == hipSuccess ? QUEST_OK : QUEST_ERR_LAUNCH; }

}  // namespace quest
