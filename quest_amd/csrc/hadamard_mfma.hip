// Fused activation kernel: block-128 Hadamard on the matrix cores, Gaussian-clip scale, INT4 codes,
// nibble packing and row sums in one pass over HBM, for rows of up to 32768 elements.
//
// This is linear_forward's activation half (gemm-quest/benchmarks/utils.py:89-100 of the
// reference) and it computes the Hadamard the way the reference states it: a product with the
// 128 x 128 matrix whose entries are +-181/2048 in the activation dtype, fp32 accumulation, one
// rounding of the result to the dtype (utils.py:17, 89-90).
//
// One wave owns 32 blocks of 128 of one row and handles nothing else: the grid has a wave per 32
// blocks and the hardware dispatcher balances them (measured faster than a persistent grid, whose
// waves reach their last rows together and leave that arithmetic uncovered by memory traffic).
// Block n is column n of the MFMA "B" operand and the Hadamard matrix is the "A" operand:
// D (128 x 32 blocks) = H (128 x 128) * X^T, as 4 row tiles x 8 k-steps of v_mfma_f32_32x32x16.
// A lane's B fragment for k-step s is the 16-byte chunk 2 s + (lane >> 5) of its block, which it
// loads straight from HBM: per instruction the wave reads 32 bytes of each block, and the eight
// instructions are in flight together, so every 128-byte line is fetched once (measured: the same
// rate as fully contiguous 16-byte-per-lane loads).  The sign of H for output 32 mt + i and input
// 8 (2 s + g) + j is (-1)^(popcount(i & 7 & j) + i3 g + i4 s0 + mt0 s1 + mt1 s2): the first two
// terms are fixed per lane, the third takes two values, the rest is uniform per instruction, so
// four register quads hold every A fragment the 32 instructions need.
// After the MFMAs lane (n, h) holds outputs 32 mt + 8 q + 4 h + e of block n: the row never leaves
// registers.  Rows longer than 4096 are split over the waves of a workgroup, which exchange only
// their partial sums of squares and of codes through LDS.
//
// Besides (or instead of) packed nibbles the codes can be written as E2M3 tiles, the operand form of the FP6 GEMM
// (gemm_e2m3.hip; layout in include/quest_hip.h): the two half-waves trade the rounded outputs so that a lane holds
// two whole groups of 32 consecutive k, each output becomes the fp16 value q + 1/2 (floor of the same nudged quotient
// the nibble path converts; the clamp is the saturation of the FP6 conversion) and v_cvt_scalef32_pk32_fp6_f16 packs
// 32 of them into the lane's 24 bytes of its fragment.
#include "common.h"
#include <type_traits>

namespace quest {
namespace hq {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));

typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));

// acc + lo(w)^2 + hi(w)^2 for a dword of two 16-bit floats (squares of 16-bit floats are exact in fp32)
template <int DT>
__device__ __forceinline__ float dot2_self(uint32_t w, float acc) {
    if constexpr (DT == QUEST_DTYPE_BF16)
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(v2bf, w), __builtin_bit_cast(v2bf, w), acc, false);
    else
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(v2h, w), __builtin_bit_cast(v2h, w), acc, false);
}

template <int DT>
__device__ __forceinline__ v16f mfma_h(const v4i &a, const v4i &b, const v16f &c) {
    if constexpr (DT == QUEST_DTYPE_BF16)
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
}

typedef unsigned int v4u __attribute__((ext_vector_type(4)));

// WPR waves share one row (32 blocks of 128 each); a workgroup holds one or two rows' worth of waves (small
// workgroups: two-wave ones measured 3 % faster than four-wave ones for whole-wave rows, eight-wave ones 5 % slower).
// TL (E2M3 tiles staged through LDS, see the kernel): the workgroup holds eight consecutive rows (four when two or
// three waves share a row), so that it owns whole 128-byte (64-byte) runs of every fragment it contributes to.
template <int WPR, int G, bool TL>
struct Shape {
    static constexpr int kRowsPerWave = 32 / G;
    static constexpr int kRows = !TL ? (WPR >= 3 ? 1 : 2) : WPR == 1 ? (8 / kRowsPerWave > 0 ? 8 / kRowsPerWave : 1) : 4;
    static constexpr int kWaves = WPR * kRows;
    static constexpr int kMinBlocks = kWaves <= 4 ? 4 : (16 / kWaves > 0 ? 16 / kWaves : 1);
    static constexpr int kTileRows = kRows * kRowsPerWave;           // rows of a workgroup
    // staging buffer: one position per (half of a k-step, k-step) of a row, the rows' 16-byte heads (8-byte tails) side
    // by side; one spare chunk per position spreads the positions over the banks
    static constexpr int kBlocks = G == 32 ? 32 * WPR : G;           // blocks of a row, rounded up
    static constexpr int kPositions = 4 * kBlocks;
    static constexpr int kHeadPitch = kTileRows * 16 + 16;
    static constexpr int kTailPitch = kTileRows * 8 + 8;
    static constexpr int kStageBytes = TL ? kPositions * (kHeadPitch + kTailPitch) : 16;
};

// What is applied to the input on its way into the transform (the producer the activation comes from):
//   kPreNone     nothing;
//   kPreRmsNorm  y = dtype(dtype(f32(x) * rsqrt(mean(x^2) + eps)) * w)    (src/models/llama.py:71-77 of the reference);
//                with add_in: x is first replaced by dtype(x + add_in) -- the residual addition in front of the norm
//                (llama.py:175-176) -- and that sum is written to sum_out (which may be x itself);
//   kPreSiluMul  y = dtype(dtype(silu(gate)) * up), gate and up the two halves of a (M, 2 K) row (llama.py:117-118).
enum { kPreNone = 0, kPreRmsNorm = 1, kPreSiluMul = 2 };

// Sum over the G lanes (G a power of two, aligned) of each half-wave that hold one row, and over the two half-waves.
template <int G>
__device__ __forceinline__ float group_sum_f(float v) {
    if constexpr (G >= 2) v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));
    if constexpr (G >= 4) v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));
    if constexpr (G >= 8) v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));
    if constexpr (G >= 16) v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xF, 0xF, true));
    if constexpr (G >= 32) v += lane_xor_f<16>(v);
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
template <int G>
__device__ __forceinline__ int group_sum_i(int v) {
    if constexpr (G >= 2) v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true);
    if constexpr (G >= 4) v += __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true);
    if constexpr (G >= 8) v += __builtin_amdgcn_update_dpp(0, v, 0x141, 0xF, 0xF, true);
    if constexpr (G >= 16) v += __builtin_amdgcn_update_dpp(0, v, 0x128, 0xF, 0xF, true);
    if constexpr (G >= 32) v += lane_xor_i<16>(v);
    const auto r = __builtin_amdgcn_permlane32_swap((unsigned)v, (unsigned)v, false, false);
    return (int)r[0] + (int)r[1];
}

// G = lanes of a half-wave per row (the row's blocks rounded up to a power of two): a wave holds 32 / G rows.
template <int DT, int WPR, int G, int PRE, bool TL>
__global__ void __launch_bounds__((64 * Shape<WPR, G, TL>::kWaves), (Shape<WPR, G, TL>::kMinBlocks))
hadamard_quantize_mfma_kernel(const uint16_t *__restrict__ x, const uint16_t *__restrict__ norm_w,
                              uint16_t *__restrict__ scale, uint32_t *__restrict__ packed, int32_t *__restrict__ row_sum,
                              uint16_t *__restrict__ x_had, uint16_t *__restrict__ pre_out, const uint16_t *add_in,
                              uint16_t *sum_out, uint8_t *__restrict__ tiles, int xcd_chunk, int K, int M, int ldx,
                              uint32_t entry_bits, float eps) {
    static_assert(WPR == 1 || G == 32, "rows shared by waves: whole waves");
    using Sh = Shape<WPR, G, TL>;
    constexpr int kRows = Sh::kRows;
    constexpr int kRowsPerWave = 32 / G;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int part = wave % WPR;               // which 32 blocks of the row
    const int row_local = wave / WPR;
    const int n = lane & 31;                   // MFMA column
    const int h = lane >> 5;
    // xcd_chunk > 0 (E2M3 tiles are written): workgroups are dealt to the eight XCDs in turn, so workgroup b of the grid
    // takes the rows of virtual workgroup (b % 8) * xcd_chunk + b / 8 -- each XCD then works through one contiguous
    // range of rows, and the 8 (16) consecutive rows that share a 128-byte line of a fragment's heads (tails) are
    // written through one L2 within a short time, where the partial lines merge
    const int vb = xcd_chunk > 0 ? (int)(blockIdx.x & 7) * xcd_chunk + (int)(blockIdx.x >> 3) : (int)blockIdx.x;
    const int row = (vb * kRows + row_local) * kRowsPerWave + n / G;
    const int blk = part * 32 + n % G;         // block of the row in this column
    const bool live = row < M && blk < (K >> 7);

    // ---- the four A fragments: +-entry with sign (-1)^(popcount(n & 7 & j) + n3 h) [* (-1)^n4] [* -1]
    v4i hv[2][2];
    {
        const uint32_t lane_flip = ((n >> 3) & 1) & h;
        uint32_t base[4];
#pragma unroll
        for (int d = 0; d < 4; d++) {
            uint32_t w = 0;
#pragma unroll
            for (int e = 0; e < 2; e++) {
                const int j = 2 * d + e;
                const uint32_t neg = (__builtin_popcount(n & 7 & j) & 1) ^ lane_flip;
                w |= (entry_bits ^ (neg << 15)) << (16 * e);
            }
            base[d] = w;
        }
        const uint32_t s0_flip = ((n >> 4) & 1) ? 0x80008000u : 0u;
#pragma unroll
        for (int d = 0; d < 4; d++) {
            hv[0][0][d] = (int)base[d];
            hv[0][1][d] = (int)(base[d] ^ 0x80008000u);
            hv[1][0][d] = (int)(base[d] ^ s0_flip);
            hv[1][1][d] = (int)(base[d] ^ s0_flip ^ 0x80008000u);
        }
    }

    // ---- B fragments straight from HBM: chunk 2 s + h of a block is bytes [32 s + 16 h, +16) of its 256.
    // Lanes without a block get an offset beyond the buffer: such loads touch no memory and return zeros.
    const int in_cols = PRE == kPreSiluMul ? 2 * K : K;
    const __amdgpu_buffer_rsrc_t xr =
        __builtin_amdgcn_make_buffer_rsrc((void *)x, 0, (int)(((long)(M - 1) * ldx + in_cols) * 2), 0x00020000);
    const uint32_t dead = 0x80000000u;
    const uint32_t ld_off = live ? (uint32_t)(row * ldx * 2 + blk * 256 + h * 16) : dead;
    v4u bq[8];
#pragma unroll
    for (int s = 0; s < 8; s++) bq[s] = __builtin_amdgcn_raw_buffer_load_b128(xr, (int)(ld_off + 32 * s), 0, 0);
    // all eight in flight before anything else: left alone the scheduler sinks the last two below the first MFMAs to
    // save registers, which costs every wave a second trip to memory
    __builtin_amdgcn_sched_barrier(0);

    if constexpr (PRE == kPreRmsNorm) {
        if (add_in != nullptr) {                 // uniform: the residual stream plus the branch that ends here
            const __amdgpu_buffer_rsrc_t ar =
                __builtin_amdgcn_make_buffer_rsrc((void *)add_in, 0, (int)((long)M * K * 2), 0x00020000);
            v4u aq[8];
#pragma unroll
            for (int s = 0; s < 8; s++) aq[s] = __builtin_amdgcn_raw_buffer_load_b128(ar, (int)(ld_off + 32 * s), 0, 0);
#pragma unroll
            for (int s = 0; s < 8; s++)
#pragma unroll
                for (int d = 0; d < 4; d++)
                    bq[s][d] = pack2_rounded_products<DT>(__fadd_rn(lo_f32<DT>(bq[s][d]), lo_f32<DT>(aq[s][d])),
                                                          __fadd_rn(hi_f32<DT>(bq[s][d]), hi_f32<DT>(aq[s][d])));
            if (live) {
                uint16_t *dst = sum_out + (size_t)row * K + blk * 128 + 8 * h;
#pragma unroll
                for (int s = 0; s < 8; s++) *reinterpret_cast<v4u *>(dst + 16 * s) = bq[s];
            }
        }
        const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc((void *)norm_w, 0, K * 2, 0x00020000);
        const uint32_t w_off = live ? (uint32_t)(blk * 256 + h * 16) : dead;
        v4u wq[8];
#pragma unroll
        for (int s = 0; s < 8; s++) wq[s] = __builtin_amdgcn_raw_buffer_load_b128(wr, (int)(w_off + 32 * s), 0, 0);
        float ss = 0.f;
#pragma unroll
        for (int s = 0; s < 8; s++)
#pragma unroll
            for (int d = 0; d < 4; d++) ss = dot2_self<DT>(bq[s][d], ss);
        float ss_row = group_sum_f<G>(ss);
        if constexpr (WPR > 1) {                 // the row's waves add their parts in wave order: the same bits in each
            __shared__ float part_pre[Sh::kWaves];
            if (lane == 0) part_pre[wave] = ss_row;
            __syncthreads();
            ss_row = 0.f;
#pragma unroll
            for (int w = 0; w < WPR; w++) ss_row += part_pre[row_local * WPR + w];
        }
        const float mean_sq = __fmul_rn(ss_row, __fdiv_rn(1.0f, (float)K));
        const float r = __frsqrt_rn(__fadd_rn(mean_sq, eps));
#pragma unroll
        for (int s = 0; s < 8; s++)
#pragma unroll
            for (int d = 0; d < 4; d++) {
                const uint32_t y = pack2_rounded_products<DT>(__fmul_rn(lo_f32<DT>(bq[s][d]), r), __fmul_rn(hi_f32<DT>(bq[s][d]), r));
                bq[s][d] = pack2_rounded_products<DT>(__fmul_rn(lo_f32<DT>(y), lo_f32<DT>(wq[s][d])),
                                                      __fmul_rn(hi_f32<DT>(y), hi_f32<DT>(wq[s][d])));
            }
    }
    if constexpr (PRE == kPreSiluMul) {
        v4u uq[8];
#pragma unroll
        for (int s = 0; s < 8; s++) uq[s] = __builtin_amdgcn_raw_buffer_load_b128(xr, (int)(ld_off + K * 2 + 32 * s), 0, 0);
#pragma unroll
        for (int s = 0; s < 8; s++)
#pragma unroll
            for (int d = 0; d < 4; d++) bq[s][d] = silu_mul_pair<DT>(bq[s][d], uq[s][d]);
    }
    if constexpr (PRE != kPreNone) {
        if (pre_out != nullptr && live) {
            uint16_t *dst = pre_out + (size_t)row * K + blk * 128 + 8 * h;
#pragma unroll
            for (int s = 0; s < 8; s++) *reinterpret_cast<v4u *>(dst + 16 * s) = bq[s];
        }
    }

    // ---- Hadamard: 8 k-steps x 4 row tiles; then round to the dtype (the transform's output exists only in dtype) and
    // sum the squares.  entry_bits == 0: no transform -- the loaded chunks are the outputs already and only have to
    // change lanes: lane (n, h) loaded the chunks whose k has bit 3 equal to h and the code below wants those whose bit 2
    // is h, so the two half-waves trade half of every chunk (nothing is multiplied: NaN and Inf stay where they are).
    uint32_t yb[4][8];                          // [mt][q * 2 + pair]: outputs 32 mt + 8 q + 4 h + {0,1} / {2,3}
    float sumsq = 0.f;
    if (entry_bits == 0) {                      // uniform
#pragma unroll
        for (int s = 0; s < 8; s++)
#pragma unroll
            for (int p = 0; p < 2; p++) {
                // outputs 16 s + 8 (q & 1) + 4 h + 2 p + {0, 1}: pair 2 h + p of the chunk held by the half-wave q & 1
                const auto sw = __builtin_amdgcn_permlane32_swap(bq[s][p], bq[s][2 + p], false, false);
#pragma unroll
                for (int qo = 0; qo < 2; qo++) {
                    const uint32_t w = sw[qo];
                    yb[s >> 1][(2 * (s & 1) + qo) * 2 + p] = w;
                    sumsq = dot2_self<DT>(w, sumsq);
                }
            }
    } else {
        v16f acc[4];
#pragma unroll
        for (int mt = 0; mt < 4; mt++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[mt][r] = 0.f;
#pragma unroll
        for (int s = 0; s < 8; s++) {
            const v4i b = __builtin_bit_cast(v4i, bq[s]);
#pragma unroll
            for (int mt = 0; mt < 4; mt++) {
                const int neg = ((mt & 1) & ((s >> 1) & 1)) ^ (((mt >> 1) & 1) & ((s >> 2) & 1));
                acc[mt] = mfma_h<DT>(hv[s & 1][neg], b, acc[mt]);
            }
        }
#pragma unroll
        for (int mt = 0; mt < 4; mt++)
#pragma unroll
            for (int q = 0; q < 4; q++)
#pragma unroll
                for (int p = 0; p < 2; p++) {
                    const uint32_t w = pack2_rne<DT>(acc[mt][q * 4 + 2 * p], acc[mt][q * 4 + 2 * p + 1]);
                    yb[mt][q * 2 + p] = w;
                    sumsq = dot2_self<DT>(w, sumsq);            // both squares straight from the packed pair
                }
    }
    // lanes without a block transformed zeros: they add nothing
    float total = G == 32 ? wave_sum_dpp_f(sumsq) : group_sum_f<G>(sumsq);
    __shared__ float part_sq[Sh::kWaves];
    __shared__ int part_sum[Sh::kWaves];
    if constexpr (WPR > 1) {
        if (lane == 0) part_sq[wave] = total;
        __syncthreads();
        total = 0.f;
#pragma unroll
        for (int w = 0; w < WPR; w++) total += part_sq[row_local * WPR + w];       // fixed order: every wave gets the same bits
    }
    const uint32_t s16 = from_f32<DT>(scale_from_sumsq(total, K));
    const bool writer = lane % G == 0 && h == 0 && part == 0 && row < M;      // one lane per row

    if (x_had != nullptr && live) {
        uint16_t *dst = x_had + (size_t)row * K + blk * 128 + 4 * h;
#pragma unroll
        for (int mt = 0; mt < 4; mt++)
#pragma unroll
            for (int q = 0; q < 4; q++)
                *reinterpret_cast<uint2 *>(dst + 32 * mt + 8 * q) = make_uint2(yb[mt][q * 2], yb[mt][q * 2 + 1]);
    }
    if (writer) scale[row] = (uint16_t)s16;

    // ---- codes as E2M3 tiles.  Rounded outputs 32 mt + 8 q + 4 h + {0..3} sit in lane (n, h); after the exchange lane
    // (n, h) holds all 32 outputs of the groups mt = 2 h and 2 h + 1: k-step 2 blk + h of the row, both halves.
    if (tiles != nullptr) {
        typedef _Float16 v32h __attribute__((ext_vector_type(32)));
        typedef _Float16 v2hh __attribute__((ext_vector_type(2)));
        typedef unsigned v6u __attribute__((ext_vector_type(6)));
        typedef unsigned v16u __attribute__((ext_vector_type(16)));
        const float sf_t = to_f32<DT>(s16);
        const float inv = quant_inv(sf_t);
        uint8_t *frag = tiles + ((size_t)(row >> 5) * (size_t)(K >> 6) + 2 * blk + h) * 1536;
        __shared__ __attribute__((aligned(16))) uint8_t stage[Sh::kStageBytes];
        auto emit = [&](auto fast_tag) {
            constexpr bool kFast = decltype(fast_tag)::value;
#pragma unroll
            for (int g = 0; g < 2; g++) {
                v16u hp;                            // dword d = 4 q + 2 h' + p: outputs 8 q + 4 h' + 2 p + {0, 1} of the group
#pragma unroll
                for (int j = 0; j < 8; j++) {       // j = 2 q + p
                    const auto sw = __builtin_amdgcn_permlane32_swap(yb[g][j], yb[g + 2][j], false, false);
#pragma unroll
                    for (int hh = 0; hh < 2; hh++) {
                        float f0, f1;
                        if constexpr (kFast) {
                            f0 = quant_floor_half<DT, 0>(sw[hh], inv);
                            f1 = quant_floor_half<DT, 1>(sw[hh], inv);
                        } else {
                            f0 = quant_code_inv(lo_f32<DT>(sw[hh]), inv);
                            f1 = quant_code_inv(hi_f32<DT>(sw[hh]), inv);
                        }
                        // to fp16 (round towards zero saturates at +-65504 instead of overflowing), then + 1/2
                        const v2hh c = __builtin_bit_cast(v2hh, __builtin_amdgcn_cvt_pkrtz(f0, f1)) + v2hh{(_Float16)0.5f, (_Float16)0.5f};
                        hp[4 * (j >> 1) + 2 * hh + (j & 1)] = __builtin_bit_cast(unsigned, c);
                    }
                }
                const v6u r = __builtin_amdgcn_cvt_scalef32_pk32_fp6_f16(__builtin_bit_cast(v32h, hp), 1.0f);
                if constexpr (TL) {
                    // position (g, h, block) of the row, this row's chunk in it
                    const int pos = (2 * g + h) * Sh::kBlocks + blk;
                    const int j = row_local * kRowsPerWave + n / G;
                    *reinterpret_cast<uint4 *>(stage + pos * Sh::kHeadPitch + j * 16) = make_uint4(r[0], r[1], r[2], r[3]);
                    *reinterpret_cast<uint2 *>(stage + Sh::kPositions * Sh::kHeadPitch + pos * Sh::kTailPitch + j * 8) = make_uint2(r[4], r[5]);
                } else if (live) {
                    const int slot = 32 * g + (row & 31);
                    *reinterpret_cast<uint4 *>(frag + slot * 16) = make_uint4(r[0], r[1], r[2], r[3]);
                    *reinterpret_cast<uint2 *>(frag + 1024 + slot * 8) = make_uint2(r[4], r[5]);
                }
            }
        };
        // degenerate rows (scale zero, Inf, NaN or outside the fast range) take the clamping form, as the nibbles do
        if (__builtin_amdgcn_ballot_w64(row < M && !quant_fast_ok(sf_t)) == 0) emit(std::true_type{}); else emit(std::false_type{});
        if constexpr (TL) {
            // The workgroup's rows are kTileRows consecutive slots of one row block: for every position their heads are
            // one contiguous run of the fragment (128 bytes for eight rows) and their tails another, written by
            // neighbouring lanes.  Rows past M inside the last row block are padding and are written like any other.
            __syncthreads();
            constexpr int kTR = Sh::kTileRows;
            const int row0 = vb * kTR;
            const int m_pad = (M + 31) & ~31;
            const size_t frag0 = (size_t)(row0 >> 5) * (size_t)(K >> 6);
            for (int u = threadIdx.x; u < Sh::kPositions * kTR; u += 64 * Sh::kWaves) {
                const int pos = u / kTR, c = u % kTR;
                const int gg = pos / (2 * Sh::kBlocks), hh = (pos / Sh::kBlocks) & 1, bb = pos % Sh::kBlocks;
                if (bb < (K >> 7) && row0 + c < m_pad)
                    *reinterpret_cast<uint4 *>(tiles + (frag0 + 2 * bb + hh) * 1536 + (32 * gg + (row0 & 31) + c) * 16) =
                        *reinterpret_cast<const uint4 *>(stage + pos * Sh::kHeadPitch + c * 16);
            }
            for (int u = threadIdx.x; u < Sh::kPositions * kTR / 2; u += 64 * Sh::kWaves) {
                const int pos = u / (kTR / 2), c = 2 * (u % (kTR / 2));
                const int gg = pos / (2 * Sh::kBlocks), hh = (pos / Sh::kBlocks) & 1, bb = pos % Sh::kBlocks;
                if (bb < (K >> 7) && row0 + c < m_pad)
                    *reinterpret_cast<uint4 *>(tiles + (frag0 + 2 * bb + hh) * 1536 + 1024 + (32 * gg + (row0 & 31) + c) * 8) =
                        *reinterpret_cast<const uint4 *>(stage + Sh::kPositions * Sh::kHeadPitch + pos * Sh::kTailPitch + c * 8);
            }
        }
    }
    if (packed == nullptr && row_sum == nullptr) return;      // uniform over the workgroup

    // ---- codes.  Outputs 8 Q + 4 h + {0..3} (Q = 4 mt + q) give one half-word c3 c2 c1 c0 of two's-complement nibbles.
    // Scales in the quantiser's fast range (everything but degenerate rows) take the clamp-free form: the code
    // arrives in the top nibble of an integer and is shifted into the half-word by one v_alignbit per code.
    const float sf = to_f32<DT>(s16);
    uint32_t hw[16];
    if (__builtin_amdgcn_ballot_w64(row < M && !quant_fast_ok(sf)) == 0) {
        const float inv28 = quant_inv28(sf);
#pragma unroll
        for (int mt = 0; mt < 4; mt++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const uint32_t w0 = yb[mt][q * 2], w1 = yb[mt][q * 2 + 1];
                uint32_t g = (uint32_t)quant_top_nibble_half<DT, 1>(w1, inv28) >> 28;
                g = push_top_nibble(g, quant_top_nibble_half<DT, 0>(w1, inv28));
                g = push_top_nibble(g, quant_top_nibble_half<DT, 1>(w0, inv28));
                hw[mt * 4 + q] = push_top_nibble(g, quant_top_nibble_half<DT, 0>(w0, inv28));
            }
    } else {
        const float inv = quant_inv(sf);
#pragma unroll
        for (int mt = 0; mt < 4; mt++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const uint32_t w0 = yb[mt][q * 2], w1 = yb[mt][q * 2 + 1];
                const uint32_t c0 = (uint32_t)quant_code_inv_i(lo_f32<DT>(w0), inv) & 15u;
                const uint32_t c1 = (uint32_t)quant_code_inv_i(hi_f32<DT>(w0), inv) & 15u;
                const uint32_t c2 = (uint32_t)quant_code_inv_i(lo_f32<DT>(w1), inv) & 15u;
                const uint32_t c3 = (uint32_t)quant_code_inv_i(hi_f32<DT>(w1), inv) & 15u;
                hw[mt * 4 + q] = (((c3 * 16 + c2) * 16 + c1) * 16) + c0;
            }
    }
    // lane (n, 0) ends with dwords 0..7 of the block's 64 packed bytes, lane (n, 1) with dwords 8..15: dword D is the
    // half-word Q = D of lane (n, 0) below that of lane (n, 1).  v_permlane32_swap hands the lower lane both half-words
    // t and the upper lane both half-words t + 8.  Every code sits in exactly one lane's dwords, so the row sum is the
    // sum of their signed nibbles.
    int isum = 0;
    uint32_t dw[8];
#pragma unroll
    for (int t = 0; t < 8; t++) {
        const auto sw = __builtin_amdgcn_permlane32_swap(hw[t], hw[t + 8], false, false);
        dw[t] = sw[0] | (sw[1] << 16);
        isum = __builtin_amdgcn_sdot8((int)dw[t], 0x11111111, isum, false);
    }
    if (packed != nullptr && live) {
        uint32_t *dst = packed + (size_t)row * (K >> 3) + blk * 16 + h * 8;
        if ((reinterpret_cast<uintptr_t>(packed) & 15) == 0) {           // uniform; rows are whole multiples of 64 bytes
            *reinterpret_cast<uint4 *>(dst) = make_uint4(dw[0], dw[1], dw[2], dw[3]);
            *reinterpret_cast<uint4 *>(dst + 4) = make_uint4(dw[4], dw[5], dw[6], dw[7]);
        } else {                                                          // a view that starts 4 bytes into an allocation
            // (volatile: kept apart from the vector stores above, which the compiler would otherwise merge with these
            // into a common, narrower sequence)
#pragma unroll
            for (int t = 0; t < 8; t++) *reinterpret_cast<volatile uint32_t *>(dst + t) = dw[t];
        }
    }
    if (row_sum != nullptr) {
        if (!live) isum = 0;                    // a dead lane's zeros need not quantise to code 0
        int t = G == 32 ? wave_sum_dpp_i(isum) : group_sum_i<G>(isum);
        if constexpr (WPR > 1) {
            if (lane == 0) part_sum[wave] = t;
            __syncthreads();
            t = 0;
#pragma unroll
            for (int w = 0; w < WPR; w++) t += part_sum[row_local * WPR + w];
        }
        if (writer) row_sum[row] = t;
    }
}

}  // namespace hq

// Whether `v` survives a round trip through the 16-bit dtype, and its bits there.
static bool representable16(float v, int dtype, uint32_t *bits) {
    uint32_t u;
    __builtin_memcpy(&u, &v, 4);
    if (dtype == QUEST_DTYPE_BF16) {
        if (u & 0xFFFFu) return false;
        *bits = u >> 16;
        return true;
    }
    const _Float16 hf = (_Float16)v;
    if ((float)hf != v) return false;
    uint16_t b;
    __builtin_memcpy(&b, &hf, 2);
    *bits = b;
    return true;
}

struct Args {
    const void *x, *norm_w;
    void *scale;
    uint8_t *packed;
    int32_t *row_sum;
    void *x_had, *pre_out;
    const void *add_in;
    void *sum_out;
    uint8_t *tiles;
    int K, M, ldx;
    uint32_t bits;
    float eps;
    hipStream_t st;
    int cus;                   // compute units of the device (only looked at when tiles are written)
};

template <int DT, int WPR, int G, int PRE, bool TL>
static void launch_shape_as(const Args &a) {
    using Sh = hq::Shape<WPR, G, TL>;
    constexpr int rows = Sh::kTileRows;                            // rows per workgroup
    int grid = (a.M + rows - 1) / rows, xcd_chunk = 0;
    if (a.tiles != nullptr) {                                     // see the kernel: a contiguous range of rows per XCD
        xcd_chunk = (grid + 7) / 8;
        grid = 8 * xcd_chunk;
    }
    hq::hadamard_quantize_mfma_kernel<DT, WPR, G, PRE, TL><<<dim3(grid), dim3(64 * Sh::kWaves), 0, a.st>>>(
        (const uint16_t *)a.x, (const uint16_t *)a.norm_w, (uint16_t *)a.scale, (uint32_t *)a.packed, a.row_sum,
        (uint16_t *)a.x_had, (uint16_t *)a.pre_out, (const uint16_t *)a.add_in, (uint16_t *)a.sum_out, a.tiles, xcd_chunk,
        a.K, a.M, a.ldx, a.bits, a.eps);
}

// Tiles go through the workgroup's LDS where a workgroup of eight (four) rows fits -- rows of 8 to 96 blocks -- and where
// such workgroups are at least two per compute unit: below that the small workgroups, which write their 16-byte pieces
// straight to the tiles, fill the device better (bf16 rows of 4096: 4.0 against 5.9 us for 512 rows, 7.3 against 7.2 us
// for 2048, 14.5 against 11.5 us for 4096).  Same arithmetic and same bytes either way.
template <int DT, int WPR, int G, int PRE>
static void launch_shape(const Args &a) {
    if constexpr (WPR <= 3 && G >= 8) {
        constexpr int rows = hq::Shape<WPR, G, true>::kTileRows;
        if (a.tiles != nullptr && (a.M + rows - 1) / rows >= 2 * a.cus) return launch_shape_as<DT, WPR, G, PRE, true>(a);
    }
    launch_shape_as<DT, WPR, G, PRE, false>(a);
}

// rows of up to 32 blocks: one wave holds 32 / G of them
template <int DT, int PRE>
static void launch_short(int g, const Args &a) {
    switch (g) {
        case 1: launch_shape<DT, 1, 1, PRE>(a); break;
        case 2: launch_shape<DT, 1, 2, PRE>(a); break;
        case 4: launch_shape<DT, 1, 4, PRE>(a); break;
        case 8: launch_shape<DT, 1, 8, PRE>(a); break;
        case 16: launch_shape<DT, 1, 16, PRE>(a); break;
        default: launch_shape<DT, 1, 32, PRE>(a); break;
    }
}

// longer rows: WPR waves per row
template <int DT, int PRE>
static void launch_long(int wpr, const Args &a) {
    switch (wpr) {
        case 2: launch_shape<DT, 2, 32, PRE>(a); break;
        case 3: launch_shape<DT, 3, 32, PRE>(a); break;
        case 4: launch_shape<DT, 4, 32, PRE>(a); break;
        case 5: launch_shape<DT, 5, 32, PRE>(a); break;
        case 6: launch_shape<DT, 6, 32, PRE>(a); break;
        case 7: launch_shape<DT, 7, 32, PRE>(a); break;
        default: launch_shape<DT, 8, 32, PRE>(a); break;
    }
}

template <int DT>
static void launch_dtype(int pre, const Args &a) {
    const int nb = a.K / 128;
    if (nb > 32) {
        const int wpr = (nb + 31) / 32;
        if (pre == hq::kPreRmsNorm) return launch_long<DT, hq::kPreRmsNorm>(wpr, a);
        if (pre == hq::kPreSiluMul) return launch_long<DT, hq::kPreSiluMul>(wpr, a);
        return launch_long<DT, hq::kPreNone>(wpr, a);
    }
    int g = 1;
    while (g < nb) g *= 2;
    if (pre == hq::kPreRmsNorm) launch_short<DT, hq::kPreRmsNorm>(g, a);
    else if (pre == hq::kPreSiluMul) launch_short<DT, hq::kPreSiluMul>(g, a);
    else launch_short<DT, hq::kPreNone>(g, a);
}

// Launches the matrix-core kernel when it applies (K a multiple of 128 up to 32768, a
// Hadamard entry the dtype represents exactly); returns QUEST_ERR_UNSUPPORTED otherwise so that the caller can take
// another path.  Whether it applies depends on K, the factor and the dtype only -- never on the number of rows or on
// where the buffers lie -- so that one shape always runs the same arithmetic.
// pre: 0 none, 1 RMSNorm (norm_w, eps; with add_in the norm of x + add_in, the sum written to sum_out), 2 SiLU(gate) * up
// with x a (M, 2 K) tensor.  tiles: the codes as E2M3 tiles (M rows; besides or instead of packed nibbles).
int launch_hadamard_quantize_mfma(int pre, const void *x, const void *norm_w, float eps, void *scale, uint8_t *packed,
                                  int32_t *row_sum, void *x_had, void *pre_out, int K, int M, float had_scale, int dtype,
                                  hipStream_t st, const void *add_in, void *sum_out, uint8_t *tiles) {
    uint32_t bits = 0;
    // (had_scale == 0: no transform; the kernel then only moves the chunks between lanes)
    if (K > 32768 || (K & 127) || had_scale < 0.f || !representable16(had_scale, dtype, &bits)) return QUEST_ERR_UNSUPPORTED;
    const int ldx = pre == hq::kPreSiluMul ? 2 * K : K;
    if (!aligned(pre_out, 16) || !aligned(norm_w, 16)) return QUEST_ERR_UNSUPPORTED;
    if (add_in != nullptr && (pre != hq::kPreRmsNorm || sum_out == nullptr || !aligned(add_in, 16) || !aligned(sum_out, 16)))
        return QUEST_ERR_UNSUPPORTED;
    // The kernel addresses its input with 32-bit byte offsets: tensors of 2 GiB and more go as several launches of
    // whole rows (same kernel, same arithmetic, so the result does not depend on where the cut falls).
    // (cuts at multiples of 32 rows: whole row blocks of the tiles)
    const long max_rows = (((1L << 31) - 1) / ((long)ldx * 2)) & ~31L;
    if (max_rows == 0) return QUEST_ERR_UNSUPPORTED;
    const size_t es = 2;
    const int cus = tiles != nullptr ? device_cu_count(st) : 0;
    for (long r0 = 0; r0 < M; r0 += max_rows) {
        const int rows = (int)(M - r0 < max_rows ? M - r0 : max_rows);
        auto at = [&](const void *p, size_t row_elems, size_t elem) -> void * {
            return p == nullptr ? nullptr : (void *)((const uint8_t *)p + (size_t)r0 * row_elems * elem);
        };
        const Args a = {at(x, ldx, es), norm_w, at(scale, 1, es), (uint8_t *)at(packed, K / 2, 1), (int32_t *)at(row_sum, 1, 4),
                        at(x_had, K, es), at(pre_out, K, es), at(add_in, K, es), at(sum_out, K, es),
                        tiles == nullptr ? nullptr : tiles + (size_t)(r0 / 32) * (size_t)(K / 64) * 1536, K, rows, ldx, bits, eps, st, cus};
        if (dtype == QUEST_DTYPE_BF16) launch_dtype<0>(pre, a);
        else launch_dtype<1>(pre, a);
    }
    return launch_status();
}

}  // namespace quest
