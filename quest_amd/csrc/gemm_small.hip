// Small-tile packed-INT4 x packed-INT4 GEMM (K % 256 == 0): a few hundred tokens.  Same arithmetic and outputs as the
// other GEMM kernels (gemm-quest/quest/matmul_kernel.cu:8-63 and gemm-quest/quest/fused_matmul_dequantize_kernel.cu:4-57
// of the reference).
//
// Between the weight-streaming kernel (a handful of tokens) and the large tiles (thousands) there are too few
// 256-token tiles to fill the chip, and a large tile that is one or two channel units wide leaves a lone wave per
// SIMD issuing a few hundred instructions per stage around four multiplications.  Here a workgroup of eight waves
// owns 64 tokens x 64 channels and splits K four ways: wave (q, c) multiplies all 64 tokens by channel half c over
// k-pair q of every 256-k stage (two accumulators; 9 nibble-splitting operations per MFMA instead of 12 for a
// 32 x 32 quadrant per wave).  Every SIMD has two waves of a tile and, with two or more tiles per CU, four or more.
// The four partial sums meet in LDS at the end, and all eight waves share the epilogue.  Operands travel as in the
// large-tile kernel: packed bytes HBM -> LDS by direct loads (stages of 256 k = two sub-stages of 64-byte rows,
// each wave bringing 16 token or channel rows), 16 packed bytes per lane per k-pair, split into the int8 vectors of
// 16 * even-k and 16 * odd-k nibbles for two MFMA k-steps.
#include "gemm_tiles.h"

namespace quest {

namespace small {

constexpr int kRowB = 64;                         // packed bytes per row per sub-stage (128 k)
constexpr int kStages = 4;
constexpr int kTB = 2;                            // token sub-tiles of 32 per wave

// Two shapes of the kernel, eight waves each:
//   Shape<1, 1, 4>   64 tokens x 64 channels; wave (q, c) multiplies all 64 tokens by channel half c (one 32-row unit)
//                    over k-pair q of the four in a stage.  16 KiB stages, 64 KiB of LDS, two workgroups per CU.
//   Shape<2, 2, 2>   128 x 128; wave (q, t, c) multiplies token half t by channel half c (two units) over the two
//                    k-pairs of sub-stage q.  Half the operand bytes and two thirds of the nibble splitting per
//                    MFMA; 32 KiB stages, 128 KiB of LDS, one workgroup per CU.
template <int TW, int NA, int KQ>
struct Shape {
    static_assert(TW * 2 * KQ == 8, "eight waves");
    static constexpr int kTokWaves = TW, kUnits = NA, kSplit = KQ;
    static constexpr int kTok = 64 * TW, kChn = 64 * NA;
    static constexpr int kHalfB = (kTok + kChn) * kRowB;          // the token rows of a sub-stage, then its channel rows
    static constexpr int kStageB = 2 * kHalfB;                    // 256 k
    static constexpr int kLoads = (kTok + kChn) / 16 / 8;         // 16-row direct loads per wave per sub-stage
    static constexpr int kAccRegs = kTB * NA * 16;
    static constexpr int kParkB = 8 * kAccRegs * 256;             // every wave's accumulators, for the K reduction
    static constexpr int kLdsB = kStages * kStageB > kParkB ? kStages * kStageB : kParkB;
    static constexpr int kPairs = 4 / KQ;                         // k-pairs per wave per stage
    static constexpr int kPieces = kTB * NA * 2 / KQ;             // epilogue pieces (32 tokens x 16 channels) per wave
    static constexpr int kWgPerCu = kLdsB <= 64 * 1024 ? 2 : 1;
};
using Tile64 = Shape<1, 1, 4>;
using Tile128 = Shape<2, 2, 2>;

template <typename S, int OUT, int EPI>
__global__ void __launch_bounds__(512, 2 * S::kWgPerCu)
gemm_w4a4_small_kernel(void *__restrict__ out, const uint8_t *__restrict__ act, const uint8_t *__restrict__ wgt,
                       const int32_t *__restrict__ a_add, const int32_t *__restrict__ b_add,
                       const uint16_t *__restrict__ a_mul, const uint16_t *__restrict__ b_mul,
                       int M, int N, int K, int tiles_t, int tiles_c, RopeArgs rope) {
    __shared__ __attribute__((aligned(1024))) uint8_t lds[S::kLdsB];
    constexpr int DT = OUT == OUT_INT32 ? 0 : OUT;
    constexpr bool GLU = EPI == kEpiGlu;
    constexpr bool ROPE = EPI == kEpiRope;            // (the caller guarantees N % 8 == 0 and a 16-byte aligned output)
    static_assert(EPI == kEpiPlain || OUT != OUT_INT32, "epilogues on 16-bit outputs only");
    constexpr int NA = S::kUnits, TW = S::kTokWaves;
    const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
    const int lane = (int)threadIdx.x & 63;
    // Workgroups are dealt to the eight XCDs in turn: all token tiles of a channel tile go to one XCD, whose L2 then
    // fetches those weight rows once.  The grid is rounded up to whole eights of channel tiles.
    const int xcd = (int)blockIdx.x & 7, local = (int)blockIdx.x >> 3;
    const int ct = (local / tiles_t) * 8 + xcd;
    const int tt = local % tiles_t;
    if (ct >= tiles_c) return;                                   // uniform: the whole workgroup
    const int tok0 = tt * S::kTok, ch0 = ct * S::kChn;
    const int kbytes = K >> 1;
    const int nk = K / 256;

    // ---- loads: waves 0-3 bring the token rows, waves 4-7 the channel rows of each sub-stage, kLoads groups of 16 each
    const bool ld_tok = wave < 4;
    const __amdgpu_buffer_rsrc_t src = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(ld_tok ? act : wgt), 0, (ld_tok ? M : N) * kbytes, 0x00020000);      // rows past the end read as zeros
    // lane p covers row p / 4 of the 16; LDS slot p (lane order) must hold chunk (p & 3) ^ ((row >> 2) & 3) of that row
    const int ld_row0 = (wave & 3) * S::kLoads * 16;
    const uint32_t voff = (uint32_t)((ld_tok ? tok0 : ch0) + ld_row0 + (lane >> 2)) * (uint32_t)kbytes +
                          (uint32_t)(((lane & 3) ^ ((lane >> 4) & 3)) * 16);
    uint8_t *const dst0 = lds + (ld_tok ? 0 : S::kTok * kRowB) + ld_row0 * kRowB;
    auto issue = [&](int kt, int slot) {
#pragma unroll
        for (int j = 0; j < S::kLoads; j++) {
            uint8_t *d = dst0 + slot * S::kStageB + j * 16 * kRowB;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(src, (__attribute__((address_space(3))) void *)d, 16,
                                                     voff + (uint32_t)(j * 16 * kbytes), kt * 128, 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(src, (__attribute__((address_space(3))) void *)(d + S::kHalfB), 16,
                                                     voff + (uint32_t)(j * 16 * kbytes), kt * 128 + 64, 0, 0);
        }
    };

    // ---- operand reads: k-pair p of the stage = 16-byte chunk 2 (p & 1) + lg of the 64-byte rows of sub-stage p >> 1;
    // the wave takes k-pairs kq kPairs .. + kPairs, row li of its token sub-tiles and of its channel units
    const int kq = wave / (2 * TW), tw = (wave >> 1) % TW, tc = wave & 1;
    const int li = lane & 31, lg = lane >> 5;
    int rd_x[S::kPairs];
#pragma unroll
    for (int i = 0; i < S::kPairs; i++) {
        const int p = kq * S::kPairs + i;
        rd_x[i] = (p >> 1) * S::kHalfB + ((2 * (p & 1) + lg) ^ ((li >> 2) & 3)) * 16;
    }
    const int rd_t = (tw * 64 + li) * kRowB;
    const int rd_c = (S::kTok + tc * NA * 32 + li) * kRowB;

    v16i acc[NA][kTB];                                   // independent chains of MFMAs
#pragma unroll
    for (int a = 0; a < NA; a++)
#pragma unroll
        for (int b = 0; b < kTB; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[a][b][r] = 0;

    // Stages 0 .. kStages - 2 in flight before the loop; past the end of K the last stage is fetched again (into a
    // free slot), which keeps the count of outstanding loads uniform.
#pragma unroll
    for (int s = 0; s < kStages - 1; s++) issue(s < nk ? s : nk - 1, s);
    for (int kt = 0; kt < nk; kt++) {
        wait_vmcnt_imm<2 * S::kLoads * (kStages - 2)>();    // this wave's share of stage kt has landed ...
        plain_barrier();                            // ... and everyone else's; the slot of stage kt - 1 is free
        const int nx = kt + kStages - 1;
        issue(nx < nk ? nx : nk - 1, nx % kStages);
        const uint8_t *sb = lds + (kt % kStages) * S::kStageB;
#pragma unroll
        for (int i = 0; i < S::kPairs; i++) {
            v4i te[kTB], to[kTB], ce[NA], co[NA];
#pragma unroll
            for (int a = 0; a < NA; a++)
                split16(*reinterpret_cast<const v4i *>(sb + rd_c + a * 32 * kRowB + rd_x[i]), ce[a], co[a]);
#pragma unroll
            for (int b = 0; b < kTB; b++)
                split16(*reinterpret_cast<const v4i *>(sb + rd_t + b * 32 * kRowB + rd_x[i]), te[b], to[b]);
#pragma unroll
            for (int a = 0; a < NA; a++)
#pragma unroll
                for (int b = 0; b < kTB; b++)
                    acc[a][b] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ce[a], te[b], acc[a][b], 0, 0, 0);
#pragma unroll
            for (int a = 0; a < NA; a++)
#pragma unroll
                for (int b = 0; b < kTB; b++)
                    acc[a][b] = __builtin_amdgcn_mfma_i32_32x32x32_i8(co[a], to[b], acc[a][b], 0, 0, 0);
        }
    }
    wait_vmcnt_imm<0>();                            // no direct-to-LDS load may still be writing ...
    plain_barrier();                                // ... and nobody still reading when the stages are reused

    // ---- the K parts meet in LDS: every wave parks its accumulators; wave q of a quadrant then sums and finishes
    // kPieces pieces of it, each a token sub-tile x 16 channels (register groups 2 pr and 2 pr + 1 of one unit)
    int32_t *red = reinterpret_cast<int32_t *>(lds);
#pragma unroll
    for (int a = 0; a < NA; a++)
#pragma unroll
        for (int b = 0; b < kTB; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) red[(wave * S::kAccRegs + (a * kTB + b) * 16 + r) * 64 + lane] = acc[a][b][r];
    __syncthreads();
    const bool vec16 = (reinterpret_cast<uintptr_t>(out) & 15) == 0;
#pragma unroll
    for (int i = 0; i < S::kPieces; i++) {
        const int piece = kq * S::kPieces + i;           // = b + kTB (a + NA pr)
        const int tb = piece % kTB, ta = (piece / kTB) % NA, pr = piece / (kTB * NA);
        int sum[8];
#pragma unroll
        for (int r = 0; r < 8; r++) {
            sum[r] = 0;
#pragma unroll
            for (int q = 0; q < S::kSplit; q++)
                sum[r] += red[((q * 2 * TW + tw * 2 + tc) * S::kAccRegs + (ta * kTB + tb) * 16 + pr * 8 + r) * 64 + lane];
        }

        // accumulator register r of lane (li, lg) is 256 x the product for token li of the sub-tile and channel
        // 8 (r / 4) + 4 lg + r % 4 of the unit; sum[r] is register 8 pr + r
        const int tok = tok0 + tw * 64 + tb * 32 + li;
        const int cb = ch0 + (tc * NA + ta) * 32 + pr * 16;      // first channel of the piece's two register groups
        const bool tok_ok = tok < M;
        if constexpr (OUT == OUT_INT32) {
            int32_t *dst = reinterpret_cast<int32_t *>(out) + (size_t)(tok_ok ? tok : 0) * N;
            const bool vec_ok = (N & 3) == 0 && vec16;           // 16-byte stores
#pragma unroll
            for (int g = 0; g < 2; g++) {
                const int c = cb + g * 8 + lg * 4;
                if (!tok_ok) continue;
                if (vec_ok) {
                    if (c < N)
                        *reinterpret_cast<int4 *>(dst + c) =
                            make_int4(sum[g * 4] >> 8, sum[g * 4 + 1] >> 8, sum[g * 4 + 2] >> 8, sum[g * 4 + 3] >> 8);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (c + e < N) dst[c + e] = sum[g * 4 + e] >> 8;
                }
            }
        } else {
            const int t_add = tok_ok ? a_add[tok] : 0;
            const float t_half_mul = tok_ok ? __fmul_rn(0.5f, to_f32<DT>(a_mul[tok])) : 0.f;
            // GLU: weight rows interleaved in eights, the output has N / 2 columns (the caller guarantees N % 8 == 0
            // and an 8-byte aligned output)
            uint16_t *dst = reinterpret_cast<uint16_t *>(out) + (size_t)(tok_ok ? tok : 0) * (GLU ? N >> 1 : N);
            const bool fast = GLU || ((N & 7) == 0 && vec16);    // 16-byte stores
            float v[2][4];
#pragma unroll
            for (int g = 0; g < 2; g++) {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int c = cb + g * 8 + lg * 4 + e;
                    const int cc = c < N ? c : N - 1;
                    // the accumulator is 256 C exactly, so 2 C is one arithmetic shift
                    const float lhs = (float)((sum[g * 4 + e] >> 7) + t_add + b_add[cc]);
                    const float rhs = __fmul_rn(t_half_mul, to_f32<DT>(b_mul[cc]));
                    v[g][e] = __fmul_rn(lhs, rhs);
                }
            }
            if (fast) {
                // the half-waves trade register groups, so that every lane stores 16 bytes = 8 consecutive channels:
                // lower half-wave group 0 complete, upper half-wave group 1
                const uint32_t x00 = pack2_rounded_products<DT>(v[0][0], v[0][1]);
                const uint32_t x01 = pack2_rounded_products<DT>(v[0][2], v[0][3]);
                const uint32_t x10 = pack2_rounded_products<DT>(v[1][0], v[1][1]);
                const uint32_t x11 = pack2_rounded_products<DT>(v[1][2], v[1][3]);
                const auto s0 = __builtin_amdgcn_permlane32_swap(x00, x10, false, false);
                const auto s1 = __builtin_amdgcn_permlane32_swap(x01, x11, false, false);
                const int c = cb + lg * 8;
                if constexpr (GLU) {
                    // the lane holds four gate rows, then the four up rows of the same outputs
                    if (tok_ok && c < N)
                        *reinterpret_cast<uint2 *>(dst + (c >> 1)) =
                            make_uint2(silu_mul_pair<DT>(s0[0], s0[1]), silu_mul_pair<DT>(s1[0], s1[1]));
                } else if (tok_ok && c < N) {
                    uint4 piece8 = make_uint4(s0[0], s1[0], s0[1], s1[1]);
                    if constexpr (ROPE) {
                        // q and k of a fused QKV projection leave rotated: the piece's four (re, im) pairs by the angles of
                        // its row's position in its sequence (the other waves of the CU cover the fetch)
                        if (c < rope.rot_cols) {
                            const int t = tok % rope.seq_len, h = c % rope.head_dim;
                            const float4 *f = reinterpret_cast<const float4 *>(rope.freqs + ((size_t)t * (rope.head_dim >> 1) + (h >> 1)) * 2);
                            const float4 cs[2] = {f[0], f[1]};
                            piece8 = rope_turn<DT>(piece8, cs);
                        }
                    }
                    *reinterpret_cast<uint4 *>(dst + c) = piece8;
                }
            } else if (!GLU && tok_ok) {
#pragma unroll
                for (int g = 0; g < 2; g++)
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const int c = cb + g * 8 + lg * 4 + e;
                        if (c < N) dst[c] = (uint16_t)from_f32<DT>(v[g][e]);
                    }
            }
        }
    }
}

}  // namespace small

template <typename S, int OUT, int EPI>
static int launch_small(void *out, const uint8_t *a, const uint8_t *b, const int32_t *a_add, const int32_t *b_add,
                             const void *a_mul, const void *b_mul, int M, int K, int N, hipStream_t st, const RopeArgs &rope) {
    const int tiles_t = (M + S::kTok - 1) / S::kTok;
    const int tiles_c = (N + S::kChn - 1) / S::kChn;
    const long grid = (long)tiles_t * ((tiles_c + 7) / 8) * 8;
    small::gemm_w4a4_small_kernel<S, OUT, EPI><<<dim3((unsigned)grid), dim3(512), 0, st>>>(
        out, a, b, a_add, b_add, (const uint16_t *)a_mul, (const uint16_t *)b_mul, M, N, K, tiles_t, tiles_c, rope);
    return launch_status();
}

template <int OUT, int EPI>
static int launch_shape(int shape, void *out, const uint8_t *a, const uint8_t *b, const int32_t *a_add, const int32_t *b_add,
                        const void *a_mul, const void *b_mul, int M, int K, int N, hipStream_t st, const RopeArgs &rope) {
    if (shape == 128) return launch_small<small::Tile128, OUT, EPI>(out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, st, rope);
    return launch_small<small::Tile64, OUT, EPI>(out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, st, rope);
}

int launch_gemm_small(int out_kind, int epi, int shape, void *out, const uint8_t *a, const uint8_t *b, const int32_t *a_add,
                      const int32_t *b_add, const void *a_mul, const void *b_mul, int M, int K, int N, hipStream_t st,
                      const RopeArgs *rope_args) {
    if ((K & 255) != 0 || (shape != 64 && shape != 128) || (epi != kEpiPlain && out_kind == OUT_INT32)) return QUEST_ERR_UNSUPPORTED;
    if (epi == kEpiRope && (rope_args == nullptr || (N & 7) != 0 || !aligned(out, 16))) return QUEST_ERR_UNSUPPORTED;
    const RopeArgs rope = epi == kEpiRope ? *rope_args : RopeArgs{nullptr, 32, 0, 32};
#define QUEST_SMALL_EPI(E)                                                                                                   \
    (out_kind == OUT_BF16 ? launch_shape<OUT_BF16, E>(shape, out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, st, rope)        \
                          : launch_shape<OUT_FP16, E>(shape, out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, st, rope))
    if (epi == kEpiGlu) return QUEST_SMALL_EPI(kEpiGlu);
    if (epi == kEpiRope) return QUEST_SMALL_EPI(kEpiRope);
    if (epi != kEpiPlain) return QUEST_ERR_UNSUPPORTED;
    if (out_kind == OUT_INT32) return launch_shape<OUT_INT32, kEpiPlain>(shape, out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, st, rope);
    return QUEST_SMALL_EPI(kEpiPlain);
#undef QUEST_SMALL_EPI
}

}  // namespace quest
