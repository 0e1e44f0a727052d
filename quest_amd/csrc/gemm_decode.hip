// Packed-INT4 x packed-INT4 GEMM for a handful of tokens (M <= 128): the weight matrix is streamed
// from HBM exactly once and that stream is the whole cost, so the kernel is laid out around it.
//
// Same arithmetic and outputs as the large GEMM (gemm-quest/quest/matmul_kernel.cu:8-63 and
// gemm-quest/quest/fused_matmul_dequantize_kernel.cu:4-57 of the reference, which run their one
// CUTLASS tile shape at every M); this is the shape the reference's decode benchmark exercises
// (gemm-quest/benchmarks/bench_e2e.py with one token per sequence).
//
// A workgroup of eight waves owns 16 output channels over the whole K; wave w takes the 256-k
// chunks w, w + 8, ...  For a chunk a lane (r = lane % 16, g = lane / 16) loads two 16-byte pieces
// of weight row r -- bytes 16 g and 64 + 16 g of the chunk's 128 -- so the wave's two loads cover one
// whole 128-byte line of each of its 16 rows, and the same two pieces of token row r.  A piece is 32
// nibbles: `w & 0xF0F0F0F0` is 16 * (odd-k nibbles), `(w << 4) & 0xF0F0F0F0` is 16 * (even-k
// nibbles), both sign-correct int8, each feeding one v_mfma_i32_16x16x64_i8 (weights as the "A"
// operand, tokens as "B"; both operands permute k identically, which a dot product ignores).  All
// of a wave's loads for up to four chunks are in flight before the first is used.  The eight partial
// 16 x 16 tiles meet in LDS, the factor 256 the nibble trick leaves is shifted out exactly, and the
// first wave(s) apply the scale epilogue and store four consecutive channels of a token per lane.
#include "common.h"

namespace quest {
namespace decode {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kWaves = 8;
constexpr int kChannels = 16;             // output channels per workgroup
constexpr int kChunkB = 128;              // packed bytes per row per chunk (256 k)
constexpr int kBatch = 2;                 // chunks whose loads are in flight together per wave: few, so that the
                                          // registers allow many waves per SIMD (8 at TM = 1) and the 256 to 688
                                          // workgroups of the layer shapes all run at once -- measured 7..23 % faster
                                          // than four chunks per wave at five waves per SIMD

__device__ __forceinline__ void split16(const v4i &p, v4i &even, v4i &odd) {
#pragma unroll
    for (int d = 0; d < 4; d++) {
        odd[d] = p[d] & (int)0xF0F0F0F0u;
        even[d] = (p[d] << 4) & (int)0xF0F0F0F0u;
    }
}

// TM = token tiles of 16 (M <= 16 TM)
template <int OUT, int TM>
__global__ void __launch_bounds__(64 * kWaves, TM == 1 ? 8 : TM == 2 ? 4 : TM == 4 ? 2 : 1)
gemm_w4a4_decode_kernel(void *__restrict__ out, const uint8_t *__restrict__ act, const uint8_t *__restrict__ wgt,
                        const int32_t *__restrict__ a_add, const int32_t *__restrict__ b_add,
                        const uint16_t *__restrict__ a_mul, const uint16_t *__restrict__ b_mul, int M, int N, int K) {
    __shared__ __attribute__((aligned(16))) int red[kWaves][TM][64][4];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 15;
    const int g = lane >> 4;
    const int row_b = K >> 1;                          // packed bytes per row
    const int ch0 = blockIdx.x * kChannels;
    const int n_chunks = (row_b + kChunkB - 1) / kChunkB;      // the last one may hold only its first 64 bytes

    // rows that do not exist get an offset beyond the buffer: such loads touch no memory and return zeros
    const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc((void *)wgt, 0, (int)((long)N * row_b), 0x00020000);
    const __amdgpu_buffer_rsrc_t ar = __builtin_amdgcn_make_buffer_rsrc((void *)act, 0, (int)((long)M * row_b), 0x00020000);
    const uint32_t dead = 0x80000000u;                 // buffers are smaller than 2^31 bytes; sums below stay under 2^32
    const uint32_t w_off = (ch0 + r < N) ? (uint32_t)((ch0 + r) * row_b + g * 16) : dead;
    uint32_t a_off[TM];
#pragma unroll
    for (int t = 0; t < TM; t++) a_off[t] = (t * 16 + r < M) ? (uint32_t)((t * 16 + r) * row_b + g * 16) : dead;

    // the waves that will finish a token tile fetch their epilogue operands now, off the critical path
    // (lane (r, g) of wave t ends up with channels ch0 + 4 g + {0..3} of token 16 t + r)
    int t_add = 0, c_add[4] = {0, 0, 0, 0};
    float t_half_mul = 0.f, c_mul[4] = {0.f, 0.f, 0.f, 0.f};
    if constexpr (OUT != OUT_INT32) {
        if (wave < TM) {
            const int tok = min(wave * 16 + r, M - 1);
            t_add = a_add[tok];
            t_half_mul = __fmul_rn(0.5f, to_f32<OUT>(a_mul[tok]));
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int che = min(ch0 + 4 * g + e, N - 1);
                c_add[e] = b_add[che];
                c_mul[e] = to_f32<OUT>(b_mul[che]);
            }
        }
    }

    v4i acc[TM];
#pragma unroll
    for (int t = 0; t < TM; t++) acc[t] = v4i{0, 0, 0, 0};

    for (int c0 = wave; c0 < n_chunks; c0 += kWaves * kBatch) {
        v4i wq[kBatch][2], aq[kBatch][TM][2];
#pragma unroll
        for (int i = 0; i < kBatch; i++) {
            const int c = c0 + i * kWaves;
            const int cb = c * kChunkB;
#pragma unroll
            for (int hlf = 0; hlf < 2; hlf++) {
                // a piece past the end of the row (chunk index too large, or the second half of a 64-byte tail) reads as zero
                const bool in_row = c < n_chunks && cb + 64 * hlf < row_b;
                const uint32_t shift = (uint32_t)(cb + 64 * hlf);
                wq[i][hlf] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(wr, (int)(in_row ? w_off + shift : dead), 0, 0));
#pragma unroll
                for (int t = 0; t < TM; t++)
                    aq[i][t][hlf] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(ar, (int)(in_row ? a_off[t] + shift : dead), 0, 0));
            }
        }
        // every load of the batch in flight before the first is used (the scheduler would otherwise sink some of
        // them between the MFMAs to save registers and pay a second trip to memory)
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < kBatch; i++)
#pragma unroll
            for (int hlf = 0; hlf < 2; hlf++) {
                v4i we, wo;
                split16(wq[i][hlf], we, wo);
#pragma unroll
                for (int t = 0; t < TM; t++) {
                    v4i ae, ao;
                    split16(aq[i][t][hlf], ae, ao);
                    acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(we, ae, acc[t], 0, 0, 0);
                    acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wo, ao, acc[t], 0, 0, 0);
                }
            }
    }

    // ---- partial tiles meet in LDS
#pragma unroll
    for (int t = 0; t < TM; t++) *reinterpret_cast<v4i *>(&red[wave][t][lane][0]) = acc[t];
    __syncthreads();
    if (wave >= TM) return;
    const int t = wave;                                  // wave t finishes token tile t
    v4i sum = v4i{0, 0, 0, 0};
#pragma unroll
    for (int w = 0; w < kWaves; w++) {
        const v4i p = *reinterpret_cast<const v4i *>(&red[w][t][lane][0]);
#pragma unroll
        for (int e = 0; e < 4; e++) sum[e] += p[e];
    }

    const int tok = t * 16 + r;
    const int ch = ch0 + 4 * g;
    if (tok >= M || ch >= N) return;
    int c[4];
#pragma unroll
    for (int e = 0; e < 4; e++) c[e] = sum[e] >> 8;      // exact: every product carries 16 * 16
    const size_t o = (size_t)tok * N + ch;
    if constexpr (OUT == OUT_INT32) {
        int32_t *dst = reinterpret_cast<int32_t *>(out) + o;
        if ((N & 3) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0) {
            *reinterpret_cast<int4 *>(dst) = make_int4(c[0], c[1], c[2], c[3]);
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (ch + e < N) dst[e] = c[e];
        }
    } else {
        uint32_t h[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const float lhs = (float)(c[e] * 2 + t_add + c_add[e]);
            const float rhs = __fmul_rn(t_half_mul, c_mul[e]);
            h[e] = from_f32<OUT>(__fmul_rn(lhs, rhs));
        }
        uint16_t *dst = reinterpret_cast<uint16_t *>(out) + o;
        if ((N & 3) == 0 && (reinterpret_cast<uintptr_t>(out) & 7) == 0) {
            *reinterpret_cast<uint2 *>(dst) = make_uint2(h[0] | (h[1] << 16), h[2] | (h[3] << 16));
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (ch + e < N) dst[e] = (uint16_t)h[e];
        }
    }
}

// ---- the same for M <= 16 with K split across workgroups --------------------------------------------------------------
// A workgroup of four waves multiplies 16 channels by one of S slices of K and leaves its partial int32 tile (1 KiB) in
// the caller's workspace; a counter per channel tile tells the workgroup that arrives last, which adds the S partial
// tiles (integers: any order gives the same sum), applies the epilogue, stores, and puts the counter back to zero.  No
// atomic touches the result.  S times the workgroups of the kernel above for the same bytes: shorter dependent chains
// per wave for long rows.  Workspace: ceil(N / 16) counters (zero before the first use, zero again after every launch),
// then, from byte kSplitPartialsAt on, ceil(N / 16) x S tiles of 256 ints.
constexpr int kSplitWaves = 4;
constexpr int kMaxSplits = 8;
constexpr size_t kSplitPartialsAt = 16384;          // room for 4096 counters: N <= 65536

template <int OUT>
__global__ void __launch_bounds__(64 * kSplitWaves, 8)
gemm_w4a4_decode_splitk_kernel(void *__restrict__ out, const uint8_t *__restrict__ act, const uint8_t *__restrict__ wgt,
                               const int32_t *__restrict__ a_add, const int32_t *__restrict__ b_add,
                               const uint16_t *__restrict__ a_mul, const uint16_t *__restrict__ b_mul, int M, int N, int K,
                               int *__restrict__ counters, int *__restrict__ partials) {
    __shared__ __attribute__((aligned(16))) int red[kSplitWaves][64][4];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 15;
    const int g = lane >> 4;
    const int row_b = K >> 1;
    const int tile = blockIdx.x;
    const int ch0 = tile * kChannels;
    const int splits = gridDim.y;
    const int n_chunks = (row_b + kChunkB - 1) / kChunkB;
    const int c_lo = (int)(((long)n_chunks * blockIdx.y) / splits);
    const int c_hi = (int)(((long)n_chunks * (blockIdx.y + 1)) / splits);

    const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc((void *)wgt, 0, (int)((long)N * row_b), 0x00020000);
    const __amdgpu_buffer_rsrc_t ar = __builtin_amdgcn_make_buffer_rsrc((void *)act, 0, (int)((long)M * row_b), 0x00020000);
    const uint32_t dead = 0x80000000u;
    const uint32_t w_off = (ch0 + r < N) ? (uint32_t)((ch0 + r) * row_b + g * 16) : dead;
    const uint32_t a_off = (r < M) ? (uint32_t)(r * row_b + g * 16) : dead;

    v4i acc = v4i{0, 0, 0, 0};
    for (int c0 = c_lo + wave; c0 < c_hi; c0 += kSplitWaves * kBatch) {
        v4i wq[kBatch][2], aq[kBatch][2];
#pragma unroll
        for (int i = 0; i < kBatch; i++) {
            const int c = c0 + i * kSplitWaves;
            const int cb = c * kChunkB;
#pragma unroll
            for (int hlf = 0; hlf < 2; hlf++) {
                const bool in_row = c < c_hi && cb + 64 * hlf < row_b;
                const uint32_t shift = (uint32_t)(cb + 64 * hlf);
                wq[i][hlf] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(wr, (int)(in_row ? w_off + shift : dead), 0, 0));
                aq[i][hlf] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(ar, (int)(in_row ? a_off + shift : dead), 0, 0));
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < kBatch; i++)
#pragma unroll
            for (int hlf = 0; hlf < 2; hlf++) {
                v4i we, wo, ae, ao;
                split16(wq[i][hlf], we, wo);
                split16(aq[i][hlf], ae, ao);
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(we, ae, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(wo, ao, acc, 0, 0, 0);
            }
    }

    // ---- the workgroup's partial tile: the four waves meet in LDS, wave 0 carries it on
    *reinterpret_cast<v4i *>(&red[wave][lane][0]) = acc;
    __syncthreads();
    if (wave != 0) return;
    v4i sum = v4i{0, 0, 0, 0};
#pragma unroll
    for (int w = 0; w < kSplitWaves; w++) {
        const v4i p = *reinterpret_cast<const v4i *>(&red[w][lane][0]);
#pragma unroll
        for (int e = 0; e < 4; e++) sum[e] += p[e];
    }
    if (splits > 1) {
        // Publish, count, and let the last arriver gather.  The slices of one channel tile may run on different XCDs, whose
        // L2 caches do not see each other's lines; a device-wide release / acquire fence would write back and invalidate a
        // whole L2 per workgroup (measured: ten times the kernel's time).  Instead the partial tiles travel past the
        // caches: stores and loads with both coherence bits set go to the memory side, the counter is a device-scope
        // atomic, and the store is complete (vmcnt) before the count.
        const __amdgpu_buffer_rsrc_t pr = __builtin_amdgcn_make_buffer_rsrc((void *)partials, 0, (int)(gridDim.x * splits * 1024), 0x00020000);
        constexpr int kPastCaches = 1 | 16;             // sc0 sc1
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(__attribute__((__vector_size__(4 * sizeof(unsigned int)))) unsigned int, sum), pr, (int)((tile * splits + blockIdx.y) * 1024 + lane * 16), 0, kPastCaches);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        int arrived = 0;
        if (lane == 0) arrived = __hip_atomic_fetch_add(counters + tile, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (__builtin_amdgcn_readfirstlane(arrived) != splits - 1) return;
        asm volatile("" ::: "memory");
        v4i part[kMaxSplits];                          // every slice's tile in flight at once; slices past the last read as zero
#pragma unroll
        for (int sl = 0; sl < kMaxSplits; sl++)
            part[sl] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(pr, sl < splits ? (int)((tile * splits + sl) * 1024 + lane * 16) : (int)0x80000000, 0, kPastCaches));
        sum = v4i{0, 0, 0, 0};
#pragma unroll
        for (int sl = 0; sl < kMaxSplits; sl++)
#pragma unroll
            for (int e = 0; e < 4; e++) sum[e] += part[sl][e];
        if (lane == 0) __hip_atomic_store(counters + tile, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);     // ready for the next launch
    }

    const int tok = r;
    const int ch = ch0 + 4 * g;
    if (tok >= M || ch >= N) return;
    int c[4];
#pragma unroll
    for (int e = 0; e < 4; e++) c[e] = sum[e] >> 8;      // exact: every product carries 16 * 16
    const size_t o = (size_t)tok * N + ch;
    if constexpr (OUT == OUT_INT32) {
        int32_t *dst = reinterpret_cast<int32_t *>(out) + o;
        if ((N & 3) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0) {
            *reinterpret_cast<int4 *>(dst) = make_int4(c[0], c[1], c[2], c[3]);
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (ch + e < N) dst[e] = c[e];
        }
    } else {
        const int t_add = a_add[tok];
        const float t_half_mul = __fmul_rn(0.5f, to_f32<OUT>(a_mul[tok]));
        uint32_t h[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int che = min(ch + e, N - 1);
            const float lhs = (float)(c[e] * 2 + t_add + b_add[che]);
            const float rhs = __fmul_rn(t_half_mul, to_f32<OUT>(b_mul[che]));
            h[e] = from_f32<OUT>(__fmul_rn(lhs, rhs));
        }
        uint16_t *dst = reinterpret_cast<uint16_t *>(out) + o;
        if ((N & 3) == 0 && (reinterpret_cast<uintptr_t>(out) & 7) == 0) {
            *reinterpret_cast<uint2 *>(dst) = make_uint2(h[0] | (h[1] << 16), h[2] | (h[3] << 16));
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (ch + e < N) dst[e] = (uint16_t)h[e];
        }
    }
}

template <int OUT, int TM>
static void launch_tm(void *out, const uint8_t *a, const uint8_t *b, const int32_t *a_add, const int32_t *b_add,
                      const void *a_mul, const void *b_mul, int M, int K, int N, hipStream_t st) {
    gemm_w4a4_decode_kernel<OUT, TM><<<dim3((N + kChannels - 1) / kChannels), dim3(64 * kWaves), 0, st>>>(
        out, a, b, a_add, b_add, (const uint16_t *)a_mul, (const uint16_t *)b_mul, M, N, K);
}

template <int OUT>
static int launch_out(void *out, const uint8_t *a, const uint8_t *b, const int32_t *a_add, const int32_t *b_add,
                      const void *a_mul, const void *b_mul, int M, int K, int N, hipStream_t st) {
    if (M <= 16) launch_tm<OUT, 1>(out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, st);
    else if (M <= 32) launch_tm<OUT, 2>(out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, st);
    else if (M <= 64) launch_tm<OUT, 4>(out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, st);
    else launch_tm<OUT, 8>(out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, st);
    return launch_status();
}

// How many slices of K pay for M <= 16 tokens.  The hand-off through memory (store past the caches, count, load) costs
// 2-2.5 us, more than the whole kernel above takes on an 8 MB layer, so slices pay only where that kernel's few
// workgroups each walk a long row: measured wins (6.9-12.3 us against 11.2-16.7 us) for K >= 32768 with N <= 2048 and
// K >= 16384 with N <= 1024, losses of 1.5-4 us everywhere else, the Llama decode layers included.  Then: enough
// workgroups to fill the chip several times over, at least two 256-k chunks per wave of a slice.
static int decode_splits(int K, int N) {
    const int tiles = (N + kChannels - 1) / kChannels;
    const int n_chunks = ((K >> 1) + kChunkB - 1) / kChunkB;
    if (!(n_chunks >= 128 && tiles <= 128) && !(n_chunks >= 64 && tiles <= 64)) return 1;
    int s = 1;
    while (s < kMaxSplits && tiles * s * 2 <= 2048 && n_chunks / (s * 2) >= kSplitWaves) s *= 2;
    return s;
}

}  // namespace decode

size_t gemm_decode_workspace_bytes(int K, int N) {
    const int tiles = (N + decode::kChannels - 1) / decode::kChannels;
    const int splits = decode::decode_splits(K, N);
    return splits < 2 ? 0 : decode::kSplitPartialsAt + (size_t)tiles * splits * 256 * sizeof(int);
}

// The split-K form: M <= 16, K % 128 == 0, N <= 65536, a workspace of gemm_decode_workspace_bytes whose counters are zero.
// QUEST_ERR_UNSUPPORTED when it does not apply or would not split (the caller then takes the kernel above).
int launch_gemm_decode_splitk(int out_kind, void *out, const uint8_t *a, const uint8_t *b, const int32_t *a_add,
                              const int32_t *b_add, const void *a_mul, const void *b_mul, int M, int K, int N, void *workspace,
                              size_t workspace_bytes, hipStream_t st) {
    if (M > 16 || (K & 127) != 0 || N > 65536 || !aligned(a, 16) || !aligned(b, 16) || !aligned(workspace, 256)) return QUEST_ERR_UNSUPPORTED;
    const int splits = decode::decode_splits(K, N);
    if (splits < 2 || workspace == nullptr || workspace_bytes < gemm_decode_workspace_bytes(K, N)) return QUEST_ERR_UNSUPPORTED;
    const dim3 grid((N + decode::kChannels - 1) / decode::kChannels, splits), block(64 * decode::kSplitWaves);
    int *counters = (int *)workspace;
    int *partials = (int *)((uint8_t *)workspace + decode::kSplitPartialsAt);
    switch (out_kind) {
        case OUT_BF16:
            decode::gemm_w4a4_decode_splitk_kernel<OUT_BF16><<<grid, block, 0, st>>>(out, a, b, a_add, b_add, (const uint16_t *)a_mul, (const uint16_t *)b_mul, M, N, K, counters, partials);
            break;
        case OUT_FP16:
            decode::gemm_w4a4_decode_splitk_kernel<OUT_FP16><<<grid, block, 0, st>>>(out, a, b, a_add, b_add, (const uint16_t *)a_mul, (const uint16_t *)b_mul, M, N, K, counters, partials);
            break;
        default:
            decode::gemm_w4a4_decode_splitk_kernel<OUT_INT32><<<grid, block, 0, st>>>(out, a, b, a_add, b_add, (const uint16_t *)a_mul, (const uint16_t *)b_mul, M, N, K, counters, partials);
            break;
    }
    return launch_status();
}

// The weight-streaming kernel applies to M <= 128 and K a multiple of 128 (whole 64-byte pieces); QUEST_ERR_UNSUPPORTED otherwise.
int launch_gemm_decode(int out_kind, void *out, const uint8_t *a, const uint8_t *b, const int32_t *a_add,
                       const int32_t *b_add, const void *a_mul, const void *b_mul, int M, int K, int N, hipStream_t st) {
    if (M > 128 || (K & 127) != 0 || !aligned(a, 16) || !aligned(b, 16)) return QUEST_ERR_UNSUPPORTED;
    switch (out_kind) {
        case OUT_BF16: return decode::launch_out<OUT_BF16>(out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, st);
        case OUT_FP16: return decode::launch_out<OUT_FP16>(out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, st);
        default: return decode::launch_out<OUT_INT32>(out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, st);
    }
}

}  // namespace quest
