// Register-staged packed-INT4 x packed-INT4 GEMM: the path for K % 128 != 0 (K % 32 == 0) and for scale vectors that
// are not 4-byte aligned.  Same arithmetic and outputs as the other GEMM kernels (gemm-quest/quest/matmul_kernel.cu:8-63
// and gemm-quest/quest/fused_matmul_dequantize_kernel.cu:4-57 of the reference).
//
// A workgroup of four waves owns a 256-token x 256-channel tile; each wave a 128 x 128
// quarter held as 4 x 4 accumulators of v_mfma_i32_32x32x32_i8.  K advances 128 elements per
// stage.  Packed bytes go HBM -> registers (16 B per lane), are split there into two int8 vectors
// holding 16 * nibble -- `w & 0xF0F0F0F0` is 16 * (odd-k nibbles), `(w << 4) & 0xF0F0F0F0` is
// 16 * (even-k nibbles), both already sign-correct int8 -- and are written to a swizzled,
// double-buffered LDS tile that the MFMA operands are read from with conflict-free 16-byte reads.
// Both operands permute k the same way, so the dot products are unchanged; every product carries
// a factor 256 that the epilogue removes with an exact arithmetic shift (|256 C| <= 2^14 K < 2^31).
// The weight rows feed the MFMA "A" side, so a lane ends up with four consecutive output channels
// of one token and stores them as one 8- or 16-byte vector.
#include "gemm_tiles.h"

namespace quest {

constexpr int kTileRows = 256;                       // rows of either operand per workgroup tile
constexpr int kStageK = 128;                         // k elements per pipeline stage
constexpr int kRowBytes = kStageK;                   // int8 bytes per row per stage in LDS
constexpr int kTileBytes = kTileRows * kRowBytes;    // 32 KiB
constexpr int kStageBytes = 2 * kTileBytes;          // channel tile + token tile
constexpr int kLdsBytes = 2 * kStageBytes;           // double buffered: 128 KiB of the CU's 160 KiB

__device__ __forceinline__ void lds_fence_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// 16-byte position swizzle inside a 128-byte LDS row: keeps both the staging writes and the MFMA
// operand reads free of bank conflicts.
__device__ __forceinline__ int swz(int row) { return (row >> 1) & 7; }

template <int OUT>
__global__ void __launch_bounds__(256)
gemm_w4a4_staged_kernel(void *__restrict__ out, const uint8_t *__restrict__ act, const uint8_t *__restrict__ wgt,
                 const int32_t *__restrict__ a_add, const int32_t *__restrict__ b_add,
                 const uint16_t *__restrict__ a_mul, const uint16_t *__restrict__ b_mul,
                 int M, int N, int K, int tiles_t) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[kLdsBytes];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wc = wave & 1;      // which 128-channel half of the tile
    const int wt = wave >> 1;     // which 128-token half
    const int li = lane & 31;
    const int lg = lane >> 5;

    // Workgroups are dealt round-robin to the 8 XCDs; renumber so that each XCD works on a
    // contiguous run of tiles and its L2 sees the same operand rows again.
    int bid = blockIdx.x;
    const int nb = gridDim.x;
    if ((nb & 7) == 0) bid = (bid & 7) * (nb >> 3) + (bid >> 3);
    const int tile_t = bid % tiles_t;
    const int tile_c = bid / tiles_t;
    const int tok0 = tile_t * kTileRows;
    const int ch0 = tile_c * kTileRows;

    const int kbytes = K >> 1;                     // packed bytes per row
    const int nk = (K + kStageK - 1) / kStageK;

    // ---- global staging: thread t fetches 16 packed bytes of rows (t/4 + 64 i), chunk t%4 --------
    const int srow = tid >> 2;
    const int sq = tid & 3;
    uint32_t po[4], qo[4];                          // byte offsets of this thread's rows (host checks < 2^31)
#pragma unroll
    for (int i = 0; i < 4; i++) {
        int c = ch0 + srow + 64 * i;
        c = c < N ? c : N - 1;
        int t = tok0 + srow + 64 * i;
        t = t < M ? t : M - 1;
        po[i] = (uint32_t)c * (uint32_t)kbytes + sq * 16;
        qo[i] = (uint32_t)t * (uint32_t)kbytes + sq * 16;
    }
    const int st_off_e = ((2 * sq) ^ swz(srow)) * 16;       // rows srow + 64 i share swz
    const int st_off_o = ((2 * sq + 1) ^ swz(srow)) * 16;

    uint4 gp[4], gq[4];

    auto gload = [&](int kt) {
        const int kb = kt * (kStageK / 2);
        const bool ok = kb + sq * 16 < kbytes;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            gp[i] = ok ? *reinterpret_cast<const uint4 *>(wgt + po[i] + kb) : make_uint4(0, 0, 0, 0);
            gq[i] = ok ? *reinterpret_cast<const uint4 *>(act + qo[i] + kb) : make_uint4(0, 0, 0, 0);
        }
    };

    auto split_store = [&](const uint4 &g, uint8_t *base) {
        uint4 e, o;
        e.x = (g.x << 4) & 0xF0F0F0F0u; o.x = g.x & 0xF0F0F0F0u;
        e.y = (g.y << 4) & 0xF0F0F0F0u; o.y = g.y & 0xF0F0F0F0u;
        e.z = (g.z << 4) & 0xF0F0F0F0u; o.z = g.z & 0xF0F0F0F0u;
        e.w = (g.w << 4) & 0xF0F0F0F0u; o.w = g.w & 0xF0F0F0F0u;
        *reinterpret_cast<uint4 *>(base + st_off_e) = e;
        *reinterpret_cast<uint4 *>(base + st_off_o) = o;
    };

    auto lds_store = [&](int stage) {
        uint8_t *sb = lds + stage * kStageBytes + srow * kRowBytes;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            split_store(gp[i], sb + i * 64 * kRowBytes);
            split_store(gq[i], sb + kTileBytes + i * 64 * kRowBytes);
        }
    };

    // ---- MFMA operand reads: lane (li, lg) takes row li of a 32-row sub-tile, 16-byte chunk 2 ks + lg
    int rd_off[4];
#pragma unroll
    for (int ks = 0; ks < 4; ks++) rd_off[ks] = li * kRowBytes + (((2 * ks + lg) ^ swz(li)) * 16);
    const int p_base = (wc * 128) * kRowBytes;
    const int q_base = kTileBytes + (wt * 128) * kRowBytes;

    v16i acc[4][4];
#pragma unroll
    for (int a = 0; a < 4; a++)
#pragma unroll
        for (int b = 0; b < 4; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[a][b][r] = 0;

    v4i pf[2][4], qf[2][4];
    auto frag_load = [&](int buf, int stage, int ks) {
        const uint8_t *sb = lds + stage * kStageBytes + rd_off[ks];
#pragma unroll
        for (int a = 0; a < 4; a++) {
            pf[buf][a] = *reinterpret_cast<const v4i *>(sb + p_base + a * 32 * kRowBytes);
            qf[buf][a] = *reinterpret_cast<const v4i *>(sb + q_base + a * 32 * kRowBytes);
        }
    };
    auto mfma_step = [&](int buf) {
#pragma unroll
        for (int a = 0; a < 4; a++)
#pragma unroll
            for (int b = 0; b < 4; b++)
                acc[a][b] = __builtin_amdgcn_mfma_i32_32x32x32_i8(pf[buf][a], qf[buf][b], acc[a][b], 0, 0, 0);
    };

    // ---- pipeline: LDS holds stage kt, registers hold the packed bytes of stage kt+1 -------------
    gload(0);
    lds_store(0);
    if (nk > 1) gload(1);
    lds_fence_barrier();
    for (int kt = 0; kt < nk; kt++) {
        const int stage = kt & 1;
        frag_load(0, stage, 0);
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            if (ks < 3) frag_load((ks + 1) & 1, stage, ks + 1);
            mfma_step(ks & 1);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (kt + 1 < nk) {
            lds_store(stage ^ 1);
            if (kt + 2 < nk) gload(kt + 2);
        }
        lds_fence_barrier();
    }

    // ---- epilogue: accumulator register r of lane (li, lg) is channel 8 (r/4) + 4 lg + r%4, token li
    const bool vec_ok = (N & 3) == 0;
#pragma unroll
    for (int b = 0; b < 4; b++) {
        const int tok = tok0 + wt * 128 + b * 32 + li;
        if (tok >= M) continue;
        int t_add = 0;
        float t_half_mul = 0.f;
        if constexpr (OUT != OUT_INT32) {
            t_add = a_add[tok];
            t_half_mul = __fmul_rn(0.5f, to_f32<OUT>(a_mul[tok]));
        }
#pragma unroll
        for (int a = 0; a < 4; a++) {
#pragma unroll
            for (int rg = 0; rg < 4; rg++) {
                const int ch = ch0 + wc * 128 + a * 32 + rg * 8 + lg * 4;
                if (ch >= N) continue;
                int c[4];
#pragma unroll
                for (int e = 0; e < 4; e++) c[e] = acc[a][b][rg * 4 + e] >> 8;
                const size_t o = (size_t)tok * N + ch;
                if constexpr (OUT == OUT_INT32) {
                    int32_t *dst = reinterpret_cast<int32_t *>(out) + o;
                    if (vec_ok) {
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
                        const int che = (ch + e < N) ? ch + e : N - 1;
                        const float lhs = (float)(c[e] * 2 + t_add + b_add[che]);
                        const float rhs = __fmul_rn(t_half_mul, to_f32<OUT>(b_mul[che]));
                        h[e] = from_f32<OUT>(__fmul_rn(lhs, rhs));
                    }
                    uint16_t *dst = reinterpret_cast<uint16_t *>(out) + o;
                    if (vec_ok) {
                        *reinterpret_cast<uint2 *>(dst) = make_uint2(h[0] | (h[1] << 16), h[2] | (h[3] << 16));
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            if (ch + e < N) dst[e] = (uint16_t)h[e];
                    }
                }
            }
        }
    }
}

template <int OUT>
static int launch_out(void *out, const uint8_t *a, const uint8_t *b, const int32_t *a_add, const int32_t *b_add,
                      const void *a_mul, const void *b_mul, int M, int K, int N, hipStream_t st) {
    const int tiles_t = (M + kTileRows - 1) / kTileRows;
    const int tiles_c = (N + kTileRows - 1) / kTileRows;
    gemm_w4a4_staged_kernel<OUT><<<dim3(tiles_t * tiles_c), dim3(256), 0, st>>>(
        out, a, b, a_add, b_add, (const uint16_t *)a_mul, (const uint16_t *)b_mul, M, N, K, tiles_t);
    return launch_status();
}

int launch_gemm_staged(int out_kind, void *out, const uint8_t *a, const uint8_t *b, const int32_t *a_add,
                       const int32_t *b_add, const void *a_mul, const void *b_mul, int M, int K, int N, hipStream_t st) {
    switch (out_kind) {
        case OUT_BF16: return launch_out<OUT_BF16>(out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, st);
        case OUT_FP16: return launch_out<OUT_FP16>(out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, st);
        default: return launch_out<OUT_INT32>(out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, st);
    }
}

}  // namespace quest
