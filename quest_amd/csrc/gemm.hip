// Packed-INT4 x packed-INT4 GEMM for gfx950 on the INT8 matrix cores, with the per-token x
// per-output-channel scale epilogue applied in registers.
//
//   C[m, n] = sum_k A[m, k] * B[n, k]          A: (M, K/2) bytes, B: (N, K/2) bytes, two signed
//                                              nibbles per byte, low nibble = even k
//   D[m, n] = dtype( f32(2 C + a_add[m] + b_add[n]) * (0.5f * a_mul[m] * b_mul[n]) )
//
// Replaces the reference's two CUTLASS instantiations (gemm-quest/quest/matmul_kernel.cu:8-63 and
// gemm-quest/quest/fused_matmul_dequantize_kernel.cu:4-57 with the functor
// gemm-quest/include/symmetric/epilogue/thread/linear_combination_dequant.h:122-185).
//
// Kernels in this file, chosen by shape in gemm_launch (the weight-streaming kernel for a handful of tokens is in
// gemm_decode.hip); all give bit-identical results:
//   gemm_w4a4_staged_kernel   K % 32 == 0 (and scale vectors that are not 4-byte aligned): operands staged through
//                             registers into int8 LDS tiles (described next);
//   gemm_w4a4_big_kernel      K % 128 == 0: the prefill kernel, persistent 256 x 256 or 256 x 128 tiles;
//   gemm_w4a4_small_kernel    K % 256 == 0, a few hundred tokens: 64 x 64 or 128 x 128 tiles, K split inside the workgroup.
//
// The staged kernel.  A workgroup of four waves owns a 256-token x 256-channel tile; each wave a 128 x 128
// quarter held as 4 x 4 accumulators of v_mfma_i32_32x32x32_i8.  K advances 128 elements per
// stage.  Packed bytes go HBM -> registers (16 B per lane), are split there into two int8 vectors
// holding 16 * nibble -- `w & 0xF0F0F0F0` is 16 * (odd-k nibbles), `(w << 4) & 0xF0F0F0F0` is
// 16 * (even-k nibbles), both already sign-correct int8 -- and are written to a swizzled,
// double-buffered LDS tile that the MFMA operands are read from with conflict-free 16-byte reads.
// Both operands permute k the same way, so the dot products are unchanged; every product carries
// a factor 256 that the epilogue removes with an exact arithmetic shift (|256 C| <= 2^14 K < 2^31).
// The weight rows feed the MFMA "A" side, so a lane ends up with four consecutive output channels
// of one token and stores them as one 8- or 16-byte vector.
#include "common.h"
#include <type_traits>

namespace quest {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

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

static int gemm_check(const void *out, const uint8_t *a, const uint8_t *b, int M, int K, int N) {
    if (!out || !a || !b) return QUEST_ERR_NULL_POINTER;
    if (M <= 0 || N <= 0 || K <= 0 || (K & 31)) return QUEST_ERR_BAD_SHAPE;
    // the accumulators hold 256 C and |C| <= 64 K: K = 131072 with all codes -8 would reach 2^31 exactly
    if (K >= 131072) return QUEST_ERR_UNSUPPORTED;
    if ((size_t)M * (K / 2) >= (1ull << 31) || (size_t)N * (K / 2) >= (1ull << 31)) return QUEST_ERR_UNSUPPORTED;  // 32-bit row offsets
    if (!aligned(a, 16) || !aligned(b, 16) || !aligned(out, 16)) return QUEST_ERR_ALIGNMENT;
    return QUEST_OK;
}

template <int OUT>
static int gemm_launch_staged(void *out, const uint8_t *a, const uint8_t *b, const int32_t *a_add, const int32_t *b_add,
                       const void *a_mul, const void *b_mul, int M, int K, int N, hipStream_t st) {
    const int tiles_t = (M + kTileRows - 1) / kTileRows;
    const int tiles_c = (N + kTileRows - 1) / kTileRows;
    gemm_w4a4_staged_kernel<OUT><<<dim3(tiles_t * tiles_c), dim3(256), 0, st>>>(
        out, a, b, a_add, b_add, (const uint16_t *)a_mul, (const uint16_t *)b_mul, M, N, K, tiles_t);
    return launch_status();
}


// How a persistent grid divides the (token tile, channel unit) cells among its workgroups.
struct Schedule {
    int tiles_t;        // token tiles of 256
    int units;          // channel units of 32
    int groups;         // channel super-groups (one per XCD when the grid allows)
    int row_tiles;      // > 0: one tile per workgroup, this many per token tile of a group (0: contiguous runs of cells)
    int by_tokens;      // the groups divide the token tiles among them (and each takes all channel units) instead of the units
};


// =================================================================================================
// Large-tile persistent kernel (K % 128 == 0): the prefill path
// =================================================================================================
// A workgroup of four waves owns 256 tokens x up to 256 (or 128) channels; wave w multiplies tokens
// [128 (w >> 1), +128) by the lower or upper half of the tile's channel units (up to 128 x 128 per
// wave: 4 x 4 accumulators in the AGPR half of the 512 registers a lone wave per SIMD has).
// Compared with staging int8 through registers this keeps the LDS pipe (the measured bottleneck of
// that variant) at a third of the traffic: packed bytes go HBM -> LDS directly
// (buffer_load_dwordx4 ... lds, stages of 128 k), a lane reads 16 packed bytes of one row
// and splits them into the int8 vectors of 16 * (even-k nibbles) and 16 * (odd-k nibbles), which
// feed two MFMA k-steps.  The stage pipeline runs on across the workgroup's tiles, and the
// epilogue's stores are left to drain under the next tile's first stages.
namespace big {

constexpr int kRows = 256;                    // token rows per tile
constexpr int kRowB = 64;                     // packed bytes per row per stage (128 k)
constexpr int kTileB = kRows * kRowB;         // 16 KiB: the token rows of a stage; the channel rows follow
constexpr int kVecParB = 2 * (kRows * 4 + kRows * 2);   // b_add, b_mul per channel and a_add, a_mul per token of one tile
constexpr int kVecB = 2 * kVecParB;                       // two tiles in flight

// Two shapes of the same kernel:
//   Wide: 256 x 256 tiles, one workgroup per CU, a wave holds 128 x 128 (256 accumulator registers) and both
//         fragment sets of the software pipeline; nothing else runs on its SIMD, so the epilogue idles the matrix pipe.
//   Duo:  256 x 128 tiles, two workgroups per CU, a wave holds 128 x 64; the two waves of a SIMD belong to different
//         tiles, so one tile's epilogue and synchronisation waits run under the other's multiplications.  Costs 1.5 x
//         the operand traffic and nibble splitting per multiply; wins where the wide shape's tiles would be narrow
//         or few (few channels) and where K is short, i.e. where the epilogue weighs most.
template <int MAXU, int STAGES, int WGS>
struct Cfg {
    static constexpr int kMaxUnits = MAXU;                    // channel units (32 rows) per tile
    static constexpr int kChnRowsPerWave = 8 * MAXU;          // channel rows each wave loads per stage
    static constexpr int kStageB = kTileB + 32 * MAXU * kRowB;
    static constexpr int kStages = STAGES;
    static constexpr int kLoads = 4 + MAXU / 2;               // buffer loads per wave per stage (16 rows each)
    static constexpr int kVecOff = STAGES * kStageB;
    static constexpr int kLdsB = kVecOff + kVecB;             // Wide: 134 KiB, Duo: 78 KiB of the CU's 160 KiB
    static constexpr int kWgPerCu = WGS;
};
using Wide = Cfg<8, 4, 1>;
using Duo = Cfg<4, 3, 2>;

// s_barrier alone: waves order their own LDS traffic with s_waitcnt, and a release / acquire fence here would
// make the compiler drain every direct-to-LDS load still in flight (vmcnt(0)), which is the pipeline
__device__ __forceinline__ void plain_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

struct Cursor {          // walks a workgroup's run of cells tile by tile, stage by stage (no divisions)
    int tt, u;               // next cell: token tile, channel unit inside the group
    int left;                // cells left in the run
    int nug, ug0;
    int tok0, ch0, width;    // current tile
    int kt;                  // next stage of the current tile
    bool valid;
};

template <typename C>
__device__ __forceinline__ void cursor_next_tile(Cursor &c) {
    if (c.left <= 0) { c.valid = false; return; }             // keeps pointing at the last tile
    int width = c.nug - c.u;
    width = width < c.left ? width : c.left;
    // kept in a scalar register: two chained minima would otherwise be selected as the vector ALU's three-operand
    // minimum, which drags the whole cursor into vector registers (and those get spilled at the register peaks)
    asm volatile("" : "+s"(width));
    width = width < C::kMaxUnits ? width : C::kMaxUnits;
    c.tok0 = c.tt * kRows;
    c.ch0 = (c.ug0 + c.u) * 32;
    c.width = width;
    c.kt = 0;
    c.valid = true;
    c.left -= width;
    c.u += width;
    if (c.u == c.nug) { c.u = 0; c.tt++; }
}

// lane number from the execution mask (volatile: never merged with an earlier copy)
__device__ __forceinline__ int fresh_lane_id() {
    int l;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(l));
    return l;
}

struct Loader {          // direct-to-LDS loads of one wave: 4 instructions of 16 token rows, 2 or 4 of 16 channel rows
    __amdgpu_buffer_rsrc_t act, wgt, badd, bmul, aadd, amul;
    uint32_t off_t, off_c;      // byte offset of this lane's first row of the load cursor's tile (+ its 16-byte chunk)
    int kbytes, nk, wave;
    int issued;                 // stages issued so far by this workgroup (slot = issued % kStages)
};

template <typename C>
__device__ __forceinline__ void loader_offsets(Loader &l, const Cursor &ld, int lane) {
    // lane p of an instruction covers row p / 4 of its 16 rows; LDS slot p (lane order) must hold chunk
    // (p & 3) ^ ((row >> 2) & 3) of that row, so the lane fetches exactly that chunk
    const int row = lane >> 2;
    const int chunk = (lane & 3) ^ ((lane >> 4) & 3);
    l.off_t = (uint32_t)(ld.tok0 + l.wave * 64 + row) * (uint32_t)l.kbytes + chunk * 16;
    l.off_c = (uint32_t)(ld.ch0 + l.wave * C::kChnRowsPerWave + row) * (uint32_t)l.kbytes + chunk * 16;
}

// The load cursor's stage goes into the next LDS slot as kLoads instructions per wave (loader_one: four of
// 16 token rows, then those of 16 channel rows), issued a few MFMAs apart because each takes the CU's address path about
// half an MFMA; loader_end then advances the cursor (into the next tile when this one is done; when nothing is
// left the last stage is fetched again, which keeps the count of outstanding loads uniform).
// Rows past the end of a matrix read as zeros.
template <typename C>
__device__ __forceinline__ void loader_one(const Loader &l, const Cursor &ld, uint8_t *lds, int j) {
    uint8_t *sb = lds + (l.issued % C::kStages) * C::kStageB;
    const int kb = ld.kt * kRowB;
    const int step = 16 * l.kbytes;
    if (j < 4)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(l.act, (__attribute__((address_space(3))) void *)(sb + (l.wave * 64 + j * 16) * kRowB), 16,
                                                 l.off_t, kb + j * step, 0, 0);
    else
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            l.wgt, (__attribute__((address_space(3))) void *)(sb + kTileB + (l.wave * C::kChnRowsPerWave + (j - 4) * 16) * kRowB), 16,
            l.off_c, kb + (j - 4) * step, 0, 0);
}
template <typename C>
__device__ __forceinline__ void loader_end(Loader &l, Cursor &ld) {
    l.issued++;
    if (++ld.kt == l.nk) {
        cursor_next_tile<C>(ld);
        if (ld.valid) loader_offsets<C>(l, ld, fresh_lane_id()); else ld.kt = l.nk - 1;
    }
}
template <typename C>
__device__ __forceinline__ void loader_issue(Loader &l, Cursor &ld, uint8_t *lds) {
#pragma unroll
    for (int j = 0; j < C::kLoads; j++) loader_one<C>(l, ld, lds, j);
    loader_end<C>(l, ld);
}

template <int N>
__device__ __forceinline__ void wait_vmcnt_imm() {
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));   // vmcnt only
}
// at most kLoads * (kStages - 3) + extra younger memory operations may still be in flight
template <typename C>
__device__ __forceinline__ void wait_stage(int extra) {
    constexpr int kBase = C::kLoads * (C::kStages - 3);
    switch (extra) {
        case 36: wait_vmcnt_imm<kBase + 36>(); break;
        case 28: wait_vmcnt_imm<kBase + 28>(); break;
        case 20: wait_vmcnt_imm<kBase + 20>(); break;
        case 12: wait_vmcnt_imm<kBase + 12>(); break;
        case 8: wait_vmcnt_imm<kBase + 8>(); break;
        case 4: wait_vmcnt_imm<kBase + 4>(); break;
        default: wait_vmcnt_imm<kBase>(); break;
    }
}

struct Pipe {            // state that lives across tiles
    int it;              // stages multiplied so far (slot = it % kStages)
    int store_extra;     // epilogue stores that may still be in flight ...
    int store_syncs;     // ... for this many more stage synchronisations
    int vec_par;
    unsigned clock;      // two workgroups per CU: the cycle counter sampled at the previous stage synchronisation ...
    int half;            // ... and which half of the grid this workgroup is in (see `sync` in big_tile)
};

__device__ __forceinline__ void split16(const v4i &p, v4i &even, v4i &odd) {
#pragma unroll
    for (int d = 0; d < 4; d++) {
        even[d] = (int)(((uint32_t)p[d] << 4) & 0xF0F0F0F0u);
        odd[d] = (int)((uint32_t)p[d] & 0xF0F0F0F0u);
    }
}

// The int8 operands of one k-pair (two MFMA k-steps): 16 * even-k nibbles and 16 * odd-k nibbles of the four token
// sub-tiles and of up to four channel sub-tiles.
struct Frags {
    v4i te[4], to[4], ce[4], co[4];
};

// One k-pair of the main loop, written as 8 NA slots of one MFMA each with the other work of the pipeline spread
// between them and the order pinned (a lone wave per SIMD issues in order: VALU work, LDS reads and the stage
// synchronisation only overlap the matrix pipe if they sit between MFMAs, which are 32 cycles apart):
//   * the MFMAs of this k-pair, operands in `cur`;
//   * `sync` runs after slot kSyncSlot (-1: none) and the stage's loads, dma(0..kLoads), follow one per few slots;
//   * NEXT: the packed fragments of the next k-pair are read from LDS in the slots after that, up to 3/8 of the
//     way, and split into `nxt` (3 VALU ops per dword) over the second half of the slots.
// TB = token sub-tiles of 32 the wave multiplies (4, or 2 when all four waves split the tokens of a narrow tile).
template <typename C, int NA, int TB, bool NEXT, int kSyncSlot, typename Sync, typename Dma>
__device__ __forceinline__ void k_pair(v16i (&acc)[NA > 0 ? NA : 1][4], const Frags &cur, Frags &nxt, const uint8_t *rd_tok,
                                       const uint8_t *rd_chn, Sync &&sync, Dma &&dma) {
    constexpr int S = 2 * TB * NA;            // slots
    constexpr int F = TB + NA;                // fragments per k-pair
    constexpr int V = F * 4;                  // dwords to split
    constexpr int R0 = kSyncSlot + 1;         // reads go into slots [R0, R1)
    constexpr int R1 = S * 3 / 8 > R0 ? S * 3 / 8 : R0 + 1;
    constexpr int U0 = S / 2 > R1 ? S / 2 : R1;      // splitting goes into slots [U0, S)
    v4i raw[8];
#pragma unroll
    for (int i = 0; i < S; i++) {
        const int a = i / (2 * TB), odd = (i / TB) & 1, b = i % TB;
        acc[a][b] = __builtin_amdgcn_mfma_i32_32x32x32_i8(odd ? cur.co[a] : cur.ce[a], odd ? cur.to[b] : cur.te[b], acc[a][b],
                                                          0, 0, 0);
        if (i == kSyncSlot) sync();
        if constexpr (kSyncSlot >= 0) {
            // the stage's kLoads direct-to-LDS loads and the cursor step (item kLoads), spread over the remaining slots
            if (i > kSyncSlot) {
#pragma unroll
                for (int j = (i - R0) * (C::kLoads + 1) / (S - R0); j < (i - R0 + 1) * (C::kLoads + 1) / (S - R0); j++) dma(j);
            }
        }
        if constexpr (NEXT) {
            if (i >= R0 && i < R1) {
#pragma unroll
                for (int r = (i - R0) * F / (R1 - R0); r < (i - R0 + 1) * F / (R1 - R0); r++)
                    raw[r] = *reinterpret_cast<const v4i *>(r < TB ? rd_tok + r * 32 * kRowB : rd_chn + (r - TB) * 32 * kRowB);
            }
            if (i >= U0) {
#pragma unroll
                for (int v = (i - U0) * V / (S - U0); v < (i - U0 + 1) * V / (S - U0); v++) {
                    const int f = v >> 2, d = v & 3;
                    const uint32_t pk = (uint32_t)raw[f][d];
                    const int ev = (int)((pk << 4) & 0xF0F0F0F0u), od = (int)(pk & 0xF0F0F0F0u);
                    if (f < TB) { nxt.te[f][d] = ev; nxt.to[f][d] = od; } else { nxt.ce[f - TB][d] = ev; nxt.co[f - TB][d] = od; }
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    }
}

template <typename C, int OUT, bool GLU, int NA, int TB>
__device__ __forceinline__ void big_tile(uint8_t *lds, Cursor &ld, Loader &ldr, Pipe &pp, void *__restrict__ out, const int32_t *__restrict__ a_add,
                                         const int32_t *__restrict__ b_add, const uint16_t *__restrict__ a_mul,
                                         const uint16_t *__restrict__ b_mul, int M, int N, int K, int tok0, int ch0,
                                         int unit0, int width) {
    constexpr int DT = OUT == OUT_INT32 ? 0 : OUT;
    constexpr int NAX = NA > 0 ? NA : 1;
    // Lane coordinates are derived afresh in every phase (here, in the loader's cursor step, in the epilogue): a value
    // computed once from threadIdx would be kept alive across the whole kernel, spilled to scratch at the register
    // peaks, and a scratch reload waits on the vector-memory counter, i.e. on every store and load in flight.
    const int lane = fresh_lane_id();
    const int wave = ldr.wave;                                      // scalar
    // the wave's token rows inside the tile: a half of 128 (the other wave of the half takes the other channel units),
    // or, in a tile of one or two channel units, a quarter of 64 with all of the tile's units
    const int tok_in_tile = TB == 4 ? (wave >> 1) * 128 : wave * 64;
    const int li = lane & 31;
    const int lg = lane >> 5;
    const int nk = K / 128;

    // operand reads: row li of a 32-row sub-tile; the 16-byte chunk 2 j + lg of its 64-byte stage row (k-pair j)
    const int rd_t = (tok_in_tile + li) * kRowB;
    const int rd_c = kTileB + (unit0 * 32 + li) * kRowB;
    int rd_j[2];
#pragma unroll
    for (int j = 0; j < 2; j++) rd_j[j] = ((2 * j + lg) ^ ((li >> 2) & 3)) * 16;

    v16i acc[NAX][4];
#pragma unroll
    for (int a = 0; a < NA; a++)
#pragma unroll
        for (int b = 0; b < TB; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[a][b][r] = 0;

    // epilogue vectors of this tile -> LDS, also by direct loads: wave w brings 64 channels of b_add and b_mul
    // and 64 tokens of a_add and a_mul (four loads per wave, counted in pp.store_extra); read back after the K loop
    uint8_t *vec = lds + C::kVecOff + pp.vec_par * kVecParB;
    int32_t *v_add = reinterpret_cast<int32_t *>(vec);
    uint16_t *v_mul = reinterpret_cast<uint16_t *>(vec + kRows * 4);
    int32_t *w_add = reinterpret_cast<int32_t *>(vec + kRows * 6);
    uint16_t *w_mul = reinterpret_cast<uint16_t *>(vec + kRows * 10);
    if constexpr (OUT != OUT_INT32) {
        // a direct load places lane l's data at 4 l bytes whatever its size, so the 16-bit vectors travel as
        // 32 dwords of two elements
        const int c = ch0 + wave * 64;
        const int t = tok0 + wave * 64;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(ldr.badd, (__attribute__((address_space(3))) void *)(v_add + wave * 64), 4,
                                                 (c + lane) * 4, 0, 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(ldr.aadd, (__attribute__((address_space(3))) void *)(w_add + wave * 64), 4,
                                                 (t + lane) * 4, 0, 0, 0);
        if (lane < 32) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(ldr.bmul, (__attribute__((address_space(3))) void *)(v_mul + wave * 64), 4,
                                                     (c + 2 * lane) * 2, 0, 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(ldr.amul, (__attribute__((address_space(3))) void *)(w_mul + wave * 64), 4,
                                                     (t + 2 * lane) * 2, 0, 0, 0);
        }
    }

    // ---- main loop: while one k-pair is multiplied the next is read from LDS and split ------------------------------
    // stage s = pp.it + kt; k-pair j of a stage is the 16-byte chunk 2 j + lg of each 64-byte stage row
    auto tok_base = [&](int slot, int j) { return lds + slot * C::kStageB + rd_j[j] + rd_t; };
    auto chn_base = [&](int slot, int j) { return lds + slot * C::kStageB + rd_j[j] + rd_c; };
    // stage s + 1 must have landed everywhere before its fragments are read; the slot of stage s - 1 is free for
    // the loads of stage s + kStages - 1 once everyone is past this barrier
    auto sync = [&]() {
        if (pp.store_syncs > 0) { wait_stage<C>(pp.store_extra); pp.store_syncs--; } else { wait_stage<C>(0); }
        plain_barrier();
        if constexpr (C::kWgPerCu > 1) {
            // Two persistent workgroups share each SIMD and the issue arbiter prefers the older wave: left alone, the
            // workgroup launched first runs at nearly full speed, finishes a third early and leaves the other to run
            // the rest by itself, without anything to overlap its waits.  Alternating the wave priority between the
            // two halves of the grid in windows of 2^14 cycles (a few stages) keeps them level.
            if ((((pp.clock >> 14) ^ pp.half) & 1) != 0) __builtin_amdgcn_s_setprio(2); else __builtin_amdgcn_s_setprio(0);
            pp.clock = (unsigned)__builtin_amdgcn_s_memtime();       // read one stage later: never waited for
        }
    };
    auto dma = [&](int j) { if (j < C::kLoads) loader_one<C>(ldr, ld, lds, j); else loader_end<C>(ldr, ld); };
    auto no_sync = []() {};
    if constexpr (NA == 0) {
        for (int kt = 0; kt < nk; kt++) { sync(); loader_issue<C>(ldr, ld, lds); pp.it++; }
    } else {
        Frags u0, u1;
        {   // prologue: the first k-pair of the tile's first stage (landed: the previous synchronisation saw to it)
            const int slot = pp.it % C::kStages;
            const uint8_t *t0 = tok_base(slot, 0), *c0 = chn_base(slot, 0);
#pragma unroll
            for (int f = 0; f < TB + NA; f++) {
                const v4i raw = *reinterpret_cast<const v4i *>(f < TB ? t0 + f * 32 * kRowB : c0 + (f - TB) * 32 * kRowB);
                v4i ev, od;
                split16(raw, ev, od);
                if (f < TB) { u0.te[f] = ev; u0.to[f] = od; } else { u0.ce[f - TB] = ev; u0.co[f - TB] = od; }
            }
        }
        for (int kt = 0; kt < nk - 1; kt++) {
            const int slot = pp.it % C::kStages, next = (pp.it + 1) % C::kStages;
            k_pair<C, NA, TB, true, 1>(acc, u0, u1, tok_base(slot, 1), chn_base(slot, 1), sync, dma);
            k_pair<C, NA, TB, true, -1>(acc, u1, u0, tok_base(next, 0), chn_base(next, 0), no_sync, dma);
            pp.it++;
        }
        {   // last stage of the tile: nothing of the next tile is read here (its channel rows sit elsewhere)
            const int slot = pp.it % C::kStages;
            k_pair<C, NA, TB, true, 1>(acc, u0, u1, tok_base(slot, 1), chn_base(slot, 1), sync, dma);
            k_pair<C, NA, TB, false, -1>(acc, u1, u0, nullptr, nullptr, no_sync, dma);
            pp.it++;
        }
    }

    // ---- epilogue -----------------------------------------------------------------------------------
    // Accumulator register r of lane (li, lg) is channel 8 (r/4) + 4 lg + r%4 of token li: a lane owns 4 consecutive
    // channels of each group of 8.  For 16-bit outputs the two half-waves trade register groups (v_permlane32_swap:
    // the lower half keeps group g and receives the upper half's part of it, the upper half does the same with
    // group g + 1), so that every lane stores 16 bytes = 8 consecutive channels and a half-wave pair covers 32
    // contiguous bytes of each token row; the four stores of a sub-tile complete its 64-byte row segments in L2.
    if constexpr (OUT != OUT_INT32) {
        // The tile's scale vectors were sent to LDS at its start; the stage synchronisations wait for them in passing
        // (the counter runs in order and they are older than the tile's own stage loads) -- but only from the
        // (kStages - 1)-th synchronisation on, the earlier ones leave the previous tile's stores and these loads in
        // flight.  A K loop shorter than that (K <= 256, or 128 with three stages) has to wait here.
        if (nk < C::kStages - 1) {
            wait_vmcnt_imm<0>();
            plain_barrier();
        }
    }
    constexpr int kEs = OUT == OUT_INT32 ? 4 : 2;                  // bytes per output element
    const bool fast = (N % (16 / kEs)) == 0;
    const bool interior = fast && tok0 + kRows <= M && ch0 + 32 * width <= N;
    // The lane's coordinates are derived afresh here: values kept alive across the main loop would be spilled to
    // scratch there, and a scratch reload waits on the vector-memory counter, i.e. on every store issued before it.
    const int lane_e = fresh_lane_id();
    const int li_e = lane_e & 31;
    const int lg_e = lane_e >> 5;
    const int tok_e = TB == 4 ? (wave >> 1) * 128 : wave * 64;      // from the scalar wave number: nothing kept alive
    if (NA > 0 && fast) {
        int t_add[4];                                              // of the tokens whose values this lane converts
        float t_half_mul[4];
#pragma unroll
        for (int b = 0; b < TB; b++) {
            t_add[b] = 0;
            t_half_mul[b] = 0.f;
            if constexpr (OUT != OUT_INT32) {
                t_add[b] = w_add[tok_e + b * 32 + li_e];
                t_half_mul[b] = __fmul_rn(0.5f, to_f32<DT>(w_mul[tok_e + b * 32 + li_e]));
            }
        }
        // GLU: the output has N / 2 columns, 16 per channel unit (see the store below)
        constexpr int kOutPerUnit = GLU ? 16 : 32;
        const int n_out = GLU ? N >> 1 : N;
        uint8_t *out_lane = reinterpret_cast<uint8_t *>(out) +
                            ((size_t)(tok0 + tok_e + li_e) * n_out + (size_t)((ch0 >> 5) + unit0) * kOutPerUnit) * kEs;
        // Loop order.  One workgroup per CU: channel unit outside, so that a unit's 32 scale values are read from
        // LDS once.  Two per CU: token sub-tile outside, so that the stores of consecutive iterations complete whole
        // 128-byte lines of the same rows (measured -3..-6 % run time at short K; nothing for the wide shape).
        constexpr bool kTokOuter = C::kWgPerCu > 1;
        // the 16 channel scale values of this lane per unit; in token-outer order all units are unpacked up front (the
        // main loop's fragment registers are free here) instead of once per token sub-tile
        constexpr int kSets = kTokOuter ? NAX : 1;
        int adds_u[kSets][16];
        float muls_u[kSets][16];
        auto load_scales = [&](int a, int (&adds)[16], float (&muls)[16]) {
#pragma unroll
            for (int rg = 0; rg < 4; rg++) {
                const int cl = (unit0 + a) * 32 + rg * 8 + lg_e * 4;      // channel inside the tile
                const int4 va = *reinterpret_cast<const int4 *>(v_add + cl);
                const uint2 vm = *reinterpret_cast<const uint2 *>(v_mul + cl);
                adds[rg * 4 + 0] = va.x; adds[rg * 4 + 1] = va.y; adds[rg * 4 + 2] = va.z; adds[rg * 4 + 3] = va.w;
                muls[rg * 4 + 0] = lo_f32<DT>(vm.x); muls[rg * 4 + 1] = hi_f32<DT>(vm.x);
                muls[rg * 4 + 2] = lo_f32<DT>(vm.y); muls[rg * 4 + 3] = hi_f32<DT>(vm.y);
            }
        };
        if constexpr (OUT != OUT_INT32 && kTokOuter) {
#pragma unroll
            for (int a = 0; a < NA; a++) load_scales(a, adds_u[a], muls_u[a]);
        }
        // interior tiles (the common case) store without the per-lane bounds tests and their exec-mask branches
        auto convert_and_store = [&](auto guarded_tag) {
        constexpr bool kGuard = decltype(guarded_tag)::value;
#pragma unroll
        for (int o = 0; o < (kTokOuter ? TB : NA); o++) {
#pragma unroll
          for (int i = 0; i < (kTokOuter ? NA : TB); i++) {
            const int a = kTokOuter ? i : o, b = kTokOuter ? o : i;
            if constexpr (OUT != OUT_INT32 && !kTokOuter) {
              if (i == 0) load_scales(a, adds_u[0], muls_u[0]);
            }
            const int (&adds)[16] = adds_u[kTokOuter ? a : 0];
            const float (&muls)[16] = muls_u[kTokOuter ? a : 0];
            {
                const bool tok_ok = tok0 + tok_e + b * 32 + li_e < M;
                uint8_t *dst = out_lane + ((size_t)b * 32 * n_out + a * kOutPerUnit) * kEs;
                if constexpr (OUT == OUT_INT32) {
#pragma unroll
                    for (int rg = 0; rg < 4; rg++) {
                        const int cl = (unit0 + a) * 32 + rg * 8 + lg_e * 4;
                        if (!kGuard || (tok_ok && ch0 + cl < N))
                            *reinterpret_cast<int4 *>(dst + (rg * 8 + lg_e * 4) * 4) =
                                make_int4(acc[a][b][rg * 4] >> 8, acc[a][b][rg * 4 + 1] >> 8, acc[a][b][rg * 4 + 2] >> 8,
                                          acc[a][b][rg * 4 + 3] >> 8);
                    }
                } else {
                    uint32_t x[4][2];
#pragma unroll
                    for (int rg = 0; rg < 4; rg++) {
                        float v[4];
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            // the accumulator is 256 C exactly, so 2 C is one arithmetic shift
                            const float lhs = (float)((acc[a][b][rg * 4 + e] >> 7) + t_add[b] + adds[rg * 4 + e]);
                            const float rhs = __fmul_rn(t_half_mul[b], muls[rg * 4 + e]);
                            v[e] = __fmul_rn(lhs, rhs);
                        }
                        x[rg][0] = pack2_rounded_products<DT>(v[0], v[1]);
                        x[rg][1] = pack2_rounded_products<DT>(v[2], v[3]);
                    }
#pragma unroll
                    for (int pr = 0; pr < 2; pr++) {
                        // lower half-wave: group 2 pr complete; upper half-wave: group 2 pr + 1 complete
                        const auto s0 = __builtin_amdgcn_permlane32_swap(x[2 * pr][0], x[2 * pr + 1][0], false, false);
                        const auto s1 = __builtin_amdgcn_permlane32_swap(x[2 * pr][1], x[2 * pr + 1][1], false, false);
                        const int cl = (unit0 + a) * 32 + (2 * pr + lg_e) * 8;
                        if constexpr (GLU) {
                            // The weight rows come interleaved in eights, four gate rows then the four up rows of the same
                            // outputs: after the swap a lane holds exactly such an eight, gates in (s0[0], s1[0]), ups in
                            // (s0[1], s1[1]), and stores dtype(dtype(silu(gate)) * up) for its four outputs.
                            if (!kGuard || (tok_ok && ch0 + cl < N))
                                *reinterpret_cast<uint2 *>(dst + (2 * pr + lg_e) * 8) =
                                    make_uint2(silu_mul_pair<DT>(s0[0], s0[1]), silu_mul_pair<DT>(s1[0], s1[1]));
                        } else if (!kGuard || (tok_ok && ch0 + cl < N)) {
                            *reinterpret_cast<uint4 *>(dst + (2 * pr + lg_e) * 16) = make_uint4(s0[0], s1[0], s0[1], s1[1]);
                        }
                    }
                }
            }
          }
        }
        };
        if (interior) convert_and_store(std::false_type{}); else convert_and_store(std::true_type{});
    } else if (NA > 0 && !GLU) {
        // generic path (N not a multiple of 8 / 4): element-wise stores straight from the accumulators
#pragma unroll
        for (int b = 0; b < TB; b++) {
            const int tok = tok0 + tok_e + b * 32 + li_e;
            if (tok >= M) continue;
            int t_add = 0;
            float t_half_mul = 0.f;
            if constexpr (OUT != OUT_INT32) {
                t_add = w_add[tok_e + b * 32 + li_e];
                t_half_mul = __fmul_rn(0.5f, to_f32<DT>(w_mul[tok_e + b * 32 + li_e]));
            }
#pragma unroll
            for (int a = 0; a < NA; a++) {
#pragma unroll
                for (int rg = 0; rg < 4; rg++) {
                    const int cl = (unit0 + a) * 32 + rg * 8 + lg_e * 4;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const int ch = ch0 + cl + e;
                        if (ch >= N) continue;
                        const int c = acc[a][b][rg * 4 + e] >> 8;
                        const size_t o = (size_t)tok * N + ch;
                        if constexpr (OUT == OUT_INT32) {
                            reinterpret_cast<int32_t *>(out)[o] = c;
                        } else {
                            const float lhs = (float)(c * 2 + t_add + v_add[cl + e]);
                            const float rhs = __fmul_rn(t_half_mul, to_f32<DT>(v_mul[cl + e]));
                            reinterpret_cast<uint16_t *>(out)[o] = (uint16_t)from_f32<DT>(__fmul_rn(lhs, rhs));
                        }
                    }
                }
            }
        }
    }
    // how many of this wave's stores the next stage synchronisations may leave in flight: exact only when every
    // store instruction of the fast path was issued with all its lanes (an interior tile), otherwise none
    // (the next tile's four vector loads, issued right after this point, are always exact)
    if constexpr (OUT != OUT_INT32) {
        pp.store_extra = (interior ? 2 * TB * NA : 0) + 4;
        pp.store_syncs = C::kStages - 2;
    } else {
        pp.store_extra = 0;
        pp.store_syncs = 0;
    }
    pp.vec_par ^= 1;
}

template <typename C, int OUT, bool GLU>
__global__ void __launch_bounds__(256, C::kWgPerCu)
gemm_w4a4_big_kernel(void *__restrict__ out, const uint8_t *__restrict__ act, const uint8_t *__restrict__ wgt,
                     const int32_t *__restrict__ a_add, const int32_t *__restrict__ b_add,
                     const uint16_t *__restrict__ a_mul, const uint16_t *__restrict__ b_mul,
                     int M, int N, int K, Schedule sch) {
    __shared__ __attribute__((aligned(1024))) uint8_t lds[C::kLdsB];
    // wave-uniform by construction; readfirstlane tells the compiler so, which keeps everything that is
    // updated under `switch (na)` below (cursors, slot numbers, LDS bases) in scalar registers; the empty
    // asm cuts the value loose from threadIdx, which would otherwise be kept (and spilled) to derive it again
    int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
    asm volatile("" : "+s"(wave));
    const int wc = wave & 1;                     // channel half this wave multiplies
    const int kbytes = K >> 1;

    const int rank = __builtin_amdgcn_readfirstlane((int)(blockIdx.x / sch.groups));
    const int grp = blockIdx.x - rank * sch.groups;
    const int per_grp = __builtin_amdgcn_readfirstlane((int)(gridDim.x / sch.groups));
    // A group (= an XCD and its L2 when there are eight) owns a slice of the channel units and all token tiles, or --
    // by_tokens -- a slice of the token tiles and all units: whichever operand is the smaller one is then the one every
    // XCD fetches whole (and keeps in its L2), and the larger one is fetched once in total.
    int ug0 = 0, ug1 = sch.units, tt_lo = 0, tt_hi = sch.tiles_t;
    if (sch.by_tokens) {
        tt_lo = __builtin_amdgcn_readfirstlane((int)(((long)grp * sch.tiles_t) / sch.groups));
        tt_hi = __builtin_amdgcn_readfirstlane((int)(((long)(grp + 1) * sch.tiles_t) / sch.groups));
    } else {
        ug0 = __builtin_amdgcn_readfirstlane((int)(((long)grp * sch.units) / sch.groups));
        ug1 = __builtin_amdgcn_readfirstlane((int)(((long)(grp + 1) * sch.units) / sch.groups));
    }
    Cursor cc, ld;
    cc.nug = ug1 - ug0;
    cc.ug0 = ug0;
    // the divisions run on the vector ALU (there is no scalar divide); readfirstlane brings the (uniform) results
    // back to scalar registers, and with them the whole cursor arithmetic of the tile loop
    const long cells = (long)(tt_hi - tt_lo) * cc.nug;
    int pos0, pos1;
    if (sch.row_tiles > 0) {
        // about one tile per workgroup: every token tile's units are cut into row_tiles tiles of equal width (+-1) and
        // workgroup `rank` takes one of them.  An even split of the cells would let runs cross token-tile boundaries,
        // and a workgroup with two tiles (each a full K loop) then takes twice as long as the others.
        const int q = sch.row_tiles;
        const int tile_t = __builtin_amdgcn_readfirstlane(rank / q);
        const int i = rank - tile_t * q;
        pos0 = tile_t * cc.nug + __builtin_amdgcn_readfirstlane((i * cc.nug) / q);
        pos1 = tile_t * cc.nug + __builtin_amdgcn_readfirstlane(((i + 1) * cc.nug) / q);
        if (tile_t >= sch.tiles_t) pos1 = pos0;
    } else {
        pos0 = __builtin_amdgcn_readfirstlane((int)((cells * rank) / per_grp));
        pos1 = __builtin_amdgcn_readfirstlane((int)((cells * (rank + 1)) / per_grp));
    }
    const int tt_rel = __builtin_amdgcn_readfirstlane(pos0 / cc.nug);
    cc.tt = tt_lo + tt_rel;
    cc.u = pos0 - tt_rel * cc.nug;
    cc.left = pos1 - pos0;
    cc.valid = false;
    cc.tok0 = cc.ch0 = cc.width = cc.kt = 0;
    ld = cc;
    cursor_next_tile<C>(cc);
    if (!cc.valid) return;                       // uniform: the whole workgroup has nothing to do
    cursor_next_tile<C>(ld);

    Loader ldr;
    ldr.act = __builtin_amdgcn_make_buffer_rsrc((void *)act, 0, M * kbytes, 0x00020000);
    ldr.wgt = __builtin_amdgcn_make_buffer_rsrc((void *)wgt, 0, N * kbytes, 0x00020000);
    ldr.badd = __builtin_amdgcn_make_buffer_rsrc((void *)b_add, 0, N * 4, 0x00020000);
    // the 16-bit scale vectors travel two per dword: an odd count ends with half a dword, which must still count as in
    // range (the dword lies inside the vector's last aligned word, so nothing outside its memory is touched; the
    // upper half belongs to a row that does not exist and is never used)
    ldr.bmul = __builtin_amdgcn_make_buffer_rsrc((void *)b_mul, 0, (N * 2 + 2) & ~3, 0x00020000);
    ldr.aadd = __builtin_amdgcn_make_buffer_rsrc((void *)a_add, 0, M * 4, 0x00020000);
    ldr.amul = __builtin_amdgcn_make_buffer_rsrc((void *)a_mul, 0, (M * 2 + 2) & ~3, 0x00020000);
    ldr.kbytes = kbytes;
    ldr.nk = K / 128;
    ldr.wave = wave;
    ldr.issued = 0;
    loader_offsets<C>(ldr, ld, fresh_lane_id());

    // ---- pipeline prologue: stages 0 .. kStages - 2 in flight, stage 0 landed
#pragma unroll
    for (int s = 0; s < C::kStages - 1; s++) loader_issue<C>(ldr, ld, lds);
    wait_vmcnt_imm<C::kLoads * (C::kStages - 2)>();
    plain_barrier();
    Pipe pp;
    pp.it = 0;
    pp.store_extra = OUT != OUT_INT32 ? 4 : 0;   // the first tile's four vector loads
    pp.store_syncs = OUT != OUT_INT32 ? C::kStages - 2 : 0;
    pp.vec_par = 0;
    pp.clock = 0;
    pp.half = blockIdx.x >= gridDim.x / 2 ? 1 : 0;
    while (cc.valid) {
        const int h0 = (cc.width + 1) >> 1;
        const int na = wc == 0 ? h0 : cc.width - h0;
        const int unit0 = wc == 0 ? 0 : h0;
#define QUEST_BIG_TILE(NA) \
    big_tile<C, OUT, GLU, NA, 4>(lds, ld, ldr, pp, out, a_add, b_add, a_mul, b_mul, M, N, K, cc.tok0, cc.ch0, unit0, cc.width)
        if (cc.width <= 2) {
            // a tile of one or two channel units (small problems, the ends of runs): every wave takes a quarter of the
            // tokens and all of the units, instead of two of the four waves idling or holding half-empty accumulators
            if (cc.width == 2)
                big_tile<C, OUT, GLU, 2, 2>(lds, ld, ldr, pp, out, a_add, b_add, a_mul, b_mul, M, N, K, cc.tok0, cc.ch0, 0, 2);
            else
                big_tile<C, OUT, GLU, 1, 2>(lds, ld, ldr, pp, out, a_add, b_add, a_mul, b_mul, M, N, K, cc.tok0, cc.ch0, 0, 1);
        } else if constexpr (C::kMaxUnits > 4) {
            switch (na) {
                case 4: QUEST_BIG_TILE(4); break;
                case 3: QUEST_BIG_TILE(3); break;
                case 2: QUEST_BIG_TILE(2); break;
                case 1: QUEST_BIG_TILE(1); break;
                default: QUEST_BIG_TILE(0); break;
            }
        } else {
            switch (na) {
                case 2: QUEST_BIG_TILE(2); break;
                case 1: QUEST_BIG_TILE(1); break;
                default: QUEST_BIG_TILE(0); break;
            }
        }
#undef QUEST_BIG_TILE
        cursor_next_tile<C>(cc);
    }
    wait_vmcnt_imm<0>();                         // no direct-to-LDS load may outlive the workgroup's LDS allocation
}

}  // namespace big

// =================================================================================================
// Small-tile kernel (K % 256 == 0): a few hundred tokens
// =================================================================================================
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

template <typename S, int OUT, bool GLU>
__global__ void __launch_bounds__(512, 2 * S::kWgPerCu)
gemm_w4a4_small_kernel(void *__restrict__ out, const uint8_t *__restrict__ act, const uint8_t *__restrict__ wgt,
                       const int32_t *__restrict__ a_add, const int32_t *__restrict__ b_add,
                       const uint16_t *__restrict__ a_mul, const uint16_t *__restrict__ b_mul,
                       int M, int N, int K, int tiles_t, int tiles_c) {
    __shared__ __attribute__((aligned(1024))) uint8_t lds[S::kLdsB];
    constexpr int DT = OUT == OUT_INT32 ? 0 : OUT;
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
        big::wait_vmcnt_imm<2 * S::kLoads * (kStages - 2)>();    // this wave's share of stage kt has landed ...
        big::plain_barrier();                            // ... and everyone else's; the slot of stage kt - 1 is free
        const int nx = kt + kStages - 1;
        issue(nx < nk ? nx : nk - 1, nx % kStages);
        const uint8_t *sb = lds + (kt % kStages) * S::kStageB;
#pragma unroll
        for (int i = 0; i < S::kPairs; i++) {
            v4i te[kTB], to[kTB], ce[NA], co[NA];
#pragma unroll
            for (int a = 0; a < NA; a++)
                big::split16(*reinterpret_cast<const v4i *>(sb + rd_c + a * 32 * kRowB + rd_x[i]), ce[a], co[a]);
#pragma unroll
            for (int b = 0; b < kTB; b++)
                big::split16(*reinterpret_cast<const v4i *>(sb + rd_t + b * 32 * kRowB + rd_x[i]), te[b], to[b]);
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
    big::wait_vmcnt_imm<0>();                            // no direct-to-LDS load may still be writing ...
    big::plain_barrier();                                // ... and nobody still reading when the stages are reused

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
                    *reinterpret_cast<uint4 *>(dst + c) = make_uint4(s0[0], s1[0], s0[1], s1[1]);
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

// Compute units of the device the stream belongs to.  Asked for at every launch (two host-side queries, no stream
// operation, nothing cached): the library keeps no state and a process may drive several devices.
static int device_cu_count(hipStream_t st) {
    int dev = 0, cus = 0;
    if (hipStreamGetDevice(st, &dev) != hipSuccess && hipGetDevice(&dev) != hipSuccess) return 256;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) return 256;
    return cus;
}

template <typename C, int OUT, bool GLU = false>
static int gemm_launch_big(void *out, const uint8_t *a, const uint8_t *b, const int32_t *a_add, const int32_t *b_add,
                           const void *a_mul, const void *b_mul, int M, int K, int N, hipStream_t st) {
    Schedule sch;
    sch.tiles_t = (M + big::kRows - 1) / big::kRows;
    sch.units = (N + 31) / 32;
    const long cells = (long)sch.tiles_t * sch.units;
    long grid = (long)C::kWgPerCu * device_cu_count(st);      // persistent: one or two workgroups per CU
    if (grid > cells) grid = cells;
    sch.groups = (grid % 8 == 0 && sch.units >= 8) ? 8 : 1;
    sch.row_tiles = 0;
    sch.by_tokens = 0;
    // More tokens than channels: the eight XCD groups divide the token tiles instead of the channel units, so that the
    // weights (the smaller operand) are what every XCD fetches whole and the activation codes cross the fabric once
    // (measured +4..7 % at M = 16384 with N = 1024..5632; no difference at M = 4096, N = 11008 either way).
    if (M > N && grid % 8 == 0 && sch.tiles_t >= 8) {
        sch.groups = 8;
        sch.by_tokens = 1;
    }
    if (!sch.by_tokens) {
        // few cells per workgroup: one tile each, cut along the channel units of single token tiles (see the kernel)
        const long per_grp = grid / sch.groups;
        const int nug = (sch.units + sch.groups - 1) / sch.groups;
        if ((long)sch.tiles_t * nug <= (long)C::kMaxUnits * per_grp) {
            for (int w = 1; w <= C::kMaxUnits; w++) {
                const int q = (nug + w - 1) / w;
                if ((long)sch.tiles_t * q <= per_grp) {
                    sch.row_tiles = q;
                    grid = (long)sch.groups * sch.tiles_t * q;
                    break;
                }
            }
        }
    }
    big::gemm_w4a4_big_kernel<C, OUT, GLU><<<dim3((unsigned)grid), dim3(256), 0, st>>>(
        out, a, b, a_add, b_add, (const uint16_t *)a_mul, (const uint16_t *)b_mul, M, N, K, sch);
    return launch_status();
}

// Which small-tile shape pays, if any (0: none, 64 or 128).
// A few hundred tokens: 64 x 64 tiles, while there are at most four of them per CU (beyond that the large tiles' operand
// reuse wins), or eight where M would leave the last 256-token tile mostly empty; with exactly four per CU the same work
// as one round of 128 x 128 tiles (half the operand bytes per MFMA) is 15-20 % faster.  Measured against the other
// kernels over M from 65 to 4096 with (K, N) from (1024, 3072) to (8192, 8192): 1.2 to 2.6 x faster where this picks
// small tiles.
// Up to 64 tokens the weight-streaming kernel is the faster one while its N / 16 workgroups are one per CU or fewer, or
// it has one or two token tiles; beyond that its time grows with its token tiles: 33 to 64 tokens (four tiles) take one
// small tile of 64 tokens per 64 channels from N > 4096 on (measured at N = 4608 .. 11264, K = 2048 and 4096: 8.3 -> 5.4 us,
// 11.2 -> 7.6 us; at N = 4096 the weight-streaming kernel is 0.6 to 1.2 us faster), 17 to 32 tokens from N > 8192 on (up to
// 2 x faster at N from 8192 to 28672).
static int small_tile_shape(int M, int K, int N, int cus) {
    if ((K & 255) != 0) return 0;
    if (M <= 64) return (M > 32 ? N > 4096 : (M > 16 && N > 8192)) ? 64 : 0;
    const long tiles = (long)((M + 63) / 64) * ((N + 63) / 64);
    const long per_cu = (tiles + cus - 1) / cus;
    if (per_cu <= 3) return 64;
    if (per_cu == 4) return (long)((M + 127) / 128) * ((N + 127) / 128) <= cus ? 128 : 64;
    return (per_cu <= 8 && M < 1024 && (M & 255) != 0) ? 64 : 0;
}

template <typename S, int OUT, bool GLU = false>
static int gemm_launch_small(void *out, const uint8_t *a, const uint8_t *b, const int32_t *a_add, const int32_t *b_add,
                             const void *a_mul, const void *b_mul, int M, int K, int N, hipStream_t st) {
    const int tiles_t = (M + S::kTok - 1) / S::kTok;
    const int tiles_c = (N + S::kChn - 1) / S::kChn;
    const long grid = (long)tiles_t * ((tiles_c + 7) / 8) * 8;
    small::gemm_w4a4_small_kernel<S, OUT, GLU><<<dim3((unsigned)grid), dim3(512), 0, st>>>(
        out, a, b, a_add, b_add, (const uint16_t *)a_mul, (const uint16_t *)b_mul, M, N, K, tiles_t, tiles_c);
    return launch_status();
}

// Wide (256 x 256 tiles, a lone wave per SIMD) has the cheaper main loop; Duo (256 x 128, two workgroups per CU)
// hides epilogues and waits.  Duo wins where there is enough work for full-width tiles on 512 workgroups (256 cells
// of 256 tokens x 32 channels per XCD group) and the epilogue weighs much: K short, or at most 16 channel units
// per group (N <= 4096), which would leave Wide with narrow tiles.  Measured over M in {1024, 4096, 16384}, K in {1024 .. 11008},
// N in {1024 .. 11008} (and again over M from 512): in total run time the rule is within 0.3 % of always picking the
// faster shape, and within 7 % on every single size.
template <int OUT, bool GLU>
static int gemm_launch_large(void *out, const uint8_t *a, const uint8_t *b, const int32_t *a_add, const int32_t *b_add,
                             const void *a_mul, const void *b_mul, int M, int K, int N, hipStream_t st) {
    const int small_shape = small_tile_shape(M, K, N, device_cu_count(st));
    if (small_shape == 64) return gemm_launch_small<small::Tile64, OUT, GLU>(out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, st);
    if (small_shape == 128) return gemm_launch_small<small::Tile128, OUT, GLU>(out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, st);
    const int units = (N + 31) / 32;
    const int per_group = units >= 8 ? units / 8 : units;
    const long cells_per_group = (long)((M + big::kRows - 1) / big::kRows) * per_group;
    // small problems (fewer cells per group than Wide has workgroups): twice the workgroups help while K is short
    const bool small = cells_per_group <= 32 && K <= (cells_per_group <= 24 ? 4096 : 2816);
    const bool duo = small || (cells_per_group >= 256 && (K <= 1024 || per_group <= 16));
    if (!duo) return gemm_launch_big<big::Wide, OUT, GLU>(out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, st);
    return gemm_launch_big<big::Duo, OUT, GLU>(out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, st);
}

template <int OUT>
static int gemm_launch(void *out, const uint8_t *a, const uint8_t *b, const int32_t *a_add, const int32_t *b_add,
                       const void *a_mul, const void *b_mul, int M, int K, int N, hipStream_t st) {
    const int small_shape = small_tile_shape(M, K, N, device_cu_count(st));
    if (small_shape == 64) return gemm_launch_small<small::Tile64, OUT>(out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, st);
    if (small_shape == 128) return gemm_launch_small<small::Tile128, OUT>(out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, st);
    // a handful of tokens: the weight-streaming kernel
    // (up to 64 of them unless the small tiles took the call above; where K rules those out, up to 128 while its
    // N / 16 workgroups still run as one round: twice as fast as large tiles that would be half empty)
    if (M <= 64 || (M <= 128 && N <= 8192)) {
        const int rc = launch_gemm_decode(OUT, out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, st);
        if (rc != QUEST_ERR_UNSUPPORTED) return rc;
    }
    // the large-tile kernel fetches the 16-bit scale vectors two per dword: 4-byte aligned vectors
    if ((K & 127) == 0 && M > 64 && aligned(b_mul, 4) && aligned(a_mul, 4))
        return gemm_launch_large<OUT, false>(out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, st);
    // K % 128 != 0, or scale vectors at odd element offsets (a sliced tensor): the register-staged kernel reads them
    // element by element
    return gemm_launch_staged<OUT>(out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, st);
}

}  // namespace quest

using namespace quest;

extern "C" int quest_matmul_int4_int4t_int32(int32_t *mat_c, const uint8_t *mat_a, const uint8_t *mat_b, int size_m,
                                             int size_k, int size_n, void *stream) {
    const int rc = gemm_check(mat_c, mat_a, mat_b, size_m, size_k, size_n);
    if (rc != QUEST_OK) return rc;
    return gemm_launch<OUT_INT32>(mat_c, mat_a, mat_b, nullptr, nullptr, nullptr, nullptr, size_m, size_k, size_n,
                                  (hipStream_t)stream);
}

extern "C" int quest_fused_matmul_dequantize_int4_int4t(void *mat_d, const uint8_t *mat_a, const uint8_t *mat_b,
                                                        const int32_t *vec_a_add, const int32_t *vec_b_add,
                                                        const void *vec_a_mul, const void *vec_b_mul, int size_m,
                                                        int size_k, int size_n, int dtype, void *stream) {
    const int rc = gemm_check(mat_d, mat_a, mat_b, size_m, size_k, size_n);
    if (rc != QUEST_OK) return rc;
    if (!vec_a_add || !vec_b_add || !vec_a_mul || !vec_b_mul) return QUEST_ERR_NULL_POINTER;
    if (!check_dtype(dtype)) return QUEST_ERR_BAD_DTYPE;
    if (dtype == QUEST_DTYPE_BF16)
        return gemm_launch<OUT_BF16>(mat_d, mat_a, mat_b, vec_a_add, vec_b_add, vec_a_mul, vec_b_mul, size_m, size_k,
                                     size_n, (hipStream_t)stream);
    return gemm_launch<OUT_FP16>(mat_d, mat_a, mat_b, vec_a_add, vec_b_add, vec_a_mul, vec_b_mul, size_m, size_k, size_n,
                                 (hipStream_t)stream);
}

extern "C" int quest_fused_matmul_dequantize_swiglu_int4_int4t(void *mat_d, const uint8_t *mat_a, const uint8_t *mat_b,
                                                               const int32_t *vec_a_add, const int32_t *vec_b_add,
                                                               const void *vec_a_mul, const void *vec_b_mul, int size_m,
                                                               int size_k, int size_n, int dtype, void *stream) {
    const int rc = gemm_check(mat_d, mat_a, mat_b, size_m, size_k, size_n);
    if (rc != QUEST_OK) return rc;
    if (!vec_a_add || !vec_b_add || !vec_a_mul || !vec_b_mul) return QUEST_ERR_NULL_POINTER;
    if (!check_dtype(dtype)) return QUEST_ERR_BAD_DTYPE;
    if (size_n & 7) return QUEST_ERR_BAD_SHAPE;                      // whole eights of weight rows: four gates, four ups
    // only the large-tile kernel has this epilogue
    if ((size_k & 127) != 0 || size_m <= 64 || !aligned(vec_b_mul, 4) || !aligned(vec_a_mul, 4) ||
        !aligned(mat_d, 8))
        return QUEST_ERR_UNSUPPORTED;
    if (dtype == QUEST_DTYPE_BF16)
        return gemm_launch_large<OUT_BF16, true>(mat_d, mat_a, mat_b, vec_a_add, vec_b_add, vec_a_mul, vec_b_mul, size_m,
                                                 size_k, size_n, (hipStream_t)stream);
    return gemm_launch_large<OUT_FP16, true>(mat_d, mat_a, mat_b, vec_a_add, vec_b_add, vec_a_mul, vec_b_mul, size_m, size_k,
                                             size_n, (hipStream_t)stream);
}
