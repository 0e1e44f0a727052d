// Large-tile persistent packed-INT4 x packed-INT4 GEMM (K % 128 == 0): the prefill path.  Same arithmetic and outputs
// as the other GEMM kernels (gemm-quest/quest/matmul_kernel.cu:8-63 and
// gemm-quest/quest/fused_matmul_dequantize_kernel.cu:4-57 of the reference, with the functor
// gemm-quest/include/symmetric/epilogue/thread/linear_combination_dequant.h:122-185).
//
// A workgroup of four waves owns 256 tokens x up to 256 (or 128) channels; wave w multiplies tokens
// [128 (w >> 1), +128) by the lower or upper half of the tile's channel units (up to 128 x 128 per
// wave: 4 x 4 accumulators in the AGPR half of the 512 registers a lone wave per SIMD has).
// Compared with staging int8 through registers this keeps the LDS pipe (the measured bottleneck of
// that variant) at a third of the traffic: packed bytes go HBM -> LDS directly
// (buffer_load_dwordx4 ... lds, stages of 128 k), a lane reads 16 packed bytes of one row
// and splits them into the int8 vectors of 16 * (even-k nibbles) and 16 * (odd-k nibbles), which
// feed two MFMA k-steps.  The stage pipeline runs on across the workgroup's tiles, and the
// epilogue's stores are left to drain under the next tile's first stages.
#include "gemm_schedule.h"

namespace quest {

namespace big {

constexpr int kRows = kBigTileRows;           // token rows per tile
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
        cursor_next_tile<C::kMaxUnits>(ld);
        if (ld.valid) loader_offsets<C>(l, ld, fresh_lane_id()); else ld.kt = l.nk - 1;
    }
}
template <typename C>
__device__ __forceinline__ void loader_issue(Loader &l, Cursor &ld, uint8_t *lds) {
#pragma unroll
    for (int j = 0; j < C::kLoads; j++) loader_one<C>(l, ld, lds, j);
    loader_end<C>(l, ld);
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

template <typename C, int OUT, int EPI, int NA, int TB>
__device__ __forceinline__ void big_tile(uint8_t *lds, Cursor &ld, Loader &ldr, Pipe &pp, void *__restrict__ out, const int32_t *__restrict__ a_add,
                                         const int32_t *__restrict__ b_add, const uint16_t *__restrict__ a_mul,
                                         const uint16_t *__restrict__ b_mul, int M, int N, int K, int tok0, int ch0,
                                         int unit0, int width, const RopeArgs &rope) {
    constexpr int DT = OUT == OUT_INT32 ? 0 : OUT;
    constexpr bool GLU = EPI == kEpiGlu;
    constexpr bool ROPE = EPI == kEpiRope;
    constexpr bool ADD = EPI == kEpiAdd;
    static_assert(EPI == kEpiPlain || OUT != OUT_INT32, "epilogues on 16-bit outputs only");
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
        // kEpiRope: the angles of this lane's sixteen-byte pieces, fetched one piece ahead in the order of the loops below
        constexpr int kOuter = kTokOuter ? TB : NA, kInner = kTokOuter ? NA : TB;
        float4 cs[2][2];
        RopeLane rl = {0, 0};
        if constexpr (ROPE) rl = rope_lane(rope, tok0 + tok_e + li_e, ch0 + unit0 * 32);
        auto fetch_angles = [&](int piece, int par) {
            const int o = piece / (2 * kInner), i = (piece >> 1) % kInner;
            rope_fetch(rope, rl, lg_e, kTokOuter ? i : o, kTokOuter ? o : i, piece & 1, cs[par]);
        };
        if constexpr (ROPE) fetch_angles(0, 0);
        // kEpiAdd: what the output holds under this lane's sixteen-byte pieces, fetched one piece ahead as well
        uint4 res[2];
        auto fetch_res = [&](int piece, int par) {
            const int o = piece / (2 * kInner), i = (piece >> 1) % kInner, pr = piece & 1;
            const int a = kTokOuter ? i : o, b = kTokOuter ? o : i;
            const bool ok = !kGuard || (tok0 + tok_e + b * 32 + li_e < M && ch0 + (unit0 + a) * 32 + (2 * pr + lg_e) * 8 < N);
            res[par] = make_uint4(0, 0, 0, 0);
            if (ok) res[par] = *reinterpret_cast<const uint4 *>(out_lane + ((size_t)b * 32 * n_out + a * kOutPerUnit) * kEs + (2 * pr + lg_e) * 16);
        };
        if constexpr (ADD) fetch_res(0, 0);
#pragma unroll
        for (int o = 0; o < kOuter; o++) {
#pragma unroll
          for (int i = 0; i < kInner; i++) {
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
                        if constexpr (ROPE || ADD) {
                            constexpr int kPieces = 2 * kOuter * kInner;
                            const int nxt = (o * kInner + i) * 2 + pr + 1;
                            if constexpr (ROPE) {
                                if (nxt < kPieces) fetch_angles(nxt, (pr + 1) & 1);
                            } else {
                                if (nxt < kPieces) fetch_res(nxt, (pr + 1) & 1);
                            }
                        }
                        if constexpr (GLU) {
                            // The weight rows come interleaved in eights, four gate rows then the four up rows of the same
                            // outputs: after the swap a lane holds exactly such an eight, gates in (s0[0], s1[0]), ups in
                            // (s0[1], s1[1]), and stores dtype(dtype(silu(gate)) * up) for its four outputs.
                            if (!kGuard || (tok_ok && ch0 + cl < N))
                                *reinterpret_cast<uint2 *>(dst + (2 * pr + lg_e) * 8) =
                                    make_uint2(silu_mul_pair<DT>(s0[0], s0[1]), silu_mul_pair<DT>(s1[0], s1[1]));
                        } else if (!kGuard || (tok_ok && ch0 + cl < N)) {
                            uint4 piece = make_uint4(s0[0], s1[0], s0[1], s1[1]);
                            if constexpr (ROPE) {
                                if (ch0 + cl < rope.rot_cols) piece = rope_turn<DT>(piece, cs[pr]);
                            }
                            if constexpr (ADD) {                  // dtype(out + dtype(product)): the residual stream's addition
                                const uint4 r = res[pr];
                                auto add2 = [](uint32_t p, uint32_t q) {
                                    return pack2_rounded_products<DT>(__fadd_rn(lo_f32<DT>(q), lo_f32<DT>(p)), __fadd_rn(hi_f32<DT>(q), hi_f32<DT>(p)));
                                };
                                piece = make_uint4(add2(piece.x, r.x), add2(piece.y, r.y), add2(piece.z, r.z), add2(piece.w, r.w));
                            }
                            *reinterpret_cast<uint4 *>(dst + (2 * pr + lg_e) * 16) = piece;
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
                            uint32_t val = from_f32<DT>(__fmul_rn(lhs, rhs));
                            if constexpr (ADD) {
                                float sum = __fadd_rn(to_f32<DT>(reinterpret_cast<uint16_t *>(out)[o]), to_f32<DT>((uint16_t)val));
                                asm volatile("" : "+v"(sum));
                                val = from_f32<DT>(sum);
                            }
                            reinterpret_cast<uint16_t *>(out)[o] = (uint16_t)val;
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

template <typename C, int OUT, int EPI>
__global__ void __launch_bounds__(256, C::kWgPerCu)
gemm_w4a4_big_kernel(void *__restrict__ out, const uint8_t *__restrict__ act, const uint8_t *__restrict__ wgt,
                     const int32_t *__restrict__ a_add, const int32_t *__restrict__ b_add,
                     const uint16_t *__restrict__ a_mul, const uint16_t *__restrict__ b_mul,
                     int M, int N, int K, Schedule sch, RopeArgs rope) {
    __shared__ __attribute__((aligned(1024))) uint8_t lds[C::kLdsB];
    // wave-uniform by construction; readfirstlane tells the compiler so, which keeps everything that is
    // updated under `switch (na)` below (cursors, slot numbers, LDS bases) in scalar registers; the empty
    // asm cuts the value loose from threadIdx, which would otherwise be kept (and spilled) to derive it again
    int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
    asm volatile("" : "+s"(wave));
    const int wc = wave & 1;                     // channel half this wave multiplies
    const int kbytes = K >> 1;

    Cursor cc, ld;
    cursor_begin(sch, cc);
    ld = cc;
    cursor_next_tile<C::kMaxUnits>(cc);
    if (!cc.valid) return;                       // uniform: the whole workgroup has nothing to do
    cursor_next_tile<C::kMaxUnits>(ld);

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
    big_tile<C, OUT, EPI, NA, 4>(lds, ld, ldr, pp, out, a_add, b_add, a_mul, b_mul, M, N, K, cc.tok0, cc.ch0, unit0, cc.width, rope)
        if (cc.width <= 2) {
            // a tile of one or two channel units (small problems, the ends of runs): every wave takes a quarter of the
            // tokens and all of the units, instead of two of the four waves idling or holding half-empty accumulators
            if (cc.width == 2)
                big_tile<C, OUT, EPI, 2, 2>(lds, ld, ldr, pp, out, a_add, b_add, a_mul, b_mul, M, N, K, cc.tok0, cc.ch0, 0, 2, rope);
            else
                big_tile<C, OUT, EPI, 1, 2>(lds, ld, ldr, pp, out, a_add, b_add, a_mul, b_mul, M, N, K, cc.tok0, cc.ch0, 0, 1, rope);
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
        cursor_next_tile<C::kMaxUnits>(cc);
    }
    wait_vmcnt_imm<0>();                         // no direct-to-LDS load may outlive the workgroup's LDS allocation
}

}  // namespace big

template <typename C, int OUT, int EPI>
static int launch_big(void *out, const uint8_t *a, const uint8_t *b, const int32_t *a_add, const int32_t *b_add,
                           const void *a_mul, const void *b_mul, int M, int K, int N, int cus, hipStream_t st, const RopeArgs &rope) {
    long grid = 0;
    const Schedule sch = make_schedule(M, N, C::kMaxUnits, C::kWgPerCu, cus, &grid);
    big::gemm_w4a4_big_kernel<C, OUT, EPI><<<dim3((unsigned)grid), dim3(256), 0, st>>>(
        out, a, b, a_add, b_add, (const uint16_t *)a_mul, (const uint16_t *)b_mul, M, N, K, sch, rope);
    return launch_status();
}

template <int OUT, int EPI>
static int launch_shape(bool duo, void *out, const uint8_t *a, const uint8_t *b, const int32_t *a_add, const int32_t *b_add,
                        const void *a_mul, const void *b_mul, int M, int K, int N, int cus, hipStream_t st, const RopeArgs &rope) {
    if (duo) return launch_big<big::Duo, OUT, EPI>(out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, cus, st, rope);
    return launch_big<big::Wide, OUT, EPI>(out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, cus, st, rope);
}

int launch_gemm_big(int out_kind, int epi, bool duo, void *out, const uint8_t *a, const uint8_t *b, const int32_t *a_add,
                    const int32_t *b_add, const void *a_mul, const void *b_mul, int M, int K, int N, int cus, hipStream_t st,
                    const RopeArgs *rope_args) {
    if ((K & 127) != 0 || cus <= 0 || (epi != kEpiPlain && out_kind == OUT_INT32)) return QUEST_ERR_UNSUPPORTED;
    if (epi == kEpiRope && rope_args == nullptr) return QUEST_ERR_NULL_POINTER;
    const RopeArgs rope = epi == kEpiRope ? *rope_args : RopeArgs{nullptr, 32, 0, 32};
#define QUEST_BIG_EPI(E)                                                                                                            \
    (out_kind == OUT_BF16 ? launch_shape<OUT_BF16, E>(duo, out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, cus, st, rope)            \
                          : launch_shape<OUT_FP16, E>(duo, out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, cus, st, rope))
    if (epi == kEpiGlu) return QUEST_BIG_EPI(kEpiGlu);
    if (epi == kEpiRope) return QUEST_BIG_EPI(kEpiRope);
    if (epi == kEpiAdd) return QUEST_BIG_EPI(kEpiAdd);
    if (epi != kEpiPlain) return QUEST_ERR_UNSUPPORTED;
    if (out_kind == OUT_INT32) return launch_shape<OUT_INT32, kEpiPlain>(duo, out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, cus, st, rope);
    return QUEST_BIG_EPI(kEpiPlain);
#undef QUEST_BIG_EPI
}

}  // namespace quest
