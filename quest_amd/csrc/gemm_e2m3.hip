// W4A4 GEMM on the FP6 (E2M3) matrix-core path of gfx950, operands in "E2M3 tiles".
//
// Both operands of the reference's fused GEMM are dequantised as (q + 1/2) * scale
// (gemm-quest/quest/quantize_kernel.cu:162, gemm-quest/benchmarks/utils.py:667-678), and its epilogue
// (gemm-quest/include/symmetric/epilogue/thread/linear_combination_dequant.h:167-181, utils.py:544) evaluates
//     D[m, n] = dtype( f32(2 C + a_add[m] + b_add[n]) * (0.5f * a_mul[m] * b_mul[n]) ),   a_add = sum_k qa,
//     b_add = sum_k qb + K/2,   C = sum_k qa qb      ==>      2 C + a_add + b_add = 2 * sum_k (qa + 1/2)(qb + 1/2).
// All sixteen values q + 1/2 (+-0.5 ... +-7.5) are exact in FP6 E2M3, every product is a multiple of 1/4 below 57 and
// every partial sum of K <= 65536 of them a multiple of 1/4 below 2^22: exactly representable in fp32, so
// v_mfma_f32_32x32x64_f8f6f4 (twice the INT8 rate) accumulates S = sum_k (qa + 1/2)(qb + 1/2) without any rounding and
// f32(2 C + a_add + b_add) is S + S bit for bit.  The outputs equal those of the INT8 kernels (gemm.hip) and of
// add_mul_vv on the exact int32 matrix; the row-sum vectors are not needed at all.
//
// Operand form.  A matrix of R rows x K codes (K % 64 == 0) is stored as ceil(R / 32) row blocks x K / 64 k-steps of
// one fragment each, row block major; a fragment is the 1536-byte register image of one MFMA operand: lane
// l = 32 g + i (row 32 rb + i, k = 64 ks + 32 g ... + 31) owns 32 codes x 6 bits = 24 bytes, code j at bits
// [6 j, 6 j + 6) -- its first 16 bytes at fragment byte 16 l ("head"), its last 8 at byte 1024 + 8 l ("tail").  Rows past
// R inside the last row block are padding (any bits are finite E2M3 values and no stored result depends on them).  Global memory -> LDS is then a linear copy (direct loads, 1 KiB per wave
// instruction) and LDS -> registers one ds_read_b128 + one ds_read_b64 per fragment at lane-linear addresses: no bank
// conflicts, no swizzle, and nothing for the vector ALU to do in the main loop.
//
// A workgroup of four waves owns 256 tokens x up to 256 channels at a time (persistent grid, schedule shared with
// gemm_big.hip); wave w multiplies tokens [128 (w >> 1), +128) by the lower or upper half of the tile's channel
// units: 4 x 4 accumulators of 32 x 32 in the AGPR half of a lone wave's 512 registers.  Six LDS slots of one
// 64-k step (24 KiB: 8 token and 8 channel fragments) form the pipeline: while step s is multiplied from registers,
// the fragments of step s + 1 are read from LDS and the direct loads of step s + 6 are issued.
#include "gemm_schedule.h"

namespace quest {
namespace e2m3 {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v2i __attribute__((ext_vector_type(2)));

constexpr int kRows = kBigTileRows;              // token rows per tile
constexpr int kMaxUnits = 8;                     // channel units (32 rows) per tile
constexpr int kHeadB = 1024, kTailB = 512, kFragB = kHeadB + kTailB;
constexpr int kFrags = 16;                       // per slot: 8 token row blocks, then 8 channel row blocks
constexpr int kHeadsB = kFrags * kHeadB;         // heads first, tails after them
constexpr int kStageB = kFrags * kFragB;         // 24 KiB
constexpr int kStages = 6;
constexpr int kTokSplit = -1;                    // XCD groups along the tokens: chosen per shape (see make_schedule)
constexpr int kLoads = 6;                        // direct loads per wave per step: four heads, two pairs of tails
constexpr int kVecParB = 2 * kRows * 2;          // a_mul of the tile's tokens and b_mul of its channels, 16-bit
constexpr int kVecOff = kStages * kStageB;
constexpr int kLdsB = kVecOff + 2 * kVecParB;    // 146 KiB of the CU's 160

struct Loader {          // direct-to-LDS loads of one wave: waves 0, 1 bring the token fragments, waves 2, 3 the channel fragments
    __amdgpu_buffer_rsrc_t src, amul, bmul;
    uint32_t off[kLoads];       // this lane's byte offsets for the load cursor's tile at its first k-step
    int pitch;                  // bytes per row block: K / 64 fragments
    int nk, wave;
    int slot;                   // LDS slot the next step goes into
};

__device__ __forceinline__ void loader_offsets(Loader &l, const Cursor &ld, int lane) {
    const int rb0 = ((l.wave < 2 ? ld.tok0 : ld.ch0) >> 5) + (l.wave & 1) * 4;
    // row blocks past the matrix give offsets past the buffer: such loads touch no memory and return zeros.  So do the
    // channel units past the tile's width (the tiles are smaller than 2 GiB): a narrow tile fetches what it multiplies,
    // while every wave still issues the same number of loads per step.
    const int units = l.wave < 2 ? 8 : ld.width;             // row blocks of this side the tile uses
    const int first = (l.wave & 1) * 4;
#pragma unroll
    for (int j = 0; j < 4; j++)
        l.off[j] = first + j < units ? (uint32_t)(rb0 + j) * (uint32_t)l.pitch + lane * 16 : 0x80000000u;
#pragma unroll
    for (int j = 0; j < 2; j++)
        l.off[4 + j] = first + 2 * j + (lane >> 5) < units
                           ? (uint32_t)(rb0 + 2 * j + (lane >> 5)) * (uint32_t)l.pitch + kHeadB + (lane & 31) * 16 : 0x80000000u;
}

// Load j of the cursor's step: the head of fragment 4 wave + j (j < 4), or the tails of fragments 4 wave + 2 (j - 4) and
// the next one, half a wave each.
__device__ __forceinline__ void loader_one(const Loader &l, const Cursor &ld, uint8_t *lds, int j) {
    uint8_t *sb = lds + l.slot * kStageB;
    uint8_t *dst = j < 4 ? sb + (4 * l.wave + j) * kHeadB : sb + kHeadsB + (4 * l.wave + 2 * (j - 4)) * kTailB;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(l.src, (__attribute__((address_space(3))) void *)dst, 16, l.off[j], ld.kt * kFragB, 0, 0);
}
// Advances the cursor (into the next tile when this one is done; when nothing is left the last step is fetched again,
// which keeps the count of outstanding loads uniform).
__device__ __forceinline__ void loader_end(Loader &l, Cursor &ld) {
    l.slot = l.slot + 1 == kStages ? 0 : l.slot + 1;
    if (++ld.kt == l.nk) {
        cursor_next_tile<kMaxUnits>(ld);
        if (ld.valid) loader_offsets(l, ld, fresh_lane_id()); else ld.kt = l.nk - 1;
    }
}
__device__ __forceinline__ void loader_issue(Loader &l, Cursor &ld, uint8_t *lds) {
#pragma unroll
    for (int j = 0; j < kLoads; j++) loader_one(l, ld, lds, j);
    loader_end(l, ld);
}

// at most the loads of steps s + 2 .. s + 5 plus `extra` younger memory operations may still be in flight
__device__ __forceinline__ void wait_stage(int extra) {
    constexpr int kBase = kLoads * (kStages - 2);
    switch (extra) {
        case 34: wait_vmcnt_imm<kBase + 34>(); break;
        case 26: wait_vmcnt_imm<kBase + 26>(); break;
        case 18: wait_vmcnt_imm<kBase + 18>(); break;
        case 10: wait_vmcnt_imm<kBase + 10>(); break;
        case 2: wait_vmcnt_imm<kBase + 2>(); break;
        default: wait_vmcnt_imm<kBase>(); break;
    }
}

struct Pipe {            // state that lives across tiles
    int cur;             // LDS slot of the step whose fragments are (to be) in registers
    int store_extra;     // epilogue stores and scale-vector loads that may still be in flight ...
    int store_syncs;     // ... for this many more step synchronisations
    int vec_par;
};

struct Frags { v8i f[8]; };                // four token fragments, then up to four channel fragments

// An FP6 operand occupies six registers: the head and the tail of a lane's 24 bytes; the upper two stay undefined.
__device__ __forceinline__ v8i read_fragment(const uint8_t *head, const uint8_t *tail) {
    const v4i h = *reinterpret_cast<const v4i *>(head);
    const v2i t = *reinterpret_cast<const v2i *>(tail);
    v8i x = __builtin_shufflevector(h, h, 0, 1, 2, 3, -1, -1, -1, -1);
    x[4] = t[0];
    x[5] = t[1];
    return x;
}

// One 64-k step: 4 NA slots of one MFMA each with the rest of the pipeline spread between them and the order pinned (a
// lone wave per SIMD issues in order, so anything that is not placed between MFMAs stalls the matrix pipe):
//   * `sync` (the next step has landed everywhere) after slot kSyncSlot, the six direct loads and the cursor step
//     (`dma`) over the slots after it;
//   * NEXT: the fragments of the next step are read from LDS (heads, tails) in the slots after the synchronisation.
template <int NA, bool NEXT, typename Sync, typename Dma>
__device__ __forceinline__ void k_step(v16f (&acc)[NA > 0 ? NA : 1][4], const Frags &cur, Frags &nxt, const uint8_t *rd_h,
                                       const uint8_t *rd_t, int unit0, int tok_frag0, Sync &&sync, Dma &&dma) {
    constexpr int S = 4 * NA;                 // slots
    constexpr int F = 4 + NA;                 // fragments to read
    constexpr int kSyncSlot = S > 4 ? 3 : 1;
    constexpr int R0 = kSyncSlot + 1;         // reads go into slots [R0, R1), direct loads into [R0, S)
    constexpr int R1 = S * 3 / 4 > R0 ? S * 3 / 4 : R0 + 1;
    if constexpr (NA == 0) {
        sync();
#pragma unroll
        for (int j = 0; j <= kLoads; j++) dma(j);
        return;
    }
#pragma unroll
    for (int i = 0; i < S; i++) {
        const int a = i / 4, b = i % 4;
        acc[a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(cur.f[4 + a], cur.f[b], acc[a][b],
                                                                    2, 2, 0, 0, 0, 0);
        if (i == kSyncSlot) sync();
        if (i > kSyncSlot) {
#pragma unroll
            for (int j = (i - R0) * (kLoads + 1) / (S - R0); j < (i - R0 + 1) * (kLoads + 1) / (S - R0); j++) dma(j);
        }
        if constexpr (NEXT) {
            if (i >= R0 && i < R1) {
#pragma unroll
                for (int r = (i - R0) * F / (R1 - R0); r < (i - R0 + 1) * F / (R1 - R0); r++) {
                    const int f = r < 4 ? tok_frag0 + r : 8 + unit0 + (r - 4);
                    nxt.f[r] = read_fragment(rd_h + f * kHeadB, rd_t + f * kTailB);
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    }
}

template <int OUT, int EPI, int NA>
__device__ __forceinline__ void tile(uint8_t *lds, Cursor &ld, Loader &ldr, Pipe &pp, void *__restrict__ out, int M, int N, int K,
                                     int tok0, int ch0, int unit0, int width, const RopeArgs &rope) {
    constexpr int DT = OUT;
    constexpr bool GLU = EPI == kEpiGlu;
    constexpr bool ADD = EPI == kEpiAdd;
    constexpr bool ROPE = EPI == kEpiRope;
    constexpr int NAX = NA > 0 ? NA : 1;
    const int wave = ldr.wave;                                      // scalar
    const int nk = K / 64;
    const int tok_frag0 = (wave >> 1) * 4;

    v16f acc[NAX][4];
#pragma unroll
    for (int a = 0; a < NA; a++)
#pragma unroll
        for (int b = 0; b < 4; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[a][b][r] = 0.f;

    // the scale vectors of this tile -> LDS by direct loads: wave w brings a_mul of 64 tokens and b_mul of 64 channels,
    // two 16-bit values per lane (a direct load places lane l's data at 4 l bytes whatever its size); read back after
    // the K loop
    uint8_t *vec = lds + kVecOff + pp.vec_par * kVecParB;
    uint16_t *t_mul = reinterpret_cast<uint16_t *>(vec);
    uint16_t *c_mul = reinterpret_cast<uint16_t *>(vec + kRows * 2);
    {
        const int lane = fresh_lane_id();
        if (lane < 32) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(ldr.amul, (__attribute__((address_space(3))) void *)(t_mul + wave * 64), 4,
                                                     (tok0 + wave * 64 + 2 * lane) * 2, 0, 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(ldr.bmul, (__attribute__((address_space(3))) void *)(c_mul + wave * 64), 4,
                                                     (ch0 + wave * 64 + 2 * lane) * 2, 0, 0, 0);
        }
    }

    // ---- main loop ---------------------------------------------------------------------------------------------------
    auto sync = [&]() {
        if (pp.store_syncs > 0) { wait_stage(pp.store_extra); pp.store_syncs--; } else { wait_stage(0); }
        plain_barrier();
    };
    auto dma = [&](int j) { if (j < kLoads) loader_one(ldr, ld, lds, j); else loader_end(ldr, ld); };
    auto head_base = [&](int slot) { return lds + slot * kStageB + fresh_lane_id() * 16; };
    auto tail_base = [&](int slot) { return lds + slot * kStageB + kHeadsB + fresh_lane_id() * 8; };
    auto next_slot = [](int s) { return s + 1 == kStages ? 0 : s + 1; };
    if constexpr (NA == 0) {
        Frags none;
        for (int kt = 0; kt < nk; kt++) {
            k_step<0, false>(acc, none, none, nullptr, nullptr, 0, 0, sync, dma);
            pp.cur = next_slot(pp.cur);
        }
    } else {
        Frags u0, u1;
        {   // the tile's first step (landed: the previous synchronisation saw to it)
            const uint8_t *h = head_base(pp.cur), *t = tail_base(pp.cur);
#pragma unroll
            for (int r = 0; r < 4 + NA; r++) {
                const int f = r < 4 ? tok_frag0 + r : 8 + unit0 + (r - 4);
                u0.f[r] = read_fragment(h + f * kHeadB, t + f * kTailB);
            }
        }
        // K % 128 == 0: an even number of steps, two per iteration (the fragment sets swap roles)
        for (int kt = 0; kt < nk - 2; kt += 2) {
            int nx = next_slot(pp.cur);
            k_step<NA, true>(acc, u0, u1, head_base(nx), tail_base(nx), unit0, tok_frag0, sync, dma);
            pp.cur = nx;
            nx = next_slot(nx);
            k_step<NA, true>(acc, u1, u0, head_base(nx), tail_base(nx), unit0, tok_frag0, sync, dma);
            pp.cur = nx;
        }
        {   // the last two steps: nothing of the next tile is read (its fragments may sit elsewhere in the slot)
            int nx = next_slot(pp.cur);
            k_step<NA, true>(acc, u0, u1, head_base(nx), tail_base(nx), unit0, tok_frag0, sync, dma);
            pp.cur = nx;
            k_step<NA, false>(acc, u1, u0, nullptr, nullptr, unit0, tok_frag0, sync, dma);
            pp.cur = next_slot(nx);
        }
    }

    // ---- epilogue ----------------------------------------------------------------------------------------------------
    // The scale vectors are older than the direct loads of the tile's step 6, so the synchronisation of its step 5 has
    // waited for them in passing; a shorter K loop waits here.
    if (nk < kStages) {
        wait_vmcnt_imm<0>();
        plain_barrier();
    }
    // Accumulator register r of lane (li, lg) is channel 8 (r / 4) + 4 lg + r % 4 of token li.  The two half-waves trade
    // register groups (v_permlane32_swap), so that every lane stores 16 bytes = 8 consecutive channels.
    const bool fast = (N % 8) == 0;
    const bool interior = fast && tok0 + kRows <= M && ch0 + 32 * width <= N;
    const int lane_e = fresh_lane_id();
    const int li_e = lane_e & 31;
    const int lg_e = lane_e >> 5;
    const int tok_e = (wave >> 1) * 128;
    constexpr int kOutPerUnit = GLU ? 16 : 32;
    const int n_out = GLU ? N >> 1 : N;
    if (NA > 0 && fast) {
        float t_half_mul[4];
#pragma unroll
        for (int b = 0; b < 4; b++) t_half_mul[b] = __fmul_rn(0.5f, to_f32<DT>(t_mul[tok_e + b * 32 + li_e]));
        uint8_t *out_lane = reinterpret_cast<uint8_t *>(out) +
                            ((size_t)(tok0 + tok_e + li_e) * n_out + (size_t)((ch0 >> 5) + unit0) * kOutPerUnit) * 2;
        auto convert_and_store = [&](auto guarded_tag) {
            constexpr bool kGuard = decltype(guarded_tag)::value;
            // kEpiAdd: what the output holds under this lane's sixteen-byte pieces, fetched one channel unit ahead of
            // the arithmetic that needs it (eight pieces per unit)
            uint4 res[2][8];
            auto fetch_unit = [&](int a, int par) {
#pragma unroll
                for (int b = 0; b < 4; b++)
#pragma unroll
                    for (int pr = 0; pr < 2; pr++) {
                        const bool ok = !kGuard || (tok0 + tok_e + b * 32 + li_e < M && ch0 + (unit0 + a) * 32 + (2 * pr + lg_e) * 8 < N);
                        res[par][b * 2 + pr] = make_uint4(0, 0, 0, 0);
                        if (ok) res[par][b * 2 + pr] = *reinterpret_cast<const uint4 *>(out_lane + ((size_t)b * 32 * n_out + a * kOutPerUnit) * 2 + (2 * pr + lg_e) * 16);
                    }
            };
            if constexpr (ADD) fetch_unit(0, 0);
            // kEpiRope: the angles of this lane's sixteen-byte pieces, fetched one piece ahead (pieces in the order of the
            // loops below: unit a, token block b, half pr)
            float4 cs[2][2];
            RopeLane rl = {0, 0};
            if constexpr (ROPE) rl = rope_lane(rope, tok0 + tok_e + li_e, ch0 + unit0 * 32);
            auto fetch_angles = [&](int piece, int par) { rope_fetch(rope, rl, lg_e, piece >> 3, (piece >> 1) & 3, piece & 1, cs[par]); };
            if constexpr (ROPE) fetch_angles(0, 0);
#pragma unroll
            for (int a = 0; a < NA; a++) {
                if constexpr (ADD) {
                    if (a + 1 < NA) fetch_unit(a + 1, (a + 1) & 1);
                }
                float muls[16];
#pragma unroll
                for (int rg = 0; rg < 4; rg++) {
                    const uint2 vm = *reinterpret_cast<const uint2 *>(c_mul + (unit0 + a) * 32 + rg * 8 + lg_e * 4);
                    muls[rg * 4 + 0] = lo_f32<DT>(vm.x); muls[rg * 4 + 1] = hi_f32<DT>(vm.x);
                    muls[rg * 4 + 2] = lo_f32<DT>(vm.y); muls[rg * 4 + 3] = hi_f32<DT>(vm.y);
                }
#pragma unroll
                for (int b = 0; b < 4; b++) {
                    const bool tok_ok = tok0 + tok_e + b * 32 + li_e < M;
                    uint8_t *dst = out_lane + ((size_t)b * 32 * n_out + a * kOutPerUnit) * 2;
                    uint32_t x[4][2];
#pragma unroll
                    for (int rg = 0; rg < 4; rg++) {
                        float v[4];
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            const float s = acc[a][b][rg * 4 + e];
                            const float lhs = __fadd_rn(s, s);                       // f32(2 C + a_add + b_add), exactly
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
                        if constexpr (ROPE) {
                            if ((a * 4 + b) * 2 + pr + 1 < 8 * NA) fetch_angles((a * 4 + b) * 2 + pr + 1, (pr + 1) & 1);
                        }
                        if constexpr (GLU) {
                            // weight rows interleaved in eights (four gate rows, the four up rows of the same outputs): a lane
                            // holds such an eight and stores dtype(dtype(silu(gate)) * up) for its four outputs
                            if (!kGuard || (tok_ok && ch0 + cl < N))
                                *reinterpret_cast<uint2 *>(dst + (2 * pr + lg_e) * 8) =
                                    make_uint2(silu_mul_pair<DT>(s0[0], s0[1]), silu_mul_pair<DT>(s1[0], s1[1]));
                        } else if (!kGuard || (tok_ok && ch0 + cl < N)) {
                            uint4 o = make_uint4(s0[0], s1[0], s0[1], s1[1]);
                            if constexpr (ROPE) {
                                if (ch0 + cl < rope.rot_cols) o = rope_turn<DT>(o, cs[pr]);
                            }
                            if constexpr (ADD) {
                                const uint4 r = res[a & 1][b * 2 + pr];
                                auto add2 = [](uint32_t p, uint32_t q) {
                                    return pack2_rounded_products<DT>(__fadd_rn(lo_f32<DT>(q), lo_f32<DT>(p)), __fadd_rn(hi_f32<DT>(q), hi_f32<DT>(p)));
                                };
                                o = make_uint4(add2(o.x, r.x), add2(o.y, r.y), add2(o.z, r.z), add2(o.w, r.w));
                            }
                            *reinterpret_cast<uint4 *>(dst + (2 * pr + lg_e) * 16) = o;
                        }
                    }
                }
            }
        };
        if (interior) convert_and_store(std::false_type{}); else convert_and_store(std::true_type{});
    } else if (NA > 0 && !GLU) {
        // N not a multiple of 8: element-wise stores straight from the accumulators
#pragma unroll
        for (int b = 0; b < 4; b++) {
            const int tok = tok0 + tok_e + b * 32 + li_e;
            if (tok >= M) continue;
            const float t_half_mul = __fmul_rn(0.5f, to_f32<DT>(t_mul[tok_e + b * 32 + li_e]));
#pragma unroll
            for (int a = 0; a < NA; a++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int cl = (unit0 + a) * 32 + (r >> 2) * 8 + lg_e * 4 + (r & 3);
                    if (ch0 + cl >= N) continue;
                    const float s = acc[a][b][r];
                    const float rhs = __fmul_rn(t_half_mul, to_f32<DT>(c_mul[cl]));
                    uint16_t *dst = reinterpret_cast<uint16_t *>(out) + (size_t)tok * N + ch0 + cl;
                    uint32_t o = from_f32<DT>(__fmul_rn(__fadd_rn(s, s), rhs));
                    if constexpr (ADD) {
                        float sum = __fadd_rn(to_f32<DT>(*dst), to_f32<DT>((uint16_t)o));
                        asm volatile("" : "+v"(sum));
                        o = from_f32<DT>(sum);
                    }
                    *dst = (uint16_t)o;
                }
        }
    }
    // how many of this wave's stores the next synchronisations may leave in flight: exact only when every store
    // instruction was issued with all its lanes (an interior tile); the next tile's two vector loads always are
    pp.store_extra = (interior ? 8 * NA : 0) + 2;
    pp.store_syncs = kStages - 1;
    pp.vec_par ^= 1;
}

template <int OUT, int EPI>
__global__ void __launch_bounds__(256, 1)
gemm_e2m3_kernel(void *__restrict__ out, const uint8_t *__restrict__ act, const uint8_t *__restrict__ wgt,
                 const uint16_t *__restrict__ a_mul, const uint16_t *__restrict__ b_mul, int M, int N, int K, Schedule sch,
                 RopeArgs rope) {
    __shared__ __attribute__((aligned(1024))) uint8_t lds[kLdsB];
    int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
    asm volatile("" : "+s"(wave));
    const int wc = wave & 1;                     // channel half this wave multiplies

    Cursor cc, ld;
    cursor_begin(sch, cc);
    ld = cc;
    cursor_next_tile<kMaxUnits>(cc);
    if (!cc.valid) return;                       // uniform: the whole workgroup has nothing to do
    cursor_next_tile<kMaxUnits>(ld);

    Loader ldr;
    const int pitch = (K / 64) * kFragB;
    const __amdgpu_buffer_rsrc_t act_r = __builtin_amdgcn_make_buffer_rsrc((void *)act, 0, ((M + 31) / 32) * pitch, 0x00020000);
    const __amdgpu_buffer_rsrc_t wgt_r = __builtin_amdgcn_make_buffer_rsrc((void *)wgt, 0, ((N + 31) / 32) * pitch, 0x00020000);
    ldr.src = wave < 2 ? act_r : wgt_r;
    // the 16-bit scale vectors travel two per dword: an odd count ends with half a dword, which must still count as in range
    ldr.amul = __builtin_amdgcn_make_buffer_rsrc((void *)a_mul, 0, (M * 2 + 2) & ~3, 0x00020000);
    ldr.bmul = __builtin_amdgcn_make_buffer_rsrc((void *)b_mul, 0, (N * 2 + 2) & ~3, 0x00020000);
    ldr.pitch = pitch;
    ldr.nk = K / 64;
    ldr.wave = wave;
    ldr.slot = 0;
    loader_offsets(ldr, ld, fresh_lane_id());

    // ---- pipeline prologue: steps 0 .. 5 in flight, step 0 landed
#pragma unroll
    for (int s = 0; s < kStages; s++) loader_issue(ldr, ld, lds);
    wait_vmcnt_imm<kLoads * (kStages - 1)>();
    plain_barrier();
    Pipe pp;
    pp.cur = 0;
    pp.store_extra = 2;                          // the first tile's two vector loads
    pp.store_syncs = kStages - 1;
    pp.vec_par = 0;
    while (cc.valid) {
        const int h0 = (cc.width + 1) >> 1;
        const int na = wc == 0 ? h0 : cc.width - h0;
        const int unit0 = wc == 0 ? 0 : h0;
#define QUEST_E2M3_TILE(NA) tile<OUT, EPI, NA>(lds, ld, ldr, pp, out, M, N, K, cc.tok0, cc.ch0, unit0, cc.width, rope)
        switch (na) {
            case 4: QUEST_E2M3_TILE(4); break;
            case 3: QUEST_E2M3_TILE(3); break;
            case 2: QUEST_E2M3_TILE(2); break;
            case 1: QUEST_E2M3_TILE(1); break;
            default: QUEST_E2M3_TILE(0); break;
        }
#undef QUEST_E2M3_TILE
        cursor_next_tile<kMaxUnits>(cc);
    }
    wait_vmcnt_imm<0>();                         // no direct-to-LDS load may outlive the workgroup's LDS allocation
}

// ---- packed INT4 codes -> E2M3 tiles -----------------------------------------------------------------------------------
// E2M3 bits of |q + 1/2| for q = 0 .. 7 (0.5 is subnormal: 0 00 100), one byte each
__device__ constexpr uint64_t kMagBits = 0x1F1D1B1916120C04ull;
__device__ __forceinline__ uint32_t e2m3_of_nibble(uint32_t n) {             // two's-complement nibble -> E2M3 bits of q + 1/2
    const uint32_t neg = (n >> 3) & 1u;
    const uint32_t idx = (n ^ (neg ? 7u : 0u)) & 7u;                          // q >= 0: q;  q < 0: -q - 1
    return ((uint32_t)(kMagBits >> (8 * idx)) & 0x3Fu) | (neg << 5);
}

// One thread per (row, 32 codes): 16 packed bytes in, 24 bytes out; a workgroup of 256 writes four whole fragments
// (k-steps ks0 .. ks0 + 3 of one row block), i.e. reads one 128-byte line of each of its 32 rows.
__global__ void __launch_bounds__(256) int4_to_e2m3_tiles_kernel(uint8_t *__restrict__ tiles, const uint8_t *__restrict__ packed,
                                                                 int rows, int K) {
    const int nks = K / 64;
    const int l = threadIdx.x & 63;
    const int ks = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int rb = blockIdx.y;
    if (ks >= nks) return;
    const int row = rb * 32 + (l & 31);
    uint32_t w[6] = {0, 0, 0, 0, 0, 0};
    if (row < rows) {
        const uint4 p = *reinterpret_cast<const uint4 *>(packed + (size_t)row * (K / 2) + (size_t)ks * 32 + (l >> 5) * 16);
        const uint32_t src[4] = {p.x, p.y, p.z, p.w};
#pragma unroll
        for (int j = 0; j < 32; j++) {
            const uint32_t c = e2m3_of_nibble((src[j >> 3] >> (4 * (j & 7))) & 15u);
            const int bit = 6 * j;
            w[bit >> 5] |= c << (bit & 31);
            if ((bit & 31) > 26) w[(bit >> 5) + 1] |= c >> (32 - (bit & 31));
        }
    }
    uint8_t *frag = tiles + ((size_t)rb * nks + ks) * kFragB;
    *reinterpret_cast<uint4 *>(frag + l * 16) = make_uint4(w[0], w[1], w[2], w[3]);
    *reinterpret_cast<uint2 *>(frag + kHeadB + l * 8) = make_uint2(w[4], w[5]);
}

}  // namespace e2m3

template <int EPI>
static int launch_e2m3(int dtype, void *out, const uint8_t *a, const uint8_t *b, const void *a_mul, const void *b_mul, int M,
                       int K, int N, int cus, hipStream_t st, RopeArgs rope = RopeArgs{nullptr, 1, 0, 2}) {
    long grid = 0;
    const Schedule sch = make_schedule(M, N, e2m3::kMaxUnits, 1, cus, &grid, e2m3::kTokSplit);
    if (dtype == QUEST_DTYPE_BF16)
        e2m3::gemm_e2m3_kernel<OUT_BF16, EPI><<<dim3((unsigned)grid), dim3(256), 0, st>>>(
            out, a, b, (const uint16_t *)a_mul, (const uint16_t *)b_mul, M, N, K, sch, rope);
    else
        e2m3::gemm_e2m3_kernel<OUT_FP16, EPI><<<dim3((unsigned)grid), dim3(256), 0, st>>>(
            out, a, b, (const uint16_t *)a_mul, (const uint16_t *)b_mul, M, N, K, sch, rope);
    return launch_status();
}

static size_t tiles_bytes(int rows, int K) { return (size_t)((rows + 31) / 32) * (size_t)(K / 64) * e2m3::kFragB; }

static int e2m3_gemm_check(const void *out, const void *a, const void *b, const void *a_mul, const void *b_mul, int M, int K,
                           int N, int dtype) {
    if (!out || !a || !b || !a_mul || !b_mul) return QUEST_ERR_NULL_POINTER;
    if (M <= 0 || N <= 0 || K <= 0 || (K & 127)) return QUEST_ERR_BAD_SHAPE;
    if (!check_dtype(dtype)) return QUEST_ERR_BAD_DTYPE;
    // every partial sum must stay an exact fp32 multiple of 1/4: 56.25 K < 2^22
    if (K > 65536) return QUEST_ERR_UNSUPPORTED;
    // 32-bit byte offsets into the tiles, with room for the eight row blocks a tile may reach past the end
    if (tiles_bytes(M + 256, K) >= (1ull << 31) || tiles_bytes(N + 256, K) >= (1ull << 31)) return QUEST_ERR_UNSUPPORTED;
    if (!aligned(a, 16) || !aligned(b, 16) || !aligned(out, 16) || !aligned(a_mul, 4) || !aligned(b_mul, 4)) return QUEST_ERR_ALIGNMENT;
    return QUEST_OK;
}

}  // namespace quest

using namespace quest;

extern "C" size_t quest_e2m3_tiles_bytes(int rows, int size_k) {
    if (rows <= 0 || size_k <= 0 || (size_k & 63)) return 0;
    return tiles_bytes(rows, size_k);
}

extern "C" int quest_int4_to_e2m3_tiles(void *tiles, const uint8_t *x_int_packed, int rows, int size_k, void *stream) {
    forget_stale_error();
    if (!tiles || !x_int_packed) return QUEST_ERR_NULL_POINTER;
    if (rows <= 0 || size_k <= 0 || (size_k & 63)) return QUEST_ERR_BAD_SHAPE;
    if (!aligned(tiles, 16) || !aligned(x_int_packed, 16)) return QUEST_ERR_ALIGNMENT;
    const int nks = size_k / 64, rbs = (rows + 31) / 32;
    if (rbs > 65535) return QUEST_ERR_UNSUPPORTED;
    e2m3::int4_to_e2m3_tiles_kernel<<<dim3((nks + 3) / 4, rbs), dim3(256), 0, (hipStream_t)stream>>>(
        (uint8_t *)tiles, x_int_packed, rows, size_k);
    return launch_status();
}

extern "C" int quest_fused_matmul_dequantize_e2m3(void *mat_d, const void *a_tiles, const void *b_tiles, const void *vec_a_mul,
                                                  const void *vec_b_mul, int size_m, int size_k, int size_n, int dtype,
                                                  void *stream) {
    forget_stale_error();
    const int rc = e2m3_gemm_check(mat_d, a_tiles, b_tiles, vec_a_mul, vec_b_mul, size_m, size_k, size_n, dtype);
    if (rc != QUEST_OK) return rc;
    return launch_e2m3<kEpiPlain>(dtype, mat_d, (const uint8_t *)a_tiles, (const uint8_t *)b_tiles, vec_a_mul, vec_b_mul, size_m,
                              size_k, size_n, device_cu_count((hipStream_t)stream), (hipStream_t)stream);
}

extern "C" int quest_fused_matmul_dequantize_add_e2m3(void *mat_d, const void *a_tiles, const void *b_tiles, const void *vec_a_mul,
                                                      const void *vec_b_mul, int size_m, int size_k, int size_n, int dtype,
                                                      void *stream) {
    forget_stale_error();
    const int rc = e2m3_gemm_check(mat_d, a_tiles, b_tiles, vec_a_mul, vec_b_mul, size_m, size_k, size_n, dtype);
    if (rc != QUEST_OK) return rc;
    return launch_e2m3<kEpiAdd>(dtype, mat_d, (const uint8_t *)a_tiles, (const uint8_t *)b_tiles, vec_a_mul, vec_b_mul, size_m,
                                      size_k, size_n, device_cu_count((hipStream_t)stream), (hipStream_t)stream);
}

extern "C" int quest_fused_matmul_dequantize_rope_e2m3(void *mat_d, const void *a_tiles, const void *b_tiles, const void *vec_a_mul,
                                                       const void *vec_b_mul, int size_m, int size_k, int size_n, int dtype,
                                                       const float *freqs_cis, int seq_len, int rot_cols, int head_dim,
                                                       void *stream) {
    forget_stale_error();
    const int rc = e2m3_gemm_check(mat_d, a_tiles, b_tiles, vec_a_mul, vec_b_mul, size_m, size_k, size_n, dtype);
    if (rc != QUEST_OK) return rc;
    if (!freqs_cis) return QUEST_ERR_NULL_POINTER;
    if (seq_len < 32 || rot_cols <= 0 || head_dim <= 0 || (head_dim & 31) || (rot_cols % head_dim) || rot_cols > size_n || (size_n & 7))
        return QUEST_ERR_BAD_SHAPE;
    if (!aligned(freqs_cis, 16)) return QUEST_ERR_ALIGNMENT;
    return launch_e2m3<kEpiRope>(dtype, mat_d, (const uint8_t *)a_tiles, (const uint8_t *)b_tiles, vec_a_mul, vec_b_mul, size_m,
                                       size_k, size_n, device_cu_count((hipStream_t)stream), (hipStream_t)stream,
                                       RopeArgs{freqs_cis, seq_len, rot_cols, head_dim});
}

extern "C" int quest_e2m3_gemm_plan(int size_m, int size_k, int size_n, int cus, int *plan) {
    if (!plan) return QUEST_ERR_NULL_POINTER;
    if (size_m <= 0 || size_n <= 0 || size_k <= 0 || (size_k & 127) || cus <= 0) return QUEST_ERR_BAD_SHAPE;
    long grid = 0;
    const Schedule sch = make_schedule(size_m, size_n, e2m3::kMaxUnits, 1, cus, &grid, e2m3::kTokSplit);
    const int v[8] = {(int)grid, sch.groups, sch.row_tiles, sch.by_tokens, e2m3::kRows, 32 * e2m3::kMaxUnits, e2m3::kStages, 64};
    for (int i = 0; i < 8; i++) plan[i] = v[i];
    return QUEST_OK;
}

extern "C" int quest_fused_matmul_dequantize_swiglu_e2m3(void *mat_d, const void *a_tiles, const void *b_tiles,
                                                         const void *vec_a_mul, const void *vec_b_mul, int size_m, int size_k,
                                                         int size_n, int dtype, void *stream) {
    forget_stale_error();
    const int rc = e2m3_gemm_check(mat_d, a_tiles, b_tiles, vec_a_mul, vec_b_mul, size_m, size_k, size_n, dtype);
    if (rc != QUEST_OK) return rc;
    if (size_n & 7) return QUEST_ERR_BAD_SHAPE;
    return launch_e2m3<kEpiGlu>(dtype, mat_d, (const uint8_t *)a_tiles, (const uint8_t *)b_tiles, vec_a_mul, vec_b_mul, size_m,
                             size_k, size_n, device_cu_count((hipStream_t)stream), (hipStream_t)stream);
}
