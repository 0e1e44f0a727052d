// Pieces shared by the tiled packed-INT4 GEMM kernels (gemm_big.hip, gemm_small.hip, gemm_staged.hip) and their
// dispatcher (gemm.hip): vector types, the barrier / wait / lane-number primitives of the direct-to-LDS pipelines,
// the nibble splitting, and the launchers each file exports.
#pragma once
#include "common.h"
#include <type_traits>

namespace quest {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kBigTileRows = 256;             // token rows per tile of the large-tile kernel

// s_barrier alone: waves order their own LDS traffic with s_waitcnt, and a release / acquire fence here would
// make the compiler drain every direct-to-LDS load still in flight (vmcnt(0)), which is the pipeline
__device__ __forceinline__ void plain_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// lane number from the execution mask (volatile: never merged with an earlier copy)
__device__ __forceinline__ int fresh_lane_id() {
    int l;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(l));
    return l;
}

template <int N>
__device__ __forceinline__ void wait_vmcnt_imm() {
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));   // vmcnt only
}

// ---- what an epilogue does with the scaled product ------------------------------------------------------------------
// kEpiPlain: store it; kEpiGlu: the gated unit over interleaved weight rows; kEpiAdd: add it to what the output holds (the
// residual stream: dtype(out + dtype(product)), the two roundings of the framework's x + linear(...),
// src/models/llama.py:175-176 of the reference); kEpiRope: the rotary embedding of the reference (llama.py:43-62) on the
// first rot_cols channels of the output -- q and k of a fused QKV projection -- applied to the rounded product before it
// is stored: channels are heads of head_dim, a head is (re, im) pairs, pair i of a head at position t = row % seq_len
// turns by freqs[t][i] = (cos, sin); fp32 products and sums in the reference's order, one more rounding to dtype.  The
// arithmetic of rope_kernel (rowops.hip).
enum { kEpiPlain = 0, kEpiGlu = 1, kEpiAdd = 2, kEpiRope = 3 };

struct RopeArgs {
    const float *freqs;                  // (seq_len, head_dim / 2, 2) fp32, 16-byte aligned
    int seq_len, rot_cols, head_dim;     // seq_len >= 32, head_dim % 32 == 0, rot_cols % head_dim == 0
};

// Where a lane's angles lie: its first token row's position in its sequence (row % seq_len: one division per tile; the
// lane's other rows are 32, 64 and 96 further on) and the place in its head of the first channel of the wave's first
// 32-channel unit (wave-uniform: a unit lies inside one head).
struct RopeLane {
    int t_first, head_at;
};
__device__ __forceinline__ RopeLane rope_lane(const RopeArgs &rope, int row_first, int ch_first) {
    // the divisor through an opaque copy: the reciprocal is then worked out here, once per tile, instead of living in a
    // vector register (or in scratch memory) across the whole tile loop
    int seq_len = rope.seq_len;
    asm volatile("" : "+s"(seq_len));
    RopeLane l;
    l.t_first = row_first % seq_len;
    l.head_at = __builtin_amdgcn_readfirstlane(ch_first % rope.head_dim);
    return l;
}
// (cos, sin) of the four pairs in the lane's sixteen-byte piece: unit a of the wave, token block b, half pr of the unit;
// the lane's half-wave lg holds the piece's channels (2 pr + lg) * 8 ... + 7 of the unit.
__device__ __forceinline__ void rope_fetch(const RopeArgs &rope, const RopeLane &l, int lg, int a, int b, int pr, float4 (&cs)[2]) {
    int h = l.head_at + a * 32;                            // a < 8 and head_dim >= 32: at most 8 wraps, uniform
    while (h >= rope.head_dim) h -= rope.head_dim;
    int t = l.t_first + b * 32;
#pragma unroll
    for (int i = 0; i < 3; i++) t = t >= rope.seq_len ? t - rope.seq_len : t;
    const uint8_t *f = reinterpret_cast<const uint8_t *>(rope.freqs) + ((uint32_t)t * (uint32_t)rope.head_dim * 4u + lg * 32u) +
                       (h * 4 + pr * 64);
    cs[0] = *reinterpret_cast<const float4 *>(f);
    cs[1] = *reinterpret_cast<const float4 *>(f + 16);
}
// the piece (four packed (re, im) pairs of 16-bit values) turned by its angles
template <int DT>
__device__ __forceinline__ uint4 rope_turn(const uint4 &o, const float4 (&cs)[2]) {
    auto turn = [](uint32_t p, float c, float sn) {
        const float re = lo_f32<DT>(p), im = hi_f32<DT>(p);
        float out_re = __fsub_rn(__fmul_rn(re, c), __fmul_rn(im, sn));
        float out_im = __fadd_rn(__fmul_rn(re, sn), __fmul_rn(im, c));
        return pack2_rounded_products<DT>(out_re, out_im);
    };
    return make_uint4(turn(o.x, cs[0].x, cs[0].y), turn(o.y, cs[0].z, cs[0].w), turn(o.z, cs[1].x, cs[1].y), turn(o.w, cs[1].z, cs[1].w));
}

// 16 packed bytes -> the int8 vectors 16 * (even-k nibbles) and 16 * (odd-k nibbles), both sign-correct
__device__ __forceinline__ void split16(const v4i &p, v4i &even, v4i &odd) {
#pragma unroll
    for (int d = 0; d < 4; d++) {
        even[d] = (int)(((uint32_t)p[d] << 4) & 0xF0F0F0F0u);
        odd[d] = (int)((uint32_t)p[d] & 0xF0F0F0F0u);
    }
}

// gemm_big.hip: the large-tile kernel (K % 128 == 0, 4-byte aligned scale vectors); `duo` picks two workgroups of
// 256 x 128 tiles per CU instead of one of 256 x 256, `epi` the epilogue (kEpiPlain, or on 16-bit outputs kEpiGlu or
// kEpiRope with its arguments in `rope`), `cus` the device's CU count (the persistent grid's size)
int launch_gemm_big(int out_kind, int epi, bool duo, void *out, const uint8_t *a, const uint8_t *b, const int32_t *a_add,
                    const int32_t *b_add, const void *a_mul, const void *b_mul, int M, int K, int N, int cus, hipStream_t st,
                    const RopeArgs *rope = nullptr);
// gemm_small.hip: tiles of `shape` x `shape` (64 or 128), K % 256 == 0; `epi` as above
int launch_gemm_small(int out_kind, int epi, int shape, void *out, const uint8_t *a, const uint8_t *b, const int32_t *a_add,
                      const int32_t *b_add, const void *a_mul, const void *b_mul, int M, int K, int N, hipStream_t st,
                      const RopeArgs *rope = nullptr);
// gemm_staged.hip: K % 32 == 0, scale vectors at any element offset
int launch_gemm_staged(int out_kind, void *out, const uint8_t *a, const uint8_t *b, const int32_t *a_add,
                       const int32_t *b_add, const void *a_mul, const void *b_mul, int M, int K, int N, hipStream_t st);

}  // namespace quest
