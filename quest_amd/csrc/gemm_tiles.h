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

// 16 packed bytes -> the int8 vectors 16 * (even-k nibbles) and 16 * (odd-k nibbles), both sign-correct
__device__ __forceinline__ void split16(const v4i &p, v4i &even, v4i &odd) {
#pragma unroll
    for (int d = 0; d < 4; d++) {
        even[d] = (int)(((uint32_t)p[d] << 4) & 0xF0F0F0F0u);
        odd[d] = (int)((uint32_t)p[d] & 0xF0F0F0F0u);
    }
}

// gemm_big.hip: the large-tile kernel (K % 128 == 0, 4-byte aligned scale vectors); `duo` picks two workgroups of
// 256 x 128 tiles per CU instead of one of 256 x 256, `glu` the SwiGLU epilogue (16-bit outputs only), `cus` the
// device's CU count (the persistent grid's size)
int launch_gemm_big(int out_kind, bool glu, bool duo, void *out, const uint8_t *a, const uint8_t *b, const int32_t *a_add,
                    const int32_t *b_add, const void *a_mul, const void *b_mul, int M, int K, int N, int cus, hipStream_t st);
// gemm_small.hip: tiles of `shape` x `shape` (64 or 128), K % 256 == 0
int launch_gemm_small(int out_kind, bool glu, int shape, void *out, const uint8_t *a, const uint8_t *b, const int32_t *a_add,
                      const int32_t *b_add, const void *a_mul, const void *b_mul, int M, int K, int N, hipStream_t st);
// gemm_staged.hip: K % 32 == 0, scale vectors at any element offset
int launch_gemm_staged(int out_kind, void *out, const uint8_t *a, const uint8_t *b, const int32_t *a_add,
                       const int32_t *b_add, const void *a_mul, const void *b_mul, int M, int K, int N, hipStream_t st);

}  // namespace quest
