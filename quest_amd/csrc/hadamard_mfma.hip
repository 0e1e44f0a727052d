// Fused activation kernel for rows of up to 4096 elements: block-128 Hadamard on the matrix
// cores, Gaussian-clip scale, INT4 codes, nibble packing and row sums in one pass over HBM.
//
// This is linear_forward's activation half (gemm-quest/benchmarks/utils.py:89-100 of the
// reference) and it computes the Hadamard the way the reference states it: a product with the
// 128 x 128 matrix whose entries are +-181/2048 in the activation dtype, fp32 accumulation, one
// rounding of the result to the dtype (utils.py:17, 89-90).
//
// One wave owns one row.  The row (up to 32 blocks of 128) goes HBM -> LDS by direct loads
// (no registers), 16 bytes per lane, fully coalesced; the wave's 8 KiB LDS strip is private, so
// there is no workgroup barrier anywhere.  Block n is column n of the MFMA "B" operand and the
// Hadamard matrix is the "A" operand:  D (128 x 32 blocks) = H (128 x 128) * X^T, as 4 row tiles
// x 8 k-steps of v_mfma_f32_32x32x16.  A lane's B fragment for k-step s is the 16-byte chunk
// 2 s + (lane >> 5) of its block, exactly what sits in LDS.  The sign of H for output 32 mt + i
// and input 8 (2 s + g) + j is (-1)^(popcount(i & 7 & j) + i3 g + i4 s0 + mt0 s1 + mt1 s2): the
// first two terms are fixed per lane, the third takes two values, the rest is uniform per
// instruction, so four register quads hold every A fragment the 32 instructions need.
// After the MFMAs lane (n, h) holds outputs 32 mt + 8 q + 4 h + e of block n: the row never
// leaves registers again.  Right after the last LDS read the next row's load is issued into the
// same strip, so it flies while this row is scaled, quantised and stored.
#include "common.h"

namespace quest {
namespace hq {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kWaveLds = 8192;                 // one row of 4096 16-bit elements
constexpr int kWavesPerBlock = 4;

template <int N>
__device__ __forceinline__ void wait_vmcnt_imm() {
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));   // vmcnt only
}
__device__ __forceinline__ void wait_vmcnt_le(int n) {      // n in {0, 1, 2, 3, 4} or those + 16
    switch (n) {
        case 0: wait_vmcnt_imm<0>(); break;
        case 1: wait_vmcnt_imm<1>(); break;
        case 2: wait_vmcnt_imm<2>(); break;
        case 3: wait_vmcnt_imm<3>(); break;
        case 4: wait_vmcnt_imm<4>(); break;
        case 17: wait_vmcnt_imm<17>(); break;
        case 18: wait_vmcnt_imm<18>(); break;
        case 19: wait_vmcnt_imm<19>(); break;
        case 20: wait_vmcnt_imm<20>(); break;
        default: wait_vmcnt_imm<0>(); break;
    }
}

template <int DT>
__device__ __forceinline__ v16f mfma_h(const v4i &a, const v4i &b, const v16f &c) {
    if constexpr (DT == QUEST_DTYPE_BF16)
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
}

template <int DT>
__global__ void __launch_bounds__(256, 3)
hadamard_quantize_mfma_kernel(const uint16_t *__restrict__ x, uint16_t *__restrict__ scale, uint32_t *__restrict__ packed,
                              int32_t *__restrict__ row_sum, uint16_t *__restrict__ x_had, int K, int M,
                              uint32_t entry_bits) {
    __shared__ __attribute__((aligned(1024))) uint8_t lds_all[kWavesPerBlock * kWaveLds];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    uint8_t *lds = lds_all + wave * kWaveLds;
    const int n = lane & 31;                   // block of the row this lane's MFMA column holds
    const int h = lane >> 5;
    const int nb = K >> 7;                     // blocks per row (<= 32)
    const int n_dma = (nb + 3) >> 2;           // 1 KiB direct loads per row
    const bool live = n < nb;

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

    // ---- direct loads: instruction i fills LDS bytes [1024 i, +1024) in lane order; the slot of lane p belongs to
    // block 4 i + p / 16, position p % 16, and holds chunk (p % 16) ^ (block & 15) of that block (conflict-free reads)
    const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc((void *)x, 0, (int)((long)M * K * 2), 0x00020000);
    auto issue_row = [&](int row) {
        const int rb = row * K * 2;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            if (i < n_dma) {
                // block = 4 i + (lane >> 4): block & 15 = ((4 i) & 15) | (lane >> 4) -> chunk = pos ^ (block & 15)
                const int blk_lo = ((4 * i) & 15) | (lane >> 4);
                const int off = (lane >> 4) * 256 + (((lane & 15) ^ blk_lo) * 16);
                __builtin_amdgcn_raw_ptr_buffer_load_lds(xr, (__attribute__((address_space(3))) void *)(lds + i * 1024), 16,
                                                         off, rb + i * 1024, 0, 0);
            }
        }
    };

    const int n_store = (packed ? 2 : 0) + 1 + (row_sum ? 1 : 0) + (x_had ? 16 : 0);
    const int wave_id = blockIdx.x * kWavesPerBlock + wave;
    const int n_waves = gridDim.x * kWavesPerBlock;
    const uint32_t perm_sel = h ? 0x03020706u : 0x05040100u;
    const int partner = (lane ^ 32) * 4;

    int row = wave_id;
    if (row < M) issue_row(row);
    int stores_pending = 0;
    for (; row < M; row += n_waves) {
        wait_vmcnt_le(stores_pending);          // the row has landed; the previous row's stores may still be in flight
        // ---- Hadamard: 8 k-steps x 4 row tiles
        v16f acc[4];
#pragma unroll
        for (int mt = 0; mt < 4; mt++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[mt][r] = 0.f;
        const uint8_t *blk = lds + n * 256;
#pragma unroll
        for (int s = 0; s < 8; s++) {
            const int c = 2 * s + h;
            const v4i b = *reinterpret_cast<const v4i *>(blk + ((c ^ (n & 15)) * 16));
#pragma unroll
            for (int mt = 0; mt < 4; mt++) {
                const int neg = ((mt & 1) & ((s >> 1) & 1)) ^ (((mt >> 1) & 1) & ((s >> 2) & 1));
                acc[mt] = mfma_h<DT>(hv[s & 1][neg], b, acc[mt]);
            }
        }
        // ---- the strip is free again: fetch the next row under the rest of this one
        const int next = row + n_waves;
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (next < M) issue_row(next);
        asm volatile("" ::: "memory");          // this row's stores stay younger than that load (see the wait above)

        // ---- round to the dtype (the transform's output exists only in dtype), sum of squares
        uint32_t yb[4][8];                      // [mt][q * 2 + pair]: outputs 32 mt + 8 q + 4 h + {0,1} / {2,3}
        float sumsq = 0.f;
#pragma unroll
        for (int mt = 0; mt < 4; mt++)
#pragma unroll
            for (int q = 0; q < 4; q++)
#pragma unroll
                for (int p = 0; p < 2; p++) {
                    const uint32_t w = pack2_from_f32<DT>(acc[mt][q * 4 + 2 * p], acc[mt][q * 4 + 2 * p + 1]);
                    yb[mt][q * 2 + p] = w;
                    const float lo = lo_f32<DT>(w), hi = hi_f32<DT>(w);
                    sumsq = __builtin_fmaf(lo, lo, sumsq);
                    sumsq = __builtin_fmaf(hi, hi, sumsq);
                }
        if (!live) sumsq = 0.f;
        const float total = wave_sum_f(sumsq);
        const uint32_t s16 = from_f32<DT>(scale_from_sumsq(total, K));
        const float inv = quant_inv(to_f32<DT>(s16));

        if (x_had != nullptr && live) {
            uint16_t *dst = x_had + (size_t)row * K + n * 128 + 4 * h;
#pragma unroll
            for (int mt = 0; mt < 4; mt++)
#pragma unroll
                for (int q = 0; q < 4; q++)
                    *reinterpret_cast<uint2 *>(dst + 32 * mt + 8 * q) = make_uint2(yb[mt][q * 2], yb[mt][q * 2 + 1]);
        }
        if (lane == 0) scale[row] = (uint16_t)s16;

        if (packed != nullptr || row_sum != nullptr) {
            // ---- codes: half-word Q = 4 mt + q holds outputs 8 Q + 4 h + {0..3} as offset-binary nibbles
            int isum = 0;
            uint32_t hw[16];
#pragma unroll
            for (int mt = 0; mt < 4; mt++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const uint32_t w0 = yb[mt][q * 2], w1 = yb[mt][q * 2 + 1];
                    const int c0 = (int)quant_code_inv(lo_f32<DT>(w0), inv);
                    const int c1 = (int)quant_code_inv(hi_f32<DT>(w0), inv);
                    const int c2 = (int)quant_code_inv(lo_f32<DT>(w1), inv);
                    const int c3 = (int)quant_code_inv(hi_f32<DT>(w1), inv);
                    isum += (c0 + c1) + (c2 + c3);
                    // sum of c_e 16^e is the offset-binary pack minus 0x8888
                    hw[mt * 4 + q] = (uint32_t)((((c3 * 16 + c2) * 16 + c1) * 16 + c0) + 0x8888);
                }
            if (packed != nullptr) {
                // lane (n, 0) ends with dwords 0..7 of the block's 64 packed bytes, lane (n, 1) with dwords 8..15
                uint32_t dw[8];
#pragma unroll
                for (int t = 0; t < 8; t++) {
                    const uint32_t own = (hw[t] & 0xFFFFu) | (hw[t + 8] << 16);
                    const uint32_t other = (uint32_t)__builtin_amdgcn_ds_bpermute(partner, (int)own);
                    dw[t] = __builtin_amdgcn_perm(other, own, perm_sel) ^ 0x88888888u;   // offset-binary -> two's complement
                }
                if (live) {
                    uint32_t *dst = packed + (size_t)row * (K >> 3) + n * 16 + h * 8;
                    *reinterpret_cast<uint4 *>(dst) = make_uint4(dw[0], dw[1], dw[2], dw[3]);
                    *reinterpret_cast<uint4 *>(dst + 4) = make_uint4(dw[4], dw[5], dw[6], dw[7]);
                }
            }
            if (row_sum != nullptr) {
                if (!live) isum = 0;
                const int t = wave_sum_i(isum);
                if (lane == 0) row_sum[row] = t;
            }
        }
        stores_pending = n_store;
    }
    wait_vmcnt_imm<0>();                        // no direct load may outlive the workgroup's LDS allocation
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

// Launches the matrix-core kernel when it applies (K a multiple of 128 up to 4096, a Hadamard entry the
// dtype represents exactly); returns QUEST_ERR_UNSUPPORTED otherwise so that the caller takes the butterfly kernel.
int launch_hadamard_quantize_mfma(const void *x, void *scale, uint8_t *packed, int32_t *row_sum, void *x_had, int K,
                                  int M, float had_scale, int dtype, hipStream_t st) {
    uint32_t bits = 0;
    if (K > 4096 || (K & 127) || had_scale <= 0.f || !representable16(had_scale, dtype, &bits)) return QUEST_ERR_UNSUPPORTED;
    if ((long)M * K * 2 >= (1L << 31)) return QUEST_ERR_UNSUPPORTED;          // 32-bit buffer offsets
    if (!aligned(packed, 16) || !aligned(x_had, 8)) return QUEST_ERR_UNSUPPORTED;
    int blocks = (M + hq::kWavesPerBlock - 1) / hq::kWavesPerBlock;
    const int cap = 3 * 256;                   // three workgroups of four waves per CU
    if (blocks > cap) blocks = cap;
    if (dtype == QUEST_DTYPE_BF16)
        hq::hadamard_quantize_mfma_kernel<0><<<dim3(blocks), dim3(256), 0, st>>>(
            (const uint16_t *)x, (uint16_t *)scale, (uint32_t *)packed, row_sum, (uint16_t *)x_had, K, M, bits);
    else
        hq::hadamard_quantize_mfma_kernel<1><<<dim3(blocks), dim3(256), 0, st>>>(
            (const uint16_t *)x, (uint16_t *)scale, (uint32_t *)packed, row_sum, (uint16_t *)x_had, K, M, bits);
    return launch_status();
}

}  // namespace quest
