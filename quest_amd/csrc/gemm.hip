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
// This file holds the checks, the choice of kernel by shape and the C entry points; all kernels give bit-identical
// results:
//   gemm_decode.hip   gemm_w4a4_decode_kernel   a handful of tokens: the weights are streamed once;
//   gemm_small.hip    gemm_w4a4_small_kernel    K % 256 == 0, a few hundred tokens: 64 x 64 or 128 x 128 tiles, K split
//                                               inside the workgroup;
//   gemm_big.hip      gemm_w4a4_big_kernel      K % 128 == 0: the prefill kernel, persistent 256 x 256 or 256 x 128 tiles;
//   gemm_staged.hip   gemm_w4a4_staged_kernel   K % 32 == 0 (and scale vectors that are not 4-byte aligned): operands
//                                               staged through registers into int8 LDS tiles.
#include "gemm_tiles.h"

#include <mutex>

namespace quest {

static int gemm_check(const void *out, const uint8_t *a, const uint8_t *b, int M, int K, int N) {
    if (!out || !a || !b) return QUEST_ERR_NULL_POINTER;
    if (M <= 0 || N <= 0 || K <= 0 || (K & 31)) return QUEST_ERR_BAD_SHAPE;
    // the accumulators hold 256 C and |C| <= 64 K: K = 131072 with all codes -8 would reach 2^31 exactly
    if (K >= 131072) return QUEST_ERR_UNSUPPORTED;
    if ((size_t)M * (K / 2) >= (1ull << 31) || (size_t)N * (K / 2) >= (1ull << 31)) return QUEST_ERR_UNSUPPORTED;  // 32-bit row offsets
    if (!aligned(a, 16) || !aligned(b, 16) || !aligned(out, 16)) return QUEST_ERR_ALIGNMENT;
    return QUEST_OK;
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

// Wide (256 x 256 tiles, a lone wave per SIMD) has the cheaper main loop; Duo (256 x 128, two workgroups per CU)
// hides epilogues and waits.  Duo wins where there is enough work for full-width tiles on 512 workgroups (256 cells
// of 256 tokens x 32 channels per XCD group) and the epilogue weighs much: K short, or at most 16 channel units
// per group (N <= 4096), which would leave Wide with narrow tiles.  Measured over M in {1024, 4096, 16384}, K in {1024 .. 11008},
// N in {1024 .. 11008} (and again over M from 512): in total run time the rule is within 0.3 % of always picking the
// faster shape, and within 7 % on every single size.
static int gemm_launch_large(int out_kind, bool glu, void *out, const uint8_t *a, const uint8_t *b, const int32_t *a_add,
                             const int32_t *b_add, const void *a_mul, const void *b_mul, int M, int K, int N, int cus,
                             hipStream_t st, const RopeArgs *rope = nullptr, bool add = false) {
    const int small_shape = small_tile_shape(M, K, N, cus);
    const int epi = add ? kEpiAdd : rope != nullptr ? kEpiRope : glu ? kEpiGlu : kEpiPlain;
    if (small_shape != 0 && add) return QUEST_ERR_UNSUPPORTED;           // the small tiles do not add into their output
    if (small_shape != 0) return launch_gemm_small(out_kind, epi, small_shape, out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, st, rope);
    const int units = (N + 31) / 32;
    const int per_group = units >= 8 ? units / 8 : units;
    const long cells_per_group = (long)((M + kBigTileRows - 1) / kBigTileRows) * per_group;
    // small problems (fewer cells per group than Wide has workgroups): twice the workgroups help while K is short
    const bool small = cells_per_group <= 32 && K <= (cells_per_group <= 24 ? 4096 : 2816);
    const bool duo = small || (cells_per_group >= 256 && (K <= 1024 || per_group <= 16));
    return launch_gemm_big(out_kind, epi, duo, out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, cus, st, rope);
}

static int gemm_launch(int out_kind, void *out, const uint8_t *a, const uint8_t *b, const int32_t *a_add, const int32_t *b_add,
                       const void *a_mul, const void *b_mul, int M, int K, int N, hipStream_t st) {
    // the device is asked for its CU count once per call, and only where a rule below uses it (not for a handful of tokens)
    const int cus = M > 64 ? device_cu_count(st) : 0;
    const int small_shape = small_tile_shape(M, K, N, cus);
    if (small_shape != 0) return launch_gemm_small(out_kind, kEpiPlain, small_shape, out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, st);
    // a handful of tokens: the weight-streaming kernel
    // (up to 64 of them unless the small tiles took the call above; where K rules those out, up to 128 while its
    // N / 16 workgroups still run as one round: twice as fast as large tiles that would be half empty)
    if (M <= 64 || (M <= 128 && N <= 8192)) {
        const int rc = launch_gemm_decode(out_kind, out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, st);
        if (rc != QUEST_ERR_UNSUPPORTED) return rc;
    }
    // the large-tile kernel fetches the 16-bit scale vectors two per dword: 4-byte aligned vectors
    if ((K & 127) == 0 && M > 64 && aligned(b_mul, 4) && aligned(a_mul, 4))
        return gemm_launch_large(out_kind, false, out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, cus, st);
    // K % 128 != 0, or scale vectors at odd element offsets (a sliced tensor): the register-staged kernel reads them
    // element by element
    return launch_gemm_staged(out_kind, out, a, b, a_add, b_add, a_mul, b_mul, M, K, N, st);
}

}  // namespace quest

using namespace quest;

extern "C" int quest_matmul_int4_int4t_int32(int32_t *mat_c, const uint8_t *mat_a, const uint8_t *mat_b, int size_m,
                                             int size_k, int size_n, void *stream) {
    forget_stale_error();
    const int rc = gemm_check(mat_c, mat_a, mat_b, size_m, size_k, size_n);
    if (rc != QUEST_OK) return rc;
    return gemm_launch(OUT_INT32, mat_c, mat_a, mat_b, nullptr, nullptr, nullptr, nullptr, size_m, size_k, size_n,
                       (hipStream_t)stream);
}

extern "C" int quest_fused_matmul_dequantize_int4_int4t(void *mat_d, const uint8_t *mat_a, const uint8_t *mat_b,
                                                        const int32_t *vec_a_add, const int32_t *vec_b_add,
                                                        const void *vec_a_mul, const void *vec_b_mul, int size_m,
                                                        int size_k, int size_n, int dtype, void *stream) {
    forget_stale_error();
    const int rc = gemm_check(mat_d, mat_a, mat_b, size_m, size_k, size_n);
    if (rc != QUEST_OK) return rc;
    if (!vec_a_add || !vec_b_add || !vec_a_mul || !vec_b_mul) return QUEST_ERR_NULL_POINTER;
    if (!check_dtype(dtype)) return QUEST_ERR_BAD_DTYPE;
    return gemm_launch(dtype == QUEST_DTYPE_BF16 ? OUT_BF16 : OUT_FP16, mat_d, mat_a, mat_b, vec_a_add, vec_b_add, vec_a_mul,
                       vec_b_mul, size_m, size_k, size_n, (hipStream_t)stream);
}

extern "C" size_t quest_gemm_workspace_bytes(int size_m, int size_k, int size_n) {
    if (size_m <= 0 || size_k <= 0 || size_n <= 0 || size_m > 16 || (size_k & 127) || size_n > 65536) return 0;
    return gemm_decode_workspace_bytes(size_k, size_n);
}

extern "C" int quest_fused_matmul_dequantize_int4_int4t_ws(void *mat_d, const uint8_t *mat_a, const uint8_t *mat_b,
                                                           const int32_t *vec_a_add, const int32_t *vec_b_add,
                                                           const void *vec_a_mul, const void *vec_b_mul, int size_m,
                                                           int size_k, int size_n, int dtype, void *workspace,
                                                           size_t workspace_bytes, void *stream) {
    forget_stale_error();
    const int rc = gemm_check(mat_d, mat_a, mat_b, size_m, size_k, size_n);
    if (rc != QUEST_OK) return rc;
    if (!vec_a_add || !vec_b_add || !vec_a_mul || !vec_b_mul) return QUEST_ERR_NULL_POINTER;
    if (!check_dtype(dtype)) return QUEST_ERR_BAD_DTYPE;
    const int out_kind = dtype == QUEST_DTYPE_BF16 ? OUT_BF16 : OUT_FP16;
    const int split = launch_gemm_decode_splitk(out_kind, mat_d, mat_a, mat_b, vec_a_add, vec_b_add, vec_a_mul, vec_b_mul, size_m,
                                                size_k, size_n, workspace, workspace_bytes, (hipStream_t)stream);
    if (split != QUEST_ERR_UNSUPPORTED) return split;
    return gemm_launch(out_kind, mat_d, mat_a, mat_b, vec_a_add, vec_b_add, vec_a_mul, vec_b_mul, size_m, size_k, size_n,
                       (hipStream_t)stream);
}

// ---- the same GEMM for callers that cannot allocate ------------------------------------------------------------------
// The split-K workspace lives in the library: one array per GPU (every device that loads this code object holds its own
// copy at its own address, zero at load, until the process ends).  In host code the array's name is only a handle for
// hipGetSymbolAddress; kernels and every other use of the memory take the address that call returns.
namespace {
constexpr size_t kScratchBytes = 16384 + (1u << 20);      // counters + 1024 partial tiles: the most any shape that splits uses
constexpr int kScratchDevices = 64;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
void *scratch_of_device[kScratchDevices];
std::mutex scratch_mutex;

int scratch_here(void **out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kScratchDevices) {
        (void)hipGetLastError();
        return QUEST_ERR_LAUNCH;
    }
    std::lock_guard<std::mutex> hold(scratch_mutex);
    if (scratch_of_device[dev] == nullptr) {
        void *p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr) {
            (void)hipGetLastError();
            return QUEST_ERR_LAUNCH;
        }
        scratch_of_device[dev] = p;
    }
    *out = scratch_of_device[dev];
    return QUEST_OK;
}
}  // namespace

extern "C" size_t quest_gemm_noalloc_scratch_bytes(void) { return kScratchBytes; }

extern "C" int quest_fused_matmul_dequantize_int4_int4t_noalloc(void *mat_d, const uint8_t *mat_a, const uint8_t *mat_b,
                                                                const int32_t *vec_a_add, const int32_t *vec_b_add,
                                                                const void *vec_a_mul, const void *vec_b_mul, int size_m,
                                                                int size_k, int size_n, int dtype, void *stream) {
    forget_stale_error();
    const int rc = gemm_check(mat_d, mat_a, mat_b, size_m, size_k, size_n);
    if (rc != QUEST_OK) return rc;
    if (!vec_a_add || !vec_b_add || !vec_a_mul || !vec_b_mul) return QUEST_ERR_NULL_POINTER;
    if (!check_dtype(dtype)) return QUEST_ERR_BAD_DTYPE;
    if (size_m > 16) return QUEST_ERR_UNSUPPORTED;                                        // the decode sizes only
    if (quest_gemm_workspace_bytes(size_m, size_k, size_n) > kScratchBytes) return QUEST_ERR_UNSUPPORTED;
    void *work = nullptr;
    const int got = scratch_here(&work);
    if (got != QUEST_OK) return got;
    const int out_kind = dtype == QUEST_DTYPE_BF16 ? OUT_BF16 : OUT_FP16;
    const int split = launch_gemm_decode_splitk(out_kind, mat_d, mat_a, mat_b, vec_a_add, vec_b_add, vec_a_mul, vec_b_mul, size_m,
                                                size_k, size_n, work, kScratchBytes, (hipStream_t)stream);
    if (split != QUEST_ERR_UNSUPPORTED) return split;
    return gemm_launch(out_kind, mat_d, mat_a, mat_b, vec_a_add, vec_b_add, vec_a_mul, vec_b_mul, size_m, size_k, size_n,
                       (hipStream_t)stream);
}

extern "C" int quest_fused_matmul_dequantize_rope_int4_int4t(void *mat_d, const uint8_t *mat_a, const uint8_t *mat_b,
                                                             const int32_t *vec_a_add, const int32_t *vec_b_add,
                                                             const void *vec_a_mul, const void *vec_b_mul, int size_m,
                                                             int size_k, int size_n, int dtype, const float *freqs_cis,
                                                             int seq_len, int rot_cols, int head_dim, void *stream) {
    forget_stale_error();
    const int rc = gemm_check(mat_d, mat_a, mat_b, size_m, size_k, size_n);
    if (rc != QUEST_OK) return rc;
    if (!vec_a_add || !vec_b_add || !vec_a_mul || !vec_b_mul || !freqs_cis) return QUEST_ERR_NULL_POINTER;
    if (!check_dtype(dtype)) return QUEST_ERR_BAD_DTYPE;
    if (seq_len < 32 || rot_cols <= 0 || head_dim <= 0 || (head_dim & 31) || (rot_cols % head_dim) || rot_cols > size_n || (size_n & 7))
        return QUEST_ERR_BAD_SHAPE;
    if (!aligned(freqs_cis, 16)) return QUEST_ERR_ALIGNMENT;
    // the large-tile and the small-tile kernels have this epilogue (the sizes the plain entry point hands to them)
    if ((size_k & 127) != 0 || size_m <= 64 || (size_m <= 128 && size_n <= 8192) || !aligned(vec_b_mul, 4) || !aligned(vec_a_mul, 4) ||
        !aligned(mat_d, 16))
        return QUEST_ERR_UNSUPPORTED;
    const RopeArgs rope = {freqs_cis, seq_len, rot_cols, head_dim};
    return gemm_launch_large(dtype == QUEST_DTYPE_BF16 ? OUT_BF16 : OUT_FP16, false, mat_d, mat_a, mat_b, vec_a_add, vec_b_add,
                             vec_a_mul, vec_b_mul, size_m, size_k, size_n, device_cu_count((hipStream_t)stream),
                             (hipStream_t)stream, &rope);
}

// Whether quest_fused_matmul_dequantize_add_int4_int4t runs this size in one launch (the large-tile kernel takes it)
static bool add_gemm_applies(int M, int K, int N, int cus) {
    return (K & 127) == 0 && M > 64 && !(M <= 128 && N <= 8192) && small_tile_shape(M, K, N, cus) == 0;
}

extern "C" int quest_fused_matmul_dequantize_add_available(int size_m, int size_k, int size_n, void *stream) {
    forget_stale_error();
    if (size_m <= 0 || size_k <= 0 || size_n <= 0) return 0;
    return add_gemm_applies(size_m, size_k, size_n, device_cu_count((hipStream_t)stream)) ? 1 : 0;
}

extern "C" int quest_fused_matmul_dequantize_add_int4_int4t(void *mat_d, const uint8_t *mat_a, const uint8_t *mat_b,
                                                            const int32_t *vec_a_add, const int32_t *vec_b_add,
                                                            const void *vec_a_mul, const void *vec_b_mul, int size_m,
                                                            int size_k, int size_n, int dtype, void *stream) {
    forget_stale_error();
    const int rc = gemm_check(mat_d, mat_a, mat_b, size_m, size_k, size_n);
    if (rc != QUEST_OK) return rc;
    if (!vec_a_add || !vec_b_add || !vec_a_mul || !vec_b_mul) return QUEST_ERR_NULL_POINTER;
    if (!check_dtype(dtype)) return QUEST_ERR_BAD_DTYPE;
    const int cus = device_cu_count((hipStream_t)stream);
    // only the large-tile kernel has this epilogue
    if (!add_gemm_applies(size_m, size_k, size_n, cus) || !aligned(vec_b_mul, 4) || !aligned(vec_a_mul, 4) || !aligned(mat_d, 16))
        return QUEST_ERR_UNSUPPORTED;
    return gemm_launch_large(dtype == QUEST_DTYPE_BF16 ? OUT_BF16 : OUT_FP16, false, mat_d, mat_a, mat_b, vec_a_add, vec_b_add,
                             vec_a_mul, vec_b_mul, size_m, size_k, size_n, cus, (hipStream_t)stream, nullptr, true);
}

extern "C" int quest_fused_matmul_dequantize_swiglu_int4_int4t(void *mat_d, const uint8_t *mat_a, const uint8_t *mat_b,
                                                               const int32_t *vec_a_add, const int32_t *vec_b_add,
                                                               const void *vec_a_mul, const void *vec_b_mul, int size_m,
                                                               int size_k, int size_n, int dtype, void *stream) {
    forget_stale_error();
    const int rc = gemm_check(mat_d, mat_a, mat_b, size_m, size_k, size_n);
    if (rc != QUEST_OK) return rc;
    if (!vec_a_add || !vec_b_add || !vec_a_mul || !vec_b_mul) return QUEST_ERR_NULL_POINTER;
    if (!check_dtype(dtype)) return QUEST_ERR_BAD_DTYPE;
    if (size_n & 7) return QUEST_ERR_BAD_SHAPE;                      // whole eights of weight rows: four gates, four ups
    // only the large-tile kernel has this epilogue
    if ((size_k & 127) != 0 || size_m <= 64 || !aligned(vec_b_mul, 4) || !aligned(vec_a_mul, 4) ||
        !aligned(mat_d, 8))
        return QUEST_ERR_UNSUPPORTED;
    return gemm_launch_large(dtype == QUEST_DTYPE_BF16 ? OUT_BF16 : OUT_FP16, true, mat_d, mat_a, mat_b, vec_a_add, vec_b_add,
                             vec_a_mul, vec_b_mul, size_m, size_k, size_n, device_cu_count((hipStream_t)stream),
                             (hipStream_t)stream);
}
