/*
 * libquest_hip -- C ABI of the MI355X (gfx950) kernels behind the `quest` Python package.
 *
 * Every entry point is what the reference's torch extension binds for the same step: it takes
 * raw device pointers, plain sizes and the HIP stream to launch on (passed as void*, i.e. a
 * hipStream_t), borrows every buffer (the caller allocates inputs and outputs), launches
 * asynchronously and never synchronises or allocates, so calls can be recorded into a HIP
 * graph.  A NULL optional output means "do not produce it".  The return value is 0 or one of
 * the negative QUEST_ERR_* codes; nothing is launched when an argument check fails.
 *
 * dtype selects the 16-bit float type of activations, scales and outputs.  The reference
 * instantiates bfloat16 only; float16 is an addition.
 *
 * Citations are file:line under gemm-quest/ of the reference.
 */
#ifndef QUEST_HIP_H
#define QUEST_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define QUEST_DTYPE_BF16 0
#define QUEST_DTYPE_FP16 1

#define QUEST_OK 0
#define QUEST_ERR_NULL_POINTER (-1)  /* a required pointer is NULL */
#define QUEST_ERR_BAD_SHAPE (-2)     /* size <= 0, odd K, K not a multiple of what the kernel needs */
#define QUEST_ERR_BAD_DTYPE (-3)     /* dtype is neither QUEST_DTYPE_BF16 nor QUEST_DTYPE_FP16 */
#define QUEST_ERR_ALIGNMENT (-4)     /* a pointer is not aligned for the vector accesses used */
#define QUEST_ERR_UNSUPPORTED (-5)   /* shape outside what this build instantiates */
#define QUEST_ERR_LAUNCH (-6)        /* hipGetLastError() after the launch was not hipSuccess */

/* ABI version of this header (major * 100 + minor). */
int quest_version(void);

/* Text for a QUEST_ERR_* code (static storage). */
const char *quest_status_string(int status);

/*
 * scale[m] = dtype( sqrt(mean_k x[m,k]^2) * fp32(2.513930578568423 * 2 / 15) + 1e-8f ), fp32 inside.
 * Replaces find_scale_int4_cuda_bf16 (quest/quantize_kernel.cu:97-117; glue quest/quantize.cpp:5-25).
 * x: (batch_size, group_size) dtype, row-major; scale: (batch_size) dtype.  group_size % 8 == 0.
 */
int quest_find_scale_int4(void *scale, const void *x, int group_size, int batch_size, int dtype, void *stream);

/*
 * q = clamp(floor(f32(x) / f32(scale[m])), -8, 7) and, each optional:
 *   x_int[m,k] = q (int8);  x_int_packed[m,j] = (q[2j+1] << 4) | (q[2j] & 0xF);
 *   x_int_row_sum[m] = sum_k q (int32);  if do_dequantize: x[m,k] = dtype(q * s + s * 0.5f) in place.
 * Replaces quantize_int4_cuda_bf16 (quest/quantize_kernel.cu:232-261; glue quest/quantize.cpp:28-70).
 * group_size % 8 == 0.
 */
int quest_quantize_int4(void *x, const void *scale, int8_t *x_int, uint8_t *x_int_packed,
                        int32_t *x_int_row_sum, int group_size, int batch_size, int do_dequantize,
                        int dtype, void *stream);

/*
 * mat_d[a,b] = dtype( f32(2 * mat_c[a,b] + vec_a_add[a] + vec_b_add[b]) * (0.5f * vec_a_mul[a] * vec_b_mul[b]) ).
 * Replaces add_mul_vv_cuda_bf16 (quest/quantize_kernel.cu:309-341; glue quest/quantize.cpp:73-105).
 */
int quest_add_mul_vv(void *mat_d, const int32_t *vec_a_add, const void *vec_a_mul,
                     const int32_t *vec_b_add, const void *vec_b_mul, const int32_t *mat_c,
                     int size_a, int size_b, int dtype, void *stream);

/*
 * mat_c (size_m, size_n) int32 = A * B^T with A (size_m, size_k/2) and B (size_n, size_k/2) packed
 * signed INT4, low nibble = even k.  Replaces matmul_int4_int4t_int32_cuda
 * (quest/matmul_kernel.cu:8-63; glue quest/matmul.cpp:52-66).  size_k % 32 == 0 (the reference's
 * CUTLASS alignment), any size_m >= 1 and size_n >= 1.  Pointers 16-byte aligned.
 */
int quest_matmul_int4_int4t_int32(int32_t *mat_c, const uint8_t *mat_a, const uint8_t *mat_b,
                                  int size_m, int size_k, int size_n, void *stream);

/*
 * mat_d (size_m, size_n) dtype = the same GEMM followed, in registers, by the add_mul_vv formula
 * above with vec_a_* indexed by row and vec_b_* by column (the int32 accumulator is used exactly,
 * where the reference's functor first rounds it to fp16).  Replaces
 * fused_matmul_dequantize_int4_int4t_bf16_cuda (quest/fused_matmul_dequantize_kernel.cu:4-57,
 * include/symmetric/epilogue/thread/linear_combination_dequant.h:122-185; glue
 * quest/fused_matmul_dequantize.cpp:20-42).
 */
int quest_fused_matmul_dequantize_int4_int4t(void *mat_d, const uint8_t *mat_a, const uint8_t *mat_b,
                                             const int32_t *vec_a_add, const int32_t *vec_b_add,
                                             const void *vec_a_mul, const void *vec_b_mul,
                                             int size_m, int size_k, int size_n, int dtype, void *stream);

/*
 * quest_fused_matmul_dequantize_int4_int4t with a caller-owned workspace, which lets a handful of tokens
 * (size_m <= 16: the decode shapes) split K across workgroups: every slice leaves its partial int32 tile in the
 * workspace and the workgroup that arrives last (a counter per channel tile, no atomics on the result) adds them --
 * integers, so the result does not depend on the order -- and applies the epilogue.  Same outputs bit for bit.
 * The reference passes no workspace to its CUTLASS GEMM (quest/matmul_kernel.cu:55: nullptr) and runs no split-K.
 * workspace: quest_gemm_workspace_bytes(size_m, size_k, size_n) bytes (0: this shape does not use one), 256-byte
 * aligned; its first 16 KiB (the counters) must be zero before the first call and are zero again after every call,
 * so one zero-initialised buffer serves any number of calls -- but calls that may overlap in time (different
 * streams) need a workspace each.  Shapes that do not split, or a workspace that is NULL or too small, run exactly as
 * quest_fused_matmul_dequantize_int4_int4t.
 */
size_t quest_gemm_workspace_bytes(int size_m, int size_k, int size_n);
int quest_fused_matmul_dequantize_int4_int4t_ws(void *mat_d, const uint8_t *mat_a, const uint8_t *mat_b,
                                                const int32_t *vec_a_add, const int32_t *vec_b_add,
                                                const void *vec_a_mul, const void *vec_b_mul, int size_m, int size_k,
                                                int size_n, int dtype, void *workspace, size_t workspace_bytes,
                                                void *stream);

/*
 * quest_fused_matmul_dequantize_int4_int4t_ws for callers that cannot allocate a workspace (code under HIP graph
 * capture, serving loops, harnesses that forbid hipMalloc): no counterpart in the reference.  The workspace is an
 * array inside the library, quest_gemm_noalloc_scratch_bytes() bytes (1,064,960) on every GPU the library runs on,
 * held until the process ends; the call allocates and frees nothing.  size_m <= 16 (QUEST_ERR_UNSUPPORTED above, or
 * if a shape ever needed more than the array holds); shapes that do not split K run the plain kernel.  Same outputs
 * bit for bit.  Every call on one GPU shares that GPU's array: calls that may overlap in time on one GPU (different
 * streams, different threads) race -- give those quest_fused_matmul_dequantize_int4_int4t_ws and a workspace each.
 * The first call on a device looks the array up (hipGetSymbolAddress); make it before capturing a graph.
 */
size_t quest_gemm_noalloc_scratch_bytes(void);
int quest_fused_matmul_dequantize_int4_int4t_noalloc(void *mat_d, const uint8_t *mat_a, const uint8_t *mat_b,
                                                     const int32_t *vec_a_add, const int32_t *vec_b_add,
                                                     const void *vec_a_mul, const void *vec_b_mul, int size_m, int size_k,
                                                     int size_n, int dtype, void *stream);

/*
 * y = block-128 Walsh-Hadamard transform of every row of x along K, fp32 butterflies, * had_scale,
 * one rounding to dtype.  had_scale = 181/2048 reproduces F.linear(x.view(-1,128), HADAMARD_MATRIX)
 * (benchmarks/utils.py:17,89-90: the matrix entries are bf16(2^-3.5) = 181/2048); had_scale = 2^-3.5
 * reproduces the weight-side hadamard_transform(..., scale=2**-3.5) (benchmarks/utils.py:38-39).
 * y may alias x.  group_size % 128 == 0.
 */
int quest_hadamard128(void *y, const void *x, int group_size, int batch_size, float had_scale,
                      int dtype, void *stream);

/*
 * One pass over x that does what linear_forward does before its GEMM (benchmarks/utils.py:89-100):
 * Hadamard (as quest_hadamard128, optional: had_scale == 0 skips it), scale (as
 * quest_find_scale_int4 on the transformed row), INT4 codes packed (as quest_quantize_int4) and
 * their row sums.  x is read once and never written.  x_had, when not NULL, receives the
 * transformed activations (dtype) the scale and codes were computed from.  scale is required;
 * x_int_packed and x_int_row_sum are optional.  group_size % 128 == 0 and <= 65536 (had_scale == 0:
 * group_size % 8 == 0, every K the GEMM takes).
 * Which arithmetic runs depends on (group_size, had_scale, dtype) only, never on batch_size or on where the buffers
 * lie: a had_scale the dtype holds exactly (181/2048) with group_size <= 32768 is the product with the +-had_scale
 * matrix on the matrix cores, fp32 accumulation, as the reference states the activation transform; any other factor
 * (2^-3.5, the weight-side one), and rows over 32768, are fp32 butterflies followed by one multiplication.  Without a
 * transform (had_scale == 0) rows of whole blocks of 128 up to 32768 run on the same matrix-core kernel with the
 * multiplications left out (the values only change lanes), other rows on the row kernel; the two differ in the order
 * of the fp32 sum of squares only (the scale may come out one ulp apart on rare rows).  The two transforms
 * agree to fp32 summation noise (<= 1e-3 relative, the transform's stated bar), so that a value on a rounding boundary
 * of the dtype may come out one ulp apart and its code one level apart: codes are reproducible for a given shape,
 * factor and dtype, not across the two.  Given the transformed tensor and the scale, codes and row sums are exactly
 * quest_quantize_int4's in both.
 */
int quest_hadamard_quantize_int4(const void *x, void *scale, uint8_t *x_int_packed,
                                 int32_t *x_int_row_sum, void *x_had, int group_size, int batch_size,
                                 float had_scale, int dtype, void *stream);

/*
 * quest_hadamard_quantize_int4 with the rule for the scale as a parameter: QUEST_SCALE_GAUSSIAN is the reference's
 * (benchmarks/utils.py:46, 207-208); QUEST_SCALE_ABSMAX sets scale = dtype(max|x| / 7.5 + 1e-8), the per-row absmax
 * rule the CPU-runnable benchmark case names for its pre-quantised weights (no counterpart in the reference's code).
 */
#define QUEST_SCALE_GAUSSIAN 0
#define QUEST_SCALE_ABSMAX 1
/* OR-ed into scale_rule: scale and codes from the transform's fp32 output and the unrounded scale (fp32 butterflies, any
 * had_scale), the arithmetic of the reference's evaluation-side fake quantiser (src/eval_hswag.py:201-214), instead of
 * from the dtype-rounded tensor that linear_forward materialises (benchmarks/utils.py:89-100).  The stored scale is still
 * rounded to dtype.  For comparing a packed model with its fake-quantised original; not bit-pinned. */
#define QUEST_QUANT_FROM_FP32 4
int quest_hadamard_quantize_int4_rule(const void *x, void *scale, uint8_t *x_int_packed, int32_t *x_int_row_sum,
                                      void *x_had, int group_size, int batch_size, float had_scale,
                                      int scale_rule, int dtype, void *stream);

/*
 * quest_fused_matmul_dequantize_int4_int4t for the gate and up projections of a SwiGLU MLP in one GEMM, with the
 * gated unit applied in the epilogue: mat_b holds the 2 H weight rows interleaved in eights -- rows 8 g .. 8 g + 3
 * the gate rows of outputs 4 g .. 4 g + 3, rows 8 g + 4 .. 8 g + 7 their up rows -- with vec_b_add / vec_b_mul in the
 * same order, and mat_d (size_m, size_n / 2) = dtype(dtype(silu(gate)) * up), gate and up being the two
 * dtype-rounded outputs the plain entry point would have written (silu(g) = g / (1 + exp(-g)) in fp32;
 * src/models/llama.py:117-118).  The (size_m, 2 H) tensor is never written.  No counterpart in the reference, which
 * runs two GEMMs and the torch expression.  size_n % 8 == 0; QUEST_ERR_UNSUPPORTED unless size_k % 128 == 0,
 * size_m > 64 (the caller then uses the plain entry point and applies the unit itself).
 */
int quest_fused_matmul_dequantize_swiglu_int4_int4t(void *mat_d, const uint8_t *mat_a, const uint8_t *mat_b,
                                                    const int32_t *vec_a_add, const int32_t *vec_b_add,
                                                    const void *vec_a_mul, const void *vec_b_mul, int size_m,
                                                    int size_k, int size_n, int dtype, void *stream);

/*
 * quest_hadamard_quantize_int4 with the producer of the activation in front, so that the normalised tensor is
 * never written: y = dtype(dtype(f32(x) * rsqrt(mean(x^2) + eps)) * norm_weight) -- the RMSNorm in front of every
 * attention and MLP block of the reference's model (src/models/llama.py:71-77, applied at llama.py:174-175) --
 * then Hadamard, scale, codes, row sums of y as above.  x_norm, when not NULL, receives y.  No counterpart in
 * the reference's quest package, which quantises a tensor the norm has already written.
 * group_size % 128 == 0, group_size <= 32768, had_scale exactly representable in dtype (181/2048 is);
 * QUEST_ERR_UNSUPPORTED otherwise (the caller then runs the norm itself and quest_hadamard_quantize_int4).
 */
int quest_rmsnorm_hadamard_quantize_int4(const void *x, const void *norm_weight, float eps, void *scale,
                                         uint8_t *x_int_packed, int32_t *x_int_row_sum, void *x_had,
                                         void *x_norm, int group_size, int batch_size, float had_scale,
                                         int dtype, void *stream);

/*
 * quest_rmsnorm_hadamard_quantize_int4 with the residual addition in front of the norm (x = x + attn(...);
 * ... ln_2(x), src/models/llama.py:175-176, and the same across two blocks): x <- dtype(x + branch) in place, one
 * rounding as the framework's addition has, then everything above on the new x.  Saves the separate addition pass
 * (two reads and a write of the residual stream).  No counterpart in the reference's quest package.  Limits and
 * error behaviour as above; x and branch are (batch_size, group_size) and must not overlap.
 */
int quest_add_rmsnorm_hadamard_quantize_int4(void *x, const void *branch, const void *norm_weight, float eps,
                                             void *scale, uint8_t *x_int_packed, int32_t *x_int_row_sum,
                                             int group_size, int batch_size, float had_scale, int dtype,
                                             void *stream);

/*
 * The same for the SwiGLU product in front of the MLP's output projection (src/models/llama.py:117-118):
 * gate_up is (batch_size, 2 * group_size), gate in the first half of each row and up in the second;
 * y = dtype(dtype(silu(gate)) * up), silu(g) = g / (1 + exp(-g)) in fp32.  x_act, when not NULL, receives y
 * (batch_size, group_size).  Limits and error behaviour as above.
 */
int quest_silu_mul_hadamard_quantize_int4(const void *gate_up, void *scale, uint8_t *x_int_packed,
                                          int32_t *x_int_row_sum, void *x_had, void *x_act, int group_size,
                                          int batch_size, float had_scale, int dtype, void *stream);

/*
 * Rotary position embedding, in place, on the first rot_cols elements of each of n_rows rows of x (row pitch
 * row_stride elements): the columns are heads of head_dim elements holding interleaved (re, im) pairs; row r is
 * position r % seq_len; freqs_cis is fp32 (seq_len, head_dim / 2, 2) = (cos, sin).  out_re = re cos - im sin,
 * out_im = re sin + im cos, every product and sum rounded to fp32, one rounding to dtype: bit for bit what
 * apply_rotary_emb (src/models/llama.py:43-62) computes for q and k.  With x the (B T, 3 d) output of the fused
 * QKV projection and rot_cols = 2 d it rotates q and k where they lie and leaves v alone.
 * head_dim % 8 == 0, rot_cols % head_dim == 0, row_stride % 8 == 0.
 */
int quest_rope_interleaved(void *x, const float *freqs_cis, int n_rows, int seq_len, int row_stride,
                           int rot_cols, int head_dim, int dtype, void *stream);

/*
 * ---- the FP6 matrix-core path: operands in "E2M3 tiles" ----------------------------------------------------------
 * Both operands of the reference's fused GEMM are dequantised as (q + 1/2) * scale (quest/quantize_kernel.cu:162,
 * benchmarks/utils.py:667-678), so 2 C + a_add + b_add of its epilogue (benchmarks/utils.py:544) is
 * 2 * sum_k (qa + 1/2)(qb + 1/2).  The sixteen values q + 1/2 are exact in FP6 E2M3 and every partial sum of up to
 * 65536 of their products is exact in fp32, so the gfx950 FP6 matrix instructions (twice the INT8 rate) give the
 * reference's outputs bit for bit.  These entry points have no counterpart in the reference's quest_c extension;
 * they are what quest_fused_matmul_dequantize_int4_int4t and quest_hadamard_quantize_int4 are for a caller that keeps
 * its codes in the operand form instead of packed nibbles.
 *
 * E2M3 tiles of a (rows, size_k) code matrix, size_k % 64 == 0: ceil(rows / 32) row blocks x size_k / 64 fragments
 * of 1536 bytes, row block major.  In fragment (rb, ks), lane l = 32 g + i (row 32 rb + i, codes k = 64 ks + 32 g ..
 * + 31) owns 32 x 6 bits, code j (the E2M3 bits of q + 1/2) at bits [6 j, 6 j + 6) of its 24 bytes: bytes 0 .. 15 at
 * fragment offset 16 l, bytes 16 .. 23 at offset 1024 + 8 l.  Rows past `rows` in the last row block are padding: any
 * content is valid there (E2M3 has no Inf or NaN) and no result depends on it.
 */

/* Bytes of the E2M3 tiles of a (rows, size_k) code matrix; 0 for an invalid shape. */
size_t quest_e2m3_tiles_bytes(int rows, int size_k);

/* tiles = the E2M3 tiles of the packed INT4 codes x_int_packed (rows, size_k / 2), low nibble = even k. */
int quest_int4_to_e2m3_tiles(void *tiles, const uint8_t *x_int_packed, int rows, int size_k, void *stream);

/*
 * mat_d (size_m, size_n) dtype = quest_fused_matmul_dequantize_int4_int4t's result for the same codes, from their
 * E2M3 tiles: dtype( f32(2 S) * (0.5f * vec_a_mul[m] * vec_b_mul[n]) ) with S = sum_k (qa + 1/2)(qb + 1/2) accumulated
 * exactly.  size_k % 128 == 0 and <= 65536; any size_m, size_n >= 1; scale vectors 4-byte aligned.
 */
int quest_fused_matmul_dequantize_e2m3(void *mat_d, const void *a_tiles, const void *b_tiles, const void *vec_a_mul,
                                       const void *vec_b_mul, int size_m, int size_k, int size_n, int dtype,
                                       void *stream);

/*
 * quest_fused_matmul_dequantize_e2m3 adding its result to what mat_d holds: mat_d <- dtype(mat_d + dtype(product)), the two
 * roundings of the framework's `x = x + linear(...)` (the residual additions of src/models/llama.py:175-176 with the
 * projection that ends the branch, in one launch: the residual stream is read and written once and the branch's output
 * never exists).  Every element of mat_d is read and written by the same lane; same shapes and limits.
 */
int quest_fused_matmul_dequantize_add_e2m3(void *mat_d, const void *a_tiles, const void *b_tiles, const void *vec_a_mul,
                                           const void *vec_b_mul, int size_m, int size_k, int size_n, int dtype,
                                           void *stream);

/*
 * quest_fused_matmul_dequantize_int4_int4t adding its result to what mat_d holds: mat_d <- dtype(mat_d + dtype(product)), the
 * two roundings of the framework's `x = x + linear(...)` (src/models/llama.py:175-176 with the projection that ends the
 * branch, in one launch), on packed codes.  Only the large-tile kernel has this epilogue: QUEST_ERR_UNSUPPORTED (nothing
 * launched) for the sizes the plain entry point gives to another kernel; quest_fused_matmul_dequantize_add_available says
 * beforehand (1 / 0) whether a size runs in one launch on the stream's device.  mat_d 16-byte aligned.
 */
int quest_fused_matmul_dequantize_add_int4_int4t(void *mat_d, const uint8_t *mat_a, const uint8_t *mat_b,
                                                 const int32_t *vec_a_add, const int32_t *vec_b_add, const void *vec_a_mul,
                                                 const void *vec_b_mul, int size_m, int size_k, int size_n, int dtype,
                                                 void *stream);
int quest_fused_matmul_dequantize_add_available(int size_m, int size_k, int size_n, void *stream);

/*
 * quest_fused_matmul_dequantize_int4_int4t with quest_rope_interleaved applied to the first rot_cols channels of its result
 * before it is stored (`self.c_attn(x)` followed by `apply_rotary_emb(q, k, freqs_cis)`, src/models/llama.py:134-140 and
 * 43-62, in one launch), on packed codes: arguments and limits as quest_fused_matmul_dequantize_rope_e2m3 below.  The
 * large-tile and the small-tile kernels have this epilogue: QUEST_ERR_UNSUPPORTED (nothing launched) for the sizes the plain
 * entry point gives to another kernel (size_m <= 64, size_m <= 128 with size_n <= 8192, size_k % 128 != 0, scale vectors or
 * output not 4- / 16-byte aligned) -- make the two calls then.
 */
int quest_fused_matmul_dequantize_rope_int4_int4t(void *mat_d, const uint8_t *mat_a, const uint8_t *mat_b,
                                                  const int32_t *vec_a_add, const int32_t *vec_b_add, const void *vec_a_mul,
                                                  const void *vec_b_mul, int size_m, int size_k, int size_n, int dtype,
                                                  const float *freqs_cis, int seq_len, int rot_cols, int head_dim,
                                                  void *stream);

/*
 * quest_fused_matmul_dequantize_e2m3 with quest_rope_interleaved applied to the first rot_cols channels of its result before
 * it is stored (the q and k of a fused QKV projection, src/models/llama.py:134-140 with apply_rotary_emb, 43-62, in the
 * projection's launch): row r is position r % seq_len of its sequence, the channels are heads of head_dim, pair i of a head
 * turns by freqs_cis[r % seq_len][i] = (cos, sin) (fp32, (seq_len, head_dim / 2, 2), 16-byte aligned).  Bit for bit the
 * two separate calls.  Limits beyond the plain entry point's: size_n % 8 == 0, head_dim % 32 == 0, rot_cols % head_dim == 0
 * and <= size_n, seq_len >= 32 (QUEST_ERR_BAD_SHAPE otherwise -- make the two calls).
 */
int quest_fused_matmul_dequantize_rope_e2m3(void *mat_d, const void *a_tiles, const void *b_tiles, const void *vec_a_mul,
                                            const void *vec_b_mul, int size_m, int size_k, int size_n, int dtype,
                                            const float *freqs_cis, int seq_len, int rot_cols, int head_dim, void *stream);

/*
 * Diagnostic (host only, nothing is launched): how quest_fused_matmul_dequantize_e2m3 divides a shape among the
 * workgroups of a device with `cus` compute units.  plan[0..7] = workgroups, scheduling groups (one per XCD when 8),
 * tiles per token tile when every workgroup gets exactly one (else 0), how many ways the groups divide the token tiles
 * (0 or 1: not at all, each group takes a slice of the channel units; g: a g x groups / g grid of groups), tile rows, tile channels at most, LDS slots, k per slot.  A measured figure that depends on
 * the schedule (HBM traffic per launch) is only valid while this plan is the one it was measured under.
 */
int quest_e2m3_gemm_plan(int size_m, int size_k, int size_n, int cus, int *plan);

/* The same with the SwiGLU epilogue of quest_fused_matmul_dequantize_swiglu_int4_int4t (b_tiles and vec_b_mul in its
 * interleaved row order); mat_d is (size_m, size_n / 2). */
int quest_fused_matmul_dequantize_swiglu_e2m3(void *mat_d, const void *a_tiles, const void *b_tiles,
                                              const void *vec_a_mul, const void *vec_b_mul, int size_m, int size_k,
                                              int size_n, int dtype, void *stream);

/*
 * quest_hadamard_quantize_int4 writing the codes as E2M3 tiles (x_tiles, quest_e2m3_tiles_bytes(batch_size,
 * group_size) bytes; rows past batch_size in the last row block are left unwritten: the GEMM never uses what it
 * computes from them).  The tiles hold exactly the codes the packed output would: x_int_packed and x_int_row_sum may
 * be asked for as well.  Only the matrix-core kernel writes tiles: had_scale must be exactly representable in dtype
 * (181/2048 is) or 0 (no transform), group_size % 128 == 0 and <= 32768; QUEST_ERR_UNSUPPORTED otherwise (the caller
 * then quantises to packed codes and converts them with quest_int4_to_e2m3_tiles).
 */
int quest_hadamard_quantize_e2m3(const void *x, void *scale, void *x_tiles, uint8_t *x_int_packed,
                                 int32_t *x_int_row_sum, void *x_had, int group_size, int batch_size, float had_scale,
                                 int dtype, void *stream);

/* quest_rmsnorm_hadamard_quantize_int4, quest_add_rmsnorm_hadamard_quantize_int4 and
 * quest_silu_mul_hadamard_quantize_int4 with the codes written as E2M3 tiles instead of packed nibbles and row sums. */
int quest_rmsnorm_hadamard_quantize_e2m3(const void *x, const void *norm_weight, float eps, void *scale, void *x_tiles,
                                         void *x_norm, int group_size, int batch_size, float had_scale, int dtype,
                                         void *stream);
int quest_add_rmsnorm_hadamard_quantize_e2m3(void *x, const void *branch, const void *norm_weight, float eps,
                                             void *scale, void *x_tiles, int group_size, int batch_size,
                                             float had_scale, int dtype, void *stream);
int quest_silu_mul_hadamard_quantize_e2m3(const void *gate_up, void *scale, void *x_tiles, void *x_act, int group_size,
                                          int batch_size, float had_scale, int dtype, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* QUEST_HIP_H */
