/*
 * sonar_marlin.h - C ABI of the MI355X (gfx950) W4A16 Marlin-family GEMM library.
 *
 * Every entry point takes plain device pointers, sizes and a HIP stream
 * (passed as void*; NULL = the null stream).  All work is enqueued on that
 * stream; nothing synchronises with the host.  Return value: 0 on success, a
 * negative SONAR_E_* code on failure; sonar_marlin_last_error() then returns a
 * message for the calling thread.  Nothing is launched when a call fails.
 *
 * The entry points replace these reference interfaces (paths relative to the
 * reference checkout):
 *   sonar_gptq_marlin_repack  -> _C::gptq_marlin_repack
 *        csrc/libtorch_stable/torch_bindings.cpp:107-109,
 *        csrc/libtorch_stable/quantization/marlin/gptq_marlin_repack.cu:285-362
 *   sonar_awq_marlin_repack   -> _C::awq_marlin_repack
 *        csrc/libtorch_stable/torch_bindings.cpp:113-115,
 *        csrc/libtorch_stable/quantization/marlin/awq_marlin_repack.cu:228-290
 *   sonar_marlin_gemm         -> _C::marlin_gemm
 *        csrc/libtorch_stable/torch_bindings.cpp:96-103,
 *        csrc/libtorch_stable/quantization/marlin/marlin.cu:546-897
 *   sonar_marlin_gemm_nvfp4   -> the same op called with b_q_type = float4_e2m1f, float8_e4m3fn
 *        block scales and a global_scale (marlin.cu:600-611,784-796)
 *   sonar_marlin_gemm_a8      -> the same op called with int8 or float8_e4m3fn activations and
 *        a_scales (marlin.cu:567-598,666-679; marlin_template.h:1302-1400,1869-1903)
 *   sonar_gptq_marlin_repack_a8 / sonar_awq_marlin_repack_a8 -> the repack ops with is_a_8bit
 *        (gptq_marlin_repack.cu:14-268, awq_marlin_repack.cu:14-212)
 *   sonar_per_token_quant_int8 / _fp8 -> per_token_quant_int8 (a Triton kernel in the reference,
 *        layers/quantization/utils/int8_utils.py:70-120) and QuantFP8 per token
 *        (layers/quantization/input_quant_fp8.py:188-204), which marlin_quant_input calls
 *   sonar_marlin_int4_fp8_preprocess -> _C::marlin_int4_fp8_preprocess
 *        csrc/libtorch_stable/quantization/marlin/marlin_int4_fp8_preprocess.cu:13-121
 *   sonar_moe_wna16_marlin_gemm -> _moe_C::moe_wna16_marlin_gemm
 *        csrc/libtorch_stable/moe/torch_bindings.cpp:76-89,
 *        csrc/libtorch_stable/moe/marlin_moe_wna16/ops.cu:544-897
 * sonar_marlin_to_gfx950 / sonar_gfx950_to_marlin have no reference
 * counterpart: they convert between the Marlin tile order that the repack ops
 * return (and every reference caller stores) and the streaming order the
 * gfx950 kernels read.
 */
#ifndef SONAR_MARLIN_H_
#define SONAR_MARLIN_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SONAR_OK 0
#define SONAR_E_INVALID (-1)       /* bad argument (shape, alignment, null pointer) */
#define SONAR_E_UNSUPPORTED (-2)   /* valid for the reference op, not built here */
#define SONAR_E_RUNTIME (-3)       /* a HIP call failed */

/* activation / output / scale element types */
#define SONAR_DTYPE_F16 0
#define SONAR_DTYPE_BF16 1
#define SONAR_DTYPE_F32 2          /* input of the per-token quantisers only */

/* 8-bit activation types of sonar_marlin_gemm_a8 */
#define SONAR_ADTYPE_INT8 0
#define SONAR_ADTYPE_FP8 1        /* float8_e4m3fn */

/* weight orders accepted by the GEMM entry points */
#define SONAR_LAYOUT_GFX950 0      /* output of sonar_marlin_to_gfx950 */

/* ScalarType ids that cross the op boundary as b_type_id
 * (aphrodite/scalar_type.py:129-156, csrc/core/scalar_type.hpp:131-164) */
#define SONAR_TYPE_UINT4B8 1125899907892224LL /* GPTQ: code - 8 */
#define SONAR_TYPE_UINT4 1125899906843648LL   /* AWQ: code - zero point */
#define SONAR_TYPE_UINT8B128 1125899923621888LL /* GPTQ 8-bit: code - 128 */
/* 8-bit floating-point codes (sign, 4 exponent bits, 3 mantissa bits, no infinities), in the 8-bit
 * weight order; b_scales then hold the scales times 2^8 (fp16) or 2^120 (bf16), as
 * fp8_fused_exponent_bias_into_scales makes them (quantization/utils/marlin_utils_fp8.py:35-46);
 * one scale per column, per group of 128 rows (marlin/generate_kernels.py:87-93) or, for MXFP8, per
 * group of 32 rows (:111-119; the torch op takes the exponent bytes of the reference's callers and
 * makes such scales of them); no act-order */
#define SONAR_TYPE_FLOAT8_E4M3FN 2814749767172868LL
/* 4-bit floating-point codes (sign, 2 exponent bits, 1 mantissa bit) in the 4-bit weight order,
 * with one power-of-two scale per column and group of 32 rows (MXFP4): bfloat16 activations only;
 * b_scales hold the block scales 2^(e - 127) as bfloat16 in marlin_permute_scales order (the
 * reference passes the exponent bytes e, reordered by mxfp4_marlin_process_scales,
 * quantization/utils/marlin_utils_fp4.py:123-135; the torch op takes those and converts them);
 * no zero points, no act-order (marlin/generate_kernels.py:102-110) */
#define SONAR_TYPE_FLOAT4_E2M1F 562949953487106LL

const char* sonar_marlin_last_error(void);
const char* sonar_marlin_version(void);

/* The launch the calling thread's last sonar_marlin_gemm / _nvfp4 / _noalloc call made with the
 * decode kernel (no counterpart in the reference; for benchmarks that quote per-launch counter
 * figures and must know that the launch shapes are still the profiled ones).  Fills
 *   out[0]  workgroups of the launch (0: the last call did not run the decode kernel)
 *   out[1]  threads per workgroup
 *   out[2]  pieces every strip was cut into along K
 *   out[3]  1 when the weight copies carried the non-temporal bit
 * and returns the number of entries written (at most n). */
int sonar_marlin_last_decode_launch(int32_t* out, int n);

/* GPTQ (K/8, N) int32, nibble k%8 of word [k/8][n] = code of W[k][n]
 * -> Marlin (K/16, 2N) int32; with num_bits == 8: (K/4, N) int32, byte k%4
 * -> Marlin (K/16, 4N) int32.  perm (int32[K], may be NULL) selects source
 * rows: output row k is source row perm[k].
 * (gptq_marlin_repack, csrc/libtorch_stable/quantization/marlin/gptq_marlin_repack.cu:285-362) */
int sonar_gptq_marlin_repack(const uint32_t* b_q_weight, const int32_t* perm,
                             uint32_t* out, int64_t size_k, int64_t size_n,
                             int num_bits, void* stream);

/* AWQ (K, N/8) int32, nibble p of word [k][n/8] = code of column
 * 8*(n/8) + {0,2,4,6,1,3,5,7}[p] -> Marlin (K/16, 2N) int32. */
int sonar_awq_marlin_repack(const uint32_t* b_q_weight, uint32_t* out,
                            int64_t size_k, int64_t size_n, int num_bits,
                            void* stream);

/* Marlin (K/16, 2N) int32 <-> gfx950 streaming order, same number of words.
 * K % 32 == 0, N % 64 == 0.  in and out must not overlap. */
int sonar_marlin_to_gfx950(const uint32_t* marlin, uint32_t* out,
                           int64_t size_k, int64_t size_n, void* stream);
int sonar_gfx950_to_marlin(const uint32_t* gfx950, uint32_t* out,
                           int64_t size_k, int64_t size_n, void* stream);

/* The same for 8-bit codes (uint8b128, float8_e4m3fn): Marlin (K/16, 4N) int32 <-> the
 * streaming order of 1-KiB blocks of 16 rows x 64 columns.  No counterpart in
 * the reference (its kernels read the Marlin order directly). */
int sonar_marlin8_to_gfx950(const uint32_t* marlin, uint32_t* out,
                            int64_t size_k, int64_t size_n, void* stream);
int sonar_gfx950_to_marlin8(const uint32_t* gfx950, uint32_t* out,
                            int64_t size_k, int64_t size_n, void* stream);

/* The repack ops with is_a_8bit = true (gptq_marlin_repack.cu:14-268, awq_marlin_repack.cu:14-212):
 * 4-bit codes into the order the reference's kernels read with 8-bit activations, tiles of
 * 32 (k) x 32 (n).  in as for the ops above, out (K/16, 2N) int32 ((K/16, 4N) for 8-bit codes, GPTQ
 * source only; no GEMM takes that order, here or in the reference).  size_k % 32 == 0,
 * size_n % 64 == 0; no perm (the reference's kernel refuses act-order with is_a_8bit). */
int sonar_gptq_marlin_repack_a8(const uint32_t* b_q_weight, uint32_t* out,
                                int64_t size_k, int64_t size_n, int num_bits, void* stream);
int sonar_awq_marlin_repack_a8(const uint32_t* b_q_weight, uint32_t* out,
                               int64_t size_k, int64_t size_n, int num_bits, void* stream);
/* That order <-> the streaming order of the gfx950 kernels (the same one as for 16-bit
 * activations).  No counterpart in the reference. */
int sonar_marlin_a8_to_gfx950(const uint32_t* marlin, uint32_t* out,
                              int64_t size_k, int64_t size_n, void* stream);
int sonar_gfx950_to_marlin_a8(const uint32_t* gfx950, uint32_t* out,
                              int64_t size_k, int64_t size_n, void* stream);

/* marlin_int4_fp8_preprocess (marlin_int4_fp8_preprocess.cu:13-121): every 4-bit code q of
 * qweight becomes sign and magnitude of q - z in a nibble: q >= z ? q - z : 15 - q.  qzeros NULL:
 * z = 8, qweight is rows * words_per_row words in any order.  qzeros given (AWQ): qweight is
 * (rows = size_k, words_per_row = size_n / 8), qzeros (size_k / group_size, size_n / 8), both in the
 * checkpoint's order.  out may be qweight. */
int sonar_marlin_int4_fp8_preprocess(const uint32_t* qweight, const uint32_t* qzeros, uint32_t* out,
                                     int64_t rows, int64_t words_per_row, int64_t group_size,
                                     void* stream);

/* Dequantised weight matrix W[K][N] (row-major, dtype elements) exactly as the
 * GEMM kernels form it in registers: round_to_dtype((code - z) * s), for
 * float8_e4m3fn round_to_dtype(value(code) * scale).  Uses the
 * same device routine as the GEMM; exists so the in-kernel values can be
 * compared bit for bit.  Arguments as for sonar_marlin_gemm. */
int sonar_marlin_dequant(const uint32_t* b_q_weight, int b_layout,
                         const void* b_scales, const uint32_t* b_zeros,
                         const int32_t* g_idx, void* w_out, int dtype,
                         int64_t b_type_id, int64_t size_n, int64_t size_k,
                         int64_t num_groups, int is_k_full, void* stream);

/* Bytes of scratch sonar_marlin_gemm needs for (size_m, size_n, size_k). */
size_t sonar_marlin_gemm_scratch_bytes(int64_t size_m, int64_t size_n, int64_t size_k);

/* C[M,N] = A[M,K] * dequant(B)[K,N] (+ bias), fp32 accumulation, result
 * rounded to dtype.
 *   a            dtype[M][a_row_stride], 16-byte aligned, a_row_stride % 8 == 0
 *   c            dtype[M][N] contiguous
 *   b_q_weight   K*N/8 words (K*N/4 for the 8-bit types) in b_layout order
 *   b_bias       dtype[N] in marlin_permute_bias order, or NULL
 *   b_scales     dtype[num_groups][N] in marlin_permute_scales order
 *   b_zeros      int32[num_groups][N/8] in marlin_zero_points order, or NULL
 *                (required iff b_type_id == SONAR_TYPE_UINT4)
 *   g_idx, perm  int32[K] each or both NULL; with both given the call is an
 *                act-order call (symmetric weights only: with b_zeros it is
 *                refused with SONAR_E_UNSUPPORTED, "Unsupported shapes", as
 *                the reference has no such kernel,
 *                marlin/generate_kernels.py:66-72): perm maps weight row k to
 *                column perm[k] of A; g_idx[k] is the group of weight row k,
 *                read only when is_k_full == 0 (a shard that does not hold
 *                whole groups: b_scales then has every group of the unsharded
 *                matrix, num_groups need not divide K, and the
 *                size_m * size_k * 2 extra scratch bytes below are required)
 *   workspace    int32[workspace_len], all zero on entry, all zero on exit;
 *                workspace_len >= number of compute units
 *   scratch      sonar_marlin_gemm_scratch_bytes() bytes, contents don't care;
 *                an act-order call given size_m * size_k * 2 bytes more uses
 *                them for a column-permuted copy of A, which is much faster
 *                than gathering A inside the GEMM
 * use_atomic_add and use_fp32_reduce are accepted for signature parity; the
 * reduction is always fp32 and deterministic. */
int sonar_marlin_gemm(const void* a, int64_t a_row_stride, void* c,
                      const uint32_t* b_q_weight, int b_layout,
                      const void* b_bias, const void* b_scales,
                      const uint32_t* b_zeros, const int32_t* g_idx,
                      const int32_t* perm, int32_t* workspace,
                      int64_t workspace_len, void* scratch,
                      size_t scratch_bytes, int dtype, int64_t b_type_id,
                      int64_t size_m, int64_t size_n, int64_t size_k,
                      int64_t num_groups, int is_k_full, int use_atomic_add,
                      int use_fp32_reduce, void* stream);

/* Per-token quantisation of the activations for sonar_marlin_gemm_a8: one fp32 scale per row.
 * int8 (per_token_quant_int8, layers/quantization/utils/int8_utils.py:70-120): scale =
 * max(absmax, 1e-10) / 127, code = x * (127 / absmax) rounded half away from zero.
 * fp8 (QuantFP8 per token, layers/quantization/input_quant_fp8.py:188-204): scale =
 * max(absmax / 448, 1 / (448 * 512)), code = float8_e4m3fn(clamp(x * (1 / scale), -448, 448)).
 *   x   dtype[rows][row_stride] (SONAR_DTYPE_F16, _BF16 or _F32); q [rows][cols]; scales float[rows] */
int sonar_per_token_quant_int8(const void* x, int dtype, int64_t row_stride, int8_t* q,
                               float* scales, int64_t rows, int64_t cols, void* stream);
int sonar_per_token_quant_fp8(const void* x, int dtype, int64_t row_stride, uint8_t* q,
                              float* scales, int64_t rows, int64_t cols, void* stream);

/* W4A8 (marlin.cu:567-598,666-679 of the reference; marlin_template.h:1302-1400,1869-1903,
 * 1955-1978): 4-bit weights, 8-bit activations with one fp32 scale per row, on the 8-bit matrix
 * cores.
 *   a            int8 (a_dtype SONAR_ADTYPE_INT8) or float8_e4m3fn bytes (SONAR_ADTYPE_FP8),
 *                [M][a_row_stride], 16-byte aligned, a_row_stride % 8 == 0
 *   a_scales     float[M]
 *   c            dtype[M][N]; dtype is also the type of b_scales (channelwise) and b_bias
 *   b_q_weight   K*N/8 words in b_layout order.  With fp8 activations the nibbles are the ones
 *                marlin_int4_fp8_preprocess leaves (sign and magnitude), as the reference's callers
 *                store them
 *   b_scales     [num_groups][N] in marlin_permute_scales(is_a_8bit=True) order (the single
 *                permutation inside every 32 columns).  int8 activations and num_groups > 1: 16-bit
 *                unsigned integers (marlin_act_int8_process_scales); otherwise numbers of dtype; with
 *                fp8 activations they carry the factor 512 the reference's callers apply
 *   b_zeros      int32[num_groups][N/8] in marlin_zero_points(is_a_8bit=True) order, iff uint4
 *   b_bias       dtype[N] in marlin_permute_bias order, or NULL
 *   scratch      sonar_marlin_gemm_a8_scratch_bytes() bytes
 * int8:  C = round(float(sum_g s[g][n] * sum_{k in g} a[m][k] * (q[k][n] - z)) * a_scales[m] + bias),
 *        the sums in wrapping 32-bit integers (exact, whatever the order); channelwise:
 *        round((float(sum_k a (q - z)) * a_scales[m]) * s[n] + bias).
 * fp8:   the same with fp32 sums and the weights (q - z) * 2^-9.
 * num_groups 1 (channelwise) or size_k / 32, / 64, / 128; size_k % 32 == 0, size_n % 64 == 0; no
 * act-order (the reference builds no such kernel).  b_type_id uint4b8 or uint4, or float4_e2m1f
 * with float8_e4m3fn activations (MXFP4 weights, "W4A8-FP4", dequant.h:474-490, marlin.cu:576-590):
 * b_scales then are exponent bytes [K/32][N] in the same order, each 6 above the checkpoint's
 * (mxfp4_marlin_process_scales with an fp8 input type), no zero points, dtype bfloat16 only
 * (marlin/generate_kernels.py:152-161; float16 is refused with SONAR_E_UNSUPPORTED), and
 * C = round((sum_g 2^(e[g][n] - 127 - 6) * sum_{k in g} a[m][k] * value(code[k][n])) * a_scales[m] + bias). */
size_t sonar_marlin_gemm_a8_scratch_bytes(int64_t size_m, int64_t size_n, int64_t size_k,
                                          int64_t num_groups);
int sonar_marlin_gemm_a8(const void* a, int64_t a_row_stride, int a_dtype, void* c,
                         const uint32_t* b_q_weight, int b_layout, const void* b_bias,
                         const void* b_scales, const float* a_scales, const uint32_t* b_zeros,
                         void* scratch, size_t scratch_bytes, int dtype, int64_t b_type_id,
                         int64_t size_m, int64_t size_n, int64_t size_k, int64_t num_groups,
                         void* stream);

/* The grouped (mixture-of-experts) form of sonar_marlin_gemm_a8: _moe_C::moe_wna16_marlin_gemm called
 * with int8 / float8_e4m3fn activations and a_scales (moe/marlin_moe_wna16/marlin_template.h:471-560,
 * 622-650,2020-2060).  Row id of sorted_token_ids: row id / top_k of a and of a_scales, row id of c
 * and of topk_weights.
 *   a          [size_m][size_k] bytes, contiguous, 8-byte aligned;  a_scales float[size_m]
 *   c          dtype[size_m * top_k][size_n]; rows of blocks whose expert id is outside
 *              [0, num_experts) are left untouched
 *   b_q_weight, b_scales, b_zeros, b_bias: as for sonar_marlin_gemm_a8 with a leading expert dimension
 * Every (block, 64-column strip) is one workgroup over the whole of K; no scratch.  The other
 * arguments as for sonar_moe_wna16_marlin_gemm. */
int sonar_moe_wna16_marlin_gemm_a8(
    const void* a, int a_dtype, void* c, const uint32_t* b_q_weight, int b_layout,
    const void* b_bias, const void* b_scales, const float* a_scales, const uint32_t* b_zeros,
    const int32_t* sorted_token_ids, int64_t sorted_len, const int32_t* expert_ids,
    const int32_t* num_tokens_past_padded, const float* topk_weights, int64_t moe_block_size,
    int64_t top_k, int mul_topk_weights, int64_t num_experts, int dtype, int64_t b_type_id,
    int64_t size_m, int64_t size_n, int64_t size_k, int64_t num_groups, void* stream);

/* NVFP4 (marlin.cu:600-611,784-796 of the reference; marlin_template.h:1661-1665;
 * marlin_utils_fp4.py:59-151): float4_e2m1f codes (b_q_weight as for the other 4-bit types),
 * one block scale per 16 rows and column, and one global scale.
 *   C = round_to_dtype((A * W) * *global_scale (+ bias)),  W[k][n] = value(code) * b_scales[k / 16][n]
 *   b_scales      dtype[size_k / 16][N] in marlin_permute_scales order: the block scales as
 *                 numbers of the activation type.  value * scale must be exact in that type
 *                 (it is for the reference's fp8 block scales: 1 + 3 mantissa bits).  The
 *                 reference's callers hold the scales as bytes of a special 8-bit format
 *                 (nvfp4_marlin_process_scales); a byte b stands for the half-precision
 *                 number with the bits b << 7 times 2^-14 (half) or 2^-126 (bfloat16), which
 *                 is what this argument takes; the torch op converts.
 *   global_scale  one float in device memory (what nvfp4_marlin_process_global_scale
 *                 returns, divided by the scale factor of the block scales)
 * dtype is SONAR_DTYPE_F16 or SONAR_DTYPE_BF16; num_groups == size_k / 16; no zero points,
 * no act-order.  The other arguments as for sonar_marlin_gemm.  sonar_marlin_dequant takes
 * the same b_scales with num_groups == size_k / 16 and returns value(code) * scale. */
int sonar_marlin_gemm_nvfp4(const void* a, int64_t a_row_stride, void* c,
                            const uint32_t* b_q_weight, int b_layout,
                            const void* b_bias, const void* b_scales,
                            const float* global_scale, int32_t* workspace,
                            int64_t workspace_len, void* scratch,
                            size_t scratch_bytes, int dtype, int64_t size_m,
                            int64_t size_n, int64_t size_k, int64_t num_groups,
                            void* stream);

/* sonar_marlin_gemm for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Same arguments without `scratch` / `scratch_bytes`: the scratch memory (fp32
 * partial tiles of strips or tiles whose K range is shared between workgroups; with act-order the
 * column-permuted copy of A when it fits) is a static array in device memory of 24 MiB, one
 * per GPU, held until the process ends.  The call allocates and frees nothing.  A call whose
 * sonar_marlin_gemm_scratch_bytes(size_m, size_n, size_k) exceeds 24 MiB (K split over many
 * workgroups of the tile kernels: 65 to 128 rows on K >= 8192, or 97 to 128 rows on N = 28672,
 * take 56 MiB) still runs: the 8 MiB of the streaming kernels always fit, and the tile kernels
 * split K only as far as their partial tiles fit (another order of summation than
 * sonar_marlin_gemm's, slower, the same tolerance).  What cannot make do is refused with
 * SONAR_E_INVALID before anything is launched: act-order with 8-bit weights or with
 * is_k_full = 0 needs the copy of A (size_m * size_k * 2 bytes) inside the array.  All calls on one
 * GPU share that GPU's array: calls that overlap in time on one GPU (two streams, two
 * threads) race and give wrong results; calls on one stream, or ordered by events, do not.
 * Nothing in the array has to be zero between calls.  The first call on a device looks the
 * array's address up (hipGetSymbolAddress); make it outside graph capture. */
int sonar_marlin_gemm_noalloc(const void* a, int64_t a_row_stride, void* c,
                              const uint32_t* b_q_weight, int b_layout,
                              const void* b_bias, const void* b_scales,
                              const uint32_t* b_zeros, const int32_t* g_idx,
                              const int32_t* perm, int32_t* workspace,
                              int64_t workspace_len, int dtype, int64_t b_type_id,
                              int64_t size_m, int64_t size_n, int64_t size_k,
                              int64_t num_groups, int is_k_full, int use_atomic_add,
                              int use_fp32_reduce, void* stream);

/* Grouped (mixture-of-experts) variant.  For block b <
 * num_tokens_past_padded[0] / moe_block_size with expert e = expert_ids[b]
 * (e < 0: skipped), each slot id = sorted_token_ids[b*moe_block_size + i] with
 * id < size_m*top_k gives C[id,:] = A[id / top_k,:] * dequant(B[e]) (+
 * bias[e]), rounded to dtype, then multiplied in dtype by
 * dtype(topk_weights[id]) when mul_topk_weights != 0.
 *   a            dtype[M][K] contiguous
 *   c            dtype[M*top_k][N] contiguous
 *   b_q_weight   num_experts * K*N/8 words (K*N/4 for the 8-bit types), each expert
 *                in b_layout order; b_type_id uint4b8, uint4, uint8b128, float8_e4m3fn
 *                or float4_e2m1f (scales as described at the type ids)
 *   b_scales     dtype[num_experts][num_groups][N]; b_zeros / b_bias likewise
 *   scratch      sonar_moe_marlin_gemm_scratch_bytes(): for 64-slot blocks the tables of
 *                row tiles and 96 MiB for fp32 partial tiles (the tile kernel cuts few
 *                tiles, or those of a short last round, along K; with less, down to
 *                the table alone, it runs without that); act-order calls run 4 to
 *                20 times faster with sorted_len * K * 2 bytes more behind that
 *                size rounded up to 256 (a column-permuted copy of A per slot;
 *                required for act-order with uint8b128)
 *   g_idx, perm  int32[num_experts][K] or NULL (act-order: symmetric weights only, refused
 *                with SONAR_E_UNSUPPORTED together with b_zeros); with is_k_full == 0 (shards that
 *                hold no whole group) g_idx is the group of
 *                every sorted row and num_groups the groups of the whole matrix
 *   sorted_token_ids int32[sorted_len], expert_ids int32[ceil(sorted_len/bs)],
 *   num_tokens_past_padded int32[1] (read on the device), topk_weights
 *   float[M*top_k]
 */
size_t sonar_moe_marlin_gemm_scratch_bytes(int64_t sorted_len, int64_t moe_block_size,
                                           int64_t size_n, int64_t size_k);
int sonar_moe_wna16_marlin_gemm(
    const void* a, void* c, const uint32_t* b_q_weight, int b_layout,
    const void* b_bias, const void* b_scales, const uint32_t* b_zeros,
    const int32_t* g_idx, const int32_t* perm, int32_t* workspace,
    int64_t workspace_len, void* scratch, size_t scratch_bytes,
    const int32_t* sorted_token_ids, int64_t sorted_len,
    const int32_t* expert_ids, const int32_t* num_tokens_past_padded,
    const float* topk_weights, int64_t moe_block_size, int64_t top_k,
    int mul_topk_weights, int64_t num_experts, int dtype, int64_t b_type_id,
    int64_t size_m, int64_t size_n, int64_t size_k, int64_t num_groups,
    int is_k_full, int use_atomic_add, int use_fp32_reduce, void* stream);

/* The grouped GEMM for NVFP4 experts (moe/marlin_moe_wna16/ops.cu of the reference called
 * with b_q_type = float4_e2m1f, float8_e4m3fn block scales and a global_scale per expert):
 * b_scales dtype[E][size_k / 16][N] as for sonar_marlin_gemm_nvfp4, global_scale float[E] in
 * device memory (row r of C is multiplied by the global scale of its block's expert before
 * the bias and the routing weight).  No zero points, no act-order; the other arguments as for
 * sonar_moe_wna16_marlin_gemm. */
int sonar_moe_wna16_marlin_gemm_nvfp4(
    const void* a, void* c, const uint32_t* b_q_weight, int b_layout,
    const void* b_bias, const void* b_scales, const float* global_scale,
    void* scratch, size_t scratch_bytes, const int32_t* sorted_token_ids,
    int64_t sorted_len, const int32_t* expert_ids,
    const int32_t* num_tokens_past_padded, const float* topk_weights,
    int64_t moe_block_size, int64_t top_k, int mul_topk_weights,
    int64_t num_experts, int dtype, int64_t size_m, int64_t size_n,
    int64_t size_k, int64_t num_groups, void* stream);

/* The small kernels around the two grouped GEMMs of a mixture-of-experts layer.
 * They have counterparts in every build of the reference (also on ROCm):
 *   sonar_moe_align_block_size -> _moe_C::moe_align_block_size
 *        csrc/libtorch_stable/moe/torch_bindings.cpp:36-41,
 *        csrc/libtorch_stable/moe/moe_align_sum_kernels.cu:626-725
 *   sonar_moe_sum              -> _moe_C::moe_sum (moe_align_sum_kernels.cu:759+)
 *   sonar_silu_and_mul         -> _C::silu_and_mul
 *        csrc/libtorch_stable/torch_bindings.cpp:640, activation_kernels.cu
 * so the torch layer registers them under its own namespace, not under _C.
 *
 * sonar_moe_align_block_size: topk_ids int32[numel] (expert of every
 * (token, k) slot).  Slots are grouped by expert, ascending slot id inside an
 * expert, every expert's run padded to a multiple of block_size with the
 * sentinel `numel`; expert_ids[b] is the expert of block b, -1 past the
 * padded total, which goes to num_tokens_post_pad[0].  With expert_map
 * (int32[num_experts], -1 = absent) slots of absent experts are dropped and
 * experts are numbered and ordered by their mapped ids.  sorted_len must be
 * at least numel + num_experts * (block_size - 1) (or numel * block_size when
 * that is smaller and numel < num_experts); offsets_scratch is int32[num_experts].
 * sonar_silu_and_mul: out[rows][d] = T(T(silu(in[r][c])) * in[r][d + c]),
 * in is [rows][2 d].  sonar_moe_sum: out[tokens][d] = T(sum_k in[t][k][d]) in fp32. */
int sonar_moe_align_block_size(const int32_t* topk_ids, int64_t numel, int64_t num_experts,
                               int64_t block_size, int32_t* sorted_token_ids, int64_t sorted_len,
                               int32_t* expert_ids, int64_t expert_len, int32_t* num_tokens_post_pad,
                               const int32_t* expert_map, int32_t* offsets_scratch, void* stream);
int sonar_silu_and_mul(void* out, const void* in, int64_t rows, int64_t d, int dtype, void* stream);
int sonar_moe_sum(void* out, const void* in, int64_t tokens, int64_t topk, int64_t d, int dtype,
                  void* stream);

/* The other gated activations apply_moe_activation dispatches between the two grouped GEMMs
 * (aphrodite/model_executor/layers/fused_moe/activation.py:128-205): in is [rows][2 d] (gate half,
 * then up half; SONAR_ACT_SWIGLUOAI: gate and up alternate), out is [rows][d], T the 16-bit type.
 *   SONAR_ACT_SILU_CLAMP  _C::silu_and_mul_with_clamp(out, in, limit, alpha, beta)
 *        (torch_bindings.cpp:644-649, activation_kernels.cu:28-76,154-160): SILU with clamp_limit,
 *        and SWIGLUOAI_UNINTERLEAVE (the experts of gpt-oss in the packed gate | up order):
 *        g = T(min(gate, limit)), u = clamp(up, -limit, limit),
 *        out = T(float(T(g / (1 + exp(-alpha g)))) * (u + beta))
 *   SONAR_ACT_GELU / SONAR_ACT_GELU_TANH  _C::gelu_and_mul / gelu_tanh_and_mul (activation_kernels.cu:172-215)
 *   SONAR_ACT_SWIGLUOAI   _C::swigluoai_and_mul(out, in, alpha = 1.702, limit = 7.0)
 *        (activation_kernels.cu:412-423): out = T((u + 1) g / (1 + exp(-alpha g))), g = min(gate, limit),
 *        u = clamp(up, -limit, limit)
 *   SONAR_ACT_SITU        _C::situ_and_mul(out, in, beta, linear_beta) (activation_kernels.cu:489-510):
 *        `alpha` carries beta, `beta` carries linear_beta (<= 0: up passes through)
 *   SONAR_ACT_SWIGLUSTEP  swiglustep_and_mul_triton (aphrodite/model_executor/layers/activation.py:27-72):
 *        out = T(min(silu(gate), limit) * clamp(up, -limit, limit)) */
#define SONAR_ACT_SILU_CLAMP 1
#define SONAR_ACT_GELU 2
#define SONAR_ACT_GELU_TANH 3
#define SONAR_ACT_SWIGLUOAI 4
#define SONAR_ACT_SITU 5
#define SONAR_ACT_SWIGLUSTEP 6
int sonar_moe_activation(void* out, const void* in, int64_t rows, int64_t d, int kind, float limit,
                         float alpha, float beta, int dtype, void* stream);

/* Diagnostics for host-side tests; no counterpart in the reference.  The tile kernels'
 * launches for a dense call (4-bit integer codes, no act-order, room for every partial
 * tile), or for a grouped call whose routing made `row_tiles` row tiles of `tile_rows`
 * rows out of at most `max_row_tiles`: one row of six int32 per workgroup that has
 * work (launch, rows of a tile, row tile, column tile, first K step, end of its K
 * steps), from the planning and mapping code the launches and the kernels run.
 * Returns the number of such workgroups (rows beyond out_rows are counted, not
 * written), -1 for arguments out of range.  Runs on the host; needs no GPU. */
int64_t sonar_debug_tile_schedule(int64_t size_m, int64_t size_n, int64_t size_k,
                                  int64_t num_groups, int32_t* out, int64_t out_rows);
int64_t sonar_debug_moe_tile_schedule(int64_t row_tiles, int64_t max_row_tiles, int64_t size_n,
                                      int64_t size_k, int tile_rows, int with_partial,
                                      int32_t* out, int64_t out_rows);

#ifdef __cplusplus
}
#endif
#endif /* SONAR_MARLIN_H_ */
