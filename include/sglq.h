/* libsglq — C ABI of the MI355X (gfx950) W8A8 quantized-linear kernels.
 *
 * Every entry point takes raw device pointers, sizes, strides (in elements) and
 * a HIP stream (hipStream_t passed as void*; NULL = the null stream).  Nothing
 * is allocated, retained or synchronised: work is enqueued on the stream and
 * the call returns.  Return value: 0 on success, otherwise one of the SGLQ_E*
 * codes; sglq_last_error() then holds a message for the calling thread.
 *
 * "Reference" below is sgl-kernel 0.3.3 inside walker-ai/sglang; each entry
 * point names the torch op it stands in for.
 */
#ifndef SGLQ_H
#define SGLQ_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SGLQ_OK 0
#define SGLQ_EINVAL 1      /* bad shape / stride / alignment / null pointer */
#define SGLQ_EUNSUPPORTED 2 /* valid in the reference but not built here */
#define SGLQ_ELAUNCH 3     /* hipGetLastError() after the launch was not hipSuccess */

/* element type codes for 16/32-bit floating inputs and outputs */
#define SGLQ_BF16 0
#define SGLQ_FP16 1
#define SGLQ_FP32 2
#define SGLQ_I32 3 /* raw accumulators (sglq_int8_mm_i32 only) */

const char* sglq_last_error(void);
int sglq_abi_version(void);

/* Replaces torch.ops.sgl_kernel.sgl_per_token_group_quant_fp8
 * (sgl-kernel/csrc/gemm/per_token_group_quant_8bit.cu:116-217,230-240; schema
 * sgl-kernel/csrc/common_extension.cc:116-119).  The UE8M0 packed-scale mode
 * (scale_ue8m0=true) is sglq_per_token_group_quant_fp8_ue8m0.
 *
 * input  [num_tokens, hidden] contiguous, in_dtype in {BF16, FP16, FP32}
 * output_q  same shape, one e4m3fn byte per element
 * output_s  fp32; element (row, g) lives at output_s[row*s_stride_row + g*s_stride_col],
 *           which covers the reference's row-major, column-major and padded
 *           column-major scale buffers (per_token_group_quant_8bit.cu:54-64,153-156)
 * group_size in {8, 16, 32, 64, 128}; hidden % group_size == 0. */
int sglq_per_token_group_quant_fp8(const void* input, int in_dtype, void* output_q, float* output_s,
                                   int64_t num_tokens, int64_t hidden, int group_size,
                                   int64_t s_stride_row, int64_t s_stride_col, float eps, float fp8_min,
                                   float fp8_max, void* stream);

/* sgl_per_token_group_quant_fp8 with scale_ue8m0 = true
 * (sgl-kernel/csrc/gemm/per_token_group_quant_8bit.cu:50-65,86-105,193-204; the
 * output tensor of python/sglang/srt/layers/quantization/fp8_kernel.py:308-320):
 * groups of 128; the scale of a group is the smallest power of two >=
 * max(max(|x|, eps) / fp8_max, 1e-10) and codes are clamp(x / scale) rounded to
 * e4m3fn.  output_s is the reference's packed int32 tensor [num_tokens, ceil4(K/128)/4]
 * with column stride s_stride_col (in 32-bit words, >= num_tokens) and row stride 1: byte
 * g % 4 of word (row, g / 4) receives the biased exponent (scale = 2^(byte - 127)) of
 * group g.  Bytes of groups beyond K/128 are left as they are (the caller zero-fills). */
int sglq_per_token_group_quant_fp8_ue8m0(const void* input, int in_dtype, void* output_q, void* output_s,
                                         int64_t num_tokens, int64_t hidden, int64_t s_stride_col, float eps,
                                         float fp8_min, float fp8_max, void* stream);

/* sglq_per_token_group_quant_fp8_ue8m0's scales as fp32 instead of packed exponent bytes: the scale of a
 * group of 128 is the smallest power of two >= max(amax / fp8_max, 1e-10) (per_token_group_quant_8bit.cu:86-89),
 * stored like sglq_per_token_group_quant_fp8 stores its scales (element (row, g) at
 * output_s[row*s_stride_row + g*s_stride_col]); the codes are the same bytes as that entry point's.  It feeds
 * sglq_fp8_blockwise_scaled_mm_ue8m0 in the place of the quantization call of
 * deepgemm_w8a8_block_fp8_linear_with_fallback (python/sglang/srt/layers/quantization/fp8_utils.py:240-246). */
int sglq_per_token_group_quant_fp8_pow2(const void* input, int in_dtype, void* output_q, float* output_s,
                                        int64_t num_tokens, int64_t hidden, int64_t s_stride_row, int64_t s_stride_col,
                                        float eps, float fp8_min, float fp8_max, void* stream);

/* Replaces torch.ops.sgl_kernel.sgl_per_token_group_quant_int8
 * (per_token_group_quant_8bit.cu:219-228; schema common_extension.cc:121-124):
 * same arithmetic with an int8 destination, the float-to-int8 cast truncating
 * toward zero as the C++ cast in per_token_group_quant_8bit.cu:111 does. */
int sglq_per_token_group_quant_int8(const void* input, int in_dtype, void* output_q, float* output_s,
                                    int64_t num_tokens, int64_t hidden, int group_size,
                                    int64_t s_stride_row, int64_t s_stride_col, float eps, float int8_min,
                                    float int8_max, void* stream);

/* Replaces torch.ops.sgl_kernel.sgl_per_tensor_quant_fp8
 * (sgl-kernel/csrc/gemm/per_tensor_quant_fp8.cu:96-123; schema
 * common_extension.cc:126-127): one scale for the whole tensor of num_elements
 * elements.  is_static == 0: *output_s must be zero on entry (the reference's
 * caller allocates it with zeros, fp8_kernel.py:1252) and receives
 * max|x| / 448 through an atomic max; is_static != 0: *output_s is read only.
 * Codes are max(min(x * (1 / *output_s), 448), -448) rounded to e4m3fn. */
int sglq_per_tensor_quant_fp8(const void* input, int in_dtype, void* output_q, float* output_s,
                              int64_t num_elements, int is_static, void* stream);

/* Replaces static_quant_fp8, a Triton kernel in the reference
 * (python/sglang/srt/layers/quantization/fp8_kernel.py:395-490; caller
 * apply_fp8_linear, fp8_utils.py:684-689): codes are
 * clamp(x * (1 / *scale), -448, 448) rounded to e4m3fn for the contiguous
 * [num_tokens, hidden] input; scale_repeat, if not NULL, receives *scale once per
 * token ([num_tokens] floats, the reference's repeat_scale=True output [M, 1]). */
int sglq_static_quant_fp8(const void* input, int in_dtype, void* output_q, const float* scale,
                          float* scale_repeat, int64_t num_tokens, int64_t hidden, void* stream);

/* Replaces torch.ops.sgl_kernel.sgl_per_token_quant_fp8
 * (sgl-kernel/csrc/gemm/per_token_quant_fp8.cu:166-227; schema
 * common_extension.cc:129-130), zero rows giving zero codes as in the
 * guarded kernel (:57).  hidden % 8 == 0 (:173).  output_s has num_tokens floats. */
int sglq_per_token_quant_fp8(const void* input, int in_dtype, void* output_q, float* output_s,
                             int64_t num_tokens, int64_t hidden, void* stream);

/* Replaces the Triton kernel behind per_token_quant_int8
 * (python/sglang/srt/layers/quantization/int8_kernel.py:20-81); the reference
 * has no compiled op for it.  row_sum may be NULL; otherwise it receives the
 * fp32-accumulated row sums in in_dtype (cal_sum=True, :43-45). */
int sglq_per_token_quant_int8(const void* input, int in_dtype, void* output_q, float* output_s,
                              void* row_sum, int64_t num_tokens, int64_t hidden, void* stream);

/* Replaces torch.ops.sgl_kernel.fp8_blockwise_scaled_mm
 * (sgl-kernel/csrc/gemm/fp8_blockwise_gemm_kernel.cu:345-423; schema
 * common_extension.cc:111-114).
 *   a   e4m3fn [M, K], row stride lda, unit column stride
 *   b   e4m3fn [K, N] column-major: element (k, n) at b[n*ldb + k]
 *   sfa fp32 [M, ceil(K/128)]  at sfa[m*sfa_stride_m + kb*sfa_stride_k]
 *   sfb fp32 [ceil(K/128), ceil(N/128)] at sfb[kb*sfb_stride_k + nb*sfb_stride_n]
 *   out [M, N] row stride ldo, out_dtype in {BF16, FP16}
 * K % 16 == 0, lda % 16 == 0, ldb % 16 == 0, a and b 16-byte aligned; N % 8 == 0,
 * ldo % 8 == 0 and out 16-byte aligned (output rows are written in 16-byte pieces; the
 * reference's own checks, fp8_blockwise_gemm_kernel.cu:383, int8_gemm_kernel.cu:679,
 * fp8_gemm_kernel.cu:1108).  The same holds for every GEMM entry point below
 * (sglq_int8_mm_i32: N % 4 == 0, ldo % 4 == 0).
 *
 * workspace (all four GEMM entry points): optional device scratch of
 * workspace_bytes bytes, 16-byte aligned, owned by the caller and not shared
 * with a call running concurrently on another stream.  Where a shape has too
 * few output tiles to fill the chip, several blocks share a tile, each with a
 * part of K (split-K), and their fp32 / int32 partial sums pass through it
 * (4 * splits * M * N bytes; the split factor is capped by what fits); it plays
 * the part of the per-call
 * workspace tensor that the reference's launchers allocate
 * (fp8_blockwise_gemm_kernel.cu:153-155).  NULL or too small only costs speed. */
int sglq_fp8_blockwise_scaled_mm(const void* a, int64_t lda, const void* b, int64_t ldb, const float* sfa,
                                 int64_t sfa_stride_m, int64_t sfa_stride_k, const float* sfb,
                                 int64_t sfb_stride_k, int64_t sfb_stride_n, void* out, int64_t ldo,
                                 int out_dtype, int64_t M, int64_t N, int64_t K, void* workspace,
                                 int64_t workspace_bytes, void* stream);

/* sglq_fp8_blockwise_scaled_mm for scales that are all powers of two (UE8M0 values held as fp32: what
 * ceil_to_ue8m0 produces, python/sglang/srt/layers/quantization/fp8_utils.py:485-486).  It stands in for the
 * DeepGEMM call of the reference's w8a8_block_fp8_matmul_deepgemm (fp8_kernel.py; a third-party kernel there),
 * whose caller deepgemm_w8a8_block_fp8_linear_with_fallback (fp8_utils.py:214-258) quantizes with such scales.
 * Same arguments, layouts and checks as sglq_fp8_blockwise_scaled_mm; for such scales the same sums formed in
 * another order (within one unit of the 16-bit output of that entry point's result, not bit-identical).  For bf16
 * outputs on the shapes of the 256- and 128-row pipelined kernels (roughly M > 128) the matrix instruction
 * applies the scales itself (v_mfma_scale_f32_16x16x128_f8f6f4 takes one exponent byte per lane and operand)
 * and accumulates in place; only the exponent bits of the scales are read there, so a scale that is not a
 * power of two is silently rounded down to one: the caller guarantees the property (it is not checked: the
 * scales are device data).  Every other shape runs exactly as sglq_fp8_blockwise_scaled_mm. */
int sglq_fp8_blockwise_scaled_mm_ue8m0(const void* a, int64_t lda, const void* b, int64_t ldb, const float* sfa,
                                       int64_t sfa_stride_m, int64_t sfa_stride_k, const float* sfb,
                                       int64_t sfb_stride_k, int64_t sfb_stride_n, void* out, int64_t ldo,
                                       int out_dtype, int64_t M, int64_t N, int64_t K, void* workspace,
                                       int64_t workspace_bytes, void* stream);

/* sglq_fp8_blockwise_scaled_mm_ue8m0 with the activation scales in the packed form that
 * sgl_per_token_group_quant_fp8 writes with scale_ue8m0 = true (sglq_per_token_group_quant_fp8_ue8m0;
 * sgl-kernel/csrc/gemm/per_token_group_quant_8bit.cu:57-64,94) and that the reference hands to DeepGEMM as it is
 * (fp8_utils.py:240-258, fp8_kernel.py:308-320): int32 words of four UE8M0 codes, byte kb % 4 of word
 * [m, kb / 4] is K block kb's code, the word at sfa_packed[m * sfa_stride_m + (kb / 4) * sfa_stride_k4] (the
 * column-major, 4-row-padded tensor of the reference: sfa_stride_m = 1, sfa_stride_k4 = M rounded up to 4).
 * K must be a multiple of 128.  The kernels whose matrix instruction applies the scales fetch the words and pick
 * the byte themselves; for every other shape the library first expands them into fp32 at the head of the
 * workspace, which must therefore hold at least M * K / 128 floats rounded up to 256 bytes (the rest serves
 * split-K as in the other entry points).  Results: those of sglq_fp8_blockwise_scaled_mm_ue8m0 on the same
 * scales as fp32, bit for bit.  sfb stays fp32 powers of two [N/128, K/128]. */
int sglq_fp8_blockwise_scaled_mm_ue8m0_packed(const void* a, int64_t lda, const void* b, int64_t ldb,
                                              const int32_t* sfa_packed, int64_t sfa_stride_m, int64_t sfa_stride_k4,
                                              const float* sfb, int64_t sfb_stride_k, int64_t sfb_stride_n, void* out,
                                              int64_t ldo, int out_dtype, int64_t M, int64_t N, int64_t K,
                                              void* workspace, int64_t workspace_bytes, void* stream);

/* sglq_fp8_blockwise_scaled_mm fused with the bias add that its caller performs on the
 * result (python/sglang/srt/layers/quantization/fp8_utils.py:207-211: the GEMM, then
 * `output += bias` on the rounded output): out = round(round(gemm) + bias), bias [N] in
 * out_dtype or NULL.  Saves one read-modify-write pass over [M, N]. */
int sglq_fp8_blockwise_scaled_mm_bias(const void* a, int64_t lda, const void* b, int64_t ldb, const float* sfa,
                                      int64_t sfa_stride_m, int64_t sfa_stride_k, const float* sfb,
                                      int64_t sfb_stride_k, int64_t sfb_stride_n, const void* bias, void* out,
                                      int64_t ldo, int out_dtype, int64_t M, int64_t N, int64_t K, void* workspace,
                                      int64_t workspace_bytes, void* stream);

/* The call pair of cutlass_w8a8_block_fp8_linear_with_fallback
 * (python/sglang/srt/layers/quantization/fp8_utils.py:204-211: per_token_group_quant_fp8 with
 * groups of 128, fp8_blockwise_scaled_mm, `output += bias`) as one entry point, the fused form
 * that the reference's CPU backend has for its INT8 path (sgl-kernel/csrc/cpu/gemm_int8.cpp:422-489):
 *   x    [M, K] contiguous activations, in_dtype in {BF16, FP16, FP32}, 16-byte aligned, K % 128 == 0
 *   b, sfb, bias (may be NULL), out: as sglq_fp8_blockwise_scaled_mm_bias
 *   eps  lower bound of a group's abs-max (the callers' 1e-10)
 * For M <= 4 (16-bit activations) on the shapes that the decode kernel without split-K takes with
 * between one and 2.5 blocks per compute unit (where it was measured faster), one
 * kernel quantizes each K block's activations in LDS right before multiplying them: no
 * quantization launch, no round trip of codes and scales through memory, no workspace.  Other
 * shapes run the quantization kernel and the GEMM one after the other; their codes and
 * column-major scales need M * K + 4 * M * K / 128 bytes (each rounded up to 256) at the head of
 * the 16-byte aligned workspace, the rest serves the GEMM's split-K as usual.  The output is
 * bit-identical to sglq_per_token_group_quant_fp8 followed by sglq_fp8_blockwise_scaled_mm(_bias). */
int sglq_w8a8_block_fp8_linear(const void* x, int in_dtype, const void* b, int64_t ldb, const float* sfb,
                               int64_t sfb_stride_k, int64_t sfb_stride_n, const void* bias, void* out, int64_t ldo,
                               int out_dtype, int64_t M, int64_t N, int64_t K, float eps, void* workspace,
                               int64_t workspace_bytes, void* stream);

/* The call pairs of the per-token linears as one entry point each:
 *   sglq_w8a8_int8_linear  per_token_quant_int8 + int8_scaled_mm, W8A8Int8LinearMethod.apply
 *                          (python/sglang/srt/layers/quantization/w8a8_int8.py:387-391);
 *   sglq_w8a8_fp8_linear   sgl_per_token_quant_fp8 + fp8_scaled_mm, apply_fp8_linear's dynamic per-token
 *                          branch (python/sglang/srt/layers/quantization/fp8_utils.py:693,725-732).
 * The fused form is the one the reference's CPU backend has, int8_scaled_mm_with_quant
 * (sgl-kernel/csrc/cpu/gemm_int8.cpp:423-489).
 *   x    [M, K] contiguous activations, in_dtype in {BF16, FP16, FP32}, 16-byte aligned
 *   b, scales_b, bias (may be NULL), out: as sglq_int8_scaled_mm / sglq_fp8_scaled_mm
 * For M <= 2 (16-bit activations, K % 128 == 0) on the shapes that the decode kernel without
 * split-K takes, one kernel forms the rows' scales in its prologue and quantizes each K block's
 * activations in LDS right before multiplying them: no quantization launch, no round trip of codes
 * and scales through memory, no workspace.  Other shapes run the quantization kernel and the GEMM
 * one after the other; their codes and row scales need M * K + 4 * M bytes (each rounded up to
 * 256) at the head of the 16-byte aligned workspace, the rest serves the GEMM's split-K as usual.
 * The output is bit-identical to the two operators called in turn. */
int sglq_w8a8_int8_linear(const void* x, int in_dtype, const void* b, int64_t ldb, const float* scales_b,
                          const void* bias, void* out, int64_t ldo, int out_dtype, int64_t M, int64_t N, int64_t K,
                          void* workspace, int64_t workspace_bytes, void* stream);
int sglq_w8a8_fp8_linear(const void* x, int in_dtype, const void* b, int64_t ldb, const float* scales_b,
                         const void* bias, void* out, int64_t ldo, int out_dtype, int64_t M, int64_t N, int64_t K,
                         void* workspace, int64_t workspace_bytes, void* stream);

/* No counterpart in the reference.  sglq_fp8_blockwise_scaled_mm for callers that cannot
 * allocate device memory (code under HIP graph capture, tight serving loops, harnesses that
 * forbid it) and therefore have no workspace to pass: the split-K partial sums go through a
 * fixed device array of SGLQ_NOALLOC_SCRATCH_BYTES inside the library (one copy per GPU, held
 * until the process ends) and the call allocates nothing.  Same arguments, checks and results
 * as sglq_fp8_blockwise_scaled_mm called with a workspace of that size: K is split (and the
 * array used) only for outputs of up to SGLQ_NOALLOC_MAX_OUTPUTS elements, two fp32 partial sums
 * each; larger outputs run unsplit without touching the array, and sizes beyond the library's
 * limits (an operand of 2 GiB or more, 2^30 rows or columns) are rejected with SGLQ_EUNSUPPORTED
 * and a message, before anything is launched.  All calls on one GPU share
 * that GPU's array: calls that overlap on one GPU (two streams, two threads) race on the
 * partial sums and must be serialised by the caller; calls in sequence on one stream are safe
 * (the array needs no clearing between calls).  The array's address is resolved per device on
 * the first call there, or by sglq_init() with that device current: call either once before
 * capturing a graph. */
#define SGLQ_NOALLOC_SCRATCH_BYTES (32ll << 20)
#define SGLQ_NOALLOC_MAX_OUTPUTS (SGLQ_NOALLOC_SCRATCH_BYTES / 8)
int sglq_init(void);
int sglq_fp8_blockwise_scaled_mm_noalloc(const void* a, int64_t lda, const void* b, int64_t ldb, const float* sfa,
                                         int64_t sfa_stride_m, int64_t sfa_stride_k, const float* sfb,
                                         int64_t sfb_stride_k, int64_t sfb_stride_n, void* out, int64_t ldo,
                                         int out_dtype, int64_t M, int64_t N, int64_t K, void* stream);

/* Replaces torch.ops.sgl_kernel.fp8_blockwise_scaled_grouped_mm
 * (sgl-kernel/csrc/moe/fp8_blockwise_moe_kernel.cu:587-754; schema
 * common_extension.cc:192-197; callers python/sglang/srt/layers/moe/cutlass_moe.py:170-213):
 * num_experts block-scaled FP8 GEMMs that share N and K in one launch sequence.  Expert e
 * multiplies rows expert_offsets[e] .. expert_offsets[e] + problem_sizes[e][0] - 1 of
 * a [total_m, K] (e4m3fn, row stride lda) with its weight b + e * b_expert_stride
 * ([N, K] rows of ldb bytes, i.e. the reference's column-major [K, N] slice) into the same
 * rows of out [total_m, N].  sfa [total_m, K/128] (element strides given; the reference's
 * K-major SM100 convention is strides (K/128, 1)), sfb element (e, kb, nb) at
 * sfb + e * sfb_expert_stride + kb * sfb_stride_k + nb * sfb_stride_n.  problem_sizes
 * ([num_experts, 3] int32, only column 0 is read: N and K are arguments) and
 * expert_offsets ([num_experts] int32) are DEVICE pointers: nothing is copied to the host.
 * The reference's pointer, stride and layout scratch tensors have no counterpart; the
 * workspace holds the tile plan, 16 * (total_m / 32 + num_experts + 1) bytes always suffice.
 * Rows outside every expert's range are left untouched. */
int sglq_fp8_blockwise_scaled_grouped_mm(const void* a, int64_t lda, const void* b, int64_t ldb,
                                         int64_t b_expert_stride, const float* sfa, int64_t sfa_stride_m,
                                         int64_t sfa_stride_k, const float* sfb, int64_t sfb_expert_stride,
                                         int64_t sfb_stride_k, int64_t sfb_stride_n, void* out, int64_t ldo,
                                         int out_dtype, const int32_t* problem_sizes, const int32_t* expert_offsets,
                                         int64_t num_experts, int64_t total_m, int64_t N, int64_t K, void* workspace,
                                         int64_t workspace_bytes, void* stream);

/* The data movement around the grouped GEMM in an MoE layer
 * (python/sglang/srt/layers/moe/cutlass_moe.py:140-222).
 *
 * sglq_prepare_moe_input replaces torch.ops.sgl_kernel.prepare_moe_input
 * (sgl-kernel/csrc/moe/prepare_moe_input.cu:13-166; schema common_extension.cc:199-203):
 * topk_ids [topk_length] int32, slot i belonging to token i / topk; outputs
 * expert_offsets [num_experts + 1], blockscale_offsets [num_experts + 1] or NULL (offsets of
 * the counts rounded up to 128), problem_sizes1 [num_experts, 3] = (count, 2 n, k),
 * problem_sizes2 = (count, k, n), input_permutation [topk_length] (expert-major position ->
 * token) and output_permutation [topk_length] (slot -> expert-major position).  Positions
 * inside an expert follow slot order (the reference's order depends on thread timing); ids
 * outside [0, num_experts) are routed nowhere.  No scratch buffer is needed.
 *
 * sglq_shuffle_rows replaces shuffle_rows (prepare_moe_input.cu:168-244):
 * output row d = input row dst2src_map[d], rows of row_bytes bytes, any element type.
 *
 * sglq_silu_and_mul replaces silu_and_mul (sgl-kernel/csrc/elementwise/activation.cu:57-60,
 * 85-103): input [num_tokens, 2 d], output [num_tokens, d] = T(silu(x[:, :d])) * x[:, d:],
 * T = dtype (SGLQ_BF16 or SGLQ_FP16); 16 bytes per lane when d is a multiple of 8 and the
 * pointers are 16-byte aligned, one element per lane otherwise.
 *
 * sglq_apply_shuffle_mul_sum replaces apply_shuffle_mul_sum (prepare_moe_input.cu:258-392):
 * output [m, row] = sum_j factors[i topk + j] * input[permutation[i topk + j]], fp32
 * accumulation in j order; factors [m topk] in dtype or NULL (all ones); input has
 * num_src_rows rows. */
int sglq_prepare_moe_input(const int32_t* topk_ids, int32_t* expert_offsets, int32_t* blockscale_offsets,
                           int32_t* problem_sizes1, int32_t* problem_sizes2, int32_t* input_permutation,
                           int32_t* output_permutation, int64_t topk_length, int64_t topk, int64_t num_experts,
                           int64_t n, int64_t k, void* stream);
int sglq_shuffle_rows(const void* input, const int32_t* dst2src_map, void* output, int64_t num_src_rows,
                      int64_t num_dst_rows, int64_t row_bytes, void* stream);
int sglq_silu_and_mul(const void* input, int dtype, void* output, int64_t num_tokens, int64_t d, void* stream);
int sglq_apply_shuffle_mul_sum(const void* input, void* output, const int32_t* permutation, const void* factors,
                               int dtype, int64_t m, int64_t topk, int64_t row, int64_t num_src_rows, void* stream);

/* sgl_per_token_group_quant_fp8 with group 128 (per_token_group_quant_8bit.cu:72-113) followed by
 * the two shuffle_rows calls that replicate codes and scales into expert-major order
 * (python/sglang/srt/layers/moe/cutlass_moe.py:156-158), in one kernel: input [num_tokens, hidden];
 * token t's codes go to rows slot_map[t * topk + j] (j < topk) of output_q [num_dst_rows, hidden]
 * and its scales to the same rows of output_s [num_dst_rows, hidden / 128] (row-major); slot_map is
 * prepare_moe_input's output_permutation; entries outside [0, num_dst_rows) are skipped.  Rows that
 * no slot names are left untouched.  Bit-identical to the three calls. */
int sglq_per_token_group_quant_fp8_scatter(const void* input, int in_dtype, void* output_q, float* output_s,
                                           const int32_t* slot_map, int64_t num_tokens, int64_t hidden, int64_t topk,
                                           int64_t num_dst_rows, float eps, void* stream);

/* silu_and_mul (activation.cu:57-60) followed by sgl_per_token_group_quant_fp8 with group 128
 * (per_token_group_quant_8bit.cu:72-113), the pair of calls of
 * python/sglang/srt/layers/moe/cutlass_moe.py:187-194, in one kernel that never writes the
 * intermediate: input [num_tokens, 2 d] in dtype (SGLQ_BF16 or SGLQ_FP16), output_q
 * [num_tokens, d] e4m3fn, output_s [num_tokens, d / 128] fp32 row-major, d a multiple of 128.
 * Codes and scales are bit-identical to sglq_silu_and_mul followed by
 * sglq_per_token_group_quant_fp8(group 128, eps, -448, 448). */
int sglq_silu_and_mul_group_quant_fp8(const void* input, int in_dtype, void* output_q, float* output_s,
                                      int64_t num_tokens, int64_t d, float eps, void* stream);

/* Replaces w8a8_block_int8_matmul, a Triton kernel in the reference
 * (python/sglang/srt/layers/quantization/int8_kernel.py:212-425; there is no
 * sgl_kernel C++ op): out[m,n] = sum_kb float(sum_{k in block kb} a[m,k] b[k,n])
 * * sfa[m,kb] * sfb[kb, n/128], the int32 block sums exact, fp32 accumulation over
 * kb, one rounding to out_dtype (Half or BFloat16).  Arguments as
 * sglq_fp8_blockwise_scaled_mm with int8 operands; the reference passes the
 * weight as stored, [N, K] row-major (= b with ldb = K), its scales
 * [N/128, K/128] (sfb_stride_k = 1, sfb_stride_n = K/128) and row-major
 * activation scales [M, K/128] (sfa_stride_m = K/128, sfa_stride_k = 1). */
int sglq_int8_blockwise_scaled_mm(const void* a, int64_t lda, const void* b, int64_t ldb, const float* sfa,
                                  int64_t sfa_stride_m, int64_t sfa_stride_k, const float* sfb,
                                  int64_t sfb_stride_k, int64_t sfb_stride_n, void* out, int64_t ldo,
                                  int out_dtype, int64_t M, int64_t N, int64_t K, void* workspace,
                                  int64_t workspace_bytes, void* stream);

/* sglq_int8_blockwise_scaled_mm fused with the bias add of its caller
 * (python/sglang/srt/layers/quantization/int8_utils.py:25-32: the matmul rounded to the
 * output type, then `output + bias`): out = round(round(gemm) + bias), bias [N] in out_dtype
 * or NULL. */
int sglq_int8_blockwise_scaled_mm_bias(const void* a, int64_t lda, const void* b, int64_t ldb, const float* sfa,
                                       int64_t sfa_stride_m, int64_t sfa_stride_k, const float* sfb,
                                       int64_t sfb_stride_k, int64_t sfb_stride_n, const void* bias, void* out,
                                       int64_t ldo, int out_dtype, int64_t M, int64_t N, int64_t K, void* workspace,
                                       int64_t workspace_bytes, void* stream);

/* Replaces torch.ops.sgl_kernel.int8_scaled_mm
 * (sgl-kernel/csrc/gemm/int8_gemm_kernel.cu:663-747; schema common_extension.cc:101-104).
 * out = float(acc) * (scales_b[n] * scales_a[m]) + bias[n], acc exact int32.
 * bias may be NULL and otherwise has out_dtype. */
int sglq_int8_scaled_mm(const void* a, int64_t lda, const void* b, int64_t ldb, const float* scales_a,
                        const float* scales_b, const void* bias, void* out, int64_t ldo, int out_dtype,
                        int64_t M, int64_t N, int64_t K, void* workspace, int64_t workspace_bytes, void* stream);

/* The INT32 accumulators of sglq_int8_scaled_mm before its epilogue, written
 * as int32 [M, N] with row stride ldo.  No counterpart op in the reference;
 * it exists so the accumulators can be compared bit for bit. */
int sglq_int8_mm_i32(const void* a, int64_t lda, const void* b, int64_t ldb, int32_t* out, int64_t ldo,
                     int64_t M, int64_t N, int64_t K, void* workspace, int64_t workspace_bytes, void* stream);

/* Replaces torch.ops.sgl_kernel.fp8_scaled_mm
 * (sgl-kernel/csrc/gemm/fp8_gemm_kernel.cu:1071-1146; schema common_extension.cc:106-109).
 * out = scales_a[m] * (scales_b[n] * sum_k a*b) + bias[n], fp32 accumulation. */
int sglq_fp8_scaled_mm(const void* a, int64_t lda, const void* b, int64_t ldb, const float* scales_a,
                       const float* scales_b, const void* bias, void* out, int64_t ldo, int out_dtype,
                       int64_t M, int64_t N, int64_t K, void* workspace, int64_t workspace_bytes, void* stream);

/* Tuned kernel selections, the counterpart of the reference's per-(N, K) JSON tables for its
 * Triton GEMMs (get_w8a8_block_fp8_configs, python/sglang/srt/layers/quantization/fp8_kernel.py:
 * 738-776, files under layers/quantization/configs/): for GEMMs of `kind` with exactly these N and
 * K and m_lo <= M <= m_hi, use kernel `tile` (a code of sglq_debug_force_tile, 0 = by shape) and
 * split-K factor `splits` (0 = by shape) instead of the built-in heuristics.  The first matching
 * entry wins; a kernel that does not apply to a shape falls through to the next one that does, so
 * no entry can make a call fail.  Results do not depend on the table beyond the summation order
 * that each kernel has anyway.  The table is guarded by a reader/writer lock: entries may be
 * added or cleared while other threads launch GEMMs. */
#define SGLQ_KIND_FP8_BLOCK 0  /* sglq_fp8_blockwise_scaled_mm(_bias) */
#define SGLQ_KIND_FP8_ROWCOL 1 /* sglq_fp8_scaled_mm */
#define SGLQ_KIND_I8_ROWCOL 2  /* sglq_int8_scaled_mm */
#define SGLQ_KIND_I8_RAW 3     /* sglq_int8_mm_i32 */
#define SGLQ_KIND_I8_BLOCK 4   /* sglq_int8_blockwise_scaled_mm(_bias) */
int sglq_tuned_add(int kind, int64_t N, int64_t K, int64_t m_lo, int64_t m_hi, int tile, int splits);
int sglq_tuned_clear(void);

/* The sglq_debug_* hooks below are for tests and measurements, are not part of the operator
 * ABI, and act on the calling thread only (thread-local state): a thread that forces a kernel
 * cannot change what GEMM calls on other threads launch.
 *
 * Test hook without a reference counterpart: non-zero (default) makes the GEMMs
 * copy global memory straight into LDS with buffer loads, zero stages the same
 * bytes through registers.  Both must give identical results. */
void sglq_debug_set_direct_lds(int on);
/* Test hook: 0 = choose the GEMM kernel and tile by shape (default); 16 / 32 = the M <= 32
 * kernel whose blocks own 16 / 32 weight rows and all of K; 64 = the split-K decode kernel
 * (M <= 512) with 128 weight rows per block, 66 = with 64 weight rows per block (M > 32);
 * 68 / 69 = the full-K decode kernel on 64 x 64 / 32 x 64 tiles (32 < M <= 1024, K >= 512);
 * 128 = the 128x128 kernel; 256 = the plain 256x256 kernel; 258 = the pipelined 256x256
 * kernel (259 = its variant whose waves write their own outputs out and whose copies run on across tile
 * boundaries: block-scaled FP8 without bias or split-K); 130 = the same kernel with 128-row tiles; 192 / 224 / 257 = the pipelined 4x2-wave
 * kernel with tiles 192 / 224 / 256 wide; 193 = that kernel on 192 x 192 tiles (block-scaled FP8 without a bias).
 * A kernel that does not apply to the shape falls through to the next one that does. */
void sglq_debug_force_tile(int tile);
/* Test hook: > 0 fixes the split-K factor of the M <= 64 kernels (0 = by shape);
 * with sglq_debug_force_tile(64 / 128 / 256): 64 = always the M <= 64 kernel where it applies. */
void sglq_debug_force_splits(int splits);
/* Test hook: fixes the grouped GEMM's row tile height (32, 64, 128: the 128-row kernel; 256: the
 * pipelined 256-row kernel; 130: the pipelined kernel with 128-row tiles); anything else restores
 * the choice from the average group size. */
void sglq_debug_grouped_tile(int rows);
/* Test and measurement hook: name of the GEMM kernel that the calling thread's last GEMM
 * call launched ("" before the first call); the string is static. */
const char* sglq_debug_last_gemm_kernel(void);
/* 1 if the calling thread's last block-scaled FP8 GEMM ran on the kernels whose MFMAs apply the scales
 * (sglq_fp8_blockwise_scaled_mm_ue8m0 on the shapes they are built for), else 0. */
int sglq_debug_last_gemm_hw_scaled(void);

#ifdef __cplusplus
}
#endif
#endif /* SGLQ_H */
