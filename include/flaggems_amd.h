/*
 * flaggems_amd -- C ABI of the MI355X (gfx950) FP8 quantized-linear kernels.
 *
 * Every entry point takes raw device pointers, element counts, element strides and a
 * HIP stream.  None of them allocates, frees, synchronises or throws: the work is
 * enqueued on `stream` and the call returns 0 (FG_OK) or a negative fg_status; the
 * text of the last error on the calling thread is available from
 * fg_last_error_string().  The caller owns every buffer, selects the device
 * (hipSetDevice / torch device guard) and validates tensor-level preconditions.
 *
 * The reference library (FlagGems) has no C ABI: its native layer is C++ functions
 * taking at::Tensor, exposed through pybind11.  Each declaration below names the
 * reference interface it stands in for (paths relative to the reference checkout).
 */
#ifndef FLAGGEMS_AMD_H_
#define FLAGGEMS_AMD_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum fg_status {
  FG_OK = 0,
  FG_ERR_INVALID_ARG = -1, /* null pointer, negative size, bad enum, bad alignment */
  FG_ERR_UNSUPPORTED = -2, /* valid request the kernels do not implement */
  FG_ERR_WORKSPACE = -3,   /* workspace missing or smaller than fg_*_workspace_bytes */
  FG_ERR_LAUNCH = -4       /* hipLaunchKernel reported an error */
} fg_status;

typedef enum fg_dtype {
  FG_BF16 = 0,
  FG_F16 = 1,
  FG_F32 = 2,
  FG_FP8_E4M3FN = 3, /* OCP e4m3fn: max 448, no inf */
  FG_FP8_E5M2 = 4    /* OCP e5m2 */
} fg_dtype;

/* How the per-group scale is derived from the group's absolute maximum. */
typedef enum fg_scale_rule {
  FG_SCALE_MUL_INV = 0, /* scale = amax * inv_fp8_max   (torch references: amax * fp32(1/448)) */
  FG_SCALE_DIV = 1      /* scale = amax / fp8_max       (reference device kernels, MoE fallback) */
} fg_scale_rule;

/* How an element is divided by its scale. */
typedef enum fg_quotient_rule {
  FG_QUOT_RECIP_MUL = 0, /* x * (1.0f / scale), both IEEE-rounded (torch_act_quant) */
  FG_QUOT_DIV = 1        /* x / scale, IEEE-rounded division   (per_token_group_quant_fp8) */
} fg_quotient_rule;

/* Optional rounding of the scale up to a power of two (UE8M0-representable). */
typedef enum fg_pow2_rule {
  FG_POW2_NONE = 0,
  FG_POW2_BITS = 1, /* exponent + (mantissa != 0), 32-bit wrap-around as in fast_round_scale */
  FG_POW2_LOG2 = 2, /* exp2(ceil(log2(max(|s|, 1e-10)))) */
  FG_POW2_BITS_CLAMPED = 3 /* |s|: exponent + (mantissa != 0) held in [1, 254], as in _ceil_to_ue8m0
                              (tests/test_fp8_einsum.py:63-67): Inf and NaN become 2^127; with this rule an
                              infinite input under such a scale gives the NaN code, as a cast that is not
                              preceded by a clamp does */
} fg_pow2_rule;

/* Library version (major*10000 + minor*100 + patch) and last error text (thread-local). */
int fg_version(void);
const char* fg_last_error_string(void);

/*
 * Capture state of a stream: 0 when `stream` is not being captured into a HIP graph, otherwise a non-zero id of the
 * capture in progress.  No reference counterpart (the reference leaves graph capture to PyTorch); the Python binding
 * uses it to decide which workspace buffer a launch may be given: a buffer allocated inside a capture belongs to that
 * graph only, and a buffer a captured launch has seen must never be released.
 */
unsigned long long fg_stream_capture_id(void* stream);

/*
 * Per-token-group FP8 quantization: for every row r and every group g of `group_size`
 * consecutive columns,
 *     amax  = max |x[r, g*G : (g+1)*G]|          (NaN propagates)
 *     amax  = max(amax, amax_floor)
 *     scale = scale_rule(amax)  then  pow2_rule(scale)
 *     q     = cast_fp8(clamp(quotient_rule(x, scale), fp8_min, fp8_max))   round-to-nearest-even
 * writes q[r*q_row_stride + c] (1 byte each) and s[r*s_row_stride + g*s_col_stride].
 *
 * x_dtype in {FG_BF16, FG_F16, FG_F32}; q_dtype in {FG_FP8_E4M3FN, FG_FP8_E5M2};
 * cols % group_size == 0; strides are in elements.  rows*cols == 0 is a no-op.
 *
 * Stands in for: per_token_group_quant_fp8 (src/flag_gems/ops/per_token_group_quant_fp8.py:227-336,
 * kernels :34-216), act_quant_triton (src/flag_gems/fused/act_quant.py:111-174, kernel :45-108),
 * the native wrapper flag_gems::act_quant_triton (cpp/lib/act_quant.cpp:26-129) and the vLLM op
 * _C::per_token_group_fp8_quant (src/flag_gems/patches/patch_vllm_all.py:425-448), which can pass
 * the caller's output buffers straight through.
 */
int fg_group_quant_fp8(const void* x, int x_dtype, int64_t rows, int64_t cols, int64_t x_row_stride,
                       void* q, int q_dtype, int64_t q_row_stride,
                       float* s, int64_t s_row_stride, int64_t s_col_stride,
                       int64_t group_size, float amax_floor, float fp8_min, float fp8_max,
                       float inv_fp8_max, int scale_rule, int quotient_rule, int pow2_rule,
                       void* stream);

/*
 * Block quantizer for weights: one fp32 scale per block_rows x block_cols block of x [rows, cols] (unit column
 * stride); blocks that hang over the matrix edge see zeros there (the reference pads with zeros) and only the
 * rows x cols codes are written.  s: [ceil(rows/block_rows), ceil(cols/block_cols)] with both strides given.
 * The rule selectors, the floor and the fp8 limits mean what they mean in fg_group_quant_fp8.  Only 128 x 128
 * blocks are implemented (FG_ERR_UNSUPPORTED otherwise).
 * The reference keeps this quantizer in torch, next to the tests and benchmarks that need block-quantized
 * weights: per_block_cast_to_fp8 (tests/test_fp8_einsum.py:89-103, benchmark/test_fp8_einsum.py:82-96), which is
 * floor 1e-4, FG_SCALE_DIV, FG_QUOT_RECIP_MUL, limits -/+448 and FG_POW2_BITS_CLAMPED when use_ue8m0 else FG_POW2_NONE.
 */
int fg_block_quant_fp8(const void* x, int x_dtype, int64_t rows, int64_t cols, int64_t x_row_stride,
                       void* q, int q_dtype, int64_t q_row_stride,
                       float* s, int64_t s_row_stride, int64_t s_col_stride,
                       int64_t block_rows, int64_t block_cols, float amax_floor, float fp8_min, float fp8_max,
                       float inv_fp8_max, int scale_rule, int quotient_rule, int pow2_rule,
                       void* stream);

/*
 * Activation fused into the quantizer: the value quantized at [r, c] is
 *     act[r, c] = silu(x[r, c]) * x[r, c + up_offset],   silu(g) = g / (1 + exp(-g)) in fp32,
 * rounded once to x's type (what a separate activation kernel would have stored) and then quantized exactly as
 * fg_group_quant_fp8 quantizes a stored act: same codes and scales, bit for bit, as fg_silu_mul followed by
 * fg_group_quant_fp8, without writing and re-reading act.  x: [rows, >= up_offset + cols]; the gate half starts
 * at column 0, the up half at column up_offset (>= cols).  group_size 64 or 128; x, its rows and the up half
 * 16-byte aligned, q rows 8-byte aligned (FG_ERR_UNSUPPORTED otherwise).  Other arguments as fg_group_quant_fp8.
 *
 * The reference runs the two steps apart between the two expert GEMMs: _silu_and_mul_kernel
 * (src/flag_gems/fused/fused_moe.py:795-800; the operator silu_and_mul, src/flag_gems/fused/silu_and_mul.py:13-18)
 * into intermediate_cache2, then moe_kernel_quantize_input -> per_token_group_quant_fp8
 * (src/flag_gems/fused/fused_moe.py:2108-2122, 642-659).
 */
int fg_silu_mul_group_quant_fp8(const void* x, int x_dtype, int64_t rows, int64_t cols, int64_t x_row_stride,
                                int64_t up_offset, void* q, int q_dtype, int64_t q_row_stride,
                                float* s, int64_t s_row_stride, int64_t s_col_stride,
                                int64_t group_size, float amax_floor, float fp8_min, float fp8_max,
                                float inv_fp8_max, int scale_rule, int quotient_rule, int pow2_rule,
                                void* stream);

/*
 * The activation alone: out[r, c] = silu(x[r, c]) * x[r, c + up_offset] in x's type, out [rows, cols] with row
 * stride out_row_stride.  cols a multiple of 8; x, out, their rows and the up half 16-byte aligned.
 * Stands in for silu_and_mul_kernel (src/flag_gems/fused/silu_and_mul.py:13-18) on the two halves of one tensor.
 */
int fg_silu_mul(const void* x, int x_dtype, int64_t rows, int64_t cols, int64_t x_row_stride, int64_t up_offset,
                void* out, int64_t out_row_stride, void* stream);

/*
 * Sum over the top-k slots of every token, the last step of an expert layer:
 *     out[t, h] = cast( sum_{k < top_k} in[t, k, h] )   (fp32 running sum in slot order, one rounding)
 * in: [tokens, top_k, hidden] of dtype FG_BF16 / FG_F16 / FG_F32 with element strides in_token_stride and
 * in_slot_stride (unit stride along hidden); out: [tokens, hidden] of the same dtype, rows out_token_stride apart.
 * hidden a multiple of 8; in, out and every row 16-byte aligned, else FG_ERR_UNSUPPORTED.
 * Stands in for moe_sum (src/flag_gems/fused/moe_sum.py:34-90), which the reference's expert layer calls on the
 * scattered, weighted results of its second GEMM (src/flag_gems/fused/fused_moe.py:2177-2182).
 */
int fg_moe_sum(const void* in, int dtype, int64_t tokens, int64_t top_k, int64_t hidden, int64_t in_token_stride,
               int64_t in_slot_stride, void* out, int64_t out_token_stride, void* stream);

/*
 * Routing by softmax: probabilities p = exp(x - max) / (sum + 1e-8) over the experts of a token (fp32), then topk rounds
 * of "largest remaining probability, the lower expert on ties".  gating: [tokens, experts] of FG_BF16 / FG_F16 / FG_F32,
 * rows row_stride elements apart; topk_weights: fp32 [tokens, topk], in descending order, divided by
 * (their sum + 1e-8) when renormalize != 0; topk_indices: [tokens, topk] of 4- or 8-byte integers (index_bytes);
 * token_expert_indices: int32 [tokens, topk] = k * tokens + t, or NULL.  topk <= 32 and <= experts <= 1024.
 * Stands in for topk_softmax (src/flag_gems/fused/topk_softmax.py:85-137, kernel :24-82), the vLLM operator
 * _moe_C::topk_softmax (src/flag_gems/patches/patch_vllm_all.py:348-353).
 */
int fg_topk_softmax(const void* gating, int dtype, int64_t tokens, int64_t experts, int64_t row_stride,
                    int64_t topk, int renormalize, float* topk_weights, void* topk_indices, int index_bytes,
                    int* token_expert_indices, void* stream);

/*
 * Group-limited routing (DeepSeek): with s = scores (scoring_func 0) or sigmoid(scores) rounded to the scores' type
 * (scoring_func 1) and sb = s + bias rounded to that type,
 *   group score  = the sum of the two largest sb of the group's experts/n_group consecutive experts (the largest counted
 *                  twice when it occurs twice), rounded to the scores' type; NaN and +inf count as -inf;
 *   groups       = the topk_group largest group scores, ties to the lower group;
 *   experts      = topk rounds of "largest remaining sb among the experts of those groups, the lower expert on ties";
 *   weights      = s of the selected experts * routed_scaling_factor, over (their sum + 1e-20) when renormalize != 0.
 * When no group score is above -inf the result is experts 0 .. topk-1 with weight 1 / topk each.
 * scores: [tokens, experts] (score_stride elements between rows), bias: [experts], both FG_BF16 / FG_F16 / FG_F32;
 * topk_values fp32 and topk_ids int32: [tokens, topk], out_stride elements between rows.
 * n_group <= 32 divides experts <= 1024; topk <= 32.
 * Stands in for grouped_topk (src/flag_gems/fused/grouped_topk.py:256-355, kernels :25-78 and :81-253), the vLLM
 * operator _moe_C::grouped_topk (src/flag_gems/patches/patch_vllm_all.py:324-345).
 */
int fg_grouped_topk(const void* scores, int dtype, int64_t tokens, int64_t experts, int64_t score_stride,
                    const void* bias, int64_t n_group, int64_t topk_group, int64_t topk, int renormalize,
                    float routed_scaling_factor, int scoring_func, float* topk_values, int* topk_ids,
                    int64_t out_stride, void* stream);

/*
 * Routing table of an expert layer for fg_grouped_block_fp8_gemm: the routed slots sorted by expert.
 *     key(s) = local expert of slot s, or num_experts if it has none
 *     sorted_slots = the slot numbers 0 .. n_slots-1 in ascending order of key, ties in slot order (int32 [n_slots])
 *     offs[e]      = number of slots with key <= e (int32 [num_experts]: the cumulative ends of the experts' segments)
 * topk_ids: [n_slots] integers of id_bytes (4 or 8) bytes, slot t * top_k + j = the j-th expert of token t.
 * expert_map (may be NULL): [map_len] integers of map_bytes (4 or 8) bytes, global expert -> local expert or -1; an id
 * outside [0, map_len), a map entry outside [0, num_experts) and, without a map, an id outside [0, num_experts) all
 * mean "no local expert": such slots sort behind offs[num_experts - 1].  One block, no workspace, nothing synchronises;
 * at most 960 experts and 65536 slots (FG_ERR_UNSUPPORTED beyond).
 * Stands in for the sorting stages of moe_align_block_size (src/flag_gems/fused/moe_align_block_size.py:405-519, the
 * expert_map convention of :817-818) without the padding to a block multiple, which the grouped GEMM here does not need.
 */
int fg_moe_sort_slots(const void* topk_ids, int id_bytes, int64_t n_slots, int64_t num_experts, const void* expert_map,
                      int map_bytes, int64_t map_len, int32_t* sorted_slots, int32_t* offs, void* stream);

/*
 * The padded routing table of the reference's moe_align_block_size (src/flag_gems/fused/moe_align_block_size.py:771-819,
 * kernels :405-519), same layout and meaning:
 *     sorted_ids [sorted_cap]   expert e's slots, in slot order, start at entry (sum over e' < e of ceil(count[e'] /
 *                               block_size)) * block_size; every entry that holds no slot is n_slots (the padding value)
 *     expert_ids [expert_ids_cap]  the expert of every block of block_size entries, -1 for blocks past the padded length
 *     num_tokens_post_pad [1]   the padded length, sum over e of ceil(count[e] / block_size) * block_size
 * topk_ids: [n_slots] integers of id_bytes (4 or 8) bytes in [0, num_experts); ids outside that range take no entry.
 * sorted_cap >= n_slots + num_experts * (block_size - 1) and expert_ids_cap >= ceil(that / block_size), the sizes the
 * reference allocates (FG_ERR_INVALID_ARG otherwise).  The reference leaves the order inside an expert's run to its
 * atomics; here it is the slot order.  expert_map is applied by the caller to expert_ids afterwards, as in the reference
 * (:817-818).  One block, no workspace; at most 960 experts and 65536 slots (FG_ERR_UNSUPPORTED beyond).
 */
int fg_moe_align_block_size(const void* topk_ids, int id_bytes, int64_t n_slots, int64_t num_experts, int64_t block_size,
                            int32_t* sorted_ids, int64_t sorted_cap, int32_t* expert_ids, int64_t expert_ids_cap,
                            int32_t* num_tokens_post_pad, void* stream);

/*
 * RMSNorm (optionally preceded by the residual add) fused into the quantizer: every row of x [rows, cols] is
 * normalised, multiplied by weight [cols] (x's type), rounded to x's type as a separate norm kernel would have
 * stored it, and quantized exactly as fg_group_quant_fp8 quantizes that stored tensor (same codes and scales, bit
 * for bit), without writing and re-reading it.
 *   residual == NULL (src/flag_gems/ops/rms_norm.py:54-66):
 *       var = sum(x^2) / cols, rrms = 1 / sqrt(var + eps), y = T(T(x * rrms) * weight), T = rounding to x's type;
 *   residual != NULL, [rows, cols] of x's type, updated in place
 *   (src/flag_gems/fused/fused_add_rms_norm.py:92-118, the kernel the reference uses for rows over 4096 elements;
 *   its kernel for shorter rows, lines 42-56, rounds differently and is not followed):
 *       t = x + residual in fp32, residual <- T(t), var = sum(t^2) / cols over the unrounded t,
 *       y = T(T(t) * rrms * weight).
 * All of it in individually rounded fp32 operations; the sum of squares runs per thread over the 8-element chunks
 * t, t + 256, ... of the row in order, then over lanes at distances 1, 2, 4, 8, 16, 32, then over the four
 * wavefronts in order (the reference leaves the order to its compiler).
 * y: NULL, or [rows, cols] that receives the normalised rows (may be x itself: the reference's fused operator
 * writes into its input).  q and s: both NULL to normalise only, else as in fg_group_quant_fp8 with group_size
 * 8, 16, 32, 64, 128, 256 or 512.  cols a multiple of 8 and at most 16384; x, residual, weight, y and their rows
 * 16-byte aligned, q rows 8-byte aligned (FG_ERR_UNSUPPORTED otherwise).
 * The reference runs the steps apart: rms_norm or fused_add_rms_norm, then the quantizer inside the linear
 * layer (src/flag_gems/ops/per_token_group_quant_fp8.py:203-297).
 */
int fg_rms_norm_group_quant_fp8(const void* x, int x_dtype, int64_t rows, int64_t cols, int64_t x_row_stride,
                                void* residual, int64_t residual_row_stride, const void* weight, float eps,
                                void* y, int64_t y_row_stride,
                                void* q, int q_dtype, int64_t q_row_stride,
                                float* s, int64_t s_row_stride, int64_t s_col_stride,
                                int64_t group_size, float amax_floor, float fp8_min, float fp8_max,
                                float inv_fp8_max, int scale_rule, int quotient_rule, int pow2_rule,
                                void* stream);

/*
 * Inverse rotary embedding fused into the group quantizer: the producer of the quantized activations of
 * DeepSeek-V4's grouped output projection (the "bhr,hdr->bhd" einsum that fg_batched_block_fp8_gemm serves).
 *   o: [tokens, heads, head_dim] of FG_BF16 / FG_F16 / FG_F32, unit stride along head_dim, element strides
 *      o_stride_token and o_stride_head; heads = groups * heads_per_group.
 *   positions: [tokens], int32 or int64 (position_bytes 4 or 8); cos_sin_cache: fp32 [cache_rows, >= rope_dim]
 *      with rows cache_stride apart, cos in the first rope_dim / 2 columns and sin in the next rope_dim / 2.
 *      A position outside [0, cache_rows) reads the nearest row (the reference reads out of bounds there).
 *   The last rope_dim values of every head are rotated back in fp32, pairs interleaved:
 *      x[2i]' = x[2i] cos_i + x[2i+1] sin_i,   x[2i+1]' = x[2i+1] cos_i - x[2i] sin_i   (each operation rounded),
 *   the first head_dim - rope_dim pass through, and every group_size values are quantized without an intermediate
 *   rounding: amax = max(max|x|, eps), scale = amax * fp32(1/448), codes = e4m3fn(clamp(x / scale, -448, 448)).
 *   q: e4m3fn, value (t, h, j) at q[(h / heads_per_group) * q_stride_group + t * q_stride_token
 *      + (h % heads_per_group) * head_dim + j]  (the reference allocates [groups, tokens, heads_per_group * head_dim]
 *      and returns its transpose, so that every group is a contiguous [tokens, K] operand).
 *   scales, pack_ue8m0 == 0: fp32, group c of head h of token t at
 *      scales[(h / heads_per_group) * scale_stride_group + t + ((h % heads_per_group) * chunks + c) * scale_stride_k],
 *      chunks = head_dim / group_size: tokens have unit stride (column-major per group).
 *   scales, pack_ue8m0 != 0: the scale is rounded up to a power of two, exp2(ceil(log2(max(scale, 1e-10)))), and one
 *      int32 per head holds the exponent fields of its (at most four) groups, group c in byte c, at
 *      scales[(h / heads_per_group) * scale_stride_group + t + (h % heads_per_group) * scale_stride_k].
 *   Rows tokens <= t < padded_tokens of the scale columns are set to zero (the reference pads the token count to a
 *   multiple of four); q has no such rows.
 * group_size 64, 128, 256 or 512 with rope_dim <= group_size, both multiples of 8; heads of o 16-byte aligned,
 * rows of q 8-byte aligned (FG_ERR_UNSUPPORTED otherwise).
 * Stands in for fused_inv_rope_fp8_quant (src/flag_gems/fused/fused_inv_rope_fp8_quant.py:164-257, kernel :38-161).
 */
int fg_inv_rope_group_quant_fp8(const void* o, int o_dtype, int64_t tokens, int64_t heads, int64_t head_dim,
                                int64_t o_stride_token, int64_t o_stride_head,
                                const void* positions, int position_bytes,
                                const float* cos_sin_cache, int64_t cache_rows, int64_t cache_stride,
                                int64_t heads_per_group, int64_t rope_dim, int64_t group_size, float eps,
                                void* q, int64_t q_stride_group, int64_t q_stride_token,
                                void* scales, int64_t scale_stride_group, int64_t scale_stride_k,
                                int64_t padded_tokens, int pack_ue8m0, void* stream);

/*
 * act_quant with the reference's fixed rules (bf16 in, e4m3fn out, floor 1e-4,
 * scale = amax * fp32(1/448), reciprocal-multiply quotient, power-of-two scale when
 * round_scale != 0), contiguous [rows, cols] input and outputs.
 * Stands in for flag_gems::act_quant_triton (cpp/lib/act_quant.cpp:26-129,
 * cpp/include/flag_gems/operators.h:59-61).
 */
int fg_act_quant_bf16(const void* x, void* y, float* s, int64_t rows, int64_t cols,
                      int64_t block_size, int round_scale, void* stream);

/*
 * Block-scaled FP8 GEMM:
 *     C[m, n] = sum_kb ( sum_{k in kb} A[m,k] * B[n,k] ) * As[m, kb] * Bs[n / block_n, kb]
 * A: e4m3fn [M, K], row stride lda, unit column stride.  B: e4m3fn [N, K], row stride ldb, unit
 * column stride.  As: fp32 [M, ceil(K/block_k)] with both strides given.  Bs: fp32
 * [ceil(N/block_n), ceil(K/block_k)] with both strides given.  C: [M, N] row stride ldc,
 * c_dtype in {FG_BF16, FG_F16, FG_F32}.  Products are accumulated in fp32 per K-block, scaled,
 * and accumulated in fp32 across K-blocks; the result is rounded once to c_dtype.
 * block_n == block_k == 128 takes the kernels built around the 16x16x128 matrix instruction.  Other block sizes with
 * block_k a multiple of 32 and block_n of 16 (64 x 64, 128 x 64, 32 x 96 ...; K a multiple of 16, 16-byte aligned rows)
 * take a tile kernel on the 16x16x32 instruction, about four times slower; everything else a plain fp32 tile kernel,
 * about fifty times slower.  (Callers with multiples of 128 do better to write the scales out per 128 x 128 block and
 * call with 128, which gives the same result.)
 * `workspace` holds split-K partial sums and, for long GEMMs, a transposed copy of As.
 * fg_block_fp8_gemm_workspace_bytes(M, N, K) says how much the kernels can use for the shape (0: none).
 * For M <= 32 that much is required when it is not 0 (FG_ERR_WORKSPACE otherwise); for larger M it is
 * optional: with less, or with a null pointer, K is never split between blocks (slower for shapes whose tile
 * count leaves much of the GPU idle; same results to within fp32 summation order; M in 33..64 then needs what
 * the decode kernels ask for, which is less) and row-major As is read as it is
 * (10-20 % slower for M in the thousands; identical results).  As with unit row stride (column-major,
 * as_row_stride == 1) is read in place in any case.  The caller zero-fills the first
 * FG_WORKSPACE_COUNTER_BYTES bytes once; every launch leaves them zero.  16-byte aligned.  Launches that
 * may run concurrently must not share a workspace.
 *
 * Stands in for: w8a8_block_fp8_matmul (src/flag_gems/ops/w8a8_block_fp8_matmul.py:173-232,
 * kernel :51-122), fp8_matmul (src/flag_gems/ops/fp8_matmul.py:137-205, kernel :58-134), the native
 * wrappers fp8_matmul / fp8_matmul_direct (cpp/lib/fp8_matmul.cpp:25-102,
 * cpp/lib/fp8_matmul_direct.cpp:25-180) and the block-wise branch of cutlass_scaled_mm
 * (src/flag_gems/fused/cutlass_scaled_mm.py:87-194).
 */
int fg_block_fp8_gemm(const void* A, int64_t lda, const void* B, int64_t ldb,
                      const float* As, int64_t as_row_stride, int64_t as_col_stride,
                      const float* Bs, int64_t bs_row_stride, int64_t bs_col_stride,
                      void* C, int64_t ldc, int c_dtype,
                      int64_t M, int64_t N, int64_t K, int64_t block_n, int64_t block_k,
                      void* workspace, size_t workspace_bytes, void* stream);

#define FG_WORKSPACE_COUNTER_BYTES 16384
size_t fg_block_fp8_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K);

/*
 * fg_block_fp8_gemm for scales the caller knows to be powers of two (fp32 values with a zero mantissa: E8M0 scales
 * widened to fp32, or the ue8m0 rounding of the quantizers).  Same arguments, same workspace rules, same result up
 * to the order of fp32 roundings: where the persistent kernel takes the problem (M > 128, K a multiple of 128,
 * 16-byte aligned rows, bf16 result) the scales go into the block-scaled form of the MFMA instruction as E8M0
 * exponents and the matrix pipe accumulates the scaled K-blocks itself, instead of one fp32 multiply-add per
 * result element and K-block; every other shape runs exactly the kernels of fg_block_fp8_gemm.  A scale that is not
 * a power of two is used as if its mantissa were zero: the caller's guarantee is not checked.
 *
 * Stands in for fp8_matmul with scale_dtype = float8_e8m0fnu (src/flag_gems/ops/fp8_matmul.py:137-205: the scales
 * arrive as E8M0 and are widened at :165-167) and for block-fp8 GEMMs whose operands were quantized with power-of-two
 * scales (per_token_cast_to_fp8 / per_block_cast_to_fp8 with use_ue8m0, tests/test_fp8_einsum.py:63-103;
 * act_quant with scale_fmt "ue8m0", src/flag_gems/fused/act_quant.py:111-174).
 */
int fg_block_fp8_gemm_pow2_scales(const void* A, int64_t lda, const void* B, int64_t ldb,
                                  const float* As, int64_t as_row_stride, int64_t as_col_stride,
                                  const float* Bs, int64_t bs_row_stride, int64_t bs_col_stride,
                                  void* C, int64_t ldc, int c_dtype,
                                  int64_t M, int64_t N, int64_t K, int64_t block_n, int64_t block_k,
                                  void* workspace, size_t workspace_bytes, void* stream);

/*
 * fg_block_fp8_gemm without the workspace arguments, for callers that cannot allocate device memory: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference (whose
 * wrappers allocate through torch).  The workspace is an array of FG_NOALLOC_SCRATCH_BYTES built into the library's
 * device code, one copy per GPU, held until the process ends; the call allocates nothing and frees nothing.  Same
 * kernels and same results as fg_block_fp8_gemm given a workspace of that size.  A shape for which
 * fg_block_fp8_gemm_workspace_bytes(M, N, K) exceeds FG_NOALLOC_SCRATCH_BYTES is refused with FG_ERR_WORKSPACE (use
 * fg_block_fp8_gemm with a workspace of the caller's).  All calls on one GPU share that GPU's array: calls that may
 * overlap on one GPU (two streams, two threads) race on the counters and partial sums and must be serialised by the
 * caller.  The first call on a device looks the array's address up; nothing but the GEMM's own kernels is ever
 * enqueued, so a call may be recorded into a graph like any other launch.  The counter area starts as zeros (a device
 * array without an initialiser is zero when the library's code is loaded) and every launch leaves it zero.
 */
#define FG_NOALLOC_SCRATCH_BYTES (32u << 20)
int fg_block_fp8_gemm_noalloc(const void* A, int64_t lda, const void* B, int64_t ldb,
                              const float* As, int64_t as_row_stride, int64_t as_col_stride,
                              const float* Bs, int64_t bs_row_stride, int64_t bs_col_stride,
                              void* C, int64_t ldc, int c_dtype,
                              int64_t M, int64_t N, int64_t K, int64_t block_n, int64_t block_k, void* stream);

/*
 * Batched block-scaled FP8 GEMM: `batch` independent problems of fg_block_fp8_gemm with the same M, N, K and
 * strides.  Matrix i of each operand starts i * <its batch stride> after matrix 0 (bytes for A and B, floats for
 * the scales, elements of c_dtype for C); row strides are free, so a [b, h, r] activation with h as the batch
 * takes lda = h * r and a_batch_stride = r.  Matrices too small to fill the GPU on their own go out in one launch
 * (the batch entry in the grid), larger ones one after the other on `stream`; the results are those of `batch`
 * calls of fg_block_fp8_gemm (the same bits, except that where K is split over blocks -- up to 128 rows, and beyond
 * while the whole batch has no more 128 x 128 tiles than the GPU has compute units -- the batch is split into fewer
 * ranges than a lone matrix, which changes the order of the fp32 partial sums), and the workspace rules are that
 * entry point's (one workspace serves the whole batch; fg_batched_block_fp8_gemm_workspace_bytes(batch, M, N, K) is
 * what the kernels can use: every entry keeps its own partial sums, and with less than that the call takes a slower
 * kernel instead of failing).
 *
 * Stands in for w8a8_block_fp8_bmm (src/flag_gems/runtime/backend/_nvidia/hopper/ops/w8a8_block_fp8_bmm.py:629-779)
 * and, through it, fp8_einsum("bhr,hdr->bhd") (.../hopper/ops/fp8_einsum.py:22-68).
 */
size_t fg_batched_block_fp8_gemm_workspace_bytes(int64_t batch, int64_t M, int64_t N, int64_t K);
int fg_batched_block_fp8_gemm(const void* A, int64_t lda, int64_t a_batch_stride,
                              const void* B, int64_t ldb, int64_t b_batch_stride,
                              const float* As, int64_t as_row_stride, int64_t as_col_stride, int64_t as_batch_stride,
                              const float* Bs, int64_t bs_row_stride, int64_t bs_col_stride, int64_t bs_batch_stride,
                              void* C, int64_t ldc, int64_t c_batch_stride, int c_dtype,
                              int64_t batch, int64_t M, int64_t N, int64_t K, int64_t block_n, int64_t block_k,
                              void* workspace, size_t workspace_bytes, void* stream);

/*
 * Grouped block-scaled FP8 GEMM (mixture-of-experts layers with the tokens sorted by expert):
 *     C[m, n] = sum_kb ( sum_{k in kb} A[m,k] * B[e(m)][n,k] ) * As[m, kb] * Bs[e(m)][n / block_n, kb]
 * where row m belongs to group e(m): group e owns rows [group_ends[e-1], group_ends[e]) with
 * group_ends[-1] = 0.  group_ends is a DEVICE table of n_groups cumulative int32 row ends, read by the
 * kernel (the host never waits for it); empty groups are allowed; rows at or past the last end are not
 * written; ends are forced into ascending order and into [0, M] before use.
 * A: e4m3fn [M, K] (all groups' rows), As: fp32 [M, K/block_k], C: bf16 [M, N], as in fg_block_fp8_gemm.
 * B: e4m3fn [n_groups, N, K]: matrix e starts b_group_stride bytes after matrix e-1, rows ldb apart.
 * Bs: fp32 [n_groups, ceil(N/block_n), K/block_k]: matrix e starts bs_group_stride floats after matrix e-1.
 * K must be a positive multiple of 128; A, B 16-byte aligned with lda, ldb, b_group_stride multiples of 16;
 * C 16-byte aligned with ldc a multiple of 8; c_dtype FG_BF16 or FG_F16 (FG_ERR_UNSUPPORTED otherwise: there is no
 * slower general path behind this entry point).
 * `workspace` (optional, 16-byte aligned, fg_grouped_block_fp8_gemm_workspace_bytes(M, N, K) bytes, first
 * FG_WORKSPACE_COUNTER_BYTES zero-filled once) lets row-major As be read from a transposed copy and, when the
 * groups average at most 128 rows (M <= 128 * n_groups), lets tiles be cut along K so that few tiles fill the GPU
 * (64 MB of partial sums; the sums are added in a fixed order, but not in the order of the call without workspace).
 * row_index (optional DEVICE table of M int32): the kernel gathers its rows itself -- row m of the sorted order
 * (the order of group_ends and of C) is row row_index[m] / index_div of A and As, which then have a_rows rows
 * (entries are forced into [0, a_rows); a_rows * lda must fit 32 bits).  This is how the reference's MoE kernel
 * reads its tokens (rows = sorted_token_ids // top_k, src/flag_gems/fused/fused_moe.py:1111): the caller need not
 * materialise the activations in expert order.  NULL: A and As are already in sorted order (a_rows ignored).
 * index_div == 0 (with c_rows > 0): A and As are in sorted order as well and row_index only addresses the scattered
 * result -- the second GEMM of an expert layer whose intermediate rows stayed in expert order.
 * c_rows > 0 (needs row_index): the results are scattered as well -- C has c_rows rows, the result of sorted row m
 * goes to row row_index[m], and entries outside [0, c_rows) are padding that stores nothing (the reference's
 * sorted_token_ids pads every expert to a multiple of its block with the value numel,
 * src/flag_gems/fused/moe_align_block_size.py:404-517).  row_weight (optional DEVICE fp32 [c_rows], with c_rows > 0):
 * the fp32 sums of sorted row m are multiplied by row_weight[row_index[m]] before the cast to bf16.  This is the
 * epilogue of the reference's MoE kernel (offs_token, token_mask, MUL_ROUTED_WEIGHT:
 * src/flag_gems/fused/fused_moe.py:1484-1509).  c_rows = 0: C has M rows in sorted order; row_weight must be NULL.
 *
 * Stands in for the block-wise fp8 branch of fused_moe_kernel (src/flag_gems/fused/fused_moe.py:1378-1450)
 * applied to rows already gathered in expert order, with the group table of aten::_scaled_grouped_mm
 * (`offs`: cumulative int32 ends, src/flag_gems/ops/scaled_grouped_mm.py:111-114,275-287).  Per group the
 * arithmetic is that of w8a8_block_fp8_matmul (src/flag_gems/ops/w8a8_block_fp8_matmul.py:51-122), which is
 * how the reference's own MoE test states it (tests/test_fused_experts_impl.py:604-662).
 */
int fg_grouped_block_fp8_gemm(const void* A, int64_t lda,
                              const void* B, int64_t ldb, int64_t b_group_stride,
                              const float* As, int64_t as_row_stride, int64_t as_col_stride,
                              const float* Bs, int64_t bs_row_stride, int64_t bs_col_stride, int64_t bs_group_stride,
                              const int32_t* group_ends, int64_t n_groups,
                              const int32_t* row_index, int64_t index_div, int64_t a_rows,
                              int64_t c_rows, const float* row_weight,
                              void* C, int64_t ldc, int c_dtype,
                              int64_t M, int64_t N, int64_t K, int64_t block_n, int64_t block_k,
                              void* workspace, size_t workspace_bytes, void* stream);
size_t fg_grouped_block_fp8_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K);

/*
 * Per-tensor / per-token x per-channel scaled FP8 GEMM with optional bias:
 *     C[m, n] = cast( (sum_k A[m,k] * B[n,k]) * a_scale[m or 0] * b_scale[n or 0] ) (+ bias[n])
 * The bias is added after the cast, in c_dtype, as the reference does.  A: e4m3fn [M, K] row stride
 * lda; B: e4m3fn given as N rows of K contiguous bytes with row stride ldb (that is the reference's
 * column-major [K, N] operand: ldb = b.stride(1)).  a_scale has M entries when a_scale_per_row != 0,
 * else 1; b_scale has N entries when b_scale_per_col != 0, else 1.  bias may be null; bias_dtype in
 * {FG_BF16, FG_F16, FG_F32}.  c_dtype in {FG_BF16, FG_F16, FG_F32, FG_FP8_E4M3FN}.
 *
 * Stands in for: cutlass_scaled_mm per-tensor/per-token path
 * (src/flag_gems/fused/cutlass_scaled_mm.py:198-344, 475-526), reached from aten::_scaled_mm
 * (src/flag_gems/ops/scaled_mm.py:333-452) and the vLLM op _C::cutlass_scaled_mm
 * (src/flag_gems/patches/patch_vllm_all.py:451-459).
 */
int fg_scaled_fp8_gemm(const void* A, int64_t lda, const void* B, int64_t ldb,
                       const float* a_scale, int a_scale_per_row,
                       const float* b_scale, int b_scale_per_col,
                       const void* bias, int bias_dtype,
                       void* C, int64_t ldc, int c_dtype,
                       int64_t M, int64_t N, int64_t K,
                       void* workspace, size_t workspace_bytes, void* stream);

size_t fg_scaled_fp8_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K);

/*
 * The same operator for operands that are not quantized (aten::_scaled_mm on bf16, fp16 or fp32 matrices):
 *     C[m, n] = cast( (sum_k A[m,k] * B[n,k]) * a_scale[m or 0] * b_scale[n or 0] + bias[n] )
 * with the sum, the scaling and the bias in fp32 and one rounding to c_dtype at the end (here the bias is added
 * BEFORE the rounding: that is what the reference's generic kernel does, unlike its cutlass path above).
 * A: [M, K] rows lda elements apart; B: N rows of K contiguous elements, ldb apart (the column-major [K, N] operand);
 * both of ab_dtype in {FG_BF16, FG_F16, FG_F32}.  c_dtype and bias_dtype in {FG_BF16, FG_F16, FG_F32}; bias may be
 * null.  K a multiple of 8 (bf16, fp16) or 4 (fp32) and operand rows 16-byte aligned, else FG_ERR_UNSUPPORTED (the
 * host pads or copies).  No workspace.
 * Stands in for scaled_mm_kernel (src/flag_gems/ops/scaled_mm.py:37-133, launched from :365-422).
 */
int fg_scaled_gemm(const void* A, int64_t lda, const void* B, int64_t ldb, int ab_dtype,
                   const float* a_scale, int a_scale_per_row,
                   const float* b_scale, int b_scale_per_col,
                   const void* bias, int bias_dtype,
                   void* C, int64_t ldc, int c_dtype,
                   int64_t M, int64_t N, int64_t K, void* stream);

/*
 * The same with int8 operands: C[m, n] = float(sum_k A[m,k] * B[n,k] in int32) * a_scale[m or 0] * b_scale[n or 0],
 * rounded to c_dtype (FG_BF16, FG_F16 or FG_F32), then + bias[n] in c_dtype.  A: int8 [M, K] rows lda apart,
 * B: int8 [N, K] rows ldb apart (the column-major [K, N] operand of the reference).  The same kernels and dispatch
 * as fg_scaled_fp8_gemm, with the int8 matrix instruction; `workspace` as for fg_block_fp8_gemm
 * (fg_scaled_int8_gemm_workspace_bytes(M, N, K); required for M <= 64 when that is not 0).  Where K is split between
 * wavefronts or blocks the int32 partial sums are added as integers: the result is float(exact sum) * scales
 * whatever the split.
 * Stands in for the int8 branch of cutlass_scaled_mm (src/flag_gems/fused/cutlass_scaled_mm.py:198-344 with an
 * int32 accumulator, dispatch :394-402).
 */
int fg_scaled_int8_gemm(const void* A, int64_t lda, const void* B, int64_t ldb,
                        const float* a_scale, int a_scale_per_row,
                        const float* b_scale, int b_scale_per_col,
                        const void* bias, int bias_dtype,
                        void* C, int64_t ldc, int c_dtype,
                        int64_t M, int64_t N, int64_t K,
                        void* workspace, size_t workspace_bytes, void* stream);
size_t fg_scaled_int8_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K);

#ifdef __cplusplus
}
#endif
#endif /* FLAGGEMS_AMD_H_ */
