/*
 * fp8k - C ABI of the MI355X (gfx950) W8A8 FP8 linear kernels.
 *
 * Every entry point takes raw device pointers, int64 sizes / element strides, small enums
 * and a hipStream_t passed as void*.  Nothing here allocates, frees, synchronises or reads
 * device memory from the host, so all calls are legal under HIP graph capture.  A call
 * returns 0 on success; otherwise a non-zero fp8k_status and a message retrievable with
 * fp8k_last_error() (thread-local).  Arguments are validated on the host before any launch.
 *
 * Each function cites the reference interface it stands in for (paths relative to the
 * SGLang checkout).
 */
#ifndef FP8K_H
#define FP8K_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  FP8K_OK = 0,
  FP8K_ERR_INVALID = 1,     /* bad argument: shape, stride, dtype, alignment, null pointer */
  FP8K_ERR_UNSUPPORTED = 2, /* valid in the reference API but not built here */
  FP8K_ERR_LAUNCH = 3,      /* HIP runtime error at launch */
  FP8K_ERR_WORKSPACE = 4    /* workspace missing or too small */
} fp8k_status;

typedef enum { FP8K_F32 = 0, FP8K_F16 = 1, FP8K_BF16 = 2 } fp8k_dtype;

/* activation of fp8k_activation */
typedef enum { FP8K_ACT_SILU = 0, FP8K_ACT_GELU = 1, FP8K_ACT_RELU2 = 2 } fp8k_activation_kind;

typedef enum {
  FP8K_SCALE_F32 = 0,         /* one float per group, addressed by (stride_m, stride_g) */
  FP8K_SCALE_UE8M0_PACKED = 1, /* int32 words, 4 exponent bytes each, word (g/4) byte (g%4) */
  FP8K_SCALE_UE8M0_F32 = 2     /* the power of two 2^ceil(log2 scale) stored as a float, addressed like FP8K_SCALE_F32
                                  (fp8k_group_quant_masked only) */
} fp8k_scale_kind;

/* Message of the last failed call on this thread ("" if none). */
const char* fp8k_last_error(void);
/* ABI version: bumped when a signature changes. */
int fp8k_abi_version(void);

/*
 * Per-token-group FP8 (OCP e4m3fn) quantisation.
 * Replaces torch.ops.sgl_kernel.sgl_per_token_group_quant_8bit
 *   (sgl-kernel/python/sgl_kernel/gemm.py:100-136, sgl-kernel/csrc/gemm/per_token_group_quant_8bit.cu:116-217);
 *   arithmetic of native_per_token_group_quant_fp8 (python/sglang/test/test_block_fp8.py:23-48).
 * x [M,K] contiguous of in_dtype; q [M,K] bytes; group_size in {16,32,64,128,256,512}, K % group_size == 0.
 * scale_kind F32: s[m*s_stride_m + g*s_stride_g] (elements), any of row-major / column-major /
 *   column-major padded.  UE8M0_PACKED: int32 word at s[(g/4)*s_stride_g + m*s_stride_m], byte g%4;
 *   every word of a touched row is written whole (unused bytes zero).
 * eps: amax floor.  For bf16 input it is rounded to bf16 first, as the torch-native path does.
 * fp8_min/fp8_max must be -448/448.
 */
int fp8k_group_quant(const void* x, void* q, void* s, int64_t M, int64_t K, int64_t group_size, float eps,
                     float fp8_min, float fp8_max, int in_dtype, int64_t s_stride_m, int64_t s_stride_g,
                     int scale_kind, void* stream);

/*
 * silu_and_mul fused into the per-token-group quantisation: quantises T(T(silu(x[m,c])) * x[m,K+c]) for c < K.
 * Replaces torch.ops.sgl_kernel.sgl_per_token_group_quant_8bit_v2 with fuse_silu_and_mul = true and no masked_m
 *   (sgl-kernel/python/sgl_kernel/gemm.py:100-136, sgl-kernel/csrc/gemm/per_token_group_quant_8bit_v2.cu:336-341;
 *   wrapper python/sglang/srt/layers/quantization/fp8_kernel.py:481-531).
 * x [M,2K] contiguous of in_dtype (gate columns first, then up); q [M,K] bytes; group_size must be 128.
 * The result is bit-identical to fp8k_silu_and_mul followed by fp8k_group_quant; scales as in fp8k_group_quant.
 */
int fp8k_silu_mul_group_quant(const void* x, void* q, void* s, int64_t M, int64_t K, int64_t group_size, float eps,
                              float fp8_min, float fp8_max, int in_dtype, int64_t s_stride_m, int64_t s_stride_g,
                              int scale_kind, void* stream);

/*
 * Masked-layout form of the two calls above: x [E, m_max, K] (or [E, m_max, 2K] with fuse_silu_and_mul), q [E, m_max, K];
 * only the first masked_m[e] rows of expert e are read and written.
 * Replaces torch.ops.sgl_kernel.sgl_per_token_group_quant_8bit_v2 with masked_m
 *   (sgl-kernel/csrc/gemm/per_token_group_quant_8bit_v2.cu, wrapper fp8_kernel.py:481-531) and the Triton
 *   silu_and_mul_masked_post_quant_fwd (python/sglang/srt/layers/moe/ep_moe/kernels.py:364-429).
 * Scales as in fp8k_group_quant with one more stride: row i of expert e, group g at
 *   s[e*s_stride_e + i*s_stride_m + g*s_stride_g] (packed UE8M0: word g/4 at (g/4)*s_stride_g); FP8K_SCALE_UE8M0_F32
 *   writes the rounded-up power of two as a float at the float position (the Triton kernel's SCALE_UE8M0 branch,
 *   ep_moe/kernels.py:348-350).
 * masked_m: int32[E] on the device.  group_size must be 128.
 */
int fp8k_group_quant_masked(const void* x, void* q, void* s, int64_t E, int64_t m_max, int64_t K, int64_t group_size,
                            float eps, float fp8_min, float fp8_max, int in_dtype, int64_t s_stride_e,
                            int64_t s_stride_m, int64_t s_stride_g, int scale_kind, int fuse_silu_and_mul,
                            const int32_t* masked_m, void* stream);

/*
 * Per-token (row) dynamic FP8 quantisation: s[m] = rowamax/448, q = clamp(x * (1/s)).
 * Replaces torch.ops.sgl_kernel.sgl_per_token_quant_fp8
 *   (sgl-kernel/python/sgl_kernel/gemm.py:155-160, sgl-kernel/csrc/gemm/per_token_quant_fp8.cu:15-236).
 * x [M,K] contiguous, K % 8 == 0; q [M,K]; s float [M].
 */
int fp8k_token_quant(const void* x, void* q, float* s, int64_t M, int64_t K, int in_dtype, void* stream);

/*
 * Per-tensor FP8 quantisation.  is_static=0: *s must be zero on entry and receives absmax/448
 * (atomic max), then q = clamp(x * (1/ *s)).  is_static=1: *s is read only.
 * Replaces torch.ops.sgl_kernel.sgl_per_tensor_quant_fp8
 *   (sgl-kernel/python/sgl_kernel/gemm.py:144-152, sgl-kernel/csrc/gemm/per_tensor_quant_fp8.cu:96-118).
 */
int fp8k_tensor_quant(const void* x, void* q, float* s, int64_t numel, int in_dtype, int is_static, void* stream);

/*
 * Block-scaled FP8 GEMM:  C[m,n] = sum_kb ( A[m,kb] . B[n,kb] ) * As[m,kb] * Bs[n/128,kb],  fp32 accumulate.
 * Replaces torch.ops.sgl_kernel.fp8_blockwise_scaled_mm
 *   (sgl-kernel/python/sgl_kernel/gemm.py:25-32, sgl-kernel/csrc/gemm/fp8_blockwise_gemm_kernel.cu:368-465)
 *   and w8a8_block_fp8_matmul (python/sglang/srt/layers/quantization/fp8_kernel.py:1072-1168).
 * A e4m3fn [M,K] row-major (lda elements between rows); B e4m3fn [N,K] row-major (ldb) - the same memory
 * as the reference's column-major mat_b [K,N]; scale block is 128 x 128.
 * As float, element (m,kb) at As[m*as_stride_m + kb*as_stride_k]; Bs float, element (nb,kb) at
 * Bs[nb*bs_stride_n + kb*bs_stride_k].  C [M,N] of out_dtype (F16/BF16), ldc elements between rows.
 * K % 16 == 0, lda % 16 == 0, ldb % 16 == 0, ldc*2 % 16 == 0.
 * workspace: device scratch of at least fp8k_block_gemm_workspace_bytes(M,N,K) bytes (may be 0 -> NULL ok): float
 *   partials of K-cut launches and, for more than 32 rows, room for a column-major copy of row-major scales_a.
 */
int fp8k_block_gemm(const void* A, const void* B, const float* As, const float* Bs, void* C, int64_t M, int64_t N,
                    int64_t K, int64_t lda, int64_t ldb, int64_t as_stride_m, int64_t as_stride_k,
                    int64_t bs_stride_n, int64_t bs_stride_k, int64_t ldc, int out_dtype, void* workspace,
                    int64_t workspace_bytes, void* stream);

/*
 * The same product with power-of-two scales that the matrix core applies itself (no float promote per K block):
 * As_packed int32 words of four UE8M0 exponent bytes, as fp8k_group_quant writes them with FP8K_SCALE_UE8M0_PACKED
 * (row m, K blocks 4j..4j+3 in the word at As_packed[m*as_stride_m + j*as_stride_w]); Bs float32, every value a power of
 * two (UE8M0-format checkpoints, or weights requantised with power-of-two scales).
 * Counterpart in the reference: the DeepGEMM path with DEEPGEMM_SCALE_UE8M0
 *   (python/sglang/srt/layers/quantization/fp8_utils.py:229-268, deep_gemm_wrapper/entrypoint.py:70-88).
 * Built for M > 128 and K % 128 == 0 (other shapes: expand the exponents to floats and call fp8k_block_gemm).
 * A Bs value that is not a power of two is used as if its mantissa were zero.
 */
int fp8k_block_gemm_ue8m0(const void* A, const void* B, const int32_t* As_packed, const float* Bs, void* C, int64_t M,
                          int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t as_stride_m, int64_t as_stride_w,
                          int64_t bs_stride_n, int64_t bs_stride_k, int64_t ldc, int out_dtype, void* workspace,
                          int64_t workspace_bytes, void* stream);
int64_t fp8k_block_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K);

/*
 * fp8k_block_gemm for callers that cannot allocate device memory or pass a workspace: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.  Same arguments and the
 * same result, bit for bit, as fp8k_block_gemm, without the workspace pair: the scratch (float partials of K-cut
 * launches, the column-major copy of row-major activation scales) is a fixed 80 MiB array in device memory that is
 * part of this library - one copy on every GPU that loads it, held until the process ends.  The call allocates and
 * frees nothing.  The first call on a device looks up the array's device address (hipGetSymbolAddress) and keeps it;
 * make that call outside a graph capture (inside one it is refused with FP8K_ERR_UNSUPPORTED).  The stream's device
 * must be the calling thread's current device (FP8K_ERR_INVALID otherwise): each GPU has its own copy of the array.  A shape whose fp8k_block_gemm_workspace_bytes exceeds 80 MiB is refused
 * with FP8K_ERR_WORKSPACE.  All calls on one GPU share the one array: calls that overlap in time on the same GPU
 * (two streams, two threads) race; nothing in the array has to be cleared between calls.
 */
int fp8k_block_gemm_noalloc(const void* A, const void* B, const float* As, const float* Bs, void* C, int64_t M,
                            int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t as_stride_m, int64_t as_stride_k,
                            int64_t bs_stride_n, int64_t bs_stride_k, int64_t ldc, int out_dtype, void* stream);

/*
 * Per-token x per-channel FP8 GEMM:  C = (A . B^T) * sa[m] * sb[n] (+ bias[n]), fp32 accumulate.
 * Replaces torch.ops.sgl_kernel.fp8_scaled_mm
 *   (sgl-kernel/python/sgl_kernel/gemm.py:35-43, sgl-kernel/csrc/gemm/fp8_gemm_kernel.cu:1450-1532).
 * Layouts as fp8k_block_gemm; sa float [M], sb float [N]; bias NULL or [N] of bias_dtype (F32/F16/BF16),
 * added in float32 before the output cast.
 */
int fp8k_scaled_mm(const void* A, const void* B, const float* sa, const float* sb, const void* bias, void* C,
                   int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int out_dtype,
                   int bias_dtype, void* workspace, int64_t workspace_bytes, void* stream);
int64_t fp8k_scaled_mm_workspace_bytes(int64_t M, int64_t N, int64_t K);

/*
 * Per-tensor FP8 quantisation of a strided [H, S, D] tensor into a contiguous [H, S, D] one (the activations of the
 * MLA absorbed products): *s must be zero on entry and receives max(absmax, eps) / 448 (atomic max), then
 * q = clamp(x * (1 / *s)).
 * Replaces per_tensor_quant_mla_fp8 (python/sglang/srt/layers/quantization/fp8_kernel.py:1172-1266, two Triton kernels).
 * Row (h, s) of x starts at x[h * x_stride_h + s * x_stride_s] (elements) and is contiguous; D % 8 == 0, rows 16-byte aligned.
 */
int fp8k_tensor_quant_mla(const void* x, void* q, float* s, int64_t H, int64_t S, int64_t D, int64_t x_stride_h,
                          int64_t x_stride_s, float eps, int in_dtype, void* stream);

/*
 * Batched FP8 GEMM with one scale per operand: C[b] = (A[b] . B[b]^T) * sa[m] * sb[n], float32 accumulation.
 * Replaces torch.ops.sgl_kernel.bmm_fp8 (sgl-kernel/python/sgl_kernel/gemm.py:45-82, sgl-kernel/csrc/gemm/bmm_fp8.cu),
 * whose per-tensor scales the caller broadcasts to the vectors sa [M] and sb [N] (shared by all batch entries).
 * A e4m3fn [batch, M, K]: entry b at A + b * a_stride_b bytes, lda bytes between rows.  B e4m3fn [batch, N, K] with K
 * contiguous - the same memory as the reference's column-major [batch, K, N] - entry b at B + b * b_stride_b, ldb
 * between rows.  C [batch, M, N] of out_dtype: entry b at C + b * c_stride_b elements, ldc elements between rows.
 * K % 128 == 0, N % 8 == 0, batch <= 65535.  No workspace.
 */
int fp8k_bmm_fp8(const void* A, const void* B, const float* sa, const float* sb, void* C, int64_t batch, int64_t M,
                 int64_t N, int64_t K, int64_t a_stride_b, int64_t lda, int64_t b_stride_b, int64_t ldb,
                 int64_t c_stride_b, int64_t ldc, int out_dtype, void* stream);

/*
 * Token alignment for the fused-MoE grouped GEMM (integer work).
 * Replaces torch.ops.sgl_kernel.moe_align_block_size
 *   (sgl-kernel/python/sgl_kernel/moe.py:6-25, sgl-kernel/csrc/moe/moe_align_kernel.cu:302-366); the caller
 *   python/sglang/srt/layers/moe/fused_moe_triton/moe_align_block_size.py:57-81 passes num_experts+1 buckets.
 * topk_ids: numel ids (int32, or int64 when ids_are_int64), values in [-1, num_buckets-1); id e goes to bucket e+1.
 * Outputs: sorted_token_ids - for every bucket in use, its flat id positions (order inside a bucket is
 *   unspecified) followed, when pad_sorted_token_ids, by the value numel up to a multiple of block_size;
 *   expert_ids[b] = bucket-1 of block b for b < post_pad/block_size; num_tokens_post_pad[0] = slots in use.
 * cumsum_buffer: num_buckets+1 ints of scratch (consumed); with it more than 8192 ids are counted and placed by one
 *   workgroup per 4096 ids (four launches); NULL: a single workgroup does all the work whatever numel is.
 * Capacities are checked against the worst case numel + min(numel, num_buckets)*(block_size-1).
 */
int fp8k_moe_align_block_size(const void* topk_ids, int ids_are_int64, int64_t numel, int64_t num_buckets,
                              int64_t block_size, int32_t* sorted_token_ids, int64_t sorted_capacity,
                              int32_t* expert_ids, int64_t expert_capacity, int32_t* num_tokens_post_pad,
                              int32_t* cumsum_buffer, int pad_sorted_token_ids, void* stream);

/*
 * Grouped block-scaled FP8 GEMM with expert indirection:
 *   C[slot, n] = w(slot) * sum_kb ( A[slot / top_k, kb] . B[e, n, kb] ) * As[slot / top_k, kb] * Bs[e, n/128, kb]
 * for every slot = sorted_token_ids[i] < num_valid_tokens, i < num_tokens_post_padded[0], with
 * e = expert_ids[i / block_m]; blocks with e < 0 write zeros; w = topk_weights[slot] or 1 when NULL.
 * Replaces invoke_fused_moe_kernel / fused_moe_kernel with use_fp8_w8a8 and block_shape [128,128]
 *   (python/sglang/srt/layers/moe/fused_moe_triton/fused_moe_triton_kernels.py:307-583, 586-790).
 * A e4m3fn [ceil(num_valid/top_k), K] (lda); B e4m3fn [E, N, K] (b_stride_e bytes between experts, ldb between
 * rows); As float (as_stride_m, as_stride_k); Bs float [E, ceil(N/128), K/128] (bs_stride_e, bs_stride_n,
 * bs_stride_k); C [num_valid_tokens, N] of out_dtype (ldc).  block_m in {16,32,64,128,256} is the block size
 * moe_align_block_size was called with; sorted_capacity = length of sorted_token_ids.  K % 128 == 0, N % 8 == 0.
 * as_sorted bit 0 (block_m >= 64): As holds one row per position of sorted_token_ids instead of one per token
 * (see fp8k_moe_sort_scales).  as_sorted bit 1 (value 2 or 3; a hint, the result does not depend on it): the table went
 * through fp8k_moe_balance_blocks, so the blocks of an expert are equally full - the 256-slot kernel then runs as one
 * walking workgroup per CU at every size instead of only up to 192 slots per expert.
 */
int fp8k_moe_block_gemm(const void* A, const void* B, const float* As, const float* Bs, void* C,
                        const int32_t* sorted_token_ids, const int32_t* expert_ids,
                        const int32_t* num_tokens_post_padded, const float* topk_weights, int64_t sorted_capacity,
                        int64_t block_m, int64_t num_valid_tokens, int64_t top_k, int64_t num_experts, int64_t N,
                        int64_t K, int64_t lda, int64_t as_stride_m, int64_t as_stride_k, int64_t b_stride_e,
                        int64_t ldb, int64_t bs_stride_e, int64_t bs_stride_n, int64_t bs_stride_k, int64_t ldc,
                        int out_dtype, int as_sorted, void* stream);

/*
 * fp8k_moe_block_gemm for scale tensors that hold only powers of two (UE8M0 checkpoints, activations quantised with
 * scale_ue8m0): same arguments, same result up to the rounding of the accumulation.  With block_m == 256 and
 * as_sorted != 0 the matrix cores apply both scales themselves (v_mfma_scale_f32_32x32x64_f8f6f4 with the exponent
 * byte of each float) and the products accumulate in place; every other block size runs the kernels of
 * fp8k_moe_block_gemm.  A scale that is not a power of two is truncated to one (its mantissa is ignored): the caller
 * vouches for the tensors, as SGLang does when DEEPGEMM_SCALE_UE8M0 is set
 *   (python/sglang/srt/layers/deep_gemm_wrapper/configurer.py, python/sglang/srt/layers/quantization/fp8_utils.py:229-268);
 * the grouped entry points this serves are python/sglang/srt/layers/deep_gemm_wrapper/entrypoint.py:26-67.
 */
int fp8k_moe_block_gemm_ue8m0(const void* A, const void* B, const float* As, const float* Bs, void* C,
                              const int32_t* sorted_token_ids, const int32_t* expert_ids,
                              const int32_t* num_tokens_post_padded, const float* topk_weights, int64_t sorted_capacity,
                              int64_t block_m, int64_t num_valid_tokens, int64_t top_k, int64_t num_experts, int64_t N,
                              int64_t K, int64_t lda, int64_t as_stride_m, int64_t as_stride_k, int64_t b_stride_e,
                              int64_t ldb, int64_t bs_stride_e, int64_t bs_stride_n, int64_t bs_stride_k, int64_t ldc,
                              int out_dtype, int as_sorted, void* stream);

/*
 * Expert-major row layout for the grouped GEMM (integer work): the (token, k) slots of topk_ids int32 [numel] sorted by
 * expert into contiguous, un-padded row ranges.
 * Replaces torch.ops.sgl_kernel.prepare_moe_input (sgl-kernel/python/sgl_kernel/moe.py:217-240,
 *   sgl-kernel/csrc/moe/prepare_moe_input.cu:12-167).
 * expert_offsets [E + 1] (start row of every expert, then the total); blockscale_offsets [E + 1] or null (the same with
 * every count rounded up to 128); problem_sizes1 [E, 3] = (rows, 2n, k); problem_sizes2 [E, 3] = (rows, k, n);
 * input_permutation [numel]: token (slot / topk) whose copy sits in that row; output_permutation [numel]: row of the
 * slot.  As in the reference the order of the rows inside one expert is not defined (atomic cursors).  Ids outside
 * [0, num_experts) take no row.  num_experts <= 4096.  One workgroup, no scratch memory (the reference allocates a
 * zeroed counter buffer per call).
 */
int fp8k_moe_prepare_input(const int32_t* topk_ids, int64_t numel, int64_t topk, int64_t num_experts, int64_t n, int64_t k,
                           int32_t* expert_offsets, int32_t* blockscale_offsets, int32_t* problem_sizes1,
                           int32_t* problem_sizes2, int32_t* input_permutation, int32_t* output_permutation, void* stream);

/*
 * output[d, :] = input[dst2src_map[d], :] for contiguous rows of row_bytes bytes (moved 16 bytes a lane when rows and
 * pointers are multiples of 16 bytes, 4 or 1 otherwise).  Replaces torch.ops.sgl_kernel.shuffle_rows (sgl-kernel/python/sgl_kernel/gemm.py:302-309,
 * prepare_moe_input.cu:169-250).  A map entry outside [0, src_rows) leaves its destination row untouched.
 */
int fp8k_shuffle_rows(const void* input, const int32_t* dst2src_map, void* output, int64_t src_rows, int64_t dst_rows,
                      int64_t row_bytes, void* stream);

/*
 * output[t, :] = sum_j factors[t * topk + j] * input[permutation[t * topk + j], :], float32 sum in ascending j, one
 * rounding to the element type; factors (same element type as the data) may be null (= 1).
 * Replaces torch.ops.sgl_kernel.apply_shuffle_mul_sum (sgl-kernel/python/sgl_kernel/moe.py:243-251,
 * prepare_moe_input.cu:252-392).  cols % 8 == 0; rows whose permutation entry is outside [0, input_rows) are skipped;
 * permutation NULL = the identity (input rows already in slot order).
 */
int fp8k_apply_shuffle_mul_sum(const void* input, void* output, const int32_t* permutation, const void* factors, int64_t m,
                               int64_t topk, int64_t cols, int64_t input_rows, int dtype, void* stream);

/*
 * Block table (sorted_token_ids / expert_ids / num_tokens_post_padded, as fp8k_moe_align_block_size writes them) for the
 * expert-major layout: expert e owns rows [expert_starts[e], expert_starts[e] + problem_sizes[3 * e]).  With it
 * fp8k_moe_block_gemm (top_k = 1, num_valid_tokens = rows) is the grouped GEMM of
 * torch.ops.sgl_kernel.fp8_blockwise_scaled_grouped_mm (sgl-kernel/python/sgl_kernel/moe.py:175-214,
 * sgl-kernel/csrc/moe/fp8_blockwise_moe_kernel.cu), which takes exactly these two tensors; the reference's pointer
 * arrays, stride vectors and scale-layout buffers are CUTLASS plumbing with no counterpart here.
 */
int fp8k_moe_blocks_from_offsets(const int32_t* expert_starts, const int32_t* problem_sizes, int64_t num_experts, int64_t rows,
                                 int64_t block_m, int32_t* sorted_token_ids, int64_t sorted_capacity, int32_t* expert_ids,
                                 int64_t expert_capacity, int32_t* num_tokens_post_pad, void* stream);

/*
 * The same block table holding token SLOTS (slot = token * topk + j, padded with num_slots) at the positions of their
 * expert-major rows: from what fp8k_moe_prepare_input wrote (expert_starts, problem_sizes, slot_rows = its
 * output_permutation) and the routed ids themselves (slots whose id is outside [0, num_experts) take no place).  With it
 * fp8k_moe_block_gemm (top_k = topk, num_valid_tokens = num_slots) gathers token slot / topk from the un-shuffled
 * activations and writes its rows in slot order: the two shuffle_rows copies that cutlass_fused_experts_fp8 makes in
 * front of its grouped GEMM (python/sglang/srt/layers/moe/cutlass_moe.py:152-154) are not needed.
 */
int fp8k_moe_slot_blocks_from_offsets(const int32_t* expert_starts, const int32_t* problem_sizes, int64_t num_experts,
                                      const int32_t* topk_ids, const int32_t* slot_rows, int64_t num_slots, int64_t block_m,
                                      int32_t* sorted_token_ids, int64_t sorted_capacity, int32_t* expert_ids,
                                      int64_t expert_capacity, int32_t* num_tokens_post_pad, void* stream);

/*
 * Grouped GEMM 1 of the fused MoE layer with silu_and_mul and the per-token-group requantisation inside its write-out
 * (256-slot blocks): what fp8k_moe_block_gemm into a 16-bit [slots, 2 I] tensor followed by
 * fp8k_silu_mul_group_quant would produce, bit for bit, without that tensor ever being written.
 * Replaces the sequence invoke_fused_moe_kernel -> silu_and_mul -> per_token_group_quant_fp8 of fused_experts_impl
 *   (python/sglang/srt/layers/moe/fused_moe_triton/fused_moe.py:498-600); the reference has the activation + quant
 *   fusion as its own kernel (sgl-kernel/csrc/gemm/per_token_group_quant_8bit_v2.cu:336-341), not inside the GEMM.
 * B e4m3fn [E, 2 I, K]: gate rows, then up rows (the checkpoint layout, no re-ordering); I % 128 == 0.
 * As_sorted: activation scales in the order of sorted_token_ids (fp8k_moe_sort_scales), as_stride_k floats between
 * K blocks.  q_out e4m3fn [slots, I] (ldq bytes between rows, row = token slot); qs_out float, the scale of
 * activation column block g of the slot at position i of sorted_token_ids at qs_out[g * qs_stride_g + i] (0 for
 * padding) - the layout fp8k_moe_block_gemm takes with as_sorted = 1.  act_dtype: the 16-bit type whose roundings
 * the write-out reproduces (the dtype the layer runs in).  eps as for fp8k_group_quant.  balanced != 0: the hint of
 * fp8k_moe_block_gemm's as_sorted bit 1 (the table went through fp8k_moe_balance_blocks).
 */
int fp8k_moe_block_gemm_silu_quant(const void* A, const void* B, const float* As_sorted, const float* Bs, void* q_out,
                                   float* qs_out, const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                   const int32_t* num_tokens_post_padded, int64_t sorted_capacity, int64_t num_valid_tokens,
                                   int64_t top_k, int64_t num_experts, int64_t N, int64_t K, int64_t lda, int64_t as_stride_k,
                                   int64_t b_stride_e, int64_t ldb, int64_t bs_stride_e, int64_t bs_stride_n,
                                   int64_t bs_stride_k, int64_t ldq, int64_t qs_stride_g, float eps, int act_dtype,
                                   int balanced, void* stream);

/*
 * No counterpart in the reference (its grouped kernel reads the table of moe_align_block_size as it is): deals the slots
 * of every expert out evenly over the blocks the expert already has.  moe_align_block_size fills all blocks of an expert
 * but the last (600 slots: 256, 256, 88); the workgroups that take those blocks against one weight tile share the tile in
 * L2 only while they keep pace, which blocks of 200, 200, 200 do and blocks of 256 and 88 do not.  sorted_out (a buffer
 * of its own, sorted_capacity entries) receives the table; expert_ids and num_tokens_post_padded stay as they are; real
 * slots still come first in every block; entries behind the blocks in use get the padding value num_valid_tokens.
 * num_experts: the experts of the aligner call (ids 0 .. num_experts-1; blocks of expert id -1 are dealt out the same way).
 */
int fp8k_moe_balance_blocks(const int32_t* sorted_token_ids, const int32_t* expert_ids,
                            const int32_t* num_tokens_post_padded, int64_t sorted_capacity, int64_t block_m,
                            int64_t num_valid_tokens, int64_t num_experts, int32_t* sorted_out, void* stream);

/*
 * Activation scales in the order of sorted_token_ids (no counterpart in the reference, whose Triton kernel gathers
 * them per K block): out[kb * sorted_capacity + i] = As[sorted_token_ids[i] / top_k, kb] for i below
 * num_tokens_post_padded[0], 0 for padding entries.  Passing `out` to fp8k_moe_block_gemm with as_stride_m = 1,
 * as_stride_k = sorted_capacity and as_sorted = 1 lets the lanes of a wave fetch their scales from one cache line
 * instead of one line per token row.
 */
int fp8k_moe_sort_scales(const float* As, float* out, const int32_t* sorted_token_ids,
                         const int32_t* num_tokens_post_padded, int64_t sorted_capacity, int64_t k_blocks, int64_t top_k,
                         int64_t num_valid_tokens, int64_t as_stride_m, int64_t as_stride_k, void* stream);

/*
 * out[r, c] = silu(x[r, c]) * x[r, d + c] for c < d, computed as the reference does for 16-bit types:
 * silu in float32, rounded to the element type, multiplied, rounded again.
 * Replaces torch.ops.sgl_kernel.silu_and_mul
 *   (sgl-kernel/python/sgl_kernel/elementwise.py:172-184, sgl-kernel/csrc/elementwise/activation.cu:85-105,
 *    sgl-kernel/include/hip/hip_act_and_mul.cuh:29-56).
 * x [rows, 2d] (ldx elements between rows), out [rows, d] (ldo); d % 8 == 0; 16-byte aligned pointers.
 */
int fp8k_silu_and_mul(const void* x, void* out, int64_t rows, int64_t d, int64_t ldx, int64_t ldo, int dtype,
                      void* stream);

/*
 * out[r, c] = gelu(x[r, c]) * x[r, d + c] for c < d with the erf form of gelu, x * 0.5 * (1 + erf(x / sqrt 2)), in
 * float32; roundings, shapes and alignment as fp8k_silu_and_mul.
 * Replaces torch.ops.sgl_kernel.gelu_and_mul
 *   (sgl-kernel/python/sgl_kernel/elementwise.py:202-214, sgl-kernel/csrc/elementwise/activation.cu:62-67,129-149);
 *   the activation="gelu" branch of fused_experts_impl calls it
 *   (python/sglang/srt/layers/moe/fused_moe_triton/fused_moe.py:561-565).
 */
int fp8k_gelu_and_mul(const void* x, void* out, int64_t rows, int64_t d, int64_t ldx, int64_t ldo, int dtype,
                      void* stream);

/*
 * out[r, c] = act(x[r, c]) for c < d: the activation of experts without a gate projection, in float32 with one rounding
 * to the element type.  kind: FP8K_ACT_SILU, FP8K_ACT_GELU (erf form), FP8K_ACT_RELU2 (relu(x)^2).
 * Replaces the tensor-library calls of the ungated branch of fused_experts_impl - F.silu, F.gelu and
 * torch.square(F.relu(.)) on the [tokens * topk, N] result of the first grouped GEMM
 *   (python/sglang/srt/layers/moe/fused_moe_triton/fused_moe.py:566-572).
 * x [rows, d] (ldx elements between rows), out [rows, d] (ldo); d % 8 == 0; 16-byte aligned pointers.
 */
int fp8k_activation(const void* x, void* out, int64_t rows, int64_t d, int64_t ldx, int64_t ldo, int kind, int dtype,
                    void* stream);

/*
 * out[t, :] = scale * sum_k x[t, k, :], float32 accumulation in ascending k, one rounding.
 * Replaces torch.ops.sgl_kernel.moe_sum_reduce
 *   (sgl-kernel/python/sgl_kernel/moe.py:83-92, sgl-kernel/csrc/moe/moe_sum_reduce.cu:56-113,227-).
 * Strides in elements; hidden % 8 == 0.
 */
int fp8k_moe_sum_reduce(const void* x, void* out, int64_t tokens, int64_t topk, int64_t hidden, int64_t stride_token,
                        int64_t stride_topk, int64_t out_stride_token, float scale, int dtype, void* stream);

/*
 * out[t, :] = sum_k x[t, k, :] as torch.ops.sgl_kernel.moe_sum computes it (sgl-kernel/python/sgl_kernel/moe.py:95-102,
 * sgl-kernel/csrc/moe/moe_sum.cu:11-69): for topk 2, 3 and 4 the sum runs in the element type, one rounding per
 * addition in ascending k; any other topk is the float32-accumulated sum of fp8k_moe_sum_reduce with scale 1.
 * Strides in elements; hidden % 8 == 0.
 */
int fp8k_moe_sum(const void* x, void* out, int64_t tokens, int64_t topk, int64_t hidden, int64_t stride_token,
                 int64_t stride_topk, int64_t out_stride_token, int dtype, void* stream);

/*
 * Grouped top-k routing with a selection bias (DeepSeek-V3 style gate).
 * Replaces torch.ops.sgl_kernel.moe_fused_gate (sgl-kernel/python/sgl_kernel/moe.py:105-137,
 *   sgl-kernel/csrc/moe/moe_fused_gate.cu:52-257, schema common_extension.cc:240-244).
 * input [num_rows, num_experts] and bias [num_experts] of `dtype`; topk_weights float32 [num_rows, topk];
 * topk_ids int32 [num_rows, topk].  num_experts a power of two, divisible by num_expert_group,
 * num_experts / num_expert_group <= 32, num_expert_group <= 64.  The last num_fused_shared_experts entries of a
 * row are the shared experts (ids num_experts + i, weight sum / routed_scaling_factor); weights are renormalised
 * to sum 1 and, if apply_routed_scaling_factor_on_output, multiplied by routed_scaling_factor.
 */
int fp8k_moe_fused_gate(const void* input, const void* bias, float* topk_weights, int32_t* topk_ids, int64_t num_rows,
                        int64_t num_experts, int64_t num_expert_group, int64_t topk_group, int64_t topk,
                        int64_t num_fused_shared_experts, double routed_scaling_factor,
                        int apply_routed_scaling_factor_on_output, int dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FP8K_H */
