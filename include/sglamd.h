/*
 * sglamd.h -- C ABI of libsglamd.so: hand-written gfx950 (MI355X) kernels for SGLang's
 * quantized-linear hot path.  Plain pointers, sizes, element strides and a hipStream_t
 * (passed as void*); no torch types.  Every entry point
 *   - validates its arguments on the host and returns SGLAMD_OK (0) or a negative
 *     SGLAMD_E* code, with the text available from sglamd_last_error();
 *   - enqueues its kernels on `stream` and returns without synchronising;
 *   - never reads device data on the host and never allocates device memory, so it can
 *     be captured into a HIP graph.
 * All pointers are device pointers unless a comment says otherwise.
 *
 * Each declaration cites the reference operator it stands in for (paths relative to the
 * SGLang tree).
 */
#ifndef SGLAMD_H_
#define SGLAMD_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element type tags */
enum {
  SGLAMD_F32 = 0,
  SGLAMD_F16 = 1,
  SGLAMD_BF16 = 2,
  SGLAMD_FP8_E4M3 = 3, /* OCP e4m3fn */
  SGLAMD_I8 = 4,
  SGLAMD_I32 = 5,
  SGLAMD_I64 = 6
};

/* status codes */
enum {
  SGLAMD_OK = 0,
  SGLAMD_EINVAL = -1,  /* an argument violates a documented precondition */
  SGLAMD_ENOTSUP = -2, /* valid in the reference, not implemented here */
  SGLAMD_EHIP = -3     /* the HIP runtime reported an error at launch */
};

/* Text of the last failure on the calling thread ("" if none). */
const char* sglamd_last_error(void);

/* Library ABI version (bumped when a signature changes). */
int sglamd_abi_version(void);

/* ------------------------------------------------------------------------------------
 * Per-token-group 8-bit quantisation.
 * Stands in for sgl_per_token_group_quant_8bit
 *   (sgl-kernel/csrc/gemm/per_token_group_quant_8bit.cu:116-217, kernel :19-114) when
 *   form == SGLAMD_QUANT_FORM_DIVIDE, and for sgl_per_token_group_quant_8bit_v2
 *   (sgl-kernel/csrc/gemm/per_token_group_quant_8bit_v2.cu:411-542, kernel :249-409,
 *   scale arithmetic :69-90) when form == SGLAMD_QUANT_FORM_RECIPROCAL.
 *
 * input    [rows, hidden] contiguous, in_dtype in {F32 (divide form only), F16, BF16}
 * output_q [rows, hidden] contiguous, q_dtype in {FP8_E4M3, I8}
 * output_s scales, one per group of `group_size` consecutive elements of a row:
 *   scale_layout SGLAMD_SCALE_ROW_MAJOR : float [rows, hidden/group_size] contiguous
 *   scale_layout SGLAMD_SCALE_COL_MAJOR : float, element (m, g) at g*scale_stride + m
 *   scale_layout SGLAMD_SCALE_COL_MAJOR_UE8M0 : bytes packed four to an int32, exponent
 *     byte of (m, g) at byte ((g/4)*scale_stride + m)*4 + g%4; when hidden/group_size is
 *     not a multiple of 4 the unused bytes of the last int32 of each row are written 0.
 * eps is the lower bound of the group absmax; min_8bit/max_8bit the clamp range.
 * ---------------------------------------------------------------------------------- */
enum { SGLAMD_SCALE_ROW_MAJOR = 0, SGLAMD_SCALE_COL_MAJOR = 1, SGLAMD_SCALE_COL_MAJOR_UE8M0 = 2 };
enum { SGLAMD_QUANT_FORM_DIVIDE = 0, SGLAMD_QUANT_FORM_RECIPROCAL = 1 };

int sglamd_per_token_group_quant_8bit(const void* input, int in_dtype, void* output_q, int q_dtype,
                                      void* output_s, int64_t rows, int64_t hidden, int group_size,
                                      int scale_layout, int64_t scale_stride, float eps, float min_8bit,
                                      float max_8bit, int form, void* stream);

/* Per-token (per-row) FP8 quantisation: scale = max|x| / 448 (no eps; an all-zero row
 * gives scale 0 and zero bytes), q = e4m3(clamp(x * (1/scale))).
 * Stands in for sgl_per_token_quant_fp8 (sgl-kernel/csrc/gemm/per_token_quant_fp8.cu:242-314,
 * arithmetic :71-105).  input [rows, hidden] contiguous F32/F16/BF16; output_s float[rows]. */
int sglamd_per_token_quant_fp8(const void* input, int in_dtype, void* output_q, float* output_s, int64_t rows,
                               int64_t hidden, void* stream);

/* Static per-tensor FP8 quantisation with a given scale (one float on the device):
 * q = e4m3(clamp(x * (1 / scale), -448, 448)); when scale_rows is not NULL the scale is also written once per
 * row (float[rows]), which is the per-token scale vector sglamd_fp8_scaled_mm takes.
 * Stands in for the Triton static_quant_fp8 (python/sglang/srt/layers/quantization/fp8_kernel.py:681-777), the
 * activation path of apply_fp8_linear for checkpoints with a static input_scale (fp8_utils.py:1518-1524).
 * input [rows, hidden] contiguous F32/F16/BF16, hidden % 8 == 0. */
int sglamd_static_quant_fp8(const void* input, int in_dtype, void* output_q, const float* scale, float* scale_rows,
                            int64_t rows, int64_t hidden, void* stream);

/* The scale of dynamic per-tensor FP8 quantisation: scale[0] = max(max|x|, eps) / fp8_max over all `numel`
 * elements of `input` (F32/F16/BF16, contiguous), in two small launches without atomics; `workspace` is 1024
 * floats of device scratch.  Followed by sglamd_static_quant_fp8 with that scale it stands in for the dynamic
 * per-tensor branch of scaled_fp8_quant (python/sglang/srt/layers/quantization/fp8_kernel.py:1693-1777;
 * arithmetic pinned by the reference's own test, test/manual/quant/test_custom_ops.py:20-44: scale =
 * max|x| / 448, q = e4m3(clamp(float(x) * (1 / scale)))); eps keeps an all-zero tensor's scale positive, as the
 * reference's native model does with 1e-12 (fp8_kernel.py:1675-1685). */
int sglamd_tensor_absmax_scale(const void* input, int in_dtype, int64_t numel, float eps, float fp8_max, float* scale,
                               float* workspace, void* stream);

/* Per-token symmetric INT8 quantisation: amax = max(max|x|, 1e-10), scale = amax/127,
 * q = int8(round_half_away_from_zero(x * (127/amax))).
 * Stands in for the Triton per_token_quant_int8
 * (python/sglang/srt/layers/quantization/int8_kernel.py:28-89). */
int sglamd_per_token_quant_int8(const void* input, int in_dtype, int8_t* output_q, float* output_s, int64_t rows,
                                int64_t hidden, void* stream);

/* Packed UE8M0 scales to fp32: out[r, g] = 2^(e - 127) as the float whose exponent field is the byte e = byte
 * (g % 4) of the int32 word packed[(r * row_step) * row_stride + (g / 4) * word_stride] (strides in words), i.e.
 * (e << 23) reinterpreted, exactly as the reference unpacks them
 * (python/sglang/srt/layers/quantization/fp8_utils.py:1348-1383).  out is float [rows, groups] contiguous.
 * Activation scales of sgl_per_token_group_quant_8bit's UE8M0 layout: row_stride 1, word_stride = the
 * column-major stride, row_step 1.  Weight scales repeated on every weight row (the layout the block GEMM's
 * packed form takes, fp8_kernel.py:1149-1174): row_step 128 picks one row per 128x128 block. */
int sglamd_ue8m0_unpack(const void* packed, int64_t row_stride, int64_t word_stride, int64_t row_step, float* out,
                        int64_t rows, int64_t groups, void* stream);

/* ------------------------------------------------------------------------------------
 * W8A8 block-scaled FP8 GEMM:
 *   out[m, n] = cast( sum_kb ( sum_{k in kb} a[m, k] * b[n, k] ) * sa[m, kb] * sb[n/128, kb] )
 * with fp32 accumulation and 128-wide K blocks / 128x128 weight blocks.
 * Stands in for fp8_blockwise_scaled_mm (sgl-kernel/csrc/gemm/fp8_blockwise_gemm_kernel.cu:425-522)
 * and for the Triton w8a8_block_fp8_matmul
 * (python/sglang/srt/layers/quantization/fp8_kernel.py:780-869,1201-1300).
 *
 * a   e4m3fn [M, K], row stride lda bytes.
 * b   e4m3fn weight stored [N, K] with K contiguous, row stride ldb bytes (the reference's
 *     "[K, N] column-major" mat_b is this same memory).
 * sa  fp32, element (m, kb) at sa[m*sa_stride_m + kb*sa_stride_k]   (M-major or row-major)
 * sb  fp32, element (nb, kb) at sb[nb*sb_stride_n + kb*sb_stride_k]
 * out [M, N] F16 or BF16, row stride ldc elements.  K % 16 == 0; partial last blocks allowed.
 * workspace / workspace_bytes: optional split-K scratch, see sglamd_gemm_workspace_bytes().
 * ---------------------------------------------------------------------------------- */
int sglamd_fp8_blockwise_scaled_mm(const void* a, int64_t lda, const void* b, int64_t ldb, const float* sa,
                                   int64_t sa_stride_m, int64_t sa_stride_k, const float* sb, int64_t sb_stride_n,
                                   int64_t sb_stride_k, void* out, int64_t ldc, int out_dtype, int64_t M, int64_t N,
                                   int64_t K, void* workspace, int64_t workspace_bytes, void* stream);

/* The same GEMM for scales that are all powers of two -- UE8M0 scales, as DeepSeek-V3.1 checkpoints and the
 * reference's DeepGEMM path carry them (python/sglang/srt/layers/quantization/fp8_kernel.py:1149-1174 with
 * scale_ue8m0, python/sglang/srt/layers/quantization/fp8_utils.py:1348-1383), expanded to fp32 by
 * sglamd_ue8m0_unpack.  Same arguments and result up to fp32 summation order; where the launch runs the persistent
 * large-tile kernel, the scales' exponent bytes go into the MFMA's block-scale operands and the K blocks add up in
 * the MFMA accumulators (no multiply-add per element and K block).  A scale that is not a power of two counts as
 * the power of two below it there; the other kernels use the scale as given. */
int sglamd_fp8_blockwise_scaled_mm_pow2(const void* a, int64_t lda, const void* b, int64_t ldb, const float* sa,
                                        int64_t sa_stride_m, int64_t sa_stride_k, const float* sb, int64_t sb_stride_n,
                                        int64_t sb_stride_k, void* out, int64_t ldc, int out_dtype, int64_t M,
                                        int64_t N, int64_t K, void* workspace, int64_t workspace_bytes, void* stream);

/* The block-scaled GEMM on int8 operands: the int32 partial product of every 128-wide K block is exact and is
 * folded as float(p) * (sa[m, kb] * sb[n/128, kb]) into the fp32 accumulator.  Same arguments as above.
 * Stands in for w8a8_block_int8_matmul (python/sglang/srt/layers/quantization/int8_kernel.py:228-441, a Triton
 * kernel in the reference; torch-native statement test/registered/quant/test_block_int8.py:41-93). */
int sglamd_int8_blockwise_scaled_mm(const void* a, int64_t lda, const void* b, int64_t ldb, const float* sa,
                                    int64_t sa_stride_m, int64_t sa_stride_k, const float* sb, int64_t sb_stride_n,
                                    int64_t sb_stride_k, void* out, int64_t ldc, int out_dtype, int64_t M, int64_t N,
                                    int64_t K, void* workspace, int64_t workspace_bytes, void* stream);

/* The block-scaled GEMM (FP8 or int8 operands, q_dtype) for scale blocks other than [128, 128]:
 *   out[m, n] = cast( sum_g ( sum_{k in group g} a[m, k] * b[n, k] ) * sa[m, g] * sb[n / block_n, g] ),
 * groups of block_k consecutive k; block_n, block_k in {64, 128} (SGLAMD_ENOTSUP otherwise).  sa holds one scale
 * per row and block_k columns, sb one per block_n x block_k weight block; strides as above.  Runs the
 * register-staged generic kernel (no workspace).  Stands in for the Triton w8a8_block_fp8_matmul /
 * w8a8_block_int8_matmul with a general block_size (python/sglang/srt/layers/quantization/fp8_kernel.py:780-869,
 * 1201-1281; int8_kernel.py:228-441), whose own tests sweep [[64,64],[64,128],[128,64],[128,128]]
 * (test/manual/quant/test_block_fp8.py:557). */
int sglamd_block_scaled_mm_any(const void* a, int64_t lda, const void* b, int64_t ldb, const float* sa,
                               int64_t sa_stride_m, int64_t sa_stride_k, const float* sb, int64_t sb_stride_n,
                               int64_t sb_stride_k, void* out, int64_t ldc, int out_dtype, int q_dtype, int64_t M,
                               int64_t N, int64_t K, int block_n, int block_k, void* stream);

/* Per-token / per-channel scaled FP8 GEMM: out = cast( acc * sb[n] * sa[m] (+ bias[n]) ).
 * Stands in for fp8_scaled_mm (sgl-kernel/csrc/gemm/fp8_gemm_kernel.cu:1095-1173, epilogue :100-137).
 * Operand layout as above; sa float[M], sb float[N], bias optional [N] in the output dtype. */
int sglamd_fp8_scaled_mm(const void* a, int64_t lda, const void* b, int64_t ldb, const float* sa, const float* sb,
                         const void* bias, void* out, int64_t ldc, int out_dtype, int64_t M, int64_t N, int64_t K,
                         void* workspace, int64_t workspace_bytes, void* stream);

/* Per-token / per-channel scaled INT8 GEMM: out = cast( float(acc_i32) * (sb[n] * sa[m]) + float(bias[n]) ).
 * Stands in for int8_scaled_mm (sgl-kernel/csrc/gemm/int8_gemm_kernel.cu:663-747; epilogue
 * sgl-kernel/csrc/cutlass_extensions/epilogue/epilogue_per_row_per_col_scale.h:232-305). */
int sglamd_int8_scaled_mm(const void* a, int64_t lda, const void* b, int64_t ldb, const float* sa, const float* sb,
                          const void* bias, void* out, int64_t ldc, int out_dtype, int64_t M, int64_t N, int64_t K,
                          void* workspace, int64_t workspace_bytes, void* stream);

/* Optional scratch for the three GEMM entry points above.  For shapes whose tile grid alone cannot fill the
 * chip (few rows or few columns with a long K) the kernels split K and sum fp32 partial tiles from
 * `workspace`; this returns the number of bytes with which that pays for (M, N, K), or 0.  The GEMMs accept
 * workspace == NULL (or a smaller buffer) and then split less or not at all; results agree to fp32 summation
 * order.  workspace must be 16-byte aligned device memory; the library never allocates it. */
int64_t sglamd_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K);

/* Which kernel the last dense GEMM call (the four entry points above) of the calling thread launched; 0 before
 * the first call.  Diagnostic with no counterpart in the reference: the kernel is chosen from the shape by launch
 * heuristics, and a parity test uses this to assert that it covers the kernel it was written for. */
#define SGLAMD_KERNEL_STREAMING 1     /* weight-streaming kernel, M <= 16 (or shapes the tile kernel does not take) */
#define SGLAMD_KERNEL_TILE64 2        /* tile kernel, 64-row tiles */
#define SGLAMD_KERNEL_TILE128 3       /* tile kernel, 128-row tiles */
#define SGLAMD_KERNEL_TILE256 4       /* tile kernel, 256-row tiles, one tile per workgroup */
#define SGLAMD_KERNEL_PERSISTENT256 5 /* 256x256 tiles, one workgroup per CU walking several tiles */
#define SGLAMD_KERNEL_GENERIC 6       /* register-staged fallback (K % 128 != 0, operands of 2 GiB and more) */
#define SGLAMD_KERNEL_PERSISTENT256_POW2 7 /* the persistent kernel applying power-of-two scales inside the MFMA */
#define SGLAMD_KERNEL_STREAMING_WIDE 8  /* weight-streaming kernel, 33..64 rows x 96..144 weight rows per workgroup */
int sglamd_last_gemm_kernel(void);
/* The same for the streaming kernel's shape: (FM << 16) | (FN << 8) | KW of the last dense launch of it on this thread
 * -- FM 16-row activation tiles, FN 16-row weight tiles per workgroup, KW waves sharing a tile's K range. */
int sglamd_last_streaming_shape(void);

/* Diagnostic with no counterpart in the reference: the byte offset inside a row at which the streaming kernel's
 * lane chunk `lchunk` (0..7) fetches its 16 bytes of K block `kb`, written to *offset; returns 1 when that piece
 * lies past the end of K (it is then not used, and the offset names a piece inside the row).  Host code; lets a
 * test sweep ragged K and assert offset + 16 <= K for every piece the kernel requests. */
int sglamd_streaming_piece_offset(int kb, int lchunk, int64_t K, int64_t* offset);

/* ------------------------------------------------------------------------------------
 * moe_align_block_size: sorts the flat top-k expert ids into per-expert spans padded to
 * `block_size`.  `num_experts` is the number of buckets: bucket b collects ids equal to
 * b - 1 (callers pass E + 1 so that bucket 0 collects the filtered id -1).
 *   sorted_token_ids[P[b] + r] = flat index of the r-th (ascending) member of bucket b;
 *     every other slot of [0, max_num_tokens_padded) is set to numel when
 *     pad_sorted_token_ids != 0;
 *   expert_ids[j] = (bucket owning slot j*block_size) - 1, for j < post_pad/block_size;
 *   num_tokens_post_pad[0] = sum_b ceil(count[b]/block_size)*block_size;
 *   cumsum_buffer (optional, num_experts + 1 ints) receives P[b] + count[b] and the total.
 * Stands in for moe_align_block_size (sgl-kernel/csrc/moe/moe_align_kernel.cu:317-383,
 * kernels :27-41,55-233); the slot order inside a span is ascending here, where the
 * reference's depends on atomics.  ids_dtype is SGLAMD_I32 or SGLAMD_I64.
 * ---------------------------------------------------------------------------------- */
int sglamd_moe_align_block_size(const void* topk_ids, int ids_dtype, int64_t numel, int num_experts, int block_size,
                                int32_t* sorted_token_ids, int64_t max_num_tokens_padded, int32_t* expert_ids,
                                int32_t* num_tokens_post_pad, int32_t* cumsum_buffer, int pad_sorted_token_ids,
                                void* stream);

/* Sorted-block grouped block-FP8 GEMM of the fused MoE: for each block j of `block_m` sorted
 * slots with expert e = expert_ids[j] and slots t = sorted_token_ids[j*block_m + r] < num_valid_tokens:
 *   c[t, n] = cast( (sum_kb (a[t / top_k, kb] . w[e, n, kb]) * a_scale[t / top_k, kb] * w_scale[e, n/128, kb])
 *                   * (mul_routed_weight ? topk_weights[t] : 1) );  zeros when e == -1.
 * Blocks at or past num_tokens_post_padded[0] are skipped.
 * Stands in for fused_moe_kernel + invoke_fused_moe_kernel
 * (python/sglang/srt/layers/moe/moe_runner/triton_utils/fused_moe_triton_kernels.py:323-638,702-930)
 * in its use_fp8_w8a8 / block_shape [128,128] configuration.
 * a e4m3fn [rows, K] (row stride lda bytes); w e4m3fn [E, N, K] (byte strides w_stride_e, w_stride_n);
 * scale strides in elements; c row stride ldc elements; block_m in {16, 32, 64, 128, 192} must equal
 * the block_size given to moe_align_block_size; max_m_blocks = ceil(len(sorted_token_ids)/block_m). */
int sglamd_fused_moe_block_fp8_gemm(const void* a, int64_t lda, const float* a_scale, int64_t as_stride_m,
                                    int64_t as_stride_k, const void* w, int64_t w_stride_e, int64_t w_stride_n,
                                    const float* w_scale, int64_t ws_stride_e, int64_t ws_stride_n,
                                    int64_t ws_stride_k, void* c, int64_t ldc, int out_dtype,
                                    const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                    const int32_t* num_tokens_post_padded, const float* topk_weights,
                                    int64_t num_valid_tokens, int top_k, int mul_routed_weight, int block_m,
                                    int64_t max_m_blocks, int64_t N, int64_t K, void* stream);

/* The same sorted-block grouped GEMM with int8 operands: the use_int8_w8a8 / block_shape [128,128]
 * configuration of fused_moe_kernel (fused_moe_triton_kernels.py:323-638; activation quantisation
 * branch :764-777; native model torch_w8a8_block_int8_moe, test/registered/quant/test_block_int8.py:101-131).
 * Arguments as above with a and w int8; every 128-deep partial dot product is exact in int32. */
int sglamd_fused_moe_block_int8_gemm(const void* a, int64_t lda, const float* a_scale, int64_t as_stride_m,
                                     int64_t as_stride_k, const void* w, int64_t w_stride_e, int64_t w_stride_n,
                                     const float* w_scale, int64_t ws_stride_e, int64_t ws_stride_n,
                                     int64_t ws_stride_k, void* c, int64_t ldc, int out_dtype,
                                     const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                     const int32_t* num_tokens_post_padded, const float* topk_weights,
                                     int64_t num_valid_tokens, int top_k, int mul_routed_weight, int block_m,
                                     int64_t max_m_blocks, int64_t N, int64_t K, void* stream);

/* The sorted-block grouped GEMM of the fused MoE in the configurations the two entry points above do not take
 * (fused_moe_kernel, fused_moe_triton_kernels.py:323-638; scale addressing :490-516, accumulation :560-585,
 * epilogue :590-606; activation quantisation per configuration :737-783).  q_dtype FP8_E4M3 or I8.
 *   block_n, block_k in {64, 128}: block-scaled as above with that scale-block shape
 *     (a_scale[t / top_k, k / block_k], w_scale[e, n / block_n, k / block_k]);
 *   block_n == block_k == 0: row-scaled -- the raw accumulator times a_scale[(t / top_k) * as_stride_m] *
 *     w_scale[e * ws_stride_e + n * ws_stride_n]: per-token x per-channel scales (per_channel_quant), or, with
 *     as_stride_m == 0 / ws_stride_n == 0, one activation scale per tensor and one weight scale per expert
 *     (as_stride_k, ws_stride_k unused).
 * bias (optional, [E, N] in the output dtype, bias_stride_e elements between experts) is added after the scales
 * and before the routing weight, as in the reference.  block_m in {16, 32, 64, 128}.  Other arguments as above. */
int sglamd_fused_moe_gemm_any(const void* a, int64_t lda, const float* a_scale, int64_t as_stride_m,
                              int64_t as_stride_k, const void* w, int64_t w_stride_e, int64_t w_stride_n,
                              const float* w_scale, int64_t ws_stride_e, int64_t ws_stride_n, int64_t ws_stride_k,
                              const void* bias, int64_t bias_stride_e, void* c, int64_t ldc, int out_dtype, int q_dtype,
                              int block_n, int block_k, const int32_t* sorted_token_ids, const int32_t* expert_ids,
                              const int32_t* num_tokens_post_padded, const float* topk_weights,
                              int64_t num_valid_tokens, int top_k, int mul_routed_weight, int block_m,
                              int64_t max_m_blocks, int64_t N, int64_t K, void* stream);

/* ------------------------------------------------------------------------------------
 * MoE routing: softmax over the experts, top-k, optional renormalisation.
 * Stands in for topk_softmax (sgl-kernel/csrc/moe/moe_topk_softmax_kernels.cu:718-810; kernels :80-146,
 * :186-262, :340-590; schema sgl-kernel/csrc/common_extension.cc:170-173).
 *
 * gating_output [num_tokens, num_experts] contiguous, g_dtype in {F32, F16, BF16}
 * topk_weights  [num_tokens, topk] float: softmax probabilities of the picked experts (of the soft-capped and
 *               biased logits when those options are used), divided by their sum when renormalize != 0
 * topk_indices  [num_tokens, topk] int32, in decreasing probability; equal probabilities pick the lower index
 * moe_softcapping != 0 applies tanh(x / c) * c first; correction_bias (float [num_experts], may be NULL) is
 * added after that.  num_experts <= 1024. */
int sglamd_topk_softmax(float* topk_weights, int32_t* topk_indices, const void* gating_output, int g_dtype,
                        int64_t num_tokens, int64_t num_experts, int64_t topk, int renormalize, float moe_softcapping,
                        const float* correction_bias, void* stream);

/* MoE routing with sigmoid scores: score[e] = 1 / (1 + exp(-x[e])); the k experts with the largest
 * score[e] + correction_bias[e] are picked (equal values pick the lower index); topk_weights holds
 * (score + bias) - bias of the picked experts in fp32, divided by their sum when renormalize != 0.
 * Stands in for topk_sigmoid (sgl-kernel/csrc/moe/moe_topk_sigmoid_kernels.cu:496-600; kernels :75-173,
 * :262-375; schema sgl-kernel/csrc/common_extension.cc:174-177).  Layouts as for sglamd_topk_softmax. */
int sglamd_topk_sigmoid(float* topk_weights, int32_t* topk_indices, const void* gating_output, int g_dtype,
                        int64_t num_tokens, int64_t num_experts, int64_t topk, int renormalize,
                        const float* correction_bias, void* stream);

/* out[t, j] = T(silu_f32(in[t, j])) * in[t, d + j]  (silu rounded to T before the multiply).
 * Stands in for silu_and_mul (sgl-kernel/csrc/elementwise/activation.cu:55-58,82-101).
 * in [rows, 2d], out [rows, d] contiguous F16/BF16, d % 8 == 0. */
int sglamd_silu_and_mul(const void* input, void* out, int dtype, int64_t rows, int64_t d, void* stream);

/* The same with gelu(x) = x * 0.5 * (1 + erf(x / sqrt 2)) and with its tanh form
 * x * 0.5 * (1 + tanh(0.7978845608 * (x + 0.044715 x^3))) in place of silu.
 * Stand in for gelu_and_mul and gelu_tanh_and_mul (sgl-kernel/csrc/elementwise/activation.cu:62-67,76-83,107-149;
 * schemas sgl-kernel/csrc/common_extension.cc:79-83).  Same layouts and limits as sglamd_silu_and_mul. */
int sglamd_gelu_and_mul(const void* input, void* out, int dtype, int64_t rows, int64_t d, void* stream);
int sglamd_gelu_tanh_and_mul(const void* input, void* out, int dtype, int64_t rows, int64_t d, void* stream);

/* out[t, j] = T(routed_scaling_factor * sum_k f32(in[t, k, j])).
 * Stands in for moe_sum_reduce (sgl-kernel/csrc/common_extension.cc:180-181; Triton twin
 * fused_moe_triton_kernels.py:1052-1137).  in [tokens, topk, d], out [tokens, d] contiguous. */
int sglamd_moe_sum_reduce(const void* input, void* out, int dtype, int64_t tokens, int topk, int64_t d,
                          float routed_scaling_factor, void* stream);

/* silu(gate) * up and per-token-group quantisation in one pass: input [rows, 2*hidden] = [gate | up],
 * x = T(T(silu_f32(gate)) * up), then quantised exactly like sglamd_per_token_group_quant_8bit on
 * x[rows, hidden].  Stands in for the fuse_silu_and_mul variant of sgl_per_token_group_quant_8bit_v2
 * (sgl-kernel/csrc/gemm/per_token_group_quant_8bit_v2.cu:307-316,349-354) without the masked layout.
 * group_size in {16, 32, 64, 128}; F16/BF16 input. */
int sglamd_silu_mul_group_quant_8bit(const void* input, int in_dtype, void* output_q, int q_dtype, void* output_s,
                                     int64_t rows, int64_t hidden, int group_size, int scale_layout,
                                     int64_t scale_stride, float eps, float min_8bit, float max_8bit, int form,
                                     void* stream);

/* The same fused quantiser on the masked ("DeepEP low-latency") layout: input [num_experts, tokens_per_expert,
 * 2*hidden], output_q [num_experts, tokens_per_expert, hidden]; of expert e only tokens t < masked_m[e] are read
 * and written, everything else is left untouched.  Scales are packed UE8M0 words, column-major per expert:
 * word(e, t, g) = output_s[e*scale_expert_stride + (g/4)*scale_hidden_stride + t] (int32 units), byte g%4; the
 * unused bytes of a token's last word are zeroed.  Reciprocal arithmetic form.
 * Stands in for sgl_per_token_group_quant_8bit_v2 with fuse_silu_and_mul, scale_ue8m0 and masked_m
 * (sgl-kernel/csrc/gemm/per_token_group_quant_8bit_v2.cu:203-247 scheduler, :318-342 scale addressing,
 *  :434-447,489-494 host side). */
int sglamd_silu_mul_group_quant_8bit_masked(const void* input, int in_dtype, void* output_q, int q_dtype,
                                            void* output_s, int64_t num_experts, int64_t tokens_per_expert,
                                            int64_t hidden, int group_size, int64_t scale_expert_stride,
                                            int64_t scale_hidden_stride, const int32_t* masked_m, float eps,
                                            float min_8bit, float max_8bit, void* stream);

/* Fused (residual add +) RMSNorm + per-token-group FP8 quantisation, optionally with a plain RMSNorm of a
 * second tensor in the same launch.  Stands in for aiter.ops.triton.fused_fp8_quant.fused_rms_fp8_group_quant,
 * which the reference calls on gfx95 to hand pre-quantised (fp8, scale) inputs to the block-FP8 linears
 * (python/sglang/srt/layers/communicator.py:552-624,
 * python/sglang/srt/models/deepseek_common/attention_forward_methods/forward_mla.py:175-203; consumed at
 * python/sglang/srt/layers/quantization/fp8.py:794-802, fp8_utils.py:779-783); the native model is
 * test/registered/quant/test_fused_rms_fp8_group_quant.py:23-52,84-95.
 *   v = f32(x1) + f32(res1);  res_out = cast(v);  y = v * rsqrt(mean(v^2) + eps1) * w1;  y1_unquantized = cast(y);
 *   per 128 columns: amax = max(max|y|, 1e-10), y1_s = amax / 448, y1_q = e4m3(clamp(y * (1 / y1_s), +-448));
 *   y2 = cast(x2 * rsqrt(mean(x2^2) + eps2) * w2).
 * x1 [M, N1] and x2 [M, N2] F16/BF16 with row strides in elements (views into a wider projection output are
 * fine); res1, res_out, y1_unquantized [M, N1] and y2 [M, N2] contiguous in the same dtype; y1_q [M, N1]
 * e4m3fn; y1_s fp32 [M, ceil(N1/128)] row-major; w1 [N1], w2 [N2] of weight_dtype (F32/F16/BF16).
 * res1, y1_unquantized and the whole second input are optional (NULL); res_out is required with res1.
 * N1, N2 multiples of 8 and at most 16384; group_size must be 128. */
int sglamd_fused_rms_fp8_group_quant(const void* x1, int64_t x1_row_stride, const void* w1, float eps1,
                                     const void* res1, int64_t M, int64_t N1, void* y1_q, float* y1_s,
                                     void* y1_unquantized, void* res_out, const void* x2, int64_t x2_row_stride,
                                     const void* w2, float eps2, int64_t N2, void* y2, int dtype, int weight_dtype,
                                     int group_size, void* stream);

/* The whole block-FP8 MoE layer from one host call (five launches on `stream`):
 *   quantise hidden (1x128 groups) + moe_align_block_size -> grouped GEMM with w13 -> silu*mul + quantise
 *   -> grouped GEMM with w2 (x routing weight) -> sum over top-k (x routed_scaling_factor).
 * Up to four tokens the activation step runs inside the two GEMMs, and a single token's sorting and quantising
 * too (four and three launches); where the sorted blocks are 128 or 192 slots tall and outnumber the compute
 * units, the first GEMM's epilogue applies silu*mul and the quantisation and writes the second GEMM's operand
 * (four launches, the same bits as the five).  The decode forms compute what the five-launch sequence computes; the bits are the
 * same when both split and walk K alike, which holds when 2I and H are at least 2048 and multiples of 32 (two
 * column tiles per workgroup in either form) and the plain launch shares K among at most four waves, as at the
 * DeepSeek-V3 dimensions; otherwise the fp32 partial sums meet in another order and the results agree to fp32
 * rounding before the 16-bit output.
 * Stands in for fused_experts_impl / _fused_moe_kernel_sequence
 * (python/sglang/srt/layers/moe/moe_runner/triton_utils/fused_moe.py:401-893) in its use_fp8_w8a8,
 * block_shape [128,128], gated-SiLU configuration.
 * hidden [M, H] F16/BF16 contiguous; w13 e4m3fn [E, 2I, H], w13_scale fp32 [E, 2I/128, H/128];
 * w2 e4m3fn [E, H, I], w2_scale [E, H/128, I/128] (all contiguous); topk_weights fp32 [M, topk];
 * topk_ids int32/int64 [M, topk] (-1 = expert not on this rank); out [M, H]; H % 128 == 0, I % 128 == 0.
 * block_m: sorted-block height (16/32/64/128/192) or 0 to choose from M*topk/E.
 * workspace: caller-provided device scratch of at least sglamd_fused_moe_block_fp8_workspace(...) bytes,
 * 256-byte aligned; nothing is allocated here. */
int64_t sglamd_fused_moe_block_fp8_workspace(int64_t M, int64_t H, int64_t I, int E, int topk, int block_m);
int sglamd_fused_moe_block_fp8(const void* hidden, int dtype, int64_t M, int64_t H, int64_t I, int E, int topk,
                               const void* w13, const float* w13_scale, const void* w2, const float* w2_scale,
                               const float* topk_weights, const void* topk_ids, int ids_dtype, void* out,
                               float routed_scaling_factor, int block_m, void* workspace, int64_t workspace_bytes,
                               void* stream);

/* sglamd_fused_moe_block_fp8 for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments and results
 * as sglamd_fused_moe_block_fp8, without the workspace: the intermediates live in a 16 MiB device array that is
 * part of the library image (sglamd_fused_moe_block_fp8_static_max_bytes(); every GPU the library runs on holds
 * it until the process ends), which covers decode-sized batches (DeepSeek-V3 layer: M <= 64).  A call whose
 * sglamd_fused_moe_block_fp8_workspace(...) exceeds the array fails with SGLAMD_EINVAL before anything is
 * launched.  Nothing in the array has to start at zero: every launch writes what the next one reads.  All
 * calls on one GPU share the array: calls that overlap on one GPU (two streams, two threads) race; calls on one
 * stream are ordered.  Calls no hipMalloc / hipFree; the array's device address is looked up on the first call
 * on each device. */
int64_t sglamd_fused_moe_block_fp8_static_max_bytes(void);
int sglamd_fused_moe_block_fp8_static(const void* hidden, int dtype, int64_t M, int64_t H, int64_t I, int E, int topk,
                                      const void* w13, const float* w13_scale, const void* w2, const float* w2_scale,
                                      const float* topk_weights, const void* topk_ids, int ids_dtype, void* out,
                                      float routed_scaling_factor, int block_m, void* stream);

/* ------------------------------------------------------------------------------------
 * Expert-major ("grouped") MoE interface: the alternative MoE backend of the reference
 * (python/sglang/srt/layers/moe/cutlass_moe.py:29-341), whose rows are physically permuted
 * into one contiguous span per expert.
 * ------------------------------------------------------------------------------------ */

/* Stands in for prepare_moe_input (sgl-kernel/csrc/moe/prepare_moe_input.cu:12-175; schema
 * sgl-kernel/csrc/common_extension.cc:205-209).  topk_ids int32 [numel] = [tokens, topk] flattened.
 *   problem_sizes1[e] = (rows_e, 2n, k), problem_sizes2[e] = (rows_e, k, n), rows_e = #{i: topk_ids[i] == e};
 *   expert_offsets[0..E] = exclusive prefix of rows_e (and the total);
 *   blockscale_offsets[0..E] (optional, may be NULL) = the same prefix with every rows_e rounded up to 128;
 *   input_permutation[pos] = i / topk and output_permutation[i] = pos, pos running over expert e's span in
 *   ascending i (the reference fills a span in the order its atomics land: any order is valid there, this
 *   one is deterministic).  Ids outside [0, E) take no part and leave output_permutation[i] untouched. */
int sglamd_prepare_moe_input(const int32_t* topk_ids, int64_t numel, int topk, int num_experts, int64_t n, int64_t k,
                             int32_t* expert_offsets, int32_t* blockscale_offsets, int32_t* problem_sizes1,
                             int32_t* problem_sizes2, int32_t* input_permutation, int32_t* output_permutation,
                             void* stream);

/* Stands in for shuffle_rows (prepare_moe_input.cu:165-246; schema common_extension.cc:211-212):
 * output row r = input row dst2src_map[r], rows of row_bytes bytes of any element type. */
int sglamd_shuffle_rows(const void* input, const int32_t* dst2src_map, void* output, int64_t num_dst_rows,
                        int64_t row_bytes, void* stream);

/* Stands in for apply_shuffle_mul_sum (prepare_moe_input.cu:248-376; schema common_extension.cc:214-215):
 *   output[i, :] = cast( sum_{j < topk} f32(factors[i*topk + j]) * f32(input[permutation[i*topk + j], :]) ),
 * fp32 accumulation in ascending j; factors (same dtype as input/output: F16 or BF16) may be NULL (all ones).
 * input [m*topk, row_stride], output [m, row_stride], both contiguous. */
int sglamd_apply_shuffle_mul_sum(const void* input, void* output, const int32_t* permutation, const void* factors,
                                 int dtype, int64_t m, int topk, int64_t row_stride, void* stream);

/* Stands in for fp8_blockwise_scaled_grouped_mm (sgl-kernel/csrc/moe/fp8_blockwise_moe_kernel.cu:650-810,
 * per-expert addressing sgl-kernel/csrc/moe/cutlass_moe_helper.cu:17-75; schema common_extension.cc:198-203):
 * for every expert e with rows_e = problem_sizes[e][0] rows starting at row expert_offsets[e]:
 *   output[r, :] = cast( sum_kb (a[r, kb] . b[e, :, kb]) * scales_a[r, kb] * scales_b[e, n/128, kb] ).
 * a e4m3fn [total_rows, K] contiguous; b e4m3fn [E, N, K] contiguous (the operator's [E, K, N] column-major
 * view); scales_a fp32 [total_rows, K/128]; scales_b fp32 [E, N/128, K/128] contiguous; output
 * [total_rows, N] F16/BF16; N % 128 == 0, K % 128 == 0.  Rows outside every expert's span are not written.
 * The reference's pointer and layout containers (a_ptrs ... layout_sfb) are CUTLASS scratch and have no
 * counterpart; workspace: at least sglamd_grouped_mm_workspace_bytes(total_rows, num_experts) bytes,
 * 16-byte aligned (the sorted-block schedule is built there; the reference passes a workspace too). */
int64_t sglamd_grouped_mm_workspace_bytes(int64_t total_rows, int num_experts);
int sglamd_fp8_blockwise_scaled_grouped_mm(void* output, int out_dtype, const void* a, const void* b,
                                           const float* scales_a, const float* scales_b, const int32_t* problem_sizes,
                                           const int32_t* expert_offsets, int num_experts, int64_t total_rows,
                                           int64_t N, int64_t K, void* workspace, int64_t workspace_bytes,
                                           void* stream);

/* ------------------------------------------------------------------------------------
 * Measured ceilings (no counterpart in the reference; launched by the benchmark only): bare loops that show what
 * the GPU gives a kernel at best, for reading the roofline fractions against.
 * sglamd_ceiling_mfma: 256 workgroups x 8 waves, each wave `iters` rounds of 8 MFMA tiles 32x32x64 (FP8:
 *   v_mfma_f32_32x32x64_f8f6f4; int8 != 0: pairs of v_mfma_i32_32x32x32_i8), operands in registers, either one
 *   constant byte or hashed bytes (random_operands != 0).  Operations per launch:
 *   256 * 8 * iters * 8 * 131072.  out: 256*512 floats of device memory (receives checksums).
 * sglamd_ceiling_hbm: dst == NULL: reads `bytes` from src with 16-byte nontemporal loads (sink: one int of device
 *   memory the kernel may write); else copies src to dst.  Buffers 16-byte aligned, bytes % 16 == 0.
 * sglamd_ceiling_hbm_lds: reads `bytes` (whole KB) of src the way the weight-streaming GEMMs fetch their operands:
 *   one workgroup per CU, eight waves each keeping sixteen 1 KB direct-to-LDS loads in flight over a contiguous
 *   share; nothing is computed or written.  The read ceiling of those kernels at the same byte count.
 * sglamd_ceiling_l2_read: one workgroup per CU (eight waves) reads its own 64 KB of src `passes` times over, so
 *   that after the first pass every load is answered by L2: through direct-to-LDS loads of 1 KB (lds != 0) or
 *   through 16-byte register loads, eight in flight per wave either way.  src holds at least 64 KB per CU;
 *   bytes moved per launch: passes * CUs * 65536.  The rate at which a CU can take operands in, whatever HBM gives.
 * sglamd_ceiling_gemm_l2_resident: the persistent 256x256 block-FP8 GEMM kernel of sglamd_fp8_blockwise_scaled_mm
 *   with every tile reading the operand panels of tile (0, 0): a, b are [256, K] e4m3 bytes, sa [K/128][256] and
 *   sb [2][K/128] floats, out [M, N] bf16 (written like the real kernel writes it; the values are those of tile
 *   (0, 0) repeated).  Same MFMA, LDS, load, barrier and store stream as the operator on an L2-resident working
 *   set; 2*M*N*K operations per launch.  Needs more 256x256 tiles than CUs, K/128 even in 4..256, N % 8 == 0. */
int sglamd_ceiling_mfma(int int8, int random_operands, int iters, float* out, void* stream);
int sglamd_ceiling_hbm(void* dst, const void* src, int64_t bytes, int* sink, void* stream);
int sglamd_ceiling_hbm_lds(const void* src, int64_t bytes, void* stream);
int sglamd_ceiling_l2_read(const void* src, int64_t bytes, int passes, int lds, int* sink, void* stream);
int sglamd_ceiling_gemm_l2_resident(const void* a, const void* b, const float* sa, const float* sb, void* out,
                                    int64_t M, int64_t N, int64_t K, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SGLAMD_H_ */
