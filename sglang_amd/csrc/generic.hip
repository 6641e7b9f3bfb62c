// Configurations of the path that the specialised kernels do not take, on the register-staged generic GEMM kernel
// (gemm_core.h): block-scaled GEMMs and fused-MoE grouped GEMMs with scale blocks of 64 or 128 in either direction,
// and the per-token / per-channel and per-tensor scaled forms of the fused-MoE grouped GEMM, with optional bias.
// Also the sigmoid router (topk_sigmoid), the twin of topk_softmax in moe.hip.
#include <math.h>

#include "gemm_core.h"

namespace sglamd {

// tile height of the generic kernel by the rows it will see
template <int MODE, typename OT, bool MOE>
static int generic_launch(const GemmArgsX& g, int bm, hipStream_t st) {
  switch (bm) {
    case 16:
      return gemm8_launch<16, 128, 1, 2, MODE, OT, MOE, GemmArgsX>(g, st);
    case 32:
      return gemm8_launch<32, 128, 1, 2, MODE, OT, MOE, GemmArgsX>(g, st);
    case 64:
      return gemm8_launch<64, 128, 2, 2, MODE, OT, MOE, GemmArgsX>(g, st);
    default:
      return gemm8_launch<128, 128, 2, 2, MODE, OT, MOE, GemmArgsX>(g, st);
  }
}

template <int MODE, bool MOE>
static int generic_out(const GemmArgsX& g, int bm, int out_dtype, hipStream_t st) {
  if (out_dtype == SGLAMD_BF16) return generic_launch<MODE, BF16, MOE>(g, bm, st);
  if (out_dtype == SGLAMD_F16) return generic_launch<MODE, F16, MOE>(g, bm, st);
  return fail(SGLAMD_EINVAL, "out_dtype must be Half or BFloat16");
}

// ---------------------------------------------------------------------------------------
// topk_sigmoid: one wavefront per token, lane l holds experts l, l + 64, ...  score = 1 / (1 + exp(-x)) (+ bias for
// the choice only: the written weight is the biased score minus the bias, as the reference computes it); k rounds
// of (value, lower index wins) arg-max by butterfly shuffles; optional division by the sum of the picked weights.
// ---------------------------------------------------------------------------------------
template <typename T, int EPL>
__global__ __launch_bounds__(256) void topk_sigmoid_kernel(const typename T::storage* __restrict__ gating,
                                                           float* __restrict__ weights, int32_t* __restrict__ ids,
                                                           int num_tokens, int num_experts, int topk, int renormalize,
                                                           const float* __restrict__ bias) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= num_tokens) return;
  const typename T::storage* g = gating + (int64_t)row * num_experts;
  float v[EPL];
#pragma unroll
  for (int j = 0; j < EPL; j++) {
    const int e = lane + 64 * j;
    float x = -10000.f;  // scores lie in (0, 1) (+ bias): an absent expert never wins against a present one
    if (e < num_experts) {
      x = 1.0f / (1.0f + expf(-T::to_f32(g[e])));
      if (bias) x = x + bias[e];
    }
    v[j] = x;
  }
  float picked = 0.f;  // lane k keeps the k-th pick
  int picked_id = 0;
  float total = 0.f;
  for (int k = 0; k < topk; k++) {
    float best = v[0];
    int best_e = lane;
#pragma unroll
    for (int j = 1; j < EPL; j++) {
      if (v[j] > best) {
        best = v[j];
        best_e = lane + 64 * j;
      }
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
      const float ob = __shfl_xor(best, off, 64);
      const int oe = __shfl_xor(best_e, off, 64);
      if (ob > best || (ob == best && oe < best_e)) {
        best = ob;
        best_e = oe;
      }
    }
    if ((best_e & 63) == lane) {
#pragma unroll
      for (int j = 0; j < EPL; j++)
        if (j == (best_e >> 6)) v[j] = -20000.f;
    }
    const float w = bias ? best - bias[best_e] : best;
    if (lane == (k & 63)) {
      picked = w;
      picked_id = best_e;
    }
    total += w;
    if ((k & 63) == 63 || k == topk - 1) {
      const int base = k & ~63;
      if (base + lane <= k) {
        weights[(int64_t)row * topk + base + lane] = picked;
        ids[(int64_t)row * topk + base + lane] = picked_id;
      }
    }
  }
  if (renormalize) {
    // every lane holds the same total; lane l re-reads exactly the entries it wrote itself (l, l + 64, ...)
    const float inv = 1.f / total;
    for (int k = lane; k < topk; k += 64) weights[(int64_t)row * topk + k] *= inv;
  }
}

// ---------------------------------------------------------------------------------------
// Largest magnitude of a tensor in two deterministic steps (no atomics, nothing to zero): every workgroup writes
// the maximum of its grid-stride share, one workgroup reduces those and writes max(amax, eps) / fp8_max.
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void absmax_partial_kernel(const typename T::storage* __restrict__ x, int64_t n,
                                                             float* __restrict__ partial) {
  __shared__ float s_max[4];
  float m = 0.f;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256)
    m = fmaxf(m, fabsf(T::to_f32(x[i])));
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
  if ((threadIdx.x & 63) == 0) s_max[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) partial[blockIdx.x] = fmaxf(fmaxf(s_max[0], s_max[1]), fmaxf(s_max[2], s_max[3]));
}

__global__ __launch_bounds__(256) void absmax_scale_kernel(const float* __restrict__ partial, int count, float eps,
                                                           float fp8_max, float* __restrict__ scale) {
  __shared__ float s_max[4];
  float m = 0.f;
  for (int i = threadIdx.x; i < count; i += 256) m = fmaxf(m, partial[i]);
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
  if ((threadIdx.x & 63) == 0) s_max[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0)
    scale[0] = fmaxf(fmaxf(fmaxf(s_max[0], s_max[1]), fmaxf(s_max[2], s_max[3])), eps) / fp8_max;
}

}  // namespace sglamd

using namespace sglamd;

extern "C" int sglamd_tensor_absmax_scale(const void* input, int in_dtype, int64_t numel, float eps, float fp8_max,
                                          float* scale, float* workspace, void* stream) {
  SGLAMD_REQUIRE(input && scale && workspace, SGLAMD_EINVAL, "tensor_absmax_scale: null pointer");
  SGLAMD_REQUIRE(numel > 0 && fp8_max > 0.f, SGLAMD_EINVAL, "tensor_absmax_scale: bad sizes");
  SGLAMD_REQUIRE(in_dtype == SGLAMD_F32 || in_dtype == SGLAMD_F16 || in_dtype == SGLAMD_BF16, SGLAMD_EINVAL,
                 "tensor_absmax_scale: input must be float32, float16 or bfloat16");
  hipStream_t st = (hipStream_t)stream;
  const int64_t want = ceil_div(numel, 256 * 16);
  const unsigned blocks = (unsigned)(want < 1 ? 1 : want > 1024 ? 1024 : want);
  if (in_dtype == SGLAMD_F32)
    hipLaunchKernelGGL(absmax_partial_kernel<F32>, dim3(blocks), dim3(256), 0, st, (const float*)input, numel, workspace);
  else if (in_dtype == SGLAMD_F16)
    hipLaunchKernelGGL(absmax_partial_kernel<F16>, dim3(blocks), dim3(256), 0, st, (const u16*)input, numel, workspace);
  else
    hipLaunchKernelGGL(absmax_partial_kernel<BF16>, dim3(blocks), dim3(256), 0, st, (const u16*)input, numel, workspace);
  int rc = check_launch("tensor_absmax(partial)");
  if (rc) return rc;
  hipLaunchKernelGGL(absmax_scale_kernel, dim3(1), dim3(256), 0, st, (const float*)workspace, (int)blocks, eps, fp8_max,
                     scale);
  return check_launch("tensor_absmax(scale)");
}

extern "C" int sglamd_topk_sigmoid(float* topk_weights, int32_t* topk_indices, const void* gating_output, int g_dtype,
                                  int64_t num_tokens, int64_t num_experts, int64_t topk, int renormalize,
                                  const float* correction_bias, void* stream) {
  SGLAMD_REQUIRE(topk_weights && topk_indices && gating_output, SGLAMD_EINVAL, "topk_sigmoid: null pointer");
  SGLAMD_REQUIRE(num_tokens >= 0 && num_experts > 0 && topk > 0, SGLAMD_EINVAL, "topk_sigmoid: bad sizes");
  SGLAMD_REQUIRE(topk <= num_experts, SGLAMD_EINVAL, "topk must be less than or equal to num_experts");
  SGLAMD_REQUIRE(num_experts <= 1024, SGLAMD_ENOTSUP, "topk_sigmoid: more than 1024 experts");
  SGLAMD_REQUIRE(g_dtype == SGLAMD_F32 || g_dtype == SGLAMD_F16 || g_dtype == SGLAMD_BF16, SGLAMD_EINVAL,
                 "gating_output must be float32, float16, or bfloat16");
  if (num_tokens == 0) return SGLAMD_OK;
  hipStream_t st = (hipStream_t)stream;
  const unsigned blocks = (unsigned)ceil_div(num_tokens, 4);
#define SGLAMD_TOPK(TT, E)                                                                                             \
  hipLaunchKernelGGL((topk_sigmoid_kernel<TT, E>), dim3(blocks), dim3(256), 0, st,                                     \
                     (const typename TT::storage*)gating_output, topk_weights, topk_indices, (int)num_tokens,          \
                     (int)num_experts, (int)topk, renormalize, correction_bias)
#define SGLAMD_TOPK_E(TT)                                                                                              \
  do {                                                                                                                 \
    if (num_experts <= 64) SGLAMD_TOPK(TT, 1);                                                                         \
    else if (num_experts <= 128) SGLAMD_TOPK(TT, 2);                                                                   \
    else if (num_experts <= 256) SGLAMD_TOPK(TT, 4);                                                                   \
    else if (num_experts <= 512) SGLAMD_TOPK(TT, 8);                                                                   \
    else SGLAMD_TOPK(TT, 16);                                                                                          \
  } while (0)
  if (g_dtype == SGLAMD_F32) SGLAMD_TOPK_E(F32);
  else if (g_dtype == SGLAMD_F16) SGLAMD_TOPK_E(F16);
  else SGLAMD_TOPK_E(BF16);
#undef SGLAMD_TOPK_E
#undef SGLAMD_TOPK
  return check_launch("topk_sigmoid");
}

static int check_block_shape(const char* op, int block_n, int block_k) {
  SGLAMD_REQUIRE((block_n == 64 || block_n == 128) && (block_k == 64 || block_k == 128), SGLAMD_ENOTSUP,
                 "%s: scale blocks of 64 or 128 in each direction are implemented (got [%d, %d])", op, block_n, block_k);
  return SGLAMD_OK;
}

extern "C" int sglamd_block_scaled_mm_any(const void* a, int64_t lda, const void* b, int64_t ldb, const float* sa,
                                          int64_t sa_stride_m, int64_t sa_stride_k, const float* sb,
                                          int64_t sb_stride_n, int64_t sb_stride_k, void* out, int64_t ldc,
                                          int out_dtype, int q_dtype, int64_t M, int64_t N, int64_t K, int block_n,
                                          int block_k, void* stream) {
  const char* op = "block_scaled_mm_any";
  SGLAMD_REQUIRE(a && b && sa && sb && out, SGLAMD_EINVAL, "%s: null pointer", op);
  SGLAMD_REQUIRE(M >= 0 && N > 0 && K > 0 && M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31), SGLAMD_EINVAL,
                 "%s: bad sizes", op);
  SGLAMD_REQUIRE(K % 16 == 0 && lda >= K && ldb >= K && ldc >= N && lda % 16 == 0 && ldb % 16 == 0, SGLAMD_EINVAL,
                 "%s: K and the row strides must be multiples of 16 bytes", op);
  SGLAMD_REQUIRE(((uintptr_t)a % 16) == 0 && ((uintptr_t)b % 16) == 0, SGLAMD_EINVAL, "%s: operands must be 16-byte aligned", op);
  SGLAMD_REQUIRE(q_dtype == SGLAMD_FP8_E4M3 || q_dtype == SGLAMD_I8, SGLAMD_EINVAL, "%s: operands must be e4m3fn or int8", op);
  int rc = check_block_shape(op, block_n, block_k);
  if (rc) return rc;
  if (M == 0) return SGLAMD_OK;
  GemmArgs g = {};
  g.A = (const uint8_t*)a;
  g.lda = lda;
  g.B = (const uint8_t*)b;
  g.ldb = ldb;
  g.sa = sa;
  g.sa_sm = sa_stride_m;
  g.sa_sk = sa_stride_k;
  g.sb = sb;
  g.sb_sn = sb_stride_n;
  g.sb_sk = sb_stride_k;
  g.C = out;
  g.ldc = ldc;
  g.M = (int)M;
  g.N = (int)N;
  g.K = (int)K;
  const GemmArgsX gx = {g, GemmExt{block_n, block_k, 1, 1, 0}};
  const int bm = M <= 16 ? 16 : M <= 32 ? 32 : M <= 64 ? 64 : 128;
  if (q_dtype == SGLAMD_I8) return generic_out<GEMM_BLOCK_INT8, false>(gx, bm, out_dtype, (hipStream_t)stream);
  return generic_out<GEMM_BLOCK_FP8, false>(gx, bm, out_dtype, (hipStream_t)stream);
}

extern "C" int sglamd_fused_moe_gemm_any(const void* a, int64_t lda, const float* a_scale, int64_t as_stride_m,
                                         int64_t as_stride_k, const void* w, int64_t w_stride_e, int64_t w_stride_n,
                                         const float* w_scale, int64_t ws_stride_e, int64_t ws_stride_n,
                                         int64_t ws_stride_k, const void* bias, int64_t bias_stride_e, void* c,
                                         int64_t ldc, int out_dtype, int q_dtype, int block_n, int block_k,
                                         const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                         const int32_t* num_tokens_post_padded, const float* topk_weights,
                                         int64_t num_valid_tokens, int top_k, int mul_routed_weight, int block_m,
                                         int64_t max_m_blocks, int64_t N, int64_t K, void* stream) {
  const char* op = "fused_moe_gemm_any";
  SGLAMD_REQUIRE(a && a_scale && w && w_scale && c && sorted_token_ids && expert_ids && num_tokens_post_padded,
                 SGLAMD_EINVAL, "%s: null pointer", op);
  SGLAMD_REQUIRE(!mul_routed_weight || topk_weights, SGLAMD_EINVAL, "%s: topk_weights missing", op);
  SGLAMD_REQUIRE(N > 0 && K > 0 && K % 16 == 0 && N < (1ll << 31) && K < (1ll << 31), SGLAMD_EINVAL, "%s: bad N/K", op);
  SGLAMD_REQUIRE(top_k >= 1 && num_valid_tokens >= 0 && num_valid_tokens < (1ll << 31), SGLAMD_EINVAL,
                 "%s: bad top_k / num_valid_tokens", op);
  SGLAMD_REQUIRE(lda % 16 == 0 && w_stride_n % 16 == 0 && w_stride_e % 16 == 0, SGLAMD_EINVAL,
                 "%s: strides must be multiples of 16 bytes", op);
  SGLAMD_REQUIRE(((uintptr_t)a % 16) == 0 && ((uintptr_t)w % 16) == 0, SGLAMD_EINVAL, "%s: operands must be 16-byte aligned", op);
  SGLAMD_REQUIRE(max_m_blocks >= 0 && max_m_blocks < (1ll << 24), SGLAMD_EINVAL, "%s: bad block count", op);
  SGLAMD_REQUIRE(q_dtype == SGLAMD_FP8_E4M3 || q_dtype == SGLAMD_I8, SGLAMD_EINVAL, "%s: operands must be e4m3fn or int8", op);
  SGLAMD_REQUIRE(block_m == 16 || block_m == 32 || block_m == 64 || block_m == 128, SGLAMD_EINVAL,
                 "%s: block_m must be 16, 32, 64 or 128 (got %d)", op, block_m);
  const bool row = block_n == 0 && block_k == 0;
  if (!row) {
    int rc = check_block_shape(op, block_n, block_k);
    if (rc) return rc;
  }
  if (max_m_blocks == 0 || num_valid_tokens == 0) return SGLAMD_OK;
  GemmArgs g = {};
  g.A = (const uint8_t*)a;
  g.lda = lda;
  g.B = (const uint8_t*)w;
  g.ldb = w_stride_n;
  g.b_expert_stride = w_stride_e;
  g.sa = a_scale;
  g.sa_sm = as_stride_m;
  g.sa_sk = as_stride_k;
  g.sb = w_scale;
  g.sb_se = ws_stride_e;
  g.sb_sn = ws_stride_n;
  g.sb_sk = ws_stride_k;
  g.bias = bias;
  g.C = c;
  g.ldc = ldc;
  g.M = (int)num_valid_tokens;
  g.N = (int)N;
  g.K = (int)K;
  g.sorted_ids = sorted_token_ids;
  g.expert_ids = expert_ids;
  g.num_post_pad = num_tokens_post_padded;
  g.topk_w = topk_weights;
  g.top_k = top_k;
  g.num_valid = (int)num_valid_tokens;
  g.mul_weight = mul_routed_weight;
  g.max_blocks_m = (int)max_m_blocks;
  hipStream_t st = (hipStream_t)stream;
  const GemmArgsX gx = {g, GemmExt{block_n, block_k, as_stride_m, ws_stride_n, bias_stride_e}};
  if (row) {
    if (q_dtype == SGLAMD_I8) return generic_out<GEMM_ROW_INT8, true>(gx, block_m, out_dtype, st);
    return generic_out<GEMM_ROW_FP8, true>(gx, block_m, out_dtype, st);
  }
  if (q_dtype == SGLAMD_I8) return generic_out<GEMM_BLOCK_INT8, true>(gx, block_m, out_dtype, st);
  return generic_out<GEMM_BLOCK_FP8, true>(gx, block_m, out_dtype, st);
}
