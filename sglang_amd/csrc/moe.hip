// Fused-MoE side of the path for gfx950: moe_align_block_size (stable counting sort into
// block-padded expert spans), the sorted-block grouped block-FP8 GEMM (same MFMA core as
// the dense GEMM, rows gathered through the sorted token list), silu_and_mul and the
// top-k sum reduce.
#include "gemm_big.h"
#include "gemm_skinny.h"
#include "quant_core.h"

namespace sglamd {

// ---------------------------------------------------------------------------------------
// moe_align_block_size: one workgroup of 1024 lanes.
//   1. every wave histograms its own contiguous chunk of the flat ids (bucket = id + 1) in LDS,
//   2. padded totals -> exclusive prefix P (wave scans + carry),
//   3. expert id of every block, total, cumsum buffer, padding fill; the per-wave counts are
//      turned into each wave's first slot per bucket (P[b] + counts of the waves in front),
//   4. stable scatter without workgroup barriers: a wave walks its chunk 64 ids at a time; a
//      lane's slot is the wave's running offset of the bucket plus the same-bucket lanes in
//      front of it, so every span is filled in ascending flat index.
// LDS: cnt[NB] | prefix[NB+1] | wavecnt[16][NB]   (NB = number of buckets)
// ---------------------------------------------------------------------------------------
template <typename IdT>
__device__ __forceinline__ void moe_align_body(const IdT* __restrict__ topk_ids, int32_t* sorted_ids,
                                               int32_t* expert_ids, int32_t* post_pad_out, int32_t* cumsum_out, int nb,
                                               int block_size, int numel, int pad_fill, int max_padded) {
  extern __shared__ int32_t lds[];
  int32_t* cnt = lds;
  int32_t* prefix = cnt + nb;
  int32_t* wavecnt = prefix + nb + 1;
  __shared__ int32_t s_carry;
  __shared__ int32_t s_wsum[16];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  for (int i = tid; i < 16 * nb; i += 1024) wavecnt[i] = 0;
  if (tid == 0) s_carry = 0;
  __syncthreads();

  // Every wave owns one contiguous chunk of the flat ids (a multiple of 64 long), so ascending flat index
  // is wave order first, position inside the wave's chunk second.
  const int chunk = ((numel + 15) / 16 + 63) & ~63;
  const int c_begin = wave * chunk, c_end = min(numel, c_begin + chunk);
  int32_t* mycnt = wavecnt + wave * nb;
  for (int i = c_begin + lane; i < c_end; i += 64) {
    const int b = (int)topk_ids[i] + 1;
    if (b >= 0 && b < nb) atomicAdd(&mycnt[b], 1);
  }
  __syncthreads();
  for (int b = tid; b < nb; b += 1024) {
    int t = 0;
    for (int w = 0; w < 16; w++) t += wavecnt[w * nb + b];
    cnt[b] = t;
  }
  __syncthreads();

  // exclusive scan of the padded counts, 1024 buckets per round
  for (int base = 0; base < nb; base += 1024) {
    const int b = base + tid;
    const int padded = b < nb ? (cnt[b] + block_size - 1) / block_size * block_size : 0;
    int incl = padded;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int v = __shfl_up(incl, off, 64);
      if (lane >= off) incl += v;
    }
    if (lane == 63) s_wsum[wave] = incl;
    __syncthreads();
    int woff = 0;
    for (int w = 0; w < wave; w++) woff += s_wsum[w];
    const int carry = s_carry;
    if (b < nb) prefix[b] = carry + woff + incl - padded;
    __syncthreads();
    if (tid == 1023) s_carry = carry + woff + incl;
    __syncthreads();
  }
  if (tid == 0) {
    prefix[nb] = s_carry;
    *post_pad_out = s_carry;
  }
  __syncthreads();

  const int post_pad = prefix[nb];
  for (int b = tid; b < nb; b += 1024) {
    // per-wave counts become the slot at which each wave starts writing bucket b
    int running = prefix[b];
    for (int w = 0; w < 16; w++) {
      const int t = wavecnt[w * nb + b];
      wavecnt[w * nb + b] = running;
      running += t;
    }
    for (int j = prefix[b] / block_size; j < prefix[b + 1] / block_size; j++) expert_ids[j] = b - 1;
    if (cumsum_out) cumsum_out[b] = prefix[b] + cnt[b];
    if (pad_fill)
      for (int j = prefix[b] + cnt[b]; j < prefix[b + 1]; j++) sorted_ids[j] = numel;
  }
  if (cumsum_out && tid == 0) cumsum_out[nb] = post_pad;
  if (pad_fill)
    for (int j = post_pad + tid; j < max_padded; j += 1024) sorted_ids[j] = numel;
  __syncthreads();

  // Stable scatter, one wave per chunk and no workgroup barrier: 64 ids at a time, a lane's slot is its wave's
  // running offset for the bucket plus the number of same-bucket lanes in front of it.
  volatile int32_t* myoff = mycnt;
  const int key_bits = 32 - __clz(max(nb - 1, 1));
  for (int base = c_begin; base < c_end; base += 64) {
    const int i = base + lane;
    int b = -1;
    if (i < c_end) {
      b = (int)topk_ids[i] + 1;
      if (b < 0 || b >= nb) b = -1;
    }
    // lanes of this wave with the same bucket: intersect, bit by bit of the bucket number, the lanes that agree
    unsigned long long m = __ballot(b >= 0);
    for (int k = 0; k < key_bits; k++) {
      const bool bit = (b >> k) & 1;
      const unsigned long long bal = __ballot(bit);
      m &= bit ? bal : ~bal;
    }
    const int rank = __popcll(m & ((1ull << lane) - 1ull));
    const int total = __popcll(m);
    const bool leader = b >= 0 && rank == 0;
    int off = 0;
    if (b >= 0) off = myoff[b];
    __builtin_amdgcn_wave_barrier();
    if (leader) myoff[b] = off + total;
    if (b >= 0) sorted_ids[off + rank] = i;
  }
}

template <typename IdT>
__global__ __launch_bounds__(1024) void moe_align_kernel(const IdT* __restrict__ topk_ids, int32_t* sorted_ids,
                                                         int32_t* expert_ids, int32_t* post_pad_out,
                                                         int32_t* cumsum_out, int nb, int block_size, int numel,
                                                         int pad_fill, int max_padded) {
  moe_align_body<IdT>(topk_ids, sorted_ids, expert_ids, post_pad_out, cumsum_out, nb, block_size, numel, pad_fill,
                      max_padded);
}

// First launch of the fused MoE layer: workgroup 0 sorts the tokens, the others quantise the hidden
// states (group 128, reciprocal form).  The two jobs are independent, so sharing a launch only removes
// one launch latency from the decode path.
template <typename IdT, typename T>
__global__ __launch_bounds__(1024) void moe_prologue_kernel(const IdT* __restrict__ topk_ids, int32_t* sorted_ids,
                                                            int32_t* expert_ids, int32_t* post_pad_out,
                                                            int32_t* cumsum_out, int nb, int block_size, int numel,
                                                            int max_padded, GroupQuantArgs qa) {
  if (blockIdx.x == 0) {
    moe_align_body<IdT>(topk_ids, sorted_ids, expert_ids, post_pad_out, cumsum_out, nb, block_size, numel, 1, max_padded);
  } else {
    group_quant_body<T, 128>(qa, (int64_t)(blockIdx.x - 1) * 1024 + threadIdx.x);
  }
}

// ---------------------------------------------------------------------------------------
// topk_softmax: routing of one token per wavefront.  Lane l holds experts l, l + 64, ...; the logits are
// (optionally) soft-capped and biased, soft-maxed in fp32 (max and sum by butterfly shuffles), then k rounds
// of arg-max pick the largest remaining probability, the lower expert index winning ties; the winner's lane
// blanks its copy.  Optional renormalisation divides by the sum of the k picked probabilities.
// ---------------------------------------------------------------------------------------
template <typename T, int EPL>
__global__ __launch_bounds__(256) void topk_softmax_kernel(const typename T::storage* __restrict__ gating,
                                                           float* __restrict__ weights, int32_t* __restrict__ ids,
                                                           int num_tokens, int num_experts, int topk, int renormalize,
                                                           float softcap, const float* __restrict__ bias) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= num_tokens) return;
  const typename T::storage* g = gating + (int64_t)row * num_experts;
  float v[EPL];
  float vmax = -INFINITY;
#pragma unroll
  for (int j = 0; j < EPL; j++) {
    const int e = lane + 64 * j;
    float x = -INFINITY;
    if (e < num_experts) {
      x = T::to_f32(g[e]);
      if (softcap != 0.f) x = tanhf(x / softcap) * softcap;
      if (bias) x += bias[e];
    }
    v[j] = x;
    vmax = fmaxf(vmax, x);
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) vmax = fmaxf(vmax, __shfl_xor(vmax, off, 64));
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < EPL; j++) {
    v[j] = (lane + 64 * j) < num_experts ? expf(v[j] - vmax) : 0.f;
    sum += v[j];
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) sum += __shfl_xor(sum, off, 64);
  const float inv = 1.f / sum;
#pragma unroll
  for (int j = 0; j < EPL; j++) v[j] = (lane + 64 * j) < num_experts ? v[j] * inv : -1.f;

  float picked = 0.f;   // lane k keeps the k-th pick
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
        if (j == (best_e >> 6)) v[j] = -1.f;
    }
    if (lane == (k & 63)) {
      picked = best;
      picked_id = best_e;
    }
    total += best;
    if ((k & 63) == 63 || k == topk - 1) {
      // flush up to 64 picks (renormalisation needs the total, so only the last flush can apply it when topk <= 64)
      const int base = k & ~63;
      if (base + lane <= k) {
        weights[(int64_t)row * topk + base + lane] = picked;
        ids[(int64_t)row * topk + base + lane] = picked_id;
      }
    }
  }
  if (renormalize) {
    const float rinv = 1.f / total;
    for (int k = lane; k < topk; k += 64) weights[(int64_t)row * topk + k] *= rinv;
  }
}

// ---------------------------------------------------------------------------------------
// silu_and_mul: out[t, j] = T(silu_f32(x[t, j])) * x[t, d + j], product rounded to T.
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void silu_and_mul_kernel(const u16* __restrict__ in, u16* __restrict__ out, int d) {
  const int64_t t = blockIdx.x;
  const u16* g = in + t * 2 * (int64_t)d;
  const u16* u = g + d;
  u16* o = out + t * (int64_t)d;
  for (int j = threadIdx.x * 8; j < d; j += 256 * 8) {
    v4i gv = *(const v4i*)(g + j), uv = *(const v4i*)(u + j);
    u16 gb[8], ub[8], ob[8];
    __builtin_memcpy(gb, &gv, 16);
    __builtin_memcpy(ub, &uv, 16);
#pragma unroll
    for (int k = 0; k < 8; k++) {
      const float x = T::to_f32(gb[k]);
      const float s = T::to_f32(T::from_f32(x / (1.0f + expf(-x))));
      ob[k] = T::from_f32(s * T::to_f32(ub[k]));
    }
    v4i ov;
    __builtin_memcpy(&ov, ob, 16);
    *(v4i*)(o + j) = ov;
  }
}

// moe_sum_reduce: out[t, j] = T(scale * sum_k f32(in[t, k, j]))
template <typename T>
__global__ __launch_bounds__(256) void moe_sum_reduce_kernel(const u16* __restrict__ in, u16* __restrict__ out,
                                                             int topk, int d, float scale) {
  const int64_t t = blockIdx.x;
  const u16* src = in + t * (int64_t)topk * d;
  u16* o = out + t * (int64_t)d;
  for (int j = (blockIdx.y * 256 + threadIdx.x) * 8; j < d; j += gridDim.y * 256 * 8) {
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int k = 0; k < topk; k++) {
      v4i v = *(const v4i*)(src + (int64_t)k * d + j);
      u16 b[8];
      __builtin_memcpy(b, &v, 16);
#pragma unroll
      for (int e = 0; e < 8; e++) acc[e] += T::to_f32(b[e]);
    }
    u16 ob[8];
#pragma unroll
    for (int e = 0; e < 8; e++) ob[e] = T::from_f32(acc[e] * scale);
    v4i ov;
    __builtin_memcpy(&ov, ob, 16);
    *(v4i*)(o + j) = ov;
  }
}

template <int MODE, typename OT>
static int dispatch_moe_gemm(const GemmArgs& g, int block_m, hipStream_t st) {
  // number of sorted blocks that will actually run is data dependent; every valid slot could own one
  const int64_t expect = g.num_valid < g.max_blocks_m ? g.num_valid : g.max_blocks_m;
  switch (block_m) {
    case 16:
      return gemm8_skinny_launch<1, MODE, OT, true>(g, st, expect);
    case 32:
      return gemm8_skinny_launch<2, MODE, OT, true>(g, st, expect);
    case 64:
      return gemm8_skinny_launch<4, MODE, OT, true>(g, st, expect);
    case 128:
      // 32x32x64-MFMA tile kernel when its preconditions hold (K % 128 == 0, operands below 2 GiB per matrix)
      if ((g.K % 128) == 0 && (g.K >> 7) <= GEMM8_BIG_MAX_KB && (int64_t)(g.num_valid / g.top_k) * g.lda < 0x7fffffffll &&
          (int64_t)g.N * g.ldb < 0x7fffffffll)
        return gemm8_big_moe_launch<MODE, OT>(g, st);
      return gemm8_launch<128, 128, 2, 2, MODE, OT, true>(g, st);
    case 192:
      // one block per expert when an expert gets 129..192 rows: its weights are streamed once
      SGLAMD_REQUIRE((g.K % 128) == 0 && (g.K >> 7) <= GEMM8_BIG_MAX_KB && (int64_t)(g.num_valid / g.top_k) * g.lda < 0x7fffffffll &&
                         (int64_t)g.N * g.ldb < 0x7fffffffll,
                     SGLAMD_EINVAL, "fused_moe_gemm: block_m 192 needs K %% 128 == 0 and operands below 2 GiB");
      return gemm8_big_moe_launch<MODE, OT, 3>(g, st);
    default:
      return fail(SGLAMD_EINVAL, "fused_moe_gemm: block_m must be 16, 32, 64, 128 or 192 (got %d)", block_m);
  }
}

}  // namespace sglamd

using namespace sglamd;

extern "C" int sglamd_moe_align_block_size(const void* topk_ids, int ids_dtype, int64_t numel, int num_experts,
                                           int block_size, int32_t* sorted_token_ids, int64_t max_num_tokens_padded,
                                           int32_t* expert_ids, int32_t* num_tokens_post_pad, int32_t* cumsum_buffer,
                                           int pad_sorted_token_ids, void* stream) {
  SGLAMD_REQUIRE(topk_ids && sorted_token_ids && expert_ids && num_tokens_post_pad, SGLAMD_EINVAL,
                 "moe_align_block_size: null pointer");
  SGLAMD_REQUIRE(ids_dtype == SGLAMD_I32 || ids_dtype == SGLAMD_I64, SGLAMD_EINVAL,
                 "moe_align_block_size: topk_ids must be int32 or int64");
  SGLAMD_REQUIRE(numel >= 0 && numel < (1ll << 30), SGLAMD_EINVAL, "moe_align_block_size: bad numel");
  SGLAMD_REQUIRE(block_size > 0, SGLAMD_EINVAL, "moe_align_block_size: block_size must be positive");
  SGLAMD_REQUIRE(num_experts > 0 && num_experts <= 2048, SGLAMD_EINVAL,
                 "moe_align_block_size: num_experts (%d) must be in [1, 2048]", num_experts);
  const size_t lds = (size_t)(3 * num_experts + 1 + 16 * num_experts) * sizeof(int32_t);
  hipStream_t st = (hipStream_t)stream;
  if (ids_dtype == SGLAMD_I32) {
    auto k = moe_align_kernel<int32_t>;
    if (lds > 64 * 1024) hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL(k, dim3(1), dim3(1024), lds, st, (const int32_t*)topk_ids, sorted_token_ids, expert_ids,
                       num_tokens_post_pad, cumsum_buffer, num_experts, block_size, (int)numel, pad_sorted_token_ids,
                       (int)max_num_tokens_padded);
  } else {
    auto k = moe_align_kernel<int64_t>;
    if (lds > 64 * 1024) hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL(k, dim3(1), dim3(1024), lds, st, (const int64_t*)topk_ids, sorted_token_ids, expert_ids,
                       num_tokens_post_pad, cumsum_buffer, num_experts, block_size, (int)numel, pad_sorted_token_ids,
                       (int)max_num_tokens_padded);
  }
  return check_launch("moe_align_block_size");
}

static int moe_block_gemm(int mode, const void* a, int64_t lda, const float* a_scale, int64_t as_stride_m,
                          int64_t as_stride_k, const void* w, int64_t w_stride_e, int64_t w_stride_n,
                          const float* w_scale, int64_t ws_stride_e, int64_t ws_stride_n, int64_t ws_stride_k, void* c,
                          int64_t ldc, int out_dtype, const int32_t* sorted_token_ids, const int32_t* expert_ids,
                          const int32_t* num_tokens_post_padded, const float* topk_weights, int64_t num_valid_tokens,
                          int top_k, int mul_routed_weight, int block_m, int64_t max_m_blocks, int64_t N, int64_t K,
                          void* stream) {
  SGLAMD_REQUIRE(a && a_scale && w && w_scale && c && sorted_token_ids && expert_ids && num_tokens_post_padded,
                 SGLAMD_EINVAL, "fused_moe_gemm: null pointer");
  SGLAMD_REQUIRE(!mul_routed_weight || topk_weights, SGLAMD_EINVAL, "fused_moe_gemm: topk_weights missing");
  SGLAMD_REQUIRE(N > 0 && K > 0 && K % 16 == 0 && N < (1ll << 31) && K < (1ll << 31), SGLAMD_EINVAL,
                 "fused_moe_gemm: bad N/K");
  SGLAMD_REQUIRE(top_k >= 1 && num_valid_tokens >= 0 && num_valid_tokens < (1ll << 31), SGLAMD_EINVAL,
                 "fused_moe_gemm: bad top_k / num_valid_tokens");
  SGLAMD_REQUIRE(lda % 16 == 0 && w_stride_n % 16 == 0 && w_stride_e % 16 == 0, SGLAMD_EINVAL,
                 "fused_moe_gemm: strides must be multiples of 16 bytes");
  SGLAMD_REQUIRE(((uintptr_t)a % 16) == 0 && ((uintptr_t)w % 16) == 0, SGLAMD_EINVAL,
                 "fused_moe_gemm: operands must be 16-byte aligned");
  SGLAMD_REQUIRE(max_m_blocks >= 0 && max_m_blocks < (1ll << 24), SGLAMD_EINVAL, "fused_moe_gemm: bad block count");
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
  if (mode == GEMM_BLOCK_INT8) {
    if (out_dtype == SGLAMD_BF16) return dispatch_moe_gemm<GEMM_BLOCK_INT8, BF16>(g, block_m, st);
    if (out_dtype == SGLAMD_F16) return dispatch_moe_gemm<GEMM_BLOCK_INT8, F16>(g, block_m, st);
  } else {
    if (out_dtype == SGLAMD_BF16) return dispatch_moe_gemm<GEMM_BLOCK_FP8, BF16>(g, block_m, st);
    if (out_dtype == SGLAMD_F16) return dispatch_moe_gemm<GEMM_BLOCK_FP8, F16>(g, block_m, st);
  }
  return fail(SGLAMD_EINVAL, "fused_moe_gemm: out_dtype must be Half or BFloat16");
}

extern "C" int sglamd_fused_moe_block_fp8_gemm(const void* a, int64_t lda, const float* a_scale, int64_t as_stride_m,
                                               int64_t as_stride_k, const void* w, int64_t w_stride_e,
                                               int64_t w_stride_n, const float* w_scale, int64_t ws_stride_e,
                                               int64_t ws_stride_n, int64_t ws_stride_k, void* c, int64_t ldc,
                                               int out_dtype, const int32_t* sorted_token_ids,
                                               const int32_t* expert_ids, const int32_t* num_tokens_post_padded,
                                               const float* topk_weights, int64_t num_valid_tokens, int top_k,
                                               int mul_routed_weight, int block_m, int64_t max_m_blocks, int64_t N,
                                               int64_t K, void* stream) {
  return moe_block_gemm(GEMM_BLOCK_FP8, a, lda, a_scale, as_stride_m, as_stride_k, w, w_stride_e, w_stride_n, w_scale,
                        ws_stride_e, ws_stride_n, ws_stride_k, c, ldc, out_dtype, sorted_token_ids, expert_ids,
                        num_tokens_post_padded, topk_weights, num_valid_tokens, top_k, mul_routed_weight, block_m,
                        max_m_blocks, N, K, stream);
}

extern "C" int sglamd_fused_moe_block_int8_gemm(const void* a, int64_t lda, const float* a_scale, int64_t as_stride_m,
                                                int64_t as_stride_k, const void* w, int64_t w_stride_e,
                                                int64_t w_stride_n, const float* w_scale, int64_t ws_stride_e,
                                                int64_t ws_stride_n, int64_t ws_stride_k, void* c, int64_t ldc,
                                                int out_dtype, const int32_t* sorted_token_ids,
                                                const int32_t* expert_ids, const int32_t* num_tokens_post_padded,
                                                const float* topk_weights, int64_t num_valid_tokens, int top_k,
                                                int mul_routed_weight, int block_m, int64_t max_m_blocks, int64_t N,
                                                int64_t K, void* stream) {
  return moe_block_gemm(GEMM_BLOCK_INT8, a, lda, a_scale, as_stride_m, as_stride_k, w, w_stride_e, w_stride_n, w_scale,
                        ws_stride_e, ws_stride_n, ws_stride_k, c, ldc, out_dtype, sorted_token_ids, expert_ids,
                        num_tokens_post_padded, topk_weights, num_valid_tokens, top_k, mul_routed_weight, block_m,
                        max_m_blocks, N, K, stream);
}

extern "C" int sglamd_topk_softmax(float* topk_weights, int32_t* topk_indices, const void* gating_output, int g_dtype,
                                  int64_t num_tokens, int64_t num_experts, int64_t topk, int renormalize,
                                  float moe_softcapping, const float* correction_bias, void* stream) {
  SGLAMD_REQUIRE(topk_weights && topk_indices && gating_output, SGLAMD_EINVAL, "topk_softmax: null pointer");
  SGLAMD_REQUIRE(num_tokens >= 0 && num_experts > 0 && topk > 0, SGLAMD_EINVAL, "topk_softmax: bad sizes");
  SGLAMD_REQUIRE(topk <= num_experts, SGLAMD_EINVAL, "topk must be less than or equal to num_experts");
  SGLAMD_REQUIRE(num_experts <= 1024, SGLAMD_ENOTSUP, "topk_softmax: more than 1024 experts");
  SGLAMD_REQUIRE(g_dtype == SGLAMD_F32 || g_dtype == SGLAMD_F16 || g_dtype == SGLAMD_BF16, SGLAMD_EINVAL,
                 "gating_output must be float32, float16, or bfloat16");
  if (num_tokens == 0) return SGLAMD_OK;
  hipStream_t st = (hipStream_t)stream;
  const unsigned blocks = (unsigned)ceil_div(num_tokens, 4);
#define SGLAMD_TOPK(TT, E)                                                                                             \
  hipLaunchKernelGGL((topk_softmax_kernel<TT, E>), dim3(blocks), dim3(256), 0, st,                                     \
                     (const typename TT::storage*)gating_output, topk_weights, topk_indices, (int)num_tokens,          \
                     (int)num_experts, (int)topk, renormalize, moe_softcapping, correction_bias)
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
  return check_launch("topk_softmax");
}

extern "C" int sglamd_silu_and_mul(const void* input, void* out, int dtype, int64_t rows, int64_t d, void* stream) {
  SGLAMD_REQUIRE(input && out, SGLAMD_EINVAL, "silu_and_mul: null pointer");
  SGLAMD_REQUIRE(rows >= 0 && d > 0 && d % 8 == 0 && d < (1ll << 30), SGLAMD_EINVAL,
                 "silu_and_mul: d (%lld) must be a positive multiple of 8", (long long)d);
  SGLAMD_REQUIRE(((uintptr_t)input % 16) == 0 && ((uintptr_t)out % 16) == 0, SGLAMD_EINVAL,
                 "silu_and_mul: pointers must be 16-byte aligned");
  if (rows == 0) return SGLAMD_OK;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == SGLAMD_BF16)
    hipLaunchKernelGGL(silu_and_mul_kernel<BF16>, dim3((unsigned)rows), dim3(256), 0, st, (const u16*)input, (u16*)out,
                       (int)d);
  else if (dtype == SGLAMD_F16)
    hipLaunchKernelGGL(silu_and_mul_kernel<F16>, dim3((unsigned)rows), dim3(256), 0, st, (const u16*)input, (u16*)out,
                       (int)d);
  else
    return fail(SGLAMD_EINVAL, "silu_and_mul: dtype must be Half or BFloat16");
  return check_launch("silu_and_mul");
}

extern "C" int sglamd_moe_sum_reduce(const void* input, void* out, int dtype, int64_t tokens, int topk, int64_t d,
                                     float routed_scaling_factor, void* stream) {
  SGLAMD_REQUIRE(input && out, SGLAMD_EINVAL, "moe_sum_reduce: null pointer");
  SGLAMD_REQUIRE(tokens >= 0 && topk >= 1 && d > 0 && d % 8 == 0 && d < (1ll << 30), SGLAMD_EINVAL,
                 "moe_sum_reduce: hidden size (%lld) must be a positive multiple of 8", (long long)d);
  if (tokens == 0) return SGLAMD_OK;
  hipStream_t st = (hipStream_t)stream;
  int64_t gy64 = ceil_div(d, 2048);
  if (gy64 > 64) gy64 = 64;
  const unsigned gy = (unsigned)gy64;
  dim3 grid((unsigned)tokens, gy);
  if (dtype == SGLAMD_BF16)
    hipLaunchKernelGGL(moe_sum_reduce_kernel<BF16>, grid, dim3(256), 0, st, (const u16*)input, (u16*)out, topk, (int)d,
                       routed_scaling_factor);
  else if (dtype == SGLAMD_F16)
    hipLaunchKernelGGL(moe_sum_reduce_kernel<F16>, grid, dim3(256), 0, st, (const u16*)input, (u16*)out, topk, (int)d,
                       routed_scaling_factor);
  else
    return fail(SGLAMD_EINVAL, "moe_sum_reduce: dtype must be Half or BFloat16");
  return check_launch("moe_sum_reduce");
}


// ---------------------------------------------------------------------------------------
// Whole block-FP8 MoE layer from one host call: quantise -> align -> grouped GEMM 1 ->
// silu*mul + quantise (one kernel) -> grouped GEMM 2 (x routing weight) -> top-k sum.
// Six launches on one stream; all intermediates live in the caller's workspace.
// ---------------------------------------------------------------------------------------
namespace {
struct MoeWs {
  int64_t sorted, expert, post, cumsum, xq, xs, c1, aq, as, c3, total;
  int64_t max_padded, max_blocks;
};
inline int64_t up256(int64_t v) { return (v + 255) & ~(int64_t)255; }
MoeWs moe_ws_layout(int64_t M, int64_t H, int64_t I, int E, int topk, int block_m) {
  MoeWs w;
  const int64_t T = M * topk;
  w.max_padded = T < E + 1 ? T * block_m : T + (int64_t)(E + 1) * (block_m - 1);
  w.max_blocks = (w.max_padded + block_m - 1) / block_m;
  int64_t o = 0;
  w.sorted = o; o = up256(o + w.max_padded * 4);
  w.expert = o; o = up256(o + w.max_blocks * 4);
  w.post = o; o = up256(o + 4);
  w.cumsum = o; o = up256(o + (int64_t)(E + 2) * 4);
  w.xq = o; o = up256(o + M * H);
  w.xs = o; o = up256(o + M * ((H + 127) / 128) * 4);
  w.c1 = o; o = up256(o + T * 2 * I * 2);
  w.aq = o; o = up256(o + T * I);
  w.as = o; o = up256(o + T * ((I + 127) / 128) * 4);
  w.c3 = o; o = up256(o + T * H * 2);
  w.total = o;
  return w;
}
int moe_auto_block(int64_t M, int E, int topk) {
  static const int forced = getenv("SGLAMD_MOE_BLOCK_M") ? atoi(getenv("SGLAMD_MOE_BLOCK_M")) : 0;  // tuning knob
  if (forced == 16 || forced == 32 || forced == 64 || forced == 128 || forced == 192) return forced;
  const double rows = (double)M * topk / (E > 0 ? E : 1);
  if (rows <= 12) return 16;
  if (rows <= 24) return 32;
  if (rows <= 96) return 64;
  // 192-slot blocks: around 128 rows per expert one block holds a whole expert, so its weights are streamed
  // once (128-slot blocks would split every second expert into a full and a nearly empty block), and with
  // more rows the taller tile still measures faster (M = 16384: 9.2 ms against 10.5 ms)
  return 192;
}
}  // namespace

extern "C" int64_t sglamd_fused_moe_block_fp8_workspace(int64_t M, int64_t H, int64_t I, int E, int topk, int block_m) {
  if (M <= 0 || H <= 0 || I <= 0 || E <= 0 || topk <= 0) return 0;
  if (block_m == 0) block_m = moe_auto_block(M, E, topk);
  return moe_ws_layout(M, H, I, E, topk, block_m).total;
}

extern "C" int sglamd_fused_moe_block_fp8(const void* hidden, int dtype, int64_t M, int64_t H, int64_t I, int E,
                                          int topk, const void* w13, const float* w13_scale, const void* w2,
                                          const float* w2_scale, const float* topk_weights, const void* topk_ids,
                                          int ids_dtype, void* out, float routed_scaling_factor, int block_m,
                                          void* workspace, int64_t workspace_bytes, void* stream) {
  SGLAMD_REQUIRE(hidden && w13 && w13_scale && w2 && w2_scale && topk_weights && topk_ids && out && workspace,
                 SGLAMD_EINVAL, "fused_moe: null pointer");
  SGLAMD_REQUIRE(M > 0 && E > 0 && topk > 0, SGLAMD_EINVAL, "fused_moe: bad M/E/topk");
  SGLAMD_REQUIRE(H % 128 == 0 && I % 128 == 0, SGLAMD_EINVAL,
                 "fused_moe: hidden (%lld) and intermediate (%lld) sizes must be multiples of 128", (long long)H,
                 (long long)I);
  SGLAMD_REQUIRE(dtype == SGLAMD_BF16 || dtype == SGLAMD_F16, SGLAMD_EINVAL, "fused_moe: dtype must be Half or BFloat16");
  if (block_m == 0) block_m = moe_auto_block(M, E, topk);
  SGLAMD_REQUIRE(block_m == 16 || block_m == 32 || block_m == 64 || block_m == 128 || block_m == 192, SGLAMD_EINVAL,
                 "fused_moe: block_m must be 16, 32, 64, 128 or 192");
  const MoeWs w = moe_ws_layout(M, H, I, E, topk, block_m);
  SGLAMD_REQUIRE(workspace_bytes >= w.total, SGLAMD_EINVAL, "fused_moe: workspace too small (%lld < %lld)",
                 (long long)workspace_bytes, (long long)w.total);
  SGLAMD_REQUIRE(((uintptr_t)workspace % 256) == 0, SGLAMD_EINVAL, "fused_moe: workspace must be 256-byte aligned");
  uint8_t* ws = (uint8_t*)workspace;
  int32_t* sorted = (int32_t*)(ws + w.sorted);
  int32_t* expert = (int32_t*)(ws + w.expert);
  int32_t* post = (int32_t*)(ws + w.post);
  int32_t* cumsum = (int32_t*)(ws + w.cumsum);
  const int64_t T = M * topk, KB1 = H / 128, KB2 = I / 128;
  SGLAMD_REQUIRE(ids_dtype == SGLAMD_I32 || ids_dtype == SGLAMD_I64, SGLAMD_EINVAL,
                 "fused_moe: topk_ids must be int32 or int64");
  SGLAMD_REQUIRE(E + 1 <= 2048 && T < (1ll << 30), SGLAMD_EINVAL, "fused_moe: too many experts or tokens");
  SGLAMD_REQUIRE(((uintptr_t)hidden % 16) == 0, SGLAMD_EINVAL, "fused_moe: hidden must be 16-byte aligned");
  int rc;
  {
    GroupQuantArgs qa = {};
    qa.in = hidden;
    qa.q = ws + w.xq;
    qa.s = ws + w.xs;
    qa.groups_per_row = (int)KB1;
    qa.num_groups = M * KB1;
    qa.layout = SGLAMD_SCALE_ROW_MAJOR;
    qa.scale_stride = 0;
    qa.eps = 1e-10f;
    qa.min8 = -448.f;
    qa.max8 = 448.f;
    qa.form = SGLAMD_QUANT_FORM_RECIPROCAL;
    qa.q_is_fp8 = 1;
    qa.fuse_silu_mul = 0;
    qa.hidden = H;
    const int nb = E + 1;
    const size_t lds = (size_t)(3 * nb + 1 + 16 * nb) * sizeof(int32_t);
    const unsigned blocks = 1 + (unsigned)ceil_div(qa.num_groups * 8, 1024);
    hipStream_t st = (hipStream_t)stream;
#define SGLAMD_PROLOGUE(IDT, TT)                                                                                       \
  do {                                                                                                                 \
    auto k = moe_prologue_kernel<IDT, TT>;                                                                             \
    if (lds > 64 * 1024) hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);    \
    hipLaunchKernelGGL(k, dim3(blocks), dim3(1024), lds, st, (const IDT*)topk_ids, sorted, expert, post, cumsum, nb,   \
                       block_m, (int)T, (int)w.max_padded, qa);                                                        \
  } while (0)
    if (ids_dtype == SGLAMD_I32) {
      if (dtype == SGLAMD_BF16) SGLAMD_PROLOGUE(int32_t, BF16);
      else SGLAMD_PROLOGUE(int32_t, F16);
    } else {
      if (dtype == SGLAMD_BF16) SGLAMD_PROLOGUE(int64_t, BF16);
      else SGLAMD_PROLOGUE(int64_t, F16);
    }
#undef SGLAMD_PROLOGUE
    rc = check_launch("moe_prologue");
    if (rc) return rc;
  }
  rc = sglamd_fused_moe_block_fp8_gemm(ws + w.xq, H, (const float*)(ws + w.xs), KB1, 1, w13, 2 * I * H, H, w13_scale,
                                       (2 * I / 128) * KB1, KB1, 1, ws + w.c1, 2 * I, dtype, sorted, expert, post,
                                       nullptr, T, topk, 0, block_m, w.max_blocks, 2 * I, H, stream);
  if (rc) return rc;
  rc = sglamd_silu_mul_group_quant_8bit(ws + w.c1, dtype, ws + w.aq, SGLAMD_FP8_E4M3, ws + w.as, T, I, 128,
                                        SGLAMD_SCALE_ROW_MAJOR, 0, 1e-10f, -448.f, 448.f,
                                        SGLAMD_QUANT_FORM_RECIPROCAL, stream);
  if (rc) return rc;
  rc = sglamd_fused_moe_block_fp8_gemm(ws + w.aq, I, (const float*)(ws + w.as), KB2, 1, w2, H * I, I, w2_scale,
                                       (H / 128) * KB2, KB2, 1, ws + w.c3, H, dtype, sorted, expert, post, topk_weights,
                                       T, 1, 1, block_m, w.max_blocks, H, I, stream);
  if (rc) return rc;
  return sglamd_moe_sum_reduce(ws + w.c3, out, dtype, M, topk, H, routed_scaling_factor, stream);
}
