// Fused-MoE side of the path for gfx950: moe_align_block_size (stable counting sort into
// block-padded expert spans), the sorted-block grouped block-FP8 GEMM (same MFMA core as
// the dense GEMM, rows gathered through the sorted token list), silu_and_mul and the
// top-k sum reduce.
#include "gemm_big.h"
#include "gemm_big_moe_persist.h"
#include "gemm_skinny.h"
#include "quant_core.h"

namespace sglamd {

// ---------------------------------------------------------------------------------------
// moe_align_block_size: `parts` workgroups of 1024 lanes that never talk to each other.  The flat ids are cut
// into 16 * parts contiguous chunks; workgroup p places the ids of chunks 16 p .. 16 p + 15, one per wave.
//   1. every wave histograms its own chunk (bucket = id + 1) in LDS; the ids of the other workgroups' chunks are
//      counted by all lanes together, those in front of this workgroup's chunks and those behind them apart
//      (each workgroup reads all ids: a few hundred KB from L2, against scattered 4-byte stores that one CU
//      issues at about one per nanosecond and that the parts share),
//   2. padded totals -> exclusive prefix P (wave scans + carry), the same in every workgroup,
//   3. expert id of every block, total, cumsum buffer, padding fill (bucket b by workgroup b % parts); the per-wave
//      counts are turned into each wave's first slot per bucket (P[b] + ids in front of the workgroup's chunks +
//      counts of the waves in front),
//   4. stable scatter without workgroup barriers: a wave walks its chunk 64 ids at a time; a
//      lane's slot is the wave's running offset of the bucket plus the same-bucket lanes in
//      front of it, so every span is filled in ascending flat index.
// LDS: cnt[NB] | prefix[NB+1] | wavecnt[16][NB]   (NB = number of buckets, at most 3072; the counts of the ids in
// front share prefix[] until the scan and live in the registers of the lanes that own their buckets after it)
// ---------------------------------------------------------------------------------------
// PREP = true turns the same sort into prepare_moe_input: block size 1 (no padding), and instead of the sorted
// slot list it emits the two permutations, the expert offsets and the per-expert problem sizes.
struct MoePrepArgs {
  int32_t* expert_offsets;      // [E + 1]
  int32_t* blockscale_offsets;  // [E + 1] or null: offsets with every expert's rows rounded up to 128
  int32_t* problem_sizes1;      // [E, 3] = (rows, 2n, k)
  int32_t* problem_sizes2;      // [E, 3] = (rows, k, n)
  int32_t* input_permutation;   // [numel]: expert-major position -> token
  int32_t* output_permutation;  // [numel]: flat (token, j) -> expert-major position
  int topk, n, k;
};

static inline size_t moe_align_lds_bytes(int nb) { return (size_t)(3 * nb + 1 + 16 * nb) * sizeof(int32_t); }
// workgroups sharing one sort: one up to 4095 ids (the decode path: nothing to share), then one per 2048 ids, 16 at most
static inline int moe_align_parts(int64_t numel) {
  if (numel < 4096) return 1;
  return (int)(numel / 2048 < 16 ? numel / 2048 : 16);
}

template <typename IdT, bool PREP = false>
__device__ __forceinline__ void moe_align_body(const IdT* __restrict__ topk_ids, int32_t* sorted_ids,
                                               int32_t* expert_ids, int32_t* post_pad_out, int32_t* cumsum_out, int nb,
                                               int block_size, int numel, int pad_fill, int max_padded, int part,
                                               int parts, MoePrepArgs pa = MoePrepArgs()) {
  extern __shared__ int32_t lds[];
  int32_t* cnt = lds;
  int32_t* prefix = cnt + nb;
  int32_t* wavecnt = prefix + nb + 1;
  int32_t* before = prefix;  // until the scan writes prefix[]
  __shared__ int32_t s_carry;
  __shared__ int32_t s_wsum[16];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  for (int i = tid; i < 16 * nb; i += 1024) wavecnt[i] = 0;
  for (int i = tid; i < nb; i += 1024) cnt[i] = 0, before[i] = 0;
  if (tid == 0) s_carry = 0;
  __syncthreads();

  // Every wave owns one contiguous chunk of the flat ids (a multiple of 64 long), so ascending flat index
  // is workgroup first, wave second, position inside the wave's chunk third.
  const int chunk = ((numel + 16 * parts - 1) / (16 * parts) + 63) & ~63;
  const int wg_begin = min(numel, part * 16 * chunk), wg_end = min(numel, wg_begin + 16 * chunk);
  const int c_begin = min(numel, wg_begin + wave * chunk), c_end = min(numel, c_begin + chunk);
  int32_t* mycnt = wavecnt + wave * nb;
  // Ids are fetched ALIGN_BATCH x 64 at a time, all loads of a batch before their first use (one load per loop
  // turn would cost the wave a full memory latency per 64 ids).
  constexpr int ALIGN_BATCH = 8;
  auto bucket_at = [&](int i, int end) -> int {
    if (i >= end) return -1;
    const int b = (int)topk_ids[i] + 1;
    return (b < 0 || b >= nb) ? -1 : b;
  };
  auto bucket_of = [&](int i) -> int { return bucket_at(i, c_end); };
  for (int base = c_begin; base < c_end; base += 64 * ALIGN_BATCH) {
    int bb[ALIGN_BATCH];
#pragma unroll
    for (int u = 0; u < ALIGN_BATCH; u++) bb[u] = bucket_of(base + u * 64 + lane);
#pragma unroll
    for (int u = 0; u < ALIGN_BATCH; u++)
      if (bb[u] >= 0) atomicAdd(&mycnt[bb[u]], 1);
  }
  // the other workgroups' ids: in front of this workgroup's chunks -> before[], behind them -> cnt[]
  for (int side = 0; side < 2; side++) {
    const int lo = side ? wg_end : 0, hi = side ? numel : wg_begin;
    int32_t* dst = side ? cnt : before;
    for (int base = lo; base < hi; base += 1024 * ALIGN_BATCH) {
      int bb[ALIGN_BATCH];
#pragma unroll
      for (int u = 0; u < ALIGN_BATCH; u++) bb[u] = bucket_at(base + u * 1024 + tid, hi);
#pragma unroll
      for (int u = 0; u < ALIGN_BATCH; u++)
        if (bb[u] >= 0) atomicAdd(&dst[bb[u]], 1);
    }
  }
  __syncthreads();
  int bef[3] = {0, 0, 0};  // before[] of buckets tid, tid + 1024, tid + 2048
  for (int b = tid; b < nb; b += 1024) {
    int t = 0;
    for (int w = 0; w < 16; w++) t += wavecnt[w * nb + b];
    const int f = before[b];
    if (b < 1024) bef[0] = f;
    else if (b < 2048) bef[1] = f;
    else bef[2] = f;
    cnt[b] += t + f;
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
    if (post_pad_out && part == 0) *post_pad_out = s_carry;
  }
  __syncthreads();

  const int post_pad = prefix[nb];
  for (int b = tid; b < nb; b += 1024) {
    // per-wave counts become the slot at which each wave starts writing bucket b
    int running = prefix[b] + (b < 1024 ? bef[0] : b < 2048 ? bef[1] : bef[2]);
    for (int w = 0; w < 16; w++) {
      const int t = wavecnt[w * nb + b];
      wavecnt[w * nb + b] = running;
      running += t;
    }
    if (b % parts != part) continue;  // the outputs of bucket b come from one workgroup
    if (PREP) {
      // bucket 0 holds the ids == -1, which take no part: positions count from the end of that bucket
      if (b >= 1) {
        const int e = b - 1;
        pa.expert_offsets[e] = prefix[b] - prefix[1];
        pa.problem_sizes1[e * 3] = cnt[b];
        pa.problem_sizes1[e * 3 + 1] = 2 * pa.n;
        pa.problem_sizes1[e * 3 + 2] = pa.k;
        pa.problem_sizes2[e * 3] = cnt[b];
        pa.problem_sizes2[e * 3 + 1] = pa.k;
        pa.problem_sizes2[e * 3 + 2] = pa.n;
      }
    } else {
      for (int j = prefix[b] / block_size; j < prefix[b + 1] / block_size; j++) expert_ids[j] = b - 1;
    }
    if (cumsum_out) cumsum_out[b] = prefix[b] + cnt[b];
    if (pad_fill)
      for (int j = prefix[b] + cnt[b]; j < prefix[b + 1]; j++) sorted_ids[j] = numel;
  }
  if (cumsum_out && tid == 0 && part == 0) cumsum_out[nb] = post_pad;
  if (PREP && tid == 0 && part == 0) {
    pa.expert_offsets[nb - 1] = post_pad - prefix[1];
    if (pa.blockscale_offsets) {
      int rounded = 0;
      for (int b = 1; b < nb; b++) {
        pa.blockscale_offsets[b - 1] = rounded;
        rounded += (cnt[b] + 127) / 128 * 128;
      }
      pa.blockscale_offsets[nb - 1] = rounded;
    }
  }
  const int prep_base = PREP ? prefix[1] : 0;
  if (pad_fill)
    for (int j = post_pad + part * 1024 + tid; j < max_padded; j += 1024 * parts) sorted_ids[j] = numel;
  __syncthreads();

  // Stable scatter, one wave per chunk and no workgroup barrier: 64 ids at a time, a lane's slot is its wave's
  // running offset for the bucket plus the number of same-bucket lanes in front of it.
  volatile int32_t* myoff = mycnt;
  const int key_bits = 32 - __clz(max(nb - 1, 1));
  for (int base0 = c_begin; base0 < c_end; base0 += 64 * ALIGN_BATCH) {
    int bb[ALIGN_BATCH];
#pragma unroll
    for (int u = 0; u < ALIGN_BATCH; u++) bb[u] = bucket_of(base0 + u * 64 + lane);
#pragma unroll
    for (int u = 0; u < ALIGN_BATCH; u++) {
      const int i = base0 + u * 64 + lane;
      const int b = bb[u];
      // lanes of this wave with the same bucket: intersect, bit by bit of the bucket number, the lanes that agree
      unsigned long long m = __ballot(b >= 0);
      if (m == 0) continue;  // past the end of the chunk (wave-uniform)
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
      if (PREP) {
        if (b >= 1) {
          const int pos = off + rank - prep_base;
          pa.input_permutation[pos] = i / pa.topk;
          pa.output_permutation[i] = pos;
        }
      } else {
        if (b >= 0) sorted_ids[off + rank] = i;
      }
    }
  }
}

template <typename IdT>
__global__ __launch_bounds__(1024) void moe_align_kernel(const IdT* __restrict__ topk_ids, int32_t* sorted_ids,
                                                         int32_t* expert_ids, int32_t* post_pad_out,
                                                         int32_t* cumsum_out, int nb, int block_size, int numel,
                                                         int pad_fill, int max_padded) {
  moe_align_body<IdT>(topk_ids, sorted_ids, expert_ids, post_pad_out, cumsum_out, nb, block_size, numel, pad_fill,
                      max_padded, (int)blockIdx.x, (int)gridDim.x);
}

// First launch of the fused MoE layer: workgroup 0 sorts the tokens, the others quantise the hidden
// states (group 128, reciprocal form).  The two jobs are independent, so sharing a launch only removes
// one launch latency from the decode path.
template <typename IdT, typename T>
__global__ __launch_bounds__(1024) void moe_prologue_kernel(const IdT* __restrict__ topk_ids, int32_t* sorted_ids,
                                                            int32_t* expert_ids, int32_t* post_pad_out,
                                                            int32_t* cumsum_out, int nb, int block_size, int numel,
                                                            int max_padded, int parts, GroupQuantArgs qa) {
  if ((int)blockIdx.x < parts) {
    moe_align_body<IdT>(topk_ids, sorted_ids, expert_ids, post_pad_out, cumsum_out, nb, block_size, numel, 1, max_padded,
                        (int)blockIdx.x, parts);
  } else {
    group_quant_body<T, 128>(qa, (int64_t)((int)blockIdx.x - parts) * 1024 + threadIdx.x);
  }
}

// prepare_moe_input: the stable sort above with block size 1, emitting permutations and problem sizes.
__global__ __launch_bounds__(1024) void moe_prepare_kernel(const int32_t* __restrict__ topk_ids, int nb, int numel,
                                                           MoePrepArgs pa) {
  moe_align_body<int32_t, true>(topk_ids, nullptr, nullptr, nullptr, nullptr, nb, 1, numel, 0, 0, (int)blockIdx.x,
                                (int)gridDim.x, pa);
}

// shuffle_rows: output row r = input row dst2src[r]; rows are moved as VEC-byte pieces.
template <typename VT>
__global__ __launch_bounds__(256) void shuffle_rows_kernel(const uint8_t* __restrict__ in, const int32_t* __restrict__ map,
                                                           uint8_t* __restrict__ out, int64_t num_dst, int64_t row_bytes) {
  const int64_t pieces = row_bytes / (int64_t)sizeof(VT);
  for (int64_t r = blockIdx.x; r < num_dst; r += gridDim.x) {
    const VT* src = (const VT*)(in + (int64_t)map[r] * row_bytes);
    VT* dst = (VT*)(out + r * row_bytes);
    for (int64_t j = threadIdx.x; j < pieces; j += 256) dst[j] = src[j];
  }
}

// apply_shuffle_mul_sum: out[i, :] = sum_j factor[i*topk + j] * in[perm[i*topk + j], :], accumulated in fp32
// in the order j = 0 .. topk-1; one workgroup per (token, 2048-column slice).
template <typename T>
__global__ __launch_bounds__(256) void shuffle_mul_sum_kernel(const u16* __restrict__ in, u16* __restrict__ out,
                                                              const int32_t* __restrict__ perm,
                                                              const u16* __restrict__ factors, int topk, int d) {
  const int i = blockIdx.x;
  const int32_t* p = perm + (int64_t)i * topk;
  const u16* f = factors ? factors + (int64_t)i * topk : nullptr;
  u16* o = out + (int64_t)i * d;
  if ((d & 7) == 0) {
    for (int j = (blockIdx.y * 256 + threadIdx.x) * 8; j < d; j += gridDim.y * 2048) {
      float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      for (int k = 0; k < topk; k++) {
        const float w = f ? T::to_f32(f[k]) : 1.f;
        const v4i v = *(const v4i*)(in + (int64_t)p[k] * d + j);
        u16 b[8];
        __builtin_memcpy(b, &v, 16);
#pragma unroll
        for (int e = 0; e < 8; e++) acc[e] = fmaf(w, T::to_f32(b[e]), acc[e]);
      }
      u16 ob[8];
#pragma unroll
      for (int e = 0; e < 8; e++) ob[e] = T::from_f32(acc[e]);
      v4i ov;
      __builtin_memcpy(&ov, ob, 16);
      *(v4i*)(o + j) = ov;
    }
  } else {
    for (int j = blockIdx.y * 256 + threadIdx.x; j < d; j += gridDim.y * 256) {
      float acc = 0.f;
      for (int k = 0; k < topk; k++)
        acc = fmaf(f ? T::to_f32(f[k]) : 1.f, T::to_f32(in[(int64_t)p[k] * d + j]), acc);
      o[j] = T::from_f32(acc);
    }
  }
}

// Sorted-block schedule of a grouped GEMM whose rows are already expert-major: expert e owns rows
// [offsets[e], offsets[e] + problem_sizes[e][0]).  Every expert gets ceil(rows / block_m) blocks; slot values
// are row numbers, slots past an expert's last row hold num_rows (the "no row" value of the GEMM kernels).
__global__ __launch_bounds__(1024) void grouped_schedule_kernel(const int32_t* __restrict__ problem_sizes,
                                                                const int32_t* __restrict__ offsets, int num_experts,
                                                                int block_m, int num_rows, int max_blocks,
                                                                int32_t* sorted_ids, int32_t* expert_ids,
                                                                int32_t* post_pad) {
  extern __shared__ int32_t lds[];  // first[E + 1]: first block of every expert
  __shared__ int32_t s_wsum[16];
  __shared__ int32_t s_carry;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (tid == 0) s_carry = 0;
  __syncthreads();
  for (int base = 0; base < num_experts; base += 1024) {
    const int e = base + tid;
    int rows = e < num_experts ? problem_sizes[e * 3] : 0;
    rows = min(max(rows, 0), num_rows);
    const int nblk = (rows + block_m - 1) / block_m;
    int incl = nblk;
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
    if (e < num_experts) lds[e] = carry + woff + incl - nblk;
    __syncthreads();
    if (tid == 1023) s_carry = carry + woff + incl;
    __syncthreads();
  }
  const int total = min(s_carry, max_blocks);
  if (tid == 0) {
    lds[num_experts] = s_carry;
    *post_pad = total * block_m;
  }
  __syncthreads();
  for (int idx = tid; idx < total * block_m; idx += 1024) {
    const int blk = idx / block_m, r = idx - blk * block_m;
    int lo = 0, hi = num_experts - 1;  // last expert whose first block is <= blk (experts without rows share a value)
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (lds[mid] <= blk) lo = mid;
      else hi = mid - 1;
    }
    const int row_in_expert = (blk - lds[lo]) * block_m + r;
    const int rows = min(max(problem_sizes[lo * 3], 0), num_rows);
    const int row = offsets[lo] + row_in_expert;
    sorted_ids[idx] = (row_in_expert < rows && row >= 0 && row < num_rows) ? row : num_rows;
    if (r == 0) expert_ids[blk] = lo;
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
// act_and_mul: out[t, j] = T(act_f32(x[t, j])) * x[t, d + j], product rounded to T.
// ACT 0: silu x / (1 + exp(-x));  1: gelu x * 0.5 * (1 + erf(x / sqrt 2));  2: the tanh form of gelu.
// ---------------------------------------------------------------------------------------
template <int ACT>
__device__ __forceinline__ float act_f32(float x) {
  if constexpr (ACT == 0) {
    return x / (1.0f + expf(-x));
  } else if constexpr (ACT == 1) {
    return x * (0.5f * (1.0f + erff(x * 0.70710678118654752440f)));
  } else {
    const float cdf = 0.5f * (1.0f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x)));
    return x * cdf;
  }
}
template <typename T, int ACT>
__global__ __launch_bounds__(256) void act_and_mul_kernel(const u16* __restrict__ in, u16* __restrict__ out, int d) {
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
      const float s = T::to_f32(T::from_f32(act_f32<ACT>(T::to_f32(gb[k]))));
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

// tuning knob: SGLAMD_MOE_PERSIST=0 runs the tall sorted blocks one tile per workgroup instead of the persistent walk
static inline bool moe_persist_enabled() {
  static const int v = getenv("SGLAMD_MOE_PERSIST") ? atoi(getenv("SGLAMD_MOE_PERSIST")) : 1;
  return v != 0;
}

// tuning knob: SGLAMD_MOE_PERSIST128=0 keeps the 128-slot sorted blocks with one tile per workgroup
static inline bool moe_persist128_enabled() {
  static const int v = getenv("SGLAMD_MOE_PERSIST128") ? atoi(getenv("SGLAMD_MOE_PERSIST128")) : 1;
  return v != 0 && moe_persist_enabled();
}

// tuning knob: SGLAMD_MOE_ACTQ=0 keeps SiLU * up and its quantisation a launch of their own behind the first GEMM
static bool moe_actq_enabled() {
  static const int v = getenv("SGLAMD_MOE_ACTQ") ? atoi(getenv("SGLAMD_MOE_ACTQ")) : 1;
  return v != 0;
}

// The persistent walk hands out tiles by position, not by arrival.  A sorted block that is an expert's second one
// finds the weights its first block has just streamed in L2 and finishes in half the time, and a fixed walk cannot
// balance that the way the dispatch order of a one-tile-per-workgroup launch does; until the tiles went to XCDs in
// contiguous ranges the walk therefore lost 5 % where half of the experts own one block and half two (6144 tokens
// on the DeepSeek-V3 layer) and was only used where every expert owns the same number.  With an expert's blocks
// meeting in one L2 it is level or ahead at every token count measured (3072 ... 12288: 0 ... -5.5 %), so it runs
// wherever there are more tiles than CUs.
template <int MODE, typename OT>
static int dispatch_moe_gemm(const GemmArgs& g, int block_m, hipStream_t st) {
  // number of sorted blocks that will actually run is data dependent; every valid slot could own one
  const int64_t expect = g.num_valid < g.max_blocks_m ? g.num_valid : g.max_blocks_m;
  const bool streaming_ok = gemm8_skinny_ok(g, g.num_valid / g.top_k);
  switch (block_m) {
    case 16:
      if (streaming_ok) return gemm8_skinny_launch<1, MODE, OT, true>(g, st, expect);
      return gemm8_launch<16, 128, 1, 2, MODE, OT, true>(g, st);  // operands of 2 GiB and more
    case 32:
      if (streaming_ok) return gemm8_skinny_launch<2, MODE, OT, true>(g, st, expect);
      return gemm8_launch<32, 128, 1, 2, MODE, OT, true>(g, st);
    case 64:
      // the tile kernel with one 32-row tile per wave when its preconditions hold: the streaming kernel spends
      // four MFMA row groups per weight fragment and falls far behind it at this height
      if ((g.K % 128) == 0 && (g.K >> 7) <= GEMM8_BIG_MAX_KB && (int64_t)(g.num_valid / g.top_k) * g.lda < 0x7fffffffll &&
          (int64_t)g.N * g.ldb < 0x7fffffffll)
        // (the persistent walk with its two stages is 12 % behind this kernel's three at this height)
        return gemm8_big_moe_launch<MODE, OT, 1>(g, st);
      if (streaming_ok) return gemm8_skinny_launch<4, MODE, OT, true>(g, st, expect);
      return gemm8_launch<64, 128, 2, 2, MODE, OT, true>(g, st);
    case 128:
      // 32x32x64-MFMA tile kernel when its preconditions hold (K % 128 == 0, operands below 2 GiB per matrix)
      if ((g.K % 128) == 0 && (g.K >> 7) <= GEMM8_BIG_MAX_KB && (int64_t)(g.num_valid / g.top_k) * g.lda < 0x7fffffffll &&
          (int64_t)g.N * g.ldb < 0x7fffffffll)
      {
        // more tiles than CUs: the persistent walk, as for the 192-slot blocks
        if (moe_persist128_enabled() && gemm8_moe_persist_ok(g) &&
            (int64_t)((g.N + 255) / 256) * g.max_blocks_m > device_cus())
          return gemm8_moe_persist_launch<MODE, OT, 2>(g, st);
        return gemm8_big_moe_launch<MODE, OT>(g, st);
      }
      return gemm8_launch<128, 128, 2, 2, MODE, OT, true>(g, st);
    case 192:
      // one block per expert when an expert gets 129..192 rows: its weights are streamed once
      SGLAMD_REQUIRE((g.K % 128) == 0 && (g.K >> 7) <= GEMM8_BIG_MAX_KB && (int64_t)(g.num_valid / g.top_k) * g.lda < 0x7fffffffll &&
                         (int64_t)g.N * g.ldb < 0x7fffffffll,
                     SGLAMD_EINVAL, "fused_moe_gemm: block_m 192 needs K %% 128 == 0 and operands below 2 GiB");
      // more tiles than CUs: one workgroup per CU walks them and requests a tile's first blocks under the
      // epilogue of the tile before
      if (moe_persist_enabled() && gemm8_moe_persist_ok(g) &&
          (int64_t)((g.N + 255) / 256) * g.max_blocks_m > device_cus())
        return gemm8_moe_persist_launch<MODE, OT, 3>(g, st);
      return gemm8_big_moe_launch<MODE, OT, 3>(g, st);
    default:
      return fail(SGLAMD_EINVAL, "fused_moe_gemm: block_m must be 16, 32, 64, 128 or 192 (got %d)", block_m);
  }
}

}  // namespace sglamd

using namespace sglamd;

// More than 64 KB of dynamic LDS (above ~850 buckets) needs the kernel's limit raised, once per kernel and device.
#define SGLAMD_RAISE_LDS(kern, lds)                                                                                    \
  do {                                                                                                                 \
    if ((lds) > 64 * 1024) {                                                                                           \
      static SmemAttrOnce attr_;                                                                                       \
      const hipError_t e_ = raise_dynamic_smem(attr_, (const void*)(kern), (int)(lds));                                \
      if (e_ != hipSuccess) return fail(SGLAMD_EHIP, "hipFuncSetAttribute: %s", hipGetErrorString(e_));                \
    }                                                                                                                  \
  } while (0)

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
  const size_t lds = moe_align_lds_bytes(num_experts);
  const unsigned parts = (unsigned)moe_align_parts(numel);
  hipStream_t st = (hipStream_t)stream;
  if (ids_dtype == SGLAMD_I32) {
    auto k = moe_align_kernel<int32_t>;
    SGLAMD_RAISE_LDS(k, lds);
    hipLaunchKernelGGL(k, dim3(parts), dim3(1024), lds, st, (const int32_t*)topk_ids, sorted_token_ids, expert_ids,
                       num_tokens_post_pad, cumsum_buffer, num_experts, block_size, (int)numel, pad_sorted_token_ids,
                       (int)max_num_tokens_padded);
  } else {
    auto k = moe_align_kernel<int64_t>;
    SGLAMD_RAISE_LDS(k, lds);
    hipLaunchKernelGGL(k, dim3(parts), dim3(1024), lds, st, (const int64_t*)topk_ids, sorted_token_ids, expert_ids,
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

template <int ACT>
static int act_and_mul_launch(const char* name, const void* input, void* out, int dtype, int64_t rows, int64_t d,
                              void* stream) {
  SGLAMD_REQUIRE(input && out, SGLAMD_EINVAL, "%s: null pointer", name);
  SGLAMD_REQUIRE(rows >= 0 && d > 0 && d % 8 == 0 && d < (1ll << 30), SGLAMD_EINVAL,
                 "%s: d (%lld) must be a positive multiple of 8", name, (long long)d);
  SGLAMD_REQUIRE(((uintptr_t)input % 16) == 0 && ((uintptr_t)out % 16) == 0, SGLAMD_EINVAL,
                 "%s: pointers must be 16-byte aligned", name);
  SGLAMD_REQUIRE(rows < (1ll << 31), SGLAMD_EINVAL, "%s: too many rows", name);
  if (rows == 0) return SGLAMD_OK;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == SGLAMD_BF16)
    hipLaunchKernelGGL((act_and_mul_kernel<BF16, ACT>), dim3((unsigned)rows), dim3(256), 0, st, (const u16*)input,
                       (u16*)out, (int)d);
  else if (dtype == SGLAMD_F16)
    hipLaunchKernelGGL((act_and_mul_kernel<F16, ACT>), dim3((unsigned)rows), dim3(256), 0, st, (const u16*)input,
                       (u16*)out, (int)d);
  else
    return fail(SGLAMD_EINVAL, "%s: dtype must be Half or BFloat16", name);
  return check_launch(name);
}

extern "C" int sglamd_silu_and_mul(const void* input, void* out, int dtype, int64_t rows, int64_t d, void* stream) {
  return act_and_mul_launch<0>("silu_and_mul", input, out, dtype, rows, d, stream);
}
extern "C" int sglamd_gelu_and_mul(const void* input, void* out, int dtype, int64_t rows, int64_t d, void* stream) {
  return act_and_mul_launch<1>("gelu_and_mul", input, out, dtype, rows, d, stream);
}
extern "C" int sglamd_gelu_tanh_and_mul(const void* input, void* out, int dtype, int64_t rows, int64_t d,
                                        void* stream) {
  return act_and_mul_launch<2>("gelu_tanh_and_mul", input, out, dtype, rows, d, stream);
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
// Expert-major ("grouped") MoE interface: prepare_moe_input / shuffle_rows /
// fp8_blockwise_scaled_grouped_mm / apply_shuffle_mul_sum.
// ---------------------------------------------------------------------------------------
extern "C" int sglamd_prepare_moe_input(const int32_t* topk_ids, int64_t numel, int topk, int num_experts, int64_t n,
                                        int64_t k, int32_t* expert_offsets, int32_t* blockscale_offsets,
                                        int32_t* problem_sizes1, int32_t* problem_sizes2, int32_t* input_permutation,
                                        int32_t* output_permutation, void* stream) {
  SGLAMD_REQUIRE(topk_ids && expert_offsets && problem_sizes1 && problem_sizes2 && input_permutation &&
                     output_permutation,
                 SGLAMD_EINVAL, "prepare_moe_input: null pointer");
  SGLAMD_REQUIRE(numel >= 0 && numel < (1ll << 30) && topk >= 1, SGLAMD_EINVAL, "prepare_moe_input: bad numel/topk");
  SGLAMD_REQUIRE(num_experts > 0 && num_experts <= 2048, SGLAMD_EINVAL,
                 "prepare_moe_input: num_experts (%d) must be in [1, 2048]", num_experts);
  SGLAMD_REQUIRE(n > 0 && k > 0 && 2 * n < (1ll << 31) && k < (1ll << 31), SGLAMD_EINVAL, "prepare_moe_input: bad n/k");
  MoePrepArgs pa;
  pa.expert_offsets = expert_offsets;
  pa.blockscale_offsets = blockscale_offsets;
  pa.problem_sizes1 = problem_sizes1;
  pa.problem_sizes2 = problem_sizes2;
  pa.input_permutation = input_permutation;
  pa.output_permutation = output_permutation;
  pa.topk = topk;
  pa.n = (int)n;
  pa.k = (int)k;
  const int nb = num_experts + 1;
  const size_t lds = moe_align_lds_bytes(nb);
  auto kern = moe_prepare_kernel;
  SGLAMD_RAISE_LDS(kern, lds);
  hipLaunchKernelGGL(kern, dim3((unsigned)moe_align_parts(numel)), dim3(1024), lds, (hipStream_t)stream, topk_ids, nb, (int)numel, pa);
  return check_launch("prepare_moe_input");
}

extern "C" int sglamd_shuffle_rows(const void* input, const int32_t* dst2src_map, void* output, int64_t num_dst_rows,
                                   int64_t row_bytes, void* stream) {
  SGLAMD_REQUIRE(input && dst2src_map && output, SGLAMD_EINVAL, "shuffle_rows: null pointer");
  SGLAMD_REQUIRE(num_dst_rows >= 0 && row_bytes > 0, SGLAMD_EINVAL, "shuffle_rows: bad sizes");
  if (num_dst_rows == 0) return SGLAMD_OK;
  const unsigned blocks = (unsigned)(num_dst_rows < 65536 ? num_dst_rows : 65536);
  hipStream_t st = (hipStream_t)stream;
  const uintptr_t both = (uintptr_t)input | (uintptr_t)output | (uintptr_t)row_bytes;
  if ((both & 15) == 0)
    hipLaunchKernelGGL(shuffle_rows_kernel<v4i>, dim3(blocks), dim3(256), 0, st, (const uint8_t*)input, dst2src_map,
                       (uint8_t*)output, num_dst_rows, row_bytes);
  else if ((both & 3) == 0)
    hipLaunchKernelGGL(shuffle_rows_kernel<int32_t>, dim3(blocks), dim3(256), 0, st, (const uint8_t*)input, dst2src_map,
                       (uint8_t*)output, num_dst_rows, row_bytes);
  else
    hipLaunchKernelGGL(shuffle_rows_kernel<uint8_t>, dim3(blocks), dim3(256), 0, st, (const uint8_t*)input, dst2src_map,
                       (uint8_t*)output, num_dst_rows, row_bytes);
  return check_launch("shuffle_rows");
}

extern "C" int sglamd_apply_shuffle_mul_sum(const void* input, void* output, const int32_t* permutation,
                                            const void* factors, int dtype, int64_t m, int topk, int64_t row_stride,
                                            void* stream) {
  SGLAMD_REQUIRE(input && output && permutation, SGLAMD_EINVAL, "apply_shuffle_mul_sum: null pointer");
  SGLAMD_REQUIRE(m >= 0 && m < (1ll << 31) && topk >= 1 && row_stride > 0 && row_stride < (1ll << 30), SGLAMD_EINVAL,
                 "apply_shuffle_mul_sum: bad sizes");
  SGLAMD_REQUIRE(dtype == SGLAMD_BF16 || dtype == SGLAMD_F16, SGLAMD_EINVAL,
                 "apply_shuffle_mul_sum: dtype must be Half or BFloat16");
  SGLAMD_REQUIRE((row_stride % 8) != 0 || (((uintptr_t)input | (uintptr_t)output) % 16) == 0, SGLAMD_EINVAL,
                 "apply_shuffle_mul_sum: pointers must be 16-byte aligned");
  if (m == 0) return SGLAMD_OK;
  int64_t gy = ceil_div(row_stride, 2048);
  if (gy > 64) gy = 64;
  dim3 grid((unsigned)m, (unsigned)gy);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == SGLAMD_BF16)
    hipLaunchKernelGGL(shuffle_mul_sum_kernel<BF16>, grid, dim3(256), 0, st, (const u16*)input, (u16*)output, permutation,
                       (const u16*)factors, topk, (int)row_stride);
  else
    hipLaunchKernelGGL(shuffle_mul_sum_kernel<F16>, grid, dim3(256), 0, st, (const u16*)input, (u16*)output, permutation,
                       (const u16*)factors, topk, (int)row_stride);
  return check_launch("apply_shuffle_mul_sum");
}

namespace {
struct GroupedWs {
  int64_t sorted, expert, post, total, max_padded, max_blocks;
};
GroupedWs grouped_ws_layout(int64_t rows, int E, int block_m) {
  GroupedWs w;
  const int64_t worst = rows + (int64_t)E * (block_m - 1);  // every expert may leave one block partly filled
  w.max_blocks = (worst + block_m - 1) / block_m;
  w.max_padded = w.max_blocks * block_m;
  int64_t o = 0;
  w.sorted = o; o = (o + w.max_padded * 4 + 255) & ~(int64_t)255;
  w.expert = o; o = (o + w.max_blocks * 4 + 255) & ~(int64_t)255;
  w.post = o; o += 256;
  w.total = o;
  return w;
}
int grouped_block_m(int64_t rows, int E);
}  // namespace

extern "C" int64_t sglamd_grouped_mm_workspace_bytes(int64_t total_rows, int num_experts) {
  if (total_rows <= 0 || num_experts <= 0) return 0;
  return grouped_ws_layout(total_rows, num_experts, grouped_block_m(total_rows, num_experts)).total;
}

extern "C" int sglamd_fp8_blockwise_scaled_grouped_mm(void* output, int out_dtype, const void* a, const void* b,
                                                      const float* scales_a, const float* scales_b,
                                                      const int32_t* problem_sizes, const int32_t* expert_offsets,
                                                      int num_experts, int64_t total_rows, int64_t N, int64_t K,
                                                      void* workspace, int64_t workspace_bytes, void* stream) {
  SGLAMD_REQUIRE(output && a && b && scales_a && scales_b && problem_sizes && expert_offsets, SGLAMD_EINVAL,
                 "fp8_blockwise_scaled_grouped_mm: null pointer");
  SGLAMD_REQUIRE(num_experts > 0 && num_experts <= 2048, SGLAMD_EINVAL,
                 "fp8_blockwise_scaled_grouped_mm: num_experts (%d) must be in [1, 2048]", num_experts);
  SGLAMD_REQUIRE(total_rows >= 0 && total_rows < (1ll << 30), SGLAMD_EINVAL,
                 "fp8_blockwise_scaled_grouped_mm: bad number of rows");
  SGLAMD_REQUIRE(N > 0 && K > 0 && N % 128 == 0 && K % 128 == 0 && N < (1ll << 31) && K < (1ll << 31), SGLAMD_EINVAL,
                 "fp8_blockwise_scaled_grouped_mm: N (%lld) and K (%lld) must be positive multiples of 128",
                 (long long)N, (long long)K);
  SGLAMD_REQUIRE((((uintptr_t)a | (uintptr_t)b) % 16) == 0, SGLAMD_EINVAL,
                 "fp8_blockwise_scaled_grouped_mm: operands must be 16-byte aligned");
  if (total_rows == 0) return SGLAMD_OK;
  const int block_m = grouped_block_m(total_rows, num_experts);
  const GroupedWs w = grouped_ws_layout(total_rows, num_experts, block_m);
  SGLAMD_REQUIRE(workspace && workspace_bytes >= w.total, SGLAMD_EINVAL,
                 "fp8_blockwise_scaled_grouped_mm: workspace too small (%lld < %lld bytes)", (long long)workspace_bytes,
                 (long long)w.total);
  SGLAMD_REQUIRE(((uintptr_t)workspace % 16) == 0, SGLAMD_EINVAL,
                 "fp8_blockwise_scaled_grouped_mm: workspace must be 16-byte aligned");
  uint8_t* ws = (uint8_t*)workspace;
  int32_t* sorted = (int32_t*)(ws + w.sorted);
  int32_t* expert = (int32_t*)(ws + w.expert);
  int32_t* post = (int32_t*)(ws + w.post);
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL(grouped_schedule_kernel, dim3(1), dim3(1024), (size_t)(num_experts + 1) * sizeof(int32_t), st,
                     problem_sizes, expert_offsets, num_experts, block_m, (int)total_rows, (int)w.max_blocks, sorted,
                     expert, post);
  int rc = check_launch("grouped_schedule");
  if (rc) return rc;
  const int64_t KB = K / 128;
  return sglamd_fused_moe_block_fp8_gemm(a, K, scales_a, KB, 1, b, N * K, K, scales_b, (N / 128) * KB, KB, 1, output, N,
                                         out_dtype, sorted, expert, post, nullptr, total_rows, 1, 0, block_m,
                                         w.max_blocks, N, K, stream);
}


// ---------------------------------------------------------------------------------------
// Whole block-FP8 MoE layer from one host call: quantise + align (one kernel) -> grouped GEMM 1 ->
// silu*mul + quantise (one kernel) -> grouped GEMM 2 (x routing weight) -> top-k sum.
// Five launches on one stream (four for up to four tokens, three for one); all intermediates live in the
// caller's workspace.
// ---------------------------------------------------------------------------------------
namespace {
struct MoeWs {
  int64_t sorted, expert, post, cumsum, xq, xs, c1, aq, as, c3, total;
  int64_t max_padded, max_blocks;
  int64_t few_padded, few_blocks;  // the same bounds for blocks of 4 (calls of at most four tokens), else 0
};
inline int64_t up256(int64_t v) { return (v + 255) & ~(int64_t)255; }
MoeWs moe_ws_layout(int64_t M, int64_t H, int64_t I, int E, int topk, int block_m) {
  MoeWs w;
  const int64_t T = M * topk;
  w.max_padded = T < E + 1 ? T * block_m : T + (int64_t)(E + 1) * (block_m - 1);
  w.max_blocks = (w.max_padded + block_m - 1) / block_m;
  w.few_padded = M > 4 ? 0 : (T < E + 1 ? T * 4 : ((T + (int64_t)(E + 1) * 3 + 3) / 4) * 4);
  w.few_blocks = w.few_padded / 4;
  int64_t o = 0;
  w.sorted = o; o = up256(o + (w.max_padded > w.few_padded ? w.max_padded : w.few_padded) * 4);
  w.expert = o; o = up256(o + (w.max_blocks > w.few_blocks ? w.max_blocks : w.few_blocks) * 4);
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
  // Measured on the DeepSeek-V3 layer (256 experts, top-8), layer time in us by block height:
  //   rows/expert    8      10     12     16     24     32     48     56     64     96     112    128
  //   16            1886   2030   2229   2896          5114
  //   64            1946   1973   1946   1978   2038   2091   2276   2456   2747   3141   3389   4147
  //   128                         1953   1970   2019   2075   2176   2220   2272   2458   2685   3236
  //   192                         1976   1989   2024   2068   2184   2233   2287   2482   2577   2672
  // The streaming kernel (16) wins while an expert's rows fit one MFMA row group.  Above that the tile kernels: 64-slot
  // blocks for a few more rows, then 128-slot blocks (from there on a launch has more tiles than CUs and runs the
  // persistent walk, whose first GEMM also applies the activation), and 192-slot blocks once experts start to
  // overflow 128 slots (an expert's second block streams nothing new but still costs a tile).
  if (rows < 10) return 16;
  if (rows < 14) return 64;
  if (rows <= 104) return 128;
  return 192;
}
int grouped_block_m(int64_t rows, int E) { return moe_auto_block(rows, E, 1); }
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
  int rc = SGLAMD_OK;
  // Decode-sized calls run with fewer launches.  Up to four tokens the activation kernel goes: the first GEMM's
  // tiles pair gate and up rows and write silu(gate) * up, the second GEMM quantises those 16-bit rows itself, at
  // most four per tile -- so these calls align the routing to blocks of 4 (a tile then holds one such block; an
  // expert named more than four times, which takes repeated ids within a token, gets several).  A single token
  // also drops the sorting / quantising launch in front: both GEMMs sort the handful of routed pairs themselves and
  // the first one quantises the hidden state itself (three launches; with more tokens the quantised rows of K = H
  // bytes each would crowd the weight rings out of LDS: measured 150 against 120 us at two tokens).  Every variant produces the bits of the five-launch sequence.
  // SGLAMD_MOE_FUSE=1 keeps the launch in front, SGLAMD_MOE_FUSE=0 the whole sequence.
  static const int fuse_level = getenv("SGLAMD_MOE_FUSE") ? atoi(getenv("SGLAMD_MOE_FUSE")) : 2;
  const bool fuse_act = fuse_level >= 1 && block_m == 16 && M <= 4 && T <= 32 && I % 256 == 0 &&
                        M * H * 2 < 0x7ffffff0ll && 2 * I * H < 0x7ffffff0ll && T * I * 2 < 0x7ffffff0ll;
  // (T <= E: the in-kernel sort may open up to one block per pair, which is what the block bound then allows)
  const bool fuse_all = fuse_act && fuse_level >= 2 && M == 1 && T <= E;
  if (!fuse_all) {
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
    const size_t lds = moe_align_lds_bytes(nb);
    const int parts = moe_align_parts(T);
    const unsigned blocks = (unsigned)parts + (unsigned)ceil_div(qa.num_groups * 8, 1024);
    hipStream_t st = (hipStream_t)stream;
#define SGLAMD_PROLOGUE(IDT, TT)                                                                                       \
  do {                                                                                                                 \
    auto k = moe_prologue_kernel<IDT, TT>;                                                                             \
    SGLAMD_RAISE_LDS(k, lds);                                                                                          \
    hipLaunchKernelGGL(k, dim3(blocks), dim3(1024), lds, st, (const IDT*)topk_ids, sorted, expert, post, cumsum, nb,   \
                       fuse_act ? 4 : block_m, (int)T, (int)(fuse_act ? w.few_padded : w.max_padded), parts, qa);      \
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
  if (fuse_act) {
    const int64_t expect = T < w.max_blocks ? T : w.max_blocks;
    GemmArgs g = {};
    if (fuse_all) {
      g.A16 = hidden;
      g.lda16 = H * 2;
      g.act_mode = 1;
      g.q_eps = 1e-10f;
      g.q_min = -448.f;
      g.q_max = 448.f;
      g.route_ids = topk_ids;
      g.route_ids_i64 = ids_dtype == SGLAMD_I64;
      g.route_experts = E;
    } else {
      g.A = ws + w.xq;
      g.lda = H;
      g.sa = (const float*)(ws + w.xs);
      g.sa_sm = KB1;
      g.sa_sk = 1;
    }
    g.B = (const uint8_t*)w13;
    g.ldb = H;
    g.b_expert_stride = 2 * I * H;
    g.sb = w13_scale;
    g.sb_se = (2 * I / 128) * KB1;
    g.sb_sn = KB1;
    g.sb_sk = 1;
    g.C = ws + w.c1;  // [T, I] activations
    g.ldc = I;
    g.M = (int)T;
    g.N = (int)(2 * I);
    g.K = (int)H;
    g.sorted_ids = sorted;
    g.expert_ids = expert;
    g.num_post_pad = post;
    g.top_k = topk;
    g.num_valid = (int)T;
    g.max_blocks_m = (int)(fuse_all ? w.max_blocks : w.few_blocks);
    g.sorted_stride = fuse_all ? 0 : 4;
    g.epi_silu = 1;
    g.act_hidden = I;
    hipStream_t st = (hipStream_t)stream;
    if (!fuse_all)
      rc = dtype == SGLAMD_BF16 ? gemm8_skinny_launch_fn<1, 2, GEMM_BLOCK_FP8, BF16, true>(g, st, expect)
                                : gemm8_skinny_launch_fn<1, 2, GEMM_BLOCK_FP8, F16, true>(g, st, expect);
    else
      rc = dtype == SGLAMD_BF16 ? gemm8_skinny_launch_fn<1, 2, GEMM_BLOCK_FP8, BF16, true, 1>(g, st, expect)
                                : gemm8_skinny_launch_fn<1, 2, GEMM_BLOCK_FP8, F16, true, 1>(g, st, expect);
    if (rc) return rc;
    GemmArgs h = {};
    h.A16 = ws + w.c1;
    h.lda16 = I * 2;
    h.act_mode = 1;
    h.q_eps = 1e-10f;
    h.q_min = -448.f;
    h.q_max = 448.f;
    h.B = (const uint8_t*)w2;
    h.ldb = I;
    h.b_expert_stride = H * I;
    h.sb = w2_scale;
    h.sb_se = (H / 128) * KB2;
    h.sb_sn = KB2;
    h.sb_sk = 1;
    h.C = ws + w.c3;
    h.ldc = H;
    h.M = (int)T;
    h.N = (int)H;
    h.K = (int)I;
    h.sorted_ids = sorted;
    h.expert_ids = expert;
    h.num_post_pad = post;
    h.topk_w = topk_weights;
    h.top_k = 1;
    h.num_valid = (int)T;
    h.mul_weight = 1;
    h.max_blocks_m = (int)(fuse_all ? w.max_blocks : w.few_blocks);
    h.sorted_stride = fuse_all ? 0 : 4;
    if (fuse_all) {
      h.route_ids = topk_ids;
      h.route_ids_i64 = ids_dtype == SGLAMD_I64;
      h.route_experts = E;
    }
    rc = dtype == SGLAMD_BF16 ? gemm8_skinny_launch_actquant<BF16>(h, (hipStream_t)stream, expect)
                              : gemm8_skinny_launch_actquant<F16>(h, (hipStream_t)stream, expect);
    if (rc) return rc;
    return sglamd_moe_sum_reduce(ws + w.c3, out, dtype, M, topk, H, routed_scaling_factor, stream);
  }
  // Where the persistent walk takes the first GEMM, its epilogue applies SiLU * up and the group quantisation
  // itself and writes the second GEMM's operand directly (same bits as the two launches it replaces).
  bool act_fused = false;
  if ((block_m == 192 || (block_m == 128 && moe_persist128_enabled())) && moe_persist_enabled() && moe_actq_enabled() &&
      I % 128 == 0) {
    GemmArgs g = {};
    g.A = ws + w.xq;
    g.lda = H;
    g.B = (const uint8_t*)w13;
    g.ldb = H;
    g.b_expert_stride = 2 * I * H;
    g.sa = (const float*)(ws + w.xs);
    g.sa_sm = KB1;
    g.sa_sk = 1;
    g.sb = w13_scale;
    g.sb_se = (2 * I / 128) * KB1;
    g.sb_sn = KB1;
    g.sb_sk = 1;
    g.C = ws + w.aq;                 // [T, I] e4m3
    g.ldc = I;
    g.A16 = ws + w.as;               // [T, I / 128] group scales, written by the kernel
    g.M = (int)T;
    g.N = (int)(2 * I);
    g.K = (int)H;
    g.sorted_ids = sorted;
    g.expert_ids = expert;
    g.num_post_pad = post;
    g.top_k = topk;
    g.num_valid = (int)T;
    g.max_blocks_m = (int)w.max_blocks;
    if (gemm8_moe_persist_ok(g) && (int64_t)(2 * I / 256) * g.max_blocks_m > device_cus()) {
      if (block_m == 192)
        rc = dtype == SGLAMD_BF16 ? gemm8_moe_persist_launch<GEMM_BLOCK_FP8, BF16, 3, true>(g, (hipStream_t)stream)
                                  : gemm8_moe_persist_launch<GEMM_BLOCK_FP8, F16, 3, true>(g, (hipStream_t)stream);
      else
        rc = dtype == SGLAMD_BF16 ? gemm8_moe_persist_launch<GEMM_BLOCK_FP8, BF16, 2, true>(g, (hipStream_t)stream)
                                  : gemm8_moe_persist_launch<GEMM_BLOCK_FP8, F16, 2, true>(g, (hipStream_t)stream);
      if (rc) return rc;
      act_fused = true;
    }
  }
  if (!act_fused) {
    rc = sglamd_fused_moe_block_fp8_gemm(ws + w.xq, H, (const float*)(ws + w.xs), KB1, 1, w13, 2 * I * H, H, w13_scale,
                                         (2 * I / 128) * KB1, KB1, 1, ws + w.c1, 2 * I, dtype, sorted, expert, post,
                                         nullptr, T, topk, 0, block_m, w.max_blocks, 2 * I, H, stream);
    if (rc) return rc;
    rc = sglamd_silu_mul_group_quant_8bit(ws + w.c1, dtype, ws + w.aq, SGLAMD_FP8_E4M3, ws + w.as, T, I, 128,
                                          SGLAMD_SCALE_ROW_MAJOR, 0, 1e-10f, -448.f, 448.f,
                                          SGLAMD_QUANT_FORM_RECIPROCAL, stream);
    if (rc) return rc;
  }
  rc = sglamd_fused_moe_block_fp8_gemm(ws + w.aq, I, (const float*)(ws + w.as), KB2, 1, w2, H * I, I, w2_scale,
                                       (H / 128) * KB2, KB2, 1, ws + w.c3, H, dtype, sorted, expert, post, topk_weights,
                                       T, 1, 1, block_m, w.max_blocks, H, I, stream);
  if (rc) return rc;
  return sglamd_moe_sum_reduce(ws + w.c3, out, dtype, M, topk, H, routed_scaling_factor, stream);
}

// ---------------------------------------------------------------------------------------
// The same layer for callers that cannot allocate device memory: the intermediates live in a
// file-scope device array instead of a caller workspace.
// ---------------------------------------------------------------------------------------
#define SGLAMD_MOE_STATIC_SCRATCH_BYTES (16ll << 20)
static __device__ __align__(256) uint8_t scratch[SGLAMD_MOE_STATIC_SCRATCH_BYTES];

// Device address of `scratch` on the current device.  Every GPU holds its own copy of the array at its own
// address, so the address is looked up once per device, with that device current, and kept.
static int moe_static_scratch(void** out) {
  static void* ptrs[32] = {};
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(SGLAMD_EHIP, "hipGetDevice: %s", hipGetErrorString(e));
  SGLAMD_REQUIRE(dev >= 0 && dev < 32, SGLAMD_ENOTSUP, "fused_moe_static: device index %d is beyond 31", dev);
  if (!ptrs[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) return fail(SGLAMD_EHIP, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
    ptrs[dev] = p;
  }
  *out = ptrs[dev];
  return SGLAMD_OK;
}

extern "C" int64_t sglamd_fused_moe_block_fp8_static_max_bytes(void) { return SGLAMD_MOE_STATIC_SCRATCH_BYTES; }

extern "C" int sglamd_fused_moe_block_fp8_static(const void* hidden, int dtype, int64_t M, int64_t H, int64_t I, int E,
                                                 int topk, const void* w13, const float* w13_scale, const void* w2,
                                                 const float* w2_scale, const float* topk_weights,
                                                 const void* topk_ids, int ids_dtype, void* out,
                                                 float routed_scaling_factor, int block_m, void* stream) {
  SGLAMD_REQUIRE(M > 0 && H > 0 && I > 0 && E > 0 && topk > 0, SGLAMD_EINVAL, "fused_moe_static: bad M/H/I/E/topk");
  const int64_t need = sglamd_fused_moe_block_fp8_workspace(M, H, I, E, topk, block_m);
  SGLAMD_REQUIRE(need > 0 && need <= SGLAMD_MOE_STATIC_SCRATCH_BYTES, SGLAMD_EINVAL,
                 "fused_moe_static: M=%lld tokens (H=%lld, I=%lld, E=%d, topk=%d) need %lld bytes of scratch, the "
                 "built-in array holds %lld; use sglamd_fused_moe_block_fp8 with a workspace",
                 (long long)M, (long long)H, (long long)I, E, topk, (long long)need,
                 (long long)SGLAMD_MOE_STATIC_SCRATCH_BYTES);
  void* ws = nullptr;
  const int rc = moe_static_scratch(&ws);
  if (rc) return rc;
  return sglamd_fused_moe_block_fp8(hidden, dtype, M, H, I, E, topk, w13, w13_scale, w2, w2_scale, topk_weights,
                                    topk_ids, ids_dtype, out, routed_scaling_factor, block_m, ws,
                                    SGLAMD_MOE_STATIC_SCRATCH_BYTES, stream);
}
