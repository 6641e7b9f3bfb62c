// Large-M FP8 GEMM for gfx950: 256 x (64*WGN) tile of C per workgroup, 2 x WGN wavefronts
// each owning 128 x 64, v_mfma_f32_32x32x64_f8f6f4, operands streamed global -> LDS with
// buffer_load ... lds (no staging registers, out-of-range rows read as zero).
//
// Why 32x32x64.  One MFMA of this shape occupies the matrix pipe for 16 passes and leaves
// about three quarters of that time free for VALU issue on the same SIMD; the 16x16x128
// shape leaves half.  The block-scaled GEMM needs one v_fma per accumulator element per
// 128-wide K block (acc += partial * scale): 16 v_fma per pair of 32x32x64 MFMAs, which fits
// in the free issue slots of this shape with room for scale and address arithmetic.
//
// LDS: rows of 128 bytes (one K block of one matrix row); the eight 16-byte chunks of a row
// are XOR-swizzled with (row >> 1) & 7.  LDS serves 256 bytes (two rows) per clock, so the
// 32-row fragment reads of the MFMA operands are conflict free.  A direct-to-LDS load writes
// the 64 lanes' 16-byte pieces to 64 consecutive slots, so the swizzle is applied on the
// global side: lane L of a load covering eight rows fetches chunk (L%8) ^ key(row) of row L/8.
// Two stages; the loads of K block kb+1 are in flight while block kb is multiplied; one
// workgroup barrier per K block.
#pragma once
#include <type_traits>

#include "gemm_core.h"

namespace sglamd {

typedef __attribute__((address_space(3))) void* lds_ptr_t;

template <int WGN, int MT>
constexpr int gemm8_big_smem() {
  return 2 * ((64 * MT + 64 * WGN) * 128 + 64 * MT * 4);
}

// MT = 32-row tiles per wave along M (4 -> 256-row workgroup tile, 2 -> 128-row tile).
// Split-K: gridDim.y slices of the K blocks; with more than one slice every workgroup stores its fp32
// partial tile (block mode: already scaled; row mode: raw accumulators) to slab blockIdx.y of g.C, which
// then points at a [slices, M, N] fp32 workspace that splitk_reduce_kernel sums.
// MOE: the row tiles are the sorted blocks of the fused-MoE schedule (block height = 64*MT): activation rows
// are gathered through sorted_token_ids (row = id / top_k, padding slots read zeros), the weight matrix and
// its scales are those of expert_ids[block], results are scattered to row id with the routing weight applied.
template <int MODE, typename OT, int WGN, int MT, bool MOE = false>
__global__ __launch_bounds__(128 * WGN) void gemm8_big_kernel(GemmArgs g) {
#if defined(__HIP_DEVICE_COMPILE__)  // the host pass only needs the launch stub; buffer-resource builtins are device-only
  constexpr int BM = 64 * MT, BN = 64 * WGN, NW = 2 * WGN, WTM = 32 * MT;
  constexpr int A_LOADS = (BM / 8) / NW;  // 1 KB (8 rows) per wave-wide load
  constexpr int B_LOADS = (BN / 8) / NW;
  constexpr int STAGE = (BM + BN) * 128 + BM * 4;
  typedef typename std::conditional<MODE == GEMM_ROW_INT8, v16i, v16f>::type acc16_t;

  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  __shared__ int s_rows[MOE ? BM : 1];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WGN, wn = wave % WGN;

  const int tiles_n = (g.N + BN - 1) / BN;
  const int tiles_m = MOE ? g.max_blocks_m : (g.M + BM - 1) / BM;
  const int pid = MOE ? (int)blockIdx.x : xcd_remap(blockIdx.x, tiles_m * tiles_n);
  int pid_m, pid_n;
  if (MOE) {
    // consecutive workgroups walk the column tiles of one sorted block: they share its gathered rows, and
    // the blocks of one expert follow each other, so its weights are re-read while still cached
    pid_m = pid / tiles_n;
    pid_n = pid % tiles_n;
  } else {
#ifndef SGLAMD_BIG_GM
#define SGLAMD_BIG_GM 8
#endif
    constexpr int GM = SGLAMD_BIG_GM;
    const int in_group = GM * tiles_n;
    const int group = pid / in_group;
    const int first_m = group * GM;
    const int gsz = min(tiles_m - first_m, GM);
    pid_m = first_m + (pid % in_group) % gsz;
    pid_n = (pid % in_group) / gsz;
  }
  const int m0 = pid_m * BM, n0 = pid_n * BN;

  int expert = 0;
  if (MOE) {
    if (m0 >= *g.num_post_pad) return;
    expert = g.expert_ids[pid_m];
    for (int r = tid; r < BM; r += 128 * WGN) s_rows[r] = g.sorted_ids[m0 + r];
    __syncthreads();
  }
  const int64_t a_rows = MOE ? g.num_valid / g.top_k : g.M;
  const uint8_t* Bmat = g.B + (MOE ? (int64_t)max(expert, 0) * g.b_expert_stride : 0);

  // Buffer descriptors: byte ranges end at the last valid row, so tile rows past M / N read zeros.
  const __amdgpu_buffer_rsrc_t rsrcA =
      __builtin_amdgcn_make_buffer_rsrc((void*)g.A, 0, (int)min(a_rows * g.lda, (int64_t)0x7fffffff), 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrcB =
      __builtin_amdgcn_make_buffer_rsrc((void*)Bmat, 0, (int)min((int64_t)g.N * g.ldb, (int64_t)0x7fffffff), 0x00020000);

  // per-lane byte offsets of this wave's loads inside the operand tiles
  uint32_t a_voff[A_LOADS], b_voff[B_LOADS];
#pragma unroll
  for (int it = 0; it < A_LOADS; it++) {
    const int row = (wave * A_LOADS + it) * 8 + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    if (MOE) {
      const int tok = s_rows[row];  // padding slots (>= num_valid) land past the descriptor's range: zeros
      a_voff[it] = tok < g.num_valid ? (uint32_t)((tok / g.top_k) * (int)g.lda + chunk * 16) : 0x7ffffff0u;
    } else {
      a_voff[it] = (uint32_t)((m0 + row) * (int)g.lda + chunk * 16);
    }
  }
#pragma unroll
  for (int it = 0; it < B_LOADS; it++) {
    const int row = (wave * B_LOADS + it) * 8 + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    b_voff[it] = (uint32_t)((n0 + row) * (int)g.ldb + chunk * 16);
  }
  // activation scales of the tile rows: waves 0..BM/64-1 fetch 64 rows each (block mode)
  int64_t srow;
  if (MOE) {
    const int tok = s_rows[min(wave * 64 + lane, BM - 1)];
    srow = tok < g.num_valid ? tok / g.top_k : 0;
  } else {
    srow = min(m0 + wave * 64 + lane, g.M - 1);
  }
  const float* sa_src = g.sa + srow * g.sa_sm;

  // K blocks of this split-K slice
  const int nkb_all = g.K >> 7;
  const int kb_begin = (int)((int64_t)nkb_all * blockIdx.y / gridDim.y);
  const int kb_end = (int)((int64_t)nkb_all * (blockIdx.y + 1) / gridDim.y);
  const int nkb = kb_end - kb_begin;

  auto issue_loads = [&](int kb, int stage) {
    uint8_t* base = smem + stage * STAGE;
    const int koff = (kb_begin + kb) << 7;
#pragma unroll
    for (int it = 0; it < A_LOADS; it++)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrcA, (lds_ptr_t)(base + (wave * A_LOADS + it) * 1024), 16, a_voff[it],
                                               koff, 0, 0);
#pragma unroll
    for (int it = 0; it < B_LOADS; it++)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrcB, (lds_ptr_t)(base + BM * 128 + (wave * B_LOADS + it) * 1024), 16,
                                               b_voff[it], koff, 0, 0);
    if (MODE == GEMM_BLOCK_FP8 && wave < BM / 64) {
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(sa_src + (int64_t)(kb_begin + kb) * g.sa_sk),
                                       (lds_ptr_t)(base + (BM + BN) * 128 + wave * 256), 4, 0, 0);
    }
  };

  // fragment of a 32x32x64 MFMA operand: lane -> row lane%32, 32 bytes at 64*h + 32*(lane/32)
  const int frow = lane & 31, fk = lane >> 5;
  auto frag = [&](const uint8_t* tile, int row, int h) -> v8i {
    const uint8_t* p = tile + row * 128;
    const int sw = (row >> 1) & 7;
    const int c = h * 4 + fk * 2;
    v4i lo = *(const v4i*)(p + ((c ^ sw) << 4));
    v4i hi = *(const v4i*)(p + (((c + 1) ^ sw) << 4));
    return v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  };

  acc16_t acc[MT][2];
#pragma unroll
  for (int i = 0; i < MT; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0;

  const float* sb_ptr = g.sb + (MOE ? (int64_t)max(expert, 0) * g.sb_se : 0) + (int64_t)(min(n0 + wn * 64, g.N - 1) >> 7) * g.sb_sn;
  float sb_next = (MODE == GEMM_BLOCK_FP8) ? sb_ptr[(int64_t)kb_begin * g.sb_sk] : 1.f;

  issue_loads(0, 0);

  for (int kb = 0; kb < nkb; kb++) {
    const int cur = kb & 1;
    // own direct-to-LDS loads of block kb have landed (vmcnt(0)); after the barrier every wave's have, and
    // every wave is done reading stage cur^1
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
#ifdef SGLAMD_EXP_NOLOAD
    if (kb == 0 && nkb > 1) issue_loads(1, 1);
#else
    if (kb + 1 < nkb) issue_loads(kb + 1, cur ^ 1);
#endif
    const float sbv = sb_next;
    if (MODE == GEMM_BLOCK_FP8 && kb + 1 < nkb) sb_next = sb_ptr[(int64_t)(kb_begin + kb + 1) * g.sb_sk];

    const uint8_t* sA = smem + cur * STAGE;
    const uint8_t* sB = sA + BM * 128;
    const float* sS = (const float*)(sA + (BM + BN) * 128);
    v8i wf[2][2];
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int h = 0; h < 2; h++) wf[j][h] = frag(sB, wn * 64 + j * 32 + frow, h);
    // The activation fragments and scale of row-tile i+1 are requested before the MFMAs of row-tile i are
    // issued, so their LDS latency is covered by a full tile pair of matrix work.
    v8i xc0 = frag(sA, wm * WTM + frow, 0), xc1 = frag(sA, wm * WTM + frow, 1);
    float sa_cur = (MODE == GEMM_BLOCK_FP8) ? sS[wm * WTM + frow] : 1.f;
#pragma unroll
    for (int i = 0; i < MT; i++) {
      v8i xn0 = xc0, xn1 = xc1;
      float sa_nxt = sa_cur;
      if (i < MT - 1) {
        const int xrow = wm * WTM + (i + 1) * 32 + frow;
        xn0 = frag(sA, xrow, 0);
        xn1 = frag(sA, xrow, 1);
        if (MODE == GEMM_BLOCK_FP8) sa_nxt = sS[xrow];
      }
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (MODE == GEMM_BLOCK_FP8) {
        const float sc = sa_cur * sbv;
#pragma unroll
        for (int j = 0; j < 2; j++) {
          v16f q;
#pragma unroll
          for (int r = 0; r < 16; r++) q[r] = 0.f;
          q = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf[j][0], xc0, q, 0, 0, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
          q = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf[j][1], xc1, q, 0, 0, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
#pragma unroll
          for (int r = 0; r < 16; r++) acc[i][j][r] = fmaf(q[r], sc, acc[i][j][r]);
        }
      } else if constexpr (MODE == GEMM_ROW_FP8) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf[j][0], xc0, acc[i][j], 0, 0, 0, 0x7f7f7f7f, 0,
                                                                      0x7f7f7f7f);
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf[j][1], xc1, acc[i][j], 0, 0, 0, 0x7f7f7f7f, 0,
                                                                      0x7f7f7f7f);
        }
      } else {
        // int8: v_mfma_i32_32x32x32_i8 takes 16 bytes per lane; the 32 bytes a lane holds per 64-byte half are two
        // such slices, and pairing low with low / high with high on both operands covers every k exactly once
#pragma unroll
        for (int j = 0; j < 2; j++) {
#pragma unroll
          for (int h = 0; h < 2; h++) {
            const v8i w = wf[j][h];
            const v8i x = h == 0 ? xc0 : xc1;
            const v4i wlo = {w[0], w[1], w[2], w[3]}, whi = {w[4], w[5], w[6], w[7]};
            const v4i xlo = {x[0], x[1], x[2], x[3]}, xhi = {x[4], x[5], x[6], x[7]};
            acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wlo, xlo, acc[i][j], 0, 0, 0);
            acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(whi, xhi, acc[i][j], 0, 0, 0);
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      xc0 = xn0;
      xc1 = xn1;
      sa_cur = sa_nxt;
    }
  }

  // epilogue: register r of tile (i, j) is C[m = .. + lane%32][n = .. + 8*(r/4) + 4*(lane/32) + r%4]
  typedef typename OT::storage OS;
  const bool split = gridDim.y > 1;
  float* slab = (float*)g.C + (int64_t)blockIdx.y * g.M * g.N;
#pragma unroll
  for (int i = 0; i < MT; i++) {
    int m = m0 + wm * WTM + i * 32 + frow;
    float wgt = 1.f;
    if (MOE) {
      m = s_rows[wm * WTM + i * 32 + frow];
      if (m >= g.num_valid) continue;
      if (g.mul_weight) wgt = g.topk_w[m];
      if (expert < 0) wgt = 0.f;
    } else if (m >= g.M) {
      continue;
    }
    float sam = 1.f;
    if (MODE != GEMM_BLOCK_FP8 && !split) sam = g.sa[m];
    OS* crow = (OS*)g.C + (int64_t)m * g.ldc;
#pragma unroll
    for (int j = 0; j < 2; j++) {
#pragma unroll
      for (int rq = 0; rq < 4; rq++) {
        const int n = n0 + wn * 64 + j * 32 + 8 * rq + 4 * fk;
        if (n >= g.N) continue;
        float v[4];
        if (split) {
          // fp32 partial sums (int8: the int32 partial sums, bit-stored in the same 4-byte slots)
          float* prow = slab + (int64_t)m * g.N + n;
#pragma unroll
          for (int r = 0; r < 4; r++) {
            if constexpr (MODE == GEMM_ROW_INT8) v[r] = __int_as_float(acc[i][j][rq * 4 + r]);
            else v[r] = acc[i][j][rq * 4 + r];
          }
          if (n + 3 < g.N && ((((uintptr_t)prow) & 15) == 0)) {
            *(v4f*)prow = v4f{v[0], v[1], v[2], v[3]};
          } else {
            for (int r = 0; r < 4 && n + r < g.N; r++) prow[r] = v[r];
          }
          continue;
        }
#pragma unroll
        for (int r = 0; r < 4; r++) v[r] = (float)acc[i][j][rq * 4 + r] * wgt;
        if constexpr (MODE != GEMM_BLOCK_FP8) {
#pragma unroll
          for (int r = 0; r < 4; r++) {
            const float sbn = (n + r) < g.N ? g.sb[n + r] : 0.f;
            if constexpr (MODE == GEMM_ROW_FP8) v[r] = v[r] * sbn * sam;
            else v[r] = v[r] * (sbn * sam);
            if (g.bias) v[r] += OT::to_f32(((const OS*)g.bias)[(n + r) < g.N ? n + r : 0]);
          }
        }
        if (n + 3 < g.N && ((((uintptr_t)(crow + n)) & 7) == 0)) {
          OS o[4] = {OT::from_f32(v[0]), OT::from_f32(v[1]), OT::from_f32(v[2]), OT::from_f32(v[3])};
          v2i w;
          __builtin_memcpy(&w, o, 8);
          *(v2i*)(crow + n) = w;
        } else {
          for (int r = 0; r < 4 && n + r < g.N; r++) crow[n + r] = OT::from_f32(v[r]);
        }
      }
    }
  }
#endif
}

// Preconditions beyond the generic kernel's: K % 128 == 0 and both operands smaller than 2 GiB
// (buffer descriptors carry 32-bit ranges and offsets).
static inline bool gemm8_big_ok(const GemmArgs& g) {
  return (g.K % 128) == 0 && (int64_t)g.M * g.lda < 0x7fffffffll && (int64_t)g.N * g.ldb < 0x7fffffffll;
}

// out[m, n] = cast(sum_s slab[s][m][n]) for block mode; row mode applies sa[m] * sb[n] (+ bias) to the sum.
template <int MODE, typename OT>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ ws, int slices, GemmArgs g) {
  typedef typename OT::storage OS;
  const int64_t total4 = ((int64_t)g.M * g.N) >> 2;  // N % 4 == 0 is a precondition of the split path
  for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < total4; idx += (int64_t)gridDim.x * 256) {
    const int64_t e = idx << 2;
    float v[4];
    if constexpr (MODE == GEMM_ROW_INT8) {
      v4i a = *(const v4i*)(ws + e);
      for (int s = 1; s < slices; s++) a += *(const v4i*)(ws + (int64_t)s * g.M * g.N + e);
#pragma unroll
      for (int r = 0; r < 4; r++) v[r] = (float)a[r];
    } else {
      v4f a = *(const v4f*)(ws + e);
      for (int s = 1; s < slices; s++) a += *(const v4f*)(ws + (int64_t)s * g.M * g.N + e);
#pragma unroll
      for (int r = 0; r < 4; r++) v[r] = a[r];
    }
    const int64_t m = e / g.N;
    const int n = (int)(e % g.N);
    if (MODE != GEMM_BLOCK_FP8) {
      const float sam = g.sa[m];
#pragma unroll
      for (int r = 0; r < 4; r++) {
        if constexpr (MODE == GEMM_ROW_FP8) v[r] = v[r] * g.sb[n + r] * sam;
        else v[r] = v[r] * (g.sb[n + r] * sam);
        if (g.bias) v[r] += OT::to_f32(((const OS*)g.bias)[n + r]);
      }
    }
    OS* crow = (OS*)g.C + m * g.ldc + n;
    OS o[4] = {OT::from_f32(v[0]), OT::from_f32(v[1]), OT::from_f32(v[2]), OT::from_f32(v[3])};
    if ((((uintptr_t)crow) & 7) == 0) {
      v2i w;
      __builtin_memcpy(&w, o, 8);
      *(v2i*)crow = w;
    } else {
#pragma unroll
      for (int r = 0; r < 4; r++) crow[r] = o[r];
    }
  }
}

// Tile height (128 or 256 rows) and number of K slices for the large-M kernel.  One workgroup occupies a
// CU, so the cost of a launch is (rounds of 256 workgroups) x (work per workgroup); the 128-row tile does
// half the work per workgroup at a somewhat lower MFMA efficiency and is preferred when it removes a mostly
// empty last round.  K is split when the tile grid alone cannot fill the chip (every slice keeps >= 8 blocks).
struct BigConfig {
  int bm, slices;
};
static inline int gemm8_big_slices(int64_t tiles, int64_t N, int64_t K) {
  const int64_t nkb = K >> 7;
  if (tiles >= 160 || (N & 3)) return 1;
  int64_t s = 256 / tiles;
  if (s > nkb / 8) s = nkb / 8;
  if (s > 16) s = 16;
  return s < 1 ? 1 : (int)s;
}
static inline BigConfig gemm8_big_config(int64_t M, int64_t N, int64_t K) {
  BigConfig best = {256, 1};
  double best_cost = 1e30;
  for (int bm = 128; bm <= 256; bm += 128) {
    if (bm == 256 && M <= 128) break;
    const int64_t tiles = ((M + bm - 1) / bm) * ((N + 255) / 256);
    const int slices = gemm8_big_slices(tiles, N, K);
    const int64_t rounds = (tiles * slices + 255) / 256;
    const double cost = (double)rounds * bm / slices * (bm == 128 ? 1.15 : 1.0) + (slices > 1 ? 8.0 : 0.0);
    if (cost < best_cost) {
      best_cost = cost;
      best = {bm, slices};
    }
  }
  return best;
}

template <int MODE, typename OT, int WGN, int MT>
static int gemm8_big_launch(const GemmArgs& g, hipStream_t st, int slices, void* workspace) {
  auto kern = gemm8_big_kernel<MODE, OT, WGN, MT>;
  constexpr int smem = gemm8_big_smem<WGN, MT>();
  hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
  if (e != hipSuccess) return fail(SGLAMD_EHIP, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  constexpr int BN = 64 * WGN, BM = 64 * MT;
  const int64_t blocks = (int64_t)((g.N + BN - 1) / BN) * ((g.M + BM - 1) / BM);
  if (blocks > 0x7fffffff) return fail(SGLAMD_EINVAL, "gemm: grid too large");
  if (slices <= 1) {
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks, 1), dim3(128 * WGN), smem, st, g);
    return check_launch("gemm8_big");
  }
  GemmArgs part = g;
  part.C = workspace;
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks, (unsigned)slices), dim3(128 * WGN), smem, st, part);
  int rc = check_launch("gemm8_big(split-K)");
  if (rc) return rc;
  const int64_t total4 = ((int64_t)g.M * g.N) >> 2;
  const unsigned rblocks = (unsigned)(total4 / 256 + 1 < 4096 ? total4 / 256 + 1 : 4096);
  hipLaunchKernelGGL((splitk_reduce_kernel<MODE, OT>), dim3(rblocks), dim3(256), 0, st, (const float*)workspace, slices,
                     g);
  return check_launch("splitk_reduce");
}

// Fused-MoE launch of the same kernel: sorted blocks of 128 slots, no split-K.
template <typename OT>
static int gemm8_big_moe_launch(const GemmArgs& g, hipStream_t st) {
  auto kern = gemm8_big_kernel<GEMM_BLOCK_FP8, OT, 4, 2, true>;
  constexpr int smem = gemm8_big_smem<4, 2>();
  hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
  if (e != hipSuccess) return fail(SGLAMD_EHIP, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  const int64_t blocks = (int64_t)((g.N + 255) / 256) * g.max_blocks_m;
  if (blocks <= 0) return SGLAMD_OK;
  if (blocks > 0x7fffffff) return fail(SGLAMD_EINVAL, "gemm: grid too large");
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks, 1), dim3(512), smem, st, g);
  return check_launch("gemm8_big(moe)");
}

}  // namespace sglamd
