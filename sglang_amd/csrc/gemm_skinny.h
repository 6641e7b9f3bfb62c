// Small-M ("decode") 8-bit GEMM for gfx950: a weight-streaming kernel.  With at most 64
// activation rows the multiply is bound by reading W once from HBM, so the kernel is organised
// around that stream and nothing else:
//   * a workgroup owns 16 weight rows (one MFMA tile of n) and all K; its KW wavefronts take the
//     128-byte K blocks round-robin (wave w: kb = w, w + KW, ...), so the waves of a workgroup read
//     adjacent 128-byte pieces of the same 16 rows;
//   * W is fetched fully coalesced: 8 lanes read one 128-byte row piece, a wave-wide 16-byte load
//     covers 8 rows, two cover the 16-row tile (measured: this pattern streams at 6.1-6.6 TB/s, the
//     MFMA operand pattern -- 16 rows x 16 bytes per 16 lanes -- only at 4.3-5.0 TB/s).  PD K blocks
//     are in flight per wave in a register ring;
//   * each wave re-shapes a block into MFMA operand layout through a private 2 KB LDS scratch
//     (swizzled ds_write_b128 / ds_read_b128, no barrier: LDS executes one wave's accesses in order);
//   * the activation tiles (FM tiles of 16 rows) and the scales are tiny and L2 resident; they are
//     fetched and re-shaped the same way alongside the weights;
//   * one v_mfma_f32_16x16x128_f8f6f4 per tile and K block with the weight fragment as first
//     operand (lane ends up with 4 consecutive n of one m), folded into the accumulator with the
//     block scale; the KW partial sums meet in LDS and leave as 8-byte stores.
// The same kernel walks the fused-MoE sorted-block schedule (MOE = true): tile rows are gathered
// through sorted_token_ids, the expert comes from expert_ids.
#pragma once
#include <stdlib.h>

// prefetch depth (K blocks in flight per wave) of the 3-4 loads-per-block configurations; tuning macro
#ifndef SGLAMD_SKINNY_PD_MID
#define SGLAMD_SKINNY_PD_MID 3
#endif

#include "gemm_core.h"

namespace sglamd {

// Byte offset inside a row at which lane chunk `lchunk` (16-byte piece lchunk of a 128-byte K block) fetches
// K block `kb`, and whether the piece lies past the end of K (ragged last block; K % 16 == 0, K >= 16).  A dead
// piece re-reads the first piece of its row, which is always inside the tensor, and is zeroed by the caller.
struct SkinnyPiece {
  int64_t offset;
  bool dead;
};
__host__ __device__ inline SkinnyPiece skinny_piece(int kb, int lchunk, int K) {
  const bool dead = ((kb << 7) + lchunk * 16) >= K;
  return {dead ? 0 : ((int64_t)kb << 7) + lchunk * 16, dead};
}

template <int FM, int FN, int MODE, typename OT, bool MOE, int KW, int PD>
__global__ __launch_bounds__(64 * KW) void gemm8_skinny_kernel(GemmArgs g) {
  typedef typename AccT<MODE>::type acc_t;
  // per-wave re-shape scratch; after the K loop the same memory carries the KW partial tiles
  __shared__ __attribute__((aligned(16))) uint8_t scratch[KW][FN + FM][2048];
  static_assert(FM * FN * 1024 <= (FN + FM) * 2048, "partial tiles must fit in the scratch");
  acc_t(*red)[FM * FN][64] = reinterpret_cast<acc_t(*)[FM * FN][64]>(&scratch[0][0][0]);
  __shared__ int s_rows[FM * 16];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int frow = lane & 15, fk = lane >> 4;

  // A workgroup owns R consecutive weight rows, R <= 16*FN: a launch may trim R so that the number of
  // workgroups is a whole multiple of the CU count (rows past R are neither fetched nor stored).
  const int R = g.rows_per_wg > 0 ? g.rows_per_wg : 16 * FN;
  const int tiles_n = (g.N + R - 1) / R;
  const int pid_n = blockIdx.x % tiles_n;
  const int pid_m = blockIdx.x / tiles_n;
  const int n0 = pid_n * R, m0 = pid_m * (16 * FM);
  const int n_end = min(g.N, n0 + R);

  int expert = 0;
  if (MOE) {
    if (m0 >= *g.num_post_pad) return;
    expert = g.expert_ids[pid_m];
    if (tid < FM * 16) s_rows[tid] = g.sorted_ids[m0 + tid];
    __syncthreads();
  }

  const int nkb = (g.K + 127) >> 7;
  const int n_my = (nkb - wave + KW - 1) / KW;  // K blocks of this wave (may be <= 0)

  // ---- per-lane source pointers: lane l reads chunk l%8 of tile rows l/8 and l/8 + 8 ------------------
  const int lrow = lane >> 3, lchunk = lane & 7;
  const uint8_t* wbase = g.B + (MOE ? (int64_t)max(expert, 0) * g.b_expert_stride : 0) + lchunk * 16;
  const uint8_t* wp0[FN];
  const uint8_t* wp1[FN];
#pragma unroll
  for (int j = 0; j < FN; j++) {
    wp0[j] = wbase + (int64_t)min(n0 + j * 16 + lrow, n_end - 1) * g.ldb;
    wp1[j] = wbase + (int64_t)min(n0 + j * 16 + lrow + 8, n_end - 1) * g.ldb;
  }
  const uint8_t* xp0[FM];
  const uint8_t* xp1[FM];
  const float* sap[FM];
#pragma unroll
  for (int i = 0; i < FM; i++) {
    int64_t r0, r1, rs;
    if (MOE) {
      const int t0 = s_rows[i * 16 + lrow], t1 = s_rows[i * 16 + lrow + 8], ts = s_rows[i * 16 + frow];
      r0 = t0 < g.num_valid ? t0 / g.top_k : 0;
      r1 = t1 < g.num_valid ? t1 / g.top_k : 0;
      rs = ts < g.num_valid ? ts / g.top_k : 0;
    } else {
      r0 = min(m0 + i * 16 + lrow, g.M - 1);
      r1 = min(m0 + i * 16 + lrow + 8, g.M - 1);
      rs = min(m0 + i * 16 + frow, g.M - 1);
    }
    xp0[i] = g.A + r0 * g.lda + lchunk * 16;
    xp1[i] = g.A + r1 * g.lda + lchunk * 16;
    sap[i] = g.sa + rs * g.sa_sm;
  }
  // weight-block scale of the 4 output columns a lane ends up with (a trimmed R may straddle a 128-row block)
  const float* sbp[FN];
#pragma unroll
  for (int j = 0; j < FN; j++)
    sbp[j] = g.sb + (MOE ? (int64_t)max(expert, 0) * g.sb_se : 0) +
             (int64_t)(min(n0 + j * 16 + 4 * fk, g.N - 1) >> 7) * g.sb_sn;
  const bool ktail = (g.K & 127) != 0;

  // wave-private LDS scratch: one 16 x 128-byte tile for W and one per activation tile
  uint8_t* wl = &scratch[wave][0][0];
  const int st0 = lrow * 128 + ((lchunk ^ ((lrow >> 1) & 7)) << 4);              // where this lane's pieces go
  const int st1 = (lrow + 8) * 128 + ((lchunk ^ (((lrow + 8) >> 1) & 7)) << 4);
  const int fsw = (frow >> 1) & 7;                                                // where its fragment comes from
  const int ld0 = frow * 128 + (((2 * fk) ^ fsw) << 4), ld1 = frow * 128 + (((2 * fk + 1) ^ fsw) << 4);

  // ---- register ring of PD K blocks ----------------------------------------------------------------
  v4i wr[PD][FN][2], xr[PD][FM][2];
  float sar[PD][FM], sbr[PD][FN];

  auto load = [&](int s, int it) {
    const int kb = wave + it * KW;
    // a 16-byte piece past the end of K (ragged last block) is not fetched: see skinny_piece; the row
    // pointers already include the lane's chunk offset
    const SkinnyPiece pc = skinny_piece(kb, lchunk, g.K);
    const bool dead = ktail && pc.dead;
    const int64_t ko = pc.offset - lchunk * 16;
#pragma unroll
    for (int j = 0; j < FN; j++) {
      wr[s][j][0] = __builtin_nontemporal_load((const v4i*)(wp0[j] + ko));
      wr[s][j][1] = __builtin_nontemporal_load((const v4i*)(wp1[j] + ko));
      if (dead) wr[s][j][0] = wr[s][j][1] = v4i{0, 0, 0, 0};
    }
#pragma unroll
    for (int i = 0; i < FM; i++) {
      xr[s][i][0] = *(const v4i*)(xp0[i] + ko);
      xr[s][i][1] = *(const v4i*)(xp1[i] + ko);
      if (dead) xr[s][i][0] = xr[s][i][1] = v4i{0, 0, 0, 0};
      if (gemm_is_block(MODE)) sar[s][i] = sap[i][(int64_t)kb * g.sa_sk];
    }
    if (gemm_is_block(MODE)) {
#pragma unroll
      for (int j = 0; j < FN; j++) sbr[s][j] = sbp[j][(int64_t)kb * g.sb_sk];
    }
  };
  auto reshape = [&](uint8_t* tile, const v4i& p0, const v4i& p1) -> v8i {
    *(v4i*)(tile + st0) = p0;
    *(v4i*)(tile + st1) = p1;
    const v4i lo = *(const v4i*)(tile + ld0), hi = *(const v4i*)(tile + ld1);
    return v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  };

  acc_t acc[FM * FN];
#pragma unroll
  for (int i = 0; i < FM * FN; i++) acc[i] = acc_t{0, 0, 0, 0};

#pragma unroll
  for (int s = 0; s < PD; s++)
    if (s < n_my) load(s, s);

  for (int it = 0; it < n_my; it += PD) {
#pragma unroll
    for (int s = 0; s < PD; s++) {
      if (it + s < n_my) {
        v8i wf[FN];
#pragma unroll
        for (int j = 0; j < FN; j++) wf[j] = reshape(wl + j * 2048, wr[s][j][0], wr[s][j][1]);
        v8i xf[FM];
#pragma unroll
        for (int i = 0; i < FM; i++) xf[i] = reshape(wl + (FN + i) * 2048, xr[s][i][0], xr[s][i][1]);
        float sav[FM], sbv[FN];
#pragma unroll
        for (int i = 0; i < FM; i++) sav[i] = gemm_is_block(MODE) ? sar[s][i] : 1.f;
#pragma unroll
        for (int j = 0; j < FN; j++) sbv[j] = gemm_is_block(MODE) ? sbr[s][j] : 1.f;
        if (it + s + PD < n_my) load(s, it + s + PD);
#pragma unroll
        for (int i = 0; i < FM; i++) {
#pragma unroll
          for (int j = 0; j < FN; j++) {
            const v8i w = wf[j];
            acc_t& a = acc[i * FN + j];
            if constexpr (MODE == GEMM_BLOCK_FP8) {
              v4f p = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(w, xf[i], v4f{0, 0, 0, 0}, 0, 0, 0, 0x7f7f7f7f, 0,
                                                                       0x7f7f7f7f);
              const float sc = sav[i] * sbv[j];
#pragma unroll
              for (int r = 0; r < 4; r++) a[r] = fmaf(p[r], sc, a[r]);
            } else if constexpr (MODE == GEMM_ROW_FP8) {
              a = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(w, xf[i], a, 0, 0, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
            } else {
              const v8i x = xf[i];
              v4i wlo = {w[0], w[1], w[2], w[3]}, whi = {w[4], w[5], w[6], w[7]};
              v4i xlo = {x[0], x[1], x[2], x[3]}, xhi = {x[4], x[5], x[6], x[7]};
              if constexpr (MODE == GEMM_BLOCK_INT8) {
                v4i p = __builtin_amdgcn_mfma_i32_16x16x64_i8(wlo, xlo, v4i{0, 0, 0, 0}, 0, 0, 0);
                p = __builtin_amdgcn_mfma_i32_16x16x64_i8(whi, xhi, p, 0, 0, 0);
                const float sc = sav[i] * sbv[j];
#pragma unroll
                for (int r = 0; r < 4; r++) a[r] = fmaf((float)p[r], sc, a[r]);
              } else {
                a = __builtin_amdgcn_mfma_i32_16x16x64_i8(wlo, xlo, a, 0, 0, 0);
                a = __builtin_amdgcn_mfma_i32_16x16x64_i8(whi, xhi, a, 0, 0, 0);
              }
            }
          }
        }
      }
    }
  }

  // ---- reduce the KW partial tiles through LDS ------------------------------------------------------
  if (KW > 1) {
    __syncthreads();  // every wave is done with its scratch
#pragma unroll
    for (int i = 0; i < FM * FN; i++) red[wave][i][lane] = acc[i];
    __syncthreads();
  }

  typedef typename OT::storage OS;
  for (int t = wave; t < FM * FN; t += KW) {
    const int i = t / FN, j = t % FN;
    acc_t a = acc[0];
    if (KW > 1) {
      a = red[0][t][lane];
#pragma unroll
      for (int w = 1; w < KW; w++) a += red[w][t][lane];
    } else {
#pragma unroll
      for (int ii = 0; ii < FM * FN; ii++)
        if (ii == t) a = acc[ii];
    }
    int64_t out_row;
    bool row_ok;
    float wgt = 1.f;
    if (MOE) {
      const int tok = s_rows[i * 16 + frow];
      row_ok = tok < g.num_valid;
      out_row = tok;
      if (row_ok && g.mul_weight) wgt = g.topk_w[tok];
    } else {
      row_ok = (m0 + i * 16 + frow) < g.M;
      out_row = m0 + i * 16 + frow;
    }
    const int n = n0 + j * 16 + 4 * fk;
    if (!row_ok || n >= n_end) continue;
    float v[4];
    float sam = 1.f;
    if (!gemm_is_block(MODE)) sam = g.sa[out_row];
#pragma unroll
    for (int r = 0; r < 4; r++) {
      if constexpr (gemm_is_block(MODE)) {
        v[r] = a[r];
      } else {
        const float sbn = (n + r) < g.N ? g.sb[n + r] : 0.f;
        if constexpr (MODE == GEMM_ROW_FP8) {
          v[r] = a[r] * sbn * sam;
        } else {
          v[r] = (float)a[r] * (sbn * sam);
        }
        if (g.bias) v[r] += OT::to_f32(((const OS*)g.bias)[(n + r) < g.N ? n + r : 0]);
      }
      if (MOE) {
        if (expert < 0) v[r] = 0.f;
        v[r] *= wgt;
      }
    }
    OS* crow = (OS*)g.C + out_row * g.ldc;
    if (n + 3 < g.N && ((((uintptr_t)(crow + n)) & 7) == 0)) {
      OS o[4] = {OT::from_f32(v[0]), OT::from_f32(v[1]), OT::from_f32(v[2]), OT::from_f32(v[3])};
      v2i w2;
      __builtin_memcpy(&w2, o, 8);
      *(v2i*)(crow + n) = w2;
    } else {
      for (int r = 0; r < 4 && n + r < g.N; r++) crow[n + r] = OT::from_f32(v[r]);
    }
  }
}

template <int FM, int FN, int MODE, typename OT, bool MOE, int KW>
static int gemm8_skinny_launch_kw(const GemmArgs& g, hipStream_t st) {
  constexpr int PD = (FM * 2 + FN * 2) <= 4 ? 4 : ((FM * 2 + FN * 2) <= 8 ? SGLAMD_SKINNY_PD_MID : 2);
  const int R = g.rows_per_wg > 0 ? g.rows_per_wg : 16 * FN;
  const int tiles_n = (g.N + R - 1) / R;
  const int tiles_m = MOE ? g.max_blocks_m : (g.M + 16 * FM - 1) / (16 * FM);
  const int64_t blocks = (int64_t)tiles_n * tiles_m;
  if (blocks <= 0) return SGLAMD_OK;
  if (blocks > 0x7fffffff) return fail(SGLAMD_EINVAL, "gemm: grid too large");
  hipLaunchKernelGGL((gemm8_skinny_kernel<FM, FN, MODE, OT, MOE, KW, PD>), dim3((unsigned)blocks), dim3(64 * KW), 0, st,
                     g);
  return check_launch("gemm8_skinny");
}

static inline int skinny_env(const char* name) {
  const char* e = getenv(name);
  return e ? atoi(e) : 0;
}

// Picks the number of waves that split K so that enough waves are resident to keep the HBM stream
// full while every wave still has a few K blocks to walk.
template <int FM, int FN, int MODE, typename OT, bool MOE>
static int gemm8_skinny_launch_fn(const GemmArgs& g, hipStream_t st, int64_t expected_tiles_m) {
  const int R = g.rows_per_wg > 0 ? g.rows_per_wg : 16 * FN;
  const int64_t tiles = (int64_t)((g.N + R - 1) / R) * (expected_tiles_m > 0 ? expected_tiles_m : 1);
  const int nkb = (g.K + 127) >> 7;
  int kw = 1;
  constexpr int KW_MAX = (FN + FM) <= 3 ? 8 : 4;  // keeps the scratch at or below 48 KB per workgroup
  while (kw < KW_MAX && tiles * kw < 4096 && nkb / (kw * 2) >= 2) kw *= 2;
  static const int force_kw = skinny_env("SGLAMD_SKINNY_KW");
  if (force_kw) kw = force_kw < KW_MAX ? force_kw : KW_MAX;
  switch (kw) {
    case 1:
      return gemm8_skinny_launch_kw<FM, FN, MODE, OT, MOE, 1>(g, st);
    case 2:
      return gemm8_skinny_launch_kw<FM, FN, MODE, OT, MOE, 2>(g, st);
    case 4:
      return gemm8_skinny_launch_kw<FM, FN, MODE, OT, MOE, 4>(g, st);
    default:
      if constexpr (KW_MAX >= 8) return gemm8_skinny_launch_kw<FM, FN, MODE, OT, MOE, 8>(g, st);
      return gemm8_skinny_launch_kw<FM, FN, MODE, OT, MOE, 4>(g, st);
  }
}

// Two weight tiles per wave share each activation fragment (halves the L2->CU activation traffic)
// whenever N leaves enough workgroups; FN = 1 otherwise.  When the dense grid is at most two rounds of
// the CUs (256 on MI355X), the rows a workgroup owns are trimmed (in steps of 4) so that the grid is a whole number of
// rounds: N = 7168 runs as 256 workgroups of 28 rows instead of 224 of 32 with 32 CUs idle.
template <int FM, int MODE, typename OT, bool MOE>
static int gemm8_skinny_launch(const GemmArgs& g0, hipStream_t st, int64_t expected_tiles_m) {
  static const int force_fn = skinny_env("SGLAMD_SKINNY_FN");
  static const int force_rows = skinny_env("SGLAMD_SKINNY_ROWS");
  GemmArgs g = g0;
  bool two = force_fn ? force_fn == 2 : (g.N % 32 == 0 && g.N >= 2048);
  if (!MOE && !force_fn && g.N >= 1024 && (g.N + (two ? 31 : 15)) / (two ? 32 : 16) <= 2 * device_cus()) {
    // cost = rounds of one workgroup per CU x rows per workgroup; ties go to the taller tile
    const int cus = device_cus();
    int best_rows = 0, best_fn = two ? 2 : 1;
    int64_t best_cost = -1;
    for (int fn = 2; fn >= 1; fn--) {
      for (int rows = 16 * fn; rows > 16 * fn - 16 && rows >= 12; rows -= 4) {
        const int64_t grid = (g.N + rows - 1) / rows;
        if (grid > 2 * cus) continue;  // trimming only pays when rounds are few
        const int64_t cost = ((grid + cus - 1) / cus) * rows;
        if (best_cost < 0 || cost < best_cost) {
          best_cost = cost;
          best_rows = rows;
          best_fn = fn;
        }
      }
    }
    two = best_fn == 2;
    g.rows_per_wg = best_rows == 16 * best_fn ? 0 : best_rows;
  }
  if (force_rows > 0 && force_rows % 4 == 0 && force_rows <= (two ? 32 : 16)) g.rows_per_wg = force_rows;
  if (two) return gemm8_skinny_launch_fn<FM, 2, MODE, OT, MOE>(g, st, expected_tiles_m);
  return gemm8_skinny_launch_fn<FM, 1, MODE, OT, MOE>(g, st, expected_tiles_m);
}

}  // namespace sglamd
