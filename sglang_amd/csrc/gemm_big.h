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
// Two or three stages.  A K block is requested in pieces, one per row tile step (a burst of 64+ wave-wide
// loads would park every wave behind the CU's vector memory pipe with an idle matrix pipe), each piece
// behind a workgroup barrier that certifies its destination rows are no longer needed: row tile i's A rows
// once every wave holds that tile's fragments, the B rows from the start of the block (the block's weight
// fragments are fetched under the last row tile of the block before).  The same barrier publishes the rows
// read next, which were requested one to two blocks earlier; vmcnt waits name exactly the piece needed.
#pragma once
#include <cmath>
#include <stdlib.h>

#include <type_traits>

#include "gemm_core.h"

namespace sglamd {

typedef __attribute__((address_space(3))) void* lds_ptr_t;

// LDS stages of the operand ring: three when they fit the 160 KB of a CU (128-row tiles), else two.  A stage in
// flight is what hides the latency of the loads, and one 48..64 KB stage per CU is not enough to stream
// weights from HBM at full rate.
constexpr int GEMM8_BIG_MAX_KB = 1024;  // K blocks per launch slice the LDS weight-scale table holds (K <= 131072)
template <int WGN, int MT>
constexpr int gemm8_big_stages() {
  return 3 * ((64 * MT + 64 * WGN) * 128 + 64 * MT * 4) + 256 + (64 * WGN / 128) * GEMM8_BIG_MAX_KB * 4 <= 160 * 1024 ? 3 : 2;
}
template <int WGN, int MT>
constexpr int gemm8_big_smem() {
  // NS stages of A rows, B rows and A-row scales; 256 bytes that absorb the scale loads of idle waves; the
  // weight-block scales of the tile's column blocks for up to GEMM8_BIG_MAX_KB K blocks
  return gemm8_big_stages<WGN, MT>() * ((64 * MT + 64 * WGN) * 128 + 64 * MT * 4) + 256 +
         (64 * WGN / 128) * GEMM8_BIG_MAX_KB * 4;
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
  typedef typename std::conditional<MODE == GEMM_ROW_INT8, v16i, v16f>::type acc16_t;  // accumulators
  typedef typename std::conditional<gemm_is_int8(MODE), v16i, v16f>::type prod16_t;    // what an MFMA returns

  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  __shared__ int s_rows[MOE ? BM : 1];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WGN, wn = wave % WGN;

  const int tiles_n = (g.N + BN - 1) / BN;
  const int tiles_m = MOE ? g.max_blocks_m : (g.M + BM - 1) / BM;
  // Hardware workgroup w runs on XCD w % 8; the remap gives each XCD one contiguous range of logical tiles.  The
  // fused-MoE grid is sized for the worst padding, so there the range is that of the sorted blocks that exist.
  const int moe_tiles = MOE ? min(tiles_m, (*g.num_post_pad + BM - 1) / BM) * tiles_n : 0;
  if (MOE && (int)blockIdx.x >= moe_tiles) return;
  const int pid = xcd_remap(blockIdx.x, MOE ? moe_tiles : tiles_m * tiles_n);
  int pid_m, pid_n;
  if (MOE) {
    // consecutive tiles (the workgroups of one XCD at a time) are the column tiles of one sorted block: they share
    // its gathered rows through that XCD's L2, and the blocks of one expert follow each other, so its weights are
    // re-read while still cached
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

  // Buffer descriptor ranges end at the last valid row, so tile rows past M / N read zeros.
  const int a_bytes = (int)min(a_rows * g.lda, (int64_t)0x7fffffff);
  const int b_bytes = (int)min((int64_t)g.N * g.ldb, (int64_t)0x7fffffff);

  // LDS map: [A stages | B stages | activation-scale stages | pad | weight scales of the whole K range].  The
  // stages of an operand lie within (or just past) 64 KB of its first byte, so a fragment read is one per-lane
  // base register plus an immediate offset that names stage and tile.
  constexpr int NS = gemm8_big_stages<WGN, MT>();
  constexpr int A_STAGE = BM * 128, B_STAGE = BN * 128, S_STAGE = BM * 4;
  constexpr int B_BASE = NS * A_STAGE, S_BASE = B_BASE + NS * B_STAGE, SB_BASE = S_BASE + NS * S_STAGE + 256;

  // ---- direct-to-LDS loads, issued in pieces ---------------------------------------------------------------
  // Requesting a whole K block at once makes every wave wait behind 64+ queued wave-wide loads (the CU's
  // vector memory pipe takes 16 cycles for each) with an idle matrix pipe, so a block is requested in MT
  // pieces, one per row tile step: piece t holds the A rows of row tile t (both wave rows) and a share of the
  // B rows.  A wave issues APT A loads, 4/MT (rounded) B loads and, with the last piece, the scale load.
  constexpr int APT = A_LOADS / MT;
  static_assert(A_LOADS % MT == 0 && B_LOADS == 4, "piece layout assumes 8 A row groups per tile and 4 B loads per wave");
  constexpr bool BLK = gemm_is_block(MODE);
  // loads of piece t per wave, and of a whole block
  auto piece_loads = [](int t) constexpr { return APT + (4 / MT + ((4 % MT) > t ? 1 : 0)) + ((BLK && t == MT - 1) ? 1 : 0); };
  constexpr int LPB = A_LOADS + B_LOADS + (BLK ? 1 : 0);

  // A load (t, u) of a wave covers 8 rows of row tile t: group gi = wave*APT + u of the tile's 8 groups, i.e.
  // wave row gi/4, rows 8*(gi%4).. inside the tile.  The swizzle key of such a row depends on gi and the lane
  // only, so one per-lane offset per u serves every t (MOE gathers its rows: one offset per load).
  uint32_t a_voff[MOE ? A_LOADS : APT], b_voff[2];
#pragma unroll
  for (int u = 0; u < APT; u++) {
    const int gi = wave * APT + u;
#pragma unroll
    for (int t = 0; t < (MOE ? MT : 1); t++) {
      const int row = (gi >> 2) * WTM + t * 32 + (gi & 3) * 8 + (lane >> 3);
      const int chunk = (lane & 7) ^ ((row >> 1) & 7);
      if (MOE) {
        const int tok = s_rows[row];  // padding slots (>= num_valid) land past the descriptor's range: zeros
        a_voff[t * APT + u] = tok < g.num_valid ? (uint32_t)((tok / g.top_k) * (int)g.lda + chunk * 16) : 0x7ffffff0u;
      } else {
        a_voff[u] = (uint32_t)((m0 + row) * (int)g.lda + chunk * 16);
      }
    }
  }
  // B load l of a wave covers rows (wave*4 + l)*8..; the key depends on the parity of l and the lane
#pragma unroll
  for (int l = 0; l < 2; l++) {
    const int row = (wave * 4 + l) * 8 + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    b_voff[l] = (uint32_t)((n0 + row) * (int)g.ldb + chunk * 16);
  }
  // activation scales of the tile rows: waves 0..BM/64-1 fetch 64 rows each (block mode)
  int srow;
  if (MOE) {
    const int tok = s_rows[min(wave * 64 + lane, BM - 1)];
    srow = tok < g.num_valid ? tok / g.top_k : 0;
  } else {
    srow = min(m0 + wave * 64 + lane, (int)g.M - 1);
  }
  const uint32_t s_voff = (uint32_t)(srow * (int)g.sa_sm) << 2;
  const int s_bytes =
      BLK ? (int)min(((a_rows - 1) * g.sa_sm + (int64_t)((g.K >> 7) - 1) * g.sa_sk + 1) * 4, (int64_t)0x7fffffff) : 0;

  // K blocks of this split-K slice
  const int nkb_all = g.K >> 7;
  const int kb_begin = (int)((int64_t)nkb_all * blockIdx.y / gridDim.y);
  const int kb_end = (int)((int64_t)nkb_all * (blockIdx.y + 1) / gridDim.y);
  const int nkb = kb_end - kb_begin;

  // The loads are written as assembly so that the compiler's own wait-count bookkeeping does not know them:
  // it treats a direct-to-LDS load as a store every later LDS read might alias and would wait for all of them
  // in front of each fragment read.  Every wait for these loads is an explicit s_waitcnt vmcnt below; the K
  // loop contains no other vector memory instruction.  Buffer descriptor: base, 0 stride, byte range, raw
  // 32-bit format; an empty range (block past the end of K) makes the load write zeros without fetching.
  const uint32_t smem_base = (uint32_t)(uintptr_t)(lds_ptr_t)smem;
  auto dma16 = [&](const void* base, int bytes, uint32_t voff, int soff, uint32_t lds_off) {
    const v4i rs = {(int)(uint32_t)(uintptr_t)base, (int)(((uint64_t)(uintptr_t)base >> 32) & 0xffff), bytes, 0x00020000};
    asm volatile("s_nop 4\n\tbuffer_load_dwordx4 %0, %1, %2 offen lds"
                 :
                 : "v"(voff), "s"(rs), "s"(soff), "{m0}"(smem_base + lds_off)
                 : "memory");
  };
  auto dma4 = [&](const void* base, int bytes, uint32_t voff, int soff, uint32_t lds_off) {
    const v4i rs = {(int)(uint32_t)(uintptr_t)base, (int)(((uint64_t)(uintptr_t)base >> 32) & 0xffff), bytes, 0x00020000};
    asm volatile("s_nop 4\n\tbuffer_load_dword %0, %1, %2 offen lds"
                 :
                 : "v"(voff), "s"(rs), "s"(soff), "{m0}"(smem_base + lds_off)
                 : "memory");
  };
  // piece t of K block kb of this slice into a stage; the scalar offset operand is not range-checked, so it
  // only carries the K offset (which stays inside a row); everything that selects the row is per lane
  // (part 0: the A loads; part 1: the B loads and the activation scales -- always issued in this order)
  auto issue_piece = [&](int kb, int stage, int t, int part) {
    const bool live = kb < nkb;
    const int koff = (kb_begin + kb) << 7;
    if (part == 0) {
#pragma unroll
      for (int u = 0; u < APT; u++) {
        const int gi = wave * APT + u;
        const uint32_t vo = MOE ? a_voff[t * APT + u] : a_voff[u] + (uint32_t)(t * 32 * (int)g.lda);
        dma16(g.A, live ? a_bytes : 0, vo, koff, stage * A_STAGE + ((gi >> 2) * WTM + t * 32 + (gi & 3) * 8) * 128);
      }
      return;
    }
#pragma unroll
    for (int l = 0; l < 4; l++) {
      if (l % MT != t) continue;
      dma16(Bmat, live ? b_bytes : 0, b_voff[l & 1] + (uint32_t)((l & 2) * 8 * (int)g.ldb), koff,
            B_BASE + stage * B_STAGE + (wave * 4 + l) * 1024);
    }
    if (BLK && t == MT - 1) {
      // waves past the last 64-row group take part with an empty range and a scratch destination, so every
      // wave issues the same number of loads
      const bool mine = wave < BM / 64;
      dma4(g.sa, (live && mine) ? s_bytes : 0, s_voff, ((kb_begin + kb) * (int)g.sa_sk) << 2,
           mine ? S_BASE + stage * S_STAGE + wave * 256 : S_BASE + NS * S_STAGE);
    }
  };

  // Fragment of a 32x32x64 MFMA operand: lane -> row lane%32, 32 bytes at 64*h + 32*(lane/32), i.e. the
  // 16-byte chunks 4h + 2*(lane/32) and the one after it, each at its swizzled position.  All fragment rows
  // of a wave are row0 + 32*t + lane%32 with row0 a multiple of 32, so the key is a function of the lane.
  const int frow = lane & 31, fk = lane >> 5;
  const int fsw = (frow >> 1) & 7;
  const uint8_t* xb[2][2];
  const uint8_t* wb[2][2];
#pragma unroll
  for (int h = 0; h < 2; h++)
#pragma unroll
    for (int c = 0; c < 2; c++) {
      const int off = (((h * 4 + fk * 2 + c) ^ fsw) << 4) + frow * 128;
      xb[h][c] = smem + wm * WTM * 128 + off;
      wb[h][c] = smem + B_BASE + wn * 64 * 128 + off;
    }
  const float* sa_lds = (const float*)(smem + S_BASE) + wm * WTM + frow;
  // x fragment of row tile t, w fragment of column tile j, both of K half h in the given stage
  auto xfrag = [&](int stage, int t, int h) -> v8i {
    const v4i lo = *(const v4i*)(xb[h][0] + stage * A_STAGE + t * 4096);
    const v4i hi = *(const v4i*)(xb[h][1] + stage * A_STAGE + t * 4096);
    return v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  };
  auto wfrag = [&](int stage, int j, int h) -> v8i {
    const v4i lo = *(const v4i*)(wb[h][0] + stage * B_STAGE + j * 4096);
    const v4i hi = *(const v4i*)(wb[h][1] + stage * B_STAGE + j * 4096);
    return v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  };
  auto xscale = [&](int stage, int t) -> float { return sa_lds[stage * BM + t * 32]; };

  acc16_t acc[MT][2];
#pragma unroll
  for (int i = 0; i < MT; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0;

  // Weight-block scales of this tile for the whole K range go to LDS once ([column block][K block]), so that
  // the K loop has no memory instruction besides the direct-to-LDS loads and LDS reads.
  float* sb_lds_all = (float*)(smem + SB_BASE);
  if (BLK) {
    const float* sb_tile = g.sb + (MOE ? (int64_t)max(expert, 0) * g.sb_se : 0);
    for (int idx = tid; idx < (BN / 128) * nkb; idx += 128 * WGN) {
      const int cb = idx / nkb, kb = idx - cb * nkb;
      sb_lds_all[cb * GEMM8_BIG_MAX_KB + kb] =
          sb_tile[(int64_t)(min(n0 + cb * 128, g.N - 1) >> 7) * g.sb_sn + (int64_t)(kb_begin + kb) * g.sb_sk];
    }
  }
  const float* sb_mine = sb_lds_all + ((wn * 64) >> 7) * GEMM8_BIG_MAX_KB;

  // MFMA of one 32x32 output tile over one 64-wide half of the K block
  auto mm_half = [&](const v8i& w, const v8i& x, prod16_t c) -> prod16_t {
    if constexpr (gemm_is_int8(MODE)) {
      // v_mfma_i32_32x32x32_i8 takes 16 bytes per lane; the 32 bytes a lane holds per 64-byte half are two
      // such slices, and pairing low with low / high with high on both operands covers every k exactly once
      const v4i wl = {w[0], w[1], w[2], w[3]}, wh = {w[4], w[5], w[6], w[7]};
      const v4i xl = {x[0], x[1], x[2], x[3]}, xh = {x[4], x[5], x[6], x[7]};
      c = __builtin_amdgcn_mfma_i32_32x32x32_i8(wl, xl, c, 0, 0, 0);
      return __builtin_amdgcn_mfma_i32_32x32x32_i8(wh, xh, c, 0, 0, 0);
    } else {
      return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(w, x, c, 0, 0, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
    }
  };

  // Prologue: the first NS K blocks requested; block 0's weight fragments, the first row tile's activation
  // fragments and the scales in registers.
#pragma unroll
  for (int st = 0; st < NS; st++)
#pragma unroll
    for (int t = 0; t < MT; t++) issue_piece(st, st, t, 0), issue_piece(st, st, t, 1);
  __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
  __syncthreads();
  v8i wf[2][2];  // [column tile j][K half h]
#pragma unroll
  for (int j = 0; j < 2; j++)
#pragma unroll
    for (int h = 0; h < 2; h++) wf[j][h] = wfrag(0, j, h);
  v8i x0 = xfrag(0, 0, 0), x1 = xfrag(0, 0, 1);
  float sa_cur = BLK ? xscale(0, 0) : 1.f;
  float sb_cur = BLK ? sb_mine[0] : 1.f;

  // Schedule of one row tile (block mode), all of it issued by one wave in this order:
  //   M1: qa  = W[0][h0] x X[h0]      M2: qa += W[0][h1] x X[h1]
  //   wait for the pieces read next, workgroup barrier, request this tile step's piece of block kb+NS
  //   16 v_fma  acc[previous tile][1] += qb * scale_prev
  //   M3: qb  = W[1][h0] x X[h0]      request X[h0] of the next tile
  //   M4: qb += W[1][h1] x X[h1]      request X[h1] of the next tile
  //   16 v_fma  acc[this tile][0] += qa * scale
  // Each group of v_fma folds a product whose last MFMA was issued 18 instructions earlier, which is the
  // distance the hardware needs between an MFMA and a VALU read of its result, so no wait states are
  // padded in, and the v_fma issue while the MFMA pair in front of them occupies the matrix pipe.  Every
  // fragment register is reloaded right after its last reader has issued, which keeps a single copy of
  // the activation fragments.  qb and scp carry the last tile's second product across K blocks (zero
  // before the first: acc += 0 * 0).
  //
  // The barrier of tile step i (after M1, M2): by then every wave holds row tile i's activation fragments
  // and, since the end of the previous block, the block's weight fragments, so row tile i's A rows and the
  // whole B stage can take block kb+NS; and the rows read next (row tile i+1, or block kb+1's first
  // fragments at the last step) are known to have landed: own loads by the vmcnt wait, everybody's by the
  // barrier.  vmcnt counts a wave's loads in issue order, so "piece P has landed" is "at most as many loads
  // outstanding as were issued after P".
  prod16_t qa, qb, zero16;
#pragma unroll
  for (int r = 0; r < 16; r++) qa[r] = 0, qb[r] = 0, zero16[r] = 0;
  float scp = 0.f;
  auto fold = [&](acc16_t& dst, const prod16_t& q, float sc) {
    if constexpr (BLK) {
#pragma unroll
      for (int r = 0; r < 16; r++) dst[r] = fmaf((float)q[r], sc, dst[r]);
    }
  };

  // One tile step of one K block; stage and tile are compile-time constants (the K loop is unrolled NS times).
  constexpr int MPH = gemm_is_int8(MODE) ? 2 : 1;  // MFMA instructions per mm_half
  constexpr int FOLDN = gemm_is_int8(MODE) ? 32 : 16;  // VALU instructions of one fold (int32 products convert first)
  auto tile_step = [&](int kb, auto stage_c, auto tile_c) {
    constexpr int cur = decltype(stage_c)::value, i = decltype(tile_c)::value;
    constexpr int nxt = (cur + 1) % NS;
    constexpr bool last = i == MT - 1;
    constexpr int prev = i == 0 ? MT - 1 : i - 1;
    // loads issued after the piece that has to be complete at this step's barrier
    constexpr int keep = [&]() constexpr {
      int n = 0;
      if (!last) {
        // A rows of row tile i+1 of this block: requested NS blocks ago with piece i+1, A loads first
        n += piece_loads(i + 1) - APT;
        for (int j = i + 2; j < MT; j++) n += piece_loads(j);
        n += (NS - 1) * LPB;
        for (int j = 0; j < i; j++) n += piece_loads(j);
      } else {
        // all of block kb+1: requested NS-1 blocks ago
        n += (NS - 2) * LPB;
        for (int j = 0; j < MT - 1; j++) n += piece_loads(j);
      }
      return n;
    }();
    static_assert(keep < 64, "vmcnt field is 6 bits");

    if constexpr (BLK) {
      qa = mm_half(wf[0][0], x0, zero16);
      qa = mm_half(wf[0][1], x1, qa);
    } else {
      acc[i][0] = mm_half(wf[0][0], x0, acc[i][0]);
      acc[i][0] = mm_half(wf[0][1], x1, acc[i][0]);
    }
    __builtin_amdgcn_sched_group_barrier(0x8, 2 * MPH, 0);
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0x0070 | (keep & 15) | ((keep >> 4) << 14));  // vmcnt(keep) lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    // the fragments pass through empty volatile statements: the MFMAs that read them stay behind the barrier
    asm volatile("" : "+v"(x0), "+v"(x1)::"memory");
    __builtin_amdgcn_sched_barrier(0);
    if (last) {
      wf[0][0] = wfrag(nxt, 0, 0);
      wf[0][1] = wfrag(nxt, 0, 1);
      __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
    }
    if constexpr (BLK) {
      fold(acc[prev][1], qb, scp);
      __builtin_amdgcn_sched_group_barrier(0x2, FOLDN, 0);
      qb = mm_half(wf[1][0], x0, zero16);
    } else {
      acc[i][1] = mm_half(wf[1][0], x0, acc[i][1]);
    }
    __builtin_amdgcn_sched_group_barrier(0x8, MPH, 0);
    // This step's piece goes out in two parts, each right behind an MFMA: all waves leave the barrier together
    // and the vector memory pipe takes 16 cycles per load, so a wave can wait at a load for a hundred cycles
    // and more; behind an MFMA the matrix pipe's queue covers that wait.
    __builtin_amdgcn_sched_barrier(0);
    issue_piece(kb + NS, cur, i, 0);
    __builtin_amdgcn_sched_barrier(0);
    float sa_nxt = 1.f, sb_nxt = sb_cur;
    if (!last) {
      x0 = xfrag(cur, i + 1, 0);
      if (BLK) sa_nxt = xscale(cur, i + 1);
      __builtin_amdgcn_sched_group_barrier(0x100, BLK ? 3 : 2, 0);
    } else {
      x0 = xfrag(nxt, 0, 0);
      wf[1][0] = wfrag(nxt, 1, 0);
      if (BLK) {
        sa_nxt = xscale(nxt, 0);
        sb_nxt = sb_mine[min(kb + 1, nkb - 1)];
      }
      __builtin_amdgcn_sched_group_barrier(0x100, BLK ? 6 : 4, 0);
    }
    if constexpr (BLK) qb = mm_half(wf[1][1], x1, qb);
    else acc[i][1] = mm_half(wf[1][1], x1, acc[i][1]);
    __builtin_amdgcn_sched_group_barrier(0x8, MPH, 0);
    __builtin_amdgcn_sched_barrier(0);
    issue_piece(kb + NS, cur, i, 1);
    __builtin_amdgcn_sched_barrier(0);
    if (!last) {
      x1 = xfrag(cur, i + 1, 1);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    } else {
      x1 = xfrag(nxt, 0, 1);
      wf[1][1] = wfrag(nxt, 1, 1);
      __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
    }
    if constexpr (BLK) {
      scp = sa_cur * sb_cur;
      sa_cur = sa_nxt;
      sb_cur = sb_nxt;
      __builtin_amdgcn_sched_group_barrier(0x2, 1, 0);
      fold(acc[i][0], qa, scp);
      __builtin_amdgcn_sched_group_barrier(0x2, FOLDN, 0);
    }
  };
  auto k_block = [&](int kb, auto stage_c) {
    tile_step(kb, stage_c, std::integral_constant<int, 0>{});
    if constexpr (MT > 1) tile_step(kb, stage_c, std::integral_constant<int, 1>{});
    if constexpr (MT > 2) tile_step(kb, stage_c, std::integral_constant<int, 2>{});
    if constexpr (MT > 3) tile_step(kb, stage_c, std::integral_constant<int, 3>{});
  };
  for (int kb = 0; kb < nkb; kb += NS) {
    k_block(kb, std::integral_constant<int, 0>{});
    if (kb + 1 < nkb) {
      k_block(kb + 1, std::integral_constant<int, 1>{});
      if constexpr (NS > 2) {
        if (kb + 2 < nkb) k_block(kb + 2, std::integral_constant<int, 2>{});
      }
    }
  }
  if constexpr (BLK) fold(acc[MT - 1][1], qb, scp);

  // Epilogue.  Register r of tile (i, j) is C[m = .. + lane%32][n = .. + 8*(r/4) + 4*(lane/32) + r%4].
  typedef typename OT::storage OS;
  static_assert(sizeof(OS) == 2, "the staged epilogue packs 2-byte outputs");
  // the trailing (empty-range) loads still write LDS: none may be in flight when the stages are reused below
  // or when the workgroup ends
  __builtin_amdgcn_s_waitcnt(0x0F70);
  if (gridDim.y > 1) {
    // split-K: fp32 partial sums (int8: the int32 sums bit-stored in the same 4-byte slots) to this slice's slab
    float* slab = (float*)g.C + (int64_t)blockIdx.y * g.M * g.N;
#pragma unroll
    for (int i = 0; i < MT; i++) {
      const int m = m0 + wm * WTM + i * 32 + frow;
      if (m >= g.M) continue;
#pragma unroll
      for (int j = 0; j < 2; j++) {
#pragma unroll
        for (int rq = 0; rq < 4; rq++) {
          const int n = n0 + wn * 64 + j * 32 + 8 * rq + 4 * fk;
          if (n >= g.N) continue;
          float v[4];
#pragma unroll
          for (int r = 0; r < 4; r++) {
            if constexpr (MODE == GEMM_ROW_INT8) v[r] = __int_as_float(acc[i][j][rq * 4 + r]);
            else v[r] = acc[i][j][rq * 4 + r];
          }
          float* prow = slab + (int64_t)m * g.N + n;
          if (n + 3 < g.N && ((((uintptr_t)prow) & 15) == 0)) {
            *(v4f*)prow = v4f{v[0], v[1], v[2], v[3]};
          } else {
            for (int r = 0; r < 4 && n + r < g.N; r++) prow[r] = v[r];
          }
        }
      }
    }
    return;
  }
  // The finished tile goes through LDS so that global stores are whole 16-byte pieces of consecutive row
  // bytes (a lane's accumulators are 4 consecutive columns of 16 different rows).  Rows are padded by 8 bytes:
  // the 32 rows a wave writes at once then fall into distinct banks.
  constexpr int CROW = BN * 2 + 8;
  static_assert(BM * CROW <= gemm8_big_smem<WGN, MT>(), "output tile must fit the operand stages");
  __syncthreads();
  // row modes: the weight-row scales (and bias) of this lane's 32 columns, fetched once for all row tiles
  float sbn[2][4][4], bia[2][4][4];
  if constexpr (!gemm_is_block(MODE)) {
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int rq = 0; rq < 4; rq++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const int nn = min(n0 + wn * 64 + j * 32 + 8 * rq + 4 * fk + r, (int)g.N - 1);
          sbn[j][rq][r] = g.sb[nn];
          bia[j][rq][r] = g.bias ? OT::to_f32(((const OS*)g.bias)[nn]) : 0.f;
        }
  }
#pragma unroll
  for (int i = 0; i < MT; i++) {
    const int rl = wm * WTM + i * 32 + frow;
    int m = m0 + rl;
    float wgt = 1.f;
    if (MOE) {
      m = s_rows[rl];
      if (g.mul_weight) wgt = g.topk_w[min(m, g.num_valid - 1)];
      if (expert < 0) wgt = 0.f;
      m = min(m, g.num_valid - 1);
    } else {
      m = min(m, (int)g.M - 1);
    }
    float sam = 1.f;
    if (!gemm_is_block(MODE)) sam = g.sa[m];
#pragma unroll
    for (int j = 0; j < 2; j++) {
#pragma unroll
      for (int rq = 0; rq < 4; rq++) {
        const int cl = wn * 64 + j * 32 + 8 * rq + 4 * fk;
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; r++) v[r] = (float)acc[i][j][rq * 4 + r] * wgt;
        if constexpr (!gemm_is_block(MODE)) {
#pragma unroll
          for (int r = 0; r < 4; r++) {
            if constexpr (MODE == GEMM_ROW_FP8) v[r] = v[r] * sbn[j][rq][r] * sam;
            else v[r] = v[r] * (sbn[j][rq][r] * sam);
            if (g.bias) v[r] += bia[j][rq][r];
          }
        }
        const v2i w = {(int)OT::pack2(v[0], v[1]), (int)OT::pack2(v[2], v[3])};
        *(v2i*)(smem + rl * CROW + cl * 2) = w;
      }
    }
  }
  __syncthreads();
  constexpr int LPR = BN / 8;         // lanes per tile row, 8 outputs (16 bytes) each
  constexpr int RPI = 64 / LPR;       // rows per wave-wide store
  const int cl = (lane % LPR) * 8;
  const int n = n0 + cl;
#pragma unroll 4
  for (int rl = wave * RPI + lane / LPR; rl < BM; rl += NW * RPI) {
    int m = m0 + rl;
    if (MOE) {
      m = s_rows[rl];
      if (m >= g.num_valid) continue;
    } else if (m >= g.M) {
      continue;
    }
    if (n >= g.N) continue;
    const uint8_t* src = smem + rl * CROW + cl * 2;
    const v2i lo = *(const v2i*)src, hi = *(const v2i*)(src + 8);
    OS* dst = (OS*)g.C + (int64_t)m * g.ldc + n;
    if (n + 8 <= g.N && ((((uintptr_t)dst) & 15) == 0)) {
      *(v4i*)dst = v4i{lo[0], lo[1], hi[0], hi[1]};
    } else {
      OS o[8];
      __builtin_memcpy(o, &lo, 8);
      __builtin_memcpy(o + 4, &hi, 8);
      for (int r = 0; r < 8 && n + r < g.N; r++) dst[r] = o[r];
    }
  }
#endif
}

// Preconditions beyond the generic kernel's: K % 128 == 0 and both operands smaller than 2 GiB
// (buffer descriptors carry 32-bit ranges and offsets).
static inline bool gemm8_big_ok(const GemmArgs& g) {
  return (g.K % 128) == 0 && (g.K >> 7) <= GEMM8_BIG_MAX_KB && (int64_t)g.M * g.lda < 0x7fffffffll &&
         (int64_t)g.N * g.ldb < 0x7fffffffll;
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
    if (!gemm_is_block(MODE)) {
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

// Tile height (64, 128 or 256 rows) and number of K slices for the large-M kernel.  One workgroup occupies a
// CU, so the cost of a launch is (rounds of one workgroup per CU) x (work per workgroup); the 128-row tile does
// half the work per workgroup at a somewhat lower MFMA efficiency and is preferred when it removes a mostly
// empty last round.  K is split when the tile grid alone cannot fill the chip (every slice keeps >= 8 blocks).
struct BigConfig {
  int bm, slices;
};
static inline int gemm8_big_slices(int64_t tiles, int64_t N, int64_t K) {
  const int64_t nkb = K >> 7;
  const int cus = device_cus();
  if (tiles >= cus * 5 / 8 || (N & 3)) return 1;
  int64_t s = cus / tiles;
  if (s > nkb / 8) s = nkb / 8;
  if (s > 16) s = 16;
  return s < 1 ? 1 : (int)s;
}
static inline BigConfig gemm8_big_config(int64_t M, int64_t N, int64_t K, bool persistent_256 = false) {
  // tuning knob: force the tile height (64, 128 or 256)
  static const int forced = getenv("SGLAMD_BIG_BM") ? atoi(getenv("SGLAMD_BIG_BM")) : 0;
  if (forced == 64 || forced == 128 || forced == 256)
    return {forced, gemm8_big_slices(((M + forced - 1) / forced) * ((N + 255) / 256), N, K)};
  if (M <= 64) {
    // one row of 64-row tiles: K is split until the grid fills the chip
    return {64, gemm8_big_slices((N + 255) / 256, N, K)};
  }
  // Cost of a launch in "tile rows over the whole K": rounds of one workgroup per CU x rows per tile / K slices,
  // weighted by what a row costs in that tile (the smaller tiles re-read more of the weights per row and fill
  // the matrix pipe less well; a 256-row launch with more tiles than CUs runs the persistent kernel when the
  // caller says so, which hides its tile boundaries), plus for split K the fp32 slabs' trip through HBM
  // (8 bytes per element and slice at ~4 TB/s against ~7.7 ns per tile row and K block).  Fitted to a sweep
  // of M = 65..2048 on the DeepSeek-V3 gate_up, down and q_b weights: within 5 % of the best height there.
  BigConfig best = {256, 1};
  double best_cost = 1e30;
  const int cus = device_cus();
  const double nkb = (double)(K >> 7);
  for (int bm = 64; bm <= 256; bm *= 2) {
    if (bm == 256 && M <= 128) break;
    const int64_t tiles = ((M + bm - 1) / bm) * ((N + 255) / 256);
    const int slices = gemm8_big_slices(tiles, N, K);
    const int64_t rounds = (tiles * slices + cus - 1) / cus;
    const double weight = bm == 64 ? 1.6 : bm == 128 ? 1.2 : (persistent_256 && tiles > cus) ? 0.88 : 1.0;
    // a single row of tiles only loads the rows that exist: M = 192 in 256-row tiles costs what 192 rows cost
    // (gate_up at M = 192: 89.6 us in 256-row tiles against 102.5 in 64-row tiles, which need two rounds)
    const double rows = M <= bm ? (double)((M + 63) / 64 * 64) : (double)bm;
    double cost = (double)rounds * rows / slices * weight;
    // one partly filled round without split K: the workgroups that do run share the fabric among fewer, so a
    // tile takes less than in a full round (fitted with the rest: cost ~ sqrt of the fill, at most a quarter off;
    // Llama-3-70B qkv at M = 512: 160 tiles of 128 rows take 47.8 us, 80 tiles of 256 rows split 3 ways 62.5)
    if (slices == 1 && rounds == 1 && tiles < cus) {
      const double fill = std::sqrt((double)tiles / cus);
      cost *= fill > 0.75 ? fill : 0.75;
    }
    if (slices > 1) cost += 4.0 + (double)slices * M * N * 8.0 / 4000.0 / (nkb * 7.7);
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
  static SmemAttrOnce attr;
  hipError_t e = raise_dynamic_smem(attr, (const void*)kern, smem);
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

// Fused-MoE launch of the same kernel: sorted blocks of 64*MT slots (128 or 192), no split-K.
template <int MODE, typename OT, int MT = 2>
static int gemm8_big_moe_launch(const GemmArgs& g, hipStream_t st) {
  auto kern = gemm8_big_kernel<MODE, OT, 4, MT, true>;
  constexpr int smem = gemm8_big_smem<4, MT>();
  static SmemAttrOnce attr;
  hipError_t e = raise_dynamic_smem(attr, (const void*)kern, smem);
  if (e != hipSuccess) return fail(SGLAMD_EHIP, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  const int64_t blocks = (int64_t)((g.N + 255) / 256) * g.max_blocks_m;
  if (blocks <= 0) return SGLAMD_OK;
  if (blocks > 0x7fffffff) return fail(SGLAMD_EINVAL, "gemm: grid too large");
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks, 1), dim3(512), smem, st, g);
  return check_launch("gemm8_big(moe)");
}

}  // namespace sglamd
