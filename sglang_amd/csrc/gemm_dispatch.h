// Which kernel a dense 8-bit GEMM call runs, by shape: shared by the per-mode translation units (gemm_mode_*.hip,
// one explicit instantiation of dispatch_out each, so that they compile in parallel) and the entry points (gemm.hip).
#pragma once
#include <stdlib.h>

#include "gemm_big.h"
#include "gemm_big_persist.h"
#include "gemm_skinny.h"

namespace sglamd {

// Width of the large-M tile in 64-column wave tiles (4 -> 256x256, 2 -> 256x128); tuning knob.
static int big_wgn() {
  static const int v = getenv("SGLAMD_BIG_WGN") ? atoi(getenv("SGLAMD_BIG_WGN")) : 4;
  return v;
}

// Rows from which the tile kernel takes over from the streaming kernel; tuning knob.
static int tile_min_m() {
  static const int v = getenv("SGLAMD_TILE_MIN_M") ? atoi(getenv("SGLAMD_TILE_MIN_M")) : 17;
  return v;
}

// 33 to 64 rows: the tile kernel (64-row tile, K split over the chip) or the streaming kernel?  Up to 32 rows the
// streaming kernel is the faster one on every weight measured (DeepSeek-V3 gate_up / down / q_b / o_proj at 17 rows:
// 54.5 / 26.1 / 12.1 / 22.8 us against 60.0 / 31.7 / 16.9 / 28.8 in 64-row tiles; at 32 rows 63.9 / 30.4 / 13.9 / 25.6
// against 61.6 / 32.6 / 17.3 / 30.0; Llama-3-70B o / gate_up / down at 24 rows 15.0 / 86.6 / 43.2 against 19.3 / 104.5 /
// 50.6).  Its four-tile form for 33..64 rows re-reads the activations too often for large weights (gate_up at 48
// rows: 83.9 us against 63.5), but a launch of the tile kernel costs more (a second kernel when K is split) and it
// needs about a hundred workgroups to hide its per-block latency, so small weights stay with the streaming kernel.
static bool small_m_uses_tile(int64_t M, int64_t N, int64_t K) {
  if (M < tile_min_m() || M <= 32) return false;
  const int64_t tiles = (N + 255) / 256;
  const int slices = gemm8_big_slices(tiles, N, K);
  if (tiles * slices >= 96) return true;
  return (slices == 1 && tiles >= 32) || K >= 6144;
}

// The wide streaming form for 33..64 rows (tuning knob: 0 switches it off).
static bool wide_streaming() {
  static const int v = getenv("SGLAMD_WIDE") ? atoi(getenv("SGLAMD_WIDE")) : 1;
  return v != 0;
}

// Workgroups of the persistent large-tile kernel: one per CU of the current device (0: kernel switched off).
static int persist_workgroups() {
  static const int off = getenv("SGLAMD_BIG_PERSIST") ? atoi(getenv("SGLAMD_BIG_PERSIST")) == 0 : 0;
  return off ? 0 : device_cus();
}

// Which kernel the last dense GEMM call of this thread launched (SGLAMD_KERNEL_* of the header): lets a test
// assert that it exercises the kernel it was written for, whatever the launch heuristics choose.
extern thread_local int last_kernel;  // defined in gemm.hip
#define RAN(code) (last_kernel = (code))

// A launch of 256x256 tiles whose last round of one tile per CU is mostly empty is cut in two along N: the
// columns that fill whole rounds, and the rest as a launch of its own, which picks the tile height and K split that
// fill the chip with what is left.
// Returns the columns of the first part (a multiple of 256), or 0 to leave the launch whole.  Measured on the
// DeepSeek-V3 gate_up weight (N = 36864, K = 7168): M = 512 179 -> 147 us, M = 1024 303 -> 279 us, while at
// M = 2048 (four and a half rounds) the two launches cost more than the half round they save.
static int64_t column_split(int64_t M, int64_t N, int64_t K) {
  static const int off = getenv("SGLAMD_BIG_COLSPLIT") ? atoi(getenv("SGLAMD_BIG_COLSPLIT")) == 0 : 0;
  if (off || M <= 128 || (N & 255)) return 0;
  const int64_t cus = device_cus();
  const int64_t tiles_m = (M + 255) / 256, tiles_n = N / 256, tiles = tiles_m * tiles_n;
  const int64_t rounds = tiles / cus, tail = tiles % cus;
  if (rounds < 1 || rounds > 2 || tail == 0 || tail * 8 > cus * 3) return 0;
  const int64_t first = rounds * cus / tiles_m;  // column tiles that make up the whole rounds
  if (first < 1 || first >= tiles_n) return 0;
  return first * 256;
}

template <int MODE, typename OT>
static int dispatch_dense(const GemmArgs& g, hipStream_t st, void* workspace, int64_t workspace_bytes,
                          bool may_split = true) {
  RAN(SGLAMD_KERNEL_STREAMING);
  const bool big = gemm8_big_ok(g);
  const int wgs = gemm_is_block(MODE) ? persist_workgroups() : 0;
  const int nkb = g.K >> 7;
  const bool persistent = wgs > 0 && (wgs & 7) == 0 && !(nkb & 1) && nkb >= 4 && nkb <= GEMM8_PERSIST_USE_MAX_KB;
  if (big && may_split && g.M > 64) {
    const BigConfig whole = gemm8_big_config(g.M, g.N, g.K, persistent);
    const int64_t n1 = whole.bm == 256 && whole.slices == 1 ? column_split(g.M, g.N, g.K) : 0;
    if (n1 > 0) {
      typedef typename OT::storage OS;
      GemmArgs head = g, rest = g;
      head.N = (int)n1;
      rest.N = g.N - (int)n1;
      rest.B = g.B + n1 * g.ldb;
      rest.C = (OS*)g.C + n1;
      rest.sb = gemm_is_block(MODE) ? g.sb + (n1 >> 7) * g.sb_sn : g.sb + n1;
      if (g.bias) rest.bias = (const OS*)g.bias + n1;
      int rc = dispatch_dense<MODE, OT>(head, st, workspace, workspace_bytes, false);
      if (rc) return rc;
      const int ran = last_kernel;
      rc = dispatch_dense<MODE, OT>(rest, st, workspace, workspace_bytes, false);
      RAN(ran);  // the kernel that did most of the work
      return rc;
    }
  }
  if (gemm8_skinny_ok(g, g.M)) {
    if (g.M > 32 && g.M <= 64 && wide_streaming() && gemm8_skinny_wide<MODE, OT>(g, st, false) > 0) {
      RAN(SGLAMD_KERNEL_STREAMING_WIDE);
      return gemm8_skinny_wide<MODE, OT>(g, st, true);
    }
    if (g.M <= 16) return gemm8_skinny_launch<1, MODE, OT, false>(g, st, 1);
    if (g.M <= 32 && !(big && small_m_uses_tile(g.M, g.N, g.K))) return gemm8_skinny_launch<2, MODE, OT, false>(g, st, 1);
    if (g.M <= 64 && !(big && small_m_uses_tile(g.M, g.N, g.K))) return gemm8_skinny_launch<4, MODE, OT, false>(g, st, 1);
  }
  {
    if (big) {
      const BigConfig cfg = gemm8_big_config(g.M, g.N, g.K, persistent);
      const int bm = cfg.bm;
      int slices = cfg.slices;
      while (slices > 1 && (int64_t)slices * g.M * g.N * 4 > workspace_bytes) slices--;
      if (!workspace || ((uintptr_t)workspace & 15)) slices = 1;
      RAN(bm == 64 ? SGLAMD_KERNEL_TILE64 : bm == 128 ? SGLAMD_KERNEL_TILE128 : SGLAMD_KERNEL_TILE256);
      if (bm == 64) return gemm8_big_launch<MODE, OT, 4, 1>(g, st, slices, workspace);
      if (bm == 128) return gemm8_big_launch<MODE, OT, 4, 2>(g, st, slices, workspace);
      if (big_wgn() == 2) return gemm8_big_launch<MODE, OT, 2, 4>(g, st, slices, workspace);
      if constexpr (gemm_is_block(MODE)) {
        if (slices == 1 && wgs > 0 && (wgs & 7) == 0 && gemm8_big_persist_ok(g, wgs)) {
          if constexpr (MODE == GEMM_BLOCK_FP8) {
            if (g.scales_pow2) {
              RAN(SGLAMD_KERNEL_PERSISTENT256_POW2);
              return gemm8_big_persist_launch<MODE, OT, true>(g, st, wgs);
            }
          }
          RAN(SGLAMD_KERNEL_PERSISTENT256);
          return gemm8_big_persist_launch<MODE, OT>(g, st, wgs);
        }
      }
      return gemm8_big_launch<MODE, OT, 4, 4>(g, st, slices, workspace);
    }
  }
  RAN(SGLAMD_KERNEL_GENERIC);
  return gemm8_launch<128, 128, 2, 2, MODE, OT, false>(g, st);
}

template <int MODE>
int dispatch_out(const GemmArgs& g, int out_dtype, hipStream_t st, void* ws, int64_t ws_bytes) {
  if (out_dtype == SGLAMD_BF16) return dispatch_dense<MODE, BF16>(g, st, ws, ws_bytes);
  if (out_dtype == SGLAMD_F16) return dispatch_dense<MODE, F16>(g, st, ws, ws_bytes);
  return fail(SGLAMD_EINVAL, "out_dtype must be Half or BFloat16");
}

}  // namespace sglamd
