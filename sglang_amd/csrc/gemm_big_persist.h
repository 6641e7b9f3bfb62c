// Persistent form of the 256x256 large-tile block-scaled GEMM for gfx950: one workgroup per CU walks its tiles
// (virtual block ids blockIdx.x, + gridDim.x, ...) and treats their K blocks as one stream.
//
// What it removes is the tile boundary of the one-tile-per-workgroup kernel: there a finished tile drains its
// loads, stages C through the operand stages, stores it and ends; the next workgroup starts, requests its
// first two K blocks and waits for them with an idle matrix pipe (13-17 us per tile at the DeepSeek-V3
// gate_up shape, a third of the launch at K = 1536).  Here
//   * the request that runs two blocks ahead of the MFMAs simply continues into the next tile: its per-lane
//     offsets are the current ones plus a per-tile delta, so the last two K blocks of a tile already fetch
//     the first two of the next, behind the same barriers and vmcnt waits as every other block;
//   * the weight-block scales of the next tile arrive the same way (in the load slot that the waves without
//     activation-scale rows have free, with the first block of a tile, into the other of two small tables);
//   * the finished tile leaves through a wave-private 32x32 staging patch beside the stages: no workgroup
//     barrier and no wait for outstanding loads.  The next tile's first vmcnt waits still see these stores
//     (vmcnt retires loads and stores in issue order, and a wait that counts only loads is then simply
//     stricter than needed), so the stores have to complete under the tile's first steps.
// Measured (MI355X, M = 4096): against one tile per workgroup it saves 7-18 % at K = 1536..1792 and 1-2 % at
// K >= 3584, where the output's way to HBM, not the boundary's bookkeeping, is what a boundary costs.
// Same MFMA schedule, piece layout and fragment addressing as gemm8_big_kernel<MODE, OT, 4, 4>; see there for
// the reasoning behind them.
#pragma once
#include "gemm_big.h"

namespace sglamd {

constexpr int GEMM8_PERSIST_MAX_KB = 256;     // two column blocks x K blocks: the 512 table entries four waves load in two slots
constexpr int GEMM8_PERSIST_USE_MAX_KB = 256;  // K blocks up to which the launcher uses it (tunable: SGLAMD_BIG_PERSIST_KB)
constexpr int gemm8_persist_smem() {
  // A stages | B stages | activation-scale stages | 256 bytes for loads that must land nowhere |
  // two weight-scale tables of 1024 floats | eight staging patches of 32 rows x 80 bytes
  return 2 * (256 * 128) + 2 * (256 * 128) + 2 * 1024 + 256 + 2 * 4096 + 8 * 2560;
}

// E8: every scale is a power of two (UE8M0 scales expanded to fp32).  The MFMA then applies them itself: its two
// block-scale operands take the exponent byte of the weight-block scale and of each lane's activation-row scale, and
// the products of all K blocks add up in the MFMA accumulators -- no partial products, no multiply-add per
// element and K block.
// L2RES (ceiling measurement only, never launched by the operators): every tile fetches the operands, scales and
// weight-scale table of tile (0, 0) and stores to its own place, so the loop runs unchanged -- same MFMAs, folds,
// LDS traffic, direct-to-LDS loads, barriers and output stores -- on a working set of two 256-row panels that
// stays in L2.  g.A / g.B then hold 256 rows each, g.M / g.N still size the tile grid and the output.  Every
// L2RES difference sits in an `if constexpr`, so the operators' instantiations compile from the same statements
// as before (the kernel uses every register it may: a reworded expression is enough to make it spill).
template <int MODE, typename OT, bool E8 = false, bool L2RES = false>
__global__ __launch_bounds__(512) void gemm8_big_persist_kernel(GemmArgs g0) {
#if defined(__HIP_DEVICE_COMPILE__)
  static_assert(gemm_is_block(MODE), "the persistent kernel is built for the block-scaled modes");
  static_assert(!E8 || MODE == GEMM_BLOCK_FP8, "scales through the MFMA's scale operands: FP8 only");
  constexpr int WGN = 4, MT = 4, NS = 2;
  constexpr int BM = 256, BN = 256, WTM = 128;
  constexpr int APT = 1;             // A loads per wave and piece (4 per block)
  constexpr int A_STAGE = BM * 128, B_STAGE = BN * 128, S_STAGE = BM * 4;
  constexpr int B_BASE = NS * A_STAGE, S_BASE = B_BASE + NS * B_STAGE, NOWHERE = S_BASE + NS * S_STAGE;
  constexpr int TBL_BASE = NOWHERE + 256, TBL_BYTES = 4096, STG_BASE = TBL_BASE + 2 * TBL_BYTES, STG_ROW = 80;
  typedef v16f acc16_t;
  typedef typename std::conditional<gemm_is_int8(MODE), v16i, v16f>::type prod16_t;
  typedef typename OT::storage OS;
  static_assert(sizeof(OS) == 2, "2-byte outputs");

  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WGN, wn = wave % WGN;

  // the tile grid and the output follow the real sizes; with L2RES the operand side sees one 256 x 256 problem
  const int grid_m = g0.M, grid_n = g0.N;
  GemmArgs g = g0;
  if constexpr (L2RES) {
    g.M = BM;
    g.N = BN;
  }
  const int tiles_n = (grid_n + BN - 1) / BN, tiles_m = (grid_m + BM - 1) / BM;
  const int total = tiles_m * tiles_n;
  const int nkb = g.K >> 7;  // even, 4..256 (checked by the launcher)
  // virtual block id -> tile origin, the mapping of gemm8_big_kernel (XCD-contiguous ranges, groups of 8 row tiles)
  auto origin = [&](int vb, int& m0, int& n0) {
    const int pid = xcd_remap(vb, total);
    constexpr int GM = SGLAMD_BIG_GM;
    const int in_group = GM * tiles_n;
    const int group = pid / in_group;
    const int first_m = group * GM;
    const int gsz = min(tiles_m - first_m, GM);
    m0 = (first_m + (pid % in_group) % gsz) * BM;
    n0 = ((pid % in_group) / gsz) * BN;
  };
  int vb = blockIdx.x;
  int m0, n0;      // origin used for the operand addresses
  int om0, on0;    // origin of the output tile (the same unless L2RES)
  origin(vb, om0, on0);
  if constexpr (L2RES) {
    m0 = 0;
    n0 = 0;
  } else {
    m0 = om0;
    n0 = on0;
  }

  const int a_bytes = (int)min((int64_t)g.M * g.lda, (int64_t)0x7fffffff);
  const int b_bytes = (int)min((int64_t)g.N * g.ldb, (int64_t)0x7fffffff);
  const int s_bytes = (int)min((((int64_t)g.M - 1) * g.sa_sm + (int64_t)(nkb - 1) * g.sa_sk + 1) * 4, (int64_t)0x7fffffff);
  const int t_bytes =
      (int)min(((int64_t)((g.N - 1) >> 7) * g.sb_sn + (int64_t)(nkb - 1) * g.sb_sk + 1) * 4, (int64_t)0x7fffffff);

  // per-lane offsets of the current tile (see gemm8_big_kernel for the row / chunk assignment)
  uint32_t a_voff, b_voff[2], s_voff;
  {
    const int row = (wave >> 2) * WTM + (wave & 3) * 8 + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    a_voff = (uint32_t)((m0 + row) * (int)g.lda + chunk * 16);
  }
#pragma unroll
  for (int l = 0; l < 2; l++) {
    const int row = (wave * 4 + l) * 8 + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    b_voff[l] = (uint32_t)((n0 + row) * (int)g.ldb + chunk * 16);
  }
  // rows past M are not clamped: their scales are never used for a stored value
  s_voff = (uint32_t)((m0 + wave * 64 + lane) * (int)g.sa_sm) << 2;
  // weight-scale table entry e = cb * nkb + kb of a tile whose first column is n0t, 64 entries per loading wave
  // and slot; the second slot (entries 256..511) is only used beyond 128 K blocks
  auto table_voff = [&](int n0t, int slot) -> uint32_t {
    const int e = slot * 256 + (wave & 3) * 64 + lane;  // loaded by waves 4..7
    const int cb = e / nkb, kbb = e - cb * nkb;
    if (cb >= BN / 128) return 0x7ffffff0u;
    return (uint32_t)((min(n0t + cb * 128, g.N - 1) >> 7) * (int)g.sb_sn + kbb * (int)g.sb_sk) << 2;
  };

  const uint32_t smem_base = (uint32_t)(uintptr_t)(lds_ptr_t)smem;
  auto dma16 = [&](const void* base, int bytes, uint32_t voff, int soff, uint32_t lds_off) {
    const v4i rs = {(int)(uint32_t)(uintptr_t)base, (int)(((uint64_t)(uintptr_t)base >> 32) & 0xffff), bytes, 0x00020000};
    asm volatile("s_nop 4\n\tbuffer_load_dwordx4 %0, %1, %2 offen lds"
                 :
                 : "v"(voff), "s"(rs), "s"(soff), "{m0}"(smem_base + lds_off)
                 : "memory");
  };
  auto dma4 = [&](int base_lo, int base_hi, int bytes, uint32_t voff, int soff, uint32_t lds_off) {
    const v4i rs = {base_lo, base_hi, __builtin_amdgcn_readfirstlane(bytes), 0x00020000};
    asm volatile("s_nop 4\n\tbuffer_load_dword %0, %1, %2 offen lds"
                 :
                 : "v"(voff), "s"(rs), "s"(soff), "{m0}"(smem_base + lds_off)
                 : "memory");
  };

  // state of the tile after the current one: whether it exists, the offset deltas that lead to it, its table
  bool has_next = false;
  uint32_t dA = 0, dB = 0, dS = 0;
  int m0n = 0, n0n = 0;
  int om0n = 0, on0n = 0;  // L2RES: the next output tile's origin
  int tcur = 0;  // which of the two tables holds the current tile's weight scales

  // per-wave constants of the scale slot (see issue_piece)
  // (each is made a scalar register here, once: inside the loops the compiler must not have to re-derive
  // that a per-wave selection is wave-uniform)
  const int mine_i = __builtin_amdgcn_readfirstlane(wave < BM / 64 ? 1 : 0);
  const uint64_t sl_base_u = (uint64_t)(uintptr_t)(mine_i ? (const void*)g.sa : (const void*)g.sb);
  const int sl_base_lo = __builtin_amdgcn_readfirstlane((int)(uint32_t)sl_base_u);
  const int sl_base_hi = __builtin_amdgcn_readfirstlane((int)((sl_base_u >> 32) & 0xffff));
  const int sl_bytes = __builtin_amdgcn_readfirstlane(mine_i ? s_bytes : t_bytes);
  const int sl_sk4 = __builtin_amdgcn_readfirstlane(mine_i ? (int)g.sa_sk << 2 : 0);
  const int sl_dst0 = __builtin_amdgcn_readfirstlane(mine_i ? S_BASE + wave * 256 : TBL_BASE + (wave - BM / 64) * 256);
  const int sl_smul = __builtin_amdgcn_readfirstlane(mine_i ? S_STAGE : 0);
  const int sl_tmask = __builtin_amdgcn_readfirstlane(mine_i ? 0 : -1);
  uint32_t sl_voff = mine_i ? s_voff : 0x7ffffff0u;  // waves 4..7: the next tile's table offsets, set per tile
  uint32_t sl_voff2 = 0x7ffffff0u;                    // waves 4..7: the same for the second table slot
  uint32_t sl_d = 0;                                  // waves 0..3: the delta that leads to the next tile's rows

  // Piece t of block kb of the stream into a stage; kb >= nkb names block kb - nkb of the next tile.
  // Loads per wave and piece: 1 A (part 0), then 1 B and with the last piece the activation scales and the
  // table slot (part 1).
  auto issue_piece = [&](int kb, int stage, int t, int part) {
    const bool nx = kb >= nkb;
    const bool live = !nx || has_next;
    const int kk = nx ? kb - nkb : kb;
    const int koff = kk << 7;
    const int gi = wave;  // APT == 1
    if (part == 0) {
      dma16(g.A, live ? a_bytes : 0, a_voff + (nx ? dA : 0u) + (uint32_t)(t * 32 * (int)g.lda), koff,
            stage * A_STAGE + ((gi >> 2) * WTM + t * 32 + (gi & 3) * 8) * 128);
      return;
    }
    {
      const int l = t;  // B load l goes with piece l % MT == l
      dma16(g.B, live ? b_bytes : 0, b_voff[l & 1] + (nx ? dB : 0u) + (uint32_t)((l & 2) * 8 * (int)g.ldb), koff,
            B_BASE + stage * B_STAGE + (wave * 4 + l) * 1024);
    }
    if (t == MT - 1) {
      // The scale slot: waves 0..3 fetch the activation scales of 64 rows each; for waves 4..7 the slot is
      // free and, with the request for local block NS of a tile, brings the next tile's weight scales (64
      // table entries each).  Both roles run the same instructions on per-wave constants (sl_*), so that no
      // loop-invariant branch exists for the compiler to clone the loop around.
      const bool second = kb == NS + 1;
      const int on = (mine_i & (int)live) | ((mine_i ^ 1) & (int)((kb == NS || (second && nkb > 128)) && has_next));
      const uint32_t dst =
          (uint32_t)(sl_dst0 + stage * sl_smul + (((tcur ^ 1) * TBL_BYTES + (second ? 1024 : 0)) & sl_tmask));
      const uint32_t vo = mine_i ? sl_voff + (nx ? sl_d : 0u) : (second ? sl_voff2 : sl_voff);
      dma4(sl_base_lo, sl_base_hi, on ? sl_bytes : 0, vo, kk * sl_sk4, (mine_i | on) ? dst : (uint32_t)NOWHERE);
    }
  };
  auto piece_loads = [](int t) constexpr { return 2 + (t == MT - 1 ? 1 : 0); };
  constexpr int LPB = 9;

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

  // the first tile's weight scales: plain loads, table 0
  float* tbl = (float*)(smem + TBL_BASE);
  for (int idx = tid; idx < (BN / 128) * nkb; idx += 512) {
    const int cb = idx / nkb, kb = idx - cb * nkb;
    tbl[idx] = g.sb[(int64_t)(min(n0 + cb * 128, g.N - 1) >> 7) * g.sb_sn + (int64_t)kb * g.sb_sk];
  }
  const int tbl_mine = (wn >> 1) * nkb;  // this wave's column block inside a table

  auto mm_half = [&](const v8i& w, const v8i& x, prod16_t c) -> prod16_t {
    if constexpr (gemm_is_int8(MODE)) {
      const v4i wl = {w[0], w[1], w[2], w[3]}, wh = {w[4], w[5], w[6], w[7]};
      const v4i xl = {x[0], x[1], x[2], x[3]}, xh = {x[4], x[5], x[6], x[7]};
      c = __builtin_amdgcn_mfma_i32_32x32x32_i8(wl, xl, c, 0, 0, 0);
      return __builtin_amdgcn_mfma_i32_32x32x32_i8(wh, xh, c, 0, 0, 0);
    } else {
      return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(w, x, c, 0, 0, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
    }
  };

  // Prologue of the stream: the first tile's first NS blocks
#pragma unroll
  for (int st = 0; st < NS; st++)
#pragma unroll
    for (int t = 0; t < MT; t++) {
      issue_piece(st, st, t, 0);
      issue_piece(st, st, t, 1);
    }
  __builtin_amdgcn_s_waitcnt(0x0070);
  __syncthreads();
  v8i wf[2][2];
#pragma unroll
  for (int j = 0; j < 2; j++)
#pragma unroll
    for (int h = 0; h < 2; h++) wf[j][h] = wfrag(0, j, h);
  v8i x0 = xfrag(0, 0, 0), x1 = xfrag(0, 0, 1);
  float sa_cur = xscale(0, 0);
  float sb_cur = tbl[tbl_mine];
  // E8: the scales' exponent bytes, as the MFMA's scale operands want them (byte 0 of a register)
  auto exponent = [](float v) -> int { return (int)((__builtin_bit_cast(uint32_t, v) >> 23) & 0xffu); };
  int sx_cur = exponent(sa_cur), sw_cur = exponent(sb_cur);
  auto mm_e8 = [&](const v8i& w, const v8i& x, acc16_t c) -> acc16_t {
    if constexpr (E8) return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(w, x, c, 0, 0, 0, sw_cur, 0, sx_cur);
    else return c;
  };

  prod16_t qa, qb, zero16;
#pragma unroll
  for (int r = 0; r < 16; r++) qa[r] = 0, qb[r] = 0, zero16[r] = 0;
  float scp = 0.f;
  auto fold = [&](acc16_t& dst, const prod16_t& q, float sc) {
#pragma unroll
    for (int r = 0; r < 16; r++) dst[r] = fmaf((float)q[r], sc, dst[r]);
  };

  constexpr int MPH = gemm_is_int8(MODE) ? 2 : 1;
  constexpr int FOLDN = gemm_is_int8(MODE) ? 32 : 16;
  // One row tile step of one K block: the schedule of gemm8_big_kernel's block mode.
  auto tile_step = [&](int kb, auto stage_c, auto tile_c) {
    constexpr int cur = decltype(stage_c)::value, i = decltype(tile_c)::value;
    constexpr int nxt = (cur + 1) % NS;
    constexpr bool last = i == MT - 1;
    constexpr int prev = i == 0 ? MT - 1 : i - 1;
    constexpr int keep = [&]() constexpr {
      int n = 0;
      if (!last) {
        n += piece_loads(i + 1) - APT;
        for (int j = i + 2; j < MT; j++) n += piece_loads(j);
        n += (NS - 1) * LPB;
        for (int j = 0; j < i; j++) n += piece_loads(j);
      } else {
        n += (NS - 2) * LPB;
        for (int j = 0; j < MT - 1; j++) n += piece_loads(j);
      }
      return n;
    }();
    static_assert(keep < 64, "vmcnt field is 6 bits");

    if constexpr (E8) {
      // the same step without partial products: MFMAs 1-2 into acc[i][0], barrier, MFMAs 3-4 into acc[i][1] with
      // the step's loads and the next step's fragments behind them
      acc[i][0] = mm_e8(wf[0][0], x0, acc[i][0]);
      acc[i][0] = mm_e8(wf[0][1], x1, acc[i][0]);
      __builtin_amdgcn_sched_group_barrier(0x8, 2, 0);
      __builtin_amdgcn_sched_barrier(0);
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_waitcnt(0x0070 | (keep & 15) | ((keep >> 4) << 14));
      __builtin_amdgcn_s_barrier();
      asm volatile("" : "+v"(x0), "+v"(x1)::"memory");
      __builtin_amdgcn_sched_barrier(0);
      if (last) {
        wf[0][0] = wfrag(nxt, 0, 0);
        wf[0][1] = wfrag(nxt, 0, 1);
        __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
      }
      acc[i][1] = mm_e8(wf[1][0], x0, acc[i][1]);
      __builtin_amdgcn_sched_group_barrier(0x8, 1, 0);
      __builtin_amdgcn_sched_barrier(0);
      issue_piece(kb + NS, cur, i, 0);
      __builtin_amdgcn_sched_barrier(0);
      float sa_n, sb_n = sb_cur;
      if (!last) {
        x0 = xfrag(cur, i + 1, 0);
        sa_n = xscale(cur, i + 1);
        __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);
      } else {
        x0 = xfrag(nxt, 0, 0);
        sa_n = xscale(nxt, 0);
        const int slot = kb + 1 < nkb ? tcur * (TBL_BYTES / 4) + tbl_mine + kb + 1 : (tcur ^ 1) * (TBL_BYTES / 4) + tbl_mine;
        sb_n = tbl[slot];
        __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
      }
      acc[i][1] = mm_e8(wf[1][1], x1, acc[i][1]);
      __builtin_amdgcn_sched_group_barrier(0x8, 1, 0);
      __builtin_amdgcn_sched_barrier(0);
      issue_piece(kb + NS, cur, i, 1);
      __builtin_amdgcn_sched_barrier(0);
      if (!last) {
        x1 = xfrag(cur, i + 1, 1);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      } else {
        // the second column tile's fragments only now: MFMA 3 and 4 read the old ones
        x1 = xfrag(nxt, 0, 1);
        wf[1][0] = wfrag(nxt, 1, 0);
        wf[1][1] = wfrag(nxt, 1, 1);
        __builtin_amdgcn_sched_group_barrier(0x100, 6, 0);
      }
      sa_cur = sa_n;
      sb_cur = sb_n;
      sx_cur = exponent(sa_n);
      sw_cur = exponent(sb_n);
      return;
    }

    qa = mm_half(wf[0][0], x0, zero16);
    qa = mm_half(wf[0][1], x1, qa);
    __builtin_amdgcn_sched_group_barrier(0x8, 2 * MPH, 0);
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0x0070 | (keep & 15) | ((keep >> 4) << 14));
    __builtin_amdgcn_s_barrier();
    asm volatile("" : "+v"(x0), "+v"(x1)::"memory");
    __builtin_amdgcn_sched_barrier(0);
    if (last) {
      wf[0][0] = wfrag(nxt, 0, 0);
      wf[0][1] = wfrag(nxt, 0, 1);
      __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
    }
    fold(acc[prev][1], qb, scp);
    __builtin_amdgcn_sched_group_barrier(0x2, FOLDN, 0);
    qb = mm_half(wf[1][0], x0, zero16);
    __builtin_amdgcn_sched_group_barrier(0x8, MPH, 0);
    // This step's piece goes out in two parts, each right behind an MFMA.  All eight waves leave the barrier
    // together and the vector memory pipe takes 16 cycles per load, so a wave can sit at a load for a hundred
    // cycles and more; behind an MFMA that wait is covered by the matrix pipe's queue (measured: +6 % on the
    // DeepSeek-V3 gate_up shape against both loads right after the barrier).
    __builtin_amdgcn_sched_barrier(0);
    issue_piece(kb + NS, cur, i, 0);
    __builtin_amdgcn_sched_barrier(0);
    float sa_nxt, sb_nxt = sb_cur;
    if (!last) {
      x0 = xfrag(cur, i + 1, 0);
      sa_nxt = xscale(cur, i + 1);
      __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);
    } else {
      x0 = xfrag(nxt, 0, 0);
      wf[1][0] = wfrag(nxt, 1, 0);
      sa_nxt = xscale(nxt, 0);
      // the block after the tile's last one is the next tile's first: its scale sits in the other table
      const int slot = kb + 1 < nkb ? tcur * (TBL_BYTES / 4) + tbl_mine + kb + 1 : (tcur ^ 1) * (TBL_BYTES / 4) + tbl_mine;
      sb_nxt = tbl[slot];
      __builtin_amdgcn_sched_group_barrier(0x100, 6, 0);
    }
    qb = mm_half(wf[1][1], x1, qb);
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
    scp = sa_cur * sb_cur;
    sa_cur = sa_nxt;
    sb_cur = sb_nxt;
    __builtin_amdgcn_sched_group_barrier(0x2, 1, 0);
    fold(acc[i][0], qa, scp);
    __builtin_amdgcn_sched_group_barrier(0x2, FOLDN, 0);
  };
  auto k_block = [&](int kb, auto stage_c) {
    tile_step(kb, stage_c, std::integral_constant<int, 0>{});
    tile_step(kb, stage_c, std::integral_constant<int, 1>{});
    tile_step(kb, stage_c, std::integral_constant<int, 2>{});
    tile_step(kb, stage_c, std::integral_constant<int, 3>{});
  };

  uint8_t* stg = smem + STG_BASE + wave * (32 * STG_ROW);
  const int c_bytes = (int)min((int64_t)(L2RES ? grid_m : g.M) * g.ldc * 2, (int64_t)0x7fffffff);
  for (;;) {
    // the tile after this one
    const int vbn = vb + (int)gridDim.x;
    has_next = vbn < total;
    if (has_next) {
      origin(vbn, m0n, n0n);
      if constexpr (L2RES) {
        om0n = m0n;
        on0n = n0n;
        m0n = 0;
        n0n = 0;
      }
      dA = (uint32_t)((m0n - m0) * (int)g.lda);
      dB = (uint32_t)((n0n - n0) * (int)g.ldb);
      dS = (uint32_t)((m0n - m0) * (int)g.sa_sm) << 2;
      const uint32_t tv = table_voff(n0n, 0), tv2 = table_voff(n0n, 1);
      sl_d = mine_i ? dS : 0u;
      sl_voff = mine_i ? sl_voff : tv;
      sl_voff2 = tv2;
    }

    for (int kb = 0; kb < nkb; kb += NS) {
      k_block(kb, std::integral_constant<int, 0>{});
      k_block(kb + 1, std::integral_constant<int, 1>{});
    }
    if constexpr (!E8) {
      fold(acc[MT - 1][1], qb, scp);
#pragma unroll
      for (int r = 0; r < 16; r++) qb[r] = 0;
      scp = 0.f;
    }

    // Epilogue: each wave moves its 128 x 64 part out in 32 x 32 patches through its own staging rows
    // (register r of patch (i, j) is C[.. + lane%32][.. + 8*(r/4) + 4*(lane/32) + r%4]); 16-byte stores,
    // four lanes per 64-byte row segment.  Whole 128-byte segments per store (patches of 16 rows x 64 columns, the
    // 32-row form does not fit beside the operand stages) were measured on the same chip in alternation: 0.2-0.7 %
    // slower, the half-masked staging writes cost more than the fuller lines save.
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < MT; i++) {
#pragma unroll
      for (int j = 0; j < 2; j++) {
#pragma unroll
        for (int rq = 0; rq < 4; rq++) {
          const v2i w = {(int)OT::pack2(acc[i][j][rq * 4], acc[i][j][rq * 4 + 1]),
                         (int)OT::pack2(acc[i][j][rq * 4 + 2], acc[i][j][rq * 4 + 3])};
          *(v2i*)(stg + frow * STG_ROW + (8 * rq + 4 * fk) * 2) = w;
        }
#pragma unroll
        for (int half = 0; half < 2; half++) {
          const int row = (lane >> 2) + 16 * half, piece = lane & 3;
          const v4i v = *(const v4i*)(stg + row * STG_ROW + piece * 16);
          const int m = (L2RES ? om0 : m0) + wm * WTM + i * 32 + row;
          const int n = (L2RES ? on0 : n0) + wn * 64 + j * 32 + piece * 8;
          // rows past M fall outside the descriptor's range and are dropped, columns past N are sent there
          const uint32_t vo = n < (L2RES ? grid_n : g.N) ? (uint32_t)((m * (int)g.ldc + n) * 2) : 0xfffffff0u;
          const v4i rs = {(int)(uint32_t)(uintptr_t)g.C, (int)(((uint64_t)(uintptr_t)g.C >> 32) & 0xffff), c_bytes, 0x00020000};
          // A store of more than 8 bytes reads its data registers in a second pass: a VALU write to them in
          // the next two issue slots (here the next patch's conversions) would be stored instead.  The compiler
          // pads this hazard for its own stores but does not look into an asm statement.
          // Nor does it pad the five wait states a VMEM instruction needs behind a VALU write of an SGPR it reads
          // (a descriptor refilled from spilled lanes by v_readlane right in front of the store): hence the s_nop 4.
          asm volatile("s_nop 4\n\tbuffer_store_dwordx4 %0, %1, %2, 0 offen\n\ts_nop 1" : : "v"(v), "v"(vo), "s"(rs) : "memory");
        }
      }
    }
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
      for (int j = 0; j < 2; j++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][j][r] = 0;
    __builtin_amdgcn_sched_barrier(0);

    if (!has_next) break;
    vb = vbn;
    m0 = m0n;
    n0 = n0n;
    if constexpr (L2RES) {
      om0 = om0n;
      on0 = on0n;
    }
    a_voff += dA;
    b_voff[0] += dB;
    b_voff[1] += dB;
    sl_voff += sl_d;  // waves 4..7: rewritten at the top of the loop
    tcur ^= 1;
  }
  // the trailing empty-range loads still write LDS: none may be in flight when the workgroup ends
  __builtin_amdgcn_s_waitcnt(0x0F70);
#endif
}

// Shapes the persistent kernel takes: more tiles than workgroups it is launched with (else there is no
// boundary to hide), an even number of K blocks that fits the scale tables, whole aligned 16-byte output
// pieces inside a 2 GiB range.
static inline bool gemm8_big_persist_ok(const GemmArgs& g, int workgroups) {
  const int64_t tiles = (int64_t)((g.M + 255) / 256) * ((g.N + 255) / 256);
  const int nkb = g.K >> 7;
  // tuning knob: the largest number of K blocks for which the persistent kernel is used (at most 256)
  static const int env_kb = getenv("SGLAMD_BIG_PERSIST_KB") ? atoi(getenv("SGLAMD_BIG_PERSIST_KB")) : 0;
  const int max_kb = env_kb > 0 ? (env_kb < GEMM8_PERSIST_MAX_KB ? env_kb : GEMM8_PERSIST_MAX_KB) : GEMM8_PERSIST_USE_MAX_KB;
  return gemm8_big_ok(g) && tiles > workgroups && tiles < 0x7fff0000 && (nkb & 1) == 0 && nkb >= 4 &&
         nkb <= max_kb && (g.N & 7) == 0 && (g.ldc & 7) == 0 && (((uintptr_t)g.C) & 15) == 0 &&
         (int64_t)g.M * g.ldc * 2 < 0x7fffffffll;
}

template <int MODE, typename OT, bool E8 = false, bool L2RES = false>
static int gemm8_big_persist_launch(const GemmArgs& g, hipStream_t st, int workgroups) {
  auto kern = gemm8_big_persist_kernel<MODE, OT, E8, L2RES>;
  constexpr int smem = gemm8_persist_smem();
  static SmemAttrOnce attr;
  hipError_t e = raise_dynamic_smem(attr, (const void*)kern, smem);
  if (e != hipSuccess) return fail(SGLAMD_EHIP, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  hipLaunchKernelGGL(kern, dim3((unsigned)workgroups), dim3(512), smem, st, g);
  return check_launch("gemm8_big_persist");
}

}  // namespace sglamd
