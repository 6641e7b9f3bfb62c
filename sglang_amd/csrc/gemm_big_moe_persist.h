// Persistent form of the fused-MoE tile kernel (gemm8_big_kernel<.., MOE>) for gfx950: one workgroup per CU walks
// the (sorted block, column tile) pairs, one per round of gridDim.x consecutive pairs.
//
// What it removes is most of a tile's fixed cost.  With one tile per workgroup every tile pays, with an idle
// matrix pipe: the dispatch of its workgroup, the read of its sorted ids, the divisions that turn them into row
// offsets, the plain loads of its weight-block scales, the first two K blocks' flight from HBM, and at the end the
// trip of the finished tile through LDS and out.  Measured on the DeepSeek-V3 layer (192-row blocks, 256 experts):
// time per round of tiles against K is a line with an intercept of 7-9 us, which is 24 % of a tile of the second
// GEMM (K = 2048) and 8 % of one of the first (K = 7168).  Here
//   * the next tile's sorted ids are read one tile ahead (into registers, then into the other of two small LDS
//     arrays), its routing weights likewise;
//   * when a tile's K loop ends, the next tile's row offsets are computed from those ids and its first two K
//     blocks and its weight-block scale table (direct-to-LDS loads, into the other of two tables) are requested
//     BEFORE the finished tile is converted and stored, so they fly under the epilogue;
//   * the finished tile leaves through wave-private 32x64 staging patches beside the stages (no workgroup barrier,
//     no use of the stages), with 16-byte stores written as assembly so that the compiler puts no wait for the
//     loads in flight in front of them.
// The K loop itself -- MFMA schedule, piece layout, fragment addressing, vmcnt waits -- is gemm8_big_kernel's with
// two stages; see there for the reasoning.  Block-scaled modes only, no split K.
// Measured (DeepSeek-V3 layer, uniform routing; one tile per workgroup -> this kernel, with the first GEMM's fused
// activation epilogue): 3072 tokens 2.61 -> 2.59 ms, 4096 2.84 -> 2.68, 5120 3.17 -> 2.96, 6144 3.99 -> 3.87,
// 7168 4.74 -> 4.58, 8192 4.77 -> 4.62, 10240 5.22 -> 5.01, 12288 6.67 -> 6.26 ms; skewed routings -3 ... -8 %.
// Whole 128-byte row segments per store instead of 64-byte halves are about 1 % of that.  A second form that also continued the request stream across the tile boundary (the last two K
// blocks of a tile fetching the first two of the next from that tile's gathered rows, every id, weight, expert id
// and scale table arriving by direct-to-LDS loads two tiles ahead, no drain between tiles) measured the same at
// K >= 2048 (grouped GEMM at K = 1024: 521 against 549 us) at 255 registers and is not kept: what a tile still costs
// beyond its K blocks (4-5 us) is the trip of its 96 KB of output, whose stores sit in front of the next tile's
// loads in the in-order vmcnt queue.
#pragma once
#include "gemm_big.h"
#include "quant_core.h"

namespace sglamd {

constexpr int GEMM8_MOE_PERSIST_MAX_KB = 256;  // 2 column blocks x K blocks: 512 table entries, one load per wave
template <int MT>
constexpr int gemm8_moe_persist_smem() {
  // two stages of A rows, B rows and A-row scales | 256 bytes for loads that must land nowhere |
  // two weight-scale tables of 512 floats | eight staging patches of 32 rows x 144 bytes
  return 2 * ((64 * MT + 256) * 128 + 64 * MT * 4) + 256 + 2 * 2048 + 8 * 4608;
}

// ACTQ (first GEMM of a gated SiLU layer, FP8): the tile pairs 128 gate rows of the weight with their 128 up rows
// -- a wave's two 32-column tiles are gate columns c .. c + 31 and up columns c .. c + 31, so both halves of an
// output sit in one lane -- and the epilogue writes what the unfused sequence's next launch would: silu(gate) * up
// rounded as silu_and_mul rounds it, group-quantised to e4m3 (one 128-wide group per row and tile, its maximum
// exchanged between the four waves that share the rows) into g.C ([pairs, N / 2] bytes, g.ldc bytes per row) and
// the group scales into g.A16 ([pairs, N / 256] floats).  The 16-bit [gate | up] rows never exist.
template <int MODE, typename OT, int MT, bool ACTQ = false>
__global__ __launch_bounds__(512) void gemm8_moe_persist_kernel(GemmArgs g) {
#if defined(__HIP_DEVICE_COMPILE__)
  static_assert(gemm_is_block(MODE), "the persistent MoE kernel is built for the block-scaled modes");
  static_assert(!ACTQ || MODE == GEMM_BLOCK_FP8, "the fused activation writes e4m3");
  constexpr int WGN = 4, NS = 2, NW = 8;
  constexpr int BM = 64 * MT, BN = 256, WTM = 32 * MT;
  constexpr int A_LOADS = (BM / 8) / NW, APT = A_LOADS / MT;
  static_assert(A_LOADS == MT && APT == 1, "one A load per wave and row tile");
  constexpr int A_STAGE = BM * 128, B_STAGE = BN * 128, S_STAGE = BM * 4;
  constexpr int B_BASE = NS * A_STAGE, S_BASE = B_BASE + NS * B_STAGE, NOWHERE = S_BASE + NS * S_STAGE;
  constexpr int TBL_BASE = NOWHERE + 256, TBL_BYTES = 2048, STG_BASE = TBL_BASE + 2 * TBL_BYTES, STG_ROW = 144;
  typedef v16f acc16_t;
  typedef typename std::conditional<gemm_is_int8(MODE), v16i, v16f>::type prod16_t;
  typedef typename OT::storage OS;
  static_assert(sizeof(OS) == 2, "2-byte outputs");

  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  __shared__ int s_rows[2][BM];    // sorted slot -> (token, k) pair id, of the current and of the next tile
  __shared__ float s_wgt[2][BM];   // the pair's routing weight (1 when the launch does not apply it)
  __shared__ float s_max[ACTQ ? 4 : 1][ACTQ ? BM : 1];  // ACTQ: a row's |activation| maximum in each wave's 32 columns

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WGN, wn = wave % WGN;

  const int tiles_n = (g.N + BN - 1) / BN;
  const int nblk = min(g.max_blocks_m, (*g.num_post_pad + BM - 1) / BM);
  const int total = nblk * tiles_n;
  const int nkb = g.K >> 7;  // 2..256 (checked by the launcher)
  // Round r of the walk gives workgroup w the tile r * G + (w + r * tiles_n) % G: every round still covers G
  // consecutive tiles (the column tiles of G / tiles_n consecutive sorted blocks, which share activation rows and,
  // for the blocks of one expert, weights), but a workgroup's position inside the round moves on by one sorted block
  // per round.  With w + r * G instead a workgroup keeps the parity of its sorted block for the whole launch, and
  // when experts own two blocks each (the first streams the expert's weights from HBM, the second finds them in L2
  // and finishes much earlier) half of the workgroups get all the slow tiles: DeepSeek-V3 layer at 8192 tokens
  // 5.60 ms against 5.06 ms with one tile per workgroup, whose dispatch order balances that by itself.
  // The position itself is XCD-aware: hardware workgroup w runs on XCD w % 8, and the workgroups of one XCD take
  // G / 8 consecutive positions, so that the column tiles of a sorted block (and the blocks of one expert) meet in
  // one L2 instead of fetching their shared rows once per XCD.
  const int G = (int)gridDim.x;
  const unsigned wpos = (unsigned)xcd_remap((int)blockIdx.x, G);
  auto tile_of_round = [&](int r) -> int { return r * G + (int)((wpos + (unsigned)(r * tiles_n)) % (unsigned)G); };
  int round = 0;
  int pid = tile_of_round(0);
  if (pid >= total) return;

  const int64_t a_rows = g.num_valid / g.top_k;
  const int a_bytes = (int)min(a_rows * g.lda, (int64_t)0x7fffffff);
  const int b_bytes = (int)min((int64_t)g.N * g.ldb, (int64_t)0x7fffffff);
  const int s_bytes = (int)min(((a_rows - 1) * g.sa_sm + (int64_t)(nkb - 1) * g.sa_sk + 1) * 4, (int64_t)0x7fffffff);
  const int t_bytes =
      (int)min(((int64_t)((g.N - 1) >> 7) * g.sb_sn + (int64_t)(nkb - 1) * g.sb_sk + 1) * 4, (int64_t)0x7fffffff);
  const int c_bytes = (int)min((int64_t)g.num_valid * g.ldc * (ACTQ ? 1 : 2), (int64_t)0x7fffffff);
  const int half_n = g.N >> 1;  // ACTQ: the weight's gate rows are 0 .. N/2 - 1, its up rows follow

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

  // ---- state of the tile whose K loop runs (or is about to) ----------------------------------------------
  int n0 = 0, expert = 0, buf = 0;
  const uint8_t* Bmat = g.B;
  uint32_t a_voff[MT], b_voff[2], s_voff = 0;
  // Row offsets, weight base and scale table of tile `p`, whose ids sit in s_rows[b]; requests the table.
  auto enter_tile = [&](int p, int b, int p_expert) {
    const int pm = p / tiles_n, pn = p - pm * tiles_n;
    n0 = pn * (ACTQ ? BN / 2 : BN);  // first output column of the tile
    expert = p_expert;
    const int ex = max(expert, 0);
    Bmat = g.B + (int64_t)ex * g.b_expert_stride;
#pragma unroll
    for (int t = 0; t < MT; t++) {
      const int row = (wave >> 2) * WTM + t * 32 + (wave & 3) * 8 + (lane >> 3);
      const int chunk = (lane & 7) ^ ((row >> 1) & 7);
      const int tok = s_rows[b][row];  // padding slots (>= num_valid) land past the descriptor's range: zeros
      a_voff[t] = tok < g.num_valid ? (uint32_t)((tok / g.top_k) * (int)g.lda + chunk * 16) : 0x7ffffff0u;
    }
#pragma unroll
    for (int l = 0; l < 2; l++) {
      const int row = (wave * 4 + l) * 8 + (lane >> 3);
      const int chunk = (lane & 7) ^ ((row >> 1) & 7);
      // ACTQ: LDS rows 64 w + 32 j + c hold gate (j = 0) / up (j = 1) row n0 + 32 w + c; a wave loads 32 of them
      const int wrow = ACTQ ? (wave & 1) * half_n + n0 + (wave >> 1) * 32 + l * 8 + (lane >> 3) : n0 + row;
      b_voff[l] = (uint32_t)(wrow * (int)g.ldb + chunk * 16);
    }
    {
      const int tok = s_rows[b][min(wave * 64 + lane, BM - 1)];
      const int srow = tok < g.num_valid ? tok / g.top_k : 0;
      s_voff = (uint32_t)(srow * (int)g.sa_sm) << 2;
    }
    // weight-block scales: entry e = cb * nkb + kb, 64 entries per wave
    const int e = wave * 64 + lane;
    const int cb = e / nkb, kbb = e - cb * nkb;
    // (ACTQ: column block 0 is the gate rows' scale block, column block 1 the up rows')
    const int sbrow = ACTQ ? (cb * half_n + n0) >> 7 : min(n0 + cb * 128, g.N - 1) >> 7;
    const uint32_t tv = cb < BN / 128 ? (uint32_t)(sbrow * (int)g.sb_sn + kbb * (int)g.sb_sk) << 2 : 0x7ffffff0u;
    dma4(g.sb + (int64_t)ex * g.sb_se, t_bytes, tv, 0, TBL_BASE + b * TBL_BYTES + wave * 256);
  };

  // piece t of K block kb of the current tile into a stage (part 0: the A load; part 1: the B loads and, with
  // the last piece, the activation scales)
  auto piece_loads = [](int t) constexpr { return APT + (4 / MT + ((4 % MT) > t ? 1 : 0)) + (t == MT - 1 ? 1 : 0); };
  constexpr int LPB = A_LOADS + 4 + 1;
  auto issue_piece = [&](int kb, int stage, int t, int part) {
    const bool live = kb < nkb;
    const int koff = kb << 7;
    if (part == 0) {
      dma16(g.A, live ? a_bytes : 0, a_voff[t], koff, stage * A_STAGE + ((wave >> 2) * WTM + t * 32 + (wave & 3) * 8) * 128);
      return;
    }
#pragma unroll
    for (int l = 0; l < 4; l++) {
      if (l % MT != t) continue;
      dma16(Bmat, live ? b_bytes : 0, b_voff[l & 1] + (uint32_t)((l & 2) * 8 * (int)g.ldb), koff,
            B_BASE + stage * B_STAGE + (wave * 4 + l) * 1024);
    }
    if (t == MT - 1) {
      const bool mine = wave < BM / 64;
      dma4(g.sa, (live && mine) ? s_bytes : 0, s_voff, (kb * (int)g.sa_sk) << 2,
           mine ? S_BASE + stage * S_STAGE + wave * 256 : NOWHERE);
    }
  };
  auto request_first_blocks = [&]() {
#pragma unroll
    for (int st = 0; st < NS; st++)
#pragma unroll
      for (int t = 0; t < MT; t++) {
        issue_piece(st, st, t, 0);
        issue_piece(st, st, t, 1);
      }
  };
  // ids of sorted block pm for this thread's slot, or a padding id when there is no such block
  auto read_id = [&](int p) -> int {
    if (p >= total || tid >= BM) return g.num_valid;
    return g.sorted_ids[(p / tiles_n) * BM + tid];
  };
  // the expert of tile p's sorted block (every lane reads the same word)
  auto read_expert = [&](int p) -> int { return p < total ? g.expert_ids[p / tiles_n] : 0; };

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

  // ---- the first tile: its ids and weights by plain loads, then like every other tile ---------------------
  {
    const int id = read_id(pid);
    if (tid < BM) {
      s_rows[0][tid] = id;
      s_wgt[0][tid] = (g.mul_weight && id < g.num_valid) ? g.topk_w[id] : 1.f;
    }
    __syncthreads();
    enter_tile(pid, 0, __builtin_amdgcn_readfirstlane(read_expert(pid)));
    request_first_blocks();
  }
  // both land under the first blocks' flight
  int id_next = read_id(tile_of_round(1));
  int ex_next = read_expert(tile_of_round(1));

  v8i wf[2][2], x0, x1;
  float sa_cur, sb_cur;
  float sb1_cur = 0.f, scp1 = 0.f;  // ACTQ: the second column tile (up rows) has a scale block of its own
  prod16_t qa, qb, zero16;
#pragma unroll
  for (int r = 0; r < 16; r++) qa[r] = 0, qb[r] = 0, zero16[r] = 0;
  float scp = 0.f;
  auto fold = [&](acc16_t& dst, const prod16_t& q, float sc) {
#pragma unroll
    for (int r = 0; r < 16; r++) dst[r] = fmaf((float)q[r], sc, dst[r]);
  };
  const float* sb_mine = nullptr;

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
    fold(acc[prev][1], qb, ACTQ ? scp1 : scp);
    __builtin_amdgcn_sched_group_barrier(0x2, FOLDN, 0);
    qb = mm_half(wf[1][0], x0, zero16);
    __builtin_amdgcn_sched_group_barrier(0x8, MPH, 0);
    __builtin_amdgcn_sched_barrier(0);
    issue_piece(kb + NS, cur, i, 0);
    __builtin_amdgcn_sched_barrier(0);
    float sa_nxt, sb_nxt = sb_cur, sb1_nxt = sb1_cur;
    if (!last) {
      x0 = xfrag(cur, i + 1, 0);
      sa_nxt = xscale(cur, i + 1);
      __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);
    } else {
      x0 = xfrag(nxt, 0, 0);
      wf[1][0] = wfrag(nxt, 1, 0);
      sa_nxt = xscale(nxt, 0);
      sb_nxt = sb_mine[min(kb + 1, nkb - 1)];
      if constexpr (ACTQ) sb1_nxt = sb_mine[nkb + min(kb + 1, nkb - 1)];
      __builtin_amdgcn_sched_group_barrier(0x100, ACTQ ? 7 : 6, 0);
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
    if constexpr (ACTQ) scp1 = sa_cur * sb1_cur;
    sa_cur = sa_nxt;
    sb_cur = sb_nxt;
    sb1_cur = sb1_nxt;
    __builtin_amdgcn_sched_group_barrier(0x2, ACTQ ? 2 : 1, 0);
    fold(acc[i][0], qa, scp);
    __builtin_amdgcn_sched_group_barrier(0x2, FOLDN, 0);
  };
  auto k_block = [&](int kb, auto stage_c) {
    tile_step(kb, stage_c, std::integral_constant<int, 0>{});
    if constexpr (MT > 1) tile_step(kb, stage_c, std::integral_constant<int, 1>{});
    if constexpr (MT > 2) tile_step(kb, stage_c, std::integral_constant<int, 2>{});
    if constexpr (MT > 3) tile_step(kb, stage_c, std::integral_constant<int, 3>{});
  };

  uint8_t* stg = smem + STG_BASE + wave * (32 * STG_ROW);
  for (;;) {
    // the tile's first two blocks, its scale table and the next tile's ids have landed (and the stores of the
    // tile before have left: vmcnt counts them too)
    __builtin_amdgcn_s_waitcnt(0x0070);
    __syncthreads();
    const int nbuf = buf ^ 1;
    const int expert_next = __builtin_amdgcn_readfirstlane(ex_next);
    float w_next = 1.f;
    if (tid < BM) {
      s_rows[nbuf][tid] = id_next;
      // in flight through the K loop; it is the oldest load outstanding there, so the loop's vmcnt waits (which
      // count loads issued later) hold as they are
      if (g.mul_weight && id_next < g.num_valid) w_next = g.topk_w[id_next];
    }
    sb_mine = (const float*)(smem + TBL_BASE + buf * TBL_BYTES) + (ACTQ ? 0 : (wn >> 1) * nkb);
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int h = 0; h < 2; h++) wf[j][h] = wfrag(0, j, h);
    x0 = xfrag(0, 0, 0);
    x1 = xfrag(0, 0, 1);
    sa_cur = xscale(0, 0);
    sb_cur = sb_mine[0];
    if constexpr (ACTQ) sb1_cur = sb_mine[nkb];

    for (int kb = 0; kb < nkb; kb += NS) {
      k_block(kb, std::integral_constant<int, 0>{});
      if (kb + 1 < nkb) k_block(kb + 1, std::integral_constant<int, 1>{});
    }
    fold(acc[MT - 1][1], qb, ACTQ ? scp1 : scp);
#pragma unroll
    for (int r = 0; r < 16; r++) qb[r] = 0;
    scp = 0.f;
    scp1 = 0.f;

    // Every wave is past its last fragment read once it has passed this barrier, and the trailing empty-range
    // loads (which still write zeros into the stages) have landed: the stages can take the next tile.
    __builtin_amdgcn_s_waitcnt(0x0070);
    if (tid < BM) s_wgt[nbuf][tid] = w_next;
    __syncthreads();
    const int n0_done = n0, expert_done = expert, buf_done = buf;
    const int next = tile_of_round(round + 1);
    const bool has_next = next < total;
    if (has_next) {
      enter_tile(next, nbuf, expert_next);
      request_first_blocks();
      id_next = read_id(tile_of_round(round + 2));
      ex_next = read_expert(tile_of_round(round + 2));
    }

    // Epilogue of the finished tile: each wave moves its (32*MT) x 64 part out in 32 x 64 patches through its own
    // staging rows (register r of tile (i, j) is C[.. + lane%32][.. + 32*j + 8*(r/4) + 4*(lane/32) + r%4]); 16-byte
    // stores, eight lanes per 128-byte row segment (a store instruction then touches 8 whole lines instead of 16
    // half lines: the vector memory pipe's cost per store follows the number of row segments), rows scattered to
    // their (token, k) pair.  Staging rows are 144 bytes apart: 16-byte aligned pieces, two-way bank conflicts on
    // the 8-byte writes at worst.
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (ACTQ) {
      // acc[i][0][r] and acc[i][1][r] are gate and up of output column n0 + 32 wn + 8 (r/4) + 4 (lane/32) + r%4.
      // Each is rounded to the 16-bit type first (the [gate | up] row the unfused sequence stores), then
      // silu(gate) is rounded, then the product: silu_and_mul's roundings; the result replaces acc[i][0][r].
      // A sorted block holds its pairs first and its padding slots behind them: a 32-row tile whose first slot is
      // padding holds nothing to store, and its conversions (an exp and a division per output) are skipped.
#pragma unroll
      for (int i = 0; i < MT; i++) {
        if (__builtin_amdgcn_readfirstlane(s_rows[buf_done][wm * WTM + i * 32]) >= g.num_valid) continue;
        const float wgt = expert_done < 0 ? 0.f : s_wgt[buf_done][wm * WTM + i * 32 + frow];
        float m = 0.f;
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const float gv = OT::to_f32(OT::from_f32(acc[i][0][r] * wgt));
          const float uv = OT::to_f32(OT::from_f32(acc[i][1][r] * wgt));
          const float sv = OT::to_f32(OT::from_f32(gv / (1.0f + expf(-gv))));
          const float y = OT::to_f32(OT::from_f32(sv * uv));
          acc[i][0][r] = y;
          m = fmaxf(m, fabsf(y));
        }
        m = fmaxf(m, __shfl_xor(m, 32, 64));
        if (fk == 0) s_max[wn][wm * WTM + i * 32 + frow] = m;
      }
      __syncthreads();
#pragma unroll
      for (int i = 0; i < MT; i++) {
        if (__builtin_amdgcn_readfirstlane(s_rows[buf_done][wm * WTM + i * 32]) >= g.num_valid) continue;
        const int trow = wm * WTM + i * 32 + frow;
        // the quantiser's reciprocal form with eps = 1e-10 (group_quant_body)
        const float amax = fmaxf(fmaxf(fmaxf(s_max[0][trow], s_max[1][trow]), fmaxf(s_max[2][trow], s_max[3][trow])), 1e-10f);
        const float mul = 448.f / amax;
#pragma unroll
        for (int rq = 0; rq < 4; rq++) {
          const uint32_t w = pack4_e4m3(clampf(acc[i][0][rq * 4] * mul, -448.f, 448.f),
                                        clampf(acc[i][0][rq * 4 + 1] * mul, -448.f, 448.f),
                                        clampf(acc[i][0][rq * 4 + 2] * mul, -448.f, 448.f),
                                        clampf(acc[i][0][rq * 4 + 3] * mul, -448.f, 448.f));
          *(uint32_t*)(stg + frow * STG_ROW + 8 * rq + 4 * fk) = w;
        }
        const int mine = s_rows[buf_done][trow];
        if (wn == 0 && fk == 0 && mine < g.num_valid)
          ((float*)g.A16)[(int64_t)mine * (half_n >> 7) + (n0_done >> 7)] = amax * (1.0f / 448.f);
        {
          // 32 rows x 32 bytes: two lanes per row, 16 bytes each
          const int row = lane >> 1, piece = lane & 1;
          const v4i v = *(const v4i*)(stg + row * STG_ROW + piece * 16);
          const int m_id = s_rows[buf_done][wm * WTM + i * 32 + row];
          const int n = n0_done + wn * 32 + piece * 16;
          const uint32_t vo = (m_id < g.num_valid && n < half_n) ? (uint32_t)(m_id * (int)g.ldc + n) : 0xfffffff0u;
          const v4i rs = {(int)(uint32_t)(uintptr_t)g.C, (int)(((uint64_t)(uintptr_t)g.C >> 32) & 0xffff), c_bytes, 0x00020000};
          asm volatile("s_nop 4\n\tbuffer_store_dwordx4 %0, %1, %2, 0 offen\n\ts_nop 1" : : "v"(v), "v"(vo), "s"(rs) : "memory");
        }
      }
    } else {
#pragma unroll
    for (int i = 0; i < MT; i++) {
      // (a 32-row tile of padding slots only: nothing to convert or store)
      if (__builtin_amdgcn_readfirstlane(s_rows[buf_done][wm * WTM + i * 32]) >= g.num_valid) continue;
      const float wgt = expert_done < 0 ? 0.f : s_wgt[buf_done][wm * WTM + i * 32 + frow];
#pragma unroll
      for (int j = 0; j < 2; j++)
#pragma unroll
        for (int rq = 0; rq < 4; rq++) {
          const v2i w = {(int)OT::pack2(acc[i][j][rq * 4] * wgt, acc[i][j][rq * 4 + 1] * wgt),
                         (int)OT::pack2(acc[i][j][rq * 4 + 2] * wgt, acc[i][j][rq * 4 + 3] * wgt)};
          *(v2i*)(stg + frow * STG_ROW + (32 * j + 8 * rq + 4 * fk) * 2) = w;
        }
#pragma unroll
      for (int q = 0; q < 4; q++) {
        const int row = (lane >> 3) + 8 * q, piece = lane & 7;
        const v4i v = *(const v4i*)(stg + row * STG_ROW + piece * 16);
        const int m = s_rows[buf_done][wm * WTM + i * 32 + row];
        const int n = n0_done + wn * 64 + piece * 8;
        // padding slots and columns past N are sent outside the descriptor's range and dropped
        const uint32_t vo = (m < g.num_valid && n < g.N) ? (uint32_t)((m * (int)g.ldc + n) * 2) : 0xfffffff0u;
        const v4i rs = {(int)(uint32_t)(uintptr_t)g.C, (int)(((uint64_t)(uintptr_t)g.C >> 32) & 0xffff), c_bytes, 0x00020000};
        // A store of more than 8 bytes reads its data registers in a second pass: a VALU write to them in the
        // next two issue slots would be stored instead; the compiler does not look into an asm statement.
        // Nor does it pad the five wait states a VMEM instruction needs behind a VALU write of an SGPR it reads:
        // when the descriptor has been spilled to VGPR lanes, v_readlane refills it right in front of the store,
        // which then goes out with the registers' old contents (seen as a memory fault) -- hence the s_nop 4.
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
    pid = next;
    round++;
    buf = nbuf;
  }
  __builtin_amdgcn_s_waitcnt(0x0070);
#endif
}

// Shapes the persistent MoE kernel takes: the tile kernel's own preconditions, K blocks that fit the scale tables,
// whole aligned 16-byte output pieces inside a 2 GiB range.
static inline bool gemm8_moe_persist_ok(const GemmArgs& g) {
  const int nkb = g.K >> 7;
  return (g.K % 128) == 0 && nkb >= 2 && nkb <= GEMM8_MOE_PERSIST_MAX_KB && (g.N & 7) == 0 && (g.ldc & 7) == 0 &&
         (((uintptr_t)g.C) & 15) == 0 && (int64_t)g.num_valid * g.ldc * 2 < 0x7fffffffll &&
         (int64_t)(g.num_valid / g.top_k) * g.lda < 0x7fffffffll && (int64_t)g.N * g.ldb < 0x7fffffffll;
}

template <int MODE, typename OT, int MT, bool ACTQ = false>
static int gemm8_moe_persist_launch(const GemmArgs& g, hipStream_t st) {
  auto kern = gemm8_moe_persist_kernel<MODE, OT, MT, ACTQ>;
  constexpr int smem = gemm8_moe_persist_smem<MT>();
  static SmemAttrOnce attr;
  hipError_t e = raise_dynamic_smem(attr, (const void*)kern, smem);
  if (e != hipSuccess) return fail(SGLAMD_EHIP, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  const int64_t tiles = (int64_t)((g.N + 255) / 256) * g.max_blocks_m;
  if (tiles <= 0) return SGLAMD_OK;
  const int64_t wgs = tiles < device_cus() ? tiles : device_cus();
  hipLaunchKernelGGL(kern, dim3((unsigned)wgs), dim3(512), smem, st, g);
  return check_launch("gemm8_moe_persist");
}

}  // namespace sglamd
