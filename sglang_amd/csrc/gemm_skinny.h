// Small-M ("decode") 8-bit GEMM for gfx950: a weight-streaming kernel.  With at most 64
// activation rows the multiply is bound by reading W once from HBM, so the kernel is organised
// around that stream and nothing else:
//   * a workgroup owns 16*FN weight rows (FN MFMA tiles of n) and all K; its KW wavefronts take the
//     128-byte K blocks round-robin (wave w: kb = w, w + KW, ...), so the waves of a workgroup read
//     adjacent 128-byte pieces of the same rows;
//   * W is fetched fully coalesced: 8 lanes read one 128-byte row piece, a wave-wide 16-byte load
//     covers 8 rows, two cover a 16-row tile (measured: this pattern streams at 6.1-6.7 TB/s, the
//     MFMA operand pattern -- 16 rows x 16 bytes per 16 lanes -- only at 4.3-5.0 TB/s);
//   * the loads go straight to LDS (buffer_load ... lds), into a per-wave ring of PD K blocks that
//     fills the CU's LDS; each piece lands at its swizzled place, so the MFMA operand fragments are
//     plain ds_read_b128, and rows / K pieces outside the tensors are never fetched (their lanes
//     carry an offset outside the buffer descriptor's range and read zeros);
//   * every wait for those loads is an explicit s_waitcnt vmcnt: left to the compiler, a register
//     ring of global loads was drained at every loop back-edge, which halves the bytes in flight;
//   * the activation tiles (FM tiles of 16 rows) and the scales are tiny and L2 resident; they are
//     fetched the same way alongside the weights;
//   * one v_mfma_f32_16x16x128_f8f6f4 per tile and K block with the weight fragment as first
//     operand (lane ends up with 4 consecutive n of one m), folded into the accumulator with the
//     block scale; the KW partial sums meet in LDS and leave as 8-byte stores.
// The same kernel walks the fused-MoE sorted-block schedule (MOE = true): tile rows are gathered
// through sorted_token_ids, the expert comes from expert_ids.
// With AQ > 0 (MoE, block FP8, at most AQ real rows per sorted block) the activations are not read as FP8 at all:
// the kernel takes the 16-bit source rows,
// quantises the tile's few rows per 128-wide group into LDS while the tile's first weight blocks are on their way,
// with the very arithmetic of the stand-alone group-quant kernel, so a decode-sized layer saves that kernel's launch.
#pragma once
#include <stdlib.h>

#include "gemm_core.h"
#include "quant_core.h"

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

// LDS of one ring slot: FN weight tiles and FM activation tiles of 16 rows x 128 bytes, then 256 bytes of
// activation-row scales and 256 bytes of weight-block scales.
// With AQ the slot only holds the FN weight tiles and the weight-block scales; the quantised activation rows of
// the whole tile live behind the rings (skinny_aq_bytes).
template <int FM, int FN, int AQ = 0>
constexpr int skinny_slot_bytes() {
  return AQ > 0 ? FN * 2048 + 256 : (FN + FM) * 2048 + 512;
}
// AQ rows of K bytes, each padded by 16 so that the rows' fragment reads spread over the banks, then their scales
static inline int skinny_aq_bytes(int aq, int K) { return aq * (K + 16) + aq * ((K + 127) >> 7) * 4; }
// Waves that may split K, and K blocks in flight per wave: the rings of all waves fill the LDS of a CU (156 KB of
// its 160), which is what keeps enough bytes in flight to stream from HBM at full rate.
template <int FM, int FN, int AQ = 0>
constexpr int skinny_kw_max() {
  return AQ == 0 && skinny_slot_bytes<FM, FN, AQ>() <= 6656 ? 8 : 4;
}
template <int FM, int FN, int AQ = 0>
constexpr int skinny_depth() {
  constexpr int d = 159744 / (skinny_kw_max<FM, FN, AQ>() * skinny_slot_bytes<FM, FN, AQ>());
  // with AQ three slots: the quantised rows need their place too, and seven one-wave workgroups still share a CU,
  // which takes the 1792 tiles of the DeepSeek-V3 layer's second GEMM in one round
  return AQ > 0 ? (d > 3 ? 3 : d) : (d > 4 ? 4 : d);
}

// Dynamic LDS of a launch: the rings of the KW waves, or, when a wave's partial tiles (FM * FN KB) do not fit its last
// ring slot (wide tiles), room for every wave's partial tiles side by side; plus the quantised rows (AQ).
template <int FM, int FN, int AQ = 0>
constexpr int skinny_smem_bytes(int kw, int extra_bytes = 0) {
  const int ring = kw * skinny_depth<FM, FN, AQ>() * skinny_slot_bytes<FM, FN, AQ>();
  const int part = FM * FN * 1024 > skinny_slot_bytes<FM, FN, AQ>() ? kw * FM * FN * 1024 : 0;
  return (ring > part ? ring : part) + extra_bytes;
}

// Operand voffset that lies past the range of every buffer descriptor used here (ranges are below 0x7ffffff0):
// a lane with this offset fetches nothing and its LDS slot receives zeros.
constexpr uint32_t SKINNY_NOWHERE = 0x7ffffff0u;

// Maximum over each aligned group of N = 4, 8 or 16 lanes, in all of them, on the DPP data path.
template <int N>
__device__ __forceinline__ float lanes_max(float v) {
  int x = __float_as_int(v);
#define SGLAMD_DPP_MAX(ctrl) \
  x = __float_as_int(fmaxf(__int_as_float(x), __int_as_float(__builtin_amdgcn_update_dpp(x, x, ctrl, 0xf, 0xf, false))))
  SGLAMD_DPP_MAX(0xB1);               // quad_perm [1, 0, 3, 2]
  SGLAMD_DPP_MAX(0x4E);               // quad_perm [2, 3, 0, 1]
  if (N >= 8) SGLAMD_DPP_MAX(0x141);  // row_half_mirror
  if (N >= 16) SGLAMD_DPP_MAX(0x140);  // row_mirror
#undef SGLAMD_DPP_MAX
  return __int_as_float(x);
}

template <int FM, int FN, int MODE, typename OT, bool MOE, int KW, int PD, int AQ = 0>
__global__ __launch_bounds__(64 * KW) void gemm8_skinny_kernel(GemmArgs g) {
#if defined(__HIP_DEVICE_COMPILE__)  // the host pass only needs the launch stub
  typedef typename AccT<MODE>::type acc_t;
  typedef typename OT::storage OS;
  constexpr bool BLK = gemm_is_block(MODE);
  constexpr int SLOT = skinny_slot_bytes<FM, FN, AQ>();
  constexpr int X_OFF = FN * 2048, SA_OFF = AQ > 0 ? 0 : (FN + FM) * 2048, SB_OFF = AQ > 0 ? FN * 2048 : SA_OFF + 256;
  // direct-to-LDS loads per K block and wave
  constexpr int LOADS = AQ > 0 ? 2 * FN + 1 : 2 * FN + 2 * FM + (BLK ? 2 : 0);
  static_assert(AQ == 0 || (MOE && MODE == GEMM_BLOCK_FP8 && FM == 1 && AQ <= 16),
                "in-kernel activation quantisation: MoE, block FP8, one row tile");
  static_assert(PD >= 1 && PD * LOADS < 64, "the vmcnt field counts up to 63 loads in flight");
  // a wave's partial tiles wait for the cross-wave sum in its last ring slot when they fit there; wide tiles put
  // them side by side over the whole ring area instead (behind a barrier: every wave's loads have landed by then)
  constexpr bool PART_IN_SLOT = FM * FN * 1024 <= SLOT;
  static_assert(PART_IN_SLOT || AQ == 0, "wide tiles do not quantise their activations");
  static_assert(PART_IN_SLOT || PD == 1, "wide tiles: no load of the next tile may be in flight while the sums meet");
  static_assert(FM <= 4 && FN <= 16, "one scale load covers 64 lanes: 4 activation tiles, 16 weight-scale slots");

  // Per wave a ring of PD slots.  The last slot of every wave doubles as the place where its partial tiles wait
  // for the cross-wave sum at the end of a tile.
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  __shared__ int s_rows[2][FM * 16];  // MoE: sorted slot ids of the tile's rows, for the current and the next tile
  // MoE with the routing sorted in the kernel (at most 32 (token, expert) pairs, at most 4 per expert): expert and
  // pair ids of each sorted block, and the number of blocks
  __shared__ int s_blk_expert[MOE ? 32 : 1], s_blk_rows[MOE ? 32 : 1][4], s_nblk;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int frow = lane & 15, fk = lane >> 4;

  // A tile is R consecutive weight rows (R <= 16*FN: a launch may trim R so that the number of tiles is a whole
  // multiple of the CU count; rows past R are neither fetched nor stored) times 16*FM activation rows.  A
  // workgroup walks tiles blockIdx.x, + gridDim.x, ...: with more tiles than resident workgroups the stream of
  // one tile continues into the next instead of ending in a workgroup's exit and another's start.
  const int R = g.rows_per_wg > 0 ? g.rows_per_wg : 16 * FN;
  const int tiles_n = (g.N + R - 1) / R;
  const int tiles_m = MOE ? g.max_blocks_m : (g.M + 16 * FM - 1) / (16 * FM);
  const int total = tiles_n * tiles_m;
  const bool self_sorted = MOE && g.route_ids != nullptr;
  if (MOE && self_sorted) {
    // What moe_align_block_size would hand over for these few pairs, in blocks of at most CAP rows (the rows a
    // tile quantises itself, four otherwise): blocks in ascending order of expert (id -1, an expert that lives
    // elsewhere, first: its rows are written as zeros), a block's pairs in ascending order of their index, ids
    // outside [-1, route_experts) dropped.  An expert with more than CAP pairs (a token that names it several
    // times) gets further blocks right behind its first.  One lane per pair; e is the id + 1, key orders the blocks.
    constexpr int CAP = AQ > 0 ? AQ : 4;
    static_assert(CAP == 1 || CAP == 2 || CAP == 4, "a block of the in-kernel sort holds 1, 2 or 4 rows");
    if (wave == 0) {
      const int numel = g.num_valid;
      int e = -1;
      if (lane < numel) {
        e = (g.route_ids_i64 ? (int)((const int64_t*)g.route_ids)[lane] : ((const int32_t*)g.route_ids)[lane]) + 1;
        if (e < 0 || e > g.route_experts) e = -1;
      }
      int slot = 0;
      for (int j = 0; j < numel; j++) {
        const int ej = __builtin_amdgcn_readlane(e, j);
        slot += (j < lane && ej == e) ? 1 : 0;
      }
      const int key = e * 32 + slot / CAP;  // at most 32 pairs
      const bool first = e >= 0 && slot % CAP == 0;
      const unsigned long long firsts = __ballot(first);
      int blk = 0;
      for (int j = 0; j < numel; j++) {
        const int kj = __builtin_amdgcn_readlane(key, j);
        blk += (((firsts >> j) & 1ull) && kj < key) ? 1 : 0;
      }
      if (lane < 32) {
#pragma unroll
        for (int q = 0; q < 4; q++) s_blk_rows[lane][q] = numel;
      }
      __builtin_amdgcn_wave_barrier();
      if (e >= 0) s_blk_rows[blk][slot % CAP] = lane;
      if (first) s_blk_expert[blk] = e - 1;
      if (lane == 0) s_nblk = __popcll(firsts);
    }
    __syncthreads();
  }
  const int bstride = (MOE && !self_sorted && g.sorted_stride > 0) ? g.sorted_stride : 16 * FM;
  const int post_pad = MOE ? __builtin_amdgcn_readfirstlane(self_sorted ? s_nblk * 16 * FM : *g.num_post_pad) : 0;
  // MoE first GEMM of a gated layer with the activation in its output: a tile pairs 16 gate rows with the 16 up
  // rows of the same columns (weight rows n and act_hidden + n) and writes silu(gate) * up, act_hidden wide.
  const bool paired = MOE && FM == 1 && FN == 2 && g.epi_silu;
  const int jstride = paired ? (int)g.act_hidden : 16;  // weight rows between a workgroup's column tiles

  const int nkb = (g.K + 127) >> 7;
  const int n_my = (nkb - wave + KW - 1) / KW;  // K blocks of this wave (may be <= 0)
  const bool ktail = (g.K & 127) != 0;
  const int64_t a_rows = MOE ? g.num_valid / g.top_k : g.M;

  // ---- what each lane fetches ----------------------------------------------------------------------------
  // A wave-wide 16-byte direct-to-LDS load writes lane l's piece to LDS slot l, so one load covers 8 rows of 128
  // bytes (8 lanes read one 128-byte row piece: the coalesced pattern that streams fastest) and two cover a
  // 16-row tile.  The 16-byte chunks of a row are XOR-swizzled with (row >> 1) & 7 for the fragment reads, and
  // since the load fixes where a lane's piece lands, the swizzle is applied on the global side: lane l fetches
  // chunk (l % 8) ^ key(row) of row l / 8 (+ 8 for the second load).
  const int lrow = lane >> 3;
  const int chunk0 = (lane & 7) ^ ((lrow >> 1) & 7), chunk1 = (lane & 7) ^ (((lrow + 8) >> 1) & 7);

  // Buffer descriptors: base, stride 0, byte range, raw 32-bit format.  The range check covers the per-lane
  // offset only, so everything that selects a row is per lane and the scalar offset carries the K position.
  auto descriptor = [](const void* base, int64_t bytes) -> v4i {
    const uint64_t b = (uint64_t)(uintptr_t)base;
    return v4i{(int)(uint32_t)b, (int)((b >> 32) & 0xffff), (int)(bytes < 0x7ffffff0ll ? bytes : 0x7ffffff0ll), 0x00020000};
  };
  const int64_t w_bytes = (int64_t)g.N * g.ldb;
  const int64_t sb_bytes = BLK ? ((int64_t)((g.N - 1) >> 7) * g.sb_sn + (int64_t)(nkb - 1) * g.sb_sk + 1) * 4 : 0;
  const v4i x_rs = descriptor(g.A, a_rows * g.lda);
  const v4i sa_rs = descriptor(g.sa, BLK ? ((a_rows - 1) * g.sa_sm + (int64_t)(nkb - 1) * g.sa_sk + 1) * 4 : 0);

  // ---- state of the tile being streamed (rewritten by setup() for the next one) ----------------------------
  int n0 = 0, n_end = 0, m0 = 0, expert = 0, rot = 0, rows_buf = 0;
  int aq_rows = 0;  // AQ: real rows of the tile's sorted block (<= AQ)
  uint32_t wv[FN][2], xv[FM][2];
  uint32_t sav_off = SKINNY_NOWHERE, sbv_off = SKINNY_NOWHERE;
  v4i w_rs = descriptor(g.B, w_bytes), sb_rs = descriptor(g.sb, sb_bytes);

  auto tile_exists = [&](int t) -> bool { return t < total && (!MOE || (t / tiles_n) * bstride < post_pad); };
  // per-lane offsets and descriptors of tile t; MoE tiles read their rows' slot ids into s_rows[buf] first
  auto setup = [&](int t, int buf) {
    const int pid_n = t % tiles_n, pid_m = t / tiles_n;
    n0 = paired ? pid_n * 16 : pid_n * R;
    m0 = pid_m * (MOE ? bstride : 16 * FM);
    n_end = paired ? n0 + 16 : min(g.N, n0 + R);
    rows_buf = buf;
    // Every tile walks the K blocks in its own rotation (the wave's j-th block is K block
    // (wave + j*KW + rot) % nkb).  Tiles that start together would otherwise all read the same K offsets of
    // different rows, and with a row stride that is a power of two (K = 8192, 16384) those addresses share a
    // few HBM channels: a plain read loop over such a matrix runs at 3.9-4.6 TB/s unrotated and 6.4-6.7 TB/s
    // rotated.  The rotation depends on the column tile only, so a row's sum is formed in the same order
    // wherever the row sits.
    // MoE launches rotate by the tile's 32-row group modulo 8, so that a tile pairing gate rows n.. with up rows
    // act_hidden + n.. (act_hidden % 256 == 0) sums in the same order as the two plain tiles that hold those rows.
    const uint32_t rot_key = MOE ? (uint32_t)((paired ? pid_n >> 1 : pid_n) & 7) : (uint32_t)pid_n;
    rot = __builtin_amdgcn_readfirstlane((int)((rot_key * 37u) % (uint32_t)nkb));
    if (MOE) {
      expert = __builtin_amdgcn_readfirstlane(self_sorted ? s_blk_expert[pid_m] : g.expert_ids[pid_m]);
      __syncthreads();  // nobody still reads this buffer for the output of the tile before the last
      if (tid < FM * 16)
        s_rows[buf][tid] = self_sorted ? (tid < 4 ? s_blk_rows[pid_m][tid] : g.num_valid)
                                       : (tid < bstride ? g.sorted_ids[m0 + tid] : g.num_valid);
      __syncthreads();
      w_rs = descriptor(g.B + (int64_t)max(expert, 0) * g.b_expert_stride, w_bytes);
      if (BLK) sb_rs = descriptor(g.sb + (int64_t)max(expert, 0) * g.sb_se, sb_bytes);
    }
#pragma unroll
    for (int j = 0; j < FN; j++) {
      const int r0 = n0 + j * jstride + lrow, r1 = r0 + 8;
      wv[j][0] = (paired || r0 < n_end) ? (uint32_t)(r0 * (int)g.ldb + chunk0 * 16) : SKINNY_NOWHERE;
      wv[j][1] = (paired || r1 < n_end) ? (uint32_t)(r1 * (int)g.ldb + chunk1 * 16) : SKINNY_NOWHERE;
    }
    if constexpr (AQ > 0) {
      const int slot_id = lane < 16 ? s_rows[buf][lane] : 0x7fffffff;
      const int real = __popcll(__ballot(slot_id < g.num_valid));  // a block's real rows come first
      aq_rows = __builtin_amdgcn_readfirstlane(real < AQ ? real : AQ);
    }
#pragma unroll
    for (int i = 0; i < (AQ > 0 ? 0 : FM); i++) {
      int r0, r1;
      if (MOE) {
        const int t0 = s_rows[buf][i * 16 + lrow], t1 = s_rows[buf][i * 16 + lrow + 8];
        r0 = t0 < g.num_valid ? t0 / g.top_k : -1;
        r1 = t1 < g.num_valid ? t1 / g.top_k : -1;
      } else {
        r0 = m0 + i * 16 + lrow < g.M ? m0 + i * 16 + lrow : -1;
        r1 = m0 + i * 16 + lrow + 8 < g.M ? m0 + i * 16 + lrow + 8 : -1;
      }
      xv[i][0] = r0 >= 0 ? (uint32_t)(r0 * (int)g.lda + chunk0 * 16) : SKINNY_NOWHERE;
      xv[i][1] = r1 >= 0 ? (uint32_t)(r1 * (int)g.lda + chunk1 * 16) : SKINNY_NOWHERE;
    }
    // scales: lane l fetches the activation scale of tile l / 16, row l % 16; lane l < 4*FN the weight-block
    // scale of the four output columns that lane (fk = l % 4) of column tile l / 4 ends up with (a trimmed R may
    // straddle a 128-row block)
    if (BLK) {
      sav_off = SKINNY_NOWHERE;
      sbv_off = SKINNY_NOWHERE;
      if (AQ == 0 && (lane >> 4) < FM) {
        int r;
        if (MOE) {
          const int tk = s_rows[buf][lane];
          r = tk < g.num_valid ? tk / g.top_k : -1;
        } else {
          r = m0 + lane < g.M ? m0 + lane : -1;
        }
        if (r >= 0) sav_off = (uint32_t)(r * (int)g.sa_sm) << 2;
      }
      if (lane < 4 * FN)
        sbv_off = (uint32_t)((min(n0 + (lane >> 2) * jstride + 4 * (lane & 3), g.N - 1) >> 7) * (int)g.sb_sn) << 2;
    }
  };

  // The loads are written as assembly: the compiler's wait-count pass neither pipelines register-destination
  // loads across the ring (it drains them at every loop back-edge) nor knows that a direct-to-LDS load completes
  // asynchronously.  Every wait for them is an explicit s_waitcnt vmcnt below.  (Loads and stores the compiler
  // issues itself in between only make both kinds of wait stricter than needed: vmcnt retires in issue order.)
  // Five wait states sit in front of every load: its descriptor and scalar offset may have been written by a VALU
  // instruction just before (v_readlane of a spilled scalar, v_readfirstlane), which a vector-memory instruction
  // must not read for 5 cycles; the compiler pads that hazard for its own instructions but does not look into
  // an asm statement (seen as loads from a stale descriptor once the kernel spilled scalars next to them).  The
  // same wait states cover the M0 write.
  const uint32_t ring = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)smem + wave * (PD * SLOT);
  auto dma16 = [&](const v4i& rs, uint32_t voff, int soff, uint32_t lds, bool nt) {
    if (nt)
      asm volatile("s_nop 4\n\tbuffer_load_dwordx4 %0, %1, %2 offen nt lds" : : "v"(voff), "s"(rs), "s"(soff), "{m0}"(lds) : "memory");
    else
      asm volatile("s_nop 4\n\tbuffer_load_dwordx4 %0, %1, %2 offen lds" : : "v"(voff), "s"(rs), "s"(soff), "{m0}"(lds) : "memory");
  };
  auto dma4 = [&](const v4i& rs, uint32_t voff, int soff, uint32_t lds) {
    asm volatile("s_nop 4\n\tbuffer_load_dword %0, %1, %2 offen lds" : : "v"(voff), "s"(rs), "s"(soff), "{m0}"(lds) : "memory");
  };
  // K block of the wave's j-th turn
  auto block_of = [&](int j) -> int {
    int kb = wave + j * KW + rot;
    if (kb >= nkb) kb -= nkb;
    return kb;
  };
  // requests K block kb of the current tile into ring slot s: LOADS loads (weights streamed past the caches)
  auto issue = [&](int s, int kb) {
    const uint32_t base = ring + s * SLOT;
    const int koff = kb << 7;
    // pieces past the end of a ragged K (K % 128 != 0, last block only) are sent nowhere: they read as zeros
    uint32_t kill0 = 0, kill1 = 0;
    if (ktail && kb == nkb - 1) {
      kill0 = skinny_piece(kb, chunk0, g.K).dead ? SKINNY_NOWHERE : 0u;
      kill1 = skinny_piece(kb, chunk1, g.K).dead ? SKINNY_NOWHERE : 0u;
    }
#pragma unroll
    for (int j = 0; j < FN; j++) {
      dma16(w_rs, wv[j][0] | kill0, koff, base + j * 2048, true);
      dma16(w_rs, wv[j][1] | kill1, koff, base + j * 2048 + 1024, true);
    }
    if constexpr (AQ > 0) {
      dma4(sb_rs, sbv_off, (kb * (int)g.sb_sk) << 2, base + SB_OFF);
    } else {
#pragma unroll
      for (int i = 0; i < FM; i++) {
        dma16(x_rs, xv[i][0] | kill0, koff, base + X_OFF + i * 2048, false);
        dma16(x_rs, xv[i][1] | kill1, koff, base + X_OFF + i * 2048 + 1024, false);
      }
      if (BLK) {
        dma4(sa_rs, sav_off, (kb * (int)g.sa_sk) << 2, base + SA_OFF);
        dma4(sb_rs, sbv_off, (kb * (int)g.sb_sk) << 2, base + SB_OFF);
      }
    }
  };

  // fragment of a 16x16x128 MFMA operand: lane -> row lane % 16, bytes 32*(lane / 16) .. +32, i.e. chunks 2*fk and
  // 2*fk + 1 at their swizzled positions
  const int fsw = (frow >> 1) & 7;
  const int ld0 = frow * 128 + (((2 * fk) ^ fsw) << 4), ld1 = frow * 128 + (((2 * fk + 1) ^ fsw) << 4);
  uint8_t* my_ring = smem + wave * (PD * SLOT);

  acc_t acc[FM * FN];

  // AQ: the tile's rows, quantised, behind the rings: AQ rows of K bytes (stride K + 16) and their group scales.
  uint8_t* xq_rows = smem + KW * PD * SLOT;
  const int xq_stride = g.K + 16;
  float* xq_scales = reinterpret_cast<float*>(xq_rows + AQ * xq_stride);
  // Quantises the real rows of the tile whose slot ids are in s_rows[buf]: per pass 16 groups of 128 over all the
  // workgroup's lanes, LPG = 4 * KW lanes per group and 128 / LPG elements per lane.  The arithmetic is
  // group_quant_body's (reciprocal form, float scales), so bytes and scales are the ones the stand-alone kernels
  // write.  The caller makes the result visible to the other waves (a workgroup barrier) before anyone reads it.
  auto quantise_rows = [&](int buf) {
   if constexpr (AQ > 0) {
    typedef typename OT::storage XS;
    constexpr int LPG = 4 * KW, EL = 128 / LPG, VEC = EL / 8;  // 16-byte loads per lane: EL 16-bit values
    static_assert(KW <= 4 && EL % 8 == 0, "a lane takes whole 16-byte pieces");
    const int sub = tid % LPG;
    // one pass of one row: the 16 groups from g0 on, this lane's EL values of its group in raw[]
    auto fetch = [&](const uint8_t* src, int g0, v4i* raw) {
      const int gi = g0 + tid / LPG;
      const int64_t eoff = (int64_t)(gi < nkb ? gi : 0) * 128 + sub * EL;  // element offset inside the row
#pragma unroll
      for (int q = 0; q < VEC; q++) raw[q] = *(const v4i*)(src + eoff * 2 + q * 16);
    };
    auto quantise = [&](int r, int g0, const v4i* raw) {
      const int gi = g0 + tid / LPG;
      float x[EL];
      XS e[EL];
      __builtin_memcpy(e, raw, EL * 2);
#pragma unroll
      for (int i = 0; i < EL; i++) x[i] = OT::to_f32(e[i]);
      float amax = g.q_eps;
#pragma unroll
      for (int i = 0; i < EL; i++) amax = fmaxf(amax, fabsf(x[i]));
      amax = lanes_max<LPG>(amax);
      const float s_store = amax * (1.0f / g.q_max);
      const float mul = g.q_max / amax;
      uint32_t o[EL / 4];
#pragma unroll
      for (int i = 0; i < EL / 4; i++)
        o[i] = pack4_e4m3(clampf(x[4 * i] * mul, g.q_min, g.q_max), clampf(x[4 * i + 1] * mul, g.q_min, g.q_max),
                          clampf(x[4 * i + 2] * mul, g.q_min, g.q_max), clampf(x[4 * i + 3] * mul, g.q_min, g.q_max));
      if (gi < nkb) {
        uint8_t* dst = xq_rows + r * xq_stride + gi * 128 + sub * EL;
        if constexpr (EL == 8) {
          *(v2i*)dst = v2i{(int)o[0], (int)o[1]};
        } else {
#pragma unroll
          for (int q = 0; q < EL / 16; q++) *(v4i*)(dst + q * 16) = v4i{(int)o[4 * q], (int)o[4 * q + 1], (int)o[4 * q + 2], (int)o[4 * q + 3]};
        }
        if (sub == 0) xq_scales[r * nkb + gi] = s_store;
      }
    };
    constexpr int MAXP = 4;  // passes whose loads are all issued before the first is used (K <= 8192)
    const int passes = (nkb + 15) >> 4;
    for (int r = 0; r < aq_rows; r++) {
      const int t = s_rows[buf][r];
      const uint8_t* src = (const uint8_t*)g.A16 + (int64_t)(t / g.top_k) * g.lda16;
      if (passes <= MAXP) {
        v4i raw[MAXP][VEC];
#pragma unroll
        for (int p = 0; p < MAXP; p++)
          if (p < passes) fetch(src, p * 16, raw[p]);
#pragma unroll
        for (int p = 0; p < MAXP; p++)
          if (p < passes) quantise(r, p * 16, raw[p]);
      } else {
        for (int g0 = 0; g0 < nkb; g0 += 16) {
          v4i raw[VEC];
          fetch(src, g0, raw);
          quantise(r, g0, raw);
        }
      }
    }
   }
  };

  // one K block out of ring slot s; `refill` >= 0 requests that K block into the slot once its fragments are in
  // registers
  auto consume = [&](int s, int kb_now, int refill) {
    const uint8_t* sl = my_ring + s * SLOT;
    v8i wf[FN], xf[FM];
    float sav[FM], sbv[FN];
#pragma unroll
    for (int j = 0; j < FN; j++) {
      const v4i lo = *(const v4i*)(sl + j * 2048 + ld0), hi = *(const v4i*)(sl + j * 2048 + ld1);
      wf[j] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    }
    if constexpr (AQ > 0) {
      // the block's real rows out of the tile's quantised rows; the other rows of the MFMA operand are zero
      v4i lo = {0, 0, 0, 0}, hi = {0, 0, 0, 0};
      sav[0] = 0.f;
      if (frow < aq_rows) {
        const uint8_t* xr = xq_rows + frow * xq_stride + (kb_now << 7) + fk * 32;
        lo = *(const v4i*)xr;
        hi = *(const v4i*)(xr + 16);
        sav[0] = xq_scales[frow * nkb + kb_now];
      }
      xf[0] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    } else {
#pragma unroll
      for (int i = 0; i < FM; i++) {
        const v4i lo = *(const v4i*)(sl + X_OFF + i * 2048 + ld0), hi = *(const v4i*)(sl + X_OFF + i * 2048 + ld1);
        xf[i] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      }
#pragma unroll
      for (int i = 0; i < FM; i++) sav[i] = BLK ? *(const float*)(sl + SA_OFF + (i * 16 + frow) * 4) : 1.f;
    }
#pragma unroll
    for (int j = 0; j < FN; j++) sbv[j] = BLK ? *(const float*)(sl + SB_OFF + (j * 4 + fk) * 4) : 1.f;
    // the slot is free once these reads have returned
    asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory");
    if (refill >= 0) issue(s, refill);
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
  };

  int tile = blockIdx.x;
  if (!tile_exists(tile)) return;
  setup(tile, 0);
#pragma unroll
  for (int s = 0; s < PD; s++)
    if (s < n_my) issue(s, block_of(s));
  if constexpr (AQ > 0) {
    quantise_rows(0);
    if (KW > 1) __syncthreads();
  }

  for (;;) {
#pragma unroll
    for (int i = 0; i < FM * FN; i++) acc[i] = acc_t{0, 0, 0, 0};
    // ---- the K loop: a ring of PD blocks in flight per wave -------------------------------------------------
    // vmcnt counts a wave's memory instructions in issue order, so "slot s has landed" is "at most as many
    // outstanding as were issued after slot s's", which is (PD - 1) * LOADS while every turn refills its slot.
    int it = 0;
    for (; it + 2 * PD <= n_my; it += PD) {
#pragma unroll
      for (int s = 0; s < PD; s++) {
        asm volatile("s_waitcnt vmcnt(%0)" : : "n"((PD - 1) * LOADS) : "memory");
        consume(s, block_of(it + s), block_of(it + s + PD));
      }
    }
    // the last PD .. 2*PD - 1 blocks (or all of them when the wave has fewer than 2*PD): the slots are drained
    // together, refilled where a block is left, and drained once more
    asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
#pragma unroll
    for (int s = 0; s < PD; s++)
      if (it + s < n_my) consume(s, block_of(it + s), it + s + PD < n_my ? block_of(it + s + PD) : -1);
    asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
#pragma unroll
    for (int s = 0; s < PD; s++)
      if (it + PD + s < n_my) consume(s, block_of(it + PD + s), -1);

    // ---- what the finished tile's output needs, then the next tile's first blocks are requested ---------------
    const int o_n0 = n0, o_n_end = n_end, o_m0 = m0, o_expert = expert, o_buf = rows_buf;
    const int next = tile + (int)gridDim.x;
    const bool has_next = tile_exists(next);
    if (has_next) {
      setup(next, o_buf ^ 1);
      // with several waves the last slot of every ring carries the partial tiles first
#pragma unroll
      for (int s = 0; s < PD - (KW > 1 ? 1 : 0); s++)
        if (s < n_my) issue(s, block_of(s));
      // every wave is past its K loop (setup's barriers), so the rows can be replaced; with several waves the
      // barriers of the reduction below stand between these writes and the next tile's first reads
      if constexpr (AQ > 0) quantise_rows(o_buf ^ 1);
    }

    // ---- reduce the KW partial tiles through LDS (every wave's own last ring slot) ------------------------------
    // wave w finishes the (i, j) tiles t = w, w + KW, ...
    // (a paired tile's two column tiles are both finished by wave 0: a lane needs the gate and the up value)
    constexpr int NT0 = (FM * FN + KW - 1) / KW;
    constexpr int NT = (MOE && FM == 1 && FN == 2 && NT0 < 2) ? 2 : NT0;
    auto tile_of = [&](int idx) -> int { return paired ? (wave == 0 ? idx : FM * FN) : wave + idx * KW; };
    acc_t sums[NT];
    if (KW > 1) {
      constexpr int PART_STRIDE = PART_IN_SLOT ? PD * SLOT : FM * FN * 1024;
      constexpr int PART_FIRST = PART_IN_SLOT ? (PD - 1) * SLOT : 0;
      // (wide tiles: the area overlaps other waves' slots, whose last loads have landed once they are here too)
      if constexpr (!PART_IN_SLOT) __syncthreads();
      acc_t* mine = reinterpret_cast<acc_t*>(smem + wave * PART_STRIDE + PART_FIRST);
#pragma unroll
      for (int i = 0; i < FM * FN; i++) mine[i * 64 + lane] = acc[i];
      __syncthreads();
#pragma unroll
      for (int idx = 0; idx < NT; idx++) {
        const int t = tile_of(idx);
        acc_t a = acc_t{0, 0, 0, 0};
        if (t < FM * FN) {
#pragma unroll
          for (int w = 0; w < KW; w++)
            a += reinterpret_cast<const acc_t*>(smem + w * PART_STRIDE + PART_FIRST)[t * 64 + lane];
        }
        sums[idx] = a;
      }
      // the partial tiles have been read: the slots that carried them take the next tile's last block
      __syncthreads();
      if (has_next && PD - 1 < n_my) issue(PD - 1, block_of(PD - 1));
    } else {
#pragma unroll
      for (int idx = 0; idx < NT; idx++) sums[idx] = idx < FM * FN ? acc[idx < FM * FN ? idx : 0] : acc_t{0, 0, 0, 0};
    }

    if constexpr (MOE && FM == 1 && FN == 2 && BLK) {
      if (paired) {
        // silu(gate) * up of the 16 x 16 patch, rounded as the stand-alone activation kernels round: the two GEMM
        // outputs to the 16-bit type first, then silu, then the product
        const int tok = s_rows[o_buf][frow];
        if (wave == 0 && tok < g.num_valid) {
          OS o[4];
#pragma unroll
          for (int r = 0; r < 4; r++) {
            float gv = (float)sums[0][r], uv = (float)sums[1][r];
            if (o_expert < 0) gv = 0.f, uv = 0.f;
            gv = OT::to_f32(OT::from_f32(gv));
            uv = OT::to_f32(OT::from_f32(uv));
            const float sv = OT::to_f32(OT::from_f32(gv / (1.0f + expf(-gv))));
            o[r] = OT::from_f32(sv * uv);
          }
          v2i w2;
          __builtin_memcpy(&w2, o, 8);
          *(v2i*)((OS*)g.C + (int64_t)tok * g.ldc + o_n0 + 4 * fk) = w2;
        }
        if (!has_next) break;
        tile = next;
        continue;
      }
    }

#pragma unroll
    for (int idx = 0; idx < NT; idx++) {
      const int t = tile_of(idx);
      if (t >= FM * FN) break;
      const int i = t / FN, j = t % FN;
      const acc_t a = sums[idx];
      int64_t out_row;
      bool row_ok;
      float wgt = 1.f;
      if (MOE) {
        const int tok = s_rows[o_buf][i * 16 + frow];
        row_ok = tok < g.num_valid;
        out_row = tok;
        if (row_ok && g.mul_weight) wgt = g.topk_w[tok];
      } else {
        row_ok = (o_m0 + i * 16 + frow) < g.M;
        out_row = o_m0 + i * 16 + frow;
      }
      const int n = o_n0 + j * 16 + 4 * fk;
      if (!row_ok || n >= o_n_end) continue;
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
          if (o_expert < 0) v[r] = 0.f;
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
    if (!has_next) break;
    tile = next;
  }
#endif
}

// Preconditions of the streaming kernel beyond the operators' own: both operands and the scale arrays are
// addressed through 32-bit buffer offsets.
static inline bool gemm8_skinny_ok(const GemmArgs& g, int64_t a_rows) {
  const int64_t nkb = (g.K + 127) >> 7;
  const bool scales_ok = (a_rows * (g.sa_sm > 0 ? g.sa_sm : 1) + nkb * (g.sa_sk > 0 ? g.sa_sk : 1)) * 4 < 0x7ffffff0ll &&
                         (((int64_t)g.N >> 7) + 1) * (g.sb_sn > 0 ? g.sb_sn : 1) * 4 + nkb * (g.sb_sk > 0 ? g.sb_sk : 1) * 4 < 0x7ffffff0ll;
  return a_rows * g.lda < 0x7ffffff0ll && (int64_t)g.N * g.ldb < 0x7ffffff0ll && scales_ok;
}

// Workgroups of one launch that a CU holds at once: bounded by the LDS rings and by 32 wavefronts.
template <int FM, int FN, int AQ = 0>
static inline int skinny_resident_per_cu(int kw, int extra_bytes = 0) {
  const int smem = skinny_smem_bytes<FM, FN, AQ>(kw, extra_bytes) + 1024;
  int n = 163840 / smem;
  if (n > 32 / kw) n = 32 / kw;
  return n < 1 ? 1 : n;
}

template <int FM, int FN, int MODE, typename OT, bool MOE, int KW, int AQ = 0>
static int gemm8_skinny_launch_kw(const GemmArgs& g, hipStream_t st) {
  constexpr int PD = skinny_depth<FM, FN, AQ>();
  const int aq_bytes = AQ > 0 ? skinny_aq_bytes(AQ, g.K) : 0;
  const int smem = skinny_smem_bytes<FM, FN, AQ>(KW, aq_bytes);
  if (smem > 160 * 1024) return fail(SGLAMD_ENOTSUP, "gemm: K = %d is too long for in-kernel activation quantisation", g.K);
  const int R = g.rows_per_wg > 0 ? g.rows_per_wg : 16 * FN;
  const int tiles_n = (g.N + R - 1) / R;
  const int tiles_m = MOE ? g.max_blocks_m : (g.M + 16 * FM - 1) / (16 * FM);
  const int64_t tiles = (int64_t)tiles_n * tiles_m;
  if (tiles <= 0) return SGLAMD_OK;
  if (tiles > 0x7fffffff) return fail(SGLAMD_EINVAL, "gemm: grid too large");
  // as many workgroups as the chip holds at once; each walks tiles blockIdx.x, + gridDim.x, ...
  const int64_t resident = (int64_t)device_cus() * skinny_resident_per_cu<FM, FN, AQ>(KW, aq_bytes);
  const unsigned blocks = (unsigned)(tiles < resident ? tiles : resident);
  auto kern = gemm8_skinny_kernel<FM, FN, MODE, OT, MOE, KW, PD, AQ>;
  if (smem > 64 * 1024) {
    static SmemAttrOnce attr;
    hipError_t e = raise_dynamic_smem(attr, (const void*)kern, smem);
    if (e != hipSuccess) return fail(SGLAMD_EHIP, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  }
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(64 * KW), smem, st, g);
  return check_launch("gemm8_skinny");
}

static inline int skinny_env(const char* name) {
  const char* e = getenv(name);
  return e ? atoi(e) : 0;
}

// Waves that split K.  A workgroup walks its tiles one after the other, and every tile ends in a drain (its last
// blocks land, the partial sums meet, the output leaves) during which that workgroup streams little: few tiles
// per workgroup ("rounds") are good, and fewer waves per workgroup mean smaller rings, more resident workgroups
// and fewer rounds.  More waves shorten a tile's chain.  Cost = rounds x kw^-0.8, fitted to sweeps of the
// DeepSeek-V3 dense and MoE decode launches (N = 36864: 4 waves in 3 rounds beat 2 in 2 and 1 in 1; the MoE
// layer's second GEMM with 16 K blocks and 1792 tiles: 1 wave in 1 round beats 4 in 4).  Every wave keeps two K
// blocks, and the workgroups resident on a CU at least 64 KB of weight bytes in flight.
template <int FM, int FN, int AQ = 0>
static inline int skinny_pick_kw(int64_t tiles, int nkb, int extra_bytes = 0) {
  static const int force_kw = skinny_env("SGLAMD_SKINNY_KW");
  constexpr int KW_MAX = skinny_kw_max<FM, FN, AQ>();
  if (force_kw) return force_kw < KW_MAX ? force_kw : KW_MAX;
  const int cus = device_cus();
  static const double weight[4] = {1.0, 0.574, 0.330, 0.189};  // kw^-0.8 for kw = 1, 2, 4, 8
  int best = 1;
  double best_cost = -1.0;
  for (int kw = 1, i = 0; kw <= KW_MAX; kw *= 2, i++) {
    if (kw > 1 && nkb / (kw * 2) < 2) break;
    const int per_cu = skinny_resident_per_cu<FM, FN, AQ>(kw, extra_bytes);
    const int64_t rounds = (tiles + (int64_t)cus * per_cu - 1) / ((int64_t)cus * per_cu);
    const int64_t active = tiles < (int64_t)cus * per_cu ? (tiles + cus - 1) / cus : per_cu;
    const int64_t in_flight = active * kw * skinny_depth<FM, FN, AQ>() * FN * 2048;
    if (in_flight < 65536 && kw < KW_MAX && nkb / (kw * 4) >= 2) continue;  // a larger kw is still to come
    const double cost = (double)rounds * weight[i];
    if (best_cost < 0 || cost < best_cost) {
      best_cost = cost;
      best = kw;
    }
  }
  return best;
}

// Shape of the last streaming launch of this thread and translation unit: (FM << 16) | (FN << 8) | KW.
extern thread_local int skinny_last_shape;  // defined in gemm.hip

template <int FM, int FN, int MODE, typename OT, bool MOE, int AQ = 0>
static int gemm8_skinny_launch_fn(const GemmArgs& g, hipStream_t st, int64_t expected_tiles_m) {
  const int R = g.rows_per_wg > 0 ? g.rows_per_wg : 16 * FN;
  const int64_t tiles = (int64_t)((g.N + R - 1) / R) * (expected_tiles_m > 0 ? expected_tiles_m : 1);
  // A launch that quantises its activations itself splits K the way the plain launch of the same shape would (up
  // to the four waves it supports): the same partial sums in the same order, so both give the same bits.
  int kw = skinny_pick_kw<FM, FN>(tiles, (g.K + 127) >> 7);
  if (AQ > 0 && kw > 4) kw = 4;
  skinny_last_shape = (FM << 16) | (FN << 8) | kw;
  switch (kw) {
    case 1:
      return gemm8_skinny_launch_kw<FM, FN, MODE, OT, MOE, 1, AQ>(g, st);
    case 2:
      return gemm8_skinny_launch_kw<FM, FN, MODE, OT, MOE, 2, AQ>(g, st);
    case 4:
      return gemm8_skinny_launch_kw<FM, FN, MODE, OT, MOE, 4, AQ>(g, st);
    default:
      if constexpr (skinny_kw_max<FM, FN, AQ>() >= 8) return gemm8_skinny_launch_kw<FM, FN, MODE, OT, MOE, 8, AQ>(g, st);
      return gemm8_skinny_launch_kw<FM, FN, MODE, OT, MOE, 4, AQ>(g, st);
  }
}

// MoE launch that quantises the activations in the kernel (see the head of this file): `g` carries the 16-bit
// source rows in A16 / lda16 (act_mode 1) and the quantisation constants; every sorted block holds at
// most four real rows (the caller launches it for at most four tokens).
template <typename OT>
static int gemm8_skinny_launch_actquant(const GemmArgs& g, hipStream_t st, int64_t expected_tiles_m) {
  return gemm8_skinny_launch_fn<1, 2, GEMM_BLOCK_FP8, OT, true, 4>(g, st, expected_tiles_m);
}

// Cost of a dense launch with FN column tiles per workgroup trimmed to `rows` weight rows, in "weight rows streamed
// by the busiest workgroup": the resident workgroups take the tiles round-robin, and every tile costs its rows
// plus its share of the activation rows (L2 hits, about a fifth of a weight byte each) plus a fixed part (drain,
// cross-wave sum, output: about 1 us, i.e. the ~27 KB a CU streams in that time).
template <int FM, int FN>
static inline double skinny_cost(const GemmArgs& g, int rows) {
  const int64_t tiles = (int64_t)((g.N + rows - 1) / rows) * ((g.M + 16 * FM - 1) / (16 * FM));
  const int nkb = (g.K + 127) >> 7;
  const int kw = skinny_pick_kw<FM, FN>(tiles, nkb);
  const int64_t resident = (int64_t)device_cus() * skinny_resident_per_cu<FM, FN>(kw);
  const int64_t rounds = (tiles + resident - 1) / resident;
  const int act_rows = g.M < 16 * FM ? g.M : 16 * FM;
  // workgroups sharing a CU share its bandwidth: a round of `per_cu` co-resident tiles takes per_cu times as long
  return (double)rounds * skinny_resident_per_cu<FM, FN>(kw) * (rows + 0.2 * act_rows + 27000.0 / g.K);
}

// Column tiles per workgroup (FN) and the rows it keeps of them.  More rows per tile mean fewer activation bytes per
// weight byte; the tile count should fill the resident workgroups a whole number of times (N = 7168 runs as 256
// tiles of 28 rows instead of 224 of 32 with 32 CUs idle).  MoE launches keep the 32-row tile of the sorted-block
// schedule's column split.
template <int FM, int MODE, typename OT, bool MOE>
static int gemm8_skinny_launch(const GemmArgs& g0, hipStream_t st, int64_t expected_tiles_m) {
  static const int force_fn = skinny_env("SGLAMD_SKINNY_FN");
  static const int force_rows = skinny_env("SGLAMD_SKINNY_ROWS");
  GemmArgs g = g0;
  int fn = (g.N % 32 == 0 && g.N >= 2048) ? 2 : 1;
  if constexpr (!MOE) {
    if (g.N >= 1024) {
      double best = -1.0;
      int best_rows = 16 * fn;
      auto consider = [&](int f, double (*cost)(const GemmArgs&, int)) {
        if (force_fn && force_fn != f) return;
        for (int rows = 16 * f; rows > 16 * f - 16 && rows >= 12; rows -= 4) {
          if (force_rows && force_rows != rows) continue;
          const double c = cost(g, rows);
          if (best < 0 || c < best - 1e-9) {
            best = c;
            best_rows = rows;
            fn = f;
          }
        }
      };
      if constexpr (FM <= 2) {
        consider(4, skinny_cost<FM, 4>);
        consider(3, skinny_cost<FM, 3>);
      }
      consider(2, skinny_cost<FM, 2>);
      consider(1, skinny_cost<FM, 1>);
      g.rows_per_wg = best_rows == 16 * fn ? 0 : best_rows;
    }
  } else if (force_fn == 1 || force_fn == 2) {
    fn = force_fn;
  }
  if constexpr (FM <= 2 && !MOE) {
    if (fn == 4) return gemm8_skinny_launch_fn<FM, 4, MODE, OT, MOE>(g, st, expected_tiles_m);
    if (fn == 3) return gemm8_skinny_launch_fn<FM, 3, MODE, OT, MOE>(g, st, expected_tiles_m);
  }
  if (fn == 2) return gemm8_skinny_launch_fn<FM, 2, MODE, OT, MOE>(g, st, expected_tiles_m);
  return gemm8_skinny_launch_fn<FM, 1, MODE, OT, MOE>(g, st, expected_tiles_m);
}

// Wide form for 33..64 activation rows on weights with many rows: four row tiles times FN = 6, 8 or 9 column tiles
// (96..144 weight rows) per workgroup, four waves that share K block by block, one ring slot per wave (the four
// slots and what is in flight to them fill most of LDS).  Per K block a workgroup then fetches 8 KB of activation
// rows for 12..18 KB of weight rows, where the two-column-tile form fetches 8 KB for 4 KB; the tile count is made a
// whole multiple of the CU count by trimming the rows per workgroup.  Returns the weight rows per workgroup it would
// use (0: the shape is not for this form) when `launch` is false.
template <int MODE, typename OT>
static int gemm8_skinny_wide(const GemmArgs& g0, hipStream_t st, bool launch) {
  const int cus = device_cus();
  const int nkb = (g0.K + 127) >> 7;
  // A tile ends in a drain (the last blocks land, the partial sums of the four waves meet in LDS, the output leaves)
  // that costs about as much as 8 K blocks: with fewer than 40 blocks per tile the tile kernel is the faster one
  // (measured on N = 24576, K = 1536: 15.2 against 12.1 us; N = 65536, K = 4224: 65.5 against 54.2 us; from K = 7168
  // on this form wins, DeepSeek-V3 gate_up at 64 / 48 / 40 rows: 57.5 / 54.2 / 54.6 against 65.0 / 63.3 / 61.9 us,
  // Llama-3-70B gate_up at 64 rows: 100.7 against 109.0 us)
  static const int min_kb = skinny_env("SGLAMD_WIDE_MIN_KB") ? skinny_env("SGLAMD_WIDE_MIN_KB") : 40;
  if (g0.M <= 32 || g0.M > 64 || nkb < min_kb || (g0.N & 3)) return 0;
  // rows per workgroup: the candidate that streams the fewest rows through the busiest CU, activation rows counted
  // at what they cost beside weight rows (L2 hits, same vector-memory path)
  int best_rows = 0;
  double best = 0.0;
  for (int rows = 144; rows >= 84; rows -= 4) {
    const int fn = (rows + 15) / 16;
    if (fn != 6 && fn != 8 && fn != 9) continue;
    const int64_t tiles = (g0.N + rows - 1) / rows;
    if (tiles * 4 < (int64_t)cus * 3) continue;  // too few workgroups to fill the chip
    const int64_t rounds = (tiles + cus - 1) / cus;
    const double cost = (double)rounds * (rows + 0.5 * 64 + 27000.0 / g0.K);
    if (best_rows == 0 || cost < best - 1e-9) {
      best = cost;
      best_rows = rows;
    }
  }
  if (!launch || best_rows == 0) return best_rows;
  GemmArgs g = g0;
  const int fn = (best_rows + 15) / 16;
  g.rows_per_wg = best_rows == 16 * fn ? 0 : best_rows;
  skinny_last_shape = (4 << 16) | (fn << 8) | 4;
  if (fn == 6) return gemm8_skinny_launch_kw<4, 6, MODE, OT, false, 4>(g, st);
  if (fn == 8) return gemm8_skinny_launch_kw<4, 8, MODE, OT, false, 4>(g, st);
  return gemm8_skinny_launch_kw<4, 9, MODE, OT, false, 4>(g, st);
}

}  // namespace sglamd
