// Tiled 8-bit GEMM core for gfx950 shared by the dense operators and the fused-MoE grouped
// GEMM.  C[m, n] = sum_k A[m, k] * B[n, k] with A [M, K] and B [N, K] both K-contiguous
// bytes (OCP e4m3fn or int8).
//
// Tiling: a workgroup of WGM x WGN wavefronts owns a BM x BN tile of C and walks K in
// 128-byte blocks (one block-scale group).  Both operand tiles are staged in LDS as rows of
// 128 bytes whose eight 16-byte chunks are XOR-swizzled by ((row >> 1) & 7): LDS serves 256 bytes
// (two rows) per clock, so the 16-row x 32-byte fragment reads touch each of the 64 banks once.  LDS is double buffered and
// the next block's global loads are in flight while the current block is multiplied.
//
// MFMA mapping: v_mfma_f32_16x16x128_f8f6f4 (or two v_mfma_i32_16x16x64_i8) with the weight
// fragment as the first operand and the activation fragment as the second, so a lane ends
// up holding four consecutive n for one m: the row scale (and the MoE routing weight) is
// one scalar per lane and the store is 8 contiguous bytes per lane.
//
// Block-scaled mode: each K block's product starts from zero and is folded into the running
// accumulator as acc += partial * (sa[m, kb] * sb[nb, kb]).
#pragma once
#include "common.h"

namespace sglamd {

enum { GEMM_BLOCK_FP8 = 0, GEMM_ROW_FP8 = 1, GEMM_ROW_INT8 = 2, GEMM_BLOCK_INT8 = 3 };
// block modes fold every 128-wide K block's partial product with sa[m, kb] * sb[n/128, kb] into an fp32
// accumulator; row modes accumulate raw products and scale once at the end
constexpr bool gemm_is_block(int mode) { return mode == GEMM_BLOCK_FP8 || mode == GEMM_BLOCK_INT8; }
constexpr bool gemm_is_int8(int mode) { return mode == GEMM_ROW_INT8 || mode == GEMM_BLOCK_INT8; }

struct GemmArgs {
  const uint8_t* A;
  int64_t lda;
  const uint8_t* B;
  int64_t ldb;
  int64_t b_expert_stride;  // MoE: bytes between experts' weight matrices
  const float* sa;          // block: sa[m*sa_sm + kb*sa_sk]; rowwise: sa[m]
  int64_t sa_sm, sa_sk;
  const float* sb;          // block: sb[e*sb_se + nb*sb_sn + kb*sb_sk]; rowwise: sb[n]
  int64_t sb_sn, sb_sk, sb_se;
  const void* bias;         // rowwise, optional, [N] in the output dtype
  void* C;
  int64_t ldc;
  int M, N, K;
  // fused-MoE schedule (unused for dense)
  const int32_t* sorted_ids;
  const int32_t* expert_ids;
  const int32_t* num_post_pad;
  const float* topk_w;
  int top_k;
  int num_valid;
  int mul_weight;
  int max_blocks_m;
  int rows_per_wg;  // skinny kernel: weight rows a workgroup owns (multiple of 4, <= 16*FN); 0 = 16*FN
  // skinny MoE kernel with in-kernel activation quantisation: the 16-bit rows that take A's place.
  // (The persistent MoE kernel with the activation in its epilogue has no such rows and finds the address of
  // the group scales it writes, fp32 [pairs, N / 256], here: one more argument word would cost a scalar register.)
  const void* A16;
  int64_t lda16;       // bytes between rows
  int act_mode;        // 1: quantise the rows of A16 in the kernel
  int64_t act_hidden;  // epi_silu: elements per half of the [gate | up] rows the weight produces
  float q_eps, q_min, q_max;
  // skinny MoE kernel, first GEMM of a gated layer: write silu(gate) * up (act_hidden wide) instead of [gate | up]
  int epi_silu;
  // skinny MoE kernel sorting the routing itself (at most 32 pairs, 4 per expert): topk_ids as handed to the layer
  const void* route_ids;
  int route_ids_i64;
  int route_experts;
  // skinny MoE kernel: entries of sorted_ids per block when that is less than the tile height (a schedule aligned
  // to blocks of 4 for tiles that hold at most 4 real rows); 0 = the tile height
  int sorted_stride;
  // block FP8: every scale is a power of two, so a kernel may apply them through the MFMA's scale operands
  int scales_pow2;
};

// What only the generic kernel takes (kept out of GemmArgs: the specialised kernels sit at the edge of their
// register budget, and every argument word costs them a scalar register).
struct GemmExt {
  // scale-block shape of the block modes, 64 or 128 each (0 = 128): sb holds one scale per block_n weight rows and
  // block_k columns, sa one per row and block_k columns
  int block_n, block_k;
  // MoE: element strides of the row modes' scales (sa[(slot / top_k) * row_sa_stride],
  // sb[expert * sb_se + n * row_sb_stride]; a stride of 0 makes the scale per tensor / per expert) and the
  // stride between the experts' bias rows (bias[expert * bias_se + n], any mode)
  int64_t row_sa_stride, row_sb_stride, bias_se;
};
struct GemmArgsX {
  GemmArgs g;
  GemmExt x;
};
__host__ __device__ inline const GemmArgs& args_base(const GemmArgs& a) { return a; }
__host__ __device__ inline const GemmArgs& args_base(const GemmArgsX& a) { return a.g; }
__host__ __device__ inline GemmExt args_ext(const GemmArgs&) { return GemmExt{0, 0, 1, 1, 0}; }
__host__ __device__ inline GemmExt args_ext(const GemmArgsX& a) { return a.x; }

// Bijective remap of the hardware workgroup id so that each of the 8 XCDs (which receive
// consecutive ids round-robin) works on one contiguous range of logical tiles and its L2
// sees a compact set of operand rows.
__device__ __forceinline__ int xcd_remap(int bid, int nblocks) {
  const int q = nblocks >> 3, r = nblocks & 7;
  const int xcd = bid & 7, idx = bid >> 3;
  const int base = xcd < r ? xcd * (q + 1) : r * (q + 1) + (xcd - r) * q;
  return base + idx;
}

template <int MODE>
struct AccT {
  typedef v4f type;
};
template <>
struct AccT<GEMM_ROW_INT8> {
  typedef v4i type;
};

template <int BM, int BN, int WGM, int WGN, int MODE, typename OT, bool MOE, typename GA = GemmArgs>
__global__ __launch_bounds__(64 * WGM * WGN) void gemm8_kernel(GA ga) {
  const GemmArgs& g = args_base(ga);
  const GemmExt gx = args_ext(ga);
  constexpr int NT = 64 * WGM * WGN;
  constexpr int WTM = BM / WGM, WTN = BN / WGN;
  constexpr int FM = WTM / 16, FN = WTN / 16;
  static_assert(WTM % 16 == 0 && WTN % 16 == 0, "wave tile must be a multiple of 16x16");
  static_assert(!gemm_is_block(MODE) || (64 % WTN == 0), "a wave's columns must stay inside one scale block (64 or 128 wide)");
  constexpr int A_CHUNKS = BM * 8, B_CHUNKS = BN * 8;
  constexpr int A_PER_T = (A_CHUNKS + NT - 1) / NT, B_PER_T = (B_CHUNKS + NT - 1) / NT;
  constexpr int STAGE = (BM + BN) * 128 + (gemm_is_block(MODE) ? BM * 8 : 0);  // scales: two 64-wide groups per row
  typedef typename AccT<MODE>::type acc_t;

  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  __shared__ int s_rows[BM];  // MoE: sorted token id per tile row (>= num_valid means padding)

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WGN, wn = wave % WGN;

  // ---- tile coordinates -------------------------------------------------------------
  const int tiles_n = (g.N + BN - 1) / BN;
  const int tiles_m = MOE ? g.max_blocks_m : (g.M + BM - 1) / BM;
  int pid = xcd_remap(blockIdx.x, tiles_m * tiles_n);
  int pid_m, pid_n;
  {
    // groups of GM row-tiles share their weight columns back to back
    constexpr int GM = MOE ? 1 : 8;
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
    for (int r = tid; r < BM; r += NT) s_rows[r] = g.sorted_ids[m0 + r];
    __syncthreads();
  }

  const uint8_t* Bbase = g.B + (MOE ? (int64_t)max(expert, 0) * g.b_expert_stride : 0);
  const float* sb_base = g.sb + (MOE ? (int64_t)max(expert, 0) * g.sb_se : 0);
  // scale-block shape (block modes): KS scale groups per 128-byte K block
  const int blk_n = gx.block_n > 0 ? gx.block_n : 128;
  const int KS = (gx.block_k > 0 && gx.block_k < 128) ? 2 : 1;
  const int nks = (g.K + (128 / KS) - 1) / (128 / KS);  // scale groups along K

  // ---- per-thread global->LDS copy plan -----------------------------------------------
  const uint8_t* a_src[A_PER_T];
  int a_dst[A_PER_T];
  bool a_ok[A_PER_T];
#pragma unroll
  for (int i = 0; i < A_PER_T; i++) {
    const int c = tid + i * NT;
    const int row = c >> 3, col = c & 7;
    int64_t src_row;
    bool ok = c < A_CHUNKS;
    if (MOE) {
      const int tok = ok ? s_rows[row] : g.num_valid;
      ok = ok && tok < g.num_valid;
      src_row = ok ? tok / g.top_k : 0;
    } else {
      ok = ok && (m0 + row) < g.M;
      src_row = ok ? m0 + row : 0;
    }
    a_ok[i] = ok;
    a_src[i] = g.A + src_row * g.lda + col * 16;
    a_dst[i] = row * 128 + ((col ^ ((row >> 1) & 7)) << 4);
  }
  const uint8_t* b_src[B_PER_T];
  int b_dst[B_PER_T];
  bool b_ok[B_PER_T];
#pragma unroll
  for (int i = 0; i < B_PER_T; i++) {
    const int c = tid + i * NT;
    const int row = c >> 3, col = c & 7;
    const bool ok = c < B_CHUNKS && (n0 + row) < g.N;
    b_ok[i] = ok;
    b_src[i] = Bbase + (int64_t)(ok ? n0 + row : 0) * g.ldb + col * 16;
    b_dst[i] = BM * 128 + row * 128 + ((col ^ ((row >> 1) & 7)) << 4);
  }
  // block mode: thread t < BM also carries the activation scale of tile row t
  const float* sa_src = nullptr;
  bool sa_ok = false;
  if (gemm_is_block(MODE) && tid < BM) {
    int64_t src_row;
    if (MOE) {
      const int tok = s_rows[tid];
      sa_ok = tok < g.num_valid;
      src_row = sa_ok ? tok / g.top_k : 0;
    } else {
      sa_ok = (m0 + tid) < g.M;
      src_row = sa_ok ? m0 + tid : 0;
    }
    sa_src = g.sa + src_row * g.sa_sm;
  }

  const int nkb = (g.K + 127) >> 7;
  v4i a_reg[A_PER_T], b_reg[B_PER_T];
  float sa_reg[2] = {0.f, 0.f};

  auto gload = [&](int kb) {
    const int kbyte = kb << 7;
#pragma unroll
    for (int i = 0; i < A_PER_T; i++) {
      const int col = (tid + i * NT) & 7;
      const bool ok = a_ok[i] && (kbyte + col * 16) < g.K;
      a_reg[i] = ok ? *(const v4i*)(a_src[i] + kbyte) : v4i{0, 0, 0, 0};
    }
#pragma unroll
    for (int i = 0; i < B_PER_T; i++) {
      const int col = (tid + i * NT) & 7;
      const bool ok = b_ok[i] && (kbyte + col * 16) < g.K;
      b_reg[i] = ok ? *(const v4i*)(b_src[i] + kbyte) : v4i{0, 0, 0, 0};
    }
    if (gemm_is_block(MODE) && tid < BM) {
      sa_reg[0] = sa_ok ? sa_src[(int64_t)(kb * KS) * g.sa_sk] : 0.f;
      sa_reg[1] = (sa_ok && KS == 2 && kb * 2 + 1 < nks) ? sa_src[(int64_t)(kb * 2 + 1) * g.sa_sk] : 0.f;
    }
  };
  auto lstore = [&](int stage) {
    uint8_t* base = smem + stage * STAGE;
#pragma unroll
    for (int i = 0; i < A_PER_T; i++)
      if (A_CHUNKS % NT == 0 || tid + i * NT < A_CHUNKS) *(v4i*)(base + a_dst[i]) = a_reg[i];
#pragma unroll
    for (int i = 0; i < B_PER_T; i++)
      if (B_CHUNKS % NT == 0 || tid + i * NT < B_CHUNKS) *(v4i*)(base + b_dst[i]) = b_reg[i];
    if (gemm_is_block(MODE) && tid < BM) {
      *(float*)(base + (BM + BN) * 128 + tid * 4) = sa_reg[0];
      *(float*)(base + (BM + BN) * 128 + (BM + tid) * 4) = sa_reg[1];
    }
  };

  // ---- fragment addressing --------------------------------------------------------------
  const int frow = lane & 15, fk = lane >> 4;  // fragment row, 32-byte k slice
  acc_t acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; i++)
#pragma unroll
    for (int j = 0; j < FN; j++) acc[i][j] = acc_t{0, 0, 0, 0};

  auto frag = [&](const uint8_t* tile, int row) -> v8i {
    const uint8_t* p = tile + row * 128;
    const int sw = (row >> 1) & 7;
    v4i lo = *(const v4i*)(p + (((2 * fk) ^ sw) << 4));
    v4i hi = *(const v4i*)(p + (((2 * fk + 1) ^ sw) << 4));
    return v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  };

  // scale block column of this wave (block mode); clamped for waves entirely past N
  const int nb_wave = min(n0 + wn * WTN, g.N - 1) / blk_n;

  gload(0);
  lstore(0);
  if (nkb > 1) gload(1);
  __syncthreads();

  for (int kb = 0; kb < nkb; kb++) {
    const int cur = kb & 1;
    if (kb + 1 < nkb) lstore(cur ^ 1);
    if (kb + 2 < nkb) gload(kb + 2);

    const uint8_t* sA = smem + cur * STAGE;
    const uint8_t* sB = sA + BM * 128;
    v8i xa[FM];
#pragma unroll
    for (int i = 0; i < FM; i++) xa[i] = frag(sA, wm * WTM + i * 16 + frow);
    // One pass per scale group of the K block (one 128-wide group, or two 64-wide ones).  A lane's 32 bytes lie
    // in the 64-byte half fk / 2, so with two groups each pass multiplies with the activation fragment zeroed in
    // the lanes of the other half: the MFMA then sums exactly one group's products.
    for (int h = 0; h < (gemm_is_block(MODE) ? KS : 1); h++) {
      float sc[FM];
      v8i xh[FM];
      const bool mine = KS == 1 || (fk >> 1) == h;
#pragma unroll
      for (int i = 0; i < FM; i++)
#pragma unroll
        for (int q = 0; q < 8; q++) xh[i][q] = mine ? xa[i][q] : 0;
      if (gemm_is_block(MODE)) {
        const int ks = kb * KS + h;
        const float sbv = ks < nks ? sb_base[(int64_t)nb_wave * g.sb_sn + (int64_t)ks * g.sb_sk] : 0.f;
        const float* sS = (const float*)(sA + (BM + BN) * 128) + h * BM;
#pragma unroll
        for (int i = 0; i < FM; i++) sc[i] = sS[wm * WTM + i * 16 + frow] * sbv;
      }
#pragma unroll
      for (int j = 0; j < FN; j++) {
        const v8i wb = frag(sB, wn * WTN + j * 16 + frow);
#pragma unroll
        for (int i = 0; i < FM; i++) {
          if constexpr (MODE == GEMM_BLOCK_FP8) {
            v4f p = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wb, xh[i], v4f{0, 0, 0, 0}, 0, 0, 0, 0x7f7f7f7f, 0,
                                                                     0x7f7f7f7f);
#pragma unroll
            for (int r = 0; r < 4; r++) acc[i][j][r] = fmaf(p[r], sc[i], acc[i][j][r]);
          } else if constexpr (MODE == GEMM_ROW_FP8) {
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wb, xh[i], acc[i][j], 0, 0, 0, 0x7f7f7f7f, 0,
                                                                         0x7f7f7f7f);
          } else {
            // int8: the 32 bytes per lane are two 16-byte k slices; A and B use the same split,
            // so pairing low with low and high with high covers the 128-byte block exactly once.
            v4i wlo = {wb[0], wb[1], wb[2], wb[3]}, whi = {wb[4], wb[5], wb[6], wb[7]};
            v4i xlo = {xh[i][0], xh[i][1], xh[i][2], xh[i][3]}, xhi = {xh[i][4], xh[i][5], xh[i][6], xh[i][7]};
            if constexpr (MODE == GEMM_BLOCK_INT8) {
              // exact int32 partial product of the scale group, folded with its scales into the fp32 accumulator
              v4i p = __builtin_amdgcn_mfma_i32_16x16x64_i8(wlo, xlo, v4i{0, 0, 0, 0}, 0, 0, 0);
              p = __builtin_amdgcn_mfma_i32_16x16x64_i8(whi, xhi, p, 0, 0, 0);
#pragma unroll
              for (int r = 0; r < 4; r++) acc[i][j][r] = fmaf((float)p[r], sc[i], acc[i][j][r]);
            } else {
              acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wlo, xlo, acc[i][j], 0, 0, 0);
              acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(whi, xhi, acc[i][j], 0, 0, 0);
            }
          }
        }
      }
    }
    __syncthreads();
  }

  // ---- epilogue: lane holds C[m = .. + frow][n = .. + 4*fk .. +3] ---------------------------
  typedef typename OT::storage OS;
#pragma unroll
  for (int i = 0; i < FM; i++) {
    const int trow = wm * WTM + i * 16 + frow;
    int64_t out_row;
    bool row_ok;
    float wgt = 1.f;
    if (MOE) {
      const int tok = s_rows[trow];
      row_ok = tok < g.num_valid;
      out_row = tok;
      if (row_ok && g.mul_weight) wgt = g.topk_w[tok];
    } else {
      row_ok = (m0 + trow) < g.M;
      out_row = m0 + trow;
    }
    if (!row_ok) continue;
    float sam = 1.f;
    if (!gemm_is_block(MODE)) sam = MOE ? g.sa[(out_row / g.top_k) * gx.row_sa_stride] : g.sa[out_row];
    OS* crow = (OS*)g.C + out_row * g.ldc;
    const OS* bias = g.bias ? (const OS*)g.bias + (MOE ? (int64_t)max(expert, 0) * gx.bias_se : 0) : nullptr;
#pragma unroll
    for (int j = 0; j < FN; j++) {
      const int n = n0 + wn * WTN + j * 16 + 4 * fk;
      if (n >= g.N) continue;
      float v[4];
#pragma unroll
      for (int r = 0; r < 4; r++) {
        if constexpr (gemm_is_block(MODE)) {
          v[r] = acc[i][j][r];
          if (MOE && bias) v[r] += OT::to_f32(bias[(n + r) < g.N ? n + r : 0]);
        } else {
          const float sbn = (n + r) < g.N ? (MOE ? sb_base[(int64_t)(n + r) * gx.row_sb_stride] : g.sb[n + r]) : 0.f;
          if constexpr (MODE == GEMM_ROW_FP8) {
            v[r] = acc[i][j][r] * sbn * sam;
          } else {
            v[r] = (float)acc[i][j][r] * (sbn * sam);
          }
          if (bias) v[r] += OT::to_f32(bias[(n + r) < g.N ? n + r : 0]);
        }
        if (MOE) {
          if (expert < 0) v[r] = 0.f;
          v[r] *= wgt;
        }
      }
      if (n + 3 < g.N) {
        OS o[4] = {OT::from_f32(v[0]), OT::from_f32(v[1]), OT::from_f32(v[2]), OT::from_f32(v[3])};
        if ((((uintptr_t)(crow + n)) & 7) == 0) {
          v2i w;
          __builtin_memcpy(&w, o, 8);
          *(v2i*)(crow + n) = w;
        } else {
#pragma unroll
          for (int r = 0; r < 4; r++) crow[n + r] = o[r];
        }
      } else {
        for (int r = 0; r < 4 && n + r < g.N; r++) crow[n + r] = OT::from_f32(v[r]);
      }
    }
  }
}

template <int BM, int BN, int MODE>
constexpr int gemm8_smem_bytes() {
  return 2 * ((BM + BN) * 128 + (gemm_is_block(MODE) ? BM * 8 : 0));
}

template <int BM, int BN, int WGM, int WGN, int MODE, typename OT, bool MOE, typename GA = GemmArgs>
static int gemm8_launch(const GA& ga, hipStream_t st) {
  const GemmArgs& g = args_base(ga);
  auto kern = gemm8_kernel<BM, BN, WGM, WGN, MODE, OT, MOE, GA>;
  constexpr int smem = gemm8_smem_bytes<BM, BN, MODE>();
  if (smem > 64 * 1024) {
    static SmemAttrOnce attr;
    hipError_t e = raise_dynamic_smem(attr, (const void*)kern, smem);
    if (e != hipSuccess) return fail(SGLAMD_EHIP, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  }
  const int tiles_n = (g.N + BN - 1) / BN;
  const int tiles_m = MOE ? g.max_blocks_m : (g.M + BM - 1) / BM;
  const int64_t blocks = (int64_t)tiles_m * tiles_n;
  if (blocks <= 0) return SGLAMD_OK;
  if (blocks > 0x7fffffff) return fail(SGLAMD_EINVAL, "gemm: grid too large");
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(64 * WGM * WGN), smem, st, ga);
  return check_launch("gemm8");
}

}  // namespace sglamd
