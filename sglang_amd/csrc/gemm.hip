// Dense 8-bit GEMM entry points: block-scaled FP8 and INT8, per-token/per-channel FP8 and INT8.  The kernels are
// instantiated in gemm_mode_*.hip (one scaling mode each); this file validates arguments and hands over.
#include "gemm_dispatch.h"

namespace sglamd {

thread_local int last_kernel = 0;
thread_local int skinny_last_shape = 0;

extern template int dispatch_out<GEMM_BLOCK_FP8>(const GemmArgs&, int, hipStream_t, void*, int64_t);
extern template int dispatch_out<GEMM_ROW_FP8>(const GemmArgs&, int, hipStream_t, void*, int64_t);
extern template int dispatch_out<GEMM_ROW_INT8>(const GemmArgs&, int, hipStream_t, void*, int64_t);
extern template int dispatch_out<GEMM_BLOCK_INT8>(const GemmArgs&, int, hipStream_t, void*, int64_t);

static int check_common(const char* op, const void* a, const void* b, const void* c, int64_t M, int64_t N, int64_t K,
                        int64_t lda, int64_t ldb, int64_t ldc) {
  SGLAMD_REQUIRE(a && b && c, SGLAMD_EINVAL, "%s: null pointer", op);
  SGLAMD_REQUIRE(M >= 0 && N > 0 && K > 0, SGLAMD_EINVAL, "%s: bad sizes M=%lld N=%lld K=%lld", op, (long long)M,
                 (long long)N, (long long)K);
  SGLAMD_REQUIRE(M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31), SGLAMD_EINVAL, "%s: size exceeds int32", op);
  SGLAMD_REQUIRE(K % 16 == 0, SGLAMD_EINVAL, "%s: K (%lld) must be a multiple of 16 bytes", op, (long long)K);
  SGLAMD_REQUIRE(lda >= K && ldb >= K && ldc >= N, SGLAMD_EINVAL, "%s: leading dimension smaller than the row", op);
  SGLAMD_REQUIRE(lda % 16 == 0 && ldb % 16 == 0, SGLAMD_EINVAL, "%s: row strides must be multiples of 16 bytes", op);
  SGLAMD_REQUIRE(((uintptr_t)a % 16) == 0 && ((uintptr_t)b % 16) == 0, SGLAMD_EINVAL,
                 "%s: operands must be 16-byte aligned", op);
  return SGLAMD_OK;
}

}  // namespace sglamd

using namespace sglamd;

static int blockwise(int mode, const char* op, const void* a, int64_t lda, const void* b, int64_t ldb, const float* sa,
                     int64_t sa_stride_m, int64_t sa_stride_k, const float* sb, int64_t sb_stride_n,
                     int64_t sb_stride_k, void* out, int64_t ldc, int out_dtype, int64_t M, int64_t N, int64_t K,
                     void* workspace, int64_t workspace_bytes, void* stream, bool scales_pow2 = false) {
  int rc = check_common(op, a, b, out, M, N, K, lda, ldb, ldc);
  if (rc) return rc;
  SGLAMD_REQUIRE(sa && sb, SGLAMD_EINVAL, "%s: null scale pointer", op);
  if (M == 0) return SGLAMD_OK;
  GemmArgs g = {};
  g.scales_pow2 = scales_pow2;
  g.A = (const uint8_t*)a;
  g.lda = lda;
  g.B = (const uint8_t*)b;
  g.ldb = ldb;
  g.sa = sa;
  g.sa_sm = sa_stride_m;
  g.sa_sk = sa_stride_k;
  g.sb = sb;
  g.sb_sn = sb_stride_n;
  g.sb_sk = sb_stride_k;
  g.C = out;
  g.ldc = ldc;
  g.M = (int)M;
  g.N = (int)N;
  g.K = (int)K;
  if (mode == GEMM_BLOCK_FP8)
    return dispatch_out<GEMM_BLOCK_FP8>(g, out_dtype, (hipStream_t)stream, workspace, workspace_bytes);
  return dispatch_out<GEMM_BLOCK_INT8>(g, out_dtype, (hipStream_t)stream, workspace, workspace_bytes);
}

extern "C" int sglamd_fp8_blockwise_scaled_mm(const void* a, int64_t lda, const void* b, int64_t ldb, const float* sa,
                                              int64_t sa_stride_m, int64_t sa_stride_k, const float* sb,
                                              int64_t sb_stride_n, int64_t sb_stride_k, void* out, int64_t ldc,
                                              int out_dtype, int64_t M, int64_t N, int64_t K, void* workspace,
                                              int64_t workspace_bytes, void* stream) {
  return blockwise(GEMM_BLOCK_FP8, "fp8_blockwise_scaled_mm", a, lda, b, ldb, sa, sa_stride_m, sa_stride_k, sb,
                   sb_stride_n, sb_stride_k, out, ldc, out_dtype, M, N, K, workspace, workspace_bytes, stream);
}

extern "C" int sglamd_fp8_blockwise_scaled_mm_pow2(const void* a, int64_t lda, const void* b, int64_t ldb,
                                                   const float* sa, int64_t sa_stride_m, int64_t sa_stride_k,
                                                   const float* sb, int64_t sb_stride_n, int64_t sb_stride_k, void* out,
                                                   int64_t ldc, int out_dtype, int64_t M, int64_t N, int64_t K,
                                                   void* workspace, int64_t workspace_bytes, void* stream) {
  return blockwise(GEMM_BLOCK_FP8, "fp8_blockwise_scaled_mm_pow2", a, lda, b, ldb, sa, sa_stride_m, sa_stride_k, sb,
                   sb_stride_n, sb_stride_k, out, ldc, out_dtype, M, N, K, workspace, workspace_bytes, stream, true);
}

extern "C" int sglamd_int8_blockwise_scaled_mm(const void* a, int64_t lda, const void* b, int64_t ldb, const float* sa,
                                               int64_t sa_stride_m, int64_t sa_stride_k, const float* sb,
                                               int64_t sb_stride_n, int64_t sb_stride_k, void* out, int64_t ldc,
                                               int out_dtype, int64_t M, int64_t N, int64_t K, void* workspace,
                                               int64_t workspace_bytes, void* stream) {
  return blockwise(GEMM_BLOCK_INT8, "int8_blockwise_scaled_mm", a, lda, b, ldb, sa, sa_stride_m, sa_stride_k, sb,
                   sb_stride_n, sb_stride_k, out, ldc, out_dtype, M, N, K, workspace, workspace_bytes, stream);
}

static int rowwise(int mode, const char* op, const void* a, int64_t lda, const void* b, int64_t ldb, const float* sa,
                   const float* sb, const void* bias, void* out, int64_t ldc, int out_dtype, int64_t M, int64_t N,
                   int64_t K, void* workspace, int64_t workspace_bytes, void* stream) {
  int rc = check_common(op, a, b, out, M, N, K, lda, ldb, ldc);
  if (rc) return rc;
  SGLAMD_REQUIRE(sa && sb, SGLAMD_EINVAL, "%s: null scale pointer", op);
  if (M == 0) return SGLAMD_OK;
  GemmArgs g = {};
  g.A = (const uint8_t*)a;
  g.lda = lda;
  g.B = (const uint8_t*)b;
  g.ldb = ldb;
  g.sa = sa;
  g.sb = sb;
  g.bias = bias;
  g.C = out;
  g.ldc = ldc;
  g.M = (int)M;
  g.N = (int)N;
  g.K = (int)K;
  if (mode == GEMM_ROW_FP8) return dispatch_out<GEMM_ROW_FP8>(g, out_dtype, (hipStream_t)stream, workspace, workspace_bytes);
  return dispatch_out<GEMM_ROW_INT8>(g, out_dtype, (hipStream_t)stream, workspace, workspace_bytes);
}

extern "C" int sglamd_fp8_scaled_mm(const void* a, int64_t lda, const void* b, int64_t ldb, const float* sa,
                                    const float* sb, const void* bias, void* out, int64_t ldc, int out_dtype,
                                    int64_t M, int64_t N, int64_t K, void* workspace, int64_t workspace_bytes,
                                    void* stream) {
  return rowwise(GEMM_ROW_FP8, "fp8_scaled_mm", a, lda, b, ldb, sa, sb, bias, out, ldc, out_dtype, M, N, K, workspace,
                 workspace_bytes, stream);
}

extern "C" int sglamd_int8_scaled_mm(const void* a, int64_t lda, const void* b, int64_t ldb, const float* sa,
                                     const float* sb, const void* bias, void* out, int64_t ldc, int out_dtype,
                                     int64_t M, int64_t N, int64_t K, void* workspace, int64_t workspace_bytes,
                                     void* stream) {
  return rowwise(GEMM_ROW_INT8, "int8_scaled_mm", a, lda, b, ldb, sa, sb, bias, out, ldc, out_dtype, M, N, K, workspace,
                 workspace_bytes, stream);
}

extern "C" int sglamd_last_gemm_kernel(void) { return last_kernel; }
extern "C" int sglamd_last_streaming_shape(void) { return skinny_last_shape; }

extern "C" int sglamd_streaming_piece_offset(int kb, int lchunk, int64_t K, int64_t* offset) {
  const SkinnyPiece pc = skinny_piece(kb, lchunk, (int)K);
  if (offset) *offset = pc.offset;
  return pc.dead ? 1 : 0;
}

// Bytes of fp32 scratch with which the GEMM entry points above can split K for this shape (0: no use for it).
extern "C" int64_t sglamd_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  if (M >= (1ll << 31) || N <= 0 || K <= 0 || (K % 128) != 0) return 0;
  if (M <= 64 && !small_m_uses_tile(M, N, K)) return 0;
  const BigConfig cfg = gemm8_big_config(M, N, K);
  int64_t need = cfg.slices > 1 ? (int64_t)cfg.slices * M * N * 4 : 0;
  // a launch of 256-row tiles cut in two along N (column_split) splits K on its second part; whether the launch
  // uses 256-row tiles depends on the operand mode, so the larger of the two needs is reported
  const int64_t n1 = M > 64 ? column_split(M, N, K) : 0;
  if (n1 > 0) {
    const int64_t rest = (int64_t)gemm8_big_config(M, N - n1, K).slices * M * (N - n1) * 4;
    if (rest > need) need = rest;
  }
  return need;
}
