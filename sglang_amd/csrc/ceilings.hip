// Loops that measure what this GPU gives a kernel at best: the matrix pipe with nothing else running, HBM
// through plain wide loads, and the large-tile GEMM's own loop on an L2-resident working set.  The roofline fractions of the real kernels are read against these as well as
// against the published peaks; they are launched from the benchmark only.
#include "gemm_big_persist.h"

namespace sglamd {

__device__ __forceinline__ uint32_t mix32(uint32_t x) {
  x ^= x >> 16;
  x *= 0x7feb352dU;
  x ^= x >> 15;
  x *= 0x846ca68bU;
  x ^= x >> 16;
  return x;
}

// 8 waves per workgroup (2 per SIMD), each with 4 x 2 accumulator tiles of 32x32 like the GEMM kernels; operands
// stay in registers.  RANDOM: operand bytes are hashed (finite e4m3 / any int8), else one constant byte: the
// chip clocks its matrix pipes by how many operand bits toggle.
template <bool INT8, bool RANDOM>
__global__ __launch_bounds__(512) void mfma_loop_kernel(float* out, int iters) {
  const uint32_t tid = threadIdx.x + blockIdx.x * 512;
  v8i a[4], b[2];
#pragma unroll
  for (int i = 0; i < 6; i++)
#pragma unroll
    for (int j = 0; j < 8; j++) {
      uint32_t h = RANDOM ? mix32(tid * 64 + i * 8 + j) : 0x38383838u;
      if (!INT8) h &= 0xbfbfbfbfu;  // exponent field below 8: no e4m3 NaN, magnitudes below 2
      (i < 4 ? a[i] : b[i - 4])[j] = (int)h;
    }
  float s = 0.f;
  if constexpr (INT8) {
    v16i acc[8];
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][r] = 0;
    for (int it = 0; it < iters; it++) {
      // int32 sums wrap, which costs nothing; the two halves of a tile are eight instructions apart
#pragma unroll
      for (int half = 0; half < 2; half++)
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
          for (int j = 0; j < 2; j++) {
            const v4i ax = {a[i][4 * half], a[i][4 * half + 1], a[i][4 * half + 2], a[i][4 * half + 3]};
            const v4i bx = {b[j][4 * half], b[j][4 * half + 1], b[j][4 * half + 2], b[j][4 * half + 3]};
            acc[i * 2 + j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ax, bx, acc[i * 2 + j], 0, 0, 0);
          }
    }
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
      for (int r = 0; r < 16; r++) s += (float)acc[i][r];
  } else {
    v16f acc[8];
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][r] = 0.f;
    for (int it = 0; it < iters; it++) {
      // eight independent accumulation chains; operands below 2 in magnitude, so the sums stay far from overflow
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
          acc[i * 2 + j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[i], b[j], acc[i * 2 + j], 0, 0, 0, 0x7f7f7f7f,
                                                                           0, 0x7f7f7f7f);
    }
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
      for (int r = 0; r < 16; r++) s += acc[i][r];
  }
  out[tid] = s;
}

// Every workgroup owns one contiguous share of the buffer; a wave takes 8 consecutive 1 KB pieces of it per step
// (16 bytes per lane and load, 8 loads in flight), the four waves interleaved.  Contiguous shares measured
// 6.9-7.0 TB/s where a grid-stride walk (each load of a thread a whole grid apart) reaches 5.5-6.1.
// The xor keeps the loads alive.
__global__ __launch_bounds__(256) void hbm_read_kernel(const v4i* __restrict__ src, int64_t n16, int* sink) {
  constexpr int UNR = 8;
  v4i acc = {0, 0, 0, 0};
  const int64_t per_wg = (n16 + gridDim.x - 1) / gridDim.x;
  const int64_t begin = (int64_t)blockIdx.x * per_wg, end = begin + per_wg < n16 ? begin + per_wg : n16;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  int64_t p = begin + (int64_t)wave * 64 * UNR;
  for (; p + 64 * UNR <= end; p += 4 * 64 * UNR) {
    v4i x[UNR];
#pragma unroll
    for (int u = 0; u < UNR; u++) x[u] = __builtin_nontemporal_load(src + p + u * 64 + lane);
#pragma unroll
    for (int u = 0; u < UNR; u++) acc ^= x[u];
  }
  for (int64_t i = p + lane; i < end && p < end; i += 64) acc ^= __builtin_nontemporal_load(src + i);  // ragged tail
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x5ca1ab1e) *sink = 1;  // practically never: the store only has to exist
}

// The same read through the path the streaming GEMMs use: one workgroup per CU, eight waves, every wave keeps
// DEPTH direct-to-LDS loads of 1 KB in flight (buffer_load_dwordx4 ... lds, non-temporal) over its contiguous share
// and never looks at what lands.  Nothing is computed and nothing leaves, so no kernel that streams its operands
// this way can be faster than this on the same bytes.
template <int DEPTH>
__global__ __launch_bounds__(512) void hbm_read_lds_kernel(const uint8_t* __restrict__ src, int64_t bytes) {
#if defined(__HIP_DEVICE_COMPILE__)
  extern __shared__ __attribute__((aligned(1024))) uint8_t ring[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t pieces = bytes >> 10;  // whole 1 KB pieces; a ragged tail below 1 KB is not read
  const int64_t waves = (int64_t)gridDim.x * 8;
  const int64_t w = (int64_t)blockIdx.x * 8 + wave;
  const int64_t begin = pieces * w / waves, end = pieces * (w + 1) / waves;
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)ring + wave * (DEPTH * 1024);
  auto issue = [&](int64_t piece, int slot) {
    const uint8_t* base = src + (piece << 10);
    const v4i rs = {(int)(uint32_t)(uintptr_t)base, (int)(((uint64_t)(uintptr_t)base >> 32) & 0xffff), 1024, 0x00020000};
    asm volatile("s_nop 4\n\tbuffer_load_dwordx4 %0, %1, 0 offen nt lds"
                 :
                 : "v"((uint32_t)(lane * 16)), "s"(rs), "{m0}"(lds0 + slot * 1024)
                 : "memory");
  };
  int64_t p = begin;
#pragma unroll
  for (int s = 0; s < DEPTH; s++)
    if (p + s < end) issue(p + s, s);
  for (p = begin + DEPTH; p + DEPTH <= end; p += DEPTH) {
#pragma unroll
    for (int s = 0; s < DEPTH; s++) {
      asm volatile("s_waitcnt vmcnt(%0)" : : "n"(DEPTH - 1) : "memory");  // slot s has landed
      issue(p + s, s);
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
  for (int s = 0; p + s < end; s++) issue(p + s, s);
  asm volatile("s_waitcnt vmcnt(0)" : : : "memory");  // nothing may be in flight when the workgroup ends
#endif
}

// What the path from L2 into a CU gives: every workgroup (one per CU, eight waves) reads its own 64 KB share of a
// buffer small enough to stay in L2, `passes` times over.  LDS: direct-to-LDS loads of 1 KB, eight in flight per
// wave, as the tile kernels issue them; else the same bytes through 16-byte register loads, eight in flight per
// wave.  The rate a tile kernel can take operands in at is bounded by the first, whatever HBM delivers.
template <bool LDS>
__global__ __launch_bounds__(512) void l2_read_kernel(const uint8_t* __restrict__ src, int passes, int* sink) {
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr int DEPTH = 8;
  extern __shared__ __attribute__((aligned(1024))) uint8_t ring[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint8_t* mine = src + ((int64_t)blockIdx.x * 8 + wave) * (DEPTH * 1024);  // this wave's 8 KB
  const v4i rs = {(int)(uint32_t)(uintptr_t)mine, (int)(((uint64_t)(uintptr_t)mine >> 32) & 0xffff), DEPTH * 1024,
                  0x00020000};
  if constexpr (LDS) {
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)ring + wave * (DEPTH * 1024);
    auto issue = [&](int s) {
      asm volatile("s_nop 4\n\tbuffer_load_dwordx4 %0, %1, 0 offen lds"
                   :
                   : "v"((uint32_t)(s * 1024 + lane * 16)), "s"(rs), "{m0}"(lds0 + s * 1024)
                   : "memory");
    };
#pragma unroll
    for (int s = 0; s < DEPTH; s++) issue(s);
    for (int p = 1; p < passes; p++) {
#pragma unroll
      for (int s = 0; s < DEPTH; s++) {
        asm volatile("s_waitcnt vmcnt(%0)" : : "n"(DEPTH - 1) : "memory");  // slot s has landed
        issue(s);
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" : : : "memory");  // nothing may be in flight when the workgroup ends
  } else {
    v4i x[DEPTH], acc = {0, 0, 0, 0};
    auto issue = [&](int s) {
      asm volatile("s_nop 4\n\tbuffer_load_dwordx4 %0, %1, %2, 0 offen" : "=v"(x[s]) : "v"((uint32_t)(s * 1024 + lane * 16)), "s"(rs) : "memory");
    };
#pragma unroll
    for (int s = 0; s < DEPTH; s++) issue(s);
    for (int p = 1; p < passes; p++) {
#pragma unroll
      for (int s = 0; s < DEPTH; s++) {
        asm volatile("s_waitcnt vmcnt(%1)" : "+v"(x[s]) : "n"(DEPTH - 1) : "memory");
        acc ^= x[s];
        issue(s);
      }
    }
#pragma unroll
    for (int s = 0; s < DEPTH; s++) {
      asm volatile("s_waitcnt vmcnt(0)" : "+v"(x[s]) : : "memory");
      acc ^= x[s];
    }
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x5ca1ab1e) *sink = 1;  // practically never: keeps the loads alive
  }
#endif
}

__global__ __launch_bounds__(256) void hbm_copy_kernel(v4i* __restrict__ dst, const v4i* __restrict__ src, int64_t n16) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += stride)
    __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

}  // namespace sglamd

using namespace sglamd;

extern "C" int sglamd_ceiling_mfma(int int8, int random_operands, int iters, float* out, void* stream) {
  SGLAMD_REQUIRE(out && iters > 0, SGLAMD_EINVAL, "ceiling_mfma: out must hold 256*512 floats, iters > 0");
  hipStream_t st = (hipStream_t)stream;
  if (int8) {
    if (random_operands) hipLaunchKernelGGL((mfma_loop_kernel<true, true>), dim3(256), dim3(512), 0, st, out, iters);
    else hipLaunchKernelGGL((mfma_loop_kernel<true, false>), dim3(256), dim3(512), 0, st, out, iters);
  } else {
    if (random_operands) hipLaunchKernelGGL((mfma_loop_kernel<false, true>), dim3(256), dim3(512), 0, st, out, iters);
    else hipLaunchKernelGGL((mfma_loop_kernel<false, false>), dim3(256), dim3(512), 0, st, out, iters);
  }
  return check_launch("ceiling_mfma");
}

extern "C" int sglamd_ceiling_hbm(void* dst, const void* src, int64_t bytes, int* sink, void* stream) {
  SGLAMD_REQUIRE(src && sink && bytes >= 16 && (bytes & 15) == 0 && (((uintptr_t)src | (uintptr_t)dst) & 15) == 0,
                 SGLAMD_EINVAL, "ceiling_hbm: 16-byte aligned buffers of a multiple of 16 bytes, and a sink word");
  hipStream_t st = (hipStream_t)stream;
  if (dst) hipLaunchKernelGGL(hbm_copy_kernel, dim3(256 * 16), dim3(256), 0, st, (v4i*)dst, (const v4i*)src, bytes >> 4);
  else hipLaunchKernelGGL(hbm_read_kernel, dim3(256 * 8), dim3(256), 0, st, (const v4i*)src, bytes >> 4, sink);
  return check_launch("ceiling_hbm");
}

// The persistent 256x256 block-FP8 kernel exactly as the operator launches it (same instantiation but for L2RES),
// except that every tile reads the operand panels of tile (0, 0): what that loop reaches when no load leaves L2.
extern "C" int sglamd_ceiling_gemm_l2_resident(const void* a, const void* b, const float* sa, const float* sb, void* out,
                                               int64_t M, int64_t N, int64_t K, void* stream) {
  SGLAMD_REQUIRE(a && b && sa && sb && out, SGLAMD_EINVAL, "ceiling_gemm_l2_resident: null pointer");
  SGLAMD_REQUIRE(M > 0 && N > 0 && K > 0 && M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31), SGLAMD_EINVAL,
                 "ceiling_gemm_l2_resident: bad sizes");
  GemmArgs g = {};
  g.A = (const uint8_t*)a;  // [256, K] e4m3 bytes
  g.lda = K;
  g.B = (const uint8_t*)b;  // [256, K]
  g.ldb = K;
  g.sa = sa;  // [K/128][256]: one scale per row and K block, rows contiguous
  g.sa_sm = 1;
  g.sa_sk = 256;
  g.sb = sb;  // [2][K/128]
  g.sb_sn = K >> 7;
  g.sb_sk = 1;
  g.C = out;  // [M, N] bf16
  g.ldc = N;
  g.M = (int)M;
  g.N = (int)N;
  g.K = (int)K;
  const int wgs = device_cus();
  SGLAMD_REQUIRE((wgs & 7) == 0 && gemm8_big_persist_ok(g, wgs), SGLAMD_EINVAL,
                 "ceiling_gemm_l2_resident: needs more 256x256 tiles than CUs, K/128 even in 4..256, N %% 8 == 0");
  return gemm8_big_persist_launch<GEMM_BLOCK_FP8, BF16, false, true>(g, (hipStream_t)stream, wgs);
}

// The read ceiling of the streaming kernels: `bytes` of src through direct-to-LDS loads, one workgroup per CU.
extern "C" int sglamd_ceiling_hbm_lds(const void* src, int64_t bytes, void* stream) {
  SGLAMD_REQUIRE(src && bytes >= 1024 && (((uintptr_t)src) & 15) == 0, SGLAMD_EINVAL,
                 "ceiling_hbm_lds: a 16-byte aligned buffer of at least 1 KB");
  constexpr int DEPTH = 16;
  auto kern = hbm_read_lds_kernel<DEPTH>;
  constexpr int smem = 8 * DEPTH * 1024;
  static SmemAttrOnce attr;
  hipError_t e = raise_dynamic_smem(attr, (const void*)kern, smem);
  if (e != hipSuccess) return fail(SGLAMD_EHIP, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  hipLaunchKernelGGL(kern, dim3((unsigned)device_cus()), dim3(512), smem, (hipStream_t)stream, (const uint8_t*)src, bytes);
  return check_launch("ceiling_hbm_lds");
}


// L2 -> CU: every CU re-reads its own 64 KB of src (device_cus() x 64 KB in all, L2 resident) `passes` times,
// through direct-to-LDS loads (lds != 0) or register loads.  Bytes moved: passes x device_cus() x 65536.
extern "C" int sglamd_ceiling_l2_read(const void* src, int64_t bytes, int passes, int lds, int* sink, void* stream) {
  const int wgs = device_cus();
  SGLAMD_REQUIRE(src && sink && passes > 0 && (((uintptr_t)src) & 15) == 0 && bytes >= (int64_t)wgs * 65536, SGLAMD_EINVAL,
                 "ceiling_l2_read: a 16-byte aligned buffer of at least 64 KB per CU, a sink word, passes > 0");
  hipStream_t st = (hipStream_t)stream;
  if (lds) {
    auto kern = l2_read_kernel<true>;
    static SmemAttrOnce attr;
    hipError_t e = raise_dynamic_smem(attr, (const void*)kern, 65536);
    if (e != hipSuccess) return fail(SGLAMD_EHIP, "hipFuncSetAttribute: %s", hipGetErrorString(e));
    hipLaunchKernelGGL(kern, dim3((unsigned)wgs), dim3(512), 65536, st, (const uint8_t*)src, passes, sink);
  } else {
    hipLaunchKernelGGL(l2_read_kernel<false>, dim3((unsigned)wgs), dim3(512), 0, st, (const uint8_t*)src, passes, sink);
  }
  return check_launch("ceiling_l2_read");
}

