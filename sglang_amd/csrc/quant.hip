// Activation quantisation kernels for gfx950: per-token-group FP8/INT8 (two arithmetic
// forms), per-token FP8 and per-token INT8.  All are HBM-streaming kernels: every lane
// moves 32 input bytes with two 16-byte loads, group maxima are reduced across the few
// lanes that share a group with wave64 cross-lane moves, and bytes leave as 16-byte
// (or 8-byte) stores.
#include <stdarg.h>
#include <stdio.h>

#include "quant_core.h"

namespace sglamd {

static thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(SGLAMD_EHIP, "%s: %s", what, hipGetErrorString(e));
  return SGLAMD_OK;
}

template <typename T, int GROUP>
__global__ __launch_bounds__(256) void group_quant_kernel(GroupQuantArgs a) {
  group_quant_body<T, GROUP>(a, (int64_t)blockIdx.x * 256 + threadIdx.x);
}

// Any group size (the divide-form operator accepts every divisor of the element count):
// one wavefront per group, scalar element loop.
template <typename T>
__global__ __launch_bounds__(256) void group_quant_generic_kernel(GroupQuantArgs a, int group) {
  typedef typename T::storage S;
  const int lane = threadIdx.x & 63;
  const int64_t g = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (g >= a.num_groups) return;
  const S* src = (const S*)a.in + g * group;
  float amax = a.eps;
  for (int i = lane; i < group; i += 64) amax = fmaxf(amax, fabsf(T::to_f32(src[i])));
  amax = group_max<64>(amax);
  const bool ue8m0 = a.layout == SGLAMD_SCALE_COL_MAJOR_UE8M0;
  float s_store, mul = 0.f;
  if (a.form == SGLAMD_QUANT_FORM_DIVIDE) {
    s_store = amax / a.max8;
    if (ue8m0) s_store = pow2_int(log2_ceil_bits(fmaxf(s_store, 1e-10f)));
  } else if (ue8m0) {
    int e = log2_ceil_bits(amax * (1.0f / a.max8));
    mul = pow2_int(-e);
    s_store = pow2_int(e);
  } else {
    s_store = amax * (1.0f / a.max8);
    mul = a.max8 / amax;
  }
  uint8_t* dst = (uint8_t*)a.q + g * group;
  for (int i = lane; i < group; i += 64) {
    float xv = T::to_f32(src[i]);
    float yv = (a.form == SGLAMD_QUANT_FORM_DIVIDE) ? xv / s_store : xv * mul;
    yv = clampf(yv, a.min8, a.max8);
    dst[i] = a.q_is_fp8 ? (uint8_t)(pack2_e4m3(yv, 0.f) & 0xff) : (uint8_t)(int)yv;
  }
  if (lane == 0) {
    const int64_t row = g / a.groups_per_row;
    const int col = (int)(g % a.groups_per_row);
    if (a.layout == SGLAMD_SCALE_ROW_MAJOR) {
      ((float*)a.s)[g] = s_store;
    } else if (a.layout == SGLAMD_SCALE_COL_MAJOR) {
      ((float*)a.s)[(int64_t)col * a.scale_stride + row] = s_store;
    } else {
      uint8_t* sp = (uint8_t*)a.s + (((int64_t)(col >> 2) * a.scale_stride + row) << 2);
      sp[col & 3] = (uint8_t)(__float_as_uint(s_store) >> 23);
      if (col == a.groups_per_row - 1) {
        for (int k = (col & 3) + 1; k < 4; k++) sp[k] = 0;
      }
    }
  }
}

template <typename T>
static int launch_group_quant(const GroupQuantArgs& a, int group, hipStream_t st) {
  constexpr int ELEMS = 32 / (int)sizeof(typename T::storage);
  auto blocks_for = [&](int lpg) { return (unsigned)ceil_div(a.num_groups * lpg, 256); };
  switch (group) {
    case 128:
      hipLaunchKernelGGL((group_quant_kernel<T, 128>), dim3(blocks_for(128 / ELEMS)), dim3(256), 0, st, a);
      break;
    case 64:
      hipLaunchKernelGGL((group_quant_kernel<T, 64>), dim3(blocks_for(64 / ELEMS)), dim3(256), 0, st, a);
      break;
    case 32:
      hipLaunchKernelGGL((group_quant_kernel<T, 32>), dim3(blocks_for(32 / ELEMS)), dim3(256), 0, st, a);
      break;
    case 16:
      hipLaunchKernelGGL((group_quant_kernel<T, 16>), dim3(blocks_for(16 / ELEMS)), dim3(256), 0, st, a);
      break;
    default:
      hipLaunchKernelGGL((group_quant_generic_kernel<T>), dim3((unsigned)ceil_div(a.num_groups, 4)), dim3(256), 0,
                         st, a, group);
  }
  return check_launch("per_token_group_quant_8bit");
}

// ---------------------------------------------------------------------------------------
// Per-token kernels: one 256-lane workgroup per row; the row is read twice (the second
// read is served by L2), maxima meet through LDS.
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ float block_max_256(float v, float* red) {
  v = group_max<64>(v);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
}

// V = elements per vector access (8, 4 or 1); rows must start V-element aligned.
template <typename T, bool INT8, int V>
__global__ __launch_bounds__(256) void per_token_quant_kernel(const void* in_, uint8_t* q, float* s, int64_t hidden) {
  typedef typename T::storage S;
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const S* src = (const S*)in_ + row * hidden;
  uint8_t* dst = q + row * hidden;
  const int64_t nvec = hidden / V;

  auto load_vec = [&](int64_t i, float* out) {
    S buf[V];
    if constexpr (V * sizeof(S) == 32) {
      v4i r0 = *((const v4i*)src + 2 * i), r1 = *((const v4i*)src + 2 * i + 1);
      __builtin_memcpy(&buf[0], &r0, 16);
      __builtin_memcpy(&buf[V / 2], &r1, 16);
    } else if constexpr (V * sizeof(S) == 16) {
      v4i r = *((const v4i*)src + i);
      __builtin_memcpy(buf, &r, 16);
    } else if constexpr (V * sizeof(S) == 8) {
      v2i r = *((const v2i*)src + i);
      __builtin_memcpy(buf, &r, 8);
    } else {
      buf[0] = src[i];
    }
#pragma unroll
    for (int j = 0; j < V; j++) out[j] = T::to_f32(buf[j]);
  };

  float amax = 0.f;
  for (int64_t i = threadIdx.x; i < nvec; i += 256) {
    float x[V];
    load_vec(i, x);
#pragma unroll
    for (int j = 0; j < V; j++) amax = fmaxf(amax, fabsf(x[j]));
  }
  amax = block_max_256(amax, red);

  float scale, mul;
  if (INT8) {
    amax = fmaxf(amax, 1e-10f);
    scale = amax / 127.0f;
    mul = 127.0f / amax;
  } else {
    scale = amax / 448.0f;
    mul = (scale == 0.f) ? 0.f : 1.0f / scale;
  }
  if (threadIdx.x == 0) s[row] = scale;

  for (int64_t i = threadIdx.x; i < nvec; i += 256) {
    float x[V];
    load_vec(i, x);
    uint8_t o[V];
    if constexpr (INT8) {
#pragma unroll
      for (int j = 0; j < V; j++) o[j] = (uint8_t)(int)roundf(x[j] * mul);
    } else if constexpr (V >= 4) {
#pragma unroll
      for (int j = 0; j < V; j += 4) {
        uint32_t w = pack4_e4m3(clampf(x[j] * mul, -448.f, 448.f), clampf(x[j + 1] * mul, -448.f, 448.f),
                                clampf(x[j + 2] * mul, -448.f, 448.f), clampf(x[j + 3] * mul, -448.f, 448.f));
        __builtin_memcpy(&o[j], &w, 4);
      }
    } else {
      o[0] = (uint8_t)(pack2_e4m3(clampf(x[0] * mul, -448.f, 448.f), 0.f) & 0xff);
    }
    if constexpr (V == 8) {
      v2i w;
      __builtin_memcpy(&w, o, 8);
      *((v2i*)dst + i) = w;
    } else if constexpr (V == 4) {
      int w;
      __builtin_memcpy(&w, o, 4);
      *((int*)dst + i) = w;
    } else {
      dst[i] = o[0];
    }
  }
}

template <typename T, bool INT8>
static void launch_per_token_t(const void* in, void* q, float* s, int64_t rows, int64_t hidden, hipStream_t st) {
  dim3 grid((unsigned)rows), block(256);
  if (hidden % 8 == 0)
    hipLaunchKernelGGL((per_token_quant_kernel<T, INT8, 8>), grid, block, 0, st, in, (uint8_t*)q, s, hidden);
  else if (hidden % 4 == 0)
    hipLaunchKernelGGL((per_token_quant_kernel<T, INT8, 4>), grid, block, 0, st, in, (uint8_t*)q, s, hidden);
  else
    hipLaunchKernelGGL((per_token_quant_kernel<T, INT8, 1>), grid, block, 0, st, in, (uint8_t*)q, s, hidden);
}

template <bool INT8>
static int launch_per_token(const void* in, int in_dtype, void* q, float* s, int64_t rows, int64_t hidden,
                            hipStream_t st) {
  switch (in_dtype) {
    case SGLAMD_BF16:
      launch_per_token_t<BF16, INT8>(in, q, s, rows, hidden, st);
      break;
    case SGLAMD_F16:
      launch_per_token_t<F16, INT8>(in, q, s, rows, hidden, st);
      break;
    case SGLAMD_F32:
      launch_per_token_t<F32, INT8>(in, q, s, rows, hidden, st);
      break;
    default:
      return fail(SGLAMD_EINVAL, "per_token_quant: input dtype must be F32, F16 or BF16");
  }
  return check_launch("per_token_quant");
}

// ---------------------------------------------------------------------------------------
// Fused (residual add +) RMSNorm + per-token-group FP8 quantisation, optionally with a second, plain
// RMSNorm of another tensor in the same launch.  One workgroup per row; a lane keeps its 8-element
// pieces of the row in registers between the sum of squares and the normalisation, so the row is read
// once.  A 128-element quant group is 16 neighbouring lanes: its maximum is four shuffles.
//   v = f32(x) + f32(res);  y = v * rsqrt(mean(v^2) + eps) * w;  amax = max(max|y|, 1e-10);
//   scale = amax / 448;  q = e4m3(clamp(y * (1 / scale)));  all in fp32, y is not rounded before quantising.
// ---------------------------------------------------------------------------------------
struct RmsQuantArgs {
  const void* x1;
  int64_t x1_stride;  // elements between rows
  const void* w1;
  const void* res1;      // optional, [M, N1] contiguous
  void* res_out;         // optional, [M, N1]: x1 + res1 in the storage dtype
  uint8_t* q;            // [M, N1] e4m3fn
  float* s;              // [M, ceil(N1 / 128)]
  void* y1;              // optional, [M, N1]: the normalised row in the storage dtype
  const void* x2;        // optional second tensor, rows of N2
  int64_t x2_stride;
  const void* w2;
  void* y2;              // [M, N2]
  int n1, n2;
  float eps1, eps2;
};

__device__ __forceinline__ float block_sum_256(float v, float* red) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
  __syncthreads();  // red may still be read by the previous use
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return (red[0] + red[1]) + (red[2] + red[3]);
}

template <typename T>
__device__ __forceinline__ void load8(const typename T::storage* p, float* out) {
  v4i r = *(const v4i*)p;
  u16 b[8];
  __builtin_memcpy(b, &r, 16);
#pragma unroll
  for (int j = 0; j < 8; j++) out[j] = T::to_f32(b[j]);
}
template <>
__device__ __forceinline__ void load8<F32>(const float* p, float* out) {
  const v4f a = *(const v4f*)p, b = *(const v4f*)(p + 4);
#pragma unroll
  for (int j = 0; j < 4; j++) {
    out[j] = a[j];
    out[4 + j] = b[j];
  }
}
template <typename T>
__device__ __forceinline__ void store8(u16* p, const float* v) {
  u16 b[8];
#pragma unroll
  for (int j = 0; j < 8; j++) b[j] = T::from_f32(v[j]);
  v4i r;
  __builtin_memcpy(&r, b, 16);
  *(v4i*)p = r;
}

// T: storage type of the activations; WT: of the norm weights; ITERS: 2048-element slices of the longest row.
template <typename T, typename WT, int ITERS>
__global__ __launch_bounds__(256) void fused_rms_group_quant_kernel(RmsQuantArgs a) {
  typedef typename WT::storage WS;
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const bool second = blockIdx.y == 1;
  const int n = second ? a.n2 : a.n1;
  const u16* x = (const u16*)(second ? a.x2 : a.x1) + row * (second ? a.x2_stride : a.x1_stride);
  const u16* res = (!second && a.res1) ? (const u16*)a.res1 + row * (int64_t)n : nullptr;
  const WS* w = (const WS*)(second ? a.w2 : a.w1);
  const float eps = second ? a.eps2 : a.eps1;

  float v[ITERS][8];
  float ss = 0.f;
#pragma unroll
  for (int it = 0; it < ITERS; it++) {
    const int c = (it * 256 + (int)threadIdx.x) * 8;
#pragma unroll
    for (int j = 0; j < 8; j++) v[it][j] = 0.f;
    if (c < n) {
      load8<T>(x + c, v[it]);
      if (res) {
        float r[8];
        load8<T>(res + c, r);
#pragma unroll
        for (int j = 0; j < 8; j++) v[it][j] += r[j];
        if (a.res_out) store8<T>((u16*)a.res_out + row * (int64_t)n + c, v[it]);
      }
#pragma unroll
      for (int j = 0; j < 8; j++) ss = fmaf(v[it][j], v[it][j], ss);
    }
  }
  ss = block_sum_256(ss, red);
  const float rnorm = rsqrtf(ss / (float)n + eps);

  const int groups = (a.n1 + 127) >> 7;
#pragma unroll
  for (int it = 0; it < ITERS; it++) {
    const int c = (it * 256 + (int)threadIdx.x) * 8;
    const bool live = c < n;
    float y[8];
    float amax = 0.f;
    if (live) {
      float wv[8];
      load8<WT>(w + c, wv);
#pragma unroll
      for (int j = 0; j < 8; j++) {
        y[j] = v[it][j] * rnorm * wv[j];
        amax = fmaxf(amax, fabsf(y[j]));
      }
    }
    if (second) {
      if (live) store8<T>((u16*)a.y2 + row * (int64_t)n + c, y);
      continue;
    }
    if (live && a.y1) store8<T>((u16*)a.y1 + row * (int64_t)n + c, y);
    if (it * 2048 >= n) continue;  // whole slice past the row: uniform for the workgroup
    amax = group_max<16>(amax);
    amax = fmaxf(amax, 1e-10f);
    const float scale = amax / 448.0f;
    const float inv = 1.0f / scale;
    if (live) {
      v2i o;
      o[0] = (int)pack4_e4m3(clampf(y[0] * inv, -448.f, 448.f), clampf(y[1] * inv, -448.f, 448.f),
                             clampf(y[2] * inv, -448.f, 448.f), clampf(y[3] * inv, -448.f, 448.f));
      o[1] = (int)pack4_e4m3(clampf(y[4] * inv, -448.f, 448.f), clampf(y[5] * inv, -448.f, 448.f),
                             clampf(y[6] * inv, -448.f, 448.f), clampf(y[7] * inv, -448.f, 448.f));
      *(v2i*)(a.q + row * (int64_t)n + c) = o;
    }
    const int grp = c >> 7;
    if ((threadIdx.x & 15) == 0 && grp < groups) a.s[row * (int64_t)groups + grp] = scale;
  }
}

template <typename T, typename WT>
static int launch_rms_quant_w(const RmsQuantArgs& a, int64_t M, hipStream_t st) {
  const int longest = a.x2 ? (a.n1 > a.n2 ? a.n1 : a.n2) : a.n1;
  dim3 grid((unsigned)M, a.x2 ? 2 : 1), block(256);
  if (longest <= 2048) hipLaunchKernelGGL((fused_rms_group_quant_kernel<T, WT, 1>), grid, block, 0, st, a);
  else if (longest <= 4096) hipLaunchKernelGGL((fused_rms_group_quant_kernel<T, WT, 2>), grid, block, 0, st, a);
  else if (longest <= 8192) hipLaunchKernelGGL((fused_rms_group_quant_kernel<T, WT, 4>), grid, block, 0, st, a);
  else hipLaunchKernelGGL((fused_rms_group_quant_kernel<T, WT, 8>), grid, block, 0, st, a);
  return check_launch("fused_rms_fp8_group_quant");
}

template <typename T>
static int launch_rms_quant(const RmsQuantArgs& a, int w_dtype, int64_t M, hipStream_t st) {
  if (w_dtype == SGLAMD_F32) return launch_rms_quant_w<T, F32>(a, M, st);
  if (w_dtype == SGLAMD_BF16) return launch_rms_quant_w<T, BF16>(a, M, st);
  if (w_dtype == SGLAMD_F16) return launch_rms_quant_w<T, F16>(a, M, st);
  return fail(SGLAMD_EINVAL, "fused_rms_fp8_group_quant: weight dtype must be F32, F16 or BF16");
}

// Packed UE8M0 scales -> fp32: out[r, g] = float with exponent byte (g % 4) of word
// in[(r * row_step) * row_stride + (g / 4) * word_stride] and zero mantissa.
__global__ __launch_bounds__(256) void ue8m0_unpack_kernel(const uint32_t* __restrict__ in, int64_t row_stride,
                                                           int64_t word_stride, int64_t row_step,
                                                           float* __restrict__ out, int64_t rows, int groups) {
  const int64_t total = rows * groups;
  for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * 256) {
    const int64_t r = idx / groups;
    const int g = (int)(idx - r * groups);
    const uint32_t w = in[r * row_step * row_stride + (int64_t)(g >> 2) * word_stride];
    out[idx] = __uint_as_float(((w >> ((g & 3) * 8)) & 0xffu) << 23);
  }
}

}  // namespace sglamd

using namespace sglamd;

extern "C" int sglamd_ue8m0_unpack(const void* packed, int64_t row_stride, int64_t word_stride, int64_t row_step,
                                   float* out, int64_t rows, int64_t groups, void* stream) {
  SGLAMD_REQUIRE(packed && out, SGLAMD_EINVAL, "ue8m0_unpack: null pointer");
  SGLAMD_REQUIRE(rows >= 0 && groups > 0 && groups < (1ll << 24) && row_step >= 1, SGLAMD_EINVAL,
                 "ue8m0_unpack: bad sizes");
  SGLAMD_REQUIRE(((uintptr_t)packed % 4) == 0, SGLAMD_EINVAL, "ue8m0_unpack: packed scales must be 4-byte aligned");
  if (rows == 0) return SGLAMD_OK;
  const int64_t total = rows * groups;
  const unsigned blocks = (unsigned)(total / 256 + 1 < 4096 ? total / 256 + 1 : 4096);
  hipLaunchKernelGGL(ue8m0_unpack_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (const uint32_t*)packed,
                     row_stride, word_stride, row_step, out, rows, (int)groups);
  return check_launch("ue8m0_unpack");
}

extern "C" const char* sglamd_last_error(void) { return g_err; }
extern "C" int sglamd_abi_version(void) { return 6; }

extern "C" int sglamd_per_token_group_quant_8bit(const void* input, int in_dtype, void* output_q, int q_dtype,
                                                 void* output_s, int64_t rows, int64_t hidden, int group_size,
                                                 int scale_layout, int64_t scale_stride, float eps, float min_8bit,
                                                 float max_8bit, int form, void* stream) {
  SGLAMD_REQUIRE(input && output_q && output_s, SGLAMD_EINVAL, "group_quant: null pointer");
  SGLAMD_REQUIRE(rows > 0 && hidden > 0, SGLAMD_EINVAL, "group_quant: empty input (rows=%lld hidden=%lld)",
                 (long long)rows, (long long)hidden);
  SGLAMD_REQUIRE(group_size > 0 && hidden % group_size == 0, SGLAMD_EINVAL,
                 "group_quant: hidden (%lld) is not a multiple of group_size (%d)", (long long)hidden, group_size);
  SGLAMD_REQUIRE(q_dtype == SGLAMD_FP8_E4M3 || q_dtype == SGLAMD_I8, SGLAMD_EINVAL,
                 "group_quant: output_q must be FP8_E4M3 or I8");
  SGLAMD_REQUIRE(form == SGLAMD_QUANT_FORM_DIVIDE || form == SGLAMD_QUANT_FORM_RECIPROCAL, SGLAMD_EINVAL,
                 "group_quant: unknown arithmetic form %d", form);
  SGLAMD_REQUIRE(scale_layout >= SGLAMD_SCALE_ROW_MAJOR && scale_layout <= SGLAMD_SCALE_COL_MAJOR_UE8M0,
                 SGLAMD_EINVAL, "group_quant: unknown scale layout %d", scale_layout);
  SGLAMD_REQUIRE(scale_layout == SGLAMD_SCALE_ROW_MAJOR || scale_stride >= rows, SGLAMD_EINVAL,
                 "group_quant: column-major scale stride (%lld) is smaller than rows (%lld)", (long long)scale_stride,
                 (long long)rows);
  SGLAMD_REQUIRE(max_8bit > 0.f && min_8bit < 0.f, SGLAMD_EINVAL, "group_quant: bad clamp range");
  const bool fast = group_size == 16 || group_size == 32 || group_size == 64 || group_size == 128;
  if (form == SGLAMD_QUANT_FORM_RECIPROCAL) {
    SGLAMD_REQUIRE(fast, SGLAMD_EINVAL, "Unsupported group_size");
    SGLAMD_REQUIRE(in_dtype == SGLAMD_F16 || in_dtype == SGLAMD_BF16, SGLAMD_EINVAL,
                   "group_quant: the reciprocal form takes 16-bit inputs only");
  }
  SGLAMD_REQUIRE(((uintptr_t)input % 16) == 0 && ((uintptr_t)output_q % 16) == 0, SGLAMD_EINVAL,
                 "group_quant: input and output_q must be 16-byte aligned");

  GroupQuantArgs a = {};
  a.in = input;
  a.q = output_q;
  a.s = output_s;
  a.groups_per_row = (int)(hidden / group_size);
  a.num_groups = rows * a.groups_per_row;
  a.layout = scale_layout;
  a.scale_stride = scale_stride;
  a.eps = eps;
  a.min8 = min_8bit;
  a.max8 = max_8bit;
  a.form = form;
  a.q_is_fp8 = q_dtype == SGLAMD_FP8_E4M3;
  a.fuse_silu_mul = 0;
  a.hidden = hidden;
  hipStream_t st = (hipStream_t)stream;
  switch (in_dtype) {
    case SGLAMD_BF16:
      return launch_group_quant<BF16>(a, group_size, st);
    case SGLAMD_F16:
      return launch_group_quant<F16>(a, group_size, st);
    case SGLAMD_F32:
      return launch_group_quant<F32>(a, group_size, st);
    default:
      return fail(SGLAMD_EINVAL, "group_quant: input dtype must be F32, F16 or BF16");
  }
}

// silu(gate) * up followed by per-token-group quantisation in one pass over the [rows, 2*hidden] input.
extern "C" int sglamd_silu_mul_group_quant_8bit(const void* input, int in_dtype, void* output_q, int q_dtype,
                                                void* output_s, int64_t rows, int64_t hidden, int group_size,
                                                int scale_layout, int64_t scale_stride, float eps, float min_8bit,
                                                float max_8bit, int form, void* stream) {
  SGLAMD_REQUIRE(input && output_q && output_s, SGLAMD_EINVAL, "silu_mul_group_quant: null pointer");
  SGLAMD_REQUIRE(rows > 0 && hidden > 0, SGLAMD_EINVAL, "silu_mul_group_quant: empty input");
  SGLAMD_REQUIRE(group_size == 16 || group_size == 32 || group_size == 64 || group_size == 128, SGLAMD_EINVAL,
                 "Unsupported group_size");
  SGLAMD_REQUIRE(hidden % group_size == 0, SGLAMD_EINVAL, "silu_mul_group_quant: hidden is not a multiple of group_size");
  SGLAMD_REQUIRE(in_dtype == SGLAMD_F16 || in_dtype == SGLAMD_BF16, SGLAMD_EINVAL,
                 "silu_mul_group_quant: input must be F16 or BF16");
  SGLAMD_REQUIRE(q_dtype == SGLAMD_FP8_E4M3 || q_dtype == SGLAMD_I8, SGLAMD_EINVAL,
                 "silu_mul_group_quant: output_q must be FP8_E4M3 or I8");
  SGLAMD_REQUIRE(form == SGLAMD_QUANT_FORM_DIVIDE || form == SGLAMD_QUANT_FORM_RECIPROCAL, SGLAMD_EINVAL,
                 "silu_mul_group_quant: unknown arithmetic form %d", form);
  SGLAMD_REQUIRE(scale_layout >= SGLAMD_SCALE_ROW_MAJOR && scale_layout <= SGLAMD_SCALE_COL_MAJOR_UE8M0, SGLAMD_EINVAL,
                 "silu_mul_group_quant: unknown scale layout %d", scale_layout);
  SGLAMD_REQUIRE(scale_layout == SGLAMD_SCALE_ROW_MAJOR || scale_stride >= rows, SGLAMD_EINVAL,
                 "silu_mul_group_quant: column-major scale stride is smaller than rows");
  SGLAMD_REQUIRE(((uintptr_t)input % 16) == 0 && ((uintptr_t)output_q % 16) == 0 && (hidden * 2) % 16 == 0,
                 SGLAMD_EINVAL, "silu_mul_group_quant: pointers and rows must be 16-byte aligned");
  GroupQuantArgs a = {};
  a.in = input;
  a.q = output_q;
  a.s = output_s;
  a.groups_per_row = (int)(hidden / group_size);
  a.num_groups = rows * a.groups_per_row;
  a.layout = scale_layout;
  a.scale_stride = scale_stride;
  a.eps = eps;
  a.min8 = min_8bit;
  a.max8 = max_8bit;
  a.form = form;
  a.q_is_fp8 = q_dtype == SGLAMD_FP8_E4M3;
  a.fuse_silu_mul = 1;
  a.hidden = hidden;
  hipStream_t st = (hipStream_t)stream;
  if (in_dtype == SGLAMD_BF16) return launch_group_quant<BF16>(a, group_size, st);
  return launch_group_quant<F16>(a, group_size, st);
}

extern "C" int sglamd_silu_mul_group_quant_8bit_masked(const void* input, int in_dtype, void* output_q, int q_dtype,
                                                       void* output_s, int64_t num_experts, int64_t tokens_per_expert,
                                                       int64_t hidden, int group_size, int64_t scale_expert_stride,
                                                       int64_t scale_hidden_stride, const int32_t* masked_m, float eps,
                                                       float min_8bit, float max_8bit, void* stream) {
  SGLAMD_REQUIRE(input && output_q && output_s && masked_m, SGLAMD_EINVAL, "silu_mul_group_quant_masked: null pointer");
  SGLAMD_REQUIRE(num_experts > 0 && tokens_per_expert > 0 && hidden > 0, SGLAMD_EINVAL,
                 "silu_mul_group_quant_masked: empty input");
  SGLAMD_REQUIRE(group_size == 16 || group_size == 32 || group_size == 64 || group_size == 128, SGLAMD_EINVAL,
                 "Unsupported group_size");
  SGLAMD_REQUIRE(hidden % group_size == 0, SGLAMD_EINVAL,
                 "silu_mul_group_quant_masked: hidden is not a multiple of group_size");
  SGLAMD_REQUIRE(in_dtype == SGLAMD_F16 || in_dtype == SGLAMD_BF16, SGLAMD_EINVAL,
                 "silu_mul_group_quant_masked: input must be F16 or BF16");
  SGLAMD_REQUIRE(q_dtype == SGLAMD_FP8_E4M3 || q_dtype == SGLAMD_I8, SGLAMD_EINVAL,
                 "silu_mul_group_quant_masked: output_q must be FP8_E4M3 or I8");
  SGLAMD_REQUIRE(scale_hidden_stride >= tokens_per_expert, SGLAMD_EINVAL,
                 "silu_mul_group_quant_masked: scale hidden stride is smaller than tokens_per_expert");
  SGLAMD_REQUIRE(scale_expert_stride >= scale_hidden_stride * ((hidden / group_size + 3) / 4), SGLAMD_EINVAL,
                 "silu_mul_group_quant_masked: scale expert stride is smaller than one expert's scale words");
  SGLAMD_REQUIRE(num_experts * tokens_per_expert < 0x7fffffffll, SGLAMD_EINVAL,
                 "silu_mul_group_quant_masked: too many rows");
  SGLAMD_REQUIRE(((uintptr_t)input % 16) == 0 && ((uintptr_t)output_q % 16) == 0 && (hidden * 2) % 16 == 0,
                 SGLAMD_EINVAL, "silu_mul_group_quant_masked: pointers and rows must be 16-byte aligned");
  GroupQuantArgs a = {};
  a.in = input;
  a.q = output_q;
  a.s = output_s;
  a.groups_per_row = (int)(hidden / group_size);
  a.num_groups = num_experts * tokens_per_expert * a.groups_per_row;
  a.layout = SGLAMD_SCALE_COL_MAJOR_UE8M0;
  a.scale_stride = scale_hidden_stride;
  a.eps = eps;
  a.min8 = min_8bit;
  a.max8 = max_8bit;
  a.form = SGLAMD_QUANT_FORM_RECIPROCAL;
  a.q_is_fp8 = q_dtype == SGLAMD_FP8_E4M3;
  a.fuse_silu_mul = 1;
  a.hidden = hidden;
  a.masked_m = masked_m;
  a.tokens_per_expert = (int)tokens_per_expert;
  a.scale_expert_stride = scale_expert_stride;
  hipStream_t st = (hipStream_t)stream;
  if (in_dtype == SGLAMD_BF16) return launch_group_quant<BF16>(a, group_size, st);
  return launch_group_quant<F16>(a, group_size, st);
}

extern "C" int sglamd_per_token_quant_fp8(const void* input, int in_dtype, void* output_q, float* output_s,
                                          int64_t rows, int64_t hidden, void* stream) {
  SGLAMD_REQUIRE(input && output_q && output_s, SGLAMD_EINVAL, "per_token_quant_fp8: null pointer");
  SGLAMD_REQUIRE(rows > 0 && hidden > 0, SGLAMD_EINVAL, "per_token_quant_fp8: empty input");
  SGLAMD_REQUIRE(hidden % 4 == 0, SGLAMD_EINVAL, "Hidden dimension must be divisible by 4, but got %lld",
                 (long long)hidden);
  SGLAMD_REQUIRE(((uintptr_t)input % 16) == 0 && ((uintptr_t)output_q % 16) == 0, SGLAMD_EINVAL,
                 "per_token_quant_fp8: pointers must be 16-byte aligned");
  return launch_per_token<false>(input, in_dtype, output_q, output_s, rows, hidden, (hipStream_t)stream);
}

// Static (per-tensor) FP8 quantisation with a scale the caller already holds on the device:
// q = e4m3(clamp(x * (1 / scale))), and optionally the scale repeated once per row for the row-scaled GEMM.
// A lane moves 16 consecutive values (32 or 64 bytes in, 16 bytes out; 8 values when the element count is not a
// multiple of 16); rows only matter for the repeated scale, so the launch is a flat grid over the elements.
template <typename T, int V>
__global__ __launch_bounds__(256) void static_quant_fp8_kernel(const typename T::storage* __restrict__ in,
                                                               uint8_t* __restrict__ q, const float* __restrict__ scale,
                                                               float* __restrict__ scale_rows, int64_t rows,
                                                               int64_t hidden) {
  typedef typename T::storage S;
  const float sc = scale[0];
  const float inv = 1.0f / sc;
  const int64_t pieces = rows * hidden / V;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < pieces; i += (int64_t)gridDim.x * 256) {
    S v[V];
    constexpr int LOADS = V * (int)sizeof(S) / 16;
    v4i raw[LOADS];
#pragma unroll
    for (int l = 0; l < LOADS; l++) raw[l] = *((const v4i*)(in + i * V) + l);
    __builtin_memcpy(v, raw, sizeof(v));
    float y[V];
#pragma unroll
    for (int k = 0; k < V; k++) y[k] = clampf(T::to_f32(v[k]) * inv, -448.f, 448.f);
    uint32_t o[V / 4];
#pragma unroll
    for (int k = 0; k < V / 4; k++) o[k] = pack4_e4m3(y[4 * k], y[4 * k + 1], y[4 * k + 2], y[4 * k + 3]);
    if constexpr (V == 16) *(v4i*)(q + i * V) = v4i{(int)o[0], (int)o[1], (int)o[2], (int)o[3]};
    else *(v2i*)(q + i * V) = v2i{(int)o[0], (int)o[1]};
  }
  if (scale_rows)
    for (int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x; r < rows; r += (int64_t)gridDim.x * 256) scale_rows[r] = sc;
}

extern "C" int sglamd_static_quant_fp8(const void* input, int in_dtype, void* output_q, const float* scale,
                                       float* scale_rows, int64_t rows, int64_t hidden, void* stream) {
  SGLAMD_REQUIRE(input && output_q && scale, SGLAMD_EINVAL, "static_quant_fp8: null pointer");
  SGLAMD_REQUIRE(rows >= 0 && hidden > 0 && rows < (1ll << 31) && hidden < (1ll << 31), SGLAMD_EINVAL,
                 "static_quant_fp8: bad sizes");
  SGLAMD_REQUIRE(hidden % 8 == 0, SGLAMD_EINVAL, "static_quant_fp8: the row length (%lld) must be a multiple of 8",
                 (long long)hidden);
  SGLAMD_REQUIRE(((uintptr_t)input % 16) == 0 && ((uintptr_t)output_q % 8) == 0, SGLAMD_EINVAL,
                 "static_quant_fp8: input must be 16-byte and output 8-byte aligned");
  if (rows == 0) return SGLAMD_OK;
  const bool wide = ((rows * hidden) % 16) == 0 && ((uintptr_t)output_q % 16) == 0;
  const int64_t pieces = rows * hidden / (wide ? 16 : 8);
  const int64_t want = (pieces + 255) / 256;
  const unsigned blocks = (unsigned)(want < (int64_t)device_cus() * 32 ? want : (int64_t)device_cus() * 32);
  hipStream_t st = (hipStream_t)stream;
#define SGLAMD_STATIC_QUANT(TT, ST)                                                                                  \
  do {                                                                                                                \
    if (wide)                                                                                                         \
      hipLaunchKernelGGL((static_quant_fp8_kernel<TT, 16>), dim3(blocks), dim3(256), 0, st, (const ST*)input,         \
                         (uint8_t*)output_q, scale, scale_rows, rows, hidden);                                        \
    else                                                                                                              \
      hipLaunchKernelGGL((static_quant_fp8_kernel<TT, 8>), dim3(blocks), dim3(256), 0, st, (const ST*)input,          \
                         (uint8_t*)output_q, scale, scale_rows, rows, hidden);                                        \
  } while (0)
  if (in_dtype == SGLAMD_BF16) SGLAMD_STATIC_QUANT(BF16, u16);
  else if (in_dtype == SGLAMD_F16) SGLAMD_STATIC_QUANT(F16, u16);
  else if (in_dtype == SGLAMD_F32) SGLAMD_STATIC_QUANT(F32, float);
  else return fail(SGLAMD_EINVAL, "static_quant_fp8: input must be Float, Half or BFloat16");
#undef SGLAMD_STATIC_QUANT
  return check_launch("static_quant_fp8");
}

extern "C" int sglamd_per_token_quant_int8(const void* input, int in_dtype, int8_t* output_q, float* output_s,
                                           int64_t rows, int64_t hidden, void* stream) {
  SGLAMD_REQUIRE(input && output_q && output_s, SGLAMD_EINVAL, "per_token_quant_int8: null pointer");
  SGLAMD_REQUIRE(rows > 0 && hidden > 0, SGLAMD_EINVAL, "per_token_quant_int8: empty input");
  SGLAMD_REQUIRE(((uintptr_t)input % 16) == 0 && ((uintptr_t)output_q % 16) == 0, SGLAMD_EINVAL,
                 "per_token_quant_int8: pointers must be 16-byte aligned");
  return launch_per_token<true>(input, in_dtype, output_q, output_s, rows, hidden, (hipStream_t)stream);
}

extern "C" int sglamd_fused_rms_fp8_group_quant(const void* x1, int64_t x1_row_stride, const void* w1, float eps1,
                                                const void* res1, int64_t M, int64_t N1, void* y1_q, float* y1_s,
                                                void* y1_unquantized, void* res_out, const void* x2,
                                                int64_t x2_row_stride, const void* w2, float eps2, int64_t N2,
                                                void* y2, int dtype, int weight_dtype, int group_size, void* stream) {
  SGLAMD_REQUIRE(x1 && w1 && y1_q && y1_s, SGLAMD_EINVAL, "fused_rms_fp8_group_quant: null pointer");
  SGLAMD_REQUIRE(group_size == 128, SGLAMD_ENOTSUP, "fused_rms_fp8_group_quant: only group_size 128 is implemented");
  SGLAMD_REQUIRE(dtype == SGLAMD_BF16 || dtype == SGLAMD_F16, SGLAMD_EINVAL,
                 "fused_rms_fp8_group_quant: activations must be Half or BFloat16");
  SGLAMD_REQUIRE(M >= 0 && M < (1ll << 31) && N1 > 0 && N1 % 8 == 0 && N1 <= 16384, SGLAMD_EINVAL,
                 "fused_rms_fp8_group_quant: row length (%lld) must be a multiple of 8, at most 16384", (long long)N1);
  SGLAMD_REQUIRE(x1_row_stride >= N1 && x1_row_stride % 8 == 0 && ((uintptr_t)x1 % 16) == 0, SGLAMD_EINVAL,
                 "fused_rms_fp8_group_quant: input rows must be 16-byte aligned");
  SGLAMD_REQUIRE((((uintptr_t)w1 | (uintptr_t)y1_q | (uintptr_t)res1 | (uintptr_t)res_out | (uintptr_t)y1_unquantized) %
                  16) == 0,
                 SGLAMD_EINVAL, "fused_rms_fp8_group_quant: pointers must be 16-byte aligned");
  SGLAMD_REQUIRE(!res1 || res_out, SGLAMD_EINVAL, "fused_rms_fp8_group_quant: res_out is required with res1");
  if (x2) {
    SGLAMD_REQUIRE(w2 && y2, SGLAMD_EINVAL, "fused_rms_fp8_group_quant: second input needs its weight and output");
    SGLAMD_REQUIRE(N2 > 0 && N2 % 8 == 0 && N2 <= 16384 && x2_row_stride >= N2 && x2_row_stride % 8 == 0, SGLAMD_EINVAL,
                   "fused_rms_fp8_group_quant: second row length (%lld) must be a multiple of 8, at most 16384",
                   (long long)N2);
    SGLAMD_REQUIRE((((uintptr_t)x2 | (uintptr_t)w2 | (uintptr_t)y2) % 16) == 0, SGLAMD_EINVAL,
                   "fused_rms_fp8_group_quant: pointers must be 16-byte aligned");
  }
  if (M == 0) return SGLAMD_OK;
  RmsQuantArgs a = {};
  a.x1 = x1;
  a.x1_stride = x1_row_stride;
  a.w1 = w1;
  a.res1 = res1;
  a.res_out = res_out;
  a.q = (uint8_t*)y1_q;
  a.s = y1_s;
  a.y1 = y1_unquantized;
  a.x2 = x2;
  a.x2_stride = x2_row_stride;
  a.w2 = w2;
  a.y2 = y2;
  a.n1 = (int)N1;
  a.n2 = x2 ? (int)N2 : 0;
  a.eps1 = eps1;
  a.eps2 = eps2;
  if (dtype == SGLAMD_BF16) return launch_rms_quant<BF16>(a, weight_dtype, M, (hipStream_t)stream);
  return launch_rms_quant<F16>(a, weight_dtype, M, (hipStream_t)stream);
}
