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

}  // namespace sglamd

using namespace sglamd;

extern "C" const char* sglamd_last_error(void) { return g_err; }
extern "C" int sglamd_abi_version(void) { return 2; }

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

extern "C" int sglamd_per_token_quant_int8(const void* input, int in_dtype, int8_t* output_q, float* output_s,
                                           int64_t rows, int64_t hidden, void* stream) {
  SGLAMD_REQUIRE(input && output_q && output_s, SGLAMD_EINVAL, "per_token_quant_int8: null pointer");
  SGLAMD_REQUIRE(rows > 0 && hidden > 0, SGLAMD_EINVAL, "per_token_quant_int8: empty input");
  SGLAMD_REQUIRE(((uintptr_t)input % 16) == 0 && ((uintptr_t)output_q % 16) == 0, SGLAMD_EINVAL,
                 "per_token_quant_int8: pointers must be 16-byte aligned");
  return launch_per_token<true>(input, in_dtype, output_q, output_s, rows, hidden, (hipStream_t)stream);
}
