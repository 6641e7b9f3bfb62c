// Shared device/host helpers for the gfx950 quantized-linear kernels.
// Everything here is HIP for CDNA4 (wave64); there is no other target.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/sglamd.h"

namespace sglamd {

// Records a message retrievable through sglamd_last_error() and returns `code`.
int fail(int code, const char* fmt, ...);

#define SGLAMD_REQUIRE(cond, code, ...) \
  do {                                  \
    if (!(cond)) return ::sglamd::fail((code), __VA_ARGS__); \
  } while (0)

// Turns the status of the launch that just happened into a C-ABI return code.
int check_launch(const char* what);

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef unsigned short u16;

__device__ __forceinline__ float bf16_bits_to_f32(u16 h) { return __uint_as_float(((uint32_t)h) << 16); }

// fp32 -> bf16 bits, round-to-nearest-even, NaN kept quiet: gfx950 converts in hardware (v_cvt_pk_bf16_f32),
// one instruction where the bit arithmetic takes seven.
__device__ __forceinline__ u16 f32_to_bf16_bits(float f) {
  const __bf16 b = (__bf16)f;
  u16 h;
  __builtin_memcpy(&h, &b, 2);
  return h;
}
// two at once: low half a, high half b
__device__ __forceinline__ uint32_t f32x2_to_bf16x2_bits(float a, float b) {
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  const bf16x2_t p = __builtin_convertvector((f32x2_t){a, b}, bf16x2_t);
  uint32_t w;
  __builtin_memcpy(&w, &p, 4);
  return w;
}

__device__ __forceinline__ float f16_bits_to_f32(u16 h) {
  _Float16 v;
  __builtin_memcpy(&v, &h, 2);
  return (float)v;
}

__device__ __forceinline__ u16 f32_to_f16_bits(float f) {
  _Float16 v = (_Float16)f;  // v_cvt_f16_f32: round-to-nearest-even
  u16 h;
  __builtin_memcpy(&h, &v, 2);
  return h;
}

// 16-bit storage tags used to pick the conversion at compile time.
struct BF16 {
  static constexpr int tag = SGLAMD_BF16;
  typedef u16 storage;
  static __device__ __forceinline__ float to_f32(u16 h) { return bf16_bits_to_f32(h); }
  static __device__ __forceinline__ u16 from_f32(float f) { return f32_to_bf16_bits(f); }
  static __device__ __forceinline__ uint32_t pack2(float a, float b) { return f32x2_to_bf16x2_bits(a, b); }
};
struct F16 {
  static constexpr int tag = SGLAMD_F16;
  typedef u16 storage;
  static __device__ __forceinline__ float to_f32(u16 h) { return f16_bits_to_f32(h); }
  static __device__ __forceinline__ u16 from_f32(float f) { return f32_to_f16_bits(f); }
  static __device__ __forceinline__ uint32_t pack2(float a, float b) {
    return (uint32_t)f32_to_f16_bits(a) | ((uint32_t)f32_to_f16_bits(b) << 16);
  }
};
struct F32 {
  static constexpr int tag = SGLAMD_F32;
  typedef float storage;
  static __device__ __forceinline__ float to_f32(float h) { return h; }
  static __device__ __forceinline__ float from_f32(float f) { return f; }
};

// Two fp32 -> two OCP e4m3fn bytes in the low half of the result (v_cvt_pk_fp8_f32,
// round-to-nearest-even; callers clamp to +-448 first, so the overflow behaviour of the
// instruction never matters).
__device__ __forceinline__ uint32_t pack2_e4m3(float a, float b) {
  return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false) & 0xffffu;
}
__device__ __forceinline__ uint32_t pack4_e4m3(float a, float b, float c, float d) {
  int w = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
  w = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, w, true);
  return (uint32_t)w;
}

__device__ __forceinline__ float clampf(float v, float lo, float hi) { return fminf(fmaxf(v, lo), hi); }

static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Compute units of the current device (cached per device; 256 when the query fails, the MI355X count).
static inline int device_cus() {
  static int cus[32] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 32) return 256;
  if (!cus[dev]) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cus[dev] = n;
  }
  return cus[dev];
}

// A kernel that asks for more than 64 KB of dynamic LDS needs hipFuncAttributeMaxDynamicSharedMemorySize
// raised once per device; `state` is one object per kernel instantiation (a function-local static).
struct SmemAttrOnce {
  int bytes[32] = {};
};
static inline hipError_t raise_dynamic_smem(SmemAttrOnce& state, const void* kern, int bytes) {
  int dev = 0;
  const bool cached = hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 32;
  if (cached && state.bytes[dev] >= bytes) return hipSuccess;
  const hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e == hipSuccess && cached) state.bytes[dev] = bytes;
  return e;
}

}  // namespace sglamd
