// Shared host/device helpers for libnf_cdna4 (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "nf_cdna4.h"

namespace nf {

// ---- error reporting -------------------------------------------------------
char* last_error_buf();
int fail(int code, const char* fmt, ...);

#define NF_REQUIRE(cond, code, ...)                 \
  do {                                              \
    if (!(cond)) return ::nf::fail(code, __VA_ARGS__); \
  } while (0)

inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail((int)e, "%s: %s", what, hipGetErrorString(e));
  return 0;
}

inline int dtype_size(int dt) { return dt == NF_F32 ? 4 : 2; }
inline bool dtype_ok(int dt) { return dt == NF_F32 || dt == NF_F16 || dt == NF_BF16; }

// ---- bf16 <-> f32 on the device --------------------------------------------
// bf16 is handled as raw uint16_t bits; round-to-nearest-even like torch.
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }

// (gfx950 converts two floats to packed bfloat16 or float16, round-to-nearest-even, in one instruction)
typedef float nf_f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 nf_bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 nf_f16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t f32x2_to_bf16x2_bits(float lo, float hi) {
  const nf_f32x2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, nf_bf16x2));
}
__device__ __forceinline__ uint32_t f32x2_to_f16x2_bits(float lo, float hi) {
  const nf_f32x2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, nf_f16x2));
}
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) { return (uint16_t)(f32x2_to_bf16x2_bits(f, 0.0f) & 0xffffu); }

__device__ __forceinline__ float f16_bits_to_f32(uint16_t b) {
  return __half2float(__ushort_as_half(b));
}
__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) { return __half_as_ushort(__float2half_rn(f)); }

// Element-type tags: load/store one element of a tensor as float.
struct F32 {
  typedef float storage;
  static constexpr int code = NF_F32;
  __device__ static __forceinline__ float to_f32(storage v) { return v; }
  __device__ static __forceinline__ storage from_f32(float f) { return f; }
};
struct F16 {
  typedef uint16_t storage;
  static constexpr int code = NF_F16;
  __device__ static __forceinline__ float to_f32(storage v) { return f16_bits_to_f32(v); }
  __device__ static __forceinline__ storage from_f32(float f) { return f32_to_f16_bits(f); }
  __device__ static __forceinline__ uint32_t pack(float lo, float hi) { return f32x2_to_f16x2_bits(lo, hi); }
};
struct BF16 {
  typedef uint16_t storage;
  static constexpr int code = NF_BF16;
  __device__ static __forceinline__ float to_f32(storage v) { return bf16_bits_to_f32(v); }
  __device__ static __forceinline__ storage from_f32(float f) { return f32_to_bf16_bits(f); }
  __device__ static __forceinline__ uint32_t pack(float lo, float hi) { return f32x2_to_bf16x2_bits(lo, hi); }
};

// Load element i of a tensor whose dtype is only known at run time (uniform branch).
__device__ __forceinline__ float load_as_f32(const void* p, int64_t i, int dt) {
  if (dt == NF_F32) return ((const float*)p)[i];
  uint16_t b = ((const uint16_t*)p)[i];
  return dt == NF_F16 ? f16_bits_to_f32(b) : bf16_bits_to_f32(b);
}

}  // namespace nf
