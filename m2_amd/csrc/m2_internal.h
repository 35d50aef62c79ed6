// Helpers shared by the translation units of libm2_amd.so (not part of the public C ABI).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/m2_amd.h"

namespace m2 {

// Records a printf-style message retrievable through m2_last_error() and returns `code`.
int set_error(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
// hipGetLastError() after a launch -> 0 or M2_ERR_LAUNCH (message recorded).
int check_launch(const char* what);
// Compute units of the current device (cached per device).
int num_cus();

// round-to-nearest-even float -> bfloat16 bits (NaN stays NaN)
// float -> bf16 bits, round to nearest even (host restatement of what v_cvt_pk_bf16_f32 does)
__host__ __device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  union { float f; uint32_t u; } v;
  v.f = f;
  if ((v.u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((v.u >> 16) | 0x40u);
  v.u += 0x7fffu + ((v.u >> 16) & 1u);
  return (uint16_t)(v.u >> 16);
}
__host__ __device__ __forceinline__ float bf16_to_f32(uint16_t h) {
  union { float f; uint32_t u; } v;
  v.u = ((uint32_t)h) << 16;
  return v.f;
}

// two floats -> packed bf16 pair (lo in bits 0..15), round to nearest even; one v_cvt_pk_bf16_f32 on the device
__host__ __device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
#if defined(__HIP_DEVICE_COMPILE__)
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  f32x2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
#else
  return (uint32_t)f32_to_bf16_bits(lo) | ((uint32_t)f32_to_bf16_bits(hi) << 16);
#endif
}
__host__ __device__ __forceinline__ uint16_t f32_to_bf16(float f) {
#if defined(__HIP_DEVICE_COMPILE__)
  return (uint16_t)pack_bf16x2(f, 0.f);            // the hardware conversion: no branches
#else
  return f32_to_bf16_bits(f);
#endif
}

}  // namespace m2
