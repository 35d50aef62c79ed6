// Pieces shared by the kernels that stream their weights through LDS with direct global -> LDS loads and apply the
// GELU gate on MFMA accumulators (mlp_fused_kernels.hip, glu_stream_kernels.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace m2 {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// x * Phi(x): the same clamped odd polynomial as the separate GLU kernel (blockdiag_kernels.hip), so both paths
// round alike.
__device__ __forceinline__ float gelu_erf_poly(float x) {
  const float xc = __builtin_amdgcn_fmed3f(x, -3.9f, 3.9f);
  const float x2 = xc * xc;
  float p = 2.7693410957e-08f;
  p = fmaf(p, x2, -1.8473178272e-06f);
  p = fmaf(p, x2, 5.2869800351e-05f);
  p = fmaf(p, x2, -8.6171873090e-04f);
  p = fmaf(p, x2, 9.0065851481e-03f);
  p = fmaf(p, x2, -6.5103946404e-02f);
  p = fmaf(p, x2, 3.9828952833e-01f);
  return x * fmaf(p, xc, 0.5f);
}

// The same polynomial cut into its eleven instructions, so that the kernel below can issue the chains of its eight
// elements side by side (step s of all eight, then step s + 1: no instruction waits for the one before it).
// Step 10 leaves gelu(x) * v in `out`; same operations in the same order as gelu_erf_poly(x) * v.
struct GeluChain {
  float xc, x2, p;
};
template <int STEP>
__device__ __forceinline__ void gelu_step(GeluChain& c, float x, float v, float& out) {
  if constexpr (STEP == 0) c.xc = __builtin_amdgcn_fmed3f(x, -3.9f, 3.9f);
  else if constexpr (STEP == 1) c.x2 = c.xc * c.xc;
  else if constexpr (STEP == 2) c.p = fmaf(2.7693410957e-08f, c.x2, -1.8473178272e-06f);
  else if constexpr (STEP == 3) c.p = fmaf(c.p, c.x2, 5.2869800351e-05f);
  else if constexpr (STEP == 4) c.p = fmaf(c.p, c.x2, -8.6171873090e-04f);
  else if constexpr (STEP == 5) c.p = fmaf(c.p, c.x2, 9.0065851481e-03f);
  else if constexpr (STEP == 6) c.p = fmaf(c.p, c.x2, -6.5103946404e-02f);
  else if constexpr (STEP == 7) c.p = fmaf(c.p, c.x2, 3.9828952833e-01f);
  else if constexpr (STEP == 8) c.p = fmaf(c.p, c.xc, 0.5f);
  else if constexpr (STEP == 9) c.p = x * c.p;
  else if constexpr (STEP == 10) out = c.p * v;
}

// s_waitcnt immediates (vmcnt in bits 3:0 and 15:14, expcnt 6:4, lgkmcnt 11:8): wait for the vector-memory
// counter only
constexpr int kWaitVm0 = 0x0F70;

// One direct global -> LDS load: every lane fetches 16 bytes from base + voff, lane l's piece lands at LDS byte
// address lds + 16 l.  Inline assembly on purpose: the compiler then neither tracks the LDS write (it would put a
// full vector-memory wait in front of every later LDS read) nor reorders it across other memory accesses; the
// kernel waits for these loads itself.
__device__ __forceinline__ void load_to_lds(unsigned lds, unsigned voff, const void* base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds), "v"(voff), "s"(base) : "memory");
}

}  // namespace m2
