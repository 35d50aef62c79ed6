// Measured ceilings of one compute unit's matrix pipe, for the roofline arguments of the GEMM-shaped kernels:
// a loop of v_mfma_f32_32x32x16_bf16 on register operands, alone or with the company the real kernels give it
// (one or two 16-byte LDS operand reads per MFMA, software-pipelined six MFMAs ahead; 4, 6 or 11 dependent fp32
// FMAs per MFMA in the same instruction stream), at one or two waves per SIMD on every compute unit.  What comes
// out is the rate this chip sustains at the clock it runs such code at, which is what a kernel's achieved
// TFLOP/s can be held against beside the published peak.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fft_regs.h"
#include "m2_internal.h"

namespace m2 {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kProbeLds = 64 * 1024;
constexpr int kProbePF = 6;        // operand reads run this many MFMAs ahead

template <int READS, int VALU, int NT>
__global__ __launch_bounds__(NT) void probe_mfma_kernel(float* __restrict__ sink, int iters) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  for (int i = tid; i < kProbeLds / 4; i += NT) reinterpret_cast<float*>(lds)[i] = i * 1e-6f;
  __syncthreads();
  floatx16 acc[6];
  static_for<0, 6>([&](auto tt) { static_for<0, 16>([&](auto vv) { acc[decltype(tt)::value][decltype(vv)::value] = 0.f; }); });
  bf16x8 b0;
  for (int i = 0; i < 8; ++i) b0[i] = (__bf16)(tid * 0.001f + i);
  float v[8];
  for (int i = 0; i < 8; ++i) v[i] = tid * 0.01f + i;
  const unsigned char* base = lds + 16 * lane;      // [block of 1 KB][lane]: conflict-free 16-byte reads
  u32x4 ring[kProbePF], ring2[kProbePF];
  static_for<0, kProbePF>([&](auto ss) {
    constexpr int s = decltype(ss)::value;
    ring[s] = *reinterpret_cast<const u32x4*>(base + 1024 * s);
    ring2[s] = *reinterpret_cast<const u32x4*>(base + 1024 * (s + 24));
  });
  for (int it = 0; it < iters; ++it) {
    static_for<0, 12>([&](auto ss) {
      constexpr int s = decltype(ss)::value;
      const bf16x8 a = READS >= 1 ? __builtin_bit_cast(bf16x8, ring[s % kProbePF]) : b0;
      const bf16x8 b = READS >= 2 ? __builtin_bit_cast(bf16x8, ring2[s % kProbePF]) : b0;
      acc[s % 6] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[s % 6], 0, 0, 0);
      if constexpr (READS >= 1) ring[s % kProbePF] = *reinterpret_cast<const u32x4*>(base + 1024 * ((s + kProbePF) % 12) + 12288 * (it & 1));
      if constexpr (READS >= 2) ring2[s % kProbePF] = *reinterpret_cast<const u32x4*>(base + 1024 * (24 + (s + kProbePF) % 12) + 12288 * (it & 1));
      static_for<0, VALU>([&](auto ee) { v[decltype(ee)::value % 8] = fmaf(v[decltype(ee)::value % 8], 1.0001f, 0.5f); });
      __builtin_amdgcn_sched_barrier(0);
    });
  }
  float s = 0.f;
  static_for<0, 6>([&](auto tt) { static_for<0, 16>([&](auto vv) { s += acc[decltype(tt)::value][decltype(vv)::value]; }); });
  for (int i = 0; i < 8; ++i) s += v[i];
  sink[(long)blockIdx.x * NT + tid] = s;
}

template <int READS, int VALU, int NT>
static int launch_probe(float* sink, int iters, hipStream_t st) {
  auto kern = probe_mfma_kernel<READS, VALU, NT>;
  hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, kProbeLds);
  if (e != hipSuccess) return set_error(M2_ERR_LAUNCH, "hipFuncSetAttribute(probe): %s", hipGetErrorString(e));
  hipLaunchKernelGGL(kern, dim3(num_cus()), dim3(NT), kProbeLds, st, sink, iters);
  return check_launch("probe_mfma");
}

}  // namespace m2

using namespace m2;

extern "C" int m2_probe_mfma_fwd(int lds_reads_per_mfma, int valu_per_mfma, int waves_per_simd, int iters, float* sink,
                                 long long* mfma_per_wave, int* waves, void* stream) {
  if (!sink || iters <= 0) return set_error(M2_ERR_ARG, "m2_probe_mfma_fwd: null sink or non-positive iters");
  if (mfma_per_wave) *mfma_per_wave = 12LL * iters;
  if (waves) *waves = num_cus() * 4 * waves_per_simd;
  hipStream_t st = (hipStream_t)stream;
#define M2_PROBE_CASE(R, V)                                                                       \
  if (lds_reads_per_mfma == R && valu_per_mfma == V)                                              \
    return waves_per_simd == 1 ? launch_probe<R, V, 256>(sink, iters, st)                         \
         : waves_per_simd == 2 ? launch_probe<R, V, 512>(sink, iters, st)                         \
         : set_error(M2_ERR_UNSUPPORTED, "m2_probe_mfma_fwd: waves_per_simd must be 1 or 2");
  M2_PROBE_CASE(0, 0) M2_PROBE_CASE(1, 0) M2_PROBE_CASE(2, 0) M2_PROBE_CASE(1, 4) M2_PROBE_CASE(1, 6) M2_PROBE_CASE(1, 11)
#undef M2_PROBE_CASE
  return set_error(M2_ERR_UNSUPPORTED, "m2_probe_mfma_fwd: (reads, valu) must be one of (0,0) (1,0) (2,0) (1,4) (1,6) (1,11)");
}
