// Types shared by the filter-generation translation units (hyena_filter_kernels.hip, filter_fused_kernels.hip):
// the pointer table of a batch of implicit filters and the helpers that turn fp32 values into bf16 parts for
// the matrix cores.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fft_regs.h"
#include "m2_internal.h"

namespace m2 {

constexpr int kOrder = 128;
constexpr int kMaxEmb = 8;

struct MlpPtrs {
  const float *w0, *b0, *w1, *b1, *w2, *b2, *w3;
};
struct FilterPtrs {
  const float *z, *t, *freq, *deltas;
  MlpPtrs mlp[2];                 // [0] forward, [1] reverse (all null when the filter is not bidirectional)
};
// the public struct is the same eighteen pointers in the same order, so a device array of it is a table of these
static_assert(sizeof(FilterPtrs) == sizeof(m2_hyena_filter_params), "pointer table layout");

// A batch of filters reaches the kernels either inside the kernel arguments (up to kMaxFilters: the entry point
// that takes a host array) or as a table in device memory (any number: the entry point for all mixers of a model).
constexpr int kMaxFilters = 4;
struct FilterBatch {
  FilterPtrs f[kMaxFilters];
};
struct TabByValue {
  FilterBatch fb;
  __device__ __forceinline__ const FilterPtrs& at(int i) const { return fb.f[i]; }
};
struct TabByPointer {
  const FilterPtrs* p;
  __device__ __forceinline__ const FilterPtrs& at(int i) const { return p[i]; }
};

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// x = hi + mid + lo with three bf16 terms: 24 mantissa bits, i.e. all of an fp32 value
__device__ __forceinline__ void split3(float x, float& hi, float& mid, float& lo) {
  hi = bf16_to_f32(f32_to_bf16(x));
  const float r = x - hi;
  mid = bf16_to_f32(f32_to_bf16(r));
  lo = r - mid;                      // the conversion of lo to bf16 happens where it is packed
}

// Spectrum kernels of a batch of mixers: blockIdx.y selects the mixer.  taps: filter f of mixer m at
// taps + (m fpm + f) d 2L; skip: device array of fpm pointers per mixer (skip weights, entries may be null);
// spectra of mixer m at spec + m spec_stride floats.  taps == nullptr: a single mixer given by the kernel's own
// taps1 / taps2 / D1 / D2 arguments.
struct SpectrumBatch {
  const float* taps;
  const float* const* skip;
  int fpm;
  long spec_stride;
};
__device__ __forceinline__ void select_mixer(const SpectrumBatch& sb, int d, int N, const float*& taps1,
                                             const float*& taps2, const float*& D1, const float*& D2, float*& spec) {
  if (sb.taps == nullptr) return;
  const int m = blockIdx.y;
  taps1 = sb.taps + (long)(m * sb.fpm) * d * N;
  taps2 = sb.fpm == 2 ? taps1 + (long)d * N : nullptr;
  D1 = sb.skip ? sb.skip[m * sb.fpm] : nullptr;
  D2 = (sb.skip && sb.fpm == 2) ? sb.skip[m * sb.fpm + 1] : nullptr;
  spec += (long)m * sb.spec_stride;
}

// launchers defined beside their kernels
int launch_filter_spectrum_any(const float* taps1, const float* taps2, const float* D1, const float* D2, float* spec,
                               int d, int L, const SpectrumBatch& sb, int nmixers, hipStream_t stream);
bool project_spectrum_supported(int L);
int launch_project_spectrum(const FilterPtrs* tab, const float* const* skip, int nmixers, int fpm, int L, int d,
                            float shift, const uint16_t* h_hi, const uint16_t* h_lo, float* spec, long spec_stride,
                            hipStream_t stream);

}  // namespace m2
