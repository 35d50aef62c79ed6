// Implicit-filter generation for short sequences (L <= 512): the 128 -> d output projection of the filter MLPs, the
// exponential decay, the placement of forward and reverse taps in the 2L window, the skip weight and the transform
// to the spectra the mixer core consumes -- as ONE kernel, so the taps never exist in memory
// (bert/src/mm/hyena_utils.py:175,201-217 last Linear + modulation, :231-236 bidirectional window,
// :24-33 rfft(k) / 2L; launch granularity of the reference's native filter kernel,
// csrc/flashmm/flash_mm.cpp:301-362).
//
// A workgroup owns 16 channels of one mixer: 16 rows of N = 2L complex points in LDS (re = filter_fn, im =
// filter_fn2), exactly one batch of rows for 16 N / 16 = N threads.  Phase 1: wave w projects the positions of
// MLP w mod nmlp (forward / reverse MLP of either filter) for the 16 channels on v_mfma_f32_16x16x32_bf16
// (W3 rows as the A operand, split into bf16 hi / lo parts in registers; the last hidden layer's activations,
// which the hidden kernel left as bf16 hi / lo parts, as the B operand; three products: fp32-grade accuracy),
// multiplies by exp(-t |delta|) + shift and drops each value at its place in the window.  Phase 2: every row is
// transformed by its N / 16 threads (same passes as the stand-alone spectrum kernel) and stored in the mixer core's
// order.  All mixers of a model go in one launch (blockIdx.y).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fft_engine.h"
#include "hyena_filter.h"

namespace m2 {

constexpr int kFusedRows = 16;      // channels per workgroup

template <class P>
__global__ __launch_bounds__(kFusedRows* P::T) void project_spectrum_kernel(
    const FilterPtrs* __restrict__ tab,         // fpm entries per mixer
    const float* const* __restrict__ skip,      // fpm skip-weight pointers per mixer (entries, or the table, may be null)
    int fpm, int d, float shift,
    const uint16_t* __restrict__ h_hi,          // (2 nfilters, L, 128) bf16: high parts of the last hidden layer
    const uint16_t* __restrict__ h_lo,          // low parts
    float4* __restrict__ spec, long spec_stride4) {
  constexpr int L = P::L, N = P::N, T = P::T, NT = kFusedRows * T, NW = NT / 64;
  extern __shared__ float2 lds[];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, i16 = lane & 15, q4 = lane >> 4;
  const int mixer = blockIdx.y, c0 = blockIdx.x * kFusedRows;
  const int nmlp = 2 * fpm;

  // parts of the window nobody writes: the second filter's component without a second filter, the reverse half
  // without reverse MLPs
  const bool bidir = tab[mixer * fpm].mlp[1].w3 != nullptr;
  if (fpm == 1 || !bidir) {
    for (int i = tid; i < kFusedRows * P::ROW_LDS; i += NT) lds[i] = make_float2(0.f, 0.f);
    __syncthreads();
  }

  // ---- phase 1: projection + decay into the window ----
  {
    const int m = wave % nmlp, which = m >> 1, dir = m & 1;
    const int f = mixer * fpm + which;
    const FilterPtrs& F = tab[f];
    const float* W3 = F.mlp[dir].w3;
    if (W3 != nullptr) {
      bf16x8 ahi[kOrder / 32], alo[kOrder / 32];
      {
        const float* wrow = W3 + (long)(c0 + i16) * kOrder + 8 * q4;
#pragma unroll
        for (int ks = 0; ks < kOrder / 32; ++ks) {
          const float4 v0 = *reinterpret_cast<const float4*>(wrow + 32 * ks);
          const float4 v1 = *reinterpret_cast<const float4*>(wrow + 32 * ks + 4);
          const float v[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
          float h[8], l[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            h[j] = bf16_to_f32(f32_to_bf16(v[j]));
            l[j] = v[j] - h[j];
          }
          const u32x4 vh = {pack_bf16x2(h[0], h[1]), pack_bf16x2(h[2], h[3]), pack_bf16x2(h[4], h[5]), pack_bf16x2(h[6], h[7])};
          const u32x4 vl = {pack_bf16x2(l[0], l[1]), pack_bf16x2(l[2], l[3]), pack_bf16x2(l[4], l[5]), pack_bf16x2(l[6], l[7])};
          ahi[ks] = __builtin_bit_cast(bf16x8, vh);
          alo[ks] = __builtin_bit_cast(bf16x8, vl);
        }
      }
      float adelta[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) adelta[j] = -fabsf(F.deltas[c0 + 4 * q4 + j]) * 1.44269504088896341f;
      const uint16_t* gh = h_hi + ((long)(2 * f + dir) * L + i16) * kOrder + 8 * q4;
      const uint16_t* gl = h_lo + ((long)(2 * f + dir) * L + i16) * kOrder + 8 * q4;
      // the waves that share an MLP take its 16-position tiles in turn
      for (int pt = wave / nmlp; pt < L / 16; pt += NW / nmlp) {
        u32x4 bh[kOrder / 32], bl[kOrder / 32];
#pragma unroll
        for (int ks = 0; ks < kOrder / 32; ++ks) {
          bh[ks] = *reinterpret_cast<const u32x4*>(gh + (long)pt * 16 * kOrder + 32 * ks);
          bl[ks] = *reinterpret_cast<const u32x4*>(gl + (long)pt * 16 * kOrder + 32 * ks);
        }
        const int p = 16 * pt + i16;
        const float tl = F.t[p];
        floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < kOrder / 32; ++ks) {      // smallest terms first
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(alo[ks], __builtin_bit_cast(bf16x8, bh[ks]), acc, 0, 0, 0);
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ahi[ks], __builtin_bit_cast(bf16x8, bl[ks]), acc, 0, 0, 0);
        }
#pragma unroll
        for (int ks = 0; ks < kOrder / 32; ++ks)
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ahi[ks], __builtin_bit_cast(bf16x8, bh[ks]), acc, 0, 0, 0);
        // accumulator element j of lane (i16, q4): channel c0 + 4 q4 + j, position p
        const int idx = dir == 0 ? p : N - 1 - p;
        float* dst = reinterpret_cast<float*>(lds + (4 * q4) * P::ROW_LDS + P::phys(idx)) + which;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          // exp(-t |delta|); the bare hardware exp2 flushes results below 2^-126 to zero, which is the value to
          // 1e-38 absolute
          const float decay = __builtin_amdgcn_exp2f(tl * adelta[j]) + shift;
          dst[(long)j * P::ROW_LDS * 2] = acc[j] * decay;
        }
      }
    }
  }

  // ---- phase 2: one row per T threads; the barrier inside twiddles_init also ends phase 1 ----
  const int rloc = tid / T, t = tid % T;
  float2* row = lds + rloc * P::ROW_LDS;
  Twiddles<P> tw;
  twiddles_init<P>(tw, t, lds + kFusedRows * P::ROW_LDS);
  int g, g2;
  paired_groups<P>(t, g, g2);
  const int c = c0 + rloc;
  if (t == 0 && skip != nullptr) {                   // the skip weight D is one more tap at lag 0
    const float* D1 = skip[mixer * fpm];
    const float* D2 = fpm == 2 ? skip[mixer * fpm + 1] : nullptr;
    float2 v = row[0];
    if (D1) v.x += D1[c];
    if (D2) v.y += D2[c];
    row[0] = v;
  }
  row_sync<P>();
  cf x[16];
  fwd_load<P, P::R1, P::S1>(x, t, row);
  forward_to_pairs<P, false>(x, t, row, tw, g, g2);
  const float scale = 0.25f / (float)N;      // the 1/2 of the even/odd split here, the 1/2 of the one in the mixer core's multiply, the 1/N of the convolution
  store_filter_spectrum<P>(x, t, scale, spec + (long)mixer * spec_stride4 + (long)c * 8 * T + t);
}

#define M2_FOR_EACH_FUSED_PLAN(X) \
  X(8, 4, 8, 1)                   \
  X(9, 8, 8, 1)                   \
  X(10, 16, 8, 1)

bool project_spectrum_supported(int L) { return L == 128 || L == 256 || L == 512; }

template <class P>
static int launch_project_spectrum_t(const FilterPtrs* tab, const float* const* skip, int nmixers, int fpm, int d,
                                     float shift, const uint16_t* h_hi, const uint16_t* h_lo, float* spec,
                                     long spec_stride, hipStream_t stream) {
  const size_t lds_bytes = (size_t)(kFusedRows * P::ROW_LDS + P::TW_LDS) * sizeof(float2);
  auto kern = project_spectrum_kernel<P>;
  if (lds_bytes > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (e != hipSuccess) return set_error(M2_ERR_LAUNCH, "hipFuncSetAttribute(project_spectrum): %s", hipGetErrorString(e));
  }
  hipLaunchKernelGGL(kern, dim3(d / kFusedRows, nmixers), dim3(kFusedRows * P::T), lds_bytes, stream, tab, skip, fpm, d,
                     shift, h_hi, h_lo, (float4*)spec, spec_stride / 4);
  return check_launch("project_spectrum");
}

int launch_project_spectrum(const FilterPtrs* tab, const float* const* skip, int nmixers, int fpm, int L, int d,
                            float shift, const uint16_t* h_hi, const uint16_t* h_lo, float* spec, long spec_stride,
                            hipStream_t stream) {
  if (d % kFusedRows != 0) return set_error(M2_ERR_UNSUPPORTED, "project_spectrum: d=%d must be a multiple of %d", d, kFusedRows);
  switch (ilog2(2 * L)) {
#define X(LOGN, R1, R2, R3) \
  case LOGN:                \
    return launch_project_spectrum_t<Plan<LOGN, R1, R2, R3>>(tab, skip, nmixers, fpm, d, shift, h_hi, h_lo, spec, spec_stride, stream);
    M2_FOR_EACH_FUSED_PLAN(X)
#undef X
  }
  return set_error(M2_ERR_UNSUPPORTED, "project_spectrum: no plan for L=%d", L);
}

}  // namespace m2
