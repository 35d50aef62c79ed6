// Long sequences (L = 2048 .. 16384): the fused mixer core and the filter-spectrum kernel with the
// row's N = 2L point transform split by frequency parity into two L-point half transforms that run one
// after the other through one L-point LDS buffer.
//
//   z[n] = a[n] + i u[n], n < L (zero for L <= n < N)
//   E[k] = Z[2k]   = FFT_L(z)[k]                O[k] = Z[2k+1] = FFT_L(z w_N^n)[k]
//   W    = spectral multiply of Z by the two filter spectra (pairs kappa <-> N - kappa: inside E that is
//          k <-> (L - k) mod L, inside O it is k <-> L - 1 - k)
//   w[n] = IFFT_L(We)[n] + w_N^-n IFFT_L(Wo)[n]  for n < L, which are the only outputs needed
//
// i.e. the first radix-2 step of a decimation-in-frequency transform whose upper input half is zero,
// and the last step of its inverse whose upper output half is dropped.  Compared with transforming all
// N points in LDS this halves the LDS footprint of a row (two workgroups fit on a compute unit and
// overlap each other's barrier and memory stalls), and with 32 points per thread each half transform
// needs three passes: radix R1 at stride L/R1, radix R2 at stride 16, radix 16 on contiguous groups.
//
// The twist w_N^n is absorbed by the first pass: with n = q + (L/R1) j it factors into a per-thread
// root b = w_N^q and the constant w_{2 R1}^j, so the odd half's first pass is "multiply input j by a
// compile-time constant, radix-R1 butterfly, twiddle with b^(2k+1)" where the even half twiddles with
// b^(2k).  The input row is staged once and kept in registers (first-pass layout) for the second half.
//
// Filter spectra: spec[channel][half][slot 0..15][work item 0..T-1] as float4 (K1.re, K1.im, K2.re,
// K2.im), in exactly the order the multiply consumes them; filter_spectrum_split_kernel writes it with
// the same passes (for the 2L-tap filters the halves are FFT_L(lo + hi) and FFT_L((lo - hi) w_N^n)).
//
// Stands in for the same reference code as fftconv_kernels.hip (bert/src/mm/hyena_utils.py:16-42,
// 231-236; bert/src/mm/monarch_mixer_sequence_mixer.py:112-147).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fft_engine.h"
#include "fft_split.h"
#include "hyena_filter.h"
#include "row_io.h"

namespace m2 {

// ------------------------------------------------------------------------------------------
// the fused mixer core
// ------------------------------------------------------------------------------------------
// FULL: short convolutions and gates (sw, sb non-null); otherwise a plain long convolution of one input.
// HAS_U: the residual long convolution of the layer input u (uin non-null).
template <class P, typename ACT, bool FULL, bool HAS_U>
__global__ __launch_bounds__(P::T) __attribute__((amdgpu_waves_per_eu(2, 2))) void mixer_split_kernel(
    const ACT* __restrict__ xproj,      // (3d, B, L): x1 | x2 | v, channel-major
    const float* __restrict__ uin,      // (d, B, L)   layer input, channel-major (may be null)
    const float* __restrict__ sw,       // (3d, 3)     short-conv taps; null = plain convolution of a (d, B, L) input
    const float* __restrict__ sb,       // (3d)        short-conv bias
    const float* __restrict__ pbias,    // (3d)        bias of the in-projection, added to xproj on load (may be null)
    const float4* __restrict__ spec,    // (d, 2, 16, T)
    ACT* __restrict__ y,                // (d, B, L)
    int B, int d) {
  constexpr int L = P::L, T = P::T;
  extern __shared__ float2 lds[];
  float2* row = lds;
  float2* tab2 = lds + P::ROW_LDS;
  const int t = threadIdx.x;
  const int n0 = 32 * t;

  tab2_init<P>(tab2);
  cf b[P::NB1];
  static_for<0, P::NB1>([&](auto ii) { b[decltype(ii)::value] = unit_root(t + T * decltype(ii)::value, P::N); });
  const SplitGroups<P> grp = split_groups<P>(t);
  phase_barrier();

  // Workgroup ids are dealt round-robin to the 8 XCDs (one L2 each).  XCD e takes the channels
  // c = e (mod 8) and runs the B rows of a channel on neighbouring workgroups at the same time, so a
  // channel's spectrum is fetched into that L2 once and shared.  (d % 8 == 0 is checked by the host.)
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, slots = gridDim.x >> 3;
  const int rows_per_xcd = (d >> 3) * B;
  for (int j = slot; j < rows_per_xcd; j += slots) {
    const int c = (j / B) * 8 + xcd, bb = j % B;

    // ---- prologue: 32 consecutive time steps per thread in chunks of 8 (a mapping with consecutive lanes on
    // consecutive 16-byte pieces was measured 7 % slower).  All loads of the row are put in
    // flight first; then short conv, gate, z = a + i u -> LDS
    GateRow<ACT, 4> gate;
    {
      RawRow<ACT, 4, true> r1, r2, rv;      // the four accesses of a thread are consecutive
      f32x4_t ru[8];
      float w1[3], w2[3], wv[3], b1 = 0.f, b2 = 0.f, bv = 0.f, p1 = 0.f, p2 = 0.f, pv = 0.f;
      static_for<0, 4>([&](auto qq) {
        constexpr int q = decltype(qq)::value;
        const int n = n0 + 8 * q;
        if constexpr (FULL) {
          r1.template fetch<q>(xproj + ((long)(0 * d + c) * B + bb) * L, n);
          rv.template fetch<q>(xproj + ((long)(2 * d + c) * B + bb) * L, n);
          r2.template fetch<q>(xproj + ((long)(1 * d + c) * B + bb) * L, n);
        } else {
          r1.template fetch<q>(xproj + ((long)c * B + bb) * L, n);
        }
        ru[2 * q] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        ru[2 * q + 1] = ru[2 * q];
        if constexpr (HAS_U) {
          const float* pu = uin + ((long)c * B + bb) * L + n;
          ru[2 * q] = *reinterpret_cast<const f32x4_t*>(pu);
          ru[2 * q + 1] = *reinterpret_cast<const f32x4_t*>(pu + 4);
        }
      });
      if constexpr (FULL) {
        const float* w = sw + (long)c * 3;
#pragma unroll
        for (int k = 0; k < 3; ++k) {
          w1[k] = w[k];
          w2[k] = w[3 * (long)d + k];
          wv[k] = w[6 * (long)d + k];
        }
        b1 = sb[c]; b2 = sb[d + c]; bv = sb[2 * d + c];
        if (pbias) { p1 = pbias[c]; p2 = pbias[d + c]; pv = pbias[2 * d + c]; }
      }
      // The bias p of the in-projection is not added to the inputs: a 3-tap convolution of (x + p) is the convolution
      // of x plus p (w0 + w1 + w2), which goes into the convolution's own bias -- except for the first two outputs
      // of a row, where one or two taps fall on the zero padding (outside the biased signal): those are corrected.
      const float f1 = b1 + p1 * (w1[0] + w1[1] + w1[2]), f2 = b2 + p2 * (w2[0] + w2[1] + w2[2]),
                  fv = bv + pv * (wv[0] + wv[1] + wv[2]);
      __builtin_amdgcn_sched_barrier(0);
      static_for<0, 4>([&](auto qq) {
        constexpr int q = decltype(qq)::value;
        const int n = n0 + 8 * q;
        float in[10], a[8], gt[8];
        if constexpr (FULL) {
          float cv[8];
          r1.template expand<q>(n, in);
          static_for<0, 8>([&](auto ee) {
            constexpr int e = decltype(ee)::value;
            a[e] = f1 + w1[0] * in[e] + w1[1] * in[e + 1] + w1[2] * in[e + 2];
          });
          rv.template expand<q>(n, in);
          static_for<0, 8>([&](auto ee) {
            constexpr int e = decltype(ee)::value;
            cv[e] = fv + wv[0] * in[e] + wv[1] * in[e + 1] + wv[2] * in[e + 2];
          });
          r2.template expand<q>(n, in);
          static_for<0, 8>([&](auto ee) {
            constexpr int e = decltype(ee)::value;
            gt[e] = f2 + w2[0] * in[e] + w2[1] * in[e + 1] + w2[2] * in[e + 2];
          });
          if constexpr (q == 0) {
            if (t == 0) {      // time steps 0 and 1 of the row
              a[0] -= p1 * (w1[0] + w1[1]); a[1] -= p1 * w1[0];
              cv[0] -= pv * (wv[0] + wv[1]); cv[1] -= pv * wv[0];
              gt[0] -= p2 * (w2[0] + w2[1]); gt[1] -= p2 * w2[0];
            }
          }
          static_for<0, 8>([&](auto ee) { a[decltype(ee)::value] *= cv[decltype(ee)::value]; });
        } else {
          // plain long convolution: xproj is a single (d, B, L) signal, no short conv, no gates
          r1.template expand<q>(n, in);
          static_for<0, 8>([&](auto ee) {
            constexpr int e = decltype(ee)::value;
            a[e] = in[e + 2];
            gt[e] = 1.f;
          });
        }
        gate.template set<q>(gt);
        const f32x4_t u0 = ru[2 * q], u1 = ru[2 * q + 1];
        float2* dst = row + sphys(n);       // 8 consecutive slots never straddle a pad
        dst[0] = make_float2(a[0], u0.x); dst[1] = make_float2(a[1], u0.y);
        dst[2] = make_float2(a[2], u0.z); dst[3] = make_float2(a[3], u0.w);
        dst[4] = make_float2(a[4], u1.x); dst[5] = make_float2(a[5], u1.y);
        dst[6] = make_float2(a[6], u1.z); dst[7] = make_float2(a[7], u1.w);
        __builtin_amdgcn_sched_barrier(0);
      });
    }
    phase_barrier();

    cf x[32], held[32];
    pass1_load<P>(x, t, row);
    static_for<0, 32>([&](auto ii) { held[decltype(ii)::value] = x[decltype(ii)::value]; });     // z, for the odd half

    const float4* sp = spec + (long)c * 32 * T + t;
    half_convolution<P, false>(x, t, row, tab2, b, sp, grp.ge, grp.gm, grp.special);
    static_for<0, 32>([&](auto ii) {       // x <- z for the odd half, held <- the even half's result
      constexpr int i = decltype(ii)::value;
      const cf e = x[i];
      x[i] = held[i];
      held[i] = e;
    });
    half_convolution<P, true>(x, t, row, tab2, b, sp + 16 * T, grp.go, grp.gc, false);
    static_for<0, 32>([&](auto ii) {
      constexpr int i = decltype(ii)::value;
      x[i] = cadd(x[i], held[i]);
    });
    pass1_store<P>(x, t, row);             // own slots: nobody else reads or writes them in the first pass
    phase_barrier();

    // ---- epilogue: 32 consecutive outputs per thread
    static_for<0, 4>([&](auto qq) {
      constexpr int q = decltype(qq)::value;
      const int n = n0 + 8 * q;
      const float2* src = row + sphys(n);
      float out[8];
      static_for<0, 8>([&](auto ee) {
        constexpr int e = decltype(ee)::value;
        const float2 v = src[e];
        out[e] = v.x * gate.template get<8 * q + e>() + v.y;
      });
      store8(y + ((long)c * B + bb) * L, n, out);
    });
    phase_barrier();      // the next row's prologue overwrites what the epilogue has just read
  }
}

// ------------------------------------------------------------------------------------------
// filter taps -> spectra in the layout above (both filters of one mixer in one complex transform)
// ------------------------------------------------------------------------------------------
template <class P, bool HAS2>
__global__ __launch_bounds__(P::T) void filter_spectrum_split_kernel(
    const float* taps1,    // (d, N) bidirectional taps of filter_fn
    const float* taps2,    // (d, N) bidirectional taps of filter_fn2 (may be null)
    const float* D1,       // (d) skip weight of filter_fn, added to tap 0 (may be null)
    const float* D2,       // (d) skip weight of filter_fn2 (may be null)
    float4* __restrict__ spec,          // (d, 2, 16, T)
    int d, SpectrumBatch sb) {
  constexpr int L = P::L, N = P::N, T = P::T;
  extern __shared__ float2 lds[];
  float2* row = lds;
  float2* tab2 = lds + P::ROW_LDS;
  const int t = threadIdx.x;
  {
    float* sp = reinterpret_cast<float*>(spec);
    select_mixer(sb, d, N, taps1, taps2, D1, D2, sp);
    spec = reinterpret_cast<float4*>(sp);
  }

  tab2_init<P>(tab2);
  cf b[P::NB1];
  static_for<0, P::NB1>([&](auto ii) { b[decltype(ii)::value] = unit_root(t + T * decltype(ii)::value, P::N); });
  const SplitGroups<P> grp = split_groups<P>(t);
  // 1/N of the convolution, 1/2 of the separation of the two packed filters, 1/2 of the separation of the two
  // packed signals in the mixer kernel (pair_multiply_half)
  const float scale = 0.25f / (float)N;
  __syncthreads();

  auto split = [&](cf za, cf zb) __attribute__((always_inline)) -> float4 {
    // K1 = (za + conj zb) * scale ; K2 = (za - conj zb) / i * scale
    return make_float4(scale * (za.re + zb.re), scale * (za.im - zb.im), scale * (za.im + zb.im),
                       scale * (zb.re - za.re));
  };

  // work item = (channel, half transform): 2 d items spread evenly over the grid.  Workgroup ids are dealt round-robin
  // to the 8 XCDs (one L2 each): XCD e takes the channels c = e (mod 8), and the two halves of a channel, which read the
  // same taps, run on neighbouring workgroups of that XCD at the same time, so the second read is an L2 hit.
  // (Needs d % 8 == 0 and an even number of workgroups per XCD; other shapes take the items in plain order.)
  const bool by_xcd = (d & 7) == 0 && (gridDim.x & 15) == 0;
  const int first = by_xcd ? (int)(blockIdx.x >> 3) : (int)blockIdx.x, step = by_xcd ? (int)(gridDim.x >> 3) : (int)gridDim.x;
  const int count = by_xcd ? (d >> 3) * 2 : 2 * d;
  for (int j = first; j < count; j += step) {
    const int c = by_xcd ? (j >> 1) * 8 + (int)(blockIdx.x & 7) : j >> 1;
    const int item = j;
    auto one_half = [&](auto hh) __attribute__((always_inline)) {
      constexpr bool ODD = decltype(hh)::value == 1;
      // z = k1 + i k2 over 2L taps; even half: z_lo + z_hi, odd half: z_lo - z_hi (its twist is in the first pass).
      // All loads of the row go in flight before the first is used.
      {
        f32x4_t lo1[8], hi1[8], lo2[8], hi2[8];
        static_for<0, 8>([&](auto qq) {
          constexpr int q = decltype(qq)::value;
          const float* p1 = taps1 + (long)c * N + 4 * (q * T + t);      // consecutive lanes, consecutive 16 bytes
          lo1[q] = *reinterpret_cast<const f32x4_t*>(p1);
          hi1[q] = *reinterpret_cast<const f32x4_t*>(p1 + L);
          if constexpr (HAS2) {
            const float* p2 = taps2 + (long)c * N + 4 * (q * T + t);
            lo2[q] = *reinterpret_cast<const f32x4_t*>(p2);
            hi2[q] = *reinterpret_cast<const f32x4_t*>(p2 + L);
          } else {
            lo2[q] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            hi2[q] = lo2[q];
          }
        });
        // the skip weight D is one more tap at lag 0
        const float dd1 = (D1 && t == 0) ? D1[c] : 0.f, dd2 = (D2 && t == 0) ? D2[c] : 0.f;
        lo1[0].x += dd1;
        lo2[0].x += dd2;
        constexpr float sgn = ODD ? -1.f : 1.f;
        static_for<0, 8>([&](auto qq) {
          constexpr int q = decltype(qq)::value;
          float2* dst = row + sphys(4 * (q * T + t));     // 4 consecutive slots never straddle a pad
          dst[0] = make_float2(lo1[q].x + sgn * hi1[q].x, lo2[q].x + sgn * hi2[q].x);
          dst[1] = make_float2(lo1[q].y + sgn * hi1[q].y, lo2[q].y + sgn * hi2[q].y);
          dst[2] = make_float2(lo1[q].z + sgn * hi1[q].z, lo2[q].z + sgn * hi2[q].z);
          dst[3] = make_float2(lo1[q].w + sgn * hi1[q].w, lo2[q].w + sgn * hi2[q].w);
        });
      }
      __syncthreads();
      cf x[32];
      pass1_load<P>(x, t, row);
      fwd_pass1<P, ODD>(x, t, row, b);
      __syncthreads();
      fwd_pass2<P>(x, t, row, tab2);
      __syncthreads();
      fwd_groups<P>(x, row, ODD ? grp.go : grp.ge, ODD ? grp.gc : grp.gm);
      __syncthreads();      // LDS is restaged by the next half / channel

      float4* sp = spec + ((long)c * 2 + (ODD ? 1 : 0)) * 16 * T + t;
      if (!ODD && grp.special) {
        const cf z0 = x[bitrev(0, 4)], zn = x[bitrev(8, 4)];
        sp[0] = make_float4(4.f * scale * z0.re, 4.f * scale * zn.re, 4.f * scale * z0.im, 4.f * scale * zn.im);
        static_for<1, 8>([&](auto ss) {
          constexpr int s = decltype(ss)::value;
          sp[s * T] = split(x[bitrev(s, 4)], x[bitrev(16 - s, 4)]);
        });
        static_for<0, 8>([&](auto ss) {
          constexpr int s = decltype(ss)::value;
          sp[(8 + s) * T] = split(x[16 + bitrev(s, 4)], x[16 + bitrev(15 - s, 4)]);
        });
      } else {
        static_for<0, 16>([&](auto ss) {
          constexpr int s = decltype(ss)::value;
          sp[s * T] = split(x[bitrev(s, 4)], x[16 + bitrev(15 - s, 4)]);
        });
      }
    };
    if (item & 1) one_half(ic<1>{});
    else one_half(ic<0>{});
  }
}

// ------------------------------------------------------------------------------------------
// host-side launchers
// ------------------------------------------------------------------------------------------
template <class P, typename ACT>
static int launch_mixer_split(const void* xproj, const float* u, const float* sw, const float* sb, const float* pbias,
                              const float* spec, void* y, int B, int d, hipStream_t stream) {
  const size_t lds_bytes = (size_t)P::WG_LDS * sizeof(float2);
  auto kern = sw ? (u ? mixer_split_kernel<P, ACT, true, true> : mixer_split_kernel<P, ACT, true, false>)
                 : mixer_split_kernel<P, ACT, false, false>;
  if (!sw && u) return set_error(M2_ERR_ARG, "mixer_split: a plain convolution takes no second input");
  if (lds_bytes > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (e != hipSuccess) return set_error(M2_ERR_LAUNCH, "hipFuncSetAttribute(mixer_split): %s", hipGetErrorString(e));
  }
  const int rows_per_xcd = (d / 8) * B;
  int per_cu = (int)((160 * 1024) / lds_bytes);
  if (per_cu < 1) per_cu = 1;
  if (per_cu > 512 / P::T) per_cu = 512 / P::T;  // two waves per SIMD at 256 registers
  int slots = (num_cus() / 8) * per_cu;          // workgroups per XCD
  if (slots > rows_per_xcd) slots = rows_per_xcd;
  const int rounds = (rows_per_xcd + slots - 1) / slots;      // every workgroup the same number of rows
  slots = (rows_per_xcd + rounds - 1) / rounds;
  hipLaunchKernelGGL(kern, dim3(8 * slots), dim3(P::T), lds_bytes, stream, (const ACT*)xproj, u, sw, sb, pbias,
                     (const float4*)spec, (ACT*)y, B, d);
  return check_launch("mixer_split");
}

template <class P>
static int launch_filter_spectrum_split_t(const float* taps1, const float* taps2, const float* D1, const float* D2,
                                          float* spec, int d, const SpectrumBatch& sb, int nmixers, hipStream_t stream) {
  const size_t lds_bytes = (size_t)P::WG_LDS * sizeof(float2);
  const bool has2 = sb.taps ? sb.fpm == 2 : taps2 != nullptr;
  auto kern = has2 ? filter_spectrum_split_kernel<P, true> : filter_spectrum_split_kernel<P, false>;
  if (lds_bytes > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (e != hipSuccess) return set_error(M2_ERR_LAUNCH, "hipFuncSetAttribute(filter_spectrum_split): %s", hipGetErrorString(e));
  }
  int per_cu = (int)((160 * 1024) / lds_bytes);
  if (per_cu < 1) per_cu = 1;
  if (per_cu > 512 / P::T) per_cu = 512 / P::T;
  // a multiple of 16 workgroups: an even number per XCD, so that the two halves of a channel run side by side
  int grid = (num_cus() * per_cu) / 16 * 16;
  if (grid > 2 * d) grid = 2 * d;
  hipLaunchKernelGGL(kern, dim3(grid, nmixers), dim3(P::T), lds_bytes, stream, taps1, taps2, D1, D2, (float4*)spec, d, sb);
  return check_launch("filter_spectrum_split");
}

#define M2_FOR_EACH_SPLIT_PLAN(X) \
  X(11, 16, 8)                    \
  X(12, 16, 16)                   \
  X(13, 32, 16)                   \
  X(14, 32, 32)

#define X(LOGL, R1, R2) static_assert(split_offsets_ok<SplitPlan<LOGL, R1, R2>>(), "LDS offsets of the split plan");
M2_FOR_EACH_SPLIT_PLAN(X)
#undef X

bool split_plan_exists(int L) {
  switch (L) {
#define X(LOGL, R1, R2) \
  case 1 << LOGL:       \
    return true;
    M2_FOR_EACH_SPLIT_PLAN(X)
#undef X
  }
  return false;
}

int launch_mixer_split_dispatch(const void* xproj, const float* u, const float* sw, const float* sb, const float* pbias,
                                const float* spec, void* y, int B, int L, int d, int act_dtype, hipStream_t stream) {
  switch (L) {
#define X(LOGL, R1, R2)                                                                                              \
  case 1 << LOGL:                                                                                                    \
    return act_dtype == M2_DTYPE_F32                                                                                 \
               ? launch_mixer_split<SplitPlan<LOGL, R1, R2>, float>(xproj, u, sw, sb, pbias, spec, y, B, d, stream)    \
               : launch_mixer_split<SplitPlan<LOGL, R1, R2>, uint16_t>(xproj, u, sw, sb, pbias, spec, y, B, d, stream);
    M2_FOR_EACH_SPLIT_PLAN(X)
#undef X
  }
  return set_error(M2_ERR_UNSUPPORTED, "mixer_split: no plan for L=%d", L);
}

int launch_filter_spectrum_split(const float* taps1, const float* taps2, const float* D1, const float* D2, float* spec,
                                 int d, int L, const SpectrumBatch& sb, int nmixers, hipStream_t stream) {
  switch (L) {
#define X(LOGL, R1, R2) \
  case 1 << LOGL:       \
    return launch_filter_spectrum_split_t<SplitPlan<LOGL, R1, R2>>(taps1, taps2, D1, D2, spec, d, sb, nmixers, stream);
    M2_FOR_EACH_SPLIT_PLAN(X)
#undef X
  }
  return set_error(M2_ERR_UNSUPPORTED, "filter_spectrum_split: no plan for L=%d", L);
}

}  // namespace m2
