// Fused Monarch-Mixer sequence-mixer core for gfx950, and the filter-spectrum kernel that feeds it.
//
// One (channel, batch) row of length L is convolved with two 2L-tap bidirectional filters by a
// single complex FFT of length N = 2L held in LDS:
//
//   z[n] = a[n] + i*u[n]           a = shortconv(v) * shortconv(x1),  u = layer input   (n < L, 0 after)
//   Z    = FFT_N(z)                in-place decimation in frequency, spectrum left digit-reversed
//   A[k] = (Z[k] + conj Z[N-k])/2, B[k] = (Z[k] - conj Z[N-k])/(2i)      (spectra of a and of u)
//   W[k] = A[k] K1[k] + i B[k] K2[k]
//   w    = IFFT_N(W) (unscaled; K carries 1/N)  ->  Re w = a (*) k1,  Im w = u (*) k2
//   y[n] = Re w[n] * shortconv(x2)[n] + Im w[n]                                        (n < L)
//
// The skip terms "+ D1 a" and "+ D2 u" of the reference are folded into tap 0 of the filters when
// their spectra are built (k[0] += D), which is the same convolution.
//
// Replaces, for the reference's torch path, bert/src/mm/monarch_mixer_sequence_mixer.py:112-147
// together with bert/src/mm/hyena_utils.py:16-42,231-236 (two fftconv_ref calls, the gating and the
// residual add); the launch granularity corresponds to the reference's optional CUDA kernel
// csrc/flashmm/mm_block_fwd_cuda.cu:173-647 but none of that code is used here.
//
// Thread mapping.  E = 16 complex points per thread, T = N/16 threads per row.  The FFT is
// R1 x R2 (x R3) x 8.  Every pass but the last is "load R points at stride S, radix-R butterfly in
// registers, twiddle, store in place".  The last forward pass and the first inverse pass are
// radix-8 on contiguous groups of 8; thread w takes group g(w) AND the group g' that holds the
// mirrored frequencies N-k, so the spectral multiply needs no exchange: it happens in registers
// between the two radix-8 transforms.  Global memory is read and written 8 consecutive time steps per
// thread (16-byte accesses); the row is staged in LDS between that layout and the first-pass layout.
// This file serves sequence lengths up to 1024; longer rows use fftconv_split_kernels.hip (2048 .. 16384)
// and fftconv_real_kernels.hip (32768).
//
// The filter spectra are stored in exactly the order the multiply consumes them
// ("native order": spec[channel][slot 0..7][w 0..T-1] as float4 = K1.re, K1.im, K2.re, K2.im for the
// frequency that sits in slot `slot` of group g(w)); the spectrum kernel below produces that order
// with the same FFT code, so the layout is private to this file.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fft_engine.h"
#include "hyena_filter.h"
#include "row_io.h"

namespace m2 {

// ------------------------------------------------------------------------------------------
// K2: the fused mixer core
// ------------------------------------------------------------------------------------------
// first forward pass when only positions [0, N/2) of the row are populated (upper half is zero)
template <class P>
__device__ __forceinline__ void fwd_load_lower(cf (&x)[16], int t, const float2* row) {
  constexpr int R = P::R1, S = P::S1, NB = 16 / R;
  static_for<0, NB>([&](auto ii) {
    constexpr int i = decltype(ii)::value;
    const float2* pb = row + P::phys(t + P::T * i);
    static_for<0, R / 2>([&](auto jj) {
      constexpr int j = decltype(jj)::value;
      x[i * R + j] = lds_get(pb, P::poff(j * S));
    });
  });
}
template <class P>
__device__ __forceinline__ void inv_store_lower(const cf (&x)[16], int t, float2* row) {
  constexpr int R = P::R1, S = P::S1, NB = 16 / R;
  static_for<0, NB>([&](auto ii) {
    constexpr int i = decltype(ii)::value;
    float2* pb = row + P::phys(t + P::T * i);
    static_for<0, R / 2>([&](auto jj) {
      constexpr int j = decltype(jj)::value;
      lds_put(pb, P::poff(j * S), x[i * R + j]);
    });
  });
}

// Per-row constants of the short convolutions, staged through LDS: the T threads of a row share one channel, so
// thread k < 15 of the row fetches constant k and all of them read the set back (one register per thread in
// flight instead of fifteen).  Order: (w0, w1, w2, conv bias, projection bias) of x1, then of v, then of x2.
constexpr int kRowConsts = 16;

template <class P, typename ACT>
__global__ __launch_bounds__(P::WG) void mixer_core_kernel(
    const ACT* __restrict__ xproj,      // (3d, B, L): x1 | x2 | v, channel-major
    const float* __restrict__ uin,      // (d, B, L)   layer input, channel-major (may be null)
    const float* __restrict__ sw,       // (3d, 3)     short-conv taps; null = plain convolution of a (d, B, L) input
    const float* __restrict__ sb,       // (3d)        short-conv bias
    const float* __restrict__ pbias,    // (3d)        bias of the in-projection, added to xproj on load (may be null)
    const float4* __restrict__ spec,    // (d, 8, T)   native-order spectra
    ACT* __restrict__ y,                // (d, B, L)
    int B, int d) {
  constexpr int L = P::L, T = P::T;
  extern __shared__ float2 lds[];
  const int tid = threadIdx.x;
  const int rloc = tid / T, t = tid % T;
  float2* row = lds + rloc * P::ROW_LDS;
  float* crow = reinterpret_cast<float*>(lds + P::RPW * P::ROW_LDS + P::TW_LDS) + rloc * kRowConsts;
  const int n0 = 8 * t;

  Twiddles<P> tw;
  twiddles_init<P>(tw, t, lds + P::RPW * P::ROW_LDS);
  int g, g2;
  paired_groups<P>(t, g, g2);

  // Workgroup ids are dealt round-robin to the 8 XCDs (one L2 each).  XCD e takes the channels
  // c = e (mod 8) and runs the B rows of a channel on neighbouring workgroups at the same time, so a
  // channel's spectrum is fetched into that L2 once and shared.  (d % 8 == 0 is checked by the host.)
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, slots = gridDim.x >> 3;
  const int rows_per_xcd = (d >> 3) * B;

  // The inputs of a row batch are requested one batch ahead: the loads of batch i + 1 are issued as soon as the
  // registers of batch i have been consumed by its prologue, and travel while batch i is transformed.  Without
  // this the workgroups of a compute unit, which start together, stay in step: all load, then all compute, and
  // memory time adds to arithmetic time instead of hiding behind it.
  RawRow<ACT, 1> r1, r2, rv;
  f32x4_t u0 = {0.f, 0.f, 0.f, 0.f}, u1 = u0;
  float cst = 0.f;
  auto fetch_batch = [&](int j0) __attribute__((always_inline)) {
    const int j = j0 + rloc;
    const int jj = j < rows_per_xcd ? j : rows_per_xcd - 1;
    const int c = (jj / B) * 8 + xcd, b = jj % B;
    if (sw) {
      r1.template fetch<0>(xproj + ((long)(0 * d + c) * B + b) * L, n0);
      rv.template fetch<0>(xproj + ((long)(2 * d + c) * B + b) * L, n0);
      r2.template fetch<0>(xproj + ((long)(1 * d + c) * B + b) * L, n0);
      if (t < 15) {
        const int grp = t / 5, k = t % 5;
        const long ch = (long)(grp == 0 ? 0 : grp == 1 ? 2 : 1) * d + c;
        cst = k < 3 ? sw[ch * 3 + k] : k == 3 ? sb[ch] : (pbias ? pbias[ch] : 0.f);
      }
    } else {
      r1.template fetch<0>(xproj + ((long)c * B + b) * L, n0);
    }
    if (uin) {
      const float* pu = uin + ((long)c * B + b) * L + n0;
      u0 = *reinterpret_cast<const f32x4_t*>(pu);
      u1 = *reinterpret_cast<const f32x4_t*>(pu + 4);
    }
  };
  if (slot * P::RPW < rows_per_xcd) fetch_batch(slot * P::RPW);

  for (int j0 = slot * P::RPW; j0 < rows_per_xcd; j0 += slots * P::RPW) {
    const int j = j0 + rloc;
    const bool valid = j < rows_per_xcd;
    const int jj = valid ? j : rows_per_xcd - 1;
    const int c = (jj / B) * 8 + xcd, b = jj % B;

    // ---- prologue: 8 consecutive time steps per thread: short conv, gate, stage z = a + i u in LDS ----
    GateRow<ACT, 1> gate;
    {
      float in[10], a[8], gt[8];
      if (sw) {
        if (t < 15) crow[t] = cst;
        row_sync<P>();
        const float4 c0 = *reinterpret_cast<const float4*>(crow), c1 = *reinterpret_cast<const float4*>(crow + 4),
                     c2 = *reinterpret_cast<const float4*>(crow + 8), c3 = *reinterpret_cast<const float4*>(crow + 12);
        const float w10 = c0.x, w11 = c0.y, w12 = c0.z, bb1 = c0.w, p1 = c1.x;
        const float wv0 = c1.y, wv1 = c1.z, wv2 = c1.w, bbv = c2.x, pv = c2.y;
        const float w20 = c2.z, w21 = c2.w, w22 = c3.x, bb2 = c3.y, p2 = c3.z;
        // The bias p of the in-projection is not added to the inputs: a 3-tap convolution of (x + p) is the
        // convolution of x plus p (w0 + w1 + w2), which goes into the convolution's own bias -- except for the first
        // two outputs of a row, where one or two taps fall on the zero padding: those are corrected.
        const float f1 = bb1 + p1 * (w10 + w11 + w12), fv = bbv + pv * (wv0 + wv1 + wv2), f2 = bb2 + p2 * (w20 + w21 + w22);
        float cv[8];
        r1.template expand<0>(n0, in);
        static_for<0, 8>([&](auto jj) {
          constexpr int j = decltype(jj)::value;
          a[j] = f1 + w10 * in[j] + w11 * in[j + 1] + w12 * in[j + 2];
        });
        rv.template expand<0>(n0, in);
        static_for<0, 8>([&](auto jj) {
          constexpr int j = decltype(jj)::value;
          cv[j] = fv + wv0 * in[j] + wv1 * in[j + 1] + wv2 * in[j + 2];
        });
        r2.template expand<0>(n0, in);
        static_for<0, 8>([&](auto jj) {
          constexpr int j = decltype(jj)::value;
          gt[j] = f2 + w20 * in[j] + w21 * in[j + 1] + w22 * in[j + 2];
        });
        if (n0 == 0) {      // time steps 0 and 1 of the row
          a[0] -= p1 * (w10 + w11); a[1] -= p1 * w10;
          cv[0] -= pv * (wv0 + wv1); cv[1] -= pv * wv0;
          gt[0] -= p2 * (w20 + w21); gt[1] -= p2 * w20;
        }
        static_for<0, 8>([&](auto jj) { a[decltype(jj)::value] *= cv[decltype(jj)::value]; });
      } else {
        // plain long convolution: xproj is a single (d, B, L) signal, no short conv, no gates
        r1.template expand<0>(n0, in);
        static_for<0, 8>([&](auto jj) {
          constexpr int j = decltype(jj)::value;
          a[j] = in[j + 2];
          gt[j] = 1.f;
        });
      }
      gate.template set<0>(gt);
      float4* dst = reinterpret_cast<float4*>(row + P::phys(n0));     // 8 consecutive slots never straddle a pad
      dst[0] = make_float4(a[0], u0.x, a[1], u0.y);
      dst[1] = make_float4(a[2], u0.z, a[3], u0.w);
      dst[2] = make_float4(a[4], u1.x, a[5], u1.y);
      dst[3] = make_float4(a[6], u1.z, a[7], u1.w);
    }
    // the next batch's loads, behind everything that read this batch's registers
    __builtin_amdgcn_sched_barrier(0);
    if (j0 + slots * P::RPW < rows_per_xcd) fetch_batch(j0 + slots * P::RPW);
    __builtin_amdgcn_sched_barrier(0);
    row_sync<P>();

    cf x[16];
    fwd_load_lower<P>(x, t, row);
    forward_to_pairs<P, true>(x, t, row, tw, g, g2);

    // ---- spectral multiply in registers ----
    {
      const float4* sp = spec + (long)c * 8 * T + t;
      float4 K[8];
      static_for<0, 8>([&](auto s) { K[decltype(s)::value] = sp[decltype(s)::value * T]; });
      if (t != 0) {
        static_for<0, 8>([&](auto jj) {
          constexpr int j = decltype(jj)::value;
          pair_multiply(x[bitrev(j, 3)], x[8 + bitrev(7 - j, 3)], K[j]);
        });
      } else {
        // group 0: slots j <-> (8-j)%8 ; DC (j=0) and Nyquist (j=4) are self-paired and real-filtered
        x[bitrev(0, 3)] = {x[bitrev(0, 3)].re * K[0].x, x[bitrev(0, 3)].im * K[0].z};
        x[bitrev(4, 3)] = {x[bitrev(4, 3)].re * K[0].y, x[bitrev(4, 3)].im * K[0].w};
        static_for<1, 4>([&](auto jj) {
          constexpr int j = decltype(jj)::value;
          pair_multiply(x[bitrev(j, 3)], x[bitrev(8 - j, 3)], K[j]);
        });
        // group RL/2 (k_low = M/2): slots j <-> 7-j inside the same group
        static_for<0, 4>([&](auto jj) {
          constexpr int j = decltype(jj)::value;
          pair_multiply(x[8 + bitrev(j, 3)], x[8 + bitrev(7 - j, 3)], K[4 + j]);
        });
      }
    }

    // ---- inverse ----
    inverse_from_pairs<P, true>(x, t, row, tw, g, g2);
    inv_store_lower<P>(x, t, row);      // only slots this thread has just read are overwritten
    row_sync<P>();

    // ---- epilogue: 8 consecutive outputs per thread ----
    {
      const float4* src = reinterpret_cast<const float4*>(row + P::phys(n0));
      const float4 o0 = src[0], o1 = src[1], o2 = src[2], o3 = src[3];
      float out[8];
      out[0] = o0.x * gate.template get<0>() + o0.y; out[1] = o0.z * gate.template get<1>() + o0.w;
      out[2] = o1.x * gate.template get<2>() + o1.y; out[3] = o1.z * gate.template get<3>() + o1.w;
      out[4] = o2.x * gate.template get<4>() + o2.y; out[5] = o2.z * gate.template get<5>() + o2.w;
      out[6] = o3.x * gate.template get<6>() + o3.y; out[7] = o3.z * gate.template get<7>() + o3.w;
      if (valid) store8(y + ((long)c * B + b) * L, n0, out);
    }
    row_sync<P>();      // the next row's prologue overwrites what the epilogue has just read
  }
}

// ------------------------------------------------------------------------------------------
// K1c: filter taps -> native-order spectra (both filters of one mixer in one complex FFT)
// ------------------------------------------------------------------------------------------
template <class P>
__global__ __launch_bounds__(P::WG) void filter_spectrum_kernel(
    const float* taps1,    // (d, N) bidirectional taps of filter_fn
    const float* taps2,    // (d, N) bidirectional taps of filter_fn2 (may be null)
    const float* D1,       // (d) skip weight of filter_fn, added to tap 0 (may be null)
    const float* D2,       // (d) skip weight of filter_fn2 (may be null)
    float4* __restrict__ spec,          // (d, 8, T)
    int d, SpectrumBatch sb) {
  constexpr int N = P::N, T = P::T;
  extern __shared__ float2 lds[];
  const int tid = threadIdx.x;
  const int rloc = tid / T, t = tid % T;
  float2* row = lds + rloc * P::ROW_LDS;
  const int n0 = 16 * t;
  {
    float* sp = reinterpret_cast<float*>(spec);
    select_mixer(sb, d, N, taps1, taps2, D1, D2, sp);
    spec = reinterpret_cast<float4*>(sp);
  }

  Twiddles<P> tw;
  twiddles_init<P>(tw, t, lds + P::RPW * P::ROW_LDS);
  int g, g2;
  paired_groups<P>(t, g, g2);
  const float scale = 0.25f / (float)N;      // the 1/2 of the even/odd split here, the 1/2 of the one in the mixer core's multiply, the 1/N of the convolution

  for (int r0 = blockIdx.x * P::RPW; r0 < d; r0 += gridDim.x * P::RPW) {
    const int r = r0 + rloc;
    const bool valid = r < d;
    const int c = valid ? r : d - 1;
    {   // 16 consecutive taps of each filter per thread -> z = k1 + i k2 staged in LDS
      const float4* p1 = reinterpret_cast<const float4*>(taps1 + (long)c * N + n0);
      float4* dst = reinterpret_cast<float4*>(row + P::phys(n0));
      static_for<0, 4>([&](auto qq) {
        constexpr int q = decltype(qq)::value;
        float4 a = p1[q];
        float4 bq = make_float4(0.f, 0.f, 0.f, 0.f);
        if (taps2) bq = reinterpret_cast<const float4*>(taps2 + (long)c * N + n0)[q];
        if (q == 0 && t == 0) {          // the skip weight D is one more tap at lag 0
          if (D1) a.x += D1[c];
          if (D2) bq.x += D2[c];
        }
        dst[2 * q] = make_float4(a.x, bq.x, a.y, bq.y);
        dst[2 * q + 1] = make_float4(a.z, bq.z, a.w, bq.w);
      });
    }
    row_sync<P>();
    cf x[16];
    fwd_load<P, P::R1, P::S1>(x, t, row);
    forward_to_pairs<P, false>(x, t, row, tw, g, g2);
    row_sync<P>();      // LDS is reused by the next row

    if (valid) store_filter_spectrum<P>(x, t, scale, spec + (long)c * 8 * T + t);
  }
}

// ------------------------------------------------------------------------------------------
// host-side dispatch
// ------------------------------------------------------------------------------------------
template <class P, typename ACT>
static int launch_mixer_core(const void* xproj, const float* u, const float* sw, const float* sb, const float* pbias,
                             const float* spec, void* y, int B, int d, hipStream_t stream) {
  const size_t lds_bytes = (size_t)P::WG_LDS * sizeof(float2) + (size_t)P::RPW * kRowConsts * sizeof(float);
  auto kern = mixer_core_kernel<P, ACT>;
  if (lds_bytes > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (e != hipSuccess) return set_error(M2_ERR_LAUNCH, "hipFuncSetAttribute(mixer_core): %s", hipGetErrorString(e));
  }
  const int rows_per_xcd = (d / 8) * B;
  const int slots_needed = (rows_per_xcd + P::RPW - 1) / P::RPW;
  // workgroups that are resident on a compute unit at once (registers or LDS, whichever binds): asked once per
  // kernel, the LDS bound is the fallback
  static int resident = 0;
  if (resident == 0) {
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, (const void*)kern, P::WG, lds_bytes) != hipSuccess || n < 1)
      n = (int)((160 * 1024) / lds_bytes) < 1 ? 1 : (int)((160 * 1024) / lds_bytes);
    resident = n;
  }
  const int per_cu = resident;
  int slots = (num_cus() / 8) * (per_cu > 8 ? 8 : per_cu);          // workgroups per XCD
  if (slots > slots_needed) slots = slots_needed;
  // every workgroup the same number of row batches: the fewest workgroups that need no extra round
  const int rounds = (slots_needed + slots - 1) / slots;
  slots = (slots_needed + rounds - 1) / rounds;
  const int grid = 8 * slots;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(P::WG), lds_bytes, stream, (const ACT*)xproj, u, sw, sb, pbias,
                     (const float4*)spec, (ACT*)y, B, d);
  return check_launch("mixer_core");
}

template <class P>
static int launch_filter_spectrum(const float* taps1, const float* taps2, const float* D1, const float* D2,
                                  float* spec, int d, const SpectrumBatch& sb, int nmixers, hipStream_t stream) {
  const size_t lds_bytes = (size_t)P::WG_LDS * sizeof(float2);
  auto kern = filter_spectrum_kernel<P>;
  if (lds_bytes > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (e != hipSuccess) return set_error(M2_ERR_LAUNCH, "hipFuncSetAttribute(filter_spectrum): %s", hipGetErrorString(e));
  }
  const int wgs_needed = (d + P::RPW - 1) / P::RPW;
  int grid = num_cus() * 2;
  if (grid > wgs_needed) grid = wgs_needed;
  hipLaunchKernelGGL(kern, dim3(grid, nmixers), dim3(P::WG), lds_bytes, stream, taps1, taps2, D1, D2, (float4*)spec, d, sb);
  return check_launch("filter_spectrum");
}

// whole-row plans, N = 2L = 256 .. 4096 (longer rows go to the split half-transform kernels)
#define M2_FOR_EACH_PLAN(X) \
  X(8, 4, 8, 1)             \
  X(9, 8, 8, 1)             \
  X(10, 16, 8, 1)           \
  X(11, 16, 16, 1)

#define X(LOGN, R1, R2, R3) static_assert(plan_offsets_ok<Plan<LOGN, R1, R2, R3>>(), "LDS offsets of the plan");
M2_FOR_EACH_PLAN(X)
#undef X

// L = 32768 (every real signal on its own, as half transforms of 16384 points), defined in fftconv_real_kernels.hip
size_t real_spectrum_bytes(int d);
int launch_mixer_real_dispatch(const void* xproj, const float* u, const float* sw, const float* sb, const float* pbias,
                               const float* spec, void* y, int B, int d, int act_dtype, hipStream_t stream);
int launch_filter_spectrum_real(const float* taps1, const float* taps2, const float* D1, const float* D2, float* spec,
                                int d, const SpectrumBatch& sb, int nmixers, hipStream_t stream);

// L = 2048 .. 16384: even/odd split half transforms, defined in fftconv_split_kernels.hip
bool split_plan_exists(int L);
int launch_mixer_split_dispatch(const void* xproj, const float* u, const float* sw, const float* sb, const float* pbias,
                                const float* spec, void* y, int B, int L, int d, int act_dtype, hipStream_t stream);
int launch_filter_spectrum_split(const float* taps1, const float* taps2, const float* D1, const float* D2, float* spec,
                                 int d, int L, const SpectrumBatch& sb, int nmixers, hipStream_t stream);

// One mixer given by pointers (sb.taps null, nmixers 1) or a batch of mixers described by `sb`.
int launch_filter_spectrum_any(const float* taps1, const float* taps2, const float* D1, const float* D2, float* spec,
                               int d, int L, const SpectrumBatch& sb, int nmixers, hipStream_t stream) {
  const int logn = ilog2(2 * L);
  if (logn == 16) return launch_filter_spectrum_real(taps1, taps2, D1, D2, spec, d, sb, nmixers, stream);
  if (split_plan_exists(L)) return launch_filter_spectrum_split(taps1, taps2, D1, D2, spec, d, L, sb, nmixers, stream);
  switch (logn) {
#define X(LOGN, R1, R2, R3) \
  case LOGN:                \
    return launch_filter_spectrum<Plan<LOGN, R1, R2, R3>>(taps1, taps2, D1, D2, spec, d, sb, nmixers, stream);
    M2_FOR_EACH_PLAN(X)
#undef X
  }
  return set_error(M2_ERR_UNSUPPORTED, "filter spectrum: no plan for L=%d", L);
}

}  // namespace m2

using namespace m2;

extern "C" int m2_fftconv_supported_seqlen(int L) {
  int n = 2 * L;
  return (n >= 256 && n <= 65536 && (n & (n - 1)) == 0) ? 1 : 0;
}

extern "C" size_t m2_filter_spectrum_bytes(int d, int L) {
  if (L == 32768) return real_spectrum_bytes(d);      // (Ke, Ko) per frequency pair and filter: 16 d L as well
  return (size_t)d * (size_t)L * 16;        // d channels x 8 slots x (2L/16) work items x float4
}

extern "C" int m2_filter_spectrum_fwd(const float* taps1, const float* taps2, const float* D1, const float* D2,
                                      float* spec, int d, int L, void* stream) {
  if (!taps1 || !spec) return set_error(M2_ERR_ARG, "m2_filter_spectrum_fwd: null pointer");
  if (d <= 0) return set_error(M2_ERR_ARG, "m2_filter_spectrum_fwd: d must be positive, got %d", d);
  if (!m2_fftconv_supported_seqlen(L))
    return set_error(M2_ERR_UNSUPPORTED, "m2_filter_spectrum_fwd: L=%d unsupported (need L a power of two in [128, 32768])", L);
  const SpectrumBatch none{nullptr, nullptr, 0, 0};
  return launch_filter_spectrum_any(taps1, taps2, D1, D2, spec, d, L, none, 1, (hipStream_t)stream);
}

extern "C" int m2_mixer_core_fwd(const void* xproj, const float* proj_bias, const float* u, const float* short_w,
                                 const float* short_b, const float* spec, void* y, int B, int L, int d, int act_dtype,
                                 void* stream) {
  if (!xproj || !short_w || !short_b || !spec || !y) return set_error(M2_ERR_ARG, "m2_mixer_core_fwd: null pointer");
  if (B <= 0 || d <= 0 || d % 8 != 0) return set_error(M2_ERR_ARG, "m2_mixer_core_fwd: need B > 0 and d a positive multiple of 8 (B=%d d=%d)", B, d);
  if ((long)B * 3 * d > 0x7fffffffL) return set_error(M2_ERR_UNSUPPORTED, "m2_mixer_core_fwd: B * 3 d = %ld rows do not fit an int", (long)B * 3 * d);
  if (act_dtype != M2_DTYPE_F32 && act_dtype != M2_DTYPE_BF16)
    return set_error(M2_ERR_ARG, "m2_mixer_core_fwd: act_dtype %d is neither M2_DTYPE_F32 nor M2_DTYPE_BF16", act_dtype);
  if (!m2_fftconv_supported_seqlen(L))
    return set_error(M2_ERR_UNSUPPORTED, "m2_mixer_core_fwd: L=%d unsupported (need L a power of two in [128, 32768])", L);
  const int logn = ilog2(2 * L);
  hipStream_t s = (hipStream_t)stream;
  if (logn == 16) return launch_mixer_real_dispatch(xproj, u, short_w, short_b, proj_bias, spec, y, B, d, act_dtype, s);
  if (split_plan_exists(L)) return launch_mixer_split_dispatch(xproj, u, short_w, short_b, proj_bias, spec, y, B, L, d, act_dtype, s);
  switch (logn) {
#define X(LOGN, R1, R2, R3)                                                                                       \
  case LOGN:                                                                                                      \
    return act_dtype == M2_DTYPE_F32                                                                              \
               ? launch_mixer_core<Plan<LOGN, R1, R2, R3>, float>(xproj, u, short_w, short_b, proj_bias, spec, y, B, d, s) \
               : launch_mixer_core<Plan<LOGN, R1, R2, R3>, uint16_t>(xproj, u, short_w, short_b, proj_bias, spec, y, B, d, s);
    M2_FOR_EACH_PLAN(X)
#undef X
  }
  return set_error(M2_ERR_UNSUPPORTED, "m2_mixer_core_fwd: no plan for L=%d", L);
}

extern "C" int m2_fftconv_fwd(const void* x, const float* spec, void* y, int B, int L, int d, int act_dtype,
                              void* stream) {
  if (!x || !spec || !y) return set_error(M2_ERR_ARG, "m2_fftconv_fwd: null pointer");
  if (B <= 0 || d <= 0 || d % 8 != 0) return set_error(M2_ERR_ARG, "m2_fftconv_fwd: need B > 0 and d a positive multiple of 8 (B=%d d=%d)", B, d);
  if ((long)B * d > 0x7fffffffL) return set_error(M2_ERR_UNSUPPORTED, "m2_fftconv_fwd: B * d = %ld rows do not fit an int", (long)B * d);
  if (act_dtype != M2_DTYPE_F32 && act_dtype != M2_DTYPE_BF16)
    return set_error(M2_ERR_ARG, "m2_fftconv_fwd: act_dtype %d is neither M2_DTYPE_F32 nor M2_DTYPE_BF16", act_dtype);
  if (!m2_fftconv_supported_seqlen(L))
    return set_error(M2_ERR_UNSUPPORTED, "m2_fftconv_fwd: L=%d unsupported (need L a power of two in [128, 32768])", L);
  const int logn = ilog2(2 * L);
  hipStream_t s = (hipStream_t)stream;
  if (logn == 16) return launch_mixer_real_dispatch(x, nullptr, nullptr, nullptr, nullptr, spec, y, B, d, act_dtype, s);
  if (split_plan_exists(L)) return launch_mixer_split_dispatch(x, nullptr, nullptr, nullptr, nullptr, spec, y, B, L, d, act_dtype, s);
  switch (logn) {
#define X(LOGN, R1, R2, R3)                                                                                  \
  case LOGN:                                                                                                 \
    return act_dtype == M2_DTYPE_F32                                                                         \
               ? launch_mixer_core<Plan<LOGN, R1, R2, R3>, float>(x, nullptr, nullptr, nullptr, nullptr, spec, y, B, d, s) \
               : launch_mixer_core<Plan<LOGN, R1, R2, R3>, uint16_t>(x, nullptr, nullptr, nullptr, nullptr, spec, y, B, d, s);
    M2_FOR_EACH_PLAN(X)
#undef X
  }
  return set_error(M2_ERR_UNSUPPORTED, "m2_fftconv_fwd: no plan for L=%d", L);
}
