// LDS-resident FFT engine shared by the long-convolution kernels.
//
// E = 16 complex points per thread, T = N/16 threads per row.  The FFT is R1 x R2 (x R3) x 8, in
// place, decimation in frequency, spectrum left digit-reversed.  Every pass but the last is "load R
// points at stride S, radix-R butterfly in registers, twiddle, store in place".  The last forward
// pass and the first inverse pass are radix-8 on contiguous groups of 8 and each thread takes TWO
// groups chosen by the caller, so that spectral work that pairs frequency k with N-k can stay in
// registers.  The inverse is the exact mirror (decimation in time, natural-order output, unscaled).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fft_regs.h"
#include "m2_internal.h"

namespace m2 {

// ------------------------------------------------------------------------------------------
// plan
// ------------------------------------------------------------------------------------------
template <int LOGN_, int R1_, int R2_, int R3_>
struct Plan {
  static constexpr int LOGN = LOGN_, N = 1 << LOGN_, L = N / 2;
  static constexpr int E = 16, RP = 8;
  static constexpr int R1 = R1_, R2 = R2_, R3 = R3_;
  static constexpr int T = N / E;            // threads per row
  static constexpr int M = N / RP;           // groups of 8 in the last pass
  static constexpr int S1 = N / R1, S2 = S1 / R2, S3 = S2 / R3;
  static constexpr int RL = (R3 > 1) ? R3 : R2;   // radix of the least significant digit of a group index
  static constexpr int WG = T < 256 ? 256 : T;    // threads per workgroup
  static constexpr int RPW = WG / T;              // rows per workgroup
  // LDS layout of a row: slot of position p is p + PA (p >> SA) + PB (p >> SB); PX more slots end the row.  All pads
  // are even numbers of 8-byte slots, so 16-byte accesses stay aligned; the values per length come from enumerating
  // the 64 banks for every access pattern of the plan (staging, the strided passes, the contiguous groups) with the
  // rows a wavefront holds side by side.
  static constexpr int SA = LOGN_ == 8 ? 4 : 5, PA = 2;
  static constexpr int SB = LOGN_ == 8 ? 7 : LOGN_ == 9 ? 8 : LOGN_ == 10 ? 7 : 9;
  static constexpr int PB = LOGN_ == 8 ? 4 : LOGN_ == 11 ? 4 : 2;
  static constexpr int PX = LOGN_ == 8 ? 8 : 0;
  __host__ __device__ static constexpr int phys(int pos) { return pos + PA * (pos >> SA) + PB * (pos >> SB); }
  // Padded offset of logical offset `o` relative to a base position, valid where adding `o` to the base carries into
  // neither bit SA nor bit SB from below (checked for every access of the plan by plan_offsets_ok).
  __host__ __device__ static constexpr int poff(int o) { return o + PA * (o >> SA) + PB * (o >> SB); }
  static constexpr int ROW_LDS = N + PA * (N >> SA) + PB * (N >> SB) + PX;    // padded complex slots per row
  static constexpr int TW_LDS = R2 * (N / R1 / R2) + (R3_ > 1 ? R3_ * (N / R1 / R2 / R3_) : 0);   // twiddle tables
  static constexpr int WG_LDS = (T < 256 ? 256 / T : 1) * ROW_LDS + TW_LDS;                         // float2 slots per workgroup
  static_assert(R1 * R2 * R3 * RP == N, "radices must multiply to N");
  static_assert(S3 == RP, "last stride");
  static_assert(R1 * R2 >= E, "passes after the first must share twiddles inside a thread");
};

// phys(base + o) == phys(base) + poff(o) for every (base, offset) pair the passes of plan P use: the strided passes
// (base = the thread's butterfly position, o = j S) and the runs of 8 / 16 consecutive slots of staging and of the
// last pass.
template <class P>
constexpr bool plan_offsets_ok() {
  for (int q = 0; q < P::N / P::R1; ++q)
    for (int j = 0; j < P::R1; ++j)
      if (P::phys(q + j * P::S1) != P::phys(q) + P::poff(j * P::S1)) return false;
  for (int q = 0; q < P::N / P::R2; ++q) {
    const int base = (q / P::S2) * (P::S2 * P::R2) + q % P::S2;
    for (int j = 0; j < P::R2; ++j)
      if (P::phys(base + j * P::S2) != P::phys(base) + P::poff(j * P::S2)) return false;
  }
  if (P::R3 > 1)
    for (int q = 0; q < P::N / P::R3; ++q) {
      const int base = (q / P::S3) * (P::S3 * P::R3) + q % P::S3;
      for (int j = 0; j < P::R3; ++j)
        if (P::phys(base + j * P::S3) != P::phys(base) + P::poff(j * P::S3)) return false;
    }
  for (int g = 0; g < P::N / 16; ++g)
    for (int j = 0; j < 16; ++j)
      if (P::phys(16 * g + j) != P::phys(16 * g) + j) return false;
  return P::ROW_LDS % 2 == 0 && P::phys(P::N - 1) < P::ROW_LDS;
}

__device__ __forceinline__ cf lds_get(const float2* p, int off) {
  float2 v = p[off];
  return {v.x, v.y};
}
__device__ __forceinline__ void lds_put(float2* p, int off, cf v) { p[off] = make_float2(v.re, v.im); }

// exp(-2*pi*i*m/n), n a power of two
__device__ __forceinline__ cf unit_root(int m, int n) {
  float s, c;
  sincospif(2.0f * (float)m / (float)n, &s, &c);
  return {c, -s};
}

// Synchronisation of the threads that share a row.  A row of up to 64 threads lies inside one wavefront
// (rows are aligned runs of T threads, T a power of two): its LDS instructions execute in program order, so a
// later read by any lane sees an earlier write by any other lane and only the compiler has to be kept from
// reordering them.  Longer rows need the workgroup barrier.
template <class P>
__device__ __forceinline__ void row_sync() {
  if constexpr (P::T <= 64) {
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
  } else {
    __syncthreads();
  }
}

// ------------------------------------------------------------------------------------------
// generic passes on the row held in LDS
// ------------------------------------------------------------------------------------------
// Twiddles.  Pass 1 twiddles w_N^(m k) are different for every thread: they are computed once per
// kernel and stay in registers.  The twiddles of the later passes depend only on (m, k) with m below
// the pass stride, i.e. they are the same small table for every row and every thread block of the
// pass: tables in LDS ([k][m], conflict-free for consecutive m), built once per workgroup.
template <class P>
struct Twiddles {
  cf p1[16 / P::R1][P::R1];     // [butterfly][k], k = 1 .. R1-1: pass-1 twiddles, in registers for the whole kernel
  const float2* tab2;           // [R2][S2]
  const float2* tab3;           // [R3][S3]   (R3 > 1 only)
  static constexpr int TAB2 = P::R2 * P::S2;
  static constexpr int TAB3 = (P::R3 > 1) ? P::R3 * P::S3 : 0;
  static constexpr int LDS_SLOTS = TAB2 + TAB3;       // float2 slots after the row buffers
};

// Must be called by every thread of the workgroup (it contains a barrier).
template <class P>
__device__ __forceinline__ void twiddles_init(Twiddles<P>& tw, int t, float2* tables) {
  constexpr int NB = 16 / P::R1;
  static_for<0, NB>([&](auto ii) {
    constexpr int i = decltype(ii)::value;
    const int q = t + P::T * i;
    const cf w = unit_root(q % P::S1, P::S1 * P::R1);
    powers<P::R1>(w, tw.p1[i]);
  });
  tw.tab2 = tables;
  tw.tab3 = tables + Twiddles<P>::TAB2;
  for (int e = threadIdx.x; e < Twiddles<P>::TAB2; e += blockDim.x) {
    const int k = e / P::S2, m = e % P::S2;
    const cf w = unit_root((k * m) % (P::S2 * P::R2), P::S2 * P::R2);
    tables[e] = make_float2(w.re, w.im);
  }
  if constexpr (P::R3 > 1) {
    for (int e = threadIdx.x; e < Twiddles<P>::TAB3; e += blockDim.x) {
      const int k = e / P::S3, m = e % P::S3;
      const cf w = unit_root((k * m) % (P::S3 * P::R3), P::S3 * P::R3);
      tables[Twiddles<P>::TAB2 + e] = make_float2(w.re, w.im);
    }
  }
  __syncthreads();
}

// pass-1 twiddles pw[k] = w^k of butterfly I of this thread
template <class P, int I>
__device__ __forceinline__ void pass1_twiddles(const Twiddles<P>& tw, cf (&pw)[P::R1]) {
  static_for<1, P::R1>([&](auto k) { pw[decltype(k)::value] = tw.p1[I][decltype(k)::value]; });
}

// twiddle w^(m k) of pass PASS (2 or 3), shared table in LDS
template <class P, int PASS, int S, int K>
__device__ __forceinline__ cf table_twiddle(const Twiddles<P>& tw, int m) {
  const float2 v = (PASS == 2 ? tw.tab2 : tw.tab3)[K * S + m];
  return {v.x, v.y};
}

// forward: registers hold natural-order inputs of E/R butterflies; butterfly, twiddle, store.
template <class P, int PASS, int R, int S, bool ZERO_UPPER>
__device__ __forceinline__ void fwd_compute_store(cf (&x)[16], int t, float2* row, const Twiddles<P>& tw) {
  constexpr int NB = 16 / R;
  static_for<0, NB>([&](auto ii) {
    constexpr int i = decltype(ii)::value;
    const int q = t + P::T * i;
    const int b = q / S, m = q % S;
    if constexpr (ZERO_UPPER) dif_zero_upper<R, i * R, 16>(x);
    else dif<R, i * R, 16>(x);
    float2* pb = row + P::phys(b * (S * R) + m);
    constexpr int bits = ilog2(R);
    cf pw[PASS == 1 ? P::R1 : 1];
    if constexpr (PASS == 1) pass1_twiddles<P, i>(tw, pw);
    static_for<0, R>([&](auto kk) {
      constexpr int k = decltype(kk)::value;
      cf v = x[i * R + bitrev(k, bits)];
      if constexpr (k > 0) {
        if constexpr (PASS == 1) v = cmul(v, pw[k]);
        else v = cmul(v, table_twiddle<P, PASS, S, k>(tw, m));
      }
      lds_put(pb, P::poff(k * S), v);
    });
  });
}

template <class P, int R, int S>
__device__ __forceinline__ void fwd_load(cf (&x)[16], int t, const float2* row) {
  constexpr int NB = 16 / R;
  static_for<0, NB>([&](auto ii) {
    constexpr int i = decltype(ii)::value;
    const int q = t + P::T * i;
    const int b = q / S, m = q % S;
    const float2* pb = row + P::phys(b * (S * R) + m);
    static_for<0, R>([&](auto jj) {
      constexpr int j = decltype(jj)::value;
      x[i * R + j] = lds_get(pb, P::poff(j * S));
    });
  });
}

// inverse: load digit k into bit-reversed register, conj twiddle, inverse butterfly (natural out)
template <class P, int PASS, int R, int S, bool LOWER_ONLY>
__device__ __forceinline__ void inv_load_compute(cf (&x)[16], int t, const float2* row, const Twiddles<P>& tw) {
  constexpr int NB = 16 / R;
  static_for<0, NB>([&](auto ii) {
    constexpr int i = decltype(ii)::value;
    const int q = t + P::T * i;
    const int b = q / S, m = q % S;
    const float2* pb = row + P::phys(b * (S * R) + m);
    constexpr int bits = ilog2(R);
    cf pw[PASS == 1 ? P::R1 : 1];
    if constexpr (PASS == 1) pass1_twiddles<P, i>(tw, pw);
    static_for<0, R>([&](auto kk) {
      constexpr int k = decltype(kk)::value;
      cf v = lds_get(pb, P::poff(k * S));
      if constexpr (k > 0) {
        if constexpr (PASS == 1) v = cmulc(v, pw[k]);
        else v = cmulc(v, table_twiddle<P, PASS, S, k>(tw, m));
      }
      x[i * R + bitrev(k, bits)] = v;
    });
    if constexpr (LOWER_ONLY) dit_lower_only<R, i * R, 16>(x);
    else dit<R, i * R, 16>(x);
  });
}

template <class P, int R, int S>
__device__ __forceinline__ void inv_store(const cf (&x)[16], int t, float2* row) {
  constexpr int NB = 16 / R;
  static_for<0, NB>([&](auto ii) {
    constexpr int i = decltype(ii)::value;
    const int q = t + P::T * i;
    const int b = q / S, m = q % S;
    float2* pb = row + P::phys(b * (S * R) + m);
    static_for<0, R>([&](auto jj) {
      constexpr int j = decltype(jj)::value;
      lds_put(pb, P::poff(j * S), x[i * R + j]);
    });
  });
}

// group taken by work item w in the paired radix-8 pass, and the group with the mirrored frequencies
template <class P>
__device__ __forceinline__ void paired_groups(int w, int& g, int& g2) {
  constexpr int RL = P::RL, R1 = P::R1, R2 = P::R2, R3 = P::R3;
  g = (w / (RL / 2)) * RL + (w % (RL / 2));
  if (w == 0) {            // groups 0 (k_low = 0) and RL/2 (k_low = M/2) are both self-mirrored
    g2 = RL / 2;
    return;
  }
  int k1 = g / (R2 * R3), k2 = (g / R3) % R2, k3 = g % R3;
  if (k1) {
    k1 = R1 - k1; k2 = R2 - 1 - k2; k3 = R3 - 1 - k3;
  } else if (k2) {
    k2 = R2 - k2; k3 = R3 - 1 - k3;
  } else {
    k3 = R3 - k3;
  }
  g2 = (k1 * R2 + k2) * R3 + k3;
}

// ------------------------------------------------------------------------------------------
// forward FFT up to (and including) the paired radix-8 pass.  On return x[0..8) holds group g
// and x[8..16) holds group g2, both in bit-reversed register order.
// ------------------------------------------------------------------------------------------
template <class P, bool ZERO_UPPER>
__device__ __forceinline__ void forward_to_pairs(cf (&x)[16], int t, float2* row, const Twiddles<P>& tw, int g, int g2) {
  fwd_compute_store<P, 1, P::R1, P::S1, ZERO_UPPER>(x, t, row, tw);
  row_sync<P>();
  fwd_load<P, P::R2, P::S2>(x, t, row);
  fwd_compute_store<P, 2, P::R2, P::S2, false>(x, t, row, tw);
  row_sync<P>();
  if constexpr (P::R3 > 1) {
    fwd_load<P, P::R3, P::S3>(x, t, row);
    fwd_compute_store<P, 3, P::R3, P::S3, false>(x, t, row, tw);
    row_sync<P>();
  }
  {
    const float2* pa = row + P::phys(g * 8);
    const float2* pb = row + P::phys(g2 * 8);
    static_for<0, 8>([&](auto jj) {
      constexpr int j = decltype(jj)::value;
      x[j] = lds_get(pa, j);
      x[8 + j] = lds_get(pb, j);
    });
  }
  dif<8, 0, 16>(x);
  dif<8, 8, 16>(x);
}

// One spectral pair: za sits at frequency k, zb at N-k.  Returns W[k] in za and W[N-k] in zb.  The 1/2 of the even/odd
// separation is folded into the stored spectra (store_filter_spectrum).
__device__ __forceinline__ void pair_multiply(cf& za, cf& zb, float4 K) {
  cf A = {za.re + zb.re, za.im - zb.im};                          // Z[k] + conj Z[N-k]
  cf Bq = {za.im + zb.im, zb.re - za.re};                         // (Z[k] - conj Z[N-k]) / i
  cf Pp = cmul(A, cf{K.x, K.y});
  cf Q = cmul(Bq, cf{K.z, K.w});
  za = {Pp.re - Q.im, Pp.im + Q.re};                               // P + iQ
  zb = {Pp.re + Q.im, Q.re - Pp.im};                               // conj(P) + i conj(Q)
}


// Inverse of forward_to_pairs: x[0..8) / x[8..16) hold groups g / g2 in bit-reversed register order.
// On return x[i R1 + j] is the (unscaled) time sample n = t + T i + j S1; with LOWER_ONLY only j < R1/2.
template <class P, bool LOWER_ONLY>
__device__ __forceinline__ void inverse_from_pairs(cf (&x)[16], int t, float2* row, const Twiddles<P>& tw, int g,
                                                   int g2) {
  dit<8, 0, 16>(x);
  dit<8, 8, 16>(x);
  {
    float2* pa = row + P::phys(g * 8);
    float2* pb = row + P::phys(g2 * 8);
    static_for<0, 8>([&](auto jj) {
      constexpr int j = decltype(jj)::value;
      lds_put(pa, j, x[j]);
      lds_put(pb, j, x[8 + j]);
    });
  }
  row_sync<P>();
  if constexpr (P::R3 > 1) {
    inv_load_compute<P, 3, P::R3, P::S3, false>(x, t, row, tw);
    inv_store<P, P::R3, P::S3>(x, t, row);
    row_sync<P>();
  }
  inv_load_compute<P, 2, P::R2, P::S2, false>(x, t, row, tw);
  inv_store<P, P::R2, P::S2>(x, t, row);
  row_sync<P>();
  inv_load_compute<P, 1, P::R1, P::S1, LOWER_ONLY>(x, t, row, tw);
}

// After forward_to_pairs on z = k1 + i k2 (two real filters packed into one complex row): separates the two
// spectra and stores them in the order the mixer core's multiply reads them, sp[slot * T] as float4 = (K1.re,
// K1.im, K2.re, K2.im) for the frequency in slot `slot` of this work item's group; work item 0 holds DC and Nyquist
// (real, packed into slot 0: multiplied directly, so without the two halves) and the two self-mirrored groups.
// `scale` carries the 1/2 of this separation, the 1/2 of the separation in pair_multiply and the 1/N of the convolution.
template <class P>
__device__ __forceinline__ void store_filter_spectrum(const cf (&x)[16], int t, float scale, float4* __restrict__ sp) {
  float4 K[8];
  auto split = [&](cf za, cf zb) -> float4 {
    // K1 = (za + conj zb) * scale ; K2 = (za - conj zb) / i * scale
    return make_float4(scale * (za.re + zb.re), scale * (za.im - zb.im), scale * (za.im + zb.im),
                       scale * (zb.re - za.re));
  };
  if (t != 0) {
    static_for<0, 8>([&](auto jj) {
      constexpr int j = decltype(jj)::value;
      K[j] = split(x[bitrev(j, 3)], x[8 + bitrev(7 - j, 3)]);
    });
  } else {
    const cf z0 = x[bitrev(0, 3)], z4 = x[bitrev(4, 3)];
    K[0] = make_float4(4.f * scale * z0.re, 4.f * scale * z4.re, 4.f * scale * z0.im, 4.f * scale * z4.im);
    static_for<1, 4>([&](auto jj) {
      constexpr int j = decltype(jj)::value;
      K[j] = split(x[bitrev(j, 3)], x[bitrev(8 - j, 3)]);
    });
    static_for<0, 4>([&](auto jj) {
      constexpr int j = decltype(jj)::value;
      K[4 + j] = split(x[8 + bitrev(j, 3)], x[8 + bitrev(7 - j, 3)]);
    });
  }
  static_for<0, 8>([&](auto s) { sp[decltype(s)::value * P::T] = K[decltype(s)::value]; });
}

}  // namespace m2
