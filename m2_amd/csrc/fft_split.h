// Device-side building blocks of the long-convolution kernels that run a row as half-length transforms
// through one LDS buffer (fftconv_split_kernels.hip, fftconv_real_kernels.hip): the plan, the LDS padding,
// the three passes of a half transform, the dealing of groups of 16 to work items, and the paired spectral
// multiply of two signals packed into one complex row.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fft_engine.h"

namespace m2 {

// LDS padding of the row buffer: one slot after every 16 and one more after every 256.  Chosen by measurement among
// the paddings whose offsets stay linear for every access pattern (split_offsets_ok below): at L = 8192 the
// bank-conflict counter of the mixer kernel reads 2.6 M cycles per launch with it against 9.4 M for two slots after
// every 32 plus one after every 512 (which a 64-bank model of 8-byte accesses rates conflict-free), 5.5 M for
// (16, 512) and 35 M for one slot after every 8; the kernel is 2 - 3 % faster.
__host__ __device__ constexpr int sphys(int pos) { return pos + (pos >> 4) + (pos >> 8); }
// Padded offset of logical offset `o` relative to a base position: valid where adding `o` to the base carries
// neither into bit 4 nor into bit 8 from below (every access in this file: offsets are multiples of 256 on a
// base below 256, multiples of 16 below 256 on a base whose low byte is below 16, or below 16 on a base
// that is a multiple of 16).
constexpr int spoff(int o) { return o + (o >> 4) + (o >> 8); }

template <int LOGL_, int R1_, int R2_>
struct SplitPlan {
  static constexpr int LOGL = LOGL_, L = 1 << LOGL_, N = 2 * L;
  static constexpr int E = 32, RP = 16;
  static constexpr int R1 = R1_, R2 = R2_;
  static constexpr int T = L / E;                 // threads per row = workgroup size
  static constexpr int M = L / RP;                // groups of 16 in the last pass
  static constexpr int S1 = L / R1, S2 = S1 / R2;
  static constexpr int NB1 = E / R1, NB2 = E / R2;
  static constexpr int ROW_LDS = L + (L >> 4) + (L >> 8);    // padded complex slots of the row buffer
  static constexpr int TAB2 = R2 * S2;            // pass-2 twiddle table
  static constexpr int WG_LDS = ROW_LDS + TAB2;   // float2 slots per workgroup
  static_assert(R1 * R2 * RP == L, "radices must multiply to L");
  static_assert(S2 == RP, "last stride");
  static_assert(R1 % 8 == 0 && R1 <= 32 && R2 <= 32, "radix range");
};

// sphys(base + o) == sphys(base) + spoff(o) for every (base, offset) pair the passes of plan P use
template <class P>
constexpr bool split_offsets_ok() {
  for (int q = 0; q < P::S1; ++q)
    for (int j = 0; j < P::R1; ++j)
      if (sphys(q + j * P::S1) != sphys(q) + spoff(j * P::S1)) return false;
  for (int q = 0; q < P::L / P::R2; ++q) {
    const int base = (q / P::S2) * (P::S2 * P::R2) + q % P::S2;
    for (int j = 0; j < P::R2; ++j)
      if (sphys(base + j * P::S2) != sphys(base) + spoff(j * P::S2)) return false;
  }
  for (int g = 0; g < P::M; ++g)
    for (int j = 0; j < 16; ++j)
      if (sphys(16 * g + j) != sphys(16 * g) + j) return false;
  return sphys(P::L - 1) < P::ROW_LDS;
}

// cos of 2 pi k / 64 for k = 0 .. 16
constexpr float kCos64[17] = {1.0f,
                              0.99518472667219688624f,
                              0.98078528040323044913f,
                              0.95694033573220886494f,
                              0.92387953251128675613f,
                              0.88192126434835502971f,
                              0.83146961230254523708f,
                              0.77301045336273696081f,
                              0.70710678118654752440f,
                              0.63439328416364549822f,
                              0.55557023301960222474f,
                              0.47139673682599764856f,
                              0.38268343236508977173f,
                              0.29028467725446236764f,
                              0.19509032201612826785f,
                              0.09801714032956060199f,
                              0.0f};
constexpr float cos64(int k) {
  k &= 63;
  return k <= 16 ? kCos64[k] : k <= 32 ? -kCos64[32 - k] : k <= 48 ? -kCos64[k - 32] : kCos64[64 - k];
}
constexpr float sin64(int k) { return cos64(k - 16 + 64); }

// multiply by exp(-+ 2 pi i K / 64): forward (INV = false) uses the minus sign
template <int K, bool INV>
__device__ __forceinline__ cf mul_w64(cf v) {
  constexpr int k = ((K % 64) + 64) % 64;
  if constexpr (k % 2 == 0) {
    return mul_w32<k / 2, INV>(v);
  } else {
    constexpr float c = cos64(k);
    constexpr float s = INV ? sin64(k) : -sin64(k);
    return {c * v.re - s * v.im, c * v.im + s * v.re};
  }
}

// ------------------------------------------------------------------------------------------
// first-pass twiddles.  b = w_N^q (kept per thread).  Even half: t_k = b^(2k); odd half: t_k = b^(2k+1).
// With k = 8 a + r they are A[a] * B[r], B[r] = (b^2)^r and A[a] = (b^2)^(8a) (times b for the odd half):
// 22 live registers instead of a table of 2 R1, one extra product per point, depth at most 7 products.
// ------------------------------------------------------------------------------------------
template <int R1>
struct Pass1Powers {
  cf B[8];
  cf A[R1 / 8];
};
template <int R1, bool ODD>
__device__ __forceinline__ void pass1_powers(cf b, Pass1Powers<R1>& p) {
  asm volatile("" : "+v"(b.re), "+v"(b.im));     // rebuilt where used: keeps them out of long-lived registers
  const cf b2 = cmul(b, b);
  p.B[1] = b2;
  p.B[2] = cmul(b2, b2);
  p.B[3] = cmul(p.B[2], b2);
  p.B[4] = cmul(p.B[2], p.B[2]);
  p.B[5] = cmul(p.B[4], b2);
  p.B[6] = cmul(p.B[4], p.B[2]);
  p.B[7] = cmul(p.B[4], p.B[3]);
  const cf a8 = cmul(p.B[4], p.B[4]);
  if constexpr (ODD) {
    p.A[0] = b;
    p.A[1] = cmul(b, a8);
  } else {
    p.A[1] = a8;
  }
  if constexpr (R1 / 8 > 2) {
    p.A[2] = cmul(p.A[1], a8);
    p.A[3] = cmul(p.A[2], a8);
  }
}
template <int R1, bool ODD, int K>
__device__ __forceinline__ cf pass1_twiddle(const Pass1Powers<R1>& p) {
  constexpr int a = K / 8, r = K % 8;
  if constexpr (!ODD && a == 0) return p.B[r];
  else if constexpr (r == 0) return p.A[a];
  else return cmul(p.A[a], p.B[r]);
}

// registers <- first-pass layout: x[i R1 + j] = row[q + S1 j], q = t + T i
template <class P>
__device__ __forceinline__ void pass1_load(cf (&x)[32], int t, const float2* row) {
  static_for<0, P::NB1>([&](auto ii) {
    constexpr int i = decltype(ii)::value;
    const float2* pb = row + sphys(t + P::T * i);
    static_for<0, P::R1>([&](auto jj) {
      constexpr int j = decltype(jj)::value;
      x[i * P::R1 + j] = lds_get(pb, spoff(j * P::S1));
    });
  });
}
template <class P>
__device__ __forceinline__ void pass1_store(const cf (&x)[32], int t, float2* row) {
  static_for<0, P::NB1>([&](auto ii) {
    constexpr int i = decltype(ii)::value;
    float2* pb = row + sphys(t + P::T * i);
    static_for<0, P::R1>([&](auto jj) {
      constexpr int j = decltype(jj)::value;
      lds_put(pb, spoff(j * P::S1), x[i * P::R1 + j]);
    });
  });
}

// forward first pass of one half transform, registers (first-pass layout) -> LDS
template <class P, bool ODD>
__device__ __forceinline__ void fwd_pass1(cf (&x)[32], int t, float2* row, const cf (&b)[P::NB1]) {
  constexpr int R = P::R1, bits = ilog2(R);
  static_for<0, P::NB1>([&](auto ii) {
    constexpr int i = decltype(ii)::value;
    if constexpr (ODD)
      static_for<1, R>([&](auto jj) {
        constexpr int j = decltype(jj)::value;
        x[i * R + j] = mul_w64<j * (32 / R), false>(x[i * R + j]);
      });
    dif<R, i * R, 32>(x);
    Pass1Powers<R> pw;
    pass1_powers<R, ODD>(b[i], pw);
    float2* pb = row + sphys(t + P::T * i);
    static_for<0, R>([&](auto kk) {
      constexpr int k = decltype(kk)::value;
      cf v = x[i * R + bitrev(k, bits)];
      if constexpr (ODD || k > 0) v = cmul(v, pass1_twiddle<R, ODD, k>(pw));
      lds_put(pb, spoff(k * P::S1), v);
    });
  });
}
// inverse first pass: LDS -> registers; x[i R1 + j] = sample q + S1 j of IFFT_L (even half) or of
// w_N^-n IFFT_L (odd half), unscaled
template <class P, bool ODD>
__device__ __forceinline__ void inv_pass1(cf (&x)[32], int t, const float2* row, const cf (&b)[P::NB1]) {
  constexpr int R = P::R1, bits = ilog2(R);
  static_for<0, P::NB1>([&](auto ii) {
    constexpr int i = decltype(ii)::value;
    Pass1Powers<R> pw;
    pass1_powers<R, ODD>(b[i], pw);
    const float2* pb = row + sphys(t + P::T * i);
    static_for<0, R>([&](auto kk) {
      constexpr int k = decltype(kk)::value;
      cf v = lds_get(pb, spoff(k * P::S1));
      if constexpr (ODD || k > 0) v = cmulc(v, pass1_twiddle<R, ODD, k>(pw));
      x[i * R + bitrev(k, bits)] = v;
    });
    dit<R, i * R, 32>(x);
    if constexpr (ODD)
      static_for<1, R>([&](auto jj) {
        constexpr int j = decltype(jj)::value;
        x[i * R + j] = mul_w64<j * (32 / R), true>(x[i * R + j]);
      });
  });
}

// second pass (radix R2 at stride 16), in place in LDS, twiddles from the shared table tab2[k][m]
template <class P>
__device__ __forceinline__ void fwd_pass2(cf (&x)[32], int t, float2* row, const float2* tab2) {
  constexpr int R = P::R2, S = P::S2, bits = ilog2(R);
  static_for<0, P::NB2>([&](auto ii) {
    constexpr int i = decltype(ii)::value;
    const int q = t + P::T * i, blk = q / S, m = q % S;
    float2* pb = row + sphys(blk * (S * R) + m);
    static_for<0, R>([&](auto jj) {
      constexpr int j = decltype(jj)::value;
      x[i * R + j] = lds_get(pb, spoff(j * S));
    });
    dif<R, i * R, 32>(x);
    static_for<0, R>([&](auto kk) {
      constexpr int k = decltype(kk)::value;
      cf v = x[i * R + bitrev(k, bits)];
      if constexpr (k > 0) {
        const float2 w = tab2[k * S + m];
        v = cmul(v, cf{w.x, w.y});
      }
      lds_put(pb, spoff(k * S), v);
    });
  });
}
template <class P>
__device__ __forceinline__ void inv_pass2(cf (&x)[32], int t, float2* row, const float2* tab2) {
  constexpr int R = P::R2, S = P::S2, bits = ilog2(R);
  static_for<0, P::NB2>([&](auto ii) {
    constexpr int i = decltype(ii)::value;
    const int q = t + P::T * i, blk = q / S, m = q % S;
    float2* pb = row + sphys(blk * (S * R) + m);
    static_for<0, R>([&](auto kk) {
      constexpr int k = decltype(kk)::value;
      cf v = lds_get(pb, spoff(k * S));
      if constexpr (k > 0) {
        const float2 w = tab2[k * S + m];
        v = cmulc(v, cf{w.x, w.y});
      }
      x[i * R + bitrev(k, bits)] = v;
    });
    dit<R, i * R, 32>(x);
    static_for<0, R>([&](auto jj) {
      constexpr int j = decltype(jj)::value;
      lds_put(pb, spoff(j * S), x[i * R + j]);
    });
  });
}

// last pass: two contiguous groups of 16 per thread, radix 16 in registers (bit-reversed order)
template <class P>
__device__ __forceinline__ void fwd_groups(cf (&x)[32], const float2* row, int ga, int gb) {
  const float2* pa = row + sphys(ga * 16);
  const float2* pb = row + sphys(gb * 16);
  static_for<0, 16>([&](auto jj) {
    constexpr int j = decltype(jj)::value;
    x[j] = lds_get(pa, j);
    x[16 + j] = lds_get(pb, j);
  });
  dif<16, 0, 32>(x);
  dif<16, 16, 32>(x);
}
template <class P>
__device__ __forceinline__ void inv_groups(cf (&x)[32], float2* row, int ga, int gb) {
  dit<16, 0, 32>(x);
  dit<16, 16, 32>(x);
  float2* pa = row + sphys(ga * 16);
  float2* pb = row + sphys(gb * 16);
  static_for<0, 16>([&](auto jj) {
    constexpr int j = decltype(jj)::value;
    lds_put(pa, j, x[j]);
    lds_put(pb, j, x[16 + j]);
  });
}

// Groups of 16 taken by work item w in the last pass.  Group index g = k1 R2 + k2 holds the frequencies
// k = k1 + R1 k2 + R1 R2 j (slot j).
// Even half: the partner is the group with the mirrored frequencies (L - k) mod L.  Work items are dealt so that
// consecutive items take consecutive groups (no LDS bank conflicts): first the groups with 1 <= k1 < R1/2 (all
// k2), whose partners have k1 > R1/2; then k1 = 0 (partners inside k1 = 0: k2 <-> R2 - k2), where the item with
// k2 = 0 is the special one that takes the two self-mirrored groups 0 and R2/2; then k1 = R1/2 (k2 <-> R2-1-k2).
// Odd half: the partner is the complement group (frequencies L - 1 - k): item w takes group w and M - 1 - w.
template <class P>
struct SplitGroups {
  int ge, gm;       // even half: group and mirrored group
  int go, gc;       // odd half: group and complement group
  bool special;     // even half: this item holds groups 0 and R2/2 (DC, Nyquist, self-mirrored slots)
};
template <class P>
__device__ __forceinline__ SplitGroups<P> split_groups(int w) {
  constexpr int R1 = P::R1, R2 = P::R2;
  constexpr int BULK = (R1 / 2 - 1) * R2;
  SplitGroups<P> s;
  s.go = w;
  s.gc = P::M - 1 - w;
  s.special = (w == BULK);
  int k1, k2;
  if (w < BULK) {
    k1 = 1 + w / R2;
    k2 = w % R2;
  } else if (w < BULK + R2 / 2) {
    k1 = 0;
    k2 = w - BULK;
  } else {
    k1 = R1 / 2;
    k2 = w - BULK - R2 / 2;
  }
  s.ge = k1 * R2 + k2;
  if (s.special) {
    s.gm = R2 / 2;
  } else if (k1) {
    s.gm = (R1 - k1) * R2 + (R2 - 1 - k2);
  } else {
    s.gm = R2 - k2;
  }
  return s;
}

// One spectral pair: za sits at frequency kappa, zb at N - kappa.  Returns W[kappa] in za and W[N - kappa] in
// zb.  The 1/2 of the even/odd separation is folded into the stored spectra.
__device__ __forceinline__ void pair_multiply_half(cf& za, cf& zb, float4 K) {
  const cf A = {za.re + zb.re, za.im - zb.im};         // Z[k] + conj Z[N-k]
  const cf Bq = {za.im + zb.im, zb.re - za.re};        // (Z[k] - conj Z[N-k]) / i
  const cf Pp = cmul(A, cf{K.x, K.y});
  const cf Q = cmul(Bq, cf{K.z, K.w});
  za = {Pp.re - Q.im, Pp.im + Q.re};                   // P + iQ
  zb = {Pp.re + Q.im, Q.re - Pp.im};                   // conj(P) + i conj(Q)
}

// spectral multiply of the 16 + 16 points a thread holds after fwd_groups, slots 8 H .. 8 H + 7.
// EVEN_SPECIAL: this is work item 0 of the even half (DC, Nyquist and the two self-mirrored groups).
template <bool EVEN_SPECIAL, int H>
__device__ __forceinline__ void multiply_batch(cf (&x)[32], const float4 (&K)[8]) {
  static_for<0, 8>([&](auto ss) {
    constexpr int s = 8 * H + decltype(ss)::value;
    const float4 k = K[decltype(ss)::value];
    if constexpr (!EVEN_SPECIAL) {
      pair_multiply_half(x[bitrev(s, 4)], x[16 + bitrev(15 - s, 4)], k);
    } else if constexpr (s == 0) {
      // DC and Nyquist are self-paired and their filter values are real: K = (K1(0), K1(N/2), K2(0), K2(N/2))
      x[bitrev(0, 4)] = {x[bitrev(0, 4)].re * k.x, x[bitrev(0, 4)].im * k.z};
      x[bitrev(8, 4)] = {x[bitrev(8, 4)].re * k.y, x[bitrev(8, 4)].im * k.w};
    } else if constexpr (s < 8) {
      pair_multiply_half(x[bitrev(s, 4)], x[bitrev(16 - s, 4)], k);              // group 0: slot s <-> 16 - s
    } else {
      pair_multiply_half(x[16 + bitrev(s - 8, 4)], x[16 + bitrev(23 - s, 4)], k);   // group R2/2: slot j <-> 15 - j
    }
  });
}
template <int H>
__device__ __forceinline__ void load_spectrum_batch(float4 (&K)[8], const float4* __restrict__ sp, int T) {
  static_for<0, 8>([&](auto s) { K[decltype(s)::value] = sp[(8 * H + decltype(s)::value) * T]; });
}

// workgroup barrier that the instruction scheduler does not move code across either: the phases on its
// two sides each fit the register budget, a merged schedule of both does not
__device__ __forceinline__ void phase_barrier() {
  __builtin_amdgcn_sched_barrier(0);
  __syncthreads();
  __builtin_amdgcn_sched_barrier(0);
}

template <class P>
__device__ __forceinline__ void tab2_init(float2* tab2) {
  for (int e = threadIdx.x; e < P::TAB2; e += blockDim.x) {
    const int k = e / P::S2, m = e % P::S2;
    const cf w = unit_root((k * m) % (P::S2 * P::R2), P::S2 * P::R2);
    tab2[e] = make_float2(w.re, w.im);
  }
}

// One half transform: forward passes from registers (first-pass layout), spectral multiply, inverse passes
// back to registers (first-pass layout).  Contains 4 barriers; touches only LDS slots this thread owns
// in the first-pass layout at entry and exit, so halves can follow each other without a barrier.
template <class P, bool ODD>
__device__ __forceinline__ void half_convolution(cf (&x)[32], int t, float2* row, const float2* tab2,
                                                 const cf (&b)[P::NB1], const float4* __restrict__ sp, int ga, int gb,
                                                 bool special) {
  fwd_pass1<P, ODD>(x, t, row, b);
  phase_barrier();
  fwd_pass2<P>(x, t, row, tab2);
  phase_barrier();
  float4 K0[8], K1[8];
  load_spectrum_batch<0>(K0, sp, P::T);
  fwd_groups<P>(x, row, ga, gb);
  __builtin_amdgcn_sched_barrier(0);
  if (!ODD && special) {
    multiply_batch<true, 0>(x, K0);
    load_spectrum_batch<1>(K1, sp, P::T);
    multiply_batch<true, 1>(x, K1);
  } else {
    multiply_batch<false, 0>(x, K0);
    load_spectrum_batch<1>(K1, sp, P::T);
    multiply_batch<false, 1>(x, K1);
  }
  __builtin_amdgcn_sched_barrier(0);
  inv_groups<P>(x, row, ga, gb);
  phase_barrier();
  inv_pass2<P>(x, t, row, tab2);
  phase_barrier();
  inv_pass1<P, ODD>(x, t, row, b);
}

}  // namespace m2
