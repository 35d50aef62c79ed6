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
#include "row_io.h"

namespace m2 {

// LDS padding of the row buffer: two slots after every 32 and one more after every 512.  With it the staging
// layout (32 consecutive slots per thread), the first pass (consecutive threads, consecutive slots at stride
// L / R1) and the second pass (16 consecutive slots per 256) are all free of bank conflicts for 8-byte
// accesses (checked by enumerating the 64 banks for every access pattern of the L = 8192 plan).
__device__ __forceinline__ int sphys(int pos) { return pos + 2 * (pos >> 5) + (pos >> 9); }
// Padded offset of logical offset `o` relative to a base position: valid where adding `o` to the base carries
// neither into bit 5 nor into bit 9 from below (every access in this file: offsets are multiples of 256 on a
// base below 256, multiples of 16 below 256 on a base whose low byte is below 16, or below 16 / 32 on a base
// that is a multiple of 16 / 32).
constexpr int spoff(int o) { return o + 2 * (o >> 5) + (o >> 9); }

template <int LOGL_, int R1_, int R2_>
struct SplitPlan {
  static constexpr int LOGL = LOGL_, L = 1 << LOGL_, N = 2 * L;
  static constexpr int E = 32, RP = 16;
  static constexpr int R1 = R1_, R2 = R2_;
  static constexpr int T = L / E;                 // threads per row = workgroup size
  static constexpr int M = L / RP;                // groups of 16 in the last pass
  static constexpr int S1 = L / R1, S2 = S1 / R2;
  static constexpr int NB1 = E / R1, NB2 = E / R2;
  static constexpr int ROW_LDS = L + 2 * (L >> 5) + (L >> 9);    // padded complex slots of the row buffer
  static constexpr int TAB2 = R2 * S2;            // pass-2 twiddle table
  static constexpr int WG_LDS = ROW_LDS + TAB2;   // float2 slots per workgroup
  static_assert(R1 * R2 * RP == L, "radices must multiply to L");
  static_assert(S2 == RP, "last stride");
  static_assert(R1 % 8 == 0 && R1 <= 32 && R2 <= 32, "radix range");
};

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
      RawRow<ACT, 4> r1, r2, rv;
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
      __builtin_amdgcn_sched_barrier(0);
      static_for<0, 4>([&](auto qq) {
        constexpr int q = decltype(qq)::value;
        const int n = n0 + 8 * q;
        float in[10], a[8], gt[8];
        if constexpr (FULL) {
          r1.template expand<q>(n, p1, in);
          static_for<0, 8>([&](auto ee) {
            constexpr int e = decltype(ee)::value;
            a[e] = b1 + w1[0] * in[e] + w1[1] * in[e + 1] + w1[2] * in[e + 2];
          });
          rv.template expand<q>(n, pv, in);
          static_for<0, 8>([&](auto ee) {
            constexpr int e = decltype(ee)::value;
            a[e] *= bv + wv[0] * in[e] + wv[1] * in[e + 1] + wv[2] * in[e + 2];
          });
          r2.template expand<q>(n, p2, in);
          static_for<0, 8>([&](auto ee) {
            constexpr int e = decltype(ee)::value;
            gt[e] = b2 + w2[0] * in[e] + w2[1] * in[e + 1] + w2[2] * in[e + 2];
          });
        } else {
          // plain long convolution: xproj is a single (d, B, L) signal, no short conv, no gates
          r1.template expand<q>(n, 0.f, in);
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
    const float* __restrict__ taps1,    // (d, N) bidirectional taps of filter_fn
    const float* __restrict__ taps2,    // (d, N) bidirectional taps of filter_fn2 (may be null)
    const float* __restrict__ D1,       // (d) skip weight of filter_fn, added to tap 0 (may be null)
    const float* __restrict__ D2,       // (d) skip weight of filter_fn2 (may be null)
    float4* __restrict__ spec,          // (d, 2, 16, T)
    int d) {
  constexpr int L = P::L, N = P::N, T = P::T;
  extern __shared__ float2 lds[];
  float2* row = lds;
  float2* tab2 = lds + P::ROW_LDS;
  const int t = threadIdx.x;

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

  // work item = (channel, half transform): 2 d items spread evenly over the grid
  for (int item = blockIdx.x; item < 2 * d; item += gridDim.x) {
    const int c = item >> 1;
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
  hipLaunchKernelGGL(kern, dim3(8 * slots), dim3(P::T), lds_bytes, stream, (const ACT*)xproj, u, sw, sb, pbias,
                     (const float4*)spec, (ACT*)y, B, d);
  return check_launch("mixer_split");
}

template <class P>
static int launch_filter_spectrum_split_t(const float* taps1, const float* taps2, const float* D1, const float* D2,
                                          float* spec, int d, hipStream_t stream) {
  const size_t lds_bytes = (size_t)P::WG_LDS * sizeof(float2);
  auto kern = taps2 ? filter_spectrum_split_kernel<P, true> : filter_spectrum_split_kernel<P, false>;
  if (lds_bytes > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (e != hipSuccess) return set_error(M2_ERR_LAUNCH, "hipFuncSetAttribute(filter_spectrum_split): %s", hipGetErrorString(e));
  }
  int per_cu = (int)((160 * 1024) / lds_bytes);
  if (per_cu < 1) per_cu = 1;
  if (per_cu > 512 / P::T) per_cu = 512 / P::T;
  int grid = num_cus() * per_cu;
  if (grid > 2 * d) grid = 2 * d;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(P::T), lds_bytes, stream, taps1, taps2, D1, D2, (float4*)spec, d);
  return check_launch("filter_spectrum_split");
}

#define M2_FOR_EACH_SPLIT_PLAN(X) \
  X(11, 16, 8)                    \
  X(12, 16, 16)                   \
  X(13, 32, 16)                   \
  X(14, 32, 32)

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
                                 int d, int L, hipStream_t stream) {
  switch (L) {
#define X(LOGL, R1, R2) \
  case 1 << LOGL:       \
    return launch_filter_spectrum_split_t<SplitPlan<LOGL, R1, R2>>(taps1, taps2, D1, D2, spec, d, stream);
    M2_FOR_EACH_SPLIT_PLAN(X)
#undef X
  }
  return set_error(M2_ERR_UNSUPPORTED, "filter_spectrum_split: no plan for L=%d", L);
}

}  // namespace m2
