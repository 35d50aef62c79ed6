// L = 32768: the fused mixer core and the filter-spectrum kernel with every real signal of a row transformed
// on its own, as H = L complex points, through the half-transform machinery of fft_split.h.
//
// A row of the N = 2L point convolution does not fit the 160 KB of LDS as one complex transform, nor as the
// two half transforms that serve L <= 16384.  Here the two real signals of the mixer (the gated short-conv
// product a, and the layer input u) are not packed into one complex row; each is convolved separately in
// polyphase form:
//
//   c[m] = s[2m] + i s[2m+1]  (m < L/2; the zero padding makes the upper half of the H = L points zero)
//   C = FFT_H(c) = Ce + i Co,   Ce = FFT_H(even samples) = (C[k] + conj C[H-k]) / 2,
//                               Co = FFT_H(odd samples)  = (C[k] - conj C[H-k]) / 2i
//   Ye = Ce Ke + w_H^k Co Ko,   Yo = Ce Ko + Co Ke        (Ke, Ko: the filter's even / odd taps, FFT_H)
//   d = IFFT_H(Ye + i Yo):      y[2m] = Re d[m], y[2m+1] = Im d[m], m < L/2
//
// The H-point transform with a zero upper half is exactly what fft_split.h runs as two half transforms of
// NS = H/2 = 16384 points (even and odd frequencies), and the pairing k <-> H - k is the mirror / complement
// pairing of its last pass, so a thread holds both members of every pair.  Per pair the spectrum buffer
// stores Ke and Ko (16 bytes) in the order the multiply consumes them; the root w_H^k is rebuilt in the multiply
// from one per-thread constant per half transform and compile-time constants:
//
//   spec[channel][filter 0..1][half 0..1] float4 (Ke, Ko)[slot 0..15][T]
//
// The filter kernel gets Ke and Ko from ONE transform per filter: the (d, 2L) taps row read as H complex
// numbers is k_even + i k_odd.
//
// A row is processed without staging through LDS: threads load and store global memory directly in the
// layout of the first pass (complex slot m = t + T j holds time steps 2m, 2m+1), where consecutive lanes
// touch consecutive 4- or 8-byte pieces.  Order per row: a -> y1 (two half transforms with filter 1),
// acc = y1 * gate, then the two half transforms of u with filter 2 are added to acc one after the other
// (u is loaded again for the second one instead of being kept in registers).
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

// One pair of the polyphase multiply: za = C[k], zb = C[H - k]; returns D[k] in za and D[H - k] in zb.
// K = (Ke, Ko) at frequency k, with the scale 1 / 4H folded in; the third factor w_H^k Ko is formed here: the root is
// beta (this thread's group, one per half transform, the same for every row) times the constant w_64^S.
template <int S>
__device__ __forceinline__ void pair_multiply_real(cf& za, cf& zb, float4 K, cf beta) {
  const cf A = {za.re + zb.re, za.im - zb.im};         // 2 Ce
  const cf Bq = {za.im + zb.im, zb.re - za.re};        // 2 Co
  const cf ke = {K.x, K.y}, ko = {K.z, K.w};
  const cf kw = cmul(beta, mul_w64<S, false>(ko));
  const cf Ye = cadd(cmul(A, ke), cmul(Bq, kw));
  const cf Yo = cadd(cmul(A, ko), cmul(Bq, ke));
  za = {Ye.re - Yo.im, Ye.im + Yo.re};                 // Ye + i Yo
  zb = {Ye.re + Yo.im, Yo.re - Ye.im};                 // conj(Ye) + i conj(Yo)
}
// self-paired frequency (k = 0 or H/2): everything is real; kw = +ko at k = 0 and -ko at k = H/2
__device__ __forceinline__ cf self_multiply_real(cf z, float ke, float ko, float kw) {
  return {z.re * ke + z.im * kw, z.re * ko + z.im * ke};
}

// spectral multiply of the 16 + 16 points a thread holds after fwd_groups, slots 4 HB .. 4 HB + 3 (same
// pairing as multiply_batch in fft_split.h)
// beta: root of the thread's group (slot s of it adds w_16^s); in the special work item of the even half the slots
// 1 .. 7 belong to group 0 (root 1) and the slots 8 .. 15 to group R2 / 2 (root beta_sp, slot s - 8 of it).
template <bool EVEN_SPECIAL, int HB>
__device__ __forceinline__ void multiply_batch_real(cf (&x)[32], const float4 (&K)[4], cf beta, cf beta_sp) {
  static_for<0, 4>([&](auto ss) {
    constexpr int s = 4 * HB + decltype(ss)::value;
    const float4 k = K[decltype(ss)::value];
    if constexpr (!EVEN_SPECIAL) {
      pair_multiply_real<4 * s>(x[bitrev(s, 4)], x[16 + bitrev(15 - s, 4)], k, beta);
    } else if constexpr (s == 0) {
      // K = (Ke(0), Ko(0), Ke(H/2), Ko(H/2))
      x[bitrev(0, 4)] = self_multiply_real(x[bitrev(0, 4)], k.x, k.y, k.y);
      x[bitrev(8, 4)] = self_multiply_real(x[bitrev(8, 4)], k.z, k.w, -k.w);
    } else if constexpr (s < 8) {
      pair_multiply_real<4 * s>(x[bitrev(s, 4)], x[bitrev(16 - s, 4)], k, cf{1.f, 0.f});
    } else {
      pair_multiply_real<4 * (s - 8)>(x[16 + bitrev(s - 8, 4)], x[16 + bitrev(23 - s, 4)], k, beta_sp);
    }
  });
}
template <int HB>
__device__ __forceinline__ void load_spectrum_batch_real(float4 (&K)[4], const float4* __restrict__ sp4, int T) {
  static_for<0, 4>([&](auto s) { K[decltype(s)::value] = sp4[(4 * HB + decltype(s)::value) * T]; });
}

// One half transform of one real signal: forward passes from registers (first-pass layout), polyphase multiply,
// inverse passes back to registers.  Same barrier structure as half_convolution in fft_split.h; the spectrum
// comes in four batches, each loaded while the one before it is multiplied.
template <class P, bool ODD>
__device__ __forceinline__ void half_convolution_real(cf (&x)[32], int t, float2* row, const float2* tab2,
                                                      const cf (&b)[P::NB1], const float4* __restrict__ sp4, cf beta,
                                                      cf beta_sp, int ga, int gb, bool special) {
  fwd_pass1<P, ODD>(x, t, row, b);
  phase_barrier();
  fwd_pass2<P>(x, t, row, tab2);
  phase_barrier();
  float4 Ka[4], Kb[4];
  load_spectrum_batch_real<0>(Ka, sp4, P::T);
  fwd_groups<P>(x, row, ga, gb);
  __builtin_amdgcn_sched_barrier(0);
  auto multiply = [&](auto sp) __attribute__((always_inline)) {
    constexpr bool S = decltype(sp)::value == 1;
    load_spectrum_batch_real<1>(Kb, sp4, P::T);
    multiply_batch_real<S, 0>(x, Ka, beta, beta_sp);
    load_spectrum_batch_real<2>(Ka, sp4, P::T);
    multiply_batch_real<S, 1>(x, Kb, beta, beta_sp);
    load_spectrum_batch_real<3>(Kb, sp4, P::T);
    multiply_batch_real<S, 2>(x, Ka, beta, beta_sp);
    multiply_batch_real<S, 3>(x, Kb, beta, beta_sp);
  };
  if (!ODD && special) multiply(ic<1>{});
  else multiply(ic<0>{});
  __builtin_amdgcn_sched_barrier(0);
  inv_groups<P>(x, row, ga, gb);
  phase_barrier();
  inv_pass2<P>(x, t, row, tab2);
  phase_barrier();
  inv_pass1<P, ODD>(x, t, row, b);
}

// floats of the spectrum buffer per (channel, filter, half): 16 slots x T work items x float4
template <class P>
constexpr long real_spec_block() { return 16L * P::T * 4; }

// ------------------------------------------------------------------------------------------
// global memory in first-pass layout: complex slot m <-> time steps 2m, 2m + 1
// ------------------------------------------------------------------------------------------
// raw bits of time steps (2m, 2m+1); m = -1 reads slot 0 instead (the caller discards it)
__device__ __forceinline__ uint32_t fetch_pair(const uint16_t* p, int m) {
  return reinterpret_cast<const uint32_t*>(p)[m < 0 ? 0 : m];
}
__device__ __forceinline__ f32x2_t fetch_pair(const float* p, int m) {
  return reinterpret_cast<const f32x2_t*>(p)[m < 0 ? 0 : m];
}
__device__ __forceinline__ float2 expand_pair(uint32_t r) {
  return make_float2(__uint_as_float(r << 16), __uint_as_float(r & 0xffff0000u));
}
__device__ __forceinline__ float2 expand_pair(f32x2_t r) { return make_float2(r.x, r.y); }
__device__ __forceinline__ void store_pair(uint16_t* p, int m, float a, float b) {
  reinterpret_cast<uint32_t*>(p)[m] = pack_bf16x2(a, b);
}
__device__ __forceinline__ void store_pair(float* p, int m, float a, float b) {
  reinterpret_cast<float2*>(p)[m] = make_float2(a, b);
}
template <typename ACT> struct PairBits;
template <> struct PairBits<uint16_t> { typedef uint32_t type; };
template <> struct PairBits<float> { typedef f32x2_t type; };

// slot of register x[i R1 + j] of thread t in the first-pass layout
template <class P>
__device__ __forceinline__ int slot_of(int t, int i, int j) { return t + P::T * i + P::S1 * j; }

// Causal 3-tap convolution of one (3d, B, L) channel at the time steps of this thread's 32 slots:
// out[r] = (sc(2m), sc(2m+1)) with sc(n) = bias + w0 in[n-2] + w1 in[n-1] + w2 in[n], in = stored value + add
// (time steps before 0 are the convolution's zero padding).  All 64 loads of a bf16 row are put in flight at once
// (64 registers); an fp32 row goes in two batches.
template <class P, typename ACT>
__device__ __forceinline__ void short_conv_slots(const ACT* __restrict__ p, int t, const float (&w)[3], float bias,
                                                 float add, cf (&out)[32]) {
  typedef typename PairBits<ACT>::type bits;
  constexpr int NB = sizeof(ACT) == 2 ? 32 : 16;      // slots per batch
  const float fbias = bias + add * (w[0] + w[1] + w[2]);
  static_for<0, 32 / NB>([&](auto hh) {
    constexpr int h0 = decltype(hh)::value * NB;
    bits prev[NB], cur[NB];
    static_for<0, NB>([&](auto rr) {
      constexpr int r = h0 + decltype(rr)::value;
      const int m = slot_of<P>(t, r / P::R1, r % P::R1);
      cur[r - h0] = fetch_pair(p, m);
      prev[r - h0] = fetch_pair(p, m - 1);
    });
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, NB>([&](auto rr) {
      constexpr int r = h0 + decltype(rr)::value;
      const int m = slot_of<P>(t, r / P::R1, r % P::R1);
      const float2 c = expand_pair(cur[r - h0]);
      float2 q = expand_pair(prev[r - h0]);
      if constexpr (r == 0) {      // only slot m = t of register 0 can be slot 0
        q.x = m > 0 ? q.x : 0.f;
        q.y = m > 0 ? q.y : 0.f;
      }
      // `add` (the in-projection's bias) is folded into the convolution's bias: conv(x + add) = conv(x) + add (w0 + w1 +
      // w2), except at time steps 0 and 1, where taps fall on the zero padding outside the biased signal
      out[r] = {fbias + w[0] * q.x + w[1] * q.y + w[2] * c.x, fbias + w[0] * q.y + w[1] * c.x + w[2] * c.y};
      if constexpr (r == 0) {
        if (m == 0) {
          out[r].re -= add * (w[0] + w[1]);
          out[r].im -= add * w[0];
        }
      }
    });
  });
}
// the signal itself (no short convolution) at this thread's slots
template <class P, typename ACT>
__device__ __forceinline__ void load_slots(const ACT* __restrict__ p, int t, cf (&out)[32]) {
  typedef typename PairBits<ACT>::type bits;
  bits cur[32];
  static_for<0, 32>([&](auto rr) {
    constexpr int r = decltype(rr)::value;
    cur[r] = fetch_pair(p, slot_of<P>(t, r / P::R1, r % P::R1));
  });
  __builtin_amdgcn_sched_barrier(0);
  static_for<0, 32>([&](auto rr) {
    constexpr int r = decltype(rr)::value;
    const float2 c = expand_pair(cur[r]);
    out[r] = {c.x, c.y};
  });
}

// ------------------------------------------------------------------------------------------
// the fused mixer core, sequence length 2 P::L
// ------------------------------------------------------------------------------------------
// FULL: short convolutions and gates (sw, sb non-null); otherwise a plain long convolution of one input.
// HAS_U: the residual long convolution of the layer input u (uin non-null).
template <class P, typename ACT, bool FULL, bool HAS_U>
__global__ __launch_bounds__(P::T) __attribute__((amdgpu_waves_per_eu(2, 2))) void mixer_real_kernel(
    const ACT* __restrict__ xproj,      // (3d, B, LS): x1 | x2 | v, channel-major
    const float* __restrict__ uin,      // (d, B, LS)  layer input, channel-major (may be null)
    const float* __restrict__ sw,       // (3d, 3)     short-conv taps
    const float* __restrict__ sb,       // (3d)        short-conv bias
    const float* __restrict__ pbias,    // (3d)        bias of the in-projection, added to xproj on load (may be null)
    const float* __restrict__ spec,     // (d, 2, 2) blocks of real_spec_block<P>() floats
    ACT* __restrict__ y,                // (d, B, LS)
    int B, int d) {
  constexpr int T = P::T;
  constexpr long LS = 2L * P::L;
  constexpr long BLK = real_spec_block<P>();
  extern __shared__ float2 lds[];
  float2* row = lds;
  float2* tab2 = lds + P::ROW_LDS;
  const int t = threadIdx.x;

  tab2_init<P>(tab2);
  cf b[P::NB1];
  static_for<0, P::NB1>([&](auto ii) { b[decltype(ii)::value] = unit_root(t + T * decltype(ii)::value, P::N); });
  const SplitGroups<P> grp = split_groups<P>(t);
  // roots of the polyphase multiply: frequency k = k0 + R1 R2 s for slot s of group g, k0 = g / R2 + R1 (g % R2), and
  // the pair at k of the half transform sits at 2 k + ODD of the H-point transform
  const cf beta_e = unit_root(2 * (grp.ge / P::R2 + P::R1 * (grp.ge % P::R2)), P::N);
  const cf beta_o = unit_root(2 * (grp.go / P::R2 + P::R1 * (grp.go % P::R2)) + 1, P::N);
  const cf beta_sp = unit_root(2 * (P::R1 * (P::R2 / 2)), P::N);
  phase_barrier();

  // workgroup -> (channel, batch row) as in mixer_split_kernel: XCD e takes the channels c = e (mod 8)
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, slots = gridDim.x >> 3;
  const int rows_per_xcd = (d >> 3) * B;
  for (int j = slot; j < rows_per_xcd; j += slots) {
    // the same for every lane: say so, so that row base addresses live in scalar registers
    const int c = __builtin_amdgcn_readfirstlane((j / B) * 8 + xcd), bb = __builtin_amdgcn_readfirstlane(j % B);
    const float* spc = spec + (long)c * 4 * BLK;
    cf x[32], acc[32];

    // ---- first signal: a = sc(x1) sc(v)  (or the plain input), convolved with filter 1
    if constexpr (FULL) {
      float w1[3], wv[3];
#pragma unroll
      for (int k = 0; k < 3; ++k) {
        w1[k] = sw[(long)c * 3 + k];
        wv[k] = sw[((long)2 * d + c) * 3 + k];
      }
      const float p1 = pbias ? pbias[c] : 0.f, pv = pbias ? pbias[2 * d + c] : 0.f;
      short_conv_slots<P, ACT>(xproj + ((long)(0 * d + c) * B + bb) * LS, t, w1, sb[c], p1, x);
      short_conv_slots<P, ACT>(xproj + ((long)(2 * d + c) * B + bb) * LS, t, wv, sb[2 * d + c], pv, acc);
      static_for<0, 32>([&](auto rr) {
        constexpr int r = decltype(rr)::value;
        x[r] = {x[r].re * acc[r].re, x[r].im * acc[r].im};
      });
    } else {
      load_slots<P, ACT>(xproj + ((long)c * B + bb) * LS, t, x);
    }
    static_for<0, 32>([&](auto rr) { acc[decltype(rr)::value] = x[decltype(rr)::value]; });     // a, for the odd half
    {
      const float4* sp4 = reinterpret_cast<const float4*>(spc) + t;
      half_convolution_real<P, false>(x, t, row, tab2, b, sp4, beta_e, beta_sp, grp.ge, grp.gm, grp.special);
    }
    static_for<0, 32>([&](auto rr) {       // x <- a for the odd half, acc <- the even half's result
      constexpr int r = decltype(rr)::value;
      const cf e = x[r];
      x[r] = acc[r];
      acc[r] = e;
    });
    {
      const float4* sp4 = reinterpret_cast<const float4*>(spc + BLK) + t;
      half_convolution_real<P, true>(x, t, row, tab2, b, sp4, beta_o, beta_sp, grp.go, grp.gc, false);
    }
    static_for<0, 32>([&](auto rr) {
      constexpr int r = decltype(rr)::value;
      acc[r] = cadd(acc[r], x[r]);
    });

    // ---- gate: acc = y1 * sc(x2)
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (FULL) {
      float w2[3];
#pragma unroll
      for (int k = 0; k < 3; ++k) w2[k] = sw[((long)d + c) * 3 + k];
      const float p2 = pbias ? pbias[d + c] : 0.f;
      short_conv_slots<P, ACT>(xproj + ((long)(1 * d + c) * B + bb) * LS, t, w2, sb[d + c], p2, x);
      static_for<0, 32>([&](auto rr) {
        constexpr int r = decltype(rr)::value;
        acc[r] = {acc[r].re * x[r].re, acc[r].im * x[r].im};
      });
    }

    // ---- second signal: the layer input u, convolved with filter 2; its two half transforms are added to acc
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (HAS_U) {
      const float* pu = uin + ((long)c * B + bb) * LS;
      load_slots<P, float>(pu, t, x);
      {
        const float4* sp4 = reinterpret_cast<const float4*>(spc + 2 * BLK) + t;
        half_convolution_real<P, false>(x, t, row, tab2, b, sp4, beta_e, beta_sp, grp.ge, grp.gm, grp.special);
      }
      static_for<0, 32>([&](auto rr) {
        constexpr int r = decltype(rr)::value;
        acc[r] = cadd(acc[r], x[r]);
      });
      __builtin_amdgcn_sched_barrier(0);
      int again = 0;
      asm volatile("" : "+v"(again));    // a second load, not the first one's registers kept across the half transform
      load_slots<P, float>(pu + again, t, x);
      {
        const float4* sp4 = reinterpret_cast<const float4*>(spc + 3 * BLK) + t;
        half_convolution_real<P, true>(x, t, row, tab2, b, sp4, beta_o, beta_sp, grp.go, grp.gc, false);
      }
      static_for<0, 32>([&](auto rr) {
        constexpr int r = decltype(rr)::value;
        acc[r] = cadd(acc[r], x[r]);
      });
    }

    ACT* py = y + ((long)c * B + bb) * LS;
    static_for<0, 32>([&](auto rr) {
      constexpr int r = decltype(rr)::value;
      store_pair(py, slot_of<P>(t, r / P::R1, r % P::R1), acc[r].re, acc[r].im);
    });
    // every half transform starts and ends in LDS slots this thread owns: no barrier between rows
  }
}

// ------------------------------------------------------------------------------------------
// filter taps -> (Ke, Ko) in the layout above; work item = (channel, filter), both half transforms
// ------------------------------------------------------------------------------------------
template <class P>
__global__ __launch_bounds__(P::T) void filter_spectrum_real_kernel(
    const float* taps1,    // (d, 2 LS) bidirectional taps of filter_fn
    const float* taps2,    // (d, 2 LS) bidirectional taps of filter_fn2 (null: its blocks are zeroed)
    const float* D1,       // (d) skip weight of filter_fn, added to tap 0 (may be null)
    const float* D2,       // (d) skip weight of filter_fn2 (may be null)
    float* __restrict__ spec, int d, SpectrumBatch sb) {
  constexpr int NS = P::L, H = P::N, T = P::T, R1 = P::R1, R2 = P::R2;
  {
    float* sp = spec;
    select_mixer(sb, d, 2 * H, taps1, taps2, D1, D2, sp);
    spec = sp;
  }
  constexpr long BLK = real_spec_block<P>();
  extern __shared__ float2 lds[];
  float2* row = lds;
  float2* tab2 = lds + P::ROW_LDS;
  const int t = threadIdx.x;

  tab2_init<P>(tab2);
  cf b[P::NB1];
  static_for<0, P::NB1>([&](auto ii) { b[decltype(ii)::value] = unit_root(t + T * decltype(ii)::value, P::N); });
  const SplitGroups<P> grp = split_groups<P>(t);
  // 1/H of the inverse, 1/2 of Ke / Ko from the packed transform, 1/2 of Ce / Co in the mixer kernel
  const float scale = 0.25f / (float)H;
  __syncthreads();

  // work item = (channel, filter): the taps row is read once; its even-half combination goes to LDS at once, the
  // odd-half combination waits in registers (64) while the even half is transformed
  for (int item = blockIdx.x; item < 2 * d; item += gridDim.x) {
    const int c = item >> 1, f = item & 1;
    const float* taps = f ? taps2 : taps1;
    const float* D = f ? D2 : D1;
    float* blk = spec + (long)item * 2 * BLK;
    if (!taps) {
      static_for<0, 2>([&](auto hh) {
        float4* z4 = reinterpret_cast<float4*>(blk + decltype(hh)::value * BLK) + t;
        static_for<0, 16>([&](auto ss) { z4[decltype(ss)::value * T] = make_float4(0.f, 0.f, 0.f, 0.f); });
      });
      continue;
    }
    // g[m] = taps[2m] + i taps[2m+1], m < H; even half: g_lo + g_hi, odd half: g_lo - g_hi
    constexpr int Q = NS / 2 / T;
    f32x4_t od[Q];
    {
      f32x4_t lo[Q], hi[Q];
      static_for<0, Q>([&](auto qq) {
        constexpr int q = decltype(qq)::value;
        const float* p = taps + (long)c * 2 * H + 4 * (q * T + t);
        lo[q] = *reinterpret_cast<const f32x4_t*>(p);
        hi[q] = *reinterpret_cast<const f32x4_t*>(p + 2 * NS);
      });
      if (D && t == 0) lo[0].x += D[c];      // the skip weight is one more tap at lag 0
      static_for<0, Q>([&](auto qq) {
        constexpr int q = decltype(qq)::value;
        float2* dst = row + sphys(2 * (q * T + t));     // 2 consecutive slots never straddle a pad
        dst[0] = make_float2(lo[q].x + hi[q].x, lo[q].y + hi[q].y);
        dst[1] = make_float2(lo[q].z + hi[q].z, lo[q].w + hi[q].w);
        od[q] = lo[q] - hi[q];
      });
    }
    auto one_half = [&](auto hh) __attribute__((always_inline)) {
      constexpr bool ODD = decltype(hh)::value == 1;
      float4* sp4 = reinterpret_cast<float4*>(blk + (ODD ? BLK : 0)) + t;
      if constexpr (ODD) {
        static_for<0, Q>([&](auto qq) {
          constexpr int q = decltype(qq)::value;
          float2* dst = row + sphys(2 * (q * T + t));
          dst[0] = make_float2(od[q].x, od[q].y);
          dst[1] = make_float2(od[q].z, od[q].w);
        });
      }
      __syncthreads();
      cf x[32];
      pass1_load<P>(x, t, row);
      fwd_pass1<P, ODD>(x, t, row, b);
      __syncthreads();
      fwd_pass2<P>(x, t, row, tab2);
      __syncthreads();
      const int ga = ODD ? grp.go : grp.ge, gb = ODD ? grp.gc : grp.gm;
      fwd_groups<P>(x, row, ga, gb);
      __syncthreads();      // LDS is restaged by the next half / item

      // (Ke, Ko) of the pair (za at frequency k of this half transform, zb at its partner)
      auto emit = [&](auto slot, cf za, cf zb) __attribute__((always_inline)) {
        sp4[decltype(slot)::value * T] = make_float4(scale * (za.re + zb.re), scale * (za.im - zb.im),
                                                     scale * (za.im + zb.im), scale * (zb.re - za.re));
      };
      if (!ODD && grp.special) {
        const cf z0 = x[bitrev(0, 4)], zn = x[bitrev(8, 4)];
        sp4[0] = make_float4(4.f * scale * z0.re, 4.f * scale * z0.im, 4.f * scale * zn.re, 4.f * scale * zn.im);
        static_for<1, 8>([&](auto ss) {
          constexpr int s = decltype(ss)::value;
          emit(ss, x[bitrev(s, 4)], x[bitrev(16 - s, 4)]);
        });
        static_for<0, 8>([&](auto ss) {
          constexpr int s = decltype(ss)::value;
          emit(ic<8 + s>{}, x[16 + bitrev(s, 4)], x[16 + bitrev(15 - s, 4)]);
        });
      } else {
        static_for<0, 16>([&](auto ss) {
          constexpr int s = decltype(ss)::value;
          emit(ss, x[bitrev(s, 4)], x[16 + bitrev(15 - s, 4)]);
        });
      }
    };
    one_half(ic<0>{});
    one_half(ic<1>{});
  }
}

// ------------------------------------------------------------------------------------------
// host-side launchers
// ------------------------------------------------------------------------------------------
typedef SplitPlan<14, 32, 32> RealPlan;      // half transforms of 16384 points: sequence length 32768
static_assert(split_offsets_ok<RealPlan>(), "LDS offsets of the split plan");

size_t real_spectrum_bytes(int d) { return (size_t)d * 4 * real_spec_block<RealPlan>() * sizeof(float); }

template <typename ACT>
static int launch_mixer_real(const void* xproj, const float* u, const float* sw, const float* sb, const float* pbias,
                             const float* spec, void* y, int B, int d, hipStream_t stream) {
  typedef RealPlan P;
  const size_t lds_bytes = (size_t)P::WG_LDS * sizeof(float2);
  auto kern = sw ? (u ? mixer_real_kernel<P, ACT, true, true> : mixer_real_kernel<P, ACT, true, false>)
                 : mixer_real_kernel<P, ACT, false, false>;
  if (!sw && u) return set_error(M2_ERR_ARG, "mixer_real: a plain convolution takes no second input");
  hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
  if (e != hipSuccess) return set_error(M2_ERR_LAUNCH, "hipFuncSetAttribute(mixer_real): %s", hipGetErrorString(e));
  const int rows_per_xcd = (d / 8) * B;
  int slots = num_cus() / 8;          // one workgroup per compute unit (140 KB of LDS)
  if (slots > rows_per_xcd) slots = rows_per_xcd;
  const int rounds = (rows_per_xcd + slots - 1) / slots;      // every workgroup the same number of rows
  slots = (rows_per_xcd + rounds - 1) / rounds;
  hipLaunchKernelGGL(kern, dim3(8 * slots), dim3(P::T), lds_bytes, stream, (const ACT*)xproj, u, sw, sb, pbias, spec,
                     (ACT*)y, B, d);
  return check_launch("mixer_real");
}

int launch_mixer_real_dispatch(const void* xproj, const float* u, const float* sw, const float* sb, const float* pbias,
                               const float* spec, void* y, int B, int d, int act_dtype, hipStream_t stream) {
  return act_dtype == M2_DTYPE_F32 ? launch_mixer_real<float>(xproj, u, sw, sb, pbias, spec, y, B, d, stream)
                                   : launch_mixer_real<uint16_t>(xproj, u, sw, sb, pbias, spec, y, B, d, stream);
}

int launch_filter_spectrum_real(const float* taps1, const float* taps2, const float* D1, const float* D2, float* spec,
                                int d, const SpectrumBatch& sb, int nmixers, hipStream_t stream) {
  typedef RealPlan P;
  const size_t lds_bytes = (size_t)P::WG_LDS * sizeof(float2);
  auto kern = filter_spectrum_real_kernel<P>;
  hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
  if (e != hipSuccess) return set_error(M2_ERR_LAUNCH, "hipFuncSetAttribute(filter_spectrum_real): %s", hipGetErrorString(e));
  int grid = num_cus();
  if (grid > 2 * d) grid = 2 * d;
  hipLaunchKernelGGL(kern, dim3(grid, nmixers), dim3(P::T), lds_bytes, stream, taps1, taps2, D1, D2, spec, d, sb);
  return check_launch("filter_spectrum_real");
}

}  // namespace m2
