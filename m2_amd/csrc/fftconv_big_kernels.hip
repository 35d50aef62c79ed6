// Long convolution for L = 32768 (FFT length N = 65536), which does not fit the 160 KB LDS.
//
// Four-step split N = 4 x NS, NS = 16384, with the radix-4 step taken first (decimation in frequency):
//
//   y_k1[n2] = ( sum_{n1<4} z[n1 NS + n2] (-i)^(n1 k1) ) w_N^(n2 k1)         k1 = 0..3, n2 < NS
//   Z[k1 + 4 k2] = FFT_NS(y_k1)[k2]                                           LDS-resident engine, digit-reversed
//
// and the mirror image on the way back:  v_k1 = IFFT_NS(W[k1 + 4 .]),
//   w[n1 NS + n2] = sum_k1 i^(n1 k1) conj(w_N^(n2 k1)) v_k1[n2]               only n1 = 0, 1 are wanted.
//
// One workgroup owns one (channel, batch) row and runs the four sub-transforms one after the other in
// the same LDS buffer, accumulating the two output halves in registers, so nothing but inputs, outputs
// and filter spectra touches memory.  What makes that possible is the choice of the two groups a thread
// takes in the engine's paired radix-8 pass.  Frequency k = k1 + 4 k2 pairs with N - k:
//   k1 = 0      <->  k1 = 0,  k2' = (NS - k2) mod NS     "mirror"      : groups (g, mirror(g)), as for N <= 16384
//   k1 = 2      <->  k1 = 2,  k2' = NS - 1 - k2          "complement"  : groups (g, comp(g))
//   k1 = 1      <->  k1 = 3,  k2' = NS - 1 - k2          "complement"  : the k1 = 1 spectrum of (g, comp(g)) is
//                                                                        kept in registers while k1 = 3 runs
// so every pair a thread needs is in its own registers.  (Index mathematics checked against numpy FFTs
// before this file was written.)
//
// Spectrum layout ("native order"), per channel: float4 spec[32][T], T = NS / 16 work items:
//   [0..8)    k1 = 0, as in the N <= 16384 kernels (slot 0 of work item 0 packs DC and Nyquist)
//   [8..16)   k1 = 2, pair j: frequency of (g, slot j), partner (comp(g), slot 7 - j)
//   [16..24)  pair j: (k1 = 1, g, j)       with partner (k1 = 3, comp(g), 7 - j)
//   [24..32)  pair j: (k1 = 1, comp(g), j) with partner (k1 = 3, g, 7 - j)
// = (N/2) float4 per channel = d L 16 bytes in total, the same size formula as the small kernels.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fft_engine.h"

namespace m2 {

using BigPlan = Plan<14, 16, 16, 8>;
constexpr int kNS = 16384;
constexpr int kBigN = 4 * kNS;

// all digits of a group index complemented: the group that holds k2' = NS - 1 - k2 (slot 7 - j)
template <class P>
__device__ __forceinline__ int complement_group(int g) {
  return P::M - 1 - g;      // digits are independent, so complementing every digit is M - 1 - g
}

// 8 consecutive activations (plus the two before) -> short-conv outputs, as in the small kernel
__device__ __forceinline__ void load10b(const float* p, int n0, float add, float (&o)[10]) {
  const float4 a = *reinterpret_cast<const float4*>(p + n0);
  const float4 b = *reinterpret_cast<const float4*>(p + n0 + 4);
  o[0] = 0.f; o[1] = 0.f;
  if (n0 > 0) {
    const float2 h = *reinterpret_cast<const float2*>(p + n0 - 2);
    o[0] = h.x + add; o[1] = h.y + add;
  }
  o[2] = a.x + add; o[3] = a.y + add; o[4] = a.z + add; o[5] = a.w + add;
  o[6] = b.x + add; o[7] = b.y + add; o[8] = b.z + add; o[9] = b.w + add;
}
__device__ __forceinline__ void load10b(const uint16_t* p, int n0, float add, float (&o)[10]) {
  const uint4 a = *reinterpret_cast<const uint4*>(p + n0);
  o[0] = 0.f; o[1] = 0.f;
  if (n0 > 0) {
    const uint32_t h = *reinterpret_cast<const uint32_t*>(p + n0 - 2);
    o[0] = __uint_as_float(h << 16) + add; o[1] = __uint_as_float(h & 0xffff0000u) + add;
  }
  o[2] = __uint_as_float(a.x << 16) + add; o[3] = __uint_as_float(a.x & 0xffff0000u) + add;
  o[4] = __uint_as_float(a.y << 16) + add; o[5] = __uint_as_float(a.y & 0xffff0000u) + add;
  o[6] = __uint_as_float(a.z << 16) + add; o[7] = __uint_as_float(a.z & 0xffff0000u) + add;
  o[8] = __uint_as_float(a.w << 16) + add; o[9] = __uint_as_float(a.w & 0xffff0000u) + add;
}
__device__ __forceinline__ void store8b(float* p, int n0, const float (&v)[8]) {
  *reinterpret_cast<float4*>(p + n0) = make_float4(v[0], v[1], v[2], v[3]);
  *reinterpret_cast<float4*>(p + n0 + 4) = make_float4(v[4], v[5], v[6], v[7]);
}
__device__ __forceinline__ void store8b(uint16_t* p, int n0, const float (&v)[8]) {
  uint4 o;
  o.x = pack_bf16x2(v[0], v[1]);
  o.y = pack_bf16x2(v[2], v[3]);
  o.z = pack_bf16x2(v[4], v[5]);
  o.w = pack_bf16x2(v[6], v[7]);
  *reinterpret_cast<uint4*>(p + n0) = o;
}

// short conv of 8 consecutive samples: out[j] = bias + w0 in[j] + w1 in[j+1] + w2 in[j+2]
__device__ __forceinline__ void conv8(const float (&in)[10], float w0, float w1, float w2, float bb, float (&o)[8]) {
  static_for<0, 8>([&](auto jj) {
    constexpr int j = decltype(jj)::value;
    o[j] = bb + w0 * in[j] + w1 * in[j + 1] + w2 * in[j + 2];
  });
}

// multiply by (-i)^k
__device__ __forceinline__ cf mul_negi_pow(cf v, int k) {
  switch (k & 3) {
    case 1: return {v.im, -v.re};
    case 2: return {-v.re, -v.im};
    case 3: return {-v.im, v.re};
    default: return v;
  }
}

struct RowSrc {             // where one row's inputs live
  const void* x1; const void* x2; const void* v; const float* u;
  float w1[3], w2[3], w3[3], b1, b2, b3, pb1, pb2, pb3;
  bool plain;
};

// a[n], u[n] for 8 consecutive n starting at n0 (n0 % 8 == 0, n0 < L)
template <typename ACT>
__device__ __forceinline__ void act8(const RowSrc& r, int n0, float (&a)[8], float (&uu)[8]) {
  float in[10];
  if (!r.plain) {
    float c[8];
    load10b(reinterpret_cast<const ACT*>(r.x1), n0, r.pb1, in);
    conv8(in, r.w1[0], r.w1[1], r.w1[2], r.b1, a);
    load10b(reinterpret_cast<const ACT*>(r.v), n0, r.pb3, in);
    conv8(in, r.w3[0], r.w3[1], r.w3[2], r.b3, c);
    static_for<0, 8>([&](auto jj) { a[decltype(jj)::value] *= c[decltype(jj)::value]; });
  } else {
    load10b(reinterpret_cast<const ACT*>(r.x1), n0, 0.f, in);
    static_for<0, 8>([&](auto jj) { a[decltype(jj)::value] = in[decltype(jj)::value + 2]; });
  }
  if (r.u) {
    const float4 u0 = *reinterpret_cast<const float4*>(r.u + n0);
    const float4 u1 = *reinterpret_cast<const float4*>(r.u + n0 + 4);
    uu[0] = u0.x; uu[1] = u0.y; uu[2] = u0.z; uu[3] = u0.w;
    uu[4] = u1.x; uu[5] = u1.y; uu[6] = u1.z; uu[7] = u1.w;
  } else {
    static_for<0, 8>([&](auto jj) { uu[decltype(jj)::value] = 0.f; });
  }
}

// Stage y_k1[16 t .. 16 t + 16) in LDS.  `quarters` = how many of the four length-NS quarters of z are
// non-zero (2 for zero-padded activations, 4 for filter taps); `loadz(n, out8)` yields z for 8 samples.
template <int QUARTERS, class LOADZ>
__device__ __forceinline__ void stage_sub_input(int k1, int t, float2* row, LOADZ&& loadz) {
  const cf step = unit_root(k1, kBigN);
  cf tw = unit_root((16 * t * k1) & (kBigN - 1), kBigN);
  float4* dst = reinterpret_cast<float4*>(row + phys(16 * t));      // 16 consecutive slots never straddle a pad
  for (int h = 0; h < 2; ++h) {
    const int n2 = 16 * t + 8 * h;
    cf y[8];
    static_for<0, 8>([&](auto jj) { y[decltype(jj)::value] = {0.f, 0.f}; });
    static_for<0, QUARTERS>([&](auto qq) {
      constexpr int n1 = decltype(qq)::value;
      cf z[8];
      loadz(n1 * kNS + n2, z);
      static_for<0, 8>([&](auto jj) {
        constexpr int j = decltype(jj)::value;
        y[j] = cadd(y[j], mul_negi_pow(z[j], n1 * k1));
      });
    });
    static_for<0, 8>([&](auto jj) {
      constexpr int j = decltype(jj)::value;
      y[j] = cmul(y[j], tw);
      tw = cmul(tw, step);
    });
    static_for<0, 4>([&](auto qq) {
      constexpr int q = decltype(qq)::value;
      dst[4 * h + q] = make_float4(y[2 * q].re, y[2 * q].im, y[2 * q + 1].re, y[2 * q + 1].im);
    });
  }
}

template <typename ACT>
__global__ __launch_bounds__(1024) void mixer_core_big_kernel(
    const ACT* __restrict__ xproj, const float* __restrict__ uin, const float* __restrict__ sw,
    const float* __restrict__ sb, const float* __restrict__ pbias, const float4* __restrict__ spec,
    ACT* __restrict__ y, int B, int d) {
  using P = BigPlan;
  constexpr int T = P::T, L = kBigN / 2;
  extern __shared__ float2 lds[];
  float2* row = lds;
  const int t = threadIdx.x;
  Twiddles<P> tw;
  twiddles_init<P>(tw, t, lds + P::RPW * P::ROW_LDS);
  int g, gm;
  paired_groups<P>(t, g, gm);
  const int gc = complement_group<P>(g);

  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, slots = gridDim.x >> 3;
  const int rows_per_xcd = (d >> 3) * B;
  for (int j0 = slot; j0 < rows_per_xcd; j0 += slots) {
    const int c = (j0 / B) * 8 + xcd, b = j0 % B;
    RowSrc src;
    src.plain = (sw == nullptr);
    if (!src.plain) {
      src.x1 = xproj + ((long)(0 * d + c) * B + b) * L;
      src.x2 = xproj + ((long)(1 * d + c) * B + b) * L;
      src.v = xproj + ((long)(2 * d + c) * B + b) * L;
      for (int j = 0; j < 3; ++j) {
        src.w1[j] = sw[(long)(0 * d + c) * 3 + j];
        src.w2[j] = sw[(long)(1 * d + c) * 3 + j];
        src.w3[j] = sw[(long)(2 * d + c) * 3 + j];
      }
      src.b1 = sb[c]; src.b2 = sb[d + c]; src.b3 = sb[2 * d + c];
      src.pb1 = pbias ? pbias[c] : 0.f; src.pb2 = pbias ? pbias[d + c] : 0.f; src.pb3 = pbias ? pbias[2 * d + c] : 0.f;
    } else {
      src.x1 = xproj + ((long)c * B + b) * L;
      src.x2 = nullptr; src.v = nullptr;
    }
    src.u = uin ? uin + ((long)c * B + b) * L : nullptr;
    auto loadz = [&](int n, cf (&z)[8]) __attribute__((always_inline)) {
      float a[8], uu[8];
      act8<ACT>(src, n, a, uu);
      static_for<0, 8>([&](auto jj) { z[decltype(jj)::value] = {a[decltype(jj)::value], uu[decltype(jj)::value]}; });
    };
    const float4* sp = spec + (long)c * 32 * T + t;

    cf acc0[16], acc1[16];      // w[n2] and w[NS + n2] at n2 = t + 1024 j
    static_for<0, 16>([&](auto jj) { acc0[decltype(jj)::value] = {0.f, 0.f}; acc1[decltype(jj)::value] = {0.f, 0.f}; });

    // forward sub-transform k1 into x: x[0..8) = group g, x[8..16) = group `gsel`
    auto forward = [&](int k1, int gsel, cf (&x)[16]) __attribute__((always_inline)) {
      stage_sub_input<2>(k1, t, row, loadz);
      __syncthreads();
      fwd_load<P, P::R1, P::S1>(x, t, row);
      forward_to_pairs<P, false>(x, t, row, tw, g, gsel);
    };
    // inverse sub-transform k1 from x, accumulate into the two output halves
    auto inverse = [&](int k1, int gsel, cf (&x)[16]) __attribute__((always_inline)) {
      inverse_from_pairs<P, false>(x, t, row, tw, g, gsel);
      __syncthreads();            // the next stage overwrites LDS that this pass has just read
      // conj(w_N^(k1 (t + 1024 j))) = conj(w_N^(k1 t)) conj(w_64^(k1 j))
      const cf base = unit_root((k1 * t) & (kBigN - 1), kBigN);
      cf p[16];
      powers<16>(unit_root(k1, 64), p);
      static_for<0, 16>([&](auto jj) {
        constexpr int j = decltype(jj)::value;
        cf v = cmulc(x[j], base);
        if constexpr (j > 0) v = cmulc(v, p[j]);
        acc0[j] = cadd(acc0[j], v);
        acc1[j] = cadd(acc1[j], mul_negi_pow(v, (4 - k1) & 3));      // i^k1 = (-i)^(4 - k1)
      });
    };

    cf x[16];
    // ---- k1 = 0: mirror pairing ----
    forward(0, gm, x);
    {
      float4 K[8];
      static_for<0, 8>([&](auto s) { K[decltype(s)::value] = sp[decltype(s)::value * T]; });
      if (t != 0) {
        static_for<0, 8>([&](auto jj) {
          constexpr int j = decltype(jj)::value;
          pair_multiply(x[bitrev(j, 3)], x[8 + bitrev(7 - j, 3)], K[j]);
        });
      } else {
        x[bitrev(0, 3)] = {x[bitrev(0, 3)].re * K[0].x, x[bitrev(0, 3)].im * K[0].z};
        x[bitrev(4, 3)] = {x[bitrev(4, 3)].re * K[0].y, x[bitrev(4, 3)].im * K[0].w};
        static_for<1, 4>([&](auto jj) {
          constexpr int j = decltype(jj)::value;
          pair_multiply(x[bitrev(j, 3)], x[bitrev(8 - j, 3)], K[j]);
        });
        static_for<0, 4>([&](auto jj) {
          constexpr int j = decltype(jj)::value;
          pair_multiply(x[8 + bitrev(j, 3)], x[8 + bitrev(7 - j, 3)], K[4 + j]);
        });
      }
    }
    inverse(0, gm, x);
    // ---- k1 = 2: complement pairing inside the sub-transform ----
    forward(2, gc, x);
    static_for<0, 8>([&](auto jj) {
      constexpr int j = decltype(jj)::value;
      pair_multiply(x[bitrev(j, 3)], x[8 + bitrev(7 - j, 3)], sp[(8 + j) * T]);
    });
    inverse(2, gc, x);
    // ---- k1 = 1 with k1 = 3 ----
    cf x1s[16];
    forward(1, gc, x1s);
    __syncthreads();
    forward(3, gc, x);
    static_for<0, 8>([&](auto jj) {
      constexpr int j = decltype(jj)::value;
      pair_multiply(x1s[bitrev(j, 3)], x[8 + bitrev(7 - j, 3)], sp[(16 + j) * T]);
      pair_multiply(x1s[8 + bitrev(j, 3)], x[bitrev(7 - j, 3)], sp[(24 + j) * T]);
    });
    inverse(3, gc, x);
    inverse(1, gc, x1s);

    // ---- epilogue: the two halves, through LDS so that every thread owns 16 consecutive outputs ----
    for (int hh = 0; hh < 2; ++hh) {
      float2* pb = row + phys(t);
      static_for<0, 16>([&](auto jj) {
        constexpr int j = decltype(jj)::value;
        lds_put(pb, poff(j * P::S1), hh == 0 ? acc0[j] : acc1[j]);
      });
      __syncthreads();
      const float4* srcl = reinterpret_cast<const float4*>(row + phys(16 * t));
      for (int h8 = 0; h8 < 2; ++h8) {
        const int n = hh * kNS + 16 * t + 8 * h8;
        float gate[8];
        if (!src.plain) {
          float in[10];
          load10b(reinterpret_cast<const ACT*>(src.x2), n, src.pb2, in);
          conv8(in, src.w2[0], src.w2[1], src.w2[2], src.b2, gate);
        } else {
          static_for<0, 8>([&](auto jj) { gate[decltype(jj)::value] = 1.f; });
        }
        float out[8];
        static_for<0, 4>([&](auto qq) {
          constexpr int q = decltype(qq)::value;
          const float4 o = srcl[4 * h8 + q];
          out[2 * q] = o.x * gate[2 * q] + o.y;
          out[2 * q + 1] = o.z * gate[2 * q + 1] + o.w;
        });
        store8b(y + ((long)c * B + b) * L, n, out);
      }
      __syncthreads();
    }
  }
}

__global__ __launch_bounds__(1024) void filter_spectrum_big_kernel(
    const float* __restrict__ taps1, const float* __restrict__ taps2, const float* __restrict__ D1,
    const float* __restrict__ D2, float4* __restrict__ spec, int d) {
  using P = BigPlan;
  constexpr int T = P::T;
  extern __shared__ float2 lds[];
  float2* row = lds;
  const int t = threadIdx.x;
  Twiddles<P> tw;
  twiddles_init<P>(tw, t, lds + P::RPW * P::ROW_LDS);
  int g, gm;
  paired_groups<P>(t, g, gm);
  const int gc = complement_group<P>(g);
  const float scale = 0.5f / (float)kBigN;

  for (int c = blockIdx.x; c < d; c += gridDim.x) {
    const float* p1 = taps1 + (long)c * kBigN;
    const float* p2 = taps2 ? taps2 + (long)c * kBigN : nullptr;
    const float d1 = D1 ? D1[c] : 0.f, d2 = D2 ? D2[c] : 0.f;
    auto loadz = [&](int n, cf (&z)[8]) __attribute__((always_inline)) {
      const float4 a0 = *reinterpret_cast<const float4*>(p1 + n), a1 = *reinterpret_cast<const float4*>(p1 + n + 4);
      float4 b0 = make_float4(0.f, 0.f, 0.f, 0.f), b1 = b0;
      if (p2) { b0 = *reinterpret_cast<const float4*>(p2 + n); b1 = *reinterpret_cast<const float4*>(p2 + n + 4); }
      z[0] = {a0.x, b0.x}; z[1] = {a0.y, b0.y}; z[2] = {a0.z, b0.z}; z[3] = {a0.w, b0.w};
      z[4] = {a1.x, b1.x}; z[5] = {a1.y, b1.y}; z[6] = {a1.z, b1.z}; z[7] = {a1.w, b1.w};
      if (n == 0) { z[0].re += d1; z[0].im += d2; }            // the skip weight is one more tap at lag 0
    };
    auto forward = [&](int k1, int gsel, cf (&x)[16]) __attribute__((always_inline)) {
      stage_sub_input<4>(k1, t, row, loadz);
      __syncthreads();
      fwd_load<P, P::R1, P::S1>(x, t, row);
      forward_to_pairs<P, false>(x, t, row, tw, g, gsel);
      __syncthreads();            // LDS is reused by the next sub-transform
    };
    auto split = [&](cf za, cf zb) -> float4 {
      return make_float4(scale * (za.re + zb.re), scale * (za.im - zb.im), scale * (za.im + zb.im),
                         scale * (zb.re - za.re));
    };
    float4* sp = spec + (long)c * 32 * T + t;
    cf x[16];
    forward(0, gm, x);
    if (t != 0) {
      static_for<0, 8>([&](auto jj) {
        constexpr int j = decltype(jj)::value;
        sp[j * T] = split(x[bitrev(j, 3)], x[8 + bitrev(7 - j, 3)]);
      });
    } else {
      const cf z0 = x[bitrev(0, 3)], z4 = x[bitrev(4, 3)];
      sp[0] = make_float4(2.f * scale * z0.re, 2.f * scale * z4.re, 2.f * scale * z0.im, 2.f * scale * z4.im);
      static_for<1, 4>([&](auto jj) {
        constexpr int j = decltype(jj)::value;
        sp[j * T] = split(x[bitrev(j, 3)], x[bitrev(8 - j, 3)]);
      });
      static_for<0, 4>([&](auto jj) {
        constexpr int j = decltype(jj)::value;
        sp[(4 + j) * T] = split(x[8 + bitrev(j, 3)], x[8 + bitrev(7 - j, 3)]);
      });
    }
    forward(2, gc, x);
    static_for<0, 8>([&](auto jj) {
      constexpr int j = decltype(jj)::value;
      sp[(8 + j) * T] = split(x[bitrev(j, 3)], x[8 + bitrev(7 - j, 3)]);
    });
    cf x1s[16];
    forward(1, gc, x1s);
    forward(3, gc, x);
    static_for<0, 8>([&](auto jj) {
      constexpr int j = decltype(jj)::value;
      sp[(16 + j) * T] = split(x1s[bitrev(j, 3)], x[8 + bitrev(7 - j, 3)]);
      sp[(24 + j) * T] = split(x1s[8 + bitrev(j, 3)], x[bitrev(7 - j, 3)]);
    });
  }
}

template <typename ACT>
int launch_mixer_core_big(const void* xproj, const float* u, const float* sw, const float* sb, const float* pbias,
                          const float* spec, void* y, int B, int d, hipStream_t stream) {
  const size_t lds_bytes = (size_t)BigPlan::WG_LDS * sizeof(float2);
  auto kern = mixer_core_big_kernel<ACT>;
  hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
  if (e != hipSuccess) return set_error(M2_ERR_LAUNCH, "hipFuncSetAttribute(mixer_core_big): %s", hipGetErrorString(e));
  const int rows_per_xcd = (d / 8) * B;
  int slots = num_cus() / 8;
  if (slots > rows_per_xcd) slots = rows_per_xcd;
  hipLaunchKernelGGL(kern, dim3(8 * slots), dim3(1024), lds_bytes, stream, (const ACT*)xproj, u, sw, sb, pbias,
                     (const float4*)spec, (ACT*)y, B, d);
  return check_launch("mixer_core_big");
}

int launch_mixer_core_big_dispatch(const void* xproj, const float* u, const float* sw, const float* sb,
                                   const float* pbias, const float* spec, void* y, int B, int d, int act_dtype,
                                   hipStream_t stream) {
  return act_dtype == M2_DTYPE_F32 ? launch_mixer_core_big<float>(xproj, u, sw, sb, pbias, spec, y, B, d, stream)
                                   : launch_mixer_core_big<uint16_t>(xproj, u, sw, sb, pbias, spec, y, B, d, stream);
}

int launch_filter_spectrum_big(const float* taps1, const float* taps2, const float* D1, const float* D2, float* spec,
                               int d, hipStream_t stream) {
  const size_t lds_bytes = (size_t)BigPlan::WG_LDS * sizeof(float2);
  hipError_t e = hipFuncSetAttribute((const void*)filter_spectrum_big_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)lds_bytes);
  if (e != hipSuccess) return set_error(M2_ERR_LAUNCH, "hipFuncSetAttribute(filter_spectrum_big): %s", hipGetErrorString(e));
  int grid = num_cus();
  if (grid > d) grid = d;
  hipLaunchKernelGGL(filter_spectrum_big_kernel, dim3(grid), dim3(1024), lds_bytes, stream, taps1, taps2, D1, D2,
                     (float4*)spec, d);
  return check_launch("filter_spectrum_big");
}

}  // namespace m2
