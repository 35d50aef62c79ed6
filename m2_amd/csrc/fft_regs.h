// In-register radix-2^k FFT building blocks for 64-wide CDNA wavefronts.
//
// A thread holds R complex points in registers.  `dif<R>` runs a forward decimation-in-frequency
// transform whose outputs land in bit-reversed register order (X_k in x[bitrev(k)]);
// `dit<R>` is its exact unscaled inverse: it consumes bit-reversed register order and leaves
// natural order.  All twiddles inside a radix-R block are compile-time constants, so the
// trivial ones (1, -i, (1-i)/sqrt2 ...) cost adds only.
#pragma once
#include <hip/hip_runtime.h>
#include <utility>

namespace m2 {

struct cf {            // complex float; kept as two scalars so that nothing is forced into pairs
  float re, im;
};

__device__ __forceinline__ cf cadd(cf a, cf b) { return {a.re + b.re, a.im + b.im}; }
__device__ __forceinline__ cf csub(cf a, cf b) { return {a.re - b.re, a.im - b.im}; }
__device__ __forceinline__ cf cmul(cf a, cf b) {
  return {a.re * b.re - a.im * b.im, a.re * b.im + a.im * b.re};
}
// a * conj(b)
__device__ __forceinline__ cf cmulc(cf a, cf b) {
  return {a.re * b.re + a.im * b.im, a.im * b.re - a.re * b.im};
}
__device__ __forceinline__ cf cconj(cf a) { return {a.re, -a.im}; }

template <int I> using ic = std::integral_constant<int, I>;

template <int B, int E, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (B < E) {
    f(ic<B>{});
    static_for<B + 1, E>(f);
  }
}

constexpr int bitrev(int v, int bits) {
  int r = 0;
  for (int i = 0; i < bits; ++i) r |= ((v >> i) & 1) << (bits - 1 - i);
  return r;
}
constexpr int ilog2(int v) { return v <= 1 ? 0 : 1 + ilog2(v >> 1); }

// cos/sin of 2*pi*k/32, k = 0..8 (first quadrant is enough; the rest by symmetry)
constexpr float kCos32[9] = {1.0f,
                             0.98078528040323044913f,
                             0.92387953251128675613f,
                             0.83146961230254523708f,
                             0.70710678118654752440f,
                             0.55557023301960222474f,
                             0.38268343236508977173f,
                             0.19509032201612826785f,
                             0.0f};
constexpr float cos32(int k) {        // k in [0, 32)
  k &= 31;
  return k <= 8 ? kCos32[k] : k <= 16 ? -kCos32[16 - k] : k <= 24 ? -kCos32[k - 16] : kCos32[32 - k];
}
constexpr float sin32(int k) { return cos32(k - 8 + 32); }

// multiply by exp(-+ 2*pi*i * K/32): forward (INV=false) uses the minus sign.
template <int K, bool INV>
__device__ __forceinline__ cf mul_w32(cf v) {
  constexpr int k = ((K % 32) + 32) % 32;
  if constexpr (k == 0) {
    return v;
  } else if constexpr (k == 16) {
    return {-v.re, -v.im};
  } else if constexpr (k == 8) {            // fwd: * (-i)   inv: * (+i)
    if constexpr (!INV) return {v.im, -v.re};
    else return {-v.im, v.re};
  } else if constexpr (k == 24) {
    if constexpr (!INV) return {-v.im, v.re};
    else return {v.im, -v.re};
  } else if constexpr (k % 8 == 4) {        // odd multiples of pi/4: (+-1 +- i)/sqrt2
    constexpr float h = 0.70710678118654752440f;
    constexpr float c = cos32(k) > 0 ? 1.0f : -1.0f;
    constexpr float s0 = sin32(k) > 0 ? 1.0f : -1.0f;
    constexpr float s = INV ? s0 : -s0;     // multiply by c + i*s (times h)
    // (re + i im)(c + i s) = (c re - s im) + i (c im + s re)
    return {h * (c * v.re - s * v.im), h * (c * v.im + s * v.re)};
  } else {
    constexpr float c = cos32(k);
    constexpr float s = INV ? sin32(k) : -sin32(k);
    return {c * v.re - s * v.im, c * v.im + s * v.re};
  }
}

// Forward DIF on x[BASE .. BASE+R): natural in, bit-reversed out.
template <int R, int BASE, int NREG>
__device__ __forceinline__ void dif(cf (&x)[NREG]) {
  if constexpr (R > 1) {
    constexpr int H = R / 2;
    static_for<0, H>([&](auto j) {
      cf a = x[BASE + j], b = x[BASE + j + H];
      x[BASE + j] = cadd(a, b);
      x[BASE + j + H] = mul_w32<j * (32 / R), false>(csub(a, b));
    });
    dif<H, BASE, NREG>(x);
    dif<H, BASE + H, NREG>(x);
  }
}

// Forward DIF when inputs BASE+R/2 .. BASE+R are known to be zero (zero-padded upper half).
template <int R, int BASE, int NREG>
__device__ __forceinline__ void dif_zero_upper(cf (&x)[NREG]) {
  constexpr int H = R / 2;
  static_for<0, H>([&](auto j) { x[BASE + j + H] = mul_w32<j * (32 / R), false>(x[BASE + j]); });
  dif<H, BASE, NREG>(x);
  dif<H, BASE + H, NREG>(x);
}

// Unscaled inverse: bit-reversed in, natural out.
template <int R, int BASE, int NREG>
__device__ __forceinline__ void dit(cf (&x)[NREG]) {
  if constexpr (R > 1) {
    constexpr int H = R / 2;
    dit<H, BASE, NREG>(x);
    dit<H, BASE + H, NREG>(x);
    static_for<0, H>([&](auto j) {
      cf a = x[BASE + j];
      cf b = mul_w32<j * (32 / R), true>(x[BASE + j + H]);
      x[BASE + j] = cadd(a, b);
      x[BASE + j + H] = csub(a, b);
    });
  }
}

// Same, but only outputs BASE .. BASE+R/2 are produced (the upper half is not needed).
template <int R, int BASE, int NREG>
__device__ __forceinline__ void dit_lower_only(cf (&x)[NREG]) {
  constexpr int H = R / 2;
  dit<H, BASE, NREG>(x);
  dit<H, BASE + H, NREG>(x);
  static_for<0, H>([&](auto j) {
    x[BASE + j] = cadd(x[BASE + j], mul_w32<j * (32 / R), true>(x[BASE + j + H]));
  });
}

// Powers w^1 .. w^(R-1) of a unit complex number with depth-log2 products.
// p[k] = w^k for k = 1..R-1; p[0] is never read.
template <int R>
__device__ __forceinline__ void powers(cf w, cf (&p)[R]) {
  p[1] = w;
  static_for<2, R>([&](auto k) {
    constexpr int a = (k + 1) / 2, b = k / 2;     // k = a + b, both already computed
    p[k] = cmul(p[a], p[b]);
  });
}

}  // namespace m2
