// Row input / output helpers shared by the long-convolution kernels: 16-byte global accesses of
// 8 consecutive activations (fp32 or bf16 storage), converted to and from fp32 registers.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "m2_internal.h"

namespace m2 {

// 8 consecutive outputs from fp32 registers, one or two 16-byte stores
__device__ __forceinline__ void store8(float* p, int n0, const float (&v)[8]) {
  *reinterpret_cast<float4*>(p + n0) = make_float4(v[0], v[1], v[2], v[3]);
  *reinterpret_cast<float4*>(p + n0 + 4) = make_float4(v[4], v[5], v[6], v[7]);
}
__device__ __forceinline__ void store8(uint16_t* p, int n0, const float (&v)[8]) {
  uint4 o;
  o.x = pack_bf16x2(v[0], v[1]);
  o.y = pack_bf16x2(v[2], v[3]);
  o.z = pack_bf16x2(v[4], v[5]);
  o.w = pack_bf16x2(v[6], v[7]);
  *reinterpret_cast<uint4*>(p + n0) = o;
}

// 8 consecutive activations starting at element n0 (n0 % 8 == 0) plus the two before them, as fp32:
// out[0], out[1] = in[n0-2], in[n0-1] (zero when n0 == 0), out[2..10) = in[n0 .. n0+8); `add` is added to every
// element that exists (the two before n0 == 0 stay zero: that is the convolution's zero padding, which sits
// outside the biased signal).  Split into the loads (`fetch`, raw bits) and the conversion (`expand`), so that a
// kernel can put all loads of a row in flight before it starts converting.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
// Raw registers of one access.  Kept as separate arrays of plain vectors (RawRow<ACT, Q>::a / b / h), not as
// an array of structs: only the former are reliably promoted to registers.
// CHAINED: the Q accesses are consecutive (access I starts where access I - 1 ends), so only access 0 fetches the
// two elements before it; the others take them from the registers of their predecessor.
template <typename ACT, int Q, bool CHAINED = false> struct RawRow;
template <int Q, bool CHAINED> struct RawRow<float, Q, CHAINED> {
  f32x4_t a[Q], b[Q];
  f32x2_t h[Q];
  template <int I> __device__ __forceinline__ void fetch(const float* p, int n0) {
    a[I] = *reinterpret_cast<const f32x4_t*>(p + n0);
    b[I] = *reinterpret_cast<const f32x4_t*>(p + n0 + 4);
    if constexpr (!(CHAINED && I > 0))
      h[I] = *reinterpret_cast<const f32x2_t*>(p + (n0 > 0 ? n0 - 2 : 0));      // unused when n0 == 0
  }
  template <int I> __device__ __forceinline__ f32x2_t before() const {
    if constexpr (CHAINED && I > 0) return f32x2_t{b[I - 1].z, b[I - 1].w};
    else return h[I];
  }
  template <int I> __device__ __forceinline__ void expand(int n0, float add, float (&o)[10]) const {
    const f32x2_t hh = before<I>();
    o[0] = n0 > 0 ? hh.x + add : 0.f;
    o[1] = n0 > 0 ? hh.y + add : 0.f;
    o[2] = a[I].x + add; o[3] = a[I].y + add; o[4] = a[I].z + add; o[5] = a[I].w + add;
    o[6] = b[I].x + add; o[7] = b[I].y + add; o[8] = b[I].z + add; o[9] = b[I].w + add;
  }
  // the same without the addend (no add instructions at all)
  template <int I> __device__ __forceinline__ void expand(int n0, float (&o)[10]) const {
    const f32x2_t hh = before<I>();
    o[0] = n0 > 0 ? hh.x : 0.f;
    o[1] = n0 > 0 ? hh.y : 0.f;
    o[2] = a[I].x; o[3] = a[I].y; o[4] = a[I].z; o[5] = a[I].w;
    o[6] = b[I].x; o[7] = b[I].y; o[8] = b[I].z; o[9] = b[I].w;
  }
};
template <int Q, bool CHAINED> struct RawRow<uint16_t, Q, CHAINED> {
  u32x4_t a[Q];
  uint32_t h[Q];
  template <int I> __device__ __forceinline__ void fetch(const uint16_t* p, int n0) {
    a[I] = *reinterpret_cast<const u32x4_t*>(p + n0);
    if constexpr (!(CHAINED && I > 0))
      h[I] = *reinterpret_cast<const uint32_t*>(p + (n0 > 0 ? n0 - 2 : 0));     // unused when n0 == 0
  }
  template <int I> __device__ __forceinline__ uint32_t before() const {
    if constexpr (CHAINED && I > 0) return a[I - 1].w;
    else return h[I];
  }
  template <int I> __device__ __forceinline__ void expand(int n0, float add, float (&o)[10]) const {
    const uint32_t hh = before<I>();
    o[0] = n0 > 0 ? __uint_as_float(hh << 16) + add : 0.f;
    o[1] = n0 > 0 ? __uint_as_float(hh & 0xffff0000u) + add : 0.f;
    o[2] = __uint_as_float(a[I].x << 16) + add; o[3] = __uint_as_float(a[I].x & 0xffff0000u) + add;
    o[4] = __uint_as_float(a[I].y << 16) + add; o[5] = __uint_as_float(a[I].y & 0xffff0000u) + add;
    o[6] = __uint_as_float(a[I].z << 16) + add; o[7] = __uint_as_float(a[I].z & 0xffff0000u) + add;
    o[8] = __uint_as_float(a[I].w << 16) + add; o[9] = __uint_as_float(a[I].w & 0xffff0000u) + add;
  }
  template <int I> __device__ __forceinline__ void expand(int n0, float (&o)[10]) const {
    const uint32_t hh = before<I>();
    o[0] = n0 > 0 ? __uint_as_float(hh << 16) : 0.f;
    o[1] = n0 > 0 ? __uint_as_float(hh & 0xffff0000u) : 0.f;
    o[2] = __uint_as_float(a[I].x << 16); o[3] = __uint_as_float(a[I].x & 0xffff0000u);
    o[4] = __uint_as_float(a[I].y << 16); o[5] = __uint_as_float(a[I].y & 0xffff0000u);
    o[6] = __uint_as_float(a[I].z << 16); o[7] = __uint_as_float(a[I].z & 0xffff0000u);
    o[8] = __uint_as_float(a[I].w << 16); o[9] = __uint_as_float(a[I].w & 0xffff0000u);
  }
};

// The gate sc(x2) of 8 Q time steps, held across the transforms.  With bf16 activations it is kept as
// packed bf16 (the reference's short convolution writes bf16 under autocast,
// bert/src/mm/monarch_mixer_sequence_mixer.py:112-118), with fp32 activations as fp32.
template <typename ACT, int Q> struct GateRow;
template <int Q> struct GateRow<float, Q> {
  float g[8 * Q];
  template <int I> __device__ __forceinline__ void set(const float (&v)[8]) {
#pragma unroll
    for (int i = 0; i < 8; ++i) g[8 * I + i] = v[i];
  }
  template <int I> __device__ __forceinline__ float get() const { return g[I]; }
};
template <int Q> struct GateRow<uint16_t, Q> {
  uint32_t g[4 * Q];
  template <int I> __device__ __forceinline__ void set(const float (&v)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) g[4 * I + i] = pack_bf16x2(v[2 * i], v[2 * i + 1]);
  }
  template <int I> __device__ __forceinline__ float get() const {
    return (I & 1) ? __uint_as_float(g[I / 2] & 0xffff0000u) : __uint_as_float(g[I / 2] << 16);
  }
};

}  // namespace m2
