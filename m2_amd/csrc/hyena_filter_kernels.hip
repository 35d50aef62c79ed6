// Implicit long-filter generation for the Monarch-Mixer sequence mixer on gfx950.
//
//   h0 = z_l (emb)  ->  h1 = sin(f.(W0 h0 + b0))  ->  h2 = sin(f.(W1 h1 + b1))  ->  h3 = sin(f.(W2 h2 + b2))
//   k[c][l] = (W3 h3)[c] * (exp(-t_l |delta_c|) + shift)
//
// (bert/src/mm/hyena_utils.py:168-175 the MLP, :50-63 Sin, :110-112 modulation, :201-217 filter /
// filter_rev, :231-236 placement of the forward and the flipped reverse taps in a 2L window.)
//
// Two kernels.  `hidden_kernel` evaluates the three sin layers for a tile of positions with the
// activations resident in LDS and writes h3 (L, 128) per MLP.  `project_kernel` is the 128 -> d
// projection as an fp32 MFMA GEMM (v_mfma_f32_32x32x2_f32) whose epilogue applies the decay and
// stores the taps channel-major, forward taps at [0, L) and reverse taps mirrored into [L, 2L).
#include <hip/hip_runtime.h>

#include "m2_internal.h"

namespace m2 {

constexpr int kOrder = 128;
constexpr int kMaxEmb = 8;
constexpr int kPosTile = 32;      // positions per workgroup in hidden_kernel

struct MlpPtrs {
  const float *w0, *b0, *w1, *b1, *w2, *b2, *w3;
};
struct FilterPtrs {
  const float *z, *t, *freq, *deltas;
  MlpPtrs mlp[2];                 // [0] forward, [1] reverse
};
constexpr int kMaxFilters = 4;
struct FilterBatch {
  FilterPtrs f[kMaxFilters];
};

// grid (L / kPosTile, 2 * nfilters), block 128: thread o owns output neuron o.
__global__ __launch_bounds__(kOrder) void hidden_kernel(FilterBatch fb, int L, int emb, float w_mod,
                                                        float* __restrict__ hidden /* (2 nf, L, 128) */) {
  __shared__ float act[2][kPosTile][kOrder];
  const int o = threadIdx.x;
  const int fi = blockIdx.y >> 1, dir = blockIdx.y & 1;
  const FilterPtrs& F = fb.f[fi];
  const MlpPtrs& W = F.mlp[dir];
  if (W.w0 == nullptr) return;                  // not bidirectional: nothing to do for dir == 1
  const int l0 = blockIdx.x * kPosTile;
  const float fo = w_mod * F.freq[o];

  // layer 0: emb -> 128
  {
    float w[kMaxEmb];
    for (int e = 0; e < kMaxEmb; ++e) w[e] = e < emb ? W.w0[o * emb + e] : 0.f;
    const float b = W.b0[o];
    for (int p = 0; p < kPosTile; ++p) {
      const float* zp = F.z + (long)(l0 + p) * emb;
      float acc = b;
      for (int e = 0; e < emb; ++e) acc += w[e] * zp[e];
      act[0][p][o] = sinf(fo * acc);
    }
  }
  __syncthreads();
  // layers 1, 2: 128 -> 128 with the weight row in registers and activations broadcast from LDS
  for (int layer = 0; layer < 2; ++layer) {
    const float* wrow = (layer == 0 ? W.w1 : W.w2) + (long)o * kOrder;
    const float b = (layer == 0 ? W.b1 : W.b2)[o];
    float4 w[kOrder / 4];
#pragma unroll
    for (int i = 0; i < kOrder / 4; ++i) w[i] = reinterpret_cast<const float4*>(wrow)[i];
    const int src = layer & 1, dst = src ^ 1;
    for (int p = 0; p < kPosTile; ++p) {
      const float4* a = reinterpret_cast<const float4*>(act[src][p]);
      float acc0 = b, acc1 = 0.f, acc2 = 0.f, acc3 = 0.f;
#pragma unroll
      for (int i = 0; i < kOrder / 4; ++i) {
        const float4 v = a[i];
        acc0 += w[i].x * v.x;
        acc1 += w[i].y * v.y;
        acc2 += w[i].z * v.z;
        acc3 += w[i].w * v.w;
      }
      const float s = sinf(fo * ((acc0 + acc1) + (acc2 + acc3)));
      if (layer == 0) act[dst][p][o] = s;
      else hidden[((long)blockIdx.y * L + l0 + p) * kOrder + o] = s;
    }
    __syncthreads();
  }
}

typedef float floatx16 __attribute__((ext_vector_type(16)));

// One wave computes a 64 (channels) x 64 (positions) tile of W3 (d x 128) * H^T (128 x L).
// grid (L / 64, d / 64, 2 * nfilters), block 64.
__global__ __launch_bounds__(64) void project_kernel(FilterBatch fb, int L, int d, float shift,
                                                     const float* __restrict__ hidden /* (2 nf, L, 128) */,
                                                     float* __restrict__ taps /* (nf, d, 2L) */) {
  const int fi = blockIdx.z >> 1, dir = blockIdx.z & 1;
  const FilterPtrs& F = fb.f[fi];
  const int lane = threadIdx.x, i32 = lane & 31, half = lane >> 5;
  const int c0 = blockIdx.y * 64, l0 = blockIdx.x * 64;
  float* out = taps + (long)fi * d * 2 * L;
  if (F.mlp[dir].w3 == nullptr) {
    // not bidirectional: the reverse half of the window is zero
    for (int r = 0; r < 64; ++r) out[(long)(c0 + r) * 2 * L + L + l0 + lane] = 0.f;
    return;
  }
  const float* A = F.mlp[dir].w3;                              // (d, 128), K contiguous
  const float* Bm = hidden + (long)blockIdx.z * L * kOrder;    // (L, 128), K contiguous
  floatx16 acc[2][2];
  for (int a = 0; a < 2; ++a)
    for (int b = 0; b < 2; ++b)
      for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;
  // lane (i32, half) holds K = 8q + 4 half + {0..3} of row i32: four MFMA steps per float4
  for (int q = 0; q < kOrder / 8; ++q) {
    float4 av[2], bv[2];
    for (int a = 0; a < 2; ++a) av[a] = *reinterpret_cast<const float4*>(A + (long)(c0 + 32 * a + i32) * kOrder + 8 * q + 4 * half);
    for (int b = 0; b < 2; ++b) bv[b] = *reinterpret_cast<const float4*>(Bm + (long)(l0 + 32 * b + i32) * kOrder + 8 * q + 4 * half);
    for (int a = 0; a < 2; ++a)
      for (int b = 0; b < 2; ++b) {
        acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[a].x, bv[b].x, acc[a][b], 0, 0, 0);
        acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[a].y, bv[b].y, acc[a][b], 0, 0, 0);
        acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[a].z, bv[b].z, acc[a][b], 0, 0, 0);
        acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[a].w, bv[b].w, acc[a][b], 0, 0, 0);
      }
  }
  // accumulator element v of lane: row (channel) = 8 (v / 4) + 4 half + v % 4, column (position) = i32
  for (int b = 0; b < 2; ++b) {
    const int l = l0 + 32 * b + i32;
    const float tl = F.t[l];
    const long pos = dir == 0 ? l : (2L * L - 1 - l);
    for (int a = 0; a < 2; ++a)
      for (int v = 0; v < 16; ++v) {
        const int c = c0 + 32 * a + 8 * (v >> 2) + 4 * half + (v & 3);
        const float decay = expf(-tl * fabsf(F.deltas[c])) + shift;
        out[(long)c * 2 * L + pos] = acc[a][b][v] * decay;
      }
  }
}

}  // namespace m2

using namespace m2;

extern "C" size_t m2_hyena_filter_workspace_bytes(int nfilters, int L, int order) {
  if (nfilters <= 0 || L <= 0 || order <= 0) return 0;
  return (size_t)2 * nfilters * L * order * sizeof(float);
}

extern "C" int m2_hyena_filter_fwd(const m2_hyena_filter_params* params, int nfilters, int L, int d, int order,
                                   int emb_dim, float w_mod, float shift, float* workspace, float* taps,
                                   void* stream) {
  if (!params || !workspace || !taps) return set_error(M2_ERR_ARG, "m2_hyena_filter_fwd: null pointer");
  if (nfilters < 1 || nfilters > kMaxFilters)
    return set_error(M2_ERR_UNSUPPORTED, "m2_hyena_filter_fwd: nfilters=%d not in [1, %d]", nfilters, kMaxFilters);
  if (order != kOrder) return set_error(M2_ERR_UNSUPPORTED, "m2_hyena_filter_fwd: order=%d, only 128 is built", order);
  if (emb_dim < 3 || emb_dim > kMaxEmb)
    return set_error(M2_ERR_UNSUPPORTED, "m2_hyena_filter_fwd: emb_dim=%d not in [3, %d]", emb_dim, kMaxEmb);
  if (L <= 0 || L % 64 != 0) return set_error(M2_ERR_UNSUPPORTED, "m2_hyena_filter_fwd: L=%d must be a positive multiple of 64", L);
  if (d <= 0 || d % 64 != 0) return set_error(M2_ERR_UNSUPPORTED, "m2_hyena_filter_fwd: d=%d must be a positive multiple of 64", d);
  FilterBatch fb;
  for (int f = 0; f < kMaxFilters; ++f) {
    const m2_hyena_filter_params& p = params[f < nfilters ? f : 0];
    if (!p.z || !p.t || !p.freq || !p.deltas || !p.w0 || !p.b0 || !p.w1 || !p.b1 || !p.w2 || !p.b2 || !p.w3)
      return set_error(M2_ERR_ARG, "m2_hyena_filter_fwd: filter %d has a null forward-MLP pointer", f);
    const bool rev = p.rw0 != nullptr;
    if (rev && (!p.rb0 || !p.rw1 || !p.rb1 || !p.rw2 || !p.rb2 || !p.rw3))
      return set_error(M2_ERR_ARG, "m2_hyena_filter_fwd: filter %d has a partly null reverse MLP", f);
    fb.f[f].z = p.z; fb.f[f].t = p.t; fb.f[f].freq = p.freq; fb.f[f].deltas = p.deltas;
    fb.f[f].mlp[0] = MlpPtrs{p.w0, p.b0, p.w1, p.b1, p.w2, p.b2, p.w3};
    fb.f[f].mlp[1] = rev ? MlpPtrs{p.rw0, p.rb0, p.rw1, p.rb1, p.rw2, p.rb2, p.rw3}
                         : MlpPtrs{nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
  }
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(hidden_kernel, dim3(L / kPosTile, 2 * nfilters), dim3(kOrder), 0, s, fb, L, emb_dim, w_mod, workspace);
  int rc = check_launch("hyena hidden_kernel");
  if (rc) return rc;
  hipLaunchKernelGGL(project_kernel, dim3(L / 64, d / 64, 2 * nfilters), dim3(64), 0, s, fb, L, d, shift, workspace, taps);
  return check_launch("hyena project_kernel");
}
