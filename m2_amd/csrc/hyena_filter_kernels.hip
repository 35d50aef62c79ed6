// Implicit long-filter generation for the Monarch-Mixer sequence mixer on gfx950.
//
//   h0 = z_l (emb)  ->  h1 = sin(f.(W0 h0 + b0))  ->  h2 = sin(f.(W1 h1 + b1))  ->  h3 = sin(f.(W2 h2 + b2))
//   k[c][l] = (W3 h3)[c] * (exp(-t_l |delta_c|) + shift)
//
// (bert/src/mm/hyena_utils.py:168-175 the MLP, :50-63 Sin, :110-112 modulation, :201-217 filter /
// filter_rev, :231-236 placement of the forward and the flipped reverse taps in a 2L window.)
//
// Three kernels.  `split_weights_kernel` re-splits the 128 x 128 weights of the two inner layers into three bf16
// parts in MFMA operand layout (a few microseconds, once per call).  `hidden_kernel` evaluates the three sin layers
// for 32 - 128 positions per workgroup: the first (emb -> 128) on the vector ALU, the two 128 x 128 layers as
// six-product split-bf16 MFMA GEMMs (v_mfma_f32_32x32x16_bf16 on the three parts of weights and activations: all
// product terms down to 2^-24, i.e. fp32 products, which matters because sin(freq * x) amplifies any rounding of
// x) with the activations resident in LDS; it writes h3 split into a bf16 high part and a bf16 low part
// (h3 = hi + lo to 16 mantissa bits).  `project_kernel` is the 128 -> d projection as a three-product split-bf16
// MFMA GEMM (W_hi h_hi + W_hi h_lo + W_lo h_hi, fp32 accumulate; 4.6e-6 relative error against fp64, measured)
// whose epilogue applies the decay and stores the taps channel-major, forward taps at [0, L) and reverse taps
// mirrored into [L, 2L).  For L >= 1024 the last two are one launch (`hidden_kernel<2, ., PROJECT = true>`: the
// workgroup that evaluated the hidden layers of 64 positions goes on to project them, h3 never leaves LDS); for
// L <= 512 the batched entry point hands h3 to the projection + spectrum kernel of filter_fused_kernels.hip instead.
#include <hip/hip_runtime.h>

#include <mutex>

#include "hyena_filter.h"

namespace m2 {

constexpr int kPosTile = 32;      // positions per workgroup in hidden_kernel

// sin(x) by two-constant Cody-Waite reduction to [-pi/2, pi/2] (fused multiply-adds keep the reduction
// exact to ~1e-15 n) and the odd Taylor polynomial to x^11 (truncation 5.6e-8 at pi/2).  Absolute error
// ~1e-7 for |x| up to ~1e4, i.e. fp32 sinf quality over the whole range freq * x can take here, at a
// third of the instructions of the libm routine (which carries a slow path for huge arguments).
__device__ __forceinline__ float sin_reduced(float x) {
  const float n = rintf(x * 0.318309886183790672f);
  float r = fmaf(-n, 3.14159274101257324f, x);
  r = fmaf(-n, -8.74227765734758577e-8f, r);
  const float r2 = r * r;
  float p = -2.50521083854417188e-8f;          // -1/11!
  p = fmaf(p, r2, 2.75573192239858907e-6f);    //  1/9!
  p = fmaf(p, r2, -1.98412698412698413e-4f);   // -1/7!
  p = fmaf(p, r2, 8.33333333333333322e-3f);    //  1/5!
  p = fmaf(p, r2, -1.66666666666666657e-1f);   // -1/3!
  const float s = fmaf(p * r2, r, r);
  return (static_cast<int>(n) & 1) ? -s : s;
}

__device__ __forceinline__ bf16x8 as_bf16x8(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  u32x4 v = {a, b, c, d};
  return __builtin_bit_cast(bf16x8, v);
}

// The 128 x 128 weights of the two inner layers, split into three bf16 parts and laid out as MFMA A operands, so
// that hidden_kernel fetches them with coalesced 16-byte loads and no arithmetic:
// wsplit[mlp][layer][part][wave w][K step ks][lane (i, h)] = 8 bf16 of row 32 w + i, K = 16 ks + 8 h .. + 7.
// The d x 128 output projection likewise, in two parts (hi, lo), for project_kernel:
// w3split[mlp][part][32-channel tile][K step ks][lane (i, h)] = 8 bf16 of row 32 tile + i, K = 16 ks + 8 h .. + 7.
constexpr int kSplitPerLayer = 3 * kOrder * kOrder;      // bf16 elements per (mlp, layer)
template <class TAB>
__global__ __launch_bounds__(256) void split_weights_kernel(TAB tab, int nmlp, int d, uint16_t* __restrict__ wsplit,
                                                            uint16_t* __restrict__ w3split) {
  const int inner_blocks = nmlp * 2 * 4 * 8 * 64 / 256;
  if ((int)blockIdx.x >= inner_blocks) {
    const int id = ((int)blockIdx.x - inner_blocks) * 256 + threadIdx.x;      // (mlp, channel tile, ks, lane)
    const int lane = id & 63, ks = (id >> 6) & 7, ct = (id >> 9) % (d / 32), m = (id >> 9) / (d / 32);
    if (m >= nmlp) return;
    const MlpPtrs& W = tab.at(m >> 1).mlp[m & 1];
    if (W.w3 == nullptr) return;
    const float* src = W.w3 + (long)(32 * ct + (lane & 31)) * kOrder + 16 * ks + 8 * (lane >> 5);
    float h[8], l[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      h[j] = bf16_to_f32(f32_to_bf16(src[j]));
      l[j] = src[j] - h[j];
    }
    u32x4* dst = reinterpret_cast<u32x4*>(w3split + (long)m * 2 * d * kOrder) + (ct * 8 + ks) * 64 + lane;
    const u32x4 vh = {pack_bf16x2(h[0], h[1]), pack_bf16x2(h[2], h[3]), pack_bf16x2(h[4], h[5]), pack_bf16x2(h[6], h[7])};
    const u32x4 vl = {pack_bf16x2(l[0], l[1]), pack_bf16x2(l[2], l[3]), pack_bf16x2(l[4], l[5]), pack_bf16x2(l[6], l[7])};
    dst[0] = vh;
    dst[d * kOrder / 8] = vl;
    return;
  }
  const int id = blockIdx.x * 256 + threadIdx.x;             // (mlp, layer, wave, ks, lane)
  const int lane = id & 63, ks = (id >> 6) & 7, w = (id >> 9) & 3, layer = (id >> 11) & 1, m = id >> 12;
  if (m >= nmlp) return;
  const MlpPtrs& W = tab.at(m >> 1).mlp[m & 1];
  if (W.w0 == nullptr) return;
  const float* src = (layer == 0 ? W.w1 : W.w2) + (long)(32 * w + (lane & 31)) * kOrder + 16 * ks + 8 * (lane >> 5);
  float h[8], md[8], l[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) split3(src[j], h[j], md[j], l[j]);
  u32x4* dst = reinterpret_cast<u32x4*>(wsplit + ((long)(m * 2 + layer)) * kSplitPerLayer) + (w * 8 + ks) * 64 + lane;
  const u32x4 vh = {pack_bf16x2(h[0], h[1]), pack_bf16x2(h[2], h[3]), pack_bf16x2(h[4], h[5]), pack_bf16x2(h[6], h[7])};
  const u32x4 vm = {pack_bf16x2(md[0], md[1]), pack_bf16x2(md[2], md[3]), pack_bf16x2(md[4], md[5]), pack_bf16x2(md[6], md[7])};
  const u32x4 vl = {pack_bf16x2(l[0], l[1]), pack_bf16x2(l[2], l[3]), pack_bf16x2(l[4], l[5]), pack_bf16x2(l[6], l[7])};
  dst[0] = vh;
  dst[kOrder * kOrder / 8] = vm;
  dst[2 * kOrder * kOrder / 8] = vl;
}

constexpr int kActRowB = 2 * kOrder + 16;     // bytes per padded bf16 row of an activation part (conflict-free 16-byte reads)

// grid (L / (32 TILES), 2 * nfilters), block 256 = 4 waves.  Wave w owns the output neurons [32 w, 32 w + 32) of all
// TILES tiles of 32 positions of the workgroup.  The activations live in LDS as three bf16 parts (hi, mid, lo:
// together the fp32 value) and every layer overwrites them in place; the two 128 x 128 layers are six-product
// split-bf16 MFMA GEMMs (all products of the three parts of either operand down to 2^-24 relative: fp32 accuracy,
// which matters because sin(freq * x) amplifies any rounding of x, at 2.7 times the rate of fp32 MFMAs), their
// weights pre-split by split_weights_kernel and held in registers for all tiles (fetching them is what a short run
// of positions per workgroup pays most for: 96 KB per workgroup and layer from L2).  Within a layer the products of
// tile i + 1 are issued together with the sin epilogue of tile i, so that matrix pipe and vector ALU overlap.
//
// PROJECT = true: the same workgroup goes on to the 128 -> d output projection of its positions (the last hidden
// layer's activations stay in LDS as bf16 hi / lo parts instead of travelling through memory): wave w takes the
// 32-channel tiles w, w + 4, ..., fetches the tile's pre-split weight rows (hi / lo parts in operand layout, from L2:
// every workgroup reads all of them once), multiplies (three products: W_hi h_hi + W_hi h_lo + W_lo h_hi), applies
// exp(-t |delta|) + shift and stores the taps channel-major with streaming stores, forward taps at [0, L), reverse taps
// mirrored into [L, 2L) (bert/src/mm/hyena_utils.py:175,213-217,233-234).
template <int TILES, class TAB, bool PROJECT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void hidden_kernel(TAB tab, int L, int emb, float w_mod,
                                                     const uint16_t* __restrict__ wsplit,
                                                     uint16_t* __restrict__ h_hi /* (2 nf, L, 128) bf16 */,
                                                     uint16_t* __restrict__ h_lo /* (2 nf, L, 128) bf16 */,
                                                     int d, float shift, const uint16_t* __restrict__ w3split,
                                                     float* __restrict__ taps /* (nf, d, 2L) */) {
  constexpr int P = 32 * TILES;
  __shared__ __attribute__((aligned(16))) unsigned char act[3][P * kActRowB];
  __shared__ float zt[P * kMaxEmb];
  const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, i32 = lane & 31, half = lane >> 5;
  const int fi = blockIdx.y >> 1, dir = blockIdx.y & 1;
  const FilterPtrs& F = tab.at(fi);
  const MlpPtrs& W = F.mlp[dir];
  const int l0 = blockIdx.x * P;
  if (W.w0 == nullptr) {                        // not bidirectional: nothing to compute for dir == 1 ...
    if constexpr (PROJECT) {                    // ... and the reverse half of the window is zero
      float* out = taps + (long)fi * d * 2 * L + (2L * L - l0 - P);
      for (int i = tid; i < d * P; i += 256) out[(long)(i / P) * 2 * L + i % P] = 0.f;
    }
    return;
  }

  auto put3 = [&](int pos, int o, float v0, float v1, float v2, float v3) __attribute__((always_inline)) {
    float h[4], m[4], l[4];
    split3(v0, h[0], m[0], l[0]); split3(v1, h[1], m[1], l[1]); split3(v2, h[2], m[2], l[2]); split3(v3, h[3], m[3], l[3]);
    const int off = pos * kActRowB + 2 * o;
    *reinterpret_cast<uint2*>(&act[0][off]) = make_uint2(pack_bf16x2(h[0], h[1]), pack_bf16x2(h[2], h[3]));
    *reinterpret_cast<uint2*>(&act[1][off]) = make_uint2(pack_bf16x2(m[0], m[1]), pack_bf16x2(m[2], m[3]));
    *reinterpret_cast<uint2*>(&act[2][off]) = make_uint2(pack_bf16x2(l[0], l[1]), pack_bf16x2(l[2], l[3]));
  };

  // Weights of an inner layer -> registers.  Requested one phase early (layer 1's before the vector-ALU layer, layer
  // 2's before the last epilogue of layer 1), so that the 24 KB per wave arrive behind other work.
  bf16x8 ah[8], am[8], al[8];
  auto load_weights = [&](int layer) __attribute__((always_inline)) {
    const u32x4* wp = reinterpret_cast<const u32x4*>(wsplit + ((long)(blockIdx.y * 2 + layer)) * kSplitPerLayer) + w * 8 * 64 + lane;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      ah[ks] = __builtin_bit_cast(bf16x8, wp[ks * 64]);
      am[ks] = __builtin_bit_cast(bf16x8, wp[ks * 64 + kOrder * kOrder / 8]);
      al[ks] = __builtin_bit_cast(bf16x8, wp[ks * 64 + 2 * kOrder * kOrder / 8]);
    }
  };
  load_weights(0);

  // layer 0 (emb -> 128) on the vector ALU: thread = (4 neurons, P / 8 positions).  The embeddings of the tile
  // (P x emb consecutive floats) go through LDS; weights beyond emb are zero so the dot product has a fixed length.
  {
    for (int i = tid; i < P * kMaxEmb; i += 256) zt[i] = i < P * emb ? F.z[(long)l0 * emb + i] : 0.f;
    const int o = 4 * (tid & 31), p0 = tid >> 5;          // positions p0, p0 + 8, ...
    float wt[4][kMaxEmb], bb[4], fo[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int e = 0; e < kMaxEmb; ++e) wt[j][e] = e < emb ? W.w0[(o + j) * emb + e] : 0.f;
      bb[j] = W.b0[o + j];
      fo[j] = w_mod * F.freq[o + j];
    }
    __syncthreads();
#pragma unroll 4
    for (int pp = 0; pp < P / 8; ++pp) {
      const int pos = p0 + 8 * pp;
      float s[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float acc = bb[j];
#pragma unroll
        for (int e = 0; e < kMaxEmb; ++e) acc += wt[j][e] * zt[pos * emb + e];      // pos emb + e < P emb + 8 <= P kMaxEmb
        s[j] = sin_reduced(fo[j] * acc);
      }
      put3(pos, o, s[0], s[1], s[2], s[3]);
    }
  }
  // layers 1, 2: D[o'][pos] = sum_o W[o'][o] act[pos][o].  A = weight rows 32 w + i32 (registers), B = positions of the
  // tile (LDS); lane (i32, half) holds K = 16 ks + 8 half .. + 7 of both.
  auto products = [&](int tile, floatx16& acc) __attribute__((always_inline)) {
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = 0.f;
    const int boff = (32 * tile + i32) * kActRowB + 16 * half;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      const bf16x8 bh = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(&act[0][boff + 32 * ks]));
      const bf16x8 bm = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(&act[1][boff + 32 * ks]));
      const bf16x8 bl = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(&act[2][boff + 32 * ks]));
      // smallest terms first
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al[ks], bh, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah[ks], bl, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(am[ks], bm, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(am[ks], bh, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah[ks], bm, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah[ks], bh, acc, 0, 0, 0);
    }
  };
  // accumulator element v: neuron 32 w + 8 (v / 4) + 4 half + v % 4, position i32 of the tile
  float fr[16], bs[16];
  auto load_scales = [&](int layer) __attribute__((always_inline)) {
    const float* bias = layer == 0 ? W.b1 : W.b2;
#pragma unroll
    for (int vq = 0; vq < 4; ++vq) {
      const int o = 32 * w + 8 * vq + 4 * half;
      const float4 fq = *reinterpret_cast<const float4*>(F.freq + o);
      const float4 bq = *reinterpret_cast<const float4*>(bias + o);
      fr[4 * vq] = w_mod * fq.x; fr[4 * vq + 1] = w_mod * fq.y; fr[4 * vq + 2] = w_mod * fq.z; fr[4 * vq + 3] = w_mod * fq.w;
      bs[4 * vq] = bq.x; bs[4 * vq + 1] = bq.y; bs[4 * vq + 2] = bq.z; bs[4 * vq + 3] = bq.w;
    }
  };
  auto epilogue = [&](auto ll, int tile, const floatx16& acc) __attribute__((always_inline)) {
    constexpr int layer = decltype(ll)::value;
    const int pos = 32 * tile + i32;
#pragma unroll
    for (int vq = 0; vq < 4; ++vq) {
      const int o = 32 * w + 8 * vq + 4 * half;
      float s[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) s[j] = sin_reduced(fr[4 * vq + j] * (acc[4 * vq + j] + bs[4 * vq + j]));
      if constexpr (layer == 0) {
        put3(pos, o, s[0], s[1], s[2], s[3]);
      } else if constexpr (PROJECT) {           // h3 = hi + lo stays in LDS (parts 0 and 1) for the projection
        float hi[4], lo[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          hi[j] = bf16_to_f32(f32_to_bf16(s[j]));
          lo[j] = s[j] - hi[j];
        }
        const int off = pos * kActRowB + 2 * o;
        *reinterpret_cast<uint2*>(&act[0][off]) = make_uint2(pack_bf16x2(hi[0], hi[1]), pack_bf16x2(hi[2], hi[3]));
        *reinterpret_cast<uint2*>(&act[1][off]) = make_uint2(pack_bf16x2(lo[0], lo[1]), pack_bf16x2(lo[2], lo[3]));
      } else {
        const long hrow = ((long)blockIdx.y * L + l0 + pos) * kOrder;
        float hi[4], lo[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          hi[j] = bf16_to_f32(f32_to_bf16(s[j]));
          lo[j] = s[j] - hi[j];
        }
        *reinterpret_cast<uint2*>(h_hi + hrow + o) = make_uint2(pack_bf16x2(hi[0], hi[1]), pack_bf16x2(hi[2], hi[3]));
        *reinterpret_cast<uint2*>(h_lo + hrow + o) = make_uint2(pack_bf16x2(lo[0], lo[1]), pack_bf16x2(lo[2], lo[3]));
      }
    }
  };
  // One layer: products(0); then for every tile "barrier; products(next tile) with epilogue(this tile)".  The barrier
  // before an epilogue says that all four waves have read that tile's operands, so it may be overwritten in place;
  // the barrier that ends the layer says that all of the layer's activations are written.
  auto layer_pass = [&](auto ll) __attribute__((always_inline)) {
    constexpr int layer = decltype(ll)::value;
    floatx16 acc[2];
    products(0, acc[0]);
    static_for<0, TILES>([&](auto tt) {
      constexpr int t = decltype(tt)::value;
      __syncthreads();
      if constexpr (t + 1 < TILES) products(t + 1, acc[(t + 1) & 1]);
      else if constexpr (layer == 0) load_weights(1);      // the products of layer 1 are done: its registers are free
      epilogue(ll, t, acc[t & 1]);
    });
    __syncthreads();
  };
  load_scales(0);
  __syncthreads();                     // layer 0's activations are complete
  layer_pass(ic<0>{});
  load_scales(1);
  layer_pass(ic<1>{});

  if constexpr (PROJECT) {
    // the barrier that ended the last layer says h3 (hi in act[0], lo in act[1]) is complete for all P positions
    float* out = taps + (long)fi * d * 2 * L;
    const u32x4* w3 = reinterpret_cast<const u32x4*>(w3split + (long)blockIdx.y * 2 * d * kOrder) + lane;
    float tl[TILES];
#pragma unroll
    for (int t = 0; t < TILES; ++t) tl[t] = F.t[l0 + 32 * t + i32];
    // A operand of a channel tile: weight rows 32 ct + i32, K = 16 ks + 8 half + {0..7}, hi / lo parts as
    // split_weights_kernel left them, and the decay rates of the lane's 16 channels
    struct TileOps {
      bf16x8 ahi[kOrder / 16], alo[kOrder / 16];
      float4 dq[4];
    };
    auto fetch_tile = [&](int ct, TileOps& o) __attribute__((always_inline)) {
#pragma unroll
      for (int ks = 0; ks < kOrder / 16; ++ks) {
        o.ahi[ks] = __builtin_bit_cast(bf16x8, w3[(ct * 8 + ks) * 64]);
        o.alo[ks] = __builtin_bit_cast(bf16x8, w3[(ct * 8 + ks) * 64 + d * kOrder / 8]);
      }
#pragma unroll
      for (int vq = 0; vq < 4; ++vq) o.dq[vq] = *reinterpret_cast<const float4*>(F.deltas + 32 * ct + 8 * vq + 4 * half);
    };
    auto project_tile = [&](int ct, const TileOps& o) __attribute__((always_inline)) {
      float adelta[16];
#pragma unroll
      for (int vq = 0; vq < 4; ++vq) {
        adelta[4 * vq] = -fabsf(o.dq[vq].x) * 1.44269504088896341f; adelta[4 * vq + 1] = -fabsf(o.dq[vq].y) * 1.44269504088896341f;
        adelta[4 * vq + 2] = -fabsf(o.dq[vq].z) * 1.44269504088896341f; adelta[4 * vq + 3] = -fabsf(o.dq[vq].w) * 1.44269504088896341f;
      }
#pragma unroll
      for (int t = 0; t < TILES; ++t) {
        const unsigned char* bh = &act[0][(32 * t + i32) * kActRowB + 16 * half];
        const unsigned char* bl = &act[1][(32 * t + i32) * kActRowB + 16 * half];
        floatx16 acc;
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[v] = 0.f;
#pragma unroll
        for (int ks = 0; ks < kOrder / 16; ++ks) {
          const bf16x8 bhi = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(bh + 32 * ks));
          const bf16x8 blo = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(bl + 32 * ks));
          acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(o.alo[ks], bhi, acc, 0, 0, 0);
          acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(o.ahi[ks], blo, acc, 0, 0, 0);
          acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(o.ahi[ks], bhi, acc, 0, 0, 0);
        }
        // accumulator element v of lane: channel 32 ct + 8 (v / 4) + 4 half + v % 4, position l0 + 32 t + i32
        const int l = l0 + 32 * t + i32;
        float* po = out + (long)(32 * ct + 4 * half) * 2 * L + (dir == 0 ? l : (2L * L - 1 - l));
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          // exp(-t |delta|); the bare hardware exp2 flushes results below 2^-126 to zero, which is the value to
          // 1e-38 absolute.  Streaming store: the taps are read once, by a later kernel
          const float decay = __builtin_amdgcn_exp2f(tl[t] * adelta[v]) + shift;
          __builtin_nontemporal_store(acc[v] * decay, po + (long)(8 * (v >> 2) + (v & 3)) * 2 * L);
        }
      }
    };
    // (a second register set that requests the next tile's operands ahead was measured: the registers it needs
    // beside the hidden layers' spill, 120 against 82 us per mixer at L = 8192)
    TileOps o;
    for (int ct = w; ct < d / 32; ct += 4) {
      fetch_tile(ct, o);
      project_tile(ct, o);
    }
  }
}

// Workgroup = 4 waves = 128 channels; wave w owns channels [c0 + 32 w, + 32) with its weight rows split
// into bf16 hi / lo parts held in registers.  The workgroup walks kPosPerWg positions in tiles of 32:
// the h3 tile (hi and lo parts, 16 KB) is fetched with coalesced 16-byte loads one tile ahead, staged in
// LDS (double buffered, rows padded to 272 bytes so that the 16-byte operand reads of 32 rows spread over
// all banks) and shared by the four waves.
// grid (L / kPosPerWg rounded up, d / 128 rounded up, 2 * nfilters).
constexpr int kPosPerWg = 512;      // at most; 32-position tiles past L are skipped
constexpr int kHRow = 2 * kOrder + 16;   // bytes per padded LDS row of one h3 part
template <class TAB>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 4))) void project_kernel(TAB tab, int L, int d, float shift,
                                                      const uint16_t* __restrict__ h_hi, const uint16_t* __restrict__ h_lo,
                                                      const uint16_t* __restrict__ w3split,
                                                      float* __restrict__ taps /* (nf, d, 2L) */) {
  __shared__ __attribute__((aligned(16))) unsigned char hbuf[2][2][32 * kHRow];     // [buffer][hi, lo][row]
  const int fi = blockIdx.z >> 1, dir = blockIdx.z & 1;
  const FilterPtrs& F = tab.at(fi);
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, i32 = lane & 31, half = lane >> 5;
  const int c0 = blockIdx.y * 128 + wave * 32;
  const bool active = c0 < d;                      // d is a multiple of 64: a wave is all in or all out
  const int lbase = blockIdx.x * kPosPerWg;
  float* out = taps + (long)fi * d * 2 * L;
  if (F.mlp[dir].w3 == nullptr) {
    // not bidirectional: the reverse half of the window is zero
    if (active)
      for (int r = 0; r < 32; ++r)
        for (int p = lane; p < kPosPerWg && lbase + p < L; p += 64) out[(long)(c0 + r) * 2 * L + L + lbase + p] = 0.f;
    return;
  }
  int ntiles = (L - lbase) / 32;
  if (ntiles > kPosPerWg / 32) ntiles = kPosPerWg / 32;

  // staging: thread -> two 16-byte pieces of each part of the (contiguous, 8 KB) tile
  const long tile_elems = 32L * kOrder;
  const uint16_t* gh = h_hi + ((long)blockIdx.z * L + lbase) * kOrder + 8 * tid;
  const uint16_t* gl = h_lo + ((long)blockIdx.z * L + lbase) * kOrder + 8 * tid;
  const int srow0 = tid >> 4, scol = (tid & 15) * 16;              // piece q covers row srow0 + 16 q
  // two register sets: the tile after next is in flight while the next one waits to be staged (a tile's product
  // takes well under a memory latency, so one tile of look-ahead left every iteration waiting for its fetch)
  u32x4 st[2][4];
  auto fetch = [&](int pt, auto ss) __attribute__((always_inline)) {
    constexpr int s = decltype(ss)::value;
    st[s][0] = *reinterpret_cast<const u32x4*>(gh + pt * tile_elems);
    st[s][1] = *reinterpret_cast<const u32x4*>(gh + pt * tile_elems + 16 * kOrder);
    st[s][2] = *reinterpret_cast<const u32x4*>(gl + pt * tile_elems);
    st[s][3] = *reinterpret_cast<const u32x4*>(gl + pt * tile_elems + 16 * kOrder);
  };
  auto stage = [&](int buf, auto ss) __attribute__((always_inline)) {
    constexpr int s = decltype(ss)::value;
    *reinterpret_cast<u32x4*>(&hbuf[buf][0][srow0 * kHRow + scol]) = st[s][0];
    *reinterpret_cast<u32x4*>(&hbuf[buf][0][(srow0 + 16) * kHRow + scol]) = st[s][1];
    *reinterpret_cast<u32x4*>(&hbuf[buf][1][srow0 * kHRow + scol]) = st[s][2];
    *reinterpret_cast<u32x4*>(&hbuf[buf][1][(srow0 + 16) * kHRow + scol]) = st[s][3];
  };
  fetch(0, ic<0>{});
  if (ntiles > 1) fetch(1, ic<1>{});

  // A operand: rows c0 + i32, K = 16 ks + 8 half + {0..7}, hi / lo parts as split_weights_kernel laid them out
  bf16x8 ahi[kOrder / 16], alo[kOrder / 16];
  float adelta[16];
  if (active) {
    const u32x4* wp = reinterpret_cast<const u32x4*>(w3split + (long)blockIdx.z * 2 * d * kOrder) + (c0 / 32) * 8 * 64 + lane;
#pragma unroll
    for (int ks = 0; ks < kOrder / 16; ++ks) {
      ahi[ks] = __builtin_bit_cast(bf16x8, wp[ks * 64]);
      alo[ks] = __builtin_bit_cast(bf16x8, wp[ks * 64 + d * kOrder / 8]);
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) adelta[v] = -fabsf(F.deltas[c0 + 8 * (v >> 2) + 4 * half + (v & 3)]) * 1.44269504088896341f;
  }
  stage(0, ic<0>{});
  __syncthreads();

  // iteration pt: tile pt is in hbuf[pt & 1], tile pt + 1 in register set (pt + 1) & 1; tile pt + 2 is requested into
  // the set tile pt was staged from
  auto iteration = [&](int pt, auto par) __attribute__((always_inline)) {
    constexpr int P = decltype(par)::value;      // pt & 1
    if (pt + 2 < ntiles) fetch(pt + 2, ic<P>{});
    if (active) {
      const unsigned char* bh = &hbuf[P][0][i32 * kHRow + 16 * half];
      const unsigned char* bl = &hbuf[P][1][i32 * kHRow + 16 * half];
      floatx16 acc;
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[v] = 0.f;
#pragma unroll
      for (int ks = 0; ks < kOrder / 16; ++ks) {
        const bf16x8 bhi = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(bh + 32 * ks));
        const bf16x8 blo = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(bl + 32 * ks));
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(alo[ks], bhi, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ahi[ks], blo, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ahi[ks], bhi, acc, 0, 0, 0);
      }
      // accumulator element v of lane: channel c0 + 8 (v / 4) + 4 half + v % 4, position i32
      const int l = lbase + pt * 32 + i32;
      const float tl = F.t[l];
      float* po = out + (long)(c0 + 4 * half) * 2 * L + (dir == 0 ? l : (2L * L - 1 - l));
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        // exp(-t |delta|); the bare hardware exp2 flushes results below 2^-126 to zero, which is the
        // value to 1e-38 absolute
        const float decay = __builtin_amdgcn_exp2f(tl * adelta[v]) + shift;
        // streaming store: the taps (100 MB per mixer at L = 8192) are read once, by a later kernel (-5 % for the call)
        __builtin_nontemporal_store(acc[v] * decay, po + (long)(8 * (v >> 2) + (v & 3)) * 2 * L);
      }
    }
    if (pt + 1 < ntiles) stage(P ^ 1, ic<P ^ 1>{});
    __syncthreads();
  };
  for (int pt = 0; pt < ntiles; pt += 2) {
    iteration(pt, ic<0>{});
    if (pt + 1 < ntiles) iteration(pt + 1, ic<1>{});
  }
}

}  // namespace m2

using namespace m2;

extern "C" size_t m2_hyena_filter_workspace_bytes(int nfilters, int L, int d, int order) {
  if (nfilters <= 0 || L <= 0 || d <= 0 || order <= 0) return 0;
  // h3 as bf16 hi / lo parts; the inner-layer weights of the 2 nfilters MLPs as three bf16 parts each; their output
  // projections as two
  return (size_t)2 * nfilters * L * order * sizeof(float) + (size_t)2 * nfilters * 2 * 3 * order * order * sizeof(uint16_t) +
         (size_t)2 * nfilters * 2 * d * order * sizeof(uint16_t);
}

// The three launches of a batch of filters (weight re-split, hidden layers, projection + decay), the table coming
// either by value or from device memory.  `w3split` / `taps` null: the projection is left to the caller (the fused
// projection + spectrum kernel of short sequences, which splits the projection weights itself).
template <class TAB>
static int filter_launches(TAB tab, int nfilters, int L, int d, int emb_dim, float w_mod, float shift, uint16_t* h_hi,
                           uint16_t* h_lo, uint16_t* wsplit, uint16_t* w3split, float* taps, hipStream_t s) {
  const int inner_blocks = 2 * nfilters * 2 * 4 * 8 * 64 / 256;
  const int split_blocks = inner_blocks + (w3split ? 2 * nfilters * (d / 32) * 8 * 64 / 256 : 0);
  hipLaunchKernelGGL(split_weights_kernel<TAB>, dim3(split_blocks), dim3(256), 0, s, tab, 2 * nfilters, d, wsplit, w3split);
  int rc = check_launch("hyena split_weights_kernel");
  if (rc) return rc;
  // positions per workgroup: longer runs amortise the weight fetch (96 KB per workgroup and layer), short sequences
  // need the workgroups spread over the chip
  if (L % 64 == 0 && L >= 1024) {     // measured at L = 8192: 26.9 us with two tiles, 29.5 with four, 32.7 with one
    if (taps && d % 32 == 0) {        // hidden layers and projection as one kernel: h3 never leaves the chip
      hipLaunchKernelGGL((hidden_kernel<2, TAB, true>), dim3(L / 64, 2 * nfilters), dim3(256), 0, s, tab, L, emb_dim, w_mod, wsplit,
                         h_hi, h_lo, d, shift, w3split, taps);
      return check_launch("hyena hidden + project kernel");
    }
    hipLaunchKernelGGL((hidden_kernel<2, TAB, false>), dim3(L / 64, 2 * nfilters), dim3(256), 0, s, tab, L, emb_dim, w_mod, wsplit,
                       h_hi, h_lo, 0, 0.f, nullptr, nullptr);
  } else {
    hipLaunchKernelGGL((hidden_kernel<1, TAB, false>), dim3(L / 32, 2 * nfilters), dim3(256), 0, s, tab, L, emb_dim, w_mod, wsplit,
                       h_hi, h_lo, 0, 0.f, nullptr, nullptr);
  }
  rc = check_launch("hyena hidden_kernel");
  if (rc || !taps) return rc;
  hipLaunchKernelGGL(project_kernel<TAB>, dim3((L + kPosPerWg - 1) / kPosPerWg, (d + 127) / 128, 2 * nfilters), dim3(256), 0, s, tab, L, d, shift,
                     h_hi, h_lo, w3split, taps);
  return check_launch("hyena project_kernel");
}

static int check_filter_sizes(const char* who, int L, int d, int order, int emb_dim) {
  if (order != kOrder) return set_error(M2_ERR_UNSUPPORTED, "%s: order=%d, only 128 is built", who, order);
  if (emb_dim < 3 || emb_dim > kMaxEmb)
    return set_error(M2_ERR_UNSUPPORTED, "%s: emb_dim=%d not in [3, %d]", who, emb_dim, kMaxEmb);
  if (L <= 0 || L % kPosTile != 0)
    return set_error(M2_ERR_UNSUPPORTED, "%s: L=%d must be a positive multiple of %d", who, L, kPosTile);
  if (d <= 0 || d % 64 != 0) return set_error(M2_ERR_UNSUPPORTED, "%s: d=%d must be a positive multiple of 64", who, d);
  return M2_OK;
}

// Shared by the two entry points that take a host array of filters: validation and the launches, `workspace`
// holding the h3 hi / lo parts and the re-split weights.
static int hyena_filter_launch(const char* who, const m2_hyena_filter_params* params, int nfilters, int L, int d,
                               int order, int emb_dim, float w_mod, float shift, void* workspace, float* taps,
                               void* stream) {
  if (nfilters < 1 || nfilters > kMaxFilters)
    return set_error(M2_ERR_UNSUPPORTED, "%s: nfilters=%d not in [1, %d]", who, nfilters, kMaxFilters);
  int rc = check_filter_sizes(who, L, d, order, emb_dim);
  if (rc) return rc;
  TabByValue tab;
  FilterBatch& fb = tab.fb;
  for (int f = 0; f < kMaxFilters; ++f) {
    const m2_hyena_filter_params& p = params[f < nfilters ? f : 0];
    if (!p.z || !p.t || !p.freq || !p.deltas || !p.w0 || !p.b0 || !p.w1 || !p.b1 || !p.w2 || !p.b2 || !p.w3)
      return set_error(M2_ERR_ARG, "%s: filter %d has a null forward-MLP pointer", who, f);
    const bool rev = p.rw0 != nullptr;
    if (rev && (!p.rb0 || !p.rw1 || !p.rb1 || !p.rw2 || !p.rb2 || !p.rw3))
      return set_error(M2_ERR_ARG, "%s: filter %d has a partly null reverse MLP", who, f);
    fb.f[f].z = p.z; fb.f[f].t = p.t; fb.f[f].freq = p.freq; fb.f[f].deltas = p.deltas;
    fb.f[f].mlp[0] = MlpPtrs{p.w0, p.b0, p.w1, p.b1, p.w2, p.b2, p.w3};
    fb.f[f].mlp[1] = rev ? MlpPtrs{p.rw0, p.rb0, p.rw1, p.rb1, p.rw2, p.rb2, p.rw3}
                         : MlpPtrs{nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
  }
  uint16_t* h_hi = reinterpret_cast<uint16_t*>(workspace);
  uint16_t* h_lo = h_hi + (size_t)2 * nfilters * L * order;
  uint16_t* wsplit = h_lo + (size_t)2 * nfilters * L * order;
  uint16_t* w3split = wsplit + (size_t)2 * nfilters * 2 * 3 * order * order;
  return filter_launches(tab, nfilters, L, d, emb_dim, w_mod, shift, h_hi, h_lo, wsplit, w3split, taps, (hipStream_t)stream);
}

extern "C" int m2_hyena_filter_fwd(const m2_hyena_filter_params* params, int nfilters, int L, int d, int order,
                                   int emb_dim, float w_mod, float shift, float* workspace, float* taps,
                                   void* stream) {
  if (!params || !workspace || !taps) return set_error(M2_ERR_ARG, "m2_hyena_filter_fwd: null pointer");
  return hyena_filter_launch("m2_hyena_filter_fwd", params, nfilters, L, d, order, emb_dim, w_mod, shift, workspace,
                             taps, stream);
}

// ---------------------------------------------------------------------------------------------
// The same computation for callers that cannot allocate a workspace: the h3 hi / lo parts go through a
// device array that is part of the library's code object.  Every GPU the library runs on holds its own copy
// of the array at its own address until the process ends; in host code the array's NAME is only a stand-in
// for the symbol, so its device address is looked up once per device (hipGetSymbolAddress) and only that
// address is ever handed to a kernel.
// ---------------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[M2_HYENA_FILTER_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {nullptr};      // device address of `scratch` on device i, once looked up

// Device address of the static scratch array on the current device (looked up on the first call per device).
int static_scratch_for_current_device(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return set_error(M2_ERR_LAUNCH, "m2_hyena_filter_fwd_static: hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices)
    return set_error(M2_ERR_UNSUPPORTED, "m2_hyena_filter_fwd_static: device index %d beyond %d", dev, kMaxDevices - 1);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr)
      return set_error(M2_ERR_LAUNCH, "m2_hyena_filter_fwd_static: hipGetSymbolAddress(scratch) on device %d: %s", dev,
                       hipGetErrorString(e));
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return M2_OK;
}
}  // namespace

extern "C" int m2_hyena_filter_fwd_static(const m2_hyena_filter_params* params, int nfilters, int L, int d, int order,
                                          int emb_dim, float w_mod, float shift, float* taps, void* stream) {
  if (!params || !taps) return set_error(M2_ERR_ARG, "m2_hyena_filter_fwd_static: null pointer");
  if (nfilters < 1 || L <= 0 || order <= 0)
    return set_error(M2_ERR_ARG, "m2_hyena_filter_fwd_static: sizes must be positive (nfilters=%d L=%d order=%d)", nfilters, L, order);
  const size_t need = m2_hyena_filter_workspace_bytes(nfilters, L, d, order);
  if (need > (size_t)M2_HYENA_FILTER_STATIC_SCRATCH_BYTES)
    return set_error(M2_ERR_UNSUPPORTED,
                     "m2_hyena_filter_fwd_static: nfilters=%d, L=%d needs %zu bytes of scratch, the static array holds %zu "
                     "(m2_hyena_filter_workspace_bytes); use m2_hyena_filter_fwd with a caller workspace",
                     nfilters, L, need, (size_t)M2_HYENA_FILTER_STATIC_SCRATCH_BYTES);
  void* ptr = nullptr;
  int rc = static_scratch_for_current_device(&ptr);
  if (rc) return rc;
  // split_weights_kernel and hidden_kernel write every element the later kernels of the same call read, so nothing
  // left by an earlier (possibly longer) call is ever read and nothing needs clearing
  return hyena_filter_launch("m2_hyena_filter_fwd_static", params, nfilters, L, d, order, emb_dim, w_mod, shift, ptr,
                             taps, stream);
}

// ---------------------------------------------------------------------------------------------
// All filters of a batch of mixers -> their spectra, the pointer table in device memory.
// ---------------------------------------------------------------------------------------------
namespace {
struct BatchLayout {
  size_t h_lo, wsplit, w3split, taps, total;      // byte offsets into the workspace (h_hi at 0)
  bool fused;                                     // projection + spectrum as one kernel, taps never in memory
};
BatchLayout batch_layout(int nmixers, int fpm, int L, int d) {
  const size_t nf = (size_t)nmixers * fpm;
  auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
  BatchLayout b;
  b.fused = project_spectrum_supported(L);
  b.h_lo = up(2 * nf * L * kOrder * sizeof(uint16_t));
  b.wsplit = b.h_lo + up(2 * nf * L * kOrder * sizeof(uint16_t));
  b.w3split = b.wsplit + up(2 * nf * 2 * 3 * kOrder * kOrder * sizeof(uint16_t));
  b.taps = b.w3split + (b.fused ? 0 : up(2 * nf * 2 * (size_t)d * kOrder * sizeof(uint16_t)));
  b.total = b.taps + (b.fused ? 0 : up(nf * (size_t)d * 2 * L * sizeof(float)));
  return b;
}
}  // namespace

extern "C" size_t m2_mixer_filters_workspace_bytes(int nmixers, int filters_per_mixer, int L, int d, int order) {
  if (nmixers <= 0 || filters_per_mixer < 1 || filters_per_mixer > 2 || L <= 0 || d <= 0 || order != kOrder) return 0;
  return batch_layout(nmixers, filters_per_mixer, L, d).total;
}

extern "C" int m2_mixer_filters_fwd(const m2_hyena_filter_params* params_dev, const float* const* skip_dev, int nmixers,
                                    int filters_per_mixer, int L, int d, int order, int emb_dim, float w_mod,
                                    float shift, void* workspace, float* spec, void* stream) {
  const char* who = "m2_mixer_filters_fwd";
  if (!params_dev || !workspace || !spec) return set_error(M2_ERR_ARG, "%s: null pointer", who);
  if (filters_per_mixer < 1 || filters_per_mixer > 2)
    return set_error(M2_ERR_ARG, "%s: filters_per_mixer=%d must be 1 or 2", who, filters_per_mixer);
  // the MLPs of the batch (two per filter) are one grid dimension of the hidden-layer launch
  if (nmixers < 1 || (long)nmixers * filters_per_mixer * 2 > 65535)
    return set_error(M2_ERR_ARG, "%s: nmixers=%d with %d filters each: at most 65535 MLPs (two per filter) per call", who, nmixers,
                     filters_per_mixer);
  int rc = check_filter_sizes(who, L, d, order, emb_dim);
  if (rc) return rc;
  if (!m2_fftconv_supported_seqlen(L))
    return set_error(M2_ERR_UNSUPPORTED, "%s: L=%d unsupported (need L a power of two in [128, 32768])", who, L);
  const int nf = nmixers * filters_per_mixer;
  const BatchLayout lay = batch_layout(nmixers, filters_per_mixer, L, d);
  unsigned char* ws = reinterpret_cast<unsigned char*>(workspace);
  uint16_t* h_hi = reinterpret_cast<uint16_t*>(ws);
  uint16_t* h_lo = reinterpret_cast<uint16_t*>(ws + lay.h_lo);
  uint16_t* wsplit = reinterpret_cast<uint16_t*>(ws + lay.wsplit);
  uint16_t* w3split = lay.fused ? nullptr : reinterpret_cast<uint16_t*>(ws + lay.w3split);
  float* taps = lay.fused ? nullptr : reinterpret_cast<float*>(ws + lay.taps);
  TabByPointer tab{reinterpret_cast<const FilterPtrs*>(params_dev)};
  hipStream_t s = (hipStream_t)stream;
  rc = filter_launches(tab, nf, L, d, emb_dim, w_mod, shift, h_hi, h_lo, wsplit, w3split, taps, s);
  if (rc) return rc;
  const long spec_stride = (long)(m2_filter_spectrum_bytes(d, L) / sizeof(float));
  if (lay.fused)
    return launch_project_spectrum(tab.p, skip_dev, nmixers, filters_per_mixer, L, d, shift, h_hi, h_lo, spec, spec_stride, s);
  SpectrumBatch sb{taps, skip_dev, filters_per_mixer, spec_stride};
  return launch_filter_spectrum_any(nullptr, nullptr, nullptr, nullptr, spec, d, L, sb, nmixers, s);
}
