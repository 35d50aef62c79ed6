// The gated block-diagonal GEMM with the GELU GLU on its accumulators for 384-wide blocks (d = 1536, nblocks = 4), and,
// with eight K steps instead of twelve and zeros beyond the block's width, for blocks of 224 .. 248 (d = 960: 240):
//
//   h = blockdiag(x, Wg)                      (M, 2I)   never materialised
//   g = gelu_erf(h[:, :I]) * h[:, I:]         (M, I)    bf16, the input of `wo`
//
// (bert/src/bert_layers.py:494-502, bert/src/mm/blockdiag_multiply.py:49-60.)  The first half of the whole-MLP
// kernel of mlp_fused_kernels.hip at twice the block width: gated columns [r I/4, (r + 1) I/4) take their gate values
// from block r / 2 of x and their paired values from block r / 2 + 2.  A workgroup of eight waves (two per SIMD) owns
// 128 rows and one r, a wave 16 rows, whose two 384-wide x blocks stay in 96 registers as MFMA B operands; the
// weights are the A operands and stream through LDS in chunks of 32 gated columns (gate rows and value rows, 48 KB),
// three stages, written by direct global -> LDS loads two chunks ahead.  Product and GLU are transposed (gated
// columns x rows of x), and the rows of a chunk are permuted so that a lane's eight accumulator elements are eight
// consecutive gated columns of its row: they leave as one 16-byte store per chunk.
//
// At this block width the second product of the MLP cannot join the first in one kernel (its 384 output columns per
// row would take another 96 accumulator registers), so `wo` stays a kernel of its own.  What this kernel replaces is
// the LDS-tiled GEMM with a GLU epilogue (blockdiag_kernels.hip), which re-reads x through LDS for every 128
// columns; here x is read once per 1536 gated columns and never passes through LDS.
//
// The weights are re-packed once (m2_glu_stream_pack) into the image of the LDS stages, 48 operand blocks of 1 KB per
// (r, chunk), so that every load instruction copies one contiguous block (the L2 delivers 62 GB/s per compute unit
// that way and 38 GB/s when a load gathers sixteen 64-byte row pieces).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fft_regs.h"
#include "m2_internal.h"
#include "mfma_stream.h"

namespace m2 {

constexpr int kSRows = 128;                 // rows per workgroup: 8 waves x 16
constexpr int kSChunk = 32;                 // gated columns per chunk
constexpr int kSBlk = 1024;                 // one operand block: 64 lanes x 16 bytes = 16 rows x 32 K
// KS = K steps (K = 32 per MFMA) of a block: 12 for 384-wide blocks, 14 for 448-wide ones, 8 for blocks of up to 256
// (the weights and the x rows are zero beyond the block's real width p).  Three LDS stages (loads two chunks ahead)
// where they fit, two (one chunk ahead) for the 56 KB chunks of 448-wide blocks.
template <int KS>
struct GluShape {
  static constexpr int kStage = 2 * 2 * KS * kSBlk;      // (gate | value) x 2 row tiles x KS K steps: 32 / 48 / 56 KB
  static constexpr int kStages = 3 * kStage <= 160 * 1024 ? 3 : 2;
  static constexpr int kLds = kStages * kStage;          // 96 / 144 / 112 KB
  static constexpr int kBatch = 4 * KS / 8;              // direct loads a wave issues per chunk: blocks / 8 waves
};
static int glu_stream_ksteps(int p) { return p == 384 ? 12 : p == 448 ? 14 : (p >= 224 && p <= 248 && p % 8 == 0) ? 8 : 0; }

// Re-packs gated_layers.weight (4, I / 2, 384) into the image of the LDS stages: for r = 0 .. 3 and chunk c (32 gated
// columns) 48 blocks of 64 lanes x 16 bytes; block ((value, t), s) = index (2 value + t) 12 + s; lane (i, q) holds row
// gamma(16 t + i) = 8 (i / 4) + 4 t + i % 4 of the chunk, K = 32 s + 8 q .. + 7.  One thread per 16-byte piece.
template <int KS>
__global__ __launch_bounds__(256) void glu_stream_pack_kernel(const uint16_t* __restrict__ wg, u32x4* __restrict__ packed, int I, int p) {
  constexpr int NB = 4 * KS;                 // operand blocks per chunk
  const int IS = I >> 2, q = I >> 1, nchunks = IS / kSChunk;
  const long piece = (long)blockIdx.x * 256 + threadIdx.x;
  const long npieces = 4l * nchunks * (GluShape<KS>::kStage / 16);
  if (piece >= npieces) return;
  const int lane = piece & 63, i16 = lane & 15, q4 = lane >> 4;
  const int blk = (piece >> 6) % NB;
  const int c = (piece / (64 * NB)) % nchunks;
  const int r = piece / (64l * NB * nchunks);
  const int s = blk % KS, t = (blk / KS) & 1, val = blk / (2 * KS);
  const int gamma = 8 * (i16 >> 2) + 4 * t + (i16 & 3);
  const int k0 = 32 * s + 8 * q4;
  u32x4 v = {0u, 0u, 0u, 0u};
  if (k0 < p)
    v = *reinterpret_cast<const u32x4*>(wg + (((long)((r >> 1) + 2 * val) * q + (long)(r & 1) * IS + c * kSChunk + gamma) * p + k0));
  packed[piece] = v;
}

template <int KS>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void glu_stream_kernel(
    const uint16_t* __restrict__ x,             // (M, 4 p) bf16
    const unsigned char* __restrict__ wpk,      // the gated weight as packed by glu_stream_pack_kernel
    uint16_t* __restrict__ out,                 // (M, I) bf16
    int M, int I, int ntiles, int p) {
  constexpr int kSKS = KS, kSStage = GluShape<KS>::kStage, kSBatch = GluShape<KS>::kBatch, kSStages = GluShape<KS>::kStages;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, i16 = lane & 15, q4 = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // Workgroup ids are dealt round-robin to the 8 XCDs (one L2 each): XCD e works on r = 2 (e % 2), 2 (e % 2) + 1, which
  // read the same two blocks of x, and on the row tiles = e / 2 (mod 4); neighbouring workgroups of an XCD take the
  // same row tile with the two r, so the second read of its x rows is an L2 hit and an L2 holds half of the weights.
  const int xcd = blockIdx.x & 7, slot = (int)(blockIdx.x >> 3);
  const int r = 2 * (xcd & 1) + (slot & 1);
  const int tile_step = 2 * (int)(gridDim.x >> 3);
  int tile = 4 * (slot >> 1) + (xcd >> 1);
  if (tile >= ntiles) return;
  const int IS = I >> 2;                  // gated columns of this r
  const int nchunks = IS / kSChunk;
  const int gb = r >> 1;                  // gate block; the value block is gb + 2
  const int d = 4 * p;

  // ---- the wave's x rows as stationary B operands: lane (n, q) holds x[row n][32 s + 8 q .. + 8) of both blocks
  bf16x8 xa[kSKS], xb[kSKS];
  auto load_x = [&](int t) __attribute__((always_inline)) {
    int row = t * kSRows + 16 * wave + i16;
    row = row < M ? row : M - 1;
    const uint16_t* pa = x + (long)row * d + gb * p + 8 * q4;
    const uint16_t* pb = pa + 2 * p;
    static_for<0, kSKS>([&](auto ss) {
      constexpr int s = decltype(ss)::value;
      if (KS != 8 || 32 * s + 8 * q4 < p) {      // narrower blocks: zeros beyond the block's width (the weights are zero there too)
        xa[s] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(pa + 32 * s));
        xb[s] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(pb + 32 * s));
      } else {
        const u32x4 z = {0u, 0u, 0u, 0u};
        xa[s] = __builtin_bit_cast(bf16x8, z);
        xb[s] = __builtin_bit_cast(bf16x8, z);
      }
    });
  };
  load_x(tile);

  // ---- staging: iteration n (counted through all tiles of the workgroup) reads stage n % 3; its loads go two
  // iterations ahead, into the stage last read in iteration n - 1.  The weights of a workgroup's r just keep cycling:
  // chunk it + 2 of a tile, or the first chunks of the next tile (same r, same weights) at a tile's end.
  const unsigned lds0 = (unsigned)(uintptr_t)smem;
  const unsigned voff = 16 * lane;
  const unsigned char* wr = wpk + (long)r * nchunks * kSStage;
  auto dma_one = [&](int stage, int chunk, auto jj) __attribute__((always_inline)) {
    constexpr int j = decltype(jj)::value;
    load_to_lds(lds0 + stage * kSStage + (wave + 8 * j) * kSBlk, voff, wr + (long)chunk * kSStage + (wave + 8 * j) * kSBlk);
  };

  floatx4 g[2], v[2];
  float gp[8], vp[8];      // the previous chunk's gate / value accumulators, in gated-column order 4 t + j
  constexpr int kNM = 4 * kSKS;      // 48 MFMAs per chunk: K step k / 4, (gate t = 0, value t = 0, gate t = 1, value t = 1) = k % 4
  constexpr int kPF = 12;            // operand reads run 12 MFMAs ahead, inside an iteration only
  auto operand_off = [&](auto kk) constexpr -> int {
    constexpr int k = decltype(kk)::value;
    constexpr int s = k / 4, sel = k % 4, t = sel >> 1, val = sel & 1;
    return ((2 * val + t) * kSKS + s) * kSBlk;
  };
  u32x4 ring[kPF];

  // prologue: the chunks of iterations 0 and (three stages) 1
  static_for<0, kSBatch>([&](auto jj) { dma_one(0, 0, jj); });
  if constexpr (kSStages == 3) static_for<0, kSBatch>([&](auto jj) { dma_one(1, nchunks > 1 ? 1 : 0, jj); });
  __builtin_amdgcn_s_waitcnt(kWaitVm0);
  __syncthreads();

  int st = 0;              // stage of the current iteration
  for (;;) {
    // The x loads complete here, once per tile (consumed before the loop, so that no "load pending" mark on the x
    // registers survives around the loop's back edge: that would put a full vector-memory wait into every iteration).
#pragma unroll
    for (int s = 0; s < kSKS; ++s) asm volatile("" : "+v"(xa[s]), "+v"(xb[s]));
    const int row = tile * kSRows + 16 * wave + i16;
    const int rowc = row < M ? row : M - 1;
    uint16_t* orow = out + (long)rowc * I + r * IS + 8 * q4;

    // gelu(gate) * value of the chunk whose accumulators sit in gp / vp: eight chains side by side, one 16-byte store
    auto finish_chunk = [&](int chunk) __attribute__((always_inline)) {
      float gl[8];
      GeluChain ch[8];
      static_for<0, 11>([&](auto stp) {
        static_for<0, 8>([&](auto ee) {
          constexpr int e = decltype(ee)::value;
          gelu_step<decltype(stp)::value>(ch[e], gp[e], vp[e], gl[e]);
        });
      });
      u32x4 pk;
      pk.x = pack_bf16x2(gl[0], gl[1]);
      pk.y = pack_bf16x2(gl[2], gl[3]);
      pk.z = pack_bf16x2(gl[4], gl[5]);
      pk.w = pack_bf16x2(gl[6], gl[7]);
      if (row < M) *reinterpret_cast<u32x4*>(orow + kSChunk * chunk) = pk;
    };

    auto iteration = [&](auto head_, int it) __attribute__((always_inline)) {
      constexpr bool HEAD = decltype(head_)::value;
      unsigned ob = 16 * lane + st * kSStage;
      asm volatile("" : "+v"(ob));
      static_for<0, kPF>([&](auto kk) {
        ring[decltype(kk)::value] = *reinterpret_cast<const u32x4*>(smem + ob + operand_off(kk));
      });
      // the previous chunk leaves while the first operands of this one travel
      if constexpr (!HEAD) finish_chunk(it - 1);
      const int st2 = st == 0 ? kSStages - 1 : st - 1;            // (st + stages - 1) % stages: the stage read in the iteration before
      const int c2 = (it + kSStages - 1) % nchunks;               // of this tile or, at its end, of the next one
      constexpr int kDmaEvery = kSStages == 3 ? 8 : 4;            // one chunk ahead only: the loads go out early in the iteration
      static_for<0, kNM>([&](auto kk) {
        constexpr int k = decltype(kk)::value;
        constexpr int s = k / 4, sel = k % 4, t = sel >> 1, val = sel & 1;
        const bf16x8 a = __builtin_bit_cast(bf16x8, ring[k % kPF]);
        floatx4& acc = val ? v[t] : g[t];
        if constexpr (s == 0) {
          const floatx4 z = {0.f, 0.f, 0.f, 0.f};
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, val ? xb[0] : xa[0], z, 0, 0, 0);
        } else {
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, val ? xb[s] : xa[s], acc, 0, 0, 0);
        }
        if constexpr (k + kPF < kNM) ring[k % kPF] = *reinterpret_cast<const u32x4*>(smem + ob + operand_off(ic<k + kPF>{}));
        // the direct loads for iteration n + 2, one every eighth MFMA
        if constexpr (k % kDmaEvery == 1 && k / kDmaEvery < kSBatch) dma_one(st2, c2, ic<k / kDmaEvery>{});
        __builtin_amdgcn_sched_barrier(0);
      });
      static_for<0, 8>([&](auto ee) {
        constexpr int e = decltype(ee)::value;
        gp[e] = g[e >> 2][e & 3];
        vp[e] = v[e >> 2][e & 3];
      });
      // everything but this wave's newest batch has landed: after the barrier the next chunk is complete for everybody
      if constexpr (kSStages == 3) __builtin_amdgcn_s_waitcnt(0x0F70 | kSBatch);
      else __builtin_amdgcn_s_waitcnt(kWaitVm0);                  // two stages: the batch just issued is the next chunk
      __syncthreads();
      __builtin_amdgcn_sched_barrier(0);
      st = st == kSStages - 1 ? 0 : st + 1;
    };
    iteration(ic<1>{}, 0);
    for (int it = 1; it < nchunks; ++it) iteration(ic<0>{}, it);

    // ---- end of the tile: the next tile's x rows are requested into the registers that have just become free, then
    // the last chunk leaves
    tile += tile_step;
    const bool more = tile < ntiles;
    if (more) load_x(tile);
    finish_chunk(nchunks - 1);
    if (!more) break;
  }
  // no load may still be in flight when the workgroup ends (its LDS goes to the next one)
  __builtin_amdgcn_s_waitcnt(kWaitVm0);
}

}  // namespace m2

using namespace m2;

extern "C" int m2_glu_stream_supported(int in_features, int intermediate, int nblocks) {
  return nblocks == 4 && in_features > 0 && in_features % 4 == 0 && glu_stream_ksteps(in_features / 4) != 0 && intermediate > 0 &&
         intermediate % (4 * kSChunk) == 0;
}

extern "C" long m2_glu_stream_packed_bytes(int in_features, int intermediate, int nblocks) {
  if (!m2_glu_stream_supported(in_features, intermediate, nblocks)) return 0;
  const int ks = glu_stream_ksteps(in_features / 4);
  return 4l * (intermediate / 4 / kSChunk) * (ks == 12 ? GluShape<12>::kStage : ks == 14 ? GluShape<14>::kStage : GluShape<8>::kStage);
}

static const char* kGluStreamShapes =
    "built for nblocks=4, in_features/4 = 384, 448 or a multiple of 8 in [224, 248], intermediate a multiple of 128";

extern "C" int m2_glu_stream_pack(const void* w_gated, void* packed, int in_features, int intermediate, int nblocks,
                                  void* stream) {
  if (!w_gated || !packed) return set_error(M2_ERR_ARG, "m2_glu_stream_pack: null pointer");
  if (!m2_glu_stream_supported(in_features, intermediate, nblocks))
    return set_error(M2_ERR_UNSUPPORTED, "m2_glu_stream_pack: %s (got nblocks=%d in=%d intermediate=%d)", kGluStreamShapes,
                     nblocks, in_features, intermediate);
  const long npieces = m2_glu_stream_packed_bytes(in_features, intermediate, nblocks) / 16;
  const int p = in_features / 4;
  const dim3 grid((unsigned)((npieces + 255) / 256));
  if (glu_stream_ksteps(p) == 12)
    hipLaunchKernelGGL(glu_stream_pack_kernel<12>, grid, dim3(256), 0, (hipStream_t)stream, (const uint16_t*)w_gated,
                       (u32x4*)packed, intermediate, p);
  else if (glu_stream_ksteps(p) == 14)
    hipLaunchKernelGGL(glu_stream_pack_kernel<14>, grid, dim3(256), 0, (hipStream_t)stream, (const uint16_t*)w_gated,
                       (u32x4*)packed, intermediate, p);
  else
    hipLaunchKernelGGL(glu_stream_pack_kernel<8>, grid, dim3(256), 0, (hipStream_t)stream, (const uint16_t*)w_gated,
                       (u32x4*)packed, intermediate, p);
  return check_launch("glu_stream_pack");
}

template <int KS>
static int launch_glu_stream(const void* x, const void* w_packed, void* out, int M, int intermediate, int p, int per_xcd,
                             int ntiles, hipStream_t stream) {
  auto kern = glu_stream_kernel<KS>;
  hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, GluShape<KS>::kLds);
  if (e != hipSuccess) return set_error(M2_ERR_LAUNCH, "hipFuncSetAttribute(glu_stream): %s", hipGetErrorString(e));
  hipLaunchKernelGGL(kern, dim3(8 * per_xcd), dim3(512), GluShape<KS>::kLds, stream, (const uint16_t*)x,
                     (const unsigned char*)w_packed, (uint16_t*)out, M, intermediate, ntiles, p);
  return check_launch("glu_stream");
}

extern "C" int m2_glu_stream_fwd(const void* x, const void* w_packed, void* out, int M, int in_features, int intermediate,
                                 int nblocks, void* stream) {
  if (!x || !w_packed || !out) return set_error(M2_ERR_ARG, "m2_glu_stream_fwd: null pointer");
  if (M <= 0) return set_error(M2_ERR_ARG, "m2_glu_stream_fwd: M=%d must be positive", M);
  if (!m2_glu_stream_supported(in_features, intermediate, nblocks))
    return set_error(M2_ERR_UNSUPPORTED, "m2_glu_stream_fwd: %s (got nblocks=%d in=%d intermediate=%d); use m2_blockdiag_glu_fwd",
                     kGluStreamShapes, nblocks, in_features, intermediate);
  const int ntiles = (M + kSRows - 1) / kSRows;
  // one persistent workgroup per compute unit (its LDS stages take most of it), an even number per XCD
  int per_xcd = (num_cus() / 8) & ~1;
  if (per_xcd < 2) per_xcd = 2;      // a device (or partition) with fewer than 16 compute units: work is dealt to 8 x per_xcd slots whatever the real count
  if (per_xcd > 2 * ((ntiles + 3) / 4)) per_xcd = 2 * ((ntiles + 3) / 4);
  const int p = in_features / 4;
  switch (glu_stream_ksteps(p)) {
    case 12: return launch_glu_stream<12>(x, w_packed, out, M, intermediate, p, per_xcd, ntiles, (hipStream_t)stream);
    case 14: return launch_glu_stream<14>(x, w_packed, out, M, intermediate, p, per_xcd, ntiles, (hipStream_t)stream);
    default: return launch_glu_stream<8>(x, w_packed, out, M, intermediate, p, per_xcd, ntiles, (hipStream_t)stream);
  }
}
