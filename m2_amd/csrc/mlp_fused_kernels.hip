// The whole Monarch GLU MLP of an M2-BERT layer as ONE kernel for d = 768 (nblocks = 4, 192-wide blocks):
//
//   h   = blockdiag(x, Wg)                      (M, 2I)   never materialised
//   g   = gelu_erf(h[:, :I]) * h[:, I:]         (M, I)    never materialised
//   out = blockdiag(g, Wo) + bias + residual    (M, d)
//
// (bert/src/bert_layers.py:482-506, bert/src/mm/blockdiag_multiply.py:49-60.)  Block structure: output block r
// of `wo` consumes the intermediate columns [r I/4, (r + 1) I/4), whose gate values come from block r / 2 of x
// and whose paired values come from block r / 2 + 2, so the MLP falls apart into four independent chains
// x[:, two blocks] -> I/4 gated columns -> 192 output columns, one per r.
//
// A workgroup of four waves owns 128 rows and one r.  Everything is computed TRANSPOSED, weights as the MFMA
// A operand (rows of the product) and the x rows as the B operand (its columns):
//
//   G^T (32 gated columns x 32 x-rows)   = Wg_chunk (32 x 192) X_a^T  and  Wv_chunk X_b^T       24 MFMAs
//   OUT^T (192 x 32 x-rows)             += Wo_chunk (192 x 32) GLU(G^T)                          12 MFMAs
//
// because then the accumulator of the first product IS the B operand of the second: lane (i, h) of
// v_mfma_f32_32x32x16_bf16 receives accumulator rows 8 (v / 4) + 4 h + v % 4 of column i, and a B operand wants
// eight consecutive K values of column i per lane.  Which gated column sits in which accumulator row is free, so
// operand row rho of a chunk is given gated column gamma(rho) = rho with bits 2 and 3 swapped: then the
// accumulator elements 8 s .. 8 s + 7 of lane (i, h) are the gated columns 16 s + 8 h .. + 7, exactly the K range
// of one 16-byte piece of a `wo` row, and the gated values go from the accumulators through gelu(gate) * value
// and the bf16 conversion straight into the next MFMA: the (M, I) intermediate never leaves the registers.
// The x rows of a wave (32 rows x two 192-wide blocks = 96 registers) are loaded once, straight from global
// memory in operand layout, and stay put.  The weights stream through LDS, 36 KB per chunk of 32 gated columns,
// in three stages, written by direct global -> LDS loads (global_load_lds_dwordx4: no registers, no LDS write
// instructions) issued two chunks ahead; every operand is one conflict-free 16-byte LDS read (a stage is laid out
// [K step][lane]).  One barrier per chunk.  One workgroup per compute unit, one wave per SIMD.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "fft_regs.h"
#include "m2_internal.h"

namespace m2 {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// x * Phi(x): the same clamped odd polynomial as the separate GLU kernel (blockdiag_kernels.hip), so both paths
// round alike.
__device__ __forceinline__ float gelu_erf_poly(float x) {
  const float xc = __builtin_amdgcn_fmed3f(x, -3.9f, 3.9f);
  const float x2 = xc * xc;
  float p = 2.7693410957e-08f;
  p = fmaf(p, x2, -1.8473178272e-06f);
  p = fmaf(p, x2, 5.2869800351e-05f);
  p = fmaf(p, x2, -8.6171873090e-04f);
  p = fmaf(p, x2, 9.0065851481e-03f);
  p = fmaf(p, x2, -6.5103946404e-02f);
  p = fmaf(p, x2, 3.9828952833e-01f);
  return x * fmaf(p, xc, 0.5f);
}

constexpr int kFP = 192;                    // block width of x and of the output (d / 4)
constexpr int kFKS = kFP / 16;              // K steps of the first products: 12
constexpr int kFRows = 128;                 // rows per workgroup
constexpr int kFChunk = 32;                 // gated columns per chunk
constexpr int kFBlk = 1024;                 // one operand block: 64 lanes x 16 bytes
constexpr int kFGV = 2 * kFKS * kFBlk;      // Wg + Wv blocks of a chunk: 24 KB
constexpr int kFWO = 12 * kFBlk;            // Wo blocks of a chunk (6 tiles x 2 K steps): 12 KB
constexpr int kFStages = 3;
constexpr int kFLds = kFStages * (kFGV + kFWO);      // 108 KB

// s_waitcnt immediates (vmcnt in bits 3:0 and 15:14, expcnt 6:4, lgkmcnt 11:8): wait for the vector-memory
// counter only
constexpr int kWaitVm0 = 0x0F70, kWaitVm9 = 0x0F79;

// One direct global -> LDS load: every lane fetches 16 bytes from base + voff, lane l's piece lands at LDS byte
// address lds + 16 l.  Inline assembly on purpose: the compiler then neither tracks the LDS write (it would put a
// full vector-memory wait in front of every later LDS read) nor reorders it across other memory accesses; the
// kernel waits for these loads itself.
__device__ __forceinline__ void load_to_lds(unsigned lds, unsigned voff, const void* base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds), "v"(voff), "s"(base) : "memory");
}

template <typename OUT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void mlp_fused_kernel(
    const uint16_t* __restrict__ x,       // (M, 768) bf16
    const uint16_t* __restrict__ wg,      // (4, I / 2, 192) bf16   gated_layers.weight
    const uint16_t* __restrict__ wo,      // (4, 192, I / 4) bf16   wo.weight
    const float* __restrict__ bias,       // (768) or null
    const uint16_t* __restrict__ resid,   // (M, 768) bf16 or null
    OUT* __restrict__ out,                // (M, 768)
    int M, int I) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, i32 = lane & 31, half = lane >> 5;
  // Workgroup ids are dealt round-robin to the 8 XCDs (one L2 each): XCD e works on output block r = e % 4 only,
  // so its L2 holds one quarter of the weights.
  const int xcd = blockIdx.x & 7;
  const int r = xcd & 3;
  const int tile = (blockIdx.x >> 3) * 2 + (xcd >> 2);
  const int m0 = tile * kFRows;
  if (m0 >= M) return;
  const int IS = I >> 2;                  // gated columns of this r
  const int q = I >> 1;                   // rows of a gated_layers block
  const int nchunks = IS / kFChunk;
  const int gb = r >> 1;                  // gate block; the value block is gb + 2
  const int d = 4 * kFP;

  // ---- the wave's x rows as stationary B operands: lane (i, h) holds x[row i][16 s + 8 h .. + 8) of both blocks
  bf16x8 xa[kFKS], xb[kFKS];
  {
    int row = m0 + 32 * wave + i32;
    row = row < M ? row : M - 1;
    const uint16_t* pa = x + (long)row * d + gb * kFP + 8 * half;
    const uint16_t* pb = pa + 2 * kFP;
    static_for<0, kFKS>([&](auto ss) {
      constexpr int s = decltype(ss)::value;
      xa[s] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(pa + 16 * s));
      xb[s] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(pb + 16 * s));
    });
  }

  // ---- staging.  A chunk is 36 operand blocks of 1 KB: Wg K steps 0 .. 11, Wv K steps 0 .. 11, Wo (tile t, K step
  // s2) 0 .. 11; wave w loads the blocks b = w + 4 j.  Lane (i, h) of a block fetches what lane (i, h) of the MFMA
  // needs: Wg / Wv row gamma(i) of the chunk, K = 16 s + 8 h .. + 7; Wo row 32 t + i, K = 16 s2 + 8 h .. + 7.
  const unsigned lds0 = (unsigned)(uintptr_t)smem;
  const int gamma = (i32 & 0x13) | ((i32 & 4) << 1) | ((i32 & 8) >> 1);
  unsigned voff_gv[6], voff_o[3];
  static_for<0, 6>([&](auto jj) {
    constexpr int j = decltype(jj)::value;
    const int b = wave + 4 * j, s = b % kFKS, val = b / kFKS;
    voff_gv[j] = (unsigned)((((long)(gb + 2 * val) * q + (long)(r & 1) * IS + gamma) * kFP + 16 * s + 8 * half) * 2);
  });
  static_for<0, 3>([&](auto jj) {
    constexpr int j = decltype(jj)::value;
    const int b = wave + 4 * j, t = b >> 1, s2 = b & 1;
    voff_o[j] = (unsigned)((((long)r * kFP + 32 * t + i32) * IS + 16 * s2 + 8 * half) * 2);
  });
  auto stage_gv = [&](int c) { return lds0 + (c % kFStages) * kFGV; };
  auto stage_wo = [&](int c) { return lds0 + kFStages * kFGV + (c % kFStages) * kFWO; };
  // Wg / Wv of chunk c -> its stage (indices past the end are clamped: nobody reads what that fetches)
  auto dma_gv = [&](int c) __attribute__((always_inline)) {
    const unsigned st = __builtin_amdgcn_readfirstlane(stage_gv(c) + wave * kFBlk);
    const int cc = c < nchunks ? c : nchunks - 1;
    const uint16_t* base = wg + (long)cc * kFChunk * kFP;
    static_for<0, 6>([&](auto jj) { load_to_lds(st + 4 * kFBlk * decltype(jj)::value, voff_gv[decltype(jj)::value], base); });
  };
  auto dma_wo = [&](int c) __attribute__((always_inline)) {
    const unsigned st = __builtin_amdgcn_readfirstlane(stage_wo(c) + wave * kFBlk);
    const int cc = c < nchunks ? c : nchunks - 1;
    const uint16_t* base = wo + cc * kFChunk;
    static_for<0, 3>([&](auto jj) { load_to_lds(st + 4 * kFBlk * decltype(jj)::value, voff_o[decltype(jj)::value], base); });
  };

  floatx16 acc_out[6];
  static_for<0, 6>([&](auto tt) {
    static_for<0, 16>([&](auto vv) { acc_out[decltype(tt)::value][decltype(vv)::value] = 0.f; });
  });

  // The instruction stream of an iteration is laid out by hand and pinned with scheduling barriers (one wave per
  // SIMD: nothing else hides a latency).  LDS operand reads run kPF MFMAs ahead through a ring of registers; the
  // MFMAs of the first products of chunk i carry the vector-ALU work of gelu(gate) * value of chunk i - 1.
  constexpr int kPF = 6;
  constexpr int kNP = 2 * kFKS;       // MFMAs of the first products per chunk: 24

  auto gelu_pack = [&](const float (&gl)[16], bf16x8 (&gt)[2]) __attribute__((always_inline)) {
    static_for<0, 2>([&](auto ss) {
      constexpr int s = decltype(ss)::value;
      u32x4 pk;
      pk.x = pack_bf16x2(gl[8 * s + 0], gl[8 * s + 1]);
      pk.y = pack_bf16x2(gl[8 * s + 2], gl[8 * s + 3]);
      pk.z = pack_bf16x2(gl[8 * s + 4], gl[8 * s + 5]);
      pk.w = pack_bf16x2(gl[8 * s + 6], gl[8 * s + 7]);
      gt[s] = __builtin_bit_cast(bf16x8, pk);
    });
  };

  // first products of chunk i into (g, v); with GLU: gelu * value of chunk i - 1, whose accumulators were copied
  // to (gp, vp) -> gt
  auto first_phase = [&](int i, floatx16& g, floatx16& v, const float (&gp)[16], const float (&vp)[16], bf16x8 (&gt)[2],
                         auto with_glu) __attribute__((always_inline)) {
    constexpr bool GLU = decltype(with_glu)::value;
    const unsigned char* ag = smem + (i % kFStages) * kFGV + 16 * lane;
    // MFMA k: K step k / 2 of the gate (k even) or value (k odd) product
    auto addr = [&](auto kk) __attribute__((always_inline)) {
      constexpr int k = decltype(kk)::value;
      return ag + ((k & 1) * kFKS + (k >> 1)) * kFBlk;
    };
    u32x4 ring[kPF];
    static_for<0, kPF>([&](auto kk) { ring[decltype(kk)::value] = *reinterpret_cast<const u32x4*>(addr(kk)); });
    float gl[16];
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, kNP>([&](auto kk) {
      constexpr int k = decltype(kk)::value;
      const bf16x8 a = __builtin_bit_cast(bf16x8, ring[k % kPF]);
      if constexpr (k == 0) {
        floatx16 z;
        static_for<0, 16>([&](auto vv) { z[decltype(vv)::value] = 0.f; });
        g = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, xa[0], z, 0, 0, 0);
      } else if constexpr (k == 1) {
        floatx16 z;
        static_for<0, 16>([&](auto vv) { z[decltype(vv)::value] = 0.f; });
        v = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, xb[0], z, 0, 0, 0);
      } else if constexpr ((k & 1) == 0) {
        g = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, xa[k >> 1], g, 0, 0, 0);
      } else {
        v = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, xb[k >> 1], v, 0, 0, 0);
      }
      if constexpr (k + kPF < kNP) ring[k % kPF] = *reinterpret_cast<const u32x4*>(addr(ic<k + kPF>{}));
      if constexpr (GLU && k < 16) gl[k] = gelu_erf_poly(gp[k]) * vp[k];
      __builtin_amdgcn_sched_barrier(0);
    });
    if constexpr (GLU) gelu_pack(gl, gt);
  };
  // second product: OUT^T += Wo_chunk (chunk c) * G^T; MFMA k = K step k / 6 of output tile k % 6, so that
  // consecutive MFMAs write different accumulators.  Along with it the accumulators (g, v) of the first products
  // just finished are copied out to (gp, vp) for the next iteration's gelu * value.
  auto second_phase = [&](int c, const bf16x8 (&gt)[2], const floatx16& g, const floatx16& v, float (&gp)[16],
                          float (&vp)[16], auto with_copy) __attribute__((always_inline)) {
    constexpr bool COPY = decltype(with_copy)::value;
    const unsigned char* ao = smem + kFStages * kFGV + (c % kFStages) * kFWO + 16 * lane;
    auto addr = [&](auto kk) __attribute__((always_inline)) {
      constexpr int k = decltype(kk)::value;
      return ao + ((k % 6) * 2 + k / 6) * kFBlk;
    };
    u32x4 ring[kPF];
    static_for<0, kPF>([&](auto kk) { ring[decltype(kk)::value] = *reinterpret_cast<const u32x4*>(addr(kk)); });
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, 12>([&](auto kk) {
      constexpr int k = decltype(kk)::value;
      acc_out[k % 6] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, ring[k % kPF]), gt[k / 6],
                                                               acc_out[k % 6], 0, 0, 0);
      if constexpr (k + kPF < 12) ring[k % kPF] = *reinterpret_cast<const u32x4*>(addr(ic<k + kPF>{}));
      if constexpr (COPY && k >= 4) {
        static_for<4 * (k - 4), 4 * (k - 3)>([&](auto ee) {
          constexpr int e = decltype(ee)::value;
          if constexpr (e < 16) gp[e] = g[e];
          else vp[e - 16] = v[e - 16];
        });
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  };

  // ---- pipeline.  Batch i of loads, issued at the top of iteration i: Wg / Wv of chunk i + 2 into the stage last
  // read as chunk i - 1 (before the barrier of iteration i), Wo of chunk i + 1 into the stage last read as chunk
  // i - 2 (Wo of chunk c is consumed one iteration later than its Wg / Wv, in iteration c + 1).  Before it reaches
  // the barrier of iteration i + 1 a wave waits until at most its newest batch is in flight, so batch i - 1 (Wg / Wv
  // of chunk i + 1, Wo of chunk i) is in LDS for everybody after that barrier.
  dma_gv(0);
  dma_gv(1);
  dma_wo(0);
  floatx16 g, v;
  float gp[16], vp[16];
  bf16x8 gt[2];
  __builtin_amdgcn_s_waitcnt(kWaitVm0);

  // iteration 0: only the first products of chunk 0
  __syncthreads();
  dma_gv(2);
  dma_wo(1);
  first_phase(0, g, v, gp, vp, gt, std::false_type{});
  static_for<0, 16>([&](auto ee) { gp[decltype(ee)::value] = g[decltype(ee)::value]; vp[decltype(ee)::value] = v[decltype(ee)::value]; });
  __builtin_amdgcn_s_waitcnt(kWaitVm9);
  for (int i = 1; i < nchunks; ++i) {
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    dma_gv(i + 2);
    dma_wo(i + 1);
    __builtin_amdgcn_sched_barrier(0);
    first_phase(i, g, v, gp, vp, gt, std::true_type{});
    __builtin_amdgcn_sched_barrier(0);
    second_phase(i - 1, gt, g, v, gp, vp, std::true_type{});
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(kWaitVm9);
  }
  // last iteration: gelu * value and the second product of the last chunk.  No load may still be in flight when
  // the workgroup ends (its LDS goes to the next one).
  __builtin_amdgcn_s_waitcnt(kWaitVm0);
  __syncthreads();
  {
    float gl[16];
    static_for<0, 16>([&](auto kk) { gl[decltype(kk)::value] = gelu_erf_poly(gp[decltype(kk)::value]) * vp[decltype(kk)::value]; });
    gelu_pack(gl, gt);
  }
  second_phase(nchunks - 1, gt, g, v, gp, vp, std::false_type{});

  // ---- epilogue: accumulator element v = 4 a + b of tile t is output column 32 t + 8 a + 4 h + b of x-row i
  const int row = m0 + 32 * wave + i32;
  if (row < M) {
    const long o0 = (long)row * d + r * kFP + 4 * half;
    static_for<0, 6>([&](auto tt) {
      constexpr int t = decltype(tt)::value;
      static_for<0, 4>([&](auto aa) {
        constexpr int a = decltype(aa)::value;
        const int col = 32 * t + 8 * a;
        float4 val = make_float4(acc_out[t][4 * a], acc_out[t][4 * a + 1], acc_out[t][4 * a + 2], acc_out[t][4 * a + 3]);
        if (bias) {
          const float4 bq = *reinterpret_cast<const float4*>(bias + r * kFP + 4 * half + col);
          val.x += bq.x; val.y += bq.y; val.z += bq.z; val.w += bq.w;
        }
        if (resid) {
          const uint2 rr = *reinterpret_cast<const uint2*>(resid + o0 + col);
          val.x += __uint_as_float(rr.x << 16); val.y += __uint_as_float(rr.x & 0xffff0000u);
          val.z += __uint_as_float(rr.y << 16); val.w += __uint_as_float(rr.y & 0xffff0000u);
        }
        if constexpr (sizeof(OUT) == 2) {
          uint2 pk;
          pk.x = pack_bf16x2(val.x, val.y);
          pk.y = pack_bf16x2(val.z, val.w);
          *reinterpret_cast<uint2*>(out + o0 + col) = pk;
        } else {
          *reinterpret_cast<float4*>(out + o0 + col) = val;
        }
      });
    });
  }
}

}  // namespace m2

using namespace m2;

extern "C" int m2_mlp_fused_supported(int in_features, int intermediate, int nblocks) {
  return nblocks == 4 && in_features == 4 * kFP && intermediate > 0 && intermediate % (4 * kFChunk) == 0;
}

extern "C" int m2_mlp_fused_fwd(const void* x, const void* w_gated, const void* w_out, const float* bias,
                                const void* residual, void* out, int M, int in_features, int intermediate, int nblocks,
                                int out_dtype, void* stream) {
  if (!x || !w_gated || !w_out || !out) return set_error(M2_ERR_ARG, "m2_mlp_fused_fwd: null pointer");
  if (M <= 0) return set_error(M2_ERR_ARG, "m2_mlp_fused_fwd: M=%d must be positive", M);
  if (out_dtype != M2_DTYPE_F32 && out_dtype != M2_DTYPE_BF16)
    return set_error(M2_ERR_ARG, "m2_mlp_fused_fwd: out_dtype %d is neither M2_DTYPE_F32 nor M2_DTYPE_BF16", out_dtype);
  if (!m2_mlp_fused_supported(in_features, intermediate, nblocks))
    return set_error(M2_ERR_UNSUPPORTED,
                     "m2_mlp_fused_fwd: built for nblocks=4, in_features=768 and intermediate a multiple of 128 "
                     "(got nblocks=%d in=%d intermediate=%d); use m2_blockdiag_glu_fwd + m2_blockdiag_linear_fwd",
                     nblocks, in_features, intermediate);
  const int ntiles = (M + kFRows - 1) / kFRows;
  const dim3 grid(8 * ((ntiles + 1) / 2));
  hipStream_t st = (hipStream_t)stream;
  if (out_dtype == M2_DTYPE_F32) {
    auto kern = mlp_fused_kernel<float>;
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, kFLds);
    if (e != hipSuccess) return set_error(M2_ERR_LAUNCH, "hipFuncSetAttribute(mlp_fused): %s", hipGetErrorString(e));
    hipLaunchKernelGGL(kern, grid, dim3(256), kFLds, st, (const uint16_t*)x, (const uint16_t*)w_gated, (const uint16_t*)w_out,
                       bias, (const uint16_t*)residual, (float*)out, M, intermediate);
  } else {
    auto kern = mlp_fused_kernel<uint16_t>;
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, kFLds);
    if (e != hipSuccess) return set_error(M2_ERR_LAUNCH, "hipFuncSetAttribute(mlp_fused): %s", hipGetErrorString(e));
    hipLaunchKernelGGL(kern, grid, dim3(256), kFLds, st, (const uint16_t*)x, (const uint16_t*)w_gated, (const uint16_t*)w_out,
                       bias, (const uint16_t*)residual, (uint16_t*)out, M, intermediate);
  }
  return check_launch("mlp_fused");
}
