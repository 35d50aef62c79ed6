// Second linear layer of the GLU MLP fused with what follows it:
//
//   s   = blockdiag_multiply(g, Wo) + bias + residual          (bert/src/bert_layers.py:504-506,
//   out = LayerNorm(s)                                           bert/src/mm/blockdiag_multiply.py:49-60)
//
// in one kernel, so that the fp32 sum s (M x d) is never written to memory.  A workgroup owns 64 full rows
// (all d = 4 q output columns): wave (k, h) holds the 32 x q accumulators of block k for row half h, the K
// dimension (p per block) is walked in chunks of 64 for all four blocks at once (global -> registers -> one
// LDS buffer, the next chunk in flight during the MFMAs).  After the GEMM the residual rows go through LDS,
// row statistics are reduced inside each wave (32 lanes per row) and across the four block-waves through
// LDS (two-pass mean / variance), and the normalised rows leave through an LDS tile, two blocks at a time,
// as bf16 rows, optional fp32 rows and the channel-major fp32 copy the next mixer reads.
//
// Needs nblocks == 4 and q = out_features / 4 a multiple of 32 up to 192 (d <= 768): the accumulators of a
// full row tile must fit the register file.  Other shapes use m2_blockdiag_linear_fwd + m2_layernorm_fwd.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fft_regs.h"
#include "m2_internal.h"

namespace m2 {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kWK = 64;                 // K per chunk
constexpr int kWRow = kWK + 8;          // bf16 elements per padded LDS row (16-byte reads of 16 rows hit distinct banks)
constexpr int kWDepth = 1;              // chunks in flight in registers (a deeper ring spills: 96 accumulators per lane)
constexpr int kWBM = 64;                // rows per workgroup

template <int QT>
struct WoLnShape {
  static constexpr int NB = 4, Q = 32 * QT, D = NB * Q;
  static constexpr int A_ELEMS = NB * kWBM * kWRow, B_ELEMS = NB * Q * kWRow;
  static constexpr size_t MAIN_BYTES = (size_t)(A_ELEMS + B_ELEMS) * sizeof(uint16_t);
  static constexpr int RROW = D + 8;                         // bf16 row of the residual tile
  static constexpr size_t RES_BYTES = (size_t)kWBM * RROW * sizeof(uint16_t);
  static constexpr size_t RED_BYTES = (size_t)2 * NB * kWBM * sizeof(float);
  static constexpr int OROW = 2 * Q + 4;                     // fp32 row of the output tile (two blocks)
  static constexpr size_t OUT_BYTES = (size_t)kWBM * OROW * sizeof(float);
  static constexpr size_t EPI_BYTES = (RES_BYTES > OUT_BYTES ? RES_BYTES : OUT_BYTES) + RED_BYTES;
  static constexpr size_t LDS_BYTES = MAIN_BYTES > EPI_BYTES ? MAIN_BYTES : EPI_BYTES;
};

template <int QT>
__global__ __launch_bounds__(512) void wo_layernorm_kernel(
    const uint16_t* __restrict__ x,       // (M, 4 p) bf16
    const uint16_t* __restrict__ w,       // (4, q, p) bf16
    const float* __restrict__ bias,       // (d) or null
    const uint16_t* __restrict__ resid,   // (M, d) bf16 or null
    const float* __restrict__ gamma, const float* __restrict__ beta, float eps,
    float* __restrict__ out_f32,          // (M, d) or null
    uint16_t* __restrict__ out_bf16,      // (M, d) or null
    float* __restrict__ out_t,            // (d, M) or null
    int M, int p) {
  using S = WoLnShape<QT>;
  constexpr int NB = S::NB, Q = S::Q, D = S::D;
  constexpr int PK = kWK / 8;                                // 16-byte pieces per row and chunk
  constexpr int A_CH = NB * kWBM * PK / 512;                 // pieces per thread and chunk: 2
  constexpr int B_CH = NB * Q * PK / 512;                    // QT
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  uint16_t* sA = reinterpret_cast<uint16_t*>(lds_raw);                       // [NB][64][kWRow]
  uint16_t* sB = sA + S::A_ELEMS;                                            // [NB][Q][kWRow]
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, i32 = lane & 31, half = lane >> 5;
  const int k = wave >> 1, h = wave & 1;
  const int m0 = blockIdx.x * kWBM;
  const long in_f = (long)NB * p;

  // per-thread source pointers / LDS offsets of the pieces it moves (fixed for the whole kernel)
  const uint16_t* pa[A_CH];
  const uint16_t* pb[B_CH];
  int la[A_CH], lb[B_CH];
  static_for<0, A_CH>([&](auto jj) {
    constexpr int j = decltype(jj)::value;
    const int id = tid + 512 * j, kc = id % PK, r = (id / PK) % kWBM, kb = id / (PK * kWBM);
    int row = m0 + r;
    row = row < M ? row : M - 1;
    pa[j] = x + (long)row * in_f + (long)kb * p + kc * 8;
    la[j] = (kb * kWBM + r) * kWRow + kc * 8;
  });
  static_for<0, B_CH>([&](auto jj) {
    constexpr int j = decltype(jj)::value;
    const int id = tid + 512 * j, kc = id % PK, rq = id / PK;              // rq = kb Q + row inside the block
    pb[j] = w + (long)rq * p + kc * 8;
    lb[j] = rq * kWRow + kc * 8;
  });
  u32x4 ra[kWDepth][A_CH], rb[kWDepth][B_CH];                 // ring: chunk c sits in slot c % kWDepth
  auto gload = [&](int c, auto slot_) __attribute__((always_inline)) {
    constexpr int sl = decltype(slot_)::value;
    static_for<0, A_CH>([&](auto jj) { ra[sl][decltype(jj)::value] = *reinterpret_cast<const u32x4*>(pa[decltype(jj)::value] + c * kWK); });
    static_for<0, B_CH>([&](auto jj) { rb[sl][decltype(jj)::value] = *reinterpret_cast<const u32x4*>(pb[decltype(jj)::value] + c * kWK); });
  };
  auto sstore = [&](auto slot_) __attribute__((always_inline)) {
    constexpr int sl = decltype(slot_)::value;
    static_for<0, A_CH>([&](auto jj) { *reinterpret_cast<u32x4*>(sA + la[decltype(jj)::value]) = ra[sl][decltype(jj)::value]; });
    static_for<0, B_CH>([&](auto jj) { *reinterpret_cast<u32x4*>(sB + lb[decltype(jj)::value]) = rb[sl][decltype(jj)::value]; });
  };

  floatx16 acc[QT];
  static_for<0, QT>([&](auto tt) { static_for<0, 16>([&](auto vv) { acc[decltype(tt)::value][decltype(vv)::value] = 0.f; }); });

  const int nchunks = p / kWK;
  const uint16_t* fa = sA + (k * kWBM + 32 * h + i32) * kWRow + 8 * half;
  const uint16_t* fb = sB + (k * Q + i32) * kWRow + 8 * half;
  auto step = [&](int c, auto slot_) __attribute__((always_inline)) {
    constexpr int sl = decltype(slot_)::value;                // c % kWDepth: the slot chunk c came from, free again
    if (c + kWDepth < nchunks) gload(c + kWDepth, ic<sl>{});
    static_for<0, kWK / 16>([&](auto kk_) {
      constexpr int kk = decltype(kk_)::value;
      const bf16x8 a = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(fa + 16 * kk));
      static_for<0, QT>([&](auto tt) {
        constexpr int t = decltype(tt)::value;
        const bf16x8 b = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(fb + 32 * t * kWRow + 16 * kk));
        acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[t], 0, 0, 0);
      });
    });
    __syncthreads();
    if (c + 1 < nchunks) sstore(ic<(sl + 1) % kWDepth>{});
    __syncthreads();
  };
  static_for<0, kWDepth>([&](auto ss) {
    if (decltype(ss)::value < nchunks) gload(decltype(ss)::value, ss);
  });
  sstore(ic<0>{});
  __syncthreads();
  int c = 0;
  for (; c + kWDepth <= nchunks; c += kWDepth)
    static_for<0, kWDepth>([&](auto ss) { step(c + decltype(ss)::value, ss); });
  static_for<0, kWDepth>([&](auto ss) {
    if (c + decltype(ss)::value < nchunks) step(c + decltype(ss)::value, ss);
  });
  // accumulator element v of tile t: row 32 h + 8 (v / 4) + 4 half + v % 4, column k Q + 32 t + i32

  // ---- residual rows through LDS (coalesced 16-byte loads), then s = acc + bias + residual ----
  uint16_t* sR = reinterpret_cast<uint16_t*>(lds_raw);                       // [64][RROW]
  constexpr size_t TILE_BYTES = S::RES_BYTES > S::OUT_BYTES ? S::RES_BYTES : S::OUT_BYTES;
  float* red = reinterpret_cast<float*>(lds_raw + TILE_BYTES);               // [2][NB][64]
  if (resid) {
    constexpr int PPR = D / 8;                                               // 16-byte pieces per row
    constexpr int NP = kWBM * PPR / 512;                                     // pieces per thread: 12 at d = 768
    static_assert(kWBM * PPR % 512 == 0, "residual tile must divide over the threads");
    // all loads first, then all LDS stores: one memory latency for the tile, not one per piece
    u32x4 rr[NP];
    static_for<0, NP>([&](auto jj) {
      constexpr int j = decltype(jj)::value;
      const int id = tid + 512 * j, r = id / PPR, pc = id % PPR;
      int row = m0 + r;
      row = row < M ? row : M - 1;
      rr[j] = *reinterpret_cast<const u32x4*>(resid + (long)row * D + 8 * pc);
    });
    static_for<0, NP>([&](auto jj) {
      constexpr int j = decltype(jj)::value;
      const int id = tid + 512 * j, r = id / PPR, pc = id % PPR;
      *reinterpret_cast<u32x4*>(sR + r * S::RROW + 8 * pc) = rr[j];
    });
    __syncthreads();
  }
  float gm[QT], bt[QT];
  static_for<0, QT>([&](auto tt) {
    constexpr int t = decltype(tt)::value;
    const int col = k * Q + 32 * t + i32;
    gm[t] = gamma[col];
    bt[t] = beta[col];
    const float bs = bias ? bias[col] : 0.f;
    static_for<0, 16>([&](auto vv) {
      constexpr int v = decltype(vv)::value;
      const int r = 32 * h + 8 * (v >> 2) + 4 * half + (v & 3);
      float add = bs;
      if (resid) add += bf16_to_f32(sR[r * S::RROW + col]);
      acc[t][v] += add;
    });
  });

  // ---- row statistics: two passes; 32 lanes of a half-wave share a row, four block-waves share it through LDS ----
  float mean[16], rstd[16];
  static_for<0, 2>([&](auto pass_) {
    constexpr int pass = decltype(pass_)::value;
    float part[16];
    static_for<0, 16>([&](auto vv) {
      constexpr int v = decltype(vv)::value;
      float sacc = 0.f;
      static_for<0, QT>([&](auto tt) {
        constexpr int t = decltype(tt)::value;
        if constexpr (pass == 0) {
          sacc += acc[t][v];
        } else {
          const float cdev = acc[t][v] - mean[v];
          sacc += cdev * cdev;
        }
      });
      part[v] = sacc;
    });
    for (int o = 16; o > 0; o >>= 1)
      static_for<0, 16>([&](auto vv) { part[decltype(vv)::value] += __shfl_xor(part[decltype(vv)::value], o); });
    float* rd = red + pass * NB * kWBM;
    if (i32 == 0)
      static_for<0, 16>([&](auto vv) {
        constexpr int v = decltype(vv)::value;
        rd[k * kWBM + 32 * h + 8 * (v >> 2) + 4 * half + (v & 3)] = part[v];
      });
    __syncthreads();
    static_for<0, 16>([&](auto vv) {
      constexpr int v = decltype(vv)::value;
      const int r = 32 * h + 8 * (v >> 2) + 4 * half + (v & 3);
      const float tot = (rd[r] + rd[kWBM + r]) + (rd[2 * kWBM + r] + rd[3 * kWBM + r]);
      if constexpr (pass == 0) mean[v] = tot * (1.0f / (float)D);
      else rstd[v] = rsqrtf(tot * (1.0f / (float)D) + eps);
    });
  });
  static_for<0, QT>([&](auto tt) {
    constexpr int t = decltype(tt)::value;
    static_for<0, 16>([&](auto vv) {
      constexpr int v = decltype(vv)::value;
      acc[t][v] = (acc[t][v] - mean[v]) * rstd[v] * gm[t] + bt[t];
    });
  });

  // ---- outputs through an LDS tile, two blocks (2 Q columns) per phase ----
  float* sO = reinterpret_cast<float*>(lds_raw);                             // [64][OROW]
  static_for<0, 2>([&](auto ph_) {
    constexpr int ph = decltype(ph_)::value;
    __syncthreads();                               // residual tile / previous phase have been read
    if ((k >> 1) == ph) {
      float* so = sO + (32 * h + 4 * half) * S::OROW + (k & 1) * Q + i32;
      static_for<0, QT>([&](auto tt) {
        constexpr int t = decltype(tt)::value;
        static_for<0, 16>([&](auto vv) {
          constexpr int v = decltype(vv)::value;
          so[(8 * (v >> 2) + (v & 3)) * S::OROW + 32 * t] = acc[t][v];
        });
      });
    }
    __syncthreads();
    const int c0 = 2 * ph * Q;                     // first output column of this phase
    if (out_bf16) {
      constexpr int PPR = 2 * Q / 8;               // pieces of 8 columns per row
      for (int id = tid; id < kWBM * PPR; id += 512) {
        const int r = id / PPR, pc = id % PPR;
        if (m0 + r < M) {
          const float4 v0 = *reinterpret_cast<const float4*>(sO + r * S::OROW + 8 * pc);
          const float4 v1 = *reinterpret_cast<const float4*>(sO + r * S::OROW + 8 * pc + 4);
          u32x4 o = {pack_bf16x2(v0.x, v0.y), pack_bf16x2(v0.z, v0.w), pack_bf16x2(v1.x, v1.y), pack_bf16x2(v1.z, v1.w)};
          *reinterpret_cast<u32x4*>(out_bf16 + (long)(m0 + r) * D + c0 + 8 * pc) = o;
        }
      }
    }
    if (out_f32) {
      constexpr int PPR = 2 * Q / 4;
      for (int id = tid; id < kWBM * PPR; id += 512) {
        const int r = id / PPR, pc = id % PPR;
        if (m0 + r < M)
          *reinterpret_cast<float4*>(out_f32 + (long)(m0 + r) * D + c0 + 4 * pc) =
              *reinterpret_cast<const float4*>(sO + r * S::OROW + 4 * pc);
      }
    }
    if (out_t) {
      // lane = (token r16, channel cc): 16 tokens x 4 channels per instruction -- the 64 LDS reads hit 64 banks
      const int r16 = lane & 15, cc = lane >> 4;
      for (int cb = 4 * wave; cb < 2 * Q; cb += 32) {
        static_for<0, 4>([&](auto rr_) {
          const int r = 16 * decltype(rr_)::value + r16;
          if (m0 + r < M) out_t[(long)(c0 + cb + cc) * M + m0 + r] = sO[r * S::OROW + cb + cc];
        });
      }
    }
  });
}

template <int QT>
static int launch_wo_layernorm(const void* x, const void* w, const float* bias, const void* resid, const float* gamma,
                               const float* beta, float eps, float* out_f32, void* out_bf16, float* out_t, int M, int p,
                               hipStream_t stream) {
  auto kern = wo_layernorm_kernel<QT>;
  const size_t lds = WoLnShape<QT>::LDS_BYTES;
  if (lds > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return set_error(M2_ERR_LAUNCH, "hipFuncSetAttribute(wo_layernorm): %s", hipGetErrorString(e));
  }
  hipLaunchKernelGGL(kern, dim3((M + kWBM - 1) / kWBM), dim3(512), lds, stream, (const uint16_t*)x, (const uint16_t*)w, bias,
                     (const uint16_t*)resid, gamma, beta, eps, out_f32, (uint16_t*)out_bf16, out_t, M, p);
  return check_launch("wo_layernorm");
}

}  // namespace m2

using namespace m2;

extern "C" int m2_blockdiag_linear_layernorm_supported(int in_features, int out_features, int nblocks) {
  if (nblocks != 4 || in_features <= 0 || out_features <= 0 || in_features % 4 || out_features % 4) return 0;
  const int p = in_features / 4, q = out_features / 4;
  return (p % kWK == 0 && q % 32 == 0 && q <= 192) ? 1 : 0;
}

extern "C" int m2_blockdiag_linear_layernorm_fwd(const void* x, const void* w, const float* bias, const void* residual,
                                                 const float* gamma, const float* beta, float eps, float* out_f32,
                                                 void* out_bf16, float* out_channel_major, int M, int in_features,
                                                 int out_features, int nblocks, void* stream) {
  if (!x || !w || !gamma || !beta) return set_error(M2_ERR_ARG, "m2_blockdiag_linear_layernorm_fwd: null pointer");
  if (M <= 0) return set_error(M2_ERR_ARG, "m2_blockdiag_linear_layernorm_fwd: M must be positive, got %d", M);
  if (!m2_blockdiag_linear_layernorm_supported(in_features, out_features, nblocks))
    return set_error(M2_ERR_UNSUPPORTED,
                     "m2_blockdiag_linear_layernorm_fwd: needs nblocks == 4, (in/4) %% 64 == 0, (out/4) %% 32 == 0 and out <= 768 "
                     "(in=%d out=%d nblocks=%d)", in_features, out_features, nblocks);
  const int p = in_features / 4, q = out_features / 4;
  hipStream_t st = (hipStream_t)stream;
  switch (q / 32) {
#define WL_CASE(QT) \
  case QT:          \
    return launch_wo_layernorm<QT>(x, w, bias, residual, gamma, beta, eps, out_f32, out_bf16, out_channel_major, M, p, st);
    WL_CASE(1) WL_CASE(2) WL_CASE(3) WL_CASE(4) WL_CASE(5) WL_CASE(6)
#undef WL_CASE
  }
  return set_error(M2_ERR_UNSUPPORTED, "m2_blockdiag_linear_layernorm_fwd: no kernel for out/4 = %d", q);
}
