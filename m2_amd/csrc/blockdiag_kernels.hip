// Block-diagonal ("Monarch") linear layers of the M2-BERT GLU MLP on bf16 MFMA, and the LayerNorm
// that closes the layer.
//
//   out[m, k q + j] = sum_i x[m, k p + i] w[k, j, i]          (bert/src/mm/blockdiag_multiply.py:19-34,49-60)
//
// Gated form: gelu_erf(gate) * value in the epilogue, where gate column j (block j / q) pairs with value
// column I + j (block j / q + nb/2)   (bert/src/bert_layers.py:482-502): `blockdiag_glu_ws3_kernel` (K <= 192,
// weights stationary in registers, software-pipelined), `blockdiag_glu_ws_kernel` (K = 256),
// `blockdiag_kernel<GLU=true>` (longer K).
// Plain form with bias and a residual (bert/src/bert_layers.py:504-506, bert/src/mm/structured_linear.py:65-69):
// `blockdiag_wide_kernel` (192-column tiles: q a multiple of 192), `blockdiag_kernel<GLU=false>` (other widths).
// `layernorm_kernel` normalises rows and writes the three forms the next layer reads.
//
// MFMA: v_mfma_f32_32x32x16_bf16.  Lane (i = lane % 32, h = lane / 32) supplies A[i][8h .. 8h+7] and
// B[8h .. 8h+7][i]; both operands are K-contiguous in memory (x row-major, w[k] is (q, p)), so every
// operand register is one 16-byte LDS read.  Accumulator element v of a lane is row 8 (v/4) + 4 h + v%4,
// column i.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fft_regs.h"
#include "m2_internal.h"

namespace m2 {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ bf16x8 ld8(const uint16_t* p) {
  return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p));
}

// x * Phi(x), Phi(x) - 1/2 = erf(x / sqrt2) / 2 as an odd polynomial of degree 13 on |x| <= 3.9 (clamped beyond,
// where Phi is within 5e-5 of 0 or 1).  Least-squares fit on Chebyshev nodes; evaluated in fp32 the result is within
// 1.8e-4 absolute of the fp64 erf form for every fp32 x in [-9, 9] (checked on the CPU), below the bf16 rounding the
// caller applies to it wherever the result is larger than 0.05 and a fraction of a per cent of the layer's output
// scale below that.  10 vector-ALU instructions and no transcendental: the GLU epilogue, not the product, bounds
// the gated kernel, so two multiply-adds less per output (degree 17 gave 7.6e-5) are worth more than the digits.
__device__ __forceinline__ float gelu_erf(float x) {
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

// ---------------------------------------------------------------------------------------------
// LDS-tiled GEMM core.  Workgroup = WR x WC waves (4 or 8); wave tile 64 x 64 (2 x 2 MFMA tiles);
// workgroup tile BM = 64 WR rows by BN = 64 WC output columns.  K advances in chunks of 64: global
// memory -> registers -> LDS (rows padded to 144 bytes so that the 16-byte operand reads of 32
// consecutive rows fall in distinct banks), double buffered, one barrier per chunk.  The finished
// tile goes back through LDS so that every global store is a full contiguous row segment.
//
// GLU: the chunk sequence runs the gate GEMM (block kb) and then the value GEMM (block kb + nb/2) of
// the same output columns; gelu(gate) is parked in registers as packed bf16 between the two.
// ---------------------------------------------------------------------------------------------
constexpr int kBK = 64;
constexpr int kLdsRow = kBK + 8;          // bf16 elements per padded LDS row (144 bytes)

// RAG: block sizes that are not multiples of the tile (p, q multiples of 8 only, e.g. the 240-wide blocks of
// d = 960): the last K chunk of a block is filled with zeros beyond p, the last column tile of a block computes
// on clamped weight rows and stores only the columns below q.
template <int WR, int WC, bool GLU, typename OUT, int NSTAGE, bool RAG = false>
__global__ __launch_bounds__(64 * WR * WC) void blockdiag_kernel(
    const uint16_t* __restrict__ x,      // (M, nb p) bf16
    const uint16_t* __restrict__ w,      // (nb, q, p) bf16
    const float* __restrict__ bias,      // (nb q) or null            [GLU: unused]
    const uint16_t* __restrict__ resid,  // (M, nb q) bf16 or null    [GLU: unused]
    OUT* __restrict__ out,               // GLU: (M, nb q / 2) ; else (M, nb q)
    int M, int nb, int p, int q) {
  constexpr int BM = 64 * WR, BN = 64 * WC, NT = 64 * WR * WC;                 // NT threads: WR x WC waves
  constexpr int A_CH = BM * (kBK / 8) / NT, B_CH = BN * (kBK / 8) / NT;        // 16-byte chunks per thread
  static_assert(A_CH >= 1 && B_CH >= 1 && (BM * (kBK / 8)) % NT == 0 && (BN * (kBK / 8)) % NT == 0, "tile must divide over the threads");
  constexpr int STAGE = (BM + BN) * kLdsRow;                                   // bf16 elements per stage
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, i32 = lane & 31, half = lane >> 5;
  const int wr = wave / WC, wc = wave % WC;
  // Workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2.  XCD e takes the row
  // tiles e, e+8, ... and walks all column tiles of one row tile back to back, so the x rows and the
  // weights of the tiles in flight on an XCD stay in that XCD's L2.
  int tile_m, tile_n;
  {
    const int ntm = (M + BM - 1) / BM, ntn = (GLU ? nb / 2 : nb) * ((q + BN - 1) / BN);
    const int id = blockIdx.x, e = id & 7, l = id >> 3;
    const int full = (ntm / 8) * 8;                   // row tiles covered by the XCD-striped part
    if (id < full * ntn) {
      tile_m = (l / ntn) * 8 + e;
      tile_n = l % ntn;
    } else {                                          // remainder rows: plain order
      const int rid = id - full * ntn;
      tile_m = full + rid / ntn;
      tile_n = rid % ntn;
    }
  }
  const int m0 = tile_m * BM;
  const int ntn_b = (q + BN - 1) / BN;                // column tiles per block
  const int blk = tile_n / ntn_b, jj = (tile_n % ntn_b) * BN;      // weight block and first row inside it (gate block for GLU)
  const int n0 = blk * q + jj;                        // first output column of the tile
  const int in_f = nb * p;
  const int out_cols = GLU ? nb * q / 2 : nb * q;
  const int kchunks = (p + kBK - 1) / kBK;
  const int kc8 = (tid & 7) * 8;                      // K offset of every 16-byte piece this thread moves (NT is a multiple of 8)
  const int nchunks = GLU ? 2 * kchunks : kchunks;

  // per-thread source rows of the 16-byte chunks it moves (fixed for the whole kernel)
  const uint16_t* pa[A_CH];
  const uint16_t* pb[B_CH];
  int la[A_CH], lb[B_CH];
  static_for<0, A_CH>([&](auto jj_) {
    constexpr int j = decltype(jj_)::value;
    const int id = tid + NT * j, r = id >> 3, kc = id & 7;
    int row = m0 + r;
    row = row < M ? row : M - 1;
    pa[j] = x + (long)row * in_f + (long)blk * p + kc * 8;
    la[j] = r * kLdsRow + kc * 8;
  });
  static_for<0, B_CH>([&](auto jj_) {
    constexpr int j = decltype(jj_)::value;
    const int id = tid + NT * j, r = id >> 3, kc = id & 7;
    int wrow = jj + r;
    if constexpr (RAG) wrow = wrow < q ? wrow : q - 1;      // columns past the block's end: computed, never stored
    pb[j] = w + ((long)blk * q + wrow) * p + kc * 8;
    lb[j] = (BM + r) * kLdsRow + kc * 8;
  });
  const long a_phase = (long)(nb / 2) * p;            // value block = gate block + nb/2
  const long b_phase = (long)(nb / 2) * q * p;

  u32x4 ra[A_CH], rb[B_CH];
  auto gload = [&](int c) __attribute__((always_inline)) {
    const int phase = GLU ? c / kchunks : 0;
    const long ao = phase * a_phase + (c % kchunks) * kBK;
    const long bo = phase * b_phase + (c % kchunks) * kBK;
    if constexpr (RAG) {
      if ((c % kchunks) * kBK + kc8 >= p) {           // beyond the block's K range: zeros on both sides
        const u32x4 z = {0u, 0u, 0u, 0u};
        static_for<0, A_CH>([&](auto jj_) { ra[decltype(jj_)::value] = z; });
        static_for<0, B_CH>([&](auto jj_) { rb[decltype(jj_)::value] = z; });
        return;
      }
    }
    static_for<0, A_CH>([&](auto jj_) { ra[decltype(jj_)::value] = *reinterpret_cast<const u32x4*>(pa[decltype(jj_)::value] + ao); });
    static_for<0, B_CH>([&](auto jj_) { rb[decltype(jj_)::value] = *reinterpret_cast<const u32x4*>(pb[decltype(jj_)::value] + bo); });
  };
  auto sstore = [&](int stage) __attribute__((always_inline)) {
    uint16_t* st = smem + stage * STAGE;
    static_for<0, A_CH>([&](auto jj_) { *reinterpret_cast<u32x4*>(st + la[decltype(jj_)::value]) = ra[decltype(jj_)::value]; });
    static_for<0, B_CH>([&](auto jj_) { *reinterpret_cast<u32x4*>(st + lb[decltype(jj_)::value]) = rb[decltype(jj_)::value]; });
  };

  // accumulators: [0] = the GEMM (gate GEMM for GLU), [1] = value GEMM (GLU only)
  floatx16 acc[GLU ? 2 : 1][2][2];
  static_for<0, (GLU ? 2 : 1)>([&](auto ss) {
    static_for<0, 4>([&](auto tt) {
      static_for<0, 16>([&](auto vv) { acc[decltype(ss)::value][decltype(tt)::value / 2][decltype(tt)::value % 2][decltype(vv)::value] = 0.f; });
    });
  });

  auto compute = [&](int stage, auto set_) __attribute__((always_inline)) {
    constexpr int set = decltype(set_)::value;
    const uint16_t* sa = smem + stage * STAGE + (wr * 64 + i32) * kLdsRow + 8 * half;
    const uint16_t* sb = smem + stage * STAGE + BM * kLdsRow + (wc * 64 + i32) * kLdsRow + 8 * half;
    static_for<0, kBK / 16>([&](auto kk_) {
      constexpr int kk = decltype(kk_)::value;
      bf16x8 av[2], bv[2];
      av[0] = ld8(sa + kk * 16);
      av[1] = ld8(sa + 32 * kLdsRow + kk * 16);
      bv[0] = ld8(sb + kk * 16);
      bv[1] = ld8(sb + 32 * kLdsRow + kk * 16);
      acc[set][0][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[0], bv[0], acc[set][0][0], 0, 0, 0);
      acc[set][0][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[0], bv[1], acc[set][0][1], 0, 0, 0);
      acc[set][1][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[1], bv[0], acc[set][1][0], 0, 0, 0);
      acc[set][1][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[1], bv[1], acc[set][1][1], 0, 0, 0);
    });
  };

  // NSTAGE == 2: double-buffered LDS, one barrier per chunk.  NSTAGE == 1: one LDS buffer and the next
  // chunk parked in registers (two barriers per chunk, but half the LDS, so more workgroups per CU
  // keep more loads in flight).
  auto step = [&](int c, auto set_) __attribute__((always_inline)) {
    if (c + 1 < nchunks) gload(c + 1);
    compute(NSTAGE == 2 ? (c & 1) : 0, set_);
    if constexpr (NSTAGE == 1) __syncthreads();
    if (c + 1 < nchunks) sstore(NSTAGE == 2 ? ((c + 1) & 1) : 0);
    __syncthreads();
  };
  gload(0);
  sstore(0);
  __syncthreads();
  for (int c = 0; c < kchunks; ++c) step(c, ic<0>{});                 // first (or only) GEMM
  if constexpr (GLU)
    for (int c = kchunks; c < nchunks; ++c) step(c, ic<1>{});         // value GEMM

  // ---- epilogue: tile -> LDS (fp32) -> coalesced rows, EP passes of BM / EP rows each ----
  constexpr int OROW = BN + 4;                          // padded fp32 row
  constexpr int EP = (WR == 4) ? 2 : 1;
  constexpr int EROWS = BM / EP;
  constexpr int TPR = BN / 4, RPI = NT / TPR;           // each thread moves 4 consecutive columns
  const int cq = (tid % TPR) * 4;
  const bool col_ok = !RAG || jj + cq < q;             // q is a multiple of 8: four columns are all in or all out
  float4 bq = make_float4(0.f, 0.f, 0.f, 0.f);
  if (!GLU && bias && col_ok) bq = *reinterpret_cast<const float4*>(bias + n0 + cq);
  for (int ep = 0; ep < EP; ++ep) {
    if (wr / (WR / EP) == ep) {
      float* so = reinterpret_cast<float*>(smem) + ((wr % (WR / EP)) * 64 + 4 * half) * OROW + wc * 64 + i32;
      static_for<0, 4>([&](auto tt) {
        constexpr int t = decltype(tt)::value, a = t / 2, b = t % 2;
        static_for<0, 16>([&](auto vv) {
          constexpr int v = decltype(vv)::value;
          float val = acc[0][a][b][v];
          if constexpr (GLU) val = gelu_erf(val) * acc[GLU ? 1 : 0][a][b][v];
          so[(32 * a + 8 * (v >> 2) + (v & 3)) * OROW + 32 * b] = val;
        });
      });
    }
    // the residual values of the pass are requested all at once, before the barrier: loaded where they are used,
    // every row of the copy loop waited a full memory latency
    constexpr int NR = EROWS / RPI;
    static_assert(EROWS % RPI == 0, "rows of a pass must divide over the threads");
    uint2 rres[NR];
    if constexpr (!GLU) {
      static_for<0, NR>([&](auto ii) {
        constexpr int i = decltype(ii)::value;
        const int row = m0 + ep * EROWS + tid / TPR + i * RPI;
        rres[i] = make_uint2(0u, 0u);
        if (resid && row < M && col_ok) rres[i] = *reinterpret_cast<const uint2*>(resid + (long)row * out_cols + n0 + cq);
      });
    }
    __syncthreads();
    const float* srow = reinterpret_cast<const float*>(smem) + cq;
    static_for<0, NR>([&](auto ii) {
      constexpr int i = decltype(ii)::value;
      const int r = tid / TPR + i * RPI;
      const int row = m0 + ep * EROWS + r;
      if (row < M && col_ok) {
        float4 v4 = *reinterpret_cast<const float4*>(srow + r * OROW);
        const long o = (long)row * out_cols + n0 + cq;
        if constexpr (!GLU) {
          v4.x += bq.x + __uint_as_float(rres[i].x << 16); v4.y += bq.y + __uint_as_float(rres[i].x & 0xffff0000u);
          v4.z += bq.z + __uint_as_float(rres[i].y << 16); v4.w += bq.w + __uint_as_float(rres[i].y & 0xffff0000u);
        }
        if constexpr (sizeof(OUT) == 2) {
          uint2 pk;
          pk.x = pack_bf16x2(v4.x, v4.y);
          pk.y = pack_bf16x2(v4.z, v4.w);
          *reinterpret_cast<uint2*>(out + o) = pk;
        } else {
          *reinterpret_cast<float4*>(out + o) = v4;
        }
      }
    });
    if (ep + 1 < EP) __syncthreads();
  }
}

template <int WR, int WC, bool GLU, typename OUT, int NSTAGE, bool RAG = false>
static int launch_blockdiag(const void* x, const void* w, const float* bias, const void* resid, void* out, int M,
                            int nb, int p, int q, int out_cols, hipStream_t stream) {
  constexpr int BM = 64 * WR, BN = 64 * WC;
  size_t lds = (size_t)NSTAGE * (BM + BN) * kLdsRow * sizeof(uint16_t);
  const size_t epi = (size_t)(BM / (WR == 4 ? 2 : 1)) * (BN + 4) * sizeof(float);
  if (epi > lds) lds = epi;
  auto kern = blockdiag_kernel<WR, WC, GLU, OUT, NSTAGE, RAG>;
  if (lds > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return set_error(M2_ERR_LAUNCH, "hipFuncSetAttribute(blockdiag): %s", hipGetErrorString(e));
  }
  dim3 grid(((M + BM - 1) / BM) * ((out_cols / q) * ((q + BN - 1) / BN)));
  hipLaunchKernelGGL(kern, grid, dim3(64 * WR * WC), lds, stream, (const uint16_t*)x, (const uint16_t*)w, bias,
                     (const uint16_t*)resid, (OUT*)out, M, nb, p, q);
  return check_launch("blockdiag");
}

// ---------------------------------------------------------------------------------------------
// Block-diagonal linear layer with a 256 x 192 workgroup tile (q a multiple of 192: d = 768, 1536).
//
// Operand delivery (L2 -> LDS -> registers) bounds these GEMMs long before the MFMA pipe does, so the tile is
// as large as the register file allows: 8 waves as 4 (row groups of 64) x 2 (column halves of 96), 6 MFMA
// tiles = 96 accumulators per lane, and with q = 192 a tile spans the whole width of a block, so every x
// element is fetched exactly once.  K advances in chunks of 64 through a double-buffered LDS stage (one
// barrier per chunk, the chunk after next in flight in registers); per K step of 16 a wave reads 2 A and 3 B
// operands for 6 MFMAs.  Epilogue: bias + bf16 residual, rows leave through LDS 64 at a time as full segments.
// ---------------------------------------------------------------------------------------------
constexpr int kWideBM = 256, kWideBN = 192;
template <typename OUT>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void blockdiag_wide_kernel(
    const uint16_t* __restrict__ x,      // (M, nb p) bf16
    const uint16_t* __restrict__ w,      // (nb, q, p) bf16
    const float* __restrict__ bias,      // (nb q) or null
    const uint16_t* __restrict__ resid,  // (M, nb q) bf16 or null
    OUT* __restrict__ out,               // (M, nb q)
    int M, int nb, int p, int q) {
  constexpr int BM = kWideBM, BN = kWideBN, NT = 512, WRG = BM / 64;
  constexpr int A_CH = BM * (kBK / 8) / NT, B_CH = BN * (kBK / 8) / NT;        // chunks of 16 bytes per thread: 4 and 3
  constexpr int STAGE = (BM + BN) * kLdsRow;
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, i32 = lane & 31, half = lane >> 5;
  const int wr = wave >> 1, wc = wave & 1;
  int tile_m, tile_n;
  {
    const int ntm = (M + BM - 1) / BM, ntn = nb * q / BN;
    const int id = blockIdx.x, e = id & 7, l = id >> 3;
    const int full = (ntm / 8) * 8;
    if (id < full * ntn) { tile_m = (l / ntn) * 8 + e; tile_n = l % ntn; }
    else { const int rid = id - full * ntn; tile_m = full + rid / ntn; tile_n = rid % ntn; }
  }
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int in_f = nb * p, out_cols = nb * q;
  const int blk = n0 / q, jj = n0 % q;
  const int nchunks = p / kBK;

  const uint16_t* pa[A_CH];
  const uint16_t* pb[B_CH];
  int la[A_CH], lb[B_CH];
  static_for<0, A_CH>([&](auto jj_) {
    constexpr int j = decltype(jj_)::value;
    const int id = tid + NT * j, r = id >> 3, kc = id & 7;
    int row = m0 + r;
    row = row < M ? row : M - 1;
    pa[j] = x + (long)row * in_f + (long)blk * p + kc * 8;
    la[j] = r * kLdsRow + kc * 8;
  });
  static_for<0, B_CH>([&](auto jj_) {
    constexpr int j = decltype(jj_)::value;
    const int id = tid + NT * j, r = id >> 3, kc = id & 7;
    pb[j] = w + ((long)blk * q + jj + r) * p + kc * 8;
    lb[j] = (BM + r) * kLdsRow + kc * 8;
  });
  // two chunks in flight in registers (ring slot = chunk & 1) on top of the one waiting in the other LDS stage:
  // with one workgroup per compute unit the loads in flight are what hides the memory latency
  u32x4 ra[2][A_CH], rb[2][B_CH];
  auto gload = [&](int c, auto slot_) __attribute__((always_inline)) {
    constexpr int sl = decltype(slot_)::value;
    static_for<0, A_CH>([&](auto jj_) { ra[sl][decltype(jj_)::value] = *reinterpret_cast<const u32x4*>(pa[decltype(jj_)::value] + c * kBK); });
    static_for<0, B_CH>([&](auto jj_) { rb[sl][decltype(jj_)::value] = *reinterpret_cast<const u32x4*>(pb[decltype(jj_)::value] + c * kBK); });
  };
  auto sstore = [&](int stage, auto slot_) __attribute__((always_inline)) {
    constexpr int sl = decltype(slot_)::value;
    uint16_t* st = smem + stage * STAGE;
    static_for<0, A_CH>([&](auto jj_) { *reinterpret_cast<u32x4*>(st + la[decltype(jj_)::value]) = ra[sl][decltype(jj_)::value]; });
    static_for<0, B_CH>([&](auto jj_) { *reinterpret_cast<u32x4*>(st + lb[decltype(jj_)::value]) = rb[sl][decltype(jj_)::value]; });
  };

  floatx16 acc[2][3];
  static_for<0, 6>([&](auto tt) {
    static_for<0, 16>([&](auto vv) { acc[decltype(tt)::value / 3][decltype(tt)::value % 3][decltype(vv)::value] = 0.f; });
  });
  auto compute = [&](int stage) __attribute__((always_inline)) {
    const uint16_t* sa = smem + stage * STAGE + (wr * 64 + i32) * kLdsRow + 8 * half;
    const uint16_t* sb = smem + stage * STAGE + (BM + wc * 96 + i32) * kLdsRow + 8 * half;
    static_for<0, kBK / 16>([&](auto kk_) {
      constexpr int kk = decltype(kk_)::value;
      bf16x8 av[2], bv[3];
      av[0] = ld8(sa + kk * 16);
      av[1] = ld8(sa + 32 * kLdsRow + kk * 16);
      static_for<0, 3>([&](auto bb) { bv[decltype(bb)::value] = ld8(sb + 32 * decltype(bb)::value * kLdsRow + kk * 16); });
      static_for<0, 6>([&](auto tt) {
        constexpr int a = decltype(tt)::value / 3, b = decltype(tt)::value % 3;
        acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[a], bv[b], acc[a][b], 0, 0, 0);
      });
    });
  };
  // chunk c is multiplied from LDS stage c & 1 while chunk c + 1 moves from ring slot (c + 1) & 1 to the other
  // stage and chunk c + 3 is requested into that slot
  auto step = [&](int c, auto par_) __attribute__((always_inline)) {
    constexpr int nx = (decltype(par_)::value + 1) & 1;          // (c + 1) & 1
    compute(c & 1);
    if (c + 1 < nchunks) {
      sstore(nx, ic<nx>{});                // that stage was last read before the barrier that ended chunk c - 1
      if (c + 3 < nchunks) gload(c + 3, ic<nx>{});
    }
    __syncthreads();
  };
  gload(0, ic<0>{});
  sstore(0, ic<0>{});
  if (nchunks > 1) gload(1, ic<1>{});
  if (nchunks > 2) gload(2, ic<0>{});
  __syncthreads();
  int c = 0;
  for (; c + 1 < nchunks; c += 2) {
    step(c, ic<0>{});
    step(c + 1, ic<1>{});
  }
  if (c < nchunks) step(c, ic<0>{});

  // ---- epilogue: 64 rows at a time (the rows of wave row group ep) through an fp32 LDS tile.  The residual
  // values of a pass are requested one pass ahead, all at once: loaded where they are used, every row of the
  // copy loop waited a full memory latency ----
  constexpr int OROW = BN + 4;
  constexpr int TPR = BN / 4, RPI = NT / TPR;           // 48 threads per row, 10 rows per sweep (32 threads idle)
  constexpr int NR = (64 + RPI - 1) / RPI;              // rows per thread and pass: 7
  float* so_base = reinterpret_cast<float*>(smem);
  const int cq = (tid % TPR) * 4, r0 = tid / TPR;
  float4 bq = make_float4(0.f, 0.f, 0.f, 0.f);
  if (bias) bq = *reinterpret_cast<const float4*>(bias + n0 + cq);
  auto row_ok = [&](int ep, int i) { return tid < TPR * RPI && r0 + i * RPI < 64 && m0 + ep * 64 + r0 + i * RPI < M; };
  uint32_t rx[2][NR], ry[2][NR];
  auto load_resid = [&](int ep, auto slot_) __attribute__((always_inline)) {
    constexpr int sl = decltype(slot_)::value;
    static_for<0, NR>([&](auto ii) {
      constexpr int i = decltype(ii)::value;
      uint2 rr = make_uint2(0u, 0u);
      if (resid && row_ok(ep, i))
        rr = *reinterpret_cast<const uint2*>(resid + (long)(m0 + ep * 64 + r0 + i * RPI) * out_cols + n0 + cq);
      rx[sl][i] = rr.x;
      ry[sl][i] = rr.y;
    });
  };
  load_resid(0, ic<0>{});
  static_for<0, WRG>([&](auto ee) {
    constexpr int ep = decltype(ee)::value, sl = ep & 1;
    if (wr == ep) {
      float* so = so_base + (4 * half) * OROW + wc * 96 + i32;
      static_for<0, 6>([&](auto tt) {
        constexpr int a = decltype(tt)::value / 3, b = decltype(tt)::value % 3;
        static_for<0, 16>([&](auto vv) {
          constexpr int v = decltype(vv)::value;
          so[(32 * a + 8 * (v >> 2) + (v & 3)) * OROW + 32 * b] = acc[a][b][v];
        });
      });
    }
    if constexpr (ep + 1 < WRG) load_resid(ep + 1, ic<(sl ^ 1)>{});
    __syncthreads();
    static_for<0, NR>([&](auto ii) {
      constexpr int i = decltype(ii)::value;
      if (row_ok(ep, i)) {
        const int r = r0 + i * RPI;
        float4 v4 = *reinterpret_cast<const float4*>(so_base + r * OROW + cq);
        const long o = (long)(m0 + ep * 64 + r) * out_cols + n0 + cq;
        v4.x += bq.x + __uint_as_float(rx[sl][i] << 16); v4.y += bq.y + __uint_as_float(rx[sl][i] & 0xffff0000u);
        v4.z += bq.z + __uint_as_float(ry[sl][i] << 16); v4.w += bq.w + __uint_as_float(ry[sl][i] & 0xffff0000u);
        if constexpr (sizeof(OUT) == 2) {
          uint2 pk;
          pk.x = pack_bf16x2(v4.x, v4.y);
          pk.y = pack_bf16x2(v4.z, v4.w);
          *reinterpret_cast<uint2*>(out + o) = pk;
        } else {
          *reinterpret_cast<float4*>(out + o) = v4;
        }
      }
    });
    __syncthreads();
  });
}

template <typename OUT>
static int launch_blockdiag_wide(const void* x, const void* w, const float* bias, const void* resid, void* out, int M,
                                 int nb, int p, int q, hipStream_t stream) {
  const size_t lds = (size_t)2 * (kWideBM + kWideBN) * kLdsRow * sizeof(uint16_t);      // 129 KB; the epilogue tile (50 KB) reuses it
  auto kern = blockdiag_wide_kernel<OUT>;
  hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return set_error(M2_ERR_LAUNCH, "hipFuncSetAttribute(blockdiag_wide): %s", hipGetErrorString(e));
  dim3 grid(((M + kWideBM - 1) / kWideBM) * (nb * q / kWideBN));
  hipLaunchKernelGGL(kern, grid, dim3(512), lds, stream, (const uint16_t*)x, (const uint16_t*)w, bias,
                     (const uint16_t*)resid, (OUT*)out, M, nb, p, q);
  return check_launch("blockdiag_wide");
}

// LayerNorm over the last dimension of x (M, d) fp32, eps inside the square root.
// Workgroup = 8 waves handles R = 8 RW rows; each wave normalises RW rows at once (all loads in flight
// together) and writes the row-major outputs from registers.  For the channel-major output the
// normalised rows also go through an LDS tile, 384 columns at a time (row pitch 386 floats, so that 32
// consecutive tokens of two neighbouring channels fall in 64 different banks; 49 KB, so that three
// workgroups share a compute unit and one's loads overlap another's stores), and are written back with
// lanes along the token axis: every store instruction covers R consecutive tokens of 64 / R channels.
// The input is read once.  PER = d / 64 values per lane.
template <int PER>
struct LnShape {
  static constexpr int RW = PER <= 16 ? 4 : 2;      // rows in flight per wave (register budget)
  static constexpr int R = 8 * RW;                  // rows per workgroup: 32 or 16
  static constexpr int PC = PER < 6 ? PER : 6;      // 64-column groups per tile pass
  static constexpr int NPASS = (PER + PC - 1) / PC;
  static constexpr int PITCH = 64 * PC + 2;
  static constexpr size_t LDS_BYTES = (size_t)R * PITCH * sizeof(float);
};
// Where the rows come from when the kernel normalises embeddings instead of a matrix:
// row m = word[ids[m]] + type[tt[m] or 0] (+ pos[pos_ids[m] or m % L]).
// Every index is clamped into its table before it is used, so a bad id reads a valid row instead of
// foreign memory; when that happens and `bad_index` is not null the kernel stores 1 there (plain vector
// store; the caller cleared it before the launch and reads it afterwards to report the error).
struct EmbedSource {
  const long long* ids;     // (M)
  const long long* tt;      // (M) or null: type 0
  const long long* pos_ids; // (M) or null: m % L
  const float* word;        // (vocab, d)
  const float* type;        // (type_vocab, d)
  const float* pos;         // (max_positions, d) or null: no position embeddings
  int L;
  int vocab, type_vocab, max_positions;      // rows of the three tables
  int* bad_index;           // or null
};
__device__ __forceinline__ long long clamp_index(long long i, int rows, bool& bad) {
  if (i < 0 || i >= rows) {
    bad = true;
    return i < 0 ? 0 : rows - 1;
  }
  return i;
}
// IN: float, or uint16_t for rows stored as bf16 (the sum the reference's autocast path feeds its LayerNorm).
template <int PER, bool EMBED, typename IN = float>
__global__ __launch_bounds__(512) void layernorm_kernel(const IN* __restrict__ x, EmbedSource src,
                                                        const float* __restrict__ gamma,
                                                        const float* __restrict__ beta, float eps,
                                                        float* __restrict__ out_f32,       // (M, d) or null
                                                        uint16_t* __restrict__ out_bf16,   // (M, d) or null
                                                        float* __restrict__ out_t,         // (d, M) or null
                                                        int M) {
  constexpr int d = 64 * PER, RW = LnShape<PER>::RW, R = LnShape<PER>::R, PITCH = LnShape<PER>::PITCH;
  constexpr int PC = LnShape<PER>::PC, NPASS = LnShape<PER>::NPASS;
  extern __shared__ float tile[];                       // [R][PITCH], used only with out_t
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int m0 = blockIdx.x * R;
  float g[PER], bt[PER];
  static_for<0, PER>([&](auto ii) {
    g[decltype(ii)::value] = gamma[lane + 64 * decltype(ii)::value];
    bt[decltype(ii)::value] = beta[lane + 64 * decltype(ii)::value];
  });
  float v[RW][PER];
  float sum[RW], sq[RW];
  static_for<0, RW>([&](auto rr_) {
    constexpr int rr = decltype(rr_)::value;
    int m = m0 + wave * RW + rr;
    m = m < M ? m : M - 1;
    if constexpr (!EMBED) {
      const IN* xr = x + (long)m * d;
      static_for<0, PER>([&](auto ii) {
        if constexpr (sizeof(IN) == 2) v[rr][decltype(ii)::value] = bf16_to_f32(xr[lane + 64 * decltype(ii)::value]);
        else v[rr][decltype(ii)::value] = xr[lane + 64 * decltype(ii)::value];
      });
    } else {
      bool bad = false;
      const float* wr = src.word + clamp_index(src.ids[m], src.vocab, bad) * d;
      const float* tr = src.type + (src.tt ? clamp_index(src.tt[m], src.type_vocab, bad) : 0) * d;
      static_for<0, PER>([&](auto ii) {
        constexpr int i = decltype(ii)::value;
        v[rr][i] = wr[lane + 64 * i] + tr[lane + 64 * i];
      });
      if (src.pos) {
        const float* pr = src.pos + (src.pos_ids ? clamp_index(src.pos_ids[m], src.max_positions, bad)
                                                 : (long long)(m % src.L)) * d;
        static_for<0, PER>([&](auto ii) {
          constexpr int i = decltype(ii)::value;
          v[rr][i] += pr[lane + 64 * i];
        });
      }
      if (bad && src.bad_index && lane == 0) *src.bad_index = 1;
    }
  });
  static_for<0, RW>([&](auto rr_) {
    constexpr int rr = decltype(rr_)::value;
    float s = 0.f;
    static_for<0, PER>([&](auto ii) { s += v[rr][decltype(ii)::value]; });
    sum[rr] = s;
  });
  for (int o = 32; o > 0; o >>= 1)
    static_for<0, RW>([&](auto rr_) { sum[decltype(rr_)::value] += __shfl_xor(sum[decltype(rr_)::value], o); });
  static_for<0, RW>([&](auto rr_) {
    constexpr int rr = decltype(rr_)::value;
    sum[rr] *= (1.0f / (float)d);
    float s = 0.f;
    static_for<0, PER>([&](auto ii) {
      const float c = v[rr][decltype(ii)::value] - sum[rr];
      s += c * c;
    });
    sq[rr] = s;
  });
  for (int o = 32; o > 0; o >>= 1)
    static_for<0, RW>([&](auto rr_) { sq[decltype(rr_)::value] += __shfl_xor(sq[decltype(rr_)::value], o); });
  static_for<0, RW>([&](auto rr_) {
    constexpr int rr = decltype(rr_)::value;
    const int m = m0 + wave * RW + rr;
    const float mean = sum[rr];
    const float rstd = rsqrtf(sq[rr] * (1.0f / (float)d) + eps);
    static_for<0, PER>([&](auto ii) {
      constexpr int i = decltype(ii)::value;
      v[rr][i] = (v[rr][i] - mean) * rstd * g[i] + bt[i];
      if (m < M) {
        if (out_f32) out_f32[(long)m * d + lane + 64 * i] = v[rr][i];
        if (out_bf16) out_bf16[(long)m * d + lane + 64 * i] = f32_to_bf16(v[rr][i]);
      }
    });
  });
  if (!out_t) return;
  // lane = (token tk, channel offset h): R tokens x (64 / R) channels per store instruction
  constexpr int CH = 64 / R;
  const int tk = lane % R, h = lane / R;
  const int mt = m0 + tk;
  static_for<0, NPASS>([&](auto pp) {
    constexpr int ps = decltype(pp)::value;
    constexpr int i0 = ps * PC, i1 = (i0 + PC < PER) ? i0 + PC : PER;      // 64-column groups of this pass
    if (ps > 0) __syncthreads();                                            // the previous pass has been read
    static_for<0, RW>([&](auto rr_) {
      constexpr int rr = decltype(rr_)::value;
      static_for<i0, i1>([&](auto ii) {
        constexpr int i = decltype(ii)::value;
        tile[(wave * RW + rr) * PITCH + lane + 64 * (i - i0)] = v[rr][i];
      });
    });
    __syncthreads();
    if (mt < M) {
      const float* src = tile + tk * PITCH + h;
      float* dst = out_t + (long)(64 * i0 + h) * M + mt;
#pragma unroll 4
      for (int c0 = wave * CH; c0 < 64 * (i1 - i0); c0 += 8 * CH) dst[(long)c0 * M] = src[c0];
    }
  });
}

// ---------------------------------------------------------------------------------------------
// Weight-stationary GLU kernel for short K (p = in_features / nblocks <= 256).
//
// With K = p as small as 192 a tiled GEMM spends its time filling and draining tiles.  Here a
// workgroup owns 128 output columns for a long run of rows: wave w keeps, for its 32 columns, the weight
// rows of BOTH GEMMs (gate block and value block) in registers for the whole run (2 x KS MFMA B
// operands), so the gate and the value of an output element meet in the same lane and gelu(gate) * value
// is applied on the accumulators.  The workgroup streams 32-row slabs of x (the K ranges of the two
// blocks) through a double-buffered LDS tile (the slab after next is in flight in registers during the
// MFMAs) and the bf16 results go through a small double-buffered LDS tile so that every global store is a
// full 256-byte row segment, written while the next slab is being multiplied.  One barrier per slab.
// ---------------------------------------------------------------------------------------------
template <int KS>        // K steps of 16: p = 16 KS
__global__ __launch_bounds__(256) void blockdiag_glu_ws_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ w,
                                                               uint16_t* __restrict__ out, int M, int nb, int q,
                                                               int rows_per_wg) {
  constexpr int p = 16 * KS;
  constexpr int AROW = p + 8;                       // padded bf16 row of an A slab
  constexpr int GROW = 128 + 8;                     // padded bf16 row of the result tile
  constexpr int CPR = 2 * (p / 8);                  // 16-byte chunks per slab row (gate K-range then value K-range)
  constexpr int NCH = 32 * CPR / 256;               // chunks per thread per slab
  constexpr int ABUF = 2 * 32 * AROW;               // bf16 elements of one A buffer
  static_assert((32 * CPR) % 256 == 0, "slab must divide over 256 threads");
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  uint16_t* sA = smem;                              // [2][2][32][AROW]
  uint16_t* sG = smem + 2 * ABUF;                   // [2][32][GROW]
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, i32 = lane & 31, half = lane >> 5;
  const int I = nb * q / 2, in_f = nb * p;
  const int nslices = I / 128;
  // XCD-aware order: XCD e takes row chunks e, e+8, ... and walks all column slices of one chunk back to back
  int slice, chunk;
  {
    const int nchunks = (M + rows_per_wg - 1) / rows_per_wg;
    const int id = blockIdx.x, e = id & 7, l = id >> 3;
    const int full = (nchunks / 8) * 8;
    if (id < full * nslices) { chunk = (l / nslices) * 8 + e; slice = l % nslices; }
    else { const int rid = id - full * nslices; chunk = full + rid / nslices; slice = rid % nslices; }
  }
  const int n0 = slice * 128;                        // first output column
  const int blk = n0 / q, jj = n0 % q;               // gate block and first weight row in it
  const int m_begin = chunk * rows_per_wg;
  const int m_end = min(M, m_begin + rows_per_wg);

  // stationary B operands: weight rows jj + 32 wave + i32 of block blk (gate) and blk + nb/2 (value),
  // K = 16 ks + 8 half + {0..7}
  bf16x8 bwg[KS], bwv[KS];
  {
    const uint16_t* wg = w + ((long)blk * q + jj + 32 * wave + i32) * p + 8 * half;
    const uint16_t* wv = wg + (long)(nb / 2) * q * p;
    static_for<0, KS>([&](auto kk) {
      bwg[decltype(kk)::value] = ld8(wg + 16 * decltype(kk)::value);
      bwv[decltype(kk)::value] = ld8(wv + 16 * decltype(kk)::value);
    });
  }
  // per-thread chunk coordinates inside a slab
  int crow[NCH], ccol[NCH], clds[NCH];
  static_for<0, NCH>([&](auto jj_) {
    constexpr int j = decltype(jj_)::value;
    const int id = tid + 256 * j, r = id / CPR, c = id % CPR, m2 = c / (p / 8), kc = c % (p / 8);
    crow[j] = r;
    ccol[j] = (blk + m2 * (nb / 2)) * p + kc * 8;
    clds[j] = (m2 * 32 + r) * AROW + kc * 8;
  });
  u32x4 ra[NCH];
  auto gload = [&](int m0) __attribute__((always_inline)) {
    static_for<0, NCH>([&](auto jj_) {
      constexpr int j = decltype(jj_)::value;
      int row = m0 + crow[j];
      row = row < M ? row : M - 1;
      ra[j] = *reinterpret_cast<const u32x4*>(x + (long)row * in_f + ccol[j]);
    });
  };
  auto sstore = [&](int buf) __attribute__((always_inline)) {
    static_for<0, NCH>([&](auto jj_) {
      *reinterpret_cast<u32x4*>(sA + buf * ABUF + clds[decltype(jj_)::value]) = ra[decltype(jj_)::value];
    });
  };
  // result tile -> global: 32 rows x 256 bytes, two 16-byte pieces per thread
  auto store_tile = [&](int buf, int m0) __attribute__((always_inline)) {
    static_for<0, 2>([&](auto jj_) {
      const int id = tid + 256 * decltype(jj_)::value, r = id >> 4, c = id & 15;
      const u32x4 v = *reinterpret_cast<const u32x4*>(sG + (buf * 32 + r) * GROW + 8 * c);
      if (m0 + r < M) *reinterpret_cast<u32x4*>(out + (long)(m0 + r) * I + n0 + 8 * c) = v;
    });
  };

  gload(m_begin);
  sstore(0);
  if (m_begin + 32 < m_end) gload(m_begin + 32);
  int s = 0;
  for (int m0 = m_begin; m0 < m_end; m0 += 32, ++s) {
    __syncthreads();      // slab s is in sA[s & 1]; result tile s - 1 is complete; buffers of s - 1 are free
    if (s > 0) store_tile((s - 1) & 1, m0 - 32);
    const uint16_t* ag = sA + (s & 1) * ABUF + i32 * AROW + 8 * half;
    const uint16_t* av = ag + 32 * AROW;
    floatx16 accg, accv;
    static_for<0, 16>([&](auto vv) { accg[decltype(vv)::value] = 0.f; accv[decltype(vv)::value] = 0.f; });
    static_for<0, KS>([&](auto kk) {
      constexpr int ks = decltype(kk)::value;
      accg = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ld8(ag + 16 * ks), bwg[ks], accg, 0, 0, 0);
      accv = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ld8(av + 16 * ks), bwv[ks], accv, 0, 0, 0);
    });
    if (m0 + 32 < m_end) {
      sstore((s + 1) & 1);                     // that buffer was last read before this slab's barrier
      if (m0 + 64 < m_end) gload(m0 + 64);
    }
    // accumulator element v: row 8 (v / 4) + 4 half + v % 4, column 32 wave + i32
    uint16_t* gt = sG + ((s & 1) * 32 + 4 * half) * GROW + 32 * wave + i32;
    static_for<0, 8>([&](auto vv) {
      constexpr int v = 2 * decltype(vv)::value;
      const uint32_t pk = pack_bf16x2(gelu_erf(accg[v]) * accv[v], gelu_erf(accg[v + 1]) * accv[v + 1]);
      gt[(8 * (v >> 2) + (v & 3)) * GROW] = (uint16_t)pk;
      gt[(8 * (v >> 2) + (v & 3) + 1) * GROW] = (uint16_t)(pk >> 16);
    });
  }
  __syncthreads();
  store_tile((s - 1) & 1, m_begin + 32 * (s - 1));
}

// The same kernel software-pipelined inside every wave: two accumulator sets, and the MFMAs of slab s + 1
// sit in the same basic block as the gelu(gate) * value epilogue of slab s, so that the vector ALU works in the
// shadow of the matrix pipe (the epilogue costs more vector-ALU cycles than the product costs MFMA cycles, and
// with one accumulator set the two were measured to run one after the other).
// NW waves per workgroup, 32 NW output columns: every column slice reads all of x again (from L2), so wider
// workgroups cut that traffic.
template <int KS, int NW>
__global__ __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(2, 2))) void blockdiag_glu_ws3_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ w,
                                                                uint16_t* __restrict__ out, int M, int nb, int q,
                                                                int rows_per_wg) {
  constexpr int p = 16 * KS;
  constexpr int AROW = p + 8;                       // padded bf16 row of an A slab
  constexpr int NT = 64 * NW, NC = 32 * NW;         // threads, output columns
  constexpr int GROW = NC + 8;                      // padded bf16 row of the result tile
  constexpr int CPR = 2 * (p / 8);                  // 16-byte chunks per slab row (gate K-range then value K-range)
  constexpr int NCH = 32 * CPR / NT;                // chunks per thread per slab
  constexpr int ABUF = 2 * 32 * AROW;               // bf16 elements of one A buffer
  static_assert((32 * CPR) % NT == 0, "slab must divide over the threads");
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  uint16_t* sA = smem;                              // [2][2][32][AROW]
  // a separate object, so that the compiler may move the epilogue's writes past the product's operand reads
  __shared__ __attribute__((aligned(16))) uint16_t sG[2 * 32 * GROW];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, i32 = lane & 31, half = lane >> 5;
  const int I = nb * q / 2, in_f = nb * p;
  const int nslices = I / NC;
  int slice, chunk;
  {
    const int nchunks = (M + rows_per_wg - 1) / rows_per_wg;
    const int id = blockIdx.x, e = id & 7, l = id >> 3;
    const int full = (nchunks / 8) * 8;
    if (id < full * nslices) { chunk = (l / nslices) * 8 + e; slice = l % nslices; }
    else { const int rid = id - full * nslices; chunk = full + rid / nslices; slice = rid % nslices; }
  }
  const int n0 = slice * NC;
  const int blk = n0 / q, jj = n0 % q;
  const int m_begin = chunk * rows_per_wg;
  const int m_end = min(M, m_begin + rows_per_wg);
  const int nslab = (m_end - m_begin + 31) / 32;

  bf16x8 bwg[KS], bwv[KS];
  {
    const uint16_t* wg = w + ((long)blk * q + jj + 32 * wave + i32) * p + 8 * half;
    const uint16_t* wv = wg + (long)(nb / 2) * q * p;
    static_for<0, KS>([&](auto kk) {
      bwg[decltype(kk)::value] = ld8(wg + 16 * decltype(kk)::value);
      bwv[decltype(kk)::value] = ld8(wv + 16 * decltype(kk)::value);
    });
  }
  int crow[NCH], ccol[NCH], clds[NCH];
  static_for<0, NCH>([&](auto jj_) {
    constexpr int j = decltype(jj_)::value;
    const int id = tid + NT * j, r = id / CPR, c = id % CPR, m2 = c / (p / 8), kc = c % (p / 8);
    crow[j] = r;
    ccol[j] = (blk + m2 * (nb / 2)) * p + kc * 8;
    clds[j] = (m2 * 32 + r) * AROW + kc * 8;
  });
  u32x4 ra[NCH];
  auto gload = [&](int m0) __attribute__((always_inline)) {
    static_for<0, NCH>([&](auto jj_) {
      constexpr int j = decltype(jj_)::value;
      int row = m0 + crow[j];
      row = row < M ? row : M - 1;
      ra[j] = *reinterpret_cast<const u32x4*>(x + (long)row * in_f + ccol[j]);
    });
  };
  auto sstore = [&](int buf) __attribute__((always_inline)) {
    static_for<0, NCH>([&](auto jj_) {
      *reinterpret_cast<u32x4*>(sA + buf * ABUF + clds[decltype(jj_)::value]) = ra[decltype(jj_)::value];
    });
  };
  auto store_tile = [&](int buf, int m0) __attribute__((always_inline)) {
    static_for<0, 32 * (NC / 8) / NT>([&](auto jj_) {       // 32 rows x NC / 8 pieces of 16 bytes
      const int id = tid + NT * decltype(jj_)::value, r = id / (NC / 8), c = id % (NC / 8);
      const u32x4 v = *reinterpret_cast<const u32x4*>(sG + (buf * 32 + r) * GROW + 8 * c);
      if (m0 + r < M) *reinterpret_cast<u32x4*>(out + (long)(m0 + r) * I + n0 + 8 * c) = v;
    });
  };
  auto product = [&](int buf, floatx16& accg, floatx16& accv) __attribute__((always_inline)) {
    const uint16_t* ag = sA + buf * ABUF + i32 * AROW + 8 * half;
    const uint16_t* av = ag + 32 * AROW;
    static_for<0, 16>([&](auto vv) { accg[decltype(vv)::value] = 0.f; accv[decltype(vv)::value] = 0.f; });
    static_for<0, KS>([&](auto kk) {
      constexpr int ks = decltype(kk)::value;
      accg = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ld8(ag + 16 * ks), bwg[ks], accg, 0, 0, 0);
      accv = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ld8(av + 16 * ks), bwv[ks], accv, 0, 0, 0);
    });
  };
  // accumulator element v: row 8 (v / 4) + 4 half + v % 4, column 32 wave + i32
  auto epilogue = [&](int buf, const floatx16& accg, const floatx16& accv) __attribute__((always_inline)) {
    uint16_t* gt = sG + (buf * 32 + 4 * half) * GROW + 32 * wave + i32;
    static_for<0, 8>([&](auto vv) {
      constexpr int v = 2 * decltype(vv)::value;
      const uint32_t pk = pack_bf16x2(gelu_erf(accg[v]) * accv[v], gelu_erf(accg[v + 1]) * accv[v + 1]);
      gt[(8 * (v >> 2) + (v & 3)) * GROW] = (uint16_t)pk;
      gt[(8 * (v >> 2) + (v & 3) + 1) * GROW] = (uint16_t)(pk >> 16);
    });
  };

  floatx16 g0, v0, g1, v1;
  gload(m_begin);
  sstore(0);
  if (nslab > 1) gload(m_begin + 32);
  __syncthreads();
  product(0, g0, v0);
  if (nslab > 1) {
    sstore(1);
    if (nslab > 2) gload(m_begin + 64);
  }
  // step s: the product of slab s + 1 and the epilogue of slab s in one basic block; tile s - 1 goes to global memory
  auto step = [&](int s, floatx16& ga, floatx16& va, floatx16& gb, floatx16& vb) __attribute__((always_inline)) {
    __syncthreads();      // slab s + 1 is in sA[(s + 1) & 1]; tile s - 1 is complete in sG[(s - 1) & 1]
    if (s > 0) store_tile((s - 1) & 1, m_begin + 32 * (s - 1));
    product((s + 1) & 1, gb, vb);
    epilogue(s & 1, ga, va);
    // issue order inside this block: one MFMA, its next operand read, then a share of the epilogue's vector ALU
    // work (about 8 instructions per MFMA) and LDS writes, so that the two pipes run side by side
    __builtin_amdgcn_sched_group_barrier(0x100, 6, 0);      // operand reads run six MFMAs ahead
    static_for<0, 2 * KS>([&](auto) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, (184 + 2 * KS - 1) / (2 * KS), 0);
      __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
    });
    if (s + 2 < nslab) {
      sstore(s & 1);                           // last read by the product of slab s, before this step's barrier
      if (s + 3 < nslab) gload(m_begin + 32 * (s + 3));
    }
  };
  auto last_step = [&](int s, floatx16& ga, floatx16& va) __attribute__((always_inline)) {
    __syncthreads();
    if (s > 0) store_tile((s - 1) & 1, m_begin + 32 * (s - 1));
    epilogue(s & 1, ga, va);
  };
  int s = 0;
  for (; s + 2 < nslab; s += 2) {
    step(s, g0, v0, g1, v1);
    step(s + 1, g1, v1, g0, v0);
  }
  if (s + 1 < nslab) {
    step(s, g0, v0, g1, v1);
    last_step(s + 1, g1, v1);
  } else {
    last_step(s, g0, v0);
  }
  __syncthreads();
  store_tile((nslab - 1) & 1, m_begin + 32 * (nslab - 1));
}

// ---------------------------------------------------------------------------------------------
// fp32 block-diagonal multiply: what the reference computes when it is called with fp32 tensors outside CUDA autocast
// (bert/src/mm/blockdiag_multiply.py:50 casts to bf16 only under autocast).  v_mfma_f32_32x32x2_f32 (exact fp32
// products, fp32 accumulation); a wave owns a 32 x 32 output tile and reads both operands straight from global
// memory in operand layout: lane (i, h) takes 4 consecutive K values of x row i and of weight row i per step, which
// feed four MFMAs (MFMA j of a step contracts K = 8 s + j from the lanes h = 0 and K = 8 s + 4 + j from h = 1).
// Not a hot path of the encoder (that runs under autocast): no LDS tiling.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void blockdiag_f32_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                            const float* __restrict__ bias, float* __restrict__ out,
                                                            int M, int nb, int p, int q) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, i32 = lane & 31, half = lane >> 5;
  const int tiles_n = (q + 31) / 32;                       // column tiles per block
  const int tile = blockIdx.x * 4 + wave;                  // over (row tile, block, column tile)
  const int ntiles = ((M + 31) / 32) * nb * tiles_n;
  if (tile >= ntiles) return;
  const int tn = tile % tiles_n, blk = (tile / tiles_n) % nb, tm = tile / (tiles_n * nb);
  int row = tm * 32 + i32, col = tn * 32 + i32;
  const bool col_ok = col < q;
  row = row < M ? row : M - 1;
  col = col_ok ? col : q - 1;
  const float* xr = x + (long)row * nb * p + (long)blk * p + 4 * half;
  const float* wr = w + ((long)blk * q + col) * p + 4 * half;
  floatx16 acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.f;
  for (int k = 0; k < p; k += 8) {
    const float4 a = *reinterpret_cast<const float4*>(xr + k);
    const float4 b = *reinterpret_cast<const float4*>(wr + k);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, b.x, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, b.y, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.z, b.z, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.w, b.w, acc, 0, 0, 0);
  }
  // accumulator element v: x row 8 (v / 4) + 4 half + v % 4 of the tile, output column i32
  if (!col_ok) return;
  const int oc = blk * q + tn * 32 + i32;
  const float bv = bias ? bias[oc] : 0.f;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int r = tm * 32 + 8 * (v >> 2) + 4 * half + (v & 3);
    if (r < M) out[(long)r * nb * q + oc] = acc[v] + bv;
  }
}

template <int KS>
static int launch_glu_ws(const void* x, const void* w, void* out, int M, int nb, int q, hipStream_t stream) {
  constexpr int p = 16 * KS;
  constexpr bool PIPELINED = KS <= 12;      // beyond that the second accumulator set does not fit the registers
  const int I = nb * q / 2;
  constexpr int NW = PIPELINED ? 8 : 4;
  const bool wide = PIPELINED && q % (32 * NW) == 0;
  const int ncols = wide ? 32 * NW : 128;
  // dynamic LDS: the A slabs, and for the plain kernel the result tiles too (the pipelined one declares them itself)
  const size_t lds = ((size_t)2 * 2 * 32 * (p + 8) + (PIPELINED ? 0 : (size_t)2 * 32 * (128 + 8))) * sizeof(uint16_t);
  auto kern = !PIPELINED ? blockdiag_glu_ws_kernel<KS> : wide ? blockdiag_glu_ws3_kernel<KS, NW> : blockdiag_glu_ws3_kernel<KS, 4>;
  if (lds > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return set_error(M2_ERR_LAUNCH, "hipFuncSetAttribute(blockdiag_glu_ws): %s", hipGetErrorString(e));
  }
  const int nslices = I / ncols;
  // Rows per workgroup (a multiple of the 32-row slab): long runs amortise the weight load and the first slab's
  // latency (worth about three slab steps), but the workgroups should fill the chip in whole rounds.  Cost model:
  // rounds x (3 + slabs per workgroup), minimised over the candidates.
  const long slots = (long)num_cus() * (wide || !PIPELINED ? 1 : 2);
  int rows = 512;
  long best = -1;
  for (int cand = 64; cand <= 4096; cand += 32) {
    const long wgs = (long)nslices * ((M + cand - 1) / cand);
    const long cost = ((wgs + slots - 1) / slots) * (3 + cand / 32);
    if (best < 0 || cost < best) { best = cost; rows = cand; }
  }
  const int nchunks = (M + rows - 1) / rows;
  hipLaunchKernelGGL(kern, dim3(nslices * nchunks), dim3(wide ? 64 * NW : 256), lds, stream, (const uint16_t*)x,
                     (const uint16_t*)w, (uint16_t*)out, M, nb, q, rows);
  return check_launch("blockdiag_glu_ws");
}

}  // namespace m2

using namespace m2;

static int check_blockdiag(const char* who, int M, int nb, int p, int q, bool glu) {
  if (M <= 0 || nb <= 0 || p <= 0 || q <= 0) return set_error(M2_ERR_ARG, "%s: sizes must be positive (M=%d nb=%d p=%d q=%d)", who, M, nb, p, q);
  if (p % 8 != 0) return set_error(M2_ERR_UNSUPPORTED, "%s: in_features/nblocks=%d must be a multiple of 8", who, p);
  if (q % 8 != 0) return set_error(M2_ERR_UNSUPPORTED, "%s: out_features/nblocks=%d must be a multiple of 8", who, q);
  if (glu && nb % 2 != 0) return set_error(M2_ERR_UNSUPPORTED, "%s: GLU pairing needs an even number of blocks, got %d", who, nb);
  return M2_OK;
}

extern "C" int m2_blockdiag_glu_fwd(const void* x, const void* w, void* out, int M, int in_features,
                                    int intermediate, int nblocks, void* stream) {
  if (!x || !w || !out) return set_error(M2_ERR_ARG, "m2_blockdiag_glu_fwd: null pointer");
  if (nblocks <= 0 || in_features % nblocks || (2 * intermediate) % nblocks)
    return set_error(M2_ERR_UNSUPPORTED, "m2_blockdiag_glu_fwd: in=%d and 2*intermediate=%d must divide by nblocks=%d",
                     in_features, 2 * intermediate, nblocks);
  const int p = in_features / nblocks, q = 2 * intermediate / nblocks;
  int rc = check_blockdiag("m2_blockdiag_glu_fwd", M, nblocks, p, q, true);
  if (rc) return rc;
  if (p % 64 != 0 || q % 64 != 0) {               // block sizes off the tile grid (d = 960: 240-wide blocks): the masked kernel
    hipStream_t st = (hipStream_t)stream;
    return q >= 128 ? launch_blockdiag<2, 2, true, uint16_t, 2, true>(x, w, nullptr, nullptr, out, M, nblocks, p, q, intermediate, st)
                    : launch_blockdiag<4, 1, true, uint16_t, 2, true>(x, w, nullptr, nullptr, out, M, nblocks, p, q, intermediate, st);
  }
  if (q % 128 == 0 && p <= 256) {                 // short K: weight-stationary kernel
    hipStream_t st = (hipStream_t)stream;
    switch (p / 16) {
      case 4: return launch_glu_ws<4>(x, w, out, M, nblocks, q, st);
      case 8: return launch_glu_ws<8>(x, w, out, M, nblocks, q, st);
      case 12: return launch_glu_ws<12>(x, w, out, M, nblocks, q, st);
      case 16: return launch_glu_ws<16>(x, w, out, M, nblocks, q, st);
      default: break;
    }
  }
  if (q % 128 == 0) {
    // 256 x 128 tiles (eight waves) once they fill the chip twice over: 3 % faster than 128 x 128 at M = 8192,
    // d = 1536 (118 - 123 against 122 - 126 us), the same results bit for bit
    if ((long)((M + 255) / 256) * (intermediate / 128) >= 2L * num_cus())
      return launch_blockdiag<4, 2, true, uint16_t, 2>(x, w, nullptr, nullptr, out, M, nblocks, p, q, intermediate, (hipStream_t)stream);
    return launch_blockdiag<2, 2, true, uint16_t, 2>(x, w, nullptr, nullptr, out, M, nblocks, p, q, intermediate, (hipStream_t)stream);
  }
  return launch_blockdiag<4, 1, true, uint16_t, 2>(x, w, nullptr, nullptr, out, M, nblocks, p, q, intermediate, (hipStream_t)stream);
}

extern "C" int m2_blockdiag_linear_fwd(const void* x, const void* w, const float* bias, const void* residual,
                                       void* out, int M, int in_features, int out_features, int nblocks,
                                       int out_dtype, void* stream) {
  if (!x || !w || !out) return set_error(M2_ERR_ARG, "m2_blockdiag_linear_fwd: null pointer");
  if (nblocks <= 0 || in_features % nblocks || out_features % nblocks)
    return set_error(M2_ERR_UNSUPPORTED, "m2_blockdiag_linear_fwd: in=%d and out=%d must divide by nblocks=%d",
                     in_features, out_features, nblocks);
  if (out_dtype != M2_DTYPE_F32 && out_dtype != M2_DTYPE_BF16)
    return set_error(M2_ERR_ARG, "m2_blockdiag_linear_fwd: out_dtype %d is neither M2_DTYPE_F32 nor M2_DTYPE_BF16", out_dtype);
  const int p = in_features / nblocks, q = out_features / nblocks;
  int rc = check_blockdiag("m2_blockdiag_linear_fwd", M, nblocks, p, q, false);
  if (rc) return rc;
  hipStream_t st = (hipStream_t)stream;
  if (p % 64 != 0 || q % 64 != 0) {               // block sizes off the tile grid: the masked kernel
    if (out_dtype == M2_DTYPE_F32)
      return q >= 128 ? launch_blockdiag<2, 2, false, float, 1, true>(x, w, bias, residual, out, M, nblocks, p, q, out_features, st)
                      : launch_blockdiag<4, 1, false, float, 1, true>(x, w, bias, residual, out, M, nblocks, p, q, out_features, st);
    return q >= 128 ? launch_blockdiag<2, 2, false, uint16_t, 1, true>(x, w, bias, residual, out, M, nblocks, p, q, out_features, st)
                    : launch_blockdiag<4, 1, false, uint16_t, 1, true>(x, w, bias, residual, out, M, nblocks, p, q, out_features, st);
  }
  // 256 x 192 tiles once there is at least one per compute unit (measured at d = 768 and 1536: below that the
  // smaller tiles of the general kernel fill the chip better)
  if (q % kWideBN == 0 && (long)((M + kWideBM - 1) / kWideBM) * (nblocks * q / kWideBN) >= num_cus())
    return out_dtype == M2_DTYPE_F32 ? launch_blockdiag_wide<float>(x, w, bias, residual, out, M, nblocks, p, q, st)
                                     : launch_blockdiag_wide<uint16_t>(x, w, bias, residual, out, M, nblocks, p, q, st);
  const bool wide = q % 128 == 0;
  if (out_dtype == M2_DTYPE_F32)
    return wide ? launch_blockdiag<2, 2, false, float, 1>(x, w, bias, residual, out, M, nblocks, p, q, out_features, st)
                : launch_blockdiag<4, 1, false, float, 1>(x, w, bias, residual, out, M, nblocks, p, q, out_features, st);
  return wide ? launch_blockdiag<2, 2, false, uint16_t, 1>(x, w, bias, residual, out, M, nblocks, p, q, out_features, st)
              : launch_blockdiag<4, 1, false, uint16_t, 1>(x, w, bias, residual, out, M, nblocks, p, q, out_features, st);
}

extern "C" int m2_blockdiag_linear_f32_fwd(const float* x, const float* w, const float* bias, float* out, int M,
                                           int in_features, int out_features, int nblocks, void* stream) {
  if (!x || !w || !out) return set_error(M2_ERR_ARG, "m2_blockdiag_linear_f32_fwd: null pointer");
  if (M <= 0 || nblocks <= 0 || in_features <= 0 || out_features <= 0 || in_features % nblocks || out_features % nblocks)
    return set_error(M2_ERR_UNSUPPORTED, "m2_blockdiag_linear_f32_fwd: in=%d and out=%d must be positive multiples of nblocks=%d",
                     in_features, out_features, nblocks);
  const int p = in_features / nblocks, q = out_features / nblocks;
  if (p % 8 != 0) return set_error(M2_ERR_UNSUPPORTED, "m2_blockdiag_linear_f32_fwd: in_features/nblocks=%d must be a multiple of 8", p);
  const long ntiles = (long)((M + 31) / 32) * nblocks * ((q + 31) / 32);
  if ((ntiles + 3) / 4 > 0x7fffffffL) return set_error(M2_ERR_UNSUPPORTED, "m2_blockdiag_linear_f32_fwd: too many tiles");
  hipLaunchKernelGGL(blockdiag_f32_kernel, dim3((unsigned)((ntiles + 3) / 4)), dim3(256), 0, (hipStream_t)stream, x, w, bias,
                     out, M, nblocks, p, q);
  return check_launch("blockdiag_f32");
}

template <bool EMBED, typename IN = float>
static int launch_layernorm(const IN* x, const EmbedSource& src, const float* gamma, const float* beta, float eps,
                            float* out_f32, void* out_bf16, float* out_channel_major, int M, int d, void* stream) {
  hipStream_t st = (hipStream_t)stream;
  uint16_t* o16 = (uint16_t*)out_bf16;
  switch (d / 64) {
#define LN_CASE(P)                                                                                                      \
  case P: {                                                                                                             \
    const size_t lds = out_channel_major ? LnShape<P>::LDS_BYTES : 0;                                                   \
    auto kern = layernorm_kernel<P, EMBED, IN>;                                                                           \
    if (lds > 64 * 1024) {                                                                                              \
      hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);     \
      if (e != hipSuccess) return set_error(M2_ERR_LAUNCH, "hipFuncSetAttribute(layernorm): %s", hipGetErrorString(e)); \
    }                                                                                                                   \
    hipLaunchKernelGGL(kern, dim3((M + LnShape<P>::R - 1) / LnShape<P>::R), dim3(512), lds, st, x, src, gamma, beta,   \
                       eps, out_f32, o16, out_channel_major, M);                                                        \
    break;                                                                                                              \
  }
    LN_CASE(1) LN_CASE(2) LN_CASE(3) LN_CASE(4) LN_CASE(5) LN_CASE(6) LN_CASE(7) LN_CASE(8) LN_CASE(9) LN_CASE(10) LN_CASE(11)
    LN_CASE(12) LN_CASE(13) LN_CASE(14) LN_CASE(15) LN_CASE(16) LN_CASE(17) LN_CASE(18) LN_CASE(19) LN_CASE(20) LN_CASE(21)
    LN_CASE(22) LN_CASE(23) LN_CASE(24) LN_CASE(25) LN_CASE(26) LN_CASE(27) LN_CASE(28) LN_CASE(29) LN_CASE(30) LN_CASE(31)
    LN_CASE(32)
#undef LN_CASE
  }
  return check_launch("layernorm");
}

extern "C" int m2_layernorm_fwd(const float* x, const float* gamma, const float* beta, float eps, float* out_f32,
                                void* out_bf16, float* out_channel_major, int M, int d, void* stream) {
  if (!x || !gamma || !beta) return set_error(M2_ERR_ARG, "m2_layernorm_fwd: null pointer");
  if (M <= 0 || d <= 0 || d % 64 != 0 || d > 2048)
    return set_error(M2_ERR_UNSUPPORTED, "m2_layernorm_fwd: need M > 0 and d a multiple of 64 up to 2048 (M=%d d=%d)", M, d);
  return launch_layernorm<false>(x, EmbedSource{}, gamma, beta, eps, out_f32, out_bf16, out_channel_major, M, d, stream);
}

extern "C" int m2_layernorm_bf16_fwd(const void* x, const float* gamma, const float* beta, float eps, float* out_f32,
                                     void* out_bf16, float* out_channel_major, int M, int d, void* stream) {
  if (!x || !gamma || !beta) return set_error(M2_ERR_ARG, "m2_layernorm_bf16_fwd: null pointer");
  if (M <= 0 || d <= 0 || d % 64 != 0 || d > 2048)
    return set_error(M2_ERR_UNSUPPORTED, "m2_layernorm_bf16_fwd: need M > 0 and d a multiple of 64 up to 2048 (M=%d d=%d)", M, d);
  return launch_layernorm<false, uint16_t>((const uint16_t*)x, EmbedSource{}, gamma, beta, eps, out_f32, out_bf16,
                                           out_channel_major, M, d, stream);
}

extern "C" int m2_embed_layernorm_fwd(const long long* input_ids, const long long* token_type_ids,
                                      const long long* position_ids, const float* word_emb, const float* type_emb,
                                      const float* pos_emb, int vocab_size, int type_vocab_size, int max_positions,
                                      const float* gamma, const float* beta, float eps, float* out_f32, void* out_bf16,
                                      float* out_channel_major, int* bad_index, int B, int L, int d, void* stream) {
  if (!input_ids || !word_emb || !type_emb || !gamma || !beta)
    return set_error(M2_ERR_ARG, "m2_embed_layernorm_fwd: null pointer");
  if (B <= 0 || L <= 0 || d <= 0 || d % 64 != 0 || d > 2048)
    return set_error(M2_ERR_UNSUPPORTED, "m2_embed_layernorm_fwd: need B, L > 0 and d a multiple of 64 up to 2048 (B=%d L=%d d=%d)", B, L, d);
  if ((long)B * L > 0x7fffffffL) return set_error(M2_ERR_UNSUPPORTED, "m2_embed_layernorm_fwd: B * L = %ld does not fit an int", (long)B * L);
  if (position_ids && !pos_emb) return set_error(M2_ERR_ARG, "m2_embed_layernorm_fwd: position_ids without a position table");
  if (vocab_size <= 0 || type_vocab_size <= 0 || (pos_emb && max_positions <= 0))
    return set_error(M2_ERR_ARG, "m2_embed_layernorm_fwd: table sizes must be positive (vocab=%d type_vocab=%d max_positions=%d)",
                     vocab_size, type_vocab_size, max_positions);
  if (pos_emb && !position_ids && L > max_positions)
    return set_error(M2_ERR_ARG, "m2_embed_layernorm_fwd: sequence length %d exceeds the position table (%d rows)", L, max_positions);
  const EmbedSource src{input_ids, token_type_ids, position_ids, word_emb, type_emb, pos_emb, L,
                        vocab_size, type_vocab_size, max_positions, bad_index};
  return launch_layernorm<true>((const float*)nullptr, src, gamma, beta, eps, out_f32, out_bf16, out_channel_major, B * L, d, stream);
}
