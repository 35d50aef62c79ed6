// Dense bf16 GEMM tiles on MFMA for the projections around the mixer core:
//
//   D[q][p] = sum_k Q[q][k] P[p][k]          P (np, K) and Q (nq, K) bf16, both K-contiguous
//
// written q-major (p contiguous).  `in_linear` of the sequence mixer (bert/src/mm/monarch_mixer_sequence_mixer.py:
// 81,108) is Q = in_linear.weight (3d, d), P = the layer input (M, d): the output is then channel-major (3d, M),
// the layout the mixer core reads, without a transpose pass and without a bias pass (the core adds the bias).
//
// Workgroup = 8 waves (two per SIMD) on a 256 (q) x 256 (p) tile, wave (wq, wp) = 64 x 128: 2 x 4 MFMA tiles of
// v_mfma_f32_32x32x16_bf16, 128 accumulators per lane.  K advances in chunks of 64 through two LDS stages of 64 KB
// that are written by direct global -> LDS loads (global_load_lds_dwordx4: no staging registers, no LDS write
// instructions).  A load instruction fetches eight rows x 128 bytes, i.e. eight whole cache lines (the L2 delivers
// whole-line gathers at twice the rate of 32- or 64-byte row pieces: measured); the 16-byte pieces of such a block are
// placed [K step][half][row], with the two halves swapped in every other block, so that an MFMA operand -- 32 rows x
// one K step, four blocks -- is one 16-byte LDS read per lane that touches every bank once per 16 lanes.  Operand registers are double-buffered per K step: the reads of step s + 1 are issued before
// the eight MFMAs of step s (6 reads per 8 MFMAs).  The finished tile goes through LDS so that every global store
// is a full row segment.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fft_regs.h"
#include "m2_internal.h"

namespace m2 {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kGT = 256;                    // tile edge (both ways)
constexpr int kGK = 64;                     // K per chunk
constexpr int kGBlk = 1024;                 // one load instruction: 64 lanes x 16 bytes = 8 rows x 64 K
constexpr int kGSide = (kGT / 8) * kGBlk;   // P (or Q) part of a stage: 32 blocks = 32 KB
constexpr int kGStage = 2 * kGSide;         // 64 KB
constexpr int kGStages = 2;
constexpr int kGOutRow = 2 * kGT + 16;      // bytes per padded row of the bf16 output tile in LDS
constexpr int kGLds = kGT * kGOutRow;       // 135168 bytes >= 2 stages

// s_waitcnt immediate (vmcnt in bits 3:0 and 15:14, expcnt 6:4, lgkmcnt 11:8): vector-memory counter to zero only
constexpr int kGWaitVm0 = 0x0F70;

// One direct global -> LDS load: every lane fetches 16 bytes from base + voff, lane l's piece lands at LDS byte
// address lds + 16 l.  Inline assembly on purpose: the compiler then neither tracks the LDS write (it would put a
// full vector-memory wait in front of every later LDS read) nor reorders it across other memory accesses; the
// kernel waits for these loads itself.
__device__ __forceinline__ void gemm_load_to_lds(unsigned lds, unsigned voff, const void* base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds), "v"(voff), "s"(base) : "memory");
}

struct GemmArgs {
  const uint16_t* P;      // (np, K) bf16, row stride ldp elements
  const uint16_t* Q;      // (nq, K) bf16, row stride ldq elements
  uint16_t* out;          // (nq, np) bf16, row stride ldo elements
  int np, nq, K;
  long ldp, ldq, ldo;
};

__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_qmajor_kernel(GemmArgs g) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, i32 = lane & 31, half = lane >> 5;
  const int wq = wave >> 1, wp = wave & 1;          // wave tile: q rows [64 wq, +64), p columns [128 wp, +128)
  // Tile order: workgroup ids are dealt round-robin to the 8 XCDs (one L2 each).  XCD e takes the p tiles e, e + 8,
  // ... (tokens for in_linear) and walks all q tiles (the whole weight matrix) of one p tile back to back, so the
  // P rows of the tiles in flight stay in that XCD's L2 and the (small) Q matrix is shared by everybody.
  const int ntp = (g.np + kGT - 1) / kGT, ntq = (g.nq + kGT - 1) / kGT;
  int tp, tq;
  {
    const int id = blockIdx.x, e = id & 7, l = id >> 3;
    const int full = (ntp / 8) * 8;
    if (id < full * ntq) { tp = (l / ntq) * 8 + e; tq = l % ntq; }
    else { const int rid = id - full * ntq; tp = full + rid / ntq; tq = rid % ntq; }
  }
  const int p0 = tp * kGT, q0 = tq * kGT;
  const int nchunks = g.K / kGK;

  // ---- staging: a stage holds 32 P blocks then 32 Q blocks, block b = rows [8 b, + 8) x the 64 K of the chunk; wave
  // w loads the blocks w, w + 8, ... of each side (4 + 4 per chunk).  Lane l of a block = (K step l / 16, slot
  // (l / 8) % 2, row l % 8); the slot holds K half (slot ^ b % 2), and b % 2 = w % 2 for all blocks of a wave.  Rows past
  // the end are clamped.
  const unsigned lds0 = (unsigned)(uintptr_t)smem;
  unsigned voff_p[4], voff_q[4];
  static_for<0, 4>([&](auto jj) {
    constexpr int j = decltype(jj)::value;
    const int b = wave + 8 * j;
    const int ks = lane >> 4, khalf = ((lane >> 3) & 1) ^ (wave & 1), r = lane & 7;
    int rp = p0 + 8 * b + r, rq = q0 + 8 * b + r;
    rp = rp < g.np ? rp : g.np - 1;
    rq = rq < g.nq ? rq : g.nq - 1;
    voff_p[j] = (unsigned)(((long)rp * g.ldp + 16 * ks + 8 * khalf) * 2);
    voff_q[j] = (unsigned)(((long)rq * g.ldq + 16 * ks + 8 * khalf) * 2);
  });
  // loads j of chunk c: one P block and one Q block
  auto dma_pair = [&](int c, auto jj) __attribute__((always_inline)) {
    constexpr int j = decltype(jj)::value;
    const unsigned st = __builtin_amdgcn_readfirstlane(lds0 + (c % kGStages) * kGStage + wave * kGBlk);
    gemm_load_to_lds(st + 8 * kGBlk * j, voff_p[j], g.P + (long)c * kGK);
    gemm_load_to_lds(st + kGSide + 8 * kGBlk * j, voff_q[j], g.Q + (long)c * kGK);
  };
  auto dma = [&](int c) __attribute__((always_inline)) { static_for<0, 4>([&](auto jj) { dma_pair(c, jj); }); };

  floatx16 acc[2][4];      // [q tile][p tile]
  static_for<0, 8>([&](auto tt) {
    static_for<0, 16>([&](auto vv) { acc[decltype(tt)::value / 4][decltype(tt)::value % 4][decltype(vv)::value] = 0.f; });
  });

  // operand reads of K step s of the chunk in stage st: 4 P blocks (A operands) and 2 Q blocks (B operands)
  u32x4 opa[2][4], opb[2][2];
  auto read_ops = [&](int st, auto ss, auto bb) __attribute__((always_inline)) {
    constexpr int s = decltype(ss)::value, bf = decltype(bb)::value;
    // lane (i32, half) of a 32-row tile: block i32 / 8 of the tile's four, slot half ^ (block % 2), row i32 % 8
    const unsigned char* base = smem + st * kGStage + (i32 >> 3) * kGBlk + (((half ^ ((i32 >> 3) & 1)) * 8 + (i32 & 7)) * 16) + s * 256;
    static_for<0, 4>([&](auto pp) {
      constexpr int pi = decltype(pp)::value;
      opa[bf][pi] = *reinterpret_cast<const u32x4*>(base + (4 * wp + pi) * 4 * kGBlk);
    });
    static_for<0, 2>([&](auto qq) {
      constexpr int qi = decltype(qq)::value;
      opb[bf][qi] = *reinterpret_cast<const u32x4*>(base + kGSide + (2 * wq + qi) * 4 * kGBlk);
    });
  };
  auto mfmas = [&](auto bb) __attribute__((always_inline)) {
    constexpr int bf = decltype(bb)::value;
    static_for<0, 4>([&](auto pp) {
      constexpr int pi = decltype(pp)::value;
      static_for<0, 2>([&](auto qq) {
        constexpr int qi = decltype(qq)::value;
        acc[qi][pi] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, opa[bf][pi]),
                                                              __builtin_bit_cast(bf16x8, opb[bf][qi]), acc[qi][pi], 0, 0, 0);
      });
    });
  };

  dma(0);
  for (int c = 0; c < nchunks; ++c) {
    __builtin_amdgcn_s_waitcnt(kGWaitVm0);      // this wave's pieces of chunk c have landed
    __syncthreads();                            // ... everybody's; and everybody is done reading chunk c - 1
    const int st = c & 1;
    const bool more = c + 1 < nchunks;
    // The reads of K step s + 1 are issued before the MFMAs of step s (scheduling barriers pin that order), and the
    // eight loads of the next chunk go out two at a time between the MFMA groups: issued together they fill the
    // memory pipeline's queue and every wave stalls behind its own loads.
    read_ops(st, ic<0>{}, ic<0>{});
    __builtin_amdgcn_sched_barrier(0);
    read_ops(st, ic<1>{}, ic<1>{});
    __builtin_amdgcn_sched_barrier(0);
    if (more) dma_pair(c + 1, ic<0>{});
    mfmas(ic<0>{});
    __builtin_amdgcn_sched_barrier(0);
    read_ops(st, ic<2>{}, ic<0>{});
    __builtin_amdgcn_sched_barrier(0);
    if (more) dma_pair(c + 1, ic<1>{});
    mfmas(ic<1>{});
    __builtin_amdgcn_sched_barrier(0);
    read_ops(st, ic<3>{}, ic<1>{});
    __builtin_amdgcn_sched_barrier(0);
    if (more) dma_pair(c + 1, ic<2>{});
    mfmas(ic<0>{});
    __builtin_amdgcn_sched_barrier(0);
    if (more) dma_pair(c + 1, ic<3>{});
    mfmas(ic<1>{});
    __builtin_amdgcn_sched_barrier(0);
  }
  __syncthreads();      // all operand reads done: the stages become the output tile

  // ---- epilogue: accumulator element v = 4 a + b of tile (qi, pi) is row q = 64 wq + 32 qi + i32,
  // column p = 128 wp + 32 pi + 8 a + 4 half + b.  The tile goes to LDS as bf16 rows of q, then out as full rows.
  static_for<0, 2>([&](auto qq) {
    constexpr int qi = decltype(qq)::value;
    unsigned char* rowp = smem + (64 * wq + 32 * qi + i32) * kGOutRow + 2 * (128 * wp + 4 * half);
    static_for<0, 4>([&](auto pp) {
      constexpr int pi = decltype(pp)::value;
      static_for<0, 4>([&](auto aa) {
        constexpr int a = decltype(aa)::value;
        uint2 pk;
        pk.x = pack_bf16x2(acc[qi][pi][4 * a], acc[qi][pi][4 * a + 1]);
        pk.y = pack_bf16x2(acc[qi][pi][4 * a + 2], acc[qi][pi][4 * a + 3]);
        *reinterpret_cast<uint2*>(rowp + 2 * (32 * pi + 8 * a)) = pk;
      });
    });
  });
  __syncthreads();
  // 256 rows x 512 bytes: a wave writes one row per instruction as 32 x 16 bytes (lanes 32 .. 63 take the next row)
  const int np_here = g.np - p0;
  for (int r = 2 * wave + half; r < kGT; r += 16) {
    const int q = q0 + r;
    if (q >= g.nq) break;
    const u32x4 v = *reinterpret_cast<const u32x4*>(smem + r * kGOutRow + 16 * i32);
    uint16_t* dst = g.out + (long)q * g.ldo + p0 + 8 * i32;
    if (8 * i32 + 8 <= np_here) {
      *reinterpret_cast<u32x4*>(dst) = v;
    } else {
      const uint16_t* e = reinterpret_cast<const uint16_t*>(&v);
      for (int k = 0; k < 8; ++k)
        if (8 * i32 + k < np_here) dst[k] = e[k];
    }
  }
}

}  // namespace m2

using namespace m2;

extern "C" int m2_gemm_bf16_supported(int np, int nq, int K) {
  return np > 0 && nq > 0 && K > 0 && K % kGK == 0;
}

extern "C" int m2_gemm_bf16_qmajor_fwd(const void* P, const void* Q, void* out, int np, int nq, int K, void* stream) {
  if (!P || !Q || !out) return set_error(M2_ERR_ARG, "m2_gemm_bf16_qmajor_fwd: null pointer");
  if (!m2_gemm_bf16_supported(np, nq, K))
    return set_error(M2_ERR_UNSUPPORTED, "m2_gemm_bf16_qmajor_fwd: need positive sizes and K a multiple of %d (np=%d nq=%d K=%d)",
                     kGK, np, nq, K);
  if ((long)np * K * 2 >= (1L << 32) || (long)nq * K * 2 >= (1L << 32))
    return set_error(M2_ERR_UNSUPPORTED, "m2_gemm_bf16_qmajor_fwd: an operand of 4 GiB or more (np=%d nq=%d K=%d)", np, nq, K);
  GemmArgs g;
  g.P = (const uint16_t*)P; g.Q = (const uint16_t*)Q; g.out = (uint16_t*)out;
  g.np = np; g.nq = nq; g.K = K;
  g.ldp = K; g.ldq = K; g.ldo = np;
  auto kern = gemm_qmajor_kernel;
  hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, kGLds);
  if (e != hipSuccess) return set_error(M2_ERR_LAUNCH, "hipFuncSetAttribute(gemm_qmajor): %s", hipGetErrorString(e));
  const int ntp = (np + kGT - 1) / kGT, ntq = (nq + kGT - 1) / kGT;
  hipLaunchKernelGGL(kern, dim3(ntp * ntq), dim3(512), kGLds, (hipStream_t)stream, g);
  return check_launch("gemm_qmajor");
}
