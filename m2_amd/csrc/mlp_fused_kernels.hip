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
// A workgroup of eight waves (two per SIMD) owns 128 rows and one r; a wave owns 16 rows.  Everything is computed
// TRANSPOSED, weights as the MFMA A operand (rows of the product) and the x rows as the B operand (its columns),
// on v_mfma_f32_16x16x32_bf16:
//
//   G^T (32 gated columns x 16 x-rows)   = Wg_chunk (32 x 192) X_a^T  and  Wv_chunk X_b^T       24 MFMAs
//   OUT^T (192 x 16 x-rows)             += Wo_chunk (192 x 32) GLU(G^T)                          12 MFMAs
//
// because then the accumulator of the first product IS the B operand of the second: lane (n, q) of the MFMA
// receives accumulator rows 4 q .. 4 q + 3 of column n, and a B operand wants the eight K values 8 q .. 8 q + 7
// of column n.  Which gated column sits in which accumulator row is free, so operand row rho = 16 t + 4 q + j of
// a chunk (t = row tile) is given gated column gamma(rho) = 8 q + 4 t + j: the eight accumulator elements of a
// lane (two row tiles x four) are then the gated columns 8 q .. 8 q + 7, exactly the K range of one 16-byte piece
// of a `wo` row, and the gated values go from the accumulators through gelu(gate) * value and the bf16
// conversion straight into the next MFMA: the (M, I) intermediate never leaves the registers.
// The x rows of a wave (16 rows x two 192-wide blocks = 48 registers) are loaded once per row tile, straight from
// global memory in operand layout, and stay put.  The weights stream through LDS, 36 KB per chunk of 32 gated
// columns, in four stages, written by direct global -> LDS loads (global_load_lds_dwordx4: no registers, no LDS
// write instructions) issued three chunks ahead; every operand is one conflict-free 16-byte LDS read (a stage is
// laid out [operand block][lane]).  One barrier per chunk; the operand reads run ahead of the MFMAs through a ring
// of registers that does not drain at the barrier (the next chunk is complete one barrier early).
//
// Every compute unit streams ALL weights of its r once per 128-row tile, from L2: 36 KB per 0.5 us of MFMA work, more
// than the L2 delivers to a compute unit at the MFMAs' pace (with that stream, the operand reads, the GELU and the
// barrier, none of which hides behind the others, a chunk takes about 1.1 us).  Measured on MI355X with all 256 compute units
// streaming (direct-to-LDS loads, L2 hits): 62 GB/s per compute unit when a load instruction covers 1 KB of
// contiguous memory, 38 GB/s when it gathers sixteen 64-byte row pieces (the operand layout taken straight from the
// row-major weights).  So the weights are re-packed once (m2_mlp_fused_pack) into the exact image of the LDS
// stages -- per (r, chunk) 36 operand blocks of 1 KB, lane-major -- and every load instruction copies one contiguous
// block.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "fft_regs.h"
#include "m2_internal.h"
#include "mfma_stream.h"

namespace m2 {

constexpr int kFP = 192;                    // block width of x and of the output (d / 4)
constexpr int kFKS = kFP / 32;              // K steps of the first products (K = 32 per MFMA): 6
constexpr int kFRows = 128;                 // rows per workgroup of 8 waves (16 per wave); the 4-wave variant for small M owns 64
constexpr int kFChunk = 32;                 // gated columns per chunk
constexpr int kFBlk = 1024;                 // one operand block: 64 lanes x 16 bytes = 16 rows x 32 K
constexpr int kFGV = 2 * 2 * kFKS * kFBlk;  // Wg + Wv of a chunk: (gate | value) x 2 row tiles x 6 K steps = 24 KB
constexpr int kFWO = 12 * kFBlk;            // Wo of a chunk: 12 output tiles of 16 columns = 12 KB
constexpr int kFStages = 4;
constexpr int kFLds = kFStages * (kFGV + kFWO);      // 144 KB
constexpr int kFChunkBytes = kFGV + kFWO;   // a chunk in the packed weights: the image of its two stages

// Re-packs gated_layers.weight (4, I / 2, 192) and wo.weight (4, 192, I / 4) into the image of the LDS stages: for
// r = 0 .. 3 and chunk c (32 gated columns) 24 Wg / Wv blocks and 12 Wo blocks of 64 lanes x 16 bytes.  One thread
// per 16-byte piece.  Lane (i, q) of Wg / Wv block ((value, t), s) holds row gamma(16 t + i) = 8 (i / 4) + 4 t + i % 4
// of the chunk, K = 32 s + 8 q .. + 7; of Wo block tau the row of output column 32 (tau / 2) + 8 (i / 4) + 4 (tau % 2) + i % 4,
// K = 8 q .. + 7 of the chunk.  With that order of the output columns lane (n, q) of the main kernel ends up with the
// columns 32 s + 8 q .. + 7 (s = 0 .. 5) of its row: they leave as six 16-byte pieces, and the four lanes of a row
// write 64 contiguous bytes per store instruction (48 consecutive columns per lane, i.e. four pieces 96 bytes
// apart per instruction, cost 26 us of stores per launch at M = 32768).
__global__ __launch_bounds__(256) void mlp_fused_pack_kernel(const uint16_t* __restrict__ wg, const uint16_t* __restrict__ wo,
                                                             u32x4* __restrict__ packed, int I) {
  const int IS = I >> 2, q = I >> 1, nchunks = IS / kFChunk;
  const long piece = (long)blockIdx.x * 256 + threadIdx.x;
  const long npieces = 4l * nchunks * (kFChunkBytes / 16);
  if (piece >= npieces) return;
  const int lane = piece & 63, i16 = lane & 15, q4 = lane >> 4;
  const int blk = (piece >> 6) % 36;
  const int c = (piece / (64 * 36)) % nchunks;
  const int r = piece / (64l * 36 * nchunks);
  const uint16_t* src;
  if (blk < 24) {
    const int s = blk % kFKS, t = (blk / kFKS) & 1, val = blk / (2 * kFKS);
    const int gamma = 8 * (i16 >> 2) + 4 * t + (i16 & 3);
    src = wg + (((long)((r >> 1) + 2 * val) * q + (long)(r & 1) * IS + c * kFChunk + gamma) * kFP + 32 * s + 8 * q4);
  } else {
    const int tau = blk - 24;
    src = wo + (((long)r * kFP + 32 * (tau >> 1) + 8 * (i16 >> 2) + 4 * (tau & 1) + (i16 & 3)) * IS + c * kFChunk + 8 * q4);
  }
  packed[piece] = *reinterpret_cast<const u32x4*>(src);
}

// WAVES = 8: the kernel as described above.  WAVES = 4: the same with workgroups of four waves and 64 rows, for row
// counts at which 128-row tiles would leave compute units without work (M < 8192: one wave per SIMD, every wave
// copies 9 of a chunk's 36 blocks).
template <typename OUT, int WAVES>
__global__ __launch_bounds__(64 * WAVES) __attribute__((amdgpu_waves_per_eu(WAVES / 4, 2))) void mlp_fused_kernel(
    const uint16_t* __restrict__ x,       // (M, 768) bf16
    const unsigned char* __restrict__ wpk,      // both weights as packed by mlp_fused_pack_kernel
    const float* __restrict__ bias,       // (768) or null
    const uint16_t* __restrict__ resid,   // (M, 768) bf16 or null
    OUT* __restrict__ out,                // (M, 768)
    int M, int I, int ntiles) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  __shared__ __attribute__((aligned(16))) float bias_s[kFP];      // this r's slice of the bias, read at every tile's end
  const int tid = threadIdx.x, lane = tid & 63, i16 = lane & 15, q4 = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // Workgroup ids are dealt round-robin to the 8 XCDs (one L2 each): XCD e works on the two output blocks
  // r = 2 (e % 2), 2 (e % 2) + 1, which are fed by the same two blocks of x, and on the row tiles = e / 2 (mod 4);
  // neighbouring workgroups of an XCD take the same row tile with the two r, so its L2 holds half of the weights
  // and the second read of a tile's x rows hits it.  A workgroup is persistent: it walks over its row tiles while
  // the weight stream through LDS just keeps cycling.  (The grid has an even number of workgroups per XCD.)
  const int xcd = blockIdx.x & 7, slot = (int)(blockIdx.x >> 3);
  const int r = 2 * (xcd & 1) + (slot & 1);
  const int tile_step = 2 * (int)(gridDim.x >> 3);
  int tile = 4 * (slot >> 1) + (xcd >> 1);
  if (tile >= ntiles) return;
  const int IS = I >> 2;                  // gated columns of this r
  const int nchunks = IS / kFChunk;
  const int gb = r >> 1;                  // gate block; the value block is gb + 2
  const int d = 4 * kFP;
  if (tid < kFP) bias_s[tid] = bias ? bias[r * kFP + tid] : 0.f;      // visible after the prologue's barrier

  // ---- the wave's x rows as stationary B operands: lane (n, q) holds x[row n][32 s + 8 q .. + 8) of both blocks
  bf16x8 xa[kFKS], xb[kFKS];
  auto load_x = [&](int t) __attribute__((always_inline)) {
    int row = t * (16 * WAVES) + 16 * wave + i16;
    row = row < M ? row : M - 1;
    const uint16_t* pa = x + (long)row * d + gb * kFP + 8 * q4;
    const uint16_t* pb = pa + 2 * kFP;
    static_for<0, kFKS>([&](auto ss) {
      constexpr int s = decltype(ss)::value;
      xa[s] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(pa + 32 * s));
      xb[s] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(pb + 32 * s));
    });
  };
  load_x(tile);

  // ---- staging.  The packed weights hold, per (r, chunk), 36 operand blocks of 1 KB, lane-major: Wg / Wv block
  // ((value, row tile t), K step s) = index (2 value + t) 6 + s, then Wo blocks tau = 0 .. 11 (the output
  // columns 32 (tau / 2) + 8 (i / 4) + 4 (tau % 2) + i % 4, i < 16); lane (i, q) of a block holds what lane (i, q) of the MFMA needs.  Wave w copies the Wg / Wv blocks
  // w, w + 8, w + 16, the Wo block w and, for w < 4, the Wo block w + 8.
  const unsigned lds0 = (unsigned)(uintptr_t)smem;
  const unsigned voff = 16 * lane;
  const unsigned char* wr = wpk + (long)r * nchunks * kFChunkBytes;
  // Iterations are counted through all tiles of the workgroup (n = 0, 1, ...); iteration n reads Wg / Wv from stage
  // n % 4 and Wo from stage (n - 1) % 4.
  auto stage_gv = [&](int n) { return (n & (kFStages - 1)) * kFGV; };
  auto stage_wo = [&](int n) { return kFStages * kFGV + ((n - 1) & (kFStages - 1)) * kFWO; };
  // Load j of the batch that feeds iteration n, which is iteration `it` (0 .. nchunks) of its tile: Wg / Wv of chunk
  // `it` (iteration nchunks only repeats the last chunk) or Wo of chunk it - 1 (iteration 0 multiplies zeros by
  // whatever finite numbers it finds: chunk 0).
  constexpr int kBatch = 36 / WAVES + (36 % WAVES ? 1 : 0);      // loads per wave and chunk: 5 (8 waves) or 9 (4 waves)
  constexpr int kGvLoads = 24 / WAVES;                             // of which Wg / Wv blocks: 3 or 6
  constexpr int kDmaEvery = 36 / kBatch;                           // one load every 7th (4th) MFMA
  auto dma_one = [&](int n, int it, auto jj) __attribute__((always_inline)) {
    constexpr int j = decltype(jj)::value;
    if constexpr (j < kGvLoads) {
      const int cc = it < nchunks ? it : nchunks - 1;
      load_to_lds(lds0 + stage_gv(n) + (wave + WAVES * j) * kFBlk, voff, wr + (long)cc * kFChunkBytes + (wave + WAVES * j) * kFBlk);
    } else {
      const int cc = it > 0 ? it - 1 : 0;
      const int tau = wave + WAVES * (j - kGvLoads);
      if (WAVES * (j - kGvLoads + 1) <= 12 || wave < 12 - WAVES * (j - kGvLoads))      // the block exists
        load_to_lds(lds0 + stage_wo(n) + tau * kFBlk, voff, wr + (long)cc * kFChunkBytes + kFGV + tau * kFBlk);
    }
  };
  // what a wave waits for before the barrier: everything but its newest batch (waves whose last Wo block does not
  // exist issue one load fewer)
  auto wait_batch = [&]() __attribute__((always_inline)) {
    if constexpr (WAVES * (kBatch - kGvLoads) <= 12) {
      __builtin_amdgcn_s_waitcnt(0x0F70 | kBatch);
    } else {
      if (wave < 12 - WAVES * (kBatch - 1 - kGvLoads)) __builtin_amdgcn_s_waitcnt(0x0F70 | kBatch);
      else __builtin_amdgcn_s_waitcnt(0x0F70 | (kBatch - 1));
    }
  };

  floatx4 acc_out[12];
  floatx4 g[2], v[2];
  float gp[8], vp[8];      // the previous chunk's gate / value accumulators, in gated-column order 4 t + j

  // ---- the instruction stream of an iteration: 36 MFMAs, laid out by hand and pinned with scheduling barriers.
  // MFMA k < 24: first products of chunk i, K step k / 4, (gate t = 0, value t = 0, gate t = 1, value t = 1) = k % 4;
  // MFMA 24 + tau: OUT^T tile tau += Wo block tau of chunk i - 1 times gelu * value of chunk i - 1.
  // The operand of MFMA k + kPF is read right after MFMA k is issued; past the end of the iteration those are the
  // first operands of the next one (its chunk has been complete in LDS since the last barrier).
  constexpr int kNM = 36;
  constexpr int kPF = 12;      // divides kNM, so that operand k of every iteration sits in ring slot k % kPF
  static_assert(kNM % kPF == 0, "the ring must close over an iteration");
  const unsigned char* lane_base = smem + 16 * lane;
  // Operand k of an iteration sits at a compile-time offset from one of two addresses (the lane's 16 bytes in the
  // iteration's Wg / Wv stage and in its Wo stage); the four addresses an iteration uses (its own and the next
  // iteration's) are formed once at its top, so that an operand read is one LDS instruction and nothing else.
  auto operand_off = [&](auto kk) constexpr -> int {
    constexpr int k = decltype(kk)::value;
    if constexpr (k < 24) {
      constexpr int s = k / 4, sel = k % 4, t = sel >> 1, val = sel & 1;
      return ((2 * val + t) * kFKS + s) * kFBlk;
    } else {
      return (k - 24) * kFBlk;
    }
  };
  auto operand_addr = [&](int n, auto kk) __attribute__((always_inline)) -> const unsigned char* {
    constexpr int k = decltype(kk)::value;
    return lane_base + (k < 24 ? stage_gv(n) : stage_wo(n)) + operand_off(kk);
  };
  u32x4 ring[kPF];
  bf16x8 gt;

  // prologue: the batches of iterations 0 .. 2; then the ring for iteration 0
  int it3 = 0;             // which iteration of its tile iteration n + 3 is
  for (int n = 0; n < 3; ++n) {
    static_for<0, kBatch>([&](auto jj) { dma_one(n, it3, jj); });
    it3 = it3 == nchunks ? 0 : it3 + 1;
  }
  __builtin_amdgcn_s_waitcnt(kWaitVm0);
  __syncthreads();
  static_for<0, kPF>([&](auto kk) { ring[decltype(kk)::value] = *reinterpret_cast<const u32x4*>(operand_addr(0, kk)); });
  {
    u32x4 z = {0u, 0u, 0u, 0u};
    gt = __builtin_bit_cast(bf16x8, z);
  }

  int n = 0;
  for (;;) {
    static_for<0, 12>([&](auto tt) {
      static_for<0, 4>([&](auto vv) { acc_out[decltype(tt)::value][decltype(vv)::value] = 0.f; });
    });
    // The x loads complete here, once per tile: consumed before the loop, the compiler has no reason to keep a
    // "load may be pending" mark on the x registers around the loop's back edge (that would put a full
    // vector-memory wait, which also waits for the direct-to-LDS loads just issued, into every iteration).
#pragma unroll
    for (int s = 0; s < kFKS; ++s) asm volatile("" : "+v"(xa[s]), "+v"(xb[s]));

    // Iteration i = 0 .. nchunks of the tile, in three copies of one body.  Iteration 0 (HEAD) has no previous chunk:
    // no gelu * value, no second product.  Iteration nchunks (TAIL) has no chunk of its own: no first products; it
    // first requests what the end of the tile needs -- the next tile's x rows into the registers that have just become
    // free, and this tile's residual rows -- so that those loads travel while the last second product runs.
    const int row = tile * (16 * WAVES) + 16 * wave + i16;
    const int rowc = row < M ? row : M - 1;
    const long o0 = (long)rowc * d + r * kFP + 8 * q4;
    u32x4 rres[6];
    auto iteration = [&](auto which_) __attribute__((always_inline)) {
      constexpr bool TAIL = decltype(which_)::value == 1, HEAD = decltype(which_)::value == 2;
      if constexpr (TAIL) {
        if (tile + tile_step < ntiles) load_x(tile + tile_step);
      }
      if constexpr (HEAD) {
        if (resid) {
          static_for<0, 6>([&](auto mm) {
            rres[decltype(mm)::value] = *reinterpret_cast<const u32x4*>(resid + o0 + 32 * decltype(mm)::value);
          });
        }
      }
      float gl[8];
      unsigned ogv0 = 16 * lane + stage_gv(n), owo0 = 16 * lane + stage_wo(n);
      unsigned ogv1 = 16 * lane + stage_gv(n + 1), owo1 = 16 * lane + stage_wo(n + 1);
      asm volatile("" : "+v"(ogv0), "+v"(owo0), "+v"(ogv1), "+v"(owo1));
      static_for<0, kNM>([&](auto kk) {
        constexpr int k = decltype(kk)::value;
        const bf16x8 a = __builtin_bit_cast(bf16x8, ring[k % kPF]);
        if constexpr (k < 24 && TAIL) {
          // nothing to multiply; the operand read below still refills the ring for the next iteration
        } else if constexpr (k < 24) {
          constexpr int s = k / 4, sel = k % 4, t = sel >> 1, val = sel & 1;
          floatx4& acc = val ? v[t] : g[t];
          if constexpr (s == 0) {
            const floatx4 z = {0.f, 0.f, 0.f, 0.f};
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, val ? xb[0] : xa[0], z, 0, 0, 0);
          } else {
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, val ? xb[s] : xa[s], acc, 0, 0, 0);
          }
        } else if constexpr (!HEAD) {
          acc_out[k - 24] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, gt, acc_out[k - 24], 0, 0, 0);
        }
        // next operand: this iteration's while k + kPF < 36, else the next iteration's
        if constexpr (k + kPF < kNM)
          ring[k % kPF] = *reinterpret_cast<const u32x4*>(smem + (k + kPF < 24 ? ogv0 : owo0) + operand_off(ic<k + kPF>{}));
        else
          ring[k % kPF] = *reinterpret_cast<const u32x4*>(smem + (k + kPF - kNM < 24 ? ogv1 : owo1) + operand_off(ic<k + kPF - kNM>{}));
        // The batch of direct loads for iteration n + 3, one load every seventh MFMA: Wg / Wv into the stage last
        // read in iteration n - 1, Wo into the one last read in iteration n - 1 as well, both before the barrier that
        // started this iteration.  (Issued together at the top, the loads of the workgroup fill the memory
        // pipeline's queue and every wave stalls behind its own loads: 21 us of 210 at M = 32768.)
        if constexpr (k % kDmaEvery == 1 && k / kDmaEvery < kBatch) dma_one(n + 3, it3, ic<k / kDmaEvery>{});
        // vector-ALU work riding along: gelu * value of the previous chunk, all eight elements in one burst behind the
        // first MFMA (measured: one element after every third MFMA 151.7 us, two after every sixth 149.8, four after
        // every twelfth 149.4, all eight at once 147.3; four instructions after every MFMA 155.0), then its
        // packing; during the second product the accumulators just finished are copied out
        if constexpr (k == 0 && !HEAD) {
          GeluChain ch[8];
          static_for<0, 11>([&](auto st) {
            static_for<0, 8>([&](auto ee) {
              constexpr int e = decltype(ee)::value;
              gelu_step<decltype(st)::value>(ch[e], gp[e], vp[e], gl[e]);
            });
          });
        }
        if constexpr (k == 23 && !HEAD) {
          u32x4 pk;
          pk.x = pack_bf16x2(gl[0], gl[1]);
          pk.y = pack_bf16x2(gl[2], gl[3]);
          pk.z = pack_bf16x2(gl[4], gl[5]);
          pk.w = pack_bf16x2(gl[6], gl[7]);
          gt = __builtin_bit_cast(bf16x8, pk);
        }
        if constexpr (k >= 28) {
          constexpr int e = k - 28;      // 0 .. 7: element 4 t + j
          gp[e] = g[e >> 2][e & 3];
          vp[e] = v[e >> 2][e & 3];
        }
        __builtin_amdgcn_sched_barrier(0);
      });
      it3 = it3 == nchunks ? 0 : it3 + 1;
      // before the barrier: everything but this wave's newest batch has landed, so after the barrier the chunks of
      // iterations n + 1 and n + 2 are complete for everybody
      wait_batch();
      __syncthreads();
      __builtin_amdgcn_sched_barrier(0);
      ++n;
    };
    iteration(ic<2>{});
    for (int i = 1; i < nchunks; ++i) iteration(ic<0>{});
    iteration(ic<1>{});

    // ---- end of the tile: this tile's results leave.  Accumulator element j of tile tau is output column
    // 32 (tau / 2) + 8 q + 4 (tau % 2) + j of x-row n (the order the packed Wo rows were given): piece m of a lane =
    // tiles 2 m and 2 m + 1 = the eight columns 32 m + 8 q .. + 7.
    tile += tile_step;
    const bool more = tile < ntiles;
    if (row < M) {
      static_for<0, 6>([&](auto mm) {
        constexpr int m = decltype(mm)::value;
        float val[8];
        static_for<0, 8>([&](auto ee) {
          constexpr int e = decltype(ee)::value;
          val[e] = acc_out[2 * m + e / 4][e % 4] + bias_s[32 * m + 8 * q4 + e];
        });
        if (resid) {
          const u32x4 rr = rres[m];
          val[0] += __uint_as_float(rr.x << 16); val[1] += __uint_as_float(rr.x & 0xffff0000u);
          val[2] += __uint_as_float(rr.y << 16); val[3] += __uint_as_float(rr.y & 0xffff0000u);
          val[4] += __uint_as_float(rr.z << 16); val[5] += __uint_as_float(rr.z & 0xffff0000u);
          val[6] += __uint_as_float(rr.w << 16); val[7] += __uint_as_float(rr.w & 0xffff0000u);
        }
        if constexpr (sizeof(OUT) == 2) {
          u32x4 pk;
          pk.x = pack_bf16x2(val[0], val[1]);
          pk.y = pack_bf16x2(val[2], val[3]);
          pk.z = pack_bf16x2(val[4], val[5]);
          pk.w = pack_bf16x2(val[6], val[7]);
          *reinterpret_cast<u32x4*>(out + o0 + 32 * m) = pk;
        } else {
          *reinterpret_cast<float4*>(out + o0 + 32 * m) = make_float4(val[0], val[1], val[2], val[3]);
          *reinterpret_cast<float4*>(out + o0 + 32 * m + 4) = make_float4(val[4], val[5], val[6], val[7]);
        }
      });
    }
    if (!more) break;
  }
  // no load may still be in flight when the workgroup ends (its LDS goes to the next one)
  __builtin_amdgcn_s_waitcnt(kWaitVm0);
}

}  // namespace m2

using namespace m2;

template <typename OUT>
static OUT* out_ptr(void (*)(const uint16_t*, const unsigned char*, const float*, const uint16_t*, OUT*, int, int, int));

extern "C" int m2_mlp_fused_supported(int in_features, int intermediate, int nblocks) {
  return nblocks == 4 && in_features == 4 * kFP && intermediate > 0 && intermediate % (4 * kFChunk) == 0;
}

extern "C" long m2_mlp_fused_packed_bytes(int in_features, int intermediate, int nblocks) {
  if (!m2_mlp_fused_supported(in_features, intermediate, nblocks)) return 0;
  return 4l * (intermediate / 4 / kFChunk) * kFChunkBytes;      // = 2 bytes x (elements of w_gated + elements of w_out)
}

extern "C" int m2_mlp_fused_pack(const void* w_gated, const void* w_out, void* packed, int in_features, int intermediate,
                                 int nblocks, void* stream) {
  if (!w_gated || !w_out || !packed) return set_error(M2_ERR_ARG, "m2_mlp_fused_pack: null pointer");
  if (!m2_mlp_fused_supported(in_features, intermediate, nblocks))
    return set_error(M2_ERR_UNSUPPORTED,
                     "m2_mlp_fused_pack: built for nblocks=4, in_features=768 and intermediate a multiple of 128 "
                     "(got nblocks=%d in=%d intermediate=%d)", nblocks, in_features, intermediate);
  const long npieces = m2_mlp_fused_packed_bytes(in_features, intermediate, nblocks) / 16;
  hipLaunchKernelGGL(mlp_fused_pack_kernel, dim3((unsigned)((npieces + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     (const uint16_t*)w_gated, (const uint16_t*)w_out, (u32x4*)packed, intermediate);
  return check_launch("mlp_fused_pack");
}

extern "C" int m2_mlp_fused_fwd(const void* x, const void* w_packed, const float* bias, const void* residual, void* out,
                                int M, int in_features, int intermediate, int nblocks, int out_dtype, void* stream) {
  if (!x || !w_packed || !out) return set_error(M2_ERR_ARG, "m2_mlp_fused_fwd: null pointer");
  if (M <= 0) return set_error(M2_ERR_ARG, "m2_mlp_fused_fwd: M=%d must be positive", M);
  if (out_dtype != M2_DTYPE_F32 && out_dtype != M2_DTYPE_BF16)
    return set_error(M2_ERR_ARG, "m2_mlp_fused_fwd: out_dtype %d is neither M2_DTYPE_F32 nor M2_DTYPE_BF16", out_dtype);
  if (!m2_mlp_fused_supported(in_features, intermediate, nblocks))
    return set_error(M2_ERR_UNSUPPORTED,
                     "m2_mlp_fused_fwd: built for nblocks=4, in_features=768 and intermediate a multiple of 128 "
                     "(got nblocks=%d in=%d intermediate=%d); use m2_blockdiag_glu_fwd + m2_blockdiag_linear_fwd",
                     nblocks, in_features, intermediate);
  // 128-row tiles and eight waves per workgroup; 64-row tiles and four waves where the 128-row tiles of the four
  // output blocks would not occupy the compute units (M < 8192 on 256 of them)
  const bool small = 4 * ((M + kFRows - 1) / kFRows) < num_cus();
  const int rows = small ? kFRows / 2 : kFRows;
  const int ntiles = (M + rows - 1) / rows;
  // one persistent workgroup per compute unit (144 KB of LDS each), an even number per XCD
  int per_xcd = (num_cus() / 8) & ~1;
  if (per_xcd < 2) per_xcd = 2;      // a device (or partition) with fewer than 16 compute units: work is dealt to 8 x per_xcd slots whatever the real count
  if (per_xcd > 2 * ((ntiles + 3) / 4)) per_xcd = 2 * ((ntiles + 3) / 4);
  const dim3 grid(8 * per_xcd);
  hipStream_t st = (hipStream_t)stream;
  auto launch = [&](auto kern, int threads) -> int {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, kFLds);
    if (e != hipSuccess) return set_error(M2_ERR_LAUNCH, "hipFuncSetAttribute(mlp_fused): %s", hipGetErrorString(e));
    hipLaunchKernelGGL(kern, grid, dim3(threads), kFLds, st, (const uint16_t*)x, (const unsigned char*)w_packed, bias,
                       (const uint16_t*)residual, (decltype(out_ptr(kern)))out, M, intermediate, ntiles);
    return 0;
  };
  int rc;
  if (out_dtype == M2_DTYPE_F32)
    rc = small ? launch(mlp_fused_kernel<float, 4>, 256) : launch(mlp_fused_kernel<float, 8>, 512);
  else
    rc = small ? launch(mlp_fused_kernel<uint16_t, 4>, 256) : launch(mlp_fused_kernel<uint16_t, 8>, 512);
  if (rc) return rc;
  return check_launch("mlp_fused");
}
