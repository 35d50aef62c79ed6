// Measured ceilings of one compute unit's matrix pipe, for the roofline arguments of the GEMM-shaped kernels:
// a loop of v_mfma_f32_32x32x16_bf16 on register operands, alone or with the company the real kernels give it
// (one or two 16-byte LDS operand reads per MFMA, software-pipelined six MFMAs ahead; 4, 6 or 11 dependent fp32
// FMAs per MFMA in the same instruction stream), at one or two waves per SIMD on every compute unit.  What comes
// out is the rate this chip sustains at the clock it runs such code at, which is what a kernel's achieved
// TFLOP/s can be held against beside the published peak.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fft_split.h"
#include "m2_internal.h"

namespace m2 {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kProbeLds = 64 * 1024;
constexpr int kProbePF = 6;        // operand reads run this many MFMAs ahead

template <int READS, int VALU, int NT>
__global__ __launch_bounds__(NT) void probe_mfma_kernel(float* __restrict__ sink, int iters) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  for (int i = tid; i < kProbeLds / 4; i += NT) reinterpret_cast<float*>(lds)[i] = i * 1e-6f;
  __syncthreads();
  floatx16 acc[6];
  static_for<0, 6>([&](auto tt) { static_for<0, 16>([&](auto vv) { acc[decltype(tt)::value][decltype(vv)::value] = 0.f; }); });
  bf16x8 b0;
  for (int i = 0; i < 8; ++i) b0[i] = (__bf16)(tid * 0.001f + i);
  float v[8];
  for (int i = 0; i < 8; ++i) v[i] = tid * 0.01f + i;
  const unsigned char* base = lds + 16 * lane;      // [block of 1 KB][lane]: conflict-free 16-byte reads
  u32x4 ring[kProbePF], ring2[kProbePF];
  static_for<0, kProbePF>([&](auto ss) {
    constexpr int s = decltype(ss)::value;
    ring[s] = *reinterpret_cast<const u32x4*>(base + 1024 * s);
    ring2[s] = *reinterpret_cast<const u32x4*>(base + 1024 * (s + 24));
  });
  for (int it = 0; it < iters; ++it) {
    static_for<0, 12>([&](auto ss) {
      constexpr int s = decltype(ss)::value;
      const bf16x8 a = READS >= 1 ? __builtin_bit_cast(bf16x8, ring[s % kProbePF]) : b0;
      const bf16x8 b = READS >= 2 ? __builtin_bit_cast(bf16x8, ring2[s % kProbePF]) : b0;
      acc[s % 6] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[s % 6], 0, 0, 0);
      if constexpr (READS >= 1) ring[s % kProbePF] = *reinterpret_cast<const u32x4*>(base + 1024 * ((s + kProbePF) % 12) + 12288 * (it & 1));
      if constexpr (READS >= 2) ring2[s % kProbePF] = *reinterpret_cast<const u32x4*>(base + 1024 * (24 + (s + kProbePF) % 12) + 12288 * (it & 1));
      static_for<0, VALU>([&](auto ee) { v[decltype(ee)::value % 8] = fmaf(v[decltype(ee)::value % 8], 1.0001f, 0.5f); });
      __builtin_amdgcn_sched_barrier(0);
    });
  }
  float s = 0.f;
  static_for<0, 6>([&](auto tt) { static_for<0, 16>([&](auto vv) { s += acc[decltype(tt)::value][decltype(vv)::value]; }); });
  for (int i = 0; i < 8; ++i) s += v[i];
  sink[(long)blockIdx.x * NT + tid] = s;
}

template <int READS, int VALU, int NT>
static int launch_probe(float* sink, int iters, hipStream_t st) {
  auto kern = probe_mfma_kernel<READS, VALU, NT>;
  hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, kProbeLds);
  if (e != hipSuccess) return set_error(M2_ERR_LAUNCH, "hipFuncSetAttribute(probe): %s", hipGetErrorString(e));
  hipLaunchKernelGGL(kern, dim3(num_cus()), dim3(NT), kProbeLds, st, sink, iters);
  return check_launch("probe_mfma");
}

// ---------------------------------------------------------------------------------------------
// One pass of the L = 8192 half transform of the long-convolution kernels (the radix-16 pass at stride 16 with its
// twiddles, fft_split.h: fwd_pass2) done two ways on a row resident in LDS, to be timed against each other:
//   MFMA = false  the butterflies on the vector ALU, as the mixer core runs them;
//   MFMA = true   the 16-point DFTs as a product with the 32 x 32 real form of the DFT matrix on
//                 v_mfma_f32_32x32x16_bf16: Y = F X with X = [Re x; Im x] (32 x 32 groups per product), every
//                 operand split into a bf16 high and low part and the three leading products summed (hi hi + hi lo
//                 + lo hi: 16 mantissa bits), the split done on the fly on the vector ALU, twiddles after it.
// A workgroup owns one row (8192 complex points) and repeats the pass `iters` times in place.
// ---------------------------------------------------------------------------------------------
typedef SplitPlan<13, 32, 16> ProbePlan;

template <bool MFMA>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void probe_dft16_kernel(float2* __restrict__ rows, int iters) {
  typedef ProbePlan P;
  extern __shared__ float2 plds[];
  float2* row = plds;
  float2* tab2 = plds + P::ROW_LDS;
  const int t = threadIdx.x, wave = t >> 6, lane = t & 63, i32 = lane & 31, half = lane >> 5;
  float2* g = rows + (long)blockIdx.x * P::L;
  tab2_init<P>(tab2);
  for (int i = t; i < P::L; i += 256) row[sphys(i)] = g[i];
  __syncthreads();
  if constexpr (!MFMA) {
    cf x[32];
    for (int it = 0; it < iters; ++it) {
      fwd_pass2<P>(x, t, row, tab2);
      __syncthreads();
    }
  } else {
    // A operands: row r of F (r < 16: Re Y_r = sum_j cos(2 pi j r / 16) Re x_j + sin(..) Im x_j; r >= 16: Im Y_k =
    // - sin Re x_j + cos Im x_j, k = r - 16), K = 16 kk + 8 half + e: kk = 0 the Re x_j coefficients, kk = 1 Im x_j
    bf16x8 ahi[2], alo[2];
    static_for<0, 2>([&](auto kk_) {
      constexpr int kk = decltype(kk_)::value;
      float hi[8], lo[8];
      for (int e = 0; e < 8; ++e) {
        const int j = 8 * half + e, k = i32 & 15;
        float sn, cs;
        sincospif(2.0f * (float)((j * k) & 15) / 16.0f, &sn, &cs);
        const float f = (i32 < 16) ? (kk == 0 ? cs : sn) : (kk == 0 ? -sn : cs);
        hi[e] = bf16_to_f32(f32_to_bf16(f));
        lo[e] = f - hi[e];
      }
      u32x4 ph = {pack_bf16x2(hi[0], hi[1]), pack_bf16x2(hi[2], hi[3]), pack_bf16x2(hi[4], hi[5]), pack_bf16x2(hi[6], hi[7])};
      u32x4 pl = {pack_bf16x2(lo[0], lo[1]), pack_bf16x2(lo[2], lo[3]), pack_bf16x2(lo[4], lo[5]), pack_bf16x2(lo[6], lo[7])};
      ahi[kk] = __builtin_bit_cast(bf16x8, ph);
      alo[kk] = __builtin_bit_cast(bf16x8, pl);
    });
    for (int it = 0; it < iters; ++it) {
      // 512 groups of 16 points per pass; a wave takes 128 of them, 32 per product
      static_for<0, 4>([&](auto ss) {
        constexpr int set = decltype(ss)::value;
        const int q = 128 * wave + 32 * set + i32, blk = q >> 4, m = q & 15;
        float2* pb = row + sphys(blk * 256 + m);
        float re[8], im[8];
        static_for<0, 8>([&](auto ee) {
          constexpr int e = decltype(ee)::value;
          const float2 v = pb[spoff(16 * e) + (half ? spoff(128) : 0)];
          re[e] = v.x;
          im[e] = v.y;
        });
        auto split = [&](const float (&x)[8], bf16x8& h8, bf16x8& l8) __attribute__((always_inline)) {
          uint32_t ph[4], pl[4];
          static_for<0, 4>([&](auto pp) {
            constexpr int pi = decltype(pp)::value;
            ph[pi] = pack_bf16x2(x[2 * pi], x[2 * pi + 1]);
            const float l0 = x[2 * pi] - __uint_as_float(ph[pi] << 16), l1 = x[2 * pi + 1] - __uint_as_float(ph[pi] & 0xffff0000u);
            pl[pi] = pack_bf16x2(l0, l1);
          });
          u32x4 a = {ph[0], ph[1], ph[2], ph[3]}, b = {pl[0], pl[1], pl[2], pl[3]};
          h8 = __builtin_bit_cast(bf16x8, a);
          l8 = __builtin_bit_cast(bf16x8, b);
        };
        bf16x8 rh, rl, ih, il;
        split(re, rh, rl);
        split(im, ih, il);
        floatx16 acc;
        static_for<0, 16>([&](auto vv) { acc[decltype(vv)::value] = 0.f; });
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(alo[0], rh, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ahi[0], rl, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(alo[1], ih, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ahi[1], il, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ahi[0], rh, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ahi[1], ih, acc, 0, 0, 0);
        // accumulator element 4 a + b: row 8 a + 4 half + b; rows below 16 are Re Y_k, rows 16 + k are Im Y_k
        static_for<0, 2>([&](auto aa) {
          constexpr int a = decltype(aa)::value;
          static_for<0, 4>([&](auto bb) {
            constexpr int b = decltype(bb)::value;
            const int k = 8 * a + 4 * half + b;
            cf y = {acc[4 * a + b], acc[4 * (a + 2) + b]};
            const float2 w = tab2[k * 16 + m];
            if (k > 0) y = cmul(y, cf{w.x, w.y});
            pb[spoff(128 * a + 16 * b) + (half ? spoff(64) : 0)] = make_float2(y.re, y.im);
          });
        });
      });
      __syncthreads();
    }
  }
  for (int i = t; i < P::L; i += 256) g[i] = row[sphys(i)];
}

// ---------------------------------------------------------------------------------------------
// L2 -> LDS stream: what one compute unit can pull out of L2 when all of them do.  Every workgroup (512 threads, one
// per compute unit) copies the same `region` (so everything is an L2 hit after the first pass) into LDS, 40 KB per
// iteration, a barrier per iteration, in one of three ways:
//   mode 0  direct loads (global_load_lds_dwordx4), an instruction gathering sixteen 64-byte row pieces (row stride
//           384 bytes: an MFMA operand block taken straight from a row-major bf16 matrix with 192 columns)
//   mode 1  direct loads, an instruction copying 1 KB of contiguous memory
//   mode 2  plain 16-byte loads into registers, software-pipelined one iteration ahead, then LDS writes
//   mode 3  direct loads, an instruction gathering eight whole 128-byte lines (row stride 1536 bytes: a 64-wide K
//           chunk of eight rows of a row-major bf16 matrix with 768 columns)
// ---------------------------------------------------------------------------------------------
template <int MODE>
__global__ __launch_bounds__(512) void probe_l2_stream_kernel(const unsigned char* __restrict__ src, long region, int iters,
                                                              float* __restrict__ sink) {
  extern __shared__ __attribute__((aligned(16))) unsigned char stage[];      // 4 stages x 40 KB
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const unsigned lds0 = (unsigned)(uintptr_t)stage;
  const unsigned voff = MODE == 0 ? (lane & 15) * 384 + (lane >> 4) * 16 : MODE == 3 ? (lane >> 3) * 1536 + (lane & 7) * 16 : lane * 16;
  const long span = region - 16 * 1536 - 1024;
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  if constexpr (MODE != 2) {
    long off = 0;
    for (int it = 0; it < iters; ++it) {
      for (int j = 0; j < 5; ++j) {
        const int blk = wave * 5 + j;
        long o = MODE == 0 ? (blk % 6) * 64 + (long)((blk / 6) * 16) * 384 + off
               : MODE == 3 ? (blk % 12) * 128 + (long)((blk / 12) * 8) * 1536 + off : off + (long)blk * 1024;
        o %= span;
        const unsigned dst = lds0 + ((it & 3) * 40 + blk) * 1024;
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(voff), "s"(src + o) : "memory");
      }
      off += MODE == 0 ? 384 * 32 : MODE == 3 ? 1536 * 32 : 40 * 1024;
      __builtin_amdgcn_s_waitcnt(0x0F70 | 5);      // all but the newest batch have landed
      __syncthreads();
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);
  } else {
    u32x4 ra[5], rb[5];
    auto ld = [&](u32x4* r, int it) __attribute__((always_inline)) {
#pragma unroll
      for (int j = 0; j < 5; ++j) r[j] = *reinterpret_cast<const u32x4*>(src + ((long)it * 40 * 1024 + (long)(wave * 5 + j) * 1024) % span + voff);
    };
    auto st = [&](const u32x4* r, int it) __attribute__((always_inline)) {
#pragma unroll
      for (int j = 0; j < 5; ++j) *reinterpret_cast<u32x4*>(stage + ((it & 3) * 40 + wave * 5 + j) * 1024 + lane * 16) = r[j];
    };
    ld(ra, 0);
    for (int it = 0; it < iters; it += 2) {
      ld(rb, it + 1);
      st(ra, it);
      __syncthreads();
      ld(ra, it + 2);
      st(rb, it + 1);
      __syncthreads();
    }
    if (ra[0].x == 0x12345678u) sink[tid] = 2.f;
  }
  __syncthreads();
  if (*reinterpret_cast<const uint32_t*>(stage + 16 * tid) == 0x12345678u) sink[tid] = 1.f;
}

}  // namespace m2

using namespace m2;

extern "C" int m2_probe_mfma_fwd(int lds_reads_per_mfma, int valu_per_mfma, int waves_per_simd, int iters, float* sink,
                                 long long* mfma_per_wave, int* waves, void* stream) {
  if (!sink || iters <= 0) return set_error(M2_ERR_ARG, "m2_probe_mfma_fwd: null sink or non-positive iters");
  if (mfma_per_wave) *mfma_per_wave = 12LL * iters;
  if (waves) *waves = num_cus() * 4 * waves_per_simd;
  hipStream_t st = (hipStream_t)stream;
#define M2_PROBE_CASE(R, V)                                                                       \
  if (lds_reads_per_mfma == R && valu_per_mfma == V)                                              \
    return waves_per_simd == 1 ? launch_probe<R, V, 256>(sink, iters, st)                         \
         : waves_per_simd == 2 ? launch_probe<R, V, 512>(sink, iters, st)                         \
         : set_error(M2_ERR_UNSUPPORTED, "m2_probe_mfma_fwd: waves_per_simd must be 1 or 2");
  M2_PROBE_CASE(0, 0) M2_PROBE_CASE(1, 0) M2_PROBE_CASE(2, 0) M2_PROBE_CASE(1, 4) M2_PROBE_CASE(1, 6) M2_PROBE_CASE(1, 11)
#undef M2_PROBE_CASE
  return set_error(M2_ERR_UNSUPPORTED, "m2_probe_mfma_fwd: (reads, valu) must be one of (0,0) (1,0) (2,0) (1,4) (1,6) (1,11)");
}

extern "C" int m2_probe_dft16_pass_fwd(int use_mfma, int iters, int nrows, float* rows, void* stream) {
  if (!rows || iters <= 0 || nrows <= 0) return set_error(M2_ERR_ARG, "m2_probe_dft16_pass_fwd: null rows or non-positive count");
  const size_t lds = (size_t)ProbePlan::WG_LDS * sizeof(float2);
  auto kern = use_mfma ? probe_dft16_kernel<true> : probe_dft16_kernel<false>;
  hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return set_error(M2_ERR_LAUNCH, "hipFuncSetAttribute(probe_dft16): %s", hipGetErrorString(e));
  hipLaunchKernelGGL(kern, dim3(nrows), dim3(256), lds, (hipStream_t)stream, reinterpret_cast<float2*>(rows), iters);
  return check_launch("probe_dft16");
}

extern "C" int m2_probe_l2_stream_fwd(int mode, int iters, const void* region, long region_bytes, float* sink, int* workgroups,
                                      void* stream) {
  if (!region || !sink || iters <= 0) return set_error(M2_ERR_ARG, "m2_probe_l2_stream_fwd: null pointer or non-positive iters");
  if (region_bytes < (1 << 20)) return set_error(M2_ERR_ARG, "m2_probe_l2_stream_fwd: region of %ld bytes, need at least 1 MiB", region_bytes);
  if (mode < 0 || mode > 3) return set_error(M2_ERR_UNSUPPORTED, "m2_probe_l2_stream_fwd: mode must be 0 .. 3");
  const int lds = 160 * 1024;
  auto kern = mode == 0 ? probe_l2_stream_kernel<0> : mode == 1 ? probe_l2_stream_kernel<1> : mode == 2 ? probe_l2_stream_kernel<2>
                        : probe_l2_stream_kernel<3>;
  hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
  if (e != hipSuccess) return set_error(M2_ERR_LAUNCH, "hipFuncSetAttribute(probe_l2_stream): %s", hipGetErrorString(e));
  if (workgroups) *workgroups = num_cus();
  hipLaunchKernelGGL(kern, dim3(num_cus()), dim3(512), lds, (hipStream_t)stream, (const unsigned char*)region, region_bytes,
                     iters & ~1, sink);
  return check_launch("probe_l2_stream");
}
