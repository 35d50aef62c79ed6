// Block-diagonal ("Monarch") linear layers of the M2-BERT GLU MLP on bf16 MFMA, and the LayerNorm
// that closes the layer.
//
//   out[m, k q + j] = sum_i x[m, k p + i] w[k, j, i]          (bert/src/mm/blockdiag_multiply.py:19-34,49-60)
//
// `blockdiag_kernel<GLU=true>`  computes gelu_erf(gate) * value in the epilogue, where gate column j
// (block j / q) pairs with value column I + j (block j / q + nb/2)   (bert/src/bert_layers.py:482-502).
// `blockdiag_kernel<GLU=false>` adds bias and a residual                (bert/src/bert_layers.py:504-506,
//                                                                        bert/src/mm/structured_linear.py:65-69).
// `layernorm_kernel` normalises rows and writes the three forms the next layer reads.
//
// MFMA: v_mfma_f32_32x32x16_bf16.  Lane (i = lane % 32, h = lane / 32) supplies A[i][8h .. 8h+7] and
// B[8h .. 8h+7][i]; both operands are K-contiguous in memory (x row-major, w[k] is (q, p)), so every
// operand register is one 16-byte load.  Accumulator element v of a lane is row 8 (v/4) + 4 h + v%4,
// column i.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "m2_internal.h"

namespace m2 {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ bf16x8 ld8(const uint16_t* p) {
  return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p));
}

__device__ __forceinline__ float gelu_erf(float x) { return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f)); }

// Workgroup = 4 waves as 2 (rows) x 2 (cols); wave tile 64 rows x 32 cols; workgroup tile 128 x 64.
// grid (ceil(M / 128), ncol_tiles) where ncol_tiles counts 64-wide tiles over the OUTPUT columns
// (I for GLU, out_features otherwise).  Requires q % 64 == 0 (GLU: (q) % 64 == 0 too), p % 16 == 0.
template <bool GLU, typename OUT>
__global__ __launch_bounds__(256) void blockdiag_kernel(
    const uint16_t* __restrict__ x,      // (M, nb p) bf16
    const uint16_t* __restrict__ w,      // (nb, q, p) bf16
    const float* __restrict__ bias,      // (nb q) or null            [GLU: unused]
    const uint16_t* __restrict__ resid,  // (M, nb q) bf16 or null    [GLU: unused]
    OUT* __restrict__ out,               // GLU: (M, nb q / 2) ; else (M, nb q)
    int M, int nb, int p, int q) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, i32 = lane & 31, half = lane >> 5;
  const int wm = wave >> 1, wn = wave & 1;
  const int m0 = blockIdx.x * 128 + wm * 64;
  const int n0 = blockIdx.y * 64 + wn * 32;          // output column of this wave's tile
  const int in_f = nb * p;
  const int blk = n0 / q, jj = n0 % q;               // block and column inside the block (gate block for GLU)
  const int out_cols = GLU ? nb * q / 2 : nb * q;

  // rows beyond M are clamped for loads and masked at the store
  int rowA[2];
  for (int a = 0; a < 2; ++a) {
    int r = m0 + 32 * a + i32;
    rowA[a] = r < M ? r : M - 1;
  }
  const uint16_t* xg = x + (long)blk * p + 8 * half;
  const uint16_t* wg = w + ((long)blk * q + jj + i32) * p + 8 * half;
  const uint16_t* xv = GLU ? x + (long)(blk + nb / 2) * p + 8 * half : nullptr;
  const uint16_t* wv = GLU ? w + ((long)(blk + nb / 2) * q + jj + i32) * p + 8 * half : nullptr;

  floatx16 accg[2], accv[2];
  for (int a = 0; a < 2; ++a)
    for (int v = 0; v < 16; ++v) { accg[a][v] = 0.f; accv[a][v] = 0.f; }

  for (int k = 0; k < p; k += 16) {
    const bf16x8 bg = ld8(wg + k);
    bf16x8 ag[2];
    for (int a = 0; a < 2; ++a) ag[a] = ld8(xg + (long)rowA[a] * in_f + k);
    for (int a = 0; a < 2; ++a) accg[a] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ag[a], bg, accg[a], 0, 0, 0);
    if constexpr (GLU) {
      const bf16x8 bv = ld8(wv + k);
      bf16x8 av[2];
      for (int a = 0; a < 2; ++a) av[a] = ld8(xv + (long)rowA[a] * in_f + k);
      for (int a = 0; a < 2; ++a) accv[a] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[a], bv, accv[a], 0, 0, 0);
    }
  }

  const int col = n0 + i32;
  const float bcol = (!GLU && bias) ? bias[col] : 0.f;
  for (int a = 0; a < 2; ++a)
    for (int v = 0; v < 16; ++v) {
      const int r = m0 + 32 * a + 8 * (v >> 2) + 4 * half + (v & 3);
      if (r >= M) continue;
      float val;
      if constexpr (GLU) {
        val = gelu_erf(accg[a][v]) * accv[a][v];
      } else {
        val = accg[a][v] + bcol;
        if (resid) val += bf16_to_f32(resid[(long)r * out_cols + col]);
      }
      if constexpr (sizeof(OUT) == 2) out[(long)r * out_cols + col] = f32_to_bf16(val);
      else out[(long)r * out_cols + col] = val;
    }
}

// LayerNorm over the last dimension of x (M, d) fp32, eps inside the square root.
// Workgroup = 256 threads handles 64 rows: phase 1 one wave per row (16 rows per wave) writes the
// row-major outputs and keeps mean / rstd in LDS; phase 2 re-reads the (cache-resident) rows with
// lanes along the token axis and writes the channel-major copy with 256-byte stores.
// d % 64 == 0, d <= 64 * kMaxPerLane.
constexpr int kMaxPerLane = 32;
__global__ __launch_bounds__(256) void layernorm_kernel(const float* __restrict__ x, const float* __restrict__ gamma,
                                                        const float* __restrict__ beta, float eps,
                                                        float* __restrict__ out_f32,       // (M, d) or null
                                                        uint16_t* __restrict__ out_bf16,   // (M, d) or null
                                                        float* __restrict__ out_t,         // (d, M) or null
                                                        int M, int d) {
  __shared__ float s_mean[64], s_rstd[64];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int m0 = blockIdx.x * 64;
  const int per = d / 64;
  for (int rr = 0; rr < 16; ++rr) {
    const int rloc = wave * 16 + rr;
    const int m = m0 + rloc;
    if (m >= M) {
      if (lane == 0) { s_mean[rloc] = 0.f; s_rstd[rloc] = 0.f; }
      continue;
    }
    const float* xr = x + (long)m * d;
    float v[kMaxPerLane];
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < kMaxPerLane; ++i)
      if (i < per) { v[i] = xr[lane + 64 * i]; sum += v[i]; }
    for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o);
    const float mean = sum / (float)d;
    float sq = 0.f;
#pragma unroll
    for (int i = 0; i < kMaxPerLane; ++i)
      if (i < per) { const float c = v[i] - mean; sq += c * c; }
    for (int o = 32; o > 0; o >>= 1) sq += __shfl_xor(sq, o);
    const float rstd = rsqrtf(sq / (float)d + eps);
    if (lane == 0) { s_mean[rloc] = mean; s_rstd[rloc] = rstd; }
#pragma unroll
    for (int i = 0; i < kMaxPerLane; ++i)
      if (i < per) {
        const int c = lane + 64 * i;
        const float o = (v[i] - mean) * rstd * gamma[c] + beta[c];
        if (out_f32) out_f32[(long)m * d + c] = o;
        if (out_bf16) out_bf16[(long)m * d + c] = f32_to_bf16(o);
      }
  }
  if (!out_t) return;
  __syncthreads();
  const int m = m0 + lane;
  const bool ok = m < M;
  const float mean = s_mean[lane], rstd = s_rstd[lane];
  const float* xr = x + (long)(ok ? m : M - 1) * d;
  for (int c0 = wave * 16; c0 < d; c0 += 64) {       // 16 channels per wave per step
    float4 q[4];
    for (int j = 0; j < 4; ++j) q[j] = *reinterpret_cast<const float4*>(xr + c0 + 4 * j);
    const float vals[16] = {q[0].x, q[0].y, q[0].z, q[0].w, q[1].x, q[1].y, q[1].z, q[1].w,
                            q[2].x, q[2].y, q[2].z, q[2].w, q[3].x, q[3].y, q[3].z, q[3].w};
    if (ok)
      for (int j = 0; j < 16; ++j) {
        const int c = c0 + j;
        out_t[(long)c * M + m] = (vals[j] - mean) * rstd * gamma[c] + beta[c];
      }
  }
}

}  // namespace m2

using namespace m2;

static int check_blockdiag(const char* who, int M, int nb, int p, int q, bool glu) {
  if (M <= 0 || nb <= 0 || p <= 0 || q <= 0) return set_error(M2_ERR_ARG, "%s: sizes must be positive (M=%d nb=%d p=%d q=%d)", who, M, nb, p, q);
  if (p % 16 != 0) return set_error(M2_ERR_UNSUPPORTED, "%s: in_features/nblocks=%d must be a multiple of 16", who, p);
  if (q % 64 != 0) return set_error(M2_ERR_UNSUPPORTED, "%s: out_features/nblocks=%d must be a multiple of 64", who, q);
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
  dim3 grid((M + 127) / 128, intermediate / 64);
  hipLaunchKernelGGL((blockdiag_kernel<true, uint16_t>), grid, dim3(256), 0, (hipStream_t)stream, (const uint16_t*)x,
                     (const uint16_t*)w, (const float*)nullptr, (const uint16_t*)nullptr, (uint16_t*)out, M, nblocks, p, q);
  return check_launch("blockdiag_glu");
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
  dim3 grid((M + 127) / 128, out_features / 64);
  if (out_dtype == M2_DTYPE_F32)
    hipLaunchKernelGGL((blockdiag_kernel<false, float>), grid, dim3(256), 0, (hipStream_t)stream, (const uint16_t*)x,
                       (const uint16_t*)w, bias, (const uint16_t*)residual, (float*)out, M, nblocks, p, q);
  else
    hipLaunchKernelGGL((blockdiag_kernel<false, uint16_t>), grid, dim3(256), 0, (hipStream_t)stream, (const uint16_t*)x,
                       (const uint16_t*)w, bias, (const uint16_t*)residual, (uint16_t*)out, M, nblocks, p, q);
  return check_launch("blockdiag_linear");
}

extern "C" int m2_layernorm_fwd(const float* x, const float* gamma, const float* beta, float eps, float* out_f32,
                                void* out_bf16, float* out_channel_major, int M, int d, void* stream) {
  if (!x || !gamma || !beta) return set_error(M2_ERR_ARG, "m2_layernorm_fwd: null pointer");
  if (M <= 0 || d <= 0 || d % 64 != 0 || d > 64 * kMaxPerLane)
    return set_error(M2_ERR_UNSUPPORTED, "m2_layernorm_fwd: need M > 0 and d a multiple of 64 up to %d (M=%d d=%d)",
                     64 * kMaxPerLane, M, d);
  hipLaunchKernelGGL(layernorm_kernel, dim3((M + 63) / 64), dim3(256), 0, (hipStream_t)stream, x, gamma, beta, eps,
                     out_f32, (uint16_t*)out_bf16, out_channel_major, M, d);
  return check_launch("layernorm");
}
