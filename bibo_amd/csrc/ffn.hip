// RMSNorm in front of the MoE block, as the caller of the block applies it: BiBoRMSNorm.forward
// (src/modeling/norm.py:19-24) inside BiBoDecoderLayer._ffn_forward (src/modeling/layers.py:59-60).
//   out = weight * round_to_dtype(x * rsqrt(mean(x^2) + eps)),   statistics in fp32
// One wave per row; the row stays in registers between the two passes when it is short enough.
#include "common.h"

namespace bibo {
namespace {

constexpr int kNormMaxPerLane = 32;      // elements a lane keeps in registers (rows up to 2048 wide)

template <typename TIn>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const TIn* __restrict__ x, const float* __restrict__ weight,
                                                      float eps, int T, int H, TIn* __restrict__ out) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= T) return;
  const TIn* xr = x + (size_t)row * H;
  TIn* orow = out + (size_t)row * H;
  float v[kNormMaxPerLane];
  float ss = 0.f;
  const bool in_regs = H <= kNormMaxPerLane * kWave;
  if (in_regs) {
#pragma unroll
    for (int u = 0; u < kNormMaxPerLane; ++u) {
      const int c = u * kWave + lane;
      v[u] = (c < H) ? to_float(xr[c]) : 0.f;
      ss = fmaf(v[u], v[u], ss);
    }
  } else {
    for (int c = lane; c < H; c += kWave) { const float f = to_float(xr[c]); ss = fmaf(f, f, ss); }
  }
  ss = wave_sum(ss);
  const float rinv = rsqrtf(ss / (float)H + eps);                                   // norm.py:22-23
  if (in_regs) {
#pragma unroll
    for (int u = 0; u < kNormMaxPerLane; ++u) {
      const int c = u * kWave + lane;
      if (c < H) orow[c] = from_float<TIn>(weight[c] * to_float(from_float<TIn>(v[u] * rinv)));   // norm.py:24
    }
  } else {
    for (int c = lane; c < H; c += kWave)
      orow[c] = from_float<TIn>(weight[c] * to_float(from_float<TIn>(to_float(xr[c]) * rinv)));
  }
}

// bf16 rows of up to 2048 elements, H % 8 == 0, 16-byte aligned: 16-byte accesses, the row stays in registers
__global__ __launch_bounds__(256) void rmsnorm_bf16x8_kernel(const bf16_t* __restrict__ x, const float* __restrict__ weight,
                                                             float eps, int T, int H, bf16_t* __restrict__ out) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= T) return;
  const int nchunk = H / 8;
  const bf16x8* xr = reinterpret_cast<const bf16x8*>(x + (size_t)row * H);
  bf16x8 v[4];
  float ss = 0.f;
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int c = u * kWave + lane;
    if (c < nchunk) {
      v[u] = xr[c];
#pragma unroll
      for (int q = 0; q < 8; ++q) ss = fmaf((float)v[u][q], (float)v[u][q], ss);
    }
  }
  ss = wave_sum(ss);
  const float rinv = rsqrtf(ss / (float)H + eps);                                   // norm.py:22-23
  bf16x8* orow = reinterpret_cast<bf16x8*>(out + (size_t)row * H);
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int c = u * kWave + lane;
    if (c < nchunk) {
      bf16x8 o;
#pragma unroll
      for (int q = 0; q < 8; ++q) o[q] = (bf16_t)(weight[c * 8 + q] * (float)(bf16_t)((float)v[u][q] * rinv));   // norm.py:24
      orow[c] = o;
    }
  }
}

// Depth mix of Block Attention Residuals (apply_attention_residual, exp/modeling_bibo.py:119-232, softmax scores,
// dense): candidates = the completed block representatives and the running prefix sum of a token; score of a
// candidate = rsqrt(mean(c^2) + eps) * <c, score_w> with score_w = norm weight * pseudo-query (fp32); out = the
// candidates averaged with the softmax of their scores, fp32, rounded once.  One wave per token, the candidates' rows
// stay in registers (two 16-byte granules per lane: H <= 1024).
constexpr int kAttnResMaxCand = 8;
struct AttnResPtrs {
  const bf16_t* c[kAttnResMaxCand];
};

__global__ __launch_bounds__(256) void attn_res_kernel(AttnResPtrs cand, int n_cand, const float* __restrict__ score_w,
                                                       float eps, int T, int H, bf16_t* __restrict__ out) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= T) return;
  const int nchunk = H / 8;
  float sw[2][8];
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int c = u * kWave + lane;
#pragma unroll
    for (int q = 0; q < 8; ++q) sw[u][q] = c < nchunk ? score_w[c * 8 + q] : 0.f;
  }
  bf16x8 v[kAttnResMaxCand][2];
  float score[kAttnResMaxCand];
  float mx = -3.0e38f;
#pragma unroll
  for (int i = 0; i < kAttnResMaxCand; ++i)
    if (i < n_cand) {
      const bf16x8* r = reinterpret_cast<const bf16x8*>(cand.c[i] + (size_t)row * H);
      float ss = 0.f, dot = 0.f;
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int c = u * kWave + lane;
        if (c < nchunk) {
          v[i][u] = r[c];
#pragma unroll
          for (int q = 0; q < 8; ++q) {
            const float f = (float)v[i][u][q];
            ss = fmaf(f, f, ss);
            dot = fmaf(f, sw[u][q], dot);
          }
        }
      }
      ss = wave_sum(ss);
      dot = wave_sum(dot);
      score[i] = dot * rsqrtf(ss / (float)H + eps);
      mx = fmaxf(mx, score[i]);
    }
  float den = 0.f;
#pragma unroll
  for (int i = 0; i < kAttnResMaxCand; ++i)
    if (i < n_cand) {
      score[i] = __expf(score[i] - mx);
      den += score[i];
    }
  const float inv = 1.f / den;
  bf16x8* orow = reinterpret_cast<bf16x8*>(out + (size_t)row * H);
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int c = u * kWave + lane;
    if (c < nchunk) {
      float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < kAttnResMaxCand; ++i)
        if (i < n_cand) {
          const float pr = score[i] * inv;
#pragma unroll
          for (int q = 0; q < 8; ++q) acc[q] = fmaf(pr, (float)v[i][u][q], acc[q]);
        }
      bf16x8 o;
#pragma unroll
      for (int q = 0; q < 8; ++q) o[q] = (bf16_t)acc[q];
      orow[c] = o;
    }
  }
}

}  // namespace

bool attn_res_supported(int H, int n_cand, int dtype) {
  return dtype == BIBO_DTYPE_BF16 && H % 8 == 0 && H <= 1024 && n_cand >= 1 && n_cand <= kAttnResMaxCand;
}

hipError_t launch_attn_res(const void* const* cands, int n_cand, const float* score_w, float eps, int T, int H, void* out,
                           hipStream_t s) {
  if (T == 0) return hipSuccess;
  AttnResPtrs p;
  for (int i = 0; i < kAttnResMaxCand; ++i) p.c[i] = static_cast<const bf16_t*>(i < n_cand ? cands[i] : cands[0]);
  hipLaunchKernelGGL(attn_res_kernel, dim3((T + 3) / 4), dim3(256), 0, s, p, n_cand, score_w, eps, T, H,
                     static_cast<bf16_t*>(out));
  return hipGetLastError();
}

hipError_t launch_rmsnorm(const void* x, const float* weight, float eps, int T, int H, int dtype, void* out,
                          hipStream_t s) {
  if (T == 0) return hipSuccess;
  const int grid = (T + 3) / 4;
  const bool vec = dtype == BIBO_DTYPE_BF16 && (H % 8) == 0 && H <= 2048 &&
                   ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
  if (vec)
    hipLaunchKernelGGL(rmsnorm_bf16x8_kernel, dim3(grid), dim3(256), 0, s, static_cast<const bf16_t*>(x), weight, eps, T, H,
                       static_cast<bf16_t*>(out));
  else if (dtype == BIBO_DTYPE_BF16)
    hipLaunchKernelGGL(rmsnorm_kernel<bf16_t>, dim3(grid), dim3(256), 0, s, static_cast<const bf16_t*>(x), weight, eps, T,
                       H, static_cast<bf16_t*>(out));
  else
    hipLaunchKernelGGL(rmsnorm_kernel<float>, dim3(grid), dim3(256), 0, s, static_cast<const float*>(x), weight, eps, T,
                       H, static_cast<float*>(out));
  return hipGetLastError();
}

}  // namespace bibo
