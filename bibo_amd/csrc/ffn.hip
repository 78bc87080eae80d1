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

}  // namespace

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
