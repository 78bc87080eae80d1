// Generic expert kernels: one workgroup per routed row, any H and I, bf16 or fp32 operands, fp32
// accumulation.  They serve shapes the MFMA tiles do not cover and fp32 modules, and double as an
// independent implementation the MFMA kernels are cross-checked against.
// Follow BiBoFusedExperts.forward, src/modeling/ffn/moe.py:73-101 of the reference.
#include "common.h"

namespace bibo {
namespace {

__device__ __forceinline__ int find_expert(const int32_t* __restrict__ offsets, int E, int row, int* sh) {
  // offsets is non-decreasing; the owner is the last expert with offsets[e] <= row < offsets[e+1]
  const int tid = threadIdx.x;
  if (tid < E && offsets[tid] <= row && row < offsets[tid + 1]) *sh = tid;
  __syncthreads();
  return *sh;
}

// hidden[row, :] = r^p * SiLU(g/r) * up   (moe.py:84-92)
template <typename TIn>
__global__ __launch_bounds__(256) void gateup_generic_kernel(const TIn* __restrict__ x, const TIn* __restrict__ wgu,
                                                             const float* __restrict__ theta,
                                                             const int32_t* __restrict__ offsets,
                                                             const int32_t* __restrict__ perm_token, int H, int E,
                                                             int I, int act, TIn* __restrict__ hidden) {
  extern __shared__ float smem[];
  float* xs = smem;            // [H]
  float* gu = smem + H;        // [2I]
  __shared__ int sh_e;
  __shared__ float red[4];
  const int row = blockIdx.x;
  if (row >= offsets[E]) return;
  const int e = find_expert(offsets, E, row, &sh_e);
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const TIn* xr = x + (size_t)perm_token[row] * H;                     // moe.py:81
  for (int h = tid; h < H; h += 256) xs[h] = to_float(xr[h]);
  __syncthreads();
  const TIn* wbase = wgu + (size_t)e * 2 * I * H;
  for (int j = wave; j < 2 * I; j += 4) {                              // moe.py:84
    const TIn* wrow = wbase + (size_t)j * H;
    float acc = 0.f;
    for (int h = lane; h < H; h += kWave) acc = fmaf(xs[h], to_float(wrow[h]), acc);
    acc = wave_sum(acc);
    if (lane == 0) gu[j] = acc;
  }
  __syncthreads();
  float ss = 0.f;
  for (int i = tid; i < I; i += 256) ss = fmaf(gu[i], gu[i], ss);
  ss = wave_sum(ss);
  if (lane == 0) red[wave] = ss;
  __syncthreads();
  const float ms = ((red[0] + red[1]) + red[2]) + red[3];
  const float r = act == BIBO_ACT_SILU ? 1.f : sqrtf(ms / (float)I + kNormSiluEps);   // moe.py:88
  const float p = radial_exponent(theta, e, act);                      // moe.py:89
  const float gain = act == BIBO_ACT_SILU ? 1.f : powf(r, p);
  for (int i = tid; i < I; i += 256) {
    const float z = gu[i] / r;
    const float act = z / (1.f + expf(-z)) * gain;                     // SiLU(g/r) * r^p
    hidden[(size_t)row * I + i] = from_float<TIn>(act * gu[I + i]);    // * up (moe.py:92)
  }
}

// yw[slot, :] = w[slot] * (hidden[row, :] @ w_down[e]^T)   (moe.py:92-93)
template <typename TIn>
__global__ __launch_bounds__(256) void down_generic_kernel(const TIn* __restrict__ hidden, const TIn* __restrict__ wd,
                                                           const float* __restrict__ w,
                                                           const int32_t* __restrict__ offsets,
                                                           const int32_t* __restrict__ perm_slot, int H, int E, int I,
                                                           float* __restrict__ yw) {
  extern __shared__ float smem[];
  float* hs = smem;            // [I]
  __shared__ int sh_e;
  const int row = blockIdx.x;
  if (row >= offsets[E]) return;
  const int e = find_expert(offsets, E, row, &sh_e);
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  for (int i = tid; i < I; i += 256) hs[i] = to_float(hidden[(size_t)row * I + i]);
  __syncthreads();
  const int slot = perm_slot[row];
  const float ws = w[slot];
  const TIn* wbase = wd + (size_t)e * H * I;
  for (int h = wave; h < H; h += 4) {
    const TIn* wrow = wbase + (size_t)h * I;
    float acc = 0.f;
    for (int i = lane; i < I; i += kWave) acc = fmaf(hs[i], to_float(wrow[i]), acc);
    acc = wave_sum(acc);
    if (lane == 0) yw[(size_t)slot * H + h] = ws * acc;
  }
}

// out[t, :] = round(residual[t, :] + sum_j contribution(t, j))  in fp32, ascending j   (moe.py:93-101; the residual
// add of the caller, src/modeling/layers.py:62, when `residual` is given).  contribution = yw[t*k + j, :] for a GLU
// expert; with `idx` given, +/- w[t,j] * x[t, :] for a +/-Identity special (moe.py:95-99) and nothing for an index
// outside [0, E_glu + n_pos + n_neg) (no kernel wrote that slot's row).
template <typename TX>
__device__ __forceinline__ bool special_slot(const CombineArgs& a, size_t slot, int* sign) {
  *sign = 0;
  if (a.idx == nullptr) return false;
  const int e = a.idx[slot];
  if ((unsigned)e >= (unsigned)(a.E_glu + a.n_pos + a.n_neg)) return true;       // skipped
  if (e < a.E_glu) return false;
  *sign = e < a.E_glu + a.n_pos ? 1 : -1;
  return true;
}

template <typename TY, typename TOut>
__global__ __launch_bounds__(256) void combine_kernel(const TY* __restrict__ yw, CombineArgs a, int T, int H, int k,
                                                      TOut* __restrict__ out) {
  const size_t n = (size_t)T * H;
  const TOut* x = static_cast<const TOut*>(a.x);
  const TOut* residual = static_cast<const TOut*>(a.residual);
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
    const size_t t = i / H, h = i - t * H;
    float acc = 0.f;
    for (int j = 0; j < k; ++j) {
      int sign;
      if (special_slot<TOut>(a, t * k + j, &sign)) {
        if (sign != 0) acc += (float)sign * a.w[t * k + j] * to_float(x[i]);
        continue;
      }
      acc += to_float(yw[(t * k + j) * H + h]);
    }
    if (residual != nullptr) acc = (a.round_block ? to_float(from_float<TOut>(acc)) : acc) + to_float(residual[i]);
    out[i] = from_float<TOut>(acc);
  }
}

// bf16 slot rows -> bf16 output, 8 columns (16 bytes) per thread, fp32 sum in ascending j
__global__ __launch_bounds__(256) void combine_bf16x8_kernel(const bf16_t* __restrict__ yw, CombineArgs a, int T, int H8,
                                                             int k, bf16_t* __restrict__ out) {
  const size_t n = (size_t)T * H8;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
    const size_t t = i / H8, c = i - t * H8;
    float acc[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) acc[q] = 0.f;
    const bf16x8* src = reinterpret_cast<const bf16x8*>(yw) + (t * k) * H8 + c;
    for (int j = 0; j < k; ++j) {
      int sign;
      if (special_slot<bf16_t>(a, t * k + j, &sign)) {
        if (sign != 0) {
          const float sw = (float)sign * a.w[t * k + j];
          const bf16x8 xv = reinterpret_cast<const bf16x8*>(a.x)[i];
#pragma unroll
          for (int q = 0; q < 8; ++q) acc[q] += sw * (float)xv[q];
        }
        continue;
      }
      const bf16x8 v = src[(size_t)j * H8];
#pragma unroll
      for (int q = 0; q < 8; ++q) acc[q] += (float)v[q];
    }
    if (a.residual != nullptr) {
      const bf16x8 r = reinterpret_cast<const bf16x8*>(a.residual)[i];
#pragma unroll
      for (int q = 0; q < 8; ++q) acc[q] = (a.round_block ? (float)(bf16_t)acc[q] : acc[q]) + (float)r[q];
    }
    bf16x8 o;
#pragma unroll
    for (int q = 0; q < 8; ++q) o[q] = (bf16_t)acc[q];
    reinterpret_cast<bf16x8*>(out)[i] = o;
  }
}

// fp32 slot rows -> bf16 output, 4 columns per thread: the decode-size combine, whose duration is one round trip of
// its loads, issues a quarter of the threads and all k loads of a thread at once.  Same sum as combine_kernel.
__global__ __launch_bounds__(256) void combine_f32x4_kernel(const float* __restrict__ yw, CombineArgs a, int T, int H4,
                                                            int k, bf16_t* __restrict__ out) {
  const size_t n = (size_t)T * H4;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
    const size_t t = i / H4, c = i - t * H4;
    floatx4 v[kMaxK];
    int sign[kMaxK];
    bool special[kMaxK];
    const floatx4* src = reinterpret_cast<const floatx4*>(yw) + (t * k) * H4 + c;
#pragma unroll
    for (int j = 0; j < kMaxK; ++j)
      if (j < k) {
        special[j] = special_slot<bf16_t>(a, t * k + j, &sign[j]);
        if (!special[j]) v[j] = src[(size_t)j * H4];
      }
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < kMaxK; ++j)
      if (j < k) {
        if (special[j]) {
          if (sign[j] != 0) {
            const float sw = (float)sign[j] * a.w[t * k + j];
            const bf16x4 xv = reinterpret_cast<const bf16x4*>(a.x)[i];
#pragma unroll
            for (int q = 0; q < 4; ++q) acc[q] += sw * (float)xv[q];
          }
        } else {
#pragma unroll
          for (int q = 0; q < 4; ++q) acc[q] += v[j][q];
        }
      }
    if (a.residual != nullptr) {
      const bf16x4 r = reinterpret_cast<const bf16x4*>(a.residual)[i];
#pragma unroll
      for (int q = 0; q < 4; ++q) acc[q] = (a.round_block ? (float)(bf16_t)acc[q] : acc[q]) + (float)r[q];
    }
    bf16x4 o = {(bf16_t)acc[0], (bf16_t)acc[1], (bf16_t)acc[2], (bf16_t)acc[3]};
    reinterpret_cast<bf16x4*>(out)[i] = o;
  }
}

}  // namespace

hipError_t launch_gateup_generic(const void* x, const void* wgu, const float* theta, const int32_t* offsets,
                                 const int32_t* perm_token, int T, int H, int E, int k, int I, int dtype, int act,
                                 void* hidden, hipStream_t s) {
  const int S = T * k;
  if (S == 0) return hipSuccess;
  const size_t shm = (size_t)(H + 2 * I) * sizeof(float);
  if (dtype == BIBO_DTYPE_BF16)
    hipLaunchKernelGGL(gateup_generic_kernel<bf16_t>, dim3(S), dim3(256), shm, s, static_cast<const bf16_t*>(x),
                       static_cast<const bf16_t*>(wgu), theta, offsets, perm_token, H, E, I, act,
                       static_cast<bf16_t*>(hidden));
  else
    hipLaunchKernelGGL(gateup_generic_kernel<float>, dim3(S), dim3(256), shm, s, static_cast<const float*>(x),
                       static_cast<const float*>(wgu), theta, offsets, perm_token, H, E, I, act,
                       static_cast<float*>(hidden));
  return hipGetLastError();
}

hipError_t launch_down_generic(const void* hidden, const void* wd, const float* w, const int32_t* offsets,
                               const int32_t* perm_slot, int T, int H, int E, int k, int I, int dtype, float* yw,
                               hipStream_t s) {
  const int S = T * k;
  if (S == 0) return hipSuccess;
  const size_t shm = (size_t)I * sizeof(float);
  if (dtype == BIBO_DTYPE_BF16)
    hipLaunchKernelGGL(down_generic_kernel<bf16_t>, dim3(S), dim3(256), shm, s, static_cast<const bf16_t*>(hidden),
                       static_cast<const bf16_t*>(wd), w, offsets, perm_slot, H, E, I, yw);
  else
    hipLaunchKernelGGL(down_generic_kernel<float>, dim3(S), dim3(256), shm, s, static_cast<const float*>(hidden),
                       static_cast<const float*>(wd), w, offsets, perm_slot, H, E, I, yw);
  return hipGetLastError();
}

hipError_t launch_combine(const void* yw, int yw_is_bf16, const CombineArgs& a, int T, int H, int k, int dtype,
                          void* out, hipStream_t s) {
  const size_t n = (size_t)T * H;
  if (n == 0) return hipSuccess;
  const int grid = (int)((n + 255) / 256 < 65536 ? (n + 255) / 256 : 65536);
  if (yw_is_bf16) {
    if (dtype != BIBO_DTYPE_BF16) return hipErrorInvalidValue;
    if ((H % 8) == 0 && ((reinterpret_cast<uintptr_t>(yw) | reinterpret_cast<uintptr_t>(out) |
                          reinterpret_cast<uintptr_t>(a.residual) | reinterpret_cast<uintptr_t>(a.x)) & 15) == 0) {
      const size_t n8 = n / 8;
      const int g8 = (int)((n8 + 255) / 256 < 65536 ? (n8 + 255) / 256 : 65536);
      hipLaunchKernelGGL(combine_bf16x8_kernel, dim3(g8), dim3(256), 0, s, static_cast<const bf16_t*>(yw), a, T, H / 8, k,
                         static_cast<bf16_t*>(out));
    } else
      hipLaunchKernelGGL((combine_kernel<bf16_t, bf16_t>), dim3(grid), dim3(256), 0, s,
                         static_cast<const bf16_t*>(yw), a, T, H, k, static_cast<bf16_t*>(out));
  } else if (dtype == BIBO_DTYPE_BF16) {
    if ((H % 4) == 0 && ((reinterpret_cast<uintptr_t>(yw) | reinterpret_cast<uintptr_t>(out) |
                          reinterpret_cast<uintptr_t>(a.residual) | reinterpret_cast<uintptr_t>(a.x)) & 15) == 0) {
      const size_t n4 = n / 4;
      const int g4 = (int)((n4 + 255) / 256 < 65536 ? (n4 + 255) / 256 : 65536);
      hipLaunchKernelGGL(combine_f32x4_kernel, dim3(g4), dim3(256), 0, s, static_cast<const float*>(yw), a, T, H / 4, k,
                         static_cast<bf16_t*>(out));
    } else
      hipLaunchKernelGGL((combine_kernel<float, bf16_t>), dim3(grid), dim3(256), 0, s, static_cast<const float*>(yw), a, T,
                         H, k, static_cast<bf16_t*>(out));
  } else {
    hipLaunchKernelGGL((combine_kernel<float, float>), dim3(grid), dim3(256), 0, s, static_cast<const float*>(yw), a, T,
                       H, k, static_cast<float*>(out));
  }
  return hipGetLastError();
}

}  // namespace bibo
