// Weight-streaming expert kernels for few rows per expert (decode shapes), bf16, gfx950.
//
// With a handful of rows per expert the layer is bound by reading every active expert's weights once
// from HBM, so the work is cut along the WEIGHT rows: a workgroup owns 64 consecutive weight rows of
// one expert (four waves x 16 rows) and multiplies them against that expert's routed rows, 16 at a
// time, with v_mfma_f32_16x16x32_bf16 (weights are the M operand, tokens the N operand).  Weight
// fragments go straight from global memory to registers: lane (r = lane%16, g = lane/16) loads the
// 32 contiguous bytes [32g, 32g+32) of every 128-byte line of weight row r, so four lanes consume a
// whole line; the token operand, staged in LDS, is read with the same K permutation.
//
//   gateup_stream_kernel : raw gate/up pre-activations  gu[row, 0..2I) fp32   (src/modeling/ffn/moe.py:84)
//   down_stream_kernel   : prologue turns a row's gate/up into r^p SiLU(g/r) up (moe.py:87-92, needs the
//                          whole gate row, which no single gate/up workgroup has), then streams w_down and
//                          writes routing-weighted rows in slot order        (moe.py:92-93)
#include "common.h"

namespace bibo {
namespace {

constexpr int kRowsPerWave = 16;
constexpr int kRowsPerWg = 64;     // weight rows per workgroup
constexpr int kTok = 16;           // routed rows multiplied per pass
constexpr int kLine = 64;          // bf16 elements per 128-byte line

// Stream `kRowsPerWave` weight rows (row stride K elements) against 16 token rows held in LDS `xs`
// (row stride K + 8 elements so the 16 lanes of a fragment read hit distinct banks).
template <int UNROLL>
__device__ __forceinline__ floatx4 stream_rows(const bf16_t* __restrict__ wrow, const bf16_t* xs, int K, int lane) {
  const int g = lane >> 4;
  const bf16_t* wp = wrow + g * 16;                            // this lane's 32 bytes of every line
  const bf16_t* xp = xs + (lane & 15) * (K + 8) + g * 16;
  floatx4 acc = {0.f, 0.f, 0.f, 0.f};
  const int nlines = K / kLine;
  int l = 0;
  for (; l + UNROLL <= nlines; l += UNROLL) {
    bf16x8 w0[UNROLL], w1[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      w0[u] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(wp + (l + u) * kLine));
      w1[u] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(wp + (l + u) * kLine + 8));
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const bf16x8 x0 = *reinterpret_cast<const bf16x8*>(xp + (l + u) * kLine);
      const bf16x8 x1 = *reinterpret_cast<const bf16x8*>(xp + (l + u) * kLine + 8);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w0[u], x0, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w1[u], x1, acc, 0, 0, 0);
    }
  }
  for (; l < nlines; ++l) {
    const bf16x8 w0 = *reinterpret_cast<const bf16x8*>(wp + l * kLine);
    const bf16x8 w1 = *reinterpret_cast<const bf16x8*>(wp + l * kLine + 8);
    const bf16x8 x0 = *reinterpret_cast<const bf16x8*>(xp + l * kLine);
    const bf16x8 x1 = *reinterpret_cast<const bf16x8*>(xp + l * kLine + 8);
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w0, x0, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w1, x1, acc, 0, 0, 0);
  }
  return acc;
}

// grid = (2I / 64, E).  gu[row, c] = x[token(row)] . w_gate_up[e, c, :]
__global__ __launch_bounds__(256) void gateup_stream_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ wgu,
                                                            const int32_t* __restrict__ offsets,
                                                            const int32_t* __restrict__ perm_token, int H, int I,
                                                            float* __restrict__ gu) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16_t* xs = reinterpret_cast<bf16_t*>(smem_raw);            // [kTok][H + 8]
  const int e = blockIdx.y;
  const int lo = offsets[e], hi = offsets[e + 1];
  if (lo == hi) return;                                        // idle expert: its weights are never read
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int c0 = blockIdx.x * kRowsPerWg + wave * kRowsPerWave;  // first weight row of this wave
  const bf16_t* wrow = wgu + ((size_t)e * 2 * I + c0 + (lane & 15)) * H;
  const int gran_per_row = H / 8;
  for (int r0 = lo; r0 < hi; r0 += kTok) {
    const int nrow = min(kTok, hi - r0);
    __syncthreads();                                           // previous pass is done with xs
    for (int i = tid; i < kTok * gran_per_row; i += 256) {
      const int t = i / gran_per_row, c = i - t * gran_per_row;
      u32x4 v = {0u, 0u, 0u, 0u};
      if (t < nrow) v = *reinterpret_cast<const u32x4*>(x + (size_t)perm_token[r0 + t] * H + c * 8);   // moe.py:81
      *reinterpret_cast<u32x4*>(xs + t * (H + 8) + c * 8) = v;
    }
    __syncthreads();
    const floatx4 acc = stream_rows<4>(wrow, xs, H, lane);
    // accumulator: lane holds token lane%16, weight rows 4*(lane/16) + i
    const int t = lane & 15;
    if (t < nrow)
      *reinterpret_cast<floatx4*>(gu + (size_t)(r0 + t) * 2 * I + c0 + 4 * (lane >> 4)) = acc;
  }
}

// grid = (H / 64, E).  yw[slot(row), c] = w[slot] * (act(row) . w_down[e, c, :])
__global__ __launch_bounds__(256) void down_stream_kernel(const float* __restrict__ gu, const bf16_t* __restrict__ wd,
                                                          const float* __restrict__ theta, const float* __restrict__ w,
                                                          const int32_t* __restrict__ offsets,
                                                          const int32_t* __restrict__ perm_slot, int H, int I,
                                                          float* __restrict__ yw) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16_t* hs = reinterpret_cast<bf16_t*>(smem_raw);            // [kTok][I + 8] activations of this pass
  __shared__ float rinv_s[kTok], gain_s[kTok];
  const int e = blockIdx.y;
  const int lo = offsets[e], hi = offsets[e + 1];
  if (lo == hi) return;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int c0 = blockIdx.x * kRowsPerWg + wave * kRowsPerWave;
  const bf16_t* wrow = wd + ((size_t)e * H + c0 + (lane & 15)) * I;
  const float p = 1.f / (1.f + __expf(-theta[e]));             // moe.py:89
  for (int r0 = lo; r0 < hi; r0 += kTok) {
    const int nrow = min(kTok, hi - r0);
    __syncthreads();
    // r = sqrt(mean(g^2) + eps) per row: one wave per 4 rows, lanes stride the I gate values (moe.py:88)
    for (int t = wave; t < kTok; t += 4) {
      float ss = 0.f;
      if (t < nrow) {
        const float* grow = gu + (size_t)(r0 + t) * 2 * I;
        for (int i = lane; i < I; i += kWave) ss = fmaf(grow[i], grow[i], ss);
      }
      ss = wave_sum(ss);
      if (lane == 0) {
        const float r2 = ss / (float)I + kNormSiluEps;
        rinv_s[t] = rsqrtf(r2);
        gain_s[t] = __expf(0.5f * p * __logf(r2));             // r^p
      }
    }
    __syncthreads();
    for (int i = tid; i < kTok * I; i += 256) {
      const int t = i / I, c = i - t * I;
      float hval = 0.f;
      if (t < nrow) {
        const float* grow = gu + (size_t)(r0 + t) * 2 * I;
        const float z = grow[c] * rinv_s[t];
        hval = z / (1.f + __expf(-z)) * gain_s[t] * grow[I + c];   // SiLU(g/r) r^p up, moe.py:89-92
      }
      hs[t * (I + 8) + c] = (bf16_t)hval;
    }
    __syncthreads();
    const floatx4 acc = stream_rows<4>(wrow, hs, I, lane);
    const int t = lane & 15;
    if (t < nrow) {
      const int slot = perm_slot[r0 + t];
      const float ws = w[slot];                                 // moe.py:93
      floatx4 o = {ws * acc[0], ws * acc[1], ws * acc[2], ws * acc[3]};
      *reinterpret_cast<floatx4*>(yw + (size_t)slot * H + c0 + 4 * (lane >> 4)) = o;
    }
  }
}

}  // namespace

bool stream_supported(int H, int I, int dtype) {
  // LDS: 16 rows of (max(H, I) + 8) bf16 within 64 KB; every K extent must be whole 128-byte lines
  return dtype == BIBO_DTYPE_BF16 && (H % 64) == 0 && (I % 64) == 0 && H <= 1984 && I <= 1984;
}

size_t stream_gu_bytes(int T, int k, int I) { return (size_t)T * k * 2 * I * sizeof(float); }

hipError_t launch_gateup_stream(const void* x, const void* wgu, const int32_t* offsets, const int32_t* perm_token,
                                int T, int H, int E, int k, int I, float* gu, hipStream_t s) {
  if (T * k == 0) return hipSuccess;
  const size_t shm = (size_t)kTok * (H + 8) * sizeof(bf16_t);
  hipLaunchKernelGGL(gateup_stream_kernel, dim3(2 * I / kRowsPerWg, E), dim3(256), shm, s,
                     static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(wgu), offsets, perm_token, H, I, gu);
  return hipGetLastError();
}

hipError_t launch_down_stream(const float* gu, const void* wd, const float* theta, const float* w,
                              const int32_t* offsets, const int32_t* perm_slot, int T, int H, int E, int k, int I,
                              float* yw, hipStream_t s) {
  if (T * k == 0) return hipSuccess;
  const size_t shm = (size_t)kTok * (I + 8) * sizeof(bf16_t);
  hipLaunchKernelGGL(down_stream_kernel, dim3(H / kRowsPerWg, E), dim3(256), shm, s, gu,
                     static_cast<const bf16_t*>(wd), theta, w, offsets, perm_slot, H, I, yw);
  return hipGetLastError();
}

}  // namespace bibo
