// Weight-streaming expert kernels for few rows per expert (decode shapes), bf16, gfx950.
//
// No permutation pass: with at most kStreamMaxSlots routed slots every workgroup finds the rows of its
// expert by scanning the routing indices itself (ascending slot order, the same order the permutation
// kernel produces), and all intermediate buffers are indexed by slot.
//
// With a handful of rows per expert the layer is bound by reading every active expert's weights once
// from HBM, so the work is cut along the WEIGHT rows: a workgroup owns 64 consecutive weight rows of
// one expert (four waves x 16 rows) and multiplies them against that expert's routed rows, 16 at a
// time, with v_mfma_f32_16x16x32_bf16 (weights are the M operand, tokens the N operand).  Weight
// fragments go straight from global memory to registers: lane (r = lane%16, g = lane/16) loads the
// 32 contiguous bytes [32g, 32g+32) of every 128-byte line of weight row r, so four lanes consume a
// whole line; the token operand, staged in LDS, is read with the same K permutation.
//
//   gateup_stream_kernel : raw gate/up pre-activations  gu[slot, 0..2I) fp32  (src/modeling/ffn/moe.py:84)
//   activate_rows_kernel : hidden[slot] = r^p SiLU(g/r) up; needs the whole gate row, which no single
//                          gate/up workgroup has, hence its own tiny launch    (moe.py:87-92)
//   down_stream_kernel   : streams w_down and writes routing-weighted rows in slot order (moe.py:92-93)
#include "common.h"

namespace bibo {
namespace {

constexpr int kRowsPerWave = 16;
constexpr int kRowsPerWg = 64;     // weight rows per workgroup
constexpr int kTok = 16;           // routed rows multiplied per pass
constexpr int kLine = 64;          // bf16 elements per 128-byte line

constexpr int kChunk = 4;          // 128-byte lines per register chunk (two chunks are alive: 64 VGPRs)
constexpr int kScan = kStreamMaxSlots / 256;   // routing indices each thread inspects

// Slots routed to expert e, ascending, into rows_s; returns how many.  All 256 threads call it; slot
// s = 256*q + tid, so slot order is (q, wave, lane).  Ends with a barrier.
__device__ __forceinline__ int expert_rows(const int32_t* __restrict__ idx, int S, int e, unsigned short* rows_s,
                                           int* cnt_s) {
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const unsigned long long lt = (1ull << lane) - 1ull;
  int v[kScan];
#pragma unroll
  for (int q = 0; q < kScan; ++q) {
    const int s = q * 256 + tid;
    v[q] = (s < S) ? idx[s] : -1;                               // all loads in flight together
  }
  int rank[kScan];
#pragma unroll
  for (int q = 0; q < kScan; ++q) {
    const unsigned long long b = __ballot(v[q] == e);
    rank[q] = __popcll(b & lt);
    if (lane == 0) cnt_s[q * 4 + wave] = __popcll(b);
  }
  __syncthreads();
  int run = 0;                                                  // exclusive prefix over the (q, wave) cells in slot order
#pragma unroll
  for (int q = 0; q < kScan; ++q)
#pragma unroll
    for (int ww = 0; ww < 4; ++ww) {
      if (ww == wave && v[q] == e) rows_s[run + rank[q]] = (unsigned short)(q * 256 + tid);
      run += cnt_s[q * 4 + ww];
    }
  __syncthreads();
  return run;
}

struct WChunk {
  bf16x8 w0[kChunk], w1[kChunk];
};

// this lane's 32 bytes of lines l .. l+kChunk-1 of its weight row (lines past nlines are skipped)
__device__ __forceinline__ void load_chunk(WChunk& c, const bf16_t* __restrict__ wp, int l, int nlines) {
#pragma unroll
  for (int u = 0; u < kChunk; ++u)
    if (l + u < nlines) {
      c.w0[u] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(wp + (l + u) * kLine));
      c.w1[u] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(wp + (l + u) * kLine + 8));
    }
}

// Stream kRowsPerWave weight rows (row stride K) against 16 token rows held in LDS `xs` (row stride K + 8
// elements, so the 16 lanes of a fragment read hit distinct banks).  `first` already holds lines 0..kChunk-1
// (loaded before the token rows were staged); each further chunk is requested one chunk ahead of its use.
__device__ __forceinline__ floatx4 stream_rows(const bf16_t* __restrict__ wrow, const bf16_t* xs, int K, int lane,
                                               const WChunk& first) {
  const int g = lane >> 4;
  const bf16_t* wp = wrow + g * 16;                            // this lane's 32 bytes of every line
  const bf16_t* xp = xs + (lane & 15) * (K + 8) + g * 16;
  floatx4 acc = {0.f, 0.f, 0.f, 0.f};
  const int nlines = K / kLine;
  WChunk cur = first, nxt;
  for (int l = 0; l < nlines; l += kChunk) {
    if (l + kChunk < nlines) load_chunk(nxt, wp, l + kChunk, nlines);
#pragma unroll
    for (int u = 0; u < kChunk; ++u)
      if (l + u < nlines) {
        const bf16x8 x0 = *reinterpret_cast<const bf16x8*>(xp + (l + u) * kLine);
        const bf16x8 x1 = *reinterpret_cast<const bf16x8*>(xp + (l + u) * kLine + 8);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur.w0[u], x0, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur.w1[u], x1, acc, 0, 0, 0);
      }
    cur = nxt;
  }
  return acc;
}

// grid = (2I / 64, E).  gu[slot, c] = x[slot / k] . w_gate_up[e, c, :]
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4))) void gateup_stream_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ wgu,
                                                            const int32_t* __restrict__ idx, int S, int k, int H, int I,
                                                            float* __restrict__ gu) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  __shared__ unsigned short rows_s[kStreamMaxSlots];   // 16-bit slot ids keep four workgroups within a CU's LDS
  __shared__ int cnt_s[kScan * 4];
  bf16_t* xs = reinterpret_cast<bf16_t*>(smem_raw);            // [kTok][H + 8]
  const int e = blockIdx.y;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int c0 = blockIdx.x * kRowsPerWg + wave * kRowsPerWave;  // first weight row of this wave
  const bf16_t* wrow = wgu + ((size_t)e * 2 * I + c0 + (lane & 15)) * H;
  WChunk first;
  load_chunk(first, wrow + (lane >> 4) * 16, 0, H / kLine);    // in flight while the rows are found and staged
  const int n = expert_rows(idx, S, e, rows_s, cnt_s);
  if (n == 0) return;                                          // idle expert
  const int gran_per_row = H / 8;
  for (int r0 = 0; r0 < n; r0 += kTok) {
    const int nrow = min(kTok, n - r0);
    __syncthreads();                                           // previous pass is done with xs
    for (int i = tid; i < kTok * gran_per_row; i += 256) {
      const int t = i / gran_per_row, c = i - t * gran_per_row;
      u32x4 v = {0u, 0u, 0u, 0u};
      if (t < nrow) v = *reinterpret_cast<const u32x4*>(x + (size_t)(rows_s[r0 + t] / k) * H + c * 8);   // moe.py:81
      *reinterpret_cast<u32x4*>(xs + t * (H + 8) + c * 8) = v;
    }
    __syncthreads();
    const floatx4 acc = stream_rows(wrow, xs, H, lane, first);
    // accumulator: lane holds row lane%16 of the pass, weight rows 4*(lane/16) + i
    const int t = lane & 15;
    if (t < nrow)
      *reinterpret_cast<floatx4*>(gu + (size_t)rows_s[r0 + t] * 2 * I + c0 + 4 * (lane >> 4)) = acc;
  }
}

// One workgroup per slot: hidden[slot] = r^p SiLU(g/r) up from the fp32 pre-activations (moe.py:87-92).
__global__ __launch_bounds__(256) void activate_rows_kernel(const float* __restrict__ gu, const float* __restrict__ theta,
                                                            const int32_t* __restrict__ idx, int E, int I,
                                                            bf16_t* __restrict__ hidden) {
  __shared__ float red[4];
  const int slot = blockIdx.x;
  const int e = idx[slot];
  if ((unsigned)e >= (unsigned)E) return;                      // no expert: the slot has no row
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const float* grow = gu + (size_t)slot * 2 * I;
  float ss = 0.f;
  for (int i = tid; i < I; i += 256) ss = fmaf(grow[i], grow[i], ss);
  ss = wave_sum(ss);
  if (lane == 0) red[wave] = ss;
  __syncthreads();
  const float r2 = (((red[0] + red[1]) + red[2]) + red[3]) / (float)I + kNormSiluEps;    // moe.py:88
  const float p = 1.f / (1.f + __expf(-theta[e]));                                        // moe.py:89
  const float rinv = rsqrtf(r2), gain = __expf(0.5f * p * __logf(r2));                     // 1/r, r^p
  for (int i = tid; i < I; i += 256) {
    const float z = grow[i] * rinv;
    hidden[(size_t)slot * I + i] = (bf16_t)(z / (1.f + __expf(-z)) * gain * grow[I + i]);
  }
}

// grid = (H / 64, E).  yw[slot, c] = w[slot] * (hidden[slot] . w_down[e, c, :])
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4))) void down_stream_kernel(const bf16_t* __restrict__ hidden, const bf16_t* __restrict__ wd,
                                                          const float* __restrict__ w, const int32_t* __restrict__ idx,
                                                          int S, int H, int I, float* __restrict__ yw) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  __shared__ unsigned short rows_s[kStreamMaxSlots];   // 16-bit slot ids keep four workgroups within a CU's LDS
  __shared__ int cnt_s[kScan * 4];
  bf16_t* hs = reinterpret_cast<bf16_t*>(smem_raw);            // [kTok][I + 8] activations of this pass
  const int e = blockIdx.y;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int c0 = blockIdx.x * kRowsPerWg + wave * kRowsPerWave;
  const bf16_t* wrow = wd + ((size_t)e * H + c0 + (lane & 15)) * I;
  WChunk first;
  load_chunk(first, wrow + (lane >> 4) * 16, 0, I / kLine);
  const int n = expert_rows(idx, S, e, rows_s, cnt_s);
  if (n == 0) return;
  const int gran_per_row = I / 8;
  for (int r0 = 0; r0 < n; r0 += kTok) {
    const int nrow = min(kTok, n - r0);
    __syncthreads();
    for (int i = tid; i < kTok * gran_per_row; i += 256) {
      const int t = i / gran_per_row, c = i - t * gran_per_row;
      u32x4 v = {0u, 0u, 0u, 0u};
      if (t < nrow) v = *reinterpret_cast<const u32x4*>(hidden + (size_t)rows_s[r0 + t] * I + c * 8);
      *reinterpret_cast<u32x4*>(hs + t * (I + 8) + c * 8) = v;
    }
    __syncthreads();
    const floatx4 acc = stream_rows(wrow, hs, I, lane, first);
    const int t = lane & 15;
    if (t < nrow) {
      const int slot = rows_s[r0 + t];
      const float ws = w[slot];                                 // moe.py:93
      floatx4 o = {ws * acc[0], ws * acc[1], ws * acc[2], ws * acc[3]};
      *reinterpret_cast<floatx4*>(yw + (size_t)slot * H + c0 + 4 * (lane >> 4)) = o;
    }
  }
}

}  // namespace

bool stream_supported(int H, int I, int dtype) {
  // LDS: 16 rows of (max(H, I) + 8) bf16 within 56 KB (next to the 8 KB row list); every K extent must be whole
  // 128-byte lines
  return dtype == BIBO_DTYPE_BF16 && (H % 64) == 0 && (I % 64) == 0 && H <= 1728 && I <= 1728;
}

size_t stream_gu_bytes(int T, int k, int I) { return (size_t)T * k * 2 * I * sizeof(float); }

hipError_t launch_gateup_stream(const void* x, const void* wgu, const int32_t* idx, int T, int H, int E, int k, int I,
                                float* gu, hipStream_t s) {
  if (T * k == 0) return hipSuccess;
  if (T * k > kStreamMaxSlots) return hipErrorInvalidValue;
  const size_t shm = (size_t)kTok * (H + 8) * sizeof(bf16_t);
  hipLaunchKernelGGL(gateup_stream_kernel, dim3(2 * I / kRowsPerWg, E), dim3(256), shm, s,
                     static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(wgu), idx, T * k, k, H, I, gu);
  return hipGetLastError();
}

hipError_t launch_down_stream(const float* gu, const void* wd, const float* theta, const float* w, const int32_t* idx,
                              int T, int H, int E, int k, int I, void* hidden, float* yw, hipStream_t s) {
  if (T * k == 0) return hipSuccess;
  if (T * k > kStreamMaxSlots) return hipErrorInvalidValue;
  bf16_t* hp = static_cast<bf16_t*>(hidden);
  hipLaunchKernelGGL(activate_rows_kernel, dim3(T * k), dim3(256), 0, s, gu, theta, idx, E, I, hp);
  const size_t shm = (size_t)kTok * (I + 8) * sizeof(bf16_t);
  hipLaunchKernelGGL(down_stream_kernel, dim3(H / kRowsPerWg, E), dim3(256), shm, s, hp,
                     static_cast<const bf16_t*>(wd), w, idx, T * k, H, I, yw);
  return hipGetLastError();
}

}  // namespace bibo
