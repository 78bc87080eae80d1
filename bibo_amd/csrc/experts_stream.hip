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
// Order of the memory requests.  A CU serves its vector loads first in, first out, and its share of the
// HBM rate is about 23 GB/s, so a small load issued behind 64 KB of weight requests waits about 3 us for
// them (and behind 192 KB about 8 us).  Every small load the multiplication depends on is therefore issued
// AHEAD of the weights it would otherwise queue behind: the routing indices before any weights, the operand
// rows before the second half of the first chunk and the second chunk, and only as much weight data is
// requested in between (kFirstLines lines per lane) as the dependent work (finding the rows) takes to complete.
//
//   gateup_stream_kernel : raw gate/up pre-activations gu[slot, 0..2I) bf16        (src/modeling/ffn/moe.py:84)
//   down_stream_kernel   : streams w_down and writes routing-weighted rows in slot order (moe.py:92-93);
//                          for I <= 512 and at most 16 rows per expert on average it also turns the expert's
//                          pre-activations into the operand rows, hidden = r^p SiLU(g/r) up (moe.py:87-92),
//                          while the weights are on their way
//   activate_rows_kernel : the same activation as a launch of its own, for wider I or more rows
#include "common.h"

namespace bibo {
namespace {

constexpr int kRowsPerWave = 16;
constexpr int kRowsPerWg = 64;     // weight rows per workgroup
constexpr int kTok = 16;           // routed rows multiplied per pass
constexpr int kLine = 64;          // bf16 elements per 128-byte line
constexpr int kChunk = 4;          // 128-byte lines per register chunk (two chunks are alive: 64 VGPRs)
constexpr int kScan = kStreamMaxSlots / 256;   // routing indices each thread inspects
constexpr int kFusedActMaxI = 512; // widest I whose activation the down kernel computes itself
static_assert(kFusedActMaxI == 2 * kChunk * kLine, "the fused-activation down kernel assumes two chunks hold a row");

struct ScanRegs {
  int v[kScan];
};

// request this thread's routing indices: slot s = 256*q + tid, so slot order is (q, wave, lane)
__device__ __forceinline__ void scan_issue(ScanRegs& r, const int32_t* __restrict__ idx, int S) {
#pragma unroll
  for (int q = 0; q < kScan; ++q) {
    const int s = q * 256 + threadIdx.x;
    r.v[q] = (s < S) ? idx[s] : -1;                             // all loads in flight together
  }
}

// Slots routed to expert e, ascending, into rows_s; returns how many.  All 256 threads call it; ends with a
// barrier.  Only the ceil(S / 256) index groups that hold slots are looked at.  The host only launches these
// kernels when no expert can get more than kStreamMaxRows rows; entries past the list's end are dropped rather
// than written all the same.
__device__ __forceinline__ int scan_finish(const ScanRegs& r, int S, int e, unsigned short* rows_s, int* cnt_s) {
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const unsigned long long lt = (1ull << lane) - 1ull;
  const int nq = (S + 255) >> 8;
  int rank[kScan];
#pragma unroll
  for (int q = 0; q < kScan; ++q)
    if (q < nq) {
      const unsigned long long b = __ballot(r.v[q] == e);
      rank[q] = __popcll(b & lt);
      if (lane == 0) cnt_s[q * 4 + wave] = __popcll(b);
    }
  __syncthreads();
  int run = 0;                                                  // exclusive prefix over the (q, wave) cells in slot order
#pragma unroll
  for (int q = 0; q < kScan; ++q)
    if (q < nq) {
#pragma unroll
      for (int ww = 0; ww < 4; ++ww) {
        if (ww == wave && r.v[q] == e && run + rank[q] < kStreamMaxRows)
          rows_s[run + rank[q]] = (unsigned short)(q * 256 + tid);
        run += cnt_s[q * 4 + ww];
      }
    }
  __syncthreads();
  return min(run, kStreamMaxRows);
}

struct WChunk {
  bf16x8 w0[kChunk], w1[kChunk];
};
// Lines of the first chunk a wave requests before its rows are known; the other lines follow the row requests.  All
// four up front put 128 KB of weight requests per CU ahead of every workgroup's row loads, which then wait for them;
// with two, the rows are back about 1.5 us earlier and the weights still keep HBM busy from the first microsecond
// (one line was as slow as four: too little in flight while the rows are found).
constexpr int kFirstLines = 2;

// this lane's 32 bytes of lines l .. l+kChunk-1 of its weight row.  kWhole: the row is a whole number of
// chunks, and a chunk that starts past its end is skipped as a whole; otherwise line by line.
// (U0, U1: only lines l + U0 .. l + U1 - 1 of the chunk)
template <bool kWhole, int U0 = 0, int U1 = kChunk>
__device__ __forceinline__ void load_chunk(WChunk& c, const bf16_t* __restrict__ wp, int l, int nlines) {
  if (kWhole && l >= nlines) return;
#pragma unroll
  for (int u = U0; u < U1; ++u)
    if (kWhole || l + u < nlines) {
      c.w0[u] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(wp + (l + u) * kLine));
      c.w1[u] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(wp + (l + u) * kLine + 8));
    }
}

// Multiply kChunk lines (from line l) of the wave's weight rows, held in `c`, with the operand rows in LDS.
template <bool kWhole>
__device__ __forceinline__ void mul_chunk(floatx4& acc, const WChunk& c, const bf16_t* xp, int l, int nlines) {
  if (kWhole && l >= nlines) return;
#pragma unroll
  for (int u = 0; u < kChunk; ++u)
    if (kWhole || l + u < nlines) {
      const bf16x8 x0 = *reinterpret_cast<const bf16x8*>(xp + (l + u) * kLine);
      const bf16x8 x1 = *reinterpret_cast<const bf16x8*>(xp + (l + u) * kLine + 8);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(c.w0[u], x0, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(c.w1[u], x1, acc, 0, 0, 0);
    }
}

// Stream kRowsPerWave weight rows (row stride K) against 16 operand rows held in LDS `xs` (row stride K + 8
// elements, so the 16 lanes of a fragment read hit distinct banks).  On entry `a` and `b` hold lines
// 0..kChunk-1 and kChunk..2*kChunk-1; each is refilled, two chunks ahead, as soon as it is consumed, so on
// return they hold other lines.
// kTwoChunks: the caller knows that the row is no longer than the two chunks (nothing is ever refilled, and the
// weight pointer is dead once they are requested).
template <bool kWhole, bool kTwoChunks = false>
__device__ __forceinline__ floatx4 stream_rows(const bf16_t* __restrict__ wp, const bf16_t* xs, int K, int lane,
                                               WChunk& a, WChunk& b) {
  const bf16_t* xp = xs + (lane & 15) * (K + 8) + (lane >> 4) * 16;
  floatx4 acc = {0.f, 0.f, 0.f, 0.f};
  const int nlines = K / kLine;
  if (kTwoChunks) {
    mul_chunk<kWhole>(acc, a, xp, 0, nlines);
    mul_chunk<kWhole>(acc, b, xp, kChunk, nlines);
    return acc;
  }
  for (int l = 0; l < nlines; l += 2 * kChunk) {
    mul_chunk<kWhole>(acc, a, xp, l, nlines);
    load_chunk<kWhole>(a, wp, l + 2 * kChunk, nlines);
    mul_chunk<kWhole>(acc, b, xp, l + kChunk, nlines);
    load_chunk<kWhole>(b, wp, l + 3 * kChunk, nlines);
  }
  return acc;
}

typedef __attribute__((address_space(3))) void stream_lds_void;
typedef const __attribute__((address_space(1))) void stream_gbl_void;

// wait until at most the kChunk lines of weights requested last are still on their way (loads complete in order)
// (EXTRA: further loads requested behind the rows, the rest of the first chunk; s_waitcnt vmcnt(8 + EXTRA) in the gfx9
// encoding: vmcnt in bits 3:0 and 15:14, expcnt and lgkmcnt left at "no wait")
template <int EXTRA>
__device__ __forceinline__ void wait_all_but_chunk(bool chunk_requested) {
  constexpr int kN = 8 + EXTRA;
  if (chunk_requested) __builtin_amdgcn_s_waitcnt((kN & 0xF) | ((kN >> 4) << 14) | (0x7 << 4) | (0xF << 8));
  else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  static_assert(2 * kChunk == 8, "the wait above counts the two loads per line of one chunk");
}

// Operand rows of slots rows_s[r0 .. r0+nrow), row (slot / div) of `src` (row length K), into xs[t][0..K) (row
// stride K + 8), by LDS-DMA: one wave instruction moves 1 KB of one row (lane L's 16 bytes land at base + 16 L),
// no registers hold the data.  The rows are requested, then (a_rest: the first pass) the lines of chunk `a` that were
// held back, then chunk `b` of the weights (lines kChunk..), and the wave then waits for its rows only.  Rows past nrow keep whatever LDS held: they only feed accumulator
// columns nobody stores.  The caller's barrier makes the rows visible to the other waves.
template <bool kWhole, int kFirst>
__device__ __forceinline__ void stage_rows(const bf16_t* __restrict__ src, const unsigned short* rows_s, int r0,
                                           int nrow, int div, int K, bf16_t* xs, WChunk& b,
                                           const bf16_t* __restrict__ wp, int nlines, bool load_b, WChunk& a, bool a_rest) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int gran = K / 8;                                      // 16-byte granules per row
  const int segs = (gran + 63) >> 6;                           // 1 KB pieces per row
  const int items = nrow * segs;
  for (int it = wave; it < items; it += 4) {
    const int t = it / segs, sg = it - t * segs;
    const int row = __builtin_amdgcn_readfirstlane((int)rows_s[r0 + t]) / div;                 // moe.py:81
    const int c = sg * 64 + lane;
    if (c < gran)
      __builtin_amdgcn_global_load_lds((stream_gbl_void*)(src + (size_t)row * K + c * 8),
                                       (stream_lds_void*)(xs + t * (K + 8) + sg * 512), 16, 0, 0);
  }
  if (a_rest) {
    load_chunk<kWhole, kFirst, kChunk>(a, wp, 0, nlines);
    if (load_b) load_chunk<kWhole>(b, wp, kChunk, nlines);
    if (kWhole) wait_all_but_chunk<2 * (kChunk - kFirst)>(load_b && nlines > kChunk);
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    return;
  }
  if (load_b) load_chunk<kWhole>(b, wp, kChunk, nlines);
  wait_all_but_chunk<0>(load_b && kWhole && nlines > kChunk);
}

// grid = (2I / 64, E).  gu[slot, c] = x[slot / k] . w_gate_up[e, c, :].  kWhole: H is a whole number of chunks.
template <bool kWhole>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4)))
void gateup_stream_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ wgu, const int32_t* __restrict__ idx,
                          int S, int k, int H, int I, bf16_t* __restrict__ gu) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  __shared__ unsigned short rows_s[kStreamMaxRows];    // 16-bit slot ids keep four workgroups within a CU's LDS
  __shared__ int cnt_s[kScan * 4];
  bf16_t* xs = reinterpret_cast<bf16_t*>(smem_raw);            // [kTok][H + 8]
  const int e = blockIdx.y;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int c0 = blockIdx.x * kRowsPerWg + wave * kRowsPerWave;  // first weight row of this wave
  // this lane's 32 bytes of every line of its weight row
  const bf16_t* wp = wgu + ((size_t)e * 2 * I + c0 + (lane & 15)) * H + (lane >> 4) * 16;
  const int nlines = H / kLine;
  const bool resident = nlines <= 2 * kChunk;                  // the two chunks hold the whole row: passes share them
  ScanRegs sr;
  scan_issue(sr, idx, S);
  WChunk ca, cb;
  load_chunk<kWhole, 0, kFirstLines>(ca, wp, 0, nlines);             // keeps HBM busy while the rows are found
  const int n = scan_finish(sr, S, e, rows_s, cnt_s);
  for (int r0 = 0; r0 < n; r0 += kTok) {
    const int nrow = min(kTok, n - r0);
    const bool reload = r0 == 0 || !resident;
    if (r0 > 0) {
      __syncthreads();                                         // the pass before is done with xs
      if (reload) load_chunk<kWhole>(ca, wp, 0, nlines);       // a further pass starts the weight rows again
    }
    stage_rows<kWhole, kFirstLines>(x, rows_s, r0, nrow, k, H, xs, cb, wp, nlines, reload, ca, r0 == 0 && kFirstLines < kChunk);
    __syncthreads();
    const floatx4 acc = stream_rows<kWhole>(wp, xs, H, lane, ca, cb);
    // accumulator: lane holds row lane%16 of the pass, weight rows 4*(lane/16) + i
    const int t = lane & 15;
    if (t < nrow) {
      bf16x4 o = {(bf16_t)acc[0], (bf16_t)acc[1], (bf16_t)acc[2], (bf16_t)acc[3]};
      *reinterpret_cast<bf16x4*>(gu + (size_t)rows_s[r0 + t] * 2 * I + c0 + 4 * (lane >> 4)) = o;
    }
  }
}

// One workgroup per slot: hidden[slot] = r^p SiLU(g/r) up from the bf16 pre-activations (moe.py:87-92).
__global__ __launch_bounds__(256) void activate_rows_kernel(const bf16_t* __restrict__ gu, const float* __restrict__ theta,
                                                            const int32_t* __restrict__ idx, int E, int I, int act,
                                                            bf16_t* __restrict__ hidden) {
  __shared__ float red[4];
  const int slot = blockIdx.x;
  const int e = idx[slot];
  if ((unsigned)e >= (unsigned)E) return;                      // no expert: the slot has no row
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const bf16_t* grow = gu + (size_t)slot * 2 * I;
  float ss = 0.f;
  for (int i = tid; i < I; i += 256) ss = fmaf((float)grow[i], (float)grow[i], ss);
  ss = wave_sum(ss);
  if (lane == 0) red[wave] = ss;
  __syncthreads();
  float rinv, gain;                                                                       // 1/r, r^p (moe.py:88-89)
  radial_row_scalars(((red[0] + red[1]) + red[2]) + red[3], I, radial_exponent(theta, e, act), act, rinv, gain);
  for (int i = tid; i < I; i += 256) {
    const float z = (float)grow[i] * rinv;
    hidden[(size_t)slot * I + i] = (bf16_t)(z / (1.f + __expf(-z)) * gain * (float)grow[I + i]);
  }
}

// Operand rows of the down projection computed in place of a copy: hidden rows of slots rows_s[r0 .. r0+nrow)
// from the bf16 pre-activations, r = sqrt(mean(g^2) + eps), hidden = r^p SiLU(g/r) up, p = sigmoid(theta)
// (moe.py:87-92), into hs[t][0..I) (row stride I + 8).  tpr = 32 or 64 threads share a row, so the workgroup
// covers 8 (or 4) rows per round; a thread owns granules part, part + tpr of the gate and of the up half.  The
// first round's loads are requested ahead of the held-back lines of chunk `a` and of chunk `b`, like the rows in
// stage_rows.
// I <= kFusedActMaxI.
template <bool kWhole, int kFirst>
__device__ __forceinline__ void stage_activated(const bf16_t* __restrict__ gu, float p, int act,
                                                const unsigned short* rows_s, int r0, int nrow, int I, bf16_t* hs,
                                                WChunk& b, const bf16_t* __restrict__ wp, int nlines, bool load_b,
                                                WChunk& a, bool a_rest) {
  constexpr int kPer = kFusedActMaxI / 8 / 32;                 // granules per thread and half at 32 threads per row
  const int tid = threadIdx.x;
  const int tpr = nrow <= 4 ? 64 : 32;
  const int row_in = tid / tpr, part = tid - row_in * tpr;
  const int gran = I / 8;
  for (int rb = 0; rb < nrow; rb += 256 / tpr) {
    const int row = rb + row_in;
    const bool live = row < nrow;                              // whole groups of tpr lanes are live or not
    const bf16_t* grow = gu + (size_t)rows_s[r0 + (live ? row : 0)] * 2 * I;
    bf16x8 g[kPer], u[kPer];
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
      const int c = part + j * tpr;
      if (live && c < gran) {
        g[j] = *reinterpret_cast<const bf16x8*>(grow + c * 8);
        u[j] = *reinterpret_cast<const bf16x8*>(grow + I + c * 8);
      }
    }
    if (rb == 0 && a_rest) load_chunk<kWhole, kFirst, kChunk>(a, wp, 0, nlines);
    if (rb == 0 && load_b) load_chunk<kWhole>(b, wp, kChunk, nlines);
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < kPer; ++j)
      if (live && part + j * tpr < gran) {
#pragma unroll
        for (int q = 0; q < 8; ++q) ss = fmaf((float)g[j][q], (float)g[j][q], ss);
      }
    for (int o = tpr >> 1; o > 0; o >>= 1) ss += __shfl_xor(ss, o, kWave);   // the row's threads are adjacent lanes
    float rinv, gain;                                                                     // 1/r, r^p (moe.py:88-89)
    radial_row_scalars(ss, I, p, act, rinv, gain);
    const float nrl = -1.4426950408889634f * rinv, rg = rinv * gain;
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
      const int c = part + j * tpr;
      if (live && c < gran) {
        bf16x8 h;
#pragma unroll
        for (int q = 0; q < 8; ++q) {
          // z / (1 + exp(-z)) * gain * up with z = g / r, constants folded per row
          const float gq = (float)g[j][q];
          const float sig = __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(gq * nrl));
          h[q] = (bf16_t)(gq * rg * sig * (float)u[j][q]);
          if (q & 1) __builtin_amdgcn_sched_barrier(0);        // two elements at a time: few temporaries alive
        }
        *reinterpret_cast<bf16x8*>(hs + row * (I + 8) + c * 8) = h;
      }
    }
  }
}

// grid = (H / 64, E).  yw[slot, c] = w[slot] * (hidden[slot] . w_down[e, c, :]).  kFusedAct: `rows_in` holds the bf16
// gate/up pre-activations [slot, 2I] and the activation `act` happens here; otherwise it holds hidden [slot, I].
// kWhole: I is a whole number of chunks.
template <bool kFusedAct, bool kWhole>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4)))
void down_stream_kernel(const bf16_t* __restrict__ rows_in, const bf16_t* __restrict__ wd, const float* __restrict__ theta,
                        const float* __restrict__ w, const int32_t* __restrict__ idx, int S, int H, int I, int act,
                        float* __restrict__ yw) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  __shared__ unsigned short rows_s[kStreamMaxRows];
  __shared__ int cnt_s[kScan * 4];
  bf16_t* hs = reinterpret_cast<bf16_t*>(smem_raw);            // [kTok][I + 8] operand rows of this pass
  const int e = blockIdx.y;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int c0 = blockIdx.x * kRowsPerWg + wave * kRowsPerWave;
  const bf16_t* wp = wd + ((size_t)e * H + c0 + (lane & 15)) * I + (lane >> 4) * 16;
  const int nlines = I / kLine;
  const bool resident = nlines <= 2 * kChunk;
  ScanRegs sr;
  scan_issue(sr, idx, S);
  const float p_e = kFusedAct ? radial_exponent(theta, e, act) : 0.f;                       // moe.py:89
  WChunk ca, cb;
  load_chunk<kWhole, 0, kFirstLines>(ca, wp, 0, nlines);
  const int n = scan_finish(sr, S, e, rows_s, cnt_s);
  for (int r0 = 0; r0 < n; r0 += kTok) {
    const int nrow = min(kTok, n - r0);
    const bool reload = r0 == 0 || !resident;
    if (r0 > 0) {
      __syncthreads();
      if (reload) load_chunk<kWhole>(ca, wp, 0, nlines);
    }
    const bool rest = r0 == 0 && kFirstLines < kChunk;
    if (kFusedAct) stage_activated<kWhole, kFirstLines>(rows_in, p_e, act, rows_s, r0, nrow, I, hs, cb, wp, nlines, reload, ca, rest);
    else stage_rows<kWhole, kFirstLines>(rows_in, rows_s, r0, nrow, 1, I, hs, cb, wp, nlines, reload, ca, rest);
    __syncthreads();
    // the fused activation is only used up to I = kFusedActMaxI = two chunks
    const floatx4 acc = stream_rows<kWhole, kFusedAct>(wp, hs, I, lane, ca, cb);
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
  // LDS: 16 rows of (max(H, I) + 8) bf16 within 56 KB (next to the 4 KB row list); every K extent must be whole
  // 128-byte lines
  return dtype == BIBO_DTYPE_BF16 && (H % 64) == 0 && (I % 64) == 0 && H <= 1728 && I <= 1728;
}

hipError_t launch_gateup_stream(const void* x, const void* wgu, const int32_t* idx, int T, int H, int E, int k, int I,
                                void* gu, hipStream_t s) {
  if (T * k == 0) return hipSuccess;
  if (T * k > kStreamMaxSlots || T > kStreamMaxRows) return hipErrorInvalidValue;
  const size_t shm = (size_t)kTok * (H + 8) * sizeof(bf16_t);
  const dim3 grid(2 * I / kRowsPerWg, E);
  if (H % (kChunk * kLine) == 0)
    hipLaunchKernelGGL(gateup_stream_kernel<true>, grid, dim3(256), shm, s, static_cast<const bf16_t*>(x),
                       static_cast<const bf16_t*>(wgu), idx, T * k, k, H, I, static_cast<bf16_t*>(gu));
  else
    hipLaunchKernelGGL(gateup_stream_kernel<false>, grid, dim3(256), shm, s, static_cast<const bf16_t*>(x),
                       static_cast<const bf16_t*>(wgu), idx, T * k, k, H, I, static_cast<bf16_t*>(gu));
  return hipGetLastError();
}

hipError_t launch_down_stream(const void* gu, const void* wd, const float* theta, const float* w, const int32_t* idx,
                              int T, int H, int E, int k, int I, int act, void* hidden, float* yw, hipStream_t s) {
  if (T * k == 0) return hipSuccess;
  if (T * k > kStreamMaxSlots || T > kStreamMaxRows) return hipErrorInvalidValue;
  const size_t shm = (size_t)kTok * (I + 8) * sizeof(bf16_t);
  const dim3 grid(H / kRowsPerWg, E);
  const bf16_t* g = static_cast<const bf16_t*>(gu);
  const bf16_t* wdp = static_cast<const bf16_t*>(wd);
  const bool whole = I % (kChunk * kLine) == 0;
  // The fused activation is computed by every one of the H/64 workgroups of an expert, once per 16-row pass:
  // cheap next to a launch for one pass, not for several
  if (I <= kFusedActMaxI && T * k <= kTok * E) {
    if (whole) hipLaunchKernelGGL((down_stream_kernel<true, true>), grid, dim3(256), shm, s, g, wdp, theta, w, idx, T * k, H, I, act, yw);
    else hipLaunchKernelGGL((down_stream_kernel<true, false>), grid, dim3(256), shm, s, g, wdp, theta, w, idx, T * k, H, I, act, yw);
  } else {
    bf16_t* hp = static_cast<bf16_t*>(hidden);
    hipLaunchKernelGGL(activate_rows_kernel, dim3(T * k), dim3(256), 0, s, g, theta, idx, E, I, act, hp);
    if (whole) hipLaunchKernelGGL((down_stream_kernel<false, true>), grid, dim3(256), shm, s, hp, wdp, theta, w, idx, T * k, H, I, act, yw);
    else hipLaunchKernelGGL((down_stream_kernel<false, false>), grid, dim3(256), shm, s, hp, wdp, theta, w, idx, T * k, H, I, act, yw);
  }
  return hipGetLastError();
}

}  // namespace bibo
