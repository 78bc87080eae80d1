// Kernel 2: per-expert histogram, prefix sum and stable permutation of the routed slots.
// Replaces the sort / bincount / cumsum / .tolist() prologue of BiBoFusedExperts.forward
// (src/modeling/ffn/moe.py:56-68) without a host synchronisation.  Row order is a stable counting
// sort of slot ids by expert, so it is identical from run to run.
#include "common.h"

namespace bibo {
namespace {

// Histogram of one chunk of kPermTokens tokens (LDS atomics; only the totals matter here).
__global__ __launch_bounds__(256) void hist_kernel(const int32_t* __restrict__ idx, int S, int E, int k,
                                                   int32_t* __restrict__ block_hist) {
  __shared__ int h[kMaxE];
  const int tid = threadIdx.x;
  if (tid < kMaxE) h[tid] = 0;
  __syncthreads();
  const int s0 = blockIdx.x * kPermTokens * k;
  const int s1 = min(S, s0 + kPermTokens * k);
  for (int s = s0 + tid; s < s1; s += 256) {
    const unsigned e = (unsigned)idx[s];
    if (e < (unsigned)E) atomicAdd(&h[e], 1);
  }
  __syncthreads();
  if (tid < kMaxE) block_hist[blockIdx.x * kMaxE + tid] = h[tid];
}

// Many histograms (large batches): sums over blocks of kHistBlock consecutive histograms, so that a scatter workgroup
// adds up the block sums and the histograms of its own block instead of every histogram in front of it.
constexpr int kHistBlock = 256;
constexpr int kTwoLevelMin = 1024;                 // histograms from which the extra launch pays

__global__ __launch_bounds__(256) void hist_blocksum_kernel(const int32_t* __restrict__ hist, int nhist,
                                                            int32_t* __restrict__ block_sum) {
  __shared__ int part[4][kMaxE];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int first = blockIdx.x * kHistBlock;
  constexpr int kPer = kHistBlock / 4;
  int v[kPer];
#pragma unroll
  for (int u = 0; u < kPer; ++u) {
    const int bb = first + wave + 4 * u;
    v[u] = bb < nhist ? hist[bb * kMaxE + lane] : 0;
  }
  int acc = 0;
#pragma unroll
  for (int u = 0; u < kPer; ++u) acc += v[u];
  part[wave][lane] = acc;
  __syncthreads();
  if (wave == 0) block_sum[blockIdx.x * kMaxE + lane] = (part[0][lane] + part[1][lane]) + (part[2][lane] + part[3][lane]);
}

// One workgroup per chunk of kPermTokens tokens, four waves of kPermTokens/4 tokens each, lane = expert for the
// bookkeeping.  (1) every wave gets the per-expert counts of its own slots; (2) the chunk histograms are
// summed (all chunks for the totals, earlier chunks for this workgroup's base), the loads issued in batches;
// (3) exclusive scan over experts; (4) every wave ranks its slots 64 at a time, slots of one expert keeping
// ascending slot order.
// HT = tokens per histogram in `hist`: kPermTokens for hist_kernel's output (the wave counts its own slots
// with ballots), 16 or 32 for the histograms the router kernel wrote per workgroup (a wave's count is the sum
// of its 32/HT histograms and no counting pass is needed).
template <int HT>
__global__ __launch_bounds__(256) void scatter_kernel(const int32_t* __restrict__ idx, int S, int E, int k,
                                                      const int32_t* __restrict__ hist, int nhist,
                                                      const int32_t* __restrict__ block_sum,
                                                      int32_t* __restrict__ counts, int32_t* __restrict__ offsets,
                                                      int32_t* __restrict__ perm_slot, int32_t* __restrict__ perm_token) {
  static_assert(kPermTokens == 128 && (HT == kPermTokens || HT == 16 || HT == 32), "a wave owns 32 tokens");
  __shared__ int part_tot[4][kMaxE], part_bef[4][kMaxE], wave_cnt[4][kMaxE];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int b = blockIdx.x;
  const int s0 = (b * kPermTokens + wave * (kPermTokens / 4)) * k;
  const int s1 = min(S, s0 + (kPermTokens / 4) * k);
  const unsigned long long lt = (1ull << lane) - 1ull;
  constexpr int kPerWg = kPermTokens / HT;          // histograms that cover this workgroup's tokens
  const int h0 = b * kPerWg;                        // the first of them

  // this wave's slots, requested before anything else: their latency passes behind the histogram sums
  constexpr int kSlotIters = (kPermTokens / 4) * kMaxK / kWave;   // 32 tokens x at most 8 slots / 64 lanes
  int ev[kSlotIters];
#pragma unroll
  for (int it = 0; it < kSlotIters; ++it) {
    const int s = s0 + it * kWave + lane;
    ev[it] = (s < s1) ? idx[s] : -1;
  }

  int mycnt = 0;                                  // slots of expert `lane` among this wave's tokens
  if constexpr (HT == kPermTokens) {
#pragma unroll
    for (int it = 0; it < kSlotIters; ++it) {
      if (s0 + it * kWave < s1) {
        const bool valid = s0 + it * kWave + lane < s1 && (unsigned)ev[it] < (unsigned)E;
        unsigned long long peers, mine;
        match64(valid ? ev[it] : 0, valid, lane, peers, mine);
        mycnt += __popcll(mine);
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < kPerWg / 4; ++i) {
      const int hh = h0 + wave * (kPerWg / 4) + i;
      if (hh < nhist) mycnt += hist[hh * kMaxE + lane];
    }
  }
  wave_cnt[wave][lane] = mycnt;

  int tot = 0, bef = 0;
  constexpr int kBatch = 64;                       // histograms requested together: one memory latency per batch
  if (block_sum == nullptr) {
    for (int bb0 = wave; bb0 < nhist; bb0 += 4 * kBatch) {
      int v[kBatch];
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        const int bb = bb0 + 4 * u;
        v[u] = (bb < nhist) ? hist[bb * kMaxE + lane] : 0;
      }
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        tot += v[u];
        bef += (bb0 + 4 * u < h0) ? v[u] : 0;
      }
    }
  } else {
    // two levels: the sums of whole blocks of histograms, then the histograms of this workgroup's own block in front
    // of its first one
    static_assert(kHistBlock == 4 * kBatch, "one batch per wave covers a block");
    const int nblk = (nhist + kHistBlock - 1) / kHistBlock, hb = h0 / kHistBlock;
    int v[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int bb = hb * kHistBlock + wave + 4 * u;
      v[u] = (bb < h0) ? hist[bb * kMaxE + lane] : 0;
    }
    for (int blk = wave; blk < nblk; blk += 4) {
      const int bs = block_sum[blk * kMaxE + lane];
      tot += bs;
      bef += blk < hb ? bs : 0;
    }
#pragma unroll
    for (int u = 0; u < kBatch; ++u) bef += v[u];
  }
  part_tot[wave][lane] = tot;
  part_bef[wave][lane] = bef;
  __syncthreads();
  const int total = (part_tot[0][lane] + part_tot[1][lane]) + (part_tot[2][lane] + part_tot[3][lane]);
  const int before = (part_bef[0][lane] + part_bef[1][lane]) + (part_bef[2][lane] + part_bef[3][lane]);
  const int incl = wave_inclusive_scan(total);
  const int excl = incl - total;
  if (b == 0 && wave == 0) {
    if (lane < E) { counts[lane] = total; offsets[lane] = excl; }
    if (lane == E - 1) offsets[E] = incl;
  }
  int cnt = excl + before;                        // next free row of expert `lane` for this wave
  for (int ww = 0; ww < wave; ++ww) cnt += wave_cnt[ww][lane];

#pragma unroll
  for (int it = 0; it < kSlotIters; ++it) {
    const int base = s0 + it * kWave;
    if (base < s1) {
      const int s = base + lane;
      const bool valid = s < s1 && (unsigned)ev[it] < (unsigned)E;
      const int e = valid ? ev[it] : 0;
      unsigned long long peers, mine;
      match64(e, valid, lane, peers, mine);
      const int pos = __shfl(cnt, e, kWave) + __popcll(peers & lt);
      if (valid) { perm_slot[pos] = s; perm_token[pos] = s / k; }
      cnt += __popcll(mine);
    }
  }
}

// Small inputs (T*k <= kSmallSlots): histogram, scan and scatter by ONE wave in one launch.  The wave spends about
// 0.7 us per 64 slots; from about 600 slots on the multi-workgroup kernels (6 us whatever the size) are faster.
constexpr int kSmallSlots = 512;

__global__ __launch_bounds__(64) void permute_small_kernel(const int32_t* __restrict__ idx, int S, int E, int k,
                                                           int32_t* __restrict__ counts, int32_t* __restrict__ offsets,
                                                           int32_t* __restrict__ perm_slot,
                                                           int32_t* __restrict__ perm_token) {
  constexpr int kChunks = kSmallSlots / kWave;
  const int lane = threadIdx.x;
  const unsigned long long lt = (1ull << lane) - 1ull;
  int ev[kChunks];                                 // every slot's expert, fetched up front: one memory latency
#pragma unroll
  for (int c = 0; c < kChunks; ++c) {
    const int s = c * kWave + lane;
    ev[c] = (s < S) ? idx[s] : -1;
  }
  int total = 0;
#pragma unroll
  for (int c = 0; c < kChunks; ++c) {
    if (c * kWave < S) {
      const bool valid = (unsigned)ev[c] < (unsigned)E;
      unsigned long long peers, mine;
      match64(valid ? ev[c] : 0, valid, lane, peers, mine);
      total += __popcll(mine);
    }
  }
  const int incl = wave_inclusive_scan(total);
  int cnt = incl - total;
  if (lane < E) { counts[lane] = total; offsets[lane] = cnt; }
  if (lane == E - 1) offsets[E] = incl;
#pragma unroll
  for (int c = 0; c < kChunks; ++c) {
    if (c * kWave < S) {
      const int s = c * kWave + lane;
      const bool valid = (unsigned)ev[c] < (unsigned)E;
      const int e = valid ? ev[c] : 0;
      unsigned long long peers, mine;
      match64(e, valid, lane, peers, mine);
      const int pos = __shfl(cnt, e, kWave) + __popcll(peers & lt);
      if (valid) { perm_slot[pos] = s; perm_token[pos] = s / k; }
      cnt += __popcll(mine);
    }
  }
}

}  // namespace

// the chunk histograms and, behind them, their block sums
size_t permute_workspace_bytes(int T) {
  const size_t nblk = (size_t)(T + kPermTokens - 1) / kPermTokens;
  return ((nblk > 0 ? nblk : 1) + nblk / kHistBlock + 1) * kMaxE * sizeof(int32_t);
}

// room for the histograms the router kernel writes, one per 16 tokens at the finest (one per 32 tokens from 8192
// tokens on, which leaves the upper half for their block sums)
size_t router_hist_bytes(int T) { return ((size_t)(T + 15) / 16 + 1) * kMaxE * sizeof(int32_t); }

// block sums of `nhist` histograms into the entries behind them, when there are enough of them to pay for the launch
static const int32_t* block_sums(int32_t* hist, int nhist, hipStream_t s) {
  if (nhist < kTwoLevelMin) return nullptr;
  int32_t* sums = hist + (size_t)nhist * kMaxE;
  hipLaunchKernelGGL(hist_blocksum_kernel, dim3((nhist + kHistBlock - 1) / kHistBlock), dim3(256), 0, s, hist, nhist, sums);
  return sums;
}

hipError_t launch_permute(const int32_t* idx, int T, int E, int k, int32_t* counts, int32_t* offsets,
                          int32_t* perm_slot, int32_t* perm_token, void* ws, hipStream_t s) {
  const int nblk = (T + kPermTokens - 1) / kPermTokens;
  int32_t* block_hist = static_cast<int32_t*>(ws);
  const int S = T * k;
  if (S <= kSmallSlots) {          // also covers T == 0: counts and offsets come out all zero
    hipLaunchKernelGGL(permute_small_kernel, dim3(1), dim3(64), 0, s, idx, S, E, k, counts, offsets, perm_slot,
                       perm_token);
    return hipGetLastError();
  }
  const int grid = nblk;
  hipLaunchKernelGGL(hist_kernel, dim3(grid), dim3(256), 0, s, idx, S, E, k, block_hist);
  hipLaunchKernelGGL(scatter_kernel<kPermTokens>, dim3(grid), dim3(256), 0, s, idx, S, E, k, block_hist, grid,
                     block_sums(block_hist, grid, s), counts, offsets, perm_slot, perm_token);
  return hipGetLastError();
}

bool permute_takes_router_hist(int T, int k) { return T * k > kSmallSlots; }

// The same permutation from the per-workgroup histograms the router kernel wrote (one per `hist_tokens` tokens):
// no histogram launch and no counting pass.
hipError_t launch_permute_from_hist(const int32_t* idx, int T, int E, int k, int32_t* hist, int hist_tokens,
                                    int32_t* counts, int32_t* offsets, int32_t* perm_slot, int32_t* perm_token,
                                    hipStream_t s) {
  const int grid = (T + kPermTokens - 1) / kPermTokens;
  const int nhist = (T + hist_tokens - 1) / hist_tokens;
  if (hist_tokens == 32)
    hipLaunchKernelGGL(scatter_kernel<32>, dim3(grid), dim3(256), 0, s, idx, T * k, E, k, hist, nhist,
                       block_sums(hist, nhist, s), counts, offsets, perm_slot, perm_token);
  else if (hist_tokens == 16)   // (fewer than 8192 tokens: never enough histograms for block sums, and no room for them)
    hipLaunchKernelGGL(scatter_kernel<16>, dim3(grid), dim3(256), 0, s, idx, T * k, E, k, hist, nhist,
                       static_cast<const int32_t*>(nullptr), counts, offsets, perm_slot, perm_token);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

}  // namespace bibo
