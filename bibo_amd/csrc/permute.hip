// Kernel 2: per-expert histogram, prefix sum and stable permutation of the routed slots.
// Replaces the sort / bincount / cumsum / .tolist() prologue of BiBoFusedExperts.forward
// (src/modeling/ffn/moe.py:56-68) without a host synchronisation.  Row order is a stable counting
// sort of slot ids by expert, so it is identical from run to run.
#include "common.h"

namespace bibo {
namespace {

// One wave per 64 tokens: LDS histogram of the chunk's slots.
__global__ __launch_bounds__(64) void hist_kernel(const int32_t* __restrict__ idx, int S, int E, int k,
                                                  int32_t* __restrict__ block_hist) {
  __shared__ int h[kMaxE];
  const int lane = threadIdx.x;
  h[lane] = 0;
  __syncthreads();
  const int s0 = blockIdx.x * kPermTokens * k;
  const int s1 = min(S, s0 + kPermTokens * k);
  for (int s = s0 + lane; s < s1; s += kWave) {
    const unsigned e = (unsigned)idx[s];
    if (e < (unsigned)E) atomicAdd(&h[e], 1);
  }
  __syncthreads();
  block_hist[blockIdx.x * kMaxE + lane] = h[lane];
}

// One wave per 64 tokens, lane = expert for the bookkeeping.  Each wave sums the chunk histograms
// (all of them for the totals, the earlier ones for its own base), scans over experts, then ranks
// its slots 64 at a time with ballots: slots of one expert keep ascending slot order.
__global__ __launch_bounds__(64) void scatter_kernel(const int32_t* __restrict__ idx, int S, int E, int k,
                                                     const int32_t* __restrict__ block_hist,
                                                     int32_t* __restrict__ counts, int32_t* __restrict__ offsets,
                                                     int32_t* __restrict__ perm_slot, int32_t* __restrict__ perm_token) {
  const int lane = threadIdx.x;
  const int b = blockIdx.x, nblk = gridDim.x;
  int total = 0, before = 0;
  for (int bb = 0; bb < nblk; ++bb) {
    const int v = block_hist[bb * kMaxE + lane];
    total += v;
    before += (bb < b) ? v : 0;
  }
  const int incl = wave_inclusive_scan(total);
  const int excl = incl - total;
  if (b == 0) {
    if (lane < E) { counts[lane] = total; offsets[lane] = excl; }
    if (lane == E - 1) offsets[E] = incl;
  }
  int cnt = excl + before;                       // next free row of expert `lane`
  const int s0 = b * kPermTokens * k;
  const int s1 = min(S, s0 + kPermTokens * k);
  const unsigned long long lt = (1ull << lane) - 1ull;
  for (int base = s0; base < s1; base += kWave) {
    const int s = base + lane;
    int e = 0;
    bool valid = s < s1;
    if (valid) { e = idx[s]; valid = (unsigned)e < (unsigned)E; }
    if (!valid) e = 0;
    const unsigned long long vmask = __ballot(valid);
    unsigned long long peers = vmask;            // lanes whose slot has my expert
    unsigned long long mine = vmask;             // lanes whose slot has expert == my lane id
#pragma unroll
    for (int bit = 0; bit < 6; ++bit) {
      const unsigned long long bb = __ballot(valid && ((e >> bit) & 1));
      peers &= ((e >> bit) & 1) ? bb : ~bb;
      mine &= ((lane >> bit) & 1) ? bb : ~bb;
    }
    const int rank = __popcll(peers & lt);
    const int pos = __shfl(cnt, e, kWave) + rank;
    if (valid) { perm_slot[pos] = s; perm_token[pos] = s / k; }
    cnt += __popcll(mine);
  }
}

}  // namespace

size_t permute_workspace_bytes(int T) {
  const size_t nblk = (size_t)(T + kPermTokens - 1) / kPermTokens;
  return (nblk > 0 ? nblk : 1) * kMaxE * sizeof(int32_t);
}

hipError_t launch_permute(const int32_t* idx, int T, int E, int k, int32_t* counts, int32_t* offsets,
                          int32_t* perm_slot, int32_t* perm_token, void* ws, hipStream_t s) {
  const int nblk = (T + kPermTokens - 1) / kPermTokens;
  int32_t* block_hist = static_cast<int32_t*>(ws);
  const int S = T * k;
  // T == 0 still has to produce counts = 0 and offsets = 0: one chunk with no slots does that.
  const int grid = nblk > 0 ? nblk : 1;
  hipLaunchKernelGGL(hist_kernel, dim3(grid), dim3(64), 0, s, idx, S, E, k, block_hist);
  hipLaunchKernelGGL(scatter_kernel, dim3(grid), dim3(64), 0, s, idx, S, E, k, block_hist, counts, offsets,
                     perm_slot, perm_token);
  return hipGetLastError();
}

}  // namespace bibo
