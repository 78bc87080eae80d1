// Kernel 1: fused router.  fp32 logits x @ w_router^T, canonical sigmoid, selection on score + bias
// (ties to the lowest expert index), gather of the unbiased scores, normalisation.
// Follows BiBoMoERouter.forward, src/modeling/ffn/router.py:25-51 of the reference.
#include "common.h"

namespace bibo {
namespace {

constexpr int kRowPad = kMaxE + 1;   // LDS row stride (floats): lane = token reads are conflict-free

// One lane owns one token: scan the E scores in ascending expert order and keep the k best
// (score + bias) in a sorted register list.  Strict '>' keeps the earlier, i.e. lower-index, expert
// ahead of an equal later one, which is the tie rule.  Emits experts in ascending index order.
__device__ __forceinline__ void select_row(const float* __restrict__ sc, const float* __restrict__ bias_s, int E,
                                           int k, int norm_mode, int32_t* __restrict__ idx_out,
                                           float* __restrict__ w_out, float* __restrict__ gap_out) {
  float sel[kMaxK];
  int id[kMaxK];
#pragma unroll
  for (int j = 0; j < kMaxK; ++j) { sel[j] = -INFINITY; id[j] = j; }
  for (int e = 0; e < E; ++e) {
    const float v = sc[e] + bias_s[e];                       // router.py:38
#pragma unroll
    for (int j = kMaxK - 1; j >= 0; --j) {
      if (j < k) {
        const bool gt_prev = (j > 0) && (v > sel[j > 0 ? j - 1 : 0]);
        if (gt_prev) { sel[j] = sel[j - (j > 0)]; id[j] = id[j - (j > 0)]; }
        else if (v > sel[j]) { sel[j] = v; id[j] = e; }
      }
    }
  }
  unsigned long long mask = 0;
#pragma unroll
  for (int j = 0; j < kMaxK; ++j)
    if (j < k) mask |= 1ull << id[j];
  // ascending expert order; weights are the UNBIASED scores (router.py:41)
  float raw[kMaxK];
  float sum = 0.f, mx = -INFINITY;
  unsigned long long m = mask;
#pragma unroll
  for (int j = 0; j < kMaxK; ++j) {
    raw[j] = 0.f;
    if (j < k) {
      const int e = __ffsll((long long)m) - 1;
      m &= m - 1;
      idx_out[j] = e;
      raw[j] = sc[e];
      sum += raw[j];                                         // sequential fp32 adds, ascending expert
      mx = fmaxf(mx, raw[j]);
    }
  }
  if (k > 1 && norm_mode == BIBO_NORM_SOFTMAX) {             // router.py:42-43
    float ex[kMaxK];
    float es = 0.f;
#pragma unroll
    for (int j = 0; j < kMaxK; ++j) { ex[j] = (j < k) ? expf(raw[j] - mx) : 0.f; es += ex[j]; }
#pragma unroll
    for (int j = 0; j < kMaxK; ++j) if (j < k) w_out[j] = ex[j] / es;
  } else if (k > 1 && norm_mode == BIBO_NORM_SUM) {          // router.py:44-45
    const float den = sum + kSumNormEps;
#pragma unroll
    for (int j = 0; j < kMaxK; ++j) if (j < k) w_out[j] = raw[j] / den;
  } else {                                                   // router.py:46-47
#pragma unroll
    for (int j = 0; j < kMaxK; ++j) if (j < k) w_out[j] = raw[j];
  }
  if (gap_out != nullptr) {                                  // router.py:33-36, unbiased scores
    float top[kMaxK + 1];
#pragma unroll
    for (int j = 0; j <= kMaxK; ++j) top[j] = -INFINITY;
    for (int e = 0; e < E; ++e) {
      const float v = sc[e];
#pragma unroll
      for (int j = kMaxK; j >= 0; --j) {
        if (j <= k) {
          const bool gt_prev = (j > 0) && (v > top[j > 0 ? j - 1 : 0]);
          if (gt_prev) top[j] = top[j - (j > 0)];
          else if (v > top[j]) top[j] = v;
        }
      }
    }
    float a = 0.f, b = 0.f;
#pragma unroll
    for (int j = 0; j <= kMaxK; ++j) { if (j == k - 1) a = top[j]; if (j == k) b = top[j]; }
    *gap_out = (k < E) ? (a - b) : 0.f;
  }
}

// ---- generic router: any H, bf16 or fp32 inputs, plain FMA -------------------------------------
constexpr int kGenTokens = 64;

template <typename TIn>
__global__ __launch_bounds__(256) void router_generic_kernel(const TIn* __restrict__ x, const TIn* __restrict__ wr,
                                                             const float* __restrict__ bias, int T, int H, int E, int k,
                                                             int norm_mode, float* __restrict__ logits,
                                                             int32_t* __restrict__ idx, float* __restrict__ w,
                                                             float* __restrict__ gap) {
  __shared__ float sc[kGenTokens * kRowPad];
  __shared__ float bias_s[kMaxE];
  const int tid = threadIdx.x;
  const int t0 = blockIdx.x * kGenTokens;
  if (tid < kMaxE) bias_s[tid] = (tid < E) ? bias[tid] : 0.f;
  {
    const int tl = tid >> 2, q = tid & 3;
    const int t = min(t0 + tl, T - 1);
    float acc[kMaxE / 4];
#pragma unroll
    for (int j = 0; j < kMaxE / 4; ++j) acc[j] = 0.f;
    const TIn* xr = x + (size_t)t * H;
    for (int h = 0; h < H; ++h) {
      const float xv = to_float(xr[h]);
#pragma unroll
      for (int j = 0; j < kMaxE / 4; ++j) {
        const int e = q + 4 * j;
        if (e < E) acc[j] = fmaf(xv, to_float(wr[(size_t)e * H + h]), acc[j]);
      }
    }
#pragma unroll
    for (int j = 0; j < kMaxE / 4; ++j) {
      const int e = q + 4 * j;
      if (e < E) sc[tl * kRowPad + e] = acc[j];
    }
  }
  __syncthreads();
  const int ntok = min(kGenTokens, T - t0);
  for (int i = tid; i < ntok * E; i += 256) {
    const int tl = i / E, e = i - tl * E;
    const float lg = sc[tl * kRowPad + e];
    if (logits != nullptr) logits[(size_t)(t0 + tl) * E + e] = lg;
    sc[tl * kRowPad + e] = sigmoid32_canonical(lg);          // router.py:31
  }
  __syncthreads();
  if (tid < ntok) {
    const int t = t0 + tid;
    select_row(sc + tid * kRowPad, bias_s, E, k, norm_mode, idx + (size_t)t * k, w + (size_t)t * k,
               gap ? gap + t : nullptr);
  }
}

// Integer key of a score whose unsigned order is the order of the floats (-0 counts as +0): the row-wide maximum
// is then one v_max_u32 per butterfly step instead of a compare-and-select on (value, expert) pairs under exec
// masks, which cost this selection 3.5 us per workgroup.
__device__ __forceinline__ unsigned order_key(float v) {
  const unsigned u = __float_as_uint(v + 0.f);
  return u ^ ((unsigned)((int)u >> 31) | 0x80000000u);
}
__device__ __forceinline__ float key_value(unsigned key) {
  return __uint_as_float((key & 0x80000000u) ? key ^ 0x80000000u : ~key);
}

template <int kCtrl>
__device__ __forceinline__ unsigned dpp_u32(unsigned v) {
  return (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, kCtrl, 0xf, 0xf, false);
}
// 16-lane butterfly on DPP row operations (a DPP row is exactly one token's 16 lanes): swap within pairs, swap
// pairs within quads, mirror within 8 lanes, mirror within 16 lanes.  Every lane ends with the row's result.
__device__ __forceinline__ unsigned row_max_u32(unsigned v) {
  v = max(v, dpp_u32<0xB1>(v));
  v = max(v, dpp_u32<0x4E>(v));
  v = max(v, dpp_u32<0x141>(v));
  return max(v, dpp_u32<0x140>(v));
}
__device__ __forceinline__ unsigned row_min_u32(unsigned v) {
  v = min(v, dpp_u32<0xB1>(v));
  v = min(v, dpp_u32<0x4E>(v));
  v = min(v, dpp_u32<0x141>(v));
  return min(v, dpp_u32<0x140>(v));
}

// Cooperative selection: 16 lanes per token, lane `seg` owns experts 4*seg .. 4*seg+3.  k rounds of
// "best remaining candidate": the row's largest key, then the lowest expert index among the lanes that hold it,
// which is the tie rule (equal floats have equal keys).  All 16 lanes end every round with the same winner.
// Returns the bit mask of the chosen experts.
__device__ __forceinline__ unsigned long long select_mask16(const float (&v)[4], int seg, int rounds, float* kth,
                                                            float* kth1) {
  unsigned key[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) key[q] = order_key(v[q]);
  unsigned taken = 0;
  unsigned long long mask = 0;
  for (int r = 0; r < rounds; ++r) {
    unsigned bk = 0, be = kMaxE;                     // a taken expert counts as key 0, below every score's key
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const unsigned kq = ((taken >> q) & 1) ? 0u : key[q];
      if (kq > bk) { bk = kq; be = seg * 4 + q; }    // strict: the lower expert of the lane keeps an equal key
    }
    const unsigned mk = row_max_u32(bk);
    be = row_min_u32(bk == mk ? be : (unsigned)kMaxE);
    be &= kMaxE - 1;
    if ((int)(be >> 2) == seg) taken |= 1u << (be & 3);
    mask |= 1ull << be;
    if (kth != nullptr) { if (r == rounds - 2) *kth = key_value(mk); if (r == rounds - 1) *kth1 = key_value(mk); }
  }
  return mask;
}

// Selection for the tokens of one workgroup whose scores sit in LDS rows `sc` (stride kRowPad):
// thread = (token tid>>4, segment tid&15); needs blockDim.x >= 16 * ntok_max.  Lane j < k of a token's 16 then
// owns output j (the j-th chosen expert in ascending order): it gathers the unbiased score, the row adds the scores
// up one after the other in that order (a serial scan over lanes, so the sum has the bits of the sequential loop),
// and every lane normalises and stores its own weight.
// Returns the bit mask of the experts chosen for this thread's token (0 for a token past the end).
__device__ __forceinline__ unsigned long long select_tokens16(const float* __restrict__ sc,
                                                              const float* __restrict__ bias_s, int E, int k,
                                                              int norm_mode, int t0, int ntok, int32_t* __restrict__ idx,
                                                              float* __restrict__ w, float* __restrict__ gap) {
  const int tid = threadIdx.x;
  const int tl = tid >> 4, seg = tid & 15;
  const bool live = tl < ntok;                       // whole 16-lane groups are live or not
  const float* row = sc + (live ? tl : 0) * kRowPad;
  float v[4], u[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int e = seg * 4 + q;
    u[q] = (e < E) ? row[e] : -INFINITY;
    v[q] = (e < E) ? row[e] + bias_s[e] : -INFINITY;                      // router.py:38
  }
  const unsigned long long mask = select_mask16(v, seg, k, nullptr, nullptr);
  float g_hi = 0.f, g_lo = 0.f;
  if (gap != nullptr && k < E) select_mask16(u, seg, k + 1, &g_hi, &g_lo);   // router.py:33-36, unbiased scores
  const bool mine = seg < k;                                              // this lane owns output `seg`
  unsigned long long m = mask;
#pragma unroll
  for (int j = 0; j < kMaxK - 1; ++j)
    if (j < seg) m &= m - 1;                                              // drop the `seg` lowest chosen experts
  const int e = mine ? __ffsll((long long)m) - 1 : 0;                     // ascending expert order
  const float raw = mine ? row[e] : 0.f;                                  // UNBIASED score, router.py:41
  // running sum in ascending j, one lane after the other: lane j ends with ((raw_0 + raw_1) + ...) + raw_j
  auto scan = [&](float x) {
    float s = x;
#pragma unroll
    for (int j = 1; j < kMaxK; ++j) {
      const float prev = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, s), 0x111, 0xf, 0xf, false));
      if (seg == j && j < k) s = prev + x;                                // row_shr:1, lane j reads lane j-1
    }
    return __shfl(s, (tid & 48) + k - 1, kWave);                          // the whole sum, from lane k-1 of the row
  };
  float wv = raw;                                                         // router.py:46-47
  if (k > 1 && norm_mode == BIBO_NORM_SOFTMAX) {                          // router.py:42-43
    const float mx = key_value(row_max_u32(mine ? order_key(raw) : 0u));
    const float ex = mine ? expf(raw - mx) : 0.f;
    wv = ex / scan(ex);
  } else if (k > 1 && norm_mode == BIBO_NORM_SUM) {                       // router.py:44-45
    wv = raw / (scan(raw) + kSumNormEps);
  }
  if (live && mine) {
    const size_t o = (size_t)(t0 + tl) * k + seg;
    idx[o] = e;
    w[o] = wv;
  }
  if (live && seg == 0 && gap != nullptr) gap[t0 + tl] = (k < E) ? (g_hi - g_lo) : 0.f;
  return live ? mask : 0ull;
}

// ---- MFMA router: bf16, H % 128 == 0 ------------------------------------------------------------
// One workgroup = TOK tokens (16 or 32), TOK/16 x 4 waves: wave (tm, en) owns the 16x16 logits tile of
// token tile tm and expert tile en over the whole K, so no partial sums cross waves and the fp32
// accumulation order is fixed.  x rows and w_router rows travel global -> LDS by LDS-DMA in K chunks of
// 128 elements (256-byte rows, one instruction fetches four whole rows per wave), double-buffered:
// fetching w_router straight into registers costs a CU about 37 GB/s, the DMA path twice that, and
// every workgroup needs all of w_router.  Granule c of row r sits at position c ^ (r & 15).
constexpr int kRouterKC = 128;                       // K elements per chunk
constexpr int kRouterGran = kRouterKC / 8;           // 16-byte granules per chunk row

typedef __attribute__((address_space(3))) void router_lds_void;
typedef const __attribute__((address_space(1))) void router_gbl_void;

// Everything after the logits of a TOK-token workgroup: canonical sigmoid on the accumulator registers, selection,
// weights, and the workgroup's histogram of selected experts.  Wave (tm, en) holds the 16x16 logits tile of token
// tile tm and expert tile en: lane = column (expert) lane%16, rows (tokens) 4*(lane/16)+i.
template <int TOK>
__device__ __forceinline__ void router_finish(const floatx4& acc, float* sc, const float* bias_s, int T, int E, int k,
                                              int norm_mode, int t0, float* __restrict__ logits, int32_t* __restrict__ idx,
                                              float* __restrict__ w, float* __restrict__ gap,
                                              int32_t* __restrict__ chunk_hist) {
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int tm = wave >> 2, en = wave & 3;
  const int r16 = lane & 15, kc = lane >> 4;
  const int ntok = min(TOK, T - t0);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int tl = tm * 16 + kc * 4 + i, e = en * 16 + r16;
    if (tl < ntok && e < E) {
      const float lg = acc[i];
      if (logits != nullptr) logits[(size_t)(t0 + tl) * E + e] = lg;
      sc[tl * kRowPad + e] = sigmoid32_canonical(lg);          // router.py:31
    }
  }
  __syncthreads();
  const unsigned long long mask = select_tokens16(sc, bias_s, E, k, norm_mode, t0, ntok, idx, w, gap);
  if (chunk_hist != nullptr) {           // histogram of this workgroup's selections, for the permutation kernel
    __shared__ unsigned long long mask_s[TOK];
    if ((tid & 15) == 0) mask_s[tid >> 4] = mask;
    __syncthreads();
    if (tid < kMaxE) {
      int c = 0;
#pragma unroll
      for (int t = 0; t < TOK; ++t) c += (int)((mask_s[t] >> tid) & 1ull);
      chunk_hist[blockIdx.x * kMaxE + tid] = c;
    }
  }
}

template <int TOK>
__global__ __launch_bounds__(TOK * 16) void router_mfma_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ wr,
                                                               const float* __restrict__ bias, int T, int H, int E,
                                                               int k, int norm_mode, float* __restrict__ logits,
                                                               int32_t* __restrict__ idx, float* __restrict__ w,
                                                               float* __restrict__ gap,
                                                               int32_t* __restrict__ chunk_hist) {
  constexpr int kThreads = TOK * 16;
  constexpr int kRows = TOK + kMaxE;                 // stage rows: tokens first, then experts
  constexpr int kPer = kRows * kRouterGran / kThreads;   // load instructions per thread and chunk
  static_assert(kRows * kRouterGran % kThreads == 0, "stage does not divide over the threads");
  __shared__ __attribute__((aligned(16))) bf16_t st0[kRows * kRouterKC];
  __shared__ __attribute__((aligned(16))) bf16_t st1[kRows * kRouterKC];
  __shared__ float sc[TOK * kRowPad];
  __shared__ float bias_s[kMaxE];
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int t0 = blockIdx.x * TOK;
  if (tid < kMaxE) bias_s[tid] = (tid < E) ? bias[tid] : 0.f;

  // thread t of load instruction i fills granule i*kThreads + t = (row, position t % 16) and fetches logical
  // granule (t % 16) ^ (row % 16) of that row
  const bf16_t* src[kPer];
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    const int row = (i * kThreads + tid) / kRouterGran;
    const int c = (tid & (kRouterGran - 1)) ^ (row & 15);
    src[i] = (row < TOK ? x + (size_t)min(t0 + row, T - 1) * H : wr + (size_t)min(row - TOK, E - 1) * H) + c * 8;
  }
  auto issue = [&](int k0, bf16_t* st) {
#pragma unroll
    for (int i = 0; i < kPer; ++i)
      __builtin_amdgcn_global_load_lds((router_gbl_void*)(src[i] + k0), (router_lds_void*)(st + (i * kThreads + wave * 64) * 8),
                                       16, 0, 0);
  };
  const int tm = wave >> 2, en = wave & 3;
  const int r16 = lane & 15, kc = lane >> 4;         // fragment row, 8-wide k chunk of a 32-wide step
  floatx4 acc = {0.f, 0.f, 0.f, 0.f};
  auto multiply = [&](const bf16_t* st) {
    const bf16_t* arow = st + (tm * 16 + r16) * kRouterKC;
    const bf16_t* brow = st + (TOK + en * 16 + r16) * kRouterKC;
#pragma unroll
    for (int s = 0; s < kRouterKC / 32; ++s) {
      const int pos = ((s * 4 + kc) ^ r16) * 8;      // both rows are r16 mod 16
      const bf16x8 a = *reinterpret_cast<const bf16x8*>(arow + pos);
      const bf16x8 b = *reinterpret_cast<const bf16x8*>(brow + pos);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc, 0, 0, 0);
    }
  };
  issue(0, st0);
  for (int k0 = 0; k0 < H; k0 += 2 * kRouterKC) {
    __builtin_amdgcn_s_waitcnt(0);                   // vmcnt(0): this thread's transfers have landed
    __syncthreads();
    if (k0 + kRouterKC < H) issue(k0 + kRouterKC, st1);
    multiply(st0);
    if (k0 + kRouterKC < H) {
      __builtin_amdgcn_s_waitcnt(0);
      __syncthreads();
      if (k0 + 2 * kRouterKC < H) issue(k0 + 2 * kRouterKC, st0);
      multiply(st1);
    }
  }
  router_finish<TOK>(acc, sc, bias_s, T, E, k, norm_mode, t0, logits, idx, w, gap, chunk_hist);
}

// ---- MFMA router with the block's input RMSNorm in front (the caller's seam) ----------------------
// out = h + moe(post_attention_layernorm(h)) (src/modeling/layers.py:57-64) needs the normalised rows twice: as the
// router's operand and as the rows the expert kernels gather.  This kernel reads the raw rows once: all H elements of
// its TOK rows arrive in LDS by LDS-DMA, one wave per row computes BiBoRMSNorm (src/modeling/norm.py:19-24) with the
// arithmetic and the summation order of rmsnorm_bf16x8_kernel (so both produce the same bits), writes the normalised
// row back to LDS in place and to `xn` in memory, and the logits are then multiplied from the resident rows while
// w_router streams through two LDS stages as in router_mfma_kernel.  x rows are stored as H/128 chunks of
// [TOK][128], granule c of a chunk row r at position c ^ (r & 15).
template <int TOK>
__global__ __launch_bounds__(TOK * 16) void router_norm_mfma_kernel(const bf16_t* __restrict__ h, const float* __restrict__ nw,
                                                                    float eps, const bf16_t* __restrict__ wr,
                                                                    const float* __restrict__ bias, int T, int H, int E,
                                                                    int k, int norm_mode, bf16_t* __restrict__ xn,
                                                                    float* __restrict__ logits, int32_t* __restrict__ idx,
                                                                    float* __restrict__ w, float* __restrict__ gap,
                                                                    int32_t* __restrict__ chunk_hist) {
  constexpr int kThreads = TOK * 16;
  constexpr int kWPer = kMaxE * kRouterGran / kThreads;      // w_router load instructions per thread and chunk
  extern __shared__ __attribute__((aligned(16))) bf16_t xs[];                 // [H/128][TOK][128]
  __shared__ __attribute__((aligned(16))) bf16_t wst0[kMaxE * kRouterKC];
  __shared__ __attribute__((aligned(16))) bf16_t wst1[kMaxE * kRouterKC];
  __shared__ float sc[TOK * kRowPad];
  __shared__ float bias_s[kMaxE];
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int t0 = blockIdx.x * TOK;
  const int nchunks = H / kRouterKC;
  if (tid < kMaxE) bias_s[tid] = (tid < E) ? bias[tid] : 0.f;

  // w_router chunk loads: thread t of instruction i fills granule i*kThreads + t = (row, position t % 16)
  const bf16_t* wsrc[kWPer];
#pragma unroll
  for (int i = 0; i < kWPer; ++i) {
    const int row = (i * kThreads + tid) / kRouterGran;
    wsrc[i] = wr + (size_t)min(row, E - 1) * H + ((tid & (kRouterGran - 1)) ^ (row & 15)) * 8;
  }
  auto issue_w = [&](int k0, bf16_t* st) {
#pragma unroll
    for (int i = 0; i < kWPer; ++i)
      __builtin_amdgcn_global_load_lds((router_gbl_void*)(wsrc[i] + k0), (router_lds_void*)(st + (i * kThreads + wave * 64) * 8),
                                       16, 0, 0);
  };
  issue_w(0, wst0);
  // the raw rows: instruction i is chunk i of every row (TOK * 16 granules = one per thread)
  {
    const int row = tid >> 4;
    const bf16_t* src = h + (size_t)min(t0 + row, T - 1) * H + ((tid & 15) ^ (row & 15)) * 8;
    for (int i = 0; i < nchunks; ++i)
      __builtin_amdgcn_global_load_lds((router_gbl_void*)(src + i * kRouterKC),
                                       (router_lds_void*)(xs + (i * kThreads + wave * 64) * 8), 16, 0, 0);
  }
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  // RMSNorm, one wave per row, four rows per wave; lane takes logical granules u*64 + lane of the row
  {
    const int ngran = H / 8;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int r = wave * 4 + j;
      bf16x8 v[4];
      bf16_t* loc[4];
      float ss = 0.f;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int c = u * kWave + lane;
        if (c < ngran) {
          loc[u] = xs + (((c >> 4) * TOK + r) * kRouterGran + ((c & 15) ^ (r & 15))) * 8;
          v[u] = *reinterpret_cast<const bf16x8*>(loc[u]);
#pragma unroll
          for (int q = 0; q < 8; ++q) ss = fmaf((float)v[u][q], (float)v[u][q], ss);
        }
      }
      ss = wave_sum(ss);
      const float rinv = rsqrtf(ss / (float)H + eps);                                   // norm.py:22-23
      const bool live = t0 + r < T;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int c = u * kWave + lane;
        if (c < ngran) {
          bf16x8 o;
#pragma unroll
          for (int q = 0; q < 8; ++q) o[q] = (bf16_t)(nw[c * 8 + q] * (float)(bf16_t)((float)v[u][q] * rinv));   // norm.py:24
          *reinterpret_cast<bf16x8*>(loc[u]) = o;
          if (live) *reinterpret_cast<bf16x8*>(xn + (size_t)(t0 + r) * H + c * 8) = o;
        }
      }
    }
  }
  const int tm = wave >> 2, en = wave & 3;
  const int r16 = lane & 15, kc = lane >> 4;
  floatx4 acc = {0.f, 0.f, 0.f, 0.f};
  auto multiply = [&](const bf16_t* xa, const bf16_t* st) {
    const bf16_t* arow = xa + (tm * 16 + r16) * kRouterKC;
    const bf16_t* brow = st + (en * 16 + r16) * kRouterKC;
#pragma unroll
    for (int s = 0; s < kRouterKC / 32; ++s) {
      const int pos = ((s * 4 + kc) ^ r16) * 8;
      const bf16x8 a = *reinterpret_cast<const bf16x8*>(arow + pos);
      const bf16x8 b = *reinterpret_cast<const bf16x8*>(brow + pos);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc, 0, 0, 0);
    }
  };
  for (int c0 = 0; c0 < nchunks; c0 += 2) {
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();                                   // first pass: also the normalised rows of the other waves
    if (c0 + 1 < nchunks) issue_w((c0 + 1) * kRouterKC, wst1);
    multiply(xs + (size_t)c0 * TOK * kRouterKC, wst0);
    if (c0 + 1 < nchunks) {
      __builtin_amdgcn_s_waitcnt(0);
      __syncthreads();
      if (c0 + 2 < nchunks) issue_w((c0 + 2) * kRouterKC, wst0);
      multiply(xs + (size_t)(c0 + 1) * TOK * kRouterKC, wst1);
    }
  }
  router_finish<TOK>(acc, sc, bias_s, T, E, k, norm_mode, t0, logits, idx, w, gap, chunk_hist);
}

// ---- MFMA router for H % 32 == 0 but not % 128: operands straight to registers, K split over 4 waves ----
constexpr int kMfmaTokens = 16;

__global__ __launch_bounds__(256) void router_mfma_split_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ wr,
                                                                const float* __restrict__ bias, int T, int H, int E,
                                                                int k, int norm_mode, float* __restrict__ logits,
                                                                int32_t* __restrict__ idx, float* __restrict__ w,
                                                                float* __restrict__ gap) {
  __shared__ float part[4 * kMfmaTokens * kRowPad];
  __shared__ float sc[kMfmaTokens * kRowPad];
  __shared__ float bias_s[kMaxE];
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int t0 = blockIdx.x * kMfmaTokens;
  if (tid < kMaxE) bias_s[tid] = (tid < E) ? bias[tid] : 0.f;

  const int r16 = lane & 15, kc = lane >> 4;                 // fragment row, 8-wide k chunk
  const bf16_t* xa = x + (size_t)min(t0 + r16, T - 1) * H + kc * 8;
  const bf16_t* wb[4];
#pragma unroll
  for (int nt = 0; nt < 4; ++nt) wb[nt] = wr + (size_t)min(nt * 16 + r16, E - 1) * H + kc * 8;
  floatx4 acc[4];
#pragma unroll
  for (int nt = 0; nt < 4; ++nt) acc[nt] = floatx4{0.f, 0.f, 0.f, 0.f};
  const int nsteps = H / 32;
  constexpr int kU = 8;                                      // K steps whose loads are issued together (160 VGPRs)
  for (int s0 = wave; s0 < nsteps; s0 += 4 * kU) {
    bf16x8 a[kU], b[kU][4];
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      const int s = s0 + 4 * u;
      if (s < nsteps) {
        a[u] = *reinterpret_cast<const bf16x8*>(xa + s * 32);
#pragma unroll
        for (int nt = 0; nt < 4; ++nt) b[u][nt] = *reinterpret_cast<const bf16x8*>(wb[nt] + s * 32);
      }
    }
#pragma unroll
    for (int u = 0; u < kU; ++u)
      if (s0 + 4 * u < nsteps) {
#pragma unroll
        for (int nt = 0; nt < 4; ++nt) acc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u], b[u][nt], acc[nt], 0, 0, 0);
      }
  }
  // D layout of the 16x16 tile: lane holds column (expert) lane%16, rows (tokens) 4*(lane/16)+i
#pragma unroll
  for (int nt = 0; nt < 4; ++nt)
#pragma unroll
    for (int i = 0; i < 4; ++i)
      part[(wave * kMfmaTokens + kc * 4 + i) * kRowPad + nt * 16 + r16] = acc[nt][i];
  __syncthreads();
  const int ntok = min(kMfmaTokens, T - t0);
  for (int i = tid; i < kMfmaTokens * kMaxE; i += 256) {
    const int tl = i >> 6, e = i & 63;
    if (tl < ntok && e < E) {
      const int o = tl * kRowPad + e;
      const float lg = ((part[o] + part[kMfmaTokens * kRowPad + o]) + part[2 * kMfmaTokens * kRowPad + o]) +
                       part[3 * kMfmaTokens * kRowPad + o];
      if (logits != nullptr) logits[(size_t)(t0 + tl) * E + e] = lg;
      sc[o] = sigmoid32_canonical(lg);                       // router.py:31
    }
  }
  __syncthreads();
  select_tokens16(sc, bias_s, E, k, norm_mode, t0, ntok, idx, w, gap);
}

}  // namespace

// The widest hidden size whose TOK raw rows fit LDS next to the w_router stages (TOK = 32: 64 KB of rows).
constexpr int kNormRouterMaxH = 1024;

bool router_norm_supported(int H, int dtype, const void* h, const void* w_router, const void* xn) {
  const bool aligned = ((reinterpret_cast<uintptr_t>(h) | reinterpret_cast<uintptr_t>(w_router) |
                         reinterpret_cast<uintptr_t>(xn)) & 15) == 0;
  return dtype == BIBO_DTYPE_BF16 && (H % kRouterKC) == 0 && H <= kNormRouterMaxH && aligned;
}

// the kernel's TOK whole rows sit in dynamic LDS: allowed once per device, for the widest rows it takes
template <int TOK>
hipError_t allow_dynamic_lds() {
  static LdsLimitOnce once;
  return once.raise(reinterpret_cast<const void*>(&router_norm_mfma_kernel<TOK>), (int)(TOK * kNormRouterMaxH * sizeof(bf16_t)));
}

// RMSNorm + router in one launch (see router_norm_mfma_kernel); `xn` receives the normalised rows.
hipError_t launch_router_norm(const void* h, const float* norm_weight, float eps, const void* w_router, const float* bias,
                              int T, int H, int E, int k, int norm_mode, void* xn, float* logits, int32_t* idx, float* w,
                              int32_t* chunk_hist, int* hist_tokens, hipStream_t s) {
  if (hist_tokens != nullptr) *hist_tokens = 0;
  if (T == 0) return hipSuccess;
  const bf16_t* hp = static_cast<const bf16_t*>(h);
  const bf16_t* wp = static_cast<const bf16_t*>(w_router);
  bf16_t* xp = static_cast<bf16_t*>(xn);
  hipError_t e;
  if (T >= 32 * 256) {
    const size_t shm = (size_t)32 * H * sizeof(bf16_t);
    if ((e = allow_dynamic_lds<32>()) != hipSuccess) return e;
    hipLaunchKernelGGL(router_norm_mfma_kernel<32>, dim3((T + 31) / 32), dim3(512), shm, s, hp, norm_weight, eps, wp, bias, T,
                       H, E, k, norm_mode, xp, logits, idx, w, nullptr, chunk_hist);
  } else {
    const size_t shm = (size_t)16 * H * sizeof(bf16_t);
    if ((e = allow_dynamic_lds<16>()) != hipSuccess) return e;
    hipLaunchKernelGGL(router_norm_mfma_kernel<16>, dim3((T + 15) / 16), dim3(256), shm, s, hp, norm_weight, eps, wp, bias, T,
                       H, E, k, norm_mode, xp, logits, idx, w, nullptr, chunk_hist);
  }
  if (hist_tokens != nullptr && chunk_hist != nullptr) *hist_tokens = T >= 32 * 256 ? 32 : 16;
  return hipGetLastError();
}

hipError_t launch_router(const void* x, const void* w_router, const float* bias, int T, int H, int E, int k, int dtype,
                         int norm_mode, float* logits, int32_t* idx, float* w, float* gap, int32_t* chunk_hist,
                         int* hist_tokens, hipStream_t s) {
  if (hist_tokens != nullptr) *hist_tokens = 0;
  if (T == 0) return hipSuccess;
  const bool aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w_router)) & 15) == 0;
  if (dtype == BIBO_DTYPE_BF16 && (H % kRouterKC) == 0 && aligned) {
    // 32 tokens per workgroup halve the w_router traffic per token; below 256 workgroups' worth of tokens the
    // smaller tile keeps more CUs busy
    if (T >= 32 * 256)
      hipLaunchKernelGGL(router_mfma_kernel<32>, dim3((T + 31) / 32), dim3(512), 0, s, static_cast<const bf16_t*>(x),
                         static_cast<const bf16_t*>(w_router), bias, T, H, E, k, norm_mode, logits, idx, w, gap,
                         chunk_hist);
    else
      hipLaunchKernelGGL(router_mfma_kernel<16>, dim3((T + 15) / 16), dim3(256), 0, s, static_cast<const bf16_t*>(x),
                         static_cast<const bf16_t*>(w_router), bias, T, H, E, k, norm_mode, logits, idx, w, gap,
                         chunk_hist);
    if (hist_tokens != nullptr && chunk_hist != nullptr) *hist_tokens = T >= 32 * 256 ? 32 : 16;
  } else if (dtype == BIBO_DTYPE_BF16 && (H % 32) == 0 && aligned) {
    const int grid = (T + kMfmaTokens - 1) / kMfmaTokens;
    hipLaunchKernelGGL(router_mfma_split_kernel, dim3(grid), dim3(256), 0, s, static_cast<const bf16_t*>(x),
                       static_cast<const bf16_t*>(w_router), bias, T, H, E, k, norm_mode, logits, idx, w, gap);
  } else {
    const int grid = (T + kGenTokens - 1) / kGenTokens;
    if (dtype == BIBO_DTYPE_BF16)
      hipLaunchKernelGGL(router_generic_kernel<bf16_t>, dim3(grid), dim3(256), 0, s, static_cast<const bf16_t*>(x),
                         static_cast<const bf16_t*>(w_router), bias, T, H, E, k, norm_mode, logits, idx, w, gap);
    else
      hipLaunchKernelGGL(router_generic_kernel<float>, dim3(grid), dim3(256), 0, s, static_cast<const float*>(x),
                         static_cast<const float*>(w_router), bias, T, H, E, k, norm_mode, logits, idx, w, gap);
  }
  return hipGetLastError();
}

}  // namespace bibo
