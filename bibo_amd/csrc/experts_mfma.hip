// Kernels 3 and 4: grouped expert GEMMs on bf16 MFMA (v_mfma_f32_32x32x16_bf16), gfx950.
//
// Both kernels compute BM = 128 permuted rows of one expert against a block of weight rows.  A
// (activations) and B (weights, stored [N,K] K-contiguous exactly as the reference keeps them) travel
// global -> LDS by LDS-DMA (global_load_lds_dwordx4) in K steps of 32 elements, double-buffered: the
// loads of step s+1 are issued while step s is multiplied, one barrier per step.  Eight waves, 2 along
// M x 4 along N, each holding MT x NTW accumulator tiles of 32x32 (192 accumulator registers at most:
// past 256 the compiler shuttles accumulators between the two register files and spills).
//
//   kernel 3 (gate/up): the workgroup covers ALL I gate columns and ALL I up columns of its rows, so the
//     row-wise mean of gate^2 that Radial NormSiLU needs is complete inside the workgroup; wave
//     (wm, wn) owns gate columns [wn*I/4, (wn+1)*I/4) and the SAME up columns, so act(gate)*up is
//     formed in registers.  Reference: src/modeling/ffn/moe.py:81-92.
//   kernel 4 (down): N is a 128*NTW wide block of hidden columns; the epilogue multiplies each row by its
//     routing weight and scatters it to slot order (token-major), where `combine` sums the k rows of a
//     token.  Reference: src/modeling/ffn/moe.py:92-93,101.
#include <utility>

#include "common.h"

namespace bibo {
namespace {

constexpr int kLoadsPerPair = 1;
constexpr int kBK = 32;        // K elements per LDS stage

struct TileMap {
  int incl;    // lane = expert: inclusive tile count
  int ntile;   // lane = expert: tiles of this expert
  int total;
};

__device__ __forceinline__ TileMap make_tile_map(const int32_t* __restrict__ offsets, int E, int BM) {
  const int lane = lane_id();
  int lo = 0, hi = 0;
  if (lane < E) { lo = offsets[lane]; hi = offsets[lane + 1]; }
  TileMap tm;
  tm.ntile = (hi - lo + BM - 1) / BM;
  tm.incl = wave_inclusive_scan(tm.ntile);
  tm.total = __shfl(tm.incl, kWave - 1, kWave);
  return tm;
}

// tile < tm.total required
__device__ __forceinline__ void find_tile(const TileMap& tm, const int32_t* __restrict__ offsets, int BM, int tile,
                                          int& expert, int& row0, int& rows) {
  const unsigned long long m = __ballot(tm.incl > tile);
  expert = __ffsll((long long)m) - 1;
  const int excl = __shfl(tm.incl - tm.ntile, expert, kWave);
  const int lo = offsets[expert], hi = offsets[expert + 1];
  row0 = lo + (tile - excl) * BM;
  rows = min(BM, hi - row0);
}

// ---- stage layout and loads ----------------------------------------------------------------------
// Stage layout: rows of 32 bf16 (64 bytes, four 16-byte granules), A rows first, then B rows, no
// padding.  Granule (row, c) is stored at position c ^ ((row >> 2) & 3) of its row, so the 16 lanes
// that read one granule column of 16 consecutive rows hit 64 distinct banks.  Tiles arrive by
// global_load_lds_dwordx4: the hardware writes lane L of a wave to LDS base + 16*L, so thread t of
// load instruction i fills granule i*256 + t = (row i*64 + t/4, position t%4) and therefore FETCHES
// logical granule (t%4) ^ ((t/16) & 3) of that row.  Two stages in separate __shared__ arrays: the
// loads of step s+1 are in flight while step s is multiplied; one barrier per step.
typedef __attribute__((address_space(3))) void lds_void;
typedef const __attribute__((address_space(1))) void gbl_void;

__device__ __forceinline__ void dma16(const bf16_t* g, bf16_t* l) {
  __builtin_amdgcn_global_load_lds((gbl_void*)g, (lds_void*)l, 16, 0, 0);
}

// WM waves along M (each MT 32-row tiles) x 4 waves along N (each NTW 32-column tiles).
template <int MT, int NTW, int WM>
struct Stripe {
  static constexpr int kThreads = 256 * WM;
  static constexpr int BM = 32 * MT * WM;
  static constexpr int BN = 128 * NTW;
  static constexpr int A_GRAN = BM * 4;                          // 16-byte granules of an A stage
  static constexpr int A_PER = (A_GRAN + kThreads - 1) / kThreads;
  static constexpr int B_PER = BN * 4 / kThreads;
  static constexpr int kStageElems = (BM + BN) * kBK;
  static_assert(BM % 16 == 0 && (BN * 4) % kThreads == 0 && (kThreads / 16) % 4 == 0, "tile / thread mismatch");
};

// Everything one thread needs to issue the load instructions of a stage.
template <typename S>
struct StripeLoader {
  const bf16_t* a_src[S::A_PER];   // row base + 8 * (swizzled granule) of the A rows this thread fetches
  const bf16_t* b_src;             // same for its first B row; later instructions step by `bstep` elements
  size_t bstep;

  static constexpr int kInstr = S::A_PER + S::B_PER;

  // load instruction `q` (0 .. kInstr-1) of the stage that starts at K offset k0
  template <int Q>
  __device__ __forceinline__ void issue(int k0, bf16_t* stage) const {
    if constexpr (Q < kInstr) {
      const int wave = threadIdx.x >> 6;
      if constexpr (Q < S::A_PER) {
        if (S::A_GRAN % S::kThreads == 0 || (Q * S::kThreads + wave * 64) < S::A_GRAN)      // wave-uniform
          dma16(a_src[Q] + k0, stage + (Q * S::kThreads + wave * 64) * 8);
      } else {
        constexpr int i = Q - S::A_PER;
        dma16(b_src + i * bstep + k0, stage + S::BM * kBK + (i * S::kThreads + wave * 64) * 8);
      }
    }
  }
  template <int... Qs>
  __device__ __forceinline__ void issue_all(int k0, bf16_t* stage, std::integer_sequence<int, Qs...>) const {
    (issue<Qs>(k0, stage), ...);
  }
  __device__ __forceinline__ void issue_stage(int k0, bf16_t* stage) const {
    issue_all(k0, stage, std::make_integer_sequence<int, kInstr>{});
  }
};

// One (k16 sub-step, N tile) pair of the software pipeline below; Q is a compile-time index so the
// scheduling hints get constant arguments.  Pair Q also issues load instruction Q of the NEXT stage
// (if there is one): spreading the loads through the MFMAs keeps the waves from queueing up at the
// texture-address unit before they start multiplying.
template <int Q, int MT, int NTW, typename S, typename FragRow>
__device__ __forceinline__ void stripe_pair(floatx16 (&acc)[MT][NTW], bf16x8 (&a)[2][MT], bf16x8 (&b)[3],
                                            const bf16_t* astage, const bf16_t* bstage, int pos0, FragRow frag_row,
                                            const StripeLoader<S>& ld, bool prefetch, int k_next, bf16_t* next_stage) {
  constexpr int kPairs = 2 * NTW;
  constexpr int s = Q / NTW, j = Q % NTW;
  // kLoadsPerPair load instructions of the next stage per pair, starting with pair 0
  constexpr int kPer = kLoadsPerPair;
  if (prefetch) {
    if constexpr (Q * kPer < StripeLoader<S>::kInstr) ld.template issue<Q * kPer>(k_next, next_stage);
    if constexpr (kPer > 1 && Q * kPer + 1 < StripeLoader<S>::kInstr) ld.template issue<Q * kPer + 1>(k_next, next_stage);
  }
  if constexpr (Q + 2 < kPairs) {
    constexpr int s2 = (Q + 2) / NTW, j2 = (Q + 2) % NTW;
    b[(Q + 2) % 3] = *reinterpret_cast<const bf16x8*>(bstage + frag_row(j2) * kBK + (pos0 ^ (s2 * 16)));
  }
  if constexpr (Q < MT) a[1][Q] = *reinterpret_cast<const bf16x8*>(astage + Q * 32 * kBK + (pos0 ^ 16));
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
    acc[mt][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[s][mt], b[Q % 3], acc[mt][j], 0, 0, 0);
  constexpr int kReads = (Q + 2 < kPairs ? 1 : 0) + (Q < MT ? 1 : 0);
  if constexpr (kReads > 0) __builtin_amdgcn_sched_group_barrier(0x100, kReads, 0);
  __builtin_amdgcn_sched_group_barrier(0x008, MT, 0);
}

template <int MT, int NTW, typename S, typename FragRow, int... Qs>
__device__ __forceinline__ void stripe_pairs(floatx16 (&acc)[MT][NTW], bf16x8 (&a)[2][MT], bf16x8 (&b)[3],
                                             const bf16_t* astage, const bf16_t* bstage, int pos0, FragRow frag_row,
                                             const StripeLoader<S>& ld, bool prefetch, int k_next, bf16_t* next_stage,
                                             std::integer_sequence<int, Qs...>) {
  (stripe_pair<Qs, MT, NTW, S>(acc, a, b, astage, bstage, pos0, frag_row, ld, prefetch, k_next, next_stage), ...);
}

// Multiply one LDS stage into the accumulators while the load instructions of the next stage are
// issued.  Software pipeline over the 2*NTW (k16 sub-step, N tile) pairs: B fragments rotate through
// three buffers and are read two pairs ahead of the MFMAs that consume them; the A fragments of the
// second sub-step are read while the first sub-step is still multiplying.
template <int MT, int NTW, int WM, typename FragRow>
__device__ __forceinline__ void stripe_compute(floatx16 (&acc)[MT][NTW], const bf16_t* stage, int wm, FragRow frag_row,
                                               const StripeLoader<Stripe<MT, NTW, WM>>& ld, bool prefetch, int k_next,
                                               bf16_t* next_stage) {
  using S = Stripe<MT, NTW, WM>;
  static_assert(StripeLoader<S>::kInstr <= 2 * (2 * NTW), "at most two load instructions per pair");
  const int lane = threadIdx.x & 63;
  const int n = lane & 31, h = lane >> 5;
  const int pos0 = (h ^ ((n >> 2) & 3)) * 8;      // element offset of logical granule h; granule 2+h is pos0 ^ 16
  const bf16_t* astage = stage + (wm * MT * 32 + n) * kBK;
  const bf16_t* bstage = stage + (S::BM + n) * kBK;
  bf16x8 a[2][MT], b[3];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) a[0][mt] = *reinterpret_cast<const bf16x8*>(astage + mt * 32 * kBK + pos0);
  b[0] = *reinterpret_cast<const bf16x8*>(bstage + frag_row(0) * kBK + pos0);
  b[1] = *reinterpret_cast<const bf16x8*>(bstage + frag_row(NTW > 1 ? 1 : 0) * kBK + (NTW > 1 ? pos0 : (pos0 ^ 16)));
  __builtin_amdgcn_sched_group_barrier(0x100, MT + 2, 0);
  stripe_pairs<MT, NTW, S>(acc, a, b, astage, bstage, pos0, frag_row, ld, prefetch, k_next, next_stage,
                           std::make_integer_sequence<int, 2 * NTW>{});
}

__device__ __forceinline__ void wait_loads_and_sync() {
  __builtin_amdgcn_s_waitcnt(0);   // vmcnt(0): this thread's LDS-DMA transfers have landed
  __syncthreads();
}

template <int MT, int NTW, int WM, typename FragRow>
__device__ __forceinline__ void stripe_mainloop_dma(floatx16 (&acc)[MT][NTW],
                                                    const StripeLoader<Stripe<MT, NTW, WM>>& ld, int K, bf16_t* st0,
                                                    bf16_t* st1, int wm, FragRow frag_row) {
  ld.issue_stage(0, st0);
  for (int k0 = 0; k0 < K; k0 += 2 * kBK) {
    wait_loads_and_sync();
    stripe_compute<MT, NTW, WM>(acc, st0, wm, frag_row, ld, k0 + kBK < K, k0 + kBK, st1);
    if (k0 + kBK < K) {
      wait_loads_and_sync();
      stripe_compute<MT, NTW, WM>(acc, st1, wm, frag_row, ld, k0 + 2 * kBK < K, k0 + 2 * kBK, st0);
    }
  }
}

// logical granule fetched by thread t (see the layout note above)
__device__ __forceinline__ int dma_chunk(int t) { return (t & 3) ^ ((t >> 4) & 3); }

// Accumulator layout of one 32x32 tile: lane holds column lane%32; register i is row
// 8*(i/4) + 4*(lane/32) + i%4.
__device__ __forceinline__ int acc_row(int i, int lane) { return 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3); }

// ---- kernel 3 ------------------------------------------------------------------------------------
template <int MT, int NT, int WM>
__global__ __launch_bounds__(256 * WM) void gateup_dma_kernel(const bf16_t* __restrict__ x,
                                                              const bf16_t* __restrict__ wgu,
                                                              const float* __restrict__ theta,
                                                              const int32_t* __restrict__ offsets,
                                                              const int32_t* __restrict__ perm_token, int H, int E,
                                                              bf16_t* __restrict__ hidden) {
  constexpr int NTW = 2 * NT;
  using S = Stripe<MT, NTW, WM>;
  constexpr int BM = S::BM;
  constexpr int I = 128 * NT;
  __shared__ __attribute__((aligned(16))) bf16_t st0[S::kStageElems];
  __shared__ __attribute__((aligned(16))) bf16_t st1[S::kStageElems];
  __shared__ float ssq[4 * BM];
  __shared__ float rinv_s[BM], gain_s[BM];

  const TileMap tm = make_tile_map(offsets, E, BM);
  const int tile = xcd_tile(blockIdx.x, tm.total);
  if (tile >= tm.total) return;
  int e, row0, rows;
  find_tile(tm, offsets, BM, tile, e, row0, rows);

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int wn = wave & 3, wm = wave >> 2;
  const int chunk = dma_chunk(tid);
  StripeLoader<S> ld;
#pragma unroll
  for (int i = 0; i < S::A_PER; ++i) {
    const int m = min((tid >> 2) + i * (S::kThreads / 4), rows - 1);     // rows past the end re-read the last valid row
    ld.a_src[i] = x + (size_t)perm_token[row0 + m] * H + chunk * 8;     // gather, moe.py:81
  }
  ld.b_src = wgu + ((size_t)e * 2 * I + (tid >> 2)) * H + chunk * 8;
  ld.bstep = (size_t)(S::kThreads / 4) * H;
  floatx16 acc[MT][NTW];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int j = 0; j < NTW; ++j)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mt][j][i] = 0.f;
  auto frag_row = [&](int j) { return (j < NT ? 0 : I) + (wn * NT + (j < NT ? j : j - NT)) * 32; };
  stripe_mainloop_dma<MT, NTW, WM>(acc, ld, H, st0, st1, wm, frag_row);

  // ---- Radial NormSiLU epilogue (moe.py:87-92) ----
  // (1) sum of gate^2 per row: registers -> 32-lane shuffle -> LDS across the four N waves;
  // (2) one thread per row turns it into 1/r and r^p; (3) every lane applies SiLU(g/r) * r^p * up and
  // parks its bf16 results in a wave-private LDS tile; (4) the tile leaves as 16-byte row segments.
  const int mbase = wm * MT * 32;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      float sq = 0.f;
#pragma unroll
      for (int j = 0; j < NT; ++j) sq = fmaf(acc[mt][j][i], acc[mt][j][i], sq);
#pragma unroll
      for (int o = 16; o > 0; o >>= 1) sq += __shfl_xor(sq, o, kWave);
      if ((lane & 31) == 0) ssq[wn * BM + mbase + mt * 32 + acc_row(i, lane)] = sq;
    }
  __syncthreads();                       // also: every wave is done reading the stage buffers
  if (tid < BM) {
    const float p = 1.f / (1.f + __expf(-theta[e]));                                  // moe.py:89
    const float ms = ((ssq[tid] + ssq[BM + tid]) + ssq[2 * BM + tid]) + ssq[3 * BM + tid];
    const float r2 = ms * (1.f / (float)I) + kNormSiluEps;                            // r^2, moe.py:88
    rinv_s[tid] = __builtin_amdgcn_rsqf(r2);
    gain_s[tid] = __builtin_amdgcn_exp2f(0.5f * p * __builtin_amdgcn_logf(r2));       // r^p = 2^(p/2 * log2 r^2)
  }
  __syncthreads();
  constexpr int kOutCols = NT * 32;                 // gate-paired columns owned by this wave
  constexpr int kOutStride = kOutCols + 8;          // bf16 elements; +16 bytes keeps the two lane halves apart
  bf16_t* otile = (wave < 4 * WM / 2 ? st0 : st1) + (wave % (4 * WM / 2)) * (MT * 32 * kOutStride);
  static_assert((4 * WM / 2) * MT * 32 * kOutStride <= S::kStageElems, "output staging does not fit a stage buffer");
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int ml = mt * 32 + acc_row(i, lane);
      const float rinv = rinv_s[mbase + ml], gain = gain_s[mbase + ml];
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        const float z = acc[mt][j][i] * rinv;
        const float sg = __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-1.44269504f * z));
        otile[ml * kOutStride + j * 32 + (lane & 31)] = (bf16_t)(z * sg * gain * acc[mt][NT + j][i]);   // SiLU(g/r) r^p up
      }
    }
  __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0): this wave's LDS writes are done (the tile is wave-private)
  __builtin_amdgcn_wave_barrier();
  constexpr int kGranPerRow = kOutCols / 8;
  const int colbase = wn * kOutCols;
  for (int g = lane; g < MT * 32 * kGranPerRow; g += kWave) {
    const int ml = g / kGranPerRow, c = g - ml * kGranPerRow;
    if (mbase + ml < rows)
      *reinterpret_cast<u32x4*>(hidden + (size_t)(row0 + mbase + ml) * I + colbase + c * 8) =
          *reinterpret_cast<const u32x4*>(otile + ml * kOutStride + c * 8);
  }
}

// ---- kernel 4 ------------------------------------------------------------------------------------
template <int MT, int NTW, int WM, typename TY>
__global__ __launch_bounds__(256 * WM) void down_dma_kernel(const bf16_t* __restrict__ hidden,
                                                            const bf16_t* __restrict__ wd, const float* __restrict__ w,
                                                            const int32_t* __restrict__ offsets,
                                                            const int32_t* __restrict__ perm_slot, int H, int E, int I,
                                                            int nblk_n, TY* __restrict__ yw) {
  using S = Stripe<MT, NTW, WM>;
  constexpr int BM = S::BM;
  constexpr int BN = S::BN;
  __shared__ __attribute__((aligned(16))) bf16_t st0[S::kStageElems];
  __shared__ __attribute__((aligned(16))) bf16_t st1[S::kStageElems];
  __shared__ int slot_s[BM];
  __shared__ float w_s[BM];

  const TileMap tm = make_tile_map(offsets, E, BM);
  const int total = tm.total * nblk_n;
  const int flat = xcd_tile(blockIdx.x, total);
  if (flat >= total) return;
  const int tile = flat / nblk_n, nb = flat - tile * nblk_n;
  int e, row0, rows;
  find_tile(tm, offsets, BM, tile, e, row0, rows);

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int wn = wave & 3, wm = wave >> 2;
  if (tid < BM) {
    const int slot = perm_slot[row0 + min(tid, rows - 1)];
    slot_s[tid] = slot;
    w_s[tid] = w[slot];
  }
  const int chunk = dma_chunk(tid);
  StripeLoader<S> ld;
#pragma unroll
  for (int i = 0; i < S::A_PER; ++i) {
    const int m = min((tid >> 2) + i * (S::kThreads / 4), rows - 1);
    ld.a_src[i] = hidden + (size_t)(row0 + m) * I + chunk * 8;
  }
  const int n0 = nb * BN;
  ld.b_src = wd + ((size_t)e * H + n0 + (tid >> 2)) * I + chunk * 8;
  ld.bstep = (size_t)(S::kThreads / 4) * I;
  floatx16 acc[MT][NTW];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int j = 0; j < NTW; ++j)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mt][j][i] = 0.f;
  auto frag_row = [&](int j) { return (wn * NTW + j) * 32; };
  stripe_mainloop_dma<MT, NTW, WM>(acc, ld, I, st0, st1, wm, frag_row);

  // Epilogue: scale by the routing weight (moe.py:93), park kPassRows rows at a time in a wave-private
  // LDS tile and scatter them to slot order as 16-byte row segments.
  const int mbase = wm * MT * 32;
  constexpr int kOutCols = NTW * 32;
  constexpr int kEltPer16 = 16 / sizeof(TY);
  constexpr int kOutStride = kOutCols + kEltPer16;  // +16 bytes keeps the two lane halves on different banks
  constexpr int kPassRows = sizeof(TY) == 2 ? 32 : 16;   // accumulator registers 8p .. 8p+7 hold rows 16p .. 16p+15
  constexpr int kPasses = 32 / kPassRows;
  static_assert((size_t)(4 * WM / 2) * kPassRows * kOutStride * sizeof(TY) <= (size_t)S::kStageElems * sizeof(bf16_t),
                "output staging does not fit a stage buffer");
  __syncthreads();                       // every wave is done reading the stage buffers
  TY* otile = reinterpret_cast<TY*>(wave < 4 * WM / 2 ? st0 : st1) + (wave % (4 * WM / 2)) * (kPassRows * kOutStride);
  constexpr int kGranPerRow = kOutCols / kEltPer16;
  const int colbase = n0 + wn * kOutCols;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int ps = 0; ps < kPasses; ++ps) {
#pragma unroll
      for (int ii = 0; ii < 16 / kPasses; ++ii) {
        const int i = ps * (16 / kPasses) + ii;
        const int ml = acc_row(i, lane) - ps * kPassRows;
        const float ws = w_s[mbase + mt * 32 + acc_row(i, lane)];
#pragma unroll
        for (int j = 0; j < NTW; ++j)
          otile[ml * kOutStride + j * 32 + (lane & 31)] = from_float<TY>(ws * acc[mt][j][i]);
      }
      __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
      __builtin_amdgcn_wave_barrier();
      for (int g = lane; g < kPassRows * kGranPerRow; g += kWave) {
        const int ml = g / kGranPerRow, c = g - ml * kGranPerRow;
        const int m = mbase + mt * 32 + ps * kPassRows + ml;
        if (m < rows)
          *reinterpret_cast<u32x4*>(yw + (size_t)slot_s[m] * H + colbase + c * kEltPer16) =
              *reinterpret_cast<const u32x4*>(otile + ml * kOutStride + c * kEltPer16);
      }
      __builtin_amdgcn_s_waitcnt(0xc07f);
      __builtin_amdgcn_wave_barrier();
    }
}

inline int round_up8(int v) { return (v + 7) & ~7; }

template <int MT, int NT, int WM>
void launch_gateup_dma_t(const bf16_t* x, const bf16_t* wgu, const float* theta, const int32_t* offsets,
                         const int32_t* perm_token, int S, int H, int E, bf16_t* hidden, hipStream_t s) {
  constexpr int BM = 32 * MT * WM;
  const int grid = round_up8(S / BM + E) + 8;
  hipLaunchKernelGGL((gateup_dma_kernel<MT, NT, WM>), dim3(grid), dim3(256 * WM), 0, s, x, wgu, theta, offsets,
                     perm_token, H, E, hidden);
}

template <int MT, int NTW, int WM, typename TY>
void launch_down_dma_t(const bf16_t* hidden, const bf16_t* wd, const float* w, const int32_t* offsets,
                       const int32_t* perm_slot, int S, int H, int E, int I, TY* yw, hipStream_t s) {
  constexpr int BM = 32 * MT * WM;
  const int nblk_n = H / (128 * NTW);
  const int grid = round_up8((S / BM + E) * nblk_n) + 8;
  hipLaunchKernelGGL((down_dma_kernel<MT, NTW, WM, TY>), dim3(grid), dim3(256 * WM), 0, s, hidden, wd, w, offsets,
                     perm_slot, H, E, I, nblk_n, yw);
}

template <typename TY>
void launch_down_dma_ty(const bf16_t* hidden, const bf16_t* wd, const float* w, const int32_t* offsets,
                        const int32_t* perm_slot, int S, int H, int E, int I, TY* yw, hipStream_t s) {
  if (H % 768 == 0) launch_down_dma_t<2, 6, 2, TY>(hidden, wd, w, offsets, perm_slot, S, H, E, I, yw, s);
  else if (H % 512 == 0) launch_down_dma_t<2, 4, 2, TY>(hidden, wd, w, offsets, perm_slot, S, H, E, I, yw, s);
  else if (H % 384 == 0) launch_down_dma_t<2, 3, 2, TY>(hidden, wd, w, offsets, perm_slot, S, H, E, I, yw, s);
  else if (H % 256 == 0) launch_down_dma_t<2, 2, 2, TY>(hidden, wd, w, offsets, perm_slot, S, H, E, I, yw, s);
  else launch_down_dma_t<2, 1, 2, TY>(hidden, wd, w, offsets, perm_slot, S, H, E, I, yw, s);
}

}  // namespace

bool mfma_supported(int H, int I, int dtype) {
  return dtype == BIBO_DTYPE_BF16 && H >= 128 && (H % 128) == 0 && (I == 128 || I == 256 || I == 384 || I == 512);
}

hipError_t launch_gateup_mfma(const void* x, const void* wgu, const float* theta, const int32_t* offsets,
                              const int32_t* perm_token, int T, int H, int E, int k, int I, void* hidden,
                              hipStream_t s) {
  const int S = T * k;
  if (S == 0) return hipSuccess;
  const bf16_t* xp = static_cast<const bf16_t*>(x);
  const bf16_t* wp = static_cast<const bf16_t*>(wgu);
  bf16_t* hp = static_cast<bf16_t*>(hidden);
  switch (I) {
    case 128: launch_gateup_dma_t<2, 1, 2>(xp, wp, theta, offsets, perm_token, S, H, E, hp, s); break;
    case 256: launch_gateup_dma_t<2, 2, 2>(xp, wp, theta, offsets, perm_token, S, H, E, hp, s); break;
    case 384: launch_gateup_dma_t<2, 3, 2>(xp, wp, theta, offsets, perm_token, S, H, E, hp, s); break;
    case 512: launch_gateup_dma_t<1, 4, 2>(xp, wp, theta, offsets, perm_token, S, H, E, hp, s); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

hipError_t launch_down_mfma(const void* hidden, const void* wd, const float* w, const int32_t* offsets,
                            const int32_t* perm_slot, int T, int H, int E, int k, int I, void* yw, hipStream_t s) {
  const int S = T * k;
  if (S == 0) return hipSuccess;
  const bf16_t* hp = static_cast<const bf16_t*>(hidden);
  const bf16_t* wp = static_cast<const bf16_t*>(wd);
  launch_down_dma_ty<bf16_t>(hp, wp, w, offsets, perm_slot, S, H, E, I, static_cast<bf16_t*>(yw), s);
  return hipGetLastError();
}

}  // namespace bibo
