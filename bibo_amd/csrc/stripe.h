// Tile machinery shared by the MFMA expert kernels (gfx950): tile lookup from the per-expert offsets,
// LDS stage layout, LDS-DMA loader and the software-pipelined stage multiply.
#pragma once

#include <utility>

#include "common.h"

namespace bibo {
namespace {

constexpr int kLoadsPerPair = 1;   // load instructions of the next stage issued per (sub-step, N tile) pair
constexpr int kBK = 32;        // default K elements per LDS stage

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
// Stage layout: rows of BK bf16 (64 bytes = four 16-byte granules for BK = 32, 128 bytes = eight for
// BK = 64), A rows first, then B rows, no padding.  Granule (row, c) is stored at position
// c ^ ((row >> 2) & 3) of its row (BK = 32) or c ^ ((row >> 1) & 7) (BK = 64), so the 16 lanes that read
// one granule column of 16 consecutive rows hit 64 distinct banks.  Tiles arrive by
// global_load_lds_dwordx4: the hardware writes lane L of a wave to LDS base + 16*L, so thread t of
// load instruction i fills granule i*kThreads + t = (row i*kThreads/GPR + t/GPR, position t%GPR) and
// therefore FETCHES logical granule (t%GPR) ^ ((t/16) & (GPR-1)) of that row.  Two stages in separate
// __shared__ arrays: the loads of step s+1 are in flight while step s is multiplied; one barrier per step.
typedef __attribute__((address_space(3))) void lds_void;
typedef const __attribute__((address_space(1))) void gbl_void;

__device__ __forceinline__ void dma16(const bf16_t* g, bf16_t* l) {
  __builtin_amdgcn_global_load_lds((gbl_void*)g, (lds_void*)l, 16, 0, 0);
}

// WM waves along M (each MT 32-row tiles) x 4 waves along N (each NTW 32-column tiles).
template <int MT, int NTW, int WM, int BK_ = kBK>
struct Stripe {
  static constexpr int BK = BK_;                                 // K elements per stage: 32 (64-byte rows) or 64
  static constexpr int GPR = BK / 8;                             // 16-byte granules per row
  static constexpr int SS = BK / 16;                             // k16 sub-steps per stage
  static constexpr int kSwzShift = GPR == 4 ? 2 : 1;             // row -> swizzle term (row >> shift) & (GPR - 1)
  static constexpr int kThreads = 256 * WM;
  static constexpr int BM = 32 * MT * WM;
  static constexpr int BN = 128 * NTW;
  static constexpr int A_GRAN = BM * GPR;                        // 16-byte granules of an A stage
  static constexpr int A_PER = (A_GRAN + kThreads - 1) / kThreads;
  static constexpr int B_PER = BN * GPR / kThreads;
  static constexpr int kRowsPerInstr = kThreads / GPR;
  static constexpr int kStageElems = (BM + BN) * BK;
  static_assert(BK == 32 || BK == 64, "stage rows are 64 or 128 bytes");
  static_assert(BM % 16 == 0 && (BN * GPR) % kThreads == 0 && kRowsPerInstr % 16 == 0, "tile / thread mismatch");
  // logical granule fetched by thread t of any load instruction (see the layout note above)
  __device__ static int dma_chunk(int t) { return (t & (GPR - 1)) ^ ((t >> 4) & (GPR - 1)); }
  // row (within one instruction's rows) thread t fetches
  __device__ static int dma_row(int t) { return t / GPR; }
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
        dma16(b_src + i * bstep + k0, stage + S::BM * S::BK + (i * S::kThreads + wave * 64) * 8);
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
  // the two halves of a stage separately: the B rows need no row indices and can be requested first
  template <int... Qs>
  __device__ __forceinline__ void issue_b_all(int k0, bf16_t* stage, std::integer_sequence<int, Qs...>) const {
    (issue<S::A_PER + Qs>(k0, stage), ...);
  }
  __device__ __forceinline__ void issue_b(int k0, bf16_t* stage) const {
    issue_b_all(k0, stage, std::make_integer_sequence<int, S::B_PER>{});
  }
  __device__ __forceinline__ void issue_a(int k0, bf16_t* stage) const {
    issue_all(k0, stage, std::make_integer_sequence<int, S::A_PER>{});
  }
};

// load instructions FIRST .. FIRST+COUNT-1 of a stage (those that exist)
template <int FIRST, int COUNT, typename Loader>
__device__ __forceinline__ void issue_some(const Loader& ld, int k_next, bf16_t* next_stage) {
  if constexpr (COUNT > 0 && FIRST < Loader::kInstr) {
    ld.template issue<FIRST>(k_next, next_stage);
    issue_some<FIRST + 1, COUNT - 1>(ld, k_next, next_stage);
  }
}

// One (k16 sub-step, N tile) pair of the software pipeline below; Q is a compile-time index so the
// scheduling hints get constant arguments.  Pair Q also issues load instruction Q of the NEXT stage
// (if there is one): spreading the loads through the MFMAs keeps the waves from queueing up at the
// texture-address unit before they start multiplying.  `a1` points at this lane's A fragment of the
// second sub-step for M tile 0; tile mt is `astride` elements further.
template <int Q, int MT, int NTW, int BK, bool TR, int NACC, int J0, int JS, typename Loader, typename FragRow, int AMT>
__device__ __forceinline__ void stripe_pair(floatx16 (&acc)[AMT][NACC], bf16x8 (&a)[2][MT], bf16x8 (&b)[3],
                                            const bf16_t* a0, int astride, const bf16_t* bstage, int pos0,
                                            FragRow frag_row, const Loader& ld, bool prefetch, int k_next,
                                            bf16_t* next_stage) {
  constexpr int SS = BK / 16;
  constexpr int kPairs = SS * NTW;
  constexpr int s = Q / NTW, j = Q % NTW;
  // kLoadsPerPair load instructions of the next stage per pair, starting with pair 0
  constexpr int kPer = (Loader::kInstr + kPairs - 1) / kPairs > kLoadsPerPair ? (Loader::kInstr + kPairs - 1) / kPairs
                                                                              : kLoadsPerPair;
  if (prefetch) issue_some<Q * kPer, kPer>(ld, k_next, next_stage);
  if constexpr (Q + 2 < kPairs) {
    constexpr int s2 = (Q + 2) / NTW, j2 = (Q + 2) % NTW;
    b[(Q + 2) % 3] = *reinterpret_cast<const bf16x8*>(bstage + frag_row(j2) * BK + (pos0 ^ (s2 * 16)));
  }
  // A fragments of the next sub-step are read during the pairs of this one: pair j reads M tile j, the
  // last pair whatever is left
  constexpr int kAFirst = j, kALast = (s + 1 < SS) ? ((j == NTW - 1) ? MT - 1 : (j < MT ? j : -1)) : -1;
#pragma unroll
  for (int mt = kAFirst; mt <= kALast; ++mt)
    a[(s + 1) & 1][mt] = *reinterpret_cast<const bf16x8*>(a0 + mt * astride + ((pos0 ^ ((s + 1) * 16)) - pos0));
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
    acc[mt][J0 + j * JS] = TR ? __builtin_amdgcn_mfma_f32_32x32x16_bf16(b[Q % 3], a[s & 1][mt], acc[mt][J0 + j * JS], 0, 0, 0)
                              : __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[s & 1][mt], b[Q % 3], acc[mt][J0 + j * JS], 0, 0, 0);
  constexpr int kReads = (Q + 2 < kPairs ? 1 : 0) + (kALast >= kAFirst ? kALast - kAFirst + 1 : 0);
  if constexpr (kReads > 0) __builtin_amdgcn_sched_group_barrier(0x100, kReads, 0);
  __builtin_amdgcn_sched_group_barrier(0x008, MT, 0);
}

template <int MT, int NTW, int BK, bool TR, int NACC, int J0, int JS, typename Loader, typename FragRow, int AMT, int... Qs>
__device__ __forceinline__ void stripe_pairs(floatx16 (&acc)[AMT][NACC], bf16x8 (&a)[2][MT], bf16x8 (&b)[3],
                                             const bf16_t* a0, int astride, const bf16_t* bstage, int pos0,
                                             FragRow frag_row, const Loader& ld, bool prefetch, int k_next,
                                             bf16_t* next_stage, std::integer_sequence<int, Qs...>) {
  (stripe_pair<Qs, MT, NTW, BK, TR, NACC, J0, JS>(acc, a, b, a0, astride, bstage, pos0, frag_row, ld, prefetch, k_next, next_stage), ...);
}

// Multiply one K step of BK into the accumulators while the load instructions of the next stage are
// issued.  Software pipeline over the (BK/16)*NTW (k16 sub-step, N tile) pairs: B fragments rotate
// through three buffers and are read two pairs ahead of the MFMAs that consume them; the A fragments
// of the next sub-step are read while the current one is still multiplying.  a0: this lane's A
// fragment of sub-step 0 for M tile 0 (position pos0 of its row; sub-step s sits at pos0 ^ 16s, M tile
// mt `astride` elements further); bstage: this lane's row of the B stage (N tile 0).  The NTW tiles multiplied
// here are columns J0, J0+JS, .. of an accumulator array NACC tiles wide.
// The accumulator array may have more M tiles (AMT) than the MT that are multiplied: the first MT are.
template <int MT, int NTW, int BK, bool TR, int NACC = NTW, int J0 = 0, int JS = 1, typename Loader, typename FragRow, int AMT>
__device__ __forceinline__ void stripe_step(floatx16 (&acc)[AMT][NACC], const bf16_t* a0, int astride, const bf16_t* bstage,
                                            int pos0, FragRow frag_row, const Loader& ld, bool prefetch, int k_next,
                                            bf16_t* next_stage) {
  constexpr int SS = BK / 16;
  bf16x8 a[2][MT], b[3];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) a[0][mt] = *reinterpret_cast<const bf16x8*>(a0 + mt * astride);
  b[0] = *reinterpret_cast<const bf16x8*>(bstage + frag_row(0) * BK + pos0);
  b[1] = *reinterpret_cast<const bf16x8*>(bstage + frag_row(NTW > 1 ? 1 : 0) * BK + (NTW > 1 ? pos0 : (pos0 ^ 16)));
  __builtin_amdgcn_sched_group_barrier(0x100, MT + 2, 0);
  stripe_pairs<MT, NTW, BK, TR, NACC, J0, JS>(acc, a, b, a0, astride, bstage, pos0, frag_row, ld, prefetch, k_next, next_stage,
                                          std::make_integer_sequence<int, SS * NTW>{});
}

// A and B both come from `stage` (A rows first).
template <int MT, int NTW, int WM, int BK, bool TR, typename FragRow>
__device__ __forceinline__ void stripe_compute(floatx16 (&acc)[MT][NTW], const bf16_t* stage, int wm, FragRow frag_row,
                                               const StripeLoader<Stripe<MT, NTW, WM, BK>>& ld, bool prefetch,
                                               int k_next, bf16_t* next_stage) {
  using S = Stripe<MT, NTW, WM, BK>;
  const int lane = threadIdx.x & 63;
  const int n = lane & 31, h = lane >> 5;
  // element offset of logical granule h of row n (all fragment rows are n plus a multiple of 32, which
  // leaves the swizzle term unchanged); granule 2s + h is pos0 ^ 16s
  const int pos0 = (h ^ ((n >> S::kSwzShift) & (S::GPR - 1))) * 8;
  const bf16_t* astage = stage + (wm * MT * 32 + n) * BK;
  const bf16_t* bstage = stage + (S::BM + n) * BK;
  stripe_step<MT, NTW, BK, TR>(acc, astage + pos0, 32 * BK, bstage, pos0, frag_row, ld, prefetch, k_next, next_stage);
}

__device__ __forceinline__ void wait_loads_and_sync() {
  __builtin_amdgcn_s_waitcnt(0);   // vmcnt(0): this thread's LDS-DMA transfers have landed
  __syncthreads();
}

// The caller has already requested stage 0 into st0 (issue_b, then issue_a once the row indices are known).
// TR = false: accumulator tile [mt][j] holds rows x columns in the MFMA D layout (lane = column, registers =
// rows, see acc_row).  TR = true: the operands are swapped and the tile is transposed: lane = ROW (lane % 32),
// register i = COLUMN acc_row(i, lane), so a lane owns runs of four consecutive columns of one row.
template <int MT, int NTW, int WM, int BK, bool TR, typename FragRow>
__device__ __forceinline__ void stripe_mainloop_dma(floatx16 (&acc)[MT][NTW],
                                                    const StripeLoader<Stripe<MT, NTW, WM, BK>>& ld, int K, bf16_t* st0,
                                                    bf16_t* st1, int wm, FragRow frag_row) {
  for (int k0 = 0; k0 < K; k0 += 2 * BK) {
    wait_loads_and_sync();
    stripe_compute<MT, NTW, WM, BK, TR>(acc, st0, wm, frag_row, ld, k0 + BK < K, k0 + BK, st1);
    if (k0 + BK < K) {
      wait_loads_and_sync();
      stripe_compute<MT, NTW, WM, BK, TR>(acc, st1, wm, frag_row, ld, k0 + 2 * BK < K, k0 + 2 * BK, st0);
    }
  }
}

// Accumulator layout of one 32x32 tile: lane holds column lane%32; register i is row
// 8*(i/4) + 4*(lane/32) + i%4.
__device__ __forceinline__ int acc_row(int i, int lane) { return 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3); }

}  // namespace
}  // namespace bibo
