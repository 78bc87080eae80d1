// Grouped GEMMs whose operands are contiguous ACROSS the contraction instead of along it ("K-major": element (k, n)
// at k * ld + n), for the backward pass on gfx950.  The two weight tensors are stored [E, 2I, H] and [E, H, I]; the
// forward pass contracts along their last dimension, the input gradients contract along the middle one, and the
// weight gradients contract along the ROWS of row-major activations.  Instead of transposed copies in memory, a
// K-major operand goes to LDS as it lies (LDS-DMA, 64 k rows x 128 n per sub-tile) and the MFMA fragments are read
// with ds_read_b64_tr_b16, which hands a lane four consecutive k of one n:
//   within a group of 16 lanes, lane r addresses 8 bytes (4 elements) M[r][0..3], and lane j receives
//   M[j / 4 + 4 i][j % 4] for i = 0..3.  With lane r pointing at (k0 + r / 4, n0 + 4 (r % 4)) the group covers a
//   4 (k) x 16 (n) block and lane j ends up with (k0 .. k0 + 3, n0 + j).
// Two such reads give the 8 consecutive k of an MFMA operand lane.
#pragma once

#include "stripe.h"

namespace bibo {
namespace {

typedef short v4i16 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) v4i16 lds_v4i16;

constexpr int kKS = 32;                 // k rows per LDS stage
constexpr int kRing = 4;                // stages in LDS: one being multiplied, two on their way, one being requested
constexpr int kSubW = 128;              // n elements per sub-tile row (256 bytes: whole 128-byte lines per DMA row)
constexpr int kSubElems = kKS * kSubW;  // 8 KB: one LDS-DMA instruction of the 512 threads
constexpr int kATile = 128 * kKS;       // row-major operand tile, 128 rows: 8 KB as well

// LDS layout of a K-major sub-tile [32 k][128 n]: 16-byte granule G of row k sits at position G ^ ((k & 3) << 2).
// The four k rows one transposed read touches then lie in four different 64-byte quarters of the 256-byte bank
// period, so the read has no bank conflicts.  Thread t of the fill writes row t / 16, position t % 16, and therefore
// fetches granule (t % 16) ^ (((t / 16) & 3) << 2) of that row.
__device__ __forceinline__ int kfill_granule(int tid) { return (tid & 15) ^ (((tid >> 4) & 3) << 2); }

// Fill one sub-tile: `row` = this thread's row (tid / 16) of the stage, already offset to the sub-tile's first
// column and to this thread's granule.
__device__ __forceinline__ void kfill_subtile(const bf16_t* row, bf16_t* sub) {
  dma16(row, sub + __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)) * 64 * 8);
}

// Per-lane element offset, inside a sub-tile, of the first transposed read of the 32 (n) x 16 (k) fragment whose
// first column is nbase (a multiple of 32): k16 step s and half ks add (16 s + 4 ks) * kSubW elements.
__device__ __forceinline__ int kfrag_offset(int lane, int nbase) {
  const int r = lane & 15, g16 = lane >> 4;
  const int kg = g16 >> 1, nblk = g16 & 1;
  const int krow = 8 * kg + (r >> 2);
  const int n = nbase + 16 * nblk + 4 * (r & 3);
  const int pos = (n >> 3) ^ ((r >> 2) << 2);                  // (k & 3) == r / 4 for every read of the fragment
  return krow * kSubW + pos * 8 + (n & 4);
}

// The fragment of k16 step S: lane (n = lane % 32, kg = lane / 32) gets k = 16 S + 8 kg .. + 8 of column nbase + n.
template <int S>
__device__ __forceinline__ bf16x8 kfrag_read(const bf16_t* sub, int off) {
  const v4i16 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16*)(sub + off + (16 * S) * kSubW));
  const v4i16 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16*)(sub + off + (16 * S + 4) * kSubW));
  typedef short v8i16 __attribute__((ext_vector_type(8)));
  const v8i16 v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  return __builtin_bit_cast(bf16x8, v);
}

// the same with the step as a loop variable of an unrolled loop (folds to one of the two)
__device__ __forceinline__ bf16x8 kfrag_read_s(const bf16_t* sub, int off, int s) {
  return s == 0 ? kfrag_read<0>(sub, off) : kfrag_read<1>(sub, off);
}

// One K stage (two k16 steps) of a wave's MT x NTW tiles as a software pipeline: the fragments of the second step
// are read while the first is multiplied, two LDS reads behind every MFMA.  read_a(s, mt) / read_b(s, j) return the
// fragments.
template <int MT, int NTW, typename ReadA, typename ReadB>
__device__ __forceinline__ void multiply_stage(floatx16 (&acc)[MT][NTW], ReadA read_a, ReadB read_b) {
  constexpr int kSteps = kKS / 16;
  bf16x8 af[2][MT], bfr[2][NTW];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) af[0][mt] = read_a(0, mt);
#pragma unroll
  for (int j = 0; j < NTW; ++j) bfr[0][j] = read_b(0, j);
#pragma unroll
  for (int s = 0; s < kSteps; ++s) {
    if (s + 1 < kSteps) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) af[(s + 1) & 1][mt] = read_a(s + 1, mt);
#pragma unroll
      for (int j = 0; j < NTW; ++j) bfr[(s + 1) & 1][j] = read_b(s + 1, j);
    }
#pragma unroll
    for (int j = 0; j < NTW; ++j)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        acc[mt][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[s & 1][j], af[s & 1][mt], acc[mt][j], 0, 0, 0);
    // order for the scheduler: an MFMA, then the next two LDS reads, and so on
#pragma unroll
    for (int i = 0; i < MT * NTW; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      if (s + 1 < kSteps) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
  }
}

// The same for a tall tile (MT = 4 row tiles per wave): 192 accumulator registers leave no room for two sets of every
// fragment, so the row operand is read one fragment ahead and only the column operand is held for a whole k16 step;
// the column fragments of the next step are read during the first NTW pairs of this one.  kARd = LDS reads per row
// fragment (1: a 16-byte read, 2: a pair of transposing reads).
template <int MT, int NTW, int kARd, typename ReadA, typename ReadB>
__device__ __forceinline__ void multiply_stage_tall(floatx16 (&acc)[MT][NTW], ReadA read_a, ReadB read_b) {
  constexpr int kSteps = kKS / 16, kPairs = kSteps * MT;
  static_assert(MT >= NTW, "a step's pairs carry the next step's column fragments");
  bf16x8 af[2], bfr[2][NTW];
#pragma unroll
  for (int j = 0; j < NTW; ++j) bfr[0][j] = read_b(0, j);
  af[0] = read_a(0, 0);
#pragma unroll
  for (int p = 0; p < kPairs; ++p) {
    const int s = p / MT, mt = p % MT;
    const bool more_a = p + 1 < kPairs, more_b = s + 1 < kSteps && mt < NTW;
    if (more_a) af[(p + 1) & 1] = read_a((p + 1) / MT, (p + 1) % MT);
    if (more_b) bfr[(s + 1) & 1][mt] = read_b(s + 1, mt);
#pragma unroll
    for (int j = 0; j < NTW; ++j)
      acc[mt][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[s & 1][j], af[p & 1], acc[mt][j], 0, 0, 0);
    if (more_a) __builtin_amdgcn_sched_group_barrier(0x100, kARd, 0);
    if (more_b) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    __builtin_amdgcn_sched_group_barrier(0x008, NTW, 0);
  }
}

// Row-major operand tile [128 rows][32 k] in the stripe layout for 64-byte rows (granule c of row r at
// c ^ ((r >> 2) & 3)): thread t of the fill writes row t / 4, position t % 4.  `row` = that row's K extent, already
// offset to the stage's first k and to this thread's granule (afill_granule).
__device__ __forceinline__ int afill_granule(int tid) { return (tid & 3) ^ ((tid >> 4) & 3); }
__device__ __forceinline__ void afill(const bf16_t* row, bf16_t* tile) {
  dma16(row, tile + __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)) * 64 * 8);
}

// The stages form a ring of four, each a __shared__ variable of its own (the compiler orders an LDS-DMA transfer
// against later reads of the same variable with a full wait).  Step i of the K loop waits until the transfers of
// stage i have landed (those of stages i + 1 and i + 2 may stay in flight: loads complete in order), meets the other
// waves, requests stage i + 3 into the buffer stage i - 1 was read from, and multiplies stage i.  Every step issues
// the same number of transfers (a request past the last stage repeats the last one), so the wait count is a constant.

// ---- input gradients: out[dst(r), n] = sum_k A[src(r), k] W[e][k, n] for the rows r of expert e ----------------
// A row-major (K contiguous), W K-major as stored: [K, N] per expert.  src(r) = a_index[r] (GATHER) or r; dst(r) =
// out_index[r] (SCATTER) or r.  Workgroup = 64 MT rows x 128 NTW columns, 2 x 4 waves, 32x32x16 MFMA, operands swapped
// so that a lane owns one output row.  K is a multiple of 128.  MT = 2: 128-row tiles, ring of four stages.  MT = 4:
// 256-row tiles for experts with many rows - an expert's weights then pass through LDS once per 256 rows instead of
// once per 128, which is what these kernels are bound by; 192 accumulator registers and 40 KB stages, ring of three.
template <int MT, int NTW, bool GATHER, bool SCATTER>
__global__ __launch_bounds__(512) void dgrad_kmajor_kernel(const bf16_t* __restrict__ A, const int32_t* __restrict__ a_index,
                                                           const bf16_t* __restrict__ W,
                                                           const int32_t* __restrict__ offsets,
                                                           const int32_t* __restrict__ out_index, int K, int N, int E,
                                                           int nblk_n, bf16_t* __restrict__ out) {
  static_assert(MT == 2 || MT == 4, "128- or 256-row tiles");
  constexpr int BM = 64 * MT, BN = kSubW * NTW;
  constexpr int R = MT == 4 ? 3 : kRing;                 // stages that fit LDS
  constexpr int kAOps = MT / 2;                          // 128-row blocks of the row operand
  constexpr int kOps = kAOps + NTW;                      // transfers per thread and stage
  __shared__ __attribute__((aligned(16))) bf16_t a0[kAOps * kATile];
  __shared__ __attribute__((aligned(16))) bf16_t a1[kAOps * kATile];
  __shared__ __attribute__((aligned(16))) bf16_t a2[kAOps * kATile];
  __shared__ __attribute__((aligned(16))) bf16_t a3[R == 4 ? kAOps * kATile : 8];
  __shared__ __attribute__((aligned(16))) bf16_t b0[NTW * kSubElems];
  __shared__ __attribute__((aligned(16))) bf16_t b1[NTW * kSubElems];
  __shared__ __attribute__((aligned(16))) bf16_t b2[NTW * kSubElems];
  __shared__ __attribute__((aligned(16))) bf16_t b3[R == 4 ? NTW * kSubElems : 8];
  __shared__ int dst_s[BM];

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
    const int r = row0 + min(tid, rows - 1);
    dst_s[tid] = SCATTER ? out_index[r] : r;
  }
  // fill side
  const bf16_t* arow[kAOps];
#pragma unroll
  for (int hb = 0; hb < kAOps; ++hb) {
    const int ar = row0 + min(hb * 128 + (tid >> 2), rows - 1);    // rows past the end re-read the last one
    arow[hb] = A + (size_t)(GATHER ? a_index[ar] : ar) * K + afill_granule(tid) * 8;
  }
  const int n0 = nb * BN;
  const bf16_t* wrow = W + (size_t)e * K * N + (size_t)(tid >> 4) * N + n0 + kfill_granule(tid) * 8;
  const int nstages = K / kKS;
  auto abuf = [&](auto bc) -> bf16_t* {
    constexpr int b = decltype(bc)::value;
    if constexpr (b == 0) return a0; else if constexpr (b == 1) return a1; else if constexpr (b == 2) return a2; else return a3;
  };
  auto bbuf = [&](auto bc) -> bf16_t* {
    constexpr int b = decltype(bc)::value;
    if constexpr (b == 0) return b0; else if constexpr (b == 1) return b1; else if constexpr (b == 2) return b2; else return b3;
  };
  auto fill = [&](auto bc, int stage) {
    const int k0 = min(stage, nstages - 1) * kKS;
#pragma unroll
    for (int hb = 0; hb < kAOps; ++hb) afill(arow[hb] + k0, abuf(bc) + hb * kATile);
    const bf16_t* w0 = wrow + (size_t)k0 * N;
#pragma unroll
    for (int j = 0; j < NTW; ++j) kfill_subtile(w0 + j * kSubW, bbuf(bc) + j * kSubElems);
  };
  using std::integral_constant;
  fill(integral_constant<int, 0>{}, 0);
  fill(integral_constant<int, 1>{}, 1);
  if constexpr (R == 4) fill(integral_constant<int, 2>{}, 2);

  floatx16 acc[MT][NTW];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int j = 0; j < NTW; ++j)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mt][j][i] = 0.f;

  // fragment side.  A: lane (n, h) reads logical granule 2 s + h of row mbase + 32 mt + n.  W: wave wn's tile j is
  // columns (wn NTW + j) 32 of the block = sub-tile (wn NTW + j) / 4, column ((wn NTW + j) % 4) 32 inside it.
  const int n = lane & 31, h = lane >> 5;
  const int mbase = wm * MT * 32;
  const int apos0 = (h ^ ((n >> 2) & 3)) * 8;
  const int aoff = (mbase + n) * kKS;
  int boff[NTW];
#pragma unroll
  for (int j = 0; j < NTW; ++j) {
    const int t32 = wn * NTW + j;
    boff[j] = (t32 >> 2) * kSubElems + kfrag_offset(lane, (t32 & 3) * 32);
  }
  // step `stage` reads buffer stage % R and requests stage + R - 1 into the buffer stage - 1 was read from
  auto step = [&](auto bc, int stage) {
    constexpr int b = decltype(bc)::value;
    sync_keep_loads<(R - 2) * kOps>();
    fill(integral_constant<int, (b + R - 1) % R>{}, stage + R - 1);
    const bf16_t* at = abuf(bc);
    const bf16_t* bt = bbuf(bc);
    auto read_a = [&](int s, int mt) { return *reinterpret_cast<const bf16x8*>(at + aoff + mt * 32 * kKS + (apos0 ^ (s * 16))); };
    auto read_b = [&](int s, int j) { return kfrag_read_s(bt, boff[j], s); };
    if constexpr (MT == 2) multiply_stage<MT, NTW>(acc, read_a, read_b);      // nstages is a multiple of 4
    else if (stage < nstages) multiply_stage_tall<MT, NTW, 1>(acc, read_a, read_b);
  };
  for (int i = 0; i < nstages; i += R) {
    step(integral_constant<int, 0>{}, i);
    step(integral_constant<int, 1>{}, i + 1);
    step(integral_constant<int, 2>{}, i + 2);
    if constexpr (R == 4) step(integral_constant<int, 3>{}, i + 3);
  }
  wait_loads_and_sync();                 // the repeated requests of the last steps have landed; every wave is done reading

  // Epilogue (accumulators transposed: lane = row, four consecutive columns per register quad): 32 rows at a time
  // through a wave-private LDS tile, out as 16-byte row segments.
  const int hh = lane >> 5;
  constexpr int kOutCols = NTW * 32;
  constexpr int kOutStride = kOutCols + 8;          // +16 bytes staggers the rows over the banks
  static_assert(3 * 32 * kOutStride <= NTW * kSubElems, "output staging does not fit a weight stage");
  bf16_t* otile = b0;                    // three waves per stage buffer
  if (wave >= 6) otile = b2; else if (wave >= 3) otile = b1;
  otile += (wave % 3) * (32 * kOutStride);
  constexpr int kGranPerRow = kOutCols / 8;
  const int colbase = n0 + wn * kOutCols;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
    for (int j = 0; j < NTW; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        bf16x4 hv;
#pragma unroll
        for (int r = 0; r < 4; ++r) hv[r] = (bf16_t)acc[mt][j][4 * q + r];
        *reinterpret_cast<bf16x4*>(otile + n * kOutStride + j * 32 + 8 * q + 4 * hh) = hv;
      }
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
    __builtin_amdgcn_wave_barrier();
    for (int g = lane; g < 32 * kGranPerRow; g += kWave) {
      const int ml = g / kGranPerRow, c = g - ml * kGranPerRow;
      const int m = mbase + mt * 32 + ml;
      if (m < rows)
        *reinterpret_cast<u32x4*>(out + (size_t)dst_s[m] * N + colbase + c * 8) =
            *reinterpret_cast<const u32x4*>(otile + ml * kOutStride + c * 8);
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_wave_barrier();
  }
}

// ---- weight gradients: dW[e][n][m] = sum over the rows r of expert e of P[srcP(r)][n] Q[srcQ(r)][m] ------------
// Both operands row-major activations, contracted over their rows: K-major both.  srcP(r) = index[r] (GATHER_P) or r,
// likewise Q.  A K stage is 32 rows; rows past the expert's end read `zrow` (zeros, at least 128 elements) on the P
// side and the expert's last row on the Q side (memory that is certainly finite, whatever the rows behind the
// expert's hold).  One workgroup per (expert, 64 MT rows of dW, 128 NTW columns of dW); MT = 4 (256 rows) halves what
// a workgroup streams of Q per row of dW, at 192 accumulator registers and a ring of three 40 KB stages.
// An expert with more than `chunk` rows is cut into chunks of that many rows, each a workgroup of its own per tile of
// dW, so that a few experts holding most of the rows do not leave a few workgroups with most of the work; such an
// expert's chunks write fp32 partial tiles to `part` (one [N, M] slot per chunk, slots numbered over all experts'
// chunks) and wgrad_reduce_block adds them in chunk order.  Experts of one chunk write dW directly.  The chunks are
// listed once per backward pass by wgrad_plan (below), so that a workgroup finds its chunk with one load.
struct WgradPlan {
  int total;         // chunks over all experts
  int n_cut;         // experts cut into more than one chunk
  int pad[2];
  // followed by int4 chunk[total] = {expert, first row, end row, chunks of that expert},
  // from entry `slots` on int4 cut[n_cut] = {expert, its first chunk, its chunks, 0},
  // and from entry `slots + E` on int4 expert[E] = {first chunk, chunks, 0, 0}
};

// One wave: lane = expert, over ALL routed experts (the +/-Identity ones have rows for the router's weight gradient).
// `slots` = the capacity of the chunk list (backward_chunk_slots).
__device__ __forceinline__ void wgrad_plan(const int32_t* __restrict__ offsets, int E, int chunk, int slots, int* __restrict__ plan) {
  const int lane = lane_id();
  int lo = 0, hi = 0;
  if (lane < E) { lo = offsets[lane]; hi = offsets[lane + 1]; }
  const int mine = lane < E ? max(1, (hi - lo + chunk - 1) / chunk) : 0;   // an idle expert keeps one (empty) chunk: its zero gradient
  const int incl = wave_inclusive_scan(mine);
  const int first = incl - mine;
  const unsigned long long cut = __ballot(mine > 1);
  if (lane == kWave - 1) { plan[0] = incl; plan[1] = __popcll(cut); }
  typedef int int4v __attribute__((ext_vector_type(4)));
  int4v* list = reinterpret_cast<int4v*>(plan + 4);
  for (int c = 0; c < mine; ++c) list[first + c] = int4v{lane, lo + c * chunk, min(lo + (c + 1) * chunk, hi), mine};
  if (mine > 1) list[slots + __popcll(cut & ((1ull << lane) - 1))] = int4v{lane, first, mine, 0};
  if (lane < E) list[slots + E + lane] = int4v{first, mine, 0, 0};
}

template <int MT, int NTW, bool GATHER_P, bool GATHER_Q>
__global__ __launch_bounds__(512) void wgrad_kmajor_kernel(const bf16_t* __restrict__ P, const bf16_t* __restrict__ Q,
                                                           const int32_t* __restrict__ index,
                                                           const int32_t* __restrict__ offsets,
                                                           const bf16_t* __restrict__ zrow, int N, int M, int E,
                                                           const int* __restrict__ plan, float* __restrict__ part,
                                                           bf16_t* __restrict__ dW) {
  static_assert(MT == 2 || MT == 4, "128 or 256 rows of dW per workgroup");
  constexpr int BM = 64 * MT, BN = kSubW * NTW;
  constexpr int R = MT == 4 ? 3 : kRing;                 // stages that fit LDS (MT = 4: 40 KB each)
  constexpr int kPOps = MT / 2;                          // 128-column sub-tiles of P
  constexpr int kOps = kPOps + NTW;
  __shared__ __attribute__((aligned(16))) bf16_t p0[kPOps * kSubElems];
  __shared__ __attribute__((aligned(16))) bf16_t p1[kPOps * kSubElems];
  __shared__ __attribute__((aligned(16))) bf16_t p2[kPOps * kSubElems];
  __shared__ __attribute__((aligned(16))) bf16_t p3[R == 4 ? kPOps * kSubElems : 8];
  __shared__ __attribute__((aligned(16))) bf16_t q0[NTW * kSubElems];
  __shared__ __attribute__((aligned(16))) bf16_t q1[NTW * kSubElems];
  __shared__ __attribute__((aligned(16))) bf16_t q2[NTW * kSubElems];
  __shared__ __attribute__((aligned(16))) bf16_t q3[R == 4 ? NTW * kSubElems : 8];
  // Workgroup ids congruent mod 8 run on one XCD: they walk a contiguous range of (expert, m block, n block) triples,
  // so the workgroups that read the same rows of Q (and of P) share that XCD's L2.
  const int nblk_n = N / BM, nblk_m = M / BN;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int total_chunks = __builtin_amdgcn_readfirstlane(plan[0]);
  // With experts cut into chunks the work per chunk is uneven (a cut expert's chunks are several times a small
  // expert's rows) and contiguous ranges of chunks per XCD would leave some XCDs with most of it: round robin then.
  const bool uneven = __builtin_amdgcn_readfirstlane(plan[1]) > 0;
  const int item = uneven ? (int)blockIdx.x : xcd_tile(blockIdx.x, total_chunks * nblk_n * nblk_m);
  if (item >= total_chunks * nblk_n * nblk_m) return;
  const int cg = item / (nblk_n * nblk_m), rest = item - cg * (nblk_n * nblk_m);      // chunk, numbered over all experts
  const int* entry = plan + 4 + 4 * cg;
  const int e = __builtin_amdgcn_readfirstlane(entry[0]);
  if (e >= E) return;                    // E = experts with weights; the chunks behind them belong to +/-Identity experts
  const int lo = __builtin_amdgcn_readfirstlane(entry[1]), hi = __builtin_amdgcn_readfirstlane(entry[2]);
  const int e_chunks = __builtin_amdgcn_readfirstlane(entry[3]);
  const int n0 = (rest % nblk_n) * BM, m0 = (rest / nblk_n) * BN;
  const int wn = wave & 3, wm = wave >> 2;
  floatx16 acc[MT][NTW];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int j = 0; j < NTW; ++j)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mt][j][i] = 0.f;

  auto pbuf = [&](auto bc) -> bf16_t* {
    constexpr int b = decltype(bc)::value;
    if constexpr (b == 0) return p0; else if constexpr (b == 1) return p1; else if constexpr (b == 2) return p2; else return p3;
  };
  auto qbuf = [&](auto bc) -> bf16_t* {
    constexpr int b = decltype(bc)::value;
    if constexpr (b == 0) return q0; else if constexpr (b == 1) return q1; else if constexpr (b == 2) return q2; else return q3;
  };
  const int nstages = (hi - lo + kKS - 1) / kKS;
  const int gofs = kfill_granule(tid) * 8;
  // This thread's row of stage `stage` (row tid / 16 of the stage's 32), the expert's last row past its end.
  auto stage_row = [&](int stage) { return lo + min(stage, nstages - 1) * kKS + (tid >> 4); };
  auto lookup = [&](int stage) {
    return (GATHER_P || GATHER_Q) ? index[min(stage_row(stage), hi - 1)] : 0;
  };
  auto fill = [&](auto bc, int stage, int ix) {
    const int r = stage_row(stage);
    const bool live = r < hi;
    const int rc = live ? r : hi - 1;
    const bf16_t* prow = live ? P + (size_t)(GATHER_P ? ix : rc) * N + n0 : zrow;
    const bf16_t* qrow = Q + (size_t)(GATHER_Q ? ix : rc) * M + m0;
#pragma unroll
    for (int j = 0; j < kPOps; ++j) kfill_subtile(prow + j * kSubW + gofs, pbuf(bc) + j * kSubElems);
#pragma unroll
    for (int j = 0; j < NTW; ++j) kfill_subtile(qrow + j * kSubW + gofs, qbuf(bc) + j * kSubElems);
  };
  int poff[MT], qoff[NTW];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int t32 = wm * MT + mt;
    poff[mt] = (t32 >> 2) * kSubElems + kfrag_offset(lane, (t32 & 3) * 32);
  }
#pragma unroll
  for (int j = 0; j < NTW; ++j) {
    const int t32 = wn * NTW + j;
    qoff[j] = (t32 >> 2) * kSubElems + kfrag_offset(lane, (t32 & 3) * 32);
  }
  using std::integral_constant;
  if (nstages > 0) {                                               // an idle expert's gradient is zero
    // The row index of a gathered operand is loaded R - 1 steps before the transfers that use it (R values rotate
    // through ix[], the index of stage s in ix[s % R]): step s requests stage s + R - 1 with the index loaded at step
    // s - R + 1 and loads the one of stage s + 2 (R - 1).  That load is one more vector-memory operation per step, so
    // the ring's wait counts it.
    constexpr int kVm = kOps + ((GATHER_P || GATHER_Q) ? 1 : 0);
    int ix[R];
    // prologue, oldest request first: stage 0, index R - 1, stage 1, index R, ... stage R - 2, index 2 R - 3
#pragma unroll
    for (int i = 0; i < R - 1; ++i) ix[i] = lookup(i);
    auto prologue = [&](auto ic) {
      constexpr int i = decltype(ic)::value;
      fill(integral_constant<int, i>{}, i, ix[i]);
      ix[(i + R - 1) % R] = lookup(i + R - 1);
    };
    prologue(integral_constant<int, 0>{});
    prologue(integral_constant<int, 1>{});
    if constexpr (R == 4) prologue(integral_constant<int, 2>{});
    auto step = [&](auto bc, int stage) {
      constexpr int b = decltype(bc)::value;
      sync_keep_loads<(R - 2) * kVm>();
      fill(integral_constant<int, (b + R - 1) % R>{}, stage + R - 1, ix[(b + R - 1) % R]);
      ix[(b + R - 2) % R] = lookup(stage + 2 * (R - 1));
      if (stage < nstages) {
        const bf16_t* pt = pbuf(bc);
        const bf16_t* qt = qbuf(bc);
        auto read_p = [&](int s, int mt) { return kfrag_read_s(pt, poff[mt], s); };
        auto read_q = [&](int s, int j) { return kfrag_read_s(qt, qoff[j], s); };
        if constexpr (MT == 2) multiply_stage<MT, NTW>(acc, read_p, read_q);
        else multiply_stage_tall<MT, NTW, 2>(acc, read_p, read_q);
      }
    };
    for (int i = 0; i < nstages; i += R) {
      step(integral_constant<int, 0>{}, i);
      step(integral_constant<int, 1>{}, i + 1);
      step(integral_constant<int, 2>{}, i + 2);
      if constexpr (R == 4) step(integral_constant<int, 3>{}, i + 3);
    }
    __builtin_amdgcn_s_waitcnt(0);       // the repeated requests of the last steps land before the workgroup ends
  }
  // accumulators transposed: lane = row n0 + wm MT 32 + 32 mt + lane % 32, register 4 q + r = column
  // m0 + (wn NTW + j) 32 + 8 q + 4 (lane / 32) + r
  const int n = lane & 31, hh = lane >> 5;
  const size_t oofs = ((size_t)n0 + wm * MT * 32 + n) * M + m0 + wn * NTW * 32 + 4 * hh;
  if (e_chunks == 1) {
    bf16_t* orow = dW + (size_t)e * N * M + oofs;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int j = 0; j < NTW; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          bf16x4 v;
#pragma unroll
          for (int r = 0; r < 4; ++r) v[r] = (bf16_t)acc[mt][j][4 * q + r];
          *reinterpret_cast<bf16x4*>(orow + (size_t)mt * 32 * M + j * 32 + 8 * q) = v;
        }
  } else {
    float* prow = part + (size_t)cg * N * M + oofs;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int j = 0; j < NTW; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          floatx4 v;
#pragma unroll
          for (int r = 0; r < 4; ++r) v[r] = acc[mt][j][4 * q + r];
          *reinterpret_cast<floatx4*>(prow + (size_t)mt * 32 * M + j * 32 + 8 * q) = v;
        }
  }
}

// For the experts that were cut into chunks (none, when the tokens are spread evenly): dW[e] = the sum of expert e's
// partial tiles, in chunk order, for both weight tensors (partials of the first in `part_a`, [.., NMa] each, of the
// second in `part_b`).  Workgroup `block` of 256 threads, a thread per four elements.  E = experts with weights.
__device__ __forceinline__ void wgrad_reduce_block(int block, const float* __restrict__ part_a, const float* __restrict__ part_b,
                                                   const int* __restrict__ plan, int slots, int NMa, int NMb, int E,
                                                   bf16_t* __restrict__ dWa, bf16_t* __restrict__ dWb) {
  const int n_cut = plan[1];
  if (n_cut == 0) return;
  const size_t i = ((size_t)block * 256 + threadIdx.x) * 4;
  const int* cut = plan + 4 + 4 * slots;
  auto reduce = [&](const float* part, int NM, bf16_t* dW, int e, int first, int n) {
    if (i >= (size_t)NM) return;
    floatx4 acc = *reinterpret_cast<const floatx4*>(part + (size_t)first * NM + i);
    for (int c = 1; c < n; ++c) {
      const floatx4 v = *reinterpret_cast<const floatx4*>(part + (size_t)(first + c) * NM + i);
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[r] += v[r];
    }
    bf16x4 o;
#pragma unroll
    for (int r = 0; r < 4; ++r) o[r] = (bf16_t)acc[r];
    *reinterpret_cast<bf16x4*>(dW + (size_t)e * NM + i) = o;
  };
  for (int q = 0; q < n_cut; ++q) {
    const int e = cut[4 * q], first = cut[4 * q + 1], n = cut[4 * q + 2];
    if (e >= E) continue;
    reduce(part_a, NMa, dWa, e, first, n);
    reduce(part_b, NMb, dWb, e, first, n);
  }
}

}  // namespace
}  // namespace bibo
