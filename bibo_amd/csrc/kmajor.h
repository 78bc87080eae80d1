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

constexpr int kKS = 64;                 // k rows per LDS stage
constexpr int kSubW = 128;              // n elements per sub-tile row (256 bytes: whole 128-byte lines per DMA row)
constexpr int kSubElems = kKS * kSubW;  // 16 KB

// LDS layout of a K-major sub-tile [64 k][128 n]: 16-byte granule G of row k sits at position G ^ ((k & 3) << 2).
// The four k rows one transposed read touches then lie in four different 64-byte quarters of the 256-byte bank
// period, so the read has no bank conflicts.

// What a thread contributes to the fill of K-major sub-tiles: with 512 threads an instruction moves 512 granules =
// 32 rows of 16, so thread t handles rows t / 16 and 32 + t / 16, position t % 16.
struct KFill {
  int krow;        // t / 16
  int gcol;        // logical granule this thread fetches for row krow AND row krow + 32 (both have the same k & 3)
  __device__ __forceinline__ void init(int tid) {
    krow = tid >> 4;
    gcol = (tid & 15) ^ ((krow & 3) << 2);
  }
};

// Fill one sub-tile from two row pointers (the rows krow and krow + 32 of the stage, already offset to the sub-tile's
// first column).
__device__ __forceinline__ void kfill_subtile(const KFill& f, const bf16_t* row_a, const bf16_t* row_b, bf16_t* sub) {
  const int wave_elems = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)) * 64 * 8;
  dma16(row_a + f.gcol * 8, sub + wave_elems);
  dma16(row_b + f.gcol * 8, sub + 512 * 8 + wave_elems);
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

// the same with the step as a loop variable of an unrolled loop (folds to one of the four)
__device__ __forceinline__ bf16x8 kfrag_read_s(const bf16_t* sub, int off, int s) {
  return s == 0 ? kfrag_read<0>(sub, off) : s == 1 ? kfrag_read<1>(sub, off) : s == 2 ? kfrag_read<2>(sub, off)
                                                                                      : kfrag_read<3>(sub, off);
}

// One K stage (four k16 steps) of a wave's MT x NTW tiles as a software pipeline: the fragments of step s + 1 are read
// while step s is multiplied, two LDS reads behind every MFMA.  read_a(s, mt) / read_b(s, j) return the fragments.
template <int MT, int NTW, typename ReadA, typename ReadB>
__device__ __forceinline__ void multiply_stage(floatx16 (&acc)[MT][NTW], ReadA read_a, ReadB read_b) {
  bf16x8 af[2][MT], bfr[2][NTW];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) af[0][mt] = read_a(0, mt);
#pragma unroll
  for (int j = 0; j < NTW; ++j) bfr[0][j] = read_b(0, j);
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    if (s < 3) {
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
      if (s < 3) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
  }
}

// Row-major A tile [128 rows][64 k] in the stripe layout (granule c of row r at c ^ ((r >> 1) & 7)): fill by 512
// threads, two instructions; thread t handles rows t / 8 and 64 + t / 8.
__device__ __forceinline__ void afill(const bf16_t* row_a, const bf16_t* row_b, bf16_t* tile) {
  const int tid = threadIdx.x;
  const int wave_elems = __builtin_amdgcn_readfirstlane(tid >> 6) * 64 * 8;
  const int g = (tid & 7) ^ ((tid >> 4) & 7);                  // rows t / 8 and 64 + t / 8 have the same (row >> 1) & 7
  dma16(row_a + g * 8, tile + wave_elems);
  dma16(row_b + g * 8, tile + 512 * 8 + wave_elems);
}

// ---- input gradients: out[dst(r), n] = sum_k A[src(r), k] W[e][k, n] for the rows r of expert e ----------------
// A row-major (K contiguous), W K-major as stored: [K, N] per expert.  src(r) = a_index[r] (GATHER) or r; dst(r) =
// out_index[r] (SCATTER) or r.  Workgroup = 128 rows x 128 NTW columns, 2 x 4 waves, 32x32x16 MFMA, operands swapped
// so that a lane owns one output row.
template <int NTW, bool GATHER, bool SCATTER>
__global__ __launch_bounds__(512) void dgrad_kmajor_kernel(const bf16_t* __restrict__ A, const int32_t* __restrict__ a_index,
                                                           const bf16_t* __restrict__ W,
                                                           const int32_t* __restrict__ offsets,
                                                           const int32_t* __restrict__ out_index, int K, int N, int E,
                                                           int nblk_n, bf16_t* __restrict__ out) {
  constexpr int MT = 2, BM = 128, BN = kSubW * NTW;
  constexpr int kATile = BM * kKS;
  __shared__ __attribute__((aligned(16))) bf16_t a0[kATile];
  __shared__ __attribute__((aligned(16))) bf16_t a1[kATile];
  __shared__ __attribute__((aligned(16))) bf16_t b0[NTW * kSubElems];
  __shared__ __attribute__((aligned(16))) bf16_t b1[NTW * kSubElems];
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
  const bf16_t* arow[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int r = row0 + min((tid >> 3) + 64 * i, rows - 1);        // rows past the end re-read the last one
    arow[i] = A + (size_t)(GATHER ? a_index[r] : r) * K;
  }
  KFill kf;
  kf.init(tid);
  const int n0 = nb * BN;
  const bf16_t* wrow = W + (size_t)e * K * N + (size_t)kf.krow * N + n0;   // row krow of the first stage; + 32 N: the other
  auto fill = [&](int k0, bf16_t* at, bf16_t* bt) {
    afill(arow[0] + k0, arow[1] + k0, at);
    const bf16_t* w0 = wrow + (size_t)k0 * N;
#pragma unroll
    for (int j = 0; j < NTW; ++j) kfill_subtile(kf, w0 + j * kSubW, w0 + (size_t)32 * N + j * kSubW, bt + j * kSubElems);
  };
  fill(0, a0, b0);

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
  const int apos0 = (h ^ ((n >> 1) & 7)) * 8;
  const int aoff = (mbase + n) * kKS;
  int boff[NTW];
#pragma unroll
  for (int j = 0; j < NTW; ++j) {
    const int t32 = wn * NTW + j;
    boff[j] = (t32 >> 2) * kSubElems + kfrag_offset(lane, (t32 & 3) * 32);
  }
  auto multiply = [&](const bf16_t* at, const bf16_t* bt) {
    multiply_stage<MT, NTW>(
        acc,
        [&](int s, int mt) { return *reinterpret_cast<const bf16x8*>(at + aoff + mt * 32 * kKS + (apos0 ^ (s * 16))); },
        [&](int s, int j) { return kfrag_read_s(bt, boff[j], s); });
  };
  for (int k0 = 0; k0 < K; k0 += 2 * kKS) {
    wait_loads_and_sync();
    if (k0 + kKS < K) fill(k0 + kKS, a1, b1);
    multiply(a0, b0);
    if (k0 + kKS < K) {
      wait_loads_and_sync();
      if (k0 + 2 * kKS < K) fill(k0 + 2 * kKS, a0, b0);
      multiply(a1, b1);
    }
  }

  // Epilogue (accumulators transposed: lane = row, four consecutive columns per register quad): 32 rows at a time
  // through a wave-private LDS tile, out as 16-byte row segments.
  const int hh = lane >> 5;
  constexpr int kOutCols = NTW * 32;
  constexpr int kOutStride = kOutCols + 8;          // +16 bytes staggers the rows over the banks
  static_assert(4 * 32 * kOutStride <= NTW * kSubElems, "output staging does not fit a weight stage");
  __syncthreads();                       // every wave is done reading the stage buffers
  bf16_t* otile = (wave < 4 ? b0 : b1) + (wave & 3) * (32 * kOutStride);
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
// likewise Q.  A K stage is 64 rows; rows past the expert's end read `zrow` (zeros, at least 128 elements) on the P
// side.  One workgroup per (expert, 128 rows of dW, 128 NTW columns of dW).
template <int NTW, bool GATHER_P, bool GATHER_Q>
__global__ __launch_bounds__(512) void wgrad_kmajor_kernel(const bf16_t* __restrict__ P, const bf16_t* __restrict__ Q,
                                                           const int32_t* __restrict__ index,
                                                           const int32_t* __restrict__ offsets,
                                                           const bf16_t* __restrict__ zrow, int N, int M, int E,
                                                           bf16_t* __restrict__ dW) {
  constexpr int MT = 2, BM = 128, BN = kSubW * NTW;
  __shared__ __attribute__((aligned(16))) bf16_t p0[kSubElems];
  __shared__ __attribute__((aligned(16))) bf16_t p1[kSubElems];
  __shared__ __attribute__((aligned(16))) bf16_t q0[NTW * kSubElems];
  __shared__ __attribute__((aligned(16))) bf16_t q1[NTW * kSubElems];
  // Workgroup ids congruent mod 8 run on one XCD: they walk a contiguous range of (expert, m block, n block) triples,
  // so the workgroups that read the same rows of Q (and of P) share that XCD's L2.
  const int nblk_n = N / BM, nblk_m = M / BN;
  const int item = xcd_tile(blockIdx.x, E * nblk_n * nblk_m);
  if (item >= E * nblk_n * nblk_m) return;
  const int e = item / (nblk_n * nblk_m), rest = item - e * (nblk_n * nblk_m);
  const int n0 = (rest % nblk_n) * BM, m0 = (rest / nblk_n) * BN;
  const int lo = offsets[e], hi = offsets[e + 1];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int wn = wave & 3, wm = wave >> 2;
  floatx16 acc[MT][NTW];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int j = 0; j < NTW; ++j)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mt][j][i] = 0.f;

  KFill kf;
  kf.init(tid);
  // rows lo + k0 + krow and + 32 of every stage; their source rows, one stage ahead of the fill that uses them
  // (a row past the expert's end reads zeros on the P side and, on the Q side, the expert's last row: memory that is
  // certainly finite, whatever the rows behind the expert's hold)
  auto source = [&](int r, const bf16_t*& prow, const bf16_t*& qrow) {
    const bool live = r < hi;
    const int rc = live ? r : hi - 1;
    const int ix = (GATHER_P || GATHER_Q) ? index[rc] : 0;
    prow = live ? P + (size_t)(GATHER_P ? ix : rc) * N + n0 : zrow;
    qrow = Q + (size_t)(GATHER_Q ? ix : rc) * M + m0;
  };
  const bf16_t *pa, *pb, *qa, *qb;
  auto fill = [&](bf16_t* pt, bf16_t* qt) {
    kfill_subtile(kf, pa, pb, pt);
#pragma unroll
    for (int j = 0; j < NTW; ++j) kfill_subtile(kf, qa + j * kSubW, qb + j * kSubW, qt + j * kSubElems);
  };
  int poff[MT], qoff[NTW];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) poff[mt] = kfrag_offset(lane, (wm * MT + mt) * 32);
#pragma unroll
  for (int j = 0; j < NTW; ++j) {
    const int t32 = wn * NTW + j;
    qoff[j] = (t32 >> 2) * kSubElems + kfrag_offset(lane, (t32 & 3) * 32);
  }
  auto multiply = [&](const bf16_t* pt, const bf16_t* qt) {
    multiply_stage<MT, NTW>(
        acc, [&](int s, int mt) { return kfrag_read_s(pt, poff[mt], s); },
        [&](int s, int j) { return kfrag_read_s(qt, qoff[j], s); });
  };
  if (hi > lo) {                                                   // an idle expert's gradient is zero
    // The source rows of a stage (two index loads per thread when an operand is gathered) are looked up a stage
    // before the fill that uses them, right after the fill before it, so the loads fly during a multiply.
    const int r_a = lo + kf.krow;
    auto sources = [&](int k0) { source(r_a + k0, pa, qa); source(r_a + k0 + 32, pb, qb); };
    sources(0);
    fill(p0, q0);
    if (lo + kKS < hi) sources(kKS);
    for (int k0 = 0; lo + k0 < hi; k0 += 2 * kKS) {
      const bool more1 = lo + k0 + kKS < hi;
      wait_loads_and_sync();
      if (more1) {
        fill(p1, q1);
        if (lo + k0 + 2 * kKS < hi) sources(k0 + 2 * kKS);
      }
      multiply(p0, q0);
      if (more1) {
        const bool more2 = lo + k0 + 2 * kKS < hi;
        wait_loads_and_sync();
        if (more2) {
          fill(p0, q0);
          if (lo + k0 + 3 * kKS < hi) sources(k0 + 3 * kKS);
        }
        multiply(p1, q1);
      }
    }
  }
  // accumulators transposed: lane = row n0 + wm MT 32 + 32 mt + lane % 32, register 4 q + r = column
  // m0 + (wn NTW + j) 32 + 8 q + 4 (lane / 32) + r
  const int n = lane & 31, hh = lane >> 5;
  bf16_t* orow = dW + ((size_t)e * N + n0 + wm * MT * 32 + n) * M + m0 + wn * NTW * 32 + 4 * hh;
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
}

}  // namespace
}  // namespace bibo
