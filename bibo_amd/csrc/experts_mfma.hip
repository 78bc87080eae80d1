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
#include "stripe.h"

namespace bibo {
namespace {

// ---- kernel 3 ------------------------------------------------------------------------------------
template <int MT, int NT, int WM>
__global__ __launch_bounds__(256 * WM) void gateup_dma_kernel(const bf16_t* __restrict__ x,
                                                              const bf16_t* __restrict__ wgu,
                                                              const float* __restrict__ theta,
                                                              const int32_t* __restrict__ offsets,
                                                              const int32_t* __restrict__ perm_token, int H, int E,
                                                              int act, bf16_t* __restrict__ hidden) {
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
  const int chunk = S::dma_chunk(tid);
  StripeLoader<S> ld;
  ld.b_src = wgu + ((size_t)e * 2 * I + S::dma_row(tid)) * H + chunk * 8;
  ld.bstep = (size_t)S::kRowsPerInstr * H;
  ld.issue_b(0, st0);                    // weight rows first: they do not wait for the row indices
#pragma unroll
  for (int i = 0; i < S::A_PER; ++i) {
    const int m = min(S::dma_row(tid) + i * S::kRowsPerInstr, rows - 1);     // rows past the end re-read the last valid row
    ld.a_src[i] = x + (size_t)perm_token[row0 + m] * H + chunk * 8;     // gather, moe.py:81
  }
  ld.issue_a(0, st0);
  floatx16 acc[MT][NTW];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int j = 0; j < NTW; ++j)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mt][j][i] = 0.f;
  auto frag_row = [&](int j) { return (j < NT ? 0 : I) + (wn * NT + (j < NT ? j : j - NT)) * 32; };
  stripe_mainloop_dma<MT, NTW, WM, S::BK, true>(acc, ld, H, st0, st1, wm, frag_row);

  // ---- Radial NormSiLU epilogue (moe.py:87-92) ----
  // The accumulators are transposed (lane = row mbase + 32*mt + lane%32, register i = column acc_row(i, lane)
  // of its 32-column tile).  (1) sum of gate^2 per row: this lane's registers, the lane with the other half
  // of the columns (lane ^ 32), then LDS across the four N waves; (2) one thread per row turns it into 1/r
  // and r^p; (3) every lane applies SiLU(g/r) * r^p * up and parks its bf16 results, four consecutive
  // columns at a time, in a wave-private LDS tile; (4) the tile leaves as 16-byte row segments.
  const int mbase = wm * MT * 32;
  const int n = lane & 31, hh = lane >> 5;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    float sq = 0.f;
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int i = 0; i < 16; ++i) sq = fmaf(acc[mt][j][i], acc[mt][j][i], sq);
    sq += __shfl_xor(sq, 32, kWave);
    if (hh == 0) ssq[wn * BM + mbase + mt * 32 + n] = sq;
  }
  __syncthreads();                       // also: every wave is done reading the stage buffers
  if (tid < BM) {
    const float p = radial_exponent(theta, e, act);                                   // moe.py:89
    const float ms = ((ssq[tid] + ssq[BM + tid]) + ssq[2 * BM + tid]) + ssq[3 * BM + tid];
    radial_row_scalars(ms, I, p, act, rinv_s[tid], gain_s[tid]);                      // 1/r and r^p, moe.py:88-89
  }
  __syncthreads();
  constexpr int kOutCols = NT * 32;                 // gate-paired columns owned by this wave
  constexpr int kOutStride = kOutCols + 8;          // bf16 elements; +16 bytes staggers the rows over the banks
  bf16_t* otile = (wave < 4 * WM / 2 ? st0 : st1) + (wave % (4 * WM / 2)) * (MT * 32 * kOutStride);
  static_assert((4 * WM / 2) * MT * 32 * kOutStride <= S::kStageElems, "output staging does not fit a stage buffer");
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int ml = mt * 32 + n;
    const float rinv = rinv_s[mbase + ml];
    const float nrl = -1.44269504f * rinv, rg = rinv * gain_s[mbase + ml];            // per-row constants
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        bf16x4 hv;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float g = acc[mt][j][4 * q + r];
          const float sg = __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(g * nrl));     // sigmoid(g/r)
          hv[r] = (bf16_t)(g * rg * sg * acc[mt][NT + j][4 * q + r]);                  // SiLU(g/r) r^p up
        }
        *reinterpret_cast<bf16x4*>(otile + ml * kOutStride + j * 32 + 8 * q + 4 * hh) = hv;
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
template <int MT, int NTW, int WM, typename TY, int BK = kBK>
__global__ __launch_bounds__(256 * WM) void down_dma_kernel(const bf16_t* __restrict__ hidden,
                                                            const bf16_t* __restrict__ wd, const float* __restrict__ w,
                                                            const int32_t* __restrict__ offsets,
                                                            const int32_t* __restrict__ perm_slot, int H, int E, int I,
                                                            int nblk_n, TY* __restrict__ yw) {
  using S = Stripe<MT, NTW, WM, BK>;
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
  const int chunk = S::dma_chunk(tid);
  StripeLoader<S> ld;
#pragma unroll
  for (int i = 0; i < S::A_PER; ++i) {
    const int m = min(S::dma_row(tid) + i * S::kRowsPerInstr, rows - 1);
    ld.a_src[i] = hidden + (size_t)(row0 + m) * I + chunk * 8;
  }
  const int n0 = nb * BN;
  ld.b_src = wd + ((size_t)e * H + n0 + S::dma_row(tid)) * I + chunk * 8;
  ld.bstep = (size_t)S::kRowsPerInstr * I;
  ld.issue_stage(0, st0);
  floatx16 acc[MT][NTW];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int j = 0; j < NTW; ++j)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mt][j][i] = 0.f;
  auto frag_row = [&](int j) { return (wn * NTW + j) * 32; };
  stripe_mainloop_dma<MT, NTW, WM, S::BK, true>(acc, ld, I, st0, st1, wm, frag_row);

  // Epilogue (accumulators transposed: lane = row, four consecutive columns per register quad): scale by the
  // routing weight (moe.py:93), park 32 rows at a time in a wave-private LDS tile and scatter them to slot
  // order as 16-byte row segments.
  static_assert(sizeof(TY) == 2, "the slot buffer of the MFMA kernels is bf16");
  const int mbase = wm * MT * 32;
  const int n = lane & 31, hh = lane >> 5;
  constexpr int kOutCols = NTW * 32;
  constexpr int kOutStride = kOutCols + 8;          // +16 bytes staggers the rows over the banks
  static_assert((4 * WM / 2) * 32 * kOutStride <= S::kStageElems, "output staging does not fit a stage buffer");
  __syncthreads();                       // every wave is done reading the stage buffers
  TY* otile = reinterpret_cast<TY*>(wave < 4 * WM / 2 ? st0 : st1) + (wave % (4 * WM / 2)) * (32 * kOutStride);
  constexpr int kGranPerRow = kOutCols / 8;
  const int colbase = n0 + wn * kOutCols;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const float ws = w_s[mbase + mt * 32 + n];
#pragma unroll
    for (int j = 0; j < NTW; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        bf16x4 hv;
#pragma unroll
        for (int r = 0; r < 4; ++r) hv[r] = (bf16_t)(ws * acc[mt][j][4 * q + r]);
        *reinterpret_cast<bf16x4*>(otile + n * kOutStride + j * 32 + 8 * q + 4 * hh) = hv;
      }
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
    __builtin_amdgcn_wave_barrier();
    for (int g = lane; g < 32 * kGranPerRow; g += kWave) {
      const int ml = g / kGranPerRow, c = g - ml * kGranPerRow;
      const int m = mbase + mt * 32 + ml;
      if (m < rows)
        *reinterpret_cast<u32x4*>(yw + (size_t)slot_s[m] * H + colbase + c * 8) =
            *reinterpret_cast<const u32x4*>(otile + ml * kOutStride + c * 8);
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_wave_barrier();
  }
}

inline int round_up8(int v) { return (v + 7) & ~7; }

template <int MT, int NT, int WM>
void launch_gateup_dma_t(const bf16_t* x, const bf16_t* wgu, const float* theta, const int32_t* offsets,
                         const int32_t* perm_token, int S, int H, int E, int act, bf16_t* hidden, hipStream_t s) {
  constexpr int BM = 32 * MT * WM;
  const int grid = round_up8(S / BM + E) + 8;
  hipLaunchKernelGGL((gateup_dma_kernel<MT, NT, WM>), dim3(grid), dim3(256 * WM), 0, s, x, wgu, theta, offsets,
                     perm_token, H, E, act, hidden);
}

template <int MT, int NTW, int WM, typename TY, int BK = kBK>
void launch_down_dma_t(const bf16_t* hidden, const bf16_t* wd, const float* w, const int32_t* offsets,
                       const int32_t* perm_slot, int S, int H, int E, int I, TY* yw, hipStream_t s) {
  constexpr int BM = 32 * MT * WM;
  const int nblk_n = H / (128 * NTW);
  const int grid = round_up8((S / BM + E) * nblk_n) + 8;
  hipLaunchKernelGGL((down_dma_kernel<MT, NTW, WM, TY, BK>), dim3(grid), dim3(256 * WM), 0, s, hidden, wd, w, offsets,
                     perm_slot, H, E, I, nblk_n, yw);
}

template <typename TY>
void launch_down_dma_ty(const bf16_t* hidden, const bf16_t* wd, const float* w, const int32_t* offsets,
                        const int32_t* perm_slot, int S, int H, int E, int I, TY* yw, hipStream_t s) {
  if (H % 768 == 0) launch_down_dma_t<2, 6, 2, TY>(hidden, wd, w, offsets, perm_slot, S, H, E, I, yw, s);
  else if (H % 512 == 0) launch_down_dma_t<2, 4, 2, TY>(hidden, wd, w, offsets, perm_slot, S, H, E, I, yw, s);
  // 128-byte stage rows (K steps of 64) fit two stages at this width and measured 8 % faster than 64-byte rows
  else if (H % 384 == 0 && I % 128 == 0) launch_down_dma_t<2, 3, 2, TY, 64>(hidden, wd, w, offsets, perm_slot, S, H, E, I, yw, s);
  else if (H % 384 == 0) launch_down_dma_t<2, 3, 2, TY>(hidden, wd, w, offsets, perm_slot, S, H, E, I, yw, s);
  else if (H % 256 == 0) launch_down_dma_t<2, 2, 2, TY>(hidden, wd, w, offsets, perm_slot, S, H, E, I, yw, s);
  else launch_down_dma_t<2, 1, 2, TY>(hidden, wd, w, offsets, perm_slot, S, H, E, I, yw, s);
}

}  // namespace

bool mfma_supported(int H, int I, int dtype) {
  return dtype == BIBO_DTYPE_BF16 && H >= 128 && (H % 128) == 0 && (I == 128 || I == 256 || I == 384 || I == 512);
}

hipError_t launch_gateup_mfma(const void* x, const void* wgu, const float* theta, const int32_t* offsets,
                              const int32_t* perm_token, int T, int H, int E, int k, int I, int act, void* hidden,
                              hipStream_t s) {
  const int S = T * k;
  if (S == 0) return hipSuccess;
  const bf16_t* xp = static_cast<const bf16_t*>(x);
  const bf16_t* wp = static_cast<const bf16_t*>(wgu);
  bf16_t* hp = static_cast<bf16_t*>(hidden);
  switch (I) {
    case 128: launch_gateup_dma_t<2, 1, 2>(xp, wp, theta, offsets, perm_token, S, H, E, act, hp, s); break;
    case 256: launch_gateup_dma_t<2, 2, 2>(xp, wp, theta, offsets, perm_token, S, H, E, act, hp, s); break;
    case 384: launch_gateup_dma_t<2, 3, 2>(xp, wp, theta, offsets, perm_token, S, H, E, act, hp, s); break;
    case 512: launch_gateup_dma_t<1, 4, 2>(xp, wp, theta, offsets, perm_token, S, H, E, act, hp, s); break;
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
