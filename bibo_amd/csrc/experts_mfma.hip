// Kernels 3 and 4: grouped expert GEMMs on bf16 MFMA (v_mfma_f32_32x32x16_bf16), gfx950.
//
// Both kernels compute a "stripe": BM permuted rows of one expert times a block of weight rows, with
// A (activations) and B (weights, stored [N,K] K-contiguous exactly as the reference keeps them)
// staged through LDS in 32-wide K steps.  Four waves split the N extent; every wave holds
// MT x NTW accumulator tiles of 32x32.
//
//   kernel 3 (gate/up): N covers all I gate columns and all I up columns of the expert, so the
//     row-wise mean of gate^2 that Radial NormSiLU needs is complete inside one workgroup; wave w
//     owns gate columns [w*I/4, (w+1)*I/4) and the SAME up columns, so act(gate)*up is formed in
//     registers.  Reference: src/modeling/ffn/moe.py:81-92.
//   kernel 4 (down): N is a block of hidden columns; the epilogue multiplies each row by its routing
//     weight and scatters it to slot order (token-major), where kernel `combine` sums the k rows of
//     a token.  Reference: src/modeling/ffn/moe.py:92-93,101.
#include "common.h"

namespace bibo {
namespace {

constexpr int kBK = 32;        // K elements per LDS stage
constexpr int kLds = 40;       // LDS row stride in bf16 (32 + 8 pad = 80 bytes: 16-byte reads conflict-free)

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

// K loop shared by both kernels.
//   a_src[i]  : per-thread global pointers of the A chunks this thread stages (row base + 8*chunk)
//   b_base    : first weight row of this workgroup's B block, row stride `ldb` elements
//   frag_row  : LDS B row of accumulator tile j of this wave is frag_row(j) + lane%32
template <int MT, int NTW, typename FragRow>
__device__ __forceinline__ void stripe_mainloop(floatx16 (&acc)[MT][NTW], const bf16_t* const* a_src,
                                                const bf16_t* __restrict__ b_base, int ldb, int K, bf16_t* As,
                                                bf16_t* Bs, FragRow frag_row) {
  constexpr int BM = 32 * MT;
  constexpr int BN = 128 * NTW;
  constexpr int A_PER = (BM * 4 + 255) / 256;
  constexpr int B_PER = BN * 4 / 256;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int crow = tid >> 2, cchunk = tid & 3;     // staging: 4 threads per 64-byte row segment
  const int frow = lane & 31, fk = (lane >> 5) * 8;   // fragment: row, k offset of this lane

  u32x4 ra[A_PER], rb[B_PER];
  const bf16_t* bsrc = b_base + (size_t)crow * ldb + cchunk * 8;
  const size_t bstep = (size_t)64 * ldb;
  constexpr bool kAFull = (A_PER * 256 == BM * 4);

#pragma unroll
  for (int i = 0; i < A_PER; ++i)
    if (kAFull || tid + i * 256 < BM * 4) ra[i] = *reinterpret_cast<const u32x4*>(a_src[i]);
#pragma unroll
  for (int i = 0; i < B_PER; ++i) rb[i] = *reinterpret_cast<const u32x4*>(bsrc + i * bstep);

  for (int k0 = 0; k0 < K; k0 += kBK) {
    __syncthreads();           // every wave is done reading the previous stage
#pragma unroll
    for (int i = 0; i < A_PER; ++i)
      if (kAFull || tid + i * 256 < BM * 4)
        *reinterpret_cast<u32x4*>(As + (crow + i * 64) * kLds + cchunk * 8) = ra[i];
#pragma unroll
    for (int i = 0; i < B_PER; ++i) *reinterpret_cast<u32x4*>(Bs + (crow + i * 64) * kLds + cchunk * 8) = rb[i];
    __syncthreads();
    if (k0 + kBK < K) {        // next stage travels while this one is multiplied
      const int k1 = k0 + kBK;
#pragma unroll
      for (int i = 0; i < A_PER; ++i)
        if (kAFull || tid + i * 256 < BM * 4) ra[i] = *reinterpret_cast<const u32x4*>(a_src[i] + k1);
#pragma unroll
      for (int i = 0; i < B_PER; ++i) rb[i] = *reinterpret_cast<const u32x4*>(bsrc + i * bstep + k1);
    }
#pragma unroll
    for (int kk = 0; kk < kBK; kk += 16) {
      bf16x8 a[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        a[mt] = *reinterpret_cast<const bf16x8*>(As + (mt * 32 + frow) * kLds + kk + fk);
#pragma unroll
      for (int j = 0; j < NTW; ++j) {
        const bf16x8 b = *reinterpret_cast<const bf16x8*>(Bs + (frag_row(j) + frow) * kLds + kk + fk);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[mt][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[mt], b, acc[mt][j], 0, 0, 0);
      }
    }
  }
}

// Accumulator layout of one 32x32 tile: lane holds column lane%32; register i is row
// 8*(i/4) + 4*(lane/32) + i%4.
__device__ __forceinline__ int acc_row(int i, int lane) { return 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3); }

// ---- kernel 3 ------------------------------------------------------------------------------------
template <int MT, int NT>
__global__ __launch_bounds__(256) void gateup_mfma_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ wgu,
                                                          const float* __restrict__ theta,
                                                          const int32_t* __restrict__ offsets,
                                                          const int32_t* __restrict__ perm_token, int H, int E,
                                                          bf16_t* __restrict__ hidden) {
  constexpr int BM = 32 * MT;
  constexpr int NTW = 2 * NT;
  constexpr int I = 128 * NT;
  constexpr int BN = 2 * I;
  constexpr int A_PER = (BM * 4 + 255) / 256;
  __shared__ __attribute__((aligned(16))) bf16_t As[BM * kLds];
  __shared__ __attribute__((aligned(16))) bf16_t Bs[BN * kLds];
  __shared__ float ssq[4 * BM];

  const TileMap tm = make_tile_map(offsets, E, BM);
  const int tile = xcd_tile(blockIdx.x, tm.total);
  if (tile >= tm.total) return;
  int e, row0, rows;
  find_tile(tm, offsets, BM, tile, e, row0, rows);

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const bf16_t* a_src[A_PER];
#pragma unroll
  for (int i = 0; i < A_PER; ++i) {
    const int m = min((tid >> 2) + i * 64, rows - 1);        // rows past the end re-read the last valid row
    a_src[i] = x + (size_t)perm_token[row0 + m] * H + (tid & 3) * 8;     // gather, moe.py:81
  }
  floatx16 acc[MT][NTW];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int j = 0; j < NTW; ++j)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mt][j][i] = 0.f;

  const bf16_t* b_base = wgu + (size_t)e * BN * H;
  // LDS rows 0..I-1 hold gate rows, I..2I-1 up rows; tiles 0..NT-1 of a wave are gate, NT..2NT-1 up
  auto frag_row = [&](int j) { return (j < NT ? 0 : I) + (wave * NT + (j < NT ? j : j - NT)) * 32; };
  stripe_mainloop<MT, NTW>(acc, a_src, b_base, H, H, As, Bs, frag_row);

  // ---- Radial NormSiLU epilogue (moe.py:87-92) ----
  // sum of gate^2 per row: over this wave's columns (registers + 32-lane reduction), then over waves
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      float s = 0.f;
#pragma unroll
      for (int j = 0; j < NT; ++j) s = fmaf(acc[mt][j][i], acc[mt][j][i], s);
#pragma unroll
      for (int o = 16; o > 0; o >>= 1) s += __shfl_xor(s, o, kWave);
      if ((lane & 31) == 0) ssq[wave * BM + mt * 32 + acc_row(i, lane)] = s;
    }
  __syncthreads();
  const float p = 1.f / (1.f + __expf(-theta[e]));                                    // moe.py:89
  const int col0 = wave * NT * 32 + (lane & 31);
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int m = mt * 32 + acc_row(i, lane);
      if (m < rows) {
        const float ms = ((ssq[m] + ssq[BM + m]) + ssq[2 * BM + m]) + ssq[3 * BM + m];
        const float r2 = ms * (1.f / (float)I) + kNormSiluEps;
        const float rinv = rsqrtf(r2);                                                // 1/r, moe.py:88
        const float gain = __expf(0.5f * p * __logf(r2));                             // r^p
        bf16_t* hrow = hidden + (size_t)(row0 + m) * I + col0;
#pragma unroll
        for (int j = 0; j < NT; ++j) {
          const float z = acc[mt][j][i] * rinv;
          const float act = z / (1.f + __expf(-z)) * gain;                            // SiLU(g/r) * r^p
          hrow[j * 32] = (bf16_t)(act * acc[mt][NT + j][i]);                          // * up
        }
      }
    }
}

// ---- kernel 4 ------------------------------------------------------------------------------------
template <int MT, int NTW, typename TY>
__global__ __launch_bounds__(256) void down_mfma_kernel(const bf16_t* __restrict__ hidden, const bf16_t* __restrict__ wd,
                                                        const float* __restrict__ w,
                                                        const int32_t* __restrict__ offsets,
                                                        const int32_t* __restrict__ perm_slot, int H, int E, int I,
                                                        int nblk_n, TY* __restrict__ yw) {
  constexpr int BM = 32 * MT;
  constexpr int BN = 128 * NTW;
  constexpr int A_PER = (BM * 4 + 255) / 256;
  __shared__ __attribute__((aligned(16))) bf16_t As[BM * kLds];
  __shared__ __attribute__((aligned(16))) bf16_t Bs[BN * kLds];
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
  if (tid < BM) {
    const int slot = perm_slot[row0 + min(tid, rows - 1)];
    slot_s[tid] = slot;
    w_s[tid] = w[slot];
  }
  const bf16_t* a_src[A_PER];
#pragma unroll
  for (int i = 0; i < A_PER; ++i) {
    const int m = min((tid >> 2) + i * 64, rows - 1);
    a_src[i] = hidden + (size_t)(row0 + m) * I + (tid & 3) * 8;
  }
  floatx16 acc[MT][NTW];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int j = 0; j < NTW; ++j)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mt][j][i] = 0.f;

  const int n0 = nb * BN;
  const bf16_t* b_base = wd + ((size_t)e * H + n0) * I;
  auto frag_row = [&](int j) { return (wave * NTW + j) * 32; };
  stripe_mainloop<MT, NTW>(acc, a_src, b_base, I, I, As, Bs, frag_row);
  // slot_s / w_s were written before the main loop's barriers, so they are visible here

  const int col0 = n0 + wave * NTW * 32 + (lane & 31);
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int m = mt * 32 + acc_row(i, lane);
      if (m < rows) {
        const float ws = w_s[m];                                                     // moe.py:93
        TY* yrow = yw + (size_t)slot_s[m] * H + col0;
#pragma unroll
        for (int j = 0; j < NTW; ++j) yrow[j * 32] = from_float<TY>(ws * acc[mt][j][i]);
      }
    }
}

inline int round_up8(int v) { return (v + 7) & ~7; }

template <int MT, int NT>
void launch_gateup_t(const bf16_t* x, const bf16_t* wgu, const float* theta, const int32_t* offsets,
                     const int32_t* perm_token, int S, int H, int E, bf16_t* hidden, hipStream_t s) {
  constexpr int BM = 32 * MT;
  const int grid = round_up8(S / BM + E) + 8;
  hipLaunchKernelGGL((gateup_mfma_kernel<MT, NT>), dim3(grid), dim3(256), 0, s, x, wgu, theta, offsets, perm_token, H,
                     E, hidden);
}

template <int MT, int NTW, typename TY>
void launch_down_t(const bf16_t* hidden, const bf16_t* wd, const float* w, const int32_t* offsets,
                   const int32_t* perm_slot, int S, int H, int E, int I, TY* yw, hipStream_t s) {
  constexpr int BM = 32 * MT;
  const int nblk_n = H / (128 * NTW);
  const int grid = round_up8((S / BM + E) * nblk_n) + 8;
  hipLaunchKernelGGL((down_mfma_kernel<MT, NTW, TY>), dim3(grid), dim3(256), 0, s, hidden, wd, w, offsets, perm_slot,
                     H, E, I, nblk_n, yw);
}

template <typename TY>
void launch_down_ty(const bf16_t* hidden, const bf16_t* wd, const float* w, const int32_t* offsets,
                    const int32_t* perm_slot, int S, int H, int E, int I, TY* yw, hipStream_t s) {
  if (H % 768 == 0) launch_down_t<2, 6, TY>(hidden, wd, w, offsets, perm_slot, S, H, E, I, yw, s);
  else if (H % 512 == 0) launch_down_t<2, 4, TY>(hidden, wd, w, offsets, perm_slot, S, H, E, I, yw, s);
  else if (H % 384 == 0) launch_down_t<2, 3, TY>(hidden, wd, w, offsets, perm_slot, S, H, E, I, yw, s);
  else if (H % 256 == 0) launch_down_t<2, 2, TY>(hidden, wd, w, offsets, perm_slot, S, H, E, I, yw, s);
  else launch_down_t<2, 1, TY>(hidden, wd, w, offsets, perm_slot, S, H, E, I, yw, s);
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
    case 128: launch_gateup_t<2, 1>(xp, wp, theta, offsets, perm_token, S, H, E, hp, s); break;
    case 256: launch_gateup_t<2, 2>(xp, wp, theta, offsets, perm_token, S, H, E, hp, s); break;
    case 384: launch_gateup_t<2, 3>(xp, wp, theta, offsets, perm_token, S, H, E, hp, s); break;
    case 512: launch_gateup_t<2, 4>(xp, wp, theta, offsets, perm_token, S, H, E, hp, s); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

hipError_t launch_down_mfma(const void* hidden, const void* wd, const float* w, const int32_t* offsets,
                            const int32_t* perm_slot, int T, int H, int E, int k, int I, void* yw, int yw_is_bf16,
                            hipStream_t s) {
  const int S = T * k;
  if (S == 0) return hipSuccess;
  const bf16_t* hp = static_cast<const bf16_t*>(hidden);
  const bf16_t* wp = static_cast<const bf16_t*>(wd);
  if (yw_is_bf16) launch_down_ty<bf16_t>(hp, wp, w, offsets, perm_slot, S, H, E, I, static_cast<bf16_t*>(yw), s);
  else launch_down_ty<float>(hp, wp, w, offsets, perm_slot, S, H, E, I, static_cast<float*>(yw), s);
  return hipGetLastError();
}

}  // namespace bibo
