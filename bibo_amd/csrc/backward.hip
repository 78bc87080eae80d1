// Backward pass of the sparse-MoE block, bf16, gfx950: the gradients torch.autograd derives for the reference's
// eager layer (src/modeling/ffn/moe.py:46-101,157-183, src/modeling/ffn/router.py:25-47) with the selection held
// fixed.  For a routed row (token t, expert e, combine weight w) the forward is
//     gu = W_gate_up[e] x_t,  r = sqrt(mean(g^2) + eps),  h = r^p SiLU(g / r) u,  y = W_down[e] h,  out_t += w y
// and the backward, for the upstream gradient d_t of out_t:
//     dh' = W_down[e]^T d_t            (grouped GEMM over the TRANSPOSED down weights)
//     dw  = <dh', h>,  dh = w dh'      (gradient of the combine weight; moe.py:93)
//     (dg, du, dtheta) from dh         (Radial NormSiLU backward, moe.py:87-92)
//     dx_t += W_gate_up[e]^T [dg, du]  (grouped GEMM over the TRANSPOSED gate/up weights)
//     dW_down[e] += (w d_t) h^T,  dW_gate_up[e] += [dg, du] x_t^T   (grouped GEMMs that contract over an expert's rows)
//     dlogit from dw (router.py:41-47), dW_router += dlogit^T x, dx += dlogit W_router.
// Every GEMM here runs on the LDS-DMA / MFMA stripe machinery of the forward kernels, which wants both operands
// contiguous along the contraction: the weights are transposed once per call, and the row-major activations that
// are contracted over ROWS (the weight gradients) are transposed into [columns][rows] buffers in which each
// expert's rows start at a multiple of 64 and are zero-padded to the next one, so that a K step never straddles
// two experts.
#include "stripe.h"

namespace bibo {
namespace {

constexpr int kPad = 64;     // an expert's rows start at a multiple of this in the transposed buffers
constexpr int kBwdBK = 64;   // K elements per LDS stage of the GEMMs here: whole 128-byte lines per row

// ---- grouped GEMM: out[dst(r), n] = sum_k A[src(r), k] W[e][n, k] for the rows r of expert e ------------------
// src(r) = a_index[r] (GATHER) or r; dst(r) = out_index[r] (SCATTER) or r.  r runs over permuted rows.
template <int MT, int NTW, int WM, bool GATHER, bool SCATTER>
__global__ __launch_bounds__(256 * WM) void ggemm_kernel(const bf16_t* __restrict__ A, const int32_t* __restrict__ a_index,
                                                         const bf16_t* __restrict__ W,
                                                         const int32_t* __restrict__ offsets,
                                                         const int32_t* __restrict__ out_index, int K, int N, int E,
                                                         int nblk_n, bf16_t* __restrict__ out) {
  using S = Stripe<MT, NTW, WM, kBwdBK>;
  constexpr int BM = S::BM;
  constexpr int BN = S::BN;
  __shared__ __attribute__((aligned(16))) bf16_t st0[S::kStageElems];
  __shared__ __attribute__((aligned(16))) bf16_t st1[S::kStageElems];
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
  const int chunk = S::dma_chunk(tid);
  StripeLoader<S> ld;
#pragma unroll
  for (int i = 0; i < S::A_PER; ++i) {
    const int r = row0 + min(S::dma_row(tid) + i * S::kRowsPerInstr, rows - 1);   // rows past the end re-read the last one
    const int src = GATHER ? a_index[r] : r;
    ld.a_src[i] = A + (size_t)src * K + chunk * 8;
  }
  const int n0 = nb * BN;
  ld.b_src = W + ((size_t)e * N + n0 + S::dma_row(tid)) * K + chunk * 8;
  ld.bstep = (size_t)S::kRowsPerInstr * K;
  ld.issue_stage(0, st0);
  floatx16 acc[MT][NTW];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int j = 0; j < NTW; ++j)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mt][j][i] = 0.f;
  auto frag_row = [&](int j) { return (wn * NTW + j) * 32; };
  stripe_mainloop_dma<MT, NTW, WM, S::BK, true>(acc, ld, K, st0, st1, wm, frag_row);

  // Epilogue (accumulators transposed: lane = row, four consecutive columns per register quad): 32 rows at a time
  // through a wave-private LDS tile, out as 16-byte row segments.
  const int mbase = wm * MT * 32;
  const int n = lane & 31, hh = lane >> 5;
  constexpr int kOutCols = NTW * 32;
  constexpr int kOutStride = kOutCols + 8;          // +16 bytes staggers the rows over the banks
  static_assert((4 * WM / 2) * 32 * kOutStride <= S::kStageElems, "output staging does not fit a stage buffer");
  __syncthreads();                       // every wave is done reading the stage buffers
  bf16_t* otile = (wave < 4 * WM / 2 ? st0 : st1) + (wave % (4 * WM / 2)) * (32 * kOutStride);
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

template <int NTW, bool GATHER, bool SCATTER>
hipError_t launch_ggemm_t(const bf16_t* A, const int32_t* a_index, const bf16_t* W, const int32_t* offsets,
                          const int32_t* out_index, int S_rows, int K, int N, int E, bf16_t* out, hipStream_t s) {
  constexpr int MT = 2, WM = 2;
  using St = Stripe<MT, NTW, WM, kBwdBK>;
  const int nblk_n = N / St::BN;
  const int tiles = (S_rows / St::BM + E) * nblk_n;
  const int grid = ((tiles + 7) & ~7) + 8;
  hipLaunchKernelGGL((ggemm_kernel<MT, NTW, WM, GATHER, SCATTER>), dim3(grid), dim3(256 * WM), 0, s, A, a_index, W,
                     offsets, out_index, K, N, E, nblk_n, out);
  return hipGetLastError();
}

template <bool GATHER, bool SCATTER>
hipError_t launch_ggemm(const bf16_t* A, const int32_t* a_index, const bf16_t* W, const int32_t* offsets,
                        const int32_t* out_index, int S_rows, int K, int N, int E, bf16_t* out, hipStream_t s) {
  if (N % 384 == 0) return launch_ggemm_t<3, GATHER, SCATTER>(A, a_index, W, offsets, out_index, S_rows, K, N, E, out, s);
  if (N % 256 == 0) return launch_ggemm_t<2, GATHER, SCATTER>(A, a_index, W, offsets, out_index, S_rows, K, N, E, out, s);
  return launch_ggemm_t<1, GATHER, SCATTER>(A, a_index, W, offsets, out_index, S_rows, K, N, E, out, s);
}

// ---- transposes ---------------------------------------------------------------------------------------------
// A 64 x 64 tile goes through LDS (row stride 66 elements: the eight column reads behind one 16-byte store touch
// different banks); global memory is read and written 16 bytes per thread, 128 contiguous bytes per row.
constexpr int kTS = 66;

// rows j = t / 8 and j + 32 of the tile, columns 8 (t % 8) .. + 8: row j of the tile is in[src(j)], scaled; src < 0: zeros
template <typename RowPtr, typename Scale>
__device__ __forceinline__ void tile_load(bf16_t (&tile)[64][kTS], RowPtr row_ptr, Scale scale) {
  const int t = threadIdx.x, cg = (t & 7) * 8;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int j = (t >> 3) + 32 * h;
    const bf16_t* src = row_ptr(j);
    bf16x8 v;
    if (src != nullptr) {
      v = *reinterpret_cast<const bf16x8*>(src + cg);
      const float sc = scale(j);
      if (sc != 1.f) {
#pragma unroll
        for (int q = 0; q < 8; ++q) v[q] = (bf16_t)(sc * (float)v[q]);
      }
    } else {
#pragma unroll
      for (int q = 0; q < 8; ++q) v[q] = (bf16_t)0.f;
    }
#pragma unroll
    for (int q = 0; q < 8; q += 2)          // 4-byte LDS writes (the row stride is not a multiple of 16 bytes)
      *reinterpret_cast<bf16x2*>(&tile[j][cg + q]) = bf16x2{v[q], v[q + 1]};
  }
}

// column c = t / 8 and c + 32 of the tile, rows 8 (t % 8) .. + 8, to out_row(c) + 8 (t % 8)
template <typename OutPtr>
__device__ __forceinline__ void tile_store_transposed(const bf16_t (&tile)[64][kTS], OutPtr out_row) {
  const int t = threadIdx.x, pg = (t & 7) * 8;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int c = (t >> 3) + 32 * h;
    bf16x8 v;
#pragma unroll
    for (int q = 0; q < 8; ++q) v[q] = tile[pg + q][c];
    *reinterpret_cast<bf16x8*>(out_row(c) + pg) = v;
  }
}

// out[b][c][r] = in[b][r][c] for b < batch.  grid = (C / 64, R / 64, batch), 256 threads.
__global__ __launch_bounds__(256) void transpose_batched_kernel(const bf16_t* __restrict__ in, int R, int C,
                                                                bf16_t* __restrict__ out) {
  __shared__ __attribute__((aligned(16))) bf16_t tile[64][kTS];
  const size_t base = (size_t)blockIdx.z * R * C;
  const int c0 = blockIdx.x * 64, r0 = blockIdx.y * 64;
  tile_load(tile, [&](int j) { return in + base + (size_t)(r0 + j) * C + c0; }, [](int) { return 1.f; });
  __syncthreads();
  tile_store_transposed(tile, [&](int c) { return out + base + (size_t)(c0 + c) * R + r0; });
}

// pad_off[e] = sum over e' < e of the rows of e' rounded up to kPad (one wave; E <= 64)
__global__ void pad_offsets_kernel(const int32_t* __restrict__ offsets, int E, int32_t* __restrict__ pad_off) {
  const int lane = threadIdx.x;
  int n = 0;
  if (lane < E) n = (offsets[lane + 1] - offsets[lane] + kPad - 1) / kPad * kPad;
  const int incl = wave_inclusive_scan(n);
  if (lane < E) pad_off[lane + 1] = incl;
  if (lane == 0) pad_off[0] = 0;
}

// outT[c][pad_off[e] + j] = scale * in[src(offsets[e] + j)][c] for the j-th row of expert e, zero in an expert's
// padding columns.  src(r) = index[r] (or r); scale = scale_by_slot[slot_of_row[r]] (or 1).  grid = (ld / 64, C / 64):
// a workgroup owns 64 columns of the padded row axis, which lie within one expert.
__global__ __launch_bounds__(256) void transpose_rows_kernel(const bf16_t* __restrict__ in,
                                                             const int32_t* __restrict__ index,
                                                             const float* __restrict__ scale_by_slot,
                                                             const int32_t* __restrict__ slot_of_row,
                                                             const int32_t* __restrict__ offsets,
                                                             const int32_t* __restrict__ pad_off, int E, int C, int ld,
                                                             bf16_t* __restrict__ outT) {
  __shared__ __attribute__((aligned(16))) bf16_t tile[64][kTS];
  __shared__ int src_s[64];
  __shared__ float scale_s[64];
  const int p0 = blockIdx.x * 64, c0 = blockIdx.y * 64;
  if (p0 >= pad_off[E]) return;
  int e = 0;
  while (pad_off[e + 1] <= p0) ++e;                            // E <= 64 steps, uniform
  if (threadIdx.x < 64) {
    const int r = offsets[e] + (p0 - pad_off[e]) + threadIdx.x;
    const bool live = r < offsets[e + 1];
    src_s[threadIdx.x] = live ? (index ? index[r] : r) : -1;
    scale_s[threadIdx.x] = (live && scale_by_slot) ? scale_by_slot[slot_of_row[r]] : 1.f;
  }
  __syncthreads();
  tile_load(tile, [&](int j) { return src_s[j] >= 0 ? in + (size_t)src_s[j] * C + c0 : nullptr; },
            [&](int j) { return scale_s[j]; });
  __syncthreads();
  tile_store_transposed(tile, [&](int c) { return outT + (size_t)(c0 + c) * ld + p0; });
}

// ---- weight gradients: dW[e][n][m] = sum over the padded rows kc of expert e of PT[n][kc] QT[m][kc] --------------
// grid = (N / BM, M / BN, E).  Both operands are row-major with leading dimension ld and contiguous along kc.
template <int MT, int NTW, int WM>
__global__ __launch_bounds__(256 * WM) void wgrad_kernel(const bf16_t* __restrict__ PT, const bf16_t* __restrict__ QT,
                                                         const int32_t* __restrict__ pad_off, int N, int M, int ld,
                                                         bf16_t* __restrict__ dW) {
  using S = Stripe<MT, NTW, WM, kBwdBK>;
  constexpr int BM = S::BM, BN = S::BN;
  __shared__ __attribute__((aligned(16))) bf16_t st0[S::kStageElems];
  __shared__ __attribute__((aligned(16))) bf16_t st1[S::kStageElems];
  const int e = blockIdx.z;
  const int n0 = blockIdx.x * BM, m0 = blockIdx.y * BN;
  const int k_lo = pad_off[e], K = pad_off[e + 1] - k_lo;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int wn = wave & 3, wm = wave >> 2;
  floatx16 acc[MT][NTW];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int j = 0; j < NTW; ++j)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mt][j][i] = 0.f;
  if (K > 0) {                                                   // an idle expert's gradient is zero
    const int chunk = S::dma_chunk(tid);
    StripeLoader<S> ldr;
#pragma unroll
    for (int i = 0; i < S::A_PER; ++i)
      ldr.a_src[i] = PT + (size_t)(n0 + S::dma_row(tid) + i * S::kRowsPerInstr) * ld + k_lo + chunk * 8;
    ldr.b_src = QT + (size_t)(m0 + S::dma_row(tid)) * ld + k_lo + chunk * 8;
    ldr.bstep = (size_t)S::kRowsPerInstr * ld;
    ldr.issue_stage(0, st0);
    auto frag_row = [&](int j) { return (wn * NTW + j) * 32; };
    stripe_mainloop_dma<MT, NTW, WM, S::BK, true>(acc, ldr, K, st0, st1, wm, frag_row);
  }
  // accumulators transposed: lane = row n0 + mbase + 32 mt + lane % 32, register 4 q + r = column
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

template <int NTW>
hipError_t launch_wgrad_t(const bf16_t* PT, const bf16_t* QT, const int32_t* pad_off, int N, int M, int ld, int E,
                          bf16_t* dW, hipStream_t s) {
  constexpr int MT = 2, WM = 2;
  using St = Stripe<MT, NTW, WM, kBwdBK>;
  hipLaunchKernelGGL((wgrad_kernel<MT, NTW, WM>), dim3(N / St::BM, M / St::BN, E), dim3(256 * WM), 0, s, PT, QT, pad_off, N,
                     M, ld, dW);
  return hipGetLastError();
}

hipError_t launch_wgrad(const bf16_t* PT, const bf16_t* QT, const int32_t* pad_off, int N, int M, int ld, int E,
                        bf16_t* dW, hipStream_t s) {
  if (M % 384 == 0) return launch_wgrad_t<3>(PT, QT, pad_off, N, M, ld, E, dW, s);
  if (M % 256 == 0) return launch_wgrad_t<2>(PT, QT, pad_off, N, M, ld, E, dW, s);
  return launch_wgrad_t<1>(PT, QT, pad_off, N, M, ld, E, dW, s);
}

// ---- Radial NormSiLU backward (moe.py:87-92), one wave per permuted row ----------------------------------------
// h = r^p a u, a = SiLU(z) = z s, s = sigmoid(z), z = g / r, a' = s (1 + z (1 - s)); with q = dh u:
//   du = dh r^p a;  dg = q r^(p-1) a' + g / (I r) sum_i q_i (p r^(p-1) a_i - r^(p-2) a'_i g_i);
//   dtheta (the row's share) = p'(theta) ln r sum_i q_i r^p a_i;  dw = <dh', h>, dh = w dh'.
// act = SiLU: h = SiLU(g) u, dg = q a'(g), no theta.  Rows of I <= kActMaxI elements.
constexpr int kActMaxI = 512;   // one 16-byte granule of the row per lane

__global__ __launch_bounds__(256) void act_bwd_kernel(const bf16_t* __restrict__ gu, const bf16_t* __restrict__ dhp,
                                                      const float* __restrict__ w, const float* __restrict__ theta,
                                                      const int32_t* __restrict__ offsets,
                                                      const int32_t* __restrict__ perm_slot, int S, int E, int I, int act,
                                                      bf16_t* __restrict__ dgu, bf16_t* __restrict__ hidden,
                                                      float* __restrict__ dw_slot, float* __restrict__ dtheta_row) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= S || row >= offsets[E]) return;                   // E = GLU experts: rows behind theirs have no activation
  int e = 0;
  {                                                            // expert of the row: offsets[e] <= row < offsets[e + 1]
    int lo = 0, hi = E;
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (offsets[mid] <= row) lo = mid; else hi = mid;
    }
    e = lo;
  }
  const int slot = perm_slot[row];
  const float ws = w[slot];
  const bool live = lane * 8 < I;
  bf16x8 gv, uv, dv;
#pragma unroll
  for (int q = 0; q < 8; ++q) gv[q] = uv[q] = dv[q] = (bf16_t)0.f;
  if (live) {
    gv = *reinterpret_cast<const bf16x8*>(gu + (size_t)row * 2 * I + lane * 8);
    uv = *reinterpret_cast<const bf16x8*>(gu + (size_t)row * 2 * I + I + lane * 8);
    dv = *reinterpret_cast<const bf16x8*>(dhp + (size_t)row * I + lane * 8);
  }
  float g[8], u[8], d[8];
  float ss = 0.f;
#pragma unroll
  for (int q = 0; q < 8; ++q) {
    g[q] = (float)gv[q]; u[q] = (float)uv[q]; d[q] = (float)dv[q];
    ss = fmaf(g[q], g[q], ss);
  }
  ss = wave_sum(ss);
  const bool radial = act != BIBO_ACT_SILU;
  float p = 0.f, rinv = 1.f, gain = 1.f;
  if (radial) {
    p = radial_exponent(theta, e, act);
    radial_row_scalars(ss, I, p, act, rinv, gain);             // 1 / r and r^p
  }
  const float r = 1.f / rinv;
  float dot_h = 0.f, sum_qa = 0.f, inner = 0.f;
  float a_[8], ad_[8];
#pragma unroll
  for (int q = 0; q < 8; ++q) {
    const float z = g[q] * rinv;
    const float s = 1.f / (1.f + __expf(-z));
    a_[q] = z * s;
    ad_[q] = s * (1.f + z * (1.f - s));
    dot_h = fmaf(d[q], gain * a_[q] * u[q], dot_h);
    const float qq = ws * d[q] * u[q];
    sum_qa = fmaf(qq, a_[q], sum_qa);
    inner = fmaf(qq, gain * rinv * (p * a_[q] - ad_[q] * z), inner);    // p r^(p-1) a - r^(p-2) a' g = r^(p-1) (p a - a' z)
  }
  dot_h = wave_sum(dot_h);
  sum_qa = wave_sum(sum_qa);
  inner = wave_sum(inner);
  if (live) {
    bf16x8 og, ou, oh;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const float dh = ws * d[q];
      float dg = dh * u[q] * gain * rinv * ad_[q];
      if (radial) dg = fmaf(g[q] * rinv / (float)I, inner, dg);
      og[q] = (bf16_t)dg;
      ou[q] = (bf16_t)(dh * gain * a_[q]);
      oh[q] = (bf16_t)(gain * a_[q] * u[q]);
    }
    *reinterpret_cast<bf16x8*>(dgu + (size_t)row * 2 * I + lane * 8) = og;
    *reinterpret_cast<bf16x8*>(dgu + (size_t)row * 2 * I + I + lane * 8) = ou;
    *reinterpret_cast<bf16x8*>(hidden + (size_t)row * I + lane * 8) = oh;
  }
  if (lane == 0) {
    dw_slot[slot] = dot_h;
    const float dp = act == BIBO_ACT_RADIAL_TANH ? 1.f - p * p : p * (1.f - p);
    dtheta_row[row] = radial ? dp * __logf(r) * gain * sum_qa : 0.f;
  }
}

// +/-Identity experts (moe.py:95-99): a slot routed to one contributes sign w x[t] to the output, so
//   dw[slot] = sign <d_out[t], x[t]>,  dx_slot[slot] = sign w[slot] d_out[t]
// (the per-slot dx rows are summed over a token's slots by dx_combine_kernel like those of the GLU experts).
// One wave per permuted row behind the GLU experts' rows: rows offsets[Eg] .. offsets[Eg + n_pos + n_neg).
__global__ __launch_bounds__(256) void special_bwd_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ d_out,
                                                          const float* __restrict__ w, const int32_t* __restrict__ offsets,
                                                          const int32_t* __restrict__ perm_slot,
                                                          const int32_t* __restrict__ perm_token, int Eg, int n_pos,
                                                          int n_neg, int H, float* __restrict__ dw_slot,
                                                          bf16_t* __restrict__ dxs) {
  const int lane = threadIdx.x & 63;
  const int row = offsets[Eg] + blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= offsets[Eg + n_pos + n_neg]) return;
  const float sign = row < offsets[Eg + n_pos] ? 1.f : -1.f;
  const int slot = perm_slot[row];
  const size_t t = (size_t)perm_token[row];
  const float sw = sign * w[slot];
  float dot = 0.f;
  for (int c = lane * 8; c < H; c += 64 * 8) {
    const bf16x8 xv = *reinterpret_cast<const bf16x8*>(x + t * H + c);
    const bf16x8 dv = *reinterpret_cast<const bf16x8*>(d_out + t * H + c);
    bf16x8 o;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      dot = fmaf((float)dv[q], (float)xv[q], dot);
      o[q] = (bf16_t)(sw * (float)dv[q]);
    }
    *reinterpret_cast<bf16x8*>(dxs + (size_t)slot * H + c) = o;
  }
  dot = wave_sum(dot);
  if (lane == 0) dw_slot[slot] = sign * dot;
}

// dtheta[e] = sum of its rows' contributions, in a fixed order (no atomics: the same bits on every call).
__global__ __launch_bounds__(256) void dtheta_reduce_kernel(const float* __restrict__ dtheta_row,
                                                            const int32_t* __restrict__ offsets,
                                                            float* __restrict__ dtheta) {
  __shared__ float red[4];
  const int e = blockIdx.x, lo = offsets[e], hi = offsets[e + 1];
  float acc = 0.f;
  for (int r = lo + threadIdx.x; r < hi; r += 256) acc += dtheta_row[r];
  acc = wave_sum(acc);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) dtheta[e] = (red[0] + red[1]) + (red[2] + red[3]);
}

// ---- router backward (router.py:31,41-47) --------------------------------------------------------------------
// One thread per token: dlogit of the k selected experts from the gradients of the combine weights.
__global__ void router_bwd_kernel(const float* __restrict__ logits, const int32_t* __restrict__ idx,
                                  const float* __restrict__ w, const float* __restrict__ dw, int T, int E, int k,
                                  int norm_mode, float* __restrict__ dl) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  float s[kMaxK], sum = 0.f, dot = 0.f;
  for (int j = 0; j < k; ++j) {
    s[j] = 1.f / (1.f + __expf(-logits[(size_t)t * E + idx[t * k + j]]));
    sum += s[j];
    dot = fmaf(dw[t * k + j], w[t * k + j], dot);
  }
  for (int j = 0; j < k; ++j) {
    float ds = dw[t * k + j];
    if (k > 1 && norm_mode == BIBO_NORM_SUM) ds = (ds - dot) / (sum + 1e-20f);
    else if (k > 1 && norm_mode == BIBO_NORM_SOFTMAX) ds = w[t * k + j] * (ds - dot);
    dl[t * k + j] = ds * s[j] * (1.f - s[j]);
  }
}

// dx[t, c] = sum_j dxs[t k + j, c] + sum_j dl[t, j] W_router[idx[t, j], c]; one thread per 8 columns.  dl == NULL: the
// slot rows alone (the experts without their router).  A slot whose expert id lies outside [0, n_experts) (padding in
// a caller's indices, which the forward pass skips) has no dxs row and no combine-weight gradient: it is left out of
// the sum and its dw_slot entry is set to zero here.
__global__ __launch_bounds__(256) void dx_combine_kernel(const bf16_t* __restrict__ dxs, const float* __restrict__ dl,
                                                         const int32_t* __restrict__ idx,
                                                         const bf16_t* __restrict__ w_router, int T, int H, int k,
                                                         int n_experts, float* __restrict__ dw_slot,
                                                         bf16_t* __restrict__ dx) {
  const int gpr = H / 8;
  const long long gid = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= (long long)T * gpr) return;
  const int t = (int)(gid / gpr), c = (int)(gid - (long long)t * gpr) * 8;
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  for (int j = 0; j < k; ++j) {
    const int e = idx[t * k + j];
    if (e < 0 || e >= n_experts) {
      if (c == 0) dw_slot[t * k + j] = 0.f;
      continue;
    }
    const bf16x8 v = *reinterpret_cast<const bf16x8*>(dxs + ((size_t)t * k + j) * H + c);
    if (dl != nullptr) {
      const bf16x8 r = *reinterpret_cast<const bf16x8*>(w_router + (size_t)e * H + c);
      const float d = dl[t * k + j];
#pragma unroll
      for (int q = 0; q < 8; ++q) acc[q] += (float)v[q] + d * (float)r[q];
    } else {
#pragma unroll
      for (int q = 0; q < 8; ++q) acc[q] += (float)v[q];
    }
  }
  bf16x8 o;
#pragma unroll
  for (int q = 0; q < 8; ++q) o[q] = (bf16_t)acc[q];
  *reinterpret_cast<bf16x8*>(dx + (size_t)t * H + c) = o;
}

// dW_router[e, c] = sum over the rows r of expert e of dl[slot(r)] x[token(r), c], in two steps.  Step 1, grid =
// (H / 256, E, kDwrSplit): block z takes the z-th of kDwrSplit equal row ranges of the expert; thread (rl = t / 32,
// cg = t % 32) adds up rows rl, rl + 8, .. of the range for columns 8 cg .. + 8 of the block's 256, the eight partial
// sums meet in LDS in a fixed order -> part[e][z][c] fp32.  Step 2 adds the kDwrSplit ranges in order.
constexpr int kDwrSplit = 8;

__global__ __launch_bounds__(256) void dwr_partial_kernel(const bf16_t* __restrict__ x, const float* __restrict__ dl,
                                                          const int32_t* __restrict__ offsets,
                                                          const int32_t* __restrict__ perm_slot,
                                                          const int32_t* __restrict__ perm_token, int H,
                                                          float* __restrict__ part) {
  __shared__ float red[8][256];
  const int e = blockIdx.y, z = blockIdx.z, cg = threadIdx.x & 31, rl = threadIdx.x >> 5;
  const int c = blockIdx.x * 256 + cg * 8;
  const int lo_e = offsets[e], n = offsets[e + 1] - lo_e;
  const int per = (n + kDwrSplit - 1) / kDwrSplit;
  const int lo = lo_e + min(z * per, n), hi = lo_e + min((z + 1) * per, n);
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (c < H)
    for (int r = lo + rl; r < hi; r += 8) {
      const float d = dl[perm_slot[r]];
      const bf16x8 v = *reinterpret_cast<const bf16x8*>(x + (size_t)perm_token[r] * H + c);
#pragma unroll
      for (int q = 0; q < 8; ++q) acc[q] = fmaf(d, (float)v[q], acc[q]);
    }
#pragma unroll
  for (int q = 0; q < 8; ++q) red[rl][cg * 8 + q] = acc[q];
  __syncthreads();
  const int col = blockIdx.x * 256 + threadIdx.x;
  if (col < H) {
    const int t = threadIdx.x;
    part[((size_t)e * kDwrSplit + z) * H + col] =
        ((red[0][t] + red[1][t]) + (red[2][t] + red[3][t])) + ((red[4][t] + red[5][t]) + (red[6][t] + red[7][t]));
  }
}

__global__ __launch_bounds__(256) void dwr_sum_kernel(const float* __restrict__ part, int H, int n, bf16_t* __restrict__ dwr) {
  const int i = blockIdx.x * 256 + threadIdx.x;                 // element of [E, H]
  if (i >= n) return;
  const int e = i / H, c = i - e * H;
  float acc = 0.f;
#pragma unroll
  for (int z = 0; z < kDwrSplit; ++z) acc += part[((size_t)e * kDwrSplit + z) * H + c];
  dwr[i] = (bf16_t)acc;
}

// zero n 4-byte words (a kernel rather than a memset node, so that the call can be captured into a graph)
__global__ void zero_words_kernel(uint32_t* __restrict__ p, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = 0u;
}

void zero_bytes(void* p, size_t bytes, hipStream_t s) {          // bytes is a multiple of 4
  const size_t n = bytes / 4;
  if (n == 0) return;
  const unsigned grid = (unsigned)((n + 255) / 256 < 2048 ? (n + 255) / 256 : 2048);
  hipLaunchKernelGGL(zero_words_kernel, dim3(grid), dim3(256), 0, s, static_cast<uint32_t*>(p), n);
}

}  // namespace

bool backward_supported(int H, int I, int k, int dtype) {
  return dtype == BIBO_DTYPE_BF16 && H >= 128 && H % 128 == 0 && I >= 128 && I % 128 == 0 && I <= kActMaxI &&
         k <= kMaxK;
}

int backward_dwr_split() { return kDwrSplit; }

// leading dimension of the transposed activation buffers: every expert's rows padded to a multiple of kPad
size_t backward_padded_rows(int T, int E, int k) { return ((size_t)T * k + (size_t)E * (kPad - 1) + kPad - 1) / kPad * kPad; }

// The launches after routing and permutation.  Buffers (bf16 unless noted): wd_t [E,I,H], wgu_t [E,H,2I], gu [S,2I],
// dhp [S,I], dgu [S,2I], hidden [S,I], dxs [S,H], p_t [max(H,2I), ld], q_t [max(H,I), ld], dw_slot [S] f32,
// dl [S] f32, dtheta_row [S] f32, dwr_part [E, backward_dwr_split(), H] f32, pad_off [E+1] i32.
hipError_t launch_backward(const void* x, const void* d_out, const void* w_router, const void* wgu, const void* wd,
                           const float* theta, const float* logits, const int32_t* idx, const float* w,
                           const int32_t* offsets, const int32_t* perm_slot, const int32_t* perm_token, int T, int H, int E,
                           int n_pos, int n_neg, int k, int I, int norm_mode, int act, const BackwardBuffers& b, void* dx,
                           void* d_w_router, void* d_wgu, void* d_wd, float* d_theta, hipStream_t s) {
  // E = GLU experts (with weights); the router and the permutation know Et experts, the +/-Identity ones last
  const int Et = E + n_pos + n_neg;
  const int S = T * k;
  const bf16_t* xp = static_cast<const bf16_t*>(x);
  const bf16_t* dop = static_cast<const bf16_t*>(d_out);
  const bf16_t* wrp = static_cast<const bf16_t*>(w_router);
  bf16_t* wd_t = static_cast<bf16_t*>(b.wd_t);
  bf16_t* wgu_t = static_cast<bf16_t*>(b.wgu_t);
  bf16_t* gu = static_cast<bf16_t*>(b.gu);
  bf16_t* dhp = static_cast<bf16_t*>(b.dhp);
  bf16_t* dgu = static_cast<bf16_t*>(b.dgu);
  bf16_t* hidden = static_cast<bf16_t*>(b.hidden);
  bf16_t* dxs = static_cast<bf16_t*>(b.dxs);
  bf16_t* p_t = static_cast<bf16_t*>(b.p_t);
  bf16_t* q_t = static_cast<bf16_t*>(b.q_t);
  const int ld = (int)backward_padded_rows(T, Et, k);
  hipError_t err = hipSuccess;
  if (S == 0) {
    zero_bytes(d_theta, (size_t)E * sizeof(float), s);
    if (d_w_router != nullptr) zero_bytes(d_w_router, (size_t)Et * H * sizeof(bf16_t), s);
    zero_bytes(d_wgu, (size_t)E * 2 * I * H * sizeof(bf16_t), s);
    zero_bytes(d_wd, (size_t)E * H * I * sizeof(bf16_t), s);
    return hipGetLastError();
  }
  hipLaunchKernelGGL(pad_offsets_kernel, dim3(1), dim3(64), 0, s, offsets, E, b.pad_off);
  // transposed weights: wd [E,H,I] -> [E,I,H]; wgu [E,2I,H] -> [E,H,2I]
  hipLaunchKernelGGL(transpose_batched_kernel, dim3(I / 64, H / 64, E), dim3(256), 0, s, static_cast<const bf16_t*>(wd), H, I,
                     wd_t);
  hipLaunchKernelGGL(transpose_batched_kernel, dim3(H / 64, 2 * I / 64, E), dim3(256), 0, s,
                     static_cast<const bf16_t*>(wgu), 2 * I, H, wgu_t);
  // pre-activations again (moe.py:84) and dh' = d W_down (both gather their rows by token)
  err = launch_ggemm<true, false>(xp, perm_token, static_cast<const bf16_t*>(wgu), offsets, nullptr, S, H, 2 * I, E, gu, s);
  if (err != hipSuccess) return err;
  err = launch_ggemm<true, false>(dop, perm_token, wd_t, offsets, nullptr, S, H, I, E, dhp, s);
  if (err != hipSuccess) return err;
  hipLaunchKernelGGL(act_bwd_kernel, dim3((S + 3) / 4), dim3(256), 0, s, gu, dhp, w, theta, offsets, perm_slot, S, E, I, act,
                     dgu, hidden, b.dw_slot, b.dtheta_row);
  hipLaunchKernelGGL(dtheta_reduce_kernel, dim3(E), dim3(256), 0, s, b.dtheta_row, offsets, d_theta);
  // dx of every slot, in slot order: [dg, du] W_gate_up
  err = launch_ggemm<false, true>(dgu, nullptr, wgu_t, offsets, perm_slot, S, 2 * I, H, E, dxs, s);
  if (err != hipSuccess) return err;
  if (n_pos + n_neg > 0)   // (as many waves as there could be rows: how many there are is only known on the device)
    hipLaunchKernelGGL(special_bwd_kernel, dim3((S + 3) / 4), dim3(256), 0, s, xp, dop, w, offsets, perm_slot, perm_token, E,
                       n_pos, n_neg, H, b.dw_slot, dxs);
  const bool with_router = w_router != nullptr;      // else: the experts alone, the caller owns the routing
  if (with_router)
    hipLaunchKernelGGL(router_bwd_kernel, dim3((T + 255) / 256), dim3(256), 0, s, logits, idx, w, b.dw_slot, T, Et, k, norm_mode,
                       b.dl);
  hipLaunchKernelGGL(dx_combine_kernel, dim3((unsigned)(((long long)T * (H / 8) + 255) / 256)), dim3(256), 0, s, dxs,
                     with_router ? b.dl : nullptr, idx, wrp, T, H, k, Et, b.dw_slot, static_cast<bf16_t*>(dx));
  if (with_router) {
    hipLaunchKernelGGL(dwr_partial_kernel, dim3((H + 255) / 256, Et, kDwrSplit), dim3(256), 0, s, xp, b.dl, offsets, perm_slot,
                       perm_token, H, b.dwr_part);
    hipLaunchKernelGGL(dwr_sum_kernel, dim3((Et * H + 255) / 256), dim3(256), 0, s, b.dwr_part, H, Et * H,
                       static_cast<bf16_t*>(d_w_router));
  }
  // weight gradients: dW_down[e] = (w d)^T h, dW_gate_up[e] = [dg, du]^T x, contracted over the expert's rows
  const dim3 tgrid_h(ld / 64, H / 64), tgrid_i(ld / 64, I / 64), tgrid_2i(ld / 64, 2 * I / 64);
  hipLaunchKernelGGL(transpose_rows_kernel, tgrid_h, dim3(256), 0, s, dop, perm_token, w, perm_slot, offsets, b.pad_off, E, H,
                     ld, p_t);
  hipLaunchKernelGGL(transpose_rows_kernel, tgrid_i, dim3(256), 0, s, hidden, nullptr, nullptr, nullptr, offsets, b.pad_off, E,
                     I, ld, q_t);
  err = launch_wgrad(p_t, q_t, b.pad_off, H, I, ld, E, static_cast<bf16_t*>(d_wd), s);
  if (err != hipSuccess) return err;
  hipLaunchKernelGGL(transpose_rows_kernel, tgrid_2i, dim3(256), 0, s, dgu, nullptr, nullptr, nullptr, offsets, b.pad_off, E,
                     2 * I, ld, p_t);
  hipLaunchKernelGGL(transpose_rows_kernel, tgrid_h, dim3(256), 0, s, xp, perm_token, nullptr, nullptr, offsets, b.pad_off, E,
                     H, ld, q_t);
  err = launch_wgrad(p_t, q_t, b.pad_off, 2 * I, H, ld, E, static_cast<bf16_t*>(d_wgu), s);
  if (err != hipSuccess) return err;
  return hipGetLastError();
}

}  // namespace bibo
