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
// Every GEMM here runs on LDS-DMA stages and 32x32x16 MFMAs.  The pre-activations are recomputed with the forward's
// operand layout (both operands contiguous along the contraction).  The input gradients contract over the middle
// dimension of the weight tensors and the weight gradients over the ROWS of row-major activations: those operands go
// to LDS as they lie in memory and are read through transposing LDS reads (kmajor.h), so nothing is transposed in
// memory and an expert's rows need no padding: a K stage that runs past an expert's last row reads a row of zeros.
#include "kmajor.h"

namespace bibo {
namespace {

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

// 256-row tiles stream an expert's weights through LDS half as often as 128-row tiles but take about 1.75 times as
// long each, and the workgroups of a launch run in rounds of one per CU (256 on this chip): the tall tiles pay when
// their rounds, weighted so, are fewer.  Only for experts that hold 192 rows on average (a 256-row tile is then at
// least half full where it matters).
inline bool tall_tiles(int S_rows, int E, long long tiles_short, long long tiles_tall) {
  constexpr long long kCUs = 256;
  const long long rs = (tiles_short + kCUs - 1) / kCUs, rt = (tiles_tall + kCUs - 1) / kCUs;
  return (long long)S_rows >= 192ll * E && rt * 7 < rs * 4;
}

template <int NTW, bool GATHER, bool SCATTER>
hipError_t launch_dgrad_t(const bf16_t* A, const int32_t* a_index, const bf16_t* W, const int32_t* offsets,
                          const int32_t* out_index, int S_rows, int K, int N, int E, bf16_t* out, hipStream_t s) {
  constexpr int BN = kSubW * NTW;
  const int nblk_n = N / BN;
  // an expert's last tile is ragged: about half a tile per expert on top of the full ones
  const bool tall = tall_tiles(S_rows, E, (long long)(S_rows / 128 + E / 2) * nblk_n, (long long)(S_rows / 256 + E / 2) * nblk_n);
  const int tiles = (S_rows / (tall ? 256 : 128) + E) * nblk_n;
  const int grid = ((tiles + 7) & ~7) + 8;
  if (tall)
    hipLaunchKernelGGL((dgrad_kmajor_kernel<4, NTW, GATHER, SCATTER>), dim3(grid), dim3(512), 0, s, A, a_index, W, offsets,
                       out_index, K, N, E, nblk_n, out);
  else
    hipLaunchKernelGGL((dgrad_kmajor_kernel<2, NTW, GATHER, SCATTER>), dim3(grid), dim3(512), 0, s, A, a_index, W, offsets,
                       out_index, K, N, E, nblk_n, out);
  return hipGetLastError();
}

// out[dst(r)] = A[src(r)] W[e] with W [E, K, N] as stored (kmajor.h)
template <bool GATHER, bool SCATTER>
hipError_t launch_dgrad(const bf16_t* A, const int32_t* a_index, const bf16_t* W, const int32_t* offsets,
                        const int32_t* out_index, int S_rows, int K, int N, int E, bf16_t* out, hipStream_t s) {
  if (N % 384 == 0) return launch_dgrad_t<3, GATHER, SCATTER>(A, a_index, W, offsets, out_index, S_rows, K, N, E, out, s);
  if (N % 256 == 0) return launch_dgrad_t<2, GATHER, SCATTER>(A, a_index, W, offsets, out_index, S_rows, K, N, E, out, s);
  return launch_dgrad_t<1, GATHER, SCATTER>(A, a_index, W, offsets, out_index, S_rows, K, N, E, out, s);
}

// dW[e] = P(rows of e)^T Q(rows of e), P [.., N] and Q [.., M] row-major (kmajor.h)
template <int MT, bool GATHER_P, bool GATHER_Q>
hipError_t launch_wgrad_t(const bf16_t* P, const bf16_t* Q, const int32_t* index, const int32_t* offsets, const bf16_t* zrow,
                          int N, int M, int E, int slots, const int* plan, float* part, bf16_t* dW, hipStream_t s) {
  const dim3 block(512);               // (the partial tiles of cut experts are added up by backward_sums_kernel)
  auto grid = [&](int bn) { return dim3((unsigned)((slots * (N / (64 * MT)) * (M / bn) + 7) & ~7)); };
  if (M % 384 == 0)
    hipLaunchKernelGGL((wgrad_kmajor_kernel<MT, 3, GATHER_P, GATHER_Q>), grid(384), block, 0, s, P, Q, index, offsets, zrow, N,
                       M, E, plan, part, dW);
  else if (M % 256 == 0)
    hipLaunchKernelGGL((wgrad_kmajor_kernel<MT, 2, GATHER_P, GATHER_Q>), grid(256), block, 0, s, P, Q, index, offsets, zrow, N,
                       M, E, plan, part, dW);
  else
    hipLaunchKernelGGL((wgrad_kmajor_kernel<MT, 1, GATHER_P, GATHER_Q>), grid(128), block, 0, s, P, Q, index, offsets, zrow, N,
                       M, E, plan, part, dW);
  return hipGetLastError();
}

// 256 rows of dW per workgroup where N allows and the experts have rows enough for the streams to matter
template <bool GATHER_P, bool GATHER_Q>
hipError_t launch_wgrad(const bf16_t* P, const bf16_t* Q, const int32_t* index, const int32_t* offsets, const bf16_t* zrow,
                        int N, int M, int S_rows, int E, int slots, const int* plan, float* part, bf16_t* dW, hipStream_t s) {
  const int bn = M % 384 == 0 ? 384 : (M % 256 == 0 ? 256 : 128);
  if (N % 256 == 0 && tall_tiles(S_rows, E, (long long)E * (N / 128) * (M / bn), (long long)E * (N / 256) * (M / bn)))
    return launch_wgrad_t<4, GATHER_P, GATHER_Q>(P, Q, index, offsets, zrow, N, M, E, slots, plan, part, dW, s);
  return launch_wgrad_t<2, GATHER_P, GATHER_Q>(P, Q, index, offsets, zrow, N, M, E, slots, plan, part, dW, s);
}

// ---- Radial NormSiLU backward (moe.py:87-92), one wave per permuted row ----------------------------------------
// h = r^p a u, a = SiLU(z) = z s, s = sigmoid(z), z = g / r, a' = s (1 + z (1 - s)); with q = dh u:
//   du = dh r^p a;  dg = q r^(p-1) a' + g / (I r) sum_i q_i (p r^(p-1) a_i - r^(p-2) a'_i g_i);
//   dtheta (the row's share) = p'(theta) ln r sum_i q_i r^p a_i;  dw = <dh', h>, dh = w dh'.
// `hidden` receives w h, the row the down projection's weight gradient contracts with d_out.
// act = SiLU: h = SiLU(g) u, dg = q a'(g), no theta.  Rows of I <= kActMaxI elements.
constexpr int kActMaxI = 512;   // one 16-byte granule of the row per lane

__global__ __launch_bounds__(256) void act_bwd_kernel(const bf16_t* __restrict__ gu, const bf16_t* __restrict__ dhp,
                                                      const float* __restrict__ w, const float* __restrict__ theta,
                                                      const int32_t* __restrict__ offsets,
                                                      const int32_t* __restrict__ perm_slot, int S, int E, int I, int act,
                                                      bf16_t* __restrict__ dgu, bf16_t* __restrict__ hidden,
                                                      float* __restrict__ dw_slot, float* __restrict__ dtheta_row,
                                                      uint32_t* __restrict__ zero_words, int n_zero_words,
                                                      int* __restrict__ plan, int n_routed, int chunk, int slots) {
  // (the first workgroup also clears the row of zeros the weight-gradient kernels read past an expert's last row and,
  // with its first wave, lists the row chunks those kernels work through)
  if (blockIdx.x == 0) {
    for (int i = threadIdx.x; i < n_zero_words; i += 256) zero_words[i] = 0u;
    if (threadIdx.x < kWave) wgrad_plan(offsets, n_routed, chunk, slots, plan);
  }
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= S) return;
  // the row's values are requested first: nothing below that decides about the row depends on them
  const bool live = lane * 8 < I;
  bf16x8 gv, uv, dv;
#pragma unroll
  for (int q = 0; q < 8; ++q) gv[q] = uv[q] = dv[q] = (bf16_t)0.f;
  if (live) {
    gv = *reinterpret_cast<const bf16x8*>(gu + (size_t)row * 2 * I + lane * 8);
    uv = *reinterpret_cast<const bf16x8*>(gu + (size_t)row * 2 * I + I + lane * 8);
    dv = *reinterpret_cast<const bf16x8*>(dhp + (size_t)row * I + lane * 8);
  }
  const int slot = perm_slot[row];
  // expert of the row: offsets[e] <= row < offsets[e + 1], one offset per lane (E <= 64) and a ballot
  const int my_off = offsets[min(lane, E)];
  const int end = E < kWave ? __shfl(my_off, E, kWave) : offsets[E];
  if (row >= end) return;                                      // E = GLU experts: rows behind theirs have no activation
  const int e = __popcll(__ballot(lane < E && my_off <= row)) - 1;
  const float ws = w[slot];
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
      oh[q] = (bf16_t)(ws * gain * a_[q] * u[q]);              // w h: the weight gradient's operand (moe.py:92-93)
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

// ---- router backward (router.py:31,41-47) --------------------------------------------------------------------
// Eight lanes per token, lane j < k for slot j: dlogit of the k selected experts from the gradients of the combine
// weights.  The sums over a token's slots are taken in ascending j by every lane, so they are the same bits in all.
__global__ __launch_bounds__(256) void router_bwd_kernel(const float* __restrict__ logits, const int32_t* __restrict__ idx,
                                                         const float* __restrict__ w, const float* __restrict__ dw, int T,
                                                         int E, int k, int norm_mode, float* __restrict__ dl) {
  static_assert(kMaxK <= 8, "eight lanes per token");
  const int gid = blockIdx.x * blockDim.x + threadIdx.x;
  const int t = gid >> 3, j = gid & 7;
  const bool live = t < T && j < k;
  float sj = 0.f, dwj = 0.f, wj = 0.f;
  if (live) {
    sj = 1.f / (1.f + __expf(-logits[(size_t)t * E + idx[t * k + j]]));
    dwj = dw[t * k + j];
    wj = w[t * k + j];
  }
  const int base = (threadIdx.x & 63) & ~7;
  float sum = 0.f, dot = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float si = __shfl(sj, base + i, kWave), di = __shfl(dwj, base + i, kWave), wi = __shfl(wj, base + i, kWave);
    if (i < k) {
      sum += si;
      dot = fmaf(di, wi, dot);
    }
  }
  if (!live) return;
  float ds = dwj;
  if (k > 1 && norm_mode == BIBO_NORM_SUM) ds = (ds - dot) / (sum + 1e-20f);
  else if (k > 1 && norm_mode == BIBO_NORM_SOFTMAX) ds = wj * (ds - dot);
  dl[t * k + j] = ds * sj * (1.f - sj);
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
// (H / 256, chunks, kDwrSplit): block (., g, z) takes the z-th of kDwrSplit equal row ranges of row chunk g of the plan
// (kmajor.h: an expert's rows, cut where an expert holds many); thread (rl = t / 32, cg = t % 32) adds up rows rl,
// rl + 8, .. of the range for columns 8 cg .. + 8 of the block's 256, the eight partial sums meet in LDS in a fixed
// order -> part[g][z][c] fp32.  Step 2 adds the ranges of an expert's chunks in order.
constexpr int kDwrSplit = 8;

__global__ __launch_bounds__(256) void dwr_partial_kernel(const bf16_t* __restrict__ x, const float* __restrict__ dl,
                                                          const int* __restrict__ plan,
                                                          const int32_t* __restrict__ perm_slot,
                                                          const int32_t* __restrict__ perm_token, int H,
                                                          float* __restrict__ part) {
  __shared__ float red[8][256];
  const int g = blockIdx.y, z = blockIdx.z, cg = threadIdx.x & 31, rl = threadIdx.x >> 5;
  if (g >= plan[0]) return;
  const int c = blockIdx.x * 256 + cg * 8;
  const int lo_e = plan[4 + 4 * g + 1], n = plan[4 + 4 * g + 2] - lo_e;
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
    part[((size_t)g * kDwrSplit + z) * H + col] =
        ((red[0][t] + red[1][t]) + (red[2][t] + red[3][t])) + ((red[4][t] + red[5][t]) + (red[6][t] + red[7][t]));
  }
}

// The last launch of the backward pass: every sum that ends one, by ranges of workgroups.
//   [0, nb_w): the partial tiles of the experts that were cut into chunks (kmajor.h) -> dW_down, dW_gate_up;
//   [nb_w, nb_w + E): dtheta[e] = the sum of the theta shares of expert e's rows, chunk by chunk of the plan and the
//     chunks in order (no atomics: the same bits on every call);
//   from nb_w + E on (when dwr != nullptr): the router's weight gradient [Et, H] = the sum over an expert's chunks
//     of dwr_partial_kernel's partial rows.
__global__ __launch_bounds__(256) void backward_sums_kernel(int nb_w, const float* __restrict__ part_a,
                                                            const float* __restrict__ part_b, const int* __restrict__ plan,
                                                            int slots, int NMa, int NMb, int E, int Et,
                                                            bf16_t* __restrict__ dWa, bf16_t* __restrict__ dWb,
                                                            const float* __restrict__ dtheta_row, float* __restrict__ dtheta,
                                                            const float* __restrict__ dwr_part, int H,
                                                            bf16_t* __restrict__ dwr) {
  const int block = blockIdx.x;
  if (block < nb_w) {
    wgrad_reduce_block(block, part_a, part_b, plan, slots, NMa, NMb, E, dWa, dWb);
    return;
  }
  const int* experts = plan + 4 + 4 * (slots + Et);            // {first chunk, chunks, ., .} per expert
  if (block < nb_w + E) {
    __shared__ float red[4];
    const int e = block - nb_w;
    const int first = experts[4 * e], chunks = experts[4 * e + 1];
    float total = 0.f;
    for (int c = 0; c < chunks; ++c) {
      const int* entry = plan + 4 + 4 * (first + c);
      float acc = 0.f;
      for (int r = entry[1] + threadIdx.x; r < entry[2]; r += 256) acc += dtheta_row[r];
      acc = wave_sum(acc);
      __syncthreads();
      if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;
      __syncthreads();
      total += (red[0] + red[1]) + (red[2] + red[3]);
    }
    if (threadIdx.x == 0) dtheta[e] = total;
    return;
  }
  if (dwr == nullptr) return;
  const int i = (block - nb_w - E) * 256 + threadIdx.x;         // element of [Et, H]
  if (i >= Et * H) return;
  const int e = i / H, c = i - e * H;
  const int first = experts[4 * e], chunks = experts[4 * e + 1];
  float acc = 0.f;
  for (int j = 0; j < chunks * kDwrSplit; ++j) acc += dwr_part[((size_t)first * kDwrSplit + j) * H + c];
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

// a row of zeros as wide as the widest weight-gradient operand: what a K stage reads past an expert's last row
// The sums over an expert's rows (weight-gradient GEMMs, router weight gradient, theta gradient) cut an expert with more
// rows than this into chunks (kmajor.h): one and a half times the average over all E routed experts, so that evenly
// routed tokens leave every expert in one piece, and at least 512.
int backward_chunk_rows(int S_rows, int E) {
  const long long c = (3ll * S_rows / (2ll * E) + 31) & ~31ll;
  return (int)(c < 512 ? 512 : c);
}
// chunks over all experts, at most
int backward_chunk_slots(int S_rows, int E) { return S_rows / backward_chunk_rows(S_rows, E) + E; }
// fp32 partial tiles of the cut experts, dW_down's and dW_gate_up's, one slot per chunk each
size_t backward_wgrad_part_bytes(int S_rows, int H, int E, int I) {
  return (size_t)backward_chunk_slots(S_rows, E) * 3 * I * H * sizeof(float);
}
// the list of chunks (kmajor.h: WgradPlan): a header, a 16-byte entry per chunk and two per expert
size_t backward_plan_bytes(int S_rows, int E) { return 16 + (size_t)(backward_chunk_slots(S_rows, E) + 2 * E) * 16; }

size_t backward_zero_row_bytes(int H, int I) { return (size_t)(H > 2 * I ? H : 2 * I) * sizeof(bf16_t); }

// The launches after routing and permutation.  Buffers (bf16 unless noted): gu [S,2I], dhp [S,I], dgu [S,2I],
// hidden [S,I], dxs [S,H], zrow [max(H, 2I)] (cleared by act_bwd_kernel), dw_slot [S] f32, dl [S] f32, dtheta_row [S] f32,
// dwr_part [backward_chunk_slots(), backward_dwr_split(), H] f32.
hipError_t launch_backward(const void* x, const void* d_out, const void* w_router, const void* wgu, const void* wd,
                           const float* theta, const float* logits, const int32_t* idx, const float* w,
                           const int32_t* offsets, const int32_t* perm_slot, const int32_t* perm_token, int T, int H, int E,
                           int n_pos, int n_neg, int k, int I, int norm_mode, int act, const BackwardBuffers& b, void* dx,
                           void* d_w_router, void* d_wgu, void* d_wd, float* d_theta, hipStream_t s, const void* gu_saved) {
  // E = GLU experts (with weights); the router and the permutation know Et experts, the +/-Identity ones last
  const int Et = E + n_pos + n_neg;
  const int S = T * k;
  const int slots = backward_chunk_slots(S, Et);      // row chunks of the plan, at most
  const bf16_t* xp = static_cast<const bf16_t*>(x);
  const bf16_t* dop = static_cast<const bf16_t*>(d_out);
  const bf16_t* wrp = static_cast<const bf16_t*>(w_router);
  const bf16_t* wgup = static_cast<const bf16_t*>(wgu);
  const bf16_t* wdp = static_cast<const bf16_t*>(wd);
  // the pre-activations: a training forward's, or recomputed below into the workspace
  const bf16_t* gu = gu_saved != nullptr ? static_cast<const bf16_t*>(gu_saved) : static_cast<const bf16_t*>(b.gu);
  bf16_t* dhp = static_cast<bf16_t*>(b.dhp);
  bf16_t* dgu = static_cast<bf16_t*>(b.dgu);
  bf16_t* hidden = static_cast<bf16_t*>(b.hidden);
  bf16_t* dxs = static_cast<bf16_t*>(b.dxs);
  bf16_t* zrow = static_cast<bf16_t*>(b.zrow);
  hipError_t err = hipSuccess;
  if (S == 0) {
    zero_bytes(d_theta, (size_t)E * sizeof(float), s);
    if (d_w_router != nullptr) zero_bytes(d_w_router, (size_t)Et * H * sizeof(bf16_t), s);
    zero_bytes(d_wgu, (size_t)E * 2 * I * H * sizeof(bf16_t), s);
    zero_bytes(d_wd, (size_t)E * H * I * sizeof(bf16_t), s);
    return hipGetLastError();
  }
  // pre-activations again (moe.py:84): x W_gate_up^T, both contiguous along H - by the first phase of the forward
  // pass's fused kernel where it takes the shape (its ring of weight stages is the faster main loop)
  if (gu_saved != nullptr)
    err = hipSuccess;
  else if (fused_supported(H, I, BIBO_DTYPE_BF16) && (long long)T * H < (1LL << 31))
    err = launch_gateup_raw(xp, wgup, offsets, perm_token, T, H, E, k, I, b.gu, s);
  else
    err = launch_ggemm<true, false>(xp, perm_token, wgup, offsets, nullptr, S, H, 2 * I, E, static_cast<bf16_t*>(b.gu), s);
  if (err != hipSuccess) return err;
  // dh' = d W_down: contracts over H, the middle dimension of w_down [E, H, I]
  err = launch_dgrad<true, false>(dop, perm_token, wdp, offsets, nullptr, S, H, I, E, dhp, s);
  if (err != hipSuccess) return err;
  hipLaunchKernelGGL(act_bwd_kernel, dim3((S + 3) / 4), dim3(256), 0, s, gu, dhp, w, theta, offsets, perm_slot, S, E, I, act,
                     dgu, hidden, b.dw_slot, b.dtheta_row, reinterpret_cast<uint32_t*>(zrow),
                     (int)(backward_zero_row_bytes(H, I) / 4), b.wgrad_plan, Et, backward_chunk_rows(S, Et), slots);
  // dx of every slot, in slot order: [dg, du] W_gate_up, contracts over the 2I rows of w_gate_up [E, 2I, H]
  err = launch_dgrad<false, true>(dgu, nullptr, wgup, offsets, perm_slot, S, 2 * I, H, E, dxs, s);
  if (err != hipSuccess) return err;
  if (n_pos + n_neg > 0)   // (as many waves as there could be rows: how many there are is only known on the device)
    hipLaunchKernelGGL(special_bwd_kernel, dim3((S + 3) / 4), dim3(256), 0, s, xp, dop, w, offsets, perm_slot, perm_token, E,
                       n_pos, n_neg, H, b.dw_slot, dxs);
  const bool with_router = w_router != nullptr;      // else: the experts alone, the caller owns the routing
  if (with_router)
    hipLaunchKernelGGL(router_bwd_kernel, dim3((T + 31) / 32), dim3(256), 0, s, logits, idx, w, b.dw_slot, T, Et, k, norm_mode,
                       b.dl);
  hipLaunchKernelGGL(dx_combine_kernel, dim3((unsigned)(((long long)T * (H / 8) + 255) / 256)), dim3(256), 0, s, dxs,
                     with_router ? b.dl : nullptr, idx, wrp, T, H, k, Et, b.dw_slot, static_cast<bf16_t*>(dx));
  if (with_router)
    hipLaunchKernelGGL(dwr_partial_kernel, dim3((H + 255) / 256, slots, kDwrSplit), dim3(256), 0, s, xp, b.dl, b.wgrad_plan,
                       perm_slot, perm_token, H, b.dwr_part);
  // weight gradients, contracted over each expert's rows: dW_down[e] = d^T (w h) (d gathered by token, `hidden`
  // already carries w), dW_gate_up[e] = [dg, du]^T x (x gathered by token)
  err = launch_wgrad<true, false>(dop, hidden, perm_token, offsets, zrow, H, I, S, E, slots, b.wgrad_plan, b.wgrad_part, static_cast<bf16_t*>(d_wd), s);
  if (err != hipSuccess) return err;
  float* part_gu = b.wgrad_part + (size_t)slots * H * I;
  err = launch_wgrad<false, true>(dgu, xp, perm_token, offsets, zrow, 2 * I, H, S, E, slots, b.wgrad_plan, part_gu, static_cast<bf16_t*>(d_wgu), s);
  if (err != hipSuccess) return err;
  // the sums that end the pass: cut experts' partial tiles, dtheta, the router's weight gradient
  const int nb_w = (int)(((size_t)2 * I * H / 4 + 255) / 256);
  const int nb_r = with_router ? (Et * H + 255) / 256 : 0;
  hipLaunchKernelGGL(backward_sums_kernel, dim3(nb_w + E + nb_r), dim3(256), 0, s, nb_w, b.wgrad_part, part_gu, b.wgrad_plan,
                     slots, H * I, 2 * I * H, E, Et, static_cast<bf16_t*>(d_wd), static_cast<bf16_t*>(d_wgu), b.dtheta_row,
                     d_theta, b.dwr_part, H, with_router ? static_cast<bf16_t*>(d_w_router) : nullptr);
  return hipGetLastError();
}

}  // namespace bibo
