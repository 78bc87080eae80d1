// Generic backward pass of the sparse-MoE block: any hidden and expert size, bf16 or fp32 operands, fp32 arithmetic.
// It serves what the MFMA backward (backward.hip) does not take: fp32 modules (the reference's own tests take their
// gradients in fp32 at tiny sizes, tests/test_moe.py:53-63, ablate/common/test_eager_radial.py:63-69) and sizes that
// are no multiples of 128.  The gradients are those torch.autograd derives for the eager layer
// (src/modeling/ffn/moe.py:46-101,157-183, src/modeling/ffn/router.py:25-47) with the selection held fixed; the
// formulas are the ones spelled out at the top of backward.hip.  One workgroup per routed row for the row-wise part,
// one workgroup per weight row for the weight gradients, which loop over an expert's rows in permuted order: every sum
// has a fixed order, so the results are the same bits on every call.
#include "common.h"

namespace bibo {
namespace {

__device__ __forceinline__ float block_sum(float v, float* red) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  v = wave_sum(v);
  __syncthreads();                                   // red may still be read from the sum before
  if (lane == 0) red[wave] = v;
  __syncthreads();
  return ((red[0] + red[1]) + red[2]) + red[3];
}

// Per routed row of a GLU expert (permuted row `row`, token t, slot s, expert e, combine weight w):
//   gu = W_gate_up[e] x_t;  dh' = W_down[e]^T d_t;  dw[s] = <dh', h>;  (dg, du, dtheta share) from dh = w dh';
//   dgu[row] = [dg, du];  hw[row] = w h;  dxs[s] = W_gate_up[e]^T [dg, du].
// Dynamic LDS: 2H + 5I floats.
template <typename TIn>
__global__ __launch_bounds__(256) void row_bwd_generic_kernel(const TIn* __restrict__ x, const TIn* __restrict__ d_out,
                                                              const TIn* __restrict__ wgu, const TIn* __restrict__ wd,
                                                              const float* __restrict__ theta, const float* __restrict__ w,
                                                              const int32_t* __restrict__ offsets,
                                                              const int32_t* __restrict__ perm_slot,
                                                              const int32_t* __restrict__ perm_token, int H, int E, int I,
                                                              int act, float* __restrict__ dgu, float* __restrict__ hw,
                                                              float* __restrict__ dxs, float* __restrict__ dw_slot,
                                                              float* __restrict__ dtheta_row) {
  extern __shared__ float smem[];
  float* xs = smem;                 // [H]
  float* ds = xs + H;               // [H]
  float* gu = ds + H;               // [2I]
  float* dhp = gu + 2 * I;          // [I]
  float* dg = dhp + I;              // [2I]  dg, then du
  __shared__ int sh_e;
  __shared__ float red[4];
  const int row = blockIdx.x;
  if (row >= offsets[E]) return;                     // E = GLU experts: rows behind theirs have no activation
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  if (tid < E && offsets[tid] <= row && row < offsets[tid + 1]) sh_e = tid;
  const int slot = perm_slot[row];
  const size_t t = (size_t)perm_token[row];
  for (int h = tid; h < H; h += 256) {
    xs[h] = to_float(x[t * H + h]);
    ds[h] = to_float(d_out[t * H + h]);
  }
  __syncthreads();
  const int e = sh_e;
  const float ws = w[slot];
  const TIn* wg = wgu + (size_t)e * 2 * I * H;
  const TIn* wdn = wd + (size_t)e * H * I;
  for (int c = wave; c < 2 * I; c += 4) {            // pre-activations (moe.py:84): one wave per weight row
    const TIn* wrow = wg + (size_t)c * H;
    float acc = 0.f;
    for (int h = lane; h < H; h += kWave) acc = fmaf(xs[h], to_float(wrow[h]), acc);
    acc = wave_sum(acc);
    if (lane == 0) gu[c] = acc;
  }
  for (int i = tid; i < I; i += 256) {               // dh' = W_down^T d: a thread per column, coalesced over i
    float acc = 0.f;
    for (int h = 0; h < H; ++h) acc = fmaf(ds[h], to_float(wdn[(size_t)h * I + i]), acc);
    dhp[i] = acc;
  }
  __syncthreads();
  float ss = 0.f;
  for (int i = tid; i < I; i += 256) ss = fmaf(gu[i], gu[i], ss);
  ss = block_sum(ss, red);
  const bool radial = act != BIBO_ACT_SILU;
  float p = 0.f, r = 1.f, gain = 1.f;
  if (radial) {
    p = radial_exponent(theta, e, act);
    r = sqrtf(ss / (float)I + kNormSiluEps);         // moe.py:88
    gain = powf(r, p);
  }
  const float rinv = 1.f / r;
  // h = r^p a u, a = z s, s = sigmoid(z), z = g / r, a' = s (1 + z (1 - s)); q = w dh' u
  float dot_h = 0.f, sum_qa = 0.f, inner = 0.f;
  for (int i = tid; i < I; i += 256) {
    const float z = gu[i] * rinv, s = 1.f / (1.f + expf(-z));
    const float a = z * s, ad = s * (1.f + z * (1.f - s));
    const float u = gu[I + i];
    dot_h = fmaf(dhp[i], gain * a * u, dot_h);
    const float q = ws * dhp[i] * u;
    sum_qa = fmaf(q, a, sum_qa);
    inner = fmaf(q, gain * rinv * (p * a - ad * z), inner);
  }
  dot_h = block_sum(dot_h, red);
  sum_qa = block_sum(sum_qa, red);
  inner = block_sum(inner, red);
  for (int i = tid; i < I; i += 256) {
    const float z = gu[i] * rinv, s = 1.f / (1.f + expf(-z));
    const float a = z * s, ad = s * (1.f + z * (1.f - s));
    const float u = gu[I + i], dh = ws * dhp[i];
    float g_ = dh * u * gain * rinv * ad;
    if (radial) g_ = fmaf(gu[i] * rinv / (float)I, inner, g_);
    const float u_ = dh * gain * a;
    dg[i] = g_;
    dg[I + i] = u_;
    dgu[(size_t)row * 2 * I + i] = g_;
    dgu[(size_t)row * 2 * I + I + i] = u_;
    hw[(size_t)row * I + i] = ws * gain * a * u;
  }
  if (tid == 0) {
    dw_slot[slot] = dot_h;
    const float dp = act == BIBO_ACT_RADIAL_TANH ? 1.f - p * p : p * (1.f - p);
    dtheta_row[row] = radial ? dp * logf(r) * gain * sum_qa : 0.f;
  }
  __syncthreads();
  for (int h = tid; h < H; h += 256) {               // dx of the slot: a thread per column, coalesced over h
    float acc = 0.f;
    for (int c = 0; c < 2 * I; ++c) acc = fmaf(dg[c], to_float(wg[(size_t)c * H + h]), acc);
    dxs[(size_t)slot * H + h] = acc;
  }
}

// +/-Identity experts (moe.py:95-99): dw[slot] = sign <d_out[t], x[t]>, dxs[slot] = sign w[slot] d_out[t].  One
// workgroup per permuted row behind the GLU experts' rows.
template <typename TIn>
__global__ __launch_bounds__(256) void special_bwd_generic_kernel(const TIn* __restrict__ x, const TIn* __restrict__ d_out,
                                                                  const float* __restrict__ w,
                                                                  const int32_t* __restrict__ offsets,
                                                                  const int32_t* __restrict__ perm_slot,
                                                                  const int32_t* __restrict__ perm_token, int Eg, int n_pos,
                                                                  int n_neg, int H, float* __restrict__ dw_slot,
                                                                  float* __restrict__ dxs) {
  __shared__ float red[4];
  const int row = offsets[Eg] + blockIdx.x;
  if (row >= offsets[Eg + n_pos + n_neg]) return;
  const float sign = row < offsets[Eg + n_pos] ? 1.f : -1.f;
  const int slot = perm_slot[row];
  const size_t t = (size_t)perm_token[row];
  const float sw = sign * w[slot];
  float dot = 0.f;
  for (int h = threadIdx.x; h < H; h += 256) {
    const float dv = to_float(d_out[t * H + h]);
    dot = fmaf(dv, to_float(x[t * H + h]), dot);
    dxs[(size_t)slot * H + h] = sw * dv;
  }
  dot = block_sum(dot, red);
  if (threadIdx.x == 0) dw_slot[slot] = sign * dot;
}

// dtheta[e] = sum of its rows' contributions, in row order
__global__ __launch_bounds__(256) void dtheta_generic_kernel(const float* __restrict__ dtheta_row,
                                                             const int32_t* __restrict__ offsets,
                                                             float* __restrict__ dtheta) {
  __shared__ float red[4];
  const int e = blockIdx.x;
  float acc = 0.f;
  for (int r = offsets[e] + threadIdx.x; r < offsets[e + 1]; r += 256) acc += dtheta_row[r];
  acc = block_sum(acc, red);
  if (threadIdx.x == 0) dtheta[e] = acc;
}

// One thread per token: dlogit of the k selected experts from the gradients of the combine weights (router.py:31,41-47).
__global__ void router_bwd_generic_kernel(const float* __restrict__ logits, const int32_t* __restrict__ idx,
                                          const float* __restrict__ w, const float* __restrict__ dw, int T, int E, int k,
                                          int norm_mode, float* __restrict__ dl) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  float s[kMaxK], sum = 0.f, dot = 0.f;
  for (int j = 0; j < k; ++j) {
    s[j] = 1.f / (1.f + expf(-logits[(size_t)t * E + idx[t * k + j]]));
    sum += s[j];
    dot = fmaf(dw[t * k + j], w[t * k + j], dot);
  }
  for (int j = 0; j < k; ++j) {
    float dsc = dw[t * k + j];
    if (k > 1 && norm_mode == BIBO_NORM_SUM) dsc = (dsc - dot) / (sum + 1e-20f);
    else if (k > 1 && norm_mode == BIBO_NORM_SOFTMAX) dsc = w[t * k + j] * (dsc - dot);
    dl[t * k + j] = dsc * s[j] * (1.f - s[j]);
  }
}

// dx[t, h] = sum_j dxs[t k + j, h] + sum_j dl[t, j] W_router[idx[t, j], h].  dl == NULL: the slot rows alone.  A slot
// whose expert id lies outside [0, n_experts) has no dxs row: left out, and its dw_slot entry is set to zero.
template <typename TIn>
__global__ __launch_bounds__(256) void dx_combine_generic_kernel(const float* __restrict__ dxs, const float* __restrict__ dl,
                                                                 const int32_t* __restrict__ idx,
                                                                 const TIn* __restrict__ w_router, int T, int H, int k,
                                                                 int n_experts, float* __restrict__ dw_slot,
                                                                 TIn* __restrict__ dx) {
  const long long gid = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= (long long)T * H) return;
  const int t = (int)(gid / H), h = (int)(gid - (long long)t * H);
  float acc = 0.f;
  for (int j = 0; j < k; ++j) {
    const int e = idx[t * k + j];
    if (e < 0 || e >= n_experts) {
      if (h == 0) dw_slot[t * k + j] = 0.f;
      continue;
    }
    acc += dxs[((size_t)t * k + j) * H + h];
    if (dl != nullptr) acc = fmaf(dl[t * k + j], to_float(w_router[(size_t)e * H + h]), acc);
  }
  dx[(size_t)t * H + h] = from_float<TIn>(acc);
}

// dW[e][n][m] = sum over the rows r of expert e, in row order, of P[srcP(r)][n] Q[srcQ(r)][m]; grid = (N, E), threads
// over m.  srcP(r) = index[r] (GATHER_P) or r, likewise Q.  P and Q may be fp32 workspace rows or operands.
template <typename TP, typename TQ, typename TOut, bool GATHER_P, bool GATHER_Q>
__global__ __launch_bounds__(256) void wgrad_generic_kernel(const TP* __restrict__ P, const TQ* __restrict__ Q,
                                                            const int32_t* __restrict__ index,
                                                            const int32_t* __restrict__ offsets, int N, int M,
                                                            TOut* __restrict__ dW) {
  const int n = blockIdx.x, e = blockIdx.y;
  const int lo = offsets[e], hi = offsets[e + 1];
  for (int m0 = 0; m0 < M; m0 += 256) {
    const int m = m0 + threadIdx.x;
    float acc = 0.f;
    for (int r = lo; r < hi; ++r) {
      const int ix = (GATHER_P || GATHER_Q) ? index[r] : 0;
      const float pv = to_float(P[(size_t)(GATHER_P ? ix : r) * N + n]);
      if (m < M) acc = fmaf(pv, to_float(Q[(size_t)(GATHER_Q ? ix : r) * M + m]), acc);
    }
    if (m < M) dW[((size_t)e * N + n) * M + m] = from_float<TOut>(acc);
  }
}

// dW_router[e, h] = sum over the rows r of expert e, in row order, of dl[slot(r)] x[token(r), h]; grid = E.
template <typename TIn>
__global__ __launch_bounds__(256) void dwr_generic_kernel(const TIn* __restrict__ x, const float* __restrict__ dl,
                                                          const int32_t* __restrict__ offsets,
                                                          const int32_t* __restrict__ perm_slot,
                                                          const int32_t* __restrict__ perm_token, int H,
                                                          TIn* __restrict__ dwr) {
  const int e = blockIdx.x;
  const int lo = offsets[e], hi = offsets[e + 1];
  for (int h = threadIdx.x; h < H; h += 256) {
    float acc = 0.f;
    for (int r = lo; r < hi; ++r) acc = fmaf(dl[perm_slot[r]], to_float(x[(size_t)perm_token[r] * H + h]), acc);
    dwr[(size_t)e * H + h] = from_float<TIn>(acc);
  }
}

template <typename TIn>
__global__ void zero_generic_kernel(TIn* __restrict__ p, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
    p[i] = from_float<TIn>(0.f);
}

template <typename TIn>
void zero_elems(TIn* p, size_t n, hipStream_t s) {
  if (n == 0) return;
  const unsigned grid = (unsigned)((n + 255) / 256 < 2048 ? (n + 255) / 256 : 2048);
  hipLaunchKernelGGL(zero_generic_kernel<TIn>, dim3(grid), dim3(256), 0, s, p, n);
}

template <typename TIn>
hipError_t launch_t(const void* x_, const void* d_out_, const void* w_router_, const void* wgu_, const void* wd_,
                    const float* theta, const float* logits, const int32_t* idx, const float* w, const int32_t* offsets,
                    const int32_t* perm_slot, const int32_t* perm_token, int T, int H, int E, int n_pos, int n_neg, int k, int I,
                    int norm_mode, int act, const GenericBackwardBuffers& b, void* dx_, void* d_w_router_, void* d_wgu_,
                    void* d_wd_, float* d_theta, hipStream_t s) {
  const TIn* x = static_cast<const TIn*>(x_);
  const TIn* d_out = static_cast<const TIn*>(d_out_);
  const TIn* w_router = static_cast<const TIn*>(w_router_);
  const TIn* wgu = static_cast<const TIn*>(wgu_);
  const TIn* wd = static_cast<const TIn*>(wd_);
  const int Et = E + n_pos + n_neg, S = T * k;
  if (S == 0) {
    zero_elems(d_theta, (size_t)E, s);
    if (d_w_router_ != nullptr) zero_elems(static_cast<TIn*>(d_w_router_), (size_t)Et * H, s);
    zero_elems(static_cast<TIn*>(d_wgu_), (size_t)E * 2 * I * H, s);
    zero_elems(static_cast<TIn*>(d_wd_), (size_t)E * H * I, s);
    return hipGetLastError();
  }
  const size_t shm = (size_t)(2 * H + 5 * I) * sizeof(float);
  hipLaunchKernelGGL(row_bwd_generic_kernel<TIn>, dim3(S), dim3(256), shm, s, x, d_out, wgu, wd, theta, w, offsets, perm_slot,
                     perm_token, H, E, I, act, b.dgu, b.hw, b.dxs, b.dw_slot, b.dtheta_row);
  hipLaunchKernelGGL(dtheta_generic_kernel, dim3(E), dim3(256), 0, s, b.dtheta_row, offsets, d_theta);
  if (n_pos + n_neg > 0)   // (as many workgroups as there could be rows: how many there are is only known on the device)
    hipLaunchKernelGGL(special_bwd_generic_kernel<TIn>, dim3(S), dim3(256), 0, s, x, d_out, w, offsets, perm_slot, perm_token, E,
                       n_pos, n_neg, H, b.dw_slot, b.dxs);
  const bool with_router = w_router != nullptr;      // else: the experts alone, the caller owns the routing
  if (with_router)
    hipLaunchKernelGGL(router_bwd_generic_kernel, dim3((T + 255) / 256), dim3(256), 0, s, logits, idx, w, b.dw_slot, T, Et, k,
                       norm_mode, b.dl);
  hipLaunchKernelGGL(dx_combine_generic_kernel<TIn>, dim3((unsigned)(((long long)T * H + 255) / 256)), dim3(256), 0, s, b.dxs,
                     with_router ? b.dl : nullptr, idx, w_router, T, H, k, Et, b.dw_slot, static_cast<TIn*>(dx_));
  if (with_router)
    hipLaunchKernelGGL(dwr_generic_kernel<TIn>, dim3(Et), dim3(256), 0, s, x, b.dl, offsets, perm_slot, perm_token, H,
                       static_cast<TIn*>(d_w_router_));
  // dW_down[e] = d^T (w h), d gathered by token; dW_gate_up[e] = [dg, du]^T x, x gathered by token
  hipLaunchKernelGGL((wgrad_generic_kernel<TIn, float, TIn, true, false>), dim3(H, E), dim3(256), 0, s, d_out, b.hw, perm_token,
                     offsets, H, I, static_cast<TIn*>(d_wd_));
  hipLaunchKernelGGL((wgrad_generic_kernel<float, TIn, TIn, false, true>), dim3(2 * I, E), dim3(256), 0, s, b.dgu, x, perm_token,
                     offsets, 2 * I, H, static_cast<TIn*>(d_wgu_));
  return hipGetLastError();
}

}  // namespace

// the row kernel keeps 2H + 5I floats of a row in dynamic LDS next to a few words of its own; 64 KB per workgroup
// need no raised limit
bool backward_generic_supported(int H, int I, int k) {
  return (size_t)(2 * H + 5 * I) * sizeof(float) + 64 <= 64 * 1024 && k <= kMaxK;
}

// Buffers (fp32): dgu [S,2I], hw [S,I], dxs [S,H], dw_slot [S], dl [S], dtheta_row [S].
hipError_t launch_backward_generic(const void* x, const void* d_out, const void* w_router, const void* wgu, const void* wd,
                                   const float* theta, const float* logits, const int32_t* idx, const float* w,
                                   const int32_t* offsets, const int32_t* perm_slot, const int32_t* perm_token, int T, int H,
                                   int E, int n_pos, int n_neg, int k, int I, int dtype, int norm_mode, int act,
                                   const GenericBackwardBuffers& b, void* dx, void* d_w_router, void* d_wgu, void* d_wd,
                                   float* d_theta, hipStream_t s) {
  if (dtype == BIBO_DTYPE_BF16)
    return launch_t<bf16_t>(x, d_out, w_router, wgu, wd, theta, logits, idx, w, offsets, perm_slot, perm_token, T, H, E, n_pos,
                            n_neg, k, I, norm_mode, act, b, dx, d_w_router, d_wgu, d_wd, d_theta, s);
  return launch_t<float>(x, d_out, w_router, wgu, wd, theta, logits, idx, w, offsets, perm_slot, perm_token, T, H, E, n_pos,
                         n_neg, k, I, norm_mode, act, b, dx, d_w_router, d_wgu, d_wd, d_theta, s);
}

}  // namespace bibo
