// Shared device helpers and host-side launcher declarations for the BiBo MoE kernels (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>

#include "../../include/bibo_moe.h"

namespace bibo {

constexpr int kWave = 64;
constexpr int kMaxE = BIBO_MOE_MAX_EXPERTS;
constexpr int kMaxK = BIBO_MOE_MAX_TOPK;
constexpr float kNormSiluEps = 1e-6f;   // src/modeling/ffn/moe.py:16
constexpr float kSumNormEps = 1e-20f;   // src/modeling/ffn/router.py:45

// tokens handled by one workgroup of the histogram / permutation kernels
constexpr int kPermTokens = 128;   // tokens per permutation workgroup (256 and 64 measured slower)
constexpr int kStreamMaxSlots = 4096;   // routed slots the weight-streaming kernels can scan per workgroup
constexpr int kStreamMaxRows = 2048;    // rows (= tokens) one expert can get in them

typedef __bf16 bf16_t;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16_t v) { return (float)v; }
template <typename T> __device__ __forceinline__ T from_float(float v);
template <> __device__ __forceinline__ float from_float<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_float<bf16_t>(float v) { return (bf16_t)v; }

__device__ __forceinline__ int lane_id() { return threadIdx.x & (kWave - 1); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}

__device__ __forceinline__ int wave_inclusive_scan(int v) {
  const int lane = lane_id();
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    int u = __shfl_up(v, o, kWave);
    if (lane >= o) v += u;
  }
  return v;
}

// Routing sigmoid: float32(1 / (1 + exp64(-x))) with exp64 a fixed sequence of IEEE double
// multiplies and adds (never fused), so that every platform produces the same bits.
//   y = clamp(-x, -200, 200); n = floor(y*log2e + 0.5); r = (y - n*LN2_HI) - n*LN2_LO;
//   p = Horner over 1/13! .. 1/0!; e = p * 2^n.
// Reference operation: torch.sigmoid on the fp32 logits, src/modeling/ffn/router.py:31.
__device__ __forceinline__ float sigmoid32_canonical(float x) {
#pragma clang fp contract(off)
  double y = -(double)x;
  y = fmin(fmax(y, -200.0), 200.0);
  const double t = y * 1.4426950408889634;
  const double n = floor(t + 0.5);
  double r = y - n * 0.693147180369123816490;
  r = r - n * 1.90821492927058770002e-10;
  double p = 1.0 / 6227020800.0;
  p = p * r; p = p + 1.0 / 479001600.0;
  p = p * r; p = p + 1.0 / 39916800.0;
  p = p * r; p = p + 1.0 / 3628800.0;
  p = p * r; p = p + 1.0 / 362880.0;
  p = p * r; p = p + 1.0 / 40320.0;
  p = p * r; p = p + 1.0 / 5040.0;
  p = p * r; p = p + 1.0 / 720.0;
  p = p * r; p = p + 1.0 / 120.0;
  p = p * r; p = p + 1.0 / 24.0;
  p = p * r; p = p + 1.0 / 6.0;
  p = p * r; p = p + 0.5;
  p = p * r; p = p + 1.0;
  p = p * r; p = p + 1.0;
  const long long bits = ((long long)((int)n + 1023)) << 52;
  const double e = p * __longlong_as_double(bits);
  const double d = 1.0 + e;
  return (float)(1.0 / d);
}

// Exponent p of the radial gain r^p for expert activation `act` (enum bibo_act): sigmoid(theta) as the
// reference module computes it (src/modeling/ffn/moe.py:89) or tanh(theta) (act code 10 of
// ablate/common/patches.py:53-61).  Plain SwiGLU has no gain: callers set r = 1 and never read theta.
__device__ __forceinline__ float radial_exponent(const float* __restrict__ theta, int e, int act) {
  if (act == BIBO_ACT_SILU) return 0.f;
  const float t = theta[e];
  return act == BIBO_ACT_RADIAL_TANH ? tanhf(t) : 1.f / (1.f + expf(-t));
}

// (1/r, r^p) of a row from its sum of squared gate values: r^2 = sum / I + eps (moe.py:88); plain SwiGLU: (1, 1).
__device__ __forceinline__ void radial_row_scalars(float sum_sq, int I, float p, int act, float& rinv, float& gain) {
  if (act == BIBO_ACT_SILU) { rinv = 1.f; gain = 1.f; return; }
  const float r2 = sum_sq * (1.f / (float)I) + kNormSiluEps;
  rinv = __builtin_amdgcn_rsqf(r2);
  gain = __builtin_amdgcn_exp2f(0.5f * p * __builtin_amdgcn_logf(r2));       // r^p = 2^(p/2 * log2 r^2)
}

// Ballot ranking of 64 consecutive slots.  `peers` = lanes whose slot has my expert, `mine` = lanes whose
// slot has the expert whose id is my lane id.
__device__ __forceinline__ void match64(int e, bool valid, int lane, unsigned long long& peers,
                                        unsigned long long& mine) {
  const unsigned long long vmask = __ballot(valid);
  peers = vmask;
  mine = vmask;
#pragma unroll
  for (int bit = 0; bit < 6; ++bit) {
    const unsigned long long bb = __ballot(valid && ((e >> bit) & 1));
    peers &= ((e >> bit) & 1) ? bb : ~bb;
    mine &= ((lane >> bit) & 1) ? bb : ~bb;
  }
}

// Workgroup barrier that lets the N most recent LDS-DMA loads of every thread stay in flight: s_waitcnt vmcnt(N)
// lgkmcnt(0) (gfx9 encoding: vmcnt in bits 3:0 and 15:14, expcnt 6:4 left at "no wait", lgkmcnt 11:8), then s_barrier.
// __syncthreads() cannot be used for this: its release fence waits for every outstanding LDS-DMA transfer.  The
// older loads have landed in every wave once all waves have passed, and every wave's LDS reads of the stage that is
// refilled next have returned.
template <int N>
__device__ __forceinline__ void sync_keep_loads() {
  __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | (0x7 << 4));
  __builtin_amdgcn_s_barrier();
}

// Map a workgroup id to a tile so that the workgroups of one XCD (ids congruent mod 8 are dispatched
// to the same XCD) walk a contiguous range of tiles: tiles of one expert then share that XCD's L2.
__device__ __forceinline__ int xcd_tile(int bid, int total) {
  const int per = (total + 7) >> 3;
  const int slot = bid >> 3;
  if (slot >= per) return total;   // no tile
  return (bid & 7) * per + slot;
}

// A kernel that wants more dynamic LDS than the default limit has to be allowed to, once per device, by a host-side
// driver call (hipFuncSetAttribute).  One of these per kernel instantiation remembers the devices on which that has
// been done, so that later launches, possibly under graph capture, go straight to the launch.
struct LdsLimitOnce {
  std::mutex m;
  bool done[64] = {};
  hipError_t raise(const void* kernel, int bytes) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const bool tracked = dev >= 0 && dev < 64;
    std::lock_guard<std::mutex> lock(m);
    if (tracked && done[dev]) return hipSuccess;
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess && tracked) done[dev] = true;
    return e;
  }
};

// ---- host-side launchers (one per translation unit) -------------------------------------------
// `chunk_hist` (or NULL): per-workgroup histograms of the selected experts, [ceil(T / *hist_tokens)][64]; *hist_tokens
// comes back 0 when the kernel that ran does not write them.
hipError_t launch_router(const void* x, const void* w_router, const float* bias, int T, int H, int E, int k, int dtype,
                         int norm_mode, float* logits, int32_t* idx, float* w, float* gap, int32_t* chunk_hist,
                         int* hist_tokens, hipStream_t s);
bool router_norm_supported(int H, int dtype, const void* h, const void* w_router, const void* xn);
hipError_t launch_router_norm(const void* h, const float* norm_weight, float eps, const void* w_router, const float* bias,
                              int T, int H, int E, int k, int norm_mode, void* xn, float* logits, int32_t* idx, float* w,
                              int32_t* chunk_hist, int* hist_tokens, hipStream_t s);
size_t permute_workspace_bytes(int T);
hipError_t launch_permute(const int32_t* idx, int T, int E, int k, int32_t* counts, int32_t* offsets,
                          int32_t* perm_slot, int32_t* perm_token, void* ws, hipStream_t s);
size_t router_hist_bytes(int T);
bool permute_takes_router_hist(int T, int k);
hipError_t launch_permute_from_hist(const int32_t* idx, int T, int E, int k, int32_t* hist, int hist_tokens,
                                    int32_t* counts, int32_t* offsets, int32_t* perm_slot, int32_t* perm_token,
                                    hipStream_t s);
hipError_t launch_gateup_generic(const void* x, const void* wgu, const float* theta, const int32_t* offsets,
                                 const int32_t* perm_token, int T, int H, int E, int k, int I, int dtype, int act,
                                 void* hidden, hipStream_t s);
hipError_t launch_down_generic(const void* hidden, const void* wd, const float* w, const int32_t* offsets,
                               const int32_t* perm_slot, int T, int H, int E, int k, int I, int dtype, float* yw,
                               hipStream_t s);
// What the combine folds in besides the slot rows; every pointer may be NULL (see combine_kernel).
struct CombineArgs {
  const int32_t* idx = nullptr;    // [T,k]; needed for specials and for skipping out-of-range slots
  const float* w = nullptr;        // [T,k]; needed for specials
  const void* x = nullptr;         // [T,H] in the output dtype; needed for specials
  int E_glu = 0, n_pos = 0, n_neg = 0;
  const void* residual = nullptr;  // [T,H] in the output dtype
  int round_block = 0;             // round the sum of the slot rows to the output dtype before the residual is added
};
hipError_t launch_combine(const void* yw, int yw_is_bf16, const CombineArgs& a, int T, int H, int k, int dtype,
                          void* out, hipStream_t s);
hipError_t launch_rmsnorm(const void* x, const float* weight, float eps, int T, int H, int dtype, void* out,
                          hipStream_t s);
bool mfma_supported(int H, int I, int dtype);
hipError_t launch_gateup_mfma(const void* x, const void* wgu, const float* theta, const int32_t* offsets,
                              const int32_t* perm_token, int T, int H, int E, int k, int I, int act, void* hidden,
                              hipStream_t s);
hipError_t launch_down_mfma(const void* hidden, const void* wd, const float* w, const int32_t* offsets,
                            const int32_t* perm_slot, int T, int H, int E, int k, int I, void* yw, hipStream_t s);

bool fused_supported(int H, int I, int dtype);
hipError_t launch_gateup_raw(const void* x, const void* wgu, const int32_t* offsets, const int32_t* perm_token, int T, int H,
                             int E, int k, int I, void* gu, hipStream_t s);
hipError_t launch_experts_fused(const void* x, const void* wgu, const void* wd, const float* theta, const float* w,
                                const int32_t* offsets, const int32_t* perm_slot, const int32_t* perm_token, int T,
                                int H, int E, int k, int I, int act, void* yw, void* preact, hipStream_t s);
bool stream_supported(int H, int I, int dtype);
hipError_t launch_gateup_stream(const void* x, const void* wgu, const int32_t* idx, int T, int H, int E, int k, int I,
                                void* gu, hipStream_t s);
hipError_t launch_down_stream(const void* gu, const void* wd, const float* theta, const float* w, const int32_t* idx,
                              int T, int H, int E, int k, int I, int act, void* hidden, float* yw, hipStream_t s);

bool attn_res_supported(int H, int n_cand, int dtype);
hipError_t launch_attn_res(const void* const* cands, int n_cand, const float* score_w, float eps, int T, int H, void* out,
                           hipStream_t s);

// ---- backward pass (backward.hip) ----
struct BackwardBuffers {
  void *gu, *dhp, *dgu, *hidden, *dxs, *zrow;                       // bf16 device buffers, sizes in launch_backward's comment
  float *dw_slot, *dl, *dtheta_row;                                 // [T*k] each
  float* dwr_part;                                                  // [backward_chunk_slots(), backward_dwr_split(), H]
  float* wgrad_part;                                                // backward_wgrad_part_bytes(): partial dW tiles of experts cut into chunks
  int* wgrad_plan;                                                  // backward_plan_bytes(): the list of row chunks, written by act_bwd_kernel
};
bool backward_supported(int H, int I, int k, int dtype);
size_t backward_zero_row_bytes(int H, int I);
int backward_chunk_rows(int S_rows, int E);
int backward_chunk_slots(int S_rows, int E);
size_t backward_wgrad_part_bytes(int S_rows, int H, int E, int I);
size_t backward_plan_bytes(int S_rows, int E);
int backward_dwr_split();
// the generic family (backward_generic.hip): any sizes, bf16 or fp32 operands; every buffer fp32
struct GenericBackwardBuffers {
  float *dgu, *hw, *dxs;                                            // [S,2I], [S,I], [S,H]
  float *dw_slot, *dl, *dtheta_row;                                 // [T*k] each
};
bool backward_generic_supported(int H, int I, int k);
hipError_t launch_backward_generic(const void* x, const void* d_out, const void* w_router, const void* wgu, const void* wd,
                                   const float* theta, const float* logits, const int32_t* idx, const float* w,
                                   const int32_t* offsets, const int32_t* perm_slot, const int32_t* perm_token, int T, int H,
                                   int E, int n_pos, int n_neg, int k, int I, int dtype, int norm_mode, int act,
                                   const GenericBackwardBuffers& b, void* dx, void* d_w_router, void* d_wgu, void* d_wd,
                                   float* d_theta, hipStream_t s);
hipError_t launch_backward(const void* x, const void* d_out, const void* w_router, const void* wgu, const void* wd,
                           const float* theta, const float* logits, const int32_t* idx, const float* w,
                           const int32_t* offsets, const int32_t* perm_slot, const int32_t* perm_token, int T, int H, int E,
                           int n_pos, int n_neg, int k, int I, int norm_mode, int act, const BackwardBuffers& b, void* dx,
                           void* d_w_router, void* d_wgu, void* d_wd, float* d_theta, hipStream_t s, const void* gu_saved = nullptr);

}  // namespace bibo
