// extern "C" entry points: host-side argument checks, workspace carving and kernel dispatch.
// Nothing here allocates or synchronises; see include/bibo_moe.h for the contract.
#include <mutex>

#include "common.h"

// Workspace of bibo_moe_forward_static: one copy per GPU, alive until the process ends.  In host code the
// name is only a handle for hipGetSymbolAddress; kernels get the per-device address looked up below.
static __device__ __align__(256) unsigned char scratch[BIBO_MOE_STATIC_SCRATCH_BYTES];

namespace {

using namespace bibo;

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// Address of `scratch` on the current device, looked up once per device.
int static_scratch(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return BIBO_ERR_UNSUPPORTED;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (p == nullptr) return (int)hipErrorInvalidSymbol;
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return BIBO_OK;
}

constexpr size_t kAlign = 256;
inline size_t align_up(size_t v) { return (v + kAlign - 1) & ~(kAlign - 1); }
inline size_t elt_size(int dtype) { return dtype == BIBO_DTYPE_BF16 ? 2 : 4; }
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
inline bool aligned_ws(const void* p) { return (reinterpret_cast<uintptr_t>(p) & (kAlign - 1)) == 0; }

inline bool act_ok(int act) { return act >= BIBO_ACT_RADIAL_SIGMOID && act <= BIBO_ACT_SILU; }

int check_dims(int T, int H, int E, int k, int I, int dtype, int n_pos = 0, int n_neg = 0) {
  if (n_pos < 0 || n_neg < 0 || n_pos + n_neg >= E) return BIBO_ERR_BAD_SHAPE;     // at least one GLU expert
  if (dtype != BIBO_DTYPE_BF16 && dtype != BIBO_DTYPE_F32) return BIBO_ERR_BAD_DTYPE;
  if (T < 0 || H < 1 || I < 1 || E < 1 || E > kMaxE || k < 1 || k > kMaxK || k > E) return BIBO_ERR_BAD_SHAPE;
  if ((long long)T * k > 0x3fffffffLL) return BIBO_ERR_BAD_SHAPE;
  return BIBO_OK;
}

// Rows per expert at or below which the weight-streaming kernels are preferred (measured against the tile kernels
// at E = 64, k = 6, whole layer).  With H and I up to 512 a wave's 16 weight rows stay in registers for all of the
// expert's rows and a further 16-row pass only costs its staging: the crossover against the fused kernel is near 24
// rows.  Wider rows are streamed again, from L2, for every pass: against the fused kernel they win up to about 10
// rows (H = 768, I = 384), against the two-kernel MFMA path (shapes the fused kernel does not take) up to about 17
// (H = 1024, I = 512).
inline long long stream_rows_per_expert(int H, int I, int dtype) {
  if (H <= 512 && I <= 512) return 24;
  return fused_supported(H, I, dtype) ? 10 : 17;
}

// `distinct`: the k experts of a token are known to differ (indices that come straight from the router kernel), so
// one expert gets at most T rows.  A caller's indices may name an expert several times per token, up to all T*k
// slots on one expert, and the row list of a streaming workgroup holds kStreamMaxRows entries.
// the fused kernel addresses hidden-state rows with 32-bit byte offsets
inline bool fused_fits(int T, int H) { return (long long)T * H < (1LL << 31); }

// what the streaming kernels can run: the slots fit a workgroup's scan and an expert's rows its row list
inline bool stream_possible(int T, int H, int E, int k, int I, int dtype, bool distinct) {
  return stream_supported(H, I, dtype) && (long long)T * k <= kStreamMaxSlots &&
         (distinct ? T : (long long)T * k) <= kStreamMaxRows;
}

// what `auto` gives them: few enough rows per expert that streaming beats the tile kernels
inline bool stream_eligible(int T, int H, int E, int k, int I, int dtype, bool distinct) {
  return stream_possible(T, H, E, k, I, dtype, distinct) && (long long)T * k <= stream_rows_per_expert(H, I, dtype) * E;
}

// `composite`: the caller is bibo_moe_experts_fwd / bibo_moe_forward, the only entry points that can run
// the streaming kernels (they hand bf16 pre-activations, not `hidden`, from one kernel to the next) and
// the fused kernel (its activations never reach memory).
int resolve_algo(int algo, int T, int H, int E, int k, int I, int dtype, bool composite, bool distinct, int* out) {
  switch (algo) {
    case BIBO_ALGO_AUTO:
      if (composite && stream_eligible(T, H, E, k, I, dtype, distinct)) *out = BIBO_ALGO_STREAM;
      else if (composite && fused_supported(H, I, dtype) && fused_fits(T, H)) *out = BIBO_ALGO_FUSED;
      else *out = mfma_supported(H, I, dtype) ? BIBO_ALGO_MFMA : BIBO_ALGO_GENERIC;
      break;
    case BIBO_ALGO_GENERIC: *out = BIBO_ALGO_GENERIC; break;
    case BIBO_ALGO_MFMA:
      if (!mfma_supported(H, I, dtype)) return BIBO_ERR_UNSUPPORTED;
      *out = BIBO_ALGO_MFMA;
      break;
    case BIBO_ALGO_STREAM:
      // more rows per expert than the limit: refused here, before anything is launched
      if (!composite || !stream_possible(T, H, E, k, I, dtype, distinct)) return BIBO_ERR_UNSUPPORTED;
      *out = BIBO_ALGO_STREAM;
      break;
    case BIBO_ALGO_FUSED:
      if (!composite || !fused_supported(H, I, dtype) || !fused_fits(T, H)) return BIBO_ERR_UNSUPPORTED;
      *out = BIBO_ALGO_FUSED;
      break;
    default: return BIBO_ERR_UNSUPPORTED;
  }
  // the generic kernels keep one activation row (H + 2I floats) in LDS
  if (*out == BIBO_ALGO_GENERIC && (size_t)(H + 2 * I) * sizeof(float) > 64 * 1024) return BIBO_ERR_UNSUPPORTED;
  return BIBO_OK;
}

struct Workspace {
  size_t hist, idx, w, counts, offsets, perm_slot, perm_token, hidden, gu, yw, total;
};

Workspace carve(int T, int H, int E, int k, int I, int dtype) {
  const size_t S = (size_t)T * k;
  Workspace ws;
  size_t o = 0;
  ws.hist = o;       o += align_up(permute_workspace_bytes(T) > router_hist_bytes(T) ? permute_workspace_bytes(T)
                                                                                    : router_hist_bytes(T));
  ws.idx = o;        o += align_up(S * sizeof(int32_t));
  ws.w = o;          o += align_up(S * sizeof(float));
  ws.counts = o;     o += align_up(kMaxE * sizeof(int32_t));
  ws.offsets = o;    o += align_up((kMaxE + 1) * sizeof(int32_t));
  ws.perm_slot = o;  o += align_up(S * sizeof(int32_t));
  ws.perm_token = o; o += align_up(S * sizeof(int32_t));
  ws.hidden = o;     o += align_up(S * (size_t)I * elt_size(dtype));
  // bf16 gate/up pre-activations, only ever used when the streaming kernels are eligible
  ws.gu = o;         o += align_up(stream_possible(T, H, E, k, I, dtype, true) ? S * (size_t)2 * I * sizeof(bf16_t) : 0);
  ws.yw = o;         o += align_up(S * (size_t)H * sizeof(float));
  ws.total = o;
  return ws;
}

inline int hip_rc(hipError_t e) { return e == hipSuccess ? BIBO_OK : (int)e; }

int gateup_dispatch(const void* x, const void* wgu, const float* theta, const int32_t* offsets,
                    const int32_t* perm_token, int T, int H, int E, int k, int I, int dtype, int algo, int act,
                    void* hidden, hipStream_t s) {
  if (algo == BIBO_ALGO_MFMA) {
    if (!aligned16(x) || !aligned16(wgu) || !aligned16(hidden)) return BIBO_ERR_MISALIGNED;
    return hip_rc(launch_gateup_mfma(x, wgu, theta, offsets, perm_token, T, H, E, k, I, act, hidden, s));
  }
  return hip_rc(launch_gateup_generic(x, wgu, theta, offsets, perm_token, T, H, E, k, I, dtype, act, hidden, s));
}

// E here and in gateup_dispatch counts the GLU experts (those that have weights)
int down_dispatch(const void* hidden, const void* wd, const float* w, const int32_t* offsets, const int32_t* perm_slot,
                  const CombineArgs& ca, int T, int H, int E, int k, int I, int dtype, int algo, void* out, float* yw,
                  hipStream_t s) {
  hipError_t e;
  if (algo == BIBO_ALGO_MFMA) {
    if (!aligned16(hidden) || !aligned16(wd)) return BIBO_ERR_MISALIGNED;
    // weighted expert outputs travel to the combine in bf16 (the reference's bf16 eager path rounds each
    // expert output to bf16 as well, moe.py:92)
    e = launch_down_mfma(hidden, wd, w, offsets, perm_slot, T, H, E, k, I, yw, s);
    if (e != hipSuccess) return (int)e;
    return hip_rc(launch_combine(yw, 1, ca, T, H, k, dtype, out, s));
  }
  e = launch_down_generic(hidden, wd, w, offsets, perm_slot, T, H, E, k, I, dtype, yw, s);
  if (e != hipSuccess) return (int)e;
  return hip_rc(launch_combine(yw, 0, ca, T, H, k, dtype, out, s));
}

// kernels 3 and 4 (+ combine) after the permutation, for the composite entry points
// Eg = GLU experts (with weights), np / nn = +/-Identity specials behind them (moe.py:39-44).
int experts_dispatch(const void* x, const void* wgu, const void* wd, const float* theta, const int32_t* idx,
                     const float* w, const int32_t* offsets, const int32_t* perm_slot, const int32_t* perm_token,
                     const void* residual, bool idx_trusted, int T, int H, int Eg, int np, int nn, int k, int I, int dtype,
                     int algo, int act, int flags, void* out, char* base, const Workspace& ws, hipStream_t s,
                     void* preact = nullptr) {
  float* yw = reinterpret_cast<float*>(base + ws.yw);
  CombineArgs ca;
  ca.residual = residual;
  ca.round_block = (residual != nullptr && (flags & BIBO_FLAG_ROUND_BLOCK_OUT)) ? 1 : 0;   // layers.py:62-63
  // indices that come straight from the router kernel are in range; a caller's may hold padding values, whose
  // slots the combine has to skip; specials are the combine's work either way (moe.py:95-99)
  if (!idx_trusted || np + nn > 0) { ca.idx = idx; ca.w = w; ca.x = x; ca.E_glu = Eg; ca.n_pos = np; ca.n_neg = nn; }
  if (algo == BIBO_ALGO_STREAM) {
    if (!aligned16(x) || !aligned16(wgu) || !aligned16(wd)) return BIBO_ERR_MISALIGNED;
    if (!stream_possible(T, H, Eg + np + nn, k, I, dtype, idx_trusted)) return BIBO_ERR_UNSUPPORTED;   // no pre-activation segment carved, or more rows than a row list holds
    void* gu = base + ws.gu;
    hipError_t e = launch_gateup_stream(x, wgu, idx, T, H, Eg, k, I, gu, s);
    if (e != hipSuccess) return (int)e;
    e = launch_down_stream(gu, wd, theta, w, idx, T, H, Eg, k, I, act, base + ws.hidden, yw, s);
    if (e != hipSuccess) return (int)e;
    return hip_rc(launch_combine(yw, 0, ca, T, H, k, dtype, out, s));
  }
  if (algo == BIBO_ALGO_FUSED) {
    if (!aligned16(x) || !aligned16(wgu) || !aligned16(wd)) return BIBO_ERR_MISALIGNED;
    hipError_t e = launch_experts_fused(x, wgu, wd, theta, w, offsets, perm_slot, perm_token, T, H, Eg, k, I, act, yw, preact, s);
    if (e != hipSuccess) return (int)e;
    return hip_rc(launch_combine(yw, 1, ca, T, H, k, dtype, out, s));
  }
  const int rc = gateup_dispatch(x, wgu, theta, offsets, perm_token, T, H, Eg, k, I, dtype, algo, act, base + ws.hidden, s);
  if (rc != BIBO_OK) return rc;
  return down_dispatch(base + ws.hidden, wd, w, offsets, perm_slot, ca, T, H, Eg, k, I, dtype, algo, out, yw, s);
}

// What a training forward leaves for its backward pass in a caller-owned buffer: the routing (selection, combine
// weights, fp32 logits), the permutation and the bf16 gate/up pre-activations of every routed row.
struct TrainState {
  size_t idx, w, logits, offsets, perm_slot, perm_token, gu, total;
};

TrainState carve_state(int T, int E, int k, int I) {
  const size_t S = (size_t)T * k;
  TrainState st;
  size_t o = 0;
  st.idx = o;        o += align_up(S * sizeof(int32_t));
  st.w = o;          o += align_up(S * sizeof(float));
  st.logits = o;     o += align_up((size_t)T * E * sizeof(float));
  st.offsets = o;    o += align_up((kMaxE + 1) * sizeof(int32_t));
  st.perm_slot = o;  o += align_up(S * sizeof(int32_t));
  st.perm_token = o; o += align_up(S * sizeof(int32_t));
  st.gu = o;         o += align_up(S * 2 * (size_t)I * sizeof(bf16_t));
  st.total = o;
  return st;
}

// The whole layer on `x`; `residual` (or NULL) is added in the combine.  With `norm_src` given, `x` is a buffer the
// router kernel first fills with RMSNorm(norm_src) (weight `norm_weight`, `eps`): the caller's seam in one read of
// the raw rows.
int forward_impl(const void* x, const void* w_router, const float* bias, const void* w_gate_up, const void* w_down,
                 const float* theta, const bibo_moe_shape* sh, int norm_mode, int algo, const void* residual, void* out,
                 int32_t* idx_out, float* w_out, int32_t* counts_out, float* logits_out, void* workspace,
                 size_t workspace_bytes, void* stream, const void* norm_src = nullptr, const float* norm_weight = nullptr,
                 float eps = 0.f, char* state = nullptr) {
  if (sh == nullptr) return BIBO_ERR_NULL_POINTER;
  const int T = sh->T, H = sh->H, E = sh->E, k = sh->k, I = sh->I, dtype = sh->dtype;
  int rc = check_dims(T, H, E, k, I, dtype, sh->n_pos, sh->n_neg);
  if (rc != BIBO_OK) return rc;
  const int Eg = E - sh->n_pos - sh->n_neg;
  if (norm_mode < BIBO_NORM_NONE || norm_mode > BIBO_NORM_SOFTMAX || !act_ok(sh->act)) return BIBO_ERR_UNSUPPORTED;
  int a;
  if ((rc = resolve_algo(algo, T, H, E, k, I, dtype, true, true, &a)) != BIBO_OK) return rc;
  if (!workspace) return BIBO_ERR_NULL_POINTER;
  if (!aligned_ws(workspace)) return BIBO_ERR_MISALIGNED;
  if (T > 0 && (!x || !w_router || !bias || !w_gate_up || !w_down || !out)) return BIBO_ERR_NULL_POINTER;
  if (T > 0 && !theta && sh->act != BIBO_ACT_SILU) return BIBO_ERR_NULL_POINTER;
  const Workspace ws = carve(T, H, E, k, I, dtype);
  if (workspace_bytes < ws.total) return BIBO_ERR_WORKSPACE_TOO_SMALL;
  char* base = static_cast<char*>(workspace);
  hipStream_t s = static_cast<hipStream_t>(stream);
  int32_t* idx = idx_out ? idx_out : reinterpret_cast<int32_t*>(base + ws.idx);
  float* w = w_out ? w_out : reinterpret_cast<float*>(base + ws.w);
  int32_t* counts = counts_out ? counts_out : reinterpret_cast<int32_t*>(base + ws.counts);
  int32_t* offsets = reinterpret_cast<int32_t*>(base + ws.offsets);
  int32_t* perm_slot = reinterpret_cast<int32_t*>(base + ws.perm_slot);
  int32_t* perm_token = reinterpret_cast<int32_t*>(base + ws.perm_token);
  void* preact = nullptr;
  if (state != nullptr) {                // a training forward: what the backward pass needs lands in the caller's state buffer
    const TrainState st = carve_state(T, E, k, I);
    idx = reinterpret_cast<int32_t*>(state + st.idx);
    w = reinterpret_cast<float*>(state + st.w);
    logits_out = reinterpret_cast<float*>(state + st.logits);
    offsets = reinterpret_cast<int32_t*>(state + st.offsets);
    perm_slot = reinterpret_cast<int32_t*>(state + st.perm_slot);
    perm_token = reinterpret_cast<int32_t*>(state + st.perm_token);
    preact = state + st.gu;
  }
  // the streaming kernels find their rows themselves; the permutation then only serves the counts
  const bool need_permute = a != BIBO_ALGO_STREAM || counts_out != nullptr || T == 0;
  // the router kernel can leave per-workgroup histograms of its selections, which save the permutation its
  // histogram launch and its counting pass
  int32_t* hist = reinterpret_cast<int32_t*>(base + ws.hist);
  int hist_tokens = 0;
  const bool want_hist = need_permute && T > 0 && permute_takes_router_hist(T, k);
  if (T > 0 && norm_src != nullptr) {
    rc = hip_rc(launch_router_norm(norm_src, norm_weight, eps, w_router, bias, T, H, E, k, norm_mode, const_cast<void*>(x),
                                   logits_out, idx, w, want_hist ? hist : nullptr, &hist_tokens, s));
    if (rc != BIBO_OK) return rc;
  } else if (T > 0 && (rc = hip_rc(launch_router(x, w_router, bias, T, H, E, k, dtype, norm_mode, logits_out, idx, w, nullptr,
                                                 want_hist ? hist : nullptr, &hist_tokens, s))) != BIBO_OK)
    return rc;
  if (need_permute) {
    const hipError_t e = (want_hist && hist_tokens > 0)
                             ? launch_permute_from_hist(idx, T, E, k, hist, hist_tokens, counts, offsets, perm_slot,
                                                        perm_token, s)
                             : launch_permute(idx, T, E, k, counts, offsets, perm_slot, perm_token, hist, s);
    if (e != hipSuccess) return (int)e;
  }
  if (T == 0) return BIBO_OK;
  return experts_dispatch(x, w_gate_up, w_down, theta, idx, w, offsets, perm_slot, perm_token, residual, true, T, H, Eg,
                          sh->n_pos, sh->n_neg, k, I, dtype, a, sh->act, sh->flags, out, base, ws, s, preact);
}


struct BackwardWorkspace {
  size_t hist, idx, w, logits, counts, offsets, perm_slot, perm_token, dw_slot, dl, dtheta_row, dwr_part, zrow, gu, dhp, dgu,
      hidden, dxs, wgrad_part, wgrad_plan, total;
};

BackwardWorkspace carve_backward(int T, int H, int E, int k, int I) {
  const size_t S = (size_t)T * k, b = sizeof(bf16_t);
  BackwardWorkspace ws;
  size_t o = 0;
  ws.hist = o;       o += align_up(permute_workspace_bytes(T) > router_hist_bytes(T) ? permute_workspace_bytes(T)
                                                                                    : router_hist_bytes(T));
  ws.idx = o;        o += align_up(S * sizeof(int32_t));
  ws.w = o;          o += align_up(S * sizeof(float));
  ws.logits = o;     o += align_up((size_t)T * E * sizeof(float));
  ws.counts = o;     o += align_up(kMaxE * sizeof(int32_t));
  ws.offsets = o;    o += align_up((kMaxE + 1) * sizeof(int32_t));
  ws.perm_slot = o;  o += align_up(S * sizeof(int32_t));
  ws.perm_token = o; o += align_up(S * sizeof(int32_t));
  ws.dw_slot = o;    o += align_up(S * sizeof(float));
  ws.dl = o;         o += align_up(S * sizeof(float));
  ws.dtheta_row = o; o += align_up(S * sizeof(float));
  ws.dwr_part = o;   o += align_up((size_t)backward_chunk_slots((int)S, E) * backward_dwr_split() * H * sizeof(float));
  ws.zrow = o;       o += align_up(backward_zero_row_bytes(H, I));
  ws.gu = o;         o += align_up(S * 2 * I * b);
  ws.dhp = o;        o += align_up(S * I * b);
  ws.dgu = o;        o += align_up(S * 2 * I * b);
  ws.hidden = o;     o += align_up(S * I * b);
  ws.dxs = o;        o += align_up(S * H * b);
  ws.wgrad_part = o; o += align_up(backward_wgrad_part_bytes((int)S, H, E, I));
  ws.wgrad_plan = o; o += align_up(backward_plan_bytes((int)S, E));
  ws.total = o;
  return ws;
}

// the generic family keeps its intermediates in fp32: [dg, du], w h and the per-slot dx rows
struct GenericBackwardWorkspace {
  size_t hist, idx, w, logits, counts, offsets, perm_slot, perm_token, dw_slot, dl, dtheta_row, dgu, hw, dxs, total;
};

GenericBackwardWorkspace carve_backward_generic(int T, int H, int E, int k, int I) {
  const size_t S = (size_t)T * k;
  GenericBackwardWorkspace ws;
  size_t o = 0;
  ws.hist = o;       o += align_up(permute_workspace_bytes(T) > router_hist_bytes(T) ? permute_workspace_bytes(T)
                                                                                    : router_hist_bytes(T));
  ws.idx = o;        o += align_up(S * sizeof(int32_t));
  ws.w = o;          o += align_up(S * sizeof(float));
  ws.logits = o;     o += align_up((size_t)T * E * sizeof(float));
  ws.counts = o;     o += align_up(kMaxE * sizeof(int32_t));
  ws.offsets = o;    o += align_up((kMaxE + 1) * sizeof(int32_t));
  ws.perm_slot = o;  o += align_up(S * sizeof(int32_t));
  ws.perm_token = o; o += align_up(S * sizeof(int32_t));
  ws.dw_slot = o;    o += align_up(S * sizeof(float));
  ws.dl = o;         o += align_up(S * sizeof(float));
  ws.dtheta_row = o; o += align_up(S * sizeof(float));
  ws.dgu = o;        o += align_up(S * 2 * I * sizeof(float));
  ws.hw = o;         o += align_up(S * I * sizeof(float));
  ws.dxs = o;        o += align_up(S * H * sizeof(float));
  ws.total = o;
  return ws;
}

// which backward family a shape runs: the MFMA kernels (bf16, H and I multiples of 128, I <= 512) or the generic ones
inline bool backward_fast(const bibo_moe_shape* sh) { return backward_supported(sh->H, sh->I, sh->k, sh->dtype); }

int backward_check(const bibo_moe_shape* sh, int norm_mode) {
  if (sh == nullptr) return BIBO_ERR_NULL_POINTER;
  const int rc = check_dims(sh->T, sh->H, sh->E, sh->k, sh->I, sh->dtype, sh->n_pos, sh->n_neg);
  if (rc != BIBO_OK) return rc;
  if (norm_mode < BIBO_NORM_NONE || norm_mode > BIBO_NORM_SOFTMAX || !act_ok(sh->act)) return BIBO_ERR_UNSUPPORTED;
  // the MFMA family (bf16, dimensions its tiles divide) or the generic one (a row of 2H + 5I floats within 64 KB)
  if (!backward_fast(sh) && !backward_generic_supported(sh->H, sh->I, sh->k)) return BIBO_ERR_UNSUPPORTED;
  return BIBO_OK;
}


// The MFMA backward family behind bibo_moe_backward and bibo_moe_backward_saved.  `state` (or NULL): what a training
// forward kept (routing, permutation, pre-activations); without it the routing and the permutation are computed again
// from x - same kernels, same inputs, hence the same selection and weights - and so are the pre-activations.
int backward_mfma(const void* x, const void* d_out, const void* w_router, const float* bias, const void* w_gate_up,
                  const void* w_down, const float* theta, const bibo_moe_shape* sh, int norm_mode, const char* state, void* d_x,
                  void* d_w_router, void* d_w_gate_up, void* d_w_down, float* d_theta, float* d_w_out, void* workspace,
                  size_t workspace_bytes, void* stream) {
  const int T = sh->T, H = sh->H, E = sh->E, k = sh->k, I = sh->I;
  int rc;
  if (!aligned16(x) || !aligned16(d_out) || !aligned16(w_router) || !aligned16(w_gate_up) || !aligned16(w_down) ||
      !aligned16(d_x) || !aligned16(d_w_gate_up) || !aligned16(d_w_down))
    return BIBO_ERR_MISALIGNED;
  const BackwardWorkspace ws = carve_backward(T, H, E, k, I);
  if (workspace_bytes < ws.total) return BIBO_ERR_WORKSPACE_TOO_SMALL;
  char* base = static_cast<char*>(workspace);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int32_t* idx; const float* w; const float* logits; const int32_t* offsets; const int32_t* perm_slot;
  const int32_t* perm_token; const void* gu_saved = nullptr;
  if (state != nullptr) {
    const TrainState st = carve_state(T, E, k, I);
    idx = reinterpret_cast<const int32_t*>(state + st.idx);
    w = reinterpret_cast<const float*>(state + st.w);
    logits = reinterpret_cast<const float*>(state + st.logits);
    offsets = reinterpret_cast<const int32_t*>(state + st.offsets);
    perm_slot = reinterpret_cast<const int32_t*>(state + st.perm_slot);
    perm_token = reinterpret_cast<const int32_t*>(state + st.perm_token);
    gu_saved = state + st.gu;
  } else {
    int32_t* idx_w = reinterpret_cast<int32_t*>(base + ws.idx);
    float* w_w = reinterpret_cast<float*>(base + ws.w);
    float* logits_w = reinterpret_cast<float*>(base + ws.logits);
    int32_t* counts = reinterpret_cast<int32_t*>(base + ws.counts);
    int32_t* offsets_w = reinterpret_cast<int32_t*>(base + ws.offsets);
    int32_t* slot_w = reinterpret_cast<int32_t*>(base + ws.perm_slot);
    int32_t* token_w = reinterpret_cast<int32_t*>(base + ws.perm_token);
    // (the router kernel leaves per-workgroup histograms of its selections for the permutation, as in the forward pass)
    int32_t* hist = reinterpret_cast<int32_t*>(base + ws.hist);
    int hist_tokens = 0;
    const bool want_hist = T > 0 && permute_takes_router_hist(T, k);
    if (T > 0 && (rc = hip_rc(launch_router(x, w_router, bias, T, H, E, k, sh->dtype, norm_mode, logits_w, idx_w, w_w, nullptr,
                                            want_hist ? hist : nullptr, &hist_tokens, s))) != BIBO_OK)
      return rc;
    rc = hip_rc((want_hist && hist_tokens > 0)
                    ? launch_permute_from_hist(idx_w, T, E, k, hist, hist_tokens, counts, offsets_w, slot_w, token_w, s)
                    : launch_permute(idx_w, T, E, k, counts, offsets_w, slot_w, token_w, hist, s));
    if (rc != BIBO_OK) return rc;
    idx = idx_w; w = w_w; logits = logits_w; offsets = offsets_w; perm_slot = slot_w; perm_token = token_w;
  }
  BackwardBuffers b;
  b.gu = base + ws.gu; b.dhp = base + ws.dhp; b.dgu = base + ws.dgu;
  b.hidden = base + ws.hidden; b.dxs = base + ws.dxs; b.zrow = base + ws.zrow;
  b.dw_slot = d_w_out ? d_w_out : reinterpret_cast<float*>(base + ws.dw_slot);
  b.dl = reinterpret_cast<float*>(base + ws.dl);
  b.dtheta_row = reinterpret_cast<float*>(base + ws.dtheta_row);
  b.dwr_part = reinterpret_cast<float*>(base + ws.dwr_part);
  b.wgrad_part = reinterpret_cast<float*>(base + ws.wgrad_part);
  b.wgrad_plan = reinterpret_cast<int*>(base + ws.wgrad_plan);
  return hip_rc(launch_backward(x, d_out, w_router, w_gate_up, w_down, theta, logits, idx, w, offsets, perm_slot, perm_token,
                                T, H, E - sh->n_pos - sh->n_neg, sh->n_pos, sh->n_neg, k, I, norm_mode, sh->act, b, d_x,
                                d_w_router, d_w_gate_up, d_w_down, d_theta, s, gu_saved));
}

// whether a shape has the training forward that keeps its state: the fused forward kernel and the MFMA backward both take it
inline bool train_state_supported(const bibo_moe_shape* sh) {
  return backward_fast(sh) && fused_supported(sh->H, sh->I, sh->dtype) && fused_fits(sh->T, sh->H);
}

}  // namespace

extern "C" {

int bibo_moe_abi_version(void) { return BIBO_MOE_ABI_VERSION; }

const char* bibo_moe_strerror(int code) {
  switch (code) {
    case BIBO_OK: return "success";
    case BIBO_ERR_NULL_POINTER: return "a required pointer is NULL";
    case BIBO_ERR_BAD_SHAPE:
      return "bad shape: need T >= 0, H, I >= 1, 1 <= E <= 64, 1 <= k <= min(E, 8), n_pos, n_neg >= 0, n_pos + n_neg < E";
    case BIBO_ERR_BAD_DTYPE: return "dtype must be BIBO_DTYPE_BF16 or BIBO_DTYPE_F32";
    case BIBO_ERR_WORKSPACE_TOO_SMALL: return "workspace smaller than bibo_moe_workspace_bytes() for this shape";
    case BIBO_ERR_MISALIGNED: return "tensor base pointers must be 16-byte aligned and the workspace 256-byte aligned";
    case BIBO_ERR_UNSUPPORTED: return "requested kernel family does not support this shape or dtype";
    case BIBO_ERR_STATIC_SCRATCH:
      return "shape needs more workspace than the static scratch array holds (BIBO_MOE_STATIC_SCRATCH_BYTES = 16 MiB); "
             "use bibo_moe_forward with a caller-owned workspace";
    default: break;
  }
  if (code > 0) return hipGetErrorString((hipError_t)code);
  return "unknown error code";
}

int bibo_moe_workspace_bytes(const bibo_moe_shape* sh, size_t* bytes) {
  if (sh == nullptr || bytes == nullptr) return BIBO_ERR_NULL_POINTER;
  const int rc = check_dims(sh->T, sh->H, sh->E, sh->k, sh->I, sh->dtype, sh->n_pos, sh->n_neg);
  if (rc != BIBO_OK) return rc;
  *bytes = carve(sh->T, sh->H, sh->E, sh->k, sh->I, sh->dtype).total;
  return BIBO_OK;
}

int bibo_moe_select_algo(const bibo_moe_shape* sh, int algo, int* selected) {
  if (sh == nullptr || selected == nullptr) return BIBO_ERR_NULL_POINTER;
  const int rc = check_dims(sh->T, sh->H, sh->E, sh->k, sh->I, sh->dtype, sh->n_pos, sh->n_neg);
  if (rc != BIBO_OK) return rc;
  return resolve_algo(algo, sh->T, sh->H, sh->E, sh->k, sh->I, sh->dtype, true, true, selected);
}

int bibo_moe_router_fwd(const void* x, const void* w_router, const float* bias, int T, int H, int E, int k, int dtype,
                        int norm_mode, float* logits, int32_t* idx, float* w, float* gap, void* stream) {
  const int rc = check_dims(T, H, E, k, 1, dtype);
  if (rc != BIBO_OK) return rc;
  if (norm_mode < BIBO_NORM_NONE || norm_mode > BIBO_NORM_SOFTMAX) return BIBO_ERR_UNSUPPORTED;
  if (T == 0) return BIBO_OK;
  if (!x || !w_router || !bias || !idx || !w) return BIBO_ERR_NULL_POINTER;
  return hip_rc(launch_router(x, w_router, bias, T, H, E, k, dtype, norm_mode, logits, idx, w, gap, nullptr, nullptr,
                              static_cast<hipStream_t>(stream)));
}

int bibo_moe_permute(const int32_t* idx, int T, int E, int k, int32_t* counts, int32_t* offsets, int32_t* perm_slot,
                     int32_t* perm_token, void* workspace, size_t workspace_bytes, void* stream) {
  const int rc = check_dims(T, 1, E, k, 1, BIBO_DTYPE_BF16);
  if (rc != BIBO_OK) return rc;
  if (!counts || !offsets || !workspace) return BIBO_ERR_NULL_POINTER;
  if (T > 0 && (!idx || !perm_slot || !perm_token)) return BIBO_ERR_NULL_POINTER;
  if (workspace_bytes < permute_workspace_bytes(T)) return BIBO_ERR_WORKSPACE_TOO_SMALL;
  return hip_rc(launch_permute(idx, T, E, k, counts, offsets, perm_slot, perm_token, workspace,
                               static_cast<hipStream_t>(stream)));
}

int bibo_moe_gateup_fwd(const void* x, const void* w_gate_up, const float* theta, const int32_t* offsets,
                        const int32_t* perm_token, int T, int H, int E, int k, int I, int dtype, int algo, int act,
                        void* hidden, void* stream) {
  int rc = check_dims(T, H, E, k, I, dtype);
  if (rc != BIBO_OK) return rc;
  if (!act_ok(act)) return BIBO_ERR_UNSUPPORTED;
  int a;
  if ((rc = resolve_algo(algo, T, H, E, k, I, dtype, false, false, &a)) != BIBO_OK) return rc;
  if (T == 0) return BIBO_OK;
  if (!x || !w_gate_up || (!theta && act != BIBO_ACT_SILU) || !offsets || !perm_token || !hidden) return BIBO_ERR_NULL_POINTER;
  return gateup_dispatch(x, w_gate_up, theta, offsets, perm_token, T, H, E, k, I, dtype, a, act, hidden,
                         static_cast<hipStream_t>(stream));
}

int bibo_moe_down_combine_fwd(const void* hidden, const void* w_down, const float* w, const int32_t* offsets,
                              const int32_t* perm_slot, int T, int H, int E, int k, int I, int dtype, int algo,
                              void* out, void* workspace, size_t workspace_bytes, void* stream) {
  int rc = check_dims(T, H, E, k, I, dtype);
  if (rc != BIBO_OK) return rc;
  int a;
  if ((rc = resolve_algo(algo, T, H, E, k, I, dtype, false, false, &a)) != BIBO_OK) return rc;
  if (T == 0) return BIBO_OK;
  if (!hidden || !w_down || !w || !offsets || !perm_slot || !out || !workspace) return BIBO_ERR_NULL_POINTER;
  if (!aligned_ws(workspace)) return BIBO_ERR_MISALIGNED;       // the slot rows live there, 16 bytes at a time
  if (workspace_bytes < (size_t)T * k * H * sizeof(float)) return BIBO_ERR_WORKSPACE_TOO_SMALL;
  return down_dispatch(hidden, w_down, w, offsets, perm_slot, CombineArgs{}, T, H, E, k, I, dtype, a, out,
                       static_cast<float*>(workspace), static_cast<hipStream_t>(stream));
}

int bibo_moe_gateup_down_fwd(const void* x, const void* w_gate_up, const void* w_down, const float* theta,
                             const float* w, const int32_t* offsets, const int32_t* perm_slot,
                             const int32_t* perm_token, int T, int H, int E, int k, int I, int dtype, int act,
                             void* yw, void* stream) {
  const int rc = check_dims(T, H, E, k, I, dtype);
  if (rc != BIBO_OK) return rc;
  if (!fused_supported(H, I, dtype) || !fused_fits(T, H) || !act_ok(act)) return BIBO_ERR_UNSUPPORTED;
  if (T == 0) return BIBO_OK;
  if (!x || !w_gate_up || !w_down || (!theta && act != BIBO_ACT_SILU) || !w || !offsets || !perm_slot || !perm_token || !yw)
    return BIBO_ERR_NULL_POINTER;
  if (!aligned16(x) || !aligned16(w_gate_up) || !aligned16(w_down) || !aligned16(yw)) return BIBO_ERR_MISALIGNED;
  return hip_rc(launch_experts_fused(x, w_gate_up, w_down, theta, w, offsets, perm_slot, perm_token, T, H, E, k, I, act,
                                     yw, nullptr, static_cast<hipStream_t>(stream)));
}

int bibo_moe_combine_fwd(const void* yw, int yw_is_bf16, int T, int H, int k, int dtype, void* out, void* stream) {
  const int rc = check_dims(T, H, k, k, 1, dtype);   // no expert dimension here: E := k, I := 1 pass the range checks
  if (rc != BIBO_OK) return rc;
  if (yw_is_bf16 && dtype != BIBO_DTYPE_BF16) return BIBO_ERR_BAD_DTYPE;
  if (T == 0) return BIBO_OK;
  if (!yw || !out) return BIBO_ERR_NULL_POINTER;
  return hip_rc(launch_combine(yw, yw_is_bf16 ? 1 : 0, CombineArgs{}, T, H, k, dtype, out, static_cast<hipStream_t>(stream)));
}

int bibo_moe_combine_ex_fwd(const void* yw, int yw_is_bf16, const int32_t* idx, const float* w, const void* x, int E_glu,
                            int n_pos, int n_neg, const void* residual, int T, int H, int k, int dtype, void* out,
                            void* stream) {
  const int rc = check_dims(T, H, k, k, 1, dtype);   // no expert dimension here: E := k, I := 1 pass the range checks
  if (rc != BIBO_OK) return rc;
  if (yw_is_bf16 && dtype != BIBO_DTYPE_BF16) return BIBO_ERR_BAD_DTYPE;
  if (E_glu < 0 || n_pos < 0 || n_neg < 0 || E_glu + n_pos + n_neg > kMaxE) return BIBO_ERR_BAD_SHAPE;
  if (T == 0) return BIBO_OK;
  if (!yw || !out) return BIBO_ERR_NULL_POINTER;
  if (n_pos + n_neg > 0 && (!idx || !w || !x)) return BIBO_ERR_NULL_POINTER;
  CombineArgs ca;
  ca.idx = idx; ca.w = w; ca.x = x; ca.E_glu = E_glu; ca.n_pos = n_pos; ca.n_neg = n_neg; ca.residual = residual;
  return hip_rc(launch_combine(yw, yw_is_bf16 ? 1 : 0, ca, T, H, k, dtype, out, static_cast<hipStream_t>(stream)));
}

int bibo_moe_experts_fwd(const void* x, const int32_t* idx, const float* w, const void* w_gate_up, const void* w_down,
                         const float* theta, const bibo_moe_shape* sh, int algo, void* out, int32_t* counts_out,
                         void* workspace, size_t workspace_bytes, void* stream) {
  if (sh == nullptr) return BIBO_ERR_NULL_POINTER;
  const int T = sh->T, H = sh->H, E = sh->E, k = sh->k, I = sh->I, dtype = sh->dtype;
  int rc = check_dims(T, H, E, k, I, dtype, sh->n_pos, sh->n_neg);
  if (rc != BIBO_OK) return rc;
  const int Eg = E - sh->n_pos - sh->n_neg;
  if (!act_ok(sh->act)) return BIBO_ERR_UNSUPPORTED;
  int a;
  // a caller's indices may repeat an expert inside a token (moe.py:46-71 accepts that)
  if ((rc = resolve_algo(algo, T, H, E, k, I, dtype, true, false, &a)) != BIBO_OK) return rc;
  if (!workspace) return BIBO_ERR_NULL_POINTER;
  if (!aligned_ws(workspace)) return BIBO_ERR_MISALIGNED;
  if (T > 0 && (!x || !idx || !w || !w_gate_up || !w_down || !out)) return BIBO_ERR_NULL_POINTER;
  if (T > 0 && !theta && sh->act != BIBO_ACT_SILU) return BIBO_ERR_NULL_POINTER;
  const Workspace ws = carve(T, H, E, k, I, dtype);
  if (workspace_bytes < ws.total) return BIBO_ERR_WORKSPACE_TOO_SMALL;
  char* base = static_cast<char*>(workspace);
  hipStream_t s = static_cast<hipStream_t>(stream);
  int32_t* counts = counts_out ? counts_out : reinterpret_cast<int32_t*>(base + ws.counts);
  int32_t* offsets = reinterpret_cast<int32_t*>(base + ws.offsets);
  int32_t* perm_slot = reinterpret_cast<int32_t*>(base + ws.perm_slot);
  int32_t* perm_token = reinterpret_cast<int32_t*>(base + ws.perm_token);
  // the streaming kernels find their rows themselves; the permutation then only serves the counts
  const bool need_permute = a != BIBO_ALGO_STREAM || counts_out != nullptr || T == 0;
  if (need_permute &&
      (rc = hip_rc(launch_permute(idx, T, E, k, counts, offsets, perm_slot, perm_token, base + ws.hist, s))) != BIBO_OK)
    return rc;
  if (T == 0) return BIBO_OK;
  return experts_dispatch(x, w_gate_up, w_down, theta, idx, w, offsets, perm_slot, perm_token, nullptr, false, T, H, Eg,
                          sh->n_pos, sh->n_neg, k, I, dtype, a, sh->act, 0, out, base, ws, s);
}

int bibo_moe_forward(const void* x, const void* w_router, const float* bias, const void* w_gate_up, const void* w_down,
                     const float* theta, const bibo_moe_shape* sh, int norm_mode, int algo, void* out, int32_t* idx_out,
                     float* w_out, int32_t* counts_out, float* logits_out, void* workspace, size_t workspace_bytes,
                     void* stream) {
  return forward_impl(x, w_router, bias, w_gate_up, w_down, theta, sh, norm_mode, algo, nullptr, out, idx_out, w_out,
                      counts_out, logits_out, workspace, workspace_bytes, stream);
}

int bibo_moe_forward_static(const void* x, const void* w_router, const float* bias, const void* w_gate_up,
                            const void* w_down, const float* theta, const bibo_moe_shape* sh, int norm_mode, int algo,
                            void* out, int32_t* idx_out, float* w_out, int32_t* counts_out, float* logits_out,
                            void* stream) {
  if (sh == nullptr) return BIBO_ERR_NULL_POINTER;
  int rc = check_dims(sh->T, sh->H, sh->E, sh->k, sh->I, sh->dtype, sh->n_pos, sh->n_neg);
  if (rc != BIBO_OK) return rc;
  if (carve(sh->T, sh->H, sh->E, sh->k, sh->I, sh->dtype).total > (size_t)BIBO_MOE_STATIC_SCRATCH_BYTES)
    return BIBO_ERR_STATIC_SCRATCH;
  void* ws = nullptr;
  if ((rc = static_scratch(&ws)) != BIBO_OK) return rc;
  return forward_impl(x, w_router, bias, w_gate_up, w_down, theta, sh, norm_mode, algo, nullptr, out, idx_out, w_out,
                      counts_out, logits_out, ws, (size_t)BIBO_MOE_STATIC_SCRATCH_BYTES, stream);
}

int bibo_moe_rmsnorm_fwd(const void* x, const float* norm_weight, float eps, int T, int H, int dtype, void* out,
                         void* stream) {
  const int rc = check_dims(T, H, 1, 1, 1, dtype);
  if (rc != BIBO_OK) return rc;
  if (T == 0) return BIBO_OK;
  if (!x || !norm_weight || !out) return BIBO_ERR_NULL_POINTER;
  return hip_rc(launch_rmsnorm(x, norm_weight, eps, T, H, dtype, out, static_cast<hipStream_t>(stream)));
}

int bibo_moe_ffn_workspace_bytes(const bibo_moe_shape* sh, size_t* out) {
  if (sh == nullptr || out == nullptr) return BIBO_ERR_NULL_POINTER;
  const int rc = check_dims(sh->T, sh->H, sh->E, sh->k, sh->I, sh->dtype, sh->n_pos, sh->n_neg);
  if (rc != BIBO_OK) return rc;
  *out = carve(sh->T, sh->H, sh->E, sh->k, sh->I, sh->dtype).total + align_up((size_t)sh->T * sh->H * elt_size(sh->dtype));
  return BIBO_OK;
}

int bibo_moe_ffn_forward(const void* h, const float* norm_weight, float eps, const void* residual, const void* w_router,
                         const float* bias, const void* w_gate_up, const void* w_down, const float* theta, const bibo_moe_shape* sh,
                         int norm_mode, int algo, void* out, int32_t* idx_out, float* w_out, int32_t* counts_out,
                         void* workspace, size_t workspace_bytes, void* stream) {
  if (sh == nullptr) return BIBO_ERR_NULL_POINTER;
  const int rc = check_dims(sh->T, sh->H, sh->E, sh->k, sh->I, sh->dtype, sh->n_pos, sh->n_neg);
  if (rc != BIBO_OK) return rc;
  if (!workspace) return BIBO_ERR_NULL_POINTER;
  if (!aligned_ws(workspace)) return BIBO_ERR_MISALIGNED;
  if (sh->T > 0 && (!h || !norm_weight || !out)) return BIBO_ERR_NULL_POINTER;
  const size_t inner = carve(sh->T, sh->H, sh->E, sh->k, sh->I, sh->dtype).total;
  const size_t xn_bytes = align_up((size_t)sh->T * sh->H * elt_size(sh->dtype));
  if (workspace_bytes < inner + xn_bytes) return BIBO_ERR_WORKSPACE_TOO_SMALL;
  void* xn = static_cast<char*>(workspace) + inner;              // post_attention_layernorm(h), layers.py:60
  // what the block's output is added to: h itself (layers.py:62-64), another tensor, or nothing
  const void* res = (sh->flags & BIBO_FLAG_NO_RESIDUAL) ? nullptr : (residual != nullptr ? residual : h);
  if (sh->T > 0 && w_router != nullptr && router_norm_supported(sh->H, sh->dtype, h, w_router, xn))
    // the router kernel normalises the rows it reads and leaves them in xn: no norm launch, one read of h
    return forward_impl(xn, w_router, bias, w_gate_up, w_down, theta, sh, norm_mode, algo, res, out, idx_out, w_out,
                        counts_out, nullptr, workspace, inner, stream, h, norm_weight, eps);
  const hipError_t e = launch_rmsnorm(h, norm_weight, eps, sh->T, sh->H, sh->dtype, xn, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return (int)e;
  return forward_impl(xn, w_router, bias, w_gate_up, w_down, theta, sh, norm_mode, algo, res, out, idx_out, w_out,
                      counts_out, nullptr, workspace, inner, stream);
}

int bibo_moe_backward_workspace_bytes(const bibo_moe_shape* sh, size_t* bytes) {
  if (bytes == nullptr) return BIBO_ERR_NULL_POINTER;
  const int rc = backward_check(sh, BIBO_NORM_SUM);
  if (rc != BIBO_OK) return rc;
  *bytes = backward_fast(sh) ? carve_backward(sh->T, sh->H, sh->E, sh->k, sh->I).total
                             : carve_backward_generic(sh->T, sh->H, sh->E, sh->k, sh->I).total;
  return BIBO_OK;
}

int bibo_moe_backward(const void* x, const void* d_out, const void* w_router, const float* bias, const void* w_gate_up,
                      const void* w_down, const float* theta, const bibo_moe_shape* sh, int norm_mode, void* d_x,
                      void* d_w_router, void* d_w_gate_up, void* d_w_down, float* d_theta, float* d_w_out,
                      void* workspace, size_t workspace_bytes, void* stream) {
  int rc = backward_check(sh, norm_mode);
  if (rc != BIBO_OK) return rc;
  const int T = sh->T, H = sh->H, E = sh->E, k = sh->k, I = sh->I;
  if (!workspace) return BIBO_ERR_NULL_POINTER;
  if (!aligned_ws(workspace)) return BIBO_ERR_MISALIGNED;
  if (!d_w_router || !d_w_gate_up || !d_w_down || !d_theta) return BIBO_ERR_NULL_POINTER;
  if (T > 0 && (!x || !d_out || !w_router || !bias || !w_gate_up || !w_down || !d_x)) return BIBO_ERR_NULL_POINTER;
  if (T > 0 && !theta && sh->act != BIBO_ACT_SILU) return BIBO_ERR_NULL_POINTER;
  if (!backward_fast(sh)) {
    const GenericBackwardWorkspace gw = carve_backward_generic(T, H, E, k, I);
    if (workspace_bytes < gw.total) return BIBO_ERR_WORKSPACE_TOO_SMALL;
    char* gb = static_cast<char*>(workspace);
    hipStream_t gs = static_cast<hipStream_t>(stream);
    int32_t* g_idx = reinterpret_cast<int32_t*>(gb + gw.idx);
    float* g_w = reinterpret_cast<float*>(gb + gw.w);
    float* g_logits = reinterpret_cast<float*>(gb + gw.logits);
    int32_t* g_offsets = reinterpret_cast<int32_t*>(gb + gw.offsets);
    int32_t* g_slot = reinterpret_cast<int32_t*>(gb + gw.perm_slot);
    int32_t* g_token = reinterpret_cast<int32_t*>(gb + gw.perm_token);
    if (T > 0 && (rc = hip_rc(launch_router(x, w_router, bias, T, H, E, k, sh->dtype, norm_mode, g_logits, g_idx, g_w, nullptr,
                                            nullptr, nullptr, gs))) != BIBO_OK)
      return rc;
    if ((rc = hip_rc(launch_permute(g_idx, T, E, k, reinterpret_cast<int32_t*>(gb + gw.counts), g_offsets, g_slot, g_token,
                                    gb + gw.hist, gs))) != BIBO_OK)
      return rc;
    GenericBackwardBuffers g;
    g.dgu = reinterpret_cast<float*>(gb + gw.dgu); g.hw = reinterpret_cast<float*>(gb + gw.hw);
    g.dxs = reinterpret_cast<float*>(gb + gw.dxs);
    g.dw_slot = d_w_out ? d_w_out : reinterpret_cast<float*>(gb + gw.dw_slot);
    g.dl = reinterpret_cast<float*>(gb + gw.dl); g.dtheta_row = reinterpret_cast<float*>(gb + gw.dtheta_row);
    return hip_rc(launch_backward_generic(x, d_out, w_router, w_gate_up, w_down, theta, g_logits, g_idx, g_w, g_offsets, g_slot,
                                          g_token, T, H, E - sh->n_pos - sh->n_neg, sh->n_pos, sh->n_neg, k, I, sh->dtype,
                                          norm_mode, sh->act, g, d_x, d_w_router, d_w_gate_up, d_w_down, d_theta, gs));
  }
  return backward_mfma(x, d_out, w_router, bias, w_gate_up, w_down, theta, sh, norm_mode, nullptr, d_x, d_w_router,
                       d_w_gate_up, d_w_down, d_theta, d_w_out, workspace, workspace_bytes, stream);
}

int bibo_moe_train_state_bytes(const bibo_moe_shape* sh, size_t* bytes) {
  if (bytes == nullptr) return BIBO_ERR_NULL_POINTER;
  const int rc = backward_check(sh, BIBO_NORM_SUM);
  if (rc != BIBO_OK) return rc;
  if (!train_state_supported(sh)) return BIBO_ERR_UNSUPPORTED;
  *bytes = carve_state(sh->T, sh->E, sh->k, sh->I).total;
  return BIBO_OK;
}

int bibo_moe_forward_train(const void* x, const void* w_router, const float* bias, const void* w_gate_up, const void* w_down,
                           const float* theta, const bibo_moe_shape* sh, int norm_mode, void* out, int32_t* counts_out,
                           void* state, size_t state_bytes, void* workspace, size_t workspace_bytes, void* stream) {
  const int rc = backward_check(sh, norm_mode);
  if (rc != BIBO_OK) return rc;
  if (!train_state_supported(sh)) return BIBO_ERR_UNSUPPORTED;
  if (state == nullptr) return BIBO_ERR_NULL_POINTER;
  if (!aligned_ws(state)) return BIBO_ERR_MISALIGNED;
  if (state_bytes < carve_state(sh->T, sh->E, sh->k, sh->I).total) return BIBO_ERR_WORKSPACE_TOO_SMALL;
  return forward_impl(x, w_router, bias, w_gate_up, w_down, theta, sh, norm_mode, BIBO_ALGO_FUSED, nullptr, out, nullptr,
                      nullptr, counts_out, nullptr, workspace, workspace_bytes, stream, nullptr, nullptr, 0.f,
                      static_cast<char*>(state));
}

int bibo_moe_backward_saved(const void* x, const void* d_out, const void* w_router, const void* w_gate_up, const void* w_down,
                            const float* theta, const bibo_moe_shape* sh, int norm_mode, const void* state,
                            size_t state_bytes, void* d_x, void* d_w_router, void* d_w_gate_up, void* d_w_down,
                            float* d_theta, float* d_w_out, void* workspace, size_t workspace_bytes, void* stream) {
  const int rc = backward_check(sh, norm_mode);
  if (rc != BIBO_OK) return rc;
  if (!train_state_supported(sh)) return BIBO_ERR_UNSUPPORTED;
  const int T = sh->T;
  if (!workspace || !state) return BIBO_ERR_NULL_POINTER;
  if (!aligned_ws(workspace) || !aligned_ws(state)) return BIBO_ERR_MISALIGNED;
  if (state_bytes < carve_state(T, sh->E, sh->k, sh->I).total) return BIBO_ERR_WORKSPACE_TOO_SMALL;
  if (!d_w_router || !d_w_gate_up || !d_w_down || !d_theta) return BIBO_ERR_NULL_POINTER;
  if (T > 0 && (!x || !d_out || !w_router || !w_gate_up || !w_down || !d_x)) return BIBO_ERR_NULL_POINTER;
  if (T > 0 && !theta && sh->act != BIBO_ACT_SILU) return BIBO_ERR_NULL_POINTER;
  return backward_mfma(x, d_out, w_router, nullptr, w_gate_up, w_down, theta, sh, norm_mode, static_cast<const char*>(state),
                       d_x, d_w_router, d_w_gate_up, d_w_down, d_theta, d_w_out, workspace, workspace_bytes, stream);
}

int bibo_moe_experts_backward(const void* x, const void* d_out, const int32_t* idx, const float* w, const void* w_gate_up,
                              const void* w_down, const float* theta, const bibo_moe_shape* sh, void* d_x, float* d_w,
                              void* d_w_gate_up, void* d_w_down, float* d_theta, void* workspace, size_t workspace_bytes,
                              void* stream) {
  int rc = backward_check(sh, BIBO_NORM_SUM);
  if (rc != BIBO_OK) return rc;
  const int T = sh->T, H = sh->H, E = sh->E, k = sh->k, I = sh->I;
  if (!workspace) return BIBO_ERR_NULL_POINTER;
  if (!aligned_ws(workspace)) return BIBO_ERR_MISALIGNED;
  if (!d_w_gate_up || !d_w_down || !d_theta) return BIBO_ERR_NULL_POINTER;
  if (T > 0 && (!x || !d_out || !idx || !w || !w_gate_up || !w_down || !d_x || !d_w)) return BIBO_ERR_NULL_POINTER;
  if (T > 0 && !theta && sh->act != BIBO_ACT_SILU) return BIBO_ERR_NULL_POINTER;
  if (!backward_fast(sh)) {
    const GenericBackwardWorkspace gw = carve_backward_generic(T, H, E, k, I);
    if (workspace_bytes < gw.total) return BIBO_ERR_WORKSPACE_TOO_SMALL;
    char* gb = static_cast<char*>(workspace);
    hipStream_t gs = static_cast<hipStream_t>(stream);
    int32_t* g_offsets = reinterpret_cast<int32_t*>(gb + gw.offsets);
    int32_t* g_slot = reinterpret_cast<int32_t*>(gb + gw.perm_slot);
    int32_t* g_token = reinterpret_cast<int32_t*>(gb + gw.perm_token);
    if ((rc = hip_rc(launch_permute(idx, T, E, k, reinterpret_cast<int32_t*>(gb + gw.counts), g_offsets, g_slot, g_token,
                                    gb + gw.hist, gs))) != BIBO_OK)
      return rc;
    GenericBackwardBuffers g;
    g.dgu = reinterpret_cast<float*>(gb + gw.dgu); g.hw = reinterpret_cast<float*>(gb + gw.hw);
    g.dxs = reinterpret_cast<float*>(gb + gw.dxs);
    g.dw_slot = d_w;
    g.dl = reinterpret_cast<float*>(gb + gw.dl); g.dtheta_row = reinterpret_cast<float*>(gb + gw.dtheta_row);
    return hip_rc(launch_backward_generic(x, d_out, nullptr, w_gate_up, w_down, theta, nullptr, idx, w, g_offsets, g_slot, g_token,
                                          T, H, E - sh->n_pos - sh->n_neg, sh->n_pos, sh->n_neg, k, I, sh->dtype, BIBO_NORM_SUM,
                                          sh->act, g, d_x, nullptr, d_w_gate_up, d_w_down, d_theta, gs));
  }
  if (!aligned16(x) || !aligned16(d_out) || !aligned16(w_gate_up) || !aligned16(w_down) || !aligned16(d_x) ||
      !aligned16(d_w_gate_up) || !aligned16(d_w_down))
    return BIBO_ERR_MISALIGNED;
  const BackwardWorkspace ws = carve_backward(T, H, E, k, I);
  if (workspace_bytes < ws.total) return BIBO_ERR_WORKSPACE_TOO_SMALL;
  char* base = static_cast<char*>(workspace);
  hipStream_t s = static_cast<hipStream_t>(stream);
  int32_t* counts = reinterpret_cast<int32_t*>(base + ws.counts);
  int32_t* offsets = reinterpret_cast<int32_t*>(base + ws.offsets);
  int32_t* perm_slot = reinterpret_cast<int32_t*>(base + ws.perm_slot);
  int32_t* perm_token = reinterpret_cast<int32_t*>(base + ws.perm_token);
  if ((rc = hip_rc(launch_permute(idx, T, E, k, counts, offsets, perm_slot, perm_token, base + ws.hist, s))) != BIBO_OK)
    return rc;
  BackwardBuffers b;
  b.gu = base + ws.gu; b.dhp = base + ws.dhp; b.dgu = base + ws.dgu;
  b.hidden = base + ws.hidden; b.dxs = base + ws.dxs; b.zrow = base + ws.zrow;
  b.dw_slot = d_w;
  b.dl = reinterpret_cast<float*>(base + ws.dl);
  b.dtheta_row = reinterpret_cast<float*>(base + ws.dtheta_row);
  b.dwr_part = reinterpret_cast<float*>(base + ws.dwr_part);
  b.wgrad_part = reinterpret_cast<float*>(base + ws.wgrad_part);
  b.wgrad_plan = reinterpret_cast<int*>(base + ws.wgrad_plan);
  return hip_rc(launch_backward(x, d_out, nullptr, w_gate_up, w_down, theta, nullptr, idx, w, offsets, perm_slot, perm_token,
                                T, H, E - sh->n_pos - sh->n_neg, sh->n_pos, sh->n_neg, k, I, BIBO_NORM_SUM, sh->act, b, d_x,
                                nullptr, d_w_gate_up, d_w_down, d_theta, s));
}

int bibo_moe_exp_attn_res_fwd(const void* const* candidates, int n_candidates, const float* score_weight, float eps, int T, int H,
                          int dtype, void* out, void* stream) {
  const int rc = check_dims(T, H, 1, 1, 1, dtype);
  if (rc != BIBO_OK) return rc;
  if (!attn_res_supported(H, n_candidates, dtype)) return BIBO_ERR_UNSUPPORTED;
  if (!candidates || !score_weight) return BIBO_ERR_NULL_POINTER;
  if (T == 0) return BIBO_OK;
  if (!out) return BIBO_ERR_NULL_POINTER;
  for (int i = 0; i < n_candidates; ++i) {
    if (!candidates[i]) return BIBO_ERR_NULL_POINTER;
    if (!aligned16(candidates[i])) return BIBO_ERR_MISALIGNED;
  }
  if (!aligned16(out)) return BIBO_ERR_MISALIGNED;
  return hip_rc(launch_attn_res(candidates, n_candidates, score_weight, eps, T, H, out, static_cast<hipStream_t>(stream)));
}

}  // extern "C"
