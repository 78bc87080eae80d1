/*
 * bibo_moe.h -- C ABI of the MI355X (gfx950) implementation of BiBo's sparse-MoE feed-forward block.
 *
 * The reference (IsNoobgrammer/BiBo) is pure Python; the interfaces below are what a binding for its
 * three nested seams would call.  Citations are paths inside the reference repository.
 *
 *   seam 1  BiBoMoELayer.forward(hidden[B,S,H]) -> [B,S,H]            src/modeling/ffn/moe.py:157-183
 *   seam 2  BiBoFusedExperts.forward(x[N,H], idx[N,k], w[N,k]) -> [N,H] src/modeling/ffn/moe.py:46-101
 *           (the method ablate/common/patches.py:157-180 rebinds to an external fused kernel)
 *   router  BiBoMoERouter.forward(hidden) -> (idx, w)                  src/modeling/ffn/router.py:28-51
 *
 * Conventions
 *   - Every pointer is a DEVICE pointer on the current HIP device unless stated otherwise.  The caller
 *     allocates inputs, outputs and the workspace; the library allocates nothing and keeps no pointer
 *     to a caller's buffer after a call returns.  Its only state across calls is set-up it remembers per
 *     device behind a mutex: the address of its static scratch array (bibo_moe_forward_static) and
 *     whether a kernel's dynamic LDS limit has been raised; neither depends on a call's arguments.
 *   - All tensors are dense row-major ("contiguous"); weights are consumed as the reference stores
 *     them: w_router [E,H], w_gate_up [E,2I,H] (rows 0..I-1 gate, I..2I-1 up), w_down [E,H,I].
 *   - `dtype` selects the element type of hidden states and the three weight tensors
 *     (BIBO_DTYPE_BF16 or BIBO_DTYPE_F32).  bias, theta, logits and routing weights are always fp32;
 *     expert indices are int32.
 *   - `stream` is a hipStream_t passed as void*; every call is stream-ordered and asynchronous and
 *     never synchronises the host.
 *   - Return value: 0 success; negative = argument error detected on the host before anything was
 *     launched (see BIBO_ERR_*); positive = hipError_t reported by a launch.
 *   - Limits: 1 <= E <= 64, 1 <= k <= min(E, 8).
 *   - Canonical orders (the reference leaves both implementation-defined): the k experts of a token
 *     are emitted in ascending expert index with top-k ties going to the lowest index; routed slots
 *     are ordered by (expert, token, slot) ascending, i.e. a stable sort of slot ids by expert.
 */
#ifndef BIBO_MOE_H
#define BIBO_MOE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BIBO_MOE_ABI_VERSION 3
#define BIBO_MOE_MAX_EXPERTS 64
#define BIBO_MOE_MAX_TOPK 8

enum bibo_dtype { BIBO_DTYPE_BF16 = 0, BIBO_DTYPE_F32 = 1 };

/* norm_topk_prob of the reference router (src/modeling/ffn/router.py:42-47) */
enum bibo_norm_mode { BIBO_NORM_NONE = 0, BIBO_NORM_SUM = 1, BIBO_NORM_SOFTMAX = 2 };

/*
 * Activation of the GLU experts.  The reference module computes RADIAL_SIGMOID (src/modeling/ffn/moe.py:87-90);
 * its training harness can switch the external kernel to the other two (act codes 8 / 10 / 0 of
 * ablate/common/patches.py:53-69):
 *   RADIAL_SIGMOID  r^p * SiLU(g/r) * up,  r = sqrt(mean_I(g^2) + 1e-6),  p = sigmoid(theta[e])     (code 8)
 *   RADIAL_TANH     the same with p = tanh(theta[e]) in (-1, 1)                                      (code 10)
 *   SILU            SiLU(g) * up, plain SwiGLU; theta is not read                                    (code 0)
 * The value 0 is the reference module's behaviour, so a zero-initialised shape means what moe.py computes.
 */
enum bibo_act { BIBO_ACT_RADIAL_SIGMOID = 0, BIBO_ACT_RADIAL_TANH = 1, BIBO_ACT_SILU = 2 };

/* bits of bibo_moe_shape.flags */
enum bibo_flags {
  /* bibo_moe_ffn_forward only: round the block's output to `dtype` before the residual is added, then round the sum
     (bf16_moe_out of the reference's decoder layer, src/modeling/layers.py:37,62-63).  Without it the sum is formed
     in fp32 and rounded once. */
  BIBO_FLAG_ROUND_BLOCK_OUT = 1,
  /* bibo_moe_ffn_forward only: no residual at all, out = moe(rmsnorm(h)): the block as the reference's experimental
     decoder layer calls it under Block Attention Residuals (exp/modeling_bibo.py:429-431), where the caller owns
     the sum. */
  BIBO_FLAG_NO_RESIDUAL = 2
};

/* kernel family for the expert GEMMs */
enum bibo_algo {
  BIBO_ALGO_AUTO = 0,    /* pick by shape */
  BIBO_ALGO_GENERIC = 1, /* one workgroup per routed row, any H and I, bf16 or fp32 */
  BIBO_ALGO_MFMA = 2,    /* grouped bf16 MFMA tiles, one kernel per GEMM; needs bf16, H % 128 == 0 and
                            I in {128,256,384,512} */
  BIBO_ALGO_STREAM = 3,  /* weight-streaming kernels for few rows per expert (decode); bf16, H and I
                            multiples of 64 up to 1728; only the composite entry points; T*k <= 40*E when
                            H, I <= 512, 32*E up to H = 768, 24*E above, and at most 4096 slots and 2048 rows per
                            expert: T <= 2048 for bibo_moe_forward / bibo_moe_ffn_forward (a token's experts are
                            distinct), T*k <= 2048 for bibo_moe_experts_fwd (a caller's indices may repeat) */
  BIBO_ALGO_FUSED = 4    /* both GEMMs of a 128-row tile in one kernel, activations stay in LDS; bf16,
                            H % 128 == 0, I in {128,256,384}; only bibo_moe_experts_fwd / bibo_moe_forward */
};

enum bibo_error {
  BIBO_OK = 0,
  BIBO_ERR_NULL_POINTER = -1,
  BIBO_ERR_BAD_SHAPE = -2,
  BIBO_ERR_BAD_DTYPE = -3,
  BIBO_ERR_WORKSPACE_TOO_SMALL = -4,
  BIBO_ERR_MISALIGNED = -5,
  BIBO_ERR_UNSUPPORTED = -6,
  BIBO_ERR_STATIC_SCRATCH = -7 /* bibo_moe_forward_static: the shape needs more than BIBO_MOE_STATIC_SCRATCH_BYTES */
};

typedef struct bibo_moe_shape {
  int32_t T; /* tokens = B*S */
  int32_t H; /* hidden size */
  int32_t E; /* routed experts = rows of w_router: GLU experts first, then +Identity, then -Identity */
  int32_t k; /* experts per token */
  int32_t I; /* expert intermediate size */
  int32_t dtype;
  int32_t n_pos; /* +Identity specials (moe.py:39-44,95-96): out += w * x; usually 0 */
  int32_t n_neg; /* -Identity specials (moe.py:97-99): out -= w * x; usually 0 */
  int32_t act;   /* enum bibo_act; 0 = the reference module's Radial NormSiLU */
  int32_t flags; /* enum bibo_flags bits; 0 = none */
} bibo_moe_shape; /* ten int32; w_gate_up, w_down and theta hold E - n_pos - n_neg (GLU) experts */

int bibo_moe_abi_version(void);

/* Static, NUL-terminated description of a negative code; for positive codes the HIP error string. */
const char* bibo_moe_strerror(int code);

/* Bytes of workspace that any entry point below needs for this shape.  The base must be 256-byte aligned
 * (segments are carved at multiples of 256 bytes and accessed 16 bytes at a time); every entry point that takes
 * a workspace returns BIBO_ERR_MISALIGNED otherwise. */
int bibo_moe_workspace_bytes(const bibo_moe_shape* shape, size_t* bytes);

/*
 * The kernel family the composite entry points (bibo_moe_experts_fwd, bibo_moe_forward, bibo_moe_ffn_forward) run
 * for this shape when asked for `algo`: *selected is one of BIBO_ALGO_GENERIC / MFMA / STREAM / FUSED (never AUTO).
 * Returns BIBO_ERR_UNSUPPORTED when `algo` names a family that cannot run the shape.  Host-side only; no
 * counterpart in the reference (its choice between eager and patched paths is made by the caller,
 * ablate/common/patches.py:402-417).
 */
int bibo_moe_select_algo(const bibo_moe_shape* shape, int algo, int* selected);

/*
 * Router: fp32 logits, sigmoid scores, selection on scores+bias, gather of the unbiased scores and
 * normalisation.  Replaces BiBoMoERouter.forward (src/modeling/ffn/router.py:28-51) and the external
 * fused router the reference once bound (legacy/bench/exp_kappa.py:142-155).
 *   x [T,H], w_router [E,H], bias fp32 [E]
 *   logits  fp32 [T,E]  optional (may be NULL)
 *   idx     int32 [T,k] ascending expert index
 *   w       fp32 [T,k]
 *   gap     fp32 [T]    optional: score_k - score_{k+1} on unbiased scores (router.py:33-36)
 */
int bibo_moe_router_fwd(const void* x, const void* w_router, const float* bias, int T, int H, int E, int k,
                        int dtype, int norm_mode, float* logits, int32_t* idx, float* w, float* gap,
                        void* stream);

/*
 * Histogram, prefix sum and stable permutation of the T*k routed slots by expert.  Replaces the
 * sort / bincount / cumsum / .tolist() prologue of BiBoFusedExperts.forward (moe.py:56-68) and the
 * bincount of BiBoMoELayer._balance_step (moe.py:141-145).
 *   idx int32 [T,k]; counts int32 [E]; offsets int32 [E+1]; perm_slot, perm_token int32 [T*k]
 * Indices outside [0,E) are ignored (their slots get no row and offsets[E] < T*k).
 * workspace: at least 256 * (max(1, ceil(T / 128)) + ceil(T / 32768) + 1) bytes (one 64-entry histogram per 128 tokens
 * and, for large batches, one sum per 256 histograms).
 */
int bibo_moe_permute(const int32_t* idx, int T, int E, int k, int32_t* counts, int32_t* offsets,
                     int32_t* perm_slot, int32_t* perm_token, void* workspace, size_t workspace_bytes,
                     void* stream);

/*
 * Grouped gate/up projection with the Radial NormSiLU epilogue r^p * SiLU(g/r) * up,
 * r = sqrt(mean_I(g^2) + 1e-6), p = sigmoid(theta[e]) (or the activation `act` names, enum bibo_act).
 * Replaces moe.py:81-90 and the `activated * up` of moe.py:92.
 *   hidden  [T*k, I] in `dtype`, rows in permuted (sorted-by-expert) order
 */
int bibo_moe_gateup_fwd(const void* x, const void* w_gate_up, const float* theta, const int32_t* offsets,
                        const int32_t* perm_token, int T, int H, int E, int k, int I, int dtype, int algo, int act,
                        void* hidden, void* stream);

/*
 * Grouped down projection; the epilogue scales each row by its routing weight and scatters it back to
 * token order, where the k rows of a token are summed in fp32 and rounded once to `dtype`.
 * Replaces the F.linear(..., down_proj) of moe.py:92, moe.py:93 and the cast of moe.py:101.
 *   hidden [T*k, I] permuted order; w fp32 [T,k]; out [T,H] in `dtype`
 */
int bibo_moe_down_combine_fwd(const void* hidden, const void* w_down, const float* w, const int32_t* offsets,
                              const int32_t* perm_slot, int T, int H, int E, int k, int I, int dtype, int algo,
                              void* out, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Both grouped projections of a 128-row tile in one launch (BIBO_ALGO_FUSED shapes only: bf16,
 * H % 128 == 0, I in {128,256,384}); the activations of moe.py:84-92 never reach memory.  Writes the
 * routing-weighted expert outputs of moe.py:92-93 in slot order: yw bf16 [T*k, H], row t*k + j belongs to
 * token t and its j-th selected expert.  Slots whose index was outside [0,E) are not written.
 */
int bibo_moe_gateup_down_fwd(const void* x, const void* w_gate_up, const void* w_down, const float* theta,
                             const float* w, const int32_t* offsets, const int32_t* perm_slot,
                             const int32_t* perm_token, int T, int H, int E, int k, int I, int dtype, int act,
                             void* yw, void* stream);

/*
 * out[t, :] = sum_j yw[t*k + j, :], summed in fp32 in ascending j and rounded once to `dtype`
 * (the index_add_ of moe.py:93 and the cast of moe.py:101).  yw [T*k, H]: bf16 when yw_is_bf16 (then
 * `dtype` must be bf16), fp32 otherwise; out [T,H] in `dtype`.
 */
int bibo_moe_combine_fwd(const void* yw, int yw_is_bf16, int T, int H, int k, int dtype, void* out, void* stream);

/*
 * The same sum with everything the composite entry points fold into it (each pointer may be NULL):
 *   idx int32 [T,k], E_glu, n_pos, n_neg: slots with idx outside [0, E_glu+n_pos+n_neg) are skipped, slots of a
 *   +/-Identity special add +/- w[slot] * x[t, :] instead of a row of yw (moe.py:95-99; needs w fp32 [T,k] and
 *   x [T,H] in `dtype`);  residual [T,H] in `dtype` is added before the rounding (layers.py:62-64).
 */
int bibo_moe_combine_ex_fwd(const void* yw, int yw_is_bf16, const int32_t* idx, const float* w, const void* x,
                            int E_glu, int n_pos, int n_neg, const void* residual, int T, int H, int k, int dtype,
                            void* out, void* stream);

/*
 * Seam 2: BiBoFusedExperts.forward(x, idx, w) (moe.py:46-101; the signature of the external
 * moe_per_expert bound at ablate/common/patches.py:165-166).  idx int32 [T,k], w fp32 [T,k], out [T,H].
 * counts_out int32 [E] optional.
 */
int bibo_moe_experts_fwd(const void* x, const int32_t* idx, const float* w, const void* w_gate_up,
                         const void* w_down, const float* theta, const bibo_moe_shape* shape, int algo,
                         void* out, int32_t* counts_out, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Seam 1: the whole layer, router included (moe.py:157-183 in eval mode; the contract of the external
 * megakernel_block minus the RMSNorm, ablate/common/patches.py:255-258).
 * Optional outputs (may be NULL): idx_out int32 [T,k], w_out fp32 [T,k], counts_out int32 [E]
 * (the per-expert token counts BiBoMoELayer._balance_step accumulates), logits_out fp32 [T,E].
 */
int bibo_moe_forward(const void* x, const void* w_router, const float* bias, const void* w_gate_up,
                     const void* w_down, const float* theta, const bibo_moe_shape* shape, int norm_mode, int algo,
                     void* out, int32_t* idx_out, float* w_out, int32_t* counts_out, float* logits_out,
                     void* workspace, size_t workspace_bytes, void* stream);

/*
 * bibo_moe_forward for callers that cannot allocate device memory or pass a workspace: code running under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.
 * Same arguments and results as bibo_moe_forward, without `workspace`: the intermediates (routing, permutation,
 * pre-activations, slot rows) live in a static device array of BIBO_MOE_STATIC_SCRATCH_BYTES that every GPU the
 * library runs on holds until the process ends.  The call allocates and frees nothing.  A shape whose
 * bibo_moe_workspace_bytes() exceeds the array is refused with BIBO_ERR_STATIC_SCRATCH before anything is
 * launched (decode-size shapes fit: T=64, H=1024, I=512 needs 2.8 MB).  All calls on one GPU share that GPU's
 * array, on whatever stream: calls that may overlap on one GPU race and must be ordered by the caller.  Nothing
 * in the array has to start at zero (every segment is written before it is read within a call), so it is
 * never cleared.  The first call on a device looks the array's address up (no stream work); make that call
 * before capturing a graph.
 */
#define BIBO_MOE_STATIC_SCRATCH_BYTES (16u << 20)
int bibo_moe_forward_static(const void* x, const void* w_router, const float* bias, const void* w_gate_up,
                            const void* w_down, const float* theta, const bibo_moe_shape* shape, int norm_mode,
                            int algo, void* out, int32_t* idx_out, float* w_out, int32_t* counts_out,
                            float* logits_out, void* stream);

/*
 * Seam 3: the caller of the block, BiBoDecoderLayer._ffn_forward (src/modeling/layers.py:57-67):
 *   out = h + moe(post_attention_layernorm(h)),  RMSNorm as BiBoRMSNorm.forward (src/modeling/norm.py:19-24)
 * with norm_weight fp32 [H].  The normalised activations live in the workspace; the residual add happens in
 * the combine, in fp32, before the single rounding to `dtype` (the reference rounds the block output first).
 * h, out [T,H] in `dtype` (out may not alias h).  Workspace size: bibo_moe_ffn_workspace_bytes.
 * `residual` [T,H] in `dtype` or NULL: what the block's output is added to.  NULL means h itself (layers.py:57-64).
 * Another tensor gives out = residual + moe(rmsnorm(h)): the experimental layer's
 * `prefix_sum = prefix_sum + mlp(post_attention_layernorm(h))` (exp/modeling_bibo.py:429-431,666) in one call;
 * out may alias residual.  With BIBO_FLAG_NO_RESIDUAL in shape->flags nothing is added and `residual` is ignored.
 */
int bibo_moe_rmsnorm_fwd(const void* x, const float* norm_weight, float eps, int T, int H, int dtype, void* out,
                         void* stream);                 /* the norm alone: out = weight * round(x * rsqrt(mean x^2 + eps)) */
int bibo_moe_ffn_workspace_bytes(const bibo_moe_shape* shape, size_t* out_bytes);
int bibo_moe_ffn_forward(const void* h, const float* norm_weight, float eps, const void* residual, const void* w_router,
                         const float* bias,
                         const void* w_gate_up, const void* w_down, const float* theta, const bibo_moe_shape* shape,
                         int norm_mode, int algo, void* out, int32_t* idx_out, float* w_out, int32_t* counts_out,
                         void* workspace, size_t workspace_bytes, void* stream);

/*
 * Backward pass of the layer: the gradients torch.autograd derives for BiBoMoELayer.forward in training
 * (src/modeling/ffn/moe.py:157-183 with the experts of moe.py:46-101 and the router of router.py:25-47) for the
 * upstream gradient d_out [T,H] of the layer's output, with the selection held fixed (the balancing bias only enters
 * the selection, router.py:38, and gets no gradient; nor does anything flow through which experts were chosen).
 * x is the block's input as in bibo_moe_forward; the routing is recomputed from it by the forward's router kernel,
 * so the selection and the combine weights are those of the forward call on the same operands.
 *   d_x [T,H], d_w_router [E,H], d_w_gate_up [Eg,2I,H], d_w_down [Eg,H,I] in `dtype`; d_theta fp32 [Eg], with
 *   Eg = E - n_pos - n_neg GLU experts
 *   (reference pins: theta receives gradient, tests/test_moe.py:53-63, ablate/common/test_eager_radial.py:63-69);
 *   d_w_out fp32 [T,k] or NULL: gradient with respect to the combine weights (router.py:47), for inspection.
 * A slot routed to a +/-Identity expert (moe.py:95-99) sends +/- w d_out[t] to d_x and +/- <d_out[t], x[t]> to its
 * combine weight, and through that to the router.
 * Two kernel families: bf16 with H and I multiples of 128 and I <= 512 runs grouped MFMA GEMMs (bf16 operands, fp32
 * accumulation, results rounded once); every other size and fp32 run generic kernels that compute in fp32 throughout
 * (fp32 operands give fp32-exact gradients, the regime of the reference's own gradient tests) and keep
 * 2H + 5I floats of a row in LDS: BIBO_ERR_UNSUPPORTED when neither applies, i.e. off the MFMA sizes with
 * (2H + 5I) * 4 + 64 > 65536.  The intermediate activations are recomputed, nothing has to be kept from the forward
 * call.  All gradients are overwritten, not accumulated.  Workspace: bibo_moe_backward_workspace_bytes (MFMA family:
 * about 12 I + 2 H bytes per routed slot plus 12 I H bytes for each of up to 1.7 E partial weight-gradient tiles, which
 * are only written for experts that hold more than 1.5 times the average number of rows; generic family: 12 I + 4 H
 * bytes per routed slot).
 */
int bibo_moe_backward_workspace_bytes(const bibo_moe_shape* shape, size_t* bytes);
int bibo_moe_backward(const void* x, const void* d_out, const void* w_router, const float* bias, const void* w_gate_up,
                      const void* w_down, const float* theta, const bibo_moe_shape* shape, int norm_mode, void* d_x,
                      void* d_w_router, void* d_w_gate_up, void* d_w_down, float* d_theta, float* d_w_out,
                      void* workspace, size_t workspace_bytes, void* stream);

/*
 * The training forward that keeps what bibo_moe_backward would compute again: the layer of bibo_moe_forward
 * (BiBoMoELayer.forward in training, src/modeling/ffn/moe.py:157-183) whose routing, permutation and bf16 gate/up
 * pre-activations (moe.py:84) land in a caller-owned `state` buffer, and the backward pass that reads them there instead
 * of running the router, the permutation and the gate/up projection a second time (about a fifth of bibo_moe_backward's
 * time; the forward call grows by the copy-out of the pre-activations).  `state`: 256-byte aligned device memory of
 * bibo_moe_train_state_bytes (about 4 I bytes per routed slot), untouched between the two calls; it belongs to ONE
 * forward call, x and the weights must be the same in both calls.  out / counts_out as in bibo_moe_forward (kernel family
 * fixed: the fused kernel); gradients, d_w_out and the workspace (bibo_moe_backward_workspace_bytes) as in
 * bibo_moe_backward, whose results bibo_moe_backward_saved reproduces bit for bit.  Shapes: bf16, H a multiple of 128,
 * I in {128, 256, 384}; BIBO_ERR_UNSUPPORTED otherwise (use bibo_moe_forward + bibo_moe_backward).  The reference keeps
 * its activations through torch.autograd; this pair is that choice made explicit.
 */
int bibo_moe_train_state_bytes(const bibo_moe_shape* shape, size_t* bytes);
int bibo_moe_forward_train(const void* x, const void* w_router, const float* bias, const void* w_gate_up, const void* w_down,
                           const float* theta, const bibo_moe_shape* shape, int norm_mode, void* out, int32_t* counts_out,
                           void* state, size_t state_bytes, void* workspace, size_t workspace_bytes, void* stream);
int bibo_moe_backward_saved(const void* x, const void* d_out, const void* w_router, const void* w_gate_up, const void* w_down,
                            const float* theta, const bibo_moe_shape* shape, int norm_mode, const void* state,
                            size_t state_bytes, void* d_x, void* d_w_router, void* d_w_gate_up, void* d_w_down,
                            float* d_theta, float* d_w_out, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Backward pass of the experts alone (what autograd derives for BiBoFusedExperts.forward, src/modeling/ffn/moe.py:46-101)
 * for a caller that owns the routing: idx int32 [T,k] (every entry a valid expert id) and w fp32 [T,k] as handed to
 * bibo_moe_experts_fwd.  d_w fp32 [T,k] is the gradient with respect to w (moe.py:93), through which the caller's own
 * router is reached; the other results and the limits are those of bibo_moe_backward, whose workspace size it shares.
 */
int bibo_moe_experts_backward(const void* x, const void* d_out, const int32_t* idx, const float* w, const void* w_gate_up,
                              const void* w_down, const float* theta, const bibo_moe_shape* shape, void* d_x, float* d_w,
                              void* d_w_gate_up, void* d_w_down, float* d_theta, void* workspace, size_t workspace_bytes,
                              void* stream);

/*
 * Depth mix of the experimental model's Block Attention Residuals: apply_attention_residual
 * (exp/modeling_bibo.py:119-232; softmax scores, dense), the operation the reference hands to its optional external
 * kernel `kernels.sm120.attn_res.attn_res(block_residual, prefix, score_weight, eps, ...)` (exp/modeling_bibo.py:44,
 * 188-190).  candidates: host array of n_candidates device pointers to [T,H] rows (the completed block
 * representatives, then the running prefix sum); score_weight fp32 [H] = norm weight * pseudo-query;
 *   score_c = rsqrt(mean(c^2) + eps) * <c, score_weight>,  out = sum_c softmax(score)_c * c   (fp32, rounded once).
 * bf16, H % 8 == 0, H <= 1024, 1 <= n_candidates <= 8 (BIBO_ERR_UNSUPPORTED otherwise).  Not part of the MoE block:
 * a caller-side kernel of the 10-layer forward the block sits in.
 */
int bibo_moe_exp_attn_res_fwd(const void* const* candidates, int n_candidates, const float* score_weight, float eps, int T, int H,
                          int dtype, void* out, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* BIBO_MOE_H */
