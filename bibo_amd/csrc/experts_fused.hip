// Kernels 3 and 4 in one launch: a workgroup takes 128 permuted rows of one expert through the gate/up
// projection, Radial NormSiLU and the down projection without the activations leaving the CU.
//
// Phase 1 (gate/up GEMM, 2 x 4 waves, v_mfma_f32_32x32x16_bf16, operands swapped so that a lane ends up with
// one ROW's values) walks K in steps of 64 elements, so every row an LDS-DMA instruction fetches is a whole
// 128-byte line: the L2 -> LDS path moves almost twice the bytes per second for whole lines than for the
// half lines of a 32-element step.  A step of all 2I weight rows would not fit LDS twice, so a step is cut
// into a gate half and an up half: while the MFMAs multiply the I gate rows of step s from one buffer, the up
// rows of step s arrive in the other, then the gate rows of step s+1 in the first, and so on; the x rows of
// step s+1 arrive in two halves over the two sub-steps of step s.
// Phase 2 turns the accumulators into bf16 activations and parks them in LDS as an operand of the second
// GEMM: rows 0..63 live in B0, rows 64..127 in B1, whose contents are dead by then; row r keeps 16-byte
// granule c at position c ^ (r & 15), which spreads the 16 lanes of a fragment read over all banks although
// the row stride is a multiple of 256 bytes.
// Phase 3 has no barriers and no LDS traffic for the weights: the eight waves split a block of 128*CT
// output columns (16*CT each), every wave multiplies ALL 128 resident rows with v_mfma_f32_16x16x32_bf16
// and pulls its own w_down rows straight from global memory into registers, up to three 128-byte K
// blocks ahead (lane (r, g) takes bytes [32g, 32g+32) of each line of weight row r; the activation fragments
// are read with the same K permutation).  Keeping the in-flight bytes in registers instead of LDS is
// what lets a CU cover the memory latency here: the activations already fill most of the LDS.
// Each block of columns is scaled by the routing weight, staged through LDS 32 rows at a time and
// scattered to slot order as whole 16-byte row segments.
// Reference: BiBoFusedExperts.forward, src/modeling/ffn/moe.py:81-93.
#include "stripe.h"

namespace bibo {
namespace {

template <int NT, int CT>
struct FusedShape {
  static constexpr int MT = 2, WM = 2, BM = 128, BK = 64;
  static constexpr int I = 128 * NT;
  static constexpr int BN2 = 128 * CT;                             // output columns per block: 8 waves x CT x 16
  static constexpr int kHalfElems = 64 * I;                        // one weight half-stage = activations of one M half
  static constexpr int kAElems = BM * BK;                          // x rows of one K step
  static constexpr int kOutRows = 32;                              // rows of a column block staged at a time
  static constexpr int kOutElems = kOutRows * BN2;
  static constexpr int kBInstr = I * (BK / 8) / 512;               // load instructions per thread and weight half-stage
  static_assert(I * (BK / 8) % 512 == 0 && BM * (BK / 8) == 2 * 512, "stage does not divide over the threads");
};

// LDS-DMA through a buffer descriptor: the address is descriptor base + 32-bit per-thread byte offset (one
// vector register) + a wave-uniform byte offset (scalar), so the loop keeps no 64-bit per-thread addresses.
__device__ __forceinline__ void dma16_buf(__amdgpu_buffer_rsrc_t rsrc, unsigned voff, unsigned soff, bf16_t* l) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_void*)l, 16, voff, soff, 0, 0);
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);   // raw buffer, 32-bit data format
}

// The load instructions one thread issues during one sub-step: the next weight half-stage and half of the
// next step's x rows.  Shaped like StripeLoader so that stripe_step can spread them between its MFMAs.
template <typename F>
struct SubLoader {
  __amdgpu_buffer_rsrc_t w_rsrc, x_rsrc;   // this expert's w_gate_up block; the hidden states
  unsigned b_voff;         // byte offset of this thread's row and granule inside the first instruction's 64 rows
  unsigned b_soff;         // byte offset of the half-stage to fetch, K offset included (uniform)
  unsigned bstep;          // bytes between the rows of consecutive instructions (uniform)
  bf16_t* b_dst;           // LDS half-stage
  unsigned a_voff;         // byte offset of this thread's token row and granule
  unsigned a_soff;         // K offset in bytes (uniform)
  bf16_t* a_dst;           // LDS position of that instruction's granules
  static constexpr int kInstr = F::kBInstr + 1;
  template <int Q>
  __device__ __forceinline__ void issue(int, bf16_t*) const {
    const int wave = threadIdx.x >> 6;
    if constexpr (Q < F::kBInstr) dma16_buf(w_rsrc, b_voff, b_soff + Q * bstep, b_dst + (Q * 512 + wave * 64) * 8);
    else if constexpr (Q == F::kBInstr) dma16_buf(x_rsrc, a_voff, a_soff, a_dst + wave * 64 * 8);
  }
};

// this lane's 32 bytes of one 128-byte K block for each of its CT weight tiles
#ifdef BIBO_P3_OLD
constexpr int W3_SECOND = 8, W3_LANE = 16;
#else
constexpr int W3_SECOND = 32, W3_LANE = 8;     // the four lanes of a row fetch 64 contiguous bytes per instruction
#endif
template <int CT>
struct WBlock {
  bf16x8 w[CT][2];
};

template <int CT>
__device__ __forceinline__ void load_wblock(WBlock<CT>& b, const bf16_t* __restrict__ wp, size_t tile_stride, int kb) {
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const bf16_t* p = wp + ct * tile_stride + kb * 64;
    b.w[ct][0] = *reinterpret_cast<const bf16x8*>(p);
    b.w[ct][1] = *reinterpret_cast<const bf16x8*>(p + W3_SECOND);
  }
}

template <int NT, int CT>
__global__ __launch_bounds__(512) void experts_fused_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ wgu,
                                                            const bf16_t* __restrict__ wd,
                                                            const float* __restrict__ theta,
                                                            const float* __restrict__ w,
                                                            const int32_t* __restrict__ offsets,
                                                            const int32_t* __restrict__ perm_slot,
                                                            const int32_t* __restrict__ perm_token, int H, int E,
                                                            int act, unsigned x_bytes, bf16_t* __restrict__ yw) {
  using F = FusedShape<NT, CT>;
  constexpr int MT = F::MT, BM = F::BM, I = F::I, BK = F::BK;
  __shared__ __attribute__((aligned(16))) bf16_t P[F::kHalfElems];    // weight half-stage 0, then activations of rows 0..63
  __shared__ __attribute__((aligned(16))) bf16_t Q[F::kHalfElems];    // weight half-stage 1, then activations of rows 64..127
  // Every buffer that is read while LDS-DMA fills another is a variable of its own: the compiler orders a DMA
  // transfer against later LDS reads of the same variable with a full wait for the transfer.
  __shared__ __attribute__((aligned(16))) bf16_t A0[F::kAElems];      // x rows of even K steps
  __shared__ __attribute__((aligned(16))) bf16_t A1[F::kAElems];      // x rows of odd K steps
  __shared__ __attribute__((aligned(16))) bf16_t O[F::kOutElems];     // output staging
  __shared__ float ssq[4 * BM];
  __shared__ float rinv_s[BM], gain_s[BM], w_s[BM];
  __shared__ int slot_s[BM];

  const TileMap tm = make_tile_map(offsets, E, BM);
  const int tile = xcd_tile(blockIdx.x, tm.total);
  if (tile >= tm.total) return;
  int e, row0, rows;
  find_tile(tm, offsets, BM, tile, e, row0, rows);
  e = __builtin_amdgcn_readfirstlane(e);                // the same for every lane: keep them in scalar registers
  row0 = __builtin_amdgcn_readfirstlane(row0);
  rows = __builtin_amdgcn_readfirstlane(rows);

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int wn = wave & 3, wm = wave >> 2;
  const int n = lane & 31;
  const int mbase = wm * MT * 32;

  // ---- phase 1: gate/up projection (moe.py:81-86) ----
  floatx16 acc[MT][2 * NT];               // [..][0..NT) gate tiles, [..][NT..2NT) the up tiles of the same columns
  {
    // DMA side: thread t of an instruction fills granule t (row t/8, position t%8) of its 64 rows and fetches
    // logical granule (t%8) ^ ((row >> 1) & 7) of that row: granule c of a stage row sits at c ^ ((row >> 1) & 7)
    const int chunk = (tid & 7) ^ ((tid >> 4) & 7);
    const int drow = tid >> 3;
    SubLoader<F> ld;
    ld.w_rsrc = make_rsrc(wgu + (size_t)e * 2 * I * H, 2u * I * H * sizeof(bf16_t));   // gate rows; the up rows are I further
    ld.x_rsrc = make_rsrc(x, x_bytes);
    const unsigned up_off = (unsigned)I * H * sizeof(bf16_t);
    ld.b_voff = ((unsigned)drow * H + chunk * 8) * sizeof(bf16_t);
    ld.bstep = 64u * H * sizeof(bf16_t);
    unsigned a_voff[2];
#pragma unroll
    for (int a = 0; a < 2; ++a) {
      const int m = min(a * 64 + drow, rows - 1);                                // rows past the end re-read the last valid row
      a_voff[a] = ((unsigned)perm_token[row0 + m] * H + chunk * 8) * sizeof(bf16_t);   // gather, moe.py:81
    }
    // prologue: gate half-stage and x rows of step 0 (weight rows first: they do not wait for the row indices)
#pragma unroll
    for (int q = 0; q < F::kBInstr; ++q) dma16_buf(ld.w_rsrc, ld.b_voff, q * ld.bstep, P + (q * 512 + wave * 64) * 8);
    dma16_buf(ld.x_rsrc, a_voff[0], 0, A0 + (wave * 64) * 8);
    dma16_buf(ld.x_rsrc, a_voff[1], 0, A0 + (512 + wave * 64) * 8);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int j = 0; j < 2 * NT; ++j)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[mt][j][i] = 0.f;
    // fragment side: lane (n, h) reads logical granule 2*ss + h of rows congruent to n mod 32
    const int pos0 = ((lane >> 5) ^ ((n >> 1) & 7)) * 8;
    auto frag_row = [&](int j) { return (wn * NT + j) * 32; };
    // one K step: x rows in `Acur`, the next step's go to `Anext`
    auto step = [&](const bf16_t* Acur, bf16_t* Anext, int k0, bool last) {
      const unsigned kb = (unsigned)k0 * sizeof(bf16_t);
      const unsigned kn = last ? kb : kb + BK * sizeof(bf16_t);                  // (the last step fetches its own x rows again: unused)
      const bf16_t* a0 = Acur + (mbase + n) * BK + pos0;
      // gate sub-step: multiplies P; the up rows of this step arrive in Q, rows 0..63 of the next x stage in Anext
      wait_loads_and_sync();
      ld.b_soff = up_off + kb; ld.b_dst = Q;
      ld.a_soff = kn; ld.a_voff = a_voff[0]; ld.a_dst = Anext;
      stripe_step<MT, NT, BK, true, 2 * NT, 0>(acc, a0, 32 * BK, P + n * BK, pos0, frag_row, ld, true, 0, nullptr);
      // up sub-step: multiplies Q; the gate rows of the next step arrive in P, rows 64..127 of the next x stage
      wait_loads_and_sync();
      ld.b_soff = kn; ld.b_dst = P;
      ld.a_voff = a_voff[1]; ld.a_dst = Anext + 512 * 8;
      stripe_step<MT, NT, BK, true, 2 * NT, NT>(acc, a0, 32 * BK, Q + n * BK, pos0, frag_row, ld, !last, 0, nullptr);
    };
    for (int k0 = 0; k0 < H; k0 += 2 * BK) {                                     // H / BK is even
      step(A0, A1, k0, false);
      step(A1, A0, k0 + BK, k0 + 2 * BK >= H);
    }
  }
  __syncthreads();                         // every wave is done with the gate/up stages

  // ---- phase 2: Radial NormSiLU (moe.py:87-92), activations to LDS ----
  // The accumulators are transposed (lane = row mbase + 32*mt + n, register i = column acc_row(i, lane) of
  // its 32-column tile), so a row's sum of gate^2 is a sum over this lane's registers, the lane with the
  // other half of the columns (lane ^ 32) and the four N waves; and every lane owns runs of four
  // consecutive columns, which leave as one 8-byte LDS write.
  const int hh = lane >> 5;
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
  __syncthreads();
  if (tid < BM) {
    const float p = radial_exponent(theta, e, act);                                   // moe.py:89
    const float ms = ((ssq[tid] + ssq[BM + tid]) + ssq[2 * BM + tid]) + ssq[3 * BM + tid];
    radial_row_scalars(ms, I, p, act, rinv_s[tid], gain_s[tid]);                      // 1/r and r^p, moe.py:88-89
    const int slot = perm_slot[row0 + min(tid, rows - 1)];
    slot_s[tid] = slot;
    w_s[tid] = w[slot];
  }
  __syncthreads();
  {
    bf16_t* hsel = wm ? Q : P;             // activations of this wave's M half, [64][I], granules swizzled
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int ml = mt * 32 + n;
      const float rinv = rinv_s[mbase + ml];
      const float nrl = -1.44269504f * rinv, rg = rinv * gain_s[mbase + ml];   // per-row constants folded once
      bf16_t* hrow = hsel + ml * I + 4 * hh;
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {        // columns (wn*NT + j)*32 + 8*q + 4*hh + 0..3: half of granule (wn*NT + j)*4 + q
          bf16x4 hv;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float g = acc[mt][j][4 * q + r];
            const float sg = __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(g * nrl));   // sigmoid(g/r)
            hv[r] = (bf16_t)(g * rg * sg * acc[mt][NT + j][4 * q + r]);                // SiLU(g/r) r^p up
          }
          const int c = (wn * NT + j) * 4 + q;
          *reinterpret_cast<bf16x4*>(hrow + (c ^ (ml & 15)) * 8) = hv;
        }
    }
  }
  __syncthreads();                         // the activation tile is complete

  // ---- phase 3: down projection, routing weight, scatter to slot order (moe.py:92-93) ----
  constexpr int KB = I / 64;                 // 128-byte K blocks
  constexpr int G = F::BN2 / 8;              // 16-byte granules per staged output row
  const int r16 = lane & 15, g4 = lane >> 4;
  const size_t tile_stride = (size_t)16 * I;
  // activation fragment of row tile rt, K block kb, half s: granule (8*kb + 2*g4 + s) ^ r16 of row 16*rt + r16
  const int nblk = H / F::BN2;
  const bf16_t* wp = wd + ((size_t)e * H + wave * (16 * CT) + r16) * I + g4 * W3_LANE;
  constexpr int D = KB > 3 ? 3 : KB - 1;      // K blocks requested ahead of the one being multiplied
  constexpr int NB = D + 1;
  WBlock<CT> wb[NB];
#pragma unroll
  for (int d = 0; d < D; ++d) load_wblock<CT>(wb[d], wp, tile_stride, d);
  for (int nb = 0; nb < nblk; ++nb) {
    const int n0 = nb * F::BN2;
    floatx4 acc2[CT][8];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
      for (int rt = 0; rt < 8; ++rt) acc2[ct][rt] = floatx4{0.f, 0.f, 0.f, 0.f};
    // Activation fragments are read a row tile ahead of the MFMAs that consume them (across K block
    // boundaries too).
    auto frag = [&](int kb, int rt, int s) {
#ifdef BIBO_P3_OLD
      const int gq = (((kb * 8 + 2 * g4) ^ r16) * 8) ^ (s * 8);
#else
      const int gq = (((kb * 8 + g4) ^ r16) * 8) ^ (s * 32);      // K elements 64 kb + 32 s + 8 g4 .. + 8 of the row
#endif
      return *reinterpret_cast<const bf16x8*>((rt < 4 ? P : Q) + ((rt & 3) * 16 + r16) * I + gq);
    };
    constexpr int AD = 1;                    // row tiles whose fragments are requested ahead (2 and 3 measured the same)
    bf16x8 xa[AD + 1][2];
#pragma unroll
    for (int g = 0; g < AD; ++g) {
      xa[g][0] = frag(g / 8, g % 8, 0);
      xa[g][1] = frag(g / 8, g % 8, 1);
    }
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
      if (kb + D < KB) load_wblock<CT>(wb[(kb + D) % NB], wp, tile_stride, kb + D);
      __builtin_amdgcn_sched_barrier(0);     // keep the loads D blocks ahead of their use
#pragma unroll
      for (int rt = 0; rt < 8; ++rt) {
        const int g = kb * 8 + rt;             // running (K block, row tile) index; fragments rotate through AD + 1 buffers
        if (g + AD < KB * 8) {
          xa[(g + AD) % (AD + 1)][0] = frag((g + AD) / 8, (g + AD) % 8, 0);
          xa[(g + AD) % (AD + 1)][1] = frag((g + AD) / 8, (g + AD) % 8, 1);
        }
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
          for (int ct = 0; ct < CT; ++ct)
            acc2[ct][rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wb[kb % NB].w[ct][s], xa[g % (AD + 1)][s], acc2[ct][rt], 0, 0, 0);
        if (g + AD < KB * 8) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 2 * CT, 0);
      }
    }
    wp += (size_t)F::BN2 * I;                                  // next block of columns: in flight during the epilogue
    if (nb + 1 < nblk) {
#pragma unroll
      for (int d = 0; d < D; ++d) load_wblock<CT>(wb[d], wp, tile_stride, d);
    }
    __builtin_amdgcn_sched_barrier(0);
    // accumulator: lane holds row 16*rt + r16, columns wave*16*CT + 16*ct + 4*g4 + i.  Staged row r keeps
    // granule c at position c ^ (r & 15): the 8-byte writes of a half wave then cover all banks.
    // (The thread index goes through an empty asm so the staging addresses are formed here, per block,
    // instead of being hoisted out of the loop and kept alive across the multiply.)
    int tid_o = tid;
    asm volatile("" : "+v"(tid_o));
    const int r16o = tid_o & 15, g4o = (tid_o >> 4) & 3;
#pragma unroll
    for (int hf = 0; hf < BM / F::kOutRows; ++hf) {
      __syncthreads();                       // the previous copy-out is done with O
#pragma unroll
      for (int rq = 0; rq < F::kOutRows / 16; ++rq) {
        const int rt = hf * (F::kOutRows / 16) + rq;
        const float ws = w_s[rt * 16 + r16o];                                            // moe.py:93
        bf16_t* orow = O + (rq * 16 + r16o) * F::BN2 + (g4o & 1) * 4;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
          const int c = wave * (2 * CT) + ct * 2 + (g4o >> 1);
          bf16x4 v;
#pragma unroll
          for (int i = 0; i < 4; ++i) v[i] = (bf16_t)(ws * acc2[ct][rt][i]);
          *reinterpret_cast<bf16x4*>(orow + (c ^ r16o) * 8) = v;
        }
      }
      __syncthreads();
#pragma unroll
      for (int q = 0; q < F::kOutRows * G / 512; ++q) {
        const int idx = q * 512 + tid_o;
        const int r = idx / G, pc = idx - r * G;
        const int m = hf * F::kOutRows + r;
        if (m < rows)
          *reinterpret_cast<u32x4*>(yw + (size_t)slot_s[m] * H + n0 + (pc ^ (r & 15)) * 8) =
              *reinterpret_cast<const u32x4*>(O + r * F::BN2 + pc * 8);
      }
    }
  }
}

template <int NT, int CT>
void launch_fused_t(const bf16_t* x, const bf16_t* wgu, const bf16_t* wd, const float* theta, const float* w,
                    const int32_t* offsets, const int32_t* perm_slot, const int32_t* perm_token, int S, int H, int E,
                    int act, unsigned x_bytes, bf16_t* yw, hipStream_t s) {
  const int grid = ((S / 128 + E + 7) & ~7) + 8;
  hipLaunchKernelGGL((experts_fused_kernel<NT, CT>), dim3(grid), dim3(512), 0, s, x, wgu, wd, theta, w, offsets,
                     perm_slot, perm_token, H, E, act, x_bytes, yw);
}

template <int NT>
void launch_fused_nt(const bf16_t* x, const bf16_t* wgu, const bf16_t* wd, const float* theta, const float* w,
                     const int32_t* offsets, const int32_t* perm_slot, const int32_t* perm_token, int S, int H, int E,
                     int act, unsigned x_bytes, bf16_t* yw, hipStream_t s) {
  if (H % 384 == 0) launch_fused_t<NT, 3>(x, wgu, wd, theta, w, offsets, perm_slot, perm_token, S, H, E, act, x_bytes, yw, s);
  else if (H % 256 == 0) launch_fused_t<NT, 2>(x, wgu, wd, theta, w, offsets, perm_slot, perm_token, S, H, E, act, x_bytes, yw, s);
  else launch_fused_t<NT, 1>(x, wgu, wd, theta, w, offsets, perm_slot, perm_token, S, H, E, act, x_bytes, yw, s);
}

}  // namespace

bool fused_supported(int H, int I, int dtype) {
  // the activation tile plus two weight stages have to fit 160 KB of LDS: I <= 384
  return dtype == BIBO_DTYPE_BF16 && H >= 128 && (H % 128) == 0 && (I == 128 || I == 256 || I == 384);
}

hipError_t launch_experts_fused(const void* x, const void* wgu, const void* wd, const float* theta, const float* w,
                                const int32_t* offsets, const int32_t* perm_slot, const int32_t* perm_token, int T,
                                int H, int E, int k, int I, int act, void* yw, hipStream_t s) {
  const int S = T * k;
  if (S == 0) return hipSuccess;
  if ((unsigned long long)T * H * sizeof(bf16_t) >= (1ull << 32)) return hipErrorInvalidValue;   // 32-bit byte offsets into x
  const unsigned xb = (unsigned)((size_t)T * H * sizeof(bf16_t));
  const bf16_t* xp = static_cast<const bf16_t*>(x);
  const bf16_t* gp = static_cast<const bf16_t*>(wgu);
  const bf16_t* dp = static_cast<const bf16_t*>(wd);
  bf16_t* yp = static_cast<bf16_t*>(yw);
  switch (I) {
    case 128: launch_fused_nt<1>(xp, gp, dp, theta, w, offsets, perm_slot, perm_token, S, H, E, act, xb, yp, s); break;
    case 256: launch_fused_nt<2>(xp, gp, dp, theta, w, offsets, perm_slot, perm_token, S, H, E, act, xb, yp, s); break;
    case 384: launch_fused_nt<3>(xp, gp, dp, theta, w, offsets, perm_slot, perm_token, S, H, E, act, xb, yp, s); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

}  // namespace bibo
