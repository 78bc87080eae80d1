// Kernels 3 and 4 in one launch: a workgroup takes 128 permuted rows of one expert through the gate/up
// projection, Radial NormSiLU and the down projection without the activations leaving the CU.
//
// Phase 1 (gate/up GEMM, 2 x 4 waves, v_mfma_f32_32x32x16_bf16, operands swapped so that a lane ends up with
// one ROW's values) walks K in steps of 64 elements, so every row an LDS-DMA instruction fetches is a whole
// 128-byte line: the L2 -> LDS path moves almost twice the bytes per second for whole lines than for the
// half lines of a 32-element step.  All 2I weight rows of a step would not fit LDS more than once, so a step
// is cut into I/128 sub-steps of 256 rows: sub-step t holds, for each of the four N waves, its t-th 32-column
// gate tile and the up tile of the same columns (16 MFMAs per wave).  The 32 KB stages form a ring of three (two
// where I < 384 meets blocks of 384 output columns, whose staging buffers leave no room): the rows of sub-step
// n + ring - 1 are requested while sub-step n is multiplied, and a wave waits only until the loads older than the
// latest sub-step's have landed (loads complete in order), so the L2 -> LDS path always has a stage or two in flight
// instead of draining at every barrier.  The x rows of step s+1 arrive during step s in a double buffer of their own
// (I = 384), or those of step s+2 in a ring of three (I < 384).
// Phase 2 turns the accumulators into bf16 activations and parks them in the stages, whose contents are dead by
// then, as an operand of the second GEMM: stage t holds columns [128t, 128t+128) of all 128 rows; row r keeps
// 16-byte granule c at position c ^ (r & 15), which spreads the 16 lanes of a fragment read over all banks
// although the row stride is 256 bytes.
// Phase 3 has no barriers and no LDS traffic for the weights: the eight waves split a block of 128*CT
// output columns (16*CT each), every wave multiplies ALL 128 resident rows with v_mfma_f32_16x16x32_bf16
// and pulls its own w_down rows straight from global memory into registers, up to three 128-byte K
// blocks ahead (the four lanes of a weight row fetch 64 contiguous bytes per instruction).  Keeping the
// in-flight bytes in registers instead of LDS is what lets a CU cover the memory latency here: the
// activations already fill most of the LDS.
// Each block of columns is scaled by the routing weight, staged through LDS 32 rows at a time (in the two x
// buffers, which are idle by then) and scattered to slot order as 256-byte row segments.
// A tile may hold fewer than 128 rows (an expert's last tile, or all of its rows).  32-row blocks without rows are
// not multiplied: the kernel body exists once per number of blocks (1 to 4), with the MFMAs, activations, down
// projection row tiles and output rounds of the missing blocks left out; every wave still issues its share of
// the weight requests.  A tile's duration hardly depends on its rows all the same (it is the stream of its
// expert's weights through one CU: 3-block tiles take as long as 4-block tiles), which is why cutting the tiles
// so that they fill whole rounds of the chip (512 tiles of 96 rows for the 410 of the prefill shape) gained nothing.
// Reference: BiBoFusedExperts.forward, src/modeling/ffn/moe.py:81-93.
#include <type_traits>

#include "stripe.h"

namespace bibo {
namespace {

template <int NT, int CT>
struct FusedShape {
  static constexpr int MT = 2, BM = 128, BK = 64;
  static constexpr int I = 128 * NT;
  static constexpr int BN2 = 128 * CT;                             // output columns per block: 8 waves x CT x 16
  // I = 384: the three stages are the three sub-steps of a K step and the x rows alternate between two buffers.
  // I < 384 with at most 256 output columns per block (kDeep): three stages all the same, walked round by the running
  // sub-step, and a third x buffer, so that x rows are requested two K steps ahead.  Otherwise two stages.
  static constexpr bool kDeep = NT < 3 && CT < 3;
  static constexpr int kRing = (NT == 3 || kDeep) ? 3 : 2;         // weight stages in LDS
  static constexpr int kDist = kRing - 1;                          // sub-steps between a stage's request and its use
  static constexpr int kStageRows = 256;                           // 4 N waves x (gate tile + up tile) x 32 rows
  static constexpr int kStageElems = kStageRows * BK;              // 32 KB = one [128][128] slice of the activations
  static constexpr int kAElems = BM * BK;                          // x rows of one K step
  static constexpr int kOutRows = 32;                              // rows of a column block staged at a time
  static constexpr int kOutElems = kOutRows * BN2;
  static constexpr int kXElems = kAElems > kOutElems ? kAElems : kOutElems;   // a buffer that serves as either
  static constexpr int kBInstr = kStageRows * (BK / 8) / 512;      // load instructions per thread and weight stage
  static_assert(kBInstr == 4 && BM * (BK / 8) == 2 * 512, "stage does not divide over the threads");
};

// LDS-DMA through a buffer descriptor: the address is descriptor base + 32-bit per-thread byte offset (one
// vector register) + a wave-uniform byte offset (scalar), so the loop keeps no 64-bit per-thread addresses.
__device__ __forceinline__ void dma16_buf(__amdgpu_buffer_rsrc_t rsrc, unsigned voff, unsigned soff, bf16_t* l) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_void*)l, 16, voff, soff, 0, 0);
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);   // raw buffer, 32-bit data format
}

// What one thread needs to request a weight stage and the x rows of a K step.
template <typename F>
struct SubLoader {
  __amdgpu_buffer_rsrc_t w_rsrc, x_rsrc;   // this expert's w_gate_up block; the hidden states
  unsigned b_voff;         // byte offset of this thread's row and granule inside an instruction's 64 rows
  unsigned b_soff;         // byte offset of the stage's first tile row, K offset included (uniform)
  unsigned bstep;          // bytes between the rows of consecutive instructions (uniform)
  bf16_t* b_dst;           // LDS stage
  unsigned a_voff[2];      // byte offsets of this thread's two token rows and granule
  unsigned a_soff;         // K offset in bytes (uniform)
  bf16_t* a_dst;           // LDS x stage
  int wave_elems;          // this wave's place in an instruction's LDS block, in elements (uniform: a scalar register,
                           // so that the LDS base of every transfer is formed by scalar instructions alone)
};

// The load instructions of one sub-step: the weight stage kDist sub-steps ahead and, in the first sub-step of a K
// step (WITH_A), the next step's x rows.  Shaped like StripeLoader so that stripe_step can spread them between its
// MFMAs.
template <typename F, bool WITH_A>
struct SubIssuer {
  const SubLoader<F>& d;
  static constexpr int kInstr = F::kBInstr + (WITH_A ? 2 : 0);
  template <int Q>
  __device__ __forceinline__ void issue(int, bf16_t*) const {
    if constexpr (Q < F::kBInstr) dma16_buf(d.w_rsrc, d.b_voff, d.b_soff + Q * d.bstep, d.b_dst + Q * 512 * 8 + d.wave_elems);
    else if constexpr (WITH_A && Q < F::kBInstr + 2)
      dma16_buf(d.x_rsrc, d.a_voff[Q - F::kBInstr], d.a_soff, d.a_dst + (Q - F::kBInstr) * 512 * 8 + d.wave_elems);
  }
};

// One 128-byte K block of a wave's 16*CT w_down rows as it comes from memory: lane l holds 16-byte piece l % 4 of
// the first (s = 0) or second (s = 1) 64 bytes of row l / 4 of column tile ct.  The four lanes of a row are
// ADJACENT, so the texture unit merges them into one 64-byte request; lanes that are 16 apart, as in the MFMA
// operand layout, are not merged and move less than half the bytes per second.
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
    b.w[ct][1] = *reinterpret_cast<const bf16x8*>(p + 32);
  }
}

// Memory order -> MFMA operand order: lane r + 16 g takes the register of lane 4 r + g (row r, piece g).  sel is
// 4 * (source lane); the exchange uses the LDS crossbar and no LDS memory.
__device__ __forceinline__ bf16x8 to_operand_lanes(bf16x8 v, int sel) {
  typedef int i32x4 __attribute__((ext_vector_type(4)));
  i32x4 u = __builtin_bit_cast(i32x4, v);
#pragma unroll
  for (int i = 0; i < 4; ++i) u[i] = __builtin_amdgcn_ds_bpermute(sel, u[i]);
  return __builtin_bit_cast(bf16x8, u);
}

// MODE 0: the forward pass.  MODE 1: the backward pass's recomputation - the kernel stops after phase 1 and writes the
// pre-activations themselves, rounded to bf16, to `preact` [S, 2I] in permuted row order (gate columns, then up
// columns), staged through the LDS stages into whole row segments.  MODE 2: the training forward - the forward pass that
// also leaves those pre-activations for its backward, in the same way (8-byte stores straight from the accumulator
// registers during phase 2 were slower: 140 against 133 us at T = 8192).
template <int NT, int CT, int MODE = 0>
__global__ __launch_bounds__(512) void experts_fused_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ wgu,
                                                            const bf16_t* __restrict__ wd,
                                                            const float* __restrict__ theta,
                                                            const float* __restrict__ w,
                                                            const int32_t* __restrict__ offsets,
                                                            const int32_t* __restrict__ perm_slot,
                                                            const int32_t* __restrict__ perm_token, int H, int E,
                                                            int act, unsigned x_bytes, bf16_t* __restrict__ yw,
                                                            bf16_t* __restrict__ preact) {
  using F = FusedShape<NT, CT>;
  constexpr int MT = F::MT, BM = F::BM, I = F::I, BK = F::BK;
  // Every buffer that is read while LDS-DMA fills another is a variable of its own: the compiler orders a DMA
  // transfer against later LDS reads of the same variable with a full wait for the transfer.
  __shared__ __attribute__((aligned(16))) bf16_t S0[F::kStageElems];  // weight stages, then the activations
  __shared__ __attribute__((aligned(16))) bf16_t S1[F::kStageElems];
  __shared__ __attribute__((aligned(16))) bf16_t S2[F::kRing == 3 ? F::kStageElems : 8];
  __shared__ __attribute__((aligned(16))) bf16_t A0[F::kXElems];      // x rows of even K steps; then output staging,
  __shared__ __attribute__((aligned(16))) bf16_t A1[F::kXElems];      // x rows of odd K steps;  alternating per 32 rows
  __shared__ __attribute__((aligned(16))) bf16_t A2[F::kDeep ? F::kAElems : 8];   // kDeep: x rows of every third K step
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
  const int nblocks = (rows + 31) >> 5;                 // 32-row blocks that hold rows: 1 .. 4

  // The rest of the kernel exists once per number of blocks, chosen here, where nothing is alive yet: the copies
  // share no values, so each gets the registers the kernel would get if it were the only one.
  auto body = [&](auto nblocks_c) {
  constexpr int kBlocks = decltype(nblocks_c)::value;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int wn = wave & 3, wm = wave >> 2;
  // M wave wm owns blocks 2 wm and 2 wm + 1; blocks without rows are not multiplied.  The two waves of a SIMD
  // belong to different M waves, so what a SIMD's MFMA pipe has to do goes with the tile's blocks either way.
  static_assert(MT == 2, "two blocks per M wave");
  const int my_blocks = __builtin_amdgcn_readfirstlane(wm == 0 ? (kBlocks < 2 ? kBlocks : 2) : (kBlocks > 2 ? kBlocks - 2 : 0));
  const int n = lane & 31;
  const int mbase = wm * MT * 32;
  auto stage = [&](auto ic) -> bf16_t* {
    constexpr int i = decltype(ic)::value;
    if constexpr (i == 0) return S0; else if constexpr (i == 1) return S1; else return S2;
  };

  // ---- phase 1: gate/up projection (moe.py:81-86) ----
  floatx16 acc[MT][2 * NT];               // [..][0..NT) gate tiles, [..][NT..2NT) the up tiles of the same columns
  {
    // DMA side: thread t of an instruction fills granule t (row t/8, position t%8) of its 64 rows and fetches
    // logical granule (t%8) ^ ((row >> 1) & 7) of that row: granule c of a stage row sits at c ^ ((row >> 1) & 7).
    // Stage row (wn*2 + gu)*32 + r of sub-step t is weight row gu*I + (wn*NT + t)*32 + r: instruction q = wn.
    const int chunk = (tid & 7) ^ ((tid >> 4) & 7);
    const int drow = tid >> 3;
    const unsigned hb = (unsigned)H * sizeof(bf16_t);                            // bytes per weight / hidden-state row
    const int nsteps = H / BK;
    SubLoader<F> ld;
    ld.w_rsrc = make_rsrc(wgu + (size_t)e * 2 * I * H, 2u * I * hb);
    ld.x_rsrc = make_rsrc(x, x_bytes);
    ld.b_voff = ((unsigned)((drow >> 5) * I + (drow & 31))) * hb + chunk * 16;
    ld.bstep = (unsigned)NT * 32 * hb;
    ld.wave_elems = __builtin_amdgcn_readfirstlane(wave) * 64 * 8;
#pragma unroll
    for (int a = 0; a < 2; ++a) {
      const int m = min(a * 64 + drow, rows - 1);                                // rows past the end re-read the last valid row
      ld.a_voff[a] = (unsigned)perm_token[row0 + m] * hb + chunk * 16;          // gather, moe.py:81
    }
    const int pos0 = ((lane >> 5) ^ ((n >> 1) & 7)) * 8;    // fragment side: lane (n, h) reads logical granule 2*ss + h of rows congruent to n mod 32
    auto frag_row = [&](int j) { return (wn * 2 + j) * 32; };
    using std::integral_constant;
    auto zero_acc = [&]() {                      // (after the prologue's requests, which do not wait for it)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int j = 0; j < 2 * NT; ++j)
#pragma unroll
          for (int i = 0; i < 16; ++i) acc[mt][j][i] = 0.f;
    };
    if constexpr (F::kDeep) {
      // Sub-step g = s NT + t reads stage g % 3 and x buffer s % 3, and requests the weight rows of sub-step g + 2
      // and, at t = 0, the x rows of step s + 2 (K steps clamped to the last one: requests past the end fetch valid
      // rows into buffers nobody reads again).  The K loop is unrolled by three steps (ph = s % 3), so every buffer is
      // chosen at compile time.  What a sub-step may leave in flight are the loads of the sub-step before it.
      auto abuf = [&](auto ic) -> bf16_t* {
        constexpr int i = decltype(ic)::value;
        if constexpr (i == 0) return A0; else if constexpr (i == 1) return A1; else return A2;
      };
      constexpr unsigned kb = BK * sizeof(bf16_t);
      // prologue, oldest first: sub-step 0, x rows of steps 0 and 1, sub-step 1
#pragma unroll
      for (int q = 0; q < F::kBInstr; ++q) dma16_buf(ld.w_rsrc, ld.b_voff, q * ld.bstep, S0 + q * 512 * 8 + ld.wave_elems);
#pragma unroll
      for (int a = 0; a < 2; ++a) dma16_buf(ld.x_rsrc, ld.a_voff[a], 0, A0 + a * 512 * 8 + ld.wave_elems);
#pragma unroll
      for (int a = 0; a < 2; ++a) dma16_buf(ld.x_rsrc, ld.a_voff[a], kb, A1 + a * 512 * 8 + ld.wave_elems);
#pragma unroll
      for (int q = 0; q < F::kBInstr; ++q)
        dma16_buf(ld.w_rsrc, ld.b_voff, (NT == 1 ? kb : 32 * hb) + q * ld.bstep, S1 + q * 512 * 8 + ld.wave_elems);
      zero_acc();
      auto substep = [&](auto mc, auto phc, auto tc, int s) {
        constexpr int nmt = decltype(mc)::value;
        constexpr int ph = decltype(phc)::value, t = decltype(tc)::value;
        constexpr int cur = (ph * NT + t) % 3, target = (ph * NT + t + 2) % 3;
        constexpr int tn = (t + 2) % NT, ds = (t + 2) / NT;
        constexpr bool after_t0 = NT == 1 || t == 1;                   // the sub-step before also requested x rows
        sync_keep_loads<F::kBInstr + (after_t0 ? 2 : 0)>();
        const bf16_t* a0 = abuf(integral_constant<int, ph>{}) + (mbase + n) * BK + pos0;
        const bf16_t* b0 = stage(integral_constant<int, cur>{}) + n * BK;
        ld.b_soff = (unsigned)tn * 32 * hb + (unsigned)min(s + ds, nsteps - 1) * kb;
        ld.b_dst = stage(integral_constant<int, target>{});
        ld.a_soff = (unsigned)min(s + 2, nsteps - 1) * kb;
        ld.a_dst = abuf(integral_constant<int, (ph + 2) % 3>{});
        const SubIssuer<F, t == 0> issuer{ld};
        if constexpr (nmt > 0)
          stripe_step<nmt, 2, BK, true, 2 * NT, t, NT>(acc, a0, 32 * BK, b0, pos0, frag_row, issuer, true, 0, nullptr);
        else
          issue_some<0, SubIssuer<F, t == 0>::kInstr>(issuer, 0, nullptr);
      };
      auto kstep = [&](auto mc, auto phc, int s) {
        substep(mc, phc, integral_constant<int, 0>{}, s);
        if constexpr (NT > 1) substep(mc, phc, integral_constant<int, 1>{}, s);
      };
      auto kloop = [&](auto mc) {
        for (int s = 0; s < nsteps; s += 3) {
          kstep(mc, integral_constant<int, 0>{}, s);
          if (s + 1 < nsteps) kstep(mc, integral_constant<int, 1>{}, s + 1);
          if (s + 2 < nsteps) kstep(mc, integral_constant<int, 2>{}, s + 2);
        }
      };
      if (my_blocks == 2) kloop(integral_constant<int, 2>{});
      else if (my_blocks == 1) kloop(integral_constant<int, 1>{});
      else kloop(integral_constant<int, 0>{});
    } else {
    // what sub-step (s, t) requests: the weight rows of sub-step (s, t) + kDist (its K step clamped to the last
    // one: requests past the end fetch valid rows into a stage nobody reads again), and at t = 0 the x rows of
    // step s + 1.  Every sub-step issues the same number of loads, so the wait counts below are constants.
    auto request = [&](auto tc, auto pc, int s) {
      constexpr int t = decltype(tc)::value, par = decltype(pc)::value;
      constexpr int tn = (t + F::kDist) % NT, ds = (t + F::kDist) / NT;
      constexpr int target = NT == 1 ? (par + ds) % 2 : tn;
      ld.b_soff = (unsigned)tn * 32 * hb + (unsigned)min(s + ds, nsteps - 1) * (unsigned)(BK * sizeof(bf16_t));
      ld.b_dst = stage(std::integral_constant<int, target>{});
      ld.a_soff = (unsigned)min(s + 1, nsteps - 1) * (unsigned)(BK * sizeof(bf16_t));
      ld.a_dst = par ? A0 : A1;
    };
    // prologue: the first kDist sub-steps' weight rows and the x rows of step 0 (weight rows first: they do not wait
    // for the row indices)
#pragma unroll
    for (int q = 0; q < F::kBInstr; ++q) dma16_buf(ld.w_rsrc, ld.b_voff, q * ld.bstep, S0 + q * 512 * 8 + ld.wave_elems);
    dma16_buf(ld.x_rsrc, ld.a_voff[0], 0, A0 + ld.wave_elems);
    dma16_buf(ld.x_rsrc, ld.a_voff[1], 0, A0 + 512 * 8 + ld.wave_elems);
    if constexpr (F::kDist == 2) {
#pragma unroll
      for (int q = 0; q < F::kBInstr; ++q)
        dma16_buf(ld.w_rsrc, ld.b_voff, 32 * hb + q * ld.bstep, S1 + q * 512 * 8 + ld.wave_elems);   // sub-step (0, 1)
    }
    zero_acc();
    auto substep = [&](auto mc, auto tc, auto pc, int s) {
      constexpr int nmt = decltype(mc)::value;           // M tiles of this wave that hold rows
      constexpr int t = decltype(tc)::value, par = decltype(pc)::value;
      constexpr int cur = NT == 1 ? par : t;
      // loads still allowed in flight: those of the sub-steps after the one whose stage is read now
      if constexpr (F::kDist == 1) sync_keep_loads<0>();
      else if constexpr (t == 1) sync_keep_loads<F::kBInstr + 2>();     // the sub-step before (t = 0) also requested x rows
      else sync_keep_loads<F::kBInstr>();
      const bf16_t* a0 = (par ? A1 : A0) + (mbase + n) * BK + pos0;
      const bf16_t* b0 = stage(std::integral_constant<int, cur>{}) + n * BK;
      request(tc, pc, s);
      const SubIssuer<F, t == 0> issuer{ld};
      if constexpr (nmt > 0)
        stripe_step<nmt, 2, BK, true, 2 * NT, t, NT>(acc, a0, 32 * BK, b0, pos0, frag_row, issuer, true, 0, nullptr);
      else
        issue_some<0, SubIssuer<F, t == 0>::kInstr>(issuer, 0, nullptr);   // its share of the requests all the same
    };
    // one copy of the K loop per number of M tiles with rows, chosen once: a choice inside the loop would meet at
    // every sub-step with all 192 accumulator registers alive
    auto kloop = [&](auto mc) {
      for (int s = 0; s < nsteps; s += 2) {                                       // H / BK is even
        substep(mc, integral_constant<int, 0>{}, integral_constant<int, 0>{}, s);
        if constexpr (NT > 1) substep(mc, integral_constant<int, 1>{}, integral_constant<int, 0>{}, s);
        if constexpr (NT > 2) substep(mc, integral_constant<int, 2>{}, integral_constant<int, 0>{}, s);
        substep(mc, integral_constant<int, 0>{}, integral_constant<int, 1>{}, s + 1);
        if constexpr (NT > 1) substep(mc, integral_constant<int, 1>{}, integral_constant<int, 1>{}, s + 1);
        if constexpr (NT > 2) substep(mc, integral_constant<int, 2>{}, integral_constant<int, 1>{}, s + 1);
      }
    };
    static_assert(MT == 2, "the three copies below are 2, 1 and 0 M tiles");
    if (my_blocks == 2) kloop(integral_constant<int, 2>{});
    else if (my_blocks == 1) kloop(integral_constant<int, 1>{});
    else kloop(integral_constant<int, 0>{});
      }
  }
  wait_loads_and_sync();                   // every transfer has landed and every wave is done with the stages

  if constexpr (MODE != 0) {
    // gate half, then up half: accumulators -> the stages in the activation layout (stage t = columns [128 t, 128 t + 128)
    // of the half, granule c of row m at c ^ (m & 15)) -> whole 256-byte row segments to memory
    const int hh = lane >> 5;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        if (mt >= my_blocks) continue;
        const int m = mbase + mt * 32 + n;
#pragma unroll
        for (int j = 0; j < NT; ++j) {
          const int tile32 = wn * NT + j;
          bf16_t* hrow = ((tile32 >> 2) == 0 ? S0 : ((tile32 >> 2) == 1 ? S1 : S2)) + m * 128 + 4 * hh;
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            bf16x4 hv;
#pragma unroll
            for (int r = 0; r < 4; ++r) hv[r] = (bf16_t)acc[mt][half * NT + j][4 * q + r];
            const int c = (tile32 & 3) * 4 + q;
            *reinterpret_cast<bf16x4*>(hrow + (c ^ (m & 15)) * 8) = hv;
          }
        }
      }
      __syncthreads();
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const bf16_t* slice = t == 0 ? S0 : (t == 1 ? S1 : S2);
        for (int g = tid; g < BM * 16; g += 512) {
          const int m = g >> 4, pos = g & 15;
          if (m < rows)
            *reinterpret_cast<u32x4*>(preact + (size_t)(row0 + m) * (2 * I) + half * I + t * 128 + ((pos ^ (m & 15)) * 8)) =
                *reinterpret_cast<const u32x4*>(slice + m * 128 + pos * 8);
        }
      }
      __syncthreads();                     // the stages are free for the other half
    }
    if constexpr (MODE == 1) return;
  }

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
  // phase 3 streams w_down through registers; its first K blocks are requested here, between the two M tiles of
  // the activation: the accumulators of the first tile are dead by then and make room, and the loads fly during
  // the rest of the activation arithmetic
  constexpr int KB = I / 64;                 // 128-byte K blocks
  const size_t tile_stride = (size_t)16 * I;
  const bf16_t* wp = wd + ((size_t)e * H + wave * (16 * CT) + (lane >> 2)) * I + (lane & 3) * 8;
  constexpr int D = KB > 3 ? 3 : KB - 1;      // K blocks requested ahead of the one being multiplied
  constexpr int NB = D + 1;
  WBlock<CT> wb[NB];
  {
    // stage t holds activation columns [128t, 128t + 128) of all 128 rows, [128][128], granules swizzled
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      if (mt == MT - 1) {
#pragma unroll
        for (int d = 0; d < D; ++d) load_wblock<CT>(wb[d], wp, tile_stride, d);
      }
      if (mt >= my_blocks) continue;          // a block without rows: nobody reads its activations
      const int m = mbase + mt * 32 + n;
      const float rinv = rinv_s[m];
      const float nrl = -1.44269504f * rinv, rg = rinv * gain_s[m];            // per-row constants folded once
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        const int tile32 = wn * NT + j;      // 32-column tile of the activation row: slice tile32 / 4, granules (tile32 % 4) * 4 + q
        bf16_t* hrow = ((tile32 >> 2) == 0 ? S0 : ((tile32 >> 2) == 1 ? S1 : S2)) + m * 128 + 4 * hh;
#pragma unroll
        for (int q = 0; q < 4; ++q) {        // columns tile32*32 + 8*q + 4*hh + 0..3: half of a granule
          bf16x4 hv;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float g = acc[mt][j][4 * q + r];
            const float sg = __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(g * nrl));   // sigmoid(g/r)
            hv[r] = (bf16_t)(g * rg * sg * acc[mt][NT + j][4 * q + r]);                // SiLU(g/r) r^p up
          }
          const int c = (tile32 & 3) * 4 + q;
          *reinterpret_cast<bf16x4*>(hrow + (c ^ (m & 15)) * 8) = hv;
        }
      }
    }
  }
  __syncthreads();                         // the activation tile is complete

  // ---- phase 3: down projection, routing weight, scatter to slot order (moe.py:92-93) ----
  const int r16 = lane & 15, g4 = lane >> 4;
  const int nblk = H / F::BN2;
  const int sel = 4 * (4 * r16 + g4);
  // One block of F::BN2 output columns for the first NRT 16-row tiles of the tile (NRT = 2 per block that holds rows).
  auto down_block = [&](auto nrt_c, int nb) {
    constexpr int NRT = decltype(nrt_c)::value;
    const int n0 = nb * F::BN2;
    floatx4 acc2[CT][NRT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
      for (int rt = 0; rt < NRT; ++rt) acc2[ct][rt] = floatx4{0.f, 0.f, 0.f, 0.f};
    // Activation fragments are read a row tile ahead of the MFMAs that consume them (across K block
    // boundaries too).
    auto frag = [&](int kb, int rt, int s) {
      // K elements 64 kb + 32 s + 8 g4 .. + 8 of row 16 rt + r16: slice kb / 2, granule (kb % 2) * 8 + 4 s + g4
      const int gq = ((((kb & 1) * 8 + g4) ^ r16) * 8) ^ (s * 32);
      const bf16_t* slice = (kb >> 1) == 0 ? S0 : ((kb >> 1) == 1 ? S1 : S2);
      return *reinterpret_cast<const bf16x8*>(slice + (rt * 16 + r16) * 128 + gq);
    };
    // The multiply walks half K blocks (32 elements, one MFMA deep): while half hs is multiplied with all NRT
    // row tiles, the weights of half hs + 1 change lanes and the activation fragment of the next row tile is read.
    bf16x8 wc[2][CT], xa[2];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) wc[0][ct] = to_operand_lanes(wb[0].w[ct][0], sel);
    xa[0] = frag(0, 0, 0);
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
      if (kb + D < KB) load_wblock<CT>(wb[(kb + D) % NB], wp, tile_stride, kb + D);
      __builtin_amdgcn_sched_barrier(0);     // keep the loads D blocks ahead of their use
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const int hs = 2 * kb + s;
#pragma unroll
        for (int rt = 0; rt < NRT; ++rt) {
          const int g = hs * NRT + rt;         // running (half K block, row tile) index
          if (g + 1 < KB * 2 * NRT) xa[(g + 1) & 1] = frag(((g + 1) / NRT) >> 1, (g + 1) % NRT, ((g + 1) / NRT) & 1);
          // the CT lane exchanges of the next half are spread over the row tiles (the last tile takes what is left)
#pragma unroll
          for (int cx = 0; cx < CT; ++cx)
            if ((cx == rt || (rt == NRT - 1 && cx > rt)) && hs + 1 < 2 * KB)
              wc[(hs + 1) & 1][cx] = to_operand_lanes(wb[((hs + 1) >> 1) % NB].w[cx][(hs + 1) & 1], sel);
#pragma unroll
          for (int ct = 0; ct < CT; ++ct)
            acc2[ct][rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wc[hs & 1][ct], xa[g & 1], acc2[ct][rt], 0, 0, 0);
        }
      }
    }
    wp += (size_t)F::BN2 * I;                                  // next block of columns: in flight during the epilogue
    if (nb + 1 < nblk) {
#pragma unroll
      for (int d = 0; d < D; ++d) load_wblock<CT>(wb[d], wp, tile_stride, d);
    }
    __builtin_amdgcn_sched_barrier(0);
    // accumulator: lane holds row 16*rt + r16, columns wave*16*CT + 16*ct + 4*g4 + i.  The block leaves 32 rows at
    // a time through the two x buffers in turn; between two barriers a wave stages the next 32 rows into one
    // buffer and copies the previous 32 out of the other.  Staged row r keeps granule c at position c ^ (r & 15): the 8-byte writes of a half wave
    // then cover all banks.  Copy-out: 16 consecutive threads move 256 contiguous bytes of one row.
    // (The thread index goes through an empty asm so the staging addresses are formed here, per block,
    // instead of being hoisted out of the loop and kept alive across the multiply.)
    int tid_o = tid;
    asm volatile("" : "+v"(tid_o));
    const int r16o = tid_o & 15, g4o = (tid_o >> 4) & 3;
    const int ro = tid_o >> 4, pco = tid_o & 15;             // copy-out: staged row, first granule position
    auto stage_rows = [&](int hf) {          // rows 32 hf .. + 32 of the block into buffer hf % 2
      bf16_t* const O = (hf & 1) ? A1 : A0;
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
    };
    auto copy_out = [&](int hf) {
      const bf16_t* const O = (hf & 1) ? A1 : A0;
      const int m = hf * F::kOutRows + ro;
      if (m < rows) {
        bf16_t* dst = yw + (size_t)slot_s[m] * H + n0;
        const bf16_t* src = O + ro * F::BN2;
#pragma unroll
        for (int q = 0; q < CT; ++q) {                         // 16 CT granules per row, 16 threads per row
          const int pc = pco + 16 * q;
          *reinterpret_cast<u32x4*>(dst + (pc ^ (ro & 15)) * 8) = *reinterpret_cast<const u32x4*>(src + pc * 8);
        }
      }
    };
    constexpr int NR = NRT * 16 / F::kOutRows;
    stage_rows(0);
#pragma unroll
    for (int hf = 0; hf < NR; ++hf) {
      __syncthreads();                       // rows of round hf are staged; round hf - 1 has left its buffer
      if (hf + 1 < NR) stage_rows(hf + 1);
      copy_out(hf);
    }
  };
  for (int nb = 0; nb < nblk; ++nb) down_block(std::integral_constant<int, 2 * kBlocks>{}, nb);
  };   // body
  if (nblocks == 4) body(std::integral_constant<int, 4>{});
  else if (nblocks == 3) body(std::integral_constant<int, 3>{});
  else if (nblocks == 2) body(std::integral_constant<int, 2>{});
  else body(std::integral_constant<int, 1>{});
}


template <int NT, int CT>
void launch_fused_t(const bf16_t* x, const bf16_t* wgu, const bf16_t* wd, const float* theta, const float* w,
                    const int32_t* offsets, const int32_t* perm_slot, const int32_t* perm_token, int S, int H, int E,
                    int act, unsigned x_bytes, bf16_t* yw, bf16_t* preact, hipStream_t s) {
  const int grid = ((S / 128 + E + 7) & ~7) + 8;
  if (preact != nullptr)
    hipLaunchKernelGGL((experts_fused_kernel<NT, CT, 2>), dim3(grid), dim3(512), 0, s, x, wgu, wd, theta, w, offsets,
                       perm_slot, perm_token, H, E, act, x_bytes, yw, preact);
  else
    hipLaunchKernelGGL((experts_fused_kernel<NT, CT, 0>), dim3(grid), dim3(512), 0, s, x, wgu, wd, theta, w, offsets,
                       perm_slot, perm_token, H, E, act, x_bytes, yw, preact);
}

template <int NT>
void launch_fused_nt(const bf16_t* x, const bf16_t* wgu, const bf16_t* wd, const float* theta, const float* w,
                     const int32_t* offsets, const int32_t* perm_slot, const int32_t* perm_token, int S, int H, int E,
                     int act, unsigned x_bytes, bf16_t* yw, bf16_t* preact, hipStream_t s) {
  // (blocks of 256 columns leave room for the third x buffer of the deeper ring where I < 384)
  if (H % 384 == 0 && (NT == 3 || H % 256 != 0))
    launch_fused_t<NT, 3>(x, wgu, wd, theta, w, offsets, perm_slot, perm_token, S, H, E, act, x_bytes, yw, preact, s);
  else if (H % 256 == 0) launch_fused_t<NT, 2>(x, wgu, wd, theta, w, offsets, perm_slot, perm_token, S, H, E, act, x_bytes, yw, preact, s);
  else launch_fused_t<NT, 1>(x, wgu, wd, theta, w, offsets, perm_slot, perm_token, S, H, E, act, x_bytes, yw, preact, s);
}

template <int NT>
void launch_raw_nt(const bf16_t* x, const bf16_t* wgu, const int32_t* offsets, const int32_t* perm_token, int S, int H, int E,
                   unsigned x_bytes, bf16_t* gu, hipStream_t s) {
  const int grid = ((S / 128 + E + 7) & ~7) + 8;
  hipLaunchKernelGGL((experts_fused_kernel<NT, 1, 1>), dim3(grid), dim3(512), 0, s, x, wgu, nullptr, nullptr, nullptr,
                     offsets, nullptr, perm_token, H, E, 0, x_bytes, nullptr, gu);
}

}  // namespace

// Phase 1 of the fused kernel alone: gu[row] = [x W_gate^T, x W_up^T] in bf16 for every permuted row (what the backward
// pass recomputes, moe.py:84).  Same shapes as launch_experts_fused.
hipError_t launch_gateup_raw(const void* x, const void* wgu, const int32_t* offsets, const int32_t* perm_token, int T, int H,
                             int E, int k, int I, void* gu, hipStream_t s) {
  const int S = T * k;
  if (S == 0) return hipSuccess;
  if ((unsigned long long)T * H * sizeof(bf16_t) >= (1ull << 32)) return hipErrorInvalidValue;
  const unsigned xb = (unsigned)((size_t)T * H * sizeof(bf16_t));
  const bf16_t* xp = static_cast<const bf16_t*>(x);
  const bf16_t* gp = static_cast<const bf16_t*>(wgu);
  bf16_t* out = static_cast<bf16_t*>(gu);
  switch (I) {
    case 128: launch_raw_nt<1>(xp, gp, offsets, perm_token, S, H, E, xb, out, s); break;
    case 256: launch_raw_nt<2>(xp, gp, offsets, perm_token, S, H, E, xb, out, s); break;
    case 384: launch_raw_nt<3>(xp, gp, offsets, perm_token, S, H, E, xb, out, s); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

bool fused_supported(int H, int I, int dtype) {
  // the activation tile plus two weight stages have to fit 160 KB of LDS: I <= 384
  return dtype == BIBO_DTYPE_BF16 && H >= 128 && (H % 128) == 0 && (I == 128 || I == 256 || I == 384);
}

hipError_t launch_experts_fused(const void* x, const void* wgu, const void* wd, const float* theta, const float* w,
                                const int32_t* offsets, const int32_t* perm_slot, const int32_t* perm_token, int T,
                                int H, int E, int k, int I, int act, void* yw, void* preact, hipStream_t s) {
  const int S = T * k;
  if (S == 0) return hipSuccess;
  if ((unsigned long long)T * H * sizeof(bf16_t) >= (1ull << 32)) return hipErrorInvalidValue;   // 32-bit byte offsets into x
  const unsigned xb = (unsigned)((size_t)T * H * sizeof(bf16_t));
  const bf16_t* xp = static_cast<const bf16_t*>(x);
  const bf16_t* gp = static_cast<const bf16_t*>(wgu);
  const bf16_t* dp = static_cast<const bf16_t*>(wd);
  bf16_t* yp = static_cast<bf16_t*>(yw);
  bf16_t* pp = static_cast<bf16_t*>(preact);
  switch (I) {
    case 128: launch_fused_nt<1>(xp, gp, dp, theta, w, offsets, perm_slot, perm_token, S, H, E, act, xb, yp, pp, s); break;
    case 256: launch_fused_nt<2>(xp, gp, dp, theta, w, offsets, perm_slot, perm_token, S, H, E, act, xb, yp, pp, s); break;
    case 384: launch_fused_nt<3>(xp, gp, dp, theta, w, offsets, perm_slot, perm_token, S, H, E, act, xb, yp, pp, s); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

}  // namespace bibo
