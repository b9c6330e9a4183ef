// Fused SageAttention forward kernel for gfx950 (MI355X).
//
// Replaces _attention_kernel of backends/_hygon/ops/sageattention/sageattention_triton.py:45-129
// (INT8 Q.K^T, fp32 base-2 online softmax, P.V with fp32 accumulation, O/l epilogue, LSE2) and adds
// causal block skipping, tail masking, FP8 P.V and packed variable-length batches.
//
// Mapping to the hardware
//   * A workgroup of NW wavefronts owns a q-tile of BM = 32*NW rows of one (batch, q-head); each
//     wavefront owns 32 query rows for the whole KV loop.
//   * Everything is computed TRANSPOSED so that a query row lives in one lane column:
//       S^T[n, m] = K[n, :] . Q[m, :]      v_mfma_i32_32x32x32_i8      A = K tile (LDS), B = Q (regs)
//       O^T[d, m] = V^T[d, n] . P^T[n, m]   v_mfma_f32_32x32x64_f8f6f4  A = V panel (LDS), B = P (regs)
//                                       or  v_mfma_f32_32x32x16_f16
//     In the 32x32 accumulator layout lane (m = lane%32, h = lane/32) holds column m, rows
//     8*(r/4) + 4*h + r%4.  So row max / row sum of query row m are in-lane reductions plus ONE
//     exchange with lane m+32 (v_permlane32_swap), the probabilities are already laid out as the
//     B operand of the second MFMA (V panels are pre-permuted to match, see sage_common.h), and the
//     running rescale / final 1/l multiply the lane's own accumulators.
//   * The INT32 accumulators start from the bit pattern of 1.5*2^23, so reading them as floats gives
//     12582912 + dot exactly: the int->float conversion is folded into the one FMA that applies
//     q_scale*k_scale and subtracts the running maximum.
//   * The running maximum is only moved when it grows by more than a threshold (lazy rescale).  The exact-exponential
//     kernels store P with a static 2^pshift so that fp8's range [2^-9, 448] is used; the FP8 kernels without LSE or an
//     explicit mask code P per (query row, 128-key tile) against the tile's own maximum (linear-mantissa e4m3 codes, no
//     v_exp_f32) and hand the tile's power of two to the P.V MFMA as its E8M0 scale operand, so every tile uses the top
//     of the code range however far it lies under the running maximum; their row sums come from the matrix pipe, unscaled
//     per tile, and are folded into the running sum with one multiply by that power of two.
//   * The tile decode (workgroup index -> head, tier, q-tile) divides by run-time values with host-made multiply-high
//     dividers (sage_launch.h: FastDiv); the first K and V tiles are requested before the Q loads.
//   * K/V tiles go global -> LDS directly (buffer_load ... lds, no registers): four slots per stream and
//     requests two tile periods ahead for FP8 P.V, two slots and one period for FP16 P.V.  The raw q-tile of
//     the variants that quantise their own Q and the V scales of the epilogue arrive the same way, and the
//     output leaves through an LDS transposition as whole rows.
//   * The wavefronts of a workgroup form two groups that run half a tile apart: while one group feeds the
//     matrix pipe (P.V of its last tile, Q.K^T of its next) the other runs the softmax of the tile in
//     between on the vector ALU.  Wavefronts w and w+4 share a SIMD and are in different groups, so each
//     SIMD always has matrix work and vector work to overlap.  One barrier per tile period hands the tile
//     slots over; the FP16 P.V kernels keep a second one in the middle of the period (their two slots are
//     what it protects the pace of), the FP8 P.V kernels, with four slots, run their two halves unsynchronised.
#pragma once
#include "sage_launch.h"
#include <atomic>
#include <cstdlib>
// Tuning constants of the matrix phase (measured: one more or one fewer fragment ahead is within +-1 %).
#define SAGE_KPF 4   // K fragments read ahead of the Q.K^T MFMA that consumes them
#define SAGE_VPF 3   // V fragment pairs read ahead of the P.V MFMA that consumes them
// Bit of the wavefront index that picks the group: wavefronts w and w + 4 share a SIMD.
#define SAGE_GSH 2

namespace sage {


constexpr float kBiasF = 12582912.0f;     // 1.5 * 2^23
constexpr int kBiasBits = 0x4B400000;     // its bit pattern; int accumulators start here
constexpr float kNegInf = -__builtin_inff();
constexpr float kMInit = -1.0e30f;
constexpr float kCodeBias = -0.3f;       // centres the linear-mantissa fp8 code of the probabilities (see softmax)

template <int PV> struct PCfg;
template <> struct PCfg<1> { static constexpr float tau = 3.0f, pshift = 5.0f; };   // fp8: p*32 <= 256 < 448
template <> struct PCfg<0> { static constexpr float tau = 8.0f, pshift = 0.0f; };   // fp16: p <= 256
// Block-scaled probability codes (FP8 P.V kernels without LSE or an explicit mask, see softmax): the largest probability of a
// query row in a 128-key tile is coded within one binade below 2^kBlockTop (code <= 126 = 448), the block's power-of-two
// scale goes to the MFMA as an E8M0 byte, kBlockScaleBias + exponent; the running maximum then only has to keep fp32 in range.
constexpr float kBlockTop = 8.75f, kBlockTau = 20.0f, kBlockMinExp = -110.0f, kBlockScaleBias = 119.0f;   // 119 = 127 - 8

// NOTE: __builtin_bit_cast applied directly to an element of an ext_vector_type value reads element
// 0 whatever the index (clang miscompiles the element lvalue), so vector elements are always passed
// BY VALUE through these two helpers.
__device__ inline float as_f(int v) { return __builtin_bit_cast(float, v); }
__device__ inline int as_i(float v) { return __builtin_bit_cast(int, v); }

// Exchange between lane l and lane l^32 (the two lanes that share a query row).
// v_permlane32_swap swaps the upper half of its first operand with the lower half of its second, so
// with both operands holding x every lane ends up with {x[l%32], x[l%32 + 32]}.
__device__ inline void xchg32(float x, float& lo, float& hi) {
  auto r = __builtin_amdgcn_permlane32_swap(as_i(x), as_i(x), false, false);
  int r0 = r[0], r1 = r[1];
  lo = as_f(r0);
  hi = as_f(r1);
}
__device__ inline float xchg32_max(float x) {
  float lo, hi;
  xchg32(x, lo, hi);
  return fmaxf(lo, hi);
}
__device__ inline float xchg32_sum(float x) {
  float lo, hi;
  xchg32(x, lo, hi);
  return lo + hi;
}

// Workgroup barrier that only orders LDS traffic: waits for this wavefront's outstanding LDS
// operations, then s_barrier (global-memory traffic issued ahead stays in flight).
__device__ inline void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// 16-byte-chunk swizzle of a K row in LDS: consecutive rows read the same logical chunk from
// different bank groups (64 banks x 4 bytes = 256 bytes per bank row).
template <int D>
__device__ inline int kswz(int n) {
  constexpr int CPR = D / 16, RPB = 256 / D;
  return (n / RPB) % CPR;
}

// LDS slots per tile stream.  FP8 P.V kernels rotate through four and request tiles two periods before
// their first use (a tile that has to come from HBM takes longer than one 2 us period: +5...8 % for
// non-causal kernels from 1k to 16k keys, neutral for causal ones; three slots measured 1-2 % slower
// than four, the slot index being a modulo in the loop).  FP16 P.V tiles are twice as large: two
// slots, one period (three slots measured 1-3 % slower there).
template <int PV, bool CAUSAL>
constexpr int attn_tile_slots() { return PV == 1 ? 4 : 2; }
template <int PV, bool CAUSAL>
constexpr int attn_tile_lead() { return attn_tile_slots<PV, CAUSAL>() > 2 ? 2 : 1; }

// Dynamic LDS of a kernel variant: the K slots and as many V slots; a kernel that quantises its own Q also
// stages the raw q-tile behind the K slots that are requested in the prologue (over slots that are idle
// until the main loop); FP8 kernels keep the D per-channel V scales behind all of that.
template <int D, int NW, int BN, int PV, bool CAUSAL, bool QF>
constexpr int attn_tile_lds_bytes() {
  constexpr int slots = attn_tile_slots<PV, CAUSAL>();
  constexpr int tiles = slots * (BN * D + BN * D * (PV ? 1 : 2));
  constexpr int qstage = attn_tile_lead<PV, CAUSAL>() * BN * D + NW * 32 * D * 2;
  return (QF && qstage > tiles) ? qstage : tiles;
}
template <int D, int NW, int BN, int PV, bool CAUSAL, bool QF>
constexpr int attn_lds_bytes() { return attn_tile_lds_bytes<D, NW, BN, PV, CAUSAL, QF>() + (PV ? D * 4 : 0); }

// Timing build (-DSAGE_TIMING=1, not the shipped library): every wavefront stamps eight points of its
// tile on the constant-rate 100 MHz counter and adds the seven intervals to per-class sums (class 0 =
// first wavefront, 1 = last, 2 = the others): [class][0..6] intervals in ticks, [class][7] wavefronts,
// [3][0] = tiles.  SAGE_T(k, x) pins stamp k after the computation of x.
// Also, in the main loop of the FP8 kernels, four stamps per period (after the even barrier, before and after the odd
// barrier, at the end of the period) are summed per group: [32 + 4 g + k] = ticks from stamp k to the next one (k = 0:
// first phase of the period, 1: wait at the odd barrier, 2: second phase, 3: wait at the even barrier), [40 + g] = periods;
// [42] / [43] = ticks per period that the issuing wavefront spends on the tile requests; [44] / [45] = ticks a wavefront
// of the kernels that quantise their own Q waits, after its last prologue request, for the raw rows to arrive.
#ifdef SAGE_TIMING
// The sums are kept in kTimingSets copies, one per workgroup index modulo kTimingSets, and added up on the host: with a
// single copy the atomics of thousands of short workgroups pile up on three cache lines and hold up the L2 channel
// they live in, tile requests included.
constexpr int kTimingSets = 256;
static __device__ unsigned long long g_tile_timing[kTimingSets][48];
// One record per workgroup of the last launch (the first kTimelineMax of them): first stamp, last stamp (ticks of the
// chip-wide 100 MHz counter), where it ran (XCC_ID << 32 | HW_ID: compute unit, shader array and engine) and its K tiles.
constexpr int kTimelineMax = 65536;
static __device__ unsigned long long g_wg_timeline[kTimelineMax][4];
#define SAGE_PH(k) do { const long long t_ = __builtin_amdgcn_s_memrealtime(); if (ph_last) ph_sum[((k) + 3) & 3] += t_ - ph_last; ph_last = t_; if ((k) == 0) ph_n++; } while (0)
#define SAGE_T(k, x) do { asm volatile("" : "+v"(x)); sage_ts[k] = __builtin_amdgcn_s_memrealtime(); } while (0)
#else
#define SAGE_PH(k) do { } while (0)
#define SAGE_T(k, x) do { } while (0)
#endif
// MASK: 0 none, 1 boolean keep-mask (bytes), 2 additive fp32 bias in base-2 score units
// (sageattention_triton.py:92-105), both [B, Hq, Sq, Skv] with element strides.
// KSUB: K scale blocks per 32 keys (1 for blocks of 32/64/128 keys, 2 for blocks of 16 keys); 3 = four interleaved scales per
// block of 32/64/128 keys, scale t for the keys n of the block with (n % 8) / 2 == t (two of them reach every lane).
// QF: the kernel reads fp16/bf16 Q and quantises its own tile (same arithmetic as quant_int8_kernel).
// KW (with KSUB == 1): 32-key groups that are known to share a K scale -- 1 for any block size from 32 keys on (every group
// looks its scale up), 2 for blocks of 64 keys and more, 4 for blocks of 128: the row maximum then runs one integer chain
// per scale and the per-scale constants of the softmax are computed once (a tenth of the vector instructions of a tile).
template <int D, int NW, int BN, int PV, bool CAUSAL, bool MSUM, int MASK, int KSUB = 1, bool QF = false, int KW = 1>
__global__ void __launch_bounds__(NW * 64) attn_kernel(AttnArgs a) {
  constexpr int GSH = SAGE_GSH;   // which bit of the wavefront index picks the group
  static_assert(NW == (2 << GSH), "the two groups pair wavefront w with w + NW/2");
  constexpr int BM = NW * 32;
  constexpr int NTHR = NW * 64;
  constexpr int KS = D / 32;   // contraction steps of S^T
  constexpr int NT = BN / 32;  // 32-row tiles of S^T
  constexpr int DTN = D / 32;  // 32-row tiles of O^T
  constexpr int VESZ = PV ? 1 : 2;
  constexpr int KBYTES = BN * D, VBYTES = BN * D * VESZ, STAGE = KBYTES + VBYTES;
  constexpr int KCHUNKS = KBYTES / 16, VCHUNKS = VBYTES / 16;
  constexpr int PANEL_BYTES = kPanelRows * D * VESZ;
  constexpr int CPR = D / 16;
  constexpr float TAU = PCfg<PV>::tau, PSHIFT = PCfg<PV>::pshift;
  constexpr int NSLOT = attn_tile_slots<PV, CAUSAL>(), LEAD = attn_tile_lead<PV, CAUSAL>();   // tiles are requested LEAD periods ahead
  // FP8 P.V: the softmax denominator of O always comes from the matrix pipe (the sum of the very fp8 values that
  // multiply V); MSUM additionally means that no fp32 sum is kept (no LSE wanted), and then the probabilities are
  // coded without v_exp_f32 (FASTP, see softmax).  FP16 P.V kernels instantiated with MSUM (no LSE wanted) take the sum
  // of the fp16-rounded probabilities from the matrix pipe as well; otherwise they sum in fp32 on the vector ALU.
  constexpr bool RSUM = PV == 1 || MSUM;
  constexpr bool FASTP = PV == 1 && MSUM && MASK == 0;
  // FP8 kernels, and FP16 ones of head_dim 128, take the row maximum in the vector phase and issue the tile requests at
  // the end of group 0's matrix phase; FP16 kernels of head_dim 64 keep the row maximum in the matrix phase (their
  // softmax, with its exponentials, is the longer one there: moving it measured -3 %, against +1 % at head_dim 128).
  constexpr bool VECMAX = PV == 1 || D == 128;

  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

#ifdef SAGE_TIMING
  long long sage_ts[8];
  for (int i = 0; i < 8; i++) sage_ts[i] = __builtin_amdgcn_s_memrealtime();
  long long ph_last = 0, ph_sum[4] = {0, 0, 0, 0}, rq_sum = 0, q_wait = 0;
  int ph_n = 0, rq_n = 0;
#endif
  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);  // wavefront index: uniform, keep it scalar
  const int m = lane & 31, h = lane >> 5;

  // ---- which tile am I: heaviest q-tiles first; q-heads sharing a KV head on one XCD ----
  // (Divisions by launch constants go through host-made multipliers, range widths are powers of two: every workgroup
  // pays for this decode before its first memory request.)
  const bool packed = a.cu_q != nullptr;
  const int G = a.G;
  const uint32_t bid = blockIdx.x;
  int rank, s, NG;
  if (packed) { rank = fastdiv(bid, a.div_heads); s = bid - rank * a.Hq; NG = a.Hkv; }
  else {
    const int U = a.B * a.Hq;
    NG = a.B * a.Hkv;
    if (a.tier_shift >= 0) {
      // Inside an XCD (workgroup index modulo 8; 32 compute units) the workgroups that run at the same time take
      // neighbouring q-tiles of FEW heads: the q-tiles of a head (by weight: rank 0 is the heaviest) are cut into ranges
      // of R consecutive ranks, and the XCD goes through a range head by head, a head's R q-tiles in a row, before it
      // moves on to the next range; 32 consecutive workgroups are therefore R q-tiles of each of 32 / R heads.  R is a
      // power of two up to 32 and at most half of a head's q-tiles (long sequences: 32, one head at a time).  The q-tiles
      // of a head walk the same K/V tiles from tile 0 on at about the same pace, so one of them fetches a tile into the
      // XCD's L2 and the others hit it there (a quarter of the L2 fills of the plain heaviest-first order, where an XCD
      // works on all its heads at once), and neighbouring q-tiles read neighbouring rows of Q.
      const int x = bid & 7, hpx = U >> 3;   // XCD, heads per XCD
      int l = bid >> 3;                      // index inside the XCD
      int rs = a.tier_shift;                 // log2 of the range width R
      if constexpr (CAUSAL) {
        // Causal q-tiles get lighter with their rank, and the ranges narrower: never more than half of the ranks that
        // are left (64 q-tiles: 32, 16, 8, 4, 2, 1, 1), so that the workgroups an XCD runs last are all short ones
        // (+2.5 % on 64 x 32 heads of 1024 rows, nothing on long sequences).
        int r0 = 0;
        for (;;) {
          while (rs > 0 && (2 << rs) > a.nqt - r0) rs--;
          if (l < (hpx << rs)) break;
          l -= hpx << rs;
          r0 += 1 << rs;
          if (r0 >= a.nqt) return;   // (a grid larger than the tile count: nothing to do)
        }
        // Inside a round (32 consecutive workgroups of the XCD: one per compute unit) the order alternates: lightest
        // q-tile first in even rounds, heaviest first in odd ones.  The hardware hands out workgroups strictly in index
        // order and round-robin over the XCD's four shader engines, so a free compute unit waits until every earlier
        // workgroup has found a place in ITS engine.  A round that starts on all compute units at once with ascending
        // cost frees them in dispatch order; the next round, started one by one as they free up, has descending cost,
        // so that it ends everywhere at the same time and the round after it starts together again -- which also
        // keeps the compute units of the XCD in step on the K/V tiles they share through its L2.  (Measured on 2 x 32 heads
        // of 16k rows, per hand-over of a compute unit from one workgroup to the next: 1.6 us this way; 6.4 us with the
        // heaviest first in every round; 4.8 us with the lightest first in every round, whose compute units also drift
        // apart and fetch 1.7 x the bytes into L2.)  Ranges
        // whose size is not a whole number of rounds (the last, lightest few) keep the plain order.
        if (((hpx << rs) & 31) == 0) {
          int j = l & 31;                      // position in the round
          j = ((l >> 5) & 1) ? 31 - j : j;
          const int hs = 5 - rs;               // log2 of the heads a round covers
          rank = r0 + ((1 << rs) - 1 - (j >> hs));
          s = x + 8 * (((l >> 5) << hs) + (j & ((1 << hs) - 1)));
        } else {
          rank = r0 + (l & ((1 << rs) - 1));
          s = x + 8 * (l >> rs);
        }
      } else {
        // all q-tiles cost the same: ranges of R ranks and one last range with the remainder
        const int nfull = a.nqt >> rs, lfull = (nfull * hpx) << rs;
        if (l < lfull) {
          const int t = fastdiv(l, a.div_range), lr = l - ((t * hpx) << rs);
          rank = (t << rs) + (lr & ((1 << rs) - 1));
          s = x + 8 * (lr >> rs);
        } else {
          const int Rt = a.nqt - (nfull << rs), lr = l - lfull, hd = fastdiv(lr, a.div_last);
          rank = (nfull << rs) + lr - hd * Rt;
          s = x + 8 * hd;
        }
      }
    } else {
      rank = fastdiv(bid, a.div_heads); s = bid - rank * U;
    }
  }
  int gi, g;
  if ((NG & 7) == 0) { const int x = s & 7, y = s >> 3, yg = fastdiv(y, a.div_G); gi = x + 8 * yg; g = y - yg * G; }
  else { gi = fastdiv(s, a.div_G); g = s - gi * G; }
  int b, kvh, qt, Lq, Lk, hq_idx;
  int64_t qoff, koff, ooff, lseoff;
  const float *qsp, *ksp;
  const uint8_t* vbase;
  int nkblk;
  if (packed) {
    if (rank >= a.ntiles[0]) return;
    int t = a.tiles[rank];
    b = t >> 16; qt = t & 0xffff; kvh = gi;
    int q0 = a.cu_q[b], k0 = a.cu_k[b];
    Lq = a.cu_q[b + 1] - q0; Lk = a.cu_k[b + 1] - k0;
    int hq = kvh * G + g;
    hq_idx = hq;
    qoff = (int64_t)q0 * a.q_sn + (int64_t)hq * a.q_sh;
    ooff = (int64_t)q0 * a.o_sn + (int64_t)hq * a.o_sh;
    koff = (int64_t)k0 * a.k_sn + (int64_t)kvh * a.k_sh;
    lseoff = (int64_t)hq * a.total_q + q0;
    qsp = a.qs + (int64_t)hq * a.qs_sh + a.cu_qblk[b];
    ksp = a.ks + (int64_t)kvh * a.ks_sh + a.cu_kblk[b];
    vbase = a.vp + ((int64_t)kvh * a.panel_sh + a.cu_panel[b]) * PANEL_BYTES;
  } else {
    b = fastdiv(gi, a.div_Hkv); kvh = gi - b * a.Hkv;
    qt = CAUSAL ? a.nqt - 1 - rank : rank;
    Lq = a.Sq; Lk = a.Skv;
    int hq = kvh * G + g;
    hq_idx = hq;
    qoff = (int64_t)b * a.q_sb + (int64_t)hq * a.q_sh;
    ooff = (int64_t)b * a.o_sb + (int64_t)hq * a.o_sh;
    koff = (int64_t)b * a.k_sb + (int64_t)kvh * a.k_sh;
    lseoff = ((int64_t)b * a.Hq + hq) * a.Sq;
    qsp = a.qs + (((int64_t)b * a.Hq + hq) * ((Lq + a.blkq - 1) >> a.blkq_shift) << a.qg_shift);
    ksp = a.ks + ((int64_t)b * a.Hkv + kvh) * ((Lk + a.blkk - 1) >> a.blkk_shift) * (KSUB == 3 ? 4 : 1);
    vbase = a.vp + ((int64_t)b * a.Hkv + kvh) * ((Lk + kPanelRows - 1) / kPanelRows) * PANEL_BYTES;
  }
  nkblk = (Lk + a.blkk - 1) >> a.blkk_shift;
  // The K scales are read through the scalar cache (constant address space): a vector load would sit
  // in the same in-order counter as the tile loads in flight and make every tile wait for them.
  const __attribute__((address_space(4))) float* ksc = (const __attribute__((address_space(4))) float*)ksp;

  const int row0 = qt * BM + w * 32;   // first query row of this wavefront
  const int my_row = row0 + m;
  const int kv_end = CAUSAL ? min(Lk, qt * BM + BM) : Lk;
  const int ntiles = (kv_end + BN - 1) / BN;
  const int wave_end = (row0 < Lq) ? (CAUSAL ? min(Lk, row0 + 32) : Lk) : 0;
  const int wave_ntiles = (wave_end + BN - 1) / BN;

  // ---- tile loads: global memory -> LDS directly (no registers), 1 KB per wavefront instruction ----
  // Lane l of a wavefront writes LDS bytes [16*l, 16*l+16) of the 1 KB piece, so the K swizzle is
  // applied on the global side: the lane fetches the 16-byte chunk that belongs in its slot.
  // K tiles and V tiles each rotate through NSLOT LDS slots.
  constexpr int KPIECES = KBYTES / 1024 / NW, VPIECES = VBYTES / 1024 / NW;
  static_assert(KPIECES * 1024 * NW == KBYTES && VPIECES * 1024 * NW == VBYTES, "tile must split into 1 KB pieces per wavefront");
  // The buffer form of the LDS load is used on purpose: the compiler treats the global form as a flat
  // access that may touch LDS and then drains every counter at each LDS read while one is in flight.
  const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc((void*)(a.k + koff), 0, 0x7fffffff, 0x00020000);
  const __amdgpu_buffer_rsrc_t vrsrc = __builtin_amdgcn_make_buffer_rsrc((void*)vbase, 0, 0x7fffffff, 0x00020000);
  auto dma16 = [&](__amdgpu_buffer_rsrc_t rsrc, int lane_offset, int uniform_offset, uint8_t* dst_uniform) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)dst_uniform, 16, lane_offset, uniform_offset, 0, 0);
  };
  auto kslot = [&](int j) { return smem + (j % NSLOT) * KBYTES; };
  auto vslot = [&](int j) { return smem + NSLOT * KBYTES + (j % NSLOT) * VBYTES; };
  // Per-lane byte offsets of this wavefront's pieces inside a tile are loop invariant; the tile index
  // only adds a uniform term.  Rows past the end of the sequence (last tile only) are clamped.
  // Piece offsets are those of the lower wavefront of the SIMD pair (wl); dw selects which wavefront's pieces a
  // request covers: dw_self for this wavefront's own (prologue), 0 and PARTNER_DW for both of the pair (main
  // loop, where one wavefront issues for two).  Offsets added per request are therefore never negative.
  constexpr int PARTNER_DW = 1 << GSH;
  const int wl = w & ~PARTNER_DW, dw_self = w - wl;
  int koffv[KPIECES], voffv[VPIECES];
#pragma unroll
  for (int i = 0; i < KPIECES; i++) {
    const int sl = (i * NW + wl) * 64 + lane, n = sl / CPR, cc = (sl % CPR) ^ kswz<D>(n);
    koffv[i] = n * (int)a.k_sn + 16 * cc;
  }
#pragma unroll
  for (int i = 0; i < VPIECES; i++) voffv[i] = (i * NW + wl) * 1024 + lane * 16;
  const int ktile_bytes = BN * (int)a.k_sn;
  // dw is a multiple of 4, so the rows move by a multiple of 16 and keep their swizzle: only the uniform offset changes.
  auto load_k = [&](int j, int dw) {
    uint8_t* dst = kslot(j) + dw * 1024;
    if (j * BN + BN <= Lk) {
      const int uo = j * ktile_bytes + dw * (64 / CPR) * (int)a.k_sn;
#pragma unroll
      for (int i = 0; i < KPIECES; i++) dma16(krsrc, koffv[i], uo, dst + (i * NW + wl) * 1024);
    } else {
#pragma unroll
      for (int i = 0; i < KPIECES; i++) {
        const int sl = (i * NW + wl + dw) * 64 + lane, n = sl / CPR, cc = (sl % CPR) ^ kswz<D>(n);
        dma16(krsrc, min(j * BN + n, Lk - 1) * (int)a.k_sn + 16 * cc, 0, dst + (i * NW + wl) * 1024);
      }
    }
  };
  auto load_v = [&](int j, int dw) {
    uint8_t* dst = vslot(j) + dw * 1024;
#pragma unroll
    for (int i = 0; i < VPIECES; i++) dma16(vrsrc, voffv[i], j * VBYTES + dw * 1024, dst + (i * NW + wl) * 1024);
  };

  // The K tiles of the lead are requested before anything waits on memory, and the per-channel V scales of the epilogue
  // come along (4 bytes per lane, D / 64 wavefronts).  Kernels that quantise their own Q put the raw q-tile's requests in
  // front of these (the quantisation is what the prologue waits for; the K tiles then arrive under it).
  float* vs_lds = reinterpret_cast<float*>(smem + attn_tile_lds_bytes<D, NW, BN, PV, CAUSAL, QF>());
  // returns the number of requests this wavefront issued
  auto request_lead_tiles = [&]() -> int {
    int n = 0;
    if (ntiles > 0) { load_k(0, dw_self); n += KPIECES; }
    if constexpr (PV == 1) {
      if (w < D / 64) {
        if (Lk > 0) {
          const __amdgpu_buffer_rsrc_t vsrsrc =
              __builtin_amdgcn_make_buffer_rsrc((void*)(a.vs + ((int64_t)b * a.Hkv + kvh) * D), 0, D * 4, 0x00020000);
          __builtin_amdgcn_raw_ptr_buffer_load_lds(vsrsrc, (__attribute__((address_space(3))) void*)(vs_lds + 64 * w), 4, lane * 4, w * 256, 0, 0);
          n += 1;
        } else {
          vs_lds[64 * w + lane] = 1.0f;   // no keys: nothing ever wrote the scales, and 0 * garbage must stay 0
        }
      }
    }
#pragma unroll
    for (int t = 1; t < LEAD; t++)
      if (t < ntiles) { load_k(t, dw_self); n += KPIECES; }
    return n;
  };
  // Tile loads complete in the order they were requested, so waiting until only the n newest are in
  // flight leaves exactly the n last requests outstanding.
  auto wait_all_but = [&](int n) {
    switch (n) {
      case 0: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
      case 1: asm volatile("s_waitcnt vmcnt(1)" ::: "memory"); break;
      case 2: asm volatile("s_waitcnt vmcnt(2)" ::: "memory"); break;
      case 3: asm volatile("s_waitcnt vmcnt(3)" ::: "memory"); break;
      case 4: asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); break;
      case 5: asm volatile("s_waitcnt vmcnt(5)" ::: "memory"); break;
      case 6: asm volatile("s_waitcnt vmcnt(6)" ::: "memory"); break;
      case 8: asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); break;
      case 10: asm volatile("s_waitcnt vmcnt(10)" ::: "memory"); break;
      case 12: asm volatile("s_waitcnt vmcnt(12)" ::: "memory"); break;
      default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
    }
  };
  if constexpr (!QF) request_lead_tiles();

  { [[maybe_unused]] int addressed = nkblk + ntiles + wave_ntiles; SAGE_T(1, addressed); }   // tile decoded, first loads requested
  // ---- Q operand: lane (m, h) holds bytes 32*ks + 16*h .. +15 of its row for every ks ----
  v4i qreg[KS];
  float qscale;
  if constexpr (!QF) {
    const int8_t* qp = a.q + qoff + (int64_t)min(my_row, Lq - 1) * a.q_sn + 16 * h;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) qreg[ks] = *reinterpret_cast<const v4i*>(qp + 32 * ks);
    // per lane: scale blocks may be smaller than a wavefront's 32 rows, and with interleaved scales the rows r, r + 8, ...
    // of a block share one of its eight
    const int qrow = min(my_row, Lq - 1);
    qscale = qsp[((qrow >> a.blkq_shift) << a.qg_shift) + (qrow & ((1 << a.qg_shift) - 1))];
  } else {
    // Quantise this wavefront's 32 rows here, exactly as quant_int8_kernel would
    // (quant_per_block.py:38-46): x32 = fp32(x) * mult, scale = max|x32| / 127 over the scale block
    // (16 rows = half a wavefront; 32, 64 or 128 rows = 1, 2 or 4 wavefronts), q = trunc(x32 / scale + 0.5 sgn).  Rows past the
    // end repeat the last row, which belongs to the same (last) scale block or to none.
#pragma clang fp contract(off)
    __shared__ float q_block_amax[NW];
    // The raw rows of this wavefront come in through LDS (1 KB per instruction, whole rows, into a region
    // that no tile uses before the first barrier of the main loop) instead of 32-byte pieces of 32 rows
    // per instruction.  16-byte units of a row are XOR-swizzled with the row index, on the global side as
    // for K.  Only this wavefront reads its region, so its own vmcnt wait is all the ordering needed.
    constexpr int QUPR = D * 2 / 16, QRPP = 64 / QUPR, QPIECES = 32 * D * 2 / 1024;
    uint8_t* qstage = smem + LEAD * KBYTES + w * (32 * D * 2);
    {
      const __amdgpu_buffer_rsrc_t qrsrc =
          __builtin_amdgcn_make_buffer_rsrc((void*)(reinterpret_cast<const u16*>(a.q_raw) + qoff), 0, 0x7fffffff, 0x00020000);
#pragma unroll
      for (int i = 0; i < QPIECES; i++) {
        const int r = i * QRPP + lane / QUPR;
        const int u = (lane % QUPR) ^ (r & (QUPR - 1));
        dma16(qrsrc, min(row0 + r, Lq - 1) * (int)a.q_sn * 2 + 16 * u, 0, qstage + i * 1024);
      }
      const int behind = request_lead_tiles();   // K tiles of the lead, V scales: they may stay in flight
#ifdef SAGE_TIMING
      const long long q_issued = __builtin_amdgcn_s_memrealtime();
#endif
      wait_all_but(behind);
#ifdef SAGE_TIMING
      q_wait = __builtin_amdgcn_s_memrealtime() - q_issued;   // from the last request of the prologue to the arrival of everything
#endif
    }
    float x[KS][16];
    float amax = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      uint4 raw[2];
#pragma unroll
      for (int e = 0; e < 2; e++)
        raw[e] = *reinterpret_cast<const uint4*>(qstage + m * (D * 2) + 16 * ((4 * ks + 2 * h + e) ^ (m & (QUPR - 1))));
      const u16* e = reinterpret_cast<const u16*>(raw);
#pragma unroll
      for (int i = 0; i < 16; i++) {
        x[ks][i] = (a.q_is_bf16 ? bf16_to_f32(e[i]) : f16_to_f32(e[i])) * a.q_mult;
        amax = fmaxf(amax, fabsf(x[ks][i]));
      }
    }
    // Scale blocks of 16 rows: the lanes of a DPP row hold 16 consecutive query rows (one column half each),
    // the other column half sits 32 lanes away.  Larger blocks span the wavefront (and its neighbours, below).
    if (a.blkq == 16) amax = xchg32_max(row16_max(amax));
    else amax = wave_max(amax);
    SAGE_T(2, amax);   // the raw Q rows have arrived
    const int wpb = a.blkq >> 5;   // wavefronts per scale block
    if (wpb > 1) {
      if (lane == 0) q_block_amax[w] = amax;
      __syncthreads();
      const int w0 = w & ~(wpb - 1);
      for (int i = 0; i < wpb; i++) amax = fmaxf(amax, q_block_amax[w0 + i]);
    }
    const float scale = fmaxf(amax / 127.0f, kScaleFloor);
    const float rcp = 1.0f / scale;
    const uint32_t sbits = __builtin_bit_cast(uint32_t, scale);
    const bool fast = ((sbits & 0x7fffffu) != 0x7fffffu) && scale < 1.0e30f;
    // (one uniform branch around the whole tile, not one per element: the two quotients are the same numbers)
    auto quantise_rows = [&](auto quotient) __attribute__((always_inline)) {
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        uint32_t packed[4] = {0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < 16; i++) {
          float z = quotient(x[ks][i]);
          z = z + __builtin_copysignf(0.5f, z);
          int qv = (int)z;
          packed[i >> 2] |= (uint32_t)(qv & 0xff) << (8 * (i & 3));
        }
        qreg[ks] = v4i{(int)packed[0], (int)packed[1], (int)packed[2], (int)packed[3]};
      }
    };
    if (fast) quantise_rows([&](float v) { return div_by_uniform(v, scale, rcp); });
    else quantise_rows([&](float v) { return v / scale; });
    qscale = scale;
  }


  v16i bias;
#pragma unroll
  for (int i = 0; i < 16; i++) bias[i] = kBiasBits;
  asm volatile("" : "+v"(bias));  // keep it in registers: it is the C operand of every first MFMA

  v16f o[DTN];
#pragma unroll
  for (int dt = 0; dt < DTN; dt++)
#pragma unroll
    for (int i = 0; i < 16; i++) o[dt][i] = 0.f;
  float m_used = kMInit, lsum = 0.f;
  // FP8 P.V: the row sums come out of the matrix pipe too, from one 16x16x128 MFMA (8 passes, half the time of
  // a P.V one) per 64 keys.  Its B operand is the very register block that multiplies V: read by that
  // instruction, lane l holds 32 codes of "column" l % 16 and k-chunk l / 16, where the 32x32x64 layout has
  // query column l % 32 and key half l / 32 -- so chunks 0 and 2 are the two key halves of query columns 0-15 and
  // chunks 1 and 3 those of columns 16-31.  The A operand selects them: row 0 is ones (fp8 1.0 = 0x38) over chunks
  // 0 and 2, row 4 over chunks 1 and 3, every other row zero.  Output row 0 lands in register 0 of lanes 0-15
  // and row 4 in register 0 of lanes 16-31: register 0 of lane l < 32 accumulates sum_n P[n][l], the softmax
  // denominator of the lane's own query row -- of the very fp8 values that multiply V.  The sum of rounded
  // values is the right denominator for O but costs LSE accuracy on rows with few keys, so kernels
  // that return LSE (MSUM false) also keep the fp32 sum of the unrounded values on the vector ALU, for LSE alone.
  v4f osum = {0.f, 0.f, 0.f, 0.f};
  // (FP16 P.V kernels that return no LSE do the same with a 16x16x32 MFMA per 16 keys: 8 halves per lane and chunk.)
  v8i ones;
  {
    const bool sel = lane == 0 || lane == 32 || lane == 20 || lane == 52;
#pragma unroll
    for (int i = 0; i < 8; i++) ones[i] = !sel ? 0 : PV == 1 ? 0x38383838 : 0x3c003c00;
  }
  asm volatile("" : "+v"(ones));

  // State that crosses phases: the raw scores of the tile in flight, its row maximum and scales, and
  // the probabilities packed as the B operand of the second MFMA.
  v16i acc[NT];
  // q_scale * k_scale per K scale block of the tile; in the accumulator layout register r of a 32-key
  // group holds keys 8*(r/4) + 4*h + r%4, so registers 0-7 belong to the first 16 keys and 8-15 to the rest.
  // With interleaved K scales (KSUB == 3) a key's scale is picked by (n % 8) / 2 = 2*h + (r % 4) / 2: two per lane and
  // 32-key group, selected by bit 1 of the register index.
  constexpr int SUBS = KSUB == 1 ? 1 : 2;   // scale values per 32-key group and lane
  static_assert(KW == 1 || (KSUB == 1 && (KW == 2 || KW == 4) && NT % KW == 0), "KW: 32-key groups per K scale");
  constexpr int GPS = KW;                    // 32-key groups that share a scale
  constexpr int NSC = NT * SUBS / GPS;
  float sc[NSC];
  auto subof = [](int r) { return KSUB == 2 ? r / 8 : KSUB == 3 ? (r >> 1) & 1 : 0; };
  auto sci = [&](int nt, int r) { return (SUBS * nt + subof(r)) / GPS; };
  // K scale i of tile j as this lane needs it (before the Q scale is multiplied in)
  auto kscale_at = [&](int j, int i) -> float {
    if constexpr (KSUB == 3) {
      const int blk = min((j * BN + 32 * (i >> 1)) >> a.blkk_shift, nkblk - 1);
      const float lo = ksc[blk * 4 + (i & 1)], hi = ksc[blk * 4 + 2 + (i & 1)];
      return h ? hi : lo;
    } else {
      return ksc[min((j * BN + (32 / KSUB) * GPS * i) >> a.blkk_shift, nkblk - 1)];
    }
  };
  float mloc = kNegInf;
  // Block-scaled codes: the E8M0 scale byte of this row's probabilities of the tile in flight, for the P.V phase.
  [[maybe_unused]] int pscale = 0;

  // ---- S^T = K . Q^T (int8 -> int32 on the biased accumulators), then mask and row maximum ----
  auto qk = [&](int j) {
    const uint8_t* kbuf = kslot(j);
    // K fragments run KPF MFMAs ahead of their use so that no MFMA waits for the LDS read issued
    // just before it; the k-step is the outer index so that consecutive MFMAs hit different accumulators.
    {
      constexpr int NF = NT * KS, KPF = SAGE_KPF;
      auto kfrag = [&](int i) {
        const int nt = i % NT, ks = i / NT, n = 32 * nt + m;
        return *reinterpret_cast<const v4i*>(kbuf + n * D + 16 * ((2 * ks + h) ^ kswz<D>(n)));
      };
      v4i kf[NF];
#pragma unroll
      for (int i = 0; i < KPF; i++) kf[i] = kfrag(i);
#pragma unroll
      for (int i = 0; i < NF; i++) {
        if (i + KPF < NF) kf[i + KPF] = kfrag(i + KPF);
        const int nt = i % NT, ks = i / NT;
        acc[nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf[i], qreg[ks], ks == 0 ? bias : acc[nt], 0, 0, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x100, KPF, 0);
#pragma unroll
      for (int i = 0; i < NF - KPF; i++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, KPF, 0);
    }
  };
  // q_scale * k_scale of the 32-key groups of tile j.  Fetched during the vector-ALU phase: a scalar
  // load in flight while K/V fragments are being read would force every LDS wait to drain the queue.
  auto load_scales = [&](int j) {
#pragma unroll
    for (int i = 0; i < NSC; i++) sc[i] = qscale * kscale_at(j, i);
  };

  auto rowmax = [&](int j) {
    const int n0 = j * BN;
    if constexpr (MASK != 0) {
      // Explicit mask: the accumulators become scores (scale applied, bias removed), the mask is
      // applied element by element, and the maximum is taken over floats.
      const int64_t mrow = (int64_t)b * a.m_sb + (int64_t)hq_idx * a.m_sh + (int64_t)min(my_row, Lq - 1) * a.m_sm;
      mloc = kNegInf;
#pragma unroll
      for (int nt = 0; nt < NT; nt++) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int n = n0 + 32 * nt + 8 * (r / 4) + 4 * h + (r % 4);
          // (the bias comes off first, exactly: the product of the biased value would have to cancel against a
          // rounded bias * scale, an error of half an ulp of that product -- 1e-3 at large scales)
          float sv = (as_f(acc[nt][r]) - kBiasF) * sc[sci(nt, r)];
          const int64_t mi = mrow + (int64_t)min(n, Lk - 1) * a.m_sn;
          if constexpr (MASK == 1) sv = reinterpret_cast<const uint8_t*>(a.mask)[mi] ? sv : kNegInf;
          else sv = __builtin_fmaf(reinterpret_cast<const float*>(a.mask)[mi], a.mask_mult, sv);
          if (n >= Lk) sv = kNegInf;
          acc[nt][r] = as_i(sv);
          mloc = fmaxf(mloc, sv);
        }
      }
      return;
    }
    // ---- masking: only tiles that cross the diagonal or the end of the sequence ----
    const bool need_mask = (CAUSAL && (n0 + BN - 1 > row0)) || (n0 + BN > Lk);
    if (need_mask) {
      // Register r of 32-key group nt holds key n0 + 32*nt + 8*(r/4) + r%4 + 4*h: it is masked when that index
      // exceeds lim.  In causal kernels (two diagonal tiles per q-tile) the bounds of lim over the wavefront (its 32
      // rows, both lane halves) sort the groups first: most are visible or masked as a whole, and only the one the
      // diagonal runs through is selected element by element.
      const int lim = (CAUSAL ? min(my_row, Lk - 1) : Lk - 1) - n0 - 4 * h;
      const int lim_hi = min(row0 + 31, Lk - 1) - n0, lim_lo = min(row0, Lk - 1) - n0 - 4;
#pragma unroll
      for (int nt = 0; nt < NT; nt++) {
        if constexpr (CAUSAL) {
          if (32 * nt + 27 <= lim_lo) continue;
          if (32 * nt > lim_hi) {
#pragma unroll
            for (int r = 0; r < 16; r++) acc[nt][r] = as_i(kNegInf);
            continue;
          }
        }
#pragma unroll
        for (int r = 0; r < 16; r++) {
          // branch-free select on the sign of (lim - index): compare-and-select would hold the lane masks
          // in scalar registers at once
          const int gone = (lim - (32 * nt + 8 * (r / 4) + (r % 4))) >> 31;
          acc[nt][r] = (acc[nt][r] & ~gone) | (as_i(kNegInf) & gone);
        }
      }
    }
    // ---- row maximum of this tile, in score units ----
    // The biased scores are positive floats (or -inf where masked), so their bit patterns order like
    // signed integers: integer max3 needs no NaN canonicalisation.
    mloc = kNegInf;
    if constexpr (GPS > 1) {
      // groups that share a scale share one integer chain
#pragma unroll
      for (int g = 0; g < NSC; g++) {
        // (one chain per 32-key group, combined at the end: independent chains issue back to back)
        int mxg[GPS];
#pragma unroll
        for (int t = 0; t < GPS; t++) {
          mxg[t] = acc[g * GPS + t][0];
#pragma unroll
          for (int r = 1; r < 16; r++) mxg[t] = max(mxg[t], acc[g * GPS + t][r]);
        }
        int mx = mxg[0];
#pragma unroll
        for (int t = 1; t < GPS; t++) mx = max(mx, mxg[t]);
        mloc = fmaxf(mloc, __builtin_fmaf(as_f(mx), sc[g], -kBiasF * sc[g]));
      }
      return;
    }
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
#pragma unroll
      for (int sub = 0; sub < SUBS; sub++) {
        float smx;
        if constexpr (KSUB == 3) {
          int mx = acc[nt][2 * sub];
#pragma unroll
          for (int r = 1; r < 16; r++)
            if (subof(r) == sub && r != 2 * sub) mx = max(mx, acc[nt][r]);
          smx = __builtin_fmaf(as_f(mx), sc[nt * SUBS + sub], -kBiasF * sc[nt * SUBS + sub]);
        } else {
          constexpr int RS = 16 / KSUB;
          int mx = acc[nt][sub * RS];
#pragma unroll
          for (int r = 1; r < RS; r++) mx = max(mx, acc[nt][sub * RS + r]);
          smx = __builtin_fmaf(as_f(mx), sc[nt * KSUB + sub], -kBiasF * sc[nt * KSUB + sub]);
        }
        mloc = fmaxf(mloc, smx);
      }
    }
  };

  // ---- online softmax of the tile whose scores are in acc: pure VALU work ----
  auto softmax = [&](int j) {
    // next tile's K scales: requested first, consumed last
    float kraw[NSC];
#pragma unroll
    for (int i = 0; i < NSC; i++) kraw[i] = kscale_at(j + 1, i);
    const float mall = xchg32_max(mloc);
    // Block-scaled codes: the matrix pipe left the sum of the previous tile's codes in osum (unscaled: in the row-sum MFMA a
    // scale block mixes two query rows); it joins the denominator with that tile's factor 2^(e - 8), which is the tile's
    // E8M0 byte moved into a float's exponent field.  Then the byte may be overwritten.
    if constexpr (FASTP) lsum = __builtin_fmaf(osum[0], as_f(pscale << 23), lsum);
    // lazy rescale: move the reference maximum only when it grew by more than TAU (block-scaled codes: only fp32's range
    // is at stake, and the threshold is far larger)
    if (__builtin_amdgcn_ballot_w64(mall > m_used + (FASTP ? kBlockTau : TAU)) != 0) {
      const float m_new = fmaxf(m_used, mall);
      const float alpha = __builtin_amdgcn_exp2f(m_used - m_new);
      lsum *= alpha;
      if constexpr (RSUM && !FASTP) osum[0] *= alpha;
#pragma unroll
      for (int dt = 0; dt < DTN; dt++)
#pragma unroll
        for (int i = 0; i < 16; i++) o[dt][i] *= alpha;
      m_used = m_new;
    }
    // P = exp2(S - m) * 2^PSHIFT, packed straight into the B operand of the second MFMA
    if constexpr (FASTP) {
      // The byte of an e4m3 number, read as an integer, is 8*(exponent + 7) + mantissa: piecewise linear in
      // log2 of the value for codes of 8 and above (the normal numbers).  So y = 8*t + 56, rounded to an integer, is
      // the fp8 code of a number within a mantissa step of 2^t, with the mantissa interpolated linearly between powers
      // of two instead of exponentially (kCodeBias centres the error of that, at most a third of a code step).  Per
      // score that is one v_fma_f32 and three quarters of a conversion instead of v_fma_f32 + v_exp_f32 + half a
      // v_cvt_pk_fp8_f32 (the vector ALU is the busier pipe): v_cvt_pknorm_u16_f32 turns two values x into
      // round(65535 * x), saturating at 0 (masked scores are -inf and give code 0); with x = (256 * y + 127.5) / 65535,
      // which the fma delivers directly, the high byte of each 16-bit result is y rounded to nearest, and one v_perm_b32
      // gathers the high bytes of four results into a dword of the B operand.
      // The linear code only spans the 14.75 binades of the normal numbers (below code 8 an e4m3 byte is linear in the
      // VALUE), so it is used block-scaled: the keys of one 128-key tile form a block per query row whose largest score
      // lands within a binade below the top code, t = s - m - e + kBlockTop with e = ceil(row maximum of the tile - m),
      // and the block's factor 2^e goes to the matrix pipe as the E8M0 scale of the B operand (v_mfma_scale_*: one scale
      // byte per lane; the hardware's scale blocks are the 32-key groups, regs 0-3 / 4-7 of the two lanes of a row, and
      // all four of a tile get the same byte here).  A key is therefore flushed to zero only when it lies 14.75 binades
      // below the largest key of ITS tile -- not below the row's running maximum, as a statically scaled code would do,
      // which loses a flat tail of many keys under a single large one.  The row sums of these very codes, with the
      // same scales, come from the matrix pipe too, so numerator and denominator of O see the same values.
      constexpr float kN = 256.0f / 65535.0f, kN8 = 8.0f * kN;
      constexpr float kC = kN * (56.0f + kCodeBias) + 127.5f / 65535.0f;
      // (a row with no visible key in the tile has maximum -inf: the clamp gives it a finite exponent, its codes are zero)
      const float e = fmaxf(__builtin_ceilf(mall - m_used), kBlockMinExp);
      const float k0 = __builtin_fmaf(-kN8, e, __builtin_fmaf(kN8, kBlockTop - m_used, kC));
      pscale = (int)(unsigned)(e + kBlockScaleBias);
#pragma unroll
      for (int nt = 0; nt < NT; nt++) {
        float c[SUBS], mul[SUBS];
#pragma unroll
        for (int sub = 0; sub < SUBS; sub++) {
          mul[sub] = kN8 * sc[(nt * SUBS + sub) / GPS];
          c[sub] = __builtin_fmaf(-kBiasF, mul[sub], k0);
        }
        float t8[16];
#pragma unroll
        for (int r = 0; r < 16; r++) t8[r] = __builtin_fmaf(as_f(acc[nt][r]), mul[subof(r)], c[subof(r)]);
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
          const unsigned w01 = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_pknorm_u16(t8[4 * q4], t8[4 * q4 + 1]));
          const unsigned w23 = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_pknorm_u16(t8[4 * q4 + 2], t8[4 * q4 + 3]));
          acc[0][4 * nt + q4] = (int)__builtin_amdgcn_perm(w23, w01, 0x07050301u);
        }
      }
    } else if constexpr (PV == 1) {
#pragma unroll
      for (int nt = 0; nt < NT; nt++) {
        float c[SUBS], mul[SUBS];
#pragma unroll
        for (int sub = 0; sub < SUBS; sub++) {
          c[sub] = MASK ? PSHIFT - m_used : __builtin_fmaf(-kBiasF, sc[(nt * SUBS + sub) / GPS], PSHIFT - m_used);
          mul[sub] = MASK ? 1.0f : sc[(nt * SUBS + sub) / GPS];   // masked variants already hold scores
        }
        float p[16];
#pragma unroll
        for (int r = 0; r < 16; r++) {
          p[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(as_f(acc[nt][r]), mul[subof(r)], c[subof(r)]));
          if constexpr (!MSUM) lsum += p[r];   // the unrounded sum, for LSE only
        }
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
          // The packed probabilities of the whole tile (NT*4 dwords) take over the registers of acc[0],
          // whose scores are consumed by then.  Both halves of each dword get written, so the 'old'
          // operand is a don't-care: it is the destination register itself.
          int d0 = __builtin_amdgcn_cvt_pk_fp8_f32(p[4 * q4], p[4 * q4 + 1], acc[0][4 * nt + q4], false);
          acc[0][4 * nt + q4] = __builtin_amdgcn_cvt_pk_fp8_f32(p[4 * q4 + 2], p[4 * q4 + 3], d0, true);
        }
      }
    } else {
#pragma unroll
      for (int nt = 0; nt < NT; nt++) {
        float c[SUBS], mul[SUBS];
#pragma unroll
        for (int sub = 0; sub < SUBS; sub++) {
          c[sub] = MASK ? PSHIFT - m_used : __builtin_fmaf(-kBiasF, sc[(nt * SUBS + sub) / GPS], PSHIFT - m_used);
          mul[sub] = MASK ? 1.0f : sc[(nt * SUBS + sub) / GPS];
        }
        // fp16 probabilities are packed in place: registers 0-7 of each accumulator take the 16 halves
        // (v_cvt_pk_f16_f32, round to nearest even) once the two scores they replace have been consumed.
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          v2f pp;
          pp[0] = __builtin_amdgcn_exp2f(__builtin_fmaf(as_f(acc[nt][r]), mul[subof(r)], c[subof(r)]));
          pp[1] = __builtin_amdgcn_exp2f(__builtin_fmaf(as_f(acc[nt][r + 1]), mul[subof(r)], c[subof(r)]));
          if constexpr (!RSUM) {
            lsum += pp[0];
            lsum += pp[1];
          }
          acc[nt][r >> 1] = __builtin_bit_cast(int, __builtin_convertvector(pp, v2h));
        }
      }
    }
#pragma unroll
    for (int i = 0; i < NSC; i++) sc[i] = qscale * kraw[i];
  };

  // ---- O^T += V^T . P^T ----
  auto pv = [&](int j) {
    const uint8_t* vbuf = vslot(j);
    if constexpr (PV == 1) {
      constexpr int NV = (BN / 64) * DTN, VPF = SAGE_VPF;
      auto vfrag = [&](int i) {
        const uint8_t* vp0 = vbuf + ((i * 2) * 64 + lane) * 16;
        v4i lo = *reinterpret_cast<const v4i*>(vp0);
        v4i hi = *reinterpret_cast<const v4i*>(vp0 + 64 * 16);
        return v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      };
      v8i vf[NV];
#pragma unroll
      for (int i = 0; i < VPF; i++) vf[i] = vfrag(i);
#pragma unroll
      for (int i = 0; i < NV; i++) {
        const int kk = i / DTN, dt = i % DTN;
        if (i + VPF < NV) vf[i + VPF] = vfrag(i + VPF);
        v8i pb;
#pragma unroll
        for (int e = 0; e < 8; e++) pb[e] = acc[0][8 * kk + e];
        if constexpr (FASTP) {
          // block-scaled codes: byte 0 of pscale is the E8M0 scale of this row's codes, V carries 2^0.  The row sums are
          // taken unscaled and per tile (the accumulator starts from zero at the tile's first step): the 16x16x128 form
          // pairs lanes l and l + 16 in one column, so its 32-element scale blocks would mix two query rows.
          if (dt == 0) {
            const v4f zero = {0.f, 0.f, 0.f, 0.f};
            osum = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ones, pb, kk == 0 ? zero : osum, 0, 0, 0, 0, 0, 0);
          }
          o[dt] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(vf[i], pb, o[dt], 0, 0, 0, 127, 0, pscale);
        } else {
          if constexpr (RSUM) {
            if (dt == 0) osum = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ones, pb, osum, 0, 0, 0, 0, 0, 0);
          }
          o[dt] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(vf[i], pb, o[dt], 0, 0, 0, 0, 0, 0);
        }
      }
      __builtin_amdgcn_sched_group_barrier(0x100, 2 * VPF, 0);
#pragma unroll
      for (int i = 0; i < NV; i++) {
        if (RSUM && i % DTN == 0) __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        if (i + VPF < NV) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      }
    } else {
      constexpr int NV = (BN / 16) * DTN, VPF = 4;
      auto vfrag = [&](int i) { return *reinterpret_cast<const v8h*>(vbuf + (i * 64 + lane) * 16); };
      v8h vf[NV];
#pragma unroll
      for (int i = 0; i < VPF; i++) vf[i] = vfrag(i);
#pragma unroll
      for (int i = 0; i < NV; i++) {
        const int k16 = i / DTN, dt = i % DTN;
        if (i + VPF < NV) vf[i + VPF] = vfrag(i + VPF);
        const int nt = k16 >> 1, half = k16 & 1;
        const v4i pw = {acc[nt][4 * half], acc[nt][4 * half + 1], acc[nt][4 * half + 2], acc[nt][4 * half + 3]};
        if constexpr (RSUM) {
          const v4i oh = {ones[0], ones[1], ones[2], ones[3]};
          if (dt == 0)
            osum = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, oh), __builtin_bit_cast(v8h, pw), osum, 0, 0, 0);
        }
        o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[i], __builtin_bit_cast(v8h, pw), o[dt], 0, 0, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x100, VPF, 0);
#pragma unroll
      for (int i = 0; i < NV; i++) {
        if (RSUM && i % DTN == 0) __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        if (i + VPF < NV) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
    }
  };

  // ---- main loop: two groups of wavefronts half a tile apart ----
  // A SIMD hosts one wavefront of each group.  In every phase one of them feeds the matrix pipe
  // (P.V of its previous tile, then Q.K^T of its next tile) while the other runs the softmax of the
  // tile in between on the vector ALU, and they swap at the next barrier: the two pipes of the SIMD
  // are kept busy at the same time instead of taking turns.
  //   phase 2j  : group 0: P.V(j-1), Q.K^T(j)      group 1: softmax(j-1)
  //   phase 2j+1: group 0: softmax(j)              group 1: P.V(j-1), Q.K^T(j)
  // K tile j is read in phases 2j and 2j+1, V tile j in phases 2j+2 and 2j+3.
  SAGE_T(3, qreg[0]);   // Q operand ready
  if (ntiles > 0) {
    const int grp = (w >> GSH) & 1;
    const int wnt = wave_ntiles;
    auto mfma_phase = [&](int j) {
      if (j >= 1 && j - 1 < wnt) pv(j - 1);
      if (j < wnt) { qk(j); rowmax(j); }
    };
    load_scales(0);
    auto even_barrier = [&](int j, int in_flight) {
      wait_all_but(in_flight);   // my pieces of K(j) and V(j-1) have landed
      lds_barrier();             // ... and everyone's; phase 2j-1 is over
#ifdef SAGE_TIMING
      if (j == 0) sage_ts[4] = __builtin_amdgcn_s_memrealtime();   // first K tile landed, all wavefronts arrived
#endif
    };
    const int first_in_flight = (LEAD == 2 && ntiles > 1) ? KPIECES : 0;   // the second K tile, requested in the prologue
    constexpr int PARTNER = PARTNER_DW;
    constexpr int NK = 2 * KPIECES, NV = 2 * VPIECES;   // requests per K / V tile of the wavefront that issues for its SIMD pair
    // Tile requests of period j, issued by one wavefront for both wavefronts of its SIMD pair: K(j+LEAD) and
    // V(j+LEAD-1), LEAD periods before their first use (a tile that has to come from HBM takes longer than one
    // period), into the slots whose last readers finished a barrier ago; with LEAD = 2, V(0) goes first in
    // period 0 and the requests of the last period may still be in flight at a barrier.
    // FP16 kernels of head_dim 128 (twelve requests per period, the V tiles being twice as large) leave the V pieces of
    // group 1's wavefronts to group 1, which requests them at the start of its matrix phase: both matrix phases then
    // carry part of the requests instead of one carrying all of them (+2 % from 4k to 16k keys).
    constexpr bool SPLIT_REQ = PV == 0 && VECMAX;
    // FP8 kernels: group 0 requests the K tile of the period (after its matrix half), group 1 the V tile, as the first
    // thing it does in the period: group 0's period (matrix half, requests, vector half) is the longer one, and V
    // requests at any other place of group 1's period, or the K requests there, measured slower (+1.4 % for this one on
    // config 2, +1.7 % on config 3, +3 % at head_dim 64).
    constexpr bool V_BY_GROUP1 = PV == 1 && LEAD == 2;
    static_assert(!SPLIT_REQ || LEAD == 1, "group 1 requests V(j) in period j");
    auto first_value_tile = [&]() { load_v(0, 0); load_v(0, PARTNER); };
    auto request_tiles = [&](int j, bool with_first_value = true) {
#ifdef SAGE_TIMING
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      const long long rq0 = __builtin_amdgcn_s_memrealtime();
#endif
      if (LEAD == 2 && j == 0 && with_first_value) first_value_tile();
      if (j + LEAD < ntiles) { load_k(j + LEAD, 0); load_k(j + LEAD, PARTNER); }
      if (!V_BY_GROUP1 && j + LEAD - 1 < ntiles) { load_v(j + LEAD - 1, 0); if (!SPLIT_REQ) load_v(j + LEAD - 1, PARTNER); }
#ifdef SAGE_TIMING
      rq_sum += __builtin_amdgcn_s_memrealtime() - rq0;   // ticks this wavefront spent issuing the requests of a period
      rq_n++;
#endif
    };
    auto issuer_in_flight = [&](int j) {
      return j == 0 ? first_in_flight : LEAD == 1 ? 0 : (j + 1 < ntiles ? NK : 0) + (!V_BY_GROUP1 && j < ntiles ? NV : 0);
    };
    // The barrier in the middle of a period only keeps the two groups in step (no tile slot changes hands there: a
    // period's requests go to slots whose last readers finished before the even barrier).  FP8 P.V kernels run without
    // it: a group that finishes its half early starts the other half at once (+1.5 % at head_dim 128, +6 % at
    // head_dim 64, where the vector half is much the longer one); FP16 P.V kernels measured equal or slower without.
    auto odd_barrier = [&]() { if constexpr (PV == 0) lds_barrier(); };
    if constexpr (VECMAX) {
      // FP8 P.V, and FP16 P.V of head_dim 128: the matrix half is nothing but MFMAs and their LDS reads (P.V of the
      // previous tile, Q.K^T of the next); the row maximum and the probabilities belong to the vector half.  Group 0
      // issues its tile requests, for both wavefronts of each SIMD pair, after its last Q.K^T MFMA (a request holds up
      // the wavefront that issues it for 40-50 ns); group 1 issues its share as said above.
      if (grp == 0) {
        for (int j = 0; j <= ntiles; j++) {
          SAGE_PH(3);
          even_barrier(j, issuer_in_flight(j));
          SAGE_PH(0);
          if (LEAD == 2 && j == 0) first_value_tile();   // V(0) has one period only: ahead of the first Q.K^T, not after it
          if (j >= 1 && j - 1 < wnt) pv(j - 1);
          if (j < wnt) qk(j);
          request_tiles(j, false);
          SAGE_PH(1);
          odd_barrier();
          SAGE_PH(2);
          if (j < wnt) { rowmax(j); softmax(j); }
        }
      } else {
        for (int j = 0; j <= ntiles; j++) {
          SAGE_PH(3);
          // (the V tile requested a period ago, for the next period, may still be in flight)
          even_barrier(j, j == 0 ? first_in_flight : (V_BY_GROUP1 && j < ntiles ? NV : 0));
          SAGE_PH(0);
          if (V_BY_GROUP1 && j + 1 < ntiles) { load_v(j + 1, 0); load_v(j + 1, PARTNER); }
          if (j >= 1 && j - 1 < wnt) { rowmax(j - 1); softmax(j - 1); }
          SAGE_PH(1);
          odd_barrier();
          SAGE_PH(2);
          if (SPLIT_REQ && j < ntiles) load_v(j, PARTNER);   // V(j) of the pair's second wavefront: LEAD is 1 here
          if (j >= 1 && j - 1 < wnt) pv(j - 1);
          if (j < wnt) qk(j);
        }
      }
    } else if (grp == 0) {
      // FP16 P.V of head_dim 64.  The even phase is as long as group 1's softmax, which must not start late: all tile loads of
      // the period are issued here, by the group whose matrix phase has slack, after its P.V.
      for (int j = 0; j <= ntiles; j++) {
        even_barrier(j, issuer_in_flight(j));
        if (j >= 1 && j - 1 < wnt) pv(j - 1);
        request_tiles(j);
        if (j < wnt) { qk(j); rowmax(j); }
        lds_barrier();
        if (j < wnt) softmax(j);
      }
    } else {
      for (int j = 0; j <= ntiles; j++) {
        even_barrier(j, j == 0 ? first_in_flight : 0);
        if (j >= 1 && j - 1 < wnt) softmax(j - 1);
        lds_barrier();
        mfma_phase(j);
      }
    }
  }

  SAGE_T(5, lsum);   // main loop done
  // ---- epilogue: O = O^T / l (* v_scale), LSE2 = m + log2(l) ----
  // The denominator of O: FP8 kernels take the matrix pipe's sum of the rounded probabilities (already the full row
  // sum: the MFMA contracts over both key halves; it sits in lanes 0-31, lanes 32-63 hold zero and get it from
  // their partner); the fp32 sum of the unrounded ones serves LSE only.
  float msum = 0.f;
  if constexpr (FASTP) msum = xchg32_sum(__builtin_fmaf(osum[0], as_f(pscale << 23), lsum));   // the last tile's sum is still pending
  else if constexpr (RSUM) msum = xchg32_sum(osum[0]);
  if constexpr (MSUM) lsum = msum;
  else lsum = xchg32_sum(lsum);
  const float den = RSUM ? msum : lsum;
  const float inv = den > 0.f ? 1.0f / den : 0.f;   // a row with no visible key yields zeros
  if (my_row < Lq) {
    if (a.lse && h == 0) {
      // lse_offset: what K smoothing removed from every logit of this row (q . k_mean, base-2 units)
      const float shift = a.lse_offset ? a.lse_offset[lseoff + my_row] : 0.f;
      a.lse[lseoff + my_row] = lsum > 0.f ? m_used + __builtin_amdgcn_logf(lsum) - PSHIFT + shift : kNegInf;
    }
  }
  // O^T (lane = row, registers = channels) goes to memory through LDS: written as stored, a wavefront
  // instruction would touch 16 bytes of 32 different rows; read back row-wise, it stores whole rows
  // (16 bytes per lane, 64 / UPR rows per instruction).  Each wavefront uses a private 32-row region
  // of the tile buffers, which every wavefront has finished reading at the barrier.  16-byte units of
  // a row are XOR-swizzled with the row index so that neither direction piles up on LDS banks.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // (the V scales, when the main loop did not run)
  lds_barrier();
  {
    constexpr int UPR = D / 8;        // 16-byte units per output row
    constexpr int RPI = 64 / UPR;     // rows per store instruction
    uint8_t* stage = smem + w * (32 * D * 2);
    // The lane index is made opaque here: addresses derived from it are then computed now, not before the
    // main loop, where they would be parked in scratch memory for its duration.
    int el = lane;
    asm volatile("" : "+v"(el));
    const int em = el & 31, eh = el >> 5;
    // (one copy of the loop per output type: the type is uniform, and converting both ways and selecting
    // per element would double the conversions)
    auto normalise_and_stage = [&](auto to_out) {
#pragma unroll
      for (int dt = 0; dt < DTN; dt++) {
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
          const int d = 32 * dt + 8 * q4 + 4 * eh;
          float f[4];
#pragma unroll
          for (int i = 0; i < 4; i++) {
            f[i] = o[dt][4 * q4 + i] * inv;
            if constexpr (PV == 1) f[i] *= vs_lds[d + i];
          }
          u16 hv[4];
#pragma unroll
          for (int i = 0; i < 4; i++) hv[i] = to_out(f[i]);
          uint2 pkd = make_uint2((uint32_t)hv[0] | ((uint32_t)hv[1] << 16), (uint32_t)hv[2] | ((uint32_t)hv[3] << 16));
          const int u = 4 * dt + q4;    // 16-byte unit of the row; h picks its half
          *reinterpret_cast<uint2*>(stage + em * (D * 2) + ((u ^ (em & (UPR - 1))) * 16) + 8 * eh) = pkd;
        }
      }
    };
    if (a.out_bf16) normalise_and_stage([](float x) { return f32_to_bf16(x); });
    else normalise_and_stage([](float x) { return f32_to_f16(x); });
    const int k16 = el % UPR, rsub = el / UPR;
#pragma unroll
    for (int i = 0; i < 32 / RPI; i++) {
      const int r = i * RPI + rsub;
      const uint4 val = *reinterpret_cast<const uint4*>(stage + r * (D * 2) + ((k16 ^ (r & (UPR - 1))) * 16));
      if (row0 + r < Lq)
        *reinterpret_cast<uint4*>(reinterpret_cast<u16*>(a.out) + ooff + (int64_t)(row0 + r) * a.o_sn + k16 * 8) = val;
    }
  }
#ifdef SAGE_TIMING
  sage_ts[6] = __builtin_amdgcn_s_memrealtime();   // stores issued
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  sage_ts[7] = __builtin_amdgcn_s_memrealtime();   // stores acknowledged
  if (ntiles == 0) sage_ts[4] = sage_ts[3];
  if (lane == 0) {
    unsigned long long* tt = g_tile_timing[blockIdx.x % kTimingSets];
    const int cls = w == 0 ? 0 : (w == NW - 1 ? 1 : 2);
    for (int i = 0; i < 7; i++) atomicAdd(&tt[cls * 8 + i], (unsigned long long)(sage_ts[i + 1] - sage_ts[i]));
    atomicAdd(&tt[cls * 8 + 7], 1ull);
    if (w == 0) atomicAdd(&tt[24], (unsigned long long)ntiles);
    if (w == NW - 1 && blockIdx.x < kTimelineMax) {
      const unsigned long long where = ((unsigned long long)__builtin_amdgcn_s_getreg(20 | (31 << 11)) << 32) |
                                       (unsigned)__builtin_amdgcn_s_getreg(4 | (31 << 11));
      unsigned long long* rec = g_wg_timeline[blockIdx.x];
      rec[0] = (unsigned long long)sage_ts[0]; rec[1] = (unsigned long long)sage_ts[7]; rec[2] = where; rec[3] = (unsigned long long)ntiles;
    }
    if (w == 1 || w == NW - 2) {   // one wavefront of each group
      const int g = (w >> GSH) & 1;
      for (int i = 0; i < 4; i++) atomicAdd(&tt[32 + 4 * g + i], (unsigned long long)ph_sum[i]);
      atomicAdd(&tt[40 + g], (unsigned long long)ph_n);
      atomicAdd(&tt[42], (unsigned long long)rq_sum);   // [42] / [43]: ticks per period spent issuing the tile requests
      atomicAdd(&tt[43], (unsigned long long)rq_n);
      atomicAdd(&tt[44], (unsigned long long)q_wait);   // [44] / [45]: ticks a wavefront waits for its raw Q rows (and the first K tile)
      atomicAdd(&tt[45], 1ull);
    }
  }
#endif
}


template <int D, int NW, int BN, int PV, bool CAUSAL, bool MSUM, int MASK, int KSUB = 1, bool QF = false, int KW = 1>
static hipError_t launch_one(const AttnArgs& a, int grid, hipStream_t st) {
  constexpr int smem = attn_lds_bytes<D, NW, BN, PV, CAUSAL, QF>();
  auto kern = attn_kernel<D, NW, BN, PV, CAUSAL, MSUM, MASK, KSUB, QF, KW>;
  // More than 64 KB of dynamic LDS has to be allowed once per kernel and device.
  constexpr int kMaxDevices = 64;
  static std::atomic<bool> attr_done[kMaxDevices] = {};   // (two host threads may make the first call at once: setting it twice is harmless)
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= kMaxDevices || !attr_done[dev].load(std::memory_order_acquire)) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return e;
    if (dev >= 0 && dev < kMaxDevices) attr_done[dev].store(true, std::memory_order_release);
  }
  kern<<<dim3(grid), dim3(NW * 64), smem, st>>>(a);
  return hipGetLastError();
}

}  // namespace sage
