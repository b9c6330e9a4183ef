// Launchers of the fused attention kernel (variants without an explicit mask) and the packed-batch plan.
#include "sage_attn_kernel.h"

namespace sage {

// ---------------------------------------------------------------------------------------------
// Variable-length plan: block offsets per sequence and the cost-ordered tile list.
// One workgroup; sequences are few (tens to thousands), tiles up to total_q/128 + nseq.
// ---------------------------------------------------------------------------------------------
constexpr int kCostBins = 2048;

__global__ void __launch_bounds__(1024) varlen_plan_kernel(const int32_t* cu_q, const int32_t* cu_k, int nseq, int total_q,
                                                           int blkq, int blkk, int bm, int bn, int causal, int32_t* plan) {
  const SagePlanLayout L = plan_layout(nseq, total_q);
  int32_t* cu_qblk = plan + L.cu_qblk;
  int32_t* cu_kblk = plan + L.cu_kblk;
  int32_t* cu_panel = plan + L.cu_panel;
  int32_t* tiles = plan + L.tiles;
  __shared__ int hist[kCostBins];
  __shared__ int start[kCostBins];
  const int tid = threadIdx.x;
  for (int i = tid; i < kCostBins; i += blockDim.x) hist[i] = 0;
  if (tid == 0) {
    int aq = 0, ak = 0, ap = 0;
    for (int i = 0; i < nseq; i++) {
      cu_qblk[i] = aq; cu_kblk[i] = ak; cu_panel[i] = ap;
      int lq = cu_q[i + 1] - cu_q[i], lk = cu_k[i + 1] - cu_k[i];
      aq += (lq + blkq - 1) / blkq; ak += (lk + blkk - 1) / blkk; ap += (lk + kPanelRows - 1) / kPanelRows;
    }
    cu_qblk[nseq] = aq; cu_kblk[nseq] = ak; cu_panel[nseq] = ap;
  }
  __syncthreads();
  auto cost_of = [&](int lq, int lk, int qt) {
    int kv_end = causal ? min(lk, (qt + 1) * bm) : lk;
    int c = (kv_end + bn - 1) / bn;
    return min(c, kCostBins - 1);
  };
  // pass 1: histogram of tile costs
  for (int i = 0; i < nseq; i++) {
    int lq = cu_q[i + 1] - cu_q[i], lk = cu_k[i + 1] - cu_k[i];
    int nqt = (lq + bm - 1) / bm;
    for (int qt = tid; qt < nqt; qt += blockDim.x) atomicAdd(&hist[cost_of(lq, lk, qt)], 1);
  }
  __syncthreads();
  // start[c] = number of tiles in more expensive bins: an exclusive scan over the bins in descending cost
  // order, two bins per thread, wavefront scans combined through LDS.
  {
    static_assert(kCostBins == 2048, "two bins per thread of a 1024-thread workgroup");
    __shared__ int wave_total[16];
    const int c0 = kCostBins - 1 - 2 * tid, c1 = c0 - 1;   // this thread's bins, the more expensive one first
    const int h0 = hist[c0], h1 = hist[c1];
    int incl = h0 + h1;
    const int lane = tid & 63, wv = tid >> 6;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int up = __shfl_up(incl, d, 64);
      if (lane >= d) incl += up;
    }
    if (lane == 63) wave_total[wv] = incl;
    __syncthreads();
    int before = 0;
    for (int i = 0; i < wv; i++) before += wave_total[i];
    const int excl = before + incl - (h0 + h1);
    start[c0] = excl;
    start[c1] = excl + h0;
    if (tid == 1023) plan[L.ntiles] = before + incl;
  }
  __syncthreads();
  // pass 2: place tiles.  Few sequences (the usual case): cost TIERS of kTierCost cost units (eight causal q-tiles of
  // 256 rows when the unit is 64 keys), most expensive tier first;
  // inside a tier sequence by sequence, and inside a sequence the heavier q-tiles first.  Consecutive entries of the
  // list run at the same time (eight of them per XCD when an XCD holds one KV head), and q-tiles of one sequence
  // walk the same K/V tiles from tile 0 on at about the same pace: one fetches a tile into the XCD's L2, the others
  // hit it there.  Ordered by cost alone, neighbours in the list belong to different sequences and share nothing.
  // The q-tiles of a sequence that fall into one tier are a contiguous range (cost does not decrease with the tile
  // index), so a tile's place is the tier's fill level plus its distance from the heaviest tile of that range.
  constexpr int kTierCost = 32, kTiers = kCostBins / kTierCost, kMaxTieredSeqs = 64;
  if (nseq <= kMaxTieredSeqs) {
    __shared__ int tier_fill[kTiers], tier_max[kTiers], tier_cnt[kTiers];
    if (tid == 0) {
      int before = 0;
      for (int t = kTiers - 1; t >= 0; t--) {
        tier_fill[t] = before;
        for (int c = 0; c < kTierCost; c++) before += hist[t * kTierCost + c];
      }
    }
    for (int i = 0; i < nseq; i++) {
      const int lq = cu_q[i + 1] - cu_q[i], lk = cu_k[i + 1] - cu_k[i];
      const int nqt = (lq + bm - 1) / bm;
      for (int t = tid; t < kTiers; t += blockDim.x) { tier_max[t] = -1; tier_cnt[t] = 0; }
      __syncthreads();
      for (int qt = tid; qt < nqt; qt += blockDim.x) {
        const int t = cost_of(lq, lk, qt) / kTierCost;
        atomicMax(&tier_max[t], qt);
        atomicAdd(&tier_cnt[t], 1);
      }
      __syncthreads();
      for (int qt = tid; qt < nqt; qt += blockDim.x) {
        const int t = cost_of(lq, lk, qt) / kTierCost;
        tiles[tier_fill[t] + tier_max[t] - qt] = (i << 16) | qt;
      }
      __syncthreads();
      for (int t = tid; t < kTiers; t += blockDim.x) tier_fill[t] += tier_cnt[t];
      __syncthreads();
    }
    return;
  }
  // Many sequences: most expensive cost bins first, in whatever order the tiles of a bin arrive.
  for (int i = 0; i < nseq; i++) {
    int lq = cu_q[i + 1] - cu_q[i], lk = cu_k[i + 1] - cu_k[i];
    int nqt = (lq + bm - 1) / bm;
    for (int qt = tid; qt < nqt; qt += blockDim.x) {
      int pos = atomicAdd(&start[cost_of(lq, lk, qt)], 1);
      tiles[pos] = (i << 16) | qt;
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Launchers
// ---------------------------------------------------------------------------------------------
AttnConfig attn_config(int D, int pv, bool packed) {
  (void)D; (void)packed;
  AttnConfig c;
  c.nw = 8;
  c.bn = 128;
  return c;
}

void finish_attn_args(AttnArgs& a, bool causal) {
  const bool packed = a.cu_q != nullptr;
  a.G = a.Hq / a.Hkv;
  const int heads = packed ? a.Hq : a.B * a.Hq, groups = packed ? a.Hkv : a.B * a.Hkv;
  a.div_G = make_fastdiv(a.G);
  a.div_Hkv = make_fastdiv(a.Hkv);
  a.div_heads = make_fastdiv(heads > 0 ? heads : 1);
  a.tier_shift = -1;
  a.div_range = a.div_last = make_fastdiv(1);
  // Per-XCD tile order (fixed-length batches whose heads and KV groups spread evenly over the eight XCDs): ranges of
  // R = 2^tier_shift consecutive q-tiles, R at most 32 and at most half of a head's q-tiles.  Causal problems with fewer than
  // 16 q-tiles per compute unit keep the plain heaviest-first order -- with so few rounds the balance of the last one
  // matters more than locality (1 x 32 heads of 4096 rows: 7 % slower with ranges) -- unless an XCD holds 16 heads or
  // more and 8 q-tiles per compute unit (4 x 32 heads of 4096 rows: 2 % faster with ranges, 8 x 32 of 2048 rows 5 %).
  if (!packed && (heads & 7) == 0 && (groups & 7) == 0 && (!causal || (int64_t)a.nqt * (heads >> 3) >= 512 || ((int64_t)a.nqt * (heads >> 3) >= 256 && (heads >> 3) >= 16))) {
    int shift = 5;
    while (shift > 0 && (2 << shift) > a.nqt) shift--;
    a.tier_shift = shift;
    const int R = 1 << shift, hpx = heads >> 3, last = a.nqt - (a.nqt >> shift << shift);
    a.div_range = make_fastdiv((uint32_t)R * hpx);
    a.div_last = make_fastdiv(last > 0 ? last : 1);
  }
}

hipError_t launch_attn(const AttnArgs& a, int D, int pv, bool causal, int grid, hipStream_t st) {
  if (grid == 0) return hipSuccess;
  if (a.mask) return launch_attn_masked(a, D, pv, grid, st);
  if (a.k_interleave) return launch_attn_kinterleaved(a, D, pv, causal, grid, st);
  if (a.blkk == 16) return launch_attn_k16(a, D, pv, causal, grid, st);
  if (a.q_raw) return launch_attn_qfused(a, D, pv, causal, grid, st);
  // Row sums on the matrix pipe unless LSE is wanted (FP16 P.V: only head_dim 64 gains by it; head_dim 128 is
  // bound by its matrix phases and keeps the sums on the vector ALU).
  const bool msum = a.lse == nullptr;
  // (K scale blocks of 64 / 128 keys: the variants that know which 32-key groups share a scale)
#define SAGE_ATTN_W(DD, PVV, BNN, MS, KWW) (causal ? launch_one<DD, 8, BNN, PVV, true, MS, 0, 1, false, KWW>(a, grid, st) : launch_one<DD, 8, BNN, PVV, false, MS, 0, 1, false, KWW>(a, grid, st))
#define SAGE_ATTN(DD, PVV, BNN, MS) (a.blkk >= 128 ? SAGE_ATTN_W(DD, PVV, BNN, MS, 4) : a.blkk == 64 ? SAGE_ATTN_W(DD, PVV, BNN, MS, 2) : SAGE_ATTN_W(DD, PVV, BNN, MS, 1))
  if (D == 128) return pv ? (msum ? SAGE_ATTN(128, 1, 128, true) : SAGE_ATTN(128, 1, 128, false)) : SAGE_ATTN(128, 0, 128, false);
  return pv ? (msum ? SAGE_ATTN(64, 1, 128, true) : SAGE_ATTN(64, 1, 128, false)) : (msum ? SAGE_ATTN(64, 0, 128, true) : SAGE_ATTN(64, 0, 128, false));
#undef SAGE_ATTN_W
#undef SAGE_ATTN
}

hipError_t launch_varlen_plan(const int32_t* cu_q, const int32_t* cu_k, int nseq, int total_q, int blkq, int blkk, int bm,
                              int bn, int causal, int32_t* plan, hipStream_t st) {
  varlen_plan_kernel<<<1, 1024, 0, st>>>(cu_q, cu_k, nseq, total_q, blkq, blkk, bm, bn, causal, plan);
  return hipGetLastError();
}

}  // namespace sage
