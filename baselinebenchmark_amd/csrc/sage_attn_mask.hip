// Fused attention kernel variants with an explicit attention mask (boolean or additive), the
// rest of the forward() contract of backends/_hygon/ops/sageattention/sageattention_triton.py:92-105.
// Also here: the variants for K scale blocks of 16 keys (the external MATE recipe (128, 16),
// backends/_mthreads/benchmarks/sage_attention_benchmark_compare.py:93).
// They live in their own translation unit so that the sets of instantiations compile in parallel.
#include "sage_attn_kernel.h"

namespace sage {

hipError_t launch_attn_masked(const AttnArgs& a, int D, int pv, int grid, hipStream_t st) {
  // K scale granularity: one scale per 32-key group or coarser, two per group (K blocks of 16 keys), or four interleaved
  // scales per block -- the masked kernels turn the accumulators into scores element by element and look the scale of
  // every element up, so the finer granularities only change that lookup.
#define SAGE_ATTN_MK(DD, PVV, BNN, KS) (a.mask_kind == 1 ? launch_one<DD, 8, BNN, PVV, false, false, 1, KS>(a, grid, st) : launch_one<DD, 8, BNN, PVV, false, false, 2, KS>(a, grid, st))
#define SAGE_ATTN_M(DD, PVV, BNN) (a.k_interleave ? SAGE_ATTN_MK(DD, PVV, BNN, 3) : a.blkk == 16 ? SAGE_ATTN_MK(DD, PVV, BNN, 2) : SAGE_ATTN_MK(DD, PVV, BNN, 1))
  if (D == 128) return pv ? SAGE_ATTN_M(128, 1, 128) : SAGE_ATTN_M(128, 0, 128);
  return pv ? SAGE_ATTN_M(64, 1, 128) : SAGE_ATTN_M(64, 0, 128);
#undef SAGE_ATTN_M
#undef SAGE_ATTN_MK
}

hipError_t launch_attn_k16(const AttnArgs& a, int D, int pv, bool causal, int grid, hipStream_t st) {
  // Row sums on the matrix pipe for FP8 P.V without LSE, as for the coarser K blocks; with a floating-point
  // Q (a.q_raw) the q-tile is quantised in the prologue.
  const bool msum = pv && a.lse == nullptr;
#define SAGE_ATTN_KQ(DD, PVV, MS, QFF) (causal ? launch_one<DD, 8, 128, PVV, true, MS, 0, 2, QFF>(a, grid, st) : launch_one<DD, 8, 128, PVV, false, MS, 0, 2, QFF>(a, grid, st))
#define SAGE_ATTN_K(DD, PVV, MS) (a.q_raw ? SAGE_ATTN_KQ(DD, PVV, MS, true) : SAGE_ATTN_KQ(DD, PVV, MS, false))
  if (D == 128) return pv ? (msum ? SAGE_ATTN_K(128, 1, true) : SAGE_ATTN_K(128, 1, false)) : SAGE_ATTN_K(128, 0, false);
  return pv ? (msum ? SAGE_ATTN_K(64, 1, true) : SAGE_ATTN_K(64, 1, false)) : SAGE_ATTN_K(64, 0, false);
#undef SAGE_ATTN_K
#undef SAGE_ATTN_KQ
}

}  // namespace sage
