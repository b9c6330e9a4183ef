// Fused attention kernel variants for four interleaved K scales per block (scale t of a block for its keys n with
// (n % 8) / 2 == t: the granularity upstream SageAttention calls per-thread for K).  Own translation unit so that the sets of
// instantiations compile in parallel.
#include "sage_attn_kernel.h"

namespace sage {

hipError_t launch_attn_kinterleaved(const AttnArgs& a, int D, int pv, bool causal, int grid, hipStream_t st) {
  // Row sums on the matrix pipe for FP8 P.V without LSE, as for the plain K blocks; with a floating-point Q (a.q_raw)
  // the q-tile is quantised in the prologue.
  const bool msum = pv && a.lse == nullptr;
#define SAGE_ATTN_TQ(DD, PVV, MS, QFF) (causal ? launch_one<DD, 8, 128, PVV, true, MS, 0, 3, QFF>(a, grid, st) : launch_one<DD, 8, 128, PVV, false, MS, 0, 3, QFF>(a, grid, st))
#define SAGE_ATTN_T(DD, PVV, MS) (a.q_raw ? SAGE_ATTN_TQ(DD, PVV, MS, true) : SAGE_ATTN_TQ(DD, PVV, MS, false))
  if (D == 128) return pv ? (msum ? SAGE_ATTN_T(128, 1, true) : SAGE_ATTN_T(128, 1, false)) : SAGE_ATTN_T(128, 0, false);
  return pv ? (msum ? SAGE_ATTN_T(64, 1, true) : SAGE_ATTN_T(64, 1, false)) : SAGE_ATTN_T(64, 0, false);
#undef SAGE_ATTN_T
#undef SAGE_ATTN_TQ
}

}  // namespace sage
