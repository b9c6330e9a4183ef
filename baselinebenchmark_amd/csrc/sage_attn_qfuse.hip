// Fused attention kernel variants that quantise their own Q tile in the prologue (the one-call
// pipeline skips the separate pass over Q: one HBM round trip less).  Own translation unit so that
// the sets of instantiations compile in parallel.
#include "sage_attn_kernel.h"

namespace sage {

hipError_t launch_attn_qfused(const AttnArgs& a, int D, int pv, bool causal, int grid, hipStream_t st) {
  const bool msum = pv && a.lse == nullptr;
#define SAGE_ATTN_Q(DD, PVV, BNN, MS) (causal ? launch_one<DD, 8, BNN, PVV, true, MS, 0, 1, true>(a, grid, st) : launch_one<DD, 8, BNN, PVV, false, MS, 0, 1, true>(a, grid, st))
  if (D == 128) return pv ? (msum ? SAGE_ATTN_Q(128, 1, 128, true) : SAGE_ATTN_Q(128, 1, 128, false)) : SAGE_ATTN_Q(128, 0, 128, false);
  return pv ? (msum ? SAGE_ATTN_Q(64, 1, 128, true) : SAGE_ATTN_Q(64, 1, 128, false)) : SAGE_ATTN_Q(64, 0, 128, false);
#undef SAGE_ATTN_Q
}

}  // namespace sage

#ifdef SAGE_TIMING
extern "C" void sage_debug_timing(long long* out) {
  hipMemcpyFromSymbol(out, HIP_SYMBOL(sage::g_dbg), sizeof(long long) * 64);
  long long z[64] = {0};
  hipMemcpyToSymbol(HIP_SYMBOL(sage::g_dbg), z, sizeof(z));
}
#endif
