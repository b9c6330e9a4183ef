// Fused attention kernel variants that quantise their own Q tile in the prologue (the one-call
// pipeline skips the separate pass over Q: one HBM round trip less).  Own translation unit so that
// the sets of instantiations compile in parallel.
#include <cstring>
#include "sage_attn_kernel.h"

namespace sage {

hipError_t launch_attn_qfused(const AttnArgs& a, int D, int pv, bool causal, int grid, hipStream_t st) {
  const bool msum = a.lse == nullptr;
#define SAGE_ATTN_QW(DD, PVV, BNN, MS, KWW) (causal ? launch_one<DD, 8, BNN, PVV, true, MS, 0, 1, true, KWW>(a, grid, st) : launch_one<DD, 8, BNN, PVV, false, MS, 0, 1, true, KWW>(a, grid, st))
#define SAGE_ATTN_Q(DD, PVV, BNN, MS) (a.blkk >= 128 ? SAGE_ATTN_QW(DD, PVV, BNN, MS, 4) : a.blkk == 64 ? SAGE_ATTN_QW(DD, PVV, BNN, MS, 2) : SAGE_ATTN_QW(DD, PVV, BNN, MS, 1))
  if (D == 128) return pv ? (msum ? SAGE_ATTN_Q(128, 1, 128, true) : SAGE_ATTN_Q(128, 1, 128, false)) : SAGE_ATTN_Q(128, 0, 128, false);
  return pv ? (msum ? SAGE_ATTN_Q(64, 1, 128, true) : SAGE_ATTN_Q(64, 1, 128, false)) : (msum ? SAGE_ATTN_Q(64, 0, 128, true) : SAGE_ATTN_Q(64, 0, 128, false));
#undef SAGE_ATTN_QW
#undef SAGE_ATTN_Q
}

}  // namespace sage

#ifdef SAGE_TIMING
// Timing build only: copies the interval sums of the kernels of this translation unit (the ones the one-call
// pipeline runs) to `out` (48 values) and clears them.  Synchronises the device.
extern "C" int sage_tile_timing(unsigned long long* out) {
  static unsigned long long sets[sage::kTimingSets][48];
  if (hipDeviceSynchronize() != hipSuccess) return -1;
  if (hipMemcpyFromSymbol(sets, HIP_SYMBOL(sage::g_tile_timing), sizeof(sets)) != hipSuccess) return -1;
  for (int i = 0; i < 48; i++) {
    out[i] = 0;
    for (int s = 0; s < sage::kTimingSets; s++) out[i] += sets[s][i];
  }
  memset(sets, 0, sizeof(sets));
  return hipMemcpyToSymbol(HIP_SYMBOL(sage::g_tile_timing), sets, sizeof(sets)) == hipSuccess ? 0 : -1;
}
// Timing build only: copies the per-workgroup records of the last launch of a kernel of this translation unit (first
// stamp, last stamp, XCC_ID << 32 | HW_ID, K tiles; four values each) for the first `count` workgroups to `out`.
// Synchronises the device.  Returns the number of records copied or -1.
extern "C" int sage_wg_timeline(unsigned long long* out, int count) {
  if (count < 0) return -1;
  if (count > sage::kTimelineMax) count = sage::kTimelineMax;
  if (hipDeviceSynchronize() != hipSuccess) return -1;
  if (hipMemcpyFromSymbol(out, HIP_SYMBOL(sage::g_wg_timeline), (size_t)count * 4 * sizeof(unsigned long long)) != hipSuccess) return -1;
  return count;
}
#endif
