// sage_sageattn_static: the one-call pipeline for callers that cannot allocate device memory (code under HIP
// graph capture, tight serving loops, harnesses that forbid allocation).  The intermediates that sage_sageattn
// keeps in a caller workspace live in a file-scope device array here.  In host code the array's name is only a
// handle, not a device address: the address is looked up once per device, with that device current, and kept.
#include "sage_launch.h"
#include "../../include/sage_mi355x.h"

#include <cstdio>
#include <mutex>

namespace sage {
int set_error(int code, const char* msg);   // sage_api.hip: fills sage_last_error() and returns code
}

namespace {

static __device__ __align__(256) unsigned char scratch[SAGE_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
std::mutex g_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

int fail_hip(hipError_t e, const char* what) {
  char msg[256];
  snprintf(msg, sizeof(msg), "%s: %s", what, hipGetErrorString(e));
  return sage::set_error(SAGE_ELAUNCH, msg);
}

// Device address of the current device's copy of `scratch` (each GPU holds its own copy at its own address).
int scratch_address(void** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail_hip(e, "hipGetDevice");
  if (dev < 0 || dev >= kMaxDevices) return sage::set_error(SAGE_EINVAL, "sage_sageattn_static: device index out of range");
  std::lock_guard<std::mutex> lock(g_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return fail_hip(e, "hipGetSymbolAddress(scratch)");
    if (!p) return sage::set_error(SAGE_ELAUNCH, "hipGetSymbolAddress(scratch) returned a null address");
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return SAGE_OK;
}

}  // namespace

extern "C" {

size_t sage_sageattn_static_capacity(void) { return (size_t)SAGE_STATIC_SCRATCH_BYTES; }

int sage_sageattn_static(const void* q, const void* k, const void* v, void* out, float* lse, int B, int Hq, int Hkv, int Sq,
                         int Skv, int D, int64_t q_sb, int64_t q_sh, int64_t q_sn, int64_t k_sb, int64_t k_sh, int64_t k_sn,
                         int64_t v_sb, int64_t v_sh, int64_t v_sn, int64_t o_sb, int64_t o_sh, int64_t o_sn, int dtype,
                         int blkq, int blkk, double sm_scale, int is_causal, int smooth_k, int pv_mode,
                         const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, int total_q, int total_k,
                         sage_stream_t stream) {
  if (blkq <= 0 || blkk <= 0 || B < 0 || Hq < 0 || Hkv <= 0 || Sq < 0 || Skv < 0 || D <= 0 || total_q < 0 || total_k < 0)
    return sage::set_error(SAGE_EINVAL, "sage_sageattn_static: bad dimension or block size");
  const size_t need = sage_sageattn_workspace_bytes_for(B, Hq, Hkv, Sq, Skv, D, blkq, blkk, pv_mode, total_q, total_k,
                                                        cu_seqlens_q != nullptr, smooth_k, lse != nullptr, 0);
  if (need > (size_t)SAGE_STATIC_SCRATCH_BYTES) {
    char msg[256];
    snprintf(msg, sizeof(msg),
             "sage_sageattn_static: this problem needs %zu bytes of intermediates, the built-in scratch array holds %zu; "
             "use sage_sageattn with a caller workspace", need, (size_t)SAGE_STATIC_SCRATCH_BYTES);
    return sage::set_error(SAGE_EWORKSPACE, msg);
  }
  void* ws = nullptr;
  if (int rc = scratch_address(&ws)) return rc;
  // Every intermediate is written before it is read within one call, so nothing has to be cleared between calls;
  // the kernels receive the looked-up address exactly as they receive a caller workspace.
  return sage_sageattn(q, k, v, out, lse, ws, (size_t)SAGE_STATIC_SCRATCH_BYTES, B, Hq, Hkv, Sq, Skv, D, q_sb, q_sh, q_sn, k_sb,
                       k_sh, k_sn, v_sb, v_sh, v_sn, o_sb, o_sh, o_sn, dtype, blkq, blkk, sm_scale, is_causal, smooth_k, pv_mode,
                       cu_seqlens_q, cu_seqlens_k, total_q, total_k, stream);
}

}  // extern "C"
