// sage_bench: a C++ benchmark driver that calls libsage_mi355x.so through its C ABI directly -- no Python, no torch.
//
//   sage_bench [--batch B] [--heads Hq] [--kv-heads Hkv] [--seq S] [--head-dim D] [--dtype bf16|fp16] [--layout HND|NHD]
//              [--causal 0|1] [--pv fp8|fp16] [--blkq n] [--blkk n] [--warmup W] [--rep R] [--static 0|1]
//
// Fills q, k, v with a fixed pseudo-random sequence on the host (k gets a per-channel offset so that K smoothing has
// work to do), copies them to the device once, runs sage_sageattn W + R times on one stream and times the R calls
// with HIP events, inputs resident in HBM.  Checks the first query row of every head: under a causal mask it sees
// only key 0, so out[row 0] must equal v[row 0] up to the rounding of the P.V format.  Prints one TSV line with the
// columns of the reference's benchmark tables (backends/_enflame/benchmarks/sage_attention_native_benchmark.py:447-455:
// latency in ms and 4*B*H*S^2*D operations per second, halved for causal).  The defaults are BASELINE config 2.
// --static 1 uses sage_sageattn_static (no workspace; small problems only).
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "sage_mi355x.h"

#define HIP_OK(x)                                                                              \
  do {                                                                                         \
    hipError_t e_ = (x);                                                                       \
    if (e_ != hipSuccess) {                                                                    \
      fprintf(stderr, "%s failed: %s\n", #x, hipGetErrorString(e_));                           \
      return 2;                                                                                \
    }                                                                                          \
  } while (0)

static uint16_t to_bits(float f, bool bf16) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if (bf16) return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
  // fp16, round to nearest even; the inputs here are small normal numbers
  uint32_t sign = (u >> 16) & 0x8000u, mant = u & 0x7fffffu;
  int32_t exp = (int32_t)((u >> 23) & 0xff) - 127 + 15;
  if (exp <= 0) return (uint16_t)sign;
  if (exp >= 31) return (uint16_t)(sign | 0x7c00u);
  uint32_t h = ((uint32_t)exp << 10) | (mant >> 13), rem = mant & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
  return (uint16_t)(sign | h);
}
static float from_bits(uint16_t h, bool bf16) {
  uint32_t u;
  if (bf16) u = (uint32_t)h << 16;
  else {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16, exp = (h >> 10) & 0x1f, mant = h & 0x3ffu;
    if (exp == 0) { float f = mant * (1.0f / 16777216.0f); return sign ? -f : f; }
    u = sign | ((exp - 15 + 127) << 23) | (mant << 13);
  }
  float f;
  memcpy(&f, &u, 4);
  return f;
}

struct Rng {   // xorshift64* and a sum of uniforms: a bell-shaped value in about [-3, 3], the same on every run
  uint64_t s;
  float next() {
    float acc = 0.f;
    for (int i = 0; i < 4; i++) {
      s ^= s >> 12; s ^= s << 25; s ^= s >> 27;
      acc += (float)((s * 0x2545F4914F6CDD1Dull) >> 40) * (1.0f / 16777216.0f);
    }
    return (acc - 2.0f) * 1.7320508f;
  }
};

int main(int argc, char** argv) {
  int B = 2, Hq = 32, Hkv = 32, S = 16384, D = 128, causal = 1, blkq = 64, blkk = 128, warmup = 10, rep = 20, use_static = 0;
  std::string dtype = "bf16", layout = "HND", pv = "fp8";
  for (int i = 1; i + 1 < argc; i += 2) {
    std::string a = argv[i];
    const char* v = argv[i + 1];
    if (a == "--batch") B = atoi(v);
    else if (a == "--heads") Hq = atoi(v);
    else if (a == "--kv-heads") Hkv = atoi(v);
    else if (a == "--seq") S = atoi(v);
    else if (a == "--head-dim") D = atoi(v);
    else if (a == "--dtype") dtype = v;
    else if (a == "--layout") layout = v;
    else if (a == "--causal") causal = atoi(v);
    else if (a == "--pv") pv = v;
    else if (a == "--blkq") blkq = atoi(v);
    else if (a == "--blkk") blkk = atoi(v);
    else if (a == "--warmup") warmup = atoi(v);
    else if (a == "--rep") rep = atoi(v);
    else if (a == "--static") use_static = atoi(v);
    else { fprintf(stderr, "unknown option %s\n", a.c_str()); return 1; }
  }
  const bool bf16 = dtype == "bf16", hnd = layout == "HND";
  const int pv_mode = pv == "fp8" ? SAGE_PV_FP8 : SAGE_PV_FP16;
  const size_t nq = (size_t)B * Hq * S * D, nk = (size_t)B * Hkv * S * D;
  auto strides = [&](int H, int64_t& sb, int64_t& sh, int64_t& sn) {
    sb = (int64_t)H * S * D;
    if (hnd) { sh = (int64_t)S * D; sn = D; } else { sh = D; sn = (int64_t)H * D; }
  };
  int64_t q_sb, q_sh, q_sn, k_sb, k_sh, k_sn;
  strides(Hq, q_sb, q_sh, q_sn);
  strides(Hkv, k_sb, k_sh, k_sn);

  std::vector<uint16_t> hq(nq), hk(nk), hv(nk);
  Rng rng{0x9E3779B97F4A7C15ull};
  for (auto& x : hq) x = to_bits(rng.next(), bf16);
  std::vector<float> offset((size_t)Hkv * D);
  for (auto& x : offset) x = 2.0f * rng.next();
  for (int b = 0; b < B; b++)
    for (int h = 0; h < Hkv; h++)
      for (int n = 0; n < S; n++)
        for (int d = 0; d < D; d++) {
          size_t i = (size_t)b * k_sb + (size_t)h * k_sh + (size_t)n * k_sn + d;
          hk[i] = to_bits(rng.next() + offset[(size_t)h * D + d], bf16);
          hv[i] = to_bits(rng.next(), bf16);
        }

  void *dq, *dk, *dv, *dout, *ws = nullptr;
  HIP_OK(hipMalloc(&dq, nq * 2));
  HIP_OK(hipMalloc(&dk, nk * 2));
  HIP_OK(hipMalloc(&dv, nk * 2));
  HIP_OK(hipMalloc(&dout, nq * 2));
  HIP_OK(hipMemcpy(dq, hq.data(), nq * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dk, hk.data(), nk * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dv, hv.data(), nk * 2, hipMemcpyHostToDevice));
  const size_t ws_bytes = sage_sageattn_workspace_bytes(B, Hq, Hkv, S, S, D, blkq, blkk, pv_mode, 0, 0, 0);
  if (!use_static) HIP_OK(hipMalloc(&ws, ws_bytes ? ws_bytes : 256));
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  hipEvent_t e0, e1;
  HIP_OK(hipEventCreate(&e0));
  HIP_OK(hipEventCreate(&e1));

  auto call = [&]() {
    if (use_static)
      return sage_sageattn_static(dq, dk, dv, dout, nullptr, B, Hq, Hkv, S, S, D, q_sb, q_sh, q_sn, k_sb, k_sh, k_sn, k_sb, k_sh,
                                  k_sn, q_sb, q_sh, q_sn, bf16 ? SAGE_DT_BF16 : SAGE_DT_F16, blkq, blkk, 0.0, causal, 1, pv_mode,
                                  nullptr, nullptr, 0, 0, stream);
    return sage_sageattn(dq, dk, dv, dout, nullptr, ws, ws_bytes, B, Hq, Hkv, S, S, D, q_sb, q_sh, q_sn, k_sb, k_sh, k_sn, k_sb,
                         k_sh, k_sn, q_sb, q_sh, q_sn, bf16 ? SAGE_DT_BF16 : SAGE_DT_F16, blkq, blkk, 0.0, causal, 1, pv_mode,
                         nullptr, nullptr, 0, 0, stream);
  };
  for (int i = 0; i < warmup; i++)
    if (int rc = call()) { fprintf(stderr, "sage_sageattn: %d %s\n", rc, sage_last_error()); return 3; }
  HIP_OK(hipStreamSynchronize(stream));
  HIP_OK(hipEventRecord(e0, stream));
  for (int i = 0; i < rep; i++)
    if (int rc = call()) { fprintf(stderr, "sage_sageattn: %d %s\n", rc, sage_last_error()); return 3; }
  HIP_OK(hipEventRecord(e1, stream));
  HIP_OK(hipStreamSynchronize(stream));
  float ms = 0.f;
  HIP_OK(hipEventElapsedTime(&ms, e0, e1));
  ms /= rep;

  // gate: query row 0 of every head (causal: it sees key 0 only)
  std::vector<uint16_t> hout(nq);
  HIP_OK(hipMemcpy(hout.data(), dout, nq * 2, hipMemcpyDeviceToHost));
  double worst = 0.0;
  bool finite = true;
  for (size_t i = 0; i < nq; i += 997) finite = finite && std::isfinite(from_bits(hout[i], bf16));
  if (causal) {
    for (int b = 0; b < B; b++)
      for (int h = 0; h < Hq; h++)
        for (int d = 0; d < D; d++) {
          float o = from_bits(hout[(size_t)b * q_sb + (size_t)h * q_sh + d], bf16);
          float v0 = from_bits(hv[(size_t)b * k_sb + (size_t)(h / (Hq / Hkv)) * k_sh + d], bf16);
          worst = std::fmax(worst, std::fabs(o - v0) / (std::fabs(v0) + 0.5));
        }
  }
  const bool pass = finite && worst < 0.08;
  const double ops = 4.0 * B * Hq * (double)S * S * D * (causal ? 0.5 : 1.0);
  printf("backend\tdtype\tlayout\tB\tHq\tHkv\tS\tD\tcausal\tpv\tblkq\tblkk\tlatency_ms\tTOPS\tgate\n");
  printf("%s\t%s\t%s\t%d\t%d\t%d\t%d\t%d\t%d\t%s\t%d\t%d\t%.4f\t%.1f\t%s\n", sage_backend_name(), dtype.c_str(), layout.c_str(), B, Hq,
         Hkv, S, D, causal, pv.c_str(), blkq, blkk, ms, ops / (ms * 1e-3) / 1e12, pass ? "PASS" : "FAIL");
  return pass ? 0 : 4;
}
