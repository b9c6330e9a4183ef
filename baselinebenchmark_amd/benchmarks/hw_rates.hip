// Micro-benchmarks of the gfx950 units the attention kernel is priced against: the two MFMA
// instructions it uses (operands from registers, and fed from LDS the way the kernel feeds them), LDS
// reads, and the vector instructions of the softmax.  They give the denominators MEASURED on the
// box next to the datasheet ones.  No counterpart in the reference: a measurement aid.
//
// One workgroup per compute unit, 1, 2 or 4 wavefronts per SIMD; the caller times the launch (the
// in-kernel clock s_memtime does not advance at wall-clock rate when wavefronts share a SIMD).
#include "../csrc/sage_common.h"
#include "hw_rates.h"

namespace sage {
namespace {

constexpr int kMbLdsInts = 16384;   // 64 KB

enum : int { MB_MFMA_I8 = 0, MB_MFMA_F8 = 1, MB_LDS = 2, MB_MFMA_I8_LDS = 3, MB_MFMA_F8_LDS = 4,
             MB_FMA = 5, MB_EXP = 6, MB_CVT_FP8 = 7, MB_SOFTMAX_MIX = 8, MB_KINDS = 9 };

template <int KIND>
__global__ void __launch_bounds__(1024) microbench_kernel(int* sink, int iters, int active_waves, float s, float c) {
  __shared__ __attribute__((aligned(16))) int buf[kMbLdsInts];
  for (int i = threadIdx.x; i < kMbLdsInts; i += blockDim.x) buf[i] = i * 7 + 1;
  __syncthreads();
  if ((int)(threadIdx.x >> 6) >= active_waves) return;
  const int lane = threadIdx.x & 63;
  int result = 0;
  if constexpr (KIND == MB_MFMA_I8 || KIND == MB_MFMA_I8_LDS || KIND == MB_LDS) {
    // per iteration: 16 fragments of 1 KB (lane-linear, conflict free) and/or 16 MFMAs on four accumulators
    const v4i* p = reinterpret_cast<const v4i*>(buf) + lane;
    v4i q = {lane, 1, 2, 3};
    v16i acc[4] = {};
    v4i sum = {0, 0, 0, 0};
    constexpr int N = 16, PF = 4;
    for (int it = 0; it < iters; it++) {
      const v4i* pp = p + (it & 3) * 1024;
      v4i f[N];
      if (KIND != MB_MFMA_I8) {
#pragma unroll
        for (int i = 0; i < PF; i++) f[i] = pp[i * 64];
      }
#pragma unroll
      for (int i = 0; i < N; i++) {
        if (KIND != MB_MFMA_I8 && i + PF < N) f[i + PF] = pp[(i + PF) * 64];
        __builtin_amdgcn_sched_barrier(0);
        if (KIND == MB_MFMA_I8) acc[i & 3] = __builtin_amdgcn_mfma_i32_32x32x32_i8(q, q, acc[i & 3], 0, 0, 0);
        if (KIND == MB_LDS) sum ^= f[i];
        if (KIND == MB_MFMA_I8_LDS) acc[i & 3] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f[i], q, acc[i & 3], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    result = sum[0] ^ sum[1] ^ sum[2] ^ sum[3];
    for (int k = 0; k < 4; k++) result ^= acc[k][0];
  } else if constexpr (KIND == MB_MFMA_F8 || KIND == MB_MFMA_F8_LDS) {
    // per iteration: 8 MFMAs f8f6f4 32x32x64 (2 KB fragment each when fed from LDS)
    const v4i* p = reinterpret_cast<const v4i*>(buf) + lane;
    v8i q8 = {lane, 1, 2, 3, 4, 5, 6, 7};
    v16f acc[4] = {};
    constexpr int N = 8, PF = 3;
    for (int it = 0; it < iters; it++) {
      const v4i* pp = p + (it & 3) * 1024;
      auto ld = [&](int i) {
        v4i lo = pp[(2 * i) * 64], hi = pp[(2 * i + 1) * 64];
        return v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      };
      v8i f[N];
      if (KIND == MB_MFMA_F8_LDS) {
#pragma unroll
        for (int i = 0; i < PF; i++) f[i] = ld(i);
      }
#pragma unroll
      for (int i = 0; i < N; i++) {
        if (KIND == MB_MFMA_F8_LDS && i + PF < N) f[i + PF] = ld(i + PF);
        __builtin_amdgcn_sched_barrier(0);
        if (KIND == MB_MFMA_F8) acc[i & 3] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(q8, q8, acc[i & 3], 0, 0, 0, 0, 0, 0);
        else acc[i & 3] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(f[i], q8, acc[i & 3], 0, 0, 0, 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    for (int k = 0; k < 4; k++) result ^= (int)acc[k][0];
  } else {
    // vector ALU: 32 independent values per lane; MB_SOFTMAX_MIX = per value one fma, one exp2, half a packed fp8 conversion
    float x[32];
    int pk[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int i = 0; i < 32; i++) x[i] = lane * 1e-3f + i * 0.01f;
    for (int it = 0; it < iters; it++) {
      if constexpr (KIND == MB_FMA) {
#pragma unroll
        for (int i = 0; i < 32; i++) x[i] = __builtin_fmaf(x[i], s, c);
      } else if constexpr (KIND == MB_EXP) {
#pragma unroll
        for (int i = 0; i < 32; i++) x[i] = __builtin_amdgcn_exp2f(x[i]);
      } else {
        float p[32];
#pragma unroll
        for (int i = 0; i < 32; i++) p[i] = KIND == MB_SOFTMAX_MIX ? __builtin_amdgcn_exp2f(__builtin_fmaf(x[i], s, c)) : x[i];
#pragma unroll
        for (int i = 0; i < 8; i++) {
          int d0 = __builtin_amdgcn_cvt_pk_fp8_f32(p[4 * i], p[4 * i + 1], pk[i], false);
          pk[i] = __builtin_amdgcn_cvt_pk_fp8_f32(p[4 * i + 2], p[4 * i + 3], d0, true);
        }
        // nothing of an iteration is loop invariant or dead
#pragma unroll
        for (int i = 0; i < 8; i++) asm volatile("" : "+v"(pk[i]));
#pragma unroll
        for (int i = 0; i < 32; i++) asm volatile("" : "+v"(x[i]));
      }
    }
    float r = 0.f;
    for (int i = 0; i < 32; i++) r += x[i];
    for (int i = 0; i < 8; i++) result ^= pk[i];
    result ^= (int)r;
  }
  sink[blockIdx.x * 1024 + threadIdx.x] = result;
}

// Co-execution of the two pipes of a SIMD: a workgroup of eight wavefronts, two per SIMD; wavefronts 0-3 issue MFMAs
// (MK 0: v_mfma_i32_32x32x32_i8, 1: v_mfma_f32_32x32x64_f8f6f4, four accumulators in turn), wavefronts 4-7 vector
// instructions (VK 0: v_fma_f32, 1: v_cvt_pk_u8_f32, 2: v_max3_i32, 3: the mix of the FP8 softmax without v_exp_f32: per
// 64 scores 64 fma + 64 cvt_pk_u8 + 32 max3; 4: the mix the kernels run now, 64 fma + 32 cvt_pknorm_u16 + 16 perm + 32 max3).  mode bit 0 / 1 switches each half on: timing a half alone and both together
// says how much the pipes slow each other down.  Per iteration: 16 MFMAs, or 64 / 64 / 32 / 160 vector instructions.
template <int MK, int VK>
__global__ void __launch_bounds__(512) coexec_kernel(int* sink, int iters, int mode, float s, float c) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  int result = 0;
  if (wave < 4) {
    if (!(mode & 1)) return;
    v8i a8 = {lane, 1, 2, 3, 4, 5, 6, 7};
    v4i a4 = {lane, 1, 2, 3};
    v16f accf[4] = {};
    v16i acci[4] = {};
    for (int it = 0; it < iters; it++) {
#pragma unroll
      for (int i = 0; i < 16; i++) {
        if constexpr (MK == 0) acci[i & 3] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a4, a4, acci[i & 3], 0, 0, 0);
        else accf[i & 3] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, a8, accf[i & 3], 0, 0, 0, 0, 0, 0);
      }
    }
    for (int k = 0; k < 4; k++) result ^= MK == 0 ? acci[k][0] : (int)accf[k][0];
  } else {
    if (!(mode & 2)) return;
    float x[16];
    unsigned pk[4] = {0, 0, 0, 0};
    int mx[4] = {0, 0, 0, 0};
    for (int i = 0; i < 16; i++) x[i] = lane * 1e-3f + i * 0.01f;
    for (int it = 0; it < iters; it++) {
#pragma unroll
      for (int u = 0; u < 4; u++) {
        if constexpr (VK == 0 || VK == 3 || VK == 4) {
#pragma unroll
          for (int i = 0; i < 16; i++) x[i] = __builtin_fmaf(x[i], s, c);
        }
        if constexpr (VK == 4) {   // two codes per conversion, one v_perm_b32 per four
#pragma unroll
          for (int i = 0; i < 16; i += 4) {
            const unsigned w01 = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_pknorm_u16(x[i], x[i + 1]));
            const unsigned w23 = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_pknorm_u16(x[i + 2], x[i + 3]));
            pk[i >> 2] ^= __builtin_amdgcn_perm(w23, w01, 0x07050301u);
          }
        }
        if constexpr (VK == 1 || VK == 3) {
#pragma unroll
          for (int i = 0; i < 16; i++) pk[i >> 2] = __builtin_amdgcn_cvt_pk_u8_f32(x[i], i & 3, pk[i >> 2]);
        }
        if constexpr (VK == 2 || VK == 3 || VK == 4) {
#pragma unroll
          for (int i = 0; i < 16; i += 2)
            mx[(i >> 1) & 3] = max(max(mx[(i >> 1) & 3], __builtin_bit_cast(int, x[i])), __builtin_bit_cast(int, x[i + 1]));
        }
        // nothing of an iteration is loop invariant or dead
#pragma unroll
        for (int i = 0; i < 4; i++) asm volatile("" : "+v"(pk[i]), "+v"(mx[i]));
#pragma unroll
        for (int i = 0; i < 16; i++) asm volatile("" : "+v"(x[i]));
      }
    }
    float r = 0.f;
    for (int i = 0; i < 16; i++) r += x[i];
    for (int i = 0; i < 4; i++) result ^= (int)pk[i] ^ mx[i];
    result ^= (int)r;
  }
  sink[blockIdx.x * 1024 + threadIdx.x] = result;
}

// ---------------------------------------------------------------------------------------------
// The steady-state tile period of the FP8 P.V attention kernel (head_dim 128, 128-key tiles) as an instruction mix
// without the attention around it: a workgroup of eight wavefronts in two groups half a period apart, one LDS-only
// barrier per period.  Per period every wavefront runs a matrix half -- P.V: 8 v_mfma_f32_32x32x64_f8f6f4 whose A
// fragments are 16 ds_read_b128 (three pairs ahead) plus 2 v_mfma_f32_16x16x128_f8f6f4 on a resident operand; Q.K^T: 16
// v_mfma_i32_32x32x32_i8 whose A fragments are 16 ds_read_b128 (four ahead), the first of each accumulator starting from
// a resident bias block -- and a vector half on the 64 scores per lane the Q.K^T left: four integer max3 chains, the
// exchange with the lane that shares the row, the block exponent and constants, 64 v_fma_f32, 32 v_cvt_pknorm_u16_f32,
// 16 v_perm_b32, whose result is the B operand of the next P.V.  Group 0 issues four 1 KB global->LDS requests after its
// matrix half, group 1 four at the start of its period (32 KB per period and workgroup, from a 1 MB window per
// XCD -- workgroup index modulo 8 -- that its L2 serves after the first pass, as the shared K/V tiles of a head are).  PARTS switches the pieces on: 1 MFMAs, 2 fragment reads from LDS
// (off: the MFMAs take resident registers), 4 the vector half, 8 the global->LDS requests.  The time of a period with
// everything on is what this schedule costs on the hardware before any attention-specific overhead (masks, rescales,
// prologue, epilogue, imbalance); with single pieces on, what each of them costs alone.
// ---------------------------------------------------------------------------------------------
template <int PARTS>
__global__ void __launch_bounds__(512) period_kernel(int* sink, const uint8_t* src, int periods, int random_operands, float s, float c) {
  constexpr bool MFMA = PARTS & 1, LDSF = PARTS & 2, VEC = PARTS & 4, DMA = PARTS & 8;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];   // 64 KB of fragments + 32 KB that the requests fill
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63, grp = wave >> 2;
  // Operand bits: a regular low-entropy pattern, or hashed bytes (what quantised data looks like to the multipliers; the
  // lowest bit of every byte cleared so that no FP8 byte is a NaN).  The instruction stream is the same either way.
  auto hashed = [](unsigned x) {
    x *= 2654435761u; x ^= x >> 15; x *= 2246822519u; x ^= x >> 13; x *= 3266489917u; x ^= x >> 16;
    return (int)(x & 0xFEFEFEFEu);
  };
  for (int i = threadIdx.x; i < 65536 / 4; i += 512)
    reinterpret_cast<int*>(smem)[i] = random_operands ? hashed(i + blockIdx.x * 16384) : i * 7 + 1;
  __syncthreads();
  const __amdgpu_buffer_rsrc_t rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)(src + (size_t)(blockIdx.x & 7) * (1u << 20)), 0, 0x7fffffff, 0x00020000);
  v4i q[4];
  v16i bias, acc[4];
  v16f o[4];
  v4f osum = {0.f, 0.f, 0.f, 0.f};
  v8i ones;
  for (int k = 0; k < 4; k++) {
    q[k] = v4i{lane + k, 1, 2, 3};
    if (random_operands)
      for (int e = 0; e < 4; e++) q[k][e] = hashed(0x40000000u + ((blockIdx.x * 512 + threadIdx.x) * 4 + k) * 4 + e);
  }
  for (int i = 0; i < 16; i++) bias[i] = 0x4B400000;
  for (int i = 0; i < 8; i++) ones[i] = (lane == 0 || lane == 32 || lane == 20 || lane == 52) ? 0x38383838 : 0;
  for (int k = 0; k < 4; k++) { acc[k] = bias; for (int i = 0; i < 16; i++) o[k][i] = 0.f; }
  asm volatile("" : "+v"(bias), "+v"(ones));
  float m_used = 0.f, lsum = 0.f, sc = s * 1e-4f;
  int pscale = 119;
  auto matrix_half = [&](int p) {
    if constexpr (!MFMA) return;
    const uint8_t* vbuf = smem + ((p & 1) ? 32768 : 0) + lane * 16;
    const uint8_t* kbuf = smem + ((p & 1) ? 0 : 32768) + 16384 + lane * 16;
    {   // P.V: the packed probabilities are registers 0..15 of acc[0]
      v8i vf[8];
      auto vfrag = [&](int i) {
        if constexpr (!LDSF) return v8i{acc[1][0], 1, 2, 3, 4, 5, 6, i};
        const v4i lo = *reinterpret_cast<const v4i*>(vbuf + (2 * i) * 1024), hi = *reinterpret_cast<const v4i*>(vbuf + (2 * i + 1) * 1024);
        return v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      };
#pragma unroll
      for (int i = 0; i < 3; i++) vf[i] = vfrag(i);
#pragma unroll
      for (int i = 0; i < 8; i++) {
        const int kk = i / 4, dt = i % 4;
        if (i + 3 < 8) vf[i + 3] = vfrag(i + 3);
        v8i pb;
#pragma unroll
        for (int e = 0; e < 8; e++) pb[e] = acc[0][8 * kk + e];
        if (dt == 0) {
          const v4f zero = {0.f, 0.f, 0.f, 0.f};
          osum = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ones, pb, kk == 0 ? zero : osum, 0, 0, 0, 0, 0, 0);
        }
        o[dt] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(vf[i], pb, o[dt], 0, 0, 0, 127, 0, pscale);
      }
      if constexpr (LDSF) {
        __builtin_amdgcn_sched_group_barrier(0x100, 6, 0);
#pragma unroll
        for (int i = 0; i < 8; i++) {
          if (i % 4 == 0) __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          if (i + 3 < 8) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        }
      }
    }
    {   // Q.K^T
      v4i kf[16];
      auto kfrag = [&](int i) {
        if constexpr (!LDSF) return v4i{(int)o[0][0], 1, 2, i};
        return *reinterpret_cast<const v4i*>(kbuf + i * 1024);
      };
#pragma unroll
      for (int i = 0; i < 4; i++) kf[i] = kfrag(i);
#pragma unroll
      for (int i = 0; i < 16; i++) {
        if (i + 4 < 16) kf[i + 4] = kfrag(i + 4);
        const int nt = i % 4, ks = i / 4;
        acc[nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf[i], q[ks], ks == 0 ? bias : acc[nt], 0, 0, 0);
      }
      if constexpr (LDSF) {
        __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
        for (int i = 0; i < 12; i++) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
      }
    }
  };
  auto vector_half = [&]() {
    if constexpr (!VEC) return;
    int mxg[4];
#pragma unroll
    for (int t = 0; t < 4; t++) {
      mxg[t] = acc[t][0];
#pragma unroll
      for (int r = 1; r < 16; r++) mxg[t] = max(mxg[t], acc[t][r]);
    }
    const int mx = max(max(mxg[0], mxg[1]), max(mxg[2], mxg[3]));
    float mloc = __builtin_fmaf(__builtin_bit_cast(float, mx), sc, -12582912.0f * sc);
    auto r2 = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(int, mloc), __builtin_bit_cast(int, mloc), false, false);
    const float mall = fmaxf(__builtin_bit_cast(float, (int)r2[0]), __builtin_bit_cast(float, (int)r2[1]));
    lsum = __builtin_fmaf(osum[0], __builtin_bit_cast(float, pscale << 23), lsum);
    if (__builtin_amdgcn_ballot_w64(mall > m_used + 1.0e30f) != 0) m_used = mall;      // (never taken: the rescale is rare)
    const float e = fmaxf(__builtin_ceilf(mall - m_used), -110.0f);
    constexpr float kN8 = 8.0f * 256.0f / 65535.0f;
    const float k0 = __builtin_fmaf(-kN8, e, __builtin_fmaf(kN8, 8.75f - m_used, c));
    pscale = (int)(unsigned)(e + 119.0f);
    const float mul = kN8 * sc, cc = __builtin_fmaf(-12582912.0f, mul, k0);
#pragma unroll
    for (int nt = 0; nt < 4; nt++) {
      float t8[16];
#pragma unroll
      for (int r = 0; r < 16; r++) t8[r] = __builtin_fmaf(__builtin_bit_cast(float, (int)acc[nt][r]), mul, cc);
#pragma unroll
      for (int q4 = 0; q4 < 4; q4++) {
        const unsigned w01 = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_pknorm_u16(t8[4 * q4], t8[4 * q4 + 1]));
        const unsigned w23 = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_pknorm_u16(t8[4 * q4 + 2], t8[4 * q4 + 3]));
        acc[0][4 * nt + q4] = (int)__builtin_amdgcn_perm(w23, w01, 0x07050301u);
      }
    }
    sc = sc * 1.0000001f;
  };
  auto requests = [&](int p) {
    if constexpr (!DMA) return;
    uint8_t* dst = smem + 65536 + (wave & 3) * 8192 + grp * 4096;       // (the data is never read: only the traffic matters)
    const int uo = ((p * 32768) & ((1 << 20) - 1)) + wave * 4096;
#pragma unroll
    for (int i = 0; i < 4; i++)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)(dst + i * 1024), 16, lane * 16, uo + i * 1024, 0, 0);
  };
  auto period_start = [&]() {
    if constexpr (DMA) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");     // the requests of the period before last have landed
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    if constexpr (!MFMA) {      // without the MFMAs nothing renews the scores: keep the vector half from being hoisted
#pragma unroll
      for (int k = 0; k < 4; k++) asm volatile("" : "+v"(acc[k]));
    }
  };
  // (one loop per group, as in the attention kernel: two copies of the matrix half inside one loop cost the compiler its
  // register allocation)
  if (grp == 0) {
    for (int p = 0; p < periods; p++) { period_start(); matrix_half(p); requests(p); vector_half(); }
  } else {
    for (int p = 0; p < periods; p++) { period_start(); requests(p); vector_half(); matrix_half(p); }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  int result = (int)lsum ^ pscale;
  for (int k = 0; k < 4; k++) result ^= acc[k][0] ^ (int)o[k][0];
  sink[blockIdx.x * 1024 + threadIdx.x] = result;
}


template <int PARTS>
hipError_t launch_period(int* sink, const uint8_t* src, int grid, int periods, int random_operands, hipStream_t st) {
  auto kern = period_kernel<PARTS>;
  static bool attr_done = false;
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 98304);
    if (e != hipSuccess) return e;
    attr_done = true;
  }
  kern<<<dim3(grid), dim3(512), 98304, st>>>(sink, src, periods, random_operands, random_operands ? 0.25f : 0.999f, 0.001f);
  return hipGetLastError();
}

template <int MK, int VK>
hipError_t launch_coexec(int* sink, int grid, int iters, int mode, hipStream_t st) {
  coexec_kernel<MK, VK><<<dim3(grid), dim3(512), 0, st>>>(sink, iters, mode, 0.999f, 0.001f);
  return hipGetLastError();
}

template <int KIND>
hipError_t launch_mb(int* sink, int grid, int waves, int iters, hipStream_t st) {
  microbench_kernel<KIND><<<dim3(grid), dim3(waves * 64), 0, st>>>(sink, iters, waves, 0.999f, 0.001f);
  return hipGetLastError();
}

}  // namespace
}  // namespace sage

extern "C" {

// Units of work one wavefront does per iteration of benchmark `kind` (MFMA: multiply-add operations
// counted as 2; LDS: bytes read; vector ALU: instructions), or 0 for an unknown kind.
double sage_microbench_units(int kind) {
  using namespace sage;
  switch (kind) {
    case MB_MFMA_I8: case MB_MFMA_I8_LDS: return 16.0 * 2 * 32 * 32 * 32;
    case MB_MFMA_F8: case MB_MFMA_F8_LDS: return 8.0 * 2 * 32 * 32 * 64;
    case MB_LDS: return 16.0 * 1024;
    case MB_FMA: case MB_EXP: return 32.0;
    case MB_CVT_FP8: return 16.0;
    case MB_SOFTMAX_MIX: return 80.0;
    default: return 0.0;
  }
}

// Launches benchmark `kind` on `grid` workgroups of 4 * waves_per_simd wavefronts (waves_per_simd 1, 2 or 4), `iters`
// iterations each.  `sink` receives one int per thread (grid * 1024 ints).  Returns 0 or a negative HWR_E* code.
int sage_microbench(int kind, int grid, int waves_per_simd, int iters, void* sink, size_t sink_bytes, void* stream) {
  using namespace sage;
  if (kind < 0 || kind >= MB_KINDS || grid <= 0 || grid > 65535 || iters <= 0 || !sink) return HWR_EINVAL;
  if (waves_per_simd != 1 && waves_per_simd != 2 && waves_per_simd != 4) return HWR_EINVAL;
  if (sink_bytes < (size_t)grid * 1024 * sizeof(int)) return HWR_ESIZE;
  int* out = (int*)sink;
  const int waves = 4 * waves_per_simd;
  hipStream_t st = (hipStream_t)stream;
  hipError_t e = hipSuccess;
  switch (kind) {
    case MB_MFMA_I8: e = launch_mb<MB_MFMA_I8>(out, grid, waves, iters, st); break;
    case MB_MFMA_F8: e = launch_mb<MB_MFMA_F8>(out, grid, waves, iters, st); break;
    case MB_LDS: e = launch_mb<MB_LDS>(out, grid, waves, iters, st); break;
    case MB_MFMA_I8_LDS: e = launch_mb<MB_MFMA_I8_LDS>(out, grid, waves, iters, st); break;
    case MB_MFMA_F8_LDS: e = launch_mb<MB_MFMA_F8_LDS>(out, grid, waves, iters, st); break;
    case MB_FMA: e = launch_mb<MB_FMA>(out, grid, waves, iters, st); break;
    case MB_EXP: e = launch_mb<MB_EXP>(out, grid, waves, iters, st); break;
    case MB_CVT_FP8: e = launch_mb<MB_CVT_FP8>(out, grid, waves, iters, st); break;
    default: e = launch_mb<MB_SOFTMAX_MIX>(out, grid, waves, iters, st); break;
  }
  return e == hipSuccess ? HWR_OK : HWR_ELAUNCH;
}

// Co-execution benchmark: `grid` workgroups of eight wavefronts, `iters` iterations; mfma_kind 0 (INT8) or 1 (FP8),
// valu_kind 0 fma, 1 cvt_pk_u8, 2 max3, 3 the mix with one conversion per code, 4 the mix with two per conversion; mode 1 = the MFMA wavefronts only, 2 = the vector wavefronts only,
// 3 = both.  Per iteration a wavefront issues 16 MFMAs, or 64 / 64 / 32 / 160 / 144 vector instructions.
// The attention kernel's steady-state tile period as an instruction mix (see period_kernel): `parts` is a sum of 1 (MFMAs),
// 2 (their A fragments come from LDS), 4 (the vector half), 8 (the global->LDS tile requests); supported: 1, 3, 4, 5, 7,
// 11, 15.  random_operands 0: regular low-entropy operand bits; 1: hashed bytes in the fragments and the resident Q operand
// (the scores then spread over a few binades below each tile's maximum, as attention scores do) -- the same
// instructions on bits that toggle.
// `src` is device memory of at least grid MiB that the requests read (fill it to match).  The caller times the launch
// and divides by `periods`.
int sage_period(int parts, int random_operands, int grid, int periods, void* sink, size_t sink_bytes, const void* src, size_t src_bytes,
                void* stream) {
  using namespace sage;
  if (grid <= 0 || grid > 65535 || periods <= 0 || !sink || !src) return HWR_EINVAL;
  if (sink_bytes < (size_t)grid * 1024 * sizeof(int) || src_bytes < (size_t)grid << 20) return HWR_ESIZE;
  int* out = (int*)sink;
  const uint8_t* in = (const uint8_t*)src;
  hipStream_t st = (hipStream_t)stream;
  hipError_t e;
  switch (parts) {
    case 1: e = launch_period<1>(out, in, grid, periods, random_operands != 0, st); break;
    case 3: e = launch_period<3>(out, in, grid, periods, random_operands != 0, st); break;
    case 4: e = launch_period<4>(out, in, grid, periods, random_operands != 0, st); break;
    case 5: e = launch_period<5>(out, in, grid, periods, random_operands != 0, st); break;
    case 7: e = launch_period<7>(out, in, grid, periods, random_operands != 0, st); break;
    case 11: e = launch_period<11>(out, in, grid, periods, random_operands != 0, st); break;
    case 15: e = launch_period<15>(out, in, grid, periods, random_operands != 0, st); break;
    default: return HWR_EINVAL;
  }
  return e == hipSuccess ? HWR_OK : HWR_ELAUNCH;
}

int sage_coexec(int mfma_kind, int valu_kind, int mode, int grid, int iters, void* sink, size_t sink_bytes, void* stream) {
  using namespace sage;
  if (mfma_kind < 0 || mfma_kind > 1 || valu_kind < 0 || valu_kind > 4 || mode < 1 || mode > 3) return HWR_EINVAL;
  if (grid <= 0 || grid > 65535 || iters <= 0 || !sink) return HWR_EINVAL;
  if (sink_bytes < (size_t)grid * 1024 * sizeof(int)) return HWR_ESIZE;
  int* out = (int*)sink;
  hipStream_t st = (hipStream_t)stream;
  hipError_t e;
#define SAGE_CX(M, V) launch_coexec<M, V>(out, grid, iters, mode, st)
  if (mfma_kind == 0) e = valu_kind == 0 ? SAGE_CX(0, 0) : valu_kind == 1 ? SAGE_CX(0, 1) : valu_kind == 2 ? SAGE_CX(0, 2) : valu_kind == 3 ? SAGE_CX(0, 3) : SAGE_CX(0, 4);
  else e = valu_kind == 0 ? SAGE_CX(1, 0) : valu_kind == 1 ? SAGE_CX(1, 1) : valu_kind == 2 ? SAGE_CX(1, 2) : valu_kind == 3 ? SAGE_CX(1, 3) : SAGE_CX(1, 4);
#undef SAGE_CX
  return e == hipSuccess ? HWR_OK : HWR_ELAUNCH;
}

}  // extern "C"
