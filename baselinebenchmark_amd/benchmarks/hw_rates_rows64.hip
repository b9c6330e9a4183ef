// The attention kernel's tile period for a design with 64 query rows per wavefront, as an instruction mix (see
// period64_kernel).  Its own translation unit: built with -mllvm -amdgpu-mfma-vgpr-form, so that the Q.K^T MFMAs leave
// their scores in registers the vector ALU can read, while the output accumulators are pinned to the accumulation
// registers by the constraints of an asm statement.  No counterpart in the reference: a measurement aid.
#include "../csrc/sage_common.h"
#include "hw_rates.h"

namespace sage {
namespace {

// ---------------------------------------------------------------------------------------------
// The same tile period for a design that is NOT the attention kernel's: one wavefront per SIMD (four per workgroup, up to
// 512 registers each), every wavefront 64 query rows (two 32-row blocks), so that every K / V fragment read from LDS
// feeds two MFMAs -- half the fragment reads per MFMA -- and the matrix pipe and the vector ALU overlap inside one
// instruction stream: 64-key steps, the Q.K^T MFMAs of step s + 1 issued between the probability codes of step s, the P.V
// MFMAs of step s between the row maxima of step s + 1 (two score buffers).  Per wavefront and 128 keys: 32 INT8 MFMAs on
// 16 ds_read_b128, 16 + 4 FP8 MFMAs on 16 ds_read_b128, the vector work of 128 scores per lane, eight 1 KB requests; one
// barrier per 128 keys.  Same work per compute unit and period as period_kernel (256 rows x 128 keys, head_dim 128).
// What it measures: whether halving the LDS bytes per MFMA buys time on this part, before anyone writes that kernel.
// ---------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256) period64_kernel(int* sink, const uint8_t* src, int periods, int random_operands, float s, float c) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];   // 64 KB of fragments + 32 KB that the requests fill
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  auto hashed = [](unsigned x) {
    x *= 2654435761u; x ^= x >> 15; x *= 2246822519u; x ^= x >> 13; x *= 3266489917u; x ^= x >> 16;
    return (int)(x & 0xFEFEFEFEu);
  };
  for (int i = threadIdx.x; i < 65536 / 4; i += 256)
    reinterpret_cast<int*>(smem)[i] = random_operands ? hashed(i + blockIdx.x * 16384) : i * 7 + 1;
  __syncthreads();
  const __amdgpu_buffer_rsrc_t rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)(src + (size_t)(blockIdx.x & 7) * (1u << 20)), 0, 0x7fffffff, 0x00020000);
  v4i q[2][4];
  v16i bias, sa[2][2], sb[2][2];
  v16f o[2][4];
  v8i ones, pa[2], pb[2];
  for (int rb = 0; rb < 2; rb++)
    for (int k = 0; k < 4; k++) {
      q[rb][k] = v4i{lane + k + rb, 1, 2, 3};
      if (random_operands)
        for (int e = 0; e < 4; e++) q[rb][k][e] = hashed(0x40000000u + (((blockIdx.x * 256 + threadIdx.x) * 2 + rb) * 4 + k) * 4 + e);
    }
  for (int i = 0; i < 16; i++) bias[i] = 0x4B400000;
  for (int i = 0; i < 8; i++) ones[i] = (lane == 0 || lane == 32 || lane == 20 || lane == 52) ? 0x38383838 : 0;
  for (int rb = 0; rb < 2; rb++) {
    for (int g = 0; g < 2; g++) { sa[rb][g] = bias; sb[rb][g] = bias; }
    for (int k = 0; k < 4; k++) for (int i = 0; i < 16; i++) o[rb][k][i] = 0.f;
    for (int i = 0; i < 8; i++) { pa[rb][i] = 0; pb[rb][i] = 0; }
  }
  asm volatile("" : "+v"(bias), "+v"(ones));
  float m_used[2] = {0.f, 0.f}, lsum[2] = {0.f, 0.f}, k0a[2] = {c, c}, k0b[2] = {c, c}, sc = s * 1e-4f;
  int psa[2] = {119, 119}, psb[2] = {119, 119};
  constexpr float kN8 = 8.0f * 256.0f / 65535.0f;
  // Fragments of the NEXT phase that are read during the current one, so that no phase starts by waiting for LDS (with
  // one wavefront per SIMD nothing else would run meanwhile): the first four K fragments, the first two V pairs.
  v4i kpre[4];
  v8i vpre[2];
  auto vfrag_at = [&](int half, int i) {
    const uint8_t* vbuf = smem + half * 8192 + lane * 16;
    const v4i lo = *reinterpret_cast<const v4i*>(vbuf + (2 * i) * 1024), hi = *reinterpret_cast<const v4i*>(vbuf + (2 * i + 1) * 1024);
    return v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  };
  auto kfrag_at = [&](int half, int i) { return *reinterpret_cast<const v4i*>(smem + 32768 + half * 8192 + lane * 16 + i * 1024); };
  // Q.K^T of one 64-key step into score buffer y (two key groups of 32, two row blocks): 8 fragments, 16 MFMAs
  auto qk = [&](v16i (&y)[2][2], int half, int next_v_half) {
    v4i kf[8];
#pragma unroll
    for (int i = 0; i < 4; i++) kf[i] = kpre[i];
    // (fragment i = key group i % 2, contraction step i / 2: the four accumulators take turns, so no MFMA waits for the
    // one before it)
#pragma unroll
    for (int i = 0; i < 8; i++) {
      if (i + 4 < 8) kf[i + 4] = kfrag_at(half, i + 4);
      const int g = i % 2, ks = i / 2;
      y[0][g] = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf[i], q[0][ks], ks == 0 ? bias : y[0][g], 0, 0, 0);
      y[1][g] = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf[i], q[1][ks], ks == 0 ? bias : y[1][g], 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 2; i++) vpre[i] = vfrag_at(next_v_half, i);
  };
  // probability codes of the scores in x -> the B operands p of the P.V MFMAs
  auto codes = [&](v16i (&x)[2][2], const float (&k0)[2], v8i (&p)[2]) {
#pragma unroll
    for (int rb = 0; rb < 2; rb++) {
      const float mul = kN8 * sc, cc = __builtin_fmaf(-12582912.0f, mul, k0[rb]);
#pragma unroll
      for (int g = 0; g < 2; g++) {
        float t8[16];
#pragma unroll
        for (int r = 0; r < 16; r++) t8[r] = __builtin_fmaf(__builtin_bit_cast(float, (int)x[rb][g][r]), mul, cc);
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
          const unsigned w01 = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_pknorm_u16(t8[4 * q4], t8[4 * q4 + 1]));
          const unsigned w23 = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_pknorm_u16(t8[4 * q4 + 2], t8[4 * q4 + 3]));
          p[rb][4 * g + q4] = (int)__builtin_amdgcn_perm(w23, w01, 0x07050301u);
        }
      }
    }
  };
  // P.V of one 64-key step (4 fragment pairs, 8 MFMAs + one row-sum MFMA per row block) with the row maxima of the NEXT
  // step's scores y woven in by hand: the P.V MFMAs are asm statements (that is what pins the output accumulators to the
  // accumulation registers), which the scheduler neither moves nor fills, so a slice of the maximum chains follows each.
  auto pv_and_rowmax = [&](const v8i (&p)[2], const int (&ps)[2], int half, v16i (&y)[2][2], int (&mx)[2][2], int next_k_half) {
    v8i vf[4];
    auto chunk = [&](int i) {      // registers 2i, 2i + 1 of the four (row block, key group) score tiles
#pragma unroll
      for (int rb = 0; rb < 2; rb++)
#pragma unroll
        for (int g = 0; g < 2; g++)
          mx[rb][g] = i == 0 ? max(y[rb][g][0], y[rb][g][1]) : max(max(mx[rb][g], y[rb][g][2 * i]), y[rb][g][2 * i + 1]);
      __builtin_amdgcn_sched_barrier(0);
    };
    vf[0] = vpre[0]; vf[1] = vpre[1];
    vf[2] = vfrag_at(half, 2); vf[3] = vfrag_at(half, 3);
#pragma unroll
    for (int i = 0; i < 4; i++) kpre[i] = kfrag_at(next_k_half, i);
    {
      const v4f zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int rb = 0; rb < 2; rb++) {
        const v4f os = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ones, p[rb], zero, 0, 0, 0, 0, 0, 0);
        lsum[rb] = __builtin_fmaf(os[0], __builtin_bit_cast(float, ps[rb] << 23), lsum[rb]);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int dt = 0; dt < 4; dt++) {
#pragma unroll
      for (int rb = 0; rb < 2; rb++) {
        asm volatile("v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[0,0,0]"
                     : "+a"(o[rb][dt]) : "v"(vf[dt]), "v"(p[rb]), "v"(127), "v"(ps[rb]));
        chunk(2 * dt + rb);
      }
    }
  };
  // (the rest of the row maximum -- exchange with the lane that shares the row, block exponent, constants of the codes --
  // is a dependent chain: it runs under the first Q.K^T MFMAs of the next phase, not after the last P.V one)
  auto finish_rowmax = [&](const int (&mx)[2][2], float (&k0)[2], int (&psn)[2]) {
#pragma unroll
    for (int rb = 0; rb < 2; rb++) {
      const int m2 = max(mx[rb][0], mx[rb][1]);
      float mloc = __builtin_fmaf(__builtin_bit_cast(float, m2), sc, -12582912.0f * sc);
      auto r2 = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(int, mloc), __builtin_bit_cast(int, mloc), false, false);
      const float mall = fmaxf(__builtin_bit_cast(float, (int)r2[0]), __builtin_bit_cast(float, (int)r2[1]));
      if (__builtin_amdgcn_ballot_w64(mall > m_used[rb] + 1.0e30f) != 0) m_used[rb] = mall;      // (never taken)
      const float e = fmaxf(__builtin_ceilf(mall - m_used[rb]), -110.0f);
      k0[rb] = __builtin_fmaf(-kN8, e, __builtin_fmaf(kN8, 8.75f - m_used[rb], c));
      psn[rb] = (int)(unsigned)(e + 119.0f);
    }
  };
  auto requests = [&](int p) {
    uint8_t* dst = smem + 65536 + wave * 8192;       // (the data is never read: only the traffic matters)
    const int uo = ((p * 32768) & ((1 << 20) - 1)) + wave * 8192;
#pragma unroll
    for (int i = 0; i < 8; i++)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)(dst + i * 1024), 16, lane * 16, uo + i * 1024, 0, 0);
  };
  // interleave patterns: an MFMA, then a share of the vector instructions of the phase (and the fragment reads in step)
  auto weave_a = [&]() {    // 16 MFMAs, 8 reads (4 first), ~130 vector instructions
#pragma unroll
    for (int i = 0; i < 16; i++) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 10, 0);
      if (i % 2 == 0) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // four K fragments, then the four reads of the V pairs
    }
  };
  int mxa[2][2], mxb[2][2];
  for (int i = 0; i < 4; i++) kpre[i] = kfrag_at(0, i);
  qk(sa, 0, 0);
  for (int i = 0; i < 4; i++) kpre[i] = kfrag_at(1, i);
  for (int rb = 0; rb < 2; rb++) for (int g = 0; g < 2; g++) { mxa[rb][g] = sa[rb][g][0]; mxb[rb][g] = 0; }
  for (int p = 0; p < periods; p++) {
    asm volatile("s_waitcnt vmcnt(8)" ::: "memory");     // the requests of the period before last have landed
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    // step 0: codes of buffer a between the Q.K^T MFMAs into buffer b; then P.V between the row maxima of b
    qk(sb, 1, 0); finish_rowmax(mxa, k0a, psa); codes(sa, k0a, pa); weave_a();
    __builtin_amdgcn_sched_barrier(0);
    pv_and_rowmax(pa, psa, 0, sb, mxb, 0);
    __builtin_amdgcn_sched_barrier(0);
    // step 1: the same with the buffers swapped (Q.K^T of the next period's first half)
    qk(sa, 0, 1); finish_rowmax(mxb, k0b, psb); codes(sb, k0b, pb); weave_a();
    __builtin_amdgcn_sched_barrier(0);
    pv_and_rowmax(pb, psb, 1, sa, mxa, 1);
    __builtin_amdgcn_sched_barrier(0);
    requests(p);
    sc = sc * 1.0000001f;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  int result = (int)(lsum[0] + lsum[1]) ^ psa[0] ^ psb[1];
  for (int rb = 0; rb < 2; rb++) for (int k = 0; k < 4; k++) result ^= (int)o[rb][k][0];
  result ^= sa[0][0][0] ^ sb[1][1][0];
  sink[blockIdx.x * 1024 + threadIdx.x] = result;
}

hipError_t launch_period64(int* sink, const uint8_t* src, int grid, int periods, int random_operands, hipStream_t st) {
  static bool attr_done = false;
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(period64_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 98304);
    if (e != hipSuccess) return e;
    attr_done = true;
  }
  period64_kernel<<<dim3(grid), dim3(256), 98304, st>>>(sink, src, periods, random_operands, random_operands ? 0.25f : 0.999f, 0.001f);
  return hipGetLastError();
}


}  // namespace
}  // namespace sage

extern "C" {
// The tile period of the 64-rows-per-wavefront design (see period64_kernel): same arguments as sage_period without `parts`.
int sage_period64(int random_operands, int grid, int periods, void* sink, size_t sink_bytes, const void* src, size_t src_bytes,
                  void* stream) {
  using namespace sage;
  if (grid <= 0 || grid > 65535 || periods <= 0 || !sink || !src) return HWR_EINVAL;
  if (sink_bytes < (size_t)grid * 1024 * sizeof(int) || src_bytes < (size_t)grid << 20) return HWR_ESIZE;
  return launch_period64((int*)sink, (const uint8_t*)src, grid, periods, random_operands != 0, (hipStream_t)stream) == hipSuccess ? HWR_OK : HWR_ELAUNCH;
}

}  // extern "C"
