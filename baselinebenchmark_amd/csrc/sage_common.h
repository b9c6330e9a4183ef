// Shared declarations for the gfx950 SageAttention kernels: vector types, wave-level helpers,
// dtype conversion, the V panel byte order and the variable-length plan layout.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace sage {

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef unsigned short u16;

constexpr int kWave = 64;
constexpr int kPanelRows = 128;  // == SAGE_PANEL_ROWS

// ---------------------------------------------------------------------------------------------
// V panel byte order.  A panel holds 128 consecutive KV rows n (0..127) of one (batch, kv head)
// for all D channels d, arranged so that one wavefront-wide 16-byte load per lane yields an MFMA
// operand of V^T (rows = 32 channels, contraction = KV rows) with no shuffling:
//
//  FP8 (1 byte/elt, 128*D bytes): index = (((ks*(D/32) + dt)*2 + half)*64 + lane)*16 + j
//      ks = n/64, lane = 32*h + (d%32), dt = d/32,
//      n%64 = 32*half + 8*(j/4) + 4*h + (j%4)          (j = 0..15, h = 0..1, half = 0..1)
//    -> operand of v_mfma_f32_32x32x64_f8f6f4: lane (d%32, h) holds 32 bytes (half 0 then 1).
//  FP16 (2 bytes/elt, 256*D bytes): index(elements) = ((ks*(D/32) + dt)*64 + lane)*8 + j
//      ks = n/16, lane = 32*h + (d%32), n%16 = 8*(j/4) + 4*h + (j%4)      (j = 0..7)
//    -> operand of v_mfma_f32_32x32x16_f16.
//
// The row order inside a lane's bytes equals the order in which a lane of the S^T = K.Q^T
// accumulator (v_mfma_i32_32x32x32_i8: register r of lane (m, h) is KV row 8*(r/4)+4*h+(r%4))
// holds the probabilities of query row m, so P never leaves registers between the two MFMAs.
// ---------------------------------------------------------------------------------------------
__host__ __device__ inline int panel_index_fp8(int n, int d, int D) {
  int ks = n >> 6, nn = n & 63;
  int half = nn >> 5, r = nn & 31;
  int a = r >> 3, h = (r >> 2) & 1, b = r & 3;
  int lane = 32 * h + (d & 31), dt = d >> 5;
  return (((ks * (D / 32) + dt) * 2 + half) * 64 + lane) * 16 + 4 * a + b;
}
__host__ __device__ inline int panel_index_fp16(int n, int d, int D) {
  int ks = n >> 4, r = n & 15;
  int a = r >> 3, h = (r >> 2) & 1, b = r & 3;
  int lane = 32 * h + (d & 31), dt = d >> 5;
  return ((ks * (D / 32) + dt) * 64 + lane) * 8 + 4 * a + b;
}

// ---------------------------------------------------------------------------------------------
// Variable-length plan: int32 arrays packed in one device buffer, offsets in ints.
// ---------------------------------------------------------------------------------------------
struct SagePlanLayout {
  int64_t cu_qblk, cu_kblk, cu_panel, ntiles, tiles, total;
};
__host__ __device__ inline SagePlanLayout plan_layout(int nseq, int total_q) {
  SagePlanLayout L;
  L.cu_qblk = 0;
  L.cu_kblk = L.cu_qblk + nseq + 1;
  L.cu_panel = L.cu_kblk + nseq + 1;
  L.ntiles = L.cu_panel + nseq + 1;
  L.tiles = L.ntiles + 1;
  // an attention q-tile never has fewer than 128 rows, so at most total_q/128 + nseq tiles exist
  L.total = L.tiles + (int64_t)total_q / 128 + nseq + 1;
  return L;
}

// ---------------------------------------------------------------------------------------------
// dtype helpers (bf16 handled as raw bits: widening is a shift, narrowing is RNE).
// ---------------------------------------------------------------------------------------------
__device__ inline float bf16_to_f32(u16 v) { return __builtin_bit_cast(float, (uint32_t)v << 16); }
// narrowing: gfx950 has a hardware round-to-nearest-even conversion (v_cvt_pk_bf16_f32)
__device__ inline u16 f32_to_bf16(float f) { return __builtin_bit_cast(u16, (__bf16)f); }
__device__ inline float f16_to_f32(u16 v) { return (float)__builtin_bit_cast(_Float16, v); }
__device__ inline u16 f32_to_f16(float f) { return __builtin_bit_cast(u16, (_Float16)f); }

template <int DT>
__device__ inline float to_f32(u16 v) {
  if constexpr (DT == 1) return bf16_to_f32(v);
  else return f16_to_f32(v);
}
template <int DT>
__device__ inline u16 from_f32(float f) {
  if constexpr (DT == 1) return f32_to_bf16(f);
  else return f32_to_f16(f);
}

// ---------------------------------------------------------------------------------------------
// Streaming accesses of the pre-pass kernels: every byte of an operand is touched once per pass and not again before
// hundreds of megabytes have gone by, so the accesses are marked non-temporal (no cache line is kept for them).  On
// this part a read-only pass over 0.5 GB measures 6.9-7.1 TB/s with such loads against 6.0-6.2 TB/s with plain ones.
// ---------------------------------------------------------------------------------------------
typedef unsigned int v4u __attribute__((ext_vector_type(4)));
__device__ inline uint4 load_stream16(const void* p) {
  const v4u v = __builtin_nontemporal_load(reinterpret_cast<const v4u*>(p));
  return make_uint4(v[0], v[1], v[2], v[3]);
}
__device__ inline void store_stream16(void* p, uint4 v) {
  const v4u t = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(t, reinterpret_cast<v4u*>(p));
}

// ---------------------------------------------------------------------------------------------
// Wavefront (64-lane) reductions with DPP inside rows of 16 lanes, then lane reads across rows.
// The result is uniform across the wavefront.
// ---------------------------------------------------------------------------------------------
template <int CTRL>
__device__ inline float dpp_f(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, x), __builtin_bit_cast(int, x),
                                                              CTRL, 0xf, 0xf, false));
}
// Maximum over the 16 lanes of a DPP row (lanes 16r .. 16r+15), in every lane of the row.
__device__ inline float row16_max(float x) {
  x = fmaxf(x, dpp_f<0xB1>(x));   // quad_perm [1,0,3,2]
  x = fmaxf(x, dpp_f<0x4E>(x));   // quad_perm [2,3,0,1]
  x = fmaxf(x, dpp_f<0x141>(x));  // row_half_mirror
  x = fmaxf(x, dpp_f<0x140>(x));  // row_mirror
  return x;
}
__device__ inline float wave_max(float x) {
  x = row16_max(x);
  float a = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 0));
  float b = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 16));
  float c = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 32));
  float d = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 48));
  return fmaxf(fmaxf(a, b), fmaxf(c, d));
}

// ---------------------------------------------------------------------------------------------
// Arithmetic shared by every place that produces INT8 operands (the standalone quantiser and the
// attention prologue that quantises its own Q tile): they must agree bit for bit.
// ---------------------------------------------------------------------------------------------
constexpr float kScaleFloor = 1.0e-12f;


// Correctly rounded x / s for a wavefront-uniform divisor whose reciprocal r = RN(1/s) is given.
// q0 = RN(x*r) is within 1 ulp of x/s; e = x - q0*s is exact in one FMA; RN(q0 + e*r) is then
// the correctly rounded quotient (Markstein's correction step), provided s's significand is not
// all ones and nothing under/overflows; the caller falls back to a true division otherwise.
__device__ inline float div_by_uniform(float x, float s, float r) {
  float q0 = x * r;
  float e = __builtin_fmaf(-q0, s, x);
  return __builtin_fmaf(e, r, q0);
}


}  // namespace sage
