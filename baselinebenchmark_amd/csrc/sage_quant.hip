// Quantisers of the SageAttention forward path for gfx950 (MI355X):
//   * per-block INT8 quantiser for Q and K (optional K-mean subtraction in the input dtype),
//   * per-(batch, head, channel) column statistics over the sequence (K mean, V abs-max),
//   * V preparation into MFMA-ready panels (fp16, or fp8-e4m3fn with per-channel scales).
// All of them are streaming kernels bound by HBM bandwidth: 128-bit loads of 8 elements per
// lane, statistics reduced with DPP inside the wavefront and through LDS across wavefronts.
//
// Arithmetic contract of the INT8 quantiser (bit-exact target): IEEE binary32 throughout,
//   backends/_enflame/ops/sage_attention/quant_per_block.py:38-46  (+ :53-54 for k - km)
//   backends/_hygon/ops/sageattention/sageattention_triton.py:35   (1e-12 floor)
#include "sage_launch.h"

#pragma clang fp contract(off)

namespace sage {

// One workgroup (256 lanes) quantises one [blk, D] tile held entirely in registers:
// pass 1 converts and reduces |x| to the tile maximum, pass 2 divides and rounds.
// A lane owns 16 consecutive channels of a row (two 128-bit loads, one 128-bit store).
// (km_lds: the K mean of this (batch, head) in LDS, D values in the input dtype, instead of a.km in global memory:
// the fused pre-pass of short sequences computes it in the same workgroup.)
// UNIT: the multiplier is 1 (every K call; x * 1.0f is x, so leaving the product out changes no bit).
template <int DT, int D, bool UNIT = false>
__device__ __forceinline__ void quant_int8_tile(const QuantArgs& a, const int blkid, const int h, const int b, const u16* km_lds) {
  constexpr int TPR = D / 16;       // lanes per row
  constexpr int RPP = 256 / TPR;    // rows per pass
  constexpr int MAXP = 128 / RPP;   // passes for the largest tile (128 rows)
  const int tid = threadIdx.x;
  const int tr = tid / TPR, tc = tid % TPR;

  int L = a.L;
  int64_t xbase, obase, sidx, dbase;
  if (a.cu_seqlens) {
    int s0 = a.cu_seqlens[b];
    L = a.cu_seqlens[b + 1] - s0;
    dbase = (int64_t)h * a.dot_total + s0;
    xbase = (int64_t)s0 * a.x_sn + (int64_t)h * a.x_sh;
    obase = (int64_t)s0 * a.o_sn + (int64_t)h * a.o_sh;
    sidx = (int64_t)h * a.scale_sh + a.cu_blocks[b] + blkid;
  } else {
    xbase = (int64_t)b * a.x_sb + (int64_t)h * a.x_sh;
    obase = (int64_t)b * a.o_sb + (int64_t)h * a.o_sh;
    sidx = (((int64_t)b * a.H + h) * ((L + a.blk - 1) / a.blk) + blkid) * a.groups;
    dbase = ((int64_t)b * a.H + h) * L;
  }
  const int n0 = blkid * a.blk;
  if (n0 >= L) return;
  const int rows = min(a.blk, L - n0);

  float kmv[16];
  const bool has_km = a.km != nullptr || km_lds != nullptr;
  if (km_lds) {
#pragma unroll
    for (int i = 0; i < 16; i++) kmv[i] = to_f32<DT>(km_lds[tc * 16 + i]);
  } else if (has_km) {
    const uint4* kp = reinterpret_cast<const uint4*>(a.km + (int64_t)b * a.km_sb + (int64_t)h * a.km_sh + tc * 16);
    uint4 raw2[2] = {kp[0], kp[1]};
    const u16* p = reinterpret_cast<const u16*>(raw2);
#pragma unroll
    for (int i = 0; i < 16; i++) kmv[i] = to_f32<DT>(p[i]);
  }
  // k - km is rounded to the input dtype (quant_per_block.py:53-54: the subtraction happens in torch, in
  // the tensor's dtype) once, while loading; both passes then see the rounded difference.
  auto smoothed = [&](u16 bits, int i) { return has_km ? from_f32<DT>(to_f32<DT>(bits) - kmv[i]) : bits; };
  auto value = [&](u16 bits) { return UNIT ? to_f32<DT>(bits) : to_f32<DT>(bits) * a.mult; };   // the fp32 value that is quantised

  // Optional side output: the dot product of every (scaled) row with a per-(batch, kv-head) vector.
  // The one-call pipeline uses it with the K mean to return the LSE of the unsmoothed logits.
  const bool has_dot = a.dot_out != nullptr;
  float dvv[16];
  if (has_dot) {
    const uint4* dp = reinterpret_cast<const uint4*>(a.dotv + (int64_t)b * a.dv_sb + (int64_t)(h / a.dv_group) * a.dv_sh + tc * 16);
    uint4 raw2[2] = {dp[0], dp[1]};
    const u16* p = reinterpret_cast<const u16*>(raw2);
#pragma unroll
    for (int i = 0; i < 16; i++) dvv[i] = to_f32<DT>(p[i]);
  }

  uint4 raw[MAXP][2];
  float amax = 0.f;
#pragma unroll
  for (int p = 0; p < MAXP; p++) {
    int r = p * RPP + tr;
    raw[p][0] = raw[p][1] = make_uint4(0, 0, 0, 0);
    float dsum = 0.f;
    if (r < rows) {
      const u16* src = a.x + xbase + (int64_t)(n0 + r) * a.x_sn + tc * 16;
      raw[p][0] = load_stream16(src);
      raw[p][1] = load_stream16(src + 8);
      if (has_km) {
        const u16* e = reinterpret_cast<const u16*>(raw[p]);
        uint32_t d[8];
#pragma unroll
        for (int i = 0; i < 8; i++) d[i] = (uint32_t)smoothed(e[2 * i], 2 * i) | ((uint32_t)smoothed(e[2 * i + 1], 2 * i + 1) << 16);
        raw[p][0] = make_uint4(d[0], d[1], d[2], d[3]);
        raw[p][1] = make_uint4(d[4], d[5], d[6], d[7]);
      }
      const u16* e = reinterpret_cast<const u16*>(raw[p]);
#pragma unroll
      for (int i = 0; i < 16; i++) amax = fmaxf(amax, fabsf(value(e[i])));
      if (has_dot) {
#pragma unroll
        for (int i = 0; i < 16; i++) dsum = __builtin_fmaf(value(e[i]), dvv[i], dsum);
      }
    }
    if (has_dot) {   // uniform branch; the TPR lanes of a row are neighbours inside one wavefront
#pragma unroll
      for (int o = 1; o < TPR; o <<= 1) dsum += __shfl_xor(dsum, o);
      if (r < rows && tc == 0) a.dot_out[dbase + n0 + r] = dsum;
    }
  }
  __shared__ float wmax[4];
  __shared__ int gmax[8];
  if (a.groups == 1) {
    amax = wave_max(amax);
    if ((tid & 63) == 0) wmax[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(wmax[0], wmax[1]), fmaxf(wmax[2], wmax[3]));
  } else {
    // Interleaved scales per block (eight: group = row % 8; four: group = (row % 8) / 2): every row this lane holds has
    // the same index modulo 8 (the passes are RPP rows apart, a multiple of 8), so the lane belongs to one group.
    // Maximum over the lanes of a row, then over the rows of the group through LDS (the values are non-negative
    // floats: their bit patterns order like integers).
    static_assert(RPP % 8 == 0, "a lane's rows must share their index modulo 8");
    if (tid < 8) gmax[tid] = 0;
    __syncthreads();
#pragma unroll
    for (int o = 1; o < TPR; o <<= 1) amax = fmaxf(amax, __shfl_xor(amax, o));
    const int gid = a.groups == 8 ? (tr & 7) : ((tr & 7) >> 1);
    if (tc == 0) atomicMax(&gmax[gid], __builtin_bit_cast(int, amax));
    __syncthreads();
    amax = __builtin_bit_cast(float, gmax[gid]);
  }
  const float scale = fmaxf(amax / 127.0f, kScaleFloor);
  if (a.groups == 1) { if (tid == 0) a.scale[sidx] = scale; }
  else if (tc == 0 && tr < a.groups) a.scale[sidx + tr] = fmaxf(__builtin_bit_cast(float, gmax[tr]) / 127.0f, kScaleFloor);   // group tr's scale

  const float rcp = 1.0f / scale;
  // The fast correction-step division needs: significand of scale not all ones, and scale and rcp
  // comfortably normal.  |quotient| <= 127.5, scale >= 1e-12.
  const uint32_t sbits = __builtin_bit_cast(uint32_t, scale);
  const bool fast = ((sbits & 0x7fffffu) != 0x7fffffu) && scale < 1.0e30f;

  // One wavefront-uniform branch around the whole second pass, not one per element (the scale is uniform over the tile,
  // or, with interleaved scales, over a lane group: if any lane of the wavefront needs the true division, all take it --
  // where the correction step applies, the two quotients are the same numbers).
  auto quantise_rows = [&](auto quotient) __attribute__((always_inline)) {
#pragma unroll
    for (int p = 0; p < MAXP; p++) {
      int r = p * RPP + tr;
      if (r < rows) {
        const u16* e = reinterpret_cast<const u16*>(raw[p]);
        uint32_t packed[4] = {0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < 16; i++) {
          // For |x| so small that the residual of the correction step is subnormal the quotient is
          // below 1e-13 in magnitude (scale >= 1e-12): whatever its last bits, it rounds to 0.
          float z = quotient(value(e[i]));
          z = z + __builtin_copysignf(0.5f, z);   // +0.5 for z >= 0 (incl. -0: -0.5 + -0 = -0.5 -> 0), else -0.5
          int q = (int)z;  // truncation toward zero
          packed[i >> 2] |= (uint32_t)(q & 0xff) << (8 * (i & 3));
        }
        store_stream16(a.out + obase + (int64_t)(n0 + r) * a.o_sn + tc * 16, make_uint4(packed[0], packed[1], packed[2], packed[3]));
      }
    }
  };
  if (__builtin_amdgcn_ballot_w64(!fast) == 0) quantise_rows([&](float x) { return div_by_uniform(x, scale, rcp); });
  else quantise_rows([&](float x) { return x / scale; });
}

template <int DT, int D>
__global__ void __launch_bounds__(256) quant_int8_kernel(QuantArgs a) {
  if (a.mult == 1.0f) quant_int8_tile<DT, D, true>(a, blockIdx.x, blockIdx.y, blockIdx.z, nullptr);
  else quant_int8_tile<DT, D, false>(a, blockIdx.x, blockIdx.y, blockIdx.z, nullptr);
}

// ---------------------------------------------------------------------------------------------
// Column statistics over the sequence: MODE 0 = float64 sum (K mean), MODE 1 = fp32 abs-max (V).
// Stage 1: one workgroup per (chunk of kChunkRows rows, head, batch) writes D partials.
// Stage 2: one workgroup per (head, batch) combines the partials in chunk order.
// ---------------------------------------------------------------------------------------------
constexpr int kChunkRows = 512;


template <int DT, int D, int MODE>
__global__ void __launch_bounds__(256) colstat_partial_kernel(ColStatArgs a) {
  using acc_t = typename std::conditional<MODE == 0, double, float>::type;
  constexpr int TPR = D / 8, RPP = 256 / TPR;
  const int chunk = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int tid = threadIdx.x, tr = tid / TPR, tc = tid % TPR;
  int L = a.L;
  int64_t xbase;
  if (a.cu_seqlens) {
    int s0 = a.cu_seqlens[b];
    L = a.cu_seqlens[b + 1] - s0;
    xbase = (int64_t)s0 * a.x_sn + (int64_t)h * a.x_sh;
  } else {
    xbase = (int64_t)b * a.x_sb + (int64_t)h * a.x_sh;
  }
  const int n0 = chunk * kChunkRows;
  if (n0 >= L) return;
  const int n1 = min(L, n0 + kChunkRows);
  acc_t acc[8];
#pragma unroll
  for (int i = 0; i < 8; i++) acc[i] = 0;
  auto fold = [&](const uint4& raw) {
    const u16* e = reinterpret_cast<const u16*>(&raw);
#pragma unroll
    for (int i = 0; i < 8; i++) {
      float x = to_f32<DT>(e[i]);
      if constexpr (MODE == 0) acc[i] += (double)x;
      else acc[i] = fmaxf(acc[i], fabsf(x));
    }
  };
  // Eight independent 16-byte loads per lane in flight (the pass is a pure read: what limits it is the bytes on their
  // way, not the arithmetic); the float64 sum of fp16/bf16 values is exact, so the order of the additions is free.
  constexpr int UNR = 8;
  const u16* base = a.x + xbase + tc * 8;
  int n = n0 + tr;
  for (; n + (UNR - 1) * RPP < n1; n += UNR * RPP) {
    uint4 raw[UNR];
#pragma unroll
    for (int u = 0; u < UNR; u++) raw[u] = load_stream16(base + (int64_t)(n + u * RPP) * a.x_sn);
#pragma unroll
    for (int u = 0; u < UNR; u++) fold(raw[u]);
  }
  for (; n < n1; n += RPP) fold(load_stream16(base + (int64_t)n * a.x_sn));
  __shared__ acc_t red[RPP][D];
#pragma unroll
  for (int i = 0; i < 8; i++) red[tr][tc * 8 + i] = acc[i];
  __syncthreads();
  if (tid < D) {
    acc_t t = red[0][tid];
    for (int r = 1; r < RPP; r++) {
      if constexpr (MODE == 0) t += red[r][tid];
      else t = fmaxf(t, red[r][tid]);
    }
    reinterpret_cast<acc_t*>(a.partial)[(((int64_t)b * a.H + h) * a.nchunk + chunk) * D + tid] = t;
  }
}

// K mean: sum partials in chunk order (float64), /L, -> fp32 -> input dtype.
template <int DT>
__global__ void kmean_finalize_kernel(const double* partial, u16* km, int H, int L, int D, int nchunk,
                                      const int32_t* cu_seqlens) {
  const int h = blockIdx.x, b = blockIdx.y, d = threadIdx.x;
  if (cu_seqlens) L = cu_seqlens[b + 1] - cu_seqlens[b];
  if (d >= D) return;
  int nc = (L + kChunkRows - 1) / kChunkRows;
  // eight partials in flight at a time (the loads are what this kernel waits for); still added in chunk order
  const double* p = partial + (((int64_t)b * H + h) * nchunk) * D + d;
  double s = 0;
  int c = 0;
  for (; c + 8 <= nc; c += 8) {
    double t[8];
#pragma unroll
    for (int i = 0; i < 8; i++) t[i] = p[(int64_t)(c + i) * D];
#pragma unroll
    for (int i = 0; i < 8; i++) s += t[i];
  }
  for (; c < nc; c++) s += p[(int64_t)c * D];
  float m = L > 0 ? (float)(s / (double)L) : 0.f;
  km[((int64_t)b * H + h) * D + d] = from_f32<DT>(m);
}

// V scale: max of partial abs-maxima, scale = max(amax/448, 1e-12).
__global__ void vscale_finalize_kernel(const float* partial, float* vscale, int H, int L, int D, int nchunk,
                                       const int32_t* cu_seqlens) {
  const int h = blockIdx.x, b = blockIdx.y, d = threadIdx.x;
  if (cu_seqlens) L = cu_seqlens[b + 1] - cu_seqlens[b];
  if (d >= D) return;
  int nc = (L + kChunkRows - 1) / kChunkRows;
  const float* p = partial + (((int64_t)b * H + h) * nchunk) * D + d;
  float m = 0.f;
  int c = 0;
  for (; c + 8 <= nc; c += 8) {
    float t[8];
#pragma unroll
    for (int i = 0; i < 8; i++) t[i] = p[(int64_t)(c + i) * D];
#pragma unroll
    for (int i = 0; i < 8; i++) m = fmaxf(m, t[i]);
  }
  for (; c < nc; c++) m = fmaxf(m, p[(int64_t)c * D]);
  vscale[((int64_t)b * H + h) * D + d] = fmaxf(m / 448.0f, kScaleFloor);
}

// ---------------------------------------------------------------------------------------------
// V preparation: one workgroup per panel (128 rows x D of one (batch, head)).
// Elements are converted, scattered into LDS in panel byte order and streamed out linearly.
// ---------------------------------------------------------------------------------------------

// (vs_lds: the per-channel V scales of this (batch, head) in LDS instead of a.vscale in global memory.)
template <int DT, int D, int PV>
__device__ __forceinline__ void prep_v_tile(const PrepVArgs& a, const int pidx, const int h, const int b, const float* vs_lds) {
  // A lane converts 4 consecutive rows x 8 consecutive channels at a time, so that the 4 row values of
  // a channel pack into one dword (fp8) or two (fp16): exactly the (b = 0..3) group of the panel
  // order.  They are staged in LDS as T[channel][row quad] and read back in panel order.
  constexpr int TPR = D / 8, RPP = 256 / TPR;   // lanes per row, row quads handled per pass
  constexpr int NQ = kPanelRows / 4;            // 32 row quads per panel
  constexpr int QPT = NQ / RPP;                 // passes
  constexpr int ESZ = (PV == 1) ? 1 : 2;
  constexpr int QW = ESZ;                       // dwords per (channel, row quad)
  constexpr int TS = NQ * QW + 1;               // dword stride of a channel in LDS (padded)
  constexpr int PANEL_BYTES = kPanelRows * D * ESZ;
  constexpr int DTN = D / 32;
  __shared__ uint32_t T[D * TS];
  const int tid = threadIdx.x, tr = tid / TPR, tc = tid % TPR;
  int L = a.L;
  int64_t vbase, pbase;
  if (a.cu_seqlens) {
    int s0 = a.cu_seqlens[b];
    L = a.cu_seqlens[b + 1] - s0;
    vbase = (int64_t)s0 * a.v_sn + (int64_t)h * a.v_sh;
    pbase = ((int64_t)h * a.panel_sh + a.cu_panels[b] + pidx) * PANEL_BYTES;
  } else {
    vbase = (int64_t)b * a.v_sb + (int64_t)h * a.v_sh;
    pbase = (((int64_t)b * a.H + h) * ((L + kPanelRows - 1) / kPanelRows) + pidx) * PANEL_BYTES;
  }
  const int n0 = pidx * kPanelRows;
  if (n0 >= L) return;
  float sc[8], rc[8];
  bool fast = true;
  if constexpr (PV == 1) {
#pragma unroll
    for (int i = 0; i < 8; i++) {
      sc[i] = vs_lds ? vs_lds[tc * 8 + i] : a.vscale[((int64_t)b * a.H + h) * D + tc * 8 + i];
      rc[i] = 1.0f / sc[i];
      fast = fast && ((__builtin_bit_cast(uint32_t, sc[i]) & 0x7fffffu) != 0x7fffffu) && sc[i] < 1.0e30f;
    }
    fast = __builtin_amdgcn_ballot_w64(!fast) == 0;   // the correction-step division for the whole wavefront, or not at all
  }
#pragma unroll
  for (int qq = 0; qq < QPT; qq++) {
    const int quad = qq * RPP + tr;
    uint4 raw[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int r = n0 + 4 * quad + j;
      raw[j] = make_uint4(0, 0, 0, 0);
      if (r < L) raw[j] = load_stream16(a.v + vbase + (int64_t)r * a.v_sn + tc * 8);
    }
#pragma unroll
    for (int i = 0; i < 8; i++) {
      float x[4];
#pragma unroll
      for (int j = 0; j < 4; j++) x[j] = to_f32<DT>(reinterpret_cast<const u16*>(&raw[j])[i]);
      uint32_t* dst = &T[(tc * 8 + i) * TS + quad * QW];
      if constexpr (PV == 1) {
        float z[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
          z[j] = fast ? div_by_uniform(x[j], sc[i], rc[i]) : x[j] / sc[i];
          z[j] = fminf(fmaxf(z[j], -448.f), 448.f);
        }
        int pk = __builtin_amdgcn_cvt_pk_fp8_f32(z[0], z[1], 0, false);
        pk = __builtin_amdgcn_cvt_pk_fp8_f32(z[2], z[3], pk, true);
        dst[0] = (uint32_t)pk;
      } else {
        dst[0] = (uint32_t)f32_to_f16(x[0]) | ((uint32_t)f32_to_f16(x[1]) << 16);
        dst[1] = (uint32_t)f32_to_f16(x[2]) | ((uint32_t)f32_to_f16(x[3]) << 16);
      }
    }
  }
  __syncthreads();
  uint4* out = reinterpret_cast<uint4*>(a.panels + pbase);
#pragma unroll
  for (int i = 0; i < PANEL_BYTES / 16 / 256; i++) {
    const int c = i * 256 + tid;           // 16-byte chunk of the panel
    const int lane = c & 63, hh = lane >> 5, d_lo = lane & 31;
    uint4 v;
    if constexpr (PV == 1) {
      // c = ((ks*DTN + dt)*2 + half)*64 + lane ; bytes 4a+b <-> row 64ks + 32half + 8a + 4h + b
      const int half = (c >> 6) & 1, dt = (c >> 7) % DTN, ks = (c >> 7) / DTN;
      const uint32_t* src = &T[(32 * dt + d_lo) * TS + 16 * ks + 8 * half + hh];
      v = make_uint4(src[0], src[2], src[4], src[6]);
    } else {
      // c = (ks16*DTN + dt)*64 + lane ; elements 4a+b <-> row 16ks16 + 8a + 4h + b
      const int dt = (c >> 6) % DTN, ks16 = (c >> 6) / DTN;
      const uint32_t* src = &T[(32 * dt + d_lo) * TS + (4 * ks16 + hh) * 2];
      v = make_uint4(src[0], src[1], src[4], src[5]);
    }
    store_stream16(out + c, v);
  }
}

template <int DT, int D, int PV>
__global__ void __launch_bounds__(256) prep_v_kernel(PrepVArgs a) {
  prep_v_tile<DT, D, PV>(a, blockIdx.x, blockIdx.y, blockIdx.z, nullptr);
}

// ---------------------------------------------------------------------------------------------
// Short sequences: every pre-pass of the one-call pipeline in ONE launch.  A workgroup is either a K tile or a V panel
// of one (batch, kv-head); it first computes the statistic its tile needs over the whole sequence itself (the K mean:
// float64 sums in the order of the two-stage kernels above -- per 512-row chunk, per-lane rows, the lanes of a channel
// in order, chunks in order -- so that the mean is the same bit pattern; the V scale: an abs-max, which has no order)
// and then runs the tile code of the kernels above.  The statistics are read again by every workgroup of the
// (batch, head): affordable while the sequence is short and the reads hit the L2; six dependent launches of a few
// microseconds each become one.
// ---------------------------------------------------------------------------------------------
template <int DT, int D, int PV>
__global__ void __launch_bounds__(256) prepass_small_kernel(QuantArgs qa, PrepVArgs va, int nk, int smooth, u16* km_out,
                                                            float* vscale_out) {
  constexpr int TPR = D / 8, RPP = 256 / TPR;
  const int h = blockIdx.y, b = blockIdx.z;
  const int tid = threadIdx.x, tr = tid / TPR, tc = tid % TPR;
  __shared__ double red[RPP][D];
  __shared__ u16 km_l[D];
  __shared__ float vs_l[D];
  if ((int)blockIdx.x < nk) {
    if (smooth) {
      const int L = qa.L;
      const int64_t xbase = (int64_t)b * qa.x_sb + (int64_t)h * qa.x_sh;
      double s = 0;
      for (int n0 = 0; n0 < L; n0 += kChunkRows) {
        const int n1 = min(L, n0 + kChunkRows);
        double acc[8];
#pragma unroll
        for (int i = 0; i < 8; i++) acc[i] = 0;
#pragma unroll 8
        for (int n = n0 + tr; n < n1; n += RPP) {   // (unrolled for loads in flight; the additions keep their order)
          uint4 raw = *reinterpret_cast<const uint4*>(qa.x + xbase + (int64_t)n * qa.x_sn + tc * 8);
          const u16* e = reinterpret_cast<const u16*>(&raw);
#pragma unroll
          for (int i = 0; i < 8; i++) acc[i] += (double)to_f32<DT>(e[i]);
        }
#pragma unroll
        for (int i = 0; i < 8; i++) red[tr][tc * 8 + i] = acc[i];
        __syncthreads();
        if (tid < D) {
          double t = red[0][tid];
          for (int r = 1; r < RPP; r++) t += red[r][tid];
          s += t;
        }
        __syncthreads();
      }
      if (tid < D) {
        const u16 m = from_f32<DT>(L > 0 ? (float)(s / (double)L) : 0.f);
        km_l[tid] = m;
        if (blockIdx.x == 0) km_out[((int64_t)b * qa.H + h) * D + tid] = m;
      }
      __syncthreads();
    }
    quant_int8_tile<DT, D, true>(qa, blockIdx.x, h, b, smooth ? km_l : nullptr);   // (K: the multiplier is 1)
  } else {
    const int pidx = blockIdx.x - nk;
    if constexpr (PV == 1) {
      const int L = va.L;
      const int64_t vbase = (int64_t)b * va.v_sb + (int64_t)h * va.v_sh;
      float acc[8];
#pragma unroll
      for (int i = 0; i < 8; i++) acc[i] = 0.f;
#pragma unroll 8
      for (int n = tr; n < L; n += RPP) {
        uint4 raw = *reinterpret_cast<const uint4*>(va.v + vbase + (int64_t)n * va.v_sn + tc * 8);
        const u16* e = reinterpret_cast<const u16*>(&raw);
#pragma unroll
        for (int i = 0; i < 8; i++) acc[i] = fmaxf(acc[i], fabsf(to_f32<DT>(e[i])));
      }
      float* redf = reinterpret_cast<float*>(&red[0][0]);
#pragma unroll
      for (int i = 0; i < 8; i++) redf[tr * D + tc * 8 + i] = acc[i];
      __syncthreads();
      if (tid < D) {
        float t = redf[tid];
        for (int r = 1; r < RPP; r++) t = fmaxf(t, redf[r * D + tid]);
        const float sc = fmaxf(t / 448.0f, kScaleFloor);
        vs_l[tid] = sc;
        if (pidx == 0) vscale_out[((int64_t)b * va.H + h) * D + tid] = sc;
      }
      __syncthreads();
    }
    prep_v_tile<DT, D, PV>(va, pidx, h, b, PV == 1 ? vs_l : nullptr);
  }
}

// ---------------------------------------------------------------------------------------------
// Host-side launchers (called from the C ABI in sage_api.hip).
// ---------------------------------------------------------------------------------------------
hipError_t launch_quant_int8(const QuantArgs& a, int dtype, int max_blocks, hipStream_t st) {
  dim3 grid(max_blocks, a.H, a.B), block(256);
  if (dtype == 0 && a.D == 64) quant_int8_kernel<0, 64><<<grid, block, 0, st>>>(a);
  else if (dtype == 0 && a.D == 128) quant_int8_kernel<0, 128><<<grid, block, 0, st>>>(a);
  else if (dtype == 1 && a.D == 64) quant_int8_kernel<1, 64><<<grid, block, 0, st>>>(a);
  else quant_int8_kernel<1, 128><<<grid, block, 0, st>>>(a);
  return hipGetLastError();
}

int colstat_chunks(int L) { return (L + kChunkRows - 1) / kChunkRows; }

template <int MODE>
static hipError_t launch_colstat(const ColStatArgs& a, int dtype, hipStream_t st) {
  dim3 grid(a.nchunk, a.H, a.B), block(256);
  if (dtype == 0 && a.D == 64) colstat_partial_kernel<0, 64, MODE><<<grid, block, 0, st>>>(a);
  else if (dtype == 0 && a.D == 128) colstat_partial_kernel<0, 128, MODE><<<grid, block, 0, st>>>(a);
  else if (dtype == 1 && a.D == 64) colstat_partial_kernel<1, 64, MODE><<<grid, block, 0, st>>>(a);
  else colstat_partial_kernel<1, 128, MODE><<<grid, block, 0, st>>>(a);
  return hipGetLastError();
}

hipError_t launch_k_mean(const ColStatArgs& a, int dtype, void* km, hipStream_t st) {
  if (a.nchunk == 0 || a.B == 0 || a.H == 0) return hipSuccess;
  hipError_t e = launch_colstat<0>(a, dtype, st);
  if (e != hipSuccess) return e;
  dim3 grid(a.H, a.B), block(a.D);
  if (dtype == 0) kmean_finalize_kernel<0><<<grid, block, 0, st>>>((const double*)a.partial, (u16*)km, a.H, a.L, a.D, a.nchunk, a.cu_seqlens);
  else kmean_finalize_kernel<1><<<grid, block, 0, st>>>((const double*)a.partial, (u16*)km, a.H, a.L, a.D, a.nchunk, a.cu_seqlens);
  return hipGetLastError();
}

hipError_t launch_v_scale(const ColStatArgs& a, int dtype, float* vscale, hipStream_t st) {
  if (a.nchunk == 0 || a.B == 0 || a.H == 0) return hipSuccess;
  hipError_t e = launch_colstat<1>(a, dtype, st);
  if (e != hipSuccess) return e;
  dim3 grid(a.H, a.B), block(a.D);
  vscale_finalize_kernel<<<grid, block, 0, st>>>((const float*)a.partial, vscale, a.H, a.L, a.D, a.nchunk, a.cu_seqlens);
  return hipGetLastError();
}

hipError_t launch_prepass_small(const QuantArgs& qa, const PrepVArgs& va, int dtype, int pv, int nk, int nv, int smooth,
                                void* km_out, float* vscale_out, hipStream_t st) {
  if (nk + nv == 0 || qa.B == 0 || qa.H == 0) return hipSuccess;
  dim3 grid(nk + nv, qa.H, qa.B), block(256);
#define SAGE_PREPASS(DT, DD, PVV) prepass_small_kernel<DT, DD, PVV><<<grid, block, 0, st>>>(qa, va, nk, smooth, (u16*)km_out, vscale_out)
  if (dtype == 0) {
    if (qa.D == 64) { if (pv) SAGE_PREPASS(0, 64, 1); else SAGE_PREPASS(0, 64, 0); }
    else { if (pv) SAGE_PREPASS(0, 128, 1); else SAGE_PREPASS(0, 128, 0); }
  } else {
    if (qa.D == 64) { if (pv) SAGE_PREPASS(1, 64, 1); else SAGE_PREPASS(1, 64, 0); }
    else { if (pv) SAGE_PREPASS(1, 128, 1); else SAGE_PREPASS(1, 128, 0); }
  }
#undef SAGE_PREPASS
  return hipGetLastError();
}

hipError_t launch_prep_v(const PrepVArgs& a, int dtype, int pv, int max_panels, hipStream_t st) {
  if (max_panels == 0 || a.B == 0 || a.H == 0) return hipSuccess;
  dim3 grid(max_panels, a.H, a.B), block(256);
#define SAGE_PREPV(DT, DD, PVV) prep_v_kernel<DT, DD, PVV><<<grid, block, 0, st>>>(a)
  if (dtype == 0) {
    if (a.D == 64) { if (pv) SAGE_PREPV(0, 64, 1); else SAGE_PREPV(0, 64, 0); }
    else { if (pv) SAGE_PREPV(0, 128, 1); else SAGE_PREPV(0, 128, 0); }
  } else {
    if (a.D == 64) { if (pv) SAGE_PREPV(1, 64, 1); else SAGE_PREPV(1, 64, 0); }
    else { if (pv) SAGE_PREPV(1, 128, 1); else SAGE_PREPV(1, 128, 0); }
  }
#undef SAGE_PREPV
  return hipGetLastError();
}

}  // namespace sage
