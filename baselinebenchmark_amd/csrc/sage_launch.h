// Host-side launcher declarations shared between the kernel translation units and the C ABI.
#pragma once
#include "sage_common.h"

namespace sage {

struct QuantArgs {
  const u16* x;
  int8_t* out;
  float* scale;
  const u16* km;
  int B, H, L, D;
  int64_t x_sb, x_sh, x_sn, o_sb, o_sh, o_sn, km_sb, km_sh;
  int blk;
  int groups;   // scales per block: 1; 8 (scale g covers the rows r of the block with r % 8 == g); 4 ((r % 8) / 2 == g); fixed-length only
  float mult;
  const int32_t* cu_seqlens;
  const int32_t* cu_blocks;
  int64_t scale_sh;
  // optional row dot products (null dot_out: off): dotv is [B, H/dv_group, D] in the input dtype,
  // dot_out is [B, H, L] (or [H, dot_total] for packed rows) fp32
  const u16* dotv;
  float* dot_out;
  int64_t dv_sb, dv_sh;
  int dv_group;
  int dot_total;
};

struct ColStatArgs {
  const u16* x;
  void* partial;  // double or float [B*H*nchunk*D]
  int B, H, L, D;
  int64_t x_sb, x_sh, x_sn;
  int nchunk;
  const int32_t* cu_seqlens;
};

struct PrepVArgs {
  const u16* v;
  uint8_t* panels;
  const float* vscale;  // [B*H*D] (fp8) or null
  int B, H, L, D;
  int64_t v_sb, v_sh, v_sn;
  const int32_t* cu_seqlens;
  const int32_t* cu_panels;
  int64_t panel_sh;
};

// Division of a 32-bit unsigned number by a launch constant as a multiply-high and two shifts (exact for every 32-bit
// dividend): the tile decode of the attention kernel divides the workgroup index by head counts that are no powers of
// two, and a true integer division is some twenty dependent instructions on this hardware, paid by every workgroup
// before its first memory request.
struct FastDiv {
  uint32_t mul, sh1, sh2;
};
inline FastDiv make_fastdiv(uint32_t d) {
  FastDiv f;
  uint32_t L = 0;
  while (L < 32 && (uint64_t(1) << L) < d) L++;               // ceil(log2 d); d >= 1
  f.mul = (uint32_t)(((uint64_t(1) << 32) * ((uint64_t(1) << L) - d)) / d + 1);
  f.sh1 = L < 1 ? L : 1;
  f.sh2 = L < 1 ? 0 : L - 1;
  return f;
}
__device__ inline uint32_t fastdiv(uint32_t n, const FastDiv& f) {
  const uint32_t t = __umulhi(f.mul, n);
  return (t + ((n - t) >> f.sh1)) >> f.sh2;
}

struct AttnArgs {
  const int8_t* q;
  const int8_t* k;
  const uint8_t* vp;
  const float* qs;
  const float* ks;
  const float* vs;
  void* out;
  float* lse;
  int B, Hq, Hkv, Sq, Skv;
  int64_t q_sb, q_sh, q_sn, k_sb, k_sh, k_sn, o_sb, o_sh, o_sn;
  int blkq, blkk;            // scale block sizes: powers of two (32, 64, 128)
  int blkq_shift, blkk_shift;  // their log2
  int qg_shift;              // log2 of the Q scales per block: 0, or 3 (eight interleaved scales: rows r, r + 8, ... share one)
  int k_interleave;          // 1: four interleaved K scales per block (scale t for the keys n with (n % 8) / 2 == t); host-side dispatch only
  int out_bf16;
  int nqt;  // q-tiles per sequence (fixed-length mode)
  // launch constants of the tile decode (filled in by finish_attn_args)
  int G;                    // q-heads per KV head
  int tier_shift;           // fixed-length mode, per-XCD tile order: log2 of the widest range of q-tiles; -1: plain order
  FastDiv div_G, div_Hkv, div_heads;   // heads = B*Hq (fixed-length) or Hq (packed)
  FastDiv div_range, div_last;         // full-attention tile order: q-tiles x heads-per-XCD of a range; width of the last range
  // packed mode (cu_q != nullptr)
  const int32_t* cu_q;
  const int32_t* cu_k;
  const int32_t* cu_qblk;
  const int32_t* cu_kblk;
  const int32_t* cu_panel;
  const int32_t* ntiles;
  const int32_t* tiles;
  int64_t qs_sh, ks_sh, panel_sh;
  int total_q;
  // explicit mask (fixed-length mode only): [B, Hq, Sq, Skv] with element strides; kind 1 = bytes
  // (non-zero keeps the key), 2 = fp32 added to the base-2 logits
  const void* mask;
  int mask_kind;
  int64_t m_sb, m_sh, m_sm, m_sn;
  float mask_mult;          // additive masks are scaled by this before they are added
  const float* lse_offset;  // added to LSE2 per query row (same layout as lse) or null
  // fused Q quantisation: fp16/bf16 Q with the strides of q (q and qs are then unused)
  const void* q_raw;
  int q_is_bf16;
  float q_mult;
};

struct AttnConfig { int nw, bn; };

hipError_t launch_quant_int8(const QuantArgs& a, int dtype, int max_blocks, hipStream_t st);
int colstat_chunks(int L);
hipError_t launch_k_mean(const ColStatArgs& a, int dtype, void* km, hipStream_t st);
hipError_t launch_v_scale(const ColStatArgs& a, int dtype, float* vscale, hipStream_t st);
hipError_t launch_prep_v(const PrepVArgs& a, int dtype, int pv, int max_panels, hipStream_t st);
// Short fixed-length sequences: K mean + K quantiser + V scale + V panels in one launch (nk K tiles and nv V panels per
// (batch, kv-head); km_out / vscale_out take the statistics; qa.km is ignored and must be null).
hipError_t launch_prepass_small(const QuantArgs& qa, const PrepVArgs& va, int dtype, int pv, int nk, int nv, int smooth,
                                void* km_out, float* vscale_out, hipStream_t st);

AttnConfig attn_config(int D, int pv, bool packed);
// Fills in the launch constants of the tile decode from the dimensions already in `a` (B, Hq, Hkv, nqt, cu_q).
void finish_attn_args(AttnArgs& a, bool causal);
hipError_t launch_attn(const AttnArgs& a, int D, int pv, bool causal, int grid, hipStream_t st);
hipError_t launch_attn_masked(const AttnArgs& a, int D, int pv, int grid, hipStream_t st);
hipError_t launch_attn_qfused(const AttnArgs& a, int D, int pv, bool causal, int grid, hipStream_t st);
hipError_t launch_attn_k16(const AttnArgs& a, int D, int pv, bool causal, int grid, hipStream_t st);
hipError_t launch_attn_kinterleaved(const AttnArgs& a, int D, int pv, bool causal, int grid, hipStream_t st);
hipError_t launch_varlen_plan(const int32_t* cu_q, const int32_t* cu_k, int nseq, int total_q, int blkq, int blkk, int bm,
                              int bn, int causal, int32_t* plan, hipStream_t st);

}  // namespace sage
