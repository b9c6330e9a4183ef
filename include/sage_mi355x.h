/*
 * sage_mi355x.h -- C ABI of libsage_mi355x.so, the MI355X (gfx950) SageAttention forward path.
 *
 * Plain pointers and sizes only; no torch types.  Every pointer is DEVICE memory owned by the
 * caller unless stated otherwise.  No entry point allocates or frees device memory, and none
 * synchronises: all work is enqueued on `stream` (a hipStream_t passed as void*; NULL = the
 * default stream).  Return value: 0 on success, a negative SAGE_E* code on failure, in which
 * case nothing was launched and sage_last_error() describes the problem (thread-local).
 *
 * Tensor addressing.  Q/K/V/out are rank-4 with a contiguous last (head_dim) axis; the caller
 * passes element strides (batch, head, sequence) so that both reference layouts are served:
 *   HND [B,H,L,D]: sb=H*L*D sh=L*D sn=D        NHD [B,L,H,D]: sb=L*H*D sh=D sn=H*D
 * (the stride selection of backends/_enflame/ops/sage_attention/quant_per_block.py:56-73 and
 *  backends/_hygon/ops/sageattention/sageattention_triton.py:132-137).
 * Packed variable-length inputs [T,H,D] are the NHD case with B = number of sequences and a
 * cu_seqlens array (int32 [B+1], device) giving each sequence's first row; sb is ignored.
 */
#ifndef SAGE_MI355X_H
#define SAGE_MI355X_H

#include <stdint.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SAGE_OK 0
#define SAGE_EINVAL (-1)   /* bad shape / stride / block size: the reference raises ValueError   */
#define SAGE_ETYPE (-2)    /* bad dtype flag: the reference raises TypeError                     */
#define SAGE_ENOTIMPL (-3) /* unsupported head_dim / block size: NotImplementedError             */
#define SAGE_ELAUNCH (-4)  /* HIP reported an error when launching                               */
#define SAGE_EWORKSPACE (-5) /* workspace too small                                              */

#define SAGE_DT_F16 0
#define SAGE_DT_BF16 1

#define SAGE_PV_FP16 0 /* P and V in fp16, fp32 accumulate (the reference's _attention_kernel)   */
#define SAGE_PV_FP8 1  /* P and V in fp8-e4m3fn, fp32 accumulate, per-channel V scale            */

/* explicit attention masks (sageattention_triton.py:180-186: MASK_KIND 1 / 2) */
#define SAGE_MASK_BOOL 1     /* bytes; non-zero = the key is visible (torch.bool)                */
#define SAGE_MASK_ADDITIVE 2 /* fp32 bias added to the logits                                    */

/* Interleaved ("per-thread") Q scales.  OR-ed into a Q block size -- `blk` of sage_quant_int8 when it quantises Q, `blkq`
 * of sage_attn_fwd, sage_attn_fwd_masked, sage_sageattn*, sage_sageattn_workspace_bytes -- it gives every block of blkq
 * rows EIGHT scales instead of one: scale g of a block covers the rows r of the block with r % 8 == g, and the scale
 * tensor holds ceil(S/blkq)*8 values per head, scale[(b*H + h)*ceil(S/blkq)*8 + block*8 + g].  This is the granularity
 * upstream SageAttention calls per-thread (its WARPQ = blkq: on its MMA fragments the rows i, i+8, i+16, ... of a
 * warp tile sit in one thread; here a query row is a lane of the transposed score tile, so a scale per row group costs
 * nothing extra in the kernel).  The reference names it as a finer granularity next to the (128, 16, -1, 1) recipe of
 * backends/_mthreads/docs/sageAttention_mthread.md:36-42 and has no code for it: the quantiser arithmetic is that of
 * quant_per_block.py:38-46 applied per row group.  Fixed-length batches only; not for K; the Q quantisation fused into the
 * attention kernel (sage_attn_fwd_qfused) does not take it -- sage_sageattn* run the standalone Q pass instead. */
#define SAGE_BLK_INTERLEAVE8 0x100
/* The same for K (upstream's per-thread K granularity, its WARPK = blkk): OR-ed into `blk` of sage_quant_int8 when it
 * quantises K and into `blkk` of sage_attn_fwd, sage_attn_fwd_qfused, sage_sageattn* and sage_sageattn_workspace_bytes,
 * every block of blkk = 32, 64 or 128 keys carries FOUR scales, scale t for the keys n of the block with (n % 8) / 2 == t
 * (keys 2t, 2t+1, 2t+8, 2t+9, ...): scale[(b*H + h)*ceil(S/blkk)*4 + block*4 + t].  In the transposed score tile a lane
 * holds keys of exactly two of the four groups per 32 keys, so the kernel applies two scales per lane and 32-key group.
 * Fixed-length batches only. */
#define SAGE_BLK_INTERLEAVE4 0x200

/* Rows of K/V covered by one V panel (see sage_prep_v). */
#define SAGE_PANEL_ROWS 128

typedef void* sage_stream_t;

/* Replaces backend_name() of backends/_hygon/ops/sageattention/sageattention_hip.py:77-79. */
const char* sage_backend_name(void);

/* Message for the last non-zero return on this thread ("" if none). */
const char* sage_last_error(void);

/*
 * Per-block INT8 quantiser for one operand.  Replaces one launch of
 * quant_per_block_int8_kernel (backends/_enflame/ops/sage_attention/quant_per_block.py:20-46,
 * launched at :82-98) including the optional `k - km` of :53-54 and the zero-tile floor of
 * backends/_hygon/ops/sageattention/sageattention_triton.py:35:
 *   x32 = fp32(round_dtype(x - km)) * mult;  scale = max(max|x32|/127, 1e-12);
 *   out = (int8) trunc(x32/scale + (x32/scale >= 0 ? 0.5 : -0.5)),  all in IEEE binary32.
 * x:      [B,H,L,D] via (x_sb,x_sh,x_sn), dtype = SAGE_DT_*.
 * km:     NULL, or per-(batch,head) channel vector in x's dtype at km + b*km_sb + h*km_sh + c.
 * out:    int8, addressed with (o_sb,o_sh,o_sn).
 * scale:  fp32; fixed-length: scale[(b*H + h)*ceil(L/blk) + block];
 *         packed: scale[h*scale_sh + cu_blocks[b] + block] (cu_blocks from sage_varlen_plan).
 * mult:   sm_scale*1.44269504 for Q (quant_per_block.py:87), 1.0 for K (:97).
 * blk in {16,32,64,128}, optionally | SAGE_BLK_INTERLEAVE8 or, for 32 rows and more, | SAGE_BLK_INTERLEAVE4 (fixed-length
 * only); D in {64,128}.  In packed mode L is the longest sequence.
 */
int sage_quant_int8(const void* x, int8_t* out, float* scale, const void* km,
                    int B, int H, int L, int D,
                    int64_t x_sb, int64_t x_sh, int64_t x_sn,
                    int64_t o_sb, int64_t o_sh, int64_t o_sn,
                    int64_t km_sb, int64_t km_sh,
                    int blk, float mult, int dtype,
                    const int32_t* cu_seqlens, const int32_t* cu_blocks, int64_t scale_sh,
                    sage_stream_t stream);

/*
 * Per-(batch, head, channel) mean of K over the sequence, written in K's dtype to
 * km[(b*H + h)*D + c].  The reference only ever receives km as an argument
 * (quant_per_block.py:49, :53-54); this computes the one SageAttention's K smoothing uses:
 * float64 sum, /L, rounded to fp32 and then to the input dtype.
 * workspace: sage_k_mean_workspace_bytes(B,H,L,D) bytes of device scratch.
 */
size_t sage_k_mean_workspace_bytes(int B, int H, int L, int D);
int sage_k_mean(const void* k, void* km, void* workspace, size_t workspace_bytes,
                int B, int H, int L, int D,
                int64_t k_sb, int64_t k_sh, int64_t k_sn, int dtype,
                const int32_t* cu_seqlens, sage_stream_t stream);

/*
 * V preparation: converts V into the MFMA-ready "panel" layout the attention kernel streams
 * (no counterpart in the reference, whose kernel reads V row-major:
 * backends/_hygon/ops/sageattention/sageattention_triton.py:114-118).
 *   SAGE_PV_FP16: values cast to fp16 (as attn_qk_int8_per_block_native.py:312 does).
 *   SAGE_PV_FP8 : v_scale[(b*H+h)*D + c] = max(max_n|v|/448, 1e-12); v8 = e4m3fn_rne(v/v_scale).
 * A panel covers SAGE_PANEL_ROWS consecutive rows of one (batch, head); rows past the end of
 * the sequence are zero.  panels: fixed-length [(b*H+h)*ceil(L/128) + p], packed
 * [h*panel_sh + cu_panels[b] + p], each panel 128*D*(1 or 2) bytes.  Byte order inside a panel
 * is documented in baselinebenchmark_amd/csrc/sage_common.h.
 * workspace: sage_prep_v_workspace_bytes(...) bytes (FP8 mode only; may be NULL for FP16).
 */
size_t sage_prep_v_workspace_bytes(int B, int H, int L, int D, int pv_mode);
size_t sage_v_panel_bytes(int B, int H, int L, int D, int pv_mode); /* fixed-length buffer size */
int sage_prep_v(const void* v, void* panels, float* v_scale, void* workspace, size_t workspace_bytes,
                int B, int H, int L, int D,
                int64_t v_sb, int64_t v_sh, int64_t v_sn, int dtype, int pv_mode,
                const int32_t* cu_seqlens, const int32_t* cu_panels, int64_t panel_sh,
                sage_stream_t stream);

/*
 * Variable-length plan (device-side scheduler).  From cu_seqlens_q/k (int32 [nseq+1], device)
 * it fills `plan` (int32, device, sage_varlen_plan_ints(nseq, total_q, blkq_min) entries) with:
 * block offsets of every sequence for the Q scales, K scales and V panels, and the list of
 * (sequence, q-tile) attention tiles ordered by decreasing cost.  Layout: see SagePlanLayout in
 * sage_common.h; sage_varlen_plan_offsets() returns the int offsets of each array in `plan`:
 * offs[0]=cu_qblk offs[1]=cu_kblk offs[2]=cu_panel offs[3]=tile count offs[4]=tiles.
 */
size_t sage_varlen_plan_ints(int nseq, int total_q);
void sage_varlen_plan_offsets(int nseq, int total_q, int64_t offs[5]);
int sage_varlen_plan(const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, int nseq,
                     int total_q, int blkq, int blkk, int is_causal,
                     int32_t* plan, size_t plan_ints, sage_stream_t stream);

/*
 * Fused attention on quantised operands.  Replaces _attention_kernel + forward
 * (backends/_hygon/ops/sageattention/sageattention_triton.py:45-129, :167-207):
 *   S = (Qi8 . Ki8^T) * (q_scale*k_scale), base-2 online softmax in fp32, O = P.V with fp32
 *   accumulation, O /= l, optional LSE2 = log2(l) + m  (lse[(b*Hq+h)*Sq + i], fp32).
 * plus causal masking (key j visible to query i iff j <= i) with block skipping, and packed
 * variable-length batches.  kvh = qh / (Hq/Hkv) (sageattention_triton.py:61).
 * q_scale/k_scale: as written by sage_quant_int8 with blkq and blkk in {16, 32, 64, 128}
 * (16: the K granularity of the external recipe (128, 16), sage_attention_benchmark_compare.py:93).
 * v_panels/v_scale: as written by sage_prep_v (v_scale NULL for SAGE_PV_FP16).
 * out: fp16/bf16 (out_dtype) addressed with (o_sb,o_sh,o_sn), base and strides multiples of 16 bytes (rows are
 * stored 16 bytes per lane); lse may be NULL.  A (batch, head) slice of k -- and of a floating-point q in
 * sage_attn_fwd_qfused -- must span less than 2 GiB (tile loads use 32-bit byte offsets): SAGE_ENOTIMPL otherwise.
 * Packed mode: cu_seqlens_q != NULL; B = nseq, Sq/Skv = longest sequences, `plan` from
 * sage_varlen_plan, total_q = number of packed query rows, scale/panel head strides given.
 */
int sage_attn_fwd(const int8_t* q, const int8_t* k, const void* v_panels,
                  const float* q_scale, const float* k_scale, const float* v_scale,
                  void* out, float* lse,
                  int B, int Hq, int Hkv, int Sq, int Skv, int D,
                  int64_t q_sb, int64_t q_sh, int64_t q_sn,
                  int64_t k_sb, int64_t k_sh, int64_t k_sn,
                  int64_t o_sb, int64_t o_sh, int64_t o_sn,
                  int blkq, int blkk, int is_causal, int pv_mode, int out_dtype,
                  const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                  const int32_t* plan, int total_q,
                  int64_t q_scale_sh, int64_t k_scale_sh, int64_t panel_sh,
                  sage_stream_t stream);

/*
 * Attention on a floating-point Q and already quantised K / V: every workgroup quantises its own
 * q-tile in the prologue with the arithmetic of sage_quant_int8 (quant_per_block.py:38-46, Q multiplier
 * (float)(sm_scale * 1.44269504) of :87; sm_scale <= 0 selects head_dim^-0.5), so the result is bit-identical
 * to sage_quant_int8 on q followed by sage_attn_fwd, without the HBM round trip of the INT8 copy of q.
 * This is what sage_sageattn runs; it also fits callers that keep K and V quantised (a KV cache) and
 * bring a fresh q.  q: fp16/bf16 (q_dtype) with element strides; everything else as in sage_attn_fwd.
 * No counterpart in the reference (its quantiser is always a separate launch, sageattention_triton.py:140-164).
 */
int sage_attn_fwd_qfused(const void* q, int q_dtype, double sm_scale,
                         const int8_t* k, const void* v_panels,
                         const float* k_scale, const float* v_scale,
                         void* out, float* lse,
                         int B, int Hq, int Hkv, int Sq, int Skv, int D,
                         int64_t q_sb, int64_t q_sh, int64_t q_sn,
                         int64_t k_sb, int64_t k_sh, int64_t k_sn,
                         int64_t o_sb, int64_t o_sh, int64_t o_sn,
                         int blkq, int blkk, int is_causal, int pv_mode, int out_dtype,
                         const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                         const int32_t* plan, int total_q,
                         int64_t k_scale_sh, int64_t panel_sh,
                         sage_stream_t stream);

/*
 * The same with an explicit mask: the attn_mask argument of forward
 * (sageattention_triton.py:167-168, :92-105; exercised by
 * backends/_hygon/test/sageattention/test_sageattention_hip.py:40-45, :65-66).
 * attn_mask is [B, Hq, Sq, Skv] addressed with ELEMENT strides (m_sb, m_sh, m_sm, m_sn; 0 broadcasts):
 *   SAGE_MASK_BOOL     : logits of keys whose byte is 0 become -inf;
 *   SAGE_MASK_ADDITIVE : the fp32 value is added to the base-2 logits (q_scale already holds
 *                        sm_scale*log2(e), so the bias is in those units, as in the reference).
 * A row with no visible key yields out = 0 and LSE2 = -inf.  Every K scale granularity is taken (blocks of 16 to 128 keys,
 * SAGE_BLK_INTERLEAVE4).  No causal flag and no packed mode here.
 */
int sage_attn_fwd_masked(const int8_t* q, const int8_t* k, const void* v_panels,
                         const float* q_scale, const float* k_scale, const float* v_scale,
                         void* out, float* lse,
                         int B, int Hq, int Hkv, int Sq, int Skv, int D,
                         int64_t q_sb, int64_t q_sh, int64_t q_sn,
                         int64_t k_sb, int64_t k_sh, int64_t k_sn,
                         int64_t o_sb, int64_t o_sh, int64_t o_sn,
                         int blkq, int blkk, int pv_mode, int out_dtype,
                         const void* attn_mask, int mask_kind,
                         int64_t m_sb, int64_t m_sh, int64_t m_sm, int64_t m_sn,
                         sage_stream_t stream);

/*
 * One-call pipeline behind sageattn(q, k, v, tensor_layout, is_causal, sm_scale, ...) -- the
 * entry point exercised at backends/_metax/benchmarks/sage_attention/benchmark.py:29 and
 * backends/_mthreads/benchmarks/sage_attention_benchmark_compare.py:300-313:
 * [K mean] -> quantise K (minus mean) -> prepare V -> attention (which quantises its own Q tiles; a
 * separate Q pass only where a mask or the LSE correction need one).
 * All intermediates live in `workspace` (sage_sageattn_workspace_bytes); nothing is allocated.
 * smooth_k != 0 subtracts the per-channel K mean.  sm_scale <= 0 selects head_dim^-0.5; the Q
 * multiplier is (float)(sm_scale * 1.44269504), the double product of quant_per_block.py:87.  Packed mode as in sage_attn_fwd
 * (cu_seqlens_* != NULL; total_q/total_k = packed row counts).
 * lse (may be NULL) receives the base-2 log-sum-exp of the logits of the ORIGINAL k: with smooth_k the
 * term q . k_mean that smoothing removed from every logit of a row is added back.
 * q, k, v and out may be arbitrary strided views (16-byte aligned rows, contiguous head_dim), e.g. slices of a
 * fused QKV buffer: the INT8 copies inside the workspace use dense strides of their own.
 */
size_t sage_sageattn_workspace_bytes(int B, int Hq, int Hkv, int Sq, int Skv, int D,
                                     int blkq, int blkk, int pv_mode, int total_q, int total_k,
                                     int varlen);
/* The same for ONE kind of call: without an explicit mask, and unless LSE is returned from smoothed keys or the Q scales
 * are interleaved, Q is quantised inside the attention kernel and its INT8 copy (a third of the upper bound) is not
 * part of the workspace.  sage_sageattn / sage_sageattn_masked accept any workspace of at least this size for the call
 * they are given; sage_sageattn_static checks it against its capacity. */
size_t sage_sageattn_workspace_bytes_for(int B, int Hq, int Hkv, int Sq, int Skv, int D,
                                         int blkq, int blkk, int pv_mode,
                                         int total_q, int total_k, int varlen,
                                         int smooth_k, int want_lse, int has_mask);
int sage_sageattn(const void* q, const void* k, const void* v, void* out, float* lse,
                  void* workspace, size_t workspace_bytes,
                  int B, int Hq, int Hkv, int Sq, int Skv, int D,
                  int64_t q_sb, int64_t q_sh, int64_t q_sn,
                  int64_t k_sb, int64_t k_sh, int64_t k_sn,
                  int64_t v_sb, int64_t v_sh, int64_t v_sn,
                  int64_t o_sb, int64_t o_sh, int64_t o_sn,
                  int dtype, int blkq, int blkk, double sm_scale, int is_causal, int smooth_k,
                  int pv_mode,
                  const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                  int total_q, int total_k,
                  sage_stream_t stream);

/*
 * sageattn with an explicit mask, the call of
 * backends/_mthreads/tests/test_sage_attention_mate.py:186-208 (attn_mask keyword) checked against
 * softmax(sm_scale * q.k^T + mask) at :171-178: here the additive mask is in NATURAL-log units on top
 * of sm_scale * q.k^T (it is multiplied by log2(e) internally); boolean masks as in
 * sage_attn_fwd_masked.  attn_mask == NULL makes it identical to sage_sageattn.
 */
int sage_sageattn_masked(const void* q, const void* k, const void* v, void* out, float* lse,
                         void* workspace, size_t workspace_bytes,
                         int B, int Hq, int Hkv, int Sq, int Skv, int D,
                         int64_t q_sb, int64_t q_sh, int64_t q_sn,
                         int64_t k_sb, int64_t k_sh, int64_t k_sn,
                         int64_t v_sb, int64_t v_sh, int64_t v_sn,
                         int64_t o_sb, int64_t o_sh, int64_t o_sn,
                         int dtype, int blkq, int blkk, double sm_scale, int is_causal, int smooth_k,
                         int pv_mode, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                         int total_q, int total_k,
                         const void* attn_mask, int mask_kind,
                         int64_t m_sb, int64_t m_sh, int64_t m_sm, int64_t m_sn,
                         sage_stream_t stream);

/*
 * sage_sageattn for callers that cannot allocate device memory or carry a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid allocation).  It has no counterpart in the reference.
 * Same arguments and results as sage_sageattn minus `workspace`/`workspace_bytes`: the intermediates (INT8 K,
 * scales, K mean, V panels, statistics partials, the packed-batch plan, INT8 Q where a separate pass is needed)
 * live in an array of SAGE_STATIC_SCRATCH_BYTES that is part of the library's device image, one copy per GPU,
 * held until the process ends.  The call allocates and frees nothing and does not synchronise.
 * The FIRST call on a device (of this entry point, and of each kernel variant it launches) additionally looks up the
 * array's address and raises the kernels' dynamic-LDS limit -- runtime calls that may allocate and are not allowed
 * while a stream is capturing: make one call of the same kind outside the capture first (tests/test_zz_no_alloc.py).
 * Limit: sage_sageattn_workspace_bytes_for(...) of the call must not exceed sage_sageattn_static_capacity()
 * (= SAGE_STATIC_SCRATCH_BYTES); larger problems return SAGE_EWORKSPACE and launch nothing.
 * All calls on one GPU share that GPU's array: calls that may overlap on one GPU (different streams, or host
 * threads without ordering between their streams) race; serialise them or use sage_sageattn.  The array keeps
 * the previous call's contents; every intermediate is rewritten before it is read, so nothing needs clearing.
 */
#define SAGE_STATIC_SCRATCH_BYTES (64u << 20)
size_t sage_sageattn_static_capacity(void);
int sage_sageattn_static(const void* q, const void* k, const void* v, void* out, float* lse,
                         int B, int Hq, int Hkv, int Sq, int Skv, int D,
                         int64_t q_sb, int64_t q_sh, int64_t q_sn,
                         int64_t k_sb, int64_t k_sh, int64_t k_sn,
                         int64_t v_sb, int64_t v_sh, int64_t v_sn,
                         int64_t o_sb, int64_t o_sh, int64_t o_sn,
                         int dtype, int blkq, int blkk, double sm_scale, int is_causal, int smooth_k,
                         int pv_mode,
                         const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                         int total_q, int total_k,
                         sage_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* SAGE_MI355X_H */
