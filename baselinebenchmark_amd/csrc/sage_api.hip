// C ABI of libsage_mi355x.so (declared in include/sage_mi355x.h): argument validation with the
// reference's error classes, workspace carving, the one-call sageattn pipeline and the launch
// geometry of every kernel.  Nothing here allocates device memory or synchronises.
#include "sage_launch.h"
#include "../../include/sage_mi355x.h"

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <cmath>
#include <cstdlib>

using namespace sage;

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int hip_fail(hipError_t e, const char* what) {
  return fail(SAGE_ELAUNCH, "%s: %s", what, hipGetErrorString(e));
}

inline size_t align_up(size_t x, size_t a = 256) { return (x + a - 1) / a * a; }

bool valid_blk_quant(int blk) { return blk == 16 || blk == 32 || blk == 64 || blk == 128; }
bool valid_blk_attn(int blk) { return blk == 16 || blk == 32 || blk == 64 || blk == 128; }
bool valid_blkk_attn(int blk) { return valid_blk_attn(blk); }
int ilog2(int x) { int r = 0; while ((1 << r) < x) r++; return r; }
// A Q block-size argument may carry SAGE_BLK_INTERLEAVE8: eight interleaved scales per block instead of one.
// ... or SAGE_BLK_INTERLEAVE4 (a K block size): four.  Both flags at once decode to 0 groups, which nothing accepts.
int blk_rows(int blk) { return blk > 0 ? (blk & ~(SAGE_BLK_INTERLEAVE8 | SAGE_BLK_INTERLEAVE4)) : blk; }
int blk_groups(int blk) {
  if (blk <= 0) return 1;
  const bool g8 = blk & SAGE_BLK_INTERLEAVE8, g4 = blk & SAGE_BLK_INTERLEAVE4;
  return g8 && g4 ? 0 : g8 ? 8 : g4 ? 4 : 1;
}

int check_common(int B, int H, int L, int D, int dtype) {
  if (B < 0 || H < 0 || L < 0) return fail(SAGE_EINVAL, "negative dimension (B=%d H=%d L=%d)", B, H, L);
  if (D != 64 && D != 128) return fail(SAGE_ENOTIMPL, "head_dim %d is not supported (64 or 128)", D);
  if (dtype != SAGE_DT_F16 && dtype != SAGE_DT_BF16) return fail(SAGE_ETYPE, "dtype flag %d is not fp16(0)/bf16(1)", dtype);
  return SAGE_OK;
}

int check_stride16(const char* name, int64_t sb, int64_t sh, int64_t sn, int esz, const void* p) {
  // 128-bit accesses: every row must start on a 16-byte boundary
  if ((sb * esz) % 16 || (sh * esz) % 16 || (sn * esz) % 16 || (reinterpret_cast<uintptr_t>(p) % 16))
    return fail(SAGE_EINVAL, "%s: base pointer and strides must be 16-byte aligned", name);
  return SAGE_OK;
}

}  // namespace

namespace sage {
int set_error(int code, const char* msg) { return fail(code, "%s", msg); }
}  // namespace sage

extern "C" {

const char* sage_backend_name(void) { return "mi355x_hip_int8_qk_fp8_fp16_pv"; }

const char* sage_last_error(void) { return g_err; }

}  // extern "C"

namespace {
struct RowDot {   // optional side output of the quantiser (see QuantArgs)
  const void* vec = nullptr;
  float* out = nullptr;
  int64_t sb = 0, sh = 0;
  int group = 1, total = 0;
};

int quant_impl(const void* x, int8_t* out, float* scale, const void* km, int B, int H, int L, int D, int64_t x_sb,
               int64_t x_sh, int64_t x_sn, int64_t o_sb, int64_t o_sh, int64_t o_sn, int64_t km_sb, int64_t km_sh, int blk,
               float mult, int dtype, const int32_t* cu_seqlens, const int32_t* cu_blocks, int64_t scale_sh,
               const RowDot& dot, sage_stream_t stream) {
  if (int rc = check_common(B, H, L, D, dtype)) return rc;
  const int groups = blk_groups(blk);
  blk = blk_rows(blk);
  if (!valid_blk_quant(blk)) return fail(SAGE_ENOTIMPL, "quantisation block %d is not supported (16, 32, 64, 128)", blk);
  if (groups == 0) return fail(SAGE_EINVAL, "SAGE_BLK_INTERLEAVE8 and SAGE_BLK_INTERLEAVE4 exclude each other");
  if (groups > 1 && cu_seqlens) return fail(SAGE_ENOTIMPL, "interleaved scales are not supported for packed batches");
  if (groups == 4 && blk == 16) return fail(SAGE_ENOTIMPL, "four interleaved scales need blocks of 32, 64 or 128 rows");
  if (B == 0 || H == 0 || L == 0) return SAGE_OK;
  if (!x || !out || !scale) return fail(SAGE_EINVAL, "null tensor pointer");
  if (cu_seqlens && !cu_blocks) return fail(SAGE_EINVAL, "packed mode needs cu_blocks");
  if (int rc = check_stride16("x", x_sb, x_sh, x_sn, 2, x)) return rc;
  if (int rc = check_stride16("out", o_sb, o_sh, o_sn, 1, out)) return rc;
  if (km && int(check_stride16("km", km_sb, km_sh, 0, 2, km))) return SAGE_EINVAL;
  QuantArgs a;
  memset(&a, 0, sizeof(a));
  a.x = (const u16*)x; a.out = out; a.scale = scale; a.km = (const u16*)km;
  a.B = B; a.H = H; a.L = L; a.D = D;
  a.x_sb = x_sb; a.x_sh = x_sh; a.x_sn = x_sn; a.o_sb = o_sb; a.o_sh = o_sh; a.o_sn = o_sn;
  a.km_sb = km_sb; a.km_sh = km_sh; a.blk = blk; a.groups = groups; a.mult = mult;
  a.cu_seqlens = cu_seqlens; a.cu_blocks = cu_blocks; a.scale_sh = scale_sh;
  a.dotv = (const u16*)dot.vec; a.dot_out = dot.out; a.dv_sb = dot.sb; a.dv_sh = dot.sh; a.dv_group = dot.group;
  a.dot_total = dot.total;
  hipError_t e = launch_quant_int8(a, dtype, (L + blk - 1) / blk, (hipStream_t)stream);
  if (e != hipSuccess) return hip_fail(e, "sage_quant_int8");
  return SAGE_OK;
}
}  // namespace

extern "C" {

int sage_quant_int8(const void* x, int8_t* out, float* scale, const void* km, int B, int H, int L, int D, int64_t x_sb,
                    int64_t x_sh, int64_t x_sn, int64_t o_sb, int64_t o_sh, int64_t o_sn, int64_t km_sb, int64_t km_sh,
                    int blk, float mult, int dtype, const int32_t* cu_seqlens, const int32_t* cu_blocks,
                    int64_t scale_sh, sage_stream_t stream) {
  return quant_impl(x, out, scale, km, B, H, L, D, x_sb, x_sh, x_sn, o_sb, o_sh, o_sn, km_sb, km_sh, blk, mult, dtype,
                    cu_seqlens, cu_blocks, scale_sh, RowDot(), stream);
}

size_t sage_k_mean_workspace_bytes(int B, int H, int L, int D) {
  return align_up((size_t)B * H * colstat_chunks(L) * D * sizeof(double));
}

int sage_k_mean(const void* k, void* km, void* workspace, size_t workspace_bytes, int B, int H, int L, int D, int64_t k_sb,
                int64_t k_sh, int64_t k_sn, int dtype, const int32_t* cu_seqlens, sage_stream_t stream) {
  if (int rc = check_common(B, H, L, D, dtype)) return rc;
  if (B == 0 || H == 0) return SAGE_OK;
  if (!k || !km || !workspace) return fail(SAGE_EINVAL, "null tensor pointer");
  if (workspace_bytes < sage_k_mean_workspace_bytes(B, H, L, D)) return fail(SAGE_EWORKSPACE, "k_mean workspace too small");
  if (int rc = check_stride16("k", k_sb, k_sh, k_sn, 2, k)) return rc;
  ColStatArgs a;
  a.x = (const u16*)k; a.partial = workspace; a.B = B; a.H = H; a.L = L; a.D = D;
  a.x_sb = k_sb; a.x_sh = k_sh; a.x_sn = k_sn; a.nchunk = colstat_chunks(L); a.cu_seqlens = cu_seqlens;
  if (a.nchunk == 0) a.nchunk = 1;  // L == 0: the finalize kernel still writes zeros
  hipError_t e = launch_k_mean(a, dtype, km, (hipStream_t)stream);
  if (e != hipSuccess) return hip_fail(e, "sage_k_mean");
  return SAGE_OK;
}

size_t sage_prep_v_workspace_bytes(int B, int H, int L, int D, int pv_mode) {
  if (pv_mode != SAGE_PV_FP8) return 0;
  int nc = colstat_chunks(L);
  return align_up((size_t)B * H * (nc ? nc : 1) * D * sizeof(float));
}

size_t sage_v_panel_bytes(int B, int H, int L, int D, int pv_mode) {
  size_t np = (L + SAGE_PANEL_ROWS - 1) / SAGE_PANEL_ROWS;
  return (size_t)B * H * np * SAGE_PANEL_ROWS * D * (pv_mode == SAGE_PV_FP8 ? 1 : 2);
}

int sage_prep_v(const void* v, void* panels, float* v_scale, void* workspace, size_t workspace_bytes, int B, int H, int L,
                int D, int64_t v_sb, int64_t v_sh, int64_t v_sn, int dtype, int pv_mode, const int32_t* cu_seqlens,
                const int32_t* cu_panels, int64_t panel_sh, sage_stream_t stream) {
  if (int rc = check_common(B, H, L, D, dtype)) return rc;
  if (pv_mode != SAGE_PV_FP16 && pv_mode != SAGE_PV_FP8) return fail(SAGE_EINVAL, "pv_mode %d unknown", pv_mode);
  if (B == 0 || H == 0 || L == 0) return SAGE_OK;
  if (!v || !panels) return fail(SAGE_EINVAL, "null tensor pointer");
  if (cu_seqlens && !cu_panels) return fail(SAGE_EINVAL, "packed mode needs cu_panels");
  if (int rc = check_stride16("v", v_sb, v_sh, v_sn, 2, v)) return rc;
  if (reinterpret_cast<uintptr_t>(panels) % 16) return fail(SAGE_EINVAL, "panels must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  if (pv_mode == SAGE_PV_FP8) {
    if (!v_scale || !workspace) return fail(SAGE_EINVAL, "fp8 mode needs v_scale and workspace");
    if (workspace_bytes < sage_prep_v_workspace_bytes(B, H, L, D, pv_mode)) return fail(SAGE_EWORKSPACE, "prep_v workspace too small");
    ColStatArgs c;
    c.x = (const u16*)v; c.partial = workspace; c.B = B; c.H = H; c.L = L; c.D = D;
    c.x_sb = v_sb; c.x_sh = v_sh; c.x_sn = v_sn; c.nchunk = colstat_chunks(L); c.cu_seqlens = cu_seqlens;
    hipError_t e = launch_v_scale(c, dtype, v_scale, st);
    if (e != hipSuccess) return hip_fail(e, "sage_prep_v(scale)");
  }
  PrepVArgs a;
  a.v = (const u16*)v; a.panels = (uint8_t*)panels; a.vscale = v_scale; a.B = B; a.H = H; a.L = L; a.D = D;
  a.v_sb = v_sb; a.v_sh = v_sh; a.v_sn = v_sn; a.cu_seqlens = cu_seqlens; a.cu_panels = cu_panels; a.panel_sh = panel_sh;
  hipError_t e = launch_prep_v(a, dtype, pv_mode, (L + SAGE_PANEL_ROWS - 1) / SAGE_PANEL_ROWS, st);
  if (e != hipSuccess) return hip_fail(e, "sage_prep_v");
  return SAGE_OK;
}

size_t sage_varlen_plan_ints(int nseq, int total_q) { return (size_t)plan_layout(nseq, total_q).total; }

void sage_varlen_plan_offsets(int nseq, int total_q, int64_t offs[5]) {
  SagePlanLayout L = plan_layout(nseq, total_q);
  offs[0] = L.cu_qblk; offs[1] = L.cu_kblk; offs[2] = L.cu_panel; offs[3] = L.ntiles; offs[4] = L.tiles;
}

int sage_varlen_plan(const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, int nseq, int total_q, int blkq, int blkk,
                     int is_causal, int32_t* plan, size_t plan_ints, sage_stream_t stream) {
  if (nseq <= 0 || nseq > 32767) return fail(SAGE_EINVAL, "number of sequences %d out of range (1..32767)", nseq);
  if (!cu_seqlens_q || !cu_seqlens_k || !plan) return fail(SAGE_EINVAL, "null pointer");
  if (!valid_blk_quant(blkq) || !valid_blk_quant(blkk)) return fail(SAGE_ENOTIMPL, "block sizes %d/%d not supported", blkq, blkk);
  if (plan_ints < sage_varlen_plan_ints(nseq, total_q)) return fail(SAGE_EWORKSPACE, "plan buffer too small");
  AttnConfig cfg = attn_config(128, 1, true);
  hipError_t e = launch_varlen_plan(cu_seqlens_q, cu_seqlens_k, nseq, total_q, blkq, blkk, cfg.nw * 32, 64, is_causal, plan,
                                    (hipStream_t)stream);
  if (e != hipSuccess) return hip_fail(e, "sage_varlen_plan");
  return SAGE_OK;
}

}  // extern "C"

namespace {
struct QRawArg {   // fp16/bf16 Q to be quantised by the attention kernel itself (q / q_scale are then ignored)
  const void* ptr = nullptr;
  int dtype = 0;
  float mult = 1.0f;
};

struct MaskArg {
  const void* ptr = nullptr;
  int kind = 0;
  int64_t sb = 0, sh = 0, sm = 0, sn = 0;
  float mult = 1.0f;   // additive masks are multiplied by this (1 for base-2 units, log2(e) for natural units)
};

int attn_impl(const int8_t* q, const int8_t* k, const void* v_panels, const float* q_scale, const float* k_scale,
              const float* v_scale, void* out, float* lse, int B, int Hq, int Hkv, int Sq, int Skv, int D, int64_t q_sb,
              int64_t q_sh, int64_t q_sn, int64_t k_sb, int64_t k_sh, int64_t k_sn, int64_t o_sb, int64_t o_sh,
              int64_t o_sn, int blkq, int blkk, int is_causal, int pv_mode, int out_dtype, const int32_t* cu_seqlens_q,
              const int32_t* cu_seqlens_k, const int32_t* plan, int total_q, int64_t q_scale_sh, int64_t k_scale_sh,
              int64_t panel_sh, const MaskArg& mask, const float* lse_offset, const QRawArg& qraw, sage_stream_t stream) {
  if (int rc = check_common(B, Hq, Sq, D, out_dtype)) return rc;
  if (Hkv <= 0 || Hq % Hkv) return fail(SAGE_EINVAL, "query heads (%d) must be divisible by KV heads (%d)", Hq, Hkv);
  if (Skv < 0) return fail(SAGE_EINVAL, "negative kv length");
  if (pv_mode != SAGE_PV_FP16 && pv_mode != SAGE_PV_FP8) return fail(SAGE_EINVAL, "pv_mode %d unknown", pv_mode);
  const int qgroups = blk_groups(blkq), kgroups = blk_groups(blkk);
  blkq = blk_rows(blkq);
  blkk = blk_rows(blkk);
  if (!valid_blk_attn(blkq) || !valid_blkk_attn(blkk))
    return fail(SAGE_ENOTIMPL, "attention needs Q and K scale blocks of 16, 32, 64 or 128 rows (got %d/%d)", blkq, blkk);
  if ((qgroups != 1 && qgroups != 8) || (kgroups != 1 && kgroups != 4))
    return fail(SAGE_ENOTIMPL, "Q scale blocks take SAGE_BLK_INTERLEAVE8, K scale blocks SAGE_BLK_INTERLEAVE4");
  if ((qgroups > 1 || kgroups > 1) && cu_seqlens_q) return fail(SAGE_ENOTIMPL, "interleaved scales are not supported for packed batches");
  if (qgroups > 1 && qraw.ptr) return fail(SAGE_ENOTIMPL, "interleaved Q scales need the standalone Q quantiser (sage_quant_int8)");
  if (kgroups > 1 && blkk == 16) return fail(SAGE_ENOTIMPL, "interleaved K scales need blocks of 32, 64 or 128 keys");
  if (B == 0 || Hq == 0 || Sq == 0) return SAGE_OK;
  if (!out || (Skv > 0 && (!k || !v_panels || !k_scale))) return fail(SAGE_EINVAL, "null tensor pointer");
  if (!qraw.ptr && (!q || !q_scale)) return fail(SAGE_EINVAL, "null tensor pointer");
  if (qraw.ptr && mask.ptr) return fail(SAGE_ENOTIMPL, "fused Q quantisation: not with an explicit mask");
  if (pv_mode == SAGE_PV_FP8 && !v_scale) return fail(SAGE_EINVAL, "fp8 P.V needs v_scale");
  if (int rc = check_stride16("q", q_sb, q_sh, q_sn, qraw.ptr ? 2 : 1, qraw.ptr ? qraw.ptr : q)) return rc;
  if (int rc = check_stride16("k", k_sb, k_sh, k_sn, 1, k)) return rc;
  if (int rc = check_stride16("out", o_sb, o_sh, o_sn, 2, out)) return rc;   // rows are stored 16 bytes per lane
  // tile loads address a row of one (batch, head) slice with 32-bit byte offsets
  if ((int64_t)Skv * k_sn >= 0x7fffffff || (qraw.ptr && (int64_t)Sq * q_sn * 2 >= 0x7fffffff))
    return fail(SAGE_ENOTIMPL, "a (batch, head) slice of q or k spans 2 GiB or more");
  const bool packed = cu_seqlens_q != nullptr;
  if (mask.ptr) {
    if (mask.kind != SAGE_MASK_BOOL && mask.kind != SAGE_MASK_ADDITIVE) return fail(SAGE_EINVAL, "mask kind %d unknown", mask.kind);
    if (packed) return fail(SAGE_ENOTIMPL, "an explicit mask is not supported for packed batches");
    if (is_causal) return fail(SAGE_ENOTIMPL, "an explicit mask cannot be combined with is_causal");
    if (mask.kind == SAGE_MASK_ADDITIVE && reinterpret_cast<uintptr_t>(mask.ptr) % 4) return fail(SAGE_EINVAL, "additive mask must be 4-byte aligned");
  }
  if (packed && (!cu_seqlens_k || !plan)) return fail(SAGE_EINVAL, "packed mode needs cu_seqlens_k and plan");
  if (packed && B > 32767) return fail(SAGE_EINVAL, "too many sequences");
  AttnConfig cfg = attn_config(D, pv_mode, packed);
  const int BM = cfg.nw * 32;
  AttnArgs a;
  memset(&a, 0, sizeof(a));
  a.q = q; a.k = k; a.vp = (const uint8_t*)v_panels; a.qs = q_scale; a.ks = k_scale; a.vs = v_scale;
  a.out = out; a.lse = lse;
  a.B = B; a.Hq = Hq; a.Hkv = Hkv; a.Sq = Sq; a.Skv = Skv;
  a.q_sb = q_sb; a.q_sh = q_sh; a.q_sn = q_sn; a.k_sb = k_sb; a.k_sh = k_sh; a.k_sn = k_sn;
  a.o_sb = o_sb; a.o_sh = o_sh; a.o_sn = o_sn;
  a.blkq = blkq; a.blkk = blkk; a.blkq_shift = ilog2(blkq); a.blkk_shift = ilog2(blkk); a.qg_shift = qgroups == 8 ? 3 : 0; a.k_interleave = kgroups == 4;
  a.out_bf16 = out_dtype == SAGE_DT_BF16;
  a.nqt = (Sq + BM - 1) / BM;
  a.mask = mask.ptr; a.mask_kind = mask.kind; a.m_sb = mask.sb; a.m_sh = mask.sh; a.m_sm = mask.sm; a.m_sn = mask.sn;
  a.mask_mult = mask.mult; a.lse_offset = lse_offset;
  a.q_raw = qraw.ptr; a.q_is_bf16 = qraw.dtype == SAGE_DT_BF16; a.q_mult = qraw.mult;
  int64_t grid;
  if (packed) {
    SagePlanLayout L = plan_layout(B, total_q);
    a.cu_q = cu_seqlens_q; a.cu_k = cu_seqlens_k;
    a.cu_qblk = plan + L.cu_qblk; a.cu_kblk = plan + L.cu_kblk; a.cu_panel = plan + L.cu_panel;
    a.ntiles = plan + L.ntiles; a.tiles = plan + L.tiles;
    a.qs_sh = q_scale_sh; a.ks_sh = k_scale_sh; a.panel_sh = panel_sh; a.total_q = total_q;
    grid = ((int64_t)total_q / BM + B) * Hq;  // upper bound on tiles; surplus workgroups exit at once
  } else {
    grid = (int64_t)a.nqt * B * Hq;
  }
  if (grid > 0x7fffffff) return fail(SAGE_EINVAL, "too many tiles for one launch");
  finish_attn_args(a, is_causal != 0);
  hipError_t e = launch_attn(a, D, pv_mode, is_causal != 0, (int)grid, (hipStream_t)stream);
  if (e != hipSuccess) return hip_fail(e, "sage_attn_fwd");
  return SAGE_OK;
}
}  // namespace

extern "C" {

int sage_attn_fwd(const int8_t* q, const int8_t* k, const void* v_panels, const float* q_scale, const float* k_scale,
                  const float* v_scale, void* out, float* lse, int B, int Hq, int Hkv, int Sq, int Skv, int D, int64_t q_sb,
                  int64_t q_sh, int64_t q_sn, int64_t k_sb, int64_t k_sh, int64_t k_sn, int64_t o_sb, int64_t o_sh,
                  int64_t o_sn, int blkq, int blkk, int is_causal, int pv_mode, int out_dtype, const int32_t* cu_seqlens_q,
                  const int32_t* cu_seqlens_k, const int32_t* plan, int total_q, int64_t q_scale_sh, int64_t k_scale_sh,
                  int64_t panel_sh, sage_stream_t stream) {
  return attn_impl(q, k, v_panels, q_scale, k_scale, v_scale, out, lse, B, Hq, Hkv, Sq, Skv, D, q_sb, q_sh, q_sn, k_sb, k_sh, k_sn, o_sb, o_sh, o_sn, blkq, blkk, is_causal, pv_mode, out_dtype, cu_seqlens_q, cu_seqlens_k, plan, total_q, q_scale_sh, k_scale_sh, panel_sh, MaskArg(), nullptr, QRawArg(), stream);
}

int sage_attn_fwd_qfused(const void* q, int q_dtype, double sm_scale, const int8_t* k, const void* v_panels,
                         const float* k_scale, const float* v_scale, void* out, float* lse, int B, int Hq, int Hkv, int Sq,
                         int Skv, int D, int64_t q_sb, int64_t q_sh, int64_t q_sn, int64_t k_sb, int64_t k_sh, int64_t k_sn,
                         int64_t o_sb, int64_t o_sh, int64_t o_sn, int blkq, int blkk, int is_causal, int pv_mode,
                         int out_dtype, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, const int32_t* plan,
                         int total_q, int64_t k_scale_sh, int64_t panel_sh, sage_stream_t stream) {
  if (q_dtype != SAGE_DT_F16 && q_dtype != SAGE_DT_BF16) return fail(SAGE_ETYPE, "q dtype flag %d is not fp16(0)/bf16(1)", q_dtype);
  if (!q) return fail(SAGE_EINVAL, "null tensor pointer");
  QRawArg qr;
  qr.ptr = q; qr.dtype = q_dtype; qr.mult = (float)((sm_scale > 0 ? sm_scale : 1.0 / sqrt((double)D)) * 1.44269504);
  return attn_impl(nullptr, k, v_panels, nullptr, k_scale, v_scale, out, lse, B, Hq, Hkv, Sq, Skv, D, q_sb, q_sh, q_sn, k_sb,
                   k_sh, k_sn, o_sb, o_sh, o_sn, blkq, blkk, is_causal, pv_mode, out_dtype, cu_seqlens_q, cu_seqlens_k, plan,
                   total_q, 0, k_scale_sh, panel_sh, MaskArg(), nullptr, qr, stream);
}

int sage_attn_fwd_masked(const int8_t* q, const int8_t* k, const void* v_panels, const float* q_scale, const float* k_scale,
                         const float* v_scale, void* out, float* lse, int B, int Hq, int Hkv, int Sq, int Skv, int D,
                         int64_t q_sb, int64_t q_sh, int64_t q_sn, int64_t k_sb, int64_t k_sh, int64_t k_sn, int64_t o_sb,
                         int64_t o_sh, int64_t o_sn, int blkq, int blkk, int pv_mode, int out_dtype, const void* attn_mask,
                         int mask_kind, int64_t m_sb, int64_t m_sh, int64_t m_sm, int64_t m_sn, sage_stream_t stream) {
  if (!attn_mask) return fail(SAGE_EINVAL, "null mask");
  MaskArg m;
  m.ptr = attn_mask; m.kind = mask_kind; m.sb = m_sb; m.sh = m_sh; m.sm = m_sm; m.sn = m_sn;
  return attn_impl(q, k, v_panels, q_scale, k_scale, v_scale, out, lse, B, Hq, Hkv, Sq, Skv, D, q_sb, q_sh, q_sn, k_sb, k_sh,
                   k_sn, o_sb, o_sh, o_sn, blkq, blkk, 0, pv_mode, out_dtype, nullptr, nullptr, nullptr, 0, 0, 0, 0, m, nullptr,
                   QRawArg(), stream);
}

// ---- one-call pipeline --------------------------------------------------------------------
namespace {
// Up to this many keys per sequence and elements of K per call the pre-passes run as one launch whose workgroups read
// their sequence's statistics themselves (sage_quant.hip: prepass_small_kernel).
constexpr int kSmallPrepassRows = 1024;
constexpr int64_t kSmallPrepassElements = (int64_t)4 << 20;
// ... and the element reads it makes: every K tile and every V panel re-reads its whole sequence, elements of K times
// (K tiles + V panels per sequence).  Measured end to end against the six launches: 8 M reads (1 x 8 heads of 1024 rows,
// head_dim 64, K blocks of 128) 30.0 against 31.2 us; 38 M (the same with K blocks of 16) 33.9 / 33.2; 100 M (1 x 32 heads
// of 1024 rows, head_dim 128, K blocks of 64) 70 / 81; 302 M (the same with K blocks of 16) 68.7 / 54.2, and 8 x 8 heads of
// 1024 rows at head_dim 64 with K blocks of 16, also 302 M, 88.9 / 50.1.
constexpr int64_t kSmallPrepassReads = (int64_t)128 << 20;
struct E2EWorkspace {
  size_t q_i8, k_i8, q_scale, k_scale, km, v_scale, panels, stat, plan, lse_off, total;
  int64_t qs_sh, ks_sh, panel_sh;
};
// What a call needs beyond K, V and their statistics: the INT8 copy of Q with its scales (only when Q is quantised by the
// stand-alone pass: an explicit mask, the LSE correction of K smoothing, interleaved Q scales) and the per-row LSE
// correction term (only when LSE is returned from smoothed keys).
bool needs_q_pass(int blkq, int has_mask, int want_lse, int smooth_k) {
  return has_mask || (want_lse && smooth_k) || blk_groups(blkq) != 1;
}
E2EWorkspace e2e_layout(int B, int Hq, int Hkv, int Sq, int Skv, int D, int blkq, int blkk, int pv, int total_q, int total_k,
                        int varlen, bool q_pass, bool lse_offset) {
  E2EWorkspace w;
  size_t off = 0;
  size_t nq = varlen ? (size_t)total_q * Hq * D : (size_t)B * Hq * Sq * D;
  size_t nk = varlen ? (size_t)total_k * Hkv * D : (size_t)B * Hkv * Skv * D;
  w.q_i8 = off; off += q_pass ? align_up(nq) : 0;
  w.k_i8 = off; off += align_up(nk);
  if (varlen) {
    w.qs_sh = total_q / blk_rows(blkq) + B; w.ks_sh = total_k / blk_rows(blkk) + B; w.panel_sh = total_k / SAGE_PANEL_ROWS + B;
    w.q_scale = off; off += q_pass ? align_up((size_t)Hq * w.qs_sh * 4) : 0;
    w.k_scale = off; off += align_up((size_t)Hkv * w.ks_sh * 4);
  } else {
    w.qs_sh = w.ks_sh = w.panel_sh = 0;
    w.q_scale = off; off += q_pass ? align_up((size_t)B * Hq * ((Sq + blk_rows(blkq) - 1) / blk_rows(blkq)) * blk_groups(blkq) * 4) : 0;
    w.k_scale = off; off += align_up((size_t)B * Hkv * ((Skv + blk_rows(blkk) - 1) / blk_rows(blkk)) * (blk_groups(blkk) ? blk_groups(blkk) : 1) * 4);
  }
  w.km = off; off += align_up((size_t)B * Hkv * D * 2);
  w.v_scale = off; off += align_up((size_t)B * Hkv * D * 4);
  size_t pbytes = varlen ? (size_t)Hkv * w.panel_sh * SAGE_PANEL_ROWS * D * (pv ? 1 : 2) : sage_v_panel_bytes(B, Hkv, Skv, D, pv);
  w.panels = off; off += align_up(pbytes);
  size_t stat = sage_k_mean_workspace_bytes(B, Hkv, Skv, D);
  size_t stat2 = sage_prep_v_workspace_bytes(B, Hkv, Skv, D, pv);
  w.stat = off; off += align_up(stat > stat2 ? stat : stat2);
  w.plan = off; off += varlen ? align_up(sage_varlen_plan_ints(B, total_q) * 4) : 0;
  w.lse_off = off; off += lse_offset ? align_up((varlen ? (size_t)Hq * total_q : (size_t)B * Hq * Sq) * 4) : 0;
  w.total = off;
  return w;
}
}  // namespace

size_t sage_sageattn_workspace_bytes(int B, int Hq, int Hkv, int Sq, int Skv, int D, int blkq, int blkk, int pv_mode,
                                     int total_q, int total_k, int varlen) {
  if (blkq <= 0 || blkk <= 0) return 0;
  return e2e_layout(B, Hq, Hkv, Sq, Skv, D, blkq, blkk, pv_mode, total_q, total_k, varlen, true, true).total;
}

size_t sage_sageattn_workspace_bytes_for(int B, int Hq, int Hkv, int Sq, int Skv, int D, int blkq, int blkk, int pv_mode,
                                         int total_q, int total_k, int varlen, int smooth_k, int want_lse, int has_mask) {
  if (blkq <= 0 || blkk <= 0) return 0;
  return e2e_layout(B, Hq, Hkv, Sq, Skv, D, blkq, blkk, pv_mode, total_q, total_k, varlen,
                    needs_q_pass(blkq, has_mask, want_lse, smooth_k), want_lse && smooth_k).total;
}

int sage_sageattn(const void* q, const void* k, const void* v, void* out, float* lse, void* workspace, size_t workspace_bytes,
                  int B, int Hq, int Hkv, int Sq, int Skv, int D, int64_t q_sb, int64_t q_sh, int64_t q_sn, int64_t k_sb,
                  int64_t k_sh, int64_t k_sn, int64_t v_sb, int64_t v_sh, int64_t v_sn, int64_t o_sb, int64_t o_sh,
                  int64_t o_sn, int dtype, int blkq, int blkk, double sm_scale, int is_causal, int smooth_k, int pv_mode,
                  const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, int total_q, int total_k, sage_stream_t stream) {
  return sage_sageattn_masked(q, k, v, out, lse, workspace, workspace_bytes, B, Hq, Hkv, Sq, Skv, D, q_sb, q_sh, q_sn, k_sb,
                              k_sh, k_sn, v_sb, v_sh, v_sn, o_sb, o_sh, o_sn, dtype, blkq, blkk, sm_scale, is_causal, smooth_k,
                              pv_mode, cu_seqlens_q, cu_seqlens_k, total_q, total_k, nullptr, 0, 0, 0, 0, 0, stream);
}

int sage_sageattn_masked(const void* q, const void* k, const void* v, void* out, float* lse, void* workspace,
                         size_t workspace_bytes, int B, int Hq, int Hkv, int Sq, int Skv, int D, int64_t q_sb, int64_t q_sh,
                         int64_t q_sn, int64_t k_sb, int64_t k_sh, int64_t k_sn, int64_t v_sb, int64_t v_sh, int64_t v_sn,
                         int64_t o_sb, int64_t o_sh, int64_t o_sn, int dtype, int blkq, int blkk, double sm_scale,
                         int is_causal, int smooth_k, int pv_mode, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                         int total_q, int total_k, const void* attn_mask, int mask_kind, int64_t m_sb, int64_t m_sh,
                         int64_t m_sm, int64_t m_sn, sage_stream_t stream) {
  if (int rc = check_common(B, Hq, Sq, D, dtype)) return rc;
  if (Hkv <= 0 || Hq % Hkv) return fail(SAGE_EINVAL, "query heads (%d) must be divisible by KV heads (%d)", Hq, Hkv);
  if (!valid_blk_attn(blk_rows(blkq)) || !valid_blkk_attn(blk_rows(blkk)))
    return fail(SAGE_ENOTIMPL, "Q and K scale blocks must be 16, 32, 64 or 128 rows (got %d/%d)", blk_rows(blkq), blk_rows(blkk));
  if ((blk_groups(blkq) != 1 && blk_groups(blkq) != 8) || (blk_groups(blkk) != 1 && blk_groups(blkk) != 4))
    return fail(SAGE_ENOTIMPL, "Q scale blocks take SAGE_BLK_INTERLEAVE8, K scale blocks SAGE_BLK_INTERLEAVE4");
  if (blk_groups(blkk) == 4 && blk_rows(blkk) == 16)
    return fail(SAGE_ENOTIMPL, "interleaved K scales need blocks of 32, 64 or 128 keys");
  if (pv_mode != SAGE_PV_FP16 && pv_mode != SAGE_PV_FP8) return fail(SAGE_EINVAL, "pv_mode %d unknown", pv_mode);
  const int varlen = cu_seqlens_q != nullptr;
  if (varlen && (blk_groups(blkq) > 1 || blk_groups(blkk) > 1)) return fail(SAGE_ENOTIMPL, "interleaved scales are not supported for packed batches");
  if (varlen && !cu_seqlens_k) return fail(SAGE_EINVAL, "packed mode needs cu_seqlens_k");
  if (B == 0 || Hq == 0 || Sq == 0) return SAGE_OK;
  if (!workspace) return fail(SAGE_EWORKSPACE, "null workspace");
  // (the workspace is laid out for what THIS call uses; sage_sageattn_workspace_bytes is the upper bound over all calls
  // of the shape, sage_sageattn_workspace_bytes_for the size for one kind of call)
  const bool q_pass = needs_q_pass(blkq, attn_mask != nullptr, lse != nullptr, smooth_k && !(!varlen && Skv == 0));
  E2EWorkspace w = e2e_layout(B, Hq, Hkv, Sq, Skv, D, blkq, blkk, pv_mode, total_q, total_k, varlen, q_pass,
                              lse != nullptr && smooth_k && !(!varlen && Skv == 0));
  if (workspace_bytes < w.total) return fail(SAGE_EWORKSPACE, "workspace too small: %zu < %zu", workspace_bytes, w.total);
  if (reinterpret_cast<uintptr_t>(workspace) % 256) return fail(SAGE_EINVAL, "workspace must be 256-byte aligned");
  uint8_t* ws = (uint8_t*)workspace;
  int8_t* q_i8 = (int8_t*)(ws + w.q_i8);
  int8_t* k_i8 = (int8_t*)(ws + w.k_i8);
  float* q_scale = (float*)(ws + w.q_scale);
  float* k_scale = (float*)(ws + w.k_scale);
  void* km = ws + w.km;
  float* v_scale = (float*)(ws + w.v_scale);
  void* panels = ws + w.panels;
  void* stat = ws + w.stat;
  int32_t* plan = varlen ? (int32_t*)(ws + w.plan) : nullptr;
  const size_t stat_bytes = w.plan - w.stat;
  // The int8 copies of q and k are the library's own tensors: they get dense strides of their own ([B,H,L,D] with
  // whole rows contiguous, or packed [T,H,D]), whatever strides the caller's q and k have (views of a fused QKV
  // buffer, sliced heads, ...), so that they always fit the workspace regions sized for B*H*L*D bytes.
  const int64_t qi_sb = varlen ? 0 : (int64_t)Hq * Sq * D, qi_sh = varlen ? D : (int64_t)Sq * D, qi_sn = varlen ? (int64_t)Hq * D : D;
  const int64_t ki_sb = varlen ? 0 : (int64_t)Hkv * Skv * D, ki_sh = varlen ? D : (int64_t)Skv * D, ki_sn = varlen ? (int64_t)Hkv * D : D;
  const int32_t *cu_qblk = nullptr, *cu_kblk = nullptr, *cu_panel = nullptr;
  if (varlen) {
    int rc = sage_varlen_plan(cu_seqlens_q, cu_seqlens_k, B, total_q, blkq, blkk, is_causal, plan,
                              sage_varlen_plan_ints(B, total_q), stream);
    if (rc) return rc;
    SagePlanLayout L = plan_layout(B, total_q);
    cu_qblk = plan + L.cu_qblk; cu_kblk = plan + L.cu_kblk; cu_panel = plan + L.cu_panel;
  }
  int rc = SAGE_OK;
  // No keys at all (fixed-length mode): nothing to smooth, quantise or lay out; the attention kernel writes zeros
  // and LSE = -inf without reading K, V or their scales.
  const bool no_keys = !varlen && Skv == 0;
  if (no_keys) smooth_k = 0;
  // Short sequences: all K and V pre-passes in one launch (every workgroup computes the statistic its tile needs over
  // the whole sequence itself); otherwise six launches, the statistics in two stages.
  const int64_t k_elements = (int64_t)B * Hkv * Skv * D;
  const int64_t rereads = (Skv + blk_rows(blkk) - 1) / blk_rows(blkk) + (Skv + kPanelRows - 1) / kPanelRows;
  const bool small_prepass = !varlen && !no_keys && Skv <= kSmallPrepassRows && k_elements <= kSmallPrepassElements &&
                             k_elements * rereads <= kSmallPrepassReads;
  if (small_prepass) {
    if (int rc2 = check_stride16("k", k_sb, k_sh, k_sn, 2, k)) return rc2;
    if (int rc2 = check_stride16("v", v_sb, v_sh, v_sn, 2, v)) return rc2;
    const int kb = blk_rows(blkk);
    QuantArgs qa;
    memset(&qa, 0, sizeof(qa));
    qa.x = (const u16*)k; qa.out = k_i8; qa.scale = k_scale; qa.km = nullptr;
    qa.B = B; qa.H = Hkv; qa.L = Skv; qa.D = D;
    qa.x_sb = k_sb; qa.x_sh = k_sh; qa.x_sn = k_sn; qa.o_sb = ki_sb; qa.o_sh = ki_sh; qa.o_sn = ki_sn;
    qa.blk = kb; qa.groups = blk_groups(blkk); qa.mult = 1.0f; qa.dv_group = 1;
    PrepVArgs va;
    memset(&va, 0, sizeof(va));
    va.v = (const u16*)v; va.panels = (uint8_t*)panels; va.vscale = v_scale; va.B = B; va.H = Hkv; va.L = Skv; va.D = D;
    va.v_sb = v_sb; va.v_sh = v_sh; va.v_sn = v_sn;
    hipError_t e = launch_prepass_small(qa, va, dtype, pv_mode == SAGE_PV_FP8, (Skv + kb - 1) / kb,
                                        (Skv + SAGE_PANEL_ROWS - 1) / SAGE_PANEL_ROWS, smooth_k != 0, km, v_scale,
                                        (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "sage_sageattn(pre-pass)");
  } else {
    if (smooth_k) {
      rc = sage_k_mean(k, km, stat, stat_bytes, B, Hkv, Skv, D, k_sb, k_sh, k_sn, dtype, cu_seqlens_k, stream);
      if (rc) return rc;
    }
    if (!no_keys) rc = sage_quant_int8(k, k_i8, k_scale, smooth_k ? km : nullptr, B, Hkv, Skv, D, k_sb, k_sh, k_sn, ki_sb, ki_sh, ki_sn,
                         (int64_t)Hkv * D, D, blkk, 1.0f, dtype, cu_seqlens_k, cu_kblk, w.ks_sh, stream);
    if (rc) return rc;
  }
  // With K smoothing every logit of a query row loses q . k_mean; the softmax does not notice but the
  // log-sum-exp does, so when LSE is requested the Q quantiser also emits that dot product (in the
  // base-2 units of the scaled Q) and the attention kernel adds it back.
  RowDot dot;
  float* lse_off = nullptr;
  if (lse && smooth_k) {
    lse_off = (float*)(ws + w.lse_off);
    dot.vec = km; dot.out = lse_off; dot.sb = (int64_t)Hkv * D; dot.sh = D; dot.group = Hq / Hkv; dot.total = total_q;
  }
  // Q is quantised by the attention kernel itself (each q-tile exactly where it is consumed) unless a
  // feature needs the standalone pass: an explicit mask or the LSE correction.
  const float q_mult = (float)((sm_scale > 0 ? sm_scale : 1.0 / sqrt((double)D)) * 1.44269504);
  const bool fuse_q = !attn_mask && !lse_off && blk_groups(blkq) == 1;   // (interleaved scales: standalone pass too)
  if (!fuse_q) {
    rc = quant_impl(q, q_i8, q_scale, nullptr, B, Hq, Sq, D, q_sb, q_sh, q_sn, qi_sb, qi_sh, qi_sn, 0, 0, blkq, q_mult, dtype,
                    cu_seqlens_q, cu_qblk, w.qs_sh, dot, stream);
    if (rc) return rc;
  }
  if (!no_keys && !small_prepass) {
    rc = sage_prep_v(v, panels, v_scale, stat, stat_bytes, B, Hkv, Skv, D, v_sb, v_sh, v_sn, dtype, pv_mode, cu_seqlens_k,
                     cu_panel, w.panel_sh, stream);
    if (rc) return rc;
  }
  QRawArg qr;
  if (fuse_q) { qr.ptr = q; qr.dtype = dtype; qr.mult = q_mult; }
  MaskArg m;
  if (attn_mask) {
    // sageattn's additive mask is in natural-log units on top of sm_scale * q.k (test_sage_attention_mate.py:171-176)
    m.ptr = attn_mask; m.kind = mask_kind; m.sb = m_sb; m.sh = m_sh; m.sm = m_sm; m.sn = m_sn; m.mult = 1.44269504f;
  }
  // the attention kernel reads either the caller's floating-point q (its strides) or the int8 copy (dense strides)
  return attn_impl(q_i8, k_i8, panels, q_scale, k_scale, pv_mode == SAGE_PV_FP8 ? v_scale : nullptr, out, lse, B, Hq, Hkv, Sq,
                   Skv, D, fuse_q ? q_sb : qi_sb, fuse_q ? q_sh : qi_sh, fuse_q ? q_sn : qi_sn, ki_sb, ki_sh, ki_sn, o_sb, o_sh,
                   o_sn, blkq, blkk, is_causal, pv_mode, dtype, cu_seqlens_q, cu_seqlens_k, plan, total_q, w.qs_sh, w.ks_sh,
                   w.panel_sh, m, lse_off, qr, stream);
}

}  // extern "C"
