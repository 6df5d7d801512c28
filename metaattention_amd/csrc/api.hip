// C ABI entry points (see include/metaattention_hip.h): argument validation,
// error strings, kernel selection.  No allocation, no synchronisation.
#include "../../include/metaattention_hip.h"
#include "attn_fwd.h"
#include "attn_bwd.h"
#include "linear_fwd.h"
#include "linear_bwd.h"
#include "mla_decode.h"

#include <atomic>
#include <cstdarg>
#include <cstdio>

namespace {
thread_local char g_err[512] = "";
int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}
}  // namespace

extern "C" {

int ma_version(void) { return MA_VERSION; }
const char* ma_last_error(void) { return g_err; }

// Strides beyond this many elements cannot belong to a tensor in device memory; bounding them keeps the kernels' 64-bit
// address arithmetic (index x stride x element size) from wrapping.
static constexpr int64_t kMaxStride = (int64_t)1 << 40;

// The kernels count work items (batch x heads x blocks of rows, kv splits included) and rows in 32-bit integers.
static bool attn_sizes_too_large(int B, int H, int Sq, int Skv) {
  const int S = Sq > Skv ? Sq : Skv;
  if (S > (1 << 24) || (int64_t)B * H > 0x7fffffff) return true;      // (step by step: the full product does not fit 64 bits for every input)
  return (int64_t)B * H * ((S + 31) / 32) * 2 > 0x7fffffff;
}

static int attn_splits(const ma_attn_params* p) {
  return ma::attn_decode_splits(p->family, p->mask == MA_MASK_CAUSAL, p->batch, p->heads, p->seqlen_q, p->seqlen_kv, p->dim_qk, p->dim_v);
}

// partial outputs [B, splits, H, Sq, Dv] in the tensor dtype, then their fp32 row scales [B, splits, H, Sq]
size_t ma_attn_workspace_bytes(const ma_attn_params* p) {
  if (!p || p->batch <= 0 || p->heads <= 0 || p->seqlen_q <= 0 || p->seqlen_kv <= 0 || p->dim_v <= 0 || p->dim_v > 65536 ||
      attn_sizes_too_large(p->batch, p->heads, p->seqlen_q, p->seqlen_kv))
    return 0;
  const int n = attn_splits(p);
  if (n <= 1) return 0;
  const size_t rows = (size_t)p->batch * n * p->heads * p->seqlen_q;
  return rows * p->dim_v * 2 + rows * sizeof(float);
}

int ma_attn_fwd(const ma_attn_params* p, ma_stream_t stream) {
  if (!p) return fail(MA_ERR_INVALID_ARG, "ma_attn_fwd: params is NULL");
  if (!p->q || !p->k || !p->v || !p->o) return fail(MA_ERR_INVALID_ARG, "ma_attn_fwd: q/k/v/o must be non-NULL");
  if (p->batch <= 0 || p->heads <= 0 || p->seqlen_q <= 0 || p->seqlen_kv <= 0 || p->dim_qk <= 0 || p->dim_v <= 0)
    return fail(MA_ERR_INVALID_ARG, "ma_attn_fwd: sizes must be positive (B=%d H=%d Sq=%d Skv=%d Dqk=%d Dv=%d)", p->batch,
                p->heads, p->seqlen_q, p->seqlen_kv, p->dim_qk, p->dim_v);
  if (attn_sizes_too_large(p->batch, p->heads, p->seqlen_q, p->seqlen_kv))
    return fail(MA_ERR_UNSUPPORTED, "ma_attn_fwd: sizes beyond the kernels' 32-bit work indices (B=%d H=%d Sq=%d Skv=%d)", p->batch, p->heads,
                p->seqlen_q, p->seqlen_kv);
  if (p->dtype != MA_BF16 && p->dtype != MA_FP16) return fail(MA_ERR_INVALID_ARG, "ma_attn_fwd: dtype %d", p->dtype);
  if (p->mask != MA_MASK_NONE && p->mask != MA_MASK_CAUSAL) return fail(MA_ERR_INVALID_ARG, "ma_attn_fwd: mask kind %d", p->mask);
  if (p->family < MA_ATTN_SOFTMAX || p->family > MA_ATTN_RETENTION)
    return fail(MA_ERR_INVALID_ARG, "ma_attn_fwd: family %d", p->family);
  if (!(p->scale > 0.f)) return fail(MA_ERR_INVALID_ARG, "ma_attn_fwd: scale must be > 0 (got %g)", (double)p->scale);
  if (p->mask == MA_MASK_CAUSAL && p->seqlen_q != p->seqlen_kv)
    return fail(MA_ERR_UNSUPPORTED, "ma_attn_fwd: causal mask needs seqlen_q == seqlen_kv (%d vs %d)", p->seqlen_q, p->seqlen_kv);
  if (p->heads_kv < 0 || (p->heads_kv > 0 && p->heads % p->heads_kv != 0))
    return fail(MA_ERR_INVALID_ARG, "ma_attn_fwd: heads (%d) must be a multiple of heads_kv (%d)", p->heads, p->heads_kv);
  if (p->kv_block_mask && (p->kv_block_size < 32 || p->kv_block_size % 32 != 0))
    return fail(MA_ERR_UNSUPPORTED, "ma_attn_fwd: kv_block_size must be a positive multiple of 32 (got %d)", p->kv_block_size);
  // (a block mask with a row per 128 queries goes with either mask: the block-sparse prefill operator)
  if ((p->kv_seqlens || (p->kv_block_mask && !p->kbm_per_query_head)) && p->mask == MA_MASK_CAUSAL)
    return fail(MA_ERR_UNSUPPORTED, "ma_attn_fwd: kv_seqlens / a kv_block_mask per kv head are for the unmasked (decode) operators");
  if (p->elem_mask) {
    if (p->mask == MA_MASK_CAUSAL || p->family == MA_ATTN_RETENTION)
      return fail(MA_ERR_UNSUPPORTED, "ma_attn_fwd: elem_mask goes with MA_MASK_NONE and the softmax / sigmoid / relu families");
    if ((uintptr_t)p->elem_mask % 4 != 0 || p->em_stride_q % 4 != 0 || p->em_stride_h % 4 != 0 || p->em_stride_b % 4 != 0)
      return fail(MA_ERR_UNSUPPORTED, "ma_attn_fwd: elem_mask rows must be 4-byte aligned");
  }
  if (p->decay_gamma && (p->family != MA_ATTN_RETENTION || p->score_mask || p->mask != MA_MASK_CAUSAL || p->dim_qk != 256 || p->dim_v != 512))
    return fail(MA_ERR_UNSUPPORTED, "ma_attn_fwd: decay_gamma replaces score_mask in the RETENTION family at Dqk 256 / Dv 512 under MA_MASK_CAUSAL");
  if (p->family == MA_ATTN_RETENTION && !p->decay_gamma) {
    if (!p->score_mask) return fail(MA_ERR_INVALID_ARG, "ma_attn_fwd: RETENTION needs score_mask (or decay_gamma)");
    if ((uintptr_t)p->score_mask % 8 != 0 || p->sm_stride_b % 4 != 0 || p->sm_stride_h % 4 != 0 || p->sm_stride_q % 4 != 0)
      return fail(MA_ERR_UNSUPPORTED, "ma_attn_fwd: score_mask must be 8-byte aligned with strides that are multiples of 4 elements");
  }
  const int64_t strides[] = {p->q_stride_s, p->q_stride_h, p->k_stride_s, p->k_stride_h, p->v_stride_s, p->v_stride_h,
                             p->o_stride_s, p->o_stride_h, p->q_stride_b, p->k_stride_b, p->v_stride_b, p->o_stride_b};
  for (int64_t s : strides)
    if (s % 8 != 0 || s > kMaxStride || s < -kMaxStride)
      return fail(MA_ERR_UNSUPPORTED, "ma_attn_fwd: strides must be multiples of 8 elements (16-byte rows) below 2^40");
  const uintptr_t ptrs[] = {(uintptr_t)p->q, (uintptr_t)p->k, (uintptr_t)p->v, (uintptr_t)p->o};
  for (uintptr_t x : ptrs)
    if (x % 16 != 0) return fail(MA_ERR_UNSUPPORTED, "ma_attn_fwd: q/k/v/o must be 16-byte aligned");

  const int64_t aux[] = {p->sm_stride_b, p->sm_stride_h, p->sm_stride_q, p->kbm_stride_b, p->kbm_stride_h, p->kbm_stride_q,
                         p->em_stride_b, p->em_stride_h, p->em_stride_q, p->sa_stride_b, p->sa_stride_h, p->sa_stride_q, p->sa_stride_kv};
  for (int64_t s : aux)
    if (s > kMaxStride || s < -kMaxStride) return fail(MA_ERR_UNSUPPORTED, "ma_attn_fwd: mask / score_add strides must stay below 2^40");

  ma::AttnArgs a{};
  a.q = p->q; a.k = p->k; a.v = p->v; a.o = p->o;
  a.row_scale = p->row_scale; a.bias_ptr = p->bias_ptr; a.smask = p->score_mask;
  a.qsb = p->q_stride_b; a.qss = p->q_stride_s; a.qsh = p->q_stride_h;
  a.ksb = p->k_stride_b; a.kss = p->k_stride_s; a.ksh = p->k_stride_h;
  a.vsb = p->v_stride_b; a.vss = p->v_stride_s; a.vsh = p->v_stride_h;
  a.osb = p->o_stride_b; a.oss = p->o_stride_s; a.osh = p->o_stride_h;
  a.msb = p->sm_stride_b; a.msh = p->sm_stride_h; a.msq = p->sm_stride_q;
  a.B = p->batch; a.H = p->heads; a.Sq = p->seqlen_q; a.Skv = p->seqlen_kv;
  a.kv_group = p->heads_kv > 0 ? p->heads / p->heads_kv : 1;
  a.kv_lens = p->kv_seqlens;
  a.kv_block_mask = p->kv_block_mask; a.kbm_sb = p->kbm_stride_b; a.kbm_sh = p->kbm_stride_h;
  a.kv_block = p->kv_block_size;
  a.kbm_sq = p->kbm_stride_q; a.kbm_by_query_head = p->kbm_per_query_head;
  a.elem_mask = p->elem_mask; a.em_sb = p->em_stride_b; a.em_sh = p->em_stride_h; a.em_sq = p->em_stride_q;
  a.n_split = 1;
  if (p->workspace && ((uintptr_t)p->workspace % 16) == 0) {
    const int n = attn_splits(p);
    if (n > 1 && p->workspace_bytes >= ma_attn_workspace_bytes(p)) {
      const size_t rows = (size_t)p->batch * n * p->heads * p->seqlen_q;
      a.n_split = n;
      a.o_part = p->workspace;
      a.lse_part = (float*)((char*)p->workspace + rows * p->dim_v * 2);
    }
  }
  a.scale = p->scale; a.bias = p->bias;
  a.decay_gamma = p->decay_gamma;
  if (p->score_add || p->pos_slope_q || p->pos_slope_kv || p->softcap != 0.f) {
    if (p->family == MA_ATTN_RETENTION)
      return fail(MA_ERR_UNSUPPORTED, "ma_attn_fwd: score_add / pos_slope / softcap go with the softmax / sigmoid / relu families");
    if (p->softcap < 0.f || (p->softcap > 0.f && p->family != MA_ATTN_SOFTMAX))
      return fail(MA_ERR_UNSUPPORTED, "ma_attn_fwd: softcap must be >= 0 and goes with the softmax family");
    if (p->score_add && (uintptr_t)p->score_add % (p->score_add_fp32 ? 4 : 2) != 0)
      return fail(MA_ERR_UNSUPPORTED, "ma_attn_fwd: score_add must be aligned to its element size");
    a.add = p->score_add; a.add_sb = p->sa_stride_b; a.add_sh = p->sa_stride_h; a.add_sq = p->sa_stride_q; a.add_sk = p->sa_stride_kv;
    a.add_f32 = p->score_add_fp32 != 0;
    a.slope_q = p->pos_slope_q; a.slope_kv = p->pos_slope_kv;
    a.softcap = p->softcap;
  }
  const int rc = ma::attn_fwd_dispatch(a, p->family, p->mask == MA_MASK_CAUSAL, p->dtype == MA_BF16, p->dim_qk, p->dim_v,
                                       (hipStream_t)stream);
  if (rc == -2)
    return fail(MA_ERR_UNSUPPORTED, "ma_attn_fwd: no kernel for family %d, Dqk=%d, Dv=%d", p->family, p->dim_qk, p->dim_v);
  if (rc != 0) return fail(MA_ERR_LAUNCH, "ma_attn_fwd: launch failed: %s", hipGetErrorString(ma::t_hip_error));
  return MA_OK;
}

size_t ma_attn_bwd_workspace_bytes(const ma_attn_bwd_params* p) {
  if (!p || p->batch <= 0 || p->heads <= 0 || p->seqlen_q <= 0 || p->family != MA_ATTN_SOFTMAX ||
      attn_sizes_too_large(p->batch, p->heads, p->seqlen_q, p->seqlen_q))
    return 0;
  return (size_t)p->batch * p->heads * p->seqlen_q * sizeof(float);
}

int ma_attn_bwd(const ma_attn_bwd_params* p, ma_stream_t stream) {
  if (!p) return fail(MA_ERR_INVALID_ARG, "ma_attn_bwd: params is NULL");
  if (!p->q || !p->k || !p->v || !p->dout || !p->dq || !p->dk || !p->dv)
    return fail(MA_ERR_INVALID_ARG, "ma_attn_bwd: q/k/v/dout/dq/dk/dv must be non-NULL");
  if (p->batch <= 0 || p->heads <= 0 || p->seqlen_q <= 0 || p->seqlen_kv <= 0 || p->dim_qk <= 0 || p->dim_v <= 0)
    return fail(MA_ERR_INVALID_ARG, "ma_attn_bwd: sizes must be positive");
  if (attn_sizes_too_large(p->batch, p->heads, p->seqlen_q, p->seqlen_kv))
    return fail(MA_ERR_UNSUPPORTED, "ma_attn_bwd: sizes beyond the kernels' 32-bit work indices (B=%d H=%d Sq=%d Skv=%d)", p->batch, p->heads,
                p->seqlen_q, p->seqlen_kv);
  if (p->dtype != MA_BF16 && p->dtype != MA_FP16) return fail(MA_ERR_INVALID_ARG, "ma_attn_bwd: dtype %d", p->dtype);
  if (p->mask != MA_MASK_NONE && p->mask != MA_MASK_CAUSAL) return fail(MA_ERR_INVALID_ARG, "ma_attn_bwd: mask kind %d", p->mask);
  if (p->family != MA_ATTN_SOFTMAX && p->family != MA_ATTN_SIGMOID && p->family != MA_ATTN_RELU && p->family != MA_ATTN_RETENTION)
    return fail(MA_ERR_UNSUPPORTED, "ma_attn_bwd: family %d has no backward kernel", p->family);
  if (p->family == MA_ATTN_RETENTION) {
    if (!p->lse || !p->score_mask || !p->score_mask_t)
      return fail(MA_ERR_INVALID_ARG, "ma_attn_bwd: RETENTION needs the forward's row scale (lse), score_mask and score_mask_t");
    if (p->elem_mask || p->kv_block_mask) return fail(MA_ERR_UNSUPPORTED, "ma_attn_bwd: RETENTION takes no element-wise or block masks");
    const int64_t ms[] = {(int64_t)(uintptr_t)p->score_mask / 2, p->sm_stride_b, p->sm_stride_h, p->sm_stride_q,
                          (int64_t)(uintptr_t)p->score_mask_t / 2, p->smt_stride_b, p->smt_stride_h, p->smt_stride_k};
    for (int64_t x : ms)
      if (x % 4 != 0) return fail(MA_ERR_UNSUPPORTED, "ma_attn_bwd: score_mask rows must be 8-byte aligned");
  }
  if (!(p->scale > 0.f)) return fail(MA_ERR_INVALID_ARG, "ma_attn_bwd: scale must be > 0 (got %g)", (double)p->scale);
  if (p->mask == MA_MASK_CAUSAL && p->seqlen_q != p->seqlen_kv)
    return fail(MA_ERR_UNSUPPORTED, "ma_attn_bwd: causal mask needs seqlen_q == seqlen_kv (%d vs %d)", p->seqlen_q, p->seqlen_kv);
  const int hkv = p->heads_kv > 0 ? p->heads_kv : p->heads;
  if (p->heads_kv < 0 || p->heads % hkv != 0)
    return fail(MA_ERR_INVALID_ARG, "ma_attn_bwd: heads (%d) must be a multiple of heads_kv (%d)", p->heads, p->heads_kv);
  if (p->family == MA_ATTN_SOFTMAX) {
    if (!p->o || !p->lse) return fail(MA_ERR_INVALID_ARG, "ma_attn_bwd: SOFTMAX needs o and lse of the forward pass");
    if (!p->workspace || p->workspace_bytes < ma_attn_bwd_workspace_bytes(p) || (uintptr_t)p->workspace % 4 != 0)
      return fail(MA_ERR_WORKSPACE, "ma_attn_bwd: workspace of %zu bytes needed", ma_attn_bwd_workspace_bytes(p));
  }
  const int64_t strides[] = {p->q_stride_b, p->q_stride_s, p->q_stride_h, p->k_stride_b, p->k_stride_s, p->k_stride_h,
                             p->v_stride_b, p->v_stride_s, p->v_stride_h, p->o_stride_b, p->o_stride_s, p->o_stride_h,
                             p->do_stride_b, p->do_stride_s, p->do_stride_h, p->dq_stride_b, p->dq_stride_s, p->dq_stride_h,
                             p->dk_stride_b, p->dk_stride_s, p->dk_stride_h, p->dv_stride_b, p->dv_stride_s, p->dv_stride_h};
  for (int64_t s : strides)
    if (s % 8 != 0 || s > kMaxStride || s < -kMaxStride)
      return fail(MA_ERR_UNSUPPORTED, "ma_attn_bwd: strides must be multiples of 8 elements (16-byte rows) below 2^40");
  const int64_t aux[] = {p->em_stride_b, p->em_stride_h, p->em_stride_q, p->emt_stride_b, p->emt_stride_h, p->emt_stride_k,
                         p->kbm_stride_b, p->kbm_stride_h, p->kbm_stride_q, p->qbm_stride_b, p->qbm_stride_h, p->qbm_stride_k,
                         p->sm_stride_b, p->sm_stride_h, p->sm_stride_q, p->smt_stride_b, p->smt_stride_h, p->smt_stride_k,
                         p->sa_stride_b, p->sa_stride_h, p->sa_stride_q, p->sa_stride_kv};
  for (int64_t s : aux)
    if (s > kMaxStride || s < -kMaxStride) return fail(MA_ERR_UNSUPPORTED, "ma_attn_bwd: mask / score_add strides must stay below 2^40");
  const uintptr_t ptrs[] = {(uintptr_t)p->q, (uintptr_t)p->k, (uintptr_t)p->v, (uintptr_t)p->o, (uintptr_t)p->dout,
                            (uintptr_t)p->dq, (uintptr_t)p->dk, (uintptr_t)p->dv};
  for (uintptr_t x : ptrs)
    if (x % 16 != 0) return fail(MA_ERR_UNSUPPORTED, "ma_attn_bwd: tensors must be 16-byte aligned");
  if (p->elem_mask || p->elem_mask_t) {
    if (!p->elem_mask || !p->elem_mask_t) return fail(MA_ERR_INVALID_ARG, "ma_attn_bwd: elem_mask and elem_mask_t go together");
    if (p->mask == MA_MASK_CAUSAL) return fail(MA_ERR_UNSUPPORTED, "ma_attn_bwd: elem_mask goes with MA_MASK_NONE");
    const int64_t ms[] = {(int64_t)(uintptr_t)p->elem_mask, p->em_stride_b, p->em_stride_h, p->em_stride_q,
                          (int64_t)(uintptr_t)p->elem_mask_t, p->emt_stride_b, p->emt_stride_h, p->emt_stride_k};
    for (int64_t x : ms)
      if (x % 4 != 0) return fail(MA_ERR_UNSUPPORTED, "ma_attn_bwd: elem_mask rows must be 4-byte aligned");
  }
  if (p->score_add || p->pos_slope_q || p->pos_slope_kv || p->softcap != 0.f) {
    if (p->family == MA_ATTN_RETENTION)
      return fail(MA_ERR_UNSUPPORTED, "ma_attn_bwd: score_add / pos_slope / softcap do not go with the retention family");
    if (p->softcap != 0.f && p->family != MA_ATTN_SOFTMAX)
      return fail(MA_ERR_UNSUPPORTED, "ma_attn_bwd: softcap goes with the softmax family only (as in ma_attn_fwd)");
    if (p->softcap < 0.f) return fail(MA_ERR_UNSUPPORTED, "ma_attn_bwd: softcap must be >= 0");
    if (p->score_add && (uintptr_t)p->score_add % (p->score_add_fp32 ? 4 : 2) != 0)
      return fail(MA_ERR_UNSUPPORTED, "ma_attn_bwd: score_add must be aligned to its element size");
  }
  if ((p->kv_block_mask != nullptr) != (p->q_block_mask != nullptr))
    return fail(MA_ERR_INVALID_ARG, "ma_attn_bwd: kv_block_mask and q_block_mask go together");
  if (p->kv_block_mask && !p->elem_mask)
    return fail(MA_ERR_UNSUPPORTED, "ma_attn_bwd: block masks come with an element-wise mask");

  ma::AttnBwdArgs a{};
  a.q = p->q; a.k = p->k; a.v = p->v; a.o = p->o; a.dout = p->dout; a.dq = p->dq; a.dk = p->dk; a.dv = p->dv;
  a.lse = p->lse; a.delta = (float*)p->workspace; a.bias_ptr = p->bias_ptr;
  a.qsb = p->q_stride_b; a.qss = p->q_stride_s; a.qsh = p->q_stride_h;
  a.ksb = p->k_stride_b; a.kss = p->k_stride_s; a.ksh = p->k_stride_h;
  a.vsb = p->v_stride_b; a.vss = p->v_stride_s; a.vsh = p->v_stride_h;
  a.osb = p->o_stride_b; a.oss = p->o_stride_s; a.osh = p->o_stride_h;
  a.dosb = p->do_stride_b; a.doss = p->do_stride_s; a.dosh = p->do_stride_h;
  a.dqsb = p->dq_stride_b; a.dqss = p->dq_stride_s; a.dqsh = p->dq_stride_h;
  a.dksb = p->dk_stride_b; a.dkss = p->dk_stride_s; a.dksh = p->dk_stride_h;
  a.dvsb = p->dv_stride_b; a.dvss = p->dv_stride_s; a.dvsh = p->dv_stride_h;
  a.B = p->batch; a.H = p->heads; a.Hkv = hkv; a.Sq = p->seqlen_q; a.Skv = p->seqlen_kv;
  a.kv_group = p->heads / hkv;
  a.add = p->score_add; a.add_sb = p->sa_stride_b; a.add_sh = p->sa_stride_h; a.add_sq = p->sa_stride_q; a.add_sk = p->sa_stride_kv;
  a.add_f32 = p->score_add_fp32 != 0;
  a.slope_q = p->pos_slope_q; a.slope_kv = p->pos_slope_kv;
  a.softcap = p->softcap;
  a.scale = p->scale; a.bias = p->bias;
  a.elem_mask = p->elem_mask; a.em_sb = p->em_stride_b; a.em_sh = p->em_stride_h; a.em_sq = p->em_stride_q;
  a.elem_mask_t = p->elem_mask_t; a.emt_sb = p->emt_stride_b; a.emt_sh = p->emt_stride_h; a.emt_sk = p->emt_stride_k;
  a.kv_block_mask = p->kv_block_mask; a.kbm_sb = p->kbm_stride_b; a.kbm_sh = p->kbm_stride_h; a.kbm_sq = p->kbm_stride_q;
  a.q_block_mask = p->q_block_mask; a.qbm_sb = p->qbm_stride_b; a.qbm_sh = p->qbm_stride_h; a.qbm_sk = p->qbm_stride_k;
  a.smask = p->score_mask; a.sm_sb = p->sm_stride_b; a.sm_sh = p->sm_stride_h; a.sm_sq = p->sm_stride_q;
  a.smask_t = p->score_mask_t; a.smt_sb = p->smt_stride_b; a.smt_sh = p->smt_stride_h; a.smt_sk = p->smt_stride_k;
  const int rc = ma::attn_bwd_dispatch(a, p->family, p->mask == MA_MASK_CAUSAL, p->dtype == MA_BF16, p->dim_qk, p->dim_v, (hipStream_t)stream);
  if (rc == -2) return fail(MA_ERR_UNSUPPORTED, "ma_attn_bwd: no kernel for family %d, Dqk=%d, Dv=%d", p->family, p->dim_qk, p->dim_v);
  if (rc != 0) return fail(MA_ERR_LAUNCH, "ma_attn_bwd: launch failed: %s", hipGetErrorString(ma::t_hip_error));
  return MA_OK;
}

static int check_linear(const ma_linear_params* p, const char* who) {
  if (!p) return fail(MA_ERR_INVALID_ARG, "%s: params is NULL", who);
  if (p->batch <= 0 || p->heads <= 0 || p->heads_q <= 0 || p->heads_k <= 0 || p->seqlen <= 0 || p->dim_k <= 0 || p->dim_v <= 0)
    return fail(MA_ERR_INVALID_ARG, "%s: sizes must be positive", who);
  if (p->dtype != MA_BF16) return fail(MA_ERR_UNSUPPORTED, "%s: only bf16 (the reference's linear kernels are bf16 only)", who);
  if (p->heads % p->heads_q != 0 || p->heads % p->heads_k != 0)
    return fail(MA_ERR_INVALID_ARG, "%s: heads (%d) must be a multiple of heads_q (%d) and heads_k (%d)", who, p->heads, p->heads_q, p->heads_k);
  if (p->segments < 0) return fail(MA_ERR_INVALID_ARG, "%s: segments must be >= 0", who);
  if (p->seqlen > (1 << 30)) return fail(MA_ERR_UNSUPPORTED, "%s: seqlen beyond 2^30", who);
  if (p->dim_k > 65536 || p->dim_v > 65536) return fail(MA_ERR_UNSUPPORTED, "%s: no kernel for dim_k=%d / dim_v=%d", who, p->dim_k, p->dim_v);
  const int64_t bh = (int64_t)p->batch * p->heads;     // (compared step by step: the full product does not fit 64 bits for every input)
  if (bh > 0x7fffffff || bh * ((p->dim_v + 63) / 64) > 0x7fffffff || bh * ((p->dim_v + 63) / 64) * (p->segments > 8 ? p->segments : 8) > 0x7fffffff)
    return fail(MA_ERR_UNSUPPORTED, "%s: grid too large", who);
  return MA_OK;
}

static ma::LinArgs linear_args(const ma_linear_params* p) {
  ma::LinArgs a{};
  a.q = p->q; a.k = p->k; a.v = p->v; a.o = p->o; a.log_decay = p->log_decay; a.v_scale = p->v_scale;
  a.q_scale = p->q_scale;
  a.out_f32 = p->out_fp32 != 0 ? 1 : 0;
  a.B = p->batch; a.H = p->heads; a.Hq = p->heads_q; a.Hk = p->heads_k; a.T = p->seqlen; a.Dv = p->dim_v;
  // a key width of 64 or 192 runs in the 128- / 256-wide kernel: the operands' rows are read as they are (general operand
  // addressing) and the rest of the contraction is zeros that are neither loaded nor multiplied
  if (p->dim_k == 64 || p->dim_k == 192) { a.q_row = a.k_row = p->dim_k; a.qk_cols = p->dim_k; }
  return a;
}
// the key width of the kernel that takes dim_k
static int linear_kernel_dk(int dim_k) { return dim_k == 64 ? 128 : dim_k == 192 ? 256 : dim_k; }

// The state of one sequence stays on chip; a workspace is only used when the sequence is cut into
// segments that run side by side (few batch x heads): it then holds the segments' fp32 end states.
// Without it (or with segments = 1) the forward pass runs as a single pass.  Returns 0 for
// arguments ma_linear_fwd would refuse and when no device is present.
size_t ma_linear_workspace_bytes(const ma_linear_params* p) {
  if (check_linear(p, "ma_linear_workspace_bytes") != MA_OK) return 0;
  size_t bytes = 0;
  if (ma::linear_fwd_dispatch(linear_args(p), linear_kernel_dk(p->dim_k), p->segments, nullptr, 0, nullptr, &bytes) != 0) return 0;
  return bytes;
}

int ma_linear_fwd(const ma_linear_params* p, ma_stream_t stream) {
  if (const int rc0 = check_linear(p, "ma_linear_fwd")) return rc0;
  if (!p->q || !p->k || !p->v || !p->o || !p->log_decay)
    return fail(MA_ERR_INVALID_ARG, "ma_linear_fwd: q/k/v/o/log_decay must be non-NULL");
  const uintptr_t ptrs[] = {(uintptr_t)p->q, (uintptr_t)p->k, (uintptr_t)p->v, (uintptr_t)p->o};
  for (uintptr_t x : ptrs)
    if (x % 16 != 0) return fail(MA_ERR_UNSUPPORTED, "ma_linear_fwd: q/k/v/o must be 16-byte aligned");
  const ma::LinArgs a = linear_args(p);
  const int rc = ma::linear_fwd_dispatch(a, linear_kernel_dk(p->dim_k), p->segments, p->workspace, p->workspace_bytes, (hipStream_t)stream, nullptr);
  if (rc == -2)
    return fail(MA_ERR_UNSUPPORTED, "ma_linear_fwd: no kernel for dim_k=%d (64, 128, 192 or 256) / dim_v=%d (multiple of 64)", p->dim_k, p->dim_v);
  if (rc != 0) return fail(MA_ERR_LAUNCH, "ma_linear_fwd: launch failed: %s", hipGetErrorString(ma::t_hip_error));
  return MA_OK;
}

static int check_linear_bwd(const ma_linear_bwd_params* p, const char* who) {
  if (!p) return fail(MA_ERR_INVALID_ARG, "%s: params is NULL", who);
  if (p->batch <= 0 || p->heads <= 0 || p->heads_q <= 0 || p->heads_k <= 0 || p->seqlen <= 0 || p->dim_k <= 0 || p->dim_v <= 0)
    return fail(MA_ERR_INVALID_ARG, "%s: sizes must be positive", who);
  if (p->dtype != MA_BF16) return fail(MA_ERR_UNSUPPORTED, "%s: only bf16 (the reference's linear kernels are bf16 only)", who);
  if (p->heads % p->heads_q != 0 || p->heads % p->heads_k != 0)
    return fail(MA_ERR_INVALID_ARG, "%s: heads (%d) must be a multiple of heads_q (%d) and heads_k (%d)", who, p->heads, p->heads_q, p->heads_k);
  if ((p->dim_k != 64 && p->dim_k != 128 && p->dim_k != 192 && p->dim_k != 256) || p->dim_v % 64 != 0 || p->dim_v > 4096)
    return fail(MA_ERR_UNSUPPORTED, "%s: dim_k=%d must be 64, 128, 192 or 256 and dim_v=%d a multiple of 64 (at most 4096)", who, p->dim_k, p->dim_v);
  const int64_t bh = (int64_t)p->batch * p->heads;     // (compared step by step: the full product does not fit 64 bits for every input)
  if (bh > 0x7fffffff || p->seqlen > (1 << 30) || bh * p->seqlen > (0x7fffffffll * 2048) / (p->dim_k > p->dim_v ? p->dim_k : p->dim_v))
    return fail(MA_ERR_UNSUPPORTED, "%s: grid too large", who);
  return MA_OK;
}

static ma::LinBwdArgs linear_bwd_args(const ma_linear_bwd_params* p) {
  ma::LinBwdArgs a{};
  a.q = p->q; a.k = p->k; a.v = p->v; a.dout = p->dout; a.log_decay = p->log_decay; a.v_scale = p->v_scale;
  a.dq = p->dq; a.dk = p->dk; a.dv = p->dv; a.dlog_decay = p->dlog_decay; a.dv_scale = p->v_scale ? p->dv_scale : nullptr;
  a.q_scale = p->q_scale;
  a.B = p->batch; a.H = p->heads; a.Hq = p->heads_q; a.Hk = p->heads_k; a.T = p->seqlen; a.Dk = p->dim_k; a.Dv = p->dim_v;
  return a;
}

// Returns 0 for arguments ma_linear_bwd would refuse.
size_t ma_linear_bwd_workspace_bytes(const ma_linear_bwd_params* p) {
  if (check_linear_bwd(p, "ma_linear_bwd_workspace_bytes") != MA_OK) return 0;
  size_t bytes = 0;
  if (ma::linear_bwd_run(linear_bwd_args(p), nullptr, 0, nullptr, &bytes) != 0) return 0;
  return bytes;
}

int ma_linear_bwd(const ma_linear_bwd_params* p, ma_stream_t stream) {
  if (const int rc0 = check_linear_bwd(p, "ma_linear_bwd")) return rc0;
  if (!p->q || !p->k || !p->v || !p->dout || !p->log_decay || !p->dq || !p->dk || !p->dv || !p->dlog_decay)
    return fail(MA_ERR_INVALID_ARG, "ma_linear_bwd: q/k/v/dout/log_decay/dq/dk/dv/dlog_decay must be non-NULL");
  const uintptr_t ptrs[] = {(uintptr_t)p->q, (uintptr_t)p->k, (uintptr_t)p->v, (uintptr_t)p->dout, (uintptr_t)p->dq, (uintptr_t)p->dk, (uintptr_t)p->dv};
  for (uintptr_t x : ptrs)
    if (x % 16 != 0) return fail(MA_ERR_UNSUPPORTED, "ma_linear_bwd: q/k/v/dout/dq/dk/dv must be 16-byte aligned");
  const int rc = ma::linear_bwd_run(linear_bwd_args(p), p->workspace, p->workspace_bytes, (hipStream_t)stream, nullptr);
  if (rc == -3)
    return fail(MA_ERR_WORKSPACE, "ma_linear_bwd: workspace missing, smaller than ma_linear_bwd_workspace_bytes (%zu) or not 256-byte aligned",
                ma_linear_bwd_workspace_bytes(p));
  if (rc == -2) return fail(MA_ERR_UNSUPPORTED, "ma_linear_bwd: no kernel for dim_k=%d / dim_v=%d", p->dim_k, p->dim_v);
  if (rc != 0) return fail(MA_ERR_LAUNCH, "ma_linear_bwd: launch failed: %s", hipGetErrorString(ma::t_hip_error));
  return MA_OK;
}

// Split count: enough workgroups to fill the device's CUs once (256 assumed where no device can be asked), each split a
// whole number of 64-row tiles, and never more splits than tiles.
int ma_mla_choose_split(const ma_mla_params* p) {
  if (!p || p->batch <= 0 || p->heads_q <= 0 || p->seqlen_kv <= 0) return 1;
  const int head_blocks = (int)(((int64_t)p->heads_q + 127) / 128);
  const int tiles = (int)(((int64_t)p->seqlen_kv + 63) / 64);
  int cus = ma::device_cus();
  if (cus <= 0) cus = 256;
  const int64_t groups = (int64_t)p->batch * head_blocks;
  int split = groups >= cus ? 1 : (int)(cus / groups);
  if (split > tiles) split = tiles;
  if (split > 64) split = 64;
  return split;
}

static int mla_split_of(const ma_mla_params* p) { return p->num_split > 0 ? p->num_split : ma_mla_choose_split(p); }

// One workgroup serves 128 heads and owns a CU: the plan has as many parts as CUs per block of heads
// (flash_api.cpp:39 with this library's block of heads).
int ma_mla_num_sm_parts(int heads_q) {
  if (heads_q <= 0) return 0;
  int cus = ma::device_cus();
  if (cus <= 0) cus = 256;
  const int64_t parts = cus / (((int64_t)heads_q + 127) / 128);
  return parts < 1 ? 1 : (int)parts;
}

int ma_mla_get_metadata(const int32_t* kv_seqlens, int batch, int num_sm_parts, int32_t* tile_scheduler_metadata, int32_t* num_splits,
                        ma_stream_t stream) {
  if (!kv_seqlens || !tile_scheduler_metadata || !num_splits) return fail(MA_ERR_INVALID_ARG, "ma_mla_get_metadata: NULL argument");
  if (batch <= 0 || num_sm_parts <= 0) return fail(MA_ERR_INVALID_ARG, "ma_mla_get_metadata: batch and num_sm_parts must be positive");
  // blocks of 64 tokens and 5 blocks of fixed cost per batch entry, as kernels/config.h:6,11
  if (ma::mla_plan_dispatch(kv_seqlens, batch, num_sm_parts, 64, 5, tile_scheduler_metadata, num_splits, (hipStream_t)stream) != 0)
    return fail(MA_ERR_LAUNCH, "ma_mla_get_metadata: launch failed: %s", hipGetErrorString(ma::t_hip_error));
  return MA_OK;
}

size_t ma_mla_workspace_bytes(const ma_mla_params* p) {
  if (!p || p->batch <= 0 || p->batch > 65535 || p->heads_q <= 0 || p->seqlen_kv <= 0 || p->dim <= 0 || p->dim > 65536 || p->num_sm_parts < 0 ||
      (int64_t)p->batch * p->heads_q > 0x7fffffff)
    return 0;
  const size_t per_slot = (size_t)p->heads_q * ((size_t)p->dim * 2 + sizeof(float));   // 2-byte partial outputs + fp32 lse
  if (p->tile_scheduler_metadata) return ((size_t)p->batch + (size_t)p->num_sm_parts) * per_slot;   // at most one piece more per part
  const int ns = mla_split_of(p);
  if (ns <= 1) return 0;
  return (size_t)p->batch * ns * per_slot;
}

int ma_mla_decode(const ma_mla_params* p, ma_stream_t stream) {
  if (!p) return fail(MA_ERR_INVALID_ARG, "ma_mla_decode: params is NULL");
  if (!p->q || !p->q_pe || !p->kv || !p->k_pe || !p->o) return fail(MA_ERR_INVALID_ARG, "ma_mla_decode: q/q_pe/kv/k_pe/o must be non-NULL");
  if (p->batch <= 0 || p->heads_q <= 0 || p->seqlen_kv <= 0)
    return fail(MA_ERR_INVALID_ARG, "ma_mla_decode: sizes must be positive (B=%d Hq=%d Skv=%d)", p->batch, p->heads_q, p->seqlen_kv);
  if (p->dtype != MA_BF16 && p->dtype != MA_FP16) return fail(MA_ERR_INVALID_ARG, "ma_mla_decode: dtype %d", p->dtype);
  if (!(p->scale > 0.f)) return fail(MA_ERR_INVALID_ARG, "ma_mla_decode: scale must be > 0");
  if (p->batch > 65535) return fail(MA_ERR_UNSUPPORTED, "ma_mla_decode: batch > 65535");
  if (p->seqlen_kv > (1 << 30)) return fail(MA_ERR_UNSUPPORTED, "ma_mla_decode: seqlen_kv beyond 2^30");
  const int64_t strides[] = {p->q_stride_b, p->q_stride_h, p->qpe_stride_b, p->qpe_stride_h, p->kv_stride_b, p->kv_stride_s,
                             p->kpe_stride_b, p->kpe_stride_s, p->o_stride_b, p->o_stride_h};
  for (int64_t s : strides)
    if (s % 8 != 0 || s > kMaxStride || s < -kMaxStride) return fail(MA_ERR_UNSUPPORTED, "ma_mla_decode: strides must be multiples of 8 elements below 2^40");
  const uintptr_t ptrs[] = {(uintptr_t)p->q, (uintptr_t)p->q_pe, (uintptr_t)p->kv, (uintptr_t)p->k_pe, (uintptr_t)p->o};
  for (uintptr_t x : ptrs)
    if (x % 16 != 0) return fail(MA_ERR_UNSUPPORTED, "ma_mla_decode: tensors must be 16-byte aligned");
  const bool planned = p->tile_scheduler_metadata != nullptr;
  if (planned) {
    if (!p->num_splits || !p->kv_seqlens || p->num_sm_parts <= 0)
      return fail(MA_ERR_INVALID_ARG, "ma_mla_decode: a work plan needs num_splits, kv_seqlens and num_sm_parts > 0");
    // (a batch entry is cut into at most one piece per part, and the combine kernel merges at most 64)
    if (p->num_sm_parts > 65535) return fail(MA_ERR_UNSUPPORTED, "ma_mla_decode: num_sm_parts > 65535");
  }
  const int ns = planned ? 1 : mla_split_of(p);
  const int tiles = (p->seqlen_kv + 63) / 64;
  if (ns > tiles || ns > 64) return fail(MA_ERR_INVALID_ARG, "ma_mla_decode: num_split %d exceeds min(kv tiles=%d, 64)", ns, tiles);
  if ((int64_t)p->batch * p->heads_q > 0x7fffffff || (int64_t)p->batch * ((p->heads_q + 127) / 128) * ns > 0x7fffffff || (planned && (int64_t)p->num_sm_parts * ((p->heads_q + 127) / 128) > 0x7fffffff))
    return fail(MA_ERR_UNSUPPORTED, "ma_mla_decode: grid too large (batch %d x heads_q %d)", p->batch, p->heads_q);
  ma::MlaArgs a{};
  a.q = p->q; a.q_pe = p->q_pe; a.kv = p->kv; a.k_pe = p->k_pe; a.o = p->o; a.lse = p->lse;
  a.qsb = p->q_stride_b; a.qsh = p->q_stride_h; a.qpsb = p->qpe_stride_b; a.qpsh = p->qpe_stride_h;
  a.kvsb = p->kv_stride_b; a.kvss = p->kv_stride_s; a.kpsb = p->kpe_stride_b; a.kpss = p->kpe_stride_s;
  a.osb = p->o_stride_b; a.osh = p->o_stride_h;
  a.B = p->batch; a.Hq = p->heads_q; a.Skv = p->seqlen_kv; a.scale = p->scale;
  a.num_split = ns;
  a.split_len = ((tiles + ns - 1) / ns) * 64;
  a.kv_lens = p->kv_seqlens;
  if (p->block_table) {
    if (p->page_size < 32 || p->page_size % 32 != 0)
      return fail(MA_ERR_UNSUPPORTED, "ma_mla_decode: page_size must be a positive multiple of 32 (got %d)", p->page_size);
    if (p->block_table_stride < 0 || p->block_table_stride > 0x7fffffff)
      return fail(MA_ERR_INVALID_ARG, "ma_mla_decode: block_table_stride %lld", (long long)p->block_table_stride);
    if ((int64_t)p->block_table_stride * p->page_size < p->seqlen_kv)
      return fail(MA_ERR_INVALID_ARG, "ma_mla_decode: block table rows of %lld pages do not cover seqlen_kv=%d", (long long)p->block_table_stride, p->seqlen_kv);
    a.block_table = p->block_table; a.bt_stride = p->block_table_stride; a.page_size = p->page_size;
    a.kvsb = 0; a.kpsb = 0;
  }
  if (planned) {
    const size_t need = ma_mla_workspace_bytes(p);
    if (!p->workspace || p->workspace_bytes < need)
      return fail(MA_ERR_WORKSPACE, "ma_mla_decode: workspace of %zu bytes needed for the work plan, got %zu", need, p->workspace_bytes);
    if ((uintptr_t)p->workspace % 16 != 0) return fail(MA_ERR_WORKSPACE, "ma_mla_decode: workspace must be 16-byte aligned");
    a.plan_meta = p->tile_scheduler_metadata; a.plan_splits = p->num_splits; a.plan_parts = p->num_sm_parts;
    a.o_part = p->workspace;
    a.lse_part = (float*)((char*)p->workspace + ((size_t)p->batch + (size_t)p->num_sm_parts) * p->heads_q * p->dim * 2);
  } else if (ns > 1) {
    const size_t need = ma_mla_workspace_bytes(p);
    if (!p->workspace || p->workspace_bytes < need)
      return fail(MA_ERR_WORKSPACE, "ma_mla_decode: workspace of %zu bytes needed for %d splits, got %zu", need, ns, p->workspace_bytes);
    if ((uintptr_t)p->workspace % 16 != 0) return fail(MA_ERR_WORKSPACE, "ma_mla_decode: workspace must be 16-byte aligned");
    a.o_part = p->workspace;
    a.lse_part = (float*)((char*)p->workspace + (size_t)p->batch * ns * p->heads_q * p->dim * 2);
  }
  const int rc = ma::mla_decode_dispatch(a, p->dtype == MA_BF16, p->dim, p->dim_pe, (hipStream_t)stream);
  if (rc == -2) return fail(MA_ERR_UNSUPPORTED, "ma_mla_decode: only dim=512, dim_pe=64 is in the kernel library (got %d, %d)", p->dim, p->dim_pe);
  if (rc != 0) return fail(MA_ERR_LAUNCH, "ma_mla_decode: launch failed: %s", hipGetErrorString(ma::t_hip_error));
  return MA_OK;
}

// ---- ma_mla_decode_noalloc: ma_mla_decode with the library's own scratch array as the workspace ----
// The array lives in the code object's global segment: each GPU the library runs on holds its own copy, at its own
// address, until the process ends.  In host code the array's name is only a handle for hipGetSymbolAddress (passing it to
// a kernel would hand the kernel a host-side address): the device address is looked up once per device, with that
// device current, and everything else uses the looked-up pointer.
// Footprint: the 40 MiB belong to the library's code object, so EVERY process that loads the library holds them on every
// GPU it initialises, whether or not it ever calls the entry point (16 processes sharing one GPU: 640 MiB of it).
#define MA_MLA_SCRATCH_BYTES (40u << 20)
#define MA_MAX_DEVICES 64
static __device__ __align__(256) unsigned char scratch[MA_MLA_SCRATCH_BYTES];
static std::atomic<void*> g_scratch_ptr[MA_MAX_DEVICES];   // by device ordinal

static void* scratch_of_current_device() {
  const int dev = ma::current_device();
  if (dev < 0 || dev >= MA_MAX_DEVICES) return nullptr;   // (the caller has checked the ordinal)
  void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (ptr) return ptr;
  if (ma::hip_check(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch))) != 0 || !ptr) return nullptr;
  g_scratch_ptr[dev].store(ptr, std::memory_order_release);   // (threads that meet here store the same address)
  return ptr;
}

size_t ma_mla_noalloc_max_workspace(void) { return MA_MLA_SCRATCH_BYTES; }

int ma_mla_decode_noalloc(const ma_mla_params* p, ma_stream_t stream) {
  if (!p) return fail(MA_ERR_INVALID_ARG, "ma_mla_decode_noalloc: params is NULL");
  if (p->batch <= 0 || p->heads_q <= 0 || p->seqlen_kv <= 0)
    return fail(MA_ERR_INVALID_ARG, "ma_mla_decode_noalloc: sizes must be positive (B=%d Hq=%d Skv=%d)", p->batch, p->heads_q, p->seqlen_kv);
  if (p->tile_scheduler_metadata && p->num_sm_parts <= 0)
    return fail(MA_ERR_INVALID_ARG, "ma_mla_decode_noalloc: a work plan needs num_sm_parts > 0");
  const size_t need = ma_mla_workspace_bytes(p);
  if (need > MA_MLA_SCRATCH_BYTES)
    return fail(MA_ERR_WORKSPACE, "ma_mla_decode_noalloc: this call needs %zu bytes of scratch, the built-in array holds %u: use ma_mla_decode with a "
                "workspace of the caller's, or fewer splits", need, (unsigned)MA_MLA_SCRATCH_BYTES);
  ma_mla_params q = *p;
  q.workspace = nullptr;
  q.workspace_bytes = 0;
  if (need > 0) {
    const int dev = ma::current_device();
    if (dev < 0 || dev >= MA_MAX_DEVICES)
      return fail(MA_ERR_UNSUPPORTED, "ma_mla_decode_noalloc: device ordinal %d is outside the %d the scratch table covers: use ma_mla_decode "
                  "with a workspace of the caller's", dev, MA_MAX_DEVICES);
    void* s = scratch_of_current_device();
    if (!s) return fail(MA_ERR_LAUNCH, "ma_mla_decode_noalloc: no address for the scratch array: %s", hipGetErrorString(ma::t_hip_error));
    q.workspace = s;
    q.workspace_bytes = MA_MLA_SCRATCH_BYTES;
  }
  return ma_mla_decode(&q, stream);
}

}  // extern "C"
