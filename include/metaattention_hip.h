/*
 * C ABI of the MI355X (gfx950) attention kernel library (forward operators and their backward).
 *
 * This is the boundary the Python host side binds with ctypes.  Each entry
 * point replaces one compiled operator that the reference builds at run time
 * from a TileLang template; the reference interface it stands in for is cited
 * per function.  Conventions (all entry points):
 *   - plain pointers and sizes only; every pointer is a device pointer to
 *     memory the CALLER owns (inputs, outputs and workspace alike);
 *   - work is enqueued on the given hipStream_t and the call returns without
 *     synchronising; the library allocates nothing.  The only state it keeps is what a first call caches per
 *     device (raised LDS limits of its kernels, the number of CUs); concurrent first calls from several host
 *     threads are safe, and so are concurrent calls afterwards;
 *   - K and V (and the latent cache of the MLA operator) must be finite everywhere, also at positions a mask
 *     hides: the kernels multiply masked positions by probabilities that are exactly 0 (and the first step of
 *     a work item multiplies one resident V sub-tile of the same batch entry and head by zeros), and 0 x inf is
 *     not 0.  The reference's kernels share this for every position inside a visited tile;
 *   - return value 0 on success, a negative MA_ERR_* code otherwise, in which
 *     case ma_last_error() (thread local) describes the problem;
 *   - strides are in ELEMENTS of the tensor's dtype; the innermost (feature)
 *     dimension of every tensor must be contiguous;
 *   - tensors may be larger than 4 GiB (bases are 64-bit).  The kernels count work items and rows in 32 bits:
 *     sequence lengths up to 2^24 (2^30 for the chunked and the MLA operators), batch x heads x ceil(seqlen / 32)
 *     below 2^30, and whatever else a call's description names; sizes beyond that come back as MA_ERR_UNSUPPORTED.
 */
#ifndef METAATTENTION_HIP_H
#define METAATTENTION_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MA_VERSION 1

enum ma_status {
  MA_OK = 0,
  MA_ERR_INVALID_ARG = -1, /* null pointer, non-positive size, bad enum */
  MA_ERR_UNSUPPORTED = -2, /* shape/dtype/variant outside the kernel library */
  MA_ERR_WORKSPACE = -3,   /* workspace missing or too small */
  MA_ERR_LAUNCH = -4       /* HIP reported a launch error */
};

enum ma_dtype { MA_BF16 = 0, MA_FP16 = 1 };

/* Row function of the parallel family.  The reference expresses these as a
 * traced score_mod + OnlineFunc pair (attention_engine/attn_engine/attn_engine.py:16-105);
 * the library holds one hand-written variant per family:
 *   SOFTMAX   p = exp(s*scale + bias - rowmax) / rowsum, final row scale = lse   (examples/mha.py:21-71)
 *   SIGMOID   p = sigmoid(s*scale + bias), no row state                           (examples/sigmoid_attn.py:17-52)
 *   RELU      p = max(s*scale + bias, 0), no row state                            (examples/reluattn.py:15-42)
 *   RETENTION p = s*scale*mask / max(sum_j |s*scale*mask|, 1), final row scale = r (examples/retention_parallel.py:31-72)
 */
enum ma_attn_family { MA_ATTN_SOFTMAX = 0, MA_ATTN_SIGMOID = 1, MA_ATTN_RELU = 2, MA_ATTN_RETENTION = 3 };

/* Structural mask of the parallel family (attn_tl.py:129-151): NONE visits
 * every kv tile; CAUSAL keeps kv_idx <= q_idx, skips tiles above the diagonal
 * and (for SOFTMAX/SIGMOID/RELU) sets masked probabilities to exactly 0. */
enum ma_mask_kind { MA_MASK_NONE = 0, MA_MASK_CAUSAL = 1 };

typedef struct ma_attn_params {
  int32_t family; /* ma_attn_family */
  int32_t dtype;  /* ma_dtype of q, k, v, o and of score_mask */
  int32_t mask;   /* ma_mask_kind */
  int32_t batch, heads, seqlen_q, seqlen_kv, dim_qk, dim_v;   /* head sizes: as listed at ma_attn_bwd_params.family */
  /* q [B,Sq,H,Dqk], k [B,Skv,Hkv,Dqk], v [B,Skv,Hkv,Dv], o [B,Sq,H,Dv]; BSHD is the
   * layout the reference operator takes (attn_tl.py:69-70) but any strides
   * with a contiguous last dimension are accepted (sequence strides of k and v
   * non-negative and below 2^26 elements). */
  const void* q; int64_t q_stride_b, q_stride_s, q_stride_h;
  const void* k; int64_t k_stride_b, k_stride_s, k_stride_h;
  const void* v; int64_t v_stride_b, v_stride_s, v_stride_h;
  void* o;       int64_t o_stride_b, o_stride_s, o_stride_h;
  /* optional fp32 [B,H,Sq] final row scale (lse for SOFTMAX, r for
   * RETENTION; lower.py:386-393); may be NULL */
  float* row_scale;
  float scale; /* multiplies q.k^T */
  float bias;  /* added after scaling ... */
  const float* bias_ptr; /* ... plus *bias_ptr if not NULL (device fp32[1], sigmoid_attn.py:54-56) */
  /* RETENTION only: elementwise score multiplier [1 or B, H, Sq, Skv] in
   * `dtype` (retention_parallel.py:96-98); stride_b may be 0 */
  const void* score_mask; int64_t sm_stride_b, sm_stride_h, sm_stride_q;
  /* grouped-query attention (attn_gqa_tl.py:21-24, :80, :95): k and v have heads_kv heads and query
   * head h reads kv head h / (heads / heads_kv); 0 means heads_kv = heads */
  int32_t heads_kv;
  /* decode-style kv selection (blockattn_decode_varlen_tl.py:16, :57-75); both optional:
   * kv_seqlens int32 [B]: keys at or beyond kv_seqlens[b] do not exist for batch entry b;
   * kv_block_mask uint8/bool [B, heads_kv, ceil(Skv / kv_block_size)]: blocks of kv_block_size keys
   * (a multiple of 32) whose entry is 0 are skipped for that (batch, kv head).  A row left with no
   * key at all gets zeros (lse = -inf). */
  int32_t kv_block_size;
  const int32_t* kv_seqlens;
  const uint8_t* kv_block_mask; int64_t kbm_stride_b, kbm_stride_h;
  /* arbitrary masks (blockattn_tl.py:123-234, where the mask_mod's code is generated into the kernel): elem_mask
   * uint8/bool [1 or B, 1 or H, Sq, Skv] (strides in bytes = elements; stride 0 broadcasts; rows 4-byte aligned),
   * 0 = the score is masked (probability exactly 0).  Not with MA_MASK_CAUSAL (the element mask says it all) nor
   * RETENTION.  With or without it, kv_block_mask may be the prefill form
   * [1 or B, 1 or heads, ceil(Sq/128), ceil(Skv/kv_block_size)] of the block-sparse prefill operator: set
   * kbm_stride_q (blocks of 128 query rows; strides 0 broadcast) and kbm_per_query_head = 1.  This form also goes
   * with MA_MASK_CAUSAL.  Beside an elem_mask, a block entry of 2 says that the element mask keeps every score of the
   * block: it is then not read for it (1, or any other non-zero value: read). */
  const uint8_t* elem_mask; int64_t em_stride_b, em_stride_h, em_stride_q;
  int64_t kbm_stride_q; int32_t kbm_per_query_head;
  /* optional; with ma_attn_workspace_bytes(&params) bytes, decode shapes (at most 32 query rows, SOFTMAX, no
   * structural mask) run as split-KV + combine (attn_decode_tl.py:63-206); without it they run unsplit */
  void* workspace; size_t workspace_bytes;
  /* additive terms of the score function, for score_mods that add custom inputs to the score (the three custom-input
   * classes of core/lower/lower.py:561-615: tensors without a seq_len_kv axis such as [batch, heads, seq_len], tiles
   * [.., seq_len, seq_len_kv], and seq_len_kv vectors) or terms linear in the indices (ALiBi).  All optional, with the
   * SOFTMAX / SIGMOID / RELU families:
   *   x = s * scale + bias + score_add[b, h, q, kv] + pos_slope_q[h] * q + pos_slope_kv[h] * kv,
   * score_add fp32 (score_add_fp32 != 0) or `dtype`, addressed with ELEMENT strides, 0 for an axis the tensor does not
   * have; pos_slope_* fp32 [heads].  softcap > 0 (SOFTMAX only): x is replaced by softcap * tanh(x) before the row
   * function.  The backward kernels do not take these. */
  const void* score_add; int64_t sa_stride_b, sa_stride_h, sa_stride_q, sa_stride_kv; int32_t score_add_fp32;
  const float* pos_slope_q; const float* pos_slope_kv;
  float softcap;
  /* RETENTION at Dqk 256 / Dv 512 under MA_MASK_CAUSAL, instead of score_mask: fp32 [heads].  Says that the multiplier is
   * the geometric decay mask of RetNet, M[h, q, kv] = decay_gamma[h]^(q - kv) for kv <= q and 0 above the diagonal
   * (examples/retention_parallel.py:11-23 builds that tensor on the host); the kernel then generates it in fp32 instead
   * of reading a [1, H, Sq, Skv] tensor once per batch entry. */
  const float* decay_gamma;
} ma_attn_params;

/* Parallel attention backward for the SOFTMAX, SIGMOID, RELU and RETENTION families.  Replaces the backward of
 * _attention (tl_template/attn/attn_tl.py:669-692): delta pre-pass, dK/dV kernel with fp32 dQ atomics,
 * dQ post-pass.  Tensors and strides as in ma_attn_params; o and lse are the forward pass's output and
 * fp32 [B,H,Sq] row scale (SOFTMAX only; may be NULL otherwise), dout is the gradient of o; dq [B,Sq,H,Dqk],
 * dk [B,Skv,Hkv,Dqk], dv [B,Skv,Hkv,Dv] are written (not accumulated into), in `dtype`.  The workspace
 * (ma_attn_bwd_workspace_bytes: fp32 [B,H,Sq]) carries delta = sum_d dout*o between the two kernels.  Sequence
 * strides of q, k, v and dout must be non-negative and below 2^26 elements (MA_ERR_UNSUPPORTED otherwise). */
typedef struct ma_attn_bwd_params {
  int32_t family; /* ma_attn_family: SOFTMAX, SIGMOID, RELU or RETENTION; head sizes (dim_qk / dim_v) 128/128, 64/64, 128/256,
                   * 256/256 and 256/512 for every family, 192/128 (DeepSeek-V2-Lite, testing/benchmark_mi250.py:40-46) for
                   * SOFTMAX, SIGMOID and RELU; others MA_ERR_UNSUPPORTED */
  int32_t dtype;
  int32_t mask;   /* ma_mask_kind */
  int32_t batch, heads, heads_kv /* 0 = heads */, seqlen_q, seqlen_kv, dim_qk, dim_v;
  const void* q;    int64_t q_stride_b, q_stride_s, q_stride_h;
  const void* k;    int64_t k_stride_b, k_stride_s, k_stride_h;
  const void* v;    int64_t v_stride_b, v_stride_s, v_stride_h;
  const void* o;    int64_t o_stride_b, o_stride_s, o_stride_h;
  const void* dout; int64_t do_stride_b, do_stride_s, do_stride_h;
  void* dq;         int64_t dq_stride_b, dq_stride_s, dq_stride_h;
  void* dk;         int64_t dk_stride_b, dk_stride_s, dk_stride_h;
  void* dv;         int64_t dv_stride_b, dv_stride_s, dv_stride_h;
  const float* lse;
  float scale, bias;
  const float* bias_ptr;
  void* workspace; size_t workspace_bytes;
  /* arbitrary masks, as elem_mask of ma_attn_params (with MA_MASK_NONE only): the same uint8/bool keep mask in both
   * orientations, strides in bytes, stride 0 broadcasts, rows 4-byte aligned.  elem_mask [1 or B, 1 or H, Sq, Skv]
   * serves the dq kernel, elem_mask_t [1 or B, 1 or H, Skv, Sq] (its transpose) the dk / dv kernels, where a lane
   * walks down a key's column; give both or neither.  (The reference generates the mask_mod's code into its backward
   * kernels as well, attn_tl.py:212-525.) */
  const uint8_t* elem_mask;   int64_t em_stride_b, em_stride_h, em_stride_q;
  const uint8_t* elem_mask_t; int64_t emt_stride_b, emt_stride_h, emt_stride_k;
  /* optional tile masks for the masks above (0 = the tile keeps nothing and is skipped; a non-zero entry for a tile
   * that keeps nothing is harmless; 2 = the element mask keeps every score of the tile and is not consulted for it), uint8/bool, strides in bytes, stride 0 broadcasts; give both or neither:
   * kv_block_mask [1 or B, 1 or H, ceil(Sq/128), ceil(Skv/32)] (the forward pass's prefill form) for the dq kernel,
   * q_block_mask  [1 or B, 1 or H, ceil(Skv/128), ceil(Sq/32)] for the dk / dv kernels. */
  const uint8_t* kv_block_mask; int64_t kbm_stride_b, kbm_stride_h, kbm_stride_q;
  const uint8_t* q_block_mask;  int64_t qbm_stride_b, qbm_stride_h, qbm_stride_k;
  /* RETENTION: p = q.k * scale * M / r with r the forward pass's row scale (passed as `lse`), which the backward
   * treats as a constant exactly as OnlineRetention.backward does (examples/retention_parallel.py:82-86:
   * dscores = dp / r; the score_mod's own derivative contributes the factor M).  score_mask is M as given to the
   * forward pass ([1 or B, H, Sq, Skv] in `dtype`), score_mask_t its transpose [1 or B, H, Skv, Sq] for the dk / dv
   * kernels; strides in elements, batch stride 0 broadcasts, rows 8-byte aligned (multiples of 4 elements). */
  const void* score_mask;   int64_t sm_stride_b, sm_stride_h, sm_stride_q;
  const void* score_mask_t; int64_t smt_stride_b, smt_stride_h, smt_stride_k;
  /* SOFTMAX, SIGMOID, RELU (softcap: SOFTMAX only, as in the forward): the additive score terms and the soft-capping of
   * ma_attn_params, exactly as given to the forward pass (the
   * reference differentiates whatever score_mod was traced, core/transform/core.py:119-199, core/lower/lower.py:510-525):
   * the scores are recomputed as x = s * scale + bias + score_add[b, h, q, kv] + pos_slope_q[h] * q + pos_slope_kv[h] * kv
   * and, with softcap > 0, softcap * tanh(x), whose derivative softcap * (1 - tanh^2 x) multiplies ds.  No gradient is
   * formed for score_add or the slopes (custom inputs get none in the reference either, attn_tl.py:669-692). */
  const void* score_add; int64_t sa_stride_b, sa_stride_h, sa_stride_q, sa_stride_kv; int32_t score_add_fp32;
  const float* pos_slope_q; const float* pos_slope_kv;
  float softcap;
} ma_attn_bwd_params;

/* Chunked linear / stateful attention forward.  Replaces the three launches
 * of LinearAttention.forward (tl_template/linear/linear_tl.py:1240-1269):
 * chunk-local cumsum (:36-60), chunk_fwd_h (:146-221), chunk_o (:322-399).
 *   o_t = q_scale * q_t . sum_{s<=t} exp(G_t - G_s) k_s^T (v_s * v_scale_s),  G = cumsum(log_decay)
 * q [B,Hq,T,Dk], k [B,Hk,T,Dk], v/o [B,H,T,Dv] (BHSD, contiguous), log_decay
 * fp32 [B,H,T]; head h reads q head h/(H/Hq) and k head h/(H/Hk) (:172,:351-352).
 * v_scale (may be NULL) is fp32 [B,H,T]: the fused per-token v modifier
 * (core/lower/lower_linear.py:211-287).  dim_k 64, 128, 192 or 256 (64 and 192 run in the 128- / 256-wide kernel, the rest of
 * the contraction being zeros that are never loaded), dim_v a multiple of 64. */
typedef struct ma_linear_params {
  int32_t dtype;
  int32_t batch, heads, heads_q, heads_k, seqlen, dim_k, dim_v, chunk;
  const void* q; const void* k; const void* v; void* o;
  const float* log_decay;
  const float* v_scale;
  float q_scale;
  int32_t segments; /* 0 = let the library choose; 1 = single pass; n = cut the sequence into at most n segments */
  int32_t out_fp32; /* non-zero: o is fp32 [B,H,T,Dv] (the backward pass builds the decay gradient from such outputs) */
  void* workspace; size_t workspace_bytes; /* see ma_linear_workspace_bytes; may be NULL (then single pass) */
} ma_linear_params;

/* Chunked linear / stateful attention backward.  Replaces LinearAttention.backward
 * (tl_template/linear/linear_tl.py:1268-1340: chunk_bwd_kernel_dh :461, chunk_bwd_dqkg :606, chunk_bwd_kernel_dv :876,
 * compute_final_dg :64-76): gradients of ma_linear_fwd's o with respect to q, k, v, log_decay and v_scale, given dout.
 * Tensors as in ma_linear_params (bf16, BHSD, contiguous, 16-byte aligned); dout [B,H,T,Dv] bf16; dq, dk, dv are bf16
 * with the shapes of q, k, v (heads that share a q / k head have their gradients summed, :1300-1303); dlog_decay fp32
 * [B,H,T]; dv_scale fp32 [B,H,T], written when v_scale is given (may then still be NULL to skip it).  dim_k 64, 128, 192 or 256,
 * dim_v a multiple of 64, at most 4096.  The workspace (ma_linear_bwd_workspace_bytes, 256-byte aligned) holds the fp32 per-head
 * gradients the decay gradient is formed from, and is required. */
typedef struct ma_linear_bwd_params {
  int32_t dtype;
  int32_t batch, heads, heads_q, heads_k, seqlen, dim_k, dim_v;
  const void* q; const void* k; const void* v; const void* dout;
  const float* log_decay;
  const float* v_scale;
  float q_scale;
  void* dq; void* dk; void* dv;
  float* dlog_decay;
  float* dv_scale;
  void* workspace; size_t workspace_bytes;
} ma_linear_bwd_params;

/* Absorbed MLA decode forward.  Replaces flash_attn_split + combine
 * (tl_template/attn/mla_decode_tl.py:154-290, wrapper :450-459):
 *   o = softmax((q.kv^T + q_pe.k_pe^T) * scale) . kv
 * q [B,Hq,D], q_pe [B,Hq,Dpe], kv [B,Skv,D], k_pe [B,Skv,Dpe], o [B,Hq,D]
 * (one latent kv head, one query token; the [B,1,Hq,.] / [B,Skv,1,.] tensors
 * of the reference are these with a unit dimension).  Partial outputs are kept in the tensors' dtype, as Output_partial
 * of the reference is (mla_decode_tl.py:160); their log-sum-exp is fp32. */
typedef struct ma_mla_params {
  int32_t dtype;
  int32_t batch, heads_q, seqlen_kv, dim, dim_pe;
  int32_t num_split; /* 0 = let the library choose */
  const void* q;    int64_t q_stride_b, q_stride_h;
  const void* q_pe; int64_t qpe_stride_b, qpe_stride_h;
  const void* kv;   int64_t kv_stride_b, kv_stride_s;
  const void* k_pe; int64_t kpe_stride_b, kpe_stride_s;
  void* o;          int64_t o_stride_b, o_stride_h;
  float* lse;       /* optional fp32 [B,Hq] natural-log lse; may be NULL */
  float scale;
  void* workspace; size_t workspace_bytes; /* see ma_mla_workspace_bytes */
  /* optional.  kv_seqlens int32 [B]: cache length of every batch entry (seqlen_kv is then the largest).
   * block_table int32 [B, block_table_stride]: paged cache as flash_mla_with_kvcache takes it
   * (cute_template_kvshared/flash_mla_interface.py:75-115): kv / k_pe address a pool of pages of page_size
   * rows (a multiple of 32; kv_stride_b / kpe_stride_b are ignored) and block_table[b][i] is the page
   * holding rows i * page_size .. of batch entry b. */
  const int32_t* kv_seqlens;
  const int32_t* block_table; int64_t block_table_stride; int32_t page_size;
  /* optional work plan for ragged batches, as written by ma_mla_get_metadata (kv_seqlens is then required and
   * num_split ignored): tile_scheduler_metadata int32 [num_sm_parts, 8], num_splits int32 [batch + 1], device memory.
   * Every workgroup then takes the contiguous run of (batch entry, token range) pieces its part of the plan names
   * instead of one of num_split equal ranges of one batch entry. */
  const int32_t* tile_scheduler_metadata;
  const int32_t* num_splits;
  int32_t num_sm_parts;
} ma_mla_params;

typedef void* ma_stream_t; /* a hipStream_t */

/* get_mla_metadata of the paged MLA interface (cute_template_kvshared/flash_mla_interface.py:57-72, kernels/
 * get_mla_metadata.cu:8-75): the number of parts the work of a launch is dealt to (one workgroup of 128 heads per CU),
 * and the plan itself, written on `stream` into device memory: tile_scheduler_metadata int32 [parts, 8] =
 * {first batch, first token, last batch, end token, split index of the first piece, 0, 0, 0} per part and num_splits
 * int32 [batch + 1], the number of pieces of the batch entries before each.  kv_seqlens is device memory, int32 [batch]. */
int ma_mla_num_sm_parts(int heads_q);
int ma_mla_get_metadata(const int32_t* kv_seqlens, int batch, int num_sm_parts, int32_t* tile_scheduler_metadata, int32_t* num_splits,
                        ma_stream_t stream);

int ma_version(void);
const char* ma_last_error(void);

/* attn_tl.py:92-190 (`main`) behind _attention.forward (:654-667); attn_decode_tl.py:63-206 for decode shapes */
size_t ma_attn_workspace_bytes(const ma_attn_params* p);
int ma_attn_fwd(const ma_attn_params* p, ma_stream_t stream);

/* attn_tl.py:669-692 (`_attention.backward`: mod_prep, mod_bwd, mod_post) */
size_t ma_attn_bwd_workspace_bytes(const ma_attn_bwd_params* p);
int ma_attn_bwd(const ma_attn_bwd_params* p, ma_stream_t stream);

/* linear_tl.py:1240-1269 */
size_t ma_linear_workspace_bytes(const ma_linear_params* p);
int ma_linear_fwd(const ma_linear_params* p, ma_stream_t stream);

/* linear_tl.py:1268-1340 */
size_t ma_linear_bwd_workspace_bytes(const ma_linear_bwd_params* p);
int ma_linear_bwd(const ma_linear_bwd_params* p, ma_stream_t stream);

/* mla_decode_tl.py:293-303 (`main_split`) */
int ma_mla_choose_split(const ma_mla_params* p);
size_t ma_mla_workspace_bytes(const ma_mla_params* p);
int ma_mla_decode(const ma_mla_params* p, ma_stream_t stream);

/* ma_mla_decode for callers that cannot allocate device memory and have no workspace at hand (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference, whose operators
 * allocate their partial results on every call.  Same arguments and results as ma_mla_decode, except that p->workspace is
 * ignored: the partial results of the kv splits go to an array inside the library, ma_mla_noalloc_max_workspace() bytes
 * (40 MiB) per GPU, held until the process ends -- by every process that loads the library and uses that GPU, whether or
 * not it calls this entry point (the array is part of the code object: 16 processes on one GPU hold 640 MiB); devices
 * beyond ordinal 63 are refused with MA_ERR_UNSUPPORTED.  A call whose ma_mla_workspace_bytes(p) exceeds that returns
 * MA_ERR_WORKSPACE.  The call itself allocates nothing and synchronises nothing.  All calls on one GPU share the array:
 * calls that overlap on one GPU (different streams, different threads) race; calls on one stream do not.  Every slot a
 * call reads it has written before, so nothing needs clearing between calls.  The first call on a device looks the
 * array's address up (and, if it is the library's first call, makes the runtime load the code object): make that call
 * outside graph capture. */
size_t ma_mla_noalloc_max_workspace(void);
int ma_mla_decode_noalloc(const ma_mla_params* p, ma_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* METAATTENTION_HIP_H */
