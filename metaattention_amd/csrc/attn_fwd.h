// Kernel-side argument block of the parallel attention forward kernels.
#pragma once
#include "common.h"

namespace ma {

struct AttnArgs {
  const void* q; const void* k; const void* v; void* o;
  float* row_scale;
  const float* bias_ptr;
  const void* smask;
  int64_t qsb, qss, qsh, ksb, kss, ksh, vsb, vss, vsh, osb, oss, osh, msb, msh, msq;
  int B, H, Sq, Skv, num_m_blocks;
  int kv_group;   // query heads per kv head (1 unless grouped-query)
  // The fields from here on are read by attn_wide_fwd_kernel only; a call at 128/128 that sets one of them is routed to
  // that kernel's 128/128 instantiation by the dispatcher instead of to attn_fwd_kernel.
  // decode-style kv selection: per-batch cache length and a per-(batch, kv head)
  // mask over blocks of kv_block keys (a multiple of 32)
  const int32_t* kv_lens;
  const uint8_t* kv_block_mask;
  int64_t kbm_sb, kbm_sh, kbm_sq;   // (kbm_sq: stride between blocks of 128 query rows; 0 for the decode form)
  int kv_block;
  int kbm_by_query_head;            // the mask's head axis counts query heads (prefill form) instead of kv heads
  // element-wise keep mask: uint8 [B|1, H|1, Sq, Skv], 0 = the score is masked
  const uint8_t* elem_mask;
  int64_t em_sb, em_sh, em_sq;
  // split-kv decode (attn_wide_fwd_kernel with one wave per workgroup): n_split kv ranges per (batch, head,
  // row block), normalised partial outputs [B, n_split, H, Sq, Dv] in the tensor dtype and their fp32
  // natural-log row scale [B, n_split, H, Sq], merged by attn_split_combine_kernel
  int n_split;
  void* o_part;
  float* lse_part;
  float scale, bias;
  // additive score terms: x = s * scale + bias + add[b, h, q, kv] + slope_q[h] * q + slope_kv[h] * kv,
  // then, with softcap > 0, x = softcap * tanh(x).  add: fp32 or the tensor dtype, element strides (0 broadcasts).
  const void* add;
  int64_t add_sb, add_sh, add_sq, add_sk;
  int add_f32;
  const float* slope_q;
  const float* slope_kv;
  float softcap;
  // retention family at Dqk 256 / Dv 512, instead of smask: fp32 [H], the multiplier is gamma[h]^(q - kv) for kv <= q, else 0
  const float* decay_gamma;
};

int attn_wide_fwd_dispatch(const AttnArgs& a, int family, bool causal, bool is_bf16, int dqk, int dv, hipStream_t stream);
// number of kv splits the decode path would use for these sizes (1: not a decode shape / nothing to gain)
int attn_decode_splits(int family, bool causal, int B, int H, int Sq, int Skv, int dqk, int dv);
int attn_fwd_dispatch(const AttnArgs& a, int family, bool causal, bool is_bf16, int dqk, int dv, hipStream_t stream);
// the retention family at Dqk 256 / Dv 512 (retention_fwd.hip); 0 ok, -1 launch failure, -2 unsupported
int retention_pair_fwd_dispatch(const AttnArgs& a, bool causal, bool is_bf16, hipStream_t stream);

}  // namespace ma
