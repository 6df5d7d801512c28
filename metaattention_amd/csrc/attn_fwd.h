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
  // decode-style kv selection (attn_wide_fwd_kernel only): per-batch cache length and a per-(batch, kv head)
  // mask over blocks of kv_block keys (a multiple of 32)
  const int32_t* kv_lens;
  const uint8_t* kv_block_mask;
  int64_t kbm_sb, kbm_sh;
  int kv_block;
  float scale, bias;
};

int attn_wide_fwd_dispatch(const AttnArgs& a, int family, bool causal, bool is_bf16, int dqk, int dv, hipStream_t stream);
int attn_fwd_dispatch(const AttnArgs& a, int family, bool causal, bool is_bf16, int dqk, int dv, hipStream_t stream);

}  // namespace ma
