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
  float scale, bias;
};

int attn_wide_fwd_dispatch(const AttnArgs& a, int family, bool causal, bool is_bf16, int dqk, int dv, hipStream_t stream);
int attn_fwd_dispatch(const AttnArgs& a, int family, bool causal, bool is_bf16, int dqk, int dv, hipStream_t stream);

}  // namespace ma
