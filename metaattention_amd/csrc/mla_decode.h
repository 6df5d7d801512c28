// Kernel-side argument block of the MLA decode kernels.
#pragma once
#include "common.h"

namespace ma {

struct MlaArgs {
  const void* q; const void* q_pe; const void* kv; const void* k_pe; void* o;
  float* lse;
  void* o_part;     // dtype [B, num_split, Hq, 512], normalised per split
  float* lse_part;  // fp32 [B, num_split, Hq], log2 domain
  int64_t qsb, qsh, qpsb, qpsh, kvsb, kvss, kpsb, kpss, osb, osh;
  int B, Hq, Skv, num_split, split_len, head_blocks;
  float scale;
};

int mla_decode_dispatch(const MlaArgs& a, bool is_bf16, int dim, int dim_pe, hipStream_t stream);

}  // namespace ma
