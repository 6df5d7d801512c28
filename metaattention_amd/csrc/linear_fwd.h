// Kernel-side argument block of the chunked linear attention forward kernel.
#pragma once
#include "common.h"

namespace ma {

struct LinArgs {
  const void* q; const void* k; const void* v; void* o;
  const float* log_decay;  // [B,H,T]
  const float* v_scale;    // [B,H,T] or null
  float q_scale;
  int B, H, Hq, Hk, T, Dv, dv_blocks;
};

int linear_fwd_dispatch(const LinArgs& a, int dk, hipStream_t stream);

}  // namespace ma
