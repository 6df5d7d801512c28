// Host-side argument block of the chunked linear attention backward operator.
#pragma once
#include "common.h"

namespace ma {

struct LinBwdArgs {
  const void* q; const void* k; const void* v; const void* dout;   // bf16: q [B,Hq,T,Dk], k [B,Hk,T,Dk], v / dout [B,H,T,Dv]
  const float* log_decay;   // [B,H,T]
  const float* v_scale;     // [B,H,T] or null
  void* dq; void* dk; void* dv;   // bf16, shaped like q, k, v
  float* dlog_decay;        // [B,H,T]
  float* dv_scale;          // [B,H,T] or null
  float q_scale;
  int B, H, Hq, Hk, T, Dk, Dv;
};

// returns 0 ok, -1 launch failure, -2 unsupported, -3 workspace too small.  With query != null nothing is launched and
// *query receives the workspace size the same call needs.
int linear_bwd_run(const LinBwdArgs& a, void* ws, size_t ws_bytes, hipStream_t stream, size_t* query);

}  // namespace ma
