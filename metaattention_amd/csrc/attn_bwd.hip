// Parallel attention backward: dispatch by head size to the translation units that hold the kernels (attn_bwd_kernels.h,
// instantiated per group of head sizes in attn_bwd_128.hip, attn_bwd_64.hip, attn_bwd_192.hip, attn_bwd_256.hip).
#include "attn_bwd.h"

namespace ma {

int attn_bwd_128_128(const AttnBwdArgs& a, int family, bool causal, bool is_bf16, hipStream_t stream);
int attn_bwd_64_64(const AttnBwdArgs& a, int family, bool causal, bool is_bf16, hipStream_t stream);
int attn_bwd_128_256(const AttnBwdArgs& a, int family, bool causal, bool is_bf16, hipStream_t stream);
int attn_bwd_256_256(const AttnBwdArgs& a, int family, bool causal, bool is_bf16, hipStream_t stream);
int attn_bwd_192_128(const AttnBwdArgs& a, int family, bool causal, bool is_bf16, hipStream_t stream);   // (the reference's DeepSeek-V2-Lite benchmark shape; not the retention family)
int attn_bwd_256_512(const AttnBwdArgs& a, int family, bool causal, bool is_bf16, hipStream_t stream);   // (256 / 512 is the head size of the retention operator itself, examples/retention_parallel.py)

// returns 0 ok, -1 launch failure, -2 unsupported
int attn_bwd_dispatch(const AttnBwdArgs& a, int family, bool causal, bool is_bf16, int dqk, int dv, hipStream_t stream) {
  // (the tile DMA addresses a tile's 32 rows with 32-bit byte offsets from its first row)
  for (int64_t row_stride : {a.qss, a.kss, a.vss, a.doss})
    if (row_stride < 0 || row_stride >= ((int64_t)1 << 26)) return -2;
  if (dqk == 128 && dv == 128) return attn_bwd_128_128(a, family, causal, is_bf16, stream);
  if (dqk == 64 && dv == 64) return attn_bwd_64_64(a, family, causal, is_bf16, stream);
  if (dqk == 128 && dv == 256) return attn_bwd_128_256(a, family, causal, is_bf16, stream);
  if (dqk == 256 && dv == 256) return attn_bwd_256_256(a, family, causal, is_bf16, stream);
  if (dqk == 192 && dv == 128) return attn_bwd_192_128(a, family, causal, is_bf16, stream);
  if (dqk == 256 && dv == 512) return attn_bwd_256_512(a, family, causal, is_bf16, stream);
  return -2;
}

}  // namespace ma
