// Parallel attention backward: the instantiations of attn_bwd_kernels.h for the head sizes 192 / 128, 128 / 256
// (one translation unit per group of head sizes, so that they compile side by side).
#include "attn_bwd_kernels.h"

namespace ma {

int attn_bwd_192_128(const AttnBwdArgs& a, int family, bool causal, bool is_bf16, hipStream_t stream) {
  return is_bf16 ? bwd_size<__bf16, 192, 128, false>(a, family, causal, stream) : bwd_size<_Float16, 192, 128, false>(a, family, causal, stream);
}

int attn_bwd_128_256(const AttnBwdArgs& a, int family, bool causal, bool is_bf16, hipStream_t stream) {
  return is_bf16 ? bwd_size<__bf16, 128, 256, true>(a, family, causal, stream) : bwd_size<_Float16, 128, 256, true>(a, family, causal, stream);
}

}  // namespace ma
