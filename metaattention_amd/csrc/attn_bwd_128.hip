// Parallel attention backward: the instantiations of attn_bwd_kernels.h for the head sizes 128 / 128
// (one translation unit per group of head sizes, so that they compile side by side).
#include "attn_bwd_kernels.h"

namespace ma {

int attn_bwd_128_128(const AttnBwdArgs& a, int family, bool causal, bool is_bf16, hipStream_t stream) {
  return is_bf16 ? bwd_size<__bf16, 128, 128, true>(a, family, causal, stream) : bwd_size<_Float16, 128, 128, true>(a, family, causal, stream);
}

}  // namespace ma
