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
  // paged cache (flash_mla_with_kvcache of cute_template_kvshared/flash_mla_interface.py:75-115): kv / k_pe then
  // address a pool of pages of page_size rows, block_table[b * bt_stride + i] is the page holding rows
  // i * page_size .. of batch entry b; kv_lens[b] (optional, also without pages) is that entry's cache length
  const int32_t* block_table;
  int64_t bt_stride;
  int page_size;
  const int32_t* kv_lens;
  // planned launch (both set, with kv_lens): plan_meta int32 [plan_parts, 8], plan_splits int32 [B + 1] as written by
  // mla_plan_dispatch; o_part / lse_part then hold plan_splits[B] <= B + plan_parts slots
  const int32_t* plan_meta;
  const int32_t* plan_splits;
  int plan_parts;
};

int mla_decode_dispatch(const MlaArgs& a, bool is_bf16, int dim, int dim_pe, hipStream_t stream);
// The work plan of get_mla_metadata (cute_template_kvshared/kernels/get_mla_metadata.cu:8-75) for `parts` workgroups
// per block of heads: meta int32 [parts, 8], splits int32 [B + 1] (device memory).  0 ok, -1 launch failure.
int mla_plan_dispatch(const int32_t* seqlens, int batch, int parts, int block_n, int overhead_blocks, int32_t* meta, int32_t* splits,
                      hipStream_t stream);

}  // namespace ma
