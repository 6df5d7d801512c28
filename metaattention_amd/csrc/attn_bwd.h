// Kernel-side argument block of the parallel attention backward kernels.
#pragma once
#include "common.h"

namespace ma {

struct AttnBwdArgs {
  const void* q; const void* k; const void* v; const void* o; const void* dout;
  void* dq; void* dk; void* dv;
  const float* lse;    // [B,H,Sq] row scale of the forward pass: natural-log sum (softmax), r (retention)
  float* delta;        // [B,H,Sq] workspace: sum_d dout * o per row (softmax)
  const float* bias_ptr;
  int64_t qsb, qss, qsh, ksb, kss, ksh, vsb, vss, vsh, osb, oss, osh, dosb, doss, dosh;
  int64_t dqsb, dqss, dqsh, dksb, dkss, dksh, dvsb, dvss, dvsh;
  int B, H, Hkv, Sq, Skv, num_blocks;
  int kv_group;   // query heads per kv head
  float scale, bias;
  // optional element-wise keep mask (0 = masked) in both orientations, strides in bytes, 0 broadcasts:
  // elem_mask [.., .., Sq, Skv] for the dq kernel (a lane walks a query row), elem_mask_t [.., .., Skv, Sq]
  // for the dk / dv kernel (a lane walks a key's column); rows are 4-byte aligned
  const uint8_t* elem_mask; int64_t em_sb, em_sh, em_sq;
  const uint8_t* elem_mask_t; int64_t emt_sb, emt_sh, emt_sk;
  // optional tile masks (0 = nothing kept in the tile: skipped), strides in bytes, 0 broadcasts:
  // kv_block_mask [.., .., ceil(Sq/128), ceil(Skv/32)] for the dq kernel (a workgroup's 128 rows x a 32-key tile),
  // q_block_mask  [.., .., ceil(Skv/128), ceil(Sq/32)] for the dk / dv kernel (a workgroup's 128 keys x a 32-row tile)
  const uint8_t* kv_block_mask; int64_t kbm_sb, kbm_sh, kbm_sq;
  const uint8_t* q_block_mask; int64_t qbm_sb, qbm_sh, qbm_sk;
  // retention family: the score multiplier of the forward pass in the tensor dtype, in both orientations (strides in
  // elements, 0 broadcasts): smask [.., H, Sq, Skv] for the dq kernel, smask_t [.., H, Skv, Sq] for the dk / dv kernels;
  // rows are 8-byte aligned.  `lse` then holds the forward's row scale r.
  const void* smask; int64_t sm_sb, sm_sh, sm_sq;
  const void* smask_t; int64_t smt_sb, smt_sh, smt_sk;
  // softmax family: additive score terms and soft-capping as in the forward pass (AttnArgs): x = s * scale + bias +
  // add[b, h, q, kv] + slope_q[h] * q + slope_kv[h] * kv, then softcap * tanh(x) when softcap > 0; add in fp32 or the
  // tensor dtype, element strides (0 broadcasts).  Any of them set selects the kernels' EXTRA instantiations.
  const void* add;
  int64_t add_sb, add_sh, add_sq, add_sk;
  int add_f32;
  const float* slope_q;
  const float* slope_kv;
  float softcap;
};

int attn_bwd_dispatch(const AttnBwdArgs& a, int family, bool causal, bool is_bf16, int dqk, int dv, hipStream_t stream);

}  // namespace ma
