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
  // sequence segments (see linear_fwd.hip): nseg segments of seg_chunks 32-token chunks; local end
  // states [group][segment][wave][registers][lane] fp32 and per-(batch*head, segment) log decays
  int nseg, seg_chunks;
  int out_f32;   // 1: o is fp32 [B,H,T,Dv] instead of bf16; 2: fp32, and the result is added to what o holds
  // General operand addressing (the backward's scans; all zero: q [B,Hq,T,Dk], k [B,Hk,T,Dk], v [B,H,T,Dv] as they
  // are): rev = the operands are read in reversed time order (token T-1-t at position t); q_row / k_row / v_row = elements
  // between consecutive tokens of an operand (a column slice of a wider tensor: the pointer carries the column offset);
  // Hv = heads of v (dividing H: head h reads v head h / (H / Hv)).
  int rev, Hv;
  int64_t q_row, k_row, v_row;
  // qk_cols (general addressing only; 0: all Dk): the q and k operands hold only this many columns (a multiple of 8); the
  // rest of the Dk-wide contraction is zeros that are never loaded (the tiles' LDS is cleared once, the loads of the missing
  // columns are switched off).
  int qk_cols;
  // rev_o (general addressing only): the outputs are written in reversed time order (row T-1-t holds the scan's token t), so
  // that a scan over reversed operands leaves its result in the operands' own order.
  int rev_o;
  // pieces (general addressing only; 0 or 1: none): the launch runs n_pieces independent scans side by side, piece p with
  // its q and k pointers moved on by p * piece_qk elements (the next slice of the contraction's columns) and its output
  // (fp32) by p * piece_o elements; the caller adds the pieces' outputs up.  Single pass only (no sequence segments).
  int n_pieces;
  int64_t piece_qk, piece_o;
  float* ws_state;
  float* ws_decay;
  // head-group range of this launch (a workgroup handles head group bg0 + its own index; bg_n groups in all; bg_n = 0: every
  // group, from 0).  The workspace of a launch with sequence segments is indexed by the launch's own group index.
  int bg0, bg_n;
};

int linear_fwd_dispatch(const LinArgs& a, int dk, int want_segments, void* ws, size_t ws_size, hipStream_t stream, size_t* query);

}  // namespace ma
