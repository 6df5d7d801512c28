// Parallel attention forward for every head size the fast kernel (attn_fwd.hip, 128/128) does not
// take, and for the normalised retention family (wide heads: Dqk 256, Dv 512), for gfx950.
//
// Same operator as attn_fwd.hip: attention_engine/core/template/tl_template/attn/attn_tl.py:92-190
// behind _attention.forward (:654-667), with the row functions of examples/mha.py (softmax),
// examples/sigmoid_attn.py, examples/reluattn.py and examples/retention_parallel.py:
//   softmax    p = exp(x - m),  o = sum p v / sum p,  lse = m + log sum p      (x = s * scale + bias)
//   sigmoid    p = 1 / (1 + exp(-x)),  masked p = 0
//   relu       p = max(x, 0),          masked p = 0
//   retention  qkm = s * scale * M,  r = max(sum_j |qkm|, 1),  o = (qkm / r) v, M a caller-supplied
//              [1|B, H, Sq, Skv] multiplier (the decay mask).  As in the reference (mask_value "0") no
//              element-wise causal mask is applied in forward: with the causal structural mask only kv
//              tiles above the workgroup's diagonal are skipped and the zeros come from M itself.
// The head sizes of the reference's own test list are covered (testing/test.py:54-63: 128/256 softmax,
// 64/64 relu, 256/512 retention) next to 256/256 and 256/512.
//
// Decode shapes (a few query rows against a long cache, softmax, no mask) run with one wave per
// workgroup and the kv sequence cut into splits, each writing a normalised partial output and its
// log-sum-exp to a workspace; attn_split_combine_kernel merges them (the split-KV scheme of
// tl_template/attn/attn_decode_tl.py:63-206 with the `combine` of examples/mha_decode.py:72-80).
//
// Structure.  One workgroup of 4 waves owns 128 query rows (32 per wave, Q fragments in registers)
// and walks the kv sequence in tiles of 32 rows; K and V tiles arrive by direct-to-LDS DMA, double
// buffered, one barrier per tile.  Scores are computed transposed (S^T = K Q^T) as in attn_fwd.hip, so
// a lane owns one query row, row statistics stay in the lane pair (l, l ^ 32) and P^T is the B operand
// of O^T += V^T P^T without a shuffle.  With Dv = 512 the fp32 accumulator takes 256 registers per lane
// and a wave runs alone on its SIMD.
//   * softmax rescales the accumulator only on tiles where some row's maximum grew;
//   * the retention row function is linear up to its final clamp, so the accumulator is kept
//     un-normalised (O = sum_j P_j V_j, r = sum_j |P_j| in fp32) and divided by max(r, 1) once at the
//     end; the online form of the reference rescales every tile and gives the same value up to rounding.
#include "attn_fwd.h"
#include <type_traits>

namespace ma {

namespace {
enum { WF_SOFTMAX = 0, WF_SIGMOID = 1, WF_RELU = 2, WF_RETENTION = 3 };   // = MA_ATTN_* of the C interface
}

template <typename T, int DQK, int DV, int FAMILY, bool CAUSAL, int NW>
__global__ __launch_bounds__(64 * NW, ((DQK + DV >= 512 || (NW == 1 && pad_width(DQK) + DV >= 384)) ? 1 : 2)) void attn_wide_fwd_kernel(const AttnArgs a) {
  using E = Elem<T>;
  using x8 = typename E::x8;
  using x4 = typename E::x4;
  constexpr int BM = 32 * NW, BN = 32;
  constexpr int KS = DQK / 16, DB = DV / 32;
  constexpr int KROW = pad_width(DQK) * 2, VROW = DV * 2;   // (LDS rows; 192-wide keys sit in 256-wide rows)
  constexpr int CPRK = pad_width(DQK) / 8, CPRV = DV / 8, USEDK = DQK / 8;
  constexpr int KTILE = BN * KROW, VTILE = BN * VROW, STAGE = KTILE + VTILE;
  constexpr int NIK = KTILE / 1024, NIV = VTILE / 1024;
  static_assert(CPRK >= 8 && CPRV >= 8 && DQK % 16 == 0 && DV % 64 == 0, "head size");

  extern __shared__ __align__(16) char smem[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(MA_LDS char*)smem;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, g = lane >> 5;

  const int nmb = a.num_m_blocks, BH = a.B * a.H;
  int bh, mb, split;
  {
    int slot;
    if ((BH & 7) == 0) {
      const int xcd = blockIdx.x & 7;
      slot = blockIdx.x >> 3;
      split = slot % a.n_split;
      slot /= a.n_split;
      bh = (slot / nmb) * 8 + xcd;
    } else {
      slot = blockIdx.x;
      split = slot % a.n_split;
      slot /= a.n_split;
      bh = slot / nmb;
    }
    mb = slot % nmb;
  }
  if (CAUSAL) mb = nmb - 1 - mb;
  const int b = bh / a.H, h = bh % a.H;
  const int m_wave = mb * BM + wave * 32, m_lane = m_wave + r;
  const int m_ld = min(m_lane, a.Sq - 1);

  x8 qf[KS];
  {
    const T* qp = (const T*)a.q + (int64_t)b * a.qsb + (int64_t)m_ld * a.qss + (int64_t)h * a.qsh + 8 * g;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) qf[ks] = *(const x8*)(qp + 16 * ks);
  }
  const char* kb = (const char*)((const T*)a.k + (int64_t)b * a.ksb + (int64_t)(h / a.kv_group) * a.ksh);
  const char* vb = (const char*)((const T*)a.v + (int64_t)b * a.vsb + (int64_t)(h / a.kv_group) * a.vsh);
  const int64_t k_row_bytes = a.kss * 2, v_row_bytes = a.vss * 2;
  const T* mrow = nullptr;
  if constexpr (FAMILY == WF_RETENTION) mrow = (const T*)a.smask + (int64_t)b * a.msb + (int64_t)h * a.msh + (int64_t)m_ld * a.msq;

  // keys beyond this batch entry's cache length do not exist (blockattn_decode_varlen_tl.py:66-75)
  const int skv = a.kv_lens ? min(a.Skv, max(a.kv_lens[b], 0)) : a.Skv;
  int n_tiles = (skv + BN - 1) / BN;
  if (CAUSAL) n_tiles = min(n_tiles, (mb * BM + BM + BN - 1) / BN);
  // tiles whose block of keys is switched off for this (batch, kv head) are skipped (:57-64)
  const uint8_t* bm_row = a.kv_block_mask ? a.kv_block_mask + (int64_t)b * a.kbm_sb +
                                                (int64_t)(a.kbm_by_query_head ? h : h / a.kv_group) * a.kbm_sh + (int64_t)mb * a.kbm_sq
                                          : nullptr;
  // element-wise keep mask of this lane's row (any mask_mod, evaluated densely by the host: blockattn_tl.py:176-190
  // generates its code into the kernel instead); the four bytes of a lane's four consecutive keys come as one word
  const uint8_t* em_row = a.elem_mask ? a.elem_mask + (int64_t)b * a.em_sb + (int64_t)h * a.em_sh + (int64_t)m_ld * a.em_sq : nullptr;
  auto load_keep = [&](int n0, uint32_t (&kp)[4]) {
#pragma unroll
    for (int q4 = 0; q4 < 4; q4++) {
      const int n = n0 + 8 * q4 + 4 * g;
      if (n + 3 < skv) {
        kp[q4] = *(const uint32_t*)(em_row + n);
      } else {
        kp[q4] = 0;
#pragma unroll
        for (int i = 0; i < 4; i++)
          if (n + i < skv) kp[q4] |= (uint32_t)em_row[n + i] << (8 * i);
      }
    }
  };
  // additive score terms of this lane's row (the score_mod's custom inputs other than the multiplier; core/lower/
  // lower.py:561-615 loads them per q tile, per kv step or as [block_M, block_N] tiles depending on their shape: here
  // one strided tensor covers all of those shapes) and terms linear in the indices; folded into the raw score as
  // extra / scale, so that everything after sees s * scale + bias + extra
  const bool has_extra = a.add || a.slope_q || a.slope_kv;
  const float inv_scale = 1.f / a.scale;
  const float sl_q = a.slope_q ? a.slope_q[h] * (float)m_ld : 0.f, sl_kv = a.slope_kv ? a.slope_kv[h] : 0.f;
  const int64_t add_row = (int64_t)b * a.add_sb + (int64_t)h * a.add_sh + (int64_t)m_ld * a.add_sq;
  auto load_extra = [&](int n0, float (&ex)[16]) {
#pragma unroll
    for (int jj = 0; jj < 16; jj++) {
      const int n = min(n0 + 8 * (jj >> 2) + 4 * g + (jj & 3), skv - 1);
      float e = sl_q + sl_kv * (float)n;
      if (a.add) e += a.add_f32 ? ((const float*)a.add)[add_row + (int64_t)n * a.add_sk] : (float)((const T*)a.add)[add_row + (int64_t)n * a.add_sk];
      ex[jj] = e * inv_scale;
    }
  };
  const int tiles_per_block = a.kv_block / BN;
  // this workgroup's share of the tiles
  const int tiles_per_split = (n_tiles + a.n_split - 1) / a.n_split;
  const int t_begin = split * tiles_per_split;
  n_tiles = min(n_tiles, t_begin + tiles_per_split);
  auto next_tile = [&](int jt) {
    if (bm_row)
      while (jt < n_tiles && !bm_row[jt / tiles_per_block]) jt++;
    return jt;
  };
  // (block mask entry 2, beside an element-wise mask: that mask keeps every score of the block and is not read for it)
  auto tile_full = [&](int jt) { return em_row && bm_row && bm_row[jt / tiles_per_block] >= 2; };

  // DMA of one tile: each instruction moves 1 KB (1024 / row bytes tile rows); lane i fetches the
  // 16-byte chunk that belongs at physical position i of that KB.  Rows beyond the sequence are clamped
  // to its last row (their scores are masked, or multiplied by a zero of M).
  TileDma<KROW, NW, USEDK> k_dma;
  TileDma<VROW, NW> v_dma;
  k_dma.init((uint32_t)k_row_bytes, wave, lane);
  v_dma.init((uint32_t)v_row_bytes, wave, lane);
  auto issue_tile = [&](int n0, int buf) {
    const uint32_t base = lds0 + buf * STAGE;
    if (n0 + BN <= skv) {   // (wave-uniform) a whole tile: scalar bases, the lane offsets computed once
      k_dma.issue(kb + (int64_t)n0 * k_row_bytes, base, wave);
      v_dma.issue(vb + (int64_t)n0 * v_row_bytes, base + KTILE, wave);
      return;
    }
    for (int ii = wave; ii < NIK + NIV; ii += NW) {
      if (ii < NIK) {
        const int row = ii * (1024 / KROW) + lane / CPRK, c = lane % CPRK;
        const int nrow = min(n0 + row, skv - 1);
        if (USEDK == CPRK || (c ^ swz_tile<CPRK>(row)) < USEDK)   // (chunks beyond the head size do not exist in memory)
          dma16(kb + nrow * k_row_bytes + ((c ^ swz_tile<CPRK>(row)) << 4), base + ii * 1024);
      } else {
        const int i2 = ii - NIK;
        const int row = i2 * (1024 / VROW) + lane / CPRV, c = lane % CPRV;
        const int nrow = min(n0 + row, skv - 1);
        dma16(vb + nrow * v_row_bytes + ((c ^ swz_tile<CPRV>(row)) << 4), base + KTILE + i2 * 1024);
      }
    }
  };
  // multiplier values of this lane's score elements: row m_lane, columns n0 + 8q4 + 4g + {0..3}
  auto load_mask = [&](int n0, x4 (&mk)[4]) {
#pragma unroll
    for (int q4 = 0; q4 < 4; q4++) {
      const int n = n0 + 8 * q4 + 4 * g;
      if (n + 3 < skv) {
        mk[q4] = *(const x4*)(mrow + n);
      } else {
#pragma unroll
        for (int i = 0; i < 4; i++) mk[q4][i] = n + i < skv ? mrow[n + i] : (T)0.f;
      }
    }
  };

  const uint32_t k_row_off = r * KROW;
  const int k_c0 = g ^ swz_tile<CPRK>(r);
  const int jr = (lane & 15) >> 2;
  const int lc = (((lane >> 4) & 1) << 1) | ((lane & 3) >> 1);
  const uint32_t v_row_off = (4 * g + jr) * VROW + (lane & 1) * 8;
  const int v_c0 = lc ^ swz_tile<CPRV>(4 * g + jr);

  f32x16 o[DB];
#pragma unroll
  for (int i = 0; i < DB; i++)
#pragma unroll
    for (int j = 0; j < 16; j++) o[i][j] = 0.f;
  float r_part = 0.f;      // this lane's share of the row sum (sum p, or sum |p| for retention)
  float row_max = -1e30f;  // softmax: running maximum of x * log2(e), the same in both lanes of a row
  const float bias = a.bias + (a.bias_ptr ? *a.bias_ptr : 0.f);
  const float c_scale = a.scale * kLog2e, c_bias = bias * kLog2e;

  x4 mk_next[4];
  uint32_t keep_next[4] = {0, 0, 0, 0};
  bool full_next = false;
  int jt = next_tile(t_begin);
  if (jt < n_tiles) {
    issue_tile(jt * BN, 0);
    full_next = tile_full(jt);
    if constexpr (FAMILY == WF_RETENTION) load_mask(jt * BN, mk_next);
    else if (em_row && !full_next) load_keep(jt * BN, keep_next);
  }

  for (int it = 0; jt < n_tiles; it++) {
    const int buf = it & 1, n0 = jt * BN;
    wait_dma();
    __syncthreads();
    jt = next_tile(jt + 1);   // from here on: the tile after this one
    x4 mk[4];
    if constexpr (FAMILY == WF_RETENTION) {
#pragma unroll
      for (int q4 = 0; q4 < 4; q4++) mk[q4] = mk_next[q4];
    }
    uint32_t keep[4];
#pragma unroll
    for (int q4 = 0; q4 < 4; q4++) keep[q4] = keep_next[q4];
    const bool full = full_next;
    if (jt < n_tiles) {
      full_next = tile_full(jt);
      if constexpr (FAMILY == WF_RETENTION) load_mask(jt * BN, mk_next);
      else if (em_row && !full_next) load_keep(jt * BN, keep_next);
      issue_tile(jt * BN, buf ^ 1);
    }
    const uint32_t kbase = lds0 + buf * STAGE, vbase = kbase + KTILE;
    float ex[16];
    if constexpr (FAMILY != WF_RETENTION) {
      if (has_extra) load_extra(n0, ex);
    }

    // ---- S^T = K Q^T
    f32x16 s;
#pragma unroll
    for (int j = 0; j < 16; j++) s[j] = 0.f;
    {
      constexpr int AH = 2, RING = 3;
      x8 kf[RING];
#pragma unroll
      for (int ks = 0; ks < AH; ks++) kf[ks] = lds_read<x8>(kbase + k_row_off + (uint32_t)((k_c0 ^ (2 * ks)) << 4));
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        if (ks + AH < KS) kf[(ks + AH) % RING] = lds_read<x8>(kbase + k_row_off + (uint32_t)((k_c0 ^ (2 * (ks + AH))) << 4));
        __builtin_amdgcn_sched_barrier(0);
        s = E::mfma32(kf[ks % RING], qf[ks], s);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // ---- P^T from S^T (lane: row m_lane, kv rows n0 + 8(jj/4) + 4g + jj%4)
    x8 pf[2];
    if constexpr (FAMILY == WF_RETENTION) {
#pragma unroll
      for (int jj = 0; jj < 16; jj++) {
        const float p = s[jj] * a.scale * (float)mk[jj >> 2][jj & 3];
        r_part += fabsf(p);
        pf[jj >> 3][jj & 7] = (T)p;
      }
    } else {
      if (has_extra) {
#pragma unroll
        for (int jj = 0; jj < 16; jj++) s[jj] += ex[jj];
      }
      if (a.softcap > 0.f) {   // x -> softcap * tanh(x), x = s * scale + bias;  tanh(x) = 1 - 2 / (1 + e^(2x))
#pragma unroll
        for (int jj = 0; jj < 16; jj++) {
          const float x = s[jj] * a.scale + bias;
          const float th = 1.f - 2.f * fast_rcp(1.f + fast_exp2(x * (2.f * kLog2e)));
          s[jj] = (a.softcap * th - bias) * inv_scale;
        }
      }
      // element-wise mask only on tiles that reach past the diagonal or the end of the sequence
      const bool edge = (CAUSAL && n0 + BN - 1 > m_wave) || n0 + BN > skv;
      if (edge) {
#pragma unroll
        for (int jj = 0; jj < 16; jj++) {
          const int n = n0 + 8 * (jj >> 2) + 4 * g + (jj & 3);
          if ((CAUSAL && n > m_lane) || n >= skv) s[jj] = -INFINITY;
        }
      }
      if (em_row && !full) {
#pragma unroll
        for (int jj = 0; jj < 16; jj++)
          if (((keep[jj >> 2] >> (8 * (jj & 3))) & 0xff) == 0) s[jj] = -INFINITY;
      }
      if constexpr (FAMILY == WF_SOFTMAX) {
        // Lazy reference: the exponentials are taken relative to row_max, which only moves when some probability of the
        // tile would exceed 2^8 (exact in fp32, in range for bf16 / fp16; the final division absorbs the offset) -- so
        // the hot path has no maximum over the scores in front of its exponentials, only one over the probabilities
        // behind them.  The first tile (row_max = -1e30: infinite probabilities) and growing scores take the cold path,
        // which moves the reference of the rows concerned to their true maximum; both lanes of a row decide alike.
        float p[16];
        float sub = c_bias - row_max;
#pragma unroll
        for (int jj = 0; jj < 16; jj++) p[jj] = fast_exp2(s[jj] * c_scale + sub);
        const float pm = fmaxf(fmaxf(fmaxf(fmaxf(p[0], p[1]), fmaxf(p[2], p[3])), fmaxf(fmaxf(p[4], p[5]), fmaxf(p[6], p[7]))),
                               fmaxf(fmaxf(fmaxf(p[8], p[9]), fmaxf(p[10], p[11])), fmaxf(fmaxf(p[12], p[13]), fmaxf(p[14], p[15]))));
        if (__any(pm > 256.f)) {
          float mx = fmaxf(fmaxf(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])), fmaxf(fmaxf(s[4], s[5]), fmaxf(s[6], s[7]))),
                           fmaxf(fmaxf(fmaxf(s[8], s[9]), fmaxf(s[10], s[11])), fmaxf(fmaxf(s[12], s[13]), fmaxf(s[14], s[15]))));
          mx = fmaxf(mx, xhalf(mx)) * c_scale + c_bias;
          // (each row decides for itself, from its own probabilities only: what another row of the wave holds -- keys a
          // causal mask hides from this one, say -- must not change this row's bits)
          const bool move = fmaxf(pm, xhalf(pm)) > 256.f;
          const float m_new = move ? fmaxf(row_max, mx) : row_max;
          const float corr = fast_exp2(row_max - m_new);
          r_part *= corr;
          if constexpr (DQK + DV >= 512) {
            // one wave per SIMD: the accumulators live in the MFMA accumulation registers and are rescaled there one at a
            // time through one vector register.  Written as C++ the compiler moves them all to vector registers first: at
            // Dv 512 it then spills 231 registers, in the loop's hot path as well (12 % of this speed), at 256 / 256 it
            // holds 438 registers instead of 326 and runs 20 % slower.
#pragma unroll
            for (int i = 0; i < DB; i++)
#pragma unroll
              for (int j = 0; j < 16; j++) {
                float t;
                asm volatile("v_accvgpr_read_b32 %1, %0\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 %0, %1" : "+a"(o[i][j]), "=&v"(t) : "v"(corr));
              }
            asm volatile("s_nop 4");   // (an accumulation register written by the vector ALU is not read by an MFMA at once)
          } else {
#pragma unroll
            for (int i = 0; i < DB; i++)
#pragma unroll
              for (int j = 0; j < 16; j++) o[i][j] *= corr;
          }
          row_max = m_new;
          sub = c_bias - row_max;
#pragma unroll
          for (int jj = 0; jj < 16; jj++) p[jj] = fast_exp2(s[jj] * c_scale + sub);
        }
#pragma unroll
        for (int jj = 0; jj < 16; jj++) {
          r_part += p[jj];
          pf[jj >> 3][jj & 7] = (T)p[jj];
        }
      } else if constexpr (FAMILY == WF_SIGMOID) {
#pragma unroll
        for (int jj = 0; jj < 16; jj++)   // sigmoid(x) = 1 / (1 + 2^(-x log2e)); s = -inf gives exactly 0
          pf[jj >> 3][jj & 7] = (T)fast_rcp(1.f + fast_exp2(-(s[jj] * c_scale + c_bias)));
      } else {
#pragma unroll
        for (int jj = 0; jj < 16; jj++) pf[jj >> 3][jj & 7] = (T)fmaxf(s[jj] * a.scale + bias, 0.f);
      }
    }
    // ---- O^T += V^T P^T
    {
      constexpr int PF = DB >= 4 ? 6 : 2 * DB;
      x4 lo[PF], hi[PF];
      auto request = [&](int idx) {   // idx = 2 db + s
        const int db = idx >> 1, sl = idx & 1;
        const uint32_t rb = vbase + v_row_off + 16 * sl * VROW;
        lo[idx % PF] = lds_read_tr4<T>(rb + (uint32_t)((v_c0 ^ (4 * db)) << 4));
        hi[idx % PF] = lds_read_tr4<T>(rb + 8 * VROW + (uint32_t)((v_c0 ^ (4 * db) ^ 2) << 4));
      };
#pragma unroll
      for (int i = 0; i < PF - 1; i++) request(i);
#pragma unroll
      for (int idx = 0; idx < 2 * DB; idx++) {
        if (idx + PF - 1 < 2 * DB) request(idx + PF - 1);
        __builtin_amdgcn_sched_barrier(0);
        x8 vf = __builtin_shufflevector(lo[idx % PF], hi[idx % PF], 0, 1, 2, 3, 4, 5, 6, 7);
        o[idx >> 1] = E::mfma32(vf, pf[idx & 1], o[idx >> 1]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  __syncthreads();   // every wave is done with the K/V buffers: they become output staging

  float inv = 1.f;
  float* rs_ptr = a.row_scale && g == 0 && m_lane < a.Sq ? a.row_scale + ((int64_t)b * a.H + h) * a.Sq + m_lane : nullptr;
  if (a.n_split > 1) rs_ptr = g == 0 && m_lane < a.Sq ? a.lse_part + (((int64_t)b * a.n_split + split) * a.H + h) * a.Sq + m_lane : nullptr;
  if constexpr (FAMILY == WF_RETENTION) {
    const float r_tot = fmaxf(r_part + xhalf(r_part), 1.f);
    inv = 1.f / r_tot;
    if (rs_ptr) *rs_ptr = r_tot;
  } else if constexpr (FAMILY == WF_SOFTMAX) {
    const float tot = r_part + xhalf(r_part);
    inv = tot > 0.f ? 1.f / tot : 0.f;   // (a row that was left no key at all gives zeros and lse = -inf)
    if (rs_ptr) *rs_ptr = tot > 0.f ? (row_max + fast_log2(tot)) * kLn2 : -INFINITY;
  }

  // ---- O: two halves of DV/2 columns through a wave-private LDS block, coalesced 16-byte stores
  constexpr int HALF = DV / 2, OROW = HALF * 2 + 16;
  const uint32_t ob = lds0 + wave * 32 * OROW;
  T* obase = (T*)a.o + (int64_t)b * a.osb + (int64_t)h * a.osh;
  int64_t o_row_stride = a.oss;
  if (a.n_split > 1) {
    obase = (T*)a.o_part + ((((int64_t)b * a.n_split + split) * a.H + h) * a.Sq) * DV;
    o_row_stride = DV;
  }
#pragma unroll
  for (int hf = 0; hf < 2; hf++) {
#pragma unroll
    for (int dbl = 0; dbl < DB / 2; dbl++)
#pragma unroll
      for (int q4 = 0; q4 < 4; q4++) {
        x4 w;
#pragma unroll
        for (int i = 0; i < 4; i++) w[i] = (T)(o[hf * (DB / 2) + dbl][4 * q4 + i] * inv);
        lds_write<x4>(ob + r * OROW + (32 * dbl + 8 * q4 + 4 * g) * 2, w);
      }
#pragma unroll
    for (int it = 0; it < 32 * (HALF / 8) / 64; it++) {
      const int ci = lane + 64 * it, row = ci / (HALF / 8), c = ci % (HALF / 8);
      const u32x4 w = lds_read<u32x4>(ob + row * OROW + c * 16);
      if (m_wave + row < a.Sq) *(u32x4*)(obase + (int64_t)(m_wave + row) * o_row_stride + hf * HALF + c * 8) = w;
    }
  }
}

// Merge of the kv splits: o = sum_s exp(lse_s - lse) o_s with lse = log sum_s exp(lse_s) (examples/mha_decode.py:72-80).
// One wave per (batch, head, row); lanes cover the value columns.
template <typename T, int DV>
__global__ __launch_bounds__(256) void attn_split_combine_kernel(const AttnArgs a) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);   // (b * H + h) * Sq + m
  const int64_t rows = (int64_t)a.B * a.H * a.Sq;
  if (row >= rows) return;
  const int m = (int)(row % a.Sq), h = (int)((row / a.Sq) % a.H), b = (int)(row / ((int64_t)a.Sq * a.H));
  const int64_t part_row = ((int64_t)b * a.n_split * a.H + h) * a.Sq + m, split_stride = (int64_t)a.H * a.Sq;
  float mx = -INFINITY;
  for (int s = 0; s < a.n_split; s++) mx = fmaxf(mx, a.lse_part[part_row + s * split_stride]);
  float tot = 0.f;
  for (int s = 0; s < a.n_split; s++) {
    const float l = a.lse_part[part_row + s * split_stride];
    tot += l == -INFINITY ? 0.f : __expf(l - mx);
  }
  constexpr int PER = DV / 64;   // value columns per lane
  float acc[PER];
#pragma unroll
  for (int i = 0; i < PER; i++) acc[i] = 0.f;
  for (int s = 0; s < a.n_split; s++) {
    const float l = a.lse_part[part_row + s * split_stride];
    if (l == -INFINITY) continue;
    const float w = __expf(l - mx) / tot;
    const T* src = (const T*)a.o_part + (part_row + s * split_stride) * DV + lane * PER;
#pragma unroll
    for (int i = 0; i < PER; i++) acc[i] += w * (float)src[i];
  }
  T* dst = (T*)a.o + (int64_t)b * a.osb + (int64_t)m * a.oss + (int64_t)h * a.osh + lane * PER;
#pragma unroll
  for (int i = 0; i < PER; i++) dst[i] = (T)acc[i];
  if (a.row_scale && lane == 0) a.row_scale[row] = tot > 0.f ? mx + __logf(tot) : -INFINITY;
}

template <typename T, int DQK, int DV, int FAMILY, bool CAUSAL, int NW = 4>
static int launch_wide(const AttnArgs& a, hipStream_t stream) {
  constexpr size_t tiles = 2 * (size_t)32 * (pad_width(DQK) + DV) * 2;
  constexpr size_t ostage = NW * 32 * (size_t)(DV + 16);
  constexpr size_t lds = tiles > ostage ? tiles : ostage;
  auto kern = attn_wide_fwd_kernel<T, DQK, DV, FAMILY, CAUSAL, NW>;
  static std::atomic<uint64_t> lds_ok{0};
  if (allow_lds(lds_ok, lds, kern) != 0) return -1;
  AttnArgs args = a;
  if (args.n_split < 1) args.n_split = 1;
  args.num_m_blocks = (a.Sq + 32 * NW - 1) / (32 * NW);
  hipLaunchKernelGGL(kern, dim3((unsigned)(args.num_m_blocks * a.B * a.H * args.n_split)), dim3(64 * NW), lds, stream, args);
  if (args.n_split > 1) {
    const int64_t rows = (int64_t)a.B * a.H * a.Sq;
    hipLaunchKernelGGL((attn_split_combine_kernel<T, DV>), dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream, args);
  }
  return launch_status();
}

// Decode shapes: at most 32 query rows per (batch, head), softmax, no structural mask.  A one-wave workgroup takes one
// (batch, head, kv split); a CU holds four of them, or as many as their two tile stages fit into its 160 KB of LDS.  The
// split count is the one with the shortest schedule, counted in tiles: rounds of resident workgroups x (tiles per split +
// a workgroup's fixed cost), plus the merge, which grows with the splits; every split gets at least 8 tiles of 32 keys.
int attn_decode_splits(int family, bool causal, int B, int H, int Sq, int Skv, int dqk, int dv) {
  if (family != WF_SOFTMAX || causal || Sq > 32) return 1;
  if (!((dqk == 128 && dv == 128) || (dqk == 64 && dv == 64) || (dqk == 128 && dv == 256) || (dqk == 256 && dv == 256) || (dqk == 192 && dv == 128))) return 1;
  const int tiles = (Skv + 31) / 32;
  const int lds = 2 * 32 * (pad_width(dqk) + dv) * 2;
  int per_cu = (160 * 1024) / lds;
  if (per_cu > 4) per_cu = 4;
  const int64_t slots = (int64_t)per_cu * 256, groups = (int64_t)B * H;
  int n_max = tiles / 8;
  if (n_max > 64) n_max = 64;
  int best = 1;
  int64_t best_cost = -1;
  for (int n = 1; n <= n_max || n == 1; n++) {
    const int64_t rounds = (groups * n + slots - 1) / slots;
    const int64_t cost = 4 * rounds * ((tiles + n - 1) / n + 3) + n;      // (in quarter tiles)
    if (best_cost < 0 || cost < best_cost) {
      best_cost = cost;
      best = n;
    }
  }
  return best;
}

template <typename T, int DQK, int DV>
static int wide_family(const AttnArgs& a, int family, bool causal, hipStream_t stream) {
  switch (family) {
    case WF_SOFTMAX:
      if constexpr (DV <= 256) {
        if (!causal && a.Sq <= 32 && a.o_part) return launch_wide<T, DQK, DV, WF_SOFTMAX, false, 1>(a, stream);   // decode
      }
      return causal ? launch_wide<T, DQK, DV, WF_SOFTMAX, true>(a, stream) : launch_wide<T, DQK, DV, WF_SOFTMAX, false>(a, stream);
    case WF_SIGMOID:
      return causal ? launch_wide<T, DQK, DV, WF_SIGMOID, true>(a, stream) : launch_wide<T, DQK, DV, WF_SIGMOID, false>(a, stream);
    case WF_RELU:
      return causal ? launch_wide<T, DQK, DV, WF_RELU, true>(a, stream) : launch_wide<T, DQK, DV, WF_RELU, false>(a, stream);
  }
  return -2;
}

template <typename T>
static int wide_dims(const AttnArgs& a, int family, bool causal, int dqk, int dv, hipStream_t stream) {
  if (family == WF_RETENTION) {
    if (dqk == 256 && dv == 512) return retention_pair_fwd_dispatch(a, causal, std::is_same<T, __bf16>::value, stream);   // retention_fwd.hip
#define MA_RET_FWD(DQ, DVV) \
  if (dqk == DQ && dv == DVV) return causal ? launch_wide<T, DQ, DVV, WF_RETENTION, true>(a, stream) : launch_wide<T, DQ, DVV, WF_RETENTION, false>(a, stream);
    MA_RET_FWD(128, 128)
    MA_RET_FWD(64, 64)
    MA_RET_FWD(128, 256)
    MA_RET_FWD(256, 256)
#undef MA_RET_FWD
    return -2;
  }
  if (dqk == 128 && dv == 128) return wide_family<T, 128, 128>(a, family, causal, stream);   // (only with kv selection: see attn_fwd_dispatch)
  if (dqk == 64 && dv == 64) return wide_family<T, 64, 64>(a, family, causal, stream);
  if (dqk == 128 && dv == 256) return wide_family<T, 128, 256>(a, family, causal, stream);
  if (dqk == 256 && dv == 256) return wide_family<T, 256, 256>(a, family, causal, stream);
  if (dqk == 192 && dv == 128) return wide_family<T, 192, 128>(a, family, causal, stream);   // (the reference's DeepSeek-V2-Lite benchmark shape)
  if (dqk == 256 && dv == 512 && (family != WF_SOFTMAX || !(a.Sq <= 32 && a.o_part))) return wide_family<T, 256, 512>(a, family, causal, stream);
  // Softmax decode (split kv, one wave per workgroup) at 256/512: a workgroup's two tile stages would take 96 KB of LDS,
  // one wave per CU.  Given the probabilities the value columns are independent, so the two halves of V and of the
  // output go through the 256/256 decode kernel one after the other (the scores are computed twice; both launches write
  // the same row scales).
  if (dqk == 256 && dv == 512) {
    AttnArgs half = a;
    const int rc = wide_family<T, 256, 256>(half, family, causal, stream);
    if (rc != 0) return rc;
    half.v = (const T*)a.v + 256;
    half.o = (T*)a.o + 256;
    return wide_family<T, 256, 256>(half, family, causal, stream);
  }
  return -2;
}

// returns 0 ok, -1 launch failure, -2 unsupported
int attn_wide_fwd_dispatch(const AttnArgs& a, int family, bool causal, bool is_bf16, int dqk, int dv, hipStream_t stream) {
  // (the tile DMA addresses a tile's 32 rows with 32-bit byte offsets from its first row)
  for (int64_t row_stride : {a.kss, a.vss})
    if (row_stride < 0 || row_stride >= ((int64_t)1 << 26)) return -2;
  return is_bf16 ? wide_dims<__bf16>(a, family, causal, dqk, dv, stream) : wide_dims<_Float16>(a, family, causal, dqk, dv, stream);
}

}  // namespace ma
