// Parallel attention backward (dq, dk, dv) for gfx950: softmax, sigmoid and relu row functions.
//
// Replaces the backward of _attention (attention_engine/core/template/tl_template/attn/attn_tl.py:
// 669-692): the delta pre-pass (:212-237), the dK/dV kernel with fp32 dQ atomics (:301-420) and the
// dQ post-pass (:239-262).  With p = rowfn(x), x = s * scale + bias, s = q.k^T:
//   softmax   p = exp(x - lse),       ds = p * (dp - delta) * scale,   delta_i = sum_d do_id * o_id
//   sigmoid   p = 1 / (1 + exp(-x)),  ds = dp * p * (1 - p) * scale
//   relu      p = max(x, 0),          ds = dp * [x > 0] * scale
//   dp = do.v^T,   dv = p^T do,   dk = ds^T q,   dq = ds k
// (p and ds are rounded to the tensor dtype before the second products, as there: :357-362; the factor
// `scale` common to dq and dk is applied once, when their accumulators are stored).
// Masks: none, causal, or an element-wise keep mask given in both orientations (the dq kernel walks a
// query row of it, the dk / dv kernel a key's column of its transpose); only tiles that a mask can
// touch evaluate it.
//
// No atomics: two kernels, each owning its outputs.
//   attn_bwd_dq_kernel   a wave owns 32 query rows and walks the kv sequence; everything transposed as in
//                        the forward kernels (S^T = K Q^T, dP^T = V dO^T: lane = query row, so lse and
//                        delta are per-lane scalars; dS^T is directly the B operand of dQ^T += K^T dS^T).
//                        It also computes delta and leaves it in the workspace for the second kernel.
//   attn_bwd_dkv_kernel  a wave owns 32 keys of one kv head (K and V fragments in registers as B
//                        operands) and walks the query rows of every query head of its group; here
//                        S = Q K^T and dP = dO V^T are NOT transposed (lane = key), so P and dS are
//                        directly the B operands of dV^T += dO^T P and dK^T += Q^T dS; lse and delta of
//                        a tile's rows come with the tile.  dk and dv in one launch or in two (then the
//                        scores are computed once more), whichever lets two waves share a SIMD.
//   attn_bwd_dkv_fused_kernel  the same work at head sizes up to 128 / 128 (any mask): dk and dv in one launch,
//                        one wave per SIMD with the 512-register budget, persistent, the loop pipelined
//                        inside the wave (see there).
// The scores are recomputed in both kernels (7 tile products instead of 5; 8 where dk and dv take two
// launches), which is what avoiding the fp32 atomics and the post-pass costs.  Tiles of 32 rows arrive by
// direct-to-LDS DMA (a wave-uniform base in scalar registers plus 32-bit lane offsets computed once),
// through a ring of stages, one barrier per tile, XOR-swizzled like the forward tiles; the column-side
// operands (K^T, dO^T, Q^T) come from the same tiles through the transposing LDS read.
#pragma once
#include "attn_bwd.h"

namespace ma {

namespace {
enum { BF_SOFTMAX = 0, BF_SIGMOID = 1, BF_RELU = 2, BF_RETENTION = 3 };   // = MA_ATTN_* of the C interface

// ds / scale (and p) of one score element: the common factor `scale` of dq and dk is applied once, when the
// accumulators are stored.  x2 = (s * scale + bias) * log2(e) for softmax / sigmoid.
// Retention (examples/retention_parallel.py:76-86 of the reference): p = s * scale * m / r with m the caller's score
// multiplier and r the row scale of the forward pass, which the backward treats as a constant (dscores = dp / r);
// `lse2` carries m / r.
template <int FAMILY>
__device__ __forceinline__ void row_fn_bwd(float s, float dp, bool masked, float c_scale, float c_bias, float scale, float bias,
                                           float lse2, float delta, float& p, float& ds) {
  if constexpr (FAMILY == BF_RETENTION) {
    p = masked ? 0.f : s * scale * lse2;
    ds = masked ? 0.f : dp * lse2;
  } else if constexpr (FAMILY == BF_SOFTMAX) {
    p = masked ? 0.f : fast_exp2(s * c_scale + lse2);   // (lse2 = c_bias - lse * log2(e), folded by the caller)
    ds = p * (dp - delta);
  } else if constexpr (FAMILY == BF_SIGMOID) {
    p = masked ? 0.f : fast_rcp(1.f + fast_exp2(-(s * c_scale + c_bias)));
    ds = dp * p * (1.f - p);
  } else {
    const float x = s * scale + bias;
    p = masked ? 0.f : fmaxf(x, 0.f);
    ds = (!masked && x > 0.f) ? dp : 0.f;
  }
}

// The same in two parts, for the pipelined kernel: p of a kept score, and ds / scale from p.
template <int FAMILY>
__device__ __forceinline__ float row_p(float s, float c_scale, float c_bias, float scale, float bias, float lse2) {
  if constexpr (FAMILY == BF_SOFTMAX) return fast_exp2(s * c_scale + lse2);
  else if constexpr (FAMILY == BF_SIGMOID) return fast_rcp(1.f + fast_exp2(-(s * c_scale + c_bias)));
  else return fmaxf(s * scale + bias, 0.f);
}
template <int FAMILY>
__device__ __forceinline__ float row_ds(float p, float dp, float delta) {
  if constexpr (FAMILY == BF_SOFTMAX) return p * (dp - delta);
  else if constexpr (FAMILY == BF_SIGMOID) return dp * p * (1.f - p);
  else return p > 0.f ? dp : 0.f;
}

// EXTRA instantiations (softmax, sigmoid, relu): the additive terms and the soft-capping of the forward pass, applied to the recomputed
// raw scores.  `extra` is (add + slope_q q + slope_kv kv) of the element; the scores stay in units of 1 / scale, so that
// everything behind sees s * scale + bias as before.  With softcap > 0, x = s * scale + bias becomes softcap * tanh(x) and
// `cap_grad` the derivative softcap * (1 - tanh^2 x), which multiplies ds; tanh(x) = 1 - 2 / (1 + e^(2x)) as in the forward.
__device__ __forceinline__ float apply_extra(float s, float extra, float scale, float inv_scale, float bias, float softcap, float& cap_grad) {
  s += extra * inv_scale;
  cap_grad = 1.f;
  if (softcap > 0.f) {
    const float x = s * scale + bias;
    const float th = 1.f - 2.f * fast_rcp(1.f + fast_exp2(x * (2.f * kLog2e)));
    s = (softcap * th - bias) * inv_scale;
    cap_grad = softcap * (1.f - th * th);
  }
  return s;
}

// DMA of a [32 x ROWB bytes] tile whose rows are `row_stride` bytes apart in memory: each instruction
// moves 1 KB; lane i fetches the 16-byte chunk that belongs at physical position i of that KB.  Rows
// beyond `limit` are clamped to the last one (whatever is computed from them is masked).
template <int ROWB, int NWAVES, int USED = ROWB / 16>
__device__ __forceinline__ void dma_tile(const char* src, int64_t row_stride, int row0, int limit, uint32_t lds_base, int wave, int lane) {
  constexpr int CPR = ROWB / 16, NI = 32 * ROWB / 1024;
  for (int ii = wave; ii < NI; ii += NWAVES) {
    const int row = ii * (1024 / ROWB) + lane / CPR, c = lane % CPR;
    const int grow = min(row0 + row, limit - 1);
    if (USED == CPR || (c ^ swz_tile<CPR>(row)) < USED)   // (chunks beyond the head size do not exist in memory)
      dma16(src + grow * row_stride + ((c ^ swz_tile<CPR>(row)) << 4), lds_base + ii * 1024);
  }
}

// Stages of the pipelined dk / dv kernel's tile ring: eight (tiles arrive four steps ahead) where they fit the LDS, else four.
constexpr int fused_stages(int dqk, int dv) { return 8 * (32 * (dqk + dv) * 2 + 512) <= 150 * 1024 ? 8 : 4; }
// Waits until at most N of this wave's vector-memory loads are outstanding (they complete in order).
template <int N>
__device__ __forceinline__ void wait_dma_but() { __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14)); }

// Retention: a wave's [32 rows x 32 columns] block of the score multiplier (64 bytes per row) by DMA into a 2 KB area of
// its own, two instructions; the 16-byte chunk c of row r sits at position c ^ ((r >> 1) & 3) of the row, so that the
// 8-byte reads of `mult_read` (lane: row r, columns 8 q4 + 4 g ..) spread over the banks.  `first` points at the wave's
// first row and the block's first column; rows from `rows_left` on are clamped to the last one.
template <typename T>
__device__ __forceinline__ void mult_dma(const T* first, int64_t row_stride, int rows_left, uint32_t lds_base, int lane) {
#pragma unroll
  for (int j = 0; j < 2; j++) {
    const int row = (lane >> 2) + 16 * j, lc = (lane & 3) ^ ((row >> 1) & 3);
    dma16(first + (int64_t)min(row, rows_left - 1) * row_stride + 8 * lc, lds_base + j * 1024);
  }
}
template <typename T>
__device__ __forceinline__ typename Elem<T>::x4 mult_read(uint32_t lds_base, int r, int g, int q4) {
  return lds_read<typename Elem<T>::x4>(lds_base + r * 64 + ((q4 ^ ((r >> 1) & 3)) << 4) + 8 * g);
}

// Element-wise keep masks: a wave's [32 rows x 32 columns] block of mask bytes by DMA into a 1 KB area of its own (one
// instruction: two lanes per row); lane (row r, half g) then reads the four bytes of columns 8 q4 + 4 g .. as one word.
__device__ __forceinline__ void keep_dma(const uint8_t* first, int64_t row_stride, int rows_left, uint32_t lds_base, int lane) {
  dma16(first + (int64_t)min(lane >> 1, rows_left - 1) * row_stride + 16 * (lane & 1), lds_base);
}
__device__ __forceinline__ uint32_t keep_read(uint32_t lds_base, int r, int g, int q4) {
  return lds_read<uint32_t>(lds_base + r * 32 + 8 * q4 + 4 * g);
}

// [32 x 32] += A B^T over DIM columns, A = the 32 rows of an LDS tile (row reads), B = fragments in registers
template <typename T, int DIM>
__device__ __forceinline__ f32x16 mm_rows(uint32_t tile, int r, int g, const typename Elem<T>::x8 (&bf)[DIM / 16]) {
  using E = Elem<T>;
  using x8 = typename E::x8;
  constexpr int ROWB = pad_width(DIM) * 2, CPR = pad_width(DIM) / 8, KS = DIM / 16, AH = 2, RING = 3;
  // (tile bases and row offsets are multiples of the row size, so the swizzled chunk index has its own address
  // bits: another k-slice is one XOR with a constant away)
  const uint32_t a0 = tile + r * ROWB + (uint32_t)((g ^ swz_tile<CPR>(r)) << 4);
  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  f32x16 acc;
  x8 af[RING];
#pragma unroll
  for (int ks = 0; ks < AH && ks < KS; ks++) af[ks] = lds_read<x8>(a0 ^ (uint32_t)(ks * 32));
#pragma unroll
  for (int ks = 0; ks < KS; ks++) {
    if (ks + AH < KS) af[(ks + AH) % RING] = lds_read<x8>(a0 ^ (uint32_t)((ks + AH) * 32));
    __builtin_amdgcn_sched_barrier(0);
    acc = E::mfma32(af[ks % RING], bf[ks], ks == 0 ? zero16 : acc);
    __builtin_amdgcn_sched_barrier(0);
  }
  return acc;
}

// acc[DIM/32 blocks of 32 columns] += (tile columns)^T . pf, where pf holds a [32 x 32] factor in
// accumulator order rounded to T (k slot i of slice s for lane half g is tile row 16s + 8(i/4) + 4g + i%4,
// which is the row order the transposing reads below fetch)
struct NoHook { __device__ __forceinline__ void operator()(int, int) const {} };
// `between(idx, n)` runs behind MFMA idx of n: vector work that the matrix pipe covers
template <typename T, int DIM, typename Hook = NoHook>
__device__ __forceinline__ void mm_cols(uint32_t tile, int lane, const typename Elem<T>::x8 (&pf)[2], f32x16 (&acc)[DIM / 32], Hook between = Hook()) {
  using E = Elem<T>;
  using x8 = typename E::x8;
  using x4 = typename E::x4;
  constexpr int ROWB = pad_width(DIM) * 2, CPR = pad_width(DIM) / 8, NB = DIM / 32, PF = NB >= 2 ? 4 : 2;
  const int g = lane >> 5, jr = (lane & 15) >> 2;
  const int lc = (((lane >> 4) & 1) << 1) | ((lane & 3) >> 1);
  const uint32_t b0 = tile + (4 * g + jr) * ROWB + (lane & 1) * 8 + (uint32_t)((lc ^ swz_tile<CPR>(4 * g + jr)) << 4);
  x4 lo[PF], hi[PF];
  auto request = [&](int idx) {   // idx = 2 block + slice
    const int db = idx >> 1, sl = idx & 1;
    lo[idx % PF] = lds_read_tr4<T>((b0 ^ (uint32_t)((4 * db) << 4)) + 16 * sl * ROWB);
    hi[idx % PF] = lds_read_tr4<T>((b0 ^ (uint32_t)(((4 * db) ^ 2) << 4)) + (16 * sl + 8) * ROWB);
  };
#pragma unroll
  for (int i = 0; i < PF - 1; i++) request(i);
#pragma unroll
  for (int idx = 0; idx < 2 * NB; idx++) {
    if (idx + PF - 1 < 2 * NB) request(idx + PF - 1);
    __builtin_amdgcn_sched_barrier(0);
    x8 af = __builtin_shufflevector(lo[idx % PF], hi[idx % PF], 0, 1, 2, 3, 4, 5, 6, 7);
    acc[idx >> 1] = E::mfma32(af, pf[idx & 1], acc[idx >> 1]);
    between(idx, 2 * NB);
    __builtin_amdgcn_sched_barrier(0);
  }
}

// a wave's [DIM x 32] accumulator (lane = output row, elements = columns) to global rows of DIM
// elements, through a wave-private LDS block in two halves, 16-byte coalesced stores
template <typename T, int DIM>
__device__ __forceinline__ void store_rows(const f32x16 (&acc)[DIM / 32], float mult, uint32_t stage, T* gbase, int64_t row_stride,
                                           int row0, int row_limit, int lane) {
  using x4 = typename Elem<T>::x4;
  constexpr int NB = DIM / 32, HALF = DIM / 2, OROW = HALF * 2 + 16;
  const int r = lane & 31, g = lane >> 5;
#pragma unroll
  for (int hp = 0; hp < 2; hp++) {
#pragma unroll
    for (int dbl = 0; dbl < NB / 2; dbl++)
#pragma unroll
      for (int q4 = 0; q4 < 4; q4++) {
        x4 w;
#pragma unroll
        for (int i = 0; i < 4; i++) w[i] = (T)(acc[hp * (NB / 2) + dbl][4 * q4 + i] * mult);
        lds_write<x4>(stage + r * OROW + (32 * dbl + 8 * q4 + 4 * g) * 2, w);
      }
#pragma unroll
    for (int it = 0; it < 32 * (HALF / 8) / 64; it++) {
      const int ci = lane + 64 * it, row = ci / (HALF / 8), c = ci % (HALF / 8);
      const u32x4 w = lds_read<u32x4>(stage + row * OROW + c * 16);
      if (row0 + row < row_limit) *(u32x4*)(gbase + (int64_t)(row0 + row) * row_stride + hp * HALF + c * 8) = w;
    }
  }
}
}  // namespace

// ------------------------------------------------------------------------------------------------
// dq (and delta)
// ------------------------------------------------------------------------------------------------
template <typename T, int DQK, int DV, int FAMILY, bool CAUSAL, bool EXTRA = false>
__global__ __launch_bounds__(256, (DQK + DV >= 512 ? 1 : 2)) void attn_bwd_dq_kernel(const AttnBwdArgs a) {
  using E = Elem<T>;
  using x8 = typename E::x8;
  constexpr int BM = 128, BN = 32;
  constexpr int KS = DQK / 16, VS = DV / 16, QB = DQK / 32;
  constexpr int KROW = pad_width(DQK) * 2, VROW = DV * 2;   // (LDS rows; 192-wide keys sit in 256-wide rows)
  constexpr int KTILE = BN * KROW, VTILE = BN * VROW, STAGE = KTILE + VTILE;

  extern __shared__ __align__(16) char smem[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(MA_LDS char*)smem;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, g = lane >> 5;

  const int nmb = a.num_blocks, BH = a.B * a.H;
  int bh, mb;
  if ((BH & 7) == 0) {
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    bh = (slot / nmb) * 8 + xcd;
    mb = slot % nmb;
  } else {
    bh = blockIdx.x / nmb;
    mb = blockIdx.x % nmb;
  }
  if (CAUSAL) mb = nmb - 1 - mb;
  const int b = bh / a.H, h = bh % a.H, hk = h / a.kv_group;
  const int m_wave = mb * BM + wave * 32, m_lane = m_wave + r;
  const int m_ld = min(m_lane, a.Sq - 1);

  // B operands of this wave's 32 rows: Q (for S^T = K Q^T) and dO (for dP^T = V dO^T)
  x8 qf[KS], dof[VS];
  float delta = 0.f, lse2 = 0.f;
  {
    const T* qp = (const T*)a.q + (int64_t)b * a.qsb + (int64_t)m_ld * a.qss + (int64_t)h * a.qsh + 8 * g;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) qf[ks] = *(const x8*)(qp + 16 * ks);
    const T* dop = (const T*)a.dout + (int64_t)b * a.dosb + (int64_t)m_ld * a.doss + (int64_t)h * a.dosh + 8 * g;
#pragma unroll
    for (int sl = 0; sl < VS; sl++) dof[sl] = *(const x8*)(dop + 16 * sl);
    if constexpr (FAMILY == BF_SOFTMAX) {
      const T* op = (const T*)a.o + (int64_t)b * a.osb + (int64_t)m_ld * a.oss + (int64_t)h * a.osh + 8 * g;
      float part = 0.f;
#pragma unroll
      for (int sl = 0; sl < VS; sl++) {
        const x8 of = *(const x8*)(op + 16 * sl);
#pragma unroll
        for (int i = 0; i < 8; i++) part += (float)dof[sl][i] * (float)of[i];
      }
      delta = part + xhalf(part);
      const int64_t ri = ((int64_t)b * a.H + h) * a.Sq + m_ld;
      lse2 = a.lse[ri] * kLog2e;
      if (g == 0 && m_lane < a.Sq) a.delta[ri] = delta;
    }
  }
  float r_inv = 1.f;   // retention: 1 / the row scale of the forward pass
  if constexpr (FAMILY == BF_RETENTION) r_inv = 1.f / a.lse[((int64_t)b * a.H + h) * a.Sq + m_ld];
  // retention: this lane's row of the score multiplier
  const T* sm_row = FAMILY == BF_RETENTION ? (const T*)a.smask + (int64_t)b * a.sm_sb + (int64_t)h * a.sm_sh + (int64_t)m_ld * a.sm_sq : nullptr;
  const char* kb = (const char*)((const T*)a.k + (int64_t)b * a.ksb + (int64_t)hk * a.ksh);
  const char* vb = (const char*)((const T*)a.v + (int64_t)b * a.vsb + (int64_t)hk * a.vsh);
  const int64_t k_row_bytes = a.kss * 2, v_row_bytes = a.vss * 2;

  int n_tiles = (a.Skv + BN - 1) / BN;
  if (CAUSAL) n_tiles = min(n_tiles, (mb * BM + BM + BN - 1) / BN);

  // retention: whole tiles of the multiplier come with the K/V tile (a 2 KB area per wave and stage behind the stages);
  // a partial last tile, or a tensor whose rows are not 16-byte aligned, is read from global memory as it is needed
  constexpr int MULT = 2 * STAGE;
  const bool mult_ok = FAMILY == BF_RETENTION && (a.sm_sq & 7) == 0 && (a.sm_sb & 7) == 0 && (a.sm_sh & 7) == 0 && ((uintptr_t)a.smask & 15) == 0;
  const bool keep_ok = FAMILY != BF_RETENTION && a.elem_mask && ((a.em_sq | a.em_sb | a.em_sh | (int64_t)(uintptr_t)a.elem_mask) & 15) == 0;
  const uint8_t* bm_full = a.kv_block_mask ? a.kv_block_mask + (int64_t)b * a.kbm_sb + (int64_t)h * a.kbm_sh + (int64_t)mb * a.kbm_sq : nullptr;
  auto tile_full = [&](int jt_) { return bm_full && bm_full[jt_] >= 2; };   // the element-wise mask keeps every score of the tile
  TileDma<KROW, 4, DQK / 8> k_dma;
  TileDma<VROW, 4> v_dma;
  k_dma.init((uint32_t)k_row_bytes, wave, lane);
  v_dma.init((uint32_t)v_row_bytes, wave, lane);
  auto issue_tile = [&](int n0, int buf) {
    if (n0 + BN <= a.Skv) {   // (wave-uniform)
      k_dma.issue(kb + (int64_t)n0 * k_row_bytes, lds0 + buf * STAGE, wave);
      v_dma.issue(vb + (int64_t)n0 * v_row_bytes, lds0 + buf * STAGE + KTILE, wave);
    } else {
      dma_tile<KROW, 4, DQK / 8>(kb, k_row_bytes, n0, a.Skv, lds0 + buf * STAGE, wave, lane);
      dma_tile<VROW, 4>(vb, v_row_bytes, n0, a.Skv, lds0 + buf * STAGE + KTILE, wave, lane);
    }
    if constexpr (FAMILY == BF_RETENTION) {
      if (mult_ok && n0 + BN <= a.Skv && m_wave < a.Sq)
        mult_dma<T>((const T*)a.smask + (int64_t)b * a.sm_sb + (int64_t)h * a.sm_sh + (int64_t)m_wave * a.sm_sq + n0, a.sm_sq, a.Sq - m_wave,
                    lds0 + MULT + (buf * 4 + wave) * 2048, lane);
    } else {
      // element-wise keep mask: whole tiles of a 16-byte aligned mask come with the K/V tile (same area, 1 KB per wave and
      // stage); a tile the block mask marks as kept in full (entry 2) needs none of it
      if (keep_ok && n0 + BN <= a.Skv && m_wave < a.Sq && !tile_full(n0 / BN))
        keep_dma(a.elem_mask + (int64_t)b * a.em_sb + (int64_t)h * a.em_sh + (int64_t)m_wave * a.em_sq + n0, a.em_sq, a.Sq - m_wave,
                 lds0 + MULT + (buf * 4 + wave) * 1024, lane);
    }
  };

  f32x16 dq[QB];
#pragma unroll
  for (int i = 0; i < QB; i++)
#pragma unroll
    for (int j = 0; j < 16; j++) dq[i][j] = 0.f;
  const float bias = a.bias + (a.bias_ptr ? *a.bias_ptr : 0.f);
  const float c_scale = a.scale * kLog2e, c_bias = bias * kLog2e;
  lse2 = c_bias - lse2;   // what the row function adds to s * c_scale

  // element-wise keep mask of this lane's query row
  const uint8_t* em_row = a.elem_mask ? a.elem_mask + (int64_t)b * a.em_sb + (int64_t)h * a.em_sh + (int64_t)m_ld * a.em_sq : nullptr;

  // tiles in which the mask keeps nothing for this workgroup's rows are never fetched
  const uint8_t* bm_row = a.kv_block_mask ? a.kv_block_mask + (int64_t)b * a.kbm_sb + (int64_t)h * a.kbm_sh + (int64_t)mb * a.kbm_sq : nullptr;
  auto next_tile = [&](int jt) {
    if (bm_row)
      while (jt < n_tiles && !bm_row[jt]) jt++;
    return jt;
  };

  int jt = next_tile(0);
  if (jt < n_tiles) issue_tile(jt * BN, 0);
  for (int it = 0; jt < n_tiles; it++) {
    const int buf = it & 1, n0 = jt * BN;
    wait_dma();
    __syncthreads();
    jt = next_tile(jt + 1);
    if (jt < n_tiles) issue_tile(jt * BN, buf ^ 1);
    const uint32_t kbase = lds0 + buf * STAGE, vbase = kbase + KTILE;

    // retention: the multipliers of this lane's 16 scores, requested before the products that hide their latency
    typename E::x4 mk[4];
    if constexpr (FAMILY == BF_RETENTION) {
      if (mult_ok && n0 + BN <= a.Skv && m_wave < a.Sq) {
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) mk[q4] = mult_read<T>(lds0 + MULT + (buf * 4 + wave) * 2048, r, g, q4);
      } else {
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
          const int n = n0 + 8 * q4 + 4 * g;
          if (n + 3 < a.Skv) {
            mk[q4] = *(const typename E::x4*)(sm_row + n);
          } else {
#pragma unroll
            for (int i = 0; i < 4; i++) mk[q4][i] = n + i < a.Skv ? sm_row[n + i] : (T)0.f;
          }
        }
      }
    }
    f32x16 s = mm_rows<T, DQK>(kbase, r, g, qf);           // S^T: lane = row m_lane, element jj = key n0 + 8(jj/4) + 4g + jj%4
    const f32x16 dp = mm_rows<T, DV>(vbase, r, g, dof);   // dP^T, same layout
    x8 dsf[2];
    float cap_grad[16];
    if constexpr (EXTRA) {
      const float inv_scale = 1.f / a.scale;
      const float sl_q = a.slope_q ? a.slope_q[h] * (float)m_ld : 0.f, sl_kv = a.slope_kv ? a.slope_kv[h] : 0.f;
      const int64_t add_row = (int64_t)b * a.add_sb + (int64_t)h * a.add_sh + (int64_t)m_ld * a.add_sq;
#pragma unroll
      for (int jj = 0; jj < 16; jj++) {
        const int n = min(n0 + 8 * (jj >> 2) + 4 * g + (jj & 3), a.Skv - 1);
        float e = sl_q + sl_kv * (float)n;
        if (a.add) e += a.add_f32 ? ((const float*)a.add)[add_row + (int64_t)n * a.add_sk] : (float)((const T*)a.add)[add_row + (int64_t)n * a.add_sk];
        s[jj] = apply_extra(s[jj], e, a.scale, inv_scale, bias, a.softcap, cap_grad[jj]);
      }
    }
    float mr[16];   // retention: multiplier / r per element
    if constexpr (FAMILY == BF_RETENTION) {
#pragma unroll
      for (int jj = 0; jj < 16; jj++) mr[jj] = (float)mk[jj >> 2][jj & 3] * r_inv;
    }
    // only tiles that touch the diagonal or the end of the keys pay for the mask (the test is wave-uniform);
    // with an element-wise mask every tile does
    const bool full = tile_full(n0 / BN);
    if ((CAUSAL && n0 + BN - 1 > m_wave) || n0 + BN > a.Skv || (em_row && !full)) {
      uint32_t keep[4] = {0x01010101u, 0x01010101u, 0x01010101u, 0x01010101u};   // the bytes of this lane's four keys per group
      if (full) {
      } else if (keep_ok && n0 + BN <= a.Skv && m_wave < a.Sq) {
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) keep[q4] = keep_read(lds0 + MULT + (buf * 4 + wave) * 1024, r, g, q4);
      } else if (em_row) {
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
          const int n = n0 + 8 * q4 + 4 * g;
          if (n + 3 < a.Skv) {
            keep[q4] = *(const uint32_t*)(em_row + n);
          } else {
            keep[q4] = 0;
#pragma unroll
            for (int i = 0; i < 4; i++)
              if (n + i < a.Skv) keep[q4] |= (uint32_t)em_row[n + i] << (8 * i);
          }
        }
      }
#pragma unroll
      for (int jj = 0; jj < 16; jj++) {
        const int n = n0 + 8 * (jj >> 2) + 4 * g + (jj & 3);
        const bool masked = (CAUSAL && n > m_lane) || n >= a.Skv || ((keep[jj >> 2] >> (8 * (jj & 3))) & 0xffu) == 0;
        float p, ds;
        row_fn_bwd<FAMILY>(s[jj], dp[jj], masked, c_scale, c_bias, a.scale, bias, FAMILY == BF_RETENTION ? mr[jj] : lse2, delta, p, ds);
        if constexpr (EXTRA) ds *= cap_grad[jj];
        dsf[jj >> 3][jj & 7] = (T)ds;
      }
    } else {
#pragma unroll
      for (int jj = 0; jj < 16; jj++) {
        float p, ds;
        row_fn_bwd<FAMILY>(s[jj], dp[jj], false, c_scale, c_bias, a.scale, bias, FAMILY == BF_RETENTION ? mr[jj] : lse2, delta, p, ds);
        if constexpr (EXTRA) ds *= cap_grad[jj];
        dsf[jj >> 3][jj & 7] = (T)ds;
      }
    }
    mm_cols<T, DQK>(kbase, lane, dsf, dq);                 // dQ^T += K^T dS^T
  }
  __syncthreads();   // every wave is done with the tiles: they become output staging

  constexpr int OROW = DQK + 16;
  T* dqb = (T*)a.dq + (int64_t)b * a.dqsb + (int64_t)h * a.dqsh;
  store_rows<T, DQK>(dq, a.scale, lds0 + wave * 32 * OROW, dqb, a.dqss, m_wave, a.Sq, lane);
}

// ------------------------------------------------------------------------------------------------
// dk, dv
// ------------------------------------------------------------------------------------------------
// WHAT: 3 = dk and dv in one launch, 1 = dv only, 2 = dk only.  Both [D x 32] accumulators plus the K and V
// fragments take 192 registers at 128/128, which leaves one wave per SIMD (forcing two makes the compiler
// spill the fragments and is slower); computing dv and dk in two launches (the scores are then computed once
// more) lets each run two waves per SIMD.
template <typename T, int DQK, int DV, int FAMILY, bool CAUSAL, int WHAT, bool EXTRA = false>
__global__ __launch_bounds__(256, (WHAT == 3 ? (DQK + DV >= 256 ? 1 : 2) : (DQK + DV >= 512 ? 1 : 2))) void attn_bwd_dkv_kernel(const AttnBwdArgs a) {
  constexpr bool DO_DV = (WHAT & 1) != 0, DO_DK = (WHAT & 2) != 0;
  using E = Elem<T>;
  using x8 = typename E::x8;
  constexpr int BNW = 128, BMT = 32;   // keys per workgroup, query rows per tile
  constexpr int KS = DQK / 16, VS = DV / 16, QB = DQK / 32, VB = DV / 32;
  constexpr int QROW = pad_width(DQK) * 2, DOROW = DV * 2;   // (LDS rows; 192-wide queries sit in 256-wide rows)
  // a stage: the Q tile and the dO tile; behind both stages, lse and delta of each stage's 32 rows (softmax; 2 x 128
  // bytes per stage -- not inside the stages: the swizzled reads address a tile as base XOR offset, which needs the
  // tile bases aligned to the row size)
  constexpr int QTILE = BMT * QROW, DOTILE = BMT * DOROW, STAGE = QTILE + DOTILE, ROWVALS = 2 * STAGE;
  // retention: behind those, a 2 KB block of the transposed multiplier per wave and stage (see the dq kernel)
  constexpr int MULT = ROWVALS + 1024;

  extern __shared__ __align__(16) char smem[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(MA_LDS char*)smem;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, g = lane >> 5;

  const int nnb = a.num_blocks, BHK = a.B * a.Hkv;
  int bhk, nb;
  if ((BHK & 7) == 0) {
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    bhk = (slot / nnb) * 8 + xcd;
    nb = slot % nnb;
  } else {
    bhk = blockIdx.x / nnb;
    nb = blockIdx.x % nnb;
  }
  const int b = bhk / a.Hkv, hk = bhk % a.Hkv;
  const int n_wave = nb * BNW + wave * 32, n_lane = n_wave + r;
  const int n_ld = min(n_lane, a.Skv - 1);

  // B operands of this wave's 32 keys: K (for S = Q K^T) and V (for dP = dO V^T)
  x8 kf[KS], vf[VS];
  {
    const T* kp = (const T*)a.k + (int64_t)b * a.ksb + (int64_t)n_ld * a.kss + (int64_t)hk * a.ksh + 8 * g;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) kf[ks] = *(const x8*)(kp + 16 * ks);
    const T* vp = (const T*)a.v + (int64_t)b * a.vsb + (int64_t)n_ld * a.vss + (int64_t)hk * a.vsh + 8 * g;
#pragma unroll
    for (int sl = 0; sl < VS; sl++) vf[sl] = *(const x8*)(vp + 16 * sl);
  }
  f32x16 dk[QB], dv[VB];
#pragma unroll
  for (int i = 0; i < QB; i++)
#pragma unroll
    for (int j = 0; j < 16; j++) dk[i][j] = 0.f;
#pragma unroll
  for (int i = 0; i < VB; i++)
#pragma unroll
    for (int j = 0; j < 16; j++) dv[i][j] = 0.f;
  const float bias = a.bias + (a.bias_ptr ? *a.bias_ptr : 0.f);
  const float c_scale = a.scale * kLog2e, c_bias = bias * kLog2e;

  // query tiles that can see this workgroup's keys, for every query head of the kv head's group
  const int t_first = CAUSAL ? (nb * BNW) / BMT : 0;
  const int t_count = (a.Sq + BMT - 1) / BMT - t_first;
  const int n_steps = t_count > 0 ? t_count * a.kv_group : 0;
  const int64_t q_row_bytes = a.qss * 2, do_row_bytes = a.doss * 2;
  // tiles in which the mask keeps nothing for this workgroup's keys are never fetched
  const uint8_t* qbm = a.q_block_mask ? a.q_block_mask + (int64_t)b * a.qbm_sb + (int64_t)nb * a.qbm_sk : nullptr;
  // (entry 2: the element-wise mask keeps every score of the tile)
  // a step = (query head of the group, tile of that head's rows), counted without divisions
  struct Pos { int step, hg, t; };
  auto advance = [&](Pos& p) {
    p.step++;
    if (++p.t == t_count) { p.t = 0; p.hg++; }
  };
  auto qbm_at = [&](const Pos& p) { return qbm[(int64_t)(hk * a.kv_group + p.hg) * a.qbm_sh + t_first + p.t]; };
  auto step_full = [&](const Pos& p) { return qbm && qbm_at(p) >= 2; };
  auto skip_empty = [&](Pos& p) {
    if (qbm)
      while (p.step < n_steps && !qbm_at(p)) advance(p);
  };
  const bool keep_ok = FAMILY != BF_RETENTION && a.elem_mask_t && ((a.emt_sk | a.emt_sb | a.emt_sh | (int64_t)(uintptr_t)a.elem_mask_t) & 15) == 0;
  const bool mult_ok = FAMILY == BF_RETENTION && (a.smt_sk & 7) == 0 && (a.smt_sb & 7) == 0 && (a.smt_sh & 7) == 0 && ((uintptr_t)a.smask_t & 15) == 0;
  TileDma<QROW, 4, DQK / 8> q_dma;
  TileDma<DOROW, 4> do_dma;
  q_dma.init((uint32_t)q_row_bytes, wave, lane);
  do_dma.init((uint32_t)do_row_bytes, wave, lane);
  auto issue_step = [&](const Pos& step, int buf) {
    const int h = hk * a.kv_group + step.hg, m0 = (t_first + step.t) * BMT;
    const char* qb = (const char*)((const T*)a.q + (int64_t)b * a.qsb + (int64_t)h * a.qsh);
    const char* dob = (const char*)((const T*)a.dout + (int64_t)b * a.dosb + (int64_t)h * a.dosh);
    if (m0 + BMT <= a.Sq) {   // (wave-uniform)
      q_dma.issue(qb + (int64_t)m0 * q_row_bytes, lds0 + buf * STAGE, wave);
      do_dma.issue(dob + (int64_t)m0 * do_row_bytes, lds0 + buf * STAGE + QTILE, wave);
    } else {
      dma_tile<QROW, 4, DQK / 8>(qb, q_row_bytes, m0, a.Sq, lds0 + buf * STAGE, wave, lane);
      dma_tile<DOROW, 4>(dob, do_row_bytes, m0, a.Sq, lds0 + buf * STAGE + QTILE, wave, lane);
    }
    if constexpr (FAMILY == BF_SOFTMAX) {
      // lse (lanes 0..31) and delta (lanes 32..63) of the tile's rows come with it: read from global memory inside
      // the loop, their latency is not covered by the little work a tile is
      // (wave 0 fetches lse, wave 1 delta: a scalar base and the lane's row; the upper lanes repeat the lower ones into
      // the other half of the wave's 256 bytes)
      if (wave < 2) {
        const float* src = (wave == 0 ? a.lse : (const float*)a.delta) + ((int64_t)b * a.H + h) * a.Sq + m0;
        dma4_so(src, (uint32_t)(min(m0 + (lane & 31), a.Sq - 1) - m0) * 4u, lds0 + ROWVALS + buf * 512 + wave * 256);
      }
    }
    if constexpr (FAMILY == BF_RETENTION) {
      // the row scales r of the tile's rows (twice: both halves of the wave fetch them) and, for whole tiles of an
      // aligned tensor, each wave's block of the transposed multiplier
      if (wave == 0)
        dma4_so(a.lse + ((int64_t)b * a.H + h) * a.Sq + m0, (uint32_t)(min(m0 + (lane & 31), a.Sq - 1) - m0) * 4u, lds0 + ROWVALS + buf * 512);
      if (mult_ok && m0 + BMT <= a.Sq && n_wave < a.Skv)
        mult_dma<T>((const T*)a.smask_t + (int64_t)b * a.smt_sb + (int64_t)h * a.smt_sh + (int64_t)n_wave * a.smt_sk + m0, a.smt_sk, a.Skv - n_wave,
                    lds0 + MULT + (buf * 4 + wave) * 2048, lane);
    } else {
      // the transposed element-wise keep mask: whole tiles of a 16-byte aligned mask come with the Q/dO tile
      if (keep_ok && m0 + BMT <= a.Sq && n_wave < a.Skv && !step_full(step))
        keep_dma(a.elem_mask_t + (int64_t)b * a.emt_sb + (int64_t)h * a.emt_sh + (int64_t)n_wave * a.emt_sk + m0, a.emt_sk, a.Skv - n_wave,
                 lds0 + MULT + (buf * 4 + wave) * 1024, lane);
    }
  };

  Pos step_next = {0, 0, 0};
  skip_empty(step_next);
  if (step_next.step < n_steps) issue_step(step_next, 0);
  for (int it = 0; step_next.step < n_steps; it++) {
    const int buf = it & 1;
    const Pos step = step_next;
    const int h = hk * a.kv_group + step.hg, m0 = (t_first + step.t) * BMT;
    wait_dma();
    __syncthreads();
    advance(step_next);
    skip_empty(step_next);
    if (step_next.step < n_steps) issue_step(step_next, buf ^ 1);
    // (a wave whose keys all lie behind this tile's rows has nothing to add; it still takes part in the barriers.  With
    // the large accumulators of the 256 / 512 head size the second way round the loop costs register copies that spill,
    // and the few such tiles are computed instead: every element of them is masked)
    if (CAUSAL && DQK + DV < 768 && m0 + BMT - 1 < n_wave) continue;
    const uint32_t qbase = lds0 + buf * STAGE, dobase = qbase + QTILE;

    // retention: 1 / r of the rows this lane holds and the multipliers of its 16 scores (from the transposed
    // multiplier tensor: this key's row, indexed by query position)
    float lse2[16], dl[16];
    if constexpr (FAMILY == BF_RETENTION) {
      const uint32_t rv = lds0 + ROWVALS + buf * 512;
      const T* smt_row = (const T*)a.smask_t + (int64_t)b * a.smt_sb + (int64_t)h * a.smt_sh + (int64_t)n_ld * a.smt_sk;
      const bool staged = mult_ok && m0 + BMT <= a.Sq && n_wave < a.Skv;
#pragma unroll
      for (int q4 = 0; q4 < 4; q4++) {
        const int m = m0 + 8 * q4 + 4 * g;
        const f32x4 tr = lds_read<f32x4>(rv + (8 * q4 + 4 * g) * 4);
        typename E::x4 tm;
        if (staged) {
          tm = mult_read<T>(lds0 + MULT + (buf * 4 + wave) * 2048, r, g, q4);
        } else {
#pragma unroll
          for (int i = 0; i < 4; i++) tm[i] = smt_row[min(m + i, a.Sq - 1)];
        }
#pragma unroll
        for (int i = 0; i < 4; i++) lse2[4 * q4 + i] = (float)tm[i] * fast_rcp(tr[i]);
      }
    }
    // lse and delta of the rows this lane holds: m0 + 8q4 + 4g + {0..3}
    if constexpr (FAMILY == BF_SOFTMAX) {
      const uint32_t rv = lds0 + ROWVALS + buf * 512;
#pragma unroll
      for (int q4 = 0; q4 < 4; q4++) {
        const f32x4 tl = lds_read<f32x4>(rv + (8 * q4 + 4 * g) * 4);
        const f32x4 td = lds_read<f32x4>(rv + 256 + (8 * q4 + 4 * g) * 4);
#pragma unroll
        for (int i = 0; i < 4; i++) {
          lse2[4 * q4 + i] = c_bias - tl[i] * kLog2e;   // what the row function adds to s * c_scale
          dl[4 * q4 + i] = td[i];
        }
      }
    }
    f32x16 s = mm_rows<T, DQK>(qbase, r, g, kf);           // S: lane = key n_lane, element jj = row m0 + 8(jj/4) + 4g + jj%4
    float cap_grad[16];
    if constexpr (EXTRA) {
      const float inv_scale = 1.f / a.scale;
      const float sl_q = a.slope_q ? a.slope_q[h] : 0.f, sl_kv = a.slope_kv ? a.slope_kv[h] * (float)n_ld : 0.f;
      const int64_t add_col = (int64_t)b * a.add_sb + (int64_t)h * a.add_sh + (int64_t)n_ld * a.add_sk;
#pragma unroll
      for (int jj = 0; jj < 16; jj++) {
        const int m = min(m0 + 8 * (jj >> 2) + 4 * g + (jj & 3), a.Sq - 1);
        float e = sl_q * (float)m + sl_kv;
        if (a.add) e += a.add_f32 ? ((const float*)a.add)[add_col + (int64_t)m * a.add_sq] : (float)((const T*)a.add)[add_col + (int64_t)m * a.add_sq];
        s[jj] = apply_extra(s[jj], e, a.scale, inv_scale, bias, a.softcap, cap_grad[jj]);
      }
    }
    f32x16 dp;
    if constexpr (DO_DK) dp = mm_rows<T, DV>(dobase, r, g, vf);   // dP, same layout
    else
#pragma unroll
      for (int j = 0; j < 16; j++) dp[j] = 0.f;
    x8 pf[2], dsf[2];
    // only tiles that touch the diagonal or an end of the sequences pay for the mask (the test is wave-uniform);
    // with an element-wise mask every tile does
    const bool full = step_full(step);
    if ((CAUSAL && n_wave + 31 > m0) || m0 + BMT > a.Sq || n_wave + 32 > a.Skv || (a.elem_mask_t && !full)) {
      uint32_t keep[4] = {0x01010101u, 0x01010101u, 0x01010101u, 0x01010101u};   // the bytes of this lane's four rows per group
      if (full) {
      } else if (keep_ok && m0 + BMT <= a.Sq && n_wave < a.Skv) {
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) keep[q4] = keep_read(lds0 + MULT + (buf * 4 + wave) * 1024, r, g, q4);
      } else if (a.elem_mask_t) {
        // the transposed mask: this key's row, indexed by query position
        const uint8_t* emt_row = a.elem_mask_t + (int64_t)b * a.emt_sb + (int64_t)h * a.emt_sh + (int64_t)n_ld * a.emt_sk;
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
          const int m = m0 + 8 * q4 + 4 * g;
          if (m + 3 < a.Sq) {
            keep[q4] = *(const uint32_t*)(emt_row + m);
          } else {
            keep[q4] = 0;
#pragma unroll
            for (int i = 0; i < 4; i++)
              if (m + i < a.Sq) keep[q4] |= (uint32_t)emt_row[m + i] << (8 * i);
          }
        }
      }
#pragma unroll
      for (int jj = 0; jj < 16; jj++) {
        const int m = m0 + 8 * (jj >> 2) + 4 * g + (jj & 3);
        const bool masked = (CAUSAL && n_lane > m) || m >= a.Sq || n_lane >= a.Skv || ((keep[jj >> 2] >> (8 * (jj & 3))) & 0xffu) == 0;
        float p, ds;
        row_fn_bwd<FAMILY>(s[jj], dp[jj], masked, c_scale, c_bias, a.scale, bias, FAMILY == BF_SOFTMAX || FAMILY == BF_RETENTION ? lse2[jj] : 0.f,
                           FAMILY == BF_SOFTMAX ? dl[jj] : 0.f, p, ds);
        if (masked) ds = 0.f;
        if constexpr (EXTRA) ds *= cap_grad[jj];
        pf[jj >> 3][jj & 7] = (T)p;
        dsf[jj >> 3][jj & 7] = (T)ds;
      }
    } else {
#pragma unroll
      for (int jj = 0; jj < 16; jj++) {
        float p, ds;
        row_fn_bwd<FAMILY>(s[jj], dp[jj], false, c_scale, c_bias, a.scale, bias, FAMILY == BF_SOFTMAX || FAMILY == BF_RETENTION ? lse2[jj] : 0.f,
                           FAMILY == BF_SOFTMAX ? dl[jj] : 0.f, p, ds);
        if constexpr (EXTRA) ds *= cap_grad[jj];
        pf[jj >> 3][jj & 7] = (T)p;
        dsf[jj >> 3][jj & 7] = (T)ds;
      }
    }
    if constexpr (DO_DV) mm_cols<T, DV>(dobase, lane, pf, dv);     // dV^T += dO^T P
    if constexpr (DO_DK) mm_cols<T, DQK>(qbase, lane, dsf, dk);    // dK^T += Q^T dS
  }
  __syncthreads();   // every wave is done with the tiles: they become output staging

  constexpr int DMAX = DQK > DV ? DQK : DV, OROW = DMAX + 16;
  const uint32_t stage = lds0 + wave * 32 * OROW;
  T* dkb = (T*)a.dk + (int64_t)b * a.dksb + (int64_t)hk * a.dksh;
  T* dvb = (T*)a.dv + (int64_t)b * a.dvsb + (int64_t)hk * a.dvsh;
  if constexpr (DO_DK) store_rows<T, DQK>(dk, a.scale, stage, dkb, a.dkss, n_wave, a.Skv, lane);
  if constexpr (DO_DV) store_rows<T, DV>(dv, 1.f, stage, dvb, a.dvss, n_wave, a.Skv, lane);
}


// ------------------------------------------------------------------------------------------------
// dk and dv in one launch: one wave per SIMD, software pipelined
// ------------------------------------------------------------------------------------------------
// Where the K and V fragments and both [D x 32] accumulators of a wave's 32 keys fit the 512 registers of a wave that has its
// SIMD to itself, dk and dv share the recomputed scores (7 tile products in all instead of 8).  With no second wave on the
// SIMD to fill the matrix pipe while one evaluates the row function or waits for LDS, the loop is pipelined inside the
// wave.  A step is ONE sequence of MFMAs:
//   phase F  S(u+1) = Q(u+1) K^T and dP(u+1) = dO(u+1) V^T of the NEXT tile, with p of the current step's 16 score elements
//            spread behind them,
//   phase V  dV^T += dO(u)^T P(u), with ds of the 16 elements behind them,
//   phase K  dK^T += Q(u)^T dS(u),
// whose LDS operand fragments travel through one ring of registers, requested AH MFMAs ahead across the phases and across
// steps (the last MFMAs of phase K request the first fragments of the next step).  Tiles come through a ring of stages, LA
// steps ahead; the step's single barrier sits between phases V and K: behind it tile u+2 is visible to every wave, and
// every wave is done with tile u-1, whose stage takes tile u+LA.  lse and delta of a tile's rows come with it.  The loop
// body is written for two steps (the registers of "this" and "the next" step swap roles) so that nothing is copied; an odd
// number of steps is padded with a step in which everything is masked.  Masked scores are set to -inf (times the sign
// of scale) before the row function, in the few tiles that touch the diagonal or an end of the sequences: p = 0 and so
// ds = 0 follow.  The retention family and the larger head sizes take the two-launch kernels above.
template <int I>
struct IntC { static constexpr int value = I; };
template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {   // f(IntC<I>()), ..., f(IntC<N - 1>()): indices that are constants by construction
  if constexpr (I < N) {
    f(IntC<I>());
    static_for<I + 1, N>(f);
  }
}

template <typename T>
struct FusedStepRegs {
  f32x16 s, dp;        // S and dP of the step's tile (lane = key, element jj = row 8(jj/4) + 4g + jj%4 of the tile)
  f32x4 tl[4], td[4];  // lse and delta of those rows (softmax)
};

// MASKS: with an element-wise keep mask (its transpose: a lane walks a key's column) and / or a tile mask.  The steps of a
// key block are then a list in LDS, built by wave 0 before the loop: the (query head, tile) pairs whose tile-mask entry is
// not 0, each with the flag "kept in full" (entry 2: the element mask is not consulted).  A wave's [32 x 32] block of mask
// bytes comes with the tile (whole tiles of a 16-byte aligned mask; others are read from global memory), and the
// masked scores are set to -inf in the same place as for the structural masks.
constexpr int FUSED_LIST_MAX = 2048;   // steps of a key block that the list holds (the launcher checks)
// Phase F of a step alternates the k slices of S and dP while both have some left, then finishes the longer contraction:
// MFMA j of the phase is slice `slice(j)` of S (`is_s(j)`) or of dP.
template <int KS, int VS>
struct PhaseF {
  static constexpr int KMIN = KS < VS ? KS : VS;
  static constexpr bool is_s(int j) { return j < 2 * KMIN ? j % 2 == 0 : KS > VS; }
  static constexpr int slice(int j) { return j < 2 * KMIN ? j / 2 : KMIN + (j - 2 * KMIN); }
};
template <typename T, int DQK, int DV, int FAMILY, bool CAUSAL, bool MASKS>
__global__ __launch_bounds__(256, 1) void attn_bwd_dkv_fused_kernel(const AttnBwdArgs a) {
  using E = Elem<T>;
  using x8 = typename E::x8;
  using x4 = typename E::x4;
  constexpr int BNW = 128, BMT = 32;
  constexpr int KS = DQK / 16, VS = DV / 16, QB = DQK / 32, VB = DV / 32;
  constexpr int QROW = pad_width(DQK) * 2, DOROW = DV * 2;   // (LDS rows; 192-wide queries sit in 256-wide rows)
  // a stage: the Q tile and the dO tile; behind the stages, 512 bytes per stage: lse (first 128) and delta (at 256) of its rows
  constexpr int QTILE = BMT * QROW, DOTILE = BMT * DOROW, STAGE = QTILE + DOTILE;
  constexpr int NST = MASKS ? 4 : fused_stages(pad_width(DQK), DV), LA = NST == 8 ? 4 : 3, ROWVALS = NST * STAGE;
  // (MASKS) behind the row values: 1 KB of mask bytes per stage and wave, then the step list and its length
  constexpr int KEEP = ROWVALS + NST * 512, LIST = KEEP + NST * 4 * 1024, LIST_N = LIST + FUSED_LIST_MAX * 4;
  // the MFMAs of a step and the fragment ring
  constexpr int NF = KS + VS, NV = 2 * VB, NK = 2 * QB, NTOT = NF + NV + NK;
  constexpr int RING = 8, AH = NK < 6 ? NK : 6;
  static_assert(NTOT % RING == 0 && AH < RING && AH <= NK && AH <= NF, "fragment ring");
  using PhF = PhaseF<KS, VS>;

  extern __shared__ __align__(16) char smem[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(MA_LDS char*)smem;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, g = lane >> 5;

  // Persistent: the grid is one workgroup per CU, and every workgroup walks items  item = blockIdx.x, + gridDim.x, ...  An
  // item is a (batch, kv head) and, under a causal mask, the PAIR of key blocks (k, n - 1 - k), which together see the
  // same number of query tiles whatever k is: every item weighs the same.  Items that follow each other on an XCD
  // (item % 8) belong to the same (batch, kv head) pairs, whose Q and dO tiles then come from that XCD's L2.
  const int nnb = a.num_blocks, BHK = a.B * a.Hkv;
  const int per_bh = CAUSAL ? (nnb + 1) / 2 : nnb, n_items = BHK * per_bh;
  for (int item = blockIdx.x; item < n_items; item += gridDim.x) {
  int bhk, ki;
  if ((BHK & 7) == 0) {
    const int slot = item >> 3;
    bhk = (slot / per_bh) * 8 + (item & 7);
    ki = slot % per_bh;
    // (without the causal pairing a key block's work depends on the mask: a workgroup, whose items are a whole number of
    // (batch, kv head) pairs apart, takes another key block each time round instead of the same one)
    if (!CAUSAL) ki = (ki + slot / per_bh) % per_bh;
  } else {
    bhk = item / per_bh;
    ki = item % per_bh;
    if (!CAUSAL) ki = (ki + bhk) % per_bh;
  }
  const int b = bhk / a.Hkv, hk = bhk % a.Hkv;
  for (int part = 0; part < (CAUSAL && ki != nnb - 1 - ki ? 2 : 1); part++) {
  const int nb = part == 0 ? ki : nnb - 1 - ki;
  const int n_wave = nb * BNW + wave * 32, n_lane = n_wave + r;
  const int n_ld = min(n_lane, a.Skv - 1);

  x8 kf[KS], vf[VS];
  {
    const T* kp = (const T*)a.k + (int64_t)b * a.ksb + (int64_t)n_ld * a.kss + (int64_t)hk * a.ksh + 8 * g;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) kf[ks] = *(const x8*)(kp + 16 * ks);
    const T* vp = (const T*)a.v + (int64_t)b * a.vsb + (int64_t)n_ld * a.vss + (int64_t)hk * a.vsh + 8 * g;
#pragma unroll
    for (int sl = 0; sl < VS; sl++) vf[sl] = *(const x8*)(vp + 16 * sl);
  }
  f32x16 dk[QB], dv[VB];
#pragma unroll
  for (int i = 0; i < QB; i++)
#pragma unroll
    for (int j = 0; j < 16; j++) dk[i][j] = 0.f;
#pragma unroll
  for (int i = 0; i < VB; i++)
#pragma unroll
    for (int j = 0; j < 16; j++) dv[i][j] = 0.f;
  const float bias = a.bias + (a.bias_ptr ? *a.bias_ptr : 0.f);
  const float c_scale = a.scale * kLog2e, c_bias = bias * kLog2e;
  const float s_masked = a.scale >= 0.f ? -__builtin_inff() : __builtin_inff();   // a score whose p is 0

  // steps: for every query head of the kv head's group, the 32-row tiles that can see this workgroup's keys
  const int t_first = CAUSAL ? (nb * BNW) / BMT : 0;
  const int t_count = (a.Sq + BMT - 1) / BMT - t_first;
  int n_steps = t_count > 0 ? t_count * a.kv_group : 0;
  const bool keep_ok = MASKS && a.elem_mask_t && ((a.emt_sk | a.emt_sb | a.emt_sh | (int64_t)(uintptr_t)a.elem_mask_t) & 15) == 0;
  if constexpr (MASKS) {
    // the step list: entry = tile | head of the group << 16 | kept in full << 31
    const uint8_t* qbm = a.q_block_mask ? a.q_block_mask + (int64_t)b * a.qbm_sb + (int64_t)nb * a.qbm_sk : nullptr;
    if (wave == 0) {
      int count = 0;
      for (int i0 = 0; i0 < n_steps; i0 += 64) {
        const int i = i0 + lane;
        bool keep = false;
        uint32_t entry = 0;
        if (i < n_steps) {
          const int hg = i / t_count, t = i - hg * t_count;
          const uint8_t e = qbm ? qbm[(int64_t)(hk * a.kv_group + hg) * a.qbm_sh + t_first + t] : (uint8_t)1;
          keep = e != 0;
          entry = (uint32_t)t | ((uint32_t)hg << 16) | (e >= 2 || !a.elem_mask_t ? 0x80000000u : 0u);
        }
        const uint64_t votes = __ballot(keep);
        if (keep) lds_write<uint32_t>(lds0 + LIST + 4 * (count + __popcll(votes & ((1ull << lane) - 1ull))), entry);
        count += __popcll(votes);
      }
      if (lane == 0) lds_write<uint32_t>(lds0 + LIST_N, (uint32_t)count);
    }
    __syncthreads();
    n_steps = __builtin_amdgcn_readfirstlane((int)lds_read<uint32_t>(lds0 + LIST_N));
  }
  // (list entries are requested a step before they are used and made wave-uniform only then: a read that is waited for
  // at once would drain the ring of operand fragments)
  auto list_request = [&](int i) { return lds_read<uint32_t>(lds0 + LIST + 4 * (i < n_steps ? i : 0)); };
  auto uniform = [&](uint32_t v) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)v); };
  const int64_t q_row_bytes = a.qss * 2, do_row_bytes = a.doss * 2;
  TileDma<QROW, 4, DQK / 8> q_dma;
  TileDma<DOROW, 4> do_dma;
  q_dma.init((uint32_t)q_row_bytes, wave, lane);
  do_dma.init((uint32_t)do_row_bytes, wave, lane);
  // what a wave issues per tile at least (with rows wider than the head size a lane may sit out some of its instructions,
  // a whole wave never does: the chunks of an instruction's rows are spread over all lanes)
  constexpr int TILE_DMAS = TileDma<QROW, 4>::NJ + TileDma<DOROW, 4>::NJ;
  auto issue_tile = [&](int hg, int t, int st, bool full = true) {
    const int h = hk * a.kv_group + hg, m0 = (t_first + t) * BMT;
    if constexpr (MASKS) {
      // the transposed element-wise keep mask: whole tiles of a 16-byte aligned mask come with the Q / dO tile
      if (keep_ok && !full && m0 + BMT <= a.Sq && n_wave < a.Skv)
        keep_dma(a.elem_mask_t + (int64_t)b * a.emt_sb + (int64_t)h * a.emt_sh + (int64_t)n_wave * a.emt_sk + m0, a.emt_sk, a.Skv - n_wave,
                 lds0 + KEEP + (st * 4 + wave) * 1024, lane);
    }
    const char* qb = (const char*)((const T*)a.q + (int64_t)b * a.qsb + (int64_t)h * a.qsh);
    const char* dob = (const char*)((const T*)a.dout + (int64_t)b * a.dosb + (int64_t)h * a.dosh);
    if (m0 + BMT <= a.Sq) {   // (wave-uniform)
      q_dma.issue(qb + (int64_t)m0 * q_row_bytes, lds0 + st * STAGE, wave);
      do_dma.issue(dob + (int64_t)m0 * do_row_bytes, lds0 + st * STAGE + QTILE, wave);
    } else {
      dma_tile<QROW, 4, DQK / 8>(qb, q_row_bytes, m0, a.Sq, lds0 + st * STAGE, wave, lane);
      dma_tile<DOROW, 4>(dob, do_row_bytes, m0, a.Sq, lds0 + st * STAGE + QTILE, wave, lane);
    }
    if constexpr (FAMILY == BF_SOFTMAX) {
      if (wave < 2) {   // wave 0 fetches lse, wave 1 delta (the upper lanes repeat the lower ones)
        const float* src = (wave == 0 ? a.lse : (const float*)a.delta) + ((int64_t)b * a.H + h) * a.Sq + m0;
        dma4_so(src, (uint32_t)(min(m0 + (lane & 31), a.Sq - 1) - m0) * 4u, lds0 + ROWVALS + st * 512 + wave * 256);
      }
    }
  };
  auto rowvals = [&](int st, FusedStepRegs<T>& x) {
    if constexpr (FAMILY == BF_SOFTMAX) {
      const uint32_t rv = lds0 + ROWVALS + st * 512;
#pragma unroll
      for (int q4 = 0; q4 < 4; q4++) {
        x.tl[q4] = lds_read<f32x4>(rv + (8 * q4 + 4 * g) * 4);
        x.td[q4] = lds_read<f32x4>(rv + 256 + (8 * q4 + 4 * g) * 4);
      }
    }
  };

  // the lane's part of the fragment addresses, relative to a tile: row reads (A operands of S and dP) and
  // transposing reads (A operands of dV^T and dK^T: the tile's columns)
  const uint32_t aq_l = (uint32_t)(r * QROW) + (uint32_t)((g ^ swz_tile<QROW / 16>(r)) << 4);
  const uint32_t ad_l = (uint32_t)(r * DOROW) + (uint32_t)((g ^ swz_tile<DV / 8>(r)) << 4);
  const int jr = (lane & 15) >> 2, lc = (((lane >> 4) & 1) << 1) | ((lane & 3) >> 1);
  const uint32_t bq_l = (uint32_t)((4 * g + jr) * QROW + (lane & 1) * 8) + (uint32_t)((lc ^ swz_tile<QROW / 16>(4 * g + jr)) << 4);
  const uint32_t bd_l = (uint32_t)((4 * g + jr) * DOROW + (lane & 1) * 8) + (uint32_t)((lc ^ swz_tile<DV / 8>(4 * g + jr)) << 4);
  // the fragment of MFMA j of a step whose current tile sits at `cur` and whose next tile at `nxt` (LDS addresses)
  auto fragment = [&](auto jc, uint32_t cur, uint32_t nxt) __attribute__((always_inline)) -> x8 {
    constexpr int j = decltype(jc)::value;
    // (consecutive MFMAs go to different accumulators: with one wave on the SIMD a dependent MFMA waits for the result
    // of the one before it.  Phase F alternates S and dP; phases V and K walk the column blocks before the k slices)
    if constexpr (j < NF && PhF::is_s(j)) {
      return lds_read<x8>((nxt + aq_l) ^ (uint32_t)(PhF::slice(j) * 32));
    } else if constexpr (j < NF) {
      return lds_read<x8>((nxt + QTILE + ad_l) ^ (uint32_t)(PhF::slice(j) * 32));
    } else {
      constexpr bool is_v = j < NF + NV;
      constexpr int idx = is_v ? j - NF : j - NF - NV, db = idx % (is_v ? VB : QB), sl = idx / (is_v ? VB : QB);
      constexpr int rowb = is_v ? DOROW : QROW;
      const uint32_t b0 = is_v ? cur + QTILE + bd_l : cur + bq_l;
      const x4 lo = lds_read_tr4<T>((b0 ^ (uint32_t)((4 * db) << 4)) + 16 * sl * rowb);
      const x4 hi = lds_read_tr4<T>((b0 ^ (uint32_t)(((4 * db) ^ 2) << 4)) + (16 * sl + 8) * rowb);
      return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
  };

  if (n_steps > 0) {
    // the next tile to fetch
    int i_hg = 0, i_t = 0, i_n = 0;
    uint32_t i_next = MASKS ? list_request(0) : 0u;   // (MASKS) the list entry of the next tile to fetch
    auto issue_next = [&]() {
      if constexpr (MASKS) {
        const uint32_t e = uniform(i_next);
        issue_tile((int)((e >> 16) & 0x7fffu), (int)(e & 0xffffu), i_n & (NST - 1), (e >> 31) != 0);
        i_n++;
        i_next = list_request(i_n);
      } else {
        issue_tile(i_hg, i_t, i_n & (NST - 1));
        i_n++;
        if (++i_t == t_count) { i_t = 0; i_hg++; }
      }
    };
#pragma unroll
    for (int i = 0; i < LA; i++)
      if (i_n < n_steps) issue_next();
    // (the padding step of an odd number of steps evaluates S, dP, lse and delta of the stage behind the last tile's:
    // where no earlier tile has been there, tile 0 goes there, so that what it computes is finite)
    if ((n_steps & 1) && n_steps < NST) {
      if constexpr (MASKS) {
        const uint32_t e = uniform(list_request(0));
        issue_tile((int)((e >> 16) & 0x7fffu), (int)(e & 0xffffu), n_steps);
      } else {
        issue_tile(0, 0, n_steps);
      }
    }
    wait_dma();
    __syncthreads();
    FusedStepRegs<T> ra, rb;
    ra.s = mm_rows<T, DQK>(lds0, r, g, kf);
    ra.dp = mm_rows<T, DV>(lds0 + QTILE, r, g, vf);
    rowvals(0, ra);
    x8 fr[RING];
    static_for<0, AH>([&](auto jc) __attribute__((always_inline)) { fr[decltype(jc)::value] = fragment(jc, lds0, lds0 + STAGE); });   // (of step 0)
    const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    int c_t = 0;   // the current step's tile within its head
    uint32_t c_next = MASKS ? list_request(0) : 0u;   // (MASKS) the list entry of the step about to begin, requested a step ahead
    auto body = [&](int u, FusedStepRegs<T>& cur, FusedStepRegs<T>& nxt) __attribute__((always_inline)) {
      const bool real = u < n_steps;                 // (the padding step: the last tile once more, everything masked)
      const uint32_t c_entry = MASKS ? uniform(c_next) : 0u;
      if constexpr (MASKS) c_next = list_request(u + 1);
      const uint32_t cur_tile = lds0 + (uint32_t)(((real ? u : n_steps - 1) & (NST - 1)) * STAGE);
      const uint32_t nxt_tile = lds0 + (uint32_t)(((u + 1) & (NST - 1)) * STAGE);
      const uint32_t nn_tile = lds0 + (uint32_t)(((u + 2) & (NST - 1)) * STAGE);
      const int m0 = real ? (t_first + (MASKS ? (int)(c_entry & 0xffffu) : c_t)) * BMT : a.Sq;
      if (++c_t == t_count) c_t = 0;
      rowvals((u + 1) & (NST - 1), nxt);             // (requested here, needed in the next step)
      // the tiles that touch the diagonal, an end of the sequences or an element-wise mask (the test is wave-uniform)
      const bool by_elem = MASKS && real && a.elem_mask_t && (c_entry >> 31) == 0;
      if ((CAUSAL && n_wave + 31 > m0) || m0 + BMT > a.Sq || n_wave + 32 > a.Skv || by_elem) {
        // (m0 through an empty asm statement: the compiler would otherwise evaluate the 32 compares in every step, ahead
        // of the branch, and turn the assignments into selects)
        int m0e = m0;
        asm volatile("; a tile that touches a mask" : "+s"(m0e));
        uint32_t keep[4] = {0x01010101u, 0x01010101u, 0x01010101u, 0x01010101u};   // the bytes of this lane's four rows per group
        if constexpr (MASKS) {
          if (by_elem) {
            if (keep_ok && m0e + BMT <= a.Sq && n_wave < a.Skv) {
#pragma unroll
              for (int q4 = 0; q4 < 4; q4++) keep[q4] = keep_read(lds0 + KEEP + ((u & (NST - 1)) * 4 + wave) * 1024, r, g, q4);
            } else {
              // this key's row of the transposed mask, indexed by query position
              const int h = hk * a.kv_group + (int)((c_entry >> 16) & 0x7fffu);
              const uint8_t* emt_row = a.elem_mask_t + (int64_t)b * a.emt_sb + (int64_t)h * a.emt_sh + (int64_t)n_ld * a.emt_sk;
#pragma unroll
              for (int q4 = 0; q4 < 4; q4++) {
                const int m = m0e + 8 * q4 + 4 * g;
                keep[q4] = 0;
#pragma unroll
                for (int i = 0; i < 4; i++)
                  if (m + i < a.Sq) keep[q4] |= (uint32_t)emt_row[m + i] << (8 * i);
              }
            }
          }
        }
#pragma unroll
        for (int jj = 0; jj < 16; jj++) {
          const int m = m0e + 8 * (jj >> 2) + 4 * g + (jj & 3);
          if ((CAUSAL && n_lane > m) || m >= a.Sq || n_lane >= a.Skv || (MASKS && ((keep[jj >> 2] >> (8 * (jj & 3))) & 0xffu) == 0)) {
            cur.s[jj] = s_masked;
            // (a row without any kept key has lse = -inf: its masked scores must still give p = 0)
            if constexpr (FAMILY == BF_SOFTMAX) cur.tl[jj >> 2][jj & 3] = 0.f;
          }
        }
      }
      x8 pf[2], dsf[2];
      float p32[16];
      static_for<0, NTOT>([&](auto jc) __attribute__((always_inline)) {
        constexpr int j = decltype(jc)::value;
        if constexpr (j == NF + NV) {
          // tile u + 2 has landed (what may still be in flight: the tiles behind it) and every wave is done with
          // tile u - 1, whose stage takes tile u + LA
          if (LA > 3 && u + LA - 1 < n_steps) wait_dma_but<(LA - 3) * TILE_DMAS>();
          else wait_dma();
          asm volatile("" ::: "memory");
          __builtin_amdgcn_s_barrier();
          asm volatile("" ::: "memory");
          if (i_n < n_steps) issue_next();
        }
        // the fragment of the MFMA AH places on (the last ones of the step: of the next step's first MFMAs)
        if constexpr (j + AH < NTOT) fr[(j + AH) % RING] = fragment(IntC<j + AH>(), cur_tile, nxt_tile);
        else fr[(j + AH) % RING] = fragment(IntC<j + AH - NTOT>(), nxt_tile, nn_tile);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (j < NF && PhF::is_s(j)) nxt.s = E::mfma32(fr[j % RING], kf[PhF::slice(j)], j == 0 ? zero16 : nxt.s);
        else if constexpr (j < NF) nxt.dp = E::mfma32(fr[j % RING], vf[PhF::slice(j)], j == 1 ? zero16 : nxt.dp);
        else if constexpr (j < NF + NV) dv[(j - NF) % VB] = E::mfma32(fr[j % RING], pf[(j - NF) / VB], dv[(j - NF) % VB]);
        else dk[(j - NF - NV) % QB] = E::mfma32(fr[j % RING], dsf[(j - NF - NV) / QB], dk[(j - NF - NV) % QB]);
        // vector work behind the MFMA: p of the step's 16 elements in phase F, ds in phase V
        if constexpr (j < NF) {
#pragma unroll
          for (int jj = j * 16 / NF; jj < (j + 1) * 16 / NF; jj++) {
            p32[jj] = row_p<FAMILY>(cur.s[jj], c_scale, c_bias, a.scale, bias, FAMILY == BF_SOFTMAX ? fmaf(cur.tl[jj >> 2][jj & 3], -kLog2e, c_bias) : 0.f);
            pf[jj >> 3][jj & 7] = (T)p32[jj];
          }
        } else if constexpr (j < NF + NV) {
#pragma unroll
          for (int jj = (j - NF) * 16 / NV; jj < (j - NF + 1) * 16 / NV; jj++)
            dsf[jj >> 3][jj & 7] = (T)row_ds<FAMILY>(p32[jj], cur.dp[jj], FAMILY == BF_SOFTMAX ? cur.td[jj >> 2][jj & 3] : 0.f);
          // (evaluated here, behind this MFMA: left alone the compiler moves it down to its use behind the barrier)
          asm volatile("" : "+v"(dsf[((j - NF) * 16 / NV) >> 3]));
        }
        __builtin_amdgcn_sched_barrier(0);
      });
    };
    for (int u = 0; u < n_steps; u += 2) {
      body(u, ra, rb);
      body(u + 1, rb, ra);
    }
  }
  wait_dma();
  __syncthreads();   // every wave is done with the tiles: they become output staging

  constexpr int DMAX = DQK > DV ? DQK : DV, OROW = DMAX + 16;
  const uint32_t stage = lds0 + wave * 32 * OROW;
  T* dkb = (T*)a.dk + (int64_t)b * a.dksb + (int64_t)hk * a.dksh;
  T* dvb = (T*)a.dv + (int64_t)b * a.dvsb + (int64_t)hk * a.dvsh;
  store_rows<T, DQK>(dk, a.scale, stage, dkb, a.dkss, n_wave, a.Skv, lane);
  store_rows<T, DV>(dv, 1.f, stage, dvb, a.dvss, n_wave, a.Skv, lane);
  __syncthreads();   // the staged output has left the stages: the next key block's tiles may arrive
  }   // the item's key blocks
  }   // items
}

// ------------------------------------------------------------------------------------------------
template <typename T, int DQK, int DV, int FAMILY, bool CAUSAL>
static int launch_bwd(const AttnBwdArgs& a, hipStream_t stream) {
  constexpr int DMAX = DQK > DV ? DQK : DV;
  // (+ the row values of the dk / dv kernels' stages and the retention family's multiplier blocks / the keep-mask blocks)
  constexpr size_t tiles = 2 * (size_t)32 * (pad_width(DQK) + DV) * 2 + 1024 + (FAMILY == BF_RETENTION ? 2 * 4 * 2048 : 2 * 4 * 1024);
  constexpr size_t ostage = 4 * 32 * (size_t)(DMAX + 16);
  constexpr size_t lds = tiles > ostage ? tiles : ostage;
  auto k1 = attn_bwd_dq_kernel<T, DQK, DV, FAMILY, CAUSAL>;
  // one dk/dv launch where both accumulators fit beside a second wave, else one launch each (at 256 / 256 the single launch
  // held both 128-register accumulators in a 512-register wave and spilled 170 registers: the whole backward at B4 H16 S4096
  // took 9.7 ms under the causal mask and 6.2 ms without; with one launch each 3.3 ms and 4.8 ms)
  constexpr bool SPLIT = DQK + DV >= 256;
  auto k2 = attn_bwd_dkv_kernel<T, DQK, DV, FAMILY, CAUSAL, SPLIT ? 1 : 3>;
  auto k3 = attn_bwd_dkv_kernel<T, DQK, DV, FAMILY, CAUSAL, 2>;
  static std::atomic<uint64_t> lds_ok{0};
  if (allow_lds(lds_ok, lds, k1, k2, k3) != 0) return -1;
  AttnBwdArgs args = a;
  if (a.add || a.slope_q || a.slope_kv || a.softcap != 0.f) {
    // additive score terms / soft-capping: instantiations of their own (not for the retention family, whose score function
    // is the multiplier tensor; soft-capping goes with softmax only, as in the forward), dk and dv by the two-launch kernels
    if constexpr (FAMILY != BF_RETENTION) {
      if (a.softcap != 0.f && FAMILY != BF_SOFTMAX) return -2;
      auto e1 = attn_bwd_dq_kernel<T, DQK, DV, FAMILY, CAUSAL, true>;
      auto e2 = attn_bwd_dkv_kernel<T, DQK, DV, FAMILY, CAUSAL, SPLIT ? 1 : 3, true>;
      auto e3 = attn_bwd_dkv_kernel<T, DQK, DV, FAMILY, CAUSAL, 2, true>;
      static std::atomic<uint64_t> elds_ok{0};
      if (allow_lds(elds_ok, lds, e1, e2, e3) != 0) return -1;
      args.num_blocks = (a.Sq + 127) / 128;
      hipLaunchKernelGGL(e1, dim3((unsigned)(args.num_blocks * a.B * a.H)), dim3(256), lds, stream, args);
      args.num_blocks = (a.Skv + 127) / 128;
      hipLaunchKernelGGL(e2, dim3((unsigned)(args.num_blocks * a.B * a.Hkv)), dim3(256), lds, stream, args);
      if (SPLIT) hipLaunchKernelGGL(e3, dim3((unsigned)(args.num_blocks * a.B * a.Hkv)), dim3(256), lds, stream, args);
      return launch_status();
    } else {
      return -2;
    }
  }
  args.num_blocks = (a.Sq + 127) / 128;
  hipLaunchKernelGGL(k1, dim3((unsigned)(args.num_blocks * a.B * a.H)), dim3(256), lds, stream, args);
  args.num_blocks = (a.Skv + 127) / 128;
  // (128 / 256 would fit the fused kernel's registers only with 60-90 spilled: measured no faster than its two launches)
  if constexpr (FAMILY != BF_RETENTION && (DQK + DV <= 256 || (DQK == 192 && DV == 128))) {
    // dk and dv by the pipelined single launch (with masks: as long as a key block's steps fit its list)
    const bool masks = a.elem_mask_t || a.q_block_mask;
    if (a.scale != 0.f && (!masks || (int64_t)((a.Sq + 31) / 32) * a.kv_group <= FUSED_LIST_MAX)) {
      constexpr size_t ftiles = fused_stages(pad_width(DQK), DV) * ((size_t)32 * (pad_width(DQK) + DV) * 2 + 512);
      constexpr size_t mtiles = 4 * ((size_t)32 * (pad_width(DQK) + DV) * 2 + 512 + 4 * 1024) + FUSED_LIST_MAX * 4 + 16;
      constexpr size_t fmax = ftiles > mtiles ? ftiles : mtiles, flds = fmax > ostage ? fmax : ostage;
      auto kf = attn_bwd_dkv_fused_kernel<T, DQK, DV, FAMILY, CAUSAL, false>;
      auto km = attn_bwd_dkv_fused_kernel<T, DQK, DV, FAMILY, CAUSAL, true>;
      static std::atomic<uint64_t> flds_ok{0};
      if (allow_lds(flds_ok, flds, kf, km) != 0) return -1;
      const int cus = device_cus();
      if (cus <= 0) return -1;
      const int items = (CAUSAL ? (args.num_blocks + 1) / 2 : args.num_blocks) * a.B * a.Hkv;
      if (masks) hipLaunchKernelGGL(km, dim3((unsigned)(items < cus ? items : cus)), dim3(256), flds, stream, args);
      else hipLaunchKernelGGL(kf, dim3((unsigned)(items < cus ? items : cus)), dim3(256), flds, stream, args);
      return launch_status();
    }
  }
  hipLaunchKernelGGL(k2, dim3((unsigned)(args.num_blocks * a.B * a.Hkv)), dim3(256), lds, stream, args);
  if (SPLIT) hipLaunchKernelGGL(k3, dim3((unsigned)(args.num_blocks * a.B * a.Hkv)), dim3(256), lds, stream, args);
  return launch_status();
}

template <typename T, int DQK, int DV>
static int bwd_family(const AttnBwdArgs& a, int family, bool causal, hipStream_t stream) {
  switch (family) {
    case BF_SOFTMAX:
      return causal ? launch_bwd<T, DQK, DV, BF_SOFTMAX, true>(a, stream) : launch_bwd<T, DQK, DV, BF_SOFTMAX, false>(a, stream);
    case BF_SIGMOID:
      return causal ? launch_bwd<T, DQK, DV, BF_SIGMOID, true>(a, stream) : launch_bwd<T, DQK, DV, BF_SIGMOID, false>(a, stream);
    case BF_RELU:
      return causal ? launch_bwd<T, DQK, DV, BF_RELU, true>(a, stream) : launch_bwd<T, DQK, DV, BF_RELU, false>(a, stream);
  }
  return -2;
}

// One head size: the retention family (where it is built at this size) or softmax / sigmoid / relu.
template <typename T, int DQK, int DV, bool RETENTION_TOO>
static int bwd_size(const AttnBwdArgs& a, int family, bool causal, hipStream_t stream) {
  if (family == BF_RETENTION) {
    if constexpr (RETENTION_TOO)
      return causal ? launch_bwd<T, DQK, DV, BF_RETENTION, true>(a, stream) : launch_bwd<T, DQK, DV, BF_RETENTION, false>(a, stream);
    else
      return -2;
  }
  return bwd_family<T, DQK, DV>(a, family, causal, stream);
}

}  // namespace ma
