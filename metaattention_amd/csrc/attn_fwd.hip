// Parallel (flash-style) attention forward for gfx950.
//
// Replaces the operator the reference renders from
// attention_engine/core/template/tl_template/attn/attn_tl.py:92-190: per Q tile,
// loop over KV tiles: S = Q K^T, elementwise score function, online row
// function, O = O * o_scale + P V.  The row functions are the fixed library
// variants documented in include/metaattention_hip.h.
//
// Mapping onto CDNA4 (wave64, v_mfma_f32_32x32x16):
//   * a workgroup is 4 waves; each wave owns 32 query rows (block_M = 128) and
//     every wave walks the same 64-row KV tiles, which arrive in LDS by
//     direct-to-LDS DMA (double buffered, one barrier per tile, no staging registers);
//   * the score tile is computed TRANSPOSED, S^T = K Q^T (A = K rows from LDS,
//     B = Q held in registers), so that in the accumulator layout every lane
//     owns ONE query row: the online row statistics are per-lane scalars, the
//     row reductions are 31 in-register ops plus one exchange with lane^32, and
//     the probabilities are already in B-operand layout for O^T += V^T P^T with
//     no LDS round trip;
//   * V^T fragments come straight out of the row-major V tile with the
//     transposing LDS read (ds_read_b64_tr_b16);
//   * both LDS tiles are XOR-swizzled at 16-byte granularity so the 128-bit K
//     reads and the transposing V reads are bank-conflict free without padding;
//   * LDS fragment reads are requested a few MFMAs ahead of their use (explicit
//     rings + scheduling barriers), and the output accumulator is only rescaled
//     when a row maximum has grown by more than 2^8 (see below).
#include "attn_fwd.h"

#include <type_traits>

namespace ma {

enum { FAM_SOFTMAX = 0, FAM_SIGMOID = 1, FAM_RELU = 2 };

template <typename T, int DQK, int DV, int FAMILY, bool CAUSAL>
__global__ __launch_bounds__(256, 2) void attn_fwd_kernel(const AttnArgs a) {
  using E = Elem<T>;
  using x8 = typename E::x8;
  using x4 = typename E::x4;
  constexpr int BM = 128, BN = 64, NB = BN / 32;
  constexpr int KS = DQK / 16;   // k-slices of the QK^T contraction
  constexpr int DB = DV / 32;    // 32-wide output column blocks
  constexpr int CPRK = DQK / 8, CPRV = DV / 8;  // 16-byte chunks per row
  constexpr int KROW = DQK * 2, VROW = DV * 2;
  constexpr int KTILE = BN * KROW, VTILE = BN * VROW;
  constexpr int NIK = KTILE / 1024, NIV = VTILE / 1024;  // DMA instructions (1 KB each) per tile
  static_assert(CPRK >= 16 && CPRV >= 16 && NIK % 4 == 0 && NIV % 4 == 0, "tile shape");

  extern __shared__ __align__(16) char smem[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(MA_LDS char*)smem;
  // [K buf0][K buf1][V buf0][V buf1]
  const uint32_t lds_k = lds0, lds_v = lds0 + 2 * KTILE;

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), r = lane & 31, g = lane >> 5;

  // workgroup -> (batch*head, q block).  Consecutive workgroup ids are dealt
  // round-robin to the 8 XCDs, so all q blocks of one (batch, head) are kept on
  // one XCD (shared K/V stays in that XCD's L2); causal q blocks run heaviest first.
  const int nmb = a.num_m_blocks, BH = a.B * a.H;
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
  const int b = bh / a.H, h = bh % a.H;
  const int m_wave = mb * BM + wave * 32;  // first query row of this wave
  const int m_lane = m_wave + r;

  // ---- Q fragments (B operand of S^T = K Q^T), kept in registers
  x8 qf[KS];
  {
    const int qrow = min(m_lane, a.Sq - 1);
    const T* qp = (const T*)a.q + (int64_t)b * a.qsb + (int64_t)qrow * a.qss + (int64_t)h * a.qsh + 8 * g;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) qf[ks] = *(const x8*)(qp + 16 * ks);
  }

  const char* kbase = (const char*)((const T*)a.k + (int64_t)b * a.ksb + (int64_t)h * a.ksh);
  const char* vbase = (const char*)((const T*)a.v + (int64_t)b * a.vsb + (int64_t)h * a.vsh);
  const int64_t k_row_bytes = a.kss * 2, v_row_bytes = a.vss * 2;

  int n_tiles = (a.Skv + BN - 1) / BN;
  if (CAUSAL) n_tiles = min(n_tiles, (mb * BM + BM + BN - 1) / BN);

  // ---- DMA of one KV tile: each instruction moves 1 KB (1024/row_bytes tile rows); lane i fetches the
  //      16-byte chunk that belongs at physical position i of that KB.  Wave w issues every 4th
  //      instruction; its rows are 4 ii + lane/16 with ii = w + 4t, so the swizzle term
  //      swz16(row) = ((lane/16) << 2) | w is the same for all of them and one per-lane 32-bit offset
  //      serves every instruction (scalar base + vector offset addressing).
  const uint32_t k_lane_off = (uint32_t)((lane / CPRK) * k_row_bytes) + (uint32_t)((((lane % CPRK) ^ swz16((lane / CPRK) | 0)) ^ (wave & 3)) << 4);
  const uint32_t v_lane_off = (uint32_t)((lane / CPRV) * v_row_bytes) + (uint32_t)((((lane % CPRV) ^ swz16((lane / CPRV) | 0)) ^ (wave & 3)) << 4);
  static_assert(1024 / KROW == 4 && 1024 / VROW == 4, "the shared lane offset assumes 4 tile rows per DMA instruction");
  auto issue_tile = [&](int n0, int buf) {
    if (n0 + BN <= a.Skv) {
#pragma unroll
      for (int t = 0; t < NIK / 4; t++) {
        const int ii = wave + 4 * t;
        dma16_so(kbase + (int64_t)(n0 + 4 * ii) * k_row_bytes, k_lane_off, lds_k + buf * KTILE + ii * 1024);
      }
#pragma unroll
      for (int t = 0; t < NIV / 4; t++) {
        const int ii = wave + 4 * t;
        dma16_so(vbase + (int64_t)(n0 + 4 * ii) * v_row_bytes, v_lane_off, lds_v + buf * VTILE + ii * 1024);
      }
    } else {   // last, partial tile: rows beyond the sequence are clamped (their scores are masked)
      for (int t = 0; t < NIK / 4; t++) {
        const int ii = wave + 4 * t;
        const int row = ii * 4 + lane / CPRK, c = lane % CPRK;
        const int nrow = min(n0 + row, a.Skv - 1);
        dma16(kbase + nrow * k_row_bytes + ((c ^ swz16(row)) << 4), lds_k + buf * KTILE + ii * 1024);
      }
      for (int t = 0; t < NIV / 4; t++) {
        const int ii = wave + 4 * t;
        const int row = ii * 4 + lane / CPRV, c = lane % CPRV;
        const int nrow = min(n0 + row, a.Skv - 1);
        dma16(vbase + nrow * v_row_bytes + ((c ^ swz16(row)) << 4), lds_v + buf * VTILE + ii * 1024);
      }
    }
  };

  // ---- per-lane LDS read addresses
  // K (A operand of S^T): row 32nb + r, logical chunk 2ks + g
  const uint32_t k_row_off = r * KROW;
  const int k_chunk0 = g ^ swz16(r);
  // V (A operand of O^T, through the transposing read): lane block = lane/16,
  // row nbase + 8*half + 4g + jr, logical chunk 4db + lc
  const int jr = (lane & 15) >> 2;
  const int lc = (((lane >> 4) & 1) << 1) | ((lane & 3) >> 1);
  const uint32_t v_row_off = (4 * g + jr) * VROW + (lane & 1) * 8;
  const int v_chunk0 = lc ^ swz16(4 * g + jr);
  constexpr int V_HALF_XOR = 2;  // swz16(row + 8) ^ swz16(row) for row < 8; swz16(row + 16) == swz16(row)
  // all lane-dependent parts of the LDS read addresses, one register each; what is added per read
  // (buffer, 32-row block, 16-row slice) is a compile-time immediate
  uint32_t k_addr[KS], v_addr[DB][2];
#pragma unroll
  for (int ks = 0; ks < KS; ks++) k_addr[ks] = lds_k + k_row_off + (uint32_t)((k_chunk0 ^ (2 * ks)) << 4);
#pragma unroll
  for (int db = 0; db < DB; db++) {
    v_addr[db][0] = lds_v + v_row_off + (uint32_t)((v_chunk0 ^ (4 * db)) << 4);
    v_addr[db][1] = lds_v + v_row_off + 8 * VROW + (uint32_t)((v_chunk0 ^ (4 * db) ^ V_HALF_XOR) << 4);
  }

  // ---- accumulators and row state
  f32x16 o[DB];
#pragma unroll
  for (int i = 0; i < DB; i++)
#pragma unroll
    for (int j = 0; j < 16; j++) o[i][j] = 0.f;
  const float bias = a.bias + (a.bias_ptr ? *a.bias_ptr : 0.f);
  const float c_scale = a.scale * kLog2e;  // scores are handled in the log2 domain
  const float c_bias = bias * kLog2e;
  float row_max = -1e30f;  // running max of (scale*s + bias) * log2e
  float row_sum = 0.f;     // this lane's share of the running sum (the other half lives in lane^32)

  // One KV tile.  BUF (LDS buffer) and MASKED are compile-time so that every LDS address is a lane
  // register plus an immediate and the unmasked tiles carry no mask code.
  auto do_tile = [&](auto buf_c, auto masked_c, const int buf_rt, const int n0) {
    constexpr bool MASKED = decltype(masked_c)::value;          // may this tile need the structural mask?
    const int BUF = decltype(buf_c)::value >= 0 ? decltype(buf_c)::value : buf_rt;   // compile-time unless -1
      // ---- S^T = K Q^T : lane holds query row r, kv rows 32nb + 8(j/4) + 4g + j%4
      f32x16 s[NB];
  #pragma unroll
      for (int nb = 0; nb < NB; nb++)
  #pragma unroll
        for (int j = 0; j < 16; j++) s[nb][j] = 0.f;
      {
        constexpr int AH = 2, RING = 3;   // K fragments are requested AH slices ahead of their MFMAs
        x8 kf[RING][NB];
        const uint32_t kb = lds_k + BUF * KTILE + k_row_off;
        auto request = [&](int ks) {
          const uint32_t coff = (uint32_t)((k_chunk0 ^ (2 * ks)) << 4);
  #pragma unroll
          for (int nb = 0; nb < NB; nb++) kf[ks % RING][nb] = lds_read<x8>(kb + nb * 32 * KROW + coff);
        };
  #pragma unroll
        for (int ks = 0; ks < AH; ks++) request(ks);
  #pragma unroll
        for (int ks = 0; ks < KS; ks++) {
          if (ks + AH < KS) request(ks + AH);
          __builtin_amdgcn_sched_barrier(0);
  #pragma unroll
          for (int nb = 0; nb < NB; nb++) s[nb] = E::mfma32(kf[ks % RING][nb], qf[ks], s[nb]);
          __builtin_amdgcn_sched_barrier(0);
        }
      }

      // ---- structural mask: exact -inf above the diagonal / beyond the cache
      if (MASKED && ((CAUSAL && (n0 + BN - 1 > m_wave)) || (n0 + BN > a.Skv))) {   // exact -inf above the diagonal / beyond the cache
        const int lim = CAUSAL ? min(m_lane, a.Skv - 1) : a.Skv - 1;  // keep n <= lim
  #pragma unroll
        for (int nb = 0; nb < NB; nb++)
  #pragma unroll
          for (int j = 0; j < 16; j++) {
            const int n = n0 + 32 * nb + 8 * (j >> 2) + 4 * g + (j & 3);
            if (n > lim) s[nb][j] = -INFINITY;
          }
      }

      // ---- row function
      if constexpr (FAMILY == FAM_SOFTMAX) {
        float mx = s[0][0];
  #pragma unroll
        for (int nb = 0; nb < NB; nb++)
  #pragma unroll
          for (int j = 0; j < 16; j++) mx = fmaxf(mx, s[nb][j]);
        mx = fmaxf(mx, xhalf(mx));
        // The running max only moves when some row's max grew by more than 2^8: until then probabilities
        // are taken relative to the stale max (at most 256: exact in fp32, in range for bf16/fp16) and the
        // accumulator needs no rescaling; the final division by row_sum absorbs the offset.
        // Each row decides for itself (rows that stay multiply by exactly 1), so a row's result never
        // depends on what other rows of its wave see.
        const float cand = fmaxf(row_max, mx * c_scale + c_bias);
        const bool move = cand - row_max > 8.f;
        if (__any(move)) {
          const float corr = move ? fast_exp2(row_max - cand) : 1.f;
          row_max = move ? cand : row_max;
          row_sum *= corr;
  #pragma unroll
          for (int i = 0; i < DB; i++)
  #pragma unroll
            for (int j = 0; j < 16; j++) o[i][j] *= corr;
        }
        const float sub = c_bias - row_max;
        float part = 0.f;
  #pragma unroll
        for (int nb = 0; nb < NB; nb++)
  #pragma unroll
          for (int j = 0; j < 16; j++) {
            const float p = fast_exp2(s[nb][j] * c_scale + sub);
            s[nb][j] = p;
            part += p;
          }
        row_sum += part;
      } else if constexpr (FAMILY == FAM_SIGMOID) {
  #pragma unroll
        for (int nb = 0; nb < NB; nb++)
  #pragma unroll
          for (int j = 0; j < 16; j++)  // sigmoid(x) = 1 / (1 + 2^(-x log2e)); s = -inf gives exactly 0
            s[nb][j] = fast_rcp(1.f + fast_exp2(-(s[nb][j] * c_scale + c_bias)));
      } else {
  #pragma unroll
        for (int nb = 0; nb < NB; nb++)
  #pragma unroll
          for (int j = 0; j < 16; j++) s[nb][j] = fmaxf(s[nb][j] * a.scale + bias, 0.f);
      }

      // ---- O^T += V^T P^T ; the k index of MFMA slice (nb, t), lane half g, slot i is
      //      kv row 32nb + 16t + 8(i/4) + 4g + i%4 on both operands
      {
        x8 pf[2 * NB];
  #pragma unroll
        for (int sl = 0; sl < 2 * NB; sl++)
  #pragma unroll
          for (int i = 0; i < 8; i++) pf[sl][i] = (T)s[sl >> 1][8 * (sl & 1) + i];
        constexpr int PF = 4, NIT = 2 * NB * DB;   // V fragments in flight; idx = sl * DB + db
        x4 lo[PF], hi[PF];
        auto request = [&](int idx) {
          const int sl = idx / DB, db = idx % DB;
          lo[idx % PF] = lds_read_tr4<T>(v_addr[db][0] + BUF * VTILE + 16 * sl * VROW);
          hi[idx % PF] = lds_read_tr4<T>(v_addr[db][1] + BUF * VTILE + 16 * sl * VROW);
        };
  #pragma unroll
        for (int i = 0; i < PF - 1; i++) request(i);
  #pragma unroll
        for (int idx = 0; idx < NIT; idx++) {
          if (idx + PF - 1 < NIT) request(idx + PF - 1);
          __builtin_amdgcn_sched_barrier(0);
          x8 vf = __builtin_shufflevector(lo[idx % PF], hi[idx % PF], 0, 1, 2, 3, 4, 5, 6, 7);
          o[idx % DB] = E::mfma32(vf, pf[idx / DB], o[idx % DB]);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
  };

  issue_tile(0, 0);

  // Tiles [0, n_fast) need no mask in any wave: they run two per iteration with compile-time buffers.
  // The remaining ones (the diagonal block of a causal workgroup, a partial last tile) take the generic path.
  using std::integral_constant;
  int n_fast = a.Skv / BN;
  if (CAUSAL) n_fast = min(n_fast, mb * BM / BN);
  n_fast &= ~1;
  int jt = 0;
  for (; jt < n_fast; jt += 2) {
    wait_dma();
    __syncthreads();   // tile jt has landed for every wave, and every wave is done reading tile jt-1
    issue_tile((jt + 1) * BN, 1);
    do_tile(integral_constant<int, 0>{}, integral_constant<bool, false>{}, 0, jt * BN);
    wait_dma();
    __syncthreads();
    if (jt + 2 < n_tiles) issue_tile((jt + 2) * BN, 0);
    do_tile(integral_constant<int, 1>{}, integral_constant<bool, false>{}, 1, (jt + 1) * BN);
  }
  for (; jt < n_tiles; jt++) {
    const int buf = jt & 1, n0 = jt * BN;
    wait_dma();
    __syncthreads();
    if (jt + 1 < n_tiles) issue_tile(n0 + BN, buf ^ 1);
    // a wave whose 32 rows all lie above this tile's first column has nothing to do in it
    if (CAUSAL && n0 > m_wave + 31) continue;
    do_tile(integral_constant<int, -1>{}, integral_constant<bool, true>{}, buf, n0);
  }
  __syncthreads();   // every wave is done with the K/V buffers: they become output staging

  // ---- epilogue: normalise, stage O through LDS (wave-private), coalesced 16-byte stores
  float inv = 1.f, lse = 0.f;
  if constexpr (FAMILY == FAM_SOFTMAX) {
    const float tot = row_sum + xhalf(row_sum);
    inv = 1.f / tot;
    lse = (row_max + fast_log2(tot)) * kLn2;
  }
  constexpr int OROW = DV * 2 + 16;  // padded staging row
  const uint32_t ob = lds0 + wave * 32 * OROW;
#pragma unroll
  for (int db = 0; db < DB; db++)
#pragma unroll
    for (int q4 = 0; q4 < 4; q4++) {
      x4 w;
#pragma unroll
      for (int i = 0; i < 4; i++) w[i] = (T)(o[db][4 * q4 + i] * inv);
      lds_write<x4>(ob + r * OROW + (32 * db + 8 * q4 + 4 * g) * 2, w);
    }
  T* obase = (T*)a.o + (int64_t)b * a.osb + (int64_t)h * a.osh;
#pragma unroll
  for (int it = 0; it < 32 * CPRV / 64; it++) {
    const int ci = lane + 64 * it, row = ci / CPRV, c = ci % CPRV;
    u32x4 w = lds_read<u32x4>(ob + row * OROW + c * 16);
    if (m_wave + row < a.Sq) *(u32x4*)(obase + (int64_t)(m_wave + row) * a.oss + c * 8) = w;
  }
  if constexpr (FAMILY == FAM_SOFTMAX) {
    if (a.row_scale && g == 0 && m_lane < a.Sq) a.row_scale[((int64_t)b * a.H + h) * a.Sq + m_lane] = lse;
  }
}

template <typename T, int DQK, int DV, int FAMILY, bool CAUSAL>
static int launch(const AttnArgs& a, hipStream_t stream) {
  constexpr int BM = 128, BN = 64;
  constexpr size_t tiles = 2 * (size_t)BN * (DQK + DV) * 2;
  constexpr size_t ostage = 4 * 32 * (size_t)(DV * 2 + 16);
  constexpr size_t lds = tiles > ostage ? tiles : ostage;
  auto kern = attn_fwd_kernel<T, DQK, DV, FAMILY, CAUSAL>;
  static bool attr_set = false;
  if (!attr_set) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) return -1;
    attr_set = true;
  }
  AttnArgs args = a;
  args.num_m_blocks = (a.Sq + BM - 1) / BM;
  const unsigned grid = (unsigned)(args.num_m_blocks * a.B * a.H);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, stream, args);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

template <typename T, int DQK, int DV>
static int dispatch_family(const AttnArgs& a, int family, bool causal, hipStream_t stream) {
  switch (family) {
    case FAM_SOFTMAX:
      return causal ? launch<T, DQK, DV, FAM_SOFTMAX, true>(a, stream) : launch<T, DQK, DV, FAM_SOFTMAX, false>(a, stream);
    case FAM_SIGMOID:
      return causal ? launch<T, DQK, DV, FAM_SIGMOID, true>(a, stream) : launch<T, DQK, DV, FAM_SIGMOID, false>(a, stream);
    case FAM_RELU:
      return causal ? launch<T, DQK, DV, FAM_RELU, true>(a, stream) : launch<T, DQK, DV, FAM_RELU, false>(a, stream);
  }
  return -2;
}

// returns 0 ok, -1 launch failure, -2 unsupported
int attn_fwd_dispatch(const AttnArgs& a, int family, bool causal, bool is_bf16, int dqk, int dv, hipStream_t stream) {
  if (family == 3) return retention_fwd_dispatch(a, causal, is_bf16, dqk, dv, stream);
  if (dqk == 128 && dv == 128) {
    return is_bf16 ? dispatch_family<__bf16, 128, 128>(a, family, causal, stream)
                   : dispatch_family<_Float16, 128, 128>(a, family, causal, stream);
  }
  return -2;
}

}  // namespace ma
