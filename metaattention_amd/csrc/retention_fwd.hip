// Normalised parallel retention forward at the wide head size (Dqk 256, Dv 512) for gfx950.
//
// Same operator as the retention family of attn_wide_fwd.hip (attn_tl.py:92-190 with the row function of
// examples/retention_parallel.py:49-72):
//   qkm = s * scale * M,  r = max(sum_j |qkm|, 1),  o = (qkm / r) v,  M a caller-supplied [1|B, H, Sq, Skv]
//   multiplier (the decay mask); mask_value "0": no element-wise causal mask in forward, only kv tiles above
//   the workgroup's diagonal are skipped and the zeros come from M itself.  Where the caller can say that M is a
//   per-head geometric decay, M[h, i, j] = gamma_h^(i-j) for j <= i and 0 above the diagonal (RetNet's mask,
//   examples/retention_parallel.py:11-23), it passes gamma [H] instead and the kernel generates M: the tensor is
//   8 MB per head at S = 2048, read again for every batch entry, and streaming it costs a quarter of the run time.
// The row function is linear up to its final clamp, so the accumulator is kept un-normalised
// (O = sum_j P_j V_j, r = sum_j |P_j| in fp32) and divided by max(r, 1) once at the end.
//
// Structure.  What bounds this shape is the rate at which a CU takes direct-to-LDS loads (about 16 B/clock, and an
// instruction holds its wave until it is taken): a workgroup that owns 128 query rows and all 512 value columns
// loads 48 KB per tile of 32 keys, 3 000 clocks of load issue against 1 700 of MFMA.  So the work is cut the other
// way: a workgroup owns 256 query rows (8 waves x 32 rows, two waves per SIMD) and HALF of the value columns, the
// two halves of a row block being two workgroups.  A tile is then the 16 KB of K plus 16 KB of V columns for twice
// the rows, a third of the load bytes per row, at the price of both workgroups computing the scores (a third more
// MFMAs): per tile and CU 2 000 clocks of loads against 2 300 of MFMA.  Every wave computes the full 32 x 32 score
// tile of its rows (Q fragments of the whole 256-wide contraction in 64 registers) and its [256 x 32] block of the
// output (128 accumulator registers): no halves to exchange, one barrier per tile.  K / V tiles arrive by DMA
// through a ring of three stages, two tiles ahead.
//   The CU takes one DMA instruction per 64 clocks; when every wave issues its four instructions of a tile behind
// the barrier, all eight stand in that queue for 2 000 clocks in which no MFMA is issued (timestamps: 2 400 clocks
// of load issue + 2 400 of arithmetic per tile, nothing overlapping).  So a wave issues its instructions one at a
// time, every eighth MFMA, and every wave at another MFMA of the eight (the loop body exists once per wave, with
// the positions as compile-time constants: a run-time test at every MFMA would cut the MFMA sequence into basic
// blocks): the queue stays short, an instruction holds its wave for little more than its own 64 clocks, and the
// other wave of the SIMD issues MFMAs meanwhile.
//   A[32 x 16]: lane holds row l%32, k = 8(l/32) .. +7;  B[16 x 32]: lane holds column l%32, same k;
//   C[32 x 32]: lane holds column l%32, element j is row 8(j/4) + 4(l/32) + j%4.
// Scores are computed transposed (S^T = K Q^T) so a lane owns one query row and P^T is the B operand of
// O^T += V^T P^T without a shuffle; V^T comes out of the row-major V tile through the transposing read.
#include "attn_fwd.h"

#include <type_traits>

namespace ma {

namespace {
constexpr int RP_DQK = 256, RP_DV = 512, RP_DVH = 256, RP_BM = 256, RP_BN = 32, RP_NW = 8, RP_NST = 3;
constexpr int RP_KROW = RP_DQK * 2, RP_VROW = RP_DVH * 2;     // bytes of a tile row (V: this workgroup's half)
constexpr int RP_CPRK = RP_DQK / 8, RP_CPRV = RP_DVH / 8;
constexpr int RP_KTILE = RP_BN * RP_KROW, RP_VTILE = RP_BN * RP_VROW, RP_STAGE = RP_KTILE + RP_VTILE;
constexpr size_t RP_OSTAGE = RP_NW * 32 * (size_t)(RP_DVH / 2 * 2 + 16);
constexpr size_t RP_LDS = RP_NST * (size_t)RP_STAGE > RP_OSTAGE ? RP_NST * (size_t)RP_STAGE : RP_OSTAGE;
}  // namespace

template <typename T, bool CAUSAL, bool GAMMA>
__global__ __launch_bounds__(64 * RP_NW, 2) void retention_cols_fwd_kernel(const AttnArgs a) {
  using E = Elem<T>;
  using x8 = typename E::x8;
  using x4 = typename E::x4;
  constexpr int KS = RP_DQK / 16;    // k-slices of the contraction (16)
  constexpr int DB = RP_DVH / 32;    // output blocks of 32 columns (8)
  constexpr int NIK = RP_KTILE / 1024, NIV = RP_VTILE / 1024, NI = (NIK + NIV) / RP_NW;   // DMA instructions per wave and tile (4)
  static_assert((NIK + NIV) % RP_NW == 0 && NIK % RP_NW == 0, "whole DMA rounds, K rounds first");

  extern __shared__ __align__(16) char smem[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(MA_LDS char*)smem;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, g = lane >> 5;

  // workgroup -> (batch * head, row block, column half); the workgroups of one (batch, head) share an XCD (its L2 holds their K / V)
  const int nmb = a.num_m_blocks, BH = a.B * a.H;
  int bh, mb, ch;
  {
    int slot = blockIdx.x;
    if ((BH & 7) == 0) {
      const int xcd = blockIdx.x & 7;
      slot = blockIdx.x >> 3;
      ch = slot & 1;
      slot >>= 1;
      bh = (slot / nmb) * 8 + xcd;
    } else {
      ch = slot & 1;
      slot >>= 1;
      bh = slot / nmb;
    }
    mb = slot % nmb;
  }
  if (CAUSAL) mb = nmb - 1 - mb;   // long rows first
  const int b = bh / a.H, h = bh % a.H;
  const int m_wave = mb * RP_BM + wave * 32, m_lane = m_wave + r;
  const int m_ld = min(m_lane, a.Sq - 1);

  // Q fragments: B operand (lane: row r, k = 8g .. 8g+7 of a slice)
  x8 qf[KS];
  {
    const T* qp = (const T*)a.q + (int64_t)b * a.qsb + (int64_t)m_ld * a.qss + (int64_t)h * a.qsh + 8 * g;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) qf[ks] = *(const x8*)(qp + 16 * ks);
  }
  const char* kb = (const char*)((const T*)a.k + (int64_t)b * a.ksb + (int64_t)(h / a.kv_group) * a.ksh);
  const char* vb = (const char*)((const T*)a.v + (int64_t)b * a.vsb + (int64_t)(h / a.kv_group) * a.vsh + ch * RP_DVH);
  const int64_t k_row_bytes = a.kss * 2, v_row_bytes = a.vss * 2;
  const T* mrow = GAMMA ? nullptr : (const T*)a.smask + (int64_t)b * a.msb + (int64_t)h * a.msh + (int64_t)m_ld * a.msq;
  // generated multiplier: gamma^(i - j) = 2^((i - j) * lg), split for element jj of a tile that starts at n0 into a
  // factor of the lane, 2^((m_lane - n0 - 4g) * lg), one exponential per tile, and a factor 2^(-(8 (jj / 4) + jj % 4) * lg)
  // that is the same for every lane and tile (at most gamma^-27: RetNet's gammas are >= 1 - 2^-5): scalar registers
  const float lg = GAMMA ? __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, __builtin_log2f(a.decay_gamma[h])))) : 0.f;
  float colf[16];
  if constexpr (GAMMA) {
#pragma unroll
    for (int jj = 0; jj < 16; jj++)
      colf[jj] = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, fast_exp2(-(float)(8 * (jj >> 2) + (jj & 3)) * lg))));
  }

  const int skv = a.Skv;
  int n_tiles = (skv + RP_BN - 1) / RP_BN;
  if (CAUSAL) n_tiles = min(n_tiles, (mb * RP_BM + RP_BM + RP_BN - 1) / RP_BN);
  // tiles above this wave's own diagonal hold only zeros of M for its rows: it skips their arithmetic
  const int my_tiles = CAUSAL ? min(n_tiles, (m_wave + 32 + RP_BN - 1) / RP_BN) : n_tiles;

  // DMA of one tile: each instruction moves 1 KB (two rows of K or of this half of V); lane i fetches the 16-byte
  // chunk that belongs at physical position i of that KB.  Rows beyond the sequence are clamped to its last row
  // (their scores are multiplied by a zero of M).
  auto issue_one = [&](int jt, int it) __attribute__((always_inline)) {
    const uint32_t base = lds0 + (jt % RP_NST) * RP_STAGE;
    const int n0 = jt * RP_BN;
    {
      const int ii = wave + RP_NW * it;
      if (it < NIK / RP_NW) {
        const int row = ii * (1024 / RP_KROW) + lane / RP_CPRK, c = lane % RP_CPRK;
        const int nrow = min(n0 + row, skv - 1);
        dma16(kb + nrow * k_row_bytes + ((c ^ swz_tile<RP_CPRK>(row)) << 4), base + ii * 1024);
      } else {
        const int i2 = ii - NIK;
        const int row = i2 * (1024 / RP_VROW) + lane / RP_CPRV, c = lane % RP_CPRV;
        const int nrow = min(n0 + row, skv - 1);
        dma16(vb + nrow * v_row_bytes + ((c ^ swz_tile<RP_CPRV>(row)) << 4), base + RP_KTILE + i2 * 1024);
      }
    }
  };
  auto issue_tile = [&](int jt) __attribute__((always_inline)) {
#pragma unroll
    for (int it = 0; it < NI; it++) issue_one(jt, it);
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

  // per-lane LDS read offsets within a stage (tile bases and row offsets are multiples of the row size, so the
  // swizzled chunk index has its own address bits: another slice or block is one XOR with a constant away)
  const uint32_t k_off = r * RP_KROW + (uint32_t)((g ^ swz_tile<RP_CPRK>(r)) << 4);
  const int jr = (lane & 15) >> 2;
  const int lc = (((lane >> 4) & 1) << 1) | ((lane & 3) >> 1);
  const uint32_t v_off = RP_KTILE + (4 * g + jr) * RP_VROW + (lane & 1) * 8 + (uint32_t)((lc ^ swz_tile<RP_CPRV>(4 * g + jr)) << 4);

  f32x16 o[DB];
#pragma unroll
  for (int i = 0; i < DB; i++)
#pragma unroll
    for (int j = 0; j < 16; j++) o[i][j] = 0.f;
  float r_part = 0.f;   // this lane's share of sum |p| of its row
  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

  if (n_tiles > 0) issue_tile(0);
  if (n_tiles > 1) issue_tile(1);
  // the tile loop, with this wave's load instructions behind MFMAs OFF, OFF + 8, OFF + 16, OFF + 24 of a tile's 32
  auto run = [&](auto off_c) __attribute__((always_inline)) {
    constexpr int OFF = decltype(off_c)::value;
    for (int jt = 0; jt < n_tiles; jt++) {
      const int n0 = jt * RP_BN;
      // this wave's loads of tile jt have landed (they complete in order: only those of tile jt+1 may be in flight)
      if (jt + 1 < n_tiles) __builtin_amdgcn_s_waitcnt(0x0F70 | NI); else wait_dma();
      __syncthreads();   // tile jt has landed for every wave; every wave is done with tile jt-1, whose stage tile jt+2 takes
      const bool load_ahead = jt + 2 < n_tiles;
      if (jt >= my_tiles) {
        if (load_ahead) issue_tile(jt + 2);
        continue;
      }
      x4 mk[4];
      if constexpr (!GAMMA) load_mask(n0, mk);
      const uint32_t base = lds0 + (jt % RP_NST) * RP_STAGE;

      // ---- S^T = K Q^T
      f32x16 s;
      {
        constexpr int AH = 2, RING = 3;
        x8 kf[RING];
        const uint32_t ka = base + k_off;
#pragma unroll
        for (int ks = 0; ks < AH; ks++) kf[ks] = lds_read<x8>(ka ^ (uint32_t)(ks * 32));
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
          if (ks + AH < KS) kf[(ks + AH) % RING] = lds_read<x8>(ka ^ (uint32_t)((ks + AH) * 32));
          __builtin_amdgcn_sched_barrier(0);
          s = E::mfma32(kf[ks % RING], qf[ks], ks == 0 ? zero16 : s);
          if (ks % 8 == OFF && load_ahead) issue_one(jt + 2, ks / 8);
          __builtin_amdgcn_sched_barrier(0);
        }
      }

      // the first fragments of P V are requested before the row function: their latency hides behind it
      const uint32_t va = base + v_off;
      constexpr int PF = 3, NPV = 2 * DB;   // fragments in flight; MFMA i: block i / 2, slice i % 2
      x4 lo[PF], hi[PF];
      auto v_request = [&](int i) {
        const int db = i >> 1, sl = i & 1;
        lo[i % PF] = lds_read_tr4<T>((va ^ (uint32_t)(db * 64)) + 16 * sl * RP_VROW);
        hi[i % PF] = lds_read_tr4<T>((va ^ (uint32_t)((db * 64) ^ 32)) + (16 * sl + 8) * RP_VROW);
      };
#pragma unroll
      for (int i = 0; i < PF - 1; i++) v_request(i);

      // ---- P^T = S^T * scale * M (lane: row m_lane, kv rows n0 + 8(jj/4) + 4g + jj%4)
      x8 pf[2];
      if constexpr (GAMMA) {
        const float rowf = a.scale * fast_exp2((float)(m_lane - n0 - 4 * g) * lg);
        if (n0 + RP_BN - 1 > m_wave) {   // (wave-uniform) the tile reaches past the diagonal of some row: zeros above it
          const int lim = m_lane - n0 - 4 * g;   // element jj is kept when 8 (jj / 4) + jj % 4 <= lim
#pragma unroll
          for (int jj = 0; jj < 16; jj++) {
            const float p = 8 * (jj >> 2) + (jj & 3) <= lim ? s[jj] * colf[jj] * rowf : 0.f;
            r_part += fabsf(p);
            pf[jj >> 3][jj & 7] = (T)p;
          }
        } else {
#pragma unroll
          for (int jj = 0; jj < 16; jj++) {
            const float p = s[jj] * colf[jj] * rowf;
            r_part += fabsf(p);
            pf[jj >> 3][jj & 7] = (T)p;
          }
        }
      } else {
#pragma unroll
        for (int jj = 0; jj < 16; jj++) {
          const float p = s[jj] * a.scale * (float)mk[jj >> 2][jj & 3];
          r_part += fabsf(p);
          pf[jj >> 3][jj & 7] = (T)p;
        }
      }

      // ---- O^T += V^T P^T
#pragma unroll
      for (int i = 0; i < NPV; i++) {
        if (i + PF - 1 < NPV) v_request(i + PF - 1);
        __builtin_amdgcn_sched_barrier(0);
        x8 vf = __builtin_shufflevector(lo[i % PF], hi[i % PF], 0, 1, 2, 3, 4, 5, 6, 7);
        o[i >> 1] = E::mfma32(vf, pf[i & 1], o[i >> 1]);
        if (i % 8 == OFF && load_ahead) issue_one(jt + 2, 2 + i / 8);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  switch (wave) {
    case 0: run(std::integral_constant<int, 0>{}); break;
    case 1: run(std::integral_constant<int, 1>{}); break;
    case 2: run(std::integral_constant<int, 2>{}); break;
    case 3: run(std::integral_constant<int, 3>{}); break;
    case 4: run(std::integral_constant<int, 4>{}); break;
    case 5: run(std::integral_constant<int, 5>{}); break;
    case 6: run(std::integral_constant<int, 6>{}); break;
    default: run(std::integral_constant<int, 7>{}); break;
  }
  __syncthreads();   // every wave is done with the K/V stages: they become output staging

  const float r_tot = fmaxf(r_part + xhalf(r_part), 1.f);
  const float inv = 1.f / r_tot;
  if (a.row_scale && ch == 0 && g == 0 && m_lane < a.Sq) a.row_scale[((int64_t)b * a.H + h) * a.Sq + m_lane] = r_tot;

  // ---- O: this wave's 256 columns in two halves of 128 through a wave-private LDS block, coalesced 16-byte stores
  constexpr int HALF = RP_DVH / 2, OROW = HALF * 2 + 16;
  const uint32_t ob = lds0 + wave * 32 * OROW;
  T* obase = (T*)a.o + (int64_t)b * a.osb + (int64_t)h * a.osh + ch * RP_DVH;
#pragma unroll
  for (int hp = 0; hp < 2; hp++) {
#pragma unroll
    for (int dbl = 0; dbl < DB / 2; dbl++)
#pragma unroll
      for (int q4 = 0; q4 < 4; q4++) {
        x4 w;
#pragma unroll
        for (int i = 0; i < 4; i++) w[i] = (T)(o[hp * (DB / 2) + dbl][4 * q4 + i] * inv);
        lds_write<x4>(ob + r * OROW + (32 * dbl + 8 * q4 + 4 * g) * 2, w);
      }
#pragma unroll
    for (int it = 0; it < 32 * (HALF / 8) / 64; it++) {
      const int ci = lane + 64 * it, row = ci / (HALF / 8), c = ci % (HALF / 8);
      const u32x4 w = lds_read<u32x4>(ob + row * OROW + c * 16);
      if (m_wave + row < a.Sq) *(u32x4*)(obase + (int64_t)(m_wave + row) * a.oss + hp * HALF + c * 8) = w;
    }
  }
}

template <typename T, bool CAUSAL, bool GAMMA>
static int launch_cols(const AttnArgs& a, hipStream_t stream) {
  auto kern = retention_cols_fwd_kernel<T, CAUSAL, GAMMA>;
  static std::atomic<uint64_t> lds_ok{0};
  if (allow_lds(lds_ok, RP_LDS, kern) != 0) return -1;
  AttnArgs args = a;
  args.num_m_blocks = (a.Sq + RP_BM - 1) / RP_BM;
  hipLaunchKernelGGL(kern, dim3((unsigned)(args.num_m_blocks * a.B * a.H * 2)), dim3(64 * RP_NW), RP_LDS, stream, args);
  return launch_status();
}

// returns 0 ok, -1 launch failure, -2 unsupported
int retention_pair_fwd_dispatch(const AttnArgs& a, bool causal, bool is_bf16, hipStream_t stream) {
  if (a.decay_gamma) {   // (the generated multiplier is lower triangular: the structural mask is the causal one)
    if (!causal) return -2;
    return is_bf16 ? launch_cols<__bf16, true, true>(a, stream) : launch_cols<_Float16, true, true>(a, stream);
  }
  if (is_bf16) return causal ? launch_cols<__bf16, true, false>(a, stream) : launch_cols<__bf16, false, false>(a, stream);
  return causal ? launch_cols<_Float16, true, false>(a, stream) : launch_cols<_Float16, false, false>(a, stream);
}

}  // namespace ma
