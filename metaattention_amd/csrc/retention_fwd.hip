// Normalised parallel retention forward at the wide head size (Dqk 256, Dv 512) for gfx950.
//
// Same operator as the retention family of attn_wide_fwd.hip (attn_tl.py:92-190 with the row function of
// examples/retention_parallel.py:49-72):
//   qkm = s * scale * M,  r = max(sum_j |qkm|, 1),  o = (qkm / r) v,  M a caller-supplied [1|B, H, Sq, Skv]
//   multiplier (the decay mask); mask_value "0": no element-wise causal mask in forward, only kv tiles above
//   the workgroup's diagonal are skipped and the zeros come from M itself.
// The row function is linear up to its final clamp, so the accumulator is kept un-normalised
// (O = sum_j P_j V_j, r = sum_j |P_j| in fp32) and divided by max(r, 1) once at the end.
//
// Structure.  A wave that owned 32 query rows and all 512 value columns would need 256 accumulator registers
// and run alone on its SIMD, every wait for an LDS operand or a direct-to-LDS load exposed.  Here two waves
// share 32 query rows and split the work along the long axes, as the MLA decode kernel does:
//   * scores:  each wave takes half of the 256-wide contraction (8 of the 16 k-slices, Q fragments of its
//     half in 32 registers), S^T_half = K_half Q_half^T; the halves are exchanged through LDS (4 KB each way)
//     and added, so both waves hold the full 32 x 32 score tile and compute the same P^T;
//   * output:  each wave takes half of the 512 value columns, O^T_half += V_half^T P^T (128 registers).
// A workgroup is 4 such pairs (128 query rows, 8 waves, two per SIMD).  K and V tiles of 32 keys arrive by
// direct-to-LDS DMA, double buffered; two barriers per tile (tile landed / halves written).
// What bounds it: a CU accepts direct-to-LDS loads at about 16 B/clock and an instruction holds its wave
// until it is accepted; the 48 KB of a tile take about as long (~3200 clocks) as the tile's arithmetic, and
// the two do not overlap while every wave issues its share behind the same barrier.  Measured and not kept:
// waves 0..3 issuing the K tile between the MFMAs of the score phase and waves 4..7 the V tile between those
// of the output phase (so that one wave of a SIMD computes while the other waits for acceptance): the
// non-issuing waves finish their short phase early and wait at the next barrier, 8 % slower.
//   A[32 x 16]: lane holds row l%32, k = 8(l/32) .. +7;  B[16 x 32]: lane holds column l%32, same k;
//   C[32 x 32]: lane holds column l%32, element j is row 8(j/4) + 4(l/32) + j%4.
// Scores are computed transposed (S^T = K Q^T) so a lane owns one query row and P^T is the B operand of
// O^T += V^T P^T without a shuffle; V^T comes out of the row-major V tile through the transposing read.
#include "attn_fwd.h"

namespace ma {

namespace {
constexpr int RP_DQK = 256, RP_DV = 512, RP_BM = 128, RP_BN = 32, RP_NW = 8;
constexpr int RP_KROW = RP_DQK * 2, RP_VROW = RP_DV * 2;
constexpr int RP_CPRK = RP_DQK / 8, RP_CPRV = RP_DV / 8;
constexpr int RP_KTILE = RP_BN * RP_KROW, RP_VTILE = RP_BN * RP_VROW, RP_STAGE = RP_KTILE + RP_VTILE;
constexpr int RP_XCHG = 4096;   // one wave's half score tile: 16 fp32 per lane
constexpr size_t RP_LDS = 2 * (size_t)RP_STAGE + RP_NW * (size_t)RP_XCHG;
}  // namespace

template <typename T, bool CAUSAL>
__global__ __launch_bounds__(64 * RP_NW, 2) void retention_pair_fwd_kernel(const AttnArgs a) {
  using E = Elem<T>;
  using x8 = typename E::x8;
  using x4 = typename E::x4;
  constexpr int KSH = RP_DQK / 16 / 2;   // k-slices per wave (8)
  constexpr int DBH = RP_DV / 32 / 2;    // output blocks of 32 columns per wave (8)
  constexpr int NIK = RP_KTILE / 1024, NIV = RP_VTILE / 1024;

  extern __shared__ __align__(16) char smem[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(MA_LDS char*)smem;
  const uint32_t lds_x = lds0 + 2 * RP_STAGE;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int hg = wave >> 1, hf = wave & 1;   // row group, half: the two waves of a pair sit on different SIMDs (wave % 4)
  const int r = lane & 31, g = lane >> 5;

  const int nmb = a.num_m_blocks, BH = a.B * a.H;
  int bh, mb;
  if ((BH & 7) == 0) {   // the row blocks of one (batch, head) share an XCD (its L2 holds their K/V)
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    bh = (slot / nmb) * 8 + xcd;
    mb = slot % nmb;
  } else {
    bh = blockIdx.x / nmb;
    mb = blockIdx.x % nmb;
  }
  if (CAUSAL) mb = nmb - 1 - mb;   // long rows first
  const int b = bh / a.H, h = bh % a.H;
  const int m_wave = mb * RP_BM + hg * 32, m_lane = m_wave + r;
  const int m_ld = min(m_lane, a.Sq - 1);

  // Q fragments of this wave's half of the contraction: B operand (lane: row r, k = 8g .. 8g+7 of a slice)
  x8 qf[KSH];
  {
    const T* qp = (const T*)a.q + (int64_t)b * a.qsb + (int64_t)m_ld * a.qss + (int64_t)h * a.qsh + 8 * g + hf * (KSH * 16);
#pragma unroll
    for (int ks = 0; ks < KSH; ks++) qf[ks] = *(const x8*)(qp + 16 * ks);
  }
  const char* kb = (const char*)((const T*)a.k + (int64_t)b * a.ksb + (int64_t)(h / a.kv_group) * a.ksh);
  const char* vb = (const char*)((const T*)a.v + (int64_t)b * a.vsb + (int64_t)(h / a.kv_group) * a.vsh);
  const int64_t k_row_bytes = a.kss * 2, v_row_bytes = a.vss * 2;
  const T* mrow = (const T*)a.smask + (int64_t)b * a.msb + (int64_t)h * a.msh + (int64_t)m_ld * a.msq;

  const int skv = a.Skv;
  int n_tiles = (skv + RP_BN - 1) / RP_BN;
  if (CAUSAL) n_tiles = min(n_tiles, (mb * RP_BM + RP_BM + RP_BN - 1) / RP_BN);

  // DMA of one tile: each instruction moves 1 KB (two K rows or one V row); lane i fetches the 16-byte chunk
  // that belongs at physical position i of that KB.  Rows beyond the sequence are clamped to its last row
  // (their scores are multiplied by a zero of M).
  auto issue_tile = [&](int n0, int buf) {
    const uint32_t base = lds0 + buf * RP_STAGE;
#pragma unroll
    for (int it = 0; it < (NIK + NIV) / RP_NW; it++) {
      const int ii = wave + RP_NW * it;
      if (ii < NIK) {
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
  static_assert((NIK + NIV) % RP_NW == 0, "whole DMA rounds");
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
  // K side (A operand): row r, logical 16-byte chunk 2 * slice + g; this wave's first slice is hf * 8
  const uint32_t k_off = r * RP_KROW + (uint32_t)(((g ^ swz_tile<RP_CPRK>(r)) << 4) ^ (hf * (KSH * 32)));
  // V side (transposing read): rows 16sl + 4g + jr (+8), chunk 4 * block + lc; this wave's first block is hf * 8
  const int jr = (lane & 15) >> 2;
  const int lc = (((lane >> 4) & 1) << 1) | ((lane & 3) >> 1);
  const uint32_t v_off = RP_KTILE + (4 * g + jr) * RP_VROW + (lane & 1) * 8 +
                         (uint32_t)(((lc ^ swz_tile<RP_CPRV>(4 * g + jr)) << 4) ^ (hf * (DBH * 64)));
  const uint32_t x_mine = lds_x + wave * RP_XCHG + lane * 16, x_other = lds_x + (wave ^ 1) * RP_XCHG + lane * 16;

  f32x16 o[DBH];
#pragma unroll
  for (int i = 0; i < DBH; i++)
#pragma unroll
    for (int j = 0; j < 16; j++) o[i][j] = 0.f;
  float r_part = 0.f;   // this lane's share of sum |p| of its row
  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

  x4 mk_next[4];
  if (n_tiles > 0) {
    issue_tile(0, 0);
    load_mask(0, mk_next);
  }
  for (int jt = 0; jt < n_tiles; jt++) {
    const int buf = jt & 1, n0 = jt * RP_BN;
    wait_dma();
    __syncthreads();   // tile jt has landed for every wave; every wave is done with tile jt-1 and with the halves of jt-1
    x4 mk[4];
#pragma unroll
    for (int q4 = 0; q4 < 4; q4++) mk[q4] = mk_next[q4];
    if (jt + 1 < n_tiles) {
      load_mask(n0 + RP_BN, mk_next);
      issue_tile(n0 + RP_BN, buf ^ 1);
    }
    const uint32_t base = lds0 + buf * RP_STAGE;

    // ---- half scores: S^T_half = K_half Q_half^T over this wave's 8 k-slices, handed to the partner
    f32x16 s;
    {
      constexpr int AH = 2, RING = 3;
      x8 kf[RING];
      const uint32_t ka = base + k_off;
#pragma unroll
      for (int ks = 0; ks < AH; ks++) kf[ks] = lds_read<x8>(ka ^ (uint32_t)(ks * 32));
#pragma unroll
      for (int ks = 0; ks < KSH; ks++) {
        if (ks + AH < KSH) kf[(ks + AH) % RING] = lds_read<x8>(ka ^ (uint32_t)((ks + AH) * 32));
        __builtin_amdgcn_sched_barrier(0);
        s = E::mfma32(kf[ks % RING], qf[ks], ks == 0 ? zero16 : s);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
#pragma unroll
    for (int j4 = 0; j4 < 4; j4++) lds_write<f32x4>(x_mine + j4 * 1024, f32x4{s[4 * j4], s[4 * j4 + 1], s[4 * j4 + 2], s[4 * j4 + 3]});
    __syncthreads();
#pragma unroll
    for (int j4 = 0; j4 < 4; j4++) {
      const f32x4 t = lds_read<f32x4>(x_other + j4 * 1024);
#pragma unroll
      for (int i = 0; i < 4; i++) s[4 * j4 + i] += t[i];
    }

    // the first fragments of P V are requested before the row function: their latency hides behind it
    const uint32_t va = base + v_off;
    constexpr int PF = 4, NPV = 2 * DBH;   // fragments in flight; MFMA i: block i / 2, slice i % 2
    x4 lo[PF], hi[PF];
    auto v_request = [&](int i) {
      const int db = i >> 1, sl = i & 1;
      lo[i % PF] = lds_read_tr4<T>((va ^ (uint32_t)(db * 64)) + 16 * sl * RP_VROW);
      hi[i % PF] = lds_read_tr4<T>((va ^ (uint32_t)((db * 64) ^ 32)) + (16 * sl + 8) * RP_VROW);
    };
#pragma unroll
    for (int i = 0; i < PF - 1; i++) v_request(i);

    // ---- P^T = S^T * scale * M (lane: row m_lane, kv rows n0 + 8(jj/4) + 4g + jj%4); both waves of the pair the same
    x8 pf[2];
#pragma unroll
    for (int jj = 0; jj < 16; jj++) {
      const float p = s[jj] * a.scale * (float)mk[jj >> 2][jj & 3];
      r_part += fabsf(p);
      pf[jj >> 3][jj & 7] = (T)p;
    }

    // ---- O^T_half += V_half^T P^T
#pragma unroll
    for (int i = 0; i < NPV; i++) {
      if (i + PF - 1 < NPV) v_request(i + PF - 1);
      __builtin_amdgcn_sched_barrier(0);
      x8 vf = __builtin_shufflevector(lo[i % PF], hi[i % PF], 0, 1, 2, 3, 4, 5, 6, 7);
      o[i >> 1] = E::mfma32(vf, pf[i & 1], o[i >> 1]);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  __syncthreads();   // every wave is done with the K/V buffers: they become output staging

  const float r_tot = fmaxf(r_part + xhalf(r_part), 1.f);
  const float inv = 1.f / r_tot;
  if (a.row_scale && hf == 0 && g == 0 && m_lane < a.Sq) a.row_scale[((int64_t)b * a.H + h) * a.Sq + m_lane] = r_tot;

  // ---- O: this wave's 256 columns in two halves of 128 through a wave-private LDS block, coalesced 16-byte stores
  constexpr int HALF = RP_DV / 4, OROW = HALF * 2 + 16;
  const uint32_t ob = lds0 + wave * 32 * OROW;
  T* obase = (T*)a.o + (int64_t)b * a.osb + (int64_t)h * a.osh + hf * (RP_DV / 2);
#pragma unroll
  for (int hp = 0; hp < 2; hp++) {
#pragma unroll
    for (int dbl = 0; dbl < DBH / 2; dbl++)
#pragma unroll
      for (int q4 = 0; q4 < 4; q4++) {
        x4 w;
#pragma unroll
        for (int i = 0; i < 4; i++) w[i] = (T)(o[hp * (DBH / 2) + dbl][4 * q4 + i] * inv);
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

template <typename T, bool CAUSAL>
static int launch_pair(const AttnArgs& a, hipStream_t stream) {
  auto kern = retention_pair_fwd_kernel<T, CAUSAL>;
  static std::atomic<uint64_t> lds_ok{0};
  if (allow_lds(lds_ok, RP_LDS, kern) != 0) return -1;
  AttnArgs args = a;
  args.num_m_blocks = (a.Sq + RP_BM - 1) / RP_BM;
  hipLaunchKernelGGL(kern, dim3((unsigned)(args.num_m_blocks * a.B * a.H)), dim3(64 * RP_NW), RP_LDS, stream, args);
  return launch_status();
}

// returns 0 ok, -1 launch failure
int retention_pair_fwd_dispatch(const AttnArgs& a, bool causal, bool is_bf16, hipStream_t stream) {
  if (is_bf16) return causal ? launch_pair<__bf16, true>(a, stream) : launch_pair<__bf16, false>(a, stream);
  return causal ? launch_pair<_Float16, true>(a, stream) : launch_pair<_Float16, false>(a, stream);
}

}  // namespace ma
