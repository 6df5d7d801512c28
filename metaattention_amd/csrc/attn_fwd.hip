// Parallel (flash-style) attention forward for gfx950.
//
// Replaces the operator the reference renders from
// attention_engine/core/template/tl_template/attn/attn_tl.py:92-190: per Q tile,
// loop over KV tiles: S = Q K^T, elementwise score function, online row
// function, O = O * o_scale + P V.  The row functions are the fixed library
// variants documented in include/metaattention_hip.h.
//
// Mapping onto CDNA4 (wave64, v_mfma_f32_32x32x16):
//   * a workgroup is 8 waves (two per SIMD, one workgroup per CU); each wave owns 32 query rows
//     (block_M = 256) and every wave walks the same 32-row KV sub-tiles, which arrive in LDS by
//     direct-to-LDS DMA through rings of 6 K and 6 V buffers (K runs 6, V 4 sub-tiles ahead; each wave
//     issues one K and one V instruction per sub-tile, spread between its MFMAs: a wave that issues a
//     burst of loads stalls on the CU's vector memory path, so also the first sub-tiles of the NEXT work
//     item are fetched one per step, by the last steps of the item before it);
//   * the score tile is computed TRANSPOSED, S^T = K Q^T (A = K rows from LDS,
//     B = Q held in registers), so that in the accumulator layout every lane
//     owns ONE query row: the online row statistics are per-lane scalars, the
//     row reductions are in-register ops plus one exchange with lane^32, and
//     the probabilities are already in B-operand layout for O^T += V^T P^T with
//     no LDS round trip;
//   * V^T fragments come straight out of the row-major V tile with the
//     transposing LDS read (ds_read_b64_tr_b16);
//   * both LDS tiles are XOR-swizzled at 16-byte granularity so the 128-bit K
//     reads and the transposing V reads are bank-conflict free without padding;
//   * two phases per sub-tile and wave, and the two waves of a SIMD in opposite phases.  Matrix phase of step u:
//     the MFMAs of P(u-1) V(u-1) and K(u+1) Q^T back to back, their fragments read from LDS a few MFMAs ahead,
//     nothing else.  Vector phase: the DMA instructions of the step, mask, exponentials, row sum, conversion of
//     sub-tile u, and the first fragment requests of the next matrix phase.  There is one workgroup barrier per
//     step; waves 0..3 pass it before their matrix phase, waves 4..7 between their matrix and their vector phase,
//     so between two barriers one wave of every SIMD runs matrix-then-vector and the other vector-then-matrix.
//     Timestamps inside the kernel: matrix phase 650 clocks (16 MFMAs), vector phase 850 (of them 200 in which the
//     wave stands still while the CU's vector memory path takes its two DMA instructions, 480 of vector ALU: a
//     v_exp_f32 holds the ALU for 16 clocks).  Interleaving both kinds of work inside each wave (one MFMA, a few
//     vector instructions, ...) measured 4 % slower, a second barrier between the phases 2 % slower (the phases
//     are not equally long, and every stall of one wave is then waited for by all);
//   * scores and probabilities of two sub-tiles are live in registers (s[u & 1], p[u & 1]);
//   * the reference point of the exponentials follows the running maximum lazily and optimistically: a
//     step takes its exponentials relative to the reference as it stands and checks afterwards whether some
//     row's scores exceeded it by more than 2^8; only then (rare) the reference moves, which is a cold path
//     that rescales the accumulator and takes that sub-tile's exponentials again (see `move_ref`).
#include "attn_fwd.h"

#include <type_traits>
#include <utility>

namespace ma {

enum { FAM_SOFTMAX = 0, FAM_SIGMOID = 1, FAM_RELU = 2 };
constexpr int ATTN_NBUF = 6;   // K and V ring slots (32-row sub-tiles)

namespace {
template <int B, int... I, typename F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
  (f(std::integral_constant<int, B + I>{}), ...);
}
// f(integral_constant<int, i>) for i in [B, E), fully unrolled with compile-time indices
template <int B, int E, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl<B>(std::make_integer_sequence<int, E - B>{}, f);
}
}  // namespace

template <typename T, int DQK, int DV, int FAMILY, bool CAUSAL>
__global__ __launch_bounds__(512, 2) void attn_fwd_kernel(const AttnArgs a) {
  using E = Elem<T>;
  using x8 = typename E::x8;
  using x4 = typename E::x4;
  using x2 = typename E::x2;
  constexpr int NW = 8, BM = 32 * NW, BN = 32, NBUF = ATTN_NBUF;
  constexpr int DK_AHEAD = 6, DV_AHEAD = 4;   // step u issues the loads of K(u + 6) and V(u + 4)
  constexpr int KS = DQK / 16;   // k-slices of the QK^T contraction
  constexpr int DB = DV / 32;    // 32-wide output column blocks
  constexpr int CPRK = DQK / 8, CPRV = DV / 8;  // 16-byte chunks per row
  constexpr int KROW = DQK * 2, VROW = DV * 2;
  constexpr int KTILE = BN * KROW, VTILE = BN * VROW;
  constexpr int NQK = KS, NPV = 2 * DB;                  // MFMAs per sub-tile
  static_assert(NBUF == 6, "the step bodies are unrolled by ring slot and by the parity of the score / probability buffers");
  static_assert(CPRK == 16 && CPRV == 16, "one DMA instruction (1 KB) covers 4 tile rows");
  static_assert(KTILE == NW * 1024 && VTILE == NW * 1024, "one K and one V DMA instruction per wave and sub-tile");
  static_assert(NQK == NPV && NQK + NPV == 16, "one MFMA pair per two score elements");
  static_assert(NBUF * KTILE <= 65536, "ring offsets must fit the 16-bit LDS instruction offset");

  extern __shared__ __align__(16) char smem[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(MA_LDS char*)smem;
  const uint32_t lds_k = lds0, lds_v = lds0 + NBUF * KTILE;   // [K ring][V ring]

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), r = lane & 31, g = lane >> 5;
  // Waves w and w + 4 share a SIMD.  Their 32-row blocks are paired as (0,7) (1,6) (2,5) (3,4) so that under
  // a causal mask, where a block's work grows with its position, every SIMD gets the same amount.
  const int row_block = wave < 4 ? wave : 11 - wave;
  const bool late = wave >= 4;   // passes the step's barrier between its two phases instead of before them

  // ---- per work item (one 256-row q block of one (batch, head)); see the item loop at the bottom
  int b = 0, h = 0, mb = 0, m_wave = 0, m_lane = 0;
  x8 qf[KS];                                   // Q fragments (B operand of S^T = K Q^T), kept in registers
  const char *kbase = nullptr, *vbase = nullptr;
  int n_sub = 0, last_sub = 0;                 // sub-tiles the workgroup walks; the last one this wave has anything to do in
  // The K/V stream runs on into the next item: the loads that an item's last steps would spend on sub-tile positions
  // past its end (n_sub, n_sub + 1, ..) fetch the first sub-tiles of the item that follows instead.  That item expects
  // sub-tile j in ring slot j, so the load bound for slot j fetches its sub-tile j, whatever the position: the next
  // item's first sub-tiles arrive in rotated order, and each slot is refilled by the usual rule (after the barrier
  // that ends the last use of what it held).  With no item after it, these loads fetch rows of the item itself.
  const char *kbase_n = nullptr, *vbase_n = nullptr;
  int v_fix = ATTN_NBUF - 1;                   // the one V slot that the item before this one could not refill (see the prologue)

  // ---- DMA of one K or V sub-tile: 8 instructions of 1 KB (4 tile rows), one per wave; lane i fetches
  //      the 16-byte chunk that belongs at physical position i of that KB.  Wave w has tile rows
  //      4w + lane/16, whose swizzle term swz16(row) = ((lane/16) << 2) | (w & 3).  Rows beyond the
  //      sequence are clamped to its last row (their scores are masked, their probabilities exactly 0),
  //      so every step issues the same two instructions without a branch, also past the end.
  //      Addressing is scalar base + 32-bit lane offset: the host checks that a (batch, head) plane of
  //      K or V spans less than 4 GB.
  const uint32_t swz_lane = (uint32_t)((((lane & 15) ^ ((lane >> 4) << 2)) ^ (wave & 3)) << 4);
  const int tile_row = 4 * wave + (lane >> 4);
  const uint32_t k_row_bytes = (uint32_t)(a.kss * 2), v_row_bytes = (uint32_t)(a.vss * 2);
  //      Positions from n_sub on fetch the next item's sub-tile `slot` (a position more than a turn of the ring past
  //      the end repeats an earlier one: the same bytes into the same slot).
  const uint32_t k_lane_off = (uint32_t)tile_row * k_row_bytes + swz_lane, v_lane_off = (uint32_t)tile_row * v_row_bytes + swz_lane;
  auto issue_rt = [&](int su, uint32_t slot, const char* cur, const char* nxt, uint32_t row_bytes, uint32_t lane_off, uint32_t lds_dst)
      __attribute__((always_inline)) {
    const bool nx = su >= n_sub;
    const int row0 = (nx ? (int)slot : su) * BN;
    const char* base = nx ? nxt : cur;
    if (row0 + BN <= a.Skv) {   // (wave-uniform) whole sub-tile inside the sequence: scalar base, the lane's constant offset
      dma16_so(base + (uint64_t)((uint32_t)row0 * row_bytes), lane_off, lds_dst);
    } else {
      const uint32_t row = (uint32_t)min(row0 + tile_row, a.Skv - 1);
      dma16_so(base, row * row_bytes + swz_lane, lds_dst);
    }
  };
  auto issue_k_rt = [&](int su, uint32_t slot) __attribute__((always_inline)) {
    issue_rt(su, slot, kbase, kbase_n, k_row_bytes, k_lane_off, lds_k + slot * KTILE + wave * 1024);
  };
  auto issue_v_rt = [&](int su, uint32_t slot) __attribute__((always_inline)) {
    issue_rt(su, slot, vbase, vbase_n, v_row_bytes, v_lane_off, lds_v + slot * VTILE + wave * 1024);
  };

  // ---- per-lane LDS read addresses: all lane-dependent parts, one register each; what is added per
  //      read (ring slot, 16-row slice) is a compile-time immediate
  // K (A operand of S^T): row r, logical chunk 2ks + g
  // V (A operand of O^T, through the transposing read): lane block = lane/16,
  //   row 16sl + 8*half + 4g + jr, logical chunk 4db + lc
  const uint32_t k_row_off = r * KROW;
  const int k_chunk0 = g ^ swz16(r);
  const int jr = (lane & 15) >> 2;
  const int lc = (((lane >> 4) & 1) << 1) | ((lane & 3) >> 1);
  const uint32_t v_row_off = (4 * g + jr) * VROW + (lane & 1) * 8;
  const int v_chunk0 = lc ^ swz16(4 * g + jr);
  constexpr int V_HALF_XOR = 2;  // swz16(row + 8) ^ swz16(row) for row < 8; swz16(row + 16) == swz16(row)
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
  const float bias = a.bias + (a.bias_ptr ? *a.bias_ptr : 0.f);
  const float c_scale = a.scale * kLog2e;  // scores are handled in the log2 domain
  const float c_bias = bias * kLog2e;
  float row_ref = 0.f;     // softmax: reference point of the exponentials, (scale * s + bias) * log2e of some earlier running max
  float row_sum = 0.f;     // this lane's share of the running sum (the other half lives in lane^32)

  // scores s[u & 1] and probabilities p[u & 1] of sub-tile u.
  // lane holds query row r; element jj of a sub-tile is kv row 8(jj/4) + 4g + jj%4.
  // p[par][sl] packs elements 8sl .. 8sl+7: the B operand of PV slice sl (k slot i of lane half g is
  // kv row 16sl + 8(i/4) + 4g + i%4, matched by the rows the transposing V reads fetch).
  f32x16 s[2];
  u32x4 p[2][2];
  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

  // structural mask of sub-tile su (scores in s[SB]): exact -inf above the diagonal / beyond the cache
  auto apply_mask = [&](auto sb_c, int su) __attribute__((always_inline)) {
    constexpr int SB = decltype(sb_c)::value;
    const int n0 = su * BN;
    if ((CAUSAL && (n0 + BN - 1 > m_wave)) || (n0 + BN > a.Skv)) {
      const int lim = CAUSAL ? min(m_lane, a.Skv - 1) : a.Skv - 1;
#pragma unroll
      for (int j = 0; j < 16; j++) {
        const int n = n0 + 8 * (j >> 2) + 4 * g + (j & 3);
        if (n > lim) s[SB][j] = -INFINITY;
      }
    }
  };

  // one score -> probability (and its contribution to the row sum); sub = c_bias - row_ref
  auto prob_one = [&](float v, float sub, float& part) __attribute__((always_inline)) -> float {
#pragma clang fp reassociate(off)   // keep the running sum a chain in element order
    if constexpr (FAMILY == FAM_SOFTMAX) {
      const float pe = fast_exp2(v * c_scale + sub);
      part += pe;
      return pe;
    } else if constexpr (FAMILY == FAM_SIGMOID) {   // sigmoid(x) = 1 / (1 + 2^(-x log2e)); s = -inf gives exactly 0
      return fast_rcp(1.f + fast_exp2(-(v * c_scale + c_bias)));
    } else {
      return fmaxf(v * a.scale + bias, 0.f);
    }
  };
  // elements e0, e0+1 packed into p[PAR]
  auto pack_pair = [&](auto par_c, auto e_c, float pe0, float pe1) __attribute__((always_inline)) {
    constexpr int PAR = decltype(par_c)::value, e0 = decltype(e_c)::value;
    x2 pk;
    pk[0] = (T)pe0;
    pk[1] = (T)pe1;
    uint32_t w = __builtin_bit_cast(uint32_t, pk);
    // (pinned where it stands: the cold path takes a step's probabilities again, and without this the compiler moves
    // the first take, exponentials and all, from between the MFMAs to behind the branch around that path)
    asm volatile("" : "+v"(w));
    p[PAR][e0 >> 3][(e0 & 7) >> 1] = w;
  };

  // Softmax, cold path.  A step takes the exponentials of its sub-tile relative to the reference point as it
  // stands (at most 2^8 while the scores stay within 8 of it: exact in fp32, in range for bf16/fp16; the final
  // division by row_sum absorbs the offset) and afterwards looks at the sub-tile's maximum `mx`.  Only if some
  // row exceeded its reference by more than 8 does the step come here: such rows move their reference up to
  // the new maximum, the accumulator and the row sum are rescaled, and the probabilities of this step's sub-tile
  // (scores in s[SB], probabilities pending in p[PAR]) are taken again.  Each row decides for itself (rows that
  // stay multiply by exactly 1), so a row's result never depends on what other rows of its wave see.
  auto move_ref = [&](auto par_c, auto sb_c, float& part) __attribute__((always_inline)) {
    constexpr int SB = decltype(sb_c)::value;
    float mx = s[SB][0];
#pragma unroll
    for (int j = 1; j < 16; j++) mx = fmaxf(mx, s[SB][j]);
    float m_lo, m_hi;
    xhalf_pair(mx, m_lo, m_hi);
    const float cand = fmaxf(m_lo, m_hi) * c_scale + c_bias;
    const bool move = cand - row_ref > 8.f;
    const float corr = move ? fast_exp2(row_ref - cand) : 1.f;
    row_ref = move ? cand : row_ref;
    row_sum *= corr;
    // In place by construction, and with the wait states that cover the longest MFMA-result-to-VALU
    // hazard (only the compiler's own instructions get those for free).
    asm volatile("s_nop 7\n s_nop 7\n s_nop 7");
#pragma unroll
    for (int i = 0; i < DB; i++)
#pragma unroll
      for (int j = 0; j < 16; j++) asm volatile("v_mul_f32 %0, %0, %1" : "+v"(o[i][j]) : "v"(corr));
    part = 0.f;
    const float sub = c_bias - row_ref;
    static_for<0, 8>([&](auto i_c) __attribute__((always_inline)) {
      constexpr int i = decltype(i_c)::value;
      const float pe0 = prob_one(s[SB][2 * i], sub, part);
      const float pe1 = prob_one(s[SB][2 * i + 1], sub, part);
      pack_pair(par_c, std::integral_constant<int, 2 * i>{}, pe0, pe1);
    });
  };

  // K and V fragments travel through small register rings and are requested PF-1 MFMA pairs ahead, across
  // step boundaries: pair i of a step is PV MFMA i (V slice i / DB, column block i % DB) and QK MFMA i
  // (k-slice i).
  constexpr int PF = 3;
  x4 lo[PF], hi[PF];
  x8 kf[PF];
  // pair I of the step whose V is in ring slot VSLOT and whose K is in ring slot KSLOT
  auto request = [&](auto i_c, auto vslot_c, auto kslot_c) __attribute__((always_inline)) {
    constexpr int I = decltype(i_c)::value, VS = decltype(vslot_c)::value, KSL = decltype(kslot_c)::value;
    constexpr int sl = I / DB, db = I % DB;
    lo[I % PF] = lds_read_tr4<T>(v_addr[db][0] + VS * VTILE + 16 * sl * VROW);
    hi[I % PF] = lds_read_tr4<T>(v_addr[db][1] + VS * VTILE + 16 * sl * VROW);
    kf[I % PF] = lds_read<x8>(k_addr[I] + KSL * KTILE);
  };

  // Step u of a wave, in two phases; SLOT = u % 6 is compile-time and fixes the ring slots and the score and
  // probability buffers (u & 1).
  // Matrix phase:
  //   O^T += V(u-1)^T P(u-1)^T   V ring slot SLOT-1, probabilities p[1-PAR]
  //   s[1-PAR] = K(u+1) Q^T      K ring slot SLOT+1
  auto g_phase = [&](auto slot_c) __attribute__((always_inline)) {
    constexpr int SLOT = decltype(slot_c)::value, PAR = SLOT & 1;
    constexpr auto vs_c = std::integral_constant<int, (SLOT + NBUF - 1) % NBUF>{};
    constexpr auto ks_c = std::integral_constant<int, (SLOT + 1) % NBUF>{};
    static_for<0, NPV>([&](auto i_c) __attribute__((always_inline)) {
      constexpr int i = decltype(i_c)::value;
      if constexpr (i + PF - 1 < NPV) request(std::integral_constant<int, i + PF - 1>{}, vs_c, ks_c);
      __builtin_amdgcn_sched_barrier(0);
      x8 vf = __builtin_shufflevector(lo[i % PF], hi[i % PF], 0, 1, 2, 3, 4, 5, 6, 7);
      o[i % DB] = E::mfma32(vf, __builtin_bit_cast(x8, p[1 - PAR][i / DB]), o[i % DB]);
      s[1 - PAR] = E::mfma32(kf[i % PF], qf[i], i == 0 ? zero16 : s[1 - PAR]);
      __builtin_amdgcn_sched_barrier(0);
    });
  };
  // Vector phase: mask, probabilities and maximum of sub-tile u from s[PAR] into p[PAR]; the loads of K(u+6) and
  // V(u+4); and, last, the first fragment requests of the next matrix phase (V(u), K(u+2)).
  auto s_phase = [&](auto slot_c, int u) __attribute__((always_inline)) {
    constexpr int SLOT = decltype(slot_c)::value, PAR = SLOT & 1;
    constexpr auto par_c = std::integral_constant<int, PAR>{};
    constexpr auto vs_next_c = std::integral_constant<int, SLOT>{};
    constexpr auto ks_next_c = std::integral_constant<int, (SLOT + 2) % NBUF>{};
    issue_k_rt(u + DK_AHEAD, (SLOT + DK_AHEAD) % NBUF);
    issue_v_rt(u + DV_AHEAD, (SLOT + DV_AHEAD) % NBUF);
    apply_mask(par_c, u);
    float part = 0.f;
    const float sub = c_bias - row_ref;
    static_for<0, 8>([&](auto i_c) __attribute__((always_inline)) {
      constexpr int i = decltype(i_c)::value;
      const float pe0 = prob_one(s[PAR][2 * i], sub, part);
      const float pe1 = prob_one(s[PAR][2 * i + 1], sub, part);
      pack_pair(par_c, std::integral_constant<int, 2 * i>{}, pe0, pe1);
    });
    if constexpr (FAMILY == FAM_SOFTMAX) {
      asm volatile("" : "+v"(part));   // (as in pack_pair)
      if (__builtin_expect(__any(!(part <= 4096.f)), 0)) move_ref(par_c, par_c, part);
      row_sum += part;
    }
    static_for<0, PF - 1>([&](auto i_c) __attribute__((always_inline)) { request(i_c, vs_next_c, ks_next_c); });
  };

  // ---- work items.  The grid is one workgroup per CU and every workgroup walks its share of the
  //      (batch*head, q block) items: a workgroup of this size owns its CU, and launching a fresh one per
  //      item leaves the CU idle for several microseconds between items.  Consecutive workgroup ids are
  //      dealt round-robin to the 8 XCDs, so XCD x takes the (batch, head) pairs with bh % 8 == x and
  //      its CUs work on the q blocks of the same few pairs at the same time (their K/V stays in that
  //      XCD's L2).  Under a causal mask a q block's work grows with its position, so the unit of work
  //      is a pair of q blocks (k, nmb-1-k) of one (batch, head): every unit weighs the same.
  //      The first sub-tiles of an item (K(0..5), V(0..3)) are fetched by the last steps of the item before it,
  //      and its Q rows are requested before that item's output is written.
  const int nmb = a.num_m_blocks, BH = a.B * a.H, G = (int)gridDim.x;
  const bool paired = CAUSAL && BH * nmb > G;               // (few items: one q block per unit, spread wide)
  const bool by_xcd = (BH & 7) == 0 && (G & 7) == 0;
  // With an even number of (batch, head) pairs per XCD the two q blocks of a unit come from two pairs: block i of pair 2s,
  // then block nmb-1-i of pair 2s+1.  Units still weigh the same, so the workgroups that share pair 2s start their first
  // items together, at key 0 of the same K/V planes: those rows are read from HBM once and need no room in L2 beyond the
  // rows in flight; only the second items, which start one after the other, need their pair's planes resident.  At
  // S = 4096 (16 q blocks, 2 MB of K/V per pair) the 32 workgroups of an XCD cover two such units of pairs: 4 MB to keep
  // in the XCD's 4 MB of L2, where both q blocks from one pair made it the planes of four pairs, 8 MB (HBM reads 0.94
  // against 1.27 GB per launch at B8 H32).  Longer sequences, whose planes do not fit either way, keep both blocks from one
  // pair: there the second items of this order, half of them long, re-read more (S = 8192: 1.5 % slower).
  const bool cross = paired && by_xcd && ((BH >> 3) & 1) == 0 && (int64_t)a.Skv * (DQK + DV) * 2 <= (2 << 20);
  const int upb = cross ? nmb : paired ? (nmb + 1) >> 1 : nmb;   // units per (batch, head), per two of them if `cross`
  const int units = cross ? (BH >> 4) * upb : by_xcd ? (BH >> 3) * upb : BH * upb;   // units of this workgroup's stream
  const int first = by_xcd ? (int)blockIdx.x >> 3 : (int)blockIdx.x, stride = by_xcd ? G >> 3 : G;
  // item cursor t = 2 * unit + half; returns the next cursor that names an item (or one past the end)
  int t_next = 0;
  auto next_item = [&](int t) -> int {
    for (;;) {
      t = (t & 1) ? t + 2 * stride - 1 : t + 1;
      if (t >= 2 * units || cross) return t;
      const int k = (t >> 1) % upb;
      if (paired ? !((t & 1) && k == nmb - 1 - k) : !(t & 1)) return t;   // (the middle block of an odd count is its own partner)
    }
  };
  // (batch, head) planes of item t
  auto planes_of = [&](int t, const char*& kb, const char*& vb, int& b_, int& h_) __attribute__((always_inline)) {
    int bh = (t >> 1) / upb;
    if (cross) bh = 2 * bh + (t & 1);
    if (by_xcd) bh = bh * 8 + ((int)blockIdx.x & 7);
    b_ = bh / a.H;
    h_ = bh % a.H;
    kb = (const char*)((const T*)a.k + (int64_t)b_ * a.ksb + (int64_t)(h_ / a.kv_group) * a.ksh);
    vb = (const char*)((const T*)a.v + (int64_t)b_ * a.vsb + (int64_t)(h_ / a.kv_group) * a.vsh);
  };
  // decode item t into the per-item variables, request its Q rows, and look up the item after it
  auto open_item = [&](int t) __attribute__((always_inline)) {
    const int k = (t >> 1) % upb;
    mb = cross ? ((t & 1) ? nmb - 1 - k : k) : paired ? ((t & 1) ? k : nmb - 1 - k) : (CAUSAL ? nmb - 1 - k : k);
    planes_of(t, kbase, vbase, b, h);
    // V positions n_sub .. n_sub + 4 of the item before this one (its steps n_sub - 4 .. n_sub) refilled every V slot
    // but the one of its own last sub-tile
    v_fix = n_sub > 0 ? (n_sub - 1) % NBUF : NBUF - 1;
    m_wave = mb * BM + row_block * 32;  // first query row of this wave
    m_lane = m_wave + r;
    n_sub = (a.Skv + BN - 1) / BN;
    if (CAUSAL) n_sub = min(n_sub, (mb * BM + BM) / BN);
    last_sub = CAUSAL ? min(n_sub - 1, m_wave / BN) : n_sub - 1;
    // Q rows, coalesced: instruction i fetches rows 4i .. 4i+3 of the wave's 32, sixteen lanes per row (the registers
    // of qf carry them until `q_fragments` turns them into fragments)
    const T* qp = (const T*)a.q + (int64_t)b * a.qsb + (int64_t)h * a.qsh + 8 * (lane & 15);
#pragma unroll
    for (int ks = 0; ks < KS; ks++) qf[ks] = *(const x8*)(qp + (int64_t)min(m_wave + 4 * ks + (lane >> 4), a.Sq - 1) * a.qss);
    t_next = next_item(t);
    if (t_next < 2 * units) {
      int b_n, h_n;
      planes_of(t_next, kbase_n, vbase_n, b_n, h_n);
    } else {
      kbase_n = kbase;
      vbase_n = vbase;
    }
  };

  // the Q rows as loaded by open_item -> fragments (lane: row r, columns 16ks + 8g ..), through this
  // wave's rows of the output staging area (16-byte chunks XOR-swizzled by row, as the output uses it)
  auto q_fragments = [&]() __attribute__((always_inline)) {
    static_assert(DQK == DV, "the staging rows hold one Q row each");
    const uint32_t qb = lds0 + NBUF * (KTILE + VTILE) + wave * 32 * VROW;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      const int row = 4 * ks + (lane >> 4);
      lds_write<x8>(qb + row * VROW + (((lane & 15) ^ (row & 15)) << 4), qf[ks]);
    }
#pragma unroll
    for (int ks = 0; ks < KS; ks++) qf[ks] = lds_read<x8>(qb + r * VROW + (((2 * ks + g) ^ (r & 15)) << 4));
  };

  int stores_behind = 0;   // output stores this wave issued after the current item's first loads
  int t_cur = 2 * first;
  // An item that nobody fetched ahead for (the first of the workgroup; the one after an item of fewer than 5 sub-tiles,
  // whose few steps do not get round the ring): K(0..5) -> slots 0..5, V(0..3) -> slots 0..3.
  auto fetch_first = [&]() __attribute__((always_inline)) {
    static_for<0, NBUF>([&](auto t_c) __attribute__((always_inline)) {
      constexpr int tt = decltype(t_c)::value;
      issue_k_rt(tt, tt);
      if constexpr (tt < DV_AHEAD) issue_v_rt(tt, tt);
    });
    v_fix = NBUF - 1;
  };
  if (t_cur < 2 * units) {
    open_item(t_cur);
    fetch_first();
  }
  while (t_cur < 2 * units) {
#pragma unroll
    for (int i = 0; i < DB; i++)
#pragma unroll
      for (int j = 0; j < 16; j++) o[i][j] = 0.f;
#pragma unroll
    for (int i = 0; i < 2; i++) p[0][i] = p[1][i] = u32x4{0u, 0u, 0u, 0u};
    row_sum = 0.f;

    // ---- schedule.  Step u (u = 0 .. last_sub + 1 for a wave): the matrix phase reads K(u+1) and V(u-1), the vector
    //      phase issues the loads of K(u+6) and V(u+4) and reads the first fragments of K(u+2) and V(u).  Barrier u
    //      stands before the matrix phase of waves 0..3 and between the two phases of waves 4..7, so it has: every
    //      matrix phase of step u-1 behind it (every wave is done reading K(<=u) and V(<=u-2), the ring slots that
    //      the loads of step u refill), every vector phase of step u before it, and of the matrix phases of step u
    //      those of waves 4..7 behind it.  What is read after it, K(u+1), K(u+2), V(u-1), V(u), must therefore have
    //      landed for every wave: K(u+2) and V(u) are the pair of step u-4, a wave's loads complete in order, and at
    //      barrier u every wave has issued the pairs of steps <= u-1, so the six instructions of steps u-3 .. u-1 may
    //      still be in flight.
    // the item's first sub-tiles (fetched by the previous item's last steps) and Q rows must have landed; the previous
    // item's output stores, issued after them, need not
    if (stores_behind == 32 * CPRV / 64 + 1) __builtin_amdgcn_s_waitcnt(0x0F70 | (32 * CPRV / 64 + 1));
    else if (stores_behind == 32 * CPRV / 64) __builtin_amdgcn_s_waitcnt(0x0F70 | (32 * CPRV / 64));
    else wait_dma();
    q_fragments();
    __syncthreads();
    // The V slot that did not get this item's sub-tile yet (slots 4 and 5 get theirs again from steps 0 and 1).  In the
    // first item of a workgroup it is slot NBUF-1: the first step multiplies that slot with zero probabilities, and
    // with V(5) in it whatever is there is finite unless this (batch, head)'s own values are not.
    {
      const uint32_t row = (uint32_t)min(v_fix * BN + tile_row, a.Skv - 1);
      dma16_so(vbase, row * v_row_bytes + swz_lane, lds_v + (uint32_t)v_fix * VTILE + wave * 1024);
    }
    {   // s[0] = K(0) Q^T.  Softmax: the row's first reference point is the maximum of this sub-tile (finite: every row
        // sees key 0).
      x8 k0[KS];
  #pragma unroll
      for (int ks = 0; ks < KS; ks++) k0[ks] = lds_read<x8>(k_addr[ks]);
  #pragma unroll
      for (int ks = 0; ks < KS; ks++) s[0] = E::mfma32(k0[ks], qf[ks], ks == 0 ? zero16 : s[0]);
      if constexpr (FAMILY == FAM_SOFTMAX) {
        apply_mask(std::integral_constant<int, 0>{}, 0);
        float mx = s[0][0];
  #pragma unroll
        for (int j = 1; j < 16; j++) mx = fmaxf(mx, s[0][j]);
        float m_lo, m_hi;
        xhalf_pair(mx, m_lo, m_hi);
        row_ref = fmaxf(m_lo, m_hi) * c_scale + c_bias;
      }
    }
    wait_dma();
    __syncthreads();   // V ring slot NBUF-1 is filled (and every wave is done reading K(0): step 0 refills its slot)
    static_for<0, PF - 1>([&](auto i_c) __attribute__((always_inline)) {   // first fragments of step 0: zeros, K(1)
      request(i_c, std::integral_constant<int, NBUF - 1>{}, std::integral_constant<int, 1>{});
    });
    const int my_steps = last_sub + 2;   // steps 0 .. last_sub + 1
    for (int u0 = 0; u0 < my_steps; u0 += NBUF) {
      static_for<0, NBUF>([&](auto slot_c) __attribute__((always_inline)) {
        constexpr int SLOT = decltype(slot_c)::value;
        const int u = u0 + SLOT;
        if (u < my_steps) {
          // (s_barrier alone: __syncthreads would also wait for the LDS reads in flight, the fragments that the vector
          // phase has requested for the matrix phase behind the barrier)
          if (!late) {
            __builtin_amdgcn_s_waitcnt(0x0F70 | 6);   // vmcnt(6)
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
          }
          g_phase(slot_c);
          if (late) {
            __builtin_amdgcn_s_waitcnt(0x0F70 | 6);
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
          }
          s_phase(slot_c, u);
        }
      });
    }
    // nothing left for this wave: keep feeding the rings and meeting the barriers of the others
    {
      uint32_t kslot = (uint32_t)((my_steps + DK_AHEAD) % NBUF), vslot = (uint32_t)((my_steps + DV_AHEAD) % NBUF);
      for (int u = my_steps; u <= n_sub; u++) {
        wait_dma();
        __syncthreads();
        issue_k_rt(u + DK_AHEAD, kslot);
        issue_v_rt(u + DV_AHEAD, vslot);
        kslot = kslot + 1 == NBUF ? 0 : kslot + 1;
        vslot = vslot + 1 == NBUF ? 0 : vslot + 1;
      }
    }

    // ---- what the epilogue needs of this item, then the next item's Q rows, then the epilogue
    T* const obase = (T*)a.o + (int64_t)b * a.osb + (int64_t)h * a.osh + (int64_t)m_wave * a.oss;
    const int m_out = m_wave;
    float* const lse_ptr = a.row_scale ? a.row_scale + ((int64_t)b * a.H + h) * a.Sq + m_lane : nullptr;
    const bool row_ok = m_lane < a.Sq;
    t_cur = t_next;
    if (t_cur < 2 * units) {
      const bool unfetched = n_sub < 5;
      open_item(t_cur);
      if (unfetched) {
        wait_dma();
        __syncthreads();   // every wave is done with the K/V rings
        fetch_first();
      }
    }

    // normalise, stage O through LDS (wave-private rows, 16-byte chunks XOR-swizzled by row so that neither
    // the 8-byte writes nor the 16-byte reads pile onto one bank group), coalesced 16-byte stores.  The
    // staging area lies behind the rings, which already hold the next item's first sub-tiles.
    float inv = 1.f, lse = 0.f;
    if constexpr (FAMILY == FAM_SOFTMAX) {
      float s_lo, s_hi;
      xhalf_pair(row_sum, s_lo, s_hi);
      const float tot = s_lo + s_hi;
      inv = 1.f / tot;
      lse = (row_ref + fast_log2(tot)) * kLn2;
    }
    // (the lane id is laundered so that the address arithmetic below is redone per item instead of being
    // hoisted out of the item loop, where it would occupy registers the main loop has no room for)
    int lane_e = lane;
    asm volatile("" : "+v"(lane_e));
    const int r_e = lane_e & 31, g_e = lane_e >> 5;
    const uint32_t ob = lds0 + NBUF * (KTILE + VTILE) + wave * 32 * VROW;
    const uint32_t ow = ob + r_e * VROW + 8 * g_e;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int q4 = 0; q4 < 4; q4++) {
        x4 w;
#pragma unroll
        for (int i = 0; i < 4; i++) w[i] = (T)(o[db][4 * q4 + i] * inv);
        lds_write<x4>(ow + (((4 * db + q4) ^ (r_e & 15)) << 4), w);
      }
    // Stores count in the same in-order counter as the loads that were just started for the next item.
    // A wave whose 32 rows all exist issues a known number of them, and the next item only waits for what
    // is older than these stores; otherwise it waits for everything.
    constexpr int NST = 32 * CPRV / 64;
    if (m_out + 32 <= a.Sq) {
#pragma unroll
      for (int it = 0; it < NST; it++) {
        const int ci = lane_e + 64 * it, row = ci / CPRV, c = ci % CPRV;
        u32x4 w = lds_read<u32x4>(ob + row * VROW + ((c ^ (row & 15)) << 4));
        *(u32x4*)(obase + (int64_t)row * a.oss + c * 8) = w;
      }
      if (FAMILY == FAM_SOFTMAX && lse_ptr) {
        if (g_e == 0) *lse_ptr = lse;
        stores_behind = NST + 1;
      } else {
        stores_behind = NST;
      }
    } else {
#pragma unroll
      for (int it = 0; it < NST; it++) {
        const int ci = lane_e + 64 * it, row = ci / CPRV, c = ci % CPRV;
        u32x4 w = lds_read<u32x4>(ob + row * VROW + ((c ^ (row & 15)) << 4));
        if (m_out + row < a.Sq) *(u32x4*)(obase + (int64_t)row * a.oss + c * 8) = w;
      }
      if constexpr (FAMILY == FAM_SOFTMAX) {
        if (lse_ptr && g_e == 0 && row_ok) *lse_ptr = lse;
      }
      stores_behind = 0;
    }
  }
}

template <typename T, int DQK, int DV, int FAMILY, bool CAUSAL>
static int launch(const AttnArgs& a, hipStream_t stream) {
  constexpr int BM = 256, BN = 32, NBUF = ATTN_NBUF;
  constexpr size_t tiles = NBUF * (size_t)BN * (DQK + DV) * 2;
  constexpr size_t lds = tiles + 8 * 32 * (size_t)DV * 2;   // rings + output staging
  auto kern = attn_fwd_kernel<T, DQK, DV, FAMILY, CAUSAL>;
  static std::atomic<uint64_t> lds_ok{0};
  if (allow_lds(lds_ok, lds, kern) != 0) return -1;
  // the kernel addresses K and V rows with 32-bit byte offsets from the (batch, head) plane
  if (a.kss < 0 || a.vss < 0 || a.kss >= ((int64_t)1 << 31) || a.vss >= ((int64_t)1 << 31) ||
      (uint64_t)a.Skv * (uint64_t)a.kss * 2 >= (1ull << 32) || (uint64_t)a.Skv * (uint64_t)a.vss * 2 >= (1ull << 32))
    return -2;
  AttnArgs args = a;
  args.num_m_blocks = (a.Sq + BM - 1) / BM;
  const int num_cus = device_cus();
  if (num_cus <= 0) return -1;
  const int n_items = args.num_m_blocks * a.B * a.H;
  const unsigned grid = (unsigned)(n_items < num_cus ? n_items : num_cus);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(512), lds, stream, args);
  return launch_status();
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
  if (family != 3 && dqk == 128 && dv == 128 && !a.kv_lens && !a.kv_block_mask && !a.o_part && !a.elem_mask && !a.add && !a.slope_q &&
      !a.slope_kv && !(a.softcap > 0.f)) {
    return is_bf16 ? dispatch_family<__bf16, 128, 128>(a, family, causal, stream)
                   : dispatch_family<_Float16, 128, 128>(a, family, causal, stream);
  }
  // 128 / 256 at prefill lengths: two launches of the 128 / 128 kernel, one per half of the value columns (given the
  // probabilities the columns are independent; the scores are computed twice, which this kernel still does in less time than
  // the general kernel needs once: 0.78 against 1.46 ms at B8 H12 S4096).  Both launches write the same row scales.
  if (family != 3 && dqk == 128 && dv == 256 && a.Sq >= 256 && !a.kv_lens && !a.kv_block_mask && !a.o_part && !a.elem_mask && !a.add &&
      !a.slope_q && !a.slope_kv && !(a.softcap > 0.f)) {
    for (int half = 0; half < 2; half++) {
      AttnArgs h = a;
      h.v = (const char*)a.v + half * 128 * 2;
      h.o = (char*)a.o + half * 128 * 2;
      const int rc = is_bf16 ? dispatch_family<__bf16, 128, 128>(h, family, causal, stream) : dispatch_family<_Float16, 128, 128>(h, family, causal, stream);
      if (rc != 0) return rc;
    }
    return 0;
  }
  // the retention family, every other head size, per-batch lengths / kv block masks / element-wise masks, split-kv decode
  return attn_wide_fwd_dispatch(a, family, causal, is_bf16, dqk, dv, stream);
}

}  // namespace ma
