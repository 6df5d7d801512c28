// Chunked linear / stateful attention forward (RetNet retention, Mamba2 SSD,
// gated retention) for gfx950.
//
// Replaces the three launches of LinearAttention.forward in
// attention_engine/core/template/tl_template/linear/linear_tl.py:1240-1269
// (chunk_local_cumsum :36-60, chunk_fwd_h :146-221, chunk_o :322-399) with ONE
// kernel that keeps the inter-chunk state on chip:
//
//   o_t = q_scale * q_t . sum_{s<=t} exp(G_t - G_s) k_s^T (v_s * vs_s),   G = cumsum(log_decay)
//
// Work split.  A workgroup owns one (batch, head) and a slice of 32*NW value
// columns; wave w owns 32 of them and the matching DK x 32 block of the fp32
// state, which lives in its accumulator registers for the whole sequence (the
// reference writes the state to HBM as bf16 every chunk and reads it back).  The
// sequence is walked in chunks of 32 tokens; per chunk and wave, with
// g = chunk-local cumsum of the log decay, everything is computed TRANSPOSED so
// each lane owns one token column:
//   A^T = K Q^T                      [32 x 32]   (every wave, redundantly: it is the B operand below)
//   P^T = A^T * q_scale * exp(g_i - g_j) * vs_j * [j <= i]
//   O^T = h^T (Q^T) * exp(g_i) q_scale + V^T P^T          [32 dv x 32 tokens]
//   h   = exp(g_last) h + K^T (V * vs * exp(g_last - g))  [DK x 32 dv]
// The state accumulator of K^T V (lane = value column, rows = key dims) is,
// register for register, the A operand of h^T Q^T, so the state never moves.
// Q/K/V chunk tiles arrive by direct-to-LDS DMA, double buffered, with a single
// workgroup barrier per chunk.
//
// Heads that share their q and k head (Mamba2: one B/C group for all heads) can be
// grouped HG to a workgroup, which then shares the Q/K tiles in LDS.
//
// Segments.  One (batch, head) is a serial chain of T/32 chunks; when batch x heads
// is too small to give every SIMD several waves, the sequence is cut into segments
// that run side by side: a first launch (MODE 1) computes, for every segment but the
// last, the state it ends in when entered with a zero state and its total log decay;
// the second launch (MODE 2) enters segment s with
//   sum_{s' < s} exp(sum_{s' < s'' < s} D[s'']) h_local[s']
// (states are exchanged in accumulator-register order, fp32, through the workspace)
// and produces the outputs.  MODE 0 is the single pass.
#include "linear_fwd.h"

namespace ma {

namespace {
constexpr int L = 32;  // tokens per chunk

template <int CTRL>
__device__ __forceinline__ float dpp_f32(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, true));
}

template <typename X8>
__device__ __forceinline__ X8 scale_bf16x8(X8 v, const float (&w)[8]) {
  X8 r;
#pragma unroll
  for (int i = 0; i < 8; i++) r[i] = (__bf16)((float)v[i] * w[i]);
  return r;
}
}  // namespace

// minimum waves per SIMD asked of the register allocator: 8 waves of one workgroup need 2; the
// two-heads-per-workgroup configuration is meant to run three workgroups of 4 waves per CU
template <int DK, int NWH, int HG>
constexpr int min_waves_per_simd() { return HG > 1 ? 3 : (NWH == 4 && DK > 128 ? 1 : 2); }

// GEN: the operands' general addressing (reversed time, row strides, v head broadcast) of LinArgs; without it the
// addressing is the plain one, with compile-time row sizes.
template <int DK, int NWH, int HG, int MODE, bool GEN = false>
__global__ __launch_bounds__(64 * NWH * HG, (min_waves_per_simd<DK, NWH, HG>())) void linear_fwd_kernel(const LinArgs a) {
  constexpr int NW = NWH * HG;
  constexpr bool ALIAS_OST = HG > 1;     // output staging block inside the wave's own (already consumed) V columns
  using T = __bf16;
  using E = Elem<T>;
  using x8 = typename E::x8;
  using x4 = typename E::x4;
  constexpr int DVS = 32 * NW;
  constexpr int RBQ = DK * 2, RBV = DVS * 2;       // row bytes
  constexpr int CPRQ = DK / 8, CPRV = DVS / 8;     // 16-byte chunks per row
  constexpr int QT = L * RBQ, VT = L * RBV;
  constexpr int STAGE = 2 * QT + VT;
  constexpr int KB = DK / 32;                      // 32-row blocks of the state
  constexpr int OROW = 64 + 16;                    // padded row of the per-wave output staging block
  constexpr int SCAL_BYTES = 3 * L * 4;            // per-wave g / pv*q_scale / w
  constexpr int NIQ = QT / 1024, NIV = VT / 1024;  // DMA instructions per tile
  static_assert(CPRQ >= 16, "DK < 128 needs its own Q/K swizzle");
  // Every wave of the workgroup needs the same 32 x 32 tile A^T = K Q^T.  With four or more waves it is computed
  // once: in 16 x 16 quadrants (v_mfma_f32_16x16x32; the quadrant of keys 16..31 x queries 0..15 lies above the
  // diagonal and is left out), each over 1 / KP of the key dims, one (quadrant, part) per wave, exchanged
  // through LDS.  16 MFMAs of 32x32x16 and 2 x DK / 16 KB of operand reads per wave become at most 4 half-size
  // MFMAs plus a 1 KB write and 4 KP KB of reads, for one more barrier per chunk.
  constexpr bool SHARE_A = NW >= 4 && MODE != 1;
  constexpr int KP = NW >= 8 ? 2 : 1;               // parts of the key dims per quadrant
  constexpr int A_ITEMS = 3 * KP;

  extern __shared__ __align__(16) char smem[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(MA_LDS char*)smem;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r0 = lane & 31;
  const uint32_t lds_scal = lds0 + 2 * STAGE + wave * SCAL_BYTES;
  const uint32_t lds_ost = lds0 + 2 * STAGE + NW * SCAL_BYTES + wave * (L * OROW);   // (unused with ALIAS_OST)
  const uint32_t lds_apart = lds0 + 2 * STAGE + NW * SCAL_BYTES + (ALIAS_OST ? 0 : NW * (L * OROW));   // A^T quadrants, 1 KB each

  // workgroup -> (head group, value slice, segment); the workgroups of one head group share
  // id % 8 (one XCD, shared L2)
  const int n_seg = MODE == 0 ? 1 : (MODE == 1 ? a.nseg - 1 : a.nseg);
  const int BG = a.bg_n > 0 ? a.bg_n : a.B * a.H / HG;     // head groups of this launch
  int bg, dvb, seg;
  {
    int slot;
    if ((BG & 7) == 0) {
      const int xcd = blockIdx.x & 7;
      slot = blockIdx.x >> 3;
      seg = slot % n_seg;
      slot /= n_seg;
      dvb = slot % a.dv_blocks;
      bg = (slot / a.dv_blocks) * 8 + xcd;
    } else {
      slot = blockIdx.x;
      seg = slot % n_seg;
      slot /= n_seg;
      dvb = slot % a.dv_blocks;
      bg = slot / a.dv_blocks;
    }
  }
  const int bg_local = bg;      // (indexes the launch's workspace)
  bg += a.bg0;
  const int hl = wave / NWH;                      // head of the group this wave works for
  const int bh0 = bg * HG, bh = bh0 + hl;
  const int b = bh0 / a.H, h0 = bh0 % a.H;        // (HG divides H, and the heads of a group share hq and hk)
  const int hq = h0 / (a.H / a.Hq), hk = h0 / (a.H / a.Hk);
  const int Tn = a.T;
  const bool rev = GEN && a.rev != 0, rev_o = GEN && a.rev_o != 0;
  const int64_t q_rb = GEN ? a.q_row * 2 : (int64_t)RBQ, k_rb = GEN ? a.k_row * 2 : (int64_t)RBQ;   // bytes between an operand's rows in memory
  const int64_t v_row_bytes = (GEN ? a.v_row : (int64_t)a.Dv) * 2;
  const int64_t bh0_v = GEN ? (int64_t)b * a.Hv + h0 / (a.H / a.Hv) : (int64_t)bh0;
  const int64_t piece = GEN ? (int64_t)blockIdx.y : 0;   // (pieces of a contraction side by side: see LinArgs)
  const char* qb = (const char*)a.q + ((int64_t)(b * a.Hq + hq) * Tn) * q_rb + piece * a.piece_qk * 2;
  const char* kb = (const char*)a.k + ((int64_t)(b * a.Hk + hk) * Tn) * k_rb + piece * a.piece_qk * 2;
  const char* vb = (const char*)a.v + bh0_v * Tn * v_row_bytes + (int64_t)dvb * (32 * NWH) * 2;
  const int64_t v_head_bytes = (int64_t)Tn * v_row_bytes;
  T* ob = (T*)a.o + (int64_t)bh * Tn * a.Dv + dvb * (32 * NWH) + 32 * (wave % NWH);
  const float* ldp = a.log_decay + (int64_t)bh * Tn;
  const float* vsp = a.v_scale ? a.v_scale + (int64_t)bh * Tn : nullptr;
  const int n_chunks_all = (Tn + L - 1) / L;
  const int c_begin = MODE == 0 ? 0 : seg * a.seg_chunks;
  const int c_end = MODE == 0 ? n_chunks_all : min(c_begin + a.seg_chunks, n_chunks_all);
  // this wave's block of the exchanged states: [segment][wave][KB*16 registers][64 lanes]
  float* ws_mine = nullptr;
  if (MODE != 0)
    ws_mine = a.ws_state + ((((int64_t)bg_local * a.dv_blocks + dvb) * (a.nseg - 1)) * NW + wave) * (int64_t)(KB * 16 * 64) + lane;
  constexpr int64_t WS_SEG = (int64_t)NW * KB * 16 * 64;

  // ---- DMA of one chunk: each instruction moves 1 KB (1024/row_bytes tile rows); lane i fetches
  //      the 16-byte chunk that belongs at physical position i of that KB.
  //      (Spreading a chunk's instructions over the chunk's phases instead of issuing them together behind the
  //      barrier was measured: no gain at the RetNet shape, 5 % slower at the Mamba2 shape.)
  const uint32_t qk_chunks = GEN && a.qk_cols > 0 ? (uint32_t)a.qk_cols / 8 : (uint32_t)CPRQ;   // 16-byte chunks of a q / k row that exist
  // (columns beyond the operand's are zeros: the 16- and 32-wide slices of the contraction that hold nothing else are skipped)
  const int qk_used = GEN && a.qk_cols > 0 ? a.qk_cols : DK;
  if (GEN && qk_chunks < (uint32_t)CPRQ) {
    // the Q and K tiles of both stages start as zeros: the missing columns are never written
    for (uint32_t off = (uint32_t)tid * 16; off < (uint32_t)(2 * QT); off += 64 * NW * 16) {
      lds_write<u32x4>(lds0 + off, u32x4{0u, 0u, 0u, 0u});
      lds_write<u32x4>(lds0 + STAGE + off, u32x4{0u, 0u, 0u, 0u});
    }
    __syncthreads();
  }
  auto issue_chunk = [&](int t0, int buf) {
    const uint32_t base = lds0 + buf * STAGE;
    constexpr int NQK = MODE == 1 ? NIQ : 2 * NIQ;      // (the state-only pass needs no Q)
    constexpr int RQ = 1024 / RBQ, RV = 1024 / RBV;     // tile rows per instruction
    static_assert(HG == 1 || RV % 4 == 0, "the V swizzle of an instruction's first row must stay inside a head's columns");
    if (t0 + L <= Tn && v_head_bytes < ((int64_t)1 << 31)) {
      // Whole chunk: no row clamping, so an instruction's source is a wave-uniform base (SGPRs) plus a
      // 32-bit lane offset.  The swizzle is a bit permutation of the row index, so it splits into the
      // lane's part (row within the instruction) and the instruction's part (its first row), and since row
      // offsets are multiples of the row size the instruction's part is one XOR on the finished lane offset.
      int ln2 = lane;
      asm volatile("" : "+v"(ln2));   // rebuilt per chunk: kept live across the chunk these would cost registers
      const int lrq = ln2 / CPRQ, lrv = ln2 / CPRV;
      // (reversed time: an instruction's rows lie behind each other in memory the other way round; its base is then
      // its LAST row's address, the lowest, and the lane's row offset counts from there)
      // With the general addressing a row distance need not be a multiple of the tile's row size, so the instruction's
      // part of the swizzle goes onto the chunk index before the row offset is added; chunks beyond the operand's columns
      // are not loaded (their LDS stays zero).
      const uint32_t cq = (uint32_t)((ln2 % CPRQ) ^ swz_tile<CPRQ>(lrq));
      const uint32_t aq = (uint32_t)(rev ? RQ - 1 - lrq : lrq) * (uint32_t)q_rb + (GEN ? 0u : cq << 4);
      const uint32_t ak = GEN ? (uint32_t)(rev ? RQ - 1 - lrq : lrq) * (uint32_t)k_rb : aq;
      const uint32_t lc0 = (ln2 % CPRV) ^ swz_tile<CPRV>(lrv);       // logical chunk: head lc / (4 NWH), then its columns
      uint32_t av = (uint32_t)(rev ? RV - 1 - lrv : lrv) * (uint32_t)v_row_bytes + ((lc0 % (4 * NWH)) << 4);
      if (HG > 1) av += (lc0 / (4 * NWH)) * (uint32_t)v_head_bytes;
#pragma unroll (DK <= 128 ? 16 : 1)   // (with a 256-wide key the state leaves no registers for an unrolled burst)
      for (int it = 0; it < (NQK + NIV + NW - 1) / NW; it++) {
        const int ii = wave + NW * it;
        if ((NQK + NIV) % NW != 0 && ii >= NQK + NIV) break;
        if (ii < NQK) {
          const int which = MODE == 1 ? 1 : ii >= NIQ, i2 = (MODE != 1 && which) ? ii - NIQ : ii;
          const int64_t row0 = rev ? Tn - t0 - (i2 + 1) * RQ : t0 + i2 * RQ;
          const char* sb = (which ? kb + row0 * k_rb : qb + row0 * q_rb);
          if constexpr (GEN) {
            const uint32_t lc = cq ^ (uint32_t)swz_tile<CPRQ>(i2 * RQ);
            if (lc < qk_chunks) dma16_so(sb, (which ? ak : aq) + (lc << 4), base + which * QT + i2 * 1024);
          } else {
            dma16_so(sb, aq ^ (uint32_t)(swz_tile<CPRQ>(i2 * RQ) << 4), base + which * QT + i2 * 1024);
          }
        } else {
          const int i2 = ii - NQK;
          const int64_t row0 = rev ? Tn - t0 - (i2 + 1) * RV : t0 + i2 * RV;
          const char* sb = vb + row0 * v_row_bytes;
          dma16_so(sb, av ^ (uint32_t)(swz_tile<CPRV>(i2 * RV) << 4), base + 2 * QT + i2 * 1024);
        }
      }
      return;
    }
    // last, partial chunk: rows beyond the sequence are clamped to its last row
#pragma unroll 1
    for (int it = 0; it < (NQK + NIV + NW - 1) / NW; it++) {
      const int ii = wave + NW * it;
      if ((NQK + NIV) % NW != 0 && ii >= NQK + NIV) break;
      if (ii < NQK) {
        const int which = MODE == 1 ? 1 : ii >= NIQ, i2 = (MODE != 1 && which) ? ii - NIQ : ii;
        const int row = i2 * RQ + lane / CPRQ, c = lane % CPRQ;
        const int tpos = min(t0 + row, Tn - 1), trow = rev ? Tn - 1 - tpos : tpos;
        const uint32_t lc = (uint32_t)(c ^ swz_tile<CPRQ>(row));
        const char* src = (which ? kb + (int64_t)trow * k_rb : qb + (int64_t)trow * q_rb) + (lc << 4);
        if (!GEN || lc < qk_chunks) dma16(src, base + which * QT + i2 * 1024);
      } else {
        const int i2 = ii - NQK;
        const int row = i2 * RV + lane / CPRV, c = lane % CPRV;
        const int tpos = min(t0 + row, Tn - 1), trow = rev ? Tn - 1 - tpos : tpos;
        const int lc = c ^ swz_tile<CPRV>(row);          // logical 16-byte chunk: head lc / (4 NWH), then its columns
        const char* src = vb + (int64_t)trow * v_row_bytes + ((lc % (4 * NWH)) << 4);
        if (HG > 1) src += (lc / (4 * NWH)) * v_head_bytes;
        dma16(src, base + 2 * QT + i2 * 1024);
      }
    }
  };

  f32x16 hst[KB];
#pragma unroll
  for (int i = 0; i < KB; i++)
#pragma unroll
    for (int j = 0; j < 16; j++) hst[i][j] = 0.f;

  // scalars of the chunk about to be processed (loaded one chunk ahead)
  const int ti = r0;
  float ld_next = 0.f, vs_next = 1.f;
  if (c_begin * L + ti < Tn) {
    ld_next = ldp[c_begin * L + ti];
    if (vsp) vs_next = vsp[c_begin * L + ti];
  }
  if (c_begin < c_end) issue_chunk(c_begin * L, 0);

  if (MODE == 2 && seg > 0) {
    // entering state: the local end states of the earlier segments, each decayed by the segments between
    const float* dec = a.ws_decay + (int64_t)(bh - a.bg0 * HG) * (a.nseg - 1);
    float acc_log = 0.f;
    for (int sp = seg - 1; sp >= 0; sp--) {
      const float coef = fast_exp2(acc_log * kLog2e);
      const float* src = ws_mine + sp * WS_SEG;
#pragma unroll
      for (int i = 0; i < KB; i++)
#pragma unroll
        for (int j = 0; j < 16; j++) hst[i][j] += coef * src[(i * 16 + j) * 64];
      acc_log += dec[sp];
    }
  }
  float seg_log = 0.f;   // MODE 1: total log decay of the segment

  for (int c = c_begin; c < c_end; c++) {
    const int buf = (c - c_begin) & 1, t0 = c * L;
    wait_dma();
    __syncthreads();
    const float ld = ld_next, vs = vs_next;
    const bool has_next = c + 1 < c_end;
    if (has_next) {
      const int tn = t0 + L + ti;
      ld_next = 0.f;
      vs_next = 1.f;
      if (tn < Tn) {
        ld_next = ldp[tn];
        if (vsp) vs_next = vsp[tn];
      }
    }
    if (has_next) issue_chunk(t0 + L, buf ^ 1);
    const uint32_t base = lds0 + buf * STAGE;
    const uint32_t qbase = base, kbase = base + QT, vbase = base + 2 * QT;

    // ---- this wave's share of A^T = K Q^T: quadrant slot 0 = keys 0..15 x queries 0..15, 1 = keys 0..15 x queries
    //      16..31, 2 = keys 16..31 x queries 16..31; A / B operand: lane holds row (column) lane % 16, k = 8 (lane / 16) .. +7
    //      of a 32-wide slice; C: lane holds column lane % 16, rows 4 (lane / 16) + {0..3}
    if constexpr (SHARE_A) {
      if (wave < A_ITEMS) {
        const int slot = wave / KP, kp = wave % KP;
        int la = lane;
        asm volatile("" : "+v"(la));
        const int rr = la & 15, kg = la >> 4;
        // (tile bases and row offsets are multiples of the row size, so the swizzled chunk index occupies its own
        // address bits: one XOR with a constant per read moves to another slice)
        constexpr int NS16 = DK / 32 / KP;
        const uint32_t c0 = (uint32_t)((kg ^ swz16(rr)) << 4) ^ (uint32_t)(kp * NS16 * 64);
        const uint32_t ka = kbase + (16 * (slot >> 1) + rr) * RBQ + c0, qa = qbase + (16 * (slot > 0) + rr) * RBQ + c0;
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s2 = 0; s2 < NS16; s2++) {
          if (GEN && (kp * NS16 + s2) * 32 >= qk_used) break;
          acc = E::mfma16(lds_read<x8>(ka ^ (uint32_t)(s2 * 64)), lds_read<x8>(qa ^ (uint32_t)(s2 * 64)), acc);
        }
        lds_write<f32x4>(lds_apart + wave * 1024 + la * 16, acc);
      }
    }

    // ---- per-lane LDS read offsets.  They are loop invariant; left outside the loop, they (and every
    //      swizzled address derived from them, dozens) stay in registers across chunks, which the state
    //      accumulator leaves no room for.  The lane id is laundered so that they are rebuilt per chunk.
    int ln = lane;
    asm volatile("" : "+v"(ln));
    const int r = ln & 31, g = ln >> 5;
    // K rows / Q rows as MFMA operands of A^T = K Q^T: row r, logical chunk 2ks + g
    const uint32_t qk_row = r * RBQ;
    const int qk_c0 = g ^ swz16(r);
    // Q^T operand of h^T Q^T: token r, key dims 32b + 16s + 4g + {0..3} and + 8: chunk 4b + 2s (+1), half g
    const uint32_t qp_row = r * RBQ + g * 8;
    const int qp_swz = swz16(r);
    // transposing reads (K^T and V^T): lane block lane/16 -> (row group g, column half), rows 16s + 4g + jr (+8)
    const int jr = (ln & 15) >> 2;
    const int lc = (((ln >> 4) & 1) << 1) | ((ln & 3) >> 1);
    const uint32_t kt_row = (4 * g + jr) * RBQ + (ln & 1) * 8;
    const int kt_c0 = lc ^ swz16(4 * g + jr);                      // rows +8 / +16: see HALF_XOR below
    const uint32_t vt_row = (4 * g + jr) * RBV + (ln & 1) * 8;
    const int vt_c0 = (4 * wave + lc) ^ swz_tile<CPRV>(4 * g + jr);
    // swz(row + 8) ^ swz(row) and swz(row + 16) ^ swz(row) for rows < 8
    constexpr int Q_X8 = 2, Q_X16 = 0;
    constexpr int V_X8 = CPRV >= 16 ? 2 : 2, V_X16 = CPRV >= 16 ? 0 : 0;


    // ---- chunk scalars: inclusive scan of the log decay over the 32 tokens (both lane halves hold a copy)
    const bool valid = t0 + ti < Tn;
    // (DPP: shifts within rows of 16 lanes, then lane 15 of rows 0 and 2 carried into rows 1 and 3; the
    // two halves of the wave scan the same 32 values)
    float gi = valid ? ld : 0.f;
    gi += dpp_f32<0x111>(gi);   // row_shr:1, lanes shifted in from outside the row read 0
    gi += dpp_f32<0x112>(gi);
    gi += dpp_f32<0x114>(gi);
    gi += dpp_f32<0x118>(gi);
    gi += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, gi), 0x142, 0xa, 0xf, false));   // row_bcast:15
    const float g_last = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, gi), 31));
    const float gi2 = gi * kLog2e, g_last2 = g_last * kLog2e;    // (exponents in the log2 domain from here on)
    const float pvq = valid ? vs * a.q_scale : 0.f;               // factor of column j in P
    const float wl = valid ? vs * fast_exp2(g_last2 - gi2) : 0.f;   // factor of row l in the state update
    const float eg = fast_exp2(gi2) * a.q_scale;                  // factor of token i in the inter-chunk term
    const float decay_all = fast_exp2(g_last2);
    if (MODE == 1) seg_log += g_last;
    if (g == 0) {
      lds_write<float>(lds_scal + ti * 4, gi2);
      lds_write<float>(lds_scal + (L + ti) * 4, pvq);
      lds_write<float>(lds_scal + (2 * L + ti) * 4, wl);
    }
    // ---- A^T = K Q^T (lane: token i = r, rows j = 8(jj/4) + 4g + jj%4)
    // two accumulation chains, so that consecutive MFMAs do not wait for each other, where registers
    // allow (with three waves per SIMD the other waves fill those gaps)
    constexpr bool TWO_CHAINS = HG == 1 && !SHARE_A;
    // (a chain's first MFMA takes the constant zero as its accumulator input: no registers to clear)
    const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    f32x16 sacc, sacc2;
#pragma unroll
    for (int j = 0; j < 16; j++) { sacc[j] = 0.f; sacc2[j] = 0.f; }
    if constexpr (SHARE_A) {
      // gather the quadrants: this lane's rows 8 q4 + 4g + {0..3} of column r sit in lane (r % 16) + 16 (2 (q4 % 2) + g)
      // of quadrant slot (q4 / 2) + (r / 16); for the quadrant that was left out this reads its neighbour, and the
      // causal select below discards it
      __syncthreads();
#pragma unroll
      for (int q4 = 0; q4 < 4; q4++) {
        const uint32_t src = lds_apart + (uint32_t)(((q4 >> 1) + (r >> 4)) * KP) * 1024 + (uint32_t)((r & 15) + 16 * (2 * (q4 & 1) + g)) * 16;
        f32x4 t = lds_read<f32x4>(src);
        if constexpr (KP == 2) {
          const f32x4 t2 = lds_read<f32x4>(src + 1024);
#pragma unroll
          for (int i = 0; i < 4; i++) t[i] += t2[i];
        }
#pragma unroll
        for (int i = 0; i < 4; i++) sacc[4 * q4 + i] = t[i];
      }
    } else if constexpr (MODE != 1) {
      constexpr int NS = DK / 16, AH = 2, RING = 3;
      x8 kf[RING], qf[RING];
      const uint32_t kq_a = kbase + qk_row + (uint32_t)(qk_c0 << 4), qq_a = qbase + qk_row + (uint32_t)(qk_c0 << 4);
      auto request = [&](int ks) {
        kf[ks % RING] = lds_read<x8>(kq_a ^ (uint32_t)(ks * 32));
        qf[ks % RING] = lds_read<x8>(qq_a ^ (uint32_t)(ks * 32));
      };
#pragma unroll
      for (int ks = 0; ks < AH; ks++) request(ks);
#pragma unroll
      for (int ks = 0; ks < NS; ks++) {
        if (GEN && ks * 16 >= qk_used) break;
        if (ks + AH < NS) request(ks + AH);
        __builtin_amdgcn_sched_barrier(0);
        if (TWO_CHAINS && (ks & 1)) sacc2 = E::mfma32(kf[ks % RING], qf[ks % RING], ks == 1 ? zero16 : sacc2);
        else sacc = E::mfma32(kf[ks % RING], qf[ks % RING], ks == 0 ? zero16 : sacc);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // rows held by this lane in a 32 x 32 accumulator block: 8q4 + 4g + {0..3}
    float gj[16], pj[16];
    uint32_t scal_g = lds_scal + 16 * g;   // one lane register; every read below is this plus an immediate
    asm volatile("" : "+v"(scal_g));
    if constexpr (MODE != 1) {
#pragma unroll
    for (int q4 = 0; q4 < 4; q4++) {
      const f32x4 tg = lds_read<f32x4>(scal_g + 32 * q4);
      const f32x4 tp = lds_read<f32x4>(scal_g + (L + 8 * q4) * 4);
#pragma unroll
      for (int i = 0; i < 4; i++) {
        gj[4 * q4 + i] = tg[i];
        pj[4 * q4 + i] = tp[i];
      }
    }
    }
    // ---- P^T: decay, per-token value scale, causal mask (exact zeros above the diagonal)
    x8 pf[2];
    if constexpr (MODE != 1) {
#pragma unroll
    for (int jj = 0; jj < 16; jj++) {
      const int j = 8 * (jj >> 2) + 4 * g + (jj & 3);
      // (above the diagonal the exponent is positive and the product may be inf or NaN: the select drops it)
      const float e = fast_exp2(gi2 - gj[jj]);
      float p = (TWO_CHAINS ? sacc[jj] + sacc2[jj] : sacc[jj]) * e * pj[jj];
      asm volatile("" : "+v"(p));   // computed for every lane, then selected: no branch per element
      pf[jj >> 3][jj & 7] = (T)(j <= ti ? p : 0.f);
    }
    }

    // ---- V^T fragments (rows = this wave's 32 value columns; k-slot i of slice s is token
    //      16s + 8(i/4) + 4g + i%4, the order P^T comes in)
    x8 vf[2];
    {
      const uint32_t va = vbase + vt_row + (uint32_t)(vt_c0 << 4);
#pragma unroll
      for (int s = 0; s < 2; s++) {
        const int cx = s ? V_X16 : 0;
        x4 lo = lds_read_tr4<T>((va ^ (uint32_t)(cx << 4)) + 16 * s * RBV);
        x4 hi = lds_read_tr4<T>((va ^ (uint32_t)((cx ^ V_X8) << 4)) + (16 * s + 8) * RBV);
        vf[s] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      }
    }

    // ---- O^T = (h^T Q^T) * eg + V^T P^T
    f32x16 o_inter, o_inter2, o_intra;
#pragma unroll
    for (int j = 0; j < 16; j++) { o_inter[j] = 0.f; o_inter2[j] = 0.f; o_intra[j] = 0.f; }
    if constexpr (MODE != 1) {
      o_intra = E::mfma32(vf[0], pf[0], zero16);
      o_intra = E::mfma32(vf[1], pf[1], o_intra);
    }
    // value-scaled V^T for the state update (k-slot i of slice s is token 16s + 8(i/4) + 4g + i%4 -> wj[8s + i])
    x8 vsf[2];
#pragma unroll
    for (int s = 0; s < 2; s++) {
      float w8[8];
#pragma unroll
      for (int h2 = 0; h2 < 2; h2++) {
        const f32x4 tw = lds_read<f32x4>(scal_g + (2 * L + 16 * s + 8 * h2) * 4);
#pragma unroll
        for (int i = 0; i < 4; i++) w8[4 * h2 + i] = tw[i];
      }
      vsf[s] = scale_bf16x8(vf[s], w8);
    }

    {
      // per 32-row state block b: inter-chunk product with the OLD state, then the state update
      constexpr int RING = 2;
      x4 qlo[RING][2], qhi[RING][2], klo[RING][2], khi[RING][2];
      const uint32_t qpa = qbase + qp_row + (uint32_t)(qp_swz << 4), kta = kbase + kt_row + (uint32_t)(kt_c0 << 4);
      auto request = [&](int bb) {
#pragma unroll
        for (int s = 0; s < 2; s++) {
          const int lcq = 4 * bb + 2 * s;
          if constexpr (MODE != 1) {
            qlo[bb % RING][s] = lds_read<x4>(qpa ^ (uint32_t)(lcq << 4));
            qhi[bb % RING][s] = lds_read<x4>(qpa ^ (uint32_t)((lcq + 1) << 4));
          }
          const int cx = s ? Q_X16 : 0;
          klo[bb % RING][s] = lds_read_tr4<T>((kta ^ (uint32_t)(((4 * bb) ^ cx) << 4)) + 16 * s * RBQ);
          khi[bb % RING][s] = lds_read_tr4<T>((kta ^ (uint32_t)(((4 * bb) ^ cx ^ Q_X8) << 4)) + (16 * s + 8) * RBQ);
        }
      };
      // operands are requested one block ahead, except where three waves per SIMD hide the LDS latency
      // and the registers are needed elsewhere
      constexpr bool AHEAD = HG == 1;
      if (AHEAD) request(0);
#pragma unroll
      for (int bb = 0; bb < KB; bb++) {
        if (GEN && bb * 32 >= qk_used) break;
        if (!AHEAD) request(bb);
        else if (bb + 1 < KB) request(bb + 1);
        __builtin_amdgcn_sched_barrier(0);
        // the old state as bf16 operands first, then the decay in place (left to itself the compiler decays into a
        // second register block while the old values are still waiting to be converted, and copies it back)
        x8 hf[2];
        if constexpr (MODE != 1) {
#pragma unroll
          for (int s = 0; s < 2; s++)
#pragma unroll
            for (int i = 0; i < 8; i++) hf[s][i] = (T)hst[bb][8 * s + i];
          __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int j = 0; j < 16; j++) hst[bb][j] *= decay_all;
        if constexpr (MODE != 1) {
#pragma unroll
          for (int s = 0; s < 2; s++) {
            x8 qf = __builtin_shufflevector(qlo[bb % RING][s], qhi[bb % RING][s], 0, 1, 2, 3, 4, 5, 6, 7);
            if (DK < 256 && HG == 1 && s) o_inter2 = E::mfma32(hf[s], qf, bb == 0 ? zero16 : o_inter2);   // (a second chain where registers allow)
            else o_inter = E::mfma32(hf[s], qf, (bb == 0 && (s == 0 || (DK < 256 && HG == 1))) ? zero16 : o_inter);
          }
        }
#pragma unroll
        for (int s = 0; s < 2; s++) {
          x8 kf = __builtin_shufflevector(klo[bb % RING][s], khi[bb % RING][s], 0, 1, 2, 3, 4, 5, 6, 7);
          hst[bb] = E::mfma32(kf, vsf[s], hst[bb]);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }

    // ---- write this wave's [32 tokens x 32 columns] block: stage (wave private), then 16-byte row pieces.
    //      With ALIAS_OST the staging block is the wave's own 4 chunks per row of the V tile just consumed
    //      (only this wave reads them, and the next DMA into this buffer is issued behind the next barrier).
    if (MODE != 1 && a.out_f32) {
      // fp32 outputs (used by the backward pass, whose decay gradient is a difference of sums over these
      // values): the same staging block, 16 columns at a time
      const int sw_r = swz_tile<CPRV>(r);
      float* ob32 = (float*)a.o + piece * a.piece_o + (int64_t)bh * Tn * a.Dv + dvb * (32 * NWH) + 32 * (wave % NWH);
#pragma unroll
      for (int half = 0; half < 2; half++) {
#pragma unroll
        for (int q2 = 0; q2 < 2; q2++) {
          const int q4 = 2 * half + q2;
          f32x4 w;
#pragma unroll
          for (int i = 0; i < 4; i++)
            w[i] = (DK < 256 && HG == 1 ? o_inter[4 * q4 + i] + o_inter2[4 * q4 + i] : o_inter[4 * q4 + i]) * eg + o_intra[4 * q4 + i];
          if (ALIAS_OST) lds_write<f32x4>(vbase + r * RBV + (uint32_t)(((4 * wave + 2 * q2 + g) ^ sw_r) << 4), w);
          else lds_write<f32x4>(lds_ost + r * OROW + (8 * q2 + 4 * g) * 4, w);
        }
#pragma unroll
        for (int it = 0; it < 2; it++) {
          const int ci = ln + 64 * it, row = ci >> 2, cc = ci & 3;
          const u32x4 w = ALIAS_OST ? lds_read<u32x4>(vbase + row * RBV + (uint32_t)(((4 * wave + cc) ^ swz_tile<CPRV>(row)) << 4))
                                    : lds_read<u32x4>(lds_ost + row * OROW + cc * 16);
          if (t0 + row < Tn) {
            f32x4* dst = (f32x4*)(ob32 + (int64_t)(rev_o ? Tn - 1 - (t0 + row) : t0 + row) * a.Dv + 16 * half + cc * 4);
            f32x4 val = __builtin_bit_cast(f32x4, w);
            if (a.out_f32 == 2) val += *dst;   // (a contraction cut into pieces: the pieces' outputs add up)
            *dst = val;
          }
        }
      }
    } else if constexpr (MODE != 1) {
      const int sw_r = swz_tile<CPRV>(r);
#pragma unroll
      for (int q4 = 0; q4 < 4; q4++) {
        x4 w;
#pragma unroll
        for (int i = 0; i < 4; i++)
          w[i] = (T)((DK < 256 && HG == 1 ? o_inter[4 * q4 + i] + o_inter2[4 * q4 + i] : o_inter[4 * q4 + i]) * eg + o_intra[4 * q4 + i]);
        if (ALIAS_OST) lds_write<x4>((vbase + r * RBV + (uint32_t)(((4 * wave) ^ sw_r) << 4) + g * 8) ^ (uint32_t)(q4 << 4), w);
        else lds_write<x4>(lds_ost + r * OROW + (8 * q4 + 4 * g) * 2, w);
      }
      // (rows 16 apart share their swizzle)
      const uint32_t ra = vbase + (ln >> 2) * RBV + (uint32_t)(((4 * wave + (ln & 3)) ^ swz_tile<CPRV>(ln >> 2)) << 4);
#pragma unroll
      for (int it = 0; it < 2; it++) {
        const int ci = ln + 64 * it, row = ci >> 2, cc = ci & 3;
        const u32x4 w = ALIAS_OST ? lds_read<u32x4>(ra + 16 * it * RBV) : lds_read<u32x4>(lds_ost + row * OROW + cc * 16);
        if (t0 + row < Tn) *(u32x4*)(ob + (int64_t)(rev_o ? Tn - 1 - (t0 + row) : t0 + row) * a.Dv + cc * 8) = w;
      }
    }
  }
  if (MODE == 1) {
    // the state this segment ends in when entered with zeros, and its total log decay
    float* dst = ws_mine + seg * WS_SEG;
#pragma unroll
    for (int i = 0; i < KB; i++)
#pragma unroll
      for (int j = 0; j < 16; j++) dst[(i * 16 + j) * 64] = hst[i][j];
    if (dvb == 0 && wave % NWH == 0 && lane == 0) a.ws_decay[(int64_t)(bh - a.bg0 * HG) * (a.nseg - 1) + seg] = seg_log;
  }
}

namespace {
// Resident workgroups per CU and the CU count, asked of the runtime once per configuration.
template <int DK, int NWH, int HG>
struct Config {
  static constexpr int NW = NWH * HG;
  static constexpr size_t stage = (size_t)L * (4 * DK + 2 * 32 * NW);
  static constexpr size_t lds = 2 * stage + NW * (3 * L * 4) + (HG > 1 ? 0 : NW * (L * 80)) + (NW >= 4 ? 3 * (NW >= 8 ? 2 : 1) * 1024 : 0);
  static constexpr int64_t ws_wave_floats = (int64_t)(DK / 32) * 16 * 64;

  static bool prepare(int& resident, int& cus) {
    // (threads that meet in a first call compute the same numbers; a device other than the first one asked is assumed to
    // be of the same kind)
    static std::atomic<uint64_t> lds_ok{0};
    static std::atomic<int> s_resident{-1};
    if (allow_lds(lds_ok, lds, linear_fwd_kernel<DK, NWH, HG, 0>, linear_fwd_kernel<DK, NWH, HG, 1>, linear_fwd_kernel<DK, NWH, HG, 2>,
                  linear_fwd_kernel<DK, NWH, HG, 0, true>, linear_fwd_kernel<DK, NWH, HG, 1, true>, linear_fwd_kernel<DK, NWH, HG, 2, true>) != 0)
      return false;
    cus = device_cus();
    if (cus <= 0) return false;
    int r = s_resident.load(std::memory_order_relaxed);
    if (r < 0) {
      if (hip_check(hipOccupancyMaxActiveBlocksPerMultiprocessor(&r, linear_fwd_kernel<DK, NWH, HG, 2>, 64 * NW, lds)) != 0) return false;
      r = r < 1 ? 1 : r;
      s_resident.store(r, std::memory_order_relaxed);
    }
    resident = r;
    return true;
  }

  // Number of segments and chunks per segment for this problem.  want: 0 = choose (as many segments as
  // keep every CU's resident workgroup slots busy, each at least 4 chunks long), n >= 1 = at most n.
  static void plan(const LinArgs& a, int want, int resident, int cus, int& nseg, int& seg_chunks) {
    const int n_chunks = (a.T + L - 1) / L;
    const int64_t groups = (int64_t)a.B * a.H / HG * (a.Dv / (32 * NWH));
    if (a.n_pieces > 1) want = 1;   // (pieces side by side run the single pass)
    int n;
    if (want >= 1) n = want;
    else {
      n = (int)((int64_t)resident * cus / groups);
      if (n > 8) n = 8;
      if (n > n_chunks / 4) n = n_chunks / 4;
    }
    if (n > n_chunks) n = n_chunks;
    if (n < 1) n = 1;
    seg_chunks = (n_chunks + n - 1) / n;
    nseg = (n_chunks + seg_chunks - 1) / seg_chunks;
  }

  static size_t ws_bytes(const LinArgs& a, int nseg) {
    if (nseg <= 1) return 0;
    const int64_t groups = (int64_t)a.B * a.H / HG * (a.Dv / (32 * NWH));
    return (size_t)((groups * (nseg - 1) * NW * ws_wave_floats + (int64_t)a.B * a.H * (nseg - 1)) * 4);
  }

  // A single pass over more head groups than the device holds at once ends in a round that is mostly empty (320 workgroups
  // on 256 CUs take as long as 512).  When the last round would be at most half full, the head groups of the full rounds run
  // the single pass and the rest is cut into sequence segments, as many as fill the device once: tail_bg head groups from
  // full_bg on, in nseg segments (tail_bg = 0: no such split).
  struct Tail { int full_bg, tail_bg, nseg, seg_chunks; };
  static Tail tail_plan(const LinArgs& a, int want, int resident, int cus) {
    Tail t{0, 0, 1, 0};
    const int dvb = a.Dv / (32 * NWH), n_chunks = (a.T + L - 1) / L;
    const int64_t BG = (int64_t)a.B * a.H / HG, per_round = (int64_t)resident * cus / dvb;     // head groups
    if (want != 0 || a.n_pieces > 1 || per_round < 1 || BG <= per_round) return t;
    const int64_t tail = BG % per_round;
    int n = tail > 0 ? (int)(per_round / tail) : 1;
    if (n > 8) n = 8;
    if (n > n_chunks / 4) n = n_chunks / 4;
    if (tail == 0 || tail * 2 > per_round || n < 2) return t;
    t.full_bg = (int)(BG - tail);
    t.tail_bg = (int)tail;
    t.seg_chunks = (n_chunks + n - 1) / n;
    t.nseg = (n_chunks + t.seg_chunks - 1) / t.seg_chunks;
    if (t.nseg < 2) t.tail_bg = 0;
    return t;
  }
  static size_t tail_ws_bytes(const Tail& t, int dvb) {
    if (t.tail_bg <= 0) return 0;
    return (size_t)(((int64_t)t.tail_bg * dvb * (t.nseg - 1) * NW * ws_wave_floats + (int64_t)t.tail_bg * HG * (t.nseg - 1)) * 4);
  }

  // query != null: only report the workspace the launch would use
  static int run(const LinArgs& a, int want_segments, void* ws, size_t ws_size, hipStream_t stream, size_t* query) {
    int resident = 1, cus = 256;
    if (!prepare(resident, cus)) {
      if (query) { *query = 0; return 0; }
      return -1;
    }
    LinArgs args = a;
    args.dv_blocks = a.Dv / (32 * NWH);
    // general operand addressing: defaults for what is left at zero; the row distances must be multiples of the tile
    // rows (the kernel XORs the swizzle of an instruction's first row onto the finished lane offset)
    const bool gen = a.rev != 0 || a.q_row != 0 || a.k_row != 0 || a.v_row != 0 || (a.Hv != 0 && a.Hv != a.H) || a.qk_cols != 0 || a.n_pieces > 1 || a.rev_o != 0;
    if (gen) {
      if (args.q_row == 0) args.q_row = DK;
      if (args.k_row == 0) args.k_row = DK;
      if (args.v_row == 0) args.v_row = a.Dv;
      if (args.Hv == 0) args.Hv = a.H;
      if (args.q_row % 8 != 0 || args.k_row % 8 != 0 || args.v_row % (32 * NWH) != 0 || args.Hv <= 0 || a.H % args.Hv != 0) return -2;
      if (a.qk_cols < 0 || a.qk_cols > DK || a.qk_cols % 8 != 0) return -2;
      if (HG > 1 && args.Hv != a.H) return -2;
      if (a.n_pieces > 1 && !a.out_f32) return -2;
    } else if (a.n_pieces > 1) {
      return -2;
    }
    const unsigned pieces = a.n_pieces > 1 ? (unsigned)a.n_pieces : 1u;
    plan(a, want_segments, resident, cus, args.nseg, args.seg_chunks);
    const Tail tail = args.nseg <= 1 ? tail_plan(a, want_segments, resident, cus) : Tail{0, 0, 1, 0};
    if (query) { *query = tail.tail_bg > 0 ? tail_ws_bytes(tail, args.dv_blocks) : ws_bytes(a, args.nseg); return 0; }
    if (args.nseg > 1 && (!ws || ws_size < ws_bytes(a, args.nseg) || ((uintptr_t)ws & 3) != 0)) args.nseg = 1;   // no workspace: single pass
    const unsigned groups = (unsigned)((int64_t)a.B * a.H / HG * args.dv_blocks);
    if (args.nseg <= 1 && tail.tail_bg > 0 && ws && ws_size >= tail_ws_bytes(tail, args.dv_blocks) && ((uintptr_t)ws & 3) == 0) {
      // the full rounds in a single pass, then the tail in segments (see tail_plan)
      LinArgs full = args;
      full.nseg = 1;
      full.bg0 = 0;
      full.bg_n = tail.full_bg;
      const unsigned g_full = (unsigned)tail.full_bg * args.dv_blocks, g_tail = (unsigned)tail.tail_bg * args.dv_blocks;
      if (gen) hipLaunchKernelGGL((linear_fwd_kernel<DK, NWH, HG, 0, true>), dim3(g_full, pieces), dim3(64 * NW), lds, stream, full);
      else hipLaunchKernelGGL((linear_fwd_kernel<DK, NWH, HG, 0>), dim3(g_full), dim3(64 * NW), lds, stream, full);
      LinArgs rest = args;
      rest.nseg = tail.nseg;
      rest.seg_chunks = tail.seg_chunks;
      rest.bg0 = tail.full_bg;
      rest.bg_n = tail.tail_bg;
      rest.ws_state = (float*)ws;
      rest.ws_decay = rest.ws_state + (int64_t)g_tail * (tail.nseg - 1) * NW * ws_wave_floats;
      if (gen) {
        hipLaunchKernelGGL((linear_fwd_kernel<DK, NWH, HG, 1, true>), dim3(g_tail * (tail.nseg - 1)), dim3(64 * NW), lds, stream, rest);
        hipLaunchKernelGGL((linear_fwd_kernel<DK, NWH, HG, 2, true>), dim3(g_tail * tail.nseg), dim3(64 * NW), lds, stream, rest);
      } else {
        hipLaunchKernelGGL((linear_fwd_kernel<DK, NWH, HG, 1>), dim3(g_tail * (tail.nseg - 1)), dim3(64 * NW), lds, stream, rest);
        hipLaunchKernelGGL((linear_fwd_kernel<DK, NWH, HG, 2>), dim3(g_tail * tail.nseg), dim3(64 * NW), lds, stream, rest);
      }
    } else if (args.nseg <= 1) {
      args.nseg = 1;
      if (gen) hipLaunchKernelGGL((linear_fwd_kernel<DK, NWH, HG, 0, true>), dim3(groups, pieces), dim3(64 * NW), lds, stream, args);
      else hipLaunchKernelGGL((linear_fwd_kernel<DK, NWH, HG, 0>), dim3(groups), dim3(64 * NW), lds, stream, args);
    } else {
      args.ws_state = (float*)ws;
      args.ws_decay = args.ws_state + (int64_t)groups * (args.nseg - 1) * NW * ws_wave_floats;
      if (gen) {
        hipLaunchKernelGGL((linear_fwd_kernel<DK, NWH, HG, 1, true>), dim3(groups * (args.nseg - 1)), dim3(64 * NW), lds, stream, args);
        hipLaunchKernelGGL((linear_fwd_kernel<DK, NWH, HG, 2, true>), dim3(groups * args.nseg), dim3(64 * NW), lds, stream, args);
      } else {
        hipLaunchKernelGGL((linear_fwd_kernel<DK, NWH, HG, 1>), dim3(groups * (args.nseg - 1)), dim3(64 * NW), lds, stream, args);
        hipLaunchKernelGGL((linear_fwd_kernel<DK, NWH, HG, 2>), dim3(groups * args.nseg), dim3(64 * NW), lds, stream, args);
      }
    }
    return launch_status();
  }
};
}  // namespace

// returns 0 ok, -1 launch failure, -2 unsupported.  With query != null nothing is launched and *query
// receives the workspace size the same call would use.
int linear_fwd_dispatch(const LinArgs& a, int dk, int want_segments, void* ws, size_t ws_size, hipStream_t stream, size_t* query) {
  const int dv = a.Dv;
  // two heads per workgroup when they share their q and k heads (Mamba2: all heads of a batch entry do)
  const bool pairable = a.H % 2 == 0 && (a.H / a.Hq) % 2 == 0 && (a.H / a.Hk) % 2 == 0 && (a.Hv == 0 || a.Hv == a.H);
  if (dk == 256) {
    if (dv % 256 == 0) return Config<256, 8, 1>::run(a, want_segments, ws, ws_size, stream, query);
    if (dv % 128 == 0) return Config<256, 4, 1>::run(a, want_segments, ws, ws_size, stream, query);
    if (dv % 64 == 0) return Config<256, 2, 1>::run(a, want_segments, ws, ws_size, stream, query);
  } else if (dk == 128) {
    if (dv % 256 == 0) return Config<128, 8, 1>::run(a, want_segments, ws, ws_size, stream, query);
    if (dv % 128 == 0) return Config<128, 4, 1>::run(a, want_segments, ws, ws_size, stream, query);
    if (dv % 64 == 0 && pairable) return Config<128, 2, 2>::run(a, want_segments, ws, ws_size, stream, query);
    if (dv % 64 == 0) return Config<128, 2, 1>::run(a, want_segments, ws, ws_size, stream, query);
  }
  return -2;
}

}  // namespace ma
