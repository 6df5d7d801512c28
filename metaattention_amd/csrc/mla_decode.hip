// Absorbed MLA decode (one query token, shared latent KV cache) for gfx950.
//
// Replaces flash_attn_split + combine of
// attention_engine/core/template/tl_template/attn/mla_decode_tl.py:154-290:
//   o[b,h,:] = softmax((q[b,h].kv[b,n] + q_pe[b,h].k_pe[b,n]) * scale) . kv[b,n]
//
// Split kernel.  A workgroup (8 waves, two per SIMD, the whole CU) owns one (batch, kv split, block of
// 128 query heads) and consumes 32-row latent sub-tiles from LDS, so the cache leaves HBM exactly once.
// At 128 heads the arithmetic is as dense as the memory stream, and what saturates first is the LDS: every
// MFMA needs a fresh 1 KB operand from it.  v_mfma_f32_32x32x16 with 32 heads per MFMA halves that
// traffic per flop, but a wave cannot hold 32 heads x (576 Q + 512 accumulator) columns.  So two waves
// share a group of 32 heads and split the work along the long axes:
//   * scores:  each wave takes half of the 576-wide contraction (18 of the 36 k-slices, Q fragments of
//     its half in 72 registers), S^T_half = KV_half Q_half^T; the halves are exchanged through LDS
//     (4 KB each way) and added, so both waves hold the full 32 x 32 score tile;
//   * softmax: computed by both (16 scores per lane; the sums a+b and b+a are the same bits);
//   * output:  each wave takes half of the 512 value columns, O^T_half += KV_half^T P^T (128 registers).
// Sub-tiles arrive by direct-to-LDS DMA (global_load_lds_dwordx4: no staging registers) through a ring of
// 3 stages, two sub-tiles ahead of their use, and a wave waits for its own share with a partial vmcnt.
//   A[32 x 16]: lane holds row l%32, k = 8(l/32) .. +7
//   B[16 x 32]: lane holds column l%32, k = 8(l/32) .. +7
//   C[32 x 32]: lane holds column l%32, element j is row 8(j/4) + 4(l/32) + j%4
// Scores are computed transposed (S^T = KV Q^T) so each lane owns one head's row statistics and the
// probabilities feed O^T += KV^T P^T straight from the accumulator registers; KV^T comes out of the same
// row-major LDS tile through the transposing read, so V is never loaded separately.
// Combine kernel: log-sum-exp merge of the partials.
#include "mla_decode.h"

namespace ma {

namespace {
constexpr int BN = 32;         // kv rows per sub-tile
constexpr int HB = 128;        // heads per workgroup
constexpr int NW = 8;          // waves per workgroup: 4 head groups x 2 halves
constexpr int D = 512, DPE = 64;
constexpr int NSTAGE = 3;
constexpr int KV_ROW = D * 2 + 32;  // bytes; each latent row is its own DMA, so rows can be padded: with a
                                   // 32 B pad consecutive rows start 8 banks apart (the transposing reads of
                                   // 8 rows x 32 B tile the 64 banks exactly) and rows 8..15 of every 16-row group
                                   // additionally swap their 16-byte chunk pairs (kv_flip) so that the 128-bit
                                   // reads of 16 rows x one chunk hit 16 different bank groups.  Every LDS
                                   // read address is then lane base + compile-time offset.
constexpr int PE_ROW = DPE * 2;    // rope rows share a DMA (8 rows per KB): XOR-swizzled instead
constexpr int KV_TILE = BN * KV_ROW;   // 33 KB
constexpr int PE_TILE = BN * PE_ROW;   // 4 KB
constexpr int STAGE = KV_TILE + PE_TILE;
constexpr int XCHG = 4096;             // one wave's half score tile: 16 fp32 per lane

__device__ __forceinline__ int kv_flip(int row) { return (row >> 3) & 1; }
__device__ __forceinline__ int swz_pe(int row) { return (row >> 1) & 7; }
}  // namespace

// PLANNED: the workgroup does not own one (batch, kv split) but the contiguous run of work that the plan gives
// its part (plan_part of the kernel below the split kernel): a sequence of pieces (batch entry, token range, split
// index), each handled like one (batch, split) of the unplanned launch.
template <typename T, bool PLANNED>
__global__ __launch_bounds__(64 * NW, 2) void mla_split_kernel(const MlaArgs a) {
  using E = Elem<T>;
  using x8 = typename E::x8;
  using x4 = typename E::x4;
  using x2 = typename E::x2;
  constexpr int NSL = (D + DPE) / 16 / 2;   // 18 k-slices of 16 per wave
  constexpr int NLAT1 = D / 16 - NSL;       // latent slices of the second half (14); its last 4 slices are the rope columns
  constexpr int DBH = D / 32 / 2;           // 8 output blocks of 32 columns per wave

  extern __shared__ __align__(16) char smem[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(MA_LDS char*)smem;
  const uint32_t lds_x = lds0 + NSTAGE * STAGE;

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int hg = wave >> 1, hf = wave & 1;   // head group, half: partners are on different SIMDs (wave % 4)
  const bool late = wave >= 4;               // head groups 2 and 3 run half a sub-tile behind (see the main loop)
  const int r = lane & 31, g = lane >> 5;
  const int hblk = blockIdx.x % a.head_blocks, bs = blockIdx.x / a.head_blocks;
  const int head = hblk * HB + hg * 32 + r;
  const int head_ld = min(head, a.Hq - 1);
  const int64_t kv_row_bytes = a.kvss * 2, pe_row_bytes = a.kpss * 2;

  // ---- the pieces of this workgroup: one (batch, split) of the uniform launch, or the run its part of the plan names
  //      (tile_scheduler_metadata[part] = {first batch, its first token, last batch, its end token, split index of the
  //      first piece}; a later piece of the run starts a batch entry: token 0, split index 0)
  int b_first, b_last, first_token = 0, last_end = 0, first_split = 0;
  if constexpr (PLANNED) {
    const int32_t* md = a.plan_meta + (int64_t)bs * 8;
    b_first = md[0]; first_token = md[1]; b_last = md[2]; last_end = md[3]; first_split = md[4];
    if (b_first >= a.B) return;   // a part the plan left without work
  } else {
    b_first = b_last = bs / a.num_split;
  }
  // per piece
  int b = 0, split = 0, n_begin = 0, skv = 0, n_end = 0, n_tiles = 0;
  bool direct = true;          // the piece is its batch entry's only one: it writes the final output
  int64_t slot = 0;            // else: its slot among the partial results
  const char* kvb = nullptr;
  const char* peb = nullptr;
  x8 qf[NSL];   // Q fragments of this wave's half of the contraction: B operand (lane: head r, k = 8g .. 8g+7 of a slice)

  // ---- DMA.  Wave w streams latent rows 4w..4w+3 of a sub-tile, one instruction per row (64 lanes x 16 B =
  //      the 1 KB row; lane i fetches the chunk that belongs at physical chunk i); waves 0..3 also fetch 8
  //      rope rows each with one more instruction.  Rows beyond the cache are clamped to its last row
  //      (their scores are masked).
  const uint32_t lane_off = (uint32_t)(lane ^ ((wave >> 1) & 1)) << 4;   // kv_flip(4w + i) = (w >> 1) & 1
  auto issue_tile = [&](int jt) {
    const uint32_t sb = lds0 + (jt % NSTAGE) * STAGE;
    const int n0 = n_begin + jt * BN;
    // where the sub-tile's first row lives: with pages, in the page the block table names (a sub-tile never
    // straddles pages: page sizes and split lengths are multiples of 32)
    int64_t row0 = n0;
    if (a.block_table) row0 = (int64_t)a.block_table[b * a.bt_stride + n0 / a.page_size] * a.page_size + n0 % a.page_size;
    const int last = skv - 1 - n0;   // rows of the sub-tile beyond the cache are clamped to its last row
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int row = wave * 4 + i;
      dma16_so(kvb + (row0 + min(row, last)) * kv_row_bytes, lane_off, sb + row * KV_ROW);
    }
    if (wave < 4) {
      const int row = wave * 8 + (lane >> 3);
      dma16(peb + (row0 + min(row, last)) * pe_row_bytes + (((lane & 7) ^ swz_pe(row)) << 4), sb + KV_TILE + wave * 8 * PE_ROW);
    }
  };

  // ---- per-lane LDS read offsets within a stage
  // K side (A operand): row r, logical 16-byte chunk 2 * slice + g; this wave's first slice is hf * 18
  const uint32_t k_off = r * KV_ROW + ((g ^ kv_flip(r)) << 4) + hf * (NSL * 32);
  const uint32_t pe_off = KV_TILE + r * PE_ROW;
  const int pe_c0 = g ^ swz_pe(r);
  // V side (transposing read): the low half of a fragment reads rows 16sl + 4g + jr (chunks not flipped), the
  // high half rows + 8 (chunk pairs flipped); chunk 4 * block + lc; this wave's first block is hf * 8
  const int jr = (lane & 15) >> 2;
  const int lc = (((lane >> 4) & 1) << 1) | ((lane & 3) >> 1);
  const uint32_t v_lo_off = (4 * g + jr) * KV_ROW + (lc << 4) + (lane & 1) * 8 + hf * (DBH * 64);
  const uint32_t v_hi_off = (4 * g + jr + 8) * KV_ROW + ((lc ^ 1) << 4) + (lane & 1) * 8 + hf * (DBH * 64);
  // exchange of the half score tiles: 4 x 16 bytes per lane, lane-major
  const uint32_t x_mine = lds_x + wave * XCHG + lane * 16, x_other = lds_x + (wave ^ 1) * XCHG + lane * 16;

  f32x16 o[DBH];
  const float c_scale = a.scale * kLog2e;
  float row_ref = -1e30f, row_sum = 0.f;
  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

  f32x16 sc;   // this wave's half scores, then the full scores, of the sub-tile it is working on

  // ---- phase A of sub-tile jt: half scores S^T_half = KV_half Q_half^T over this wave's 18 k-slices, handed to the partner
  auto half_scores = [&](int jt) {
    const uint32_t base = lds0 + (jt % NSTAGE) * STAGE;
    constexpr int AH = 2, RING = AH + 1;
    x8 kf[RING];
    uint32_t kb = base + k_off, pb = base + pe_off;
    asm volatile("" : "+v"(kb), "+v"(pb));   // one address register + immediates for the reads below
    // the last four slices of the second half are the rope columns (their own, XOR-swizzled tile)
    uint32_t tail[NSL - NLAT1];
#pragma unroll
    for (int j = 0; j < NSL - NLAT1; j++) tail[j] = hf ? pb + (uint32_t)((pe_c0 ^ (2 * j)) << 4) : kb + 32 * (NLAT1 + j);
    auto request = [&](int sl) {
      kf[sl % RING] = lds_read<x8>(sl < NLAT1 ? kb + 32 * sl : tail[sl < NLAT1 ? 0 : sl - NLAT1]);
    };
#pragma unroll
    for (int sl = 0; sl < AH; sl++) request(sl);
#pragma unroll
    for (int sl = 0; sl < NSL; sl++) {
      if (sl + AH < NSL) request(sl + AH);
      __builtin_amdgcn_sched_barrier(0);   // keep the requests ahead of the MFMAs that hide their latency
      sc = E::mfma32(kf[sl % RING], qf[sl], sl == 0 ? zero16 : sc);
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int j4 = 0; j4 < 4; j4++) lds_write<f32x4>(x_mine + j4 * 1024, f32x4{sc[4 * j4], sc[4 * j4 + 1], sc[4 * j4 + 2], sc[4 * j4 + 3]});
  };

  // ---- phase B of sub-tile jt (a barrier after the partner's phase A): add the halves, softmax, O^T_half += KV_half^T P^T
  auto softmax_pv = [&](int jt) {
    const int n0 = n_begin + jt * BN;
    const uint32_t base = lds0 + (jt % NSTAGE) * STAGE;
#pragma unroll
    for (int j4 = 0; j4 < 4; j4++) {
      const f32x4 t = lds_read<f32x4>(x_other + j4 * 1024);
#pragma unroll
      for (int i = 0; i < 4; i++) sc[4 * j4 + i] += t[i];
    }

    // the first fragments of P V are requested before the softmax: their latency hides behind it
    uint32_t vlo = base + v_lo_off, vhi = base + v_hi_off;
    asm volatile("" : "+v"(vlo), "+v"(vhi));
    constexpr int PF = 3, NPV = 2 * DBH;   // fragments in flight; MFMA i: slice i / DBH, block i % DBH
    x4 lo[PF], hi[PF];
    auto v_request = [&](int i) {
      const int sl = i / DBH, db = i % DBH;
      lo[i % PF] = lds_read_tr4<T>(vlo + 16 * sl * KV_ROW + 64 * db);
      hi[i % PF] = lds_read_tr4<T>(vhi + 16 * sl * KV_ROW + 64 * db);
    };
#pragma unroll
    for (int i = 0; i < PF - 1; i++) v_request(i);

    // mask, online softmax in the log2 domain: lane holds head r, kv rows 8(j/4) + 4g + j%4
    if (n0 + BN > n_end) {
#pragma unroll
      for (int j = 0; j < 16; j++)
        if (n0 + 8 * (j >> 2) + 4 * g + (j & 3) >= n_end) sc[j] = -INFINITY;
    }
    float mx = sc[0];
#pragma unroll
    for (int j = 1; j < 16; j++) mx = fmaxf(mx, sc[j]);
    {
      float m_lo, m_hi;
      xhalf_pair(mx, m_lo, m_hi);
      mx = fmaxf(m_lo, m_hi);
    }
    // The reference point of the exponentials only moves when some head's max grew by more than 2^8: until
    // then the probabilities are taken relative to the stale reference (at most 256, exact in fp32 / in
    // range for bf16 and fp16) and the 128 accumulator registers need no rescaling.  The final
    // normalisation by row_sum absorbs the offset.  Each head decides for itself.
    const float cand = fmaxf(row_ref, mx * c_scale);
    const bool move = cand - row_ref > 8.f;
    if (__any(move)) {
      const float corr = move ? fast_exp2(row_ref - cand) : 1.f;
      row_ref = move ? cand : row_ref;
      row_sum *= corr;
#pragma unroll
      for (int i = 0; i < DBH; i++)
#pragma unroll
        for (int j = 0; j < 16; j++) asm volatile("v_mul_f32 %0, %0, %1" : "+v"(o[i][j]) : "v"(corr));
    }
    // probabilities, packed as the B operand of P V: p[sl] holds elements 8sl .. 8sl+7 (k slot i of lane
    // half g is kv row 16sl + 8(i/4) + 4g + i%4, matched by the rows the transposing V reads fetch)
    x8 p[2];
    float part = 0.f;
#pragma unroll
    for (int j = 0; j < 16; j++) {
      const float pe = fast_exp2(sc[j] * c_scale - row_ref);
      part += pe;
      p[j >> 3][j & 7] = (T)pe;
    }
    row_sum += part;

#pragma unroll
    for (int i = 0; i < NPV; i++) {
      if (i + PF - 1 < NPV) v_request(i + PF - 1);
      __builtin_amdgcn_sched_barrier(0);
      x8 vf = __builtin_shufflevector(lo[i % PF], hi[i % PF], 0, 1, 2, 3, 4, 5, 6, 7);
      o[i % DBH] = E::mfma32(vf, p[i / DBH], o[i % DBH]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // Two barriers per sub-tile: [barrier, phase A, barrier, phase B].  Head groups 2 and 3 (waves 4..7) pass one
  // barrier more before their first sub-tile and groups 0 and 1 one more after their last, so the late groups
  // run half a sub-tile behind: while an early wave is in phase A the late wave on its SIMD is in phase B of
  // the sub-tile before, and the other way round.  One wave's softmax (vector ALU) then always runs beside the
  // other wave's MFMAs instead of both doing the same thing at the same time.  With the global barrier count
  // k = 1, 2, ..: early waves run A(j) after k = 2j+1 and B(j) after 2j+2, late waves A(j) after 2j+2 and B(j)
  // after 2j+3.  Sub-tile j is read from k = 2j+1 on, so every wave has waited for its own loads of it before
  // that barrier; its stage is free after k = 2j+4, which is where sub-tile j+3 is requested.
  auto wait_tile = [&](int t) {   // this wave's loads of sub-tile t have landed (they complete in order: only those of t+1 may be in flight)
    if (t + 1 < n_tiles) {
      if (wave < 4) __builtin_amdgcn_s_waitcnt(0x0F70 | 5); else __builtin_amdgcn_s_waitcnt(0x0F70 | 4);
    } else {
      wait_dma();
    }
  };
  for (b = b_first; b <= b_last; b++) {
  // ---- this piece
  if constexpr (PLANNED) {
    skv = min(a.Skv, max(a.kv_lens[b], 0));
    n_begin = b == b_first ? first_token : 0;
    n_end = min(b == b_last ? last_end : skv, skv);
    split = b == b_first ? first_split : 0;
    const int first_slot = a.plan_splits[b];
    direct = a.plan_splits[b + 1] - first_slot == 1;
    slot = first_slot + split;
  } else {
    split = bs % a.num_split;
    n_begin = split * a.split_len;
    skv = a.kv_lens ? min(a.Skv, max(a.kv_lens[b], 0)) : a.Skv;   // this batch entry's cache length
    n_end = min(n_begin + a.split_len, skv);
    direct = a.num_split == 1;
    slot = (int64_t)b * a.num_split + split;
  }
  n_tiles = n_end > n_begin ? (n_end - n_begin + BN - 1) / BN : 0;
  kvb = (const char*)a.kv + (int64_t)b * a.kvsb * 2;
  peb = (const char*)a.k_pe + (int64_t)b * a.kpsb * 2;
  {
    const T* qp = (const T*)a.q + (int64_t)b * a.qsb + (int64_t)head_ld * a.qsh + 8 * g + hf * (NSL * 16);
    const T* qpe = (const T*)a.q_pe + (int64_t)b * a.qpsb + (int64_t)head_ld * a.qpsh + 8 * g;
#pragma unroll
    for (int sl = 0; sl < NSL; sl++) {
      const T* src = (hf == 1 && sl >= NLAT1) ? qpe + 16 * (sl - NLAT1) : qp + 16 * sl;
      qf[sl] = *(const x8*)src;
    }
  }
#pragma unroll
  for (int i = 0; i < DBH; i++)
#pragma unroll
    for (int j = 0; j < 16; j++) o[i][j] = 0.f;
  row_ref = -1e30f;
  row_sum = 0.f;
  if (n_tiles > 0) issue_tile(0);
  if (n_tiles > 1) issue_tile(1);

  if (late) {
    wait_tile(0);
    __syncthreads();
  }
  for (int jt = 0; jt < n_tiles; jt++) {
    if (!late) wait_tile(jt);
    __syncthreads();
    if (late && jt + 2 < n_tiles) issue_tile(jt + 2);
    half_scores(jt);
    if (late && jt + 1 < n_tiles) wait_tile(jt + 1);
    __syncthreads();
    if (!late && jt + 2 < n_tiles) issue_tile(jt + 2);
    softmax_pv(jt);
  }
  if (!late) __syncthreads();

  // ---- epilogue: lane holds head r, output columns 256 hf + 32db + 8(j/4) + 4g + j%4
  float t_lo, t_hi;
  xhalf_pair(row_sum, t_lo, t_hi);
  const float tot = t_lo + t_hi;
  const bool empty = n_tiles == 0;
  const float inv = empty ? 0.f : 1.f / tot;
  const float lse2 = empty ? -INFINITY : row_ref + fast_log2(tot);   // log2 domain
  // Stage the wave's 32 heads x 256 columns through LDS (the stages are free now) so that every head's
  // half row leaves as 512 contiguous bytes in 16-byte pieces; chunks are XOR-swizzled by head so that
  // neither the 8-byte writes nor the 16-byte reads pile onto one bank group.
  __syncthreads();   // every wave is done with the last sub-tile
  {
    constexpr int SROW = D;   // bytes: 256 columns of T
    const uint32_t sb = lds0 + wave * 32 * SROW;
#pragma unroll
    for (int db = 0; db < DBH; db++)
#pragma unroll
      for (int q4 = 0; q4 < 4; q4++) {
        x4 w;
#pragma unroll
        for (int i = 0; i < 4; i++) w[i] = (T)(o[db][4 * q4 + i] * inv);
        lds_write<x4>(sb + r * SROW + (((4 * db + q4) ^ (r & 31)) << 4) + 8 * g, w);
      }
    T* obase = direct ? (T*)a.o + (int64_t)b * a.osb : (T*)a.o_part + slot * a.Hq * D;
    const int64_t ostride = direct ? a.osh : D;
    const int head0 = hblk * HB + hg * 32;
#pragma unroll
    for (int it = 0; it < 32 * (SROW / 16) / 64; it++) {
      const int ci = lane + 64 * it, row = ci / (SROW / 16), c = ci % (SROW / 16);
      const u32x4 w = lds_read<u32x4>(sb + row * SROW + ((c ^ (row & 31)) << 4));
      if (head0 + row < a.Hq) *(u32x4*)(obase + (int64_t)(head0 + row) * ostride + hf * (D / 2) + c * 8) = w;
    }
  }
  if (head < a.Hq && hf == 0 && g == 0) {
    if (direct) {
      if (a.lse) a.lse[(int64_t)b * a.Hq + head] = lse2 * kLn2;
    } else {
      a.lse_part[slot * a.Hq + head] = lse2;
    }
  }
  if (PLANNED && b < b_last) __syncthreads();   // the staged output has left the stages: the next piece may fill them
  }   // pieces
}

// Four (batch, head) pairs per workgroup: 64 threads x 8 output columns each.
template <typename T>
__global__ __launch_bounds__(256) void mla_combine_kernel(const MlaArgs a) {
  using x8 = typename Elem<T>::x8;
  const int tid = threadIdx.x & 63;
  const int64_t bh = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (bh >= (int64_t)a.B * a.Hq) return;
  const int b = (int)(bh / a.Hq), head = (int)(bh % a.Hq);
  // the partial results of this batch entry: num_split slots from b * num_split on, or what the plan says (an entry with
  // a single piece has written its output itself)
  int ns = a.num_split;
  int64_t first = (int64_t)b * ns;
  if (a.plan_splits) {
    first = a.plan_splits[b];
    ns = a.plan_splits[b + 1] - (int)first;
    if (ns <= 1) return;
  }
  const float* lp = a.lse_part + first * a.Hq + head;
  if (ns > 64) {
    // (only a plan can cut a batch entry into this many pieces: one very long sequence on many parts)
    float mx = -INFINITY;
    for (int s2 = tid; s2 < ns; s2 += 64) mx = fmaxf(mx, lp[(int64_t)s2 * a.Hq]);
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) mx = fmaxf(mx, __shfl_xor(mx, m, 64));
    // (every piece empty: mx = -inf; the weights are then 0, the output zeros and the lse -inf, as the unsplit launch gives)
    const float mref = mx == -INFINITY ? 0.f : mx;
    float sum = 0.f;
    for (int s2 = tid; s2 < ns; s2 += 64) sum += fast_exp2(lp[(int64_t)s2 * a.Hq] - mref);
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) sum += __shfl_xor(sum, m, 64);
    const float inv = sum > 0.f ? 1.f / sum : 0.f;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    const T* pp = (const T*)a.o_part + (first * a.Hq + head) * D + tid * 8;
    for (int s2 = 0; s2 < ns; s2++) {
      const float w = fast_exp2(lp[(int64_t)s2 * a.Hq] - mref) * inv;
      const x8 v = *(const x8*)(pp + (int64_t)s2 * a.Hq * D);
#pragma unroll
      for (int i = 0; i < 8; i++) acc[i] += (float)v[i] * w;
    }
    x8 w;
#pragma unroll
    for (int i = 0; i < 8; i++) w[i] = (T)acc[i];
    *(x8*)((T*)a.o + (int64_t)b * a.osb + (int64_t)head * a.osh + tid * 8) = w;
    if (a.lse && tid == 0) a.lse[(int64_t)b * a.Hq + head] = sum > 0.f ? (mx + fast_log2(sum)) * kLn2 : -INFINITY;
    return;
  }
  // lane s of the wave holds the log-sum-exp of split s (at most 64 splits here): one load, wave reductions
  const float my = tid < ns ? lp[(int64_t)tid * a.Hq] : -INFINITY;
  float mx = my;
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) mx = fmaxf(mx, __shfl_xor(mx, m, 64));
  // (every piece empty: mx = -inf; weights 0, output zeros, lse -inf, as the unsplit launch gives)
  const float e = (tid < ns && mx != -INFINITY) ? fast_exp2(my - mx) : 0.f;
  float sum = e;
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) sum += __shfl_xor(sum, m, 64);
  const float wgt = sum > 0.f ? e / sum : 0.f;
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const T* pp = (const T*)a.o_part + (first * a.Hq + head) * D + tid * 8;
  int s0 = 0;
  for (; s0 + 4 <= ns; s0 += 4) {   // four independent loads in flight
    x8 v[4];
#pragma unroll
    for (int k = 0; k < 4; k++) v[k] = *(const x8*)(pp + (int64_t)(s0 + k) * a.Hq * D);
#pragma unroll
    for (int k = 0; k < 4; k++) {
      const float w = __shfl(wgt, s0 + k, 64);
#pragma unroll
      for (int i = 0; i < 8; i++) acc[i] += (float)v[k][i] * w;
    }
  }
  for (; s0 < ns; s0++) {
    const float w = __shfl(wgt, s0, 64);
    const x8 v = *(const x8*)(pp + (int64_t)s0 * a.Hq * D);
#pragma unroll
    for (int i = 0; i < 8; i++) acc[i] += (float)v[i] * w;
  }
  x8 w;
#pragma unroll
  for (int i = 0; i < 8; i++) w[i] = (T)acc[i];
  *(x8*)((T*)a.o + (int64_t)b * a.osb + (int64_t)head * a.osh + tid * 8) = w;
  if (a.lse && tid == 0) a.lse[(int64_t)b * a.Hq + head] = sum > 0.f ? (mx + fast_log2(sum)) * kLn2 : -INFINITY;
}

// The work plan of get_mla_metadata.cu:8-75, one lane: cache blocks of block_n tokens plus a fixed overhead per batch
// entry are dealt to `parts` workgroups in order, each taking about total / parts (+ overhead); a batch entry cut by a
// part boundary gets one more split.  meta[p] = {first batch, first token, last batch, end token, split index of the
// first piece, 0, 0, 0}; splits[b] = number of pieces of the batch entries before b.
__global__ __launch_bounds__(64) void mla_plan_kernel(const int32_t* seqlens, int batch, int parts, int block_n, int overhead,
                                                      int32_t* meta, int32_t* splits) {
  if (threadIdx.x != 0) return;
  int total = 0;
  for (int i = 0; i < batch; i++) total += (max(seqlens[i], 0) + block_n - 1) / block_n + overhead;
  const int payload = max((total + parts - 1) / parts + overhead, 2 * overhead);
  int now_idx = 0, now_block = 0, now_split = 0, cum = 0;
  splits[0] = 0;
  for (int p = 0; p < parts; p++) {
    int32_t* m = meta + (int64_t)p * 8;
    m[0] = now_idx;
    m[1] = now_block * block_n;
    m[4] = now_split;
    int remain = payload;
    while (now_idx < batch) {
      const int blocks = (max(seqlens[now_idx], 0) + block_n - 1) / block_n;
      const int left = blocks - now_block;
      if (remain >= left + overhead) {
        cum += now_split + 1;
        splits[now_idx + 1] = cum;
        remain -= left + overhead;
        now_idx++;
        now_block = 0;
        now_split = 0;
      } else {
        if (remain - overhead > 0) {
          now_block += remain - overhead;
          now_split++;
          remain = 0;
        }
        break;
      }
    }
    m[2] = now_block > 0 ? now_idx : now_idx - 1;
    m[3] = now_block > 0 ? now_block * block_n : (now_idx > 0 ? max(seqlens[now_idx - 1], 0) : 0);
    m[5] = m[6] = m[7] = 0;
  }
}

int mla_plan_dispatch(const int32_t* seqlens, int batch, int parts, int block_n, int overhead_blocks, int32_t* meta, int32_t* splits,
                      hipStream_t stream) {
  hipLaunchKernelGGL(mla_plan_kernel, dim3(1), dim3(64), 0, stream, seqlens, batch, parts, block_n, overhead_blocks, meta, splits);
  return launch_status();
}

template <typename T>
static int launch_t(const MlaArgs& a, hipStream_t stream) {
  constexpr size_t lds = NSTAGE * (size_t)STAGE + NW * (size_t)XCHG;
  auto kern = mla_split_kernel<T, false>;
  auto kern_planned = mla_split_kernel<T, true>;
  static std::atomic<uint64_t> lds_ok{0};
  if (allow_lds(lds_ok, lds, kern, kern_planned) != 0) return -1;
  MlaArgs args = a;
  args.head_blocks = (a.Hq + HB - 1) / HB;
  if (a.plan_meta) {
    hipLaunchKernelGGL(kern_planned, dim3((unsigned)(a.plan_parts * args.head_blocks)), dim3(64 * NW), lds, stream, args);
    if (launch_status() != 0) return -1;
    hipLaunchKernelGGL(mla_combine_kernel<T>, dim3((unsigned)(((int64_t)a.B * a.Hq + 3) / 4)), dim3(256), 0, stream, args);
    return launch_status();
  }
  const unsigned grid = (unsigned)(a.B * a.num_split * args.head_blocks);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * NW), lds, stream, args);
  if (launch_status() != 0) return -1;
  if (a.num_split > 1) {
    hipLaunchKernelGGL(mla_combine_kernel<T>, dim3((unsigned)(((int64_t)a.B * a.Hq + 3) / 4)), dim3(256), 0, stream, a);
    if (launch_status() != 0) return -1;
  }
  return 0;
}

int mla_decode_dispatch(const MlaArgs& a, bool is_bf16, int dim, int dim_pe, hipStream_t stream) {
  if (dim != D || dim_pe != DPE) return -2;
  return is_bf16 ? launch_t<__bf16>(a, stream) : launch_t<_Float16>(a, stream);
}

}  // namespace ma
