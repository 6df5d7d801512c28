// Absorbed MLA decode (one query token, shared latent KV cache) for gfx950.
//
// Replaces flash_attn_split + combine of
// attention_engine/core/template/tl_template/attn/mla_decode_tl.py:154-290:
//   o[b,h,:] = softmax((q[b,h].kv[b,n] + q_pe[b,h].k_pe[b,n]) * scale) . kv[b,n]
//
// Split kernel.  A workgroup (8 waves, two per SIMD, the whole CU) owns one (batch, kv split, block of
// 128 query heads); wave w owns heads 16w..16w+15 and all eight waves consume the same 32-row latent
// sub-tiles from LDS, so the cache leaves HBM exactly once.  Sub-tiles arrive by direct-to-LDS DMA
// (global_load_lds_dwordx4: no staging registers; the registers hold the 576-wide Q fragments and the
// 512 x 16 fp32 output accumulator of the wave) through a ring of 4 stages, three sub-tiles ahead of their
// use, and a wave waits for its own share with a partial vmcnt before the one barrier per sub-tile.
// v_mfma_f32_16x16x32 is used throughout:
//   A[16 x 32]: lane holds row l%16, k = 8(l/16) .. +7
//   B[32 x 16]: lane holds column l%16, k = 8(l/16) .. +7
//   C[16 x 16]: lane holds column l%16, element j is row 4(l/16) + j
// Scores are computed transposed (S^T = KV Q^T) so each lane owns one head's
// row statistics and the probabilities feed O^T += KV^T P^T straight from the
// accumulator registers; KV^T comes out of the same row-major LDS tile through
// the transposing read, so V is never loaded separately.  Within a wave the phases of a sub-tile run one
// after the other (scores, softmax, P V); the second wave on the SIMD fills the gaps.
// Combine kernel: log-sum-exp merge of the fp32 partials.
#include "mla_decode.h"

namespace ma {

namespace {
constexpr int BN = 32;         // kv rows per sub-tile
constexpr int HB = 128;        // heads per workgroup
constexpr int NW = 8;          // waves per workgroup
constexpr int D = 512, DPE = 64;
constexpr int NSTAGE = 4;
constexpr int KV_ROW = D * 2 + 32;  // bytes; each latent row is its own DMA, so rows can be padded: with a
                                   // 32 B pad consecutive rows start 8 banks apart (the transposing reads of
                                   // 8 rows x 32 B tile the 64 banks exactly) and rows 8..15 of a 16-row group
                                   // additionally swap their 16-byte chunk pairs (kv_flip) so that the 128-bit
                                   // reads of 16 rows x one chunk hit 16 different bank groups.  Every LDS
                                   // read address is then lane base + compile-time offset.
constexpr int PE_ROW = DPE * 2;    // rope rows share a DMA (8 rows per KB): XOR-swizzled instead
constexpr int KV_TILE = BN * KV_ROW;   // 33 KB
constexpr int PE_TILE = BN * PE_ROW;   // 4 KB
constexpr int STAGE = KV_TILE + PE_TILE;

__device__ __forceinline__ int kv_flip(int row) { return (row >> 3) & 1; }
__device__ __forceinline__ int swz_pe(int row) { return (row >> 1) & 7; }

__device__ __forceinline__ float xlane(float x, int mask) { return __shfl_xor(x, mask, 64); }
}  // namespace

template <typename T>
__global__ __launch_bounds__(64 * NW, 2) void mla_split_kernel(const MlaArgs a) {
  using E = Elem<T>;
  using x8 = typename E::x8;
  using x4 = typename E::x4;
  constexpr int KS = D / 32, KSPE = DPE / 32, DB = D / 16, NB = BN / 16;

  extern __shared__ __align__(16) char smem[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(MA_LDS char*)smem;

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, q = lane >> 4;
  const int hblk = blockIdx.x % a.head_blocks, bs = blockIdx.x / a.head_blocks;
  const int b = bs / a.num_split, split = bs % a.num_split;
  const int head = hblk * HB + wave * 16 + r;
  const int head_ld = min(head, a.Hq - 1);

  const int n_begin = split * a.split_len;
  const int n_end = min(n_begin + a.split_len, a.Skv);
  const int n_tiles = n_end > n_begin ? (n_end - n_begin + BN - 1) / BN : 0;

  // ---- Q fragments: B operand of S^T = KV Q^T
  x8 qf[KS + KSPE];
  {
    const T* qp = (const T*)a.q + (int64_t)b * a.qsb + (int64_t)head_ld * a.qsh + 8 * q;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) qf[ks] = *(const x8*)(qp + 32 * ks);
    const T* qpe = (const T*)a.q_pe + (int64_t)b * a.qpsb + (int64_t)head_ld * a.qpsh + 8 * q;
#pragma unroll
    for (int ks = 0; ks < KSPE; ks++) qf[KS + ks] = *(const x8*)(qpe + 32 * ks);
  }

  const char* kvb = (const char*)a.kv + (int64_t)b * a.kvsb * 2;
  const char* peb = (const char*)a.k_pe + (int64_t)b * a.kpsb * 2;
  const int64_t kv_row_bytes = a.kvss * 2, pe_row_bytes = a.kpss * 2;

  // ---- DMA.  Wave w streams latent rows 4w..4w+3 of a sub-tile, one instruction per row (64 lanes x 16 B =
  //      the 1 KB row; lane i fetches the chunk that belongs at physical chunk i); waves 0..3 also fetch 8
  //      rope rows each with one more instruction.  Rows beyond the cache are clamped to its last row
  //      (their scores are masked).  NDMA is the wave's instruction count per sub-tile.
  const int NDMA = wave < 4 ? 5 : 4;
  const uint32_t lane_off = (uint32_t)(lane ^ ((wave >> 1) & 1)) << 4;   // kv_flip(4w + i) = (w >> 1) & 1
  auto issue_tile = [&](int jt) {
    const uint32_t sb = lds0 + (jt & (NSTAGE - 1)) * STAGE;
    const int n0 = n_begin + jt * BN;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int row = wave * 4 + i;
      const int nrow = min(n0 + row, a.Skv - 1);
      dma16_so(kvb + nrow * kv_row_bytes, lane_off, sb + row * KV_ROW);
    }
    if (wave < 4) {
      const int row = wave * 8 + (lane >> 3);
      const int nrow = min(n0 + row, a.Skv - 1);
      dma16(peb + nrow * pe_row_bytes + (((lane & 7) ^ swz_pe(row)) << 4), sb + KV_TILE + wave * 8 * PE_ROW);
    }
  };

  // ---- per-lane LDS read offsets within a stage
  // K side (A operand): row 16nb + r, logical 16-byte chunk 4ks + q
  const uint32_t k_row_off = r * KV_ROW + (q ^ kv_flip(r)) * 16;
  const uint32_t pe_row_off = KV_TILE + r * PE_ROW;
  const int pe_chunk0 = q ^ swz_pe(r);
  // V side (transposing read): lane block q reads rows 4q + jr (and + 16), columns 16db + 4(l%4)..+3
  const int jr = r >> 2;
  const uint32_t v_row_off = (4 * q + jr) * KV_ROW + ((((lane & 3) >> 1) ^ kv_flip(4 * q + jr)) << 4) + (lane & 1) * 8;

  f32x4 o[DB];
#pragma unroll
  for (int i = 0; i < DB; i++) o[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  const float c_scale = a.scale * kLog2e;
  float row_max = -1e30f, row_sum = 0.f;

  if (n_tiles > 0) issue_tile(0);
  if (n_tiles > 1) issue_tile(1);
  if (n_tiles > 2) issue_tile(2);

  for (int jt = 0; jt < n_tiles; jt++) {
    // Sub-tile jt has landed for every wave (a wave's loads complete in order: only those of the up to two
    // later sub-tiles may still be in flight) and every wave is done with sub-tile jt-1, whose stage
    // takes sub-tile jt+3.
    if (jt + 2 < n_tiles) {
      if (wave < 4) __builtin_amdgcn_s_waitcnt(0x0F70 | 10); else __builtin_amdgcn_s_waitcnt(0x0F70 | 8);
    } else if (jt + 1 < n_tiles) {
      if (wave < 4) __builtin_amdgcn_s_waitcnt(0x0F70 | 5); else __builtin_amdgcn_s_waitcnt(0x0F70 | 4);
    } else {
      wait_dma();
    }
    __syncthreads();
    if (jt + 3 < n_tiles) issue_tile(jt + 3);
    const int n0 = n_begin + jt * BN;
    uint32_t base = lds0 + (jt & (NSTAGE - 1)) * STAGE;

    // ---- S^T = KV Q^T + K_pe Q_pe^T : lane holds head r, kv rows 16nb + 4q + j
    f32x4 s[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) s[nb] = f32x4{0.f, 0.f, 0.f, 0.f};
    {
      // fragments are requested AH slices ahead of the MFMAs that consume them
      constexpr int AH = 2, RING = AH + 1, NSL = KS + KSPE;
      x8 kf[RING][NB];
      uint32_t kb = base + k_row_off, pb = base + pe_row_off;
      asm volatile("" : "+v"(kb), "+v"(pb));   // one address register + immediates for every read below
      auto request = [&](int ks) {
        if (ks < KS) {
#pragma unroll
          for (int nb = 0; nb < NB; nb++) kf[ks % RING][nb] = lds_read<x8>(kb + nb * 16 * KV_ROW + ks * 64);
        } else {
          const uint32_t coff = (uint32_t)((pe_chunk0 ^ (4 * (ks - KS))) << 4);
#pragma unroll
          for (int nb = 0; nb < NB; nb++) kf[ks % RING][nb] = lds_read<x8>(pb + nb * 16 * PE_ROW + coff);
        }
      };
#pragma unroll
      for (int ks = 0; ks < AH; ks++) request(ks);
#pragma unroll
      for (int ks = 0; ks < NSL; ks++) {
        if (ks + AH < NSL) request(ks + AH);
        __builtin_amdgcn_sched_barrier(0);   // keep the requests ahead of the MFMAs that hide their latency
#pragma unroll
        for (int nb = 0; nb < NB; nb++) s[nb] = E::mfma16(kf[ks % RING][nb], qf[ks], s[nb]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }

    if (n0 + BN > n_end) {
#pragma unroll
      for (int nb = 0; nb < NB; nb++)
#pragma unroll
        for (int j = 0; j < 4; j++)
          if (n0 + 16 * nb + 4 * q + j >= n_end) s[nb][j] = -INFINITY;
    }

    // ---- online softmax in the log2 domain (the 4 lanes l%16 == r own one head)
    float mx = s[0][0];
#pragma unroll
    for (int nb = 0; nb < NB; nb++)
#pragma unroll
      for (int j = 0; j < 4; j++) mx = fmaxf(mx, s[nb][j]);
    mx = fmaxf(mx, xlane(mx, 16));
    mx = fmaxf(mx, xlane(mx, 32));
    // The running max is only moved when some head's max grew by more than 2^8: until then the
    // probabilities are taken relative to the stale max (at most 256, exact in fp32 / bf16 range) and the
    // 128 accumulator registers need no rescaling.  The final normalisation by row_sum absorbs the offset.
    const float cand = fmaxf(row_max, mx * c_scale);
    const bool move = cand - row_max > 8.f;   // per head: heads that stay multiply by exactly 1
    if (__any(move)) {
      const float corr = move ? fast_exp2(row_max - cand) : 1.f;
      row_max = move ? cand : row_max;
      row_sum *= corr;
#pragma unroll
      for (int i = 0; i < DB; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) asm volatile("v_mul_f32 %0, %0, %1" : "+v"(o[i][j]) : "v"(corr));
    }
    float part = 0.f;
#pragma unroll
    for (int nb = 0; nb < NB; nb++)
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const float p = fast_exp2(s[nb][j] * c_scale - row_max);
        s[nb][j] = p;
        part += p;
      }
    row_sum += part;

    // ---- O^T += KV^T P^T ; lane block q, k slot i is kv row 16(i/4) + 4q + i%4 on both operands
    {
      x8 pf;
#pragma unroll
      for (int i = 0; i < 4; i++) {
        pf[i] = (T)s[0][i];
        pf[4 + i] = (T)s[1][i];
      }
      uint32_t rb = base + v_row_off;
      asm volatile("" : "+v"(rb));
      constexpr int PF = 4;   // V fragments in flight
      x4 lo[PF], hi[PF];
#pragma unroll
      for (int i = 0; i < PF - 1; i++) {
        lo[i] = lds_read_tr4<T>(rb + i * 32);
        hi[i] = lds_read_tr4<T>(rb + 16 * KV_ROW + i * 32);
      }
#pragma unroll
      for (int db = 0; db < DB; db++) {
        if (db + PF - 1 < DB) {
          lo[(db + PF - 1) % PF] = lds_read_tr4<T>(rb + (db + PF - 1) * 32);
          hi[(db + PF - 1) % PF] = lds_read_tr4<T>(rb + 16 * KV_ROW + (db + PF - 1) * 32);
        }
        __builtin_amdgcn_sched_barrier(0);
        x8 vf = __builtin_shufflevector(lo[db % PF], hi[db % PF], 0, 1, 2, 3, 4, 5, 6, 7);
        o[db] = E::mfma16(vf, pf, o[db]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }

  // ---- epilogue: lane holds head r, output columns 16db + 4q + j
  float tot = row_sum + xlane(row_sum, 16);
  tot += xlane(tot, 32);
  const bool empty = n_tiles == 0;
  const float inv = empty ? 0.f : 1.f / tot;
  const float lse2 = empty ? -INFINITY : row_max + fast_log2(tot);   // log2 domain
  if (head < a.Hq) {
    if (a.num_split == 1) {
      T* op = (T*)a.o + (int64_t)b * a.osb + (int64_t)head * a.osh + 4 * q;
#pragma unroll
      for (int db = 0; db < DB; db++) {
        x4 w;
#pragma unroll
        for (int i = 0; i < 4; i++) w[i] = (T)(o[db][i] * inv);
        *(x4*)(op + 16 * db) = w;
      }
      if (a.lse && q == 0) a.lse[(int64_t)b * a.Hq + head] = lse2 * kLn2;
    } else {
      T* op = (T*)a.o_part + (((int64_t)b * a.num_split + split) * a.Hq + head) * D + 4 * q;
#pragma unroll
      for (int db = 0; db < DB; db++) {
        x4 w;
#pragma unroll
        for (int i = 0; i < 4; i++) w[i] = (T)(o[db][i] * inv);
        *(x4*)(op + 16 * db) = w;
      }
      if (q == 0) a.lse_part[((int64_t)b * a.num_split + split) * a.Hq + head] = lse2;
    }
  }
}

// Four (batch, head) pairs per workgroup: 64 threads x 8 output columns each.
template <typename T>
__global__ __launch_bounds__(256) void mla_combine_kernel(const MlaArgs a) {
  using x8 = typename Elem<T>::x8;
  const int tid = threadIdx.x & 63;
  const int64_t bh = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (bh >= (int64_t)a.B * a.Hq) return;
  const int b = (int)(bh / a.Hq), head = (int)(bh % a.Hq);
  const int ns = a.num_split;
  // lane s of the wave holds the log-sum-exp of split s (at most 64 splits): one load, wave reductions
  const float* lp = a.lse_part + (int64_t)b * ns * a.Hq + head;
  const float my = tid < ns ? lp[(int64_t)tid * a.Hq] : -INFINITY;
  float mx = my;
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) mx = fmaxf(mx, __shfl_xor(mx, m, 64));
  const float e = tid < ns ? fast_exp2(my - mx) : 0.f;
  float sum = e;
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) sum += __shfl_xor(sum, m, 64);
  const float wgt = e / sum;
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const T* pp = (const T*)a.o_part + ((int64_t)b * ns * a.Hq + head) * D + tid * 8;
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
  if (a.lse && tid == 0) a.lse[(int64_t)b * a.Hq + head] = (mx + fast_log2(sum)) * kLn2;
}

template <typename T>
static int launch_t(const MlaArgs& a, hipStream_t stream) {
  constexpr size_t lds = NSTAGE * (size_t)STAGE;
  auto kern = mla_split_kernel<T>;
  static bool attr_set = false;
  if (!attr_set) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) return -1;
    attr_set = true;
  }
  MlaArgs args = a;
  args.head_blocks = (a.Hq + HB - 1) / HB;
  const unsigned grid = (unsigned)(a.B * a.num_split * args.head_blocks);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * NW), lds, stream, args);
  if (hipGetLastError() != hipSuccess) return -1;
  if (a.num_split > 1) {
    hipLaunchKernelGGL(mla_combine_kernel<T>, dim3((unsigned)(((int64_t)a.B * a.Hq + 3) / 4)), dim3(256), 0, stream, a);
    if (hipGetLastError() != hipSuccess) return -1;
  }
  return 0;
}

int mla_decode_dispatch(const MlaArgs& a, bool is_bf16, int dim, int dim_pe, hipStream_t stream) {
  if (dim != D || dim_pe != DPE) return -2;
  return is_bf16 ? launch_t<__bf16>(a, stream) : launch_t<_Float16>(a, stream);
}

}  // namespace ma
