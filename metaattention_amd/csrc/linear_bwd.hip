// Chunked linear / stateful attention backward (RetNet retention, Mamba2 SSD, gated retention) for gfx950.
//
// Replaces LinearAttention.backward of attention_engine/core/template/tl_template/linear/linear_tl.py:1268-1340
// (chunk_bwd_kernel_dh :461, chunk_bwd_dqkg :606, chunk_bwd_kernel_dv :876, compute_final_dg :64-76).  The reference
// materialises the forward state h and its gradient dh per chunk in HBM (bf16) and then visits the chunks in parallel.
// Here no state ever leaves the chip.  With
//   A_ts = q_scale (q_t . k_s) exp(G_t - G_s) [s <= t],   u = v * v_scale,   o = A u,   G = cumsum(log_decay)
// the three gradients
//   dq_t = q_scale sum_{s<=t} exp(G_t - G_s) (do_t . u_s) k_s
//   du_s = sum_{t>=s} A_ts do_t
//   dk_s = q_scale sum_{t>=s} exp(G_t - G_s) (do_t . u_s) q_t
// are the forward operator LA(q, k, v) itself on permuted operands, the two sums over LATER tokens on the time-reversed
// sequence with the log decay shifted by one token:
//   dq = LA(do, v, k; v_scale)      du = R LA(R k, R q, R do)      dk = v_scale * R LA(R v, R do, R q)      (R reverses time)
// so the backward pass is three scans of the forward kernel (linear_fwd.hip: state in accumulator registers, fp32
// outputs), each contraction cut into the 128 / 256 wide pieces that kernel takes (their fp32 outputs add up); the scans
// read their operands in place (reversed time, column slices, shared heads and the zero padding of a narrow piece are
// the scan kernel's general operand addressing).  Plus the small kernels of this file:
// the shifted reversed log decay, and the epilogue that forms dv, dv_scale, the per-token decay gradient
//   dG_t = q_t . dq_t - k_t . dk_t        (fp32 products of the fp32 scan outputs)
// sums the heads that share a q / k head (:1300-1303), converts, and turns dG into dlog_decay by a reversed running sum
// in fp32 (compute_final_dg).
#include "linear_bwd.h"

#include "linear_fwd.h"

namespace ma {

namespace {

// g_rev[b, h, t'] = log_decay[b, h, T - t'] for t' >= 1, 0 for t' = 0: the decay between reversed tokens t' - 1 and t'
__global__ __launch_bounds__(256) void shift_rev_kernel(float* __restrict__ dst, const float* __restrict__ src, int T, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const int t = (int)(i % T);
  dst[i] = t >= 1 ? src[i - t + (T - t)] : 0.f;
}

// sum over the LPT lanes (a power of two) that share a token
template <int LPT>
__device__ __forceinline__ float lanes_sum(float x) {
#pragma unroll
  for (int off = LPT / 2; off >= 1; off >>= 1) x += __shfl_xor(x, off, 64);
  return x;
}

// LPT lanes per (batch, head, token), four columns per lane and round.  dqh [B,H,T,Dk] fp32 (time order), dkh_rev [B,H,T,Dk]
// and du_rev [B,H,T,Dv] fp32 (reversed time order, dk before its v_scale factor).  Writes dG, dv, dv_scale and, where every
// head has its own q / k head, dq / dk.  du_rev null: dv has been written by the scan itself (no v_scale: dv = du).
// With np > 1 the scan outputs dqh and dkh_rev are np pieces (partial sums over slices of the contraction), piece_stride
// floats apart, which are added up here.
template <int LPT>
__global__ __launch_bounds__(256) void grads_kernel(LinBwdArgs a, const float* __restrict__ dqh, const float* __restrict__ dkh_rev,
                                                   const float* __restrict__ du_rev, float* __restrict__ dG, int np, int64_t piece_stride) {
  const int sub = threadIdx.x % LPT;
  const int64_t tok = ((int64_t)blockIdx.x * 256 + threadIdx.x) / LPT;
  const bool live = tok < (int64_t)a.B * a.H * a.T;   // (dead lanes take part in the shuffles with zeros)
  const int64_t tk = live ? tok : 0;
  const int t = (int)(tk % a.T);
  const int64_t bh = tk / a.T;
  const int h = (int)(bh % a.H);
  const int64_t b = bh / a.H;
  const int64_t rtok = bh * a.T + (a.T - 1 - t);
  const float vs = a.v_scale ? a.v_scale[tk] : 1.f;
  const int hq = h / (a.H / a.Hq), hk = h / (a.H / a.Hk);
  const __bf16* qrow = (const __bf16*)a.q + ((b * a.Hq + hq) * a.T + t) * (int64_t)a.Dk;
  const __bf16* krow = (const __bf16*)a.k + ((b * a.Hk + hk) * a.T + t) * (int64_t)a.Dk;
  float acc = 0.f, acc_vs = 0.f;
  if (live) {
    for (int c = 4 * sub; c < a.Dk; c += 4 * LPT) {
      f32x4 gq = *(const f32x4*)(dqh + tk * a.Dk + c);
      f32x4 gk = *(const f32x4*)(dkh_rev + rtok * a.Dk + c);
      for (int p = 1; p < np; p++) {
        gq += *(const f32x4*)(dqh + p * piece_stride + tk * a.Dk + c);
        gk += *(const f32x4*)(dkh_rev + p * piece_stride + rtok * a.Dk + c);
      }
      const bf16x4 qv = *(const bf16x4*)(qrow + c), kv = *(const bf16x4*)(krow + c);
#pragma unroll
      for (int i = 0; i < 4; i++) {
        gk[i] *= vs;
        acc += (float)qv[i] * gq[i] - (float)kv[i] * gk[i];
      }
      if (a.Hq == a.H) {
        bf16x4 w;
#pragma unroll
        for (int i = 0; i < 4; i++) w[i] = (__bf16)gq[i];
        *(bf16x4*)((__bf16*)a.dq + tk * a.Dk + c) = w;
      }
      if (a.Hk == a.H) {
        bf16x4 w;
#pragma unroll
        for (int i = 0; i < 4; i++) w[i] = (__bf16)gk[i];
        *(bf16x4*)((__bf16*)a.dk + tk * a.Dk + c) = w;
      }
    }
    for (int c = 4 * sub; du_rev && c < a.Dv; c += 4 * LPT) {
      const f32x4 gu = *(const f32x4*)(du_rev + rtok * a.Dv + c);
      const bf16x4 vv = *(const bf16x4*)((const __bf16*)a.v + tk * a.Dv + c);
      bf16x4 w;
#pragma unroll
      for (int i = 0; i < 4; i++) {
        acc_vs += (float)vv[i] * gu[i];
        w[i] = (__bf16)(gu[i] * vs);
      }
      *(bf16x4*)((__bf16*)a.dv + tk * a.Dv + c) = w;
    }
  }
  acc = lanes_sum<LPT>(acc);
  acc_vs = lanes_sum<LPT>(acc_vs);
  if (live && sub == 0) {
    dG[tk] = acc;
    if (a.dv_scale) a.dv_scale[tk] = acc_vs;
  }
}

// The same for heads that share their q and k heads in groups of G = H / Hq (Hq == Hk < H): LPT lanes per (batch, shared
// head, token) walk the G heads of the group, so that dq and dk of the shared head -- the sums over the group
// (linear_tl.py:1300-1303) -- are formed while the per-head scan outputs pass through once.
// DKB: the dk scan has left its per-head output as bf16 in time order (dkh_rev then points at [B,H,T,Dk] bf16; the
// reference rounds its per-head dk to the tensor dtype before the group sum as well), and the k . dk term of the decay
// gradient comes from the du scan instead, in fp32: k_s . dk_s = sum_{t>=s} A_ts (do_t . u_s) = u_s . du_s = v_scale_s (v_s . du_s).
template <int LPT, bool DKB = false>
__global__ __launch_bounds__(256) void grads_shared_kernel(LinBwdArgs a, const float* __restrict__ dqh, const float* __restrict__ dkh_rev,
                                                          const float* __restrict__ du_rev, float* __restrict__ dG, int np, int64_t piece_stride) {
  const int sub = threadIdx.x % LPT;
  const int64_t tok = ((int64_t)blockIdx.x * 256 + threadIdx.x) / LPT;
  const bool live = tok < (int64_t)a.B * a.Hq * a.T;   // (dead lanes take part in the shuffles with zeros)
  const int64_t tg = live ? tok : 0;
  const int t = (int)(tg % a.T);
  const int64_t bg = tg / a.T;
  const int g = (int)(bg % a.Hq), G = a.H / a.Hq;
  const int64_t b = bg / a.Hq;
  const int c = 4 * sub;                               // (4 LPT >= Dk: one group of four key columns per lane)
  const bool has_c = live && c < a.Dk;
  f32x4 qv = {0.f, 0.f, 0.f, 0.f}, kv = {0.f, 0.f, 0.f, 0.f}, sq = {0.f, 0.f, 0.f, 0.f}, sk = {0.f, 0.f, 0.f, 0.f};
  if (has_c) {
    const bf16x4 q4 = *(const bf16x4*)((const __bf16*)a.q + tg * a.Dk + c), k4 = *(const bf16x4*)((const __bf16*)a.k + tg * a.Dk + c);
#pragma unroll
    for (int i = 0; i < 4; i++) { qv[i] = (float)q4[i]; kv[i] = (float)k4[i]; }
  }
  // What head j + 1 needs is requested before head j is worked on (the compiler cannot move a load above the stores
  // of the head before, which it must assume to alias).
  struct Row { f32x4 gq, gk, gu; bf16x4 vv; float vs; };
  const int cv0 = 4 * sub;
  const bool has_v = live && du_rev && cv0 < a.Dv;
  auto load_row = [&](int j) {
    Row r{};
    const int64_t bh = b * a.H + (int64_t)g * G + j, tk = bh * a.T + t, rtok = bh * a.T + (a.T - 1 - t);
    r.vs = a.v_scale ? a.v_scale[tk] : 1.f;
    if (has_c) {
      r.gq = *(const f32x4*)(dqh + tk * a.Dk + c);
      if constexpr (DKB) {
        const bf16x4 g4 = *(const bf16x4*)((const __bf16*)dkh_rev + tk * a.Dk + c);
#pragma unroll
        for (int i = 0; i < 4; i++) r.gk[i] = (float)g4[i];
      } else {
        r.gk = *(const f32x4*)(dkh_rev + rtok * a.Dk + c);
      }
    }
    if (has_v) {
      r.gu = *(const f32x4*)(du_rev + rtok * a.Dv + cv0);
      r.vv = *(const bf16x4*)((const __bf16*)a.v + tk * a.Dv + cv0);
    }
    return r;
  };
  constexpr int PF = 3;   // heads ahead
  Row ring[PF];
#pragma unroll
  for (int i = 0; i < PF; i++) ring[i] = i < G ? load_row(i) : Row{};
  for (int j = 0; j < G; j++) {
    const int64_t bh = b * a.H + (int64_t)g * G + j, tk = bh * a.T + t, rtok = bh * a.T + (a.T - 1 - t);
    const Row row = ring[0];
#pragma unroll
    for (int i = 0; i + 1 < PF; i++) ring[i] = ring[i + 1];
    if (j + PF < G) ring[PF - 1] = load_row(j + PF);
    const float vs = row.vs;
    float acc = 0.f, acc_vs = 0.f;
    if (has_c) {
      f32x4 gq = row.gq, gk = row.gk;
      for (int p = 1; p < np; p++) {
        gq += *(const f32x4*)(dqh + p * piece_stride + tk * a.Dk + c);
        if constexpr (!DKB) gk += *(const f32x4*)(dkh_rev + p * piece_stride + rtok * a.Dk + c);
      }
#pragma unroll
      for (int i = 0; i < 4; i++) {
        gk[i] *= vs;
        acc += DKB ? qv[i] * gq[i] : qv[i] * gq[i] - kv[i] * gk[i];
        sq[i] += gq[i];
        sk[i] += gk[i];
      }
    }
    if (has_v) {
      for (int cv = cv0; cv < a.Dv; cv += 4 * LPT) {
        const f32x4 gu = cv == cv0 ? row.gu : *(const f32x4*)(du_rev + rtok * a.Dv + cv);
        const bf16x4 vv = cv == cv0 ? row.vv : *(const bf16x4*)((const __bf16*)a.v + tk * a.Dv + cv);
        bf16x4 w;
#pragma unroll
        for (int i = 0; i < 4; i++) {
          acc_vs += (float)vv[i] * gu[i];
          w[i] = (__bf16)(gu[i] * vs);
        }
        *(bf16x4*)((__bf16*)a.dv + tk * a.Dv + cv) = w;
      }
    }
    acc = lanes_sum<LPT>(acc);
    acc_vs = lanes_sum<LPT>(acc_vs);
    if (live && sub == 0) {
      dG[tk] = DKB ? acc - vs * acc_vs : acc;
      if (a.dv_scale) a.dv_scale[tk] = acc_vs;
    }
  }
  if (has_c) {
    bf16x4 wq, wk;
#pragma unroll
    for (int i = 0; i < 4; i++) { wq[i] = (__bf16)sq[i]; wk[i] = (__bf16)sk[i]; }
    *(bf16x4*)((__bf16*)a.dq + tg * a.Dk + c) = wq;
    *(bf16x4*)((__bf16*)a.dk + tg * a.Dk + c) = wk;
  }
}

// dst [B, Hg, T, D] bf16 = sum over the G = H / Hg heads of a group of src [B, H, T, D] fp32 (row T - 1 - t when rev),
// each times scale[b, h, t] when scale is given.  One thread per 4 columns.
// (np pieces of src, piece_stride floats apart, are added up as well)
__global__ __launch_bounds__(256) void group_sum_kernel(__bf16* __restrict__ dst, const float* __restrict__ src, const float* __restrict__ scale,
                                                       int H, int Hg, int T, int D, int rev, int64_t n4, int np, int64_t piece_stride) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n4) return;
  const int cpr = D / 4;
  const int c = 4 * (int)(i % cpr);
  const int64_t row = i / cpr;
  const int t = (int)(row % T);
  const int64_t bg = row / T;
  const int g = (int)(bg % Hg);
  const int64_t b = bg / Hg;
  const int G = H / Hg, ts = rev ? T - 1 - t : t;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int j = 0; j < G; j++) {
    const int64_t bh = b * H + g * G + j;
    f32x4 x = *(const f32x4*)(src + (bh * T + ts) * (int64_t)D + c);
    for (int p = 1; p < np; p++) x += *(const f32x4*)(src + p * piece_stride + (bh * T + ts) * (int64_t)D + c);
    const float s = scale ? scale[bh * T + t] : 1.f;
#pragma unroll
    for (int k = 0; k < 4; k++) acc[k] += x[k] * s;
  }
  bf16x4 w;
#pragma unroll
  for (int k = 0; k < 4; k++) w[k] = (__bf16)acc[k];
  *(bf16x4*)(dst + row * D + c) = w;
}

// dlog_decay[b, h, t] = sum_{t' >= t} dG[b, h, t']: one workgroup of 256 threads per (batch, head), blocks of 2048 tokens from
// the end, eight consecutive tokens per thread (its own running sum), the threads' totals scanned through the wave and LDS
__global__ __launch_bounds__(256) void suffix_sum_kernel(float* __restrict__ dst, const float* __restrict__ dG, int T) {
  __shared__ float wave_total[4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const float* src = dG + (int64_t)blockIdx.x * T;
  float* out = dst + (int64_t)blockIdx.x * T;
  float carry = 0.f;   // sum of everything behind the block
  for (int t0 = (T - 1) / 2048 * 2048; t0 >= 0; t0 -= 2048) {
    const int t = t0 + 8 * tid;
    float x[8];
#pragma unroll
    for (int i = 0; i < 8; i++) x[i] = t + i < T ? src[t + i] : 0.f;
#pragma unroll
    for (int i = 6; i >= 0; i--) x[i] += x[i + 1];   // x[i] = sum of this thread's tokens i..7
    // sum of the totals of the later lanes of the wave, then of the later waves
    float incl = x[0];
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const float y = __shfl_down(incl, off, 64);
      if (lane + off < 64) incl += y;
    }
    if (lane == 0) wave_total[wave] = incl;
    __syncthreads();
    float behind = carry + (incl - x[0]);
    float block_total = 0.f;
#pragma unroll
    for (int w = 3; w >= 0; w--) {
      if (w > wave) behind += wave_total[w];
      block_total += wave_total[w];
    }
#pragma unroll
    for (int i = 0; i < 8; i++)
      if (t + i < T) out[t + i] = x[i] + behind;
    carry += block_total;
    __syncthreads();
  }
}

inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

// the widths the scan kernel contracts over: pieces of 256 columns, a remainder (or a narrow operand) as 128 or 256
struct Slices {
  int n = 0, c0[16], w[16];
  explicit Slices(int width) {
    for (int c = 0; c < width && n < 16;) {
      const int rest = width - c;
      w[n] = rest > 128 ? 256 : 128;
      c0[n] = c;
      c += w[n];
      n++;
    }
  }
};

}  // namespace

int linear_bwd_run(const LinBwdArgs& a, void* ws, size_t ws_bytes, hipStream_t stream, size_t* query) {
  if ((a.Dk != 64 && a.Dk != 128 && a.Dk != 192 && a.Dk != 256) || a.Dv % 64 != 0 || a.Dv > 16 * 256) return -2;
  // (a key width of 64 or 192 is contracted in the 128- / 256-wide scan kernel: the missing columns are zeros that are never loaded)
  const int DKP = a.Dk <= 128 ? 128 : 256, dk_cols = a.Dk == DKP ? 0 : a.Dk;
  const int64_t BHT = (int64_t)a.B * a.H * a.T;
  const Slices sl(a.Dv);   // contraction of the dq and dk scans

  // workspace: fp32 scan outputs, dG, reversed log decay, the scan kernel's own workspace
  size_t off = 0;
  auto take = [&](size_t bytes) { const size_t o = off; off += align256(bytes); return o; };
  // (a contraction of equal pieces that are all read in place runs its pieces side by side, each with an output of its own)
  const bool side_by_side = sl.n > 1 && a.Dv % sl.w[0] == 0 && sl.w[sl.n - 1] == sl.w[0];
  const int np = side_by_side ? sl.n : 1;
  const int64_t piece_stride = BHT * a.Dk;
  const size_t o_dqh = take((size_t)np * BHT * a.Dk * 4), o_dkh = take((size_t)np * BHT * a.Dk * 4), o_du = take((size_t)BHT * a.Dv * 4);
  const size_t o_dG = take((size_t)BHT * 4), o_grev = take((size_t)BHT * 4);
  // the scan kernel's workspace (sequence segments): the largest any of the scans asks for
  size_t scan_ws = 0;
  {
    LinArgs la{};
    la.B = a.B; la.H = a.H; la.T = a.T;
    size_t need = 0;
    la.Hq = la.Hk = a.H; la.Dv = a.Dk;
    for (int s = 0; s < sl.n; s++)
      if (linear_fwd_dispatch(la, sl.w[s], 0, nullptr, 0, nullptr, &need) == 0 && need > scan_ws) scan_ws = need;
    la.Hq = a.Hk; la.Hk = a.Hq; la.Dv = a.Dv;
    la.qk_cols = dk_cols;
    if (dk_cols) la.q_row = la.k_row = a.Dk;
    if (linear_fwd_dispatch(la, DKP, 0, nullptr, 0, nullptr, &need) == 0 && need > scan_ws) scan_ws = need;
  }
  const size_t o_scan = take(scan_ws);
  if (query) { *query = off; return 0; }
  if (!ws || ws_bytes < off || ((uintptr_t)ws & 255) != 0) return -3;
  char* base = (char*)ws;
  float *dqh = (float*)(base + o_dqh), *dkh = (float*)(base + o_dkh), *du = (float*)(base + o_du), *dG = (float*)(base + o_dG), *grev = (float*)(base + o_grev);
  void* scan = scan_ws ? base + o_scan : nullptr;
  // an operand of a scan as the scan kernel reads it in place: heads, elements between its tokens (the pointer carries a
  // column offset)
  struct Operand { const void* p; int heads; int64_t row; };
  // (out_bf16: the output goes out as bf16 in the operands' own time order instead of fp32 in scan order)
  auto scan_launch = [&](Operand q, Operand k, Operand v, bool reversed, int dk, int dv, const float* g, const float* vs, void* out,
                         bool accumulate, int pieces = 1, int qk_cols = 0, bool out_bf16 = false) -> int {
    LinArgs la{};
    la.q = q.p; la.k = k.p; la.v = v.p; la.o = out; la.log_decay = g; la.v_scale = vs; la.q_scale = a.q_scale;
    la.B = a.B; la.H = a.H; la.Hq = q.heads; la.Hk = k.heads; la.Hv = v.heads; la.T = a.T; la.Dv = dv;
    la.q_row = q.row; la.k_row = k.row; la.v_row = v.row; la.rev = reversed ? 1 : 0;
    la.out_f32 = out_bf16 ? 0 : (accumulate ? 2 : 1);
    la.rev_o = out_bf16 && reversed ? 1 : 0;
    if (pieces > 1) { la.n_pieces = pieces; la.piece_qk = dk; la.piece_o = piece_stride; }
    la.qk_cols = qk_cols;
    return linear_fwd_dispatch(la, dk, 0, scan, scan_ws, stream, nullptr);
  };
  const __bf16 *q_p = (const __bf16*)a.q, *k_p = (const __bf16*)a.k, *v_p = (const __bf16*)a.v, *do_p = (const __bf16*)a.dout;
  // the columns of piece s that exist (a last piece may reach beyond the value columns: the scan kernel pads with zeros)
  auto piece_cols = [&](int s) { return sl.c0[s] + sl.w[s] <= a.Dv ? 0 : a.Dv - sl.c0[s]; };

  hipLaunchKernelGGL(shift_rev_kernel, dim3((unsigned)((BHT + 255) / 256)), dim3(256), 0, stream, grev, a.log_decay, a.T, BHT);

  // dq (per head) = LA(do, v, k; v_scale), contraction over the value columns; k is read with its own heads
  if (side_by_side) {
    if (const int rc = scan_launch(Operand{do_p, a.H, a.Dv}, Operand{v_p, a.H, a.Dv}, Operand{k_p, a.Hk, a.Dk}, false, sl.w[0], a.Dk, a.log_decay, a.v_scale,
                                   dqh, false, np))
      return rc;
  }
  for (int s = 0; s < sl.n && !side_by_side; s++) {
    Operand qs{do_p + sl.c0[s], a.H, a.Dv}, ks{v_p + sl.c0[s], a.H, a.Dv};
    if (const int rc = scan_launch(qs, ks, Operand{k_p, a.Hk, a.Dk}, false, sl.w[s], a.Dk, a.log_decay, a.v_scale, dqh, s > 0, 1, piece_cols(s))) return rc;
  }

  // du (reversed) = LA(R k, R q, R do), contraction over the key columns: the operands are read in reversed time in place.
  // Without a v_scale dv is du itself, and the scan writes it: bf16, rows back in time order.
  const bool direct_dv = !a.v_scale && !a.dv_scale;
  if (const int rc = scan_launch(Operand{k_p, a.Hk, a.Dk}, Operand{q_p, a.Hq, a.Dk}, Operand{do_p, a.H, a.Dv}, true, DKP, a.Dv, grev, nullptr,
                                 direct_dv ? a.dv : (void*)du, false, 1, dk_cols, direct_dv))
    return rc;
  if (direct_dv) du = nullptr;

  // dk (per head, reversed, before its v_scale factor) = LA(R v, R do, R q), contraction over the value columns.
  // Heads in groups that share q and k, with a v_scale and a contraction of one piece (Mamba2): the scan leaves bf16 in
  // time order (see grads_shared_kernel).
  const bool dk_bf16 = a.Hq == a.Hk && a.Hq != a.H && du && sl.n == 1;
  if (side_by_side) {
    if (const int rc = scan_launch(Operand{v_p, a.H, a.Dv}, Operand{do_p, a.H, a.Dv}, Operand{q_p, a.Hq, a.Dk}, true, sl.w[0], a.Dk, grev, nullptr, dkh, false, np))
      return rc;
  }
  for (int s = 0; s < sl.n && !side_by_side; s++) {
    Operand qs{v_p + sl.c0[s], a.H, a.Dv}, ks{do_p + sl.c0[s], a.H, a.Dv};
    if (const int rc = scan_launch(qs, ks, Operand{q_p, a.Hq, a.Dk}, true, sl.w[s], a.Dk, grev, nullptr, dkh, s > 0, 1, piece_cols(s), dk_bf16)) return rc;
  }

  if (a.Hq == a.Hk && a.Hq != a.H) {
    // heads in groups that share q and k: gradients, group sums and conversions in one pass over the scan outputs
    const int64_t n_tok = (int64_t)a.B * a.Hq * a.T;
    const dim3 grid64((unsigned)((n_tok + 3) / 4)), grid32((unsigned)((n_tok + 7) / 8));
    if (a.Dk > 128 && dk_bf16)
      hipLaunchKernelGGL((grads_shared_kernel<64, true>), grid64, dim3(256), 0, stream, a, (const float*)dqh, (const float*)dkh, (const float*)du, dG, np,
                         piece_stride);
    else if (a.Dk > 128)
      hipLaunchKernelGGL(grads_shared_kernel<64>, grid64, dim3(256), 0, stream, a, (const float*)dqh, (const float*)dkh, (const float*)du, dG, np, piece_stride);
    else if (dk_bf16)
      hipLaunchKernelGGL((grads_shared_kernel<32, true>), grid32, dim3(256), 0, stream, a, (const float*)dqh, (const float*)dkh, (const float*)du, dG, np,
                         piece_stride);
    else
      hipLaunchKernelGGL(grads_shared_kernel<32>, grid32, dim3(256), 0, stream, a, (const float*)dqh, (const float*)dkh, (const float*)du, dG, np, piece_stride);
    hipLaunchKernelGGL(suffix_sum_kernel, dim3((unsigned)(a.B * a.H)), dim3(256), 0, stream, a.dlog_decay, (const float*)dG, a.T);
    return launch_status();
  }
  if ((a.Dk > a.Dv ? a.Dk : a.Dv) >= 256)
    hipLaunchKernelGGL(grads_kernel<64>, dim3((unsigned)((BHT + 3) / 4)), dim3(256), 0, stream, a, (const float*)dqh, (const float*)dkh, (const float*)du, dG,
                       np, piece_stride);
  else
    hipLaunchKernelGGL(grads_kernel<32>, dim3((unsigned)((BHT + 7) / 8)), dim3(256), 0, stream, a, (const float*)dqh, (const float*)dkh, (const float*)du, dG,
                       np, piece_stride);
  if (a.Hq != a.H) {
    const int64_t n4 = (int64_t)a.B * a.Hq * a.T * (a.Dk / 4);
    hipLaunchKernelGGL(group_sum_kernel, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, stream, (__bf16*)a.dq, (const float*)dqh, (const float*)nullptr,
                       a.H, a.Hq, a.T, a.Dk, 0, n4, np, piece_stride);
  }
  if (a.Hk != a.H) {
    const int64_t n4 = (int64_t)a.B * a.Hk * a.T * (a.Dk / 4);
    hipLaunchKernelGGL(group_sum_kernel, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, stream, (__bf16*)a.dk, (const float*)dkh, a.v_scale, a.H, a.Hk,
                       a.T, a.Dk, 1, n4, np, piece_stride);
  }
  hipLaunchKernelGGL(suffix_sum_kernel, dim3((unsigned)(a.B * a.H)), dim3(256), 0, stream, a.dlog_decay, (const float*)dG, a.T);
  return launch_status();
}

}  // namespace ma
