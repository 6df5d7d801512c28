// Ceiling probes for the MFMA kernels of this library on gfx950.  Not part of the operator library: a separate small
// shared object that bench.py --probe loads to measure, on the box it runs on, what the instruction mix of the parallel
// attention forward can reach at best, and how fast a CU can stream global memory into LDS.
//
// probe 1 (ma_probe_attention_step): one workgroup of 8 waves per CU (two per SIMD), every wave owning 32 query rows,
// runs the per-step work of a flash-attention forward at head size 128 over a 32-key sub-tile in a loop with nothing
// else around it: 8 MFMAs of S^T = K Q^T and 8 of O^T += V^T P^T (v_mfma_f32_32x32x16_bf16), optionally the vector work of
// the 16 score elements a lane owns (scale, exponential, row sum, conversion to bf16), the 24 LDS fragment reads, one
// workgroup barrier per step, and the two direct-to-LDS load instructions per wave that fetch the next sub-tile (from an
// L2-resident window).  Operands are either constants or pseudo-random bf16 values of the spread real inputs have: the
// instruction stream is the same, the switching activity is not, and the chip's power management answers the latter
// with a lower clock.  The cycle counter of one wave and the wall time of the launch are both returned.
//
// probe 3 (ma_probe_issue_hold): how many cycles a direct-to-LDS load instruction holds the wave that issues it, by the number
// of waves of the CU issuing at the same time, the number of instructions per burst and where the data comes from.
//
// probe 2 (ma_probe_stream_to_lds): 8 waves per CU stream a window of global memory into LDS with direct-to-LDS loads,
// `depth` instructions (1 KB each) in flight per wave; the window is chosen to fit L2, the last-level cache, or neither.
#include "../common.h"

using namespace ma;

namespace {

enum { PROBE_VECTOR = 1, PROBE_LDS = 2, PROBE_BARRIER = 4, PROBE_DMA = 8, PROBE_DMA_MID = 16 };

template <int MODE, bool RANDOM>
__global__ __launch_bounds__(512, 2) void attention_step_kernel(float* out, int iters, float cs, float sub, long long* clk, const char* gbuf) {
  extern __shared__ __align__(16) char smem[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(MA_LDS char*)smem;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), r = lane & 31, g = lane >> 5;
  // a K tile and a V tile of 32 rows x 128 columns (8 KB each), swizzled as the forward kernel keeps them
  for (int i = tid; i < 16384 / 4; i += 512) {
    uint32_t h = (uint32_t)i * 2654435761u;
    h ^= h >> 15; h *= 2246822519u; h ^= h >> 13;
    // two bf16 values with random sign, exponent 2^-2 .. 2^1 and random mantissa
    const uint32_t lo16 = 0x3e80u + (h & 0x017fu) + ((h >> 9) & 1u) * 0x8000u, hi16 = 0x3e80u + ((h >> 16) & 0x017fu) + ((h >> 31) & 1u) * 0x8000u;
    ((MA_LDS uint32_t*)smem)[i] = RANDOM ? (hi16 << 16 | lo16) : 0x3c003c00u;
  }
  __syncthreads();
  bf16x8 qf[8];
#pragma unroll
  for (int ks = 0; ks < 8; ks++)
#pragma unroll
    for (int e = 0; e < 8; e++)
      qf[ks][e] = RANDOM ? (__bf16)(0.37f * (float)(((lane * 7 + e * 13 + ks * 5) % 11) - 5)) : (__bf16)(0.01f * ((lane + e + ks) & 7));
  f32x16 o[4], s[2];
  u32x4 p[2][2];
#pragma unroll
  for (int b = 0; b < 4; b++)
#pragma unroll
    for (int j = 0; j < 16; j++) o[b][j] = 0.f;
#pragma unroll
  for (int a = 0; a < 2; a++) {
#pragma unroll
    for (int j = 0; j < 16; j++) s[a][j] = 0.01f * j;
    p[a][0] = p[a][1] = u32x4{0x3c003c00u, 0x3c003c00u, 0x3c003c00u, 0x3c003c00u};
  }
  const uint32_t k_addr = lds0 + r * 256 + ((g ^ swz16(r)) << 4);
  const int jr = (lane & 15) >> 2, lc = (((lane >> 4) & 1) << 1) | ((lane & 3) >> 1);
  const uint32_t v_addr = lds0 + 8192 + (4 * g + jr) * 256 + (lane & 1) * 8 + ((lc ^ swz16(4 * g + jr)) << 4);
  constexpr int PFD = 2;   // fragments are requested two MFMA pairs ahead
  bf16x8 kf = qf[0], kfr[PFD + 1];
  bf16x4 lo = {0, 0, 0, 0}, hi = {0, 0, 0, 0}, lor[PFD + 1], hir[PFD + 1];
#pragma unroll
  for (int i = 0; i < PFD + 1; i++) { kfr[i] = kf; lor[i] = lo; hir[i] = lo; }
  float row_sum = 0.f;
  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const char* gwin = gbuf + (size_t)blockIdx.x * 1048576;   // 1 MB per workgroup, walked round and round: stays in L2
  uint32_t goff = 0, ring = 0;
  const long long t0 = __builtin_readcyclecounter();
  auto step = [&](auto par_c) __attribute__((always_inline)) {
    constexpr int PAR = decltype(par_c)::value;
    float part = 0.f;
    if (MODE & PROBE_DMA) __builtin_amdgcn_s_waitcnt(0x0F70 | 6);
    if (MODE & PROBE_BARRIER) __syncthreads();
    // the next sub-tile: 16 KB per workgroup, into a ring of 4 slots behind the two tiles that are read; both instructions of
    // a wave at the start of the step, or (PROBE_DMA_MID) one behind the third and one behind the sixth MFMA pair
    auto load_part = [&](int part) __attribute__((always_inline)) {
      dma16_so(gwin + goff + part * 8192, (uint32_t)(wave * 1024 + lane * 16), lds0 + 16384 + ring * 16384 + part * 8192 + wave * 1024);
    };
    if ((MODE & PROBE_DMA) && !(MODE & PROBE_DMA_MID)) {
      load_part(0);
      load_part(1);
    }
    uint32_t ka = k_addr, va = v_addr;
    asm volatile("" : "+v"(ka), "+v"(va));   // (the addresses are the same every step; keep the reads inside the loop)
    if (!(MODE & PROBE_LDS)) asm volatile("" : "+v"(kf), "+v"(lo), "+v"(hi));
#pragma unroll
    for (int i = 0; i < 8; i++) {
      if (MODE & PROBE_LDS) {
        const int fn = (i + PFD) & 7;
        kfr[(i + PFD) % (PFD + 1)] = lds_read<bf16x8>(ka + (fn << 5));
        lor[(i + PFD) % (PFD + 1)] = lds_read_tr4<__bf16>(va + (fn & 3) * 64 + (fn >> 2) * 16 * 256);
        hir[(i + PFD) % (PFD + 1)] = lds_read_tr4<__bf16>(va + (fn & 3) * 64 + (fn >> 2) * 16 * 256 + 8 * 256);
        __builtin_amdgcn_sched_barrier(0);
        kf = kfr[i % (PFD + 1)]; lo = lor[i % (PFD + 1)]; hi = hir[i % (PFD + 1)];
      }
      const bf16x8 vf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      o[i & 3] = Elem<__bf16>::mfma32(vf, __builtin_bit_cast(bf16x8, p[1 - PAR][i >> 2]), o[i & 3]);
      s[1 - PAR] = Elem<__bf16>::mfma32(kf, qf[i], i == 0 ? zero16 : s[1 - PAR]);
      if (MODE & PROBE_VECTOR) {
        const float pe0 = fast_exp2(s[PAR][2 * i] * cs + sub), pe1 = fast_exp2(s[PAR][2 * i + 1] * cs + sub);
        part += pe0;
        part += pe1;
        bf16x2 pk;
        pk[0] = (__bf16)pe0;
        pk[1] = (__bf16)pe1;
        uint32_t w = __builtin_bit_cast(uint32_t, pk);
        asm volatile("" : "+v"(w));
        p[PAR][i >> 2][i & 3] = w;
      }
      if ((MODE & PROBE_DMA) && (MODE & PROBE_DMA_MID) && (i == 2 || i == 5)) load_part(i == 5);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (MODE & PROBE_DMA) {
      goff = (goff + 16384) & (1048576 - 1);
      ring = ring == 3 ? 0 : ring + 1;
    }
    row_sum += part;
  };
  for (int it = 0; it < iters; it += 2) {
    step(std::integral_constant<int, 0>{});
    step(std::integral_constant<int, 1>{});
  }
  if (MODE & PROBE_DMA) __builtin_amdgcn_s_waitcnt(0x0F70);
  const long long t1 = __builtin_readcyclecounter();
  float acc = row_sum;
#pragma unroll
  for (int b = 0; b < 4; b++)
#pragma unroll
    for (int j = 0; j < 16; j++) acc += o[b][j];
#pragma unroll
  for (int a = 0; a < 2; a++)
#pragma unroll
    for (int j = 0; j < 16; j++) acc += s[a][j];
  out[blockIdx.x * blockDim.x + tid] = acc;
  if (blockIdx.x == 0 && tid == 0) clk[0] = t1 - t0;
}

template <int DEPTH>
__global__ __launch_bounds__(512) void stream_kernel(const char* src, size_t region_bytes, int iters, uint32_t* sink) {
  extern __shared__ __align__(16) char smem[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(MA_LDS char*)smem;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const size_t window = region_bytes / gridDim.x / 8192 * 8192;   // bytes per workgroup
  const char* base = src + (size_t)blockIdx.x * window;
  size_t off = 0;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int d = 0; d < DEPTH; d++) {
      dma16(base + off + (size_t)wave * 1024 + lane * 16, lds0 + (uint32_t)((d * 8 + wave) * 1024));
      off += 8192;
      if (off + 8192 > window) off = 0;
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);
  }
  __syncthreads();
  const u32x4 v = *(MA_LDS u32x4*)(uintptr_t)(lds0 + threadIdx.x * 16);
  if (v[0] == 0x12345678u) sink[0] = v[1];
}

// probe 3: how long does a direct-to-LDS load instruction hold the wave that issues it?  `nwaves` of the 8 waves of every
// workgroup (one workgroup per CU) issue `per_round` instructions (1 KB each) back to back, then wait for them, `rounds`
// times, walking a window of global memory; the cycle counter brackets the issue alone.  clk[0] = cycles wave 0 of
// workgroup 0 spent issuing, clk[1] = its cycles in all (issue + wait).
// KIND 0: global_load_lds_dwordx4 (1 KB per instruction), 1: global_load_lds_dword (256 B), 2: global_load_dwordx4 into
// registers (1 KB; the registers are stored to LDS with ds_write_b128 after the wait, outside the bracket).  A burst is NB
// instructions, fully unrolled, each at the address of the one before plus 8 KB (one 64-bit add between them); the window
// wrap is handled between the rounds, outside the bracket.
template <int KIND, int NB>
__global__ __launch_bounds__(512) void issue_hold_kernel(const char* src, size_t region_bytes, int nwaves, int rounds, long long* clk) {
  extern __shared__ __align__(16) char smem[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(MA_LDS char*)smem;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  if (wave >= nwaves) return;
  const size_t window = region_bytes / gridDim.x / 8192 * 8192;
  const char* base = src + (size_t)blockIdx.x * window + (size_t)wave * 1024 + lane * (KIND == 1 ? 4 : 16);
  size_t off = 0;
  long long t_issue = 0;
  u32x4 regs[NB];
#pragma unroll
  for (int i = 0; i < NB; i++) regs[i] = u32x4{0u, 0u, 0u, 0u};
  const long long t0 = __builtin_readcyclecounter();
  for (int r = 0; r < rounds; r++) {
    const char* p = base + off;
    uint32_t m0v = lds0 + (uint32_t)(wave * 1024);
    asm volatile("" : "+v"(p));
    const long long a0 = __builtin_readcyclecounter();
#pragma unroll
    for (int i = 0; i < NB; i++) {
      if constexpr (KIND == 2) asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(regs[i]) : "v"(p) : "memory");
      else if constexpr (KIND == 0) asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(m0v), "v"(p) : "memory");
      else asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" : : "s"(m0v), "v"(p) : "memory");
      p += 8192;
    }
    t_issue += __builtin_readcyclecounter() - a0;
    off += (size_t)NB * 8192;
    if (off + (size_t)NB * 8192 > window) off = 0;
    __builtin_amdgcn_s_waitcnt(0x0F70);
    if constexpr (KIND == 2) {
#pragma unroll
      for (int i = 0; i < NB; i++) {
        asm volatile("" : "+v"(regs[i]));
        lds_write<u32x4>(lds0 + (uint32_t)(((i & 7) * 8 + wave) * 1024 + lane * 16), regs[i]);
      }
    }
  }
  const long long t1 = __builtin_readcyclecounter();
  if (blockIdx.x == 0 && wave == 0 && lane == 0) { clk[0] = t_issue; clk[1] = t1 - t0; }
}

struct Buffers {
  float* out = nullptr;
  long long* clk = nullptr;
  char* gbuf = nullptr;
  size_t gbytes = 0;
};
Buffers g_buf;

int ensure(size_t gbytes) {
  if (!g_buf.out && hipMalloc(&g_buf.out, 256 * 512 * sizeof(float)) != hipSuccess) return -1;
  if (!g_buf.clk && hipMalloc(&g_buf.clk, 64) != hipSuccess) return -1;
  if (g_buf.gbytes < gbytes) {
    if (g_buf.gbuf) (void)hipFree(g_buf.gbuf);
    g_buf.gbuf = nullptr;
    g_buf.gbytes = 0;
    if (hipMalloc(&g_buf.gbuf, gbytes) != hipSuccess) return -1;
    if (hipMemset(g_buf.gbuf, 1, gbytes) != hipSuccess) return -1;
    g_buf.gbytes = gbytes;
  }
  return 0;
}

template <typename K, typename... A>
int timed(K kern, dim3 grid, dim3 block, size_t lds, float* ms, A... args) {
  if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) return -1;
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return -1;
  (void)hipEventRecord(e0, nullptr);
  hipLaunchKernelGGL(kern, grid, block, lds, nullptr, args...);
  (void)hipEventRecord(e1, nullptr);
  const hipError_t err = hipEventSynchronize(e1);
  (void)hipEventElapsedTime(ms, e0, e1);
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  return err == hipSuccess && hipGetLastError() == hipSuccess ? 0 : -1;
}

template <int MODE>
int run_step(int random_operands, int iters, float* ms) {
  constexpr size_t lds = 16384 + 4 * 16384;
  if (random_operands) return timed(attention_step_kernel<MODE, true>, dim3(256), dim3(512), lds, ms, g_buf.out, iters, 0.1f, -1.f, g_buf.clk, (const char*)g_buf.gbuf);
  return timed(attention_step_kernel<MODE, false>, dim3(256), dim3(512), lds, ms, g_buf.out, iters, 0.1f, -1.f, g_buf.clk, (const char*)g_buf.gbuf);
}

}  // namespace

extern "C" {

// mode: bit mask of 1 (vector work), 2 (LDS fragment reads), 4 (barrier per step), 8 (direct-to-LDS loads), 16 (those loads
// between the MFMAs of the step instead of at its start); only the masks 0, 1, 2, 3, 7, 15 and 31 are built.  Runs `iters` steps per wave on 256 workgroups twice (the first run is a warm-up) and
// returns the wall time per step in nanoseconds and the cycle count per step seen by wave 0 of workgroup 0.  Returns 0
// on success, -1 on a HIP failure, -2 for a mask that is not built.
int ma_probe_attention_step(int mode, int random_operands, int iters, double* ns_per_step, double* cycles_per_step) {
  if (iters < 2 || ensure((size_t)256 << 20) != 0) return -1;
  iters &= ~1;
  float ms = 0.f;
  int rc = -2;
  for (int rep = 0; rep < 2; rep++) {
    const int n = rep == 0 ? 200 : iters;
    switch (mode) {
      case 0: rc = run_step<0>(random_operands, n, &ms); break;
      case 1: rc = run_step<1>(random_operands, n, &ms); break;
      case 2: rc = run_step<2>(random_operands, n, &ms); break;
      case 3: rc = run_step<3>(random_operands, n, &ms); break;
      case 7: rc = run_step<7>(random_operands, n, &ms); break;
      case 15: rc = run_step<15>(random_operands, n, &ms); break;
      case 31: rc = run_step<31>(random_operands, n, &ms); break;
      default: return -2;
    }
    if (rc != 0) return rc;
  }
  long long c = 0;
  if (hipMemcpy(&c, g_buf.clk, sizeof(c), hipMemcpyDeviceToHost) != hipSuccess) return -1;
  *ns_per_step = (double)ms * 1e6 / iters;
  *cycles_per_step = (double)c / iters;
  return 0;
}

// Streams `region_bytes` (split evenly over 256 workgroups, each walking its window round and round) into LDS with `depth`
// (2 or 6) 1 KB direct-to-LDS instructions in flight per wave, `iters` rounds; returns GB/s over the whole chip.
int ma_probe_stream_to_lds(size_t region_bytes, int depth, int iters, double* gb_per_s) {
  if (region_bytes < ((size_t)256 << 13) || ensure(region_bytes) != 0) return -1;
  float ms = 0.f;
  int rc = -2;
  for (int rep = 0; rep < 2; rep++) {
    const int n = rep == 0 ? 20 : iters;
    if (depth == 2) rc = timed(stream_kernel<2>, dim3(256), dim3(512), (size_t)65536, &ms, (const char*)g_buf.gbuf, region_bytes, n, (uint32_t*)g_buf.clk);
    else if (depth == 6) rc = timed(stream_kernel<6>, dim3(256), dim3(512), (size_t)65536, &ms, (const char*)g_buf.gbuf, region_bytes, n, (uint32_t*)g_buf.clk);
    else return -2;
    if (rc != 0) return rc;
  }
  *gb_per_s = 256.0 * iters * depth * 8192.0 / ((double)ms * 1e-3) / 1e9;
  return 0;
}

// `nwaves` (1..8) waves per CU issue `per_round` (1, 2, 4 or 8) load instructions back to back per round, 200 rounds, from a region
// of `region_bytes`; kind 0: global_load_lds_dwordx4 (1 KB), 1: global_load_lds_dword (256 B), 2: global_load_dwordx4 into
// registers (1 KB); the bracket of a burst of 1 also holds the two cycle-counter reads (subtract the 1-instruction figure
// from 8 x the 8-instruction figure and divide by 7 for the cost of one more instruction); returns the cycles one instruction holds its wave at issue and the cycles per
// instruction including the wait for the round's data (wave 0 of workgroup 0).
int ma_probe_issue_hold(int kind, size_t region_bytes, int nwaves, int per_round, double* issue_cycles_per_instr, double* total_cycles_per_instr) {
  if (kind < 0 || kind > 2 || nwaves < 1 || nwaves > 8 || (per_round != 1 && per_round != 2 && per_round != 4 && per_round != 8) || region_bytes < ((size_t)256 << 16) || ensure(region_bytes) != 0)
    return -1;
  float ms = 0.f;
  const int rounds = 200;
  auto go = [&](auto kern) { return timed(kern, dim3(256), dim3(512), (size_t)65536, &ms, (const char*)g_buf.gbuf, region_bytes, nwaves, rounds, g_buf.clk); };
  for (int rep = 0; rep < 2; rep++) {
    int rc;
    if (per_round == 1) rc = kind == 0 ? go(issue_hold_kernel<0, 1>) : kind == 1 ? go(issue_hold_kernel<1, 1>) : go(issue_hold_kernel<2, 1>);
    else if (per_round == 2) rc = kind == 0 ? go(issue_hold_kernel<0, 2>) : kind == 1 ? go(issue_hold_kernel<1, 2>) : go(issue_hold_kernel<2, 2>);
    else if (per_round == 4) rc = kind == 0 ? go(issue_hold_kernel<0, 4>) : kind == 1 ? go(issue_hold_kernel<1, 4>) : go(issue_hold_kernel<2, 4>);
    else rc = kind == 0 ? go(issue_hold_kernel<0, 8>) : kind == 1 ? go(issue_hold_kernel<1, 8>) : go(issue_hold_kernel<2, 8>);
    if (rc != 0) return -1;
  }
  long long c[2] = {0, 0};
  if (hipMemcpy(c, g_buf.clk, sizeof(c), hipMemcpyDeviceToHost) != hipSuccess) return -1;
  *issue_cycles_per_instr = (double)c[0] / ((double)rounds * per_round);
  *total_cycles_per_instr = (double)c[1] / ((double)rounds * per_round);
  return 0;
}

}  // extern "C"
