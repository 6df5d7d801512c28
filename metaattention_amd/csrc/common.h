// Shared device helpers for the gfx950 kernels: 64-lane MFMA fragments,
// LDS swizzles, cross-half exchange.  gfx950 only; there is no other target.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "host_util.h"

namespace ma {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

#define MA_LDS __attribute__((address_space(3)))

// Element traits.  Fragment conventions of v_mfma_f32_32x32x16_{bf16,f16}
// (lane l, r = l % 32, g = l / 32), verified on hardware:
//   A[32 x 16]: lane holds row r, k = 8g .. 8g+7
//   B[16 x 32]: lane holds column r, k = 8g .. 8g+7
//   C[32 x 32]: lane holds column r, element j (0..15) is row 8(j/4) + 4g + j%4
template <typename T> struct Elem;
template <> struct Elem<__bf16> {
  using x8 = bf16x8; using x4 = bf16x4; using x2 = bf16x2;
  static __device__ __forceinline__ f32x16 mfma32(x8 a, x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 mfma16(x8 a, x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct Elem<_Float16> {
  using x8 = f16x8; using x4 = f16x4; using x2 = f16x2;
  static __device__ __forceinline__ f32x16 mfma32(x8 a, x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 mfma16(x8 a, x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};

// Transposing LDS read (ds_read_b64_tr_b16).  Within each block of 16 lanes,
// lane j supplies the address of 4 consecutive 16-bit elements; result lane i
// receives element (i % 4) of lanes i/4, 4 + i/4, 8 + i/4, 12 + i/4.  With
// lanes 4r..4r+3 pointing at 16 consecutive columns of row r (r = 0..3), lane
// i ends up with column i of rows 0..3: a 4-deep column read of a row-major
// tile, which is the K-major operand MFMA wants.  (Mapping verified on hardware.)
template <typename T>
__device__ __forceinline__ typename Elem<T>::x4 lds_read_tr4(uint32_t lds_byte_addr) {
  s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((MA_LDS s16x4*)(uintptr_t)lds_byte_addr);
  return __builtin_bit_cast(typename Elem<T>::x4, v);
}

template <typename V>
__device__ __forceinline__ V lds_read(uint32_t lds_byte_addr) {
  return *(const MA_LDS V*)(uintptr_t)lds_byte_addr;
}
template <typename V>
__device__ __forceinline__ void lds_write(uint32_t lds_byte_addr, V v) {
  *(MA_LDS V*)(uintptr_t)lds_byte_addr = v;
}

// value held by lane (l ^ 32)
__device__ __forceinline__ float xhalf(float x) {
  return __shfl_xor(x, 32, 64);
}

// The two halves of the wave exchange x: for every lane, {lo, hi} = {x of the lane's own half, x of lane^32}
// in an order that is the same for both lanes of a pair -- enough for symmetric combinations (max, sum),
// and one v_permlane32_swap instead of a trip through the LDS crossbar.
__device__ __forceinline__ void xhalf_pair(float x, float& lo, float& hi) {
  const uint32_t u = __builtin_bit_cast(uint32_t, x);
  const auto rr = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  lo = __builtin_bit_cast(float, (uint32_t)rr[0]);
  hi = __builtin_bit_cast(float, (uint32_t)rr[1]);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

// Direct-to-LDS load of 64 x 16 bytes (global_load_lds_dwordx4): lane i's 16 bytes
// land at lds_base + 16 i; every lane chooses its own global source address.
// Issued through inline asm so that the compiler does not serialise later LDS
// reads behind it; completion is awaited explicitly with wait_dma() before the
// barrier that publishes the data.  lds_base must be wave-uniform.
__device__ __forceinline__ void dma16(const void* gptr, uint32_t lds_base) {
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %1, off\n\t"
      :
      : "s"(__builtin_amdgcn_readfirstlane(lds_base)), "v"(gptr)
      : "memory");
}
// Direct-to-LDS load of 64 x 4 bytes (global_load_lds_dword): lane i's dword lands at lds_base + 4 i.
__device__ __forceinline__ void dma4(const void* gptr, uint32_t lds_base) {
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dword %1, off\n\t"
      :
      : "s"(__builtin_amdgcn_readfirstlane(lds_base)), "v"(gptr)
      : "memory");
}
// Same with a wave-uniform 64-bit base (scalar registers) plus a per-lane 32-bit byte offset.
__device__ __forceinline__ void dma16_so(const void* base_uniform, uint32_t lane_off, uint32_t lds_base) {
  const uint64_t b = (uint64_t)(uintptr_t)base_uniform;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)b), hi = __builtin_amdgcn_readfirstlane((uint32_t)(b >> 32));
  const uint64_t sb = ((uint64_t)hi << 32) | lo;
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %1, %2\n\t"
      :
      : "s"(__builtin_amdgcn_readfirstlane(lds_base)), "v"(lane_off), "s"(sb)
      : "memory");
}
__device__ __forceinline__ void dma4_so(const void* base_uniform, uint32_t lane_off, uint32_t lds_base) {
  const uint64_t b = (uint64_t)(uintptr_t)base_uniform;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)b), hi = __builtin_amdgcn_readfirstlane((uint32_t)(b >> 32));
  const uint64_t sb = ((uint64_t)hi << 32) | lo;
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dword %1, %2\n\t"
      :
      : "s"(__builtin_amdgcn_readfirstlane(lds_base)), "v"(lane_off), "s"(sb)
      : "memory");
}
// vmcnt(0), other counters untouched.  The builtin (rather than asm) also tells the
// compiler's own wait-count bookkeeping that no vector-memory load is pending any more.
__device__ __forceinline__ void wait_dma() { __builtin_amdgcn_s_waitcnt(0x0F70); }
// vmcnt(N): at most the N most recent vector-memory instructions of this wave are still in flight (they complete in order)
template <int N>
__device__ __forceinline__ void wait_vm() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

// XOR swizzle (in 16-byte chunks) of a row-major LDS tile with >= 16 chunks per row:
// a bijection on the low 4 row bits, so 128-bit reads of 16 consecutive rows at one
// logical chunk hit 16 different bank groups, and the 8 rows x 4 chunks touched by a
// transposing read spread evenly over the banks.
__device__ __forceinline__ int swz16(int row) { return ((row & 3) << 2) | ((row >> 2) & 3); }

// The same for any row length: with 8 chunks per row (128-byte rows) two rows span the banks, so the
// row's bit 1 goes to chunk bit 2 and row bits 2..3 to chunk bits 0..1.
template <int CPR>
__device__ __forceinline__ int swz_tile(int row) {
  if constexpr (CPR >= 16) return swz16(row);
  return (((row >> 1) & 1) << 2) | ((row >> 2) & 3);
}

// DMA of a [32 rows x ROWB bytes] tile, XOR-swizzled in 16-byte chunks, whose 32 rows all lie inside the tensor (NWAVES
// waves share the tile's instructions of 1 KB each: lane i fetches the chunk that belongs at physical position i of that
// KB).  The byte offsets of a lane (tile row * row stride + swizzled chunk) are computed once, and a tile's DMA is then
// its wave-uniform first-row address in scalar registers plus those 32-bit offsets: no per-lane 64-bit address
// arithmetic inside the loops.  The swizzle term repeats every 16 rows, so instructions of a wave that are a multiple
// of 16 rows apart share an offset and the row distance goes into the scalar base.
// Head sizes that are not powers of two (192) live in LDS rows of the next power of two: the swizzles and the XOR
// addressing of the k-slices need row sizes that are powers of two.  The columns beyond the head size are neither loaded
// nor read.
constexpr int pad_width(int d) { return d <= 64 ? 64 : d <= 128 ? 128 : d <= 256 ? 256 : 512; }

// (USED: the 16-byte chunks of a row that exist in memory; a lane whose chunk lies beyond them sits the instruction out)
template <int ROWB, int NWAVES, int USED = ROWB / 16>
struct TileDma {
  static constexpr int CPR = ROWB / 16, RPI = 1024 / ROWB, NI = 32 * ROWB / 1024, NJ = NI / NWAVES;
  static constexpr int RPJ = NWAVES * RPI;   // rows between consecutive instructions of a wave
  static constexpr int NOFF = RPJ % 16 == 0 ? 1 : (16 % RPJ == 0 && 16 / RPJ < NJ ? 16 / RPJ : NJ);
  static_assert(NI % NWAVES == 0, "a tile is a whole number of instructions per wave");
  uint32_t off[NOFF];
  bool on[USED < CPR ? NOFF : 1];
  uint32_t stride;
  __device__ __forceinline__ void init(uint32_t row_stride, int wave, int lane) {
    stride = row_stride;
#pragma unroll
    for (int j = 0; j < NOFF; j++) {
      const int row = (wave + NWAVES * j) * RPI + lane / CPR, c = lane % CPR;
      off[j] = (uint32_t)row * row_stride + (uint32_t)((c ^ swz_tile<CPR>(row)) << 4);
      if constexpr (USED < CPR) on[j] = (c ^ swz_tile<CPR>(row)) < USED;
    }
  }
  __device__ __forceinline__ void issue(const char* first_row, uint32_t lds_base, int wave) const {
#pragma unroll
    for (int j = 0; j < NJ; j++) {
      if constexpr (USED < CPR) {
        if (!on[j % NOFF]) continue;
      }
      dma16_so(first_row + (uint64_t)((uint32_t)((j / NOFF) * NOFF * RPJ) * stride), off[j % NOFF], lds_base + (wave + NWAVES * j) * 1024);
    }
  }
};

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

}  // namespace ma
