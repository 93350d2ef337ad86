// Shared device-side definitions for the gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16_t;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

// log2 of the f32 literal 2.71828175f, the base the reference C backend uses
// for unary pow (compiler/src/lower/exec_plan_to_module.rs:630-633):
// powf(2.71828175f, x) == exp2(x * I_LOG2_E32).
#define I_LOG2_E32 1.44269499718f

#define WAVE 64

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Exchange a value between lane l and lane l^32.
__device__ __forceinline__ float xhalf(float x) { return __shfl_xor(x, 32, 64); }

// Both half-waves' copies of a value: after the call lo = x[lane & 31], hi = x[(lane & 31) + 32]
// in every lane.  v_permlane32_swap exchanges the upper half of its first register with the
// lower half of its second.  It is issued as inline assembly on two registers that both hold x
// (the compiler builtin mis-assigns the second result on this toolchain); the s_nop cover the
// VALU-write -> permlane read wait states the compiler would otherwise insert itself.
__device__ __forceinline__ void both_halves(float x, float& lo, float& hi) {
  float a = x, b = x;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  lo = a;
  hi = b;
}
// max / sum of a value over the two half-waves (lanes l and l^32), result in both.
__device__ __forceinline__ float half_max(float x) {
  float lo, hi;
  both_halves(x, lo, hi);
  return fmaxf(lo, hi);
}
__device__ __forceinline__ float half_sum(float x) {
  float lo, hi;
  both_halves(x, lo, hi);
  return lo + hi;
}

__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x = fmaxf(x, __shfl_xor(x, o, 64));
  return x;
}
__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o, 64);
  return x;
}

__device__ __forceinline__ u32x4 ldg128(const void* p) { return *reinterpret_cast<const u32x4*>(p); }

// Effective score scale in the log2 domain.  exp is spelled pow(2.71828175f, x)
// by the reference, i.e. exp2(x * I_LOG2_E32).
__device__ __forceinline__ float load_scale(const float* ptr, float value) {
  return (ptr ? *ptr : 1.0f) * value;
}

// Workgroups are dealt round-robin to the 8 XCDs, each with a private L2.  The tiles of all groups in sequence
// (`per_group` tiles per group, e.g. the query tiles of one attention head after those of the one before) are cut
// into 8 equal runs, one per XCD: workgroup id (xcd = id % 8, slot = id / 8) takes number xcd * ceil(T / 8) + slot
// of the sequence.  The workgroups of an XCD thus walk consecutive tiles of one group after the other (a head's K/V
// stay in that XCD's L2) and every XCD has work whatever the number of groups: a single head is spread over all
// eight.  Launch with at least 8 * ceil(T / 8) workgroups; one without a tile gets group == groups.
__device__ __forceinline__ void xcd_map(uint32_t id, uint32_t per_group, uint32_t groups, uint32_t& group, uint32_t& tile) {
  const uint32_t total = groups * per_group, per_xcd = (total + 7u) / 8u;
  const uint32_t slot = id >> 3, at = (id & 7u) * per_xcd + slot;
  if (slot >= per_xcd || at >= total) {
    group = groups;
    tile = 0;
    return;
  }
  group = at / per_group;
  tile = at - group * per_group;
}

// Output tile of a large-tile GEMM workgroup.  The tiles are numbered block by block (blocks of 4 x 8 tiles, the
// blocks of one block column after the other, blocks at the far edges being as small as the tile grid leaves
// them; inside a block the m index runs fastest), and that sequence is cut into 8 equal runs, one per XCD:
// workgroup id (xcd = id % 8, slot = id / 8) takes tile number xcd * ceil(T / 8) + slot of it.  The 32 CUs
// of an XCD thus work on consecutive tiles (at most 1024 rows of A and 2048 of B at a time, shared through the
// XCD's L2), and the XCDs get the same number of tiles to within one: with whole blocks dealt out to XCDs
// instead, 22 x 22 tiles (18 blocks) cost three rounds of workgroups where two suffice.
// Launch with 8 * ceil(T / 8) workgroups per batch (so that id % 8 is the XCD in every batch).  `batch` rotates
// which XCD takes which run: when T is not a multiple of 8 the short and the empty runs then fall on a different
// XCD in every batch (one tile per batch: batch b runs on XCD (8 - b) % 8 instead of all of them on XCD 0).
// Returns false for a workgroup that has no tile.
__device__ __forceinline__ bool gemm_tile_of_workgroup(uint32_t id, uint32_t batch, uint32_t tiles_m, uint32_t tiles_n,
                                                       uint32_t& tm, uint32_t& tn) {
  const uint32_t total = tiles_m * tiles_n, per_xcd = (total + 7) / 8;
  const uint32_t slot = id >> 3, at = ((id + batch) & 7u) * per_xcd + slot;
  if (slot >= per_xcd || at >= total) return false;
  const uint32_t column = tiles_m * 8;            // tiles in a full block column
  const uint32_t bn = at / column, in_column = at - bn * column;
  const uint32_t wn = min(8u, tiles_n - 8 * bn);  // width of this block column, in tiles
  const uint32_t bm = in_column / (4 * wn), in_block = in_column - bm * 4 * wn;
  const uint32_t hm = min(4u, tiles_m - 4 * bm);  // height of this block
  tm = 4 * bm + in_block % hm;
  tn = 8 * bn + in_block / hm;
  return true;
}

// One 16-byte-per-lane global -> LDS transfer.  `lds_base` (wave-uniform) is where lane 0's
// 16 bytes land; lane l lands at lds_base + 16 l.  `base` is wave-uniform, `voff` per lane.
// The compiler is not told that LDS is written: completion is awaited explicitly with
// dma_wait_all() before the barrier that publishes the tile.
__device__ __forceinline__ void dma16(const void* base, uint32_t voff, uint32_t lds_base) {
  asm volatile(
      "s_mov_b32 m0, %2\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %0, %1"
      :
      : "v"(voff), "s"(base), "s"(lds_base)
      : "memory");
}
__device__ __forceinline__ void dma_wait_all() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// The two device clocks: the shader clock (s_memtime: it follows the frequency the power manager grants) and the
// constant 100 MHz clock (s_memrealtime).  A workgroup that is asked to (clock != nullptr) subtracts both readings
// from clock[0] and clock[1] when it starts and adds them when it ends (unsigned arithmetic: the sums come out as
// the time the workgroups were resident on either clock); nothing is held in registers in between.
__device__ __forceinline__ void clock_note(unsigned long long* clock, bool leaving) {
  if (clock && threadIdx.x == 0) {
    const unsigned long long shader = __builtin_amdgcn_s_memtime(), constant = __builtin_amdgcn_s_memrealtime();
    atomicAdd(clock, leaving ? shader : 0ull - shader);
    atomicAdd(clock + 1, leaving ? constant : 0ull - constant);
  }
}

__device__ __forceinline__ uint32_t lds_address(const void* p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)p;
}
