// Host stand-in for <hip/hip_runtime.h>, used only by the CPU emulation tests: it lets the HIP source that
// the backend generates be compiled as ordinary C++ and run one "work-item" at a time.
#pragma once
#include <math.h>
#include <stddef.h>

struct shim_dim3 {
  unsigned x, y, z;
};
static thread_local shim_dim3 blockIdx, threadIdx, blockDim, gridDim;

extern "C" __attribute__((visibility("default"))) inline void shim_set_ids(unsigned bx, unsigned tx, unsigned bdx,
                                                                             unsigned gdx) {
  blockIdx = {bx, 0, 0};
  threadIdx = {tx, 0, 0};
  blockDim = {bdx, 1, 1};
  gridDim = {gdx, 1, 1};
}
// force an out-of-line copy of the inline function into every kernel library
static void (*const shim_keep_set_ids)(unsigned, unsigned, unsigned, unsigned) __attribute__((used)) = shim_set_ids;

// __syncthreads(): when the emulation runs the work-items of a workgroup as real threads (workgroups of more
// than one wavefront), it hands every thread a barrier to wait on; work-items run one after the other have none.
static thread_local void (*shim_barrier_fn)(void*) = nullptr;
static thread_local void* shim_barrier_arg = nullptr;
extern "C" __attribute__((visibility("default"))) inline void shim_set_barrier(void (*fn)(void*), void* arg) {
  shim_barrier_fn = fn;
  shim_barrier_arg = arg;
}
static void (*const shim_keep_set_barrier)(void (*)(void*), void*) __attribute__((used)) = shim_set_barrier;
static inline void __syncthreads() {
  if (shim_barrier_fn) shim_barrier_fn(shim_barrier_arg);
}

// The wavefront form of a generated kernel: 64 consecutive work-items of a workgroup are the lanes of a
// wavefront.  The emulation hands each of the 64 threads its wavefront's barrier and exchange slots;
// ILANG_WAVE_SYNC() makes the statements that all lanes execute alike happen in lockstep, as on the device.
struct shim_wave_ctx {
  void (*wait)(void*);
  void* barrier;
  float* slots;  // 64
};
static thread_local shim_wave_ctx shim_wave = {nullptr, nullptr, nullptr};
extern "C" __attribute__((visibility("default"))) inline void shim_set_wave(void (*wait)(void*), void* barrier, float* slots) {
  shim_wave = {wait, barrier, slots};
}
static void (*const shim_keep_set_wave)(void (*)(void*), void*, float*) __attribute__((used)) = shim_set_wave;
static inline void shim_wave_sync() {
  if (!shim_wave.wait) __builtin_trap();  // a wavefront kernel launched with work-items that run one after the other
  shim_wave.wait(shim_wave.barrier);
}
#define ILANG_WAVE_SYNC() shim_wave_sync()
static inline float __shfl_xor(float v, int lane_xor) {
  const unsigned lane = threadIdx.x % 64;
  shim_wave.slots[lane] = v;
  shim_wave_sync();
  const float r = shim_wave.slots[lane ^ (unsigned)lane_xor];
  shim_wave_sync();
  return r;
}

#define __global__ __attribute__((visibility("default")))
#define __launch_bounds__(...)
#define __device__
#define __forceinline__ inline
