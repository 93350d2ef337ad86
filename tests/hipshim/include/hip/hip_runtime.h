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

#define __global__ __attribute__((visibility("default")))
#define __launch_bounds__(...)
#define __device__
#define __forceinline__ inline
