// Kernel argument blocks shared by the device code and the host launcher.
// Each kernel takes exactly one of these by value.
#pragma once
#include <stdint.h>

enum { I_DT_F32 = 0, I_DT_BF16 = 1 };

struct AttnParams {
  const void* q;   // [bh, nq, d]
  const void* k;   // [bh, nk, d]
  const void* v;   // [bh, nk, dv]
  void* o;         // [bh, nq, dv]
  uint32_t bh, nq, nk, d, dv;
  uint32_t nqt;        // query tiles per head
  uint32_t out_bf16;   // 0: f32 output, 1: bf16 output
  // score scale = scale_value * (scale_ptr ? *scale_ptr : 1), any finite value
  const float* scale_ptr;  // optional rank-0 f32 operand in device memory
  float scale_value;
  // The keys of a head split over workgroups (the direct kernels, bf16 and f32; 0 or 1: not split).  bh then counts
  // (head, part) pairs: part s attends the keys kv_chunk * s .. + kv_chunk (what is left of nk for the last one)
  // and writes its normalised f32 result to o[head * kv_splits + s][nq][dv] and log2 of its sum of exponentials
  // (relative to nothing: reference included) to lse[head * kv_splits + s][nq]; attn_kv_merge combines them.
  uint32_t kv_splits;
  uint32_t kv_chunk;  // a multiple of 64
  float* lse;
  // Optional (the bf16 direct-to-LDS kernels): two 64-bit counters to which every workgroup adds what its first wave
  // saw pass between entry and exit on the shader clock (s_memtime, which follows the clock the power manager
  // grants) and on the constant 100 MHz clock (s_memrealtime).  clock[0] / clock[1] * 0.1 is the average shader
  // clock in GHz over the launch, weighted by the time the workgroups were resident.
  unsigned long long* clock;
};

// One wavefront that reads both clocks, sleeps until `ticks` of the 100 MHz clock have passed, reads them again and
// adds the differences to out[0] (shader clock) and out[1] (100 MHz clock): the shader clock under whatever else
// the GPU runs meanwhile, for kernels that cannot count for themselves.
struct ClockProbeParams {
  unsigned long long* out;
  uint32_t ticks;  // of 10 ns; the host bounds it to two seconds
};

// out[b][r][:] = sum_s w_s partial[b * splits + s][r][:],  w_s = 2^lse[b * splits + s][r] / sum_t 2^lse[b * splits + t][r]
struct AttnMergeParams {
  const float* partial;  // [heads * splits, nq, dv]
  const float* lse;      // [heads * splits, nq]
  void* out;             // [heads, nq, dv] f32 or bf16
  uint32_t heads, splits, nq, dv;  // dv a multiple of 4
  uint32_t out_bf16;
};

struct GemmParams {
  const void* a;   // [bh, m, k]
  const void* b;   // [bh, n, k]
  void* c;         // [bh, m, n]  f32, or bf16 when out_bf16 is set (bf16 operands only)
  uint32_t bh, m, n, k;
  uint32_t tiles_m, tiles_n;
  uint32_t out_bf16;  // 0: f32 output, 1: the f32 sums are rounded to bf16 on the way out
  // The k loop split over workgroups (the direct kernels, NT and NN; 0 or 1: not split).  blockIdx.y then counts
  // (batch, split) pairs; split s contracts k_chunk * s .. + k_chunk (what is left of k for the last one) and
  // writes its f32 partial products to c[(batch * splits + s)][m][n], a temporary that splitk_reduce adds up.
  uint32_t splits;
  uint32_t k_chunk;   // a multiple of 64
};

// out[b][i] = sum over s < splits of partial[b][s][i], i < count (count a multiple of 4); out f32 or bf16
struct SplitReduceParams {
  const float* partial;
  void* out;
  uint32_t batches, splits;
  uint64_t count;
  uint32_t out_bf16;
};

struct SoftmaxParams {
  const float* x;
  float* y;
  uint32_t rows, cols;
  // the "softmax of scale * x" kernels only: scale = scale_value * (scale_ptr ? *scale_ptr : 1)
  const float* scale_ptr;
  float scale_value;
  // A row in parts over workgroups (row_*_parts_* kernels: fewer rows than CUs, very long rows): blockIdx.x counts
  // (row, part) pairs, part s covers the accesses part_chunks * s .. + part_chunks of its row; the first kernel
  // leaves each part's running max and sum of exponentials in stats[row][part][2], the second combines them.
  float* stats;
  uint32_t parts, part_chunks;
};

struct ConvertParams {
  const void* src;
  void* dst;
  uint64_t n;
};

// dst[b][c][r] = src[b][r][c] for b < bh, r < rows, c < cols; elements of 2 or 4 bytes
// dst[r][c] = c < cols ? src[r][c] : 0 for r < rows, c < cols_padded; elements of 2 or 4 bytes
struct PadParams {
  const void* src;
  void* dst;
  uint64_t rows;
  uint32_t cols, cols_padded;
};

struct TransposeParams {
  const void* src;
  void* dst;
  uint32_t bh, rows, cols;
  uint32_t tiles_r, tiles_c;  // 64 x 64 tiles
};

