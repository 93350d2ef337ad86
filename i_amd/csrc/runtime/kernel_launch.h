// Host-side launchers for the hand-written gfx950 kernels.  They validate the
// operand shapes against what each kernel and its grid assume, pick the
// kernel variant, and enqueue it on `stream`.  All pointers are device memory.
#pragma once
#include <cstddef>

#include "hip_rt.h"

namespace ihip {

enum DType { F32 = 0, BF16 = 1 };

// o[bh,nq,dv] = softmax(s * q[bh,nq,d] k[bh,nk,d]^T) v[bh,nk,dv],  s = scale * (scale_ptr ? *scale_ptr : 1)
// in_dtype applies to q, k, v; out_dtype to o (F32 or BF16; BF16 only with bf16 inputs).
// scale_ptr, when given, is a rank-0 f32 operand in device memory, read by the kernel.
// query_tile is the query-row tile the schedule asks for (the product of the split factors of the row
// index; 0 = no preference): 128 and 256 select the 4- and 8-wave workgroup of the direct-to-LDS kernel, any other
// value leaves the choice to the launcher.
Err launch_attention(const void* q, const void* k, const void* v, void* o, DType in_dtype, DType out_dtype, size_t bh,
                     size_t nq, size_t nk, size_t d, size_t dv, const float* scale_ptr, float scale, hipStream_t stream,
                     size_t query_tile = 0);
bool attention_supported(DType in_dtype, size_t d, size_t dv);

// c[bh,m,n] (f32) = a[bh,m,k] b[bh,n,k]^T, a and b bf16
// tile_m x tile_n is the output tile the schedule asks for (0 = no preference): 256 x 256 and 128 x 128 select
// the kernel with that workgroup tile (when its requirements hold), anything else leaves the choice to the launcher.
Err launch_gemm_nt_bf16(const void* a, const void* b, float* c, size_t bh, size_t m, size_t n, size_t k,
                        hipStream_t stream, size_t tile_m = 0, size_t tile_n = 0);
bool gemm_nt_bf16_supported(size_t k);

// c[bh,m,n] (f32) = a[bh,m,k] b[bh,k,n], a and b bf16, on the direct kernels with a row-major right operand.
// Needs k % 64 == 0 and n % 8 == 0 (gemm_nn_bf16_supported); callers transpose b and use the NT kernels otherwise.
Err launch_gemm_nn_bf16(const void* a, const void* b, float* c, size_t bh, size_t m, size_t n, size_t k,
                        hipStream_t stream, size_t tile_m = 0, size_t tile_n = 0);
bool gemm_nn_bf16_supported(size_t bh, size_t m, size_t n, size_t k);

// c[bh,m,n] = a[bh,m,k] b[bh,n,k]^T, all f32, products and sums in f32 (f32 MFMA); needs k % 32 == 0
Err launch_gemm_nt_f32(const float* a, const float* b, float* c, size_t bh, size_t m, size_t n, size_t k,
                       hipStream_t stream);
bool gemm_nt_f32_supported(size_t k);

// y[rows,cols] = row softmax of x, f32
// mode 0: softmax; 1: y = x - rowmax(x) (row_max_shift); 2: y = x / rowsum(x) (row_normalize); 3: y = exp(x)
Err launch_row_softmax(const float* x, float* y, size_t rows, size_t cols, hipStream_t stream, int mode = 0);

// dst[b][c][r] = src[b][r][c]; elem_bytes is 2 or 4.  An NN product that the direct kernels cannot read runs as transpose + NT kernel.
Err launch_transpose(const void* src, void* dst, size_t bh, size_t rows, size_t cols, size_t elem_bytes,
                     hipStream_t stream);

Err launch_convert(const void* src, void* dst, DType from, DType to, size_t n, hipStream_t stream);

}  // namespace ihip
