// Single translation unit for the gfx950 code object (i_kernels_gfx950.hsaco).
// Every entry point is extern "C" so the host side can look it up by name with
// hipModuleGetFunction; each takes one parameter block by value (params.h).
#include "attention_bf16.h"
#include "attention_bf16_direct.h"
#include "attention_f32.h"
#include "attention_f32_direct.h"
#include "gemm_nt_bf16.h"
#include "gemm_nt_f32_direct.h"
#include "gemm_nt_bf16_mfma16.h"
#include "row_softmax.h"

// attn_fwd_bf16_d<D>_bn<BN>: d == dv == D exactly; ..._any: d, dv <= D (multiples of 8), guarded columns
#define ATTN_BF16(DPAD, BN, NW, OCC)                                                                          \
  extern "C" __global__ void __launch_bounds__(NW * 64, OCC) attn_fwd_bf16_d##DPAD##_bn##BN(AttnParams p) {   \
    attn_fwd_bf16_body<DPAD, BN, NW, true>(p);                                                                \
  }                                                                                                           \
  extern "C" __global__ void __launch_bounds__(NW * 64, OCC) attn_fwd_bf16_d##DPAD##_bn##BN##_any(AttnParams p) { \
    attn_fwd_bf16_body<DPAD, BN, NW, false>(p);                                                               \
  }
ATTN_BF16(64, 64, 4, 2)
ATTN_BF16(128, 64, 4, 2)

// attn_fwd_bf16_d<D>_bn<BN>_direct[_w2|_w8][_f32scale]: d == dv == D, K/V tiles of BN keys loaded from global memory
// straight into LDS; 4 waves (128 queries) per workgroup, _w2: two waves (64 queries), _w8: eight waves (256
// queries, one workgroup per CU); _f32scale: the score scale is applied in f32 instead of being folded into Q
#define ATTN_BF16_DIRECT(DPAD, BN, NW, OCC, SUFFIX, PRECISE)                                                     \
  extern "C" __global__ void __launch_bounds__(NW * 64, OCC) attn_fwd_bf16_d##DPAD##_bn##BN##_direct##SUFFIX(AttnParams p) { \
    attn_fwd_bf16_direct_body<DPAD, BN, NW, PRECISE>(p);                                                         \
  }
ATTN_BF16_DIRECT(64, 64, 4, 2, , false)
ATTN_BF16_DIRECT(128, 64, 4, 2, , false)
ATTN_BF16_DIRECT(128, 64, 8, 1, _w8, false)
ATTN_BF16_DIRECT(64, 64, 8, 1, _w8, false)
ATTN_BF16_DIRECT(128, 64, 2, 1, _w2, false)
ATTN_BF16_DIRECT(64, 64, 2, 1, _w2, false)
// 32-key tiles (the schedule's j:32)
ATTN_BF16_DIRECT(128, 32, 2, 1, _w2, false)
ATTN_BF16_DIRECT(128, 32, 4, 2, , false)
ATTN_BF16_DIRECT(128, 32, 8, 1, _w8, false)
ATTN_BF16_DIRECT(64, 32, 2, 1, _w2, false)
ATTN_BF16_DIRECT(64, 32, 4, 2, , false)
// f32 score scale
ATTN_BF16_DIRECT(128, 64, 4, 2, _f32scale, true)
ATTN_BF16_DIRECT(128, 64, 8, 1, _w8_f32scale, true)
ATTN_BF16_DIRECT(64, 64, 4, 2, _f32scale, true)
ATTN_BF16_DIRECT(64, 64, 8, 1, _w8_f32scale, true)
// head sizes below DPAD that are multiples of 8: LDS rows padded with zeros
#define ATTN_BF16_DIRECT_PAD(DPAD, BN, NW, OCC, SUFFIX, PRECISE)                                                 \
  extern "C" __global__ void __launch_bounds__(NW * 64, OCC) attn_fwd_bf16_d##DPAD##_bn##BN##_direct##SUFFIX##_pad(AttnParams p) { \
    attn_fwd_bf16_direct_body<DPAD, BN, NW, PRECISE, true>(p);                                                    \
  }
ATTN_BF16_DIRECT_PAD(128, 64, 4, 2, , false)
ATTN_BF16_DIRECT_PAD(128, 64, 8, 1, _w8, false)
ATTN_BF16_DIRECT_PAD(64, 64, 4, 2, , false)
ATTN_BF16_DIRECT_PAD(64, 64, 8, 1, _w8, false)
ATTN_BF16_DIRECT_PAD(128, 64, 4, 2, _f32scale, true)
ATTN_BF16_DIRECT_PAD(128, 64, 8, 1, _w8_f32scale, true)
ATTN_BF16_DIRECT_PAD(64, 64, 4, 2, _f32scale, true)
ATTN_BF16_DIRECT_PAD(64, 64, 8, 1, _w8_f32scale, true)
// head sizes above 128 up to 256: one wave per SIMD (all its registers), 128 query rows per workgroup, 32-key tiles
ATTN_BF16_DIRECT(256, 32, 4, 1, , false)
ATTN_BF16_DIRECT_PAD(256, 32, 4, 1, , false)
ATTN_BF16_DIRECT(256, 32, 4, 1, _f32scale, true)
ATTN_BF16_DIRECT_PAD(256, 32, 4, 1, _f32scale, true)
// d = 64 with 64 queries per wave (two query blocks): 8 waves, 512 query rows per workgroup, 32-key tiles
extern "C" __global__ void __launch_bounds__(512, 1) attn_fwd_bf16_d64_bn32_q64(AttnParams p) {
  attn_fwd_bf16_direct_body<64, 32, 8, false, false, 2>(p);
}

#define ATTN_F32(DPAD, BN, NW)                                                             \
  extern "C" __global__ void __launch_bounds__(NW * 64) attn_fwd_f32_d##DPAD##_bn##BN(AttnParams p) { \
    attn_fwd_f32_body<DPAD, BN, NW>(p);                                                    \
  }
// d == dv in {64, 128}, K and V tiles moved global -> LDS directly (attention_f32_direct.h)
#define ATTN_F32_DIRECT(DPAD)                                                                                   \
  extern "C" __global__ void __launch_bounds__(256, 2) attn_fwd_f32_d##DPAD##_bn32_direct(AttnParams p) {        \
    attn_fwd_f32_direct_body<DPAD, 4>(p);                                                                       \
  }
ATTN_F32_DIRECT(64)
ATTN_F32_DIRECT(128)
// ... head sizes below DPAD that are multiples of 4: LDS rows padded with zeros
#define ATTN_F32_DIRECT_PAD(DPAD)                                                                               \
  extern "C" __global__ void __launch_bounds__(256, 2) attn_fwd_f32_d##DPAD##_bn32_direct_pad(AttnParams p) {    \
    attn_fwd_f32_direct_body<DPAD, 4, true>(p);                                                                 \
  }
ATTN_F32_DIRECT_PAD(64)
ATTN_F32_DIRECT_PAD(128)
ATTN_F32(32, 32, 4)
ATTN_F32(64, 32, 4)
ATTN_F32(128, 32, 4)

extern "C" __global__ void __launch_bounds__(256, 2) gemm_nt_bf16_128x128x64(GemmParams p) {
  gemm_nt_bf16_body<128, 128, 64, 2, 2>(p);
}

extern "C" __global__ void __launch_bounds__(512, 1) gemm_nt_bf16_256x256x64_direct(GemmParams p) {
  gemm_nt_mfma16_body<256, 2, 4>(p);
}
// 128 x 128 tiles, 4 waves, two workgroups per CU: mid-size problems
extern "C" __global__ void __launch_bounds__(256, 2) gemm_nt_bf16_128x128x64_direct(GemmParams p) {
  gemm_nt_mfma16_body<128, 2, 2>(p);
}
// row-major right operand: c[m,n] = sum_k a[m,k] * b[k,n]
extern "C" __global__ void __launch_bounds__(512, 1) gemm_nn_bf16_256x256x64_direct(GemmParams p) {
  gemm_nt_mfma16_body<256, 2, 4, true>(p);
}
extern "C" __global__ void __launch_bounds__(256, 2) gemm_nn_bf16_128x128x64_direct(GemmParams p) {
  gemm_nt_mfma16_body<128, 2, 2, true>(p);
}
// k a multiple of 8 but not of 64: the last slab partial
// ..._w4: the 256 x 256 tile with four waves of 128 x 128 (one per SIMD, its 256 accumulator registers in the
// accumulation file): a third fewer operand reads from LDS per matrix instruction than with eight waves
extern "C" __global__ void __launch_bounds__(256, 1) gemm_nt_bf16_256x256x64_direct_w4(GemmParams p) {
  gemm_nt_mfma16_body<256, 2, 2>(p);
}
extern "C" __global__ void __launch_bounds__(256, 1) gemm_nt_bf16_256x256x64_direct_ktail_w4(GemmParams p) {
  gemm_nt_mfma16_body<256, 2, 2, false, true>(p);
}
// 192 rows of A against 256 rows of B, four waves of 96 x 128 (6 x 8 accumulators): for sizes whose 256 x 256 tiles
// leave a partly empty last round of workgroups (3072^3: 192 of these fill three quarters of the CUs at once,
// where 144 tiles of 256 x 256 fill 56 %; 6144^3: three full rounds instead of 2.25)
extern "C" __global__ void __launch_bounds__(256, 1) gemm_nt_bf16_192x256x64_direct_w4(GemmParams p) {
  gemm_nt_mfma16_body<192, 2, 2, false, false, 256>(p);
}
extern "C" __global__ void __launch_bounds__(256, 1) gemm_nt_bf16_192x256x64_direct_ktail_w4(GemmParams p) {
  gemm_nt_mfma16_body<192, 2, 2, false, true, 256>(p);
}
// ... and 256 rows of A against 192 rows of B (four waves of 128 x 96), for the same sizes when it is n that 256 cuts badly
extern "C" __global__ void __launch_bounds__(256, 1) gemm_nt_bf16_256x192x64_direct_w4(GemmParams p) {
  gemm_nt_mfma16_body<256, 2, 2, false, false, 192>(p);
}
extern "C" __global__ void __launch_bounds__(256, 1) gemm_nt_bf16_256x192x64_direct_ktail_w4(GemmParams p) {
  gemm_nt_mfma16_body<256, 2, 2, false, true, 192>(p);
}
extern "C" __global__ void __launch_bounds__(256, 1) gemm_nn_bf16_256x256x64_direct_w4(GemmParams p) {
  gemm_nt_mfma16_body<256, 2, 2, true>(p);
}
extern "C" __global__ void __launch_bounds__(256, 1) gemm_nn_bf16_256x256x64_direct_ktail_w4(GemmParams p) {
  gemm_nt_mfma16_body<256, 2, 2, true, true>(p);
}
extern "C" __global__ void __launch_bounds__(512, 1) gemm_nt_bf16_256x256x64_direct_ktail(GemmParams p) {
  gemm_nt_mfma16_body<256, 2, 4, false, true>(p);
}
extern "C" __global__ void __launch_bounds__(512, 1) gemm_nn_bf16_256x256x64_direct_ktail(GemmParams p) {
  gemm_nt_mfma16_body<256, 2, 4, true, true>(p);
}
extern "C" __global__ void __launch_bounds__(256, 2) gemm_nt_bf16_128x128x64_direct_ktail(GemmParams p) {
  gemm_nt_mfma16_body<128, 2, 2, false, true>(p);
}
extern "C" __global__ void __launch_bounds__(256, 2) gemm_nn_bf16_128x128x64_direct_ktail(GemmParams p) {
  gemm_nt_mfma16_body<128, 2, 2, true, true>(p);
}
extern "C" __global__ void __launch_bounds__(256, 2) gemm_nt_f32_128x128x32_direct(GemmParams p) {
  gemm_nt_f32_direct_body<128, 2, 2>(p);
}
// f32 operands, f32 MFMA: the arithmetic type of the reference
extern "C" __global__ void __launch_bounds__(512, 1) gemm_nt_f32_256x256x32_direct(GemmParams p) {
  gemm_nt_f32_direct_body<256, 2, 4>(p);
}
// k that is a multiple of 4 but not of 32: the last slab partial
extern "C" __global__ void __launch_bounds__(256, 2) gemm_nt_f32_128x128x32_direct_ktail(GemmParams p) {
  gemm_nt_f32_direct_body<128, 2, 2, true>(p);
}
extern "C" __global__ void __launch_bounds__(512, 1) gemm_nt_f32_256x256x32_direct_ktail(GemmParams p) {
  gemm_nt_f32_direct_body<256, 2, 4, true>(p);
}

// row_<op>_wave_{v,s}<NV>, row_<op>_sub_{v,s}<G>, row_<op>_group_{v,s}<NV> and row_<op>_block[_v] for op = softmax,
// shift (x - row max), norm (x / row sum), exp, scaled_softmax
#define ROW_WAVE(OP, MODE, NV)                                                                     \
  extern "C" __global__ void __launch_bounds__(256) row_##OP##_wave_v##NV(SoftmaxParams p) {       \
    row_softmax_wave_body<NV, true, MODE>(p);                                                      \
  }                                                                                                \
  extern "C" __global__ void __launch_bounds__(256) row_##OP##_wave_s##NV(SoftmaxParams p) {       \
    row_softmax_wave_body<NV, false, MODE>(p);                                                     \
  }
// row_<op>_group_{v,s}<NV>: 8192 < cols <= 4096 * NV, one workgroup of 16 wavefronts per row, row in registers
// (no s16: element-wise loads of 64 values per lane do not fit 128 registers; such rows take the two-pass kernel)
#define ROW_GROUP_V(OP, MODE, NV)                                                                  \
  extern "C" __global__ void __launch_bounds__(1024) row_##OP##_group_v##NV(SoftmaxParams p) {     \
    row_softmax_group_body<NV, true, MODE>(p);                                                     \
  }
#define ROW_GROUP(OP, MODE, NV)                                                                    \
  ROW_GROUP_V(OP, MODE, NV)                                                                        \
  extern "C" __global__ void __launch_bounds__(1024) row_##OP##_group_s##NV(SoftmaxParams p) {     \
    row_softmax_group_body<NV, false, MODE>(p);                                                    \
  }
// row_<op>_sub_{v,s}<G>: cols <= 4 G <= 128, G lanes per row (64 / G rows per wavefront)
#define ROW_SUB(OP, MODE, G)                                                                       \
  extern "C" __global__ void __launch_bounds__(256) row_##OP##_sub_v##G(SoftmaxParams p) {         \
    row_softmax_sub_body<G, true, MODE>(p);                                                        \
  }                                                                                                \
  extern "C" __global__ void __launch_bounds__(256) row_##OP##_sub_s##G(SoftmaxParams p) {         \
    row_softmax_sub_body<G, false, MODE>(p);                                                       \
  }
#define ROW_OP(OP, MODE)                                                                           \
  ROW_WAVE(OP, MODE, 1) ROW_WAVE(OP, MODE, 2) ROW_WAVE(OP, MODE, 4) ROW_WAVE(OP, MODE, 8)          \
  ROW_WAVE(OP, MODE, 16) ROW_WAVE(OP, MODE, 32)                                                    \
  ROW_GROUP(OP, MODE, 4) ROW_GROUP(OP, MODE, 8) ROW_GROUP_V(OP, MODE, 16)                           \
  ROW_SUB(OP, MODE, 1) ROW_SUB(OP, MODE, 2) ROW_SUB(OP, MODE, 4) ROW_SUB(OP, MODE, 8)              \
  ROW_SUB(OP, MODE, 16) ROW_SUB(OP, MODE, 32)                                                      \
  extern "C" __global__ void __launch_bounds__(1024) row_##OP##_block(SoftmaxParams p) {           \
    row_softmax_block_body<MODE, false>(p);                                                        \
  }                                                                                                \
  extern "C" __global__ void __launch_bounds__(1024) row_##OP##_block_v(SoftmaxParams p) {         \
    row_softmax_block_body<MODE, true>(p);                                                         \
  }
#define ROW_PARTS(OP, MODE)                                                                                   \
  extern "C" __global__ void __launch_bounds__(1024) row_##OP##_parts_stats(SoftmaxParams p) {                \
    row_softmax_parts_body<MODE, false, 0>(p);                                                                \
  }                                                                                                           \
  extern "C" __global__ void __launch_bounds__(1024) row_##OP##_parts_stats_v(SoftmaxParams p) {              \
    row_softmax_parts_body<MODE, true, 0>(p);                                                                 \
  }                                                                                                           \
  extern "C" __global__ void __launch_bounds__(1024) row_##OP##_parts_apply(SoftmaxParams p) {                \
    row_softmax_parts_body<MODE, false, 1>(p);                                                                \
  }                                                                                                           \
  extern "C" __global__ void __launch_bounds__(1024) row_##OP##_parts_apply_v(SoftmaxParams p) {              \
    row_softmax_parts_body<MODE, true, 1>(p);                                                                 \
  }
ROW_OP(softmax, 0)
ROW_PARTS(softmax, 0)
ROW_PARTS(scaled_softmax, 4)
ROW_OP(shift, 1)
ROW_OP(norm, 2)
ROW_OP(exp, 3)
ROW_OP(scaled_softmax, 4)  // the middle kernel of attention in three kernels (head sizes above 128)

extern "C" __global__ void __launch_bounds__(256) convert_f32_to_bf16(ConvertParams p) {
  const float* s = reinterpret_cast<const float*>(p.src);
  bf16_t* d = reinterpret_cast<bf16_t*>(p.dst);
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < p.n; i += (uint64_t)gridDim.x * blockDim.x)
    d[i] = (bf16_t)s[i];
}
extern "C" __global__ void __launch_bounds__(256) convert_bf16_to_f32(ConvertParams p) {
  const bf16_t* s = reinterpret_cast<const bf16_t*>(p.src);
  float* d = reinterpret_cast<float*>(p.dst);
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < p.n; i += (uint64_t)gridDim.x * blockDim.x)
    d[i] = (float)s[i];
}

// Batched matrix transpose through a padded 64 x 64 LDS tile (reads and writes both run along rows).  It feeds
// the NT GEMM kernels with the right operand of an NN product.
template <typename T>
__device__ __forceinline__ void transpose_body(const TransposeParams& p) {
  __shared__ T tile[64][65];
  const uint32_t per_batch = p.tiles_r * p.tiles_c;
  const uint32_t b = blockIdx.x / per_batch, t = blockIdx.x % per_batch;
  const uint32_t r0 = (t / p.tiles_c) * 64, c0 = (t % p.tiles_c) * 64;
  const T* src = reinterpret_cast<const T*>(p.src) + (size_t)b * p.rows * p.cols;
  T* dst = reinterpret_cast<T*>(p.dst) + (size_t)b * p.rows * p.cols;
  const uint32_t x = threadIdx.x & 63, y0 = threadIdx.x >> 6;
#pragma unroll 4
  for (uint32_t y = y0; y < 64; y += 4)
    if (r0 + y < p.rows && c0 + x < p.cols) tile[y][x] = src[(size_t)(r0 + y) * p.cols + c0 + x];
  __syncthreads();
#pragma unroll 4
  for (uint32_t y = y0; y < 64; y += 4)
    if (c0 + y < p.cols && r0 + x < p.rows) dst[(size_t)(c0 + y) * p.rows + r0 + x] = tile[x][y];
}
// the partial products of a GEMM whose k loop was split over workgroups, added up in split order
extern "C" __global__ void __launch_bounds__(256) splitk_reduce(SplitReduceParams p) {
  const uint64_t quads = p.count / 4, total = (uint64_t)p.batches * quads;
  for (uint64_t at = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; at < total; at += (uint64_t)gridDim.x * blockDim.x) {
    const uint64_t b = at / quads, i = at - b * quads;
    const f32x4* src = reinterpret_cast<const f32x4*>(p.partial + (size_t)b * p.splits * p.count) + i;
    f32x4 sum = src[0];
#pragma unroll 8
    for (uint32_t s = 1; s < p.splits; ++s) sum += src[(size_t)s * quads];  // (unrolled: eight loads in flight per lane)
    if (p.out_bf16) {
      bf16x4 v;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = (bf16_t)sum[e];
      reinterpret_cast<bf16x4*>(p.out)[at] = v;
    } else {
      reinterpret_cast<f32x4*>(p.out)[at] = sum;
    }
  }
}

// the parts of an attention whose keys were split over workgroups, put together: each part's rows are normalised
// by their own sum of exponentials, whose base-2 logarithm weighs them here (relative to the largest of the row)
extern "C" __global__ void __launch_bounds__(256) attn_kv_merge(AttnMergeParams p) {
  const uint32_t quads = p.dv / 4;
  const uint64_t rows = (uint64_t)p.heads * p.nq, total = rows * quads;
  for (uint64_t at = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; at < total; at += (uint64_t)gridDim.x * blockDim.x) {
    const uint64_t row = at / quads;
    const uint32_t quad = (uint32_t)(at - row * quads);
    const uint64_t head = row / p.nq;
    const uint32_t r = (uint32_t)(row - head * p.nq);
    const float* lse = p.lse + (size_t)head * p.splits * p.nq + r;
    const f32x4* src = reinterpret_cast<const f32x4*>(p.partial + ((size_t)head * p.splits * p.nq + r) * p.dv) + quad;
    float top = lse[0];
    for (uint32_t s = 1; s < p.splits; ++s) top = fmaxf(top, lse[(size_t)s * p.nq]);
    f32x4 sum = {0.0f, 0.0f, 0.0f, 0.0f};
    float weights = 0.0f;
    for (uint32_t s = 0; s < p.splits; ++s) {
      const float w = exp2f(lse[(size_t)s * p.nq] - top);
      weights += w;
      sum += w * src[(size_t)s * p.nq * quads];
    }
    sum *= 1.0f / weights;
    if (p.out_bf16) {
      bf16x4 v;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = (bf16_t)sum[e];
      reinterpret_cast<bf16x4*>(p.out)[at] = v;
    } else {
      reinterpret_cast<f32x4*>(p.out)[at] = sum;
    }
  }
}

// rows copied into rows of cols_padded elements, the tail zeroed: what gives a product whose contracted extent the
// matrix-instruction kernels cannot take (k % 8 != 0 in bf16, k % 4 != 0 in f32) operands they can
template <class T>
__device__ __forceinline__ void pad_rows_body(const PadParams& p) {
  const T* src = reinterpret_cast<const T*>(p.src);
  T* dst = reinterpret_cast<T*>(p.dst);
  const uint64_t total = p.rows * p.cols_padded;
  for (uint64_t at = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; at < total; at += (uint64_t)gridDim.x * blockDim.x) {
    const uint64_t r = at / p.cols_padded;
    const uint32_t c = (uint32_t)(at - r * p.cols_padded);
    dst[at] = c < p.cols ? src[r * p.cols + c] : T(0);
  }
}
extern "C" __global__ void __launch_bounds__(256) pad_rows_b16(PadParams p) { pad_rows_body<uint16_t>(p); }
extern "C" __global__ void __launch_bounds__(256) pad_rows_b32(PadParams p) { pad_rows_body<uint32_t>(p); }

// see ClockProbeParams
extern "C" __global__ void __launch_bounds__(64) shader_clock_probe(ClockProbeParams p) {
  const uint64_t shader0 = __builtin_amdgcn_s_memtime(), constant0 = __builtin_amdgcn_s_memrealtime();
  uint64_t constant1 = constant0;
  // (the loop ends on the constant clock, and after a bounded number of sleeps whatever that clock reads)
  for (uint32_t n = 0; n < (1u << 22) && constant1 - constant0 < p.ticks; ++n) {
    __builtin_amdgcn_s_sleep(64);
    constant1 = __builtin_amdgcn_s_memrealtime();
  }
  const uint64_t shader1 = __builtin_amdgcn_s_memtime();
  if (threadIdx.x == 0) {
    atomicAdd(p.out, (unsigned long long)(shader1 - shader0));
    atomicAdd(p.out + 1, (unsigned long long)(constant1 - constant0));
  }
}

extern "C" __global__ void __launch_bounds__(256) transpose_b16(TransposeParams p) { transpose_body<uint16_t>(p); }
extern "C" __global__ void __launch_bounds__(256) transpose_b32(TransposeParams p) { transpose_body<uint32_t>(p); }

