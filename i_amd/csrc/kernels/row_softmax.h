// Row softmax  y[i,:] = exp(x[i,:] - max_i) / sum_j exp(x[i,j] - max_i)  in f32.
//
// Device form of  row_max_shift >> exp >> row_normalize  (README.md:19-25).
// The reference's valid schedules materialise the shifted / exponentiated row
// (three kernels, ilang-python/flash-attn.py:60-62); here the row lives in
// registers, so HBM sees exactly one read and one write per element.
// One wavefront owns one row; reductions use cross-lane shuffles only.  Loads and stores are non-temporal: with
// ordinary loads the kernel looks 12 % faster when it is timed on one buffer over and over (the input then comes
// partly out of the 256 MiB Infinity Cache) and is 6 % slower on inputs that really come from HBM.
//
// The same kernels also run the two halves on their own (template parameter MODE), which is how the reference's
// naive three-kernel schedule reaches them:  row_max_shift  y = x - max_j x  (flash-attn.py:60) and
// row_normalize  y = x / sum_j x  (flash-attn.py:62); and the elementwise exp between them (flash-attn.py:61, mode 3)
// with the exponential the fused form uses.
#pragma once
#include "common.h"
#include "params.h"

// NV = float4 chunks per lane; covers cols <= 256 * NV.  VEC: cols % 4 == 0.
// MODE (0 softmax, 1 x - max, 2 x / sum, 3 exp, 4 softmax of scale * x) is a template parameter: as a run-time switch the four bodies
// cost the softmax a third of its registers' worth of occupancy and 13 % of its bandwidth.
template <int NV, bool VEC, int MODE>
__device__ __forceinline__ void row_softmax_wave_body(const SoftmaxParams& p) {
  const int lane = threadIdx.x & 63;
  const uint32_t row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (row >= p.rows) return;
  const float* __restrict__ x = p.x + (size_t)row * p.cols;
  float* __restrict__ y = p.y + (size_t)row * p.cols;

  f32x4 r[NV];
  float mx = -INFINITY;
  const float pad = MODE == 2 ? 0.0f : -INFINITY;  // neutral for the reduction of the mode
  const float sc = MODE == 4 ? load_scale(p.scale_ptr, p.scale_value) : 1.0f;  // mode 4: softmax(scale * x)
#pragma unroll
  for (int t = 0; t < NV; ++t) {
    const uint32_t col = 4u * (lane + 64 * t);
    if (VEC) {
      if (col < p.cols) {
        r[t] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(x + col));
        if constexpr (MODE == 4) r[t] *= sc;
      } else {
        r[t] = f32x4{pad, pad, pad, pad};
      }
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) r[t][e] = (col + e < p.cols) ? (MODE == 4 ? x[col + e] * sc : x[col + e]) : pad;
    }
    mx = fmaxf(fmaxf(fmaxf(r[t][0], r[t][1]), fmaxf(r[t][2], r[t][3])), mx);
  }
  if constexpr (MODE == 3) {  // exp(x), elementwise
#pragma unroll
    for (int t = 0; t < NV; ++t) {
      const uint32_t col = 4u * (lane + 64 * t);
      f32x4 v;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = fast_exp2(r[t][e] * I_LOG2_E32);
      if (VEC) {
        if (col < p.cols) __builtin_nontemporal_store(v, reinterpret_cast<f32x4*>(y + col));
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (col + e < p.cols) y[col + e] = v[e];
      }
    }
    return;
  }
  if constexpr (MODE == 2) {  // row_normalize: x / sum(x)
    float total = 0.0f;
#pragma unroll
    for (int t = 0; t < NV; ++t) total += (r[t][0] + r[t][1]) + (r[t][2] + r[t][3]);
    total = wave_sum(total);
    // a true division per element, as the reference's `a / b`: the kernel is HBM-bound either way
#pragma unroll
    for (int t = 0; t < NV; ++t) {
      const uint32_t col = 4u * (lane + 64 * t);
      if (VEC) {
        if (col < p.cols) __builtin_nontemporal_store(r[t] / total, reinterpret_cast<f32x4*>(y + col));
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (col + e < p.cols) y[col + e] = r[t][e] / total;
      }
    }
    return;
  }
  mx = wave_max(mx);
  if constexpr (MODE == 1) {  // row_max_shift: x - max(x)
#pragma unroll
    for (int t = 0; t < NV; ++t) {
      const uint32_t col = 4u * (lane + 64 * t);
      if (VEC) {
        if (col < p.cols) __builtin_nontemporal_store(r[t] - mx, reinterpret_cast<f32x4*>(y + col));
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (col + e < p.cols) y[col + e] = r[t][e] - mx;
      }
    }
    return;
  }
  const float mb = mx * I_LOG2_E32;
  float sum = 0.0f;
#pragma unroll
  for (int t = 0; t < NV; ++t)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float v = fast_exp2(__builtin_fmaf(r[t][e], I_LOG2_E32, -mb));
      r[t][e] = v;
      sum += v;
    }
  sum = wave_sum(sum);
  const float inv = 1.0f / sum;
#pragma unroll
  for (int t = 0; t < NV; ++t) {
    const uint32_t col = 4u * (lane + 64 * t);
    if (VEC) {
      if (col < p.cols) __builtin_nontemporal_store(r[t] * inv, reinterpret_cast<f32x4*>(y + col));
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (col + e < p.cols) y[col + e] = r[t][e] * inv;
    }
  }
}

// Rows of 8192 < cols <= 65536: one workgroup of 16 wavefronts owns one row, which still lives in registers
// (NV float4 chunks per lane, cols <= 4096 * NV), so HBM again sees one read and one write per element; the row
// max and the row sum cross the wavefronts through 16 words of LDS.
template <int NV, bool VEC, int MODE>
__device__ __forceinline__ void row_softmax_group_body(const SoftmaxParams& p) {
  constexpr int NW = 16;
  __shared__ float red[2][NW];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint32_t row = blockIdx.x;
  const float* __restrict__ x = p.x + (size_t)row * p.cols;
  float* __restrict__ y = p.y + (size_t)row * p.cols;

  f32x4 r[NV];
  float mx = -INFINITY;
  const float pad = MODE == 2 ? 0.0f : -INFINITY;  // neutral for the reduction of the mode
  const float sc = MODE == 4 ? load_scale(p.scale_ptr, p.scale_value) : 1.0f;  // mode 4: softmax(scale * x)
#pragma unroll
  for (int t = 0; t < NV; ++t) {
    const uint32_t col = 4u * (tid + 64 * NW * t);
    if (VEC) {
      if (col < p.cols) {
        r[t] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(x + col));
        if constexpr (MODE == 4) r[t] *= sc;
      } else {
        r[t] = f32x4{pad, pad, pad, pad};
      }
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) r[t][e] = (col + e < p.cols) ? (MODE == 4 ? x[col + e] * sc : x[col + e]) : pad;
    }
    mx = fmaxf(fmaxf(fmaxf(r[t][0], r[t][1]), fmaxf(r[t][2], r[t][3])), mx);
  }
  auto store = [&](int t, f32x4 v) {
    const uint32_t col = 4u * (tid + 64 * NW * t);
    if (VEC) {
      if (col < p.cols) __builtin_nontemporal_store(v, reinterpret_cast<f32x4*>(y + col));
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (col + e < p.cols) y[col + e] = v[e];
    }
  };
  // every lane gets the reduction over the 16 wavefronts' partial results, combined in wavefront order
  auto across_waves = [&](float v, int slot, auto combine) {
    if (lane == 0) red[slot][wave] = v;
    __syncthreads();
    float total = red[slot][0];
#pragma unroll
    for (int w = 1; w < NW; ++w) total = combine(total, red[slot][w]);
    return total;
  };
  if constexpr (MODE == 3) {  // exp(x), elementwise
#pragma unroll
    for (int t = 0; t < NV; ++t) {
      f32x4 v;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = fast_exp2(r[t][e] * I_LOG2_E32);
      store(t, v);
    }
    return;
  }
  if constexpr (MODE == 2) {  // row_normalize: x / sum(x)
    float total = 0.0f;
#pragma unroll
    for (int t = 0; t < NV; ++t) total += (r[t][0] + r[t][1]) + (r[t][2] + r[t][3]);
    total = across_waves(wave_sum(total), 0, [](float a, float b) { return a + b; });
#pragma unroll
    for (int t = 0; t < NV; ++t) store(t, r[t] / total);
    return;
  }
  mx = across_waves(wave_max(mx), 0, [](float a, float b) { return fmaxf(a, b); });
  if constexpr (MODE == 1) {  // row_max_shift: x - max(x)
#pragma unroll
    for (int t = 0; t < NV; ++t) store(t, r[t] - mx);
    return;
  }
  const float mb = mx * I_LOG2_E32;
  float sum = 0.0f;
#pragma unroll
  for (int t = 0; t < NV; ++t)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float v = fast_exp2(__builtin_fmaf(r[t][e], I_LOG2_E32, -mb));
      r[t][e] = v;
      sum += v;
    }
  sum = across_waves(wave_sum(sum), 1, [](float a, float b) { return a + b; });
  const float inv = 1.0f / sum;
#pragma unroll
  for (int t = 0; t < NV; ++t) store(t, r[t] * inv);
}

// Any width: one workgroup per row, three passes over the row (max, sum, write).
template <int MODE>
__device__ __forceinline__ void row_softmax_block_body(const SoftmaxParams& p) {
  __shared__ float red[16];
  const uint32_t row = blockIdx.x;
  const float* __restrict__ x = p.x + (size_t)row * p.cols;
  float* __restrict__ y = p.y + (size_t)row * p.cols;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  if constexpr (MODE == 3) {  // exp(x), elementwise
    for (uint32_t j = threadIdx.x; j < p.cols; j += blockDim.x) y[j] = fast_exp2(x[j] * I_LOG2_E32);
    return;
  }
  if constexpr (MODE == 2) {  // row_normalize
    float total = 0.0f;
    for (uint32_t j = threadIdx.x; j < p.cols; j += blockDim.x) total += x[j];
    total = wave_sum(total);
    if (lane == 0) red[wave] = total;
    __syncthreads();
    total = 0.0f;
    for (int w = 0; w < nw; ++w) total += red[w];
    for (uint32_t j = threadIdx.x; j < p.cols; j += blockDim.x) y[j] = x[j] / total;
    return;
  }
  const float sc = MODE == 4 ? load_scale(p.scale_ptr, p.scale_value) : 1.0f;  // mode 4: softmax(scale * x)
  float mx = -INFINITY;
  for (uint32_t j = threadIdx.x; j < p.cols; j += blockDim.x) mx = fmaxf(mx, x[j] * sc);
  mx = wave_max(mx);
  if (lane == 0) red[wave] = mx;
  __syncthreads();
  mx = red[0];
  for (int w = 1; w < nw; ++w) mx = fmaxf(mx, red[w]);
  __syncthreads();
  if constexpr (MODE == 1) {  // row_max_shift
    for (uint32_t j = threadIdx.x; j < p.cols; j += blockDim.x) y[j] = x[j] - mx;
    return;
  }
  const float mb = mx * I_LOG2_E32;
  float sum = 0.0f;
  for (uint32_t j = threadIdx.x; j < p.cols; j += blockDim.x) sum += fast_exp2(__builtin_fmaf(x[j] * sc, I_LOG2_E32, -mb));
  sum = wave_sum(sum);
  if (lane == 0) red[wave] = sum;
  __syncthreads();
  sum = 0.0f;
  for (int w = 0; w < nw; ++w) sum += red[w];
  const float inv = 1.0f / sum;
  for (uint32_t j = threadIdx.x; j < p.cols; j += blockDim.x)
    y[j] = fast_exp2(__builtin_fmaf(x[j] * sc, I_LOG2_E32, -mb)) * inv;
}
