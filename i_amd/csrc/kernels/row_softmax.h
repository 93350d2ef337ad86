// Row softmax  y[i,:] = exp(x[i,:] - max_i) / sum_j exp(x[i,j] - max_i)  in f32.
//
// Device form of  row_max_shift >> exp >> row_normalize  (README.md:19-25).
// The reference's valid schedules materialise the shifted / exponentiated row
// (three kernels, ilang-python/flash-attn.py:60-62); here the row lives in
// registers, so HBM sees exactly one read and one write per element.
// One wavefront owns one row (a group of lanes for rows of at most 128 columns, a workgroup for rows beyond
// 8192); reductions use cross-lane shuffles, and 16 words of LDS across wavefronts.  Loads and stores are non-temporal: with
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

// Rows of at most 128 columns: G lanes own one row (4 G >= cols, one float4 chunk per lane), so a wavefront
// works on 64 / G rows at once and its loads cover consecutive rows; the reductions are butterflies inside the
// groups of G lanes.  (With a wavefront per row, a row of 16 columns occupied 4 lanes of 64.)
template <int G, bool VEC, int MODE>
__device__ __forceinline__ void row_softmax_sub_body(const SoftmaxParams& p) {
  const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const uint64_t row = gid / G;
  const uint32_t col = 4u * (uint32_t)(gid % G);
  const bool live = row < p.rows;  // lanes of rows past the end take part in the exchanges with neutral values
  const float* __restrict__ x = p.x + row * p.cols;
  float* __restrict__ y = p.y + row * p.cols;
  const float pad = MODE == 2 ? 0.0f : -INFINITY;
  const float sc = MODE == 4 ? load_scale(p.scale_ptr, p.scale_value) : 1.0f;
  f32x4 r = {pad, pad, pad, pad};
  if (live) {
    if (VEC) {
      if (col < p.cols) {
        r = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(x + col));
        if constexpr (MODE == 4) r *= sc;
      }
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (col + e < p.cols) r[e] = MODE == 4 ? x[col + e] * sc : x[col + e];
    }
  }
  auto store = [&](f32x4 v) {
    if (!live) return;
    if (VEC) {
      if (col < p.cols) __builtin_nontemporal_store(v, reinterpret_cast<f32x4*>(y + col));
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (col + e < p.cols) y[col + e] = v[e];
    }
  };
  auto group_max = [](float v) {
#pragma unroll
    for (int o = G / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
  };
  auto group_sum = [](float v) {
#pragma unroll
    for (int o = G / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
  };
  if constexpr (MODE == 3) {
    f32x4 v;
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = fast_exp2(r[e] * I_LOG2_E32);
    store(v);
    return;
  }
  if constexpr (MODE == 2) {
    const float total = group_sum((r[0] + r[1]) + (r[2] + r[3]));
    store(r / total);
    return;
  }
  const float mx = group_max(fmaxf(fmaxf(r[0], r[1]), fmaxf(r[2], r[3])));
  if constexpr (MODE == 1) {
    store(r - mx);
    return;
  }
  const float mb = mx * I_LOG2_E32;
  float sum = 0.0f;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    r[e] = fast_exp2(__builtin_fmaf(r[e], I_LOG2_E32, -mb));
    sum += r[e];
  }
  sum = group_sum(sum);
  store(r * (1.0f / sum));
}

// Any width (rows beyond what a workgroup's registers hold): one workgroup of 16 wavefronts per row and two
// passes over it.  The first pass takes the row max and the row sum together: every lane keeps a running max m
// and the sum of exp(x - m) over what it has seen, rescaling the sum when its max moves, and lanes, then
// wavefronts, combine their (m, sum) pairs the same way; the second pass writes.  HBM sees the row twice on the
// way in at most (the second read of a row of a few hundred KiB comes out of the caches) and once on the way out.
// VEC: cols % 4 == 0 and 16-byte aligned rows, float4 accesses.
template <int MODE, bool VEC>
__device__ __forceinline__ void row_softmax_block_body(const SoftmaxParams& p) {
  __shared__ float red[2][16];
  const uint32_t row = blockIdx.x;
  const float* __restrict__ x = p.x + (size_t)row * p.cols;
  float* __restrict__ y = p.y + (size_t)row * p.cols;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  constexpr int W = VEC ? 4 : 1;                    // elements per access
  const uint32_t chunks = VEC ? p.cols / 4 : p.cols;
  auto load = [&](uint32_t c) {
    f32x4 v;
    if constexpr (VEC) v = *reinterpret_cast<const f32x4*>(x + 4 * (size_t)c);
    else v[0] = x[c];
    return v;
  };
  auto store = [&](uint32_t c, f32x4 v) {
    if constexpr (VEC) __builtin_nontemporal_store(v, reinterpret_cast<f32x4*>(y + 4 * (size_t)c));
    else y[c] = v[0];
  };
  if constexpr (MODE == 3) {  // exp(x), elementwise
#pragma unroll 4
    for (uint32_t c = threadIdx.x; c < chunks; c += blockDim.x) {
      f32x4 v = load(c);
#pragma unroll
      for (int e = 0; e < W; ++e) v[e] = fast_exp2(v[e] * I_LOG2_E32);
      store(c, v);
    }
    return;
  }
  // the reduction of a per-lane value over the workgroup (every lane gets it), wavefront partials in order
  auto over_workgroup = [&](float v, auto combine) {
    if (lane == 0) red[0][wave] = v;
    __syncthreads();
    float total = red[0][0];
    for (int w = 1; w < nw; ++w) total = combine(total, red[0][w]);
    return total;
  };
  if constexpr (MODE == 2) {  // row_normalize
    float total = 0.0f;
#pragma unroll 4
    for (uint32_t c = threadIdx.x; c < chunks; c += blockDim.x) {
      const f32x4 v = load(c);
#pragma unroll
      for (int e = 0; e < W; ++e) total += v[e];
    }
    total = over_workgroup(wave_sum(total), [](float a, float b) { return a + b; });
#pragma unroll 4
    for (uint32_t c = threadIdx.x; c < chunks; c += blockDim.x) {
      f32x4 v = load(c);
#pragma unroll
      for (int e = 0; e < W; ++e) v[e] = v[e] / total;
      store(c, v);
    }
    return;
  }
  if constexpr (MODE == 1) {  // row_max_shift
    float mx = -INFINITY;
#pragma unroll 4
    for (uint32_t c = threadIdx.x; c < chunks; c += blockDim.x) {
      const f32x4 v = load(c);
#pragma unroll
      for (int e = 0; e < W; ++e) mx = fmaxf(mx, v[e]);
    }
    mx = over_workgroup(wave_max(mx), [](float a, float b) { return fmaxf(a, b); });
#pragma unroll 4
    for (uint32_t c = threadIdx.x; c < chunks; c += blockDim.x) {
      f32x4 v = load(c);
#pragma unroll
      for (int e = 0; e < W; ++e) v[e] -= mx;
      store(c, v);
    }
    return;
  }
  const float sc = MODE == 4 ? load_scale(p.scale_ptr, p.scale_value) : 1.0f;  // mode 4: softmax(scale * x)
  // (m, s): the running max of t = scale * x * log2(e) and the sum of exp2(t - m) over the elements seen
  float m = -INFINITY, s = 0.0f;
  auto weight = [](float from, float to) { return from == to ? 1.0f : fast_exp2(from - to); };  // (-inf to -inf: nothing seen yet)
  auto merge = [&](float& ma, float& sa, float mb, float sb) {
    const float mn = fmaxf(ma, mb);
    sa = sa * weight(ma, mn) + sb * weight(mb, mn);
    ma = mn;
  };
#pragma unroll 4
  for (uint32_t c = threadIdx.x; c < chunks; c += blockDim.x) {
    f32x4 v = load(c);
    float cm = -INFINITY;
#pragma unroll
    for (int e = 0; e < W; ++e) {
      v[e] = v[e] * sc * I_LOG2_E32;
      cm = fmaxf(cm, v[e]);
    }
    const float mn = fmaxf(m, cm);
    s *= weight(m, mn);
#pragma unroll
    for (int e = 0; e < W; ++e) s += fast_exp2(v[e] - mn);
    m = mn;
  }
  // lanes, then wavefronts
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float mo = __shfl_xor(m, o, 64), so = __shfl_xor(s, o, 64);
    merge(m, s, mo, so);
  }
  if (lane == 0) {
    red[0][wave] = m;
    red[1][wave] = s;
  }
  __syncthreads();
  m = red[0][0];
  s = red[1][0];
  for (int w = 1; w < nw; ++w) merge(m, s, red[0][w], red[1][w]);
  const float inv = 1.0f / s;
#pragma unroll 4
  for (uint32_t c = threadIdx.x; c < chunks; c += blockDim.x) {
    f32x4 v = load(c);
#pragma unroll
    for (int e = 0; e < W; ++e) v[e] = fast_exp2(v[e] * sc * I_LOG2_E32 - m) * inv;
    store(c, v);
  }
}

// A row in parts over workgroups, for softmax of a few very long rows (fewer rows than CUs): workgroup (row, part)
// takes the accesses part_chunks * part .. + part_chunks of its row.  PASS 0 computes the part's (m, s) pair as
// the block kernel's first pass does and stores it; PASS 1 (a second launch) combines the pairs of its row in part
// order and writes its part of the result.  HBM sees the row twice on the way in, once on the way out.
template <int MODE, bool VEC, int PASS>
__device__ __forceinline__ void row_softmax_parts_body(const SoftmaxParams& p) {
  static_assert(MODE == 0 || MODE == 4, "softmax only");
  __shared__ float red[2][16];
  const uint32_t row = blockIdx.x / p.parts, part = blockIdx.x - row * p.parts;
  const float* __restrict__ x = p.x + (size_t)row * p.cols;
  float* __restrict__ y = p.y + (size_t)row * p.cols;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  constexpr int W = VEC ? 4 : 1;
  const uint32_t chunks = VEC ? p.cols / 4 : p.cols;
  const uint32_t first = part * p.part_chunks, last = first + p.part_chunks < chunks ? first + p.part_chunks : chunks;
  auto load = [&](uint32_t c) {
    f32x4 v;
    if constexpr (VEC) v = *reinterpret_cast<const f32x4*>(x + 4 * (size_t)c);
    else v[0] = x[c];
    return v;
  };
  const float sc = MODE == 4 ? load_scale(p.scale_ptr, p.scale_value) : 1.0f;
  auto weight = [](float from, float to) { return from == to ? 1.0f : fast_exp2(from - to); };
  auto merge = [&](float& ma, float& sa, float mb, float sb) {
    const float mn = fmaxf(ma, mb);
    sa = sa * weight(ma, mn) + sb * weight(mb, mn);
    ma = mn;
  };
  float* stats = p.stats + (size_t)row * p.parts * 2;
  if constexpr (PASS == 0) {
    float m = -INFINITY, s = 0.0f;
#pragma unroll 4
    for (uint32_t c = first + threadIdx.x; c < last; c += blockDim.x) {
      f32x4 v = load(c);
      float cm = -INFINITY;
#pragma unroll
      for (int e = 0; e < W; ++e) {
        v[e] = v[e] * sc * I_LOG2_E32;
        cm = fmaxf(cm, v[e]);
      }
      const float mn = fmaxf(m, cm);
      s *= weight(m, mn);
#pragma unroll
      for (int e = 0; e < W; ++e) s += fast_exp2(v[e] - mn);
      m = mn;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float mo = __shfl_xor(m, o, 64), so = __shfl_xor(s, o, 64);
      merge(m, s, mo, so);
    }
    if (lane == 0) {
      red[0][wave] = m;
      red[1][wave] = s;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      m = red[0][0];
      s = red[1][0];
      for (int w = 1; w < nw; ++w) merge(m, s, red[0][w], red[1][w]);
      stats[2 * part] = m;
      stats[2 * part + 1] = s;
    }
  } else {
    float m = stats[0], s = stats[1];
    for (uint32_t t = 1; t < p.parts; ++t) merge(m, s, stats[2 * t], stats[2 * t + 1]);
    const float inv = 1.0f / s;
#pragma unroll 4
    for (uint32_t c = first + threadIdx.x; c < last; c += blockDim.x) {
      f32x4 v = load(c);
#pragma unroll
      for (int e = 0; e < W; ++e) v[e] = fast_exp2(v[e] * sc * I_LOG2_E32 - m) * inv;
      if constexpr (VEC) __builtin_nontemporal_store(v, reinterpret_cast<f32x4*>(y + 4 * (size_t)c));
      else y[c] = v[0];
    }
  }
}

