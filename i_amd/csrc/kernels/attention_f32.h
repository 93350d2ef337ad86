// FlashAttention forward for f32 inputs (full f32 arithmetic) on gfx950.
//
// Same fused nest and the same lane mapping as the bf16 kernel (one query per
// lane, S^T and O^T accumulators), with v_mfma_f32_32x32x2_f32 so that products
// and sums stay in IEEE f32 as in the reference C backend
// (ilang-python/annotated-flashattn.c:52-310).  Arbitrary d, dv <= DPAD and
// arbitrary nq, nk (tail guards as in the reference's `tile*F + inner < dim`).
#pragma once
#include "common.h"
#include "params.h"

template <int DPAD, int BN>
struct AttnF32Smem {
  static constexpr int KS = DPAD + 1;  // odd stride: lanes of one half-wave hit distinct banks
  static constexpr int VS = DPAD + 4;
  float k[BN * KS];
  float v[BN * VS];
};

template <int DPAD, int BN, int NWAVES>
__device__ __forceinline__ void attn_fwd_f32_body(const AttnParams& p) {
  constexpr int NT = NWAVES * WAVE;
  constexpr int BM = 32 * NWAVES;
  constexpr int KSTEPS = DPAD / 2;
  constexpr int KT = BN / 32;
  constexpr int DT = DPAD / 32;
  using Smem = AttnF32Smem<DPAD, BN>;
  __shared__ __attribute__((aligned(16))) Smem sm;

  uint32_t head, qt;
  xcd_map(blockIdx.x, p.nqt, p.bh, head, qt);
  if (head >= p.bh) return;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int c = lane & 31;
  const int h = lane >> 5;

  const float* __restrict__ Q = reinterpret_cast<const float*>(p.q) + (size_t)head * p.nq * p.d;
  const float* __restrict__ K = reinterpret_cast<const float*>(p.k) + (size_t)head * p.nk * p.d;
  const float* __restrict__ V = reinterpret_cast<const float*>(p.v) + (size_t)head * p.nk * p.dv;

  const float scale_raw = load_scale(p.scale_ptr, p.scale_value);
  const float qsign = scale_raw < 0.0f ? -1.0f : 1.0f;  // negative scale folded into Q
  const float scale_log2 = fabsf(scale_raw) * I_LOG2_E32;

  const uint32_t qrow = qt * BM + wave * 32 + c;
  float qf[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) {
    const uint32_t col = 2 * ks + h;
    qf[ks] = (qrow < p.nq && col < p.d) ? qsign * Q[(size_t)qrow * p.d + col] : 0.0f;
  }

  f32x16 o[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[t][i] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;

  const uint32_t ntiles = (p.nk + BN - 1) / BN;
  for (uint32_t j = 0; j < ntiles; ++j) {
    const uint32_t key0 = j * BN;
    for (int idx = tid; idx < BN * DPAD; idx += NT) {
      const int row = idx / DPAD, col = idx % DPAD;
      const bool okr = key0 + row < p.nk;
      sm.k[row * Smem::KS + col] = (okr && (uint32_t)col < p.d) ? K[(size_t)(key0 + row) * p.d + col] : 0.0f;
      sm.v[row * Smem::VS + col] = (okr && (uint32_t)col < p.dv) ? V[(size_t)(key0 + row) * p.dv + col] : 0.0f;
    }
    __syncthreads();

    f32x16 s[KT];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int i = 0; i < 16; ++i) s[kt][i] = 0.0f;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks)
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) {
        const float a = sm.k[(32 * kt + c) * Smem::KS + 2 * ks + h];
        s[kt] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, qf[ks], s[kt], 0, 0, 0);
      }

    if (key0 + BN > p.nk) {
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const uint32_t key = key0 + 32 * kt + 8 * (i >> 2) + 4 * h + (i & 3);
          if (key >= p.nk) s[kt][i] = -INFINITY;
        }
    }

    float mx = s[0][0];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[kt][i]);
    mx = fmaxf(mx, xhalf(mx));
    const float m_new = fmaxf(m_run, mx);
    const float alpha = m_run == -INFINITY ? 0.0f : fast_exp2((m_run - m_new) * scale_log2);
    const float mb = m_new * scale_log2;
    m_run = m_new;

    float psum = 0.0f;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float e = fast_exp2(__builtin_fmaf(s[kt][i], scale_log2, -mb));
        s[kt][i] = e;
        psum += e;
      }
    // keys past nk take no weight (spelled out rather than left to exp(-inf): a zero scale
    // turns the masked score into 0 * inf)
    if (key0 + BN > p.nk) {
      psum = 0.0f;
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const uint32_t key = key0 + 32 * kt + 8 * (i >> 2) + 4 * h + (i & 3);
          if (key >= p.nk) s[kt][i] = 0.0f;
          psum += s[kt][i];
        }
    }
    l_run = l_run * alpha + psum;

#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[t][i] *= alpha;

    // O^T += V^T P^T, one key per k-slot: lane half h supplies key 8(i/4)+4h+i%4.
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int key = 32 * kt + 8 * (i >> 2) + 4 * h + (i & 3);
#pragma unroll
        for (int t = 0; t < DT; ++t) {
          const float a = sm.v[key * Smem::VS + 32 * t + c];
          o[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, s[kt][i], o[t], 0, 0, 0);
        }
      }
    __syncthreads();
  }

  const float l_tot = l_run + xhalf(l_run);
  const float inv = 1.0f / l_tot;
  if (qrow < p.nq) {
    float* O = reinterpret_cast<float*>(p.o) + ((size_t)head * p.nq + qrow) * p.dv;
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const uint32_t col = 32 * t + 8 * (i >> 2) + 4 * h + (i & 3);
        if (col < p.dv) O[col] = o[t][i] * inv;
      }
  }
}
