// FlashAttention forward for bf16 inputs with f32 accumulation (gfx950).
//
// This is the device form of the fused loop nest that the 𝚒 schedule
//   mm_t >> [scale] >> row_max_shift >> exp >> row_normalize >> mm
// lowers to (reference emission: ilang-python/annotated-flashattn.c:52-310):
// the K/V tile loop `j` is the outer sequential loop, the score tile and the
// probability tile never leave the chip (storage folding), and the row max /
// row sum are carried as running values with exp-shift corrections applied to
// the sum and to the output accumulator (online-reduction rewriting).
//
// Mapping to the machine
//   workgroup  = one query tile of BM = 32 * NWAVES rows of one (batch, head)
//   wavefront  = 32 query rows; every lane owns ONE query (lane & 31), the two
//                half-waves own disjoint key subsets
//   QK^T       = computed transposed, S^T = K_tile * Q^T, with
//                v_mfma_f32_32x32x16_bf16: A = K rows from LDS, B = Q^T held in
//                registers for the whole kernel.  In the accumulator layout a
//                lane then holds 16 keys of its own query, so the row max and
//                row sum are in-lane reductions plus one half-wave exchange.
//   PV         = O^T += V_tile^T * P^T: the S^T accumulators, rounded to bf16,
//                are already in B-operand layout (keys x query); A = V^T read
//                from an LDS tile that was transposed while being staged.
//   running m/l = one scalar per lane; the output rescale is a lane-scalar
//                multiply of the O^T accumulators.
// The per-tile normalisation the reference emits (P/l and O*l_old/l) is
// algebraically the deferred form used here: O = (sum_j e^{s_j-m} v_j) / l.
#pragma once
#include <type_traits>

#include "common.h"
#include "params.h"

template <int DPAD, int BN>
struct AttnBf16Smem {
  static constexpr int KS = DPAD + 8;  // K tile row stride (elements); +16 B keeps b128 reads conflict-free
  static constexpr int VS = BN + 8;    // V^T tile row stride
  bf16_t k[2][BN * KS];
  bf16_t vt[2][DPAD * VS];
};

// EXACT: d == dv == DPAD, so no column guards are needed anywhere.
template <int DPAD, int BN, int NWAVES, bool EXACT>
__device__ __forceinline__ void attn_fwd_bf16_body(const AttnParams& p) {
  constexpr int NT = NWAVES * WAVE;
  constexpr int BM = 32 * NWAVES;
  constexpr int KSTEPS = DPAD / 16;  // k-steps of the QK^T contraction
  constexpr int KT = BN / 32;        // 32-key accumulator tiles
  constexpr int DT = DPAD / 32;      // 32-column output tiles
  constexpr int CH = DPAD / 8;       // 16-byte chunks per K/V row
  constexpr int K_ITERS = (BN * CH + NT - 1) / NT;
  constexpr int V_TASKS = (BN / 4) * CH;  // (4 keys) x (8 columns) blocks
  constexpr int V_ITERS = (V_TASKS + NT - 1) / NT;
  static_assert((BN * CH) % NT == 0 || K_ITERS == 1, "K staging assumes whole iterations");
  using Smem = AttnBf16Smem<DPAD, BN>;
  __shared__ __attribute__((aligned(16))) Smem sm;

  uint32_t head, qt;
  xcd_map(blockIdx.x, p.nqt, p.bh, head, qt);
  if (head >= p.bh) return;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int c = lane & 31;  // query column within the wave / A-operand row
  const int h = lane >> 5;  // half-wave
  const uint32_t d = EXACT ? DPAD : p.d;
  const uint32_t dv = EXACT ? DPAD : p.dv;

  const bf16_t* __restrict__ Q = reinterpret_cast<const bf16_t*>(p.q) + (size_t)head * p.nq * d;
  const bf16_t* __restrict__ K = reinterpret_cast<const bf16_t*>(p.k) + (size_t)head * p.nk * d;
  const bf16_t* __restrict__ V = reinterpret_cast<const bf16_t*>(p.v) + (size_t)head * p.nk * dv;

  // A negative scale is folded into Q (sign flip is exact), so the running max
  // can be tracked on the raw scores: max_j(s_j * scale) == scale * max_j(s_j).
  const float scale_raw = load_scale(p.scale_ptr, p.scale_value);
  const uint32_t sign_flip = scale_raw < 0.0f ? 0x80008000u : 0u;
  const float scale_log2 = fabsf(scale_raw) * I_LOG2_E32;

  // Q^T fragments (B operand): lane (c, h) holds q[row][16*ks + 8*h .. +8].
  const uint32_t qrow = qt * BM + wave * 32 + c;
  bf16x8 qf[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) {
    u32x4 z = {0, 0, 0, 0};
    const uint32_t col = 16 * ks + 8 * h;
    if (qrow < p.nq && (EXACT || col < d)) z = ldg128(Q + (size_t)qrow * d + col);
    z ^= sign_flip;
    qf[ks] = __builtin_bit_cast(bf16x8, z);
  }

  f32x16 o[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[t][i] = 0.0f;
  float m_run = -INFINITY;  // running max of the raw scores
  float l_run = 0.0f;       // running sum over this half-wave's keys

  u32x4 kreg[K_ITERS];
  u32x4 vreg[V_ITERS][4];

  // Staging addresses: a wave-uniform base (scalar registers) plus one 32-bit per-lane offset.
  static_assert(NT % CH == 0, "a staging iteration covers whole rows");
  constexpr int ROWS_PER_IT = NT / CH;
  const uint32_t krow0 = tid / CH, kch = tid % CH;
  const uint32_t koff = krow0 * d + 8 * kch;
  // V is staged as (4 keys) x (8 columns) blocks.  The key group varies fastest across lanes:
  // the 16 lanes that share a column block then write one contiguous 128-byte run of a V^T row
  // (no LDS bank conflicts); the price is 16-byte global loads from 16 different rows per quarter wave.
  constexpr int VG = BN / 4;  // key groups per tile
  static_assert(NT % VG == 0, "a staging iteration covers whole column blocks");
  constexpr int VCH_PER_IT = NT / VG;
  const uint32_t vg = tid % VG, vch0 = tid / VG;
  const uint32_t voff = 4 * vg * dv + 8 * vch0;

  // MASKED: the tile may run past nk (or past d / dv when !EXACT): guard every load.
  auto load_tile = [&](uint32_t key0, auto masked_tag) {
    constexpr bool MASKED = decltype(masked_tag)::value;
#pragma unroll
    for (int it = 0; it < K_ITERS; ++it) {
      const bf16_t* base = K + (size_t)(key0 + it * ROWS_PER_IT) * d;
      if constexpr (MASKED || !EXACT) {
        u32x4 z = {0, 0, 0, 0};
        if (tid + it * NT < BN * CH && key0 + it * ROWS_PER_IT + krow0 < p.nk && 8u * kch < d) z = ldg128(base + koff);
        kreg[it] = z;
      } else {
        kreg[it] = ldg128(base + koff);
      }
    }
#pragma unroll
    for (int it = 0; it < V_ITERS; ++it) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const bf16_t* base = V + (size_t)(key0 + r) * dv + 8 * it * VCH_PER_IT;
        if constexpr (MASKED || !EXACT || (V_TASKS % NT) != 0) {
          u32x4 z = {0, 0, 0, 0};
          if (tid + it * NT < V_TASKS && key0 + 4 * vg + r < p.nk && 8u * (vch0 + it * VCH_PER_IT) < dv)
            z = ldg128(base + voff);
          vreg[it][r] = z;
        } else {
          vreg[it][r] = ldg128(base + voff);
        }
      }
    }
  };

  auto store_tile = [&](int buf) {
#pragma unroll
    for (int it = 0; it < K_ITERS; ++it) {
      const int idx = tid + it * NT;
      const int row = idx / CH, ch = idx % CH;
      if (idx < BN * CH) *reinterpret_cast<u32x4*>(&sm.k[buf][row * Smem::KS + 8 * ch]) = kreg[it];
    }
    // V^T with the key order the PV B-operand (= S^T accumulator layout) needs:
    // key 16s + 8a + 4hh + cc  ->  position 16s + 8hh + 4a + cc.
    const int pos0 = 16 * (vg >> 2) + 8 * (vg & 1) + 4 * ((vg >> 1) & 1);
#pragma unroll
    for (int it = 0; it < V_ITERS; ++it) {
      const int dc = vch0 + it * VCH_PER_IT;
      if (tid + it * NT < V_TASKS) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const uint32_t sel = (e & 1) ? 0x07060302u : 0x05040100u;
          u32x2 w;
          w[0] = __builtin_amdgcn_perm(vreg[it][1][e >> 1], vreg[it][0][e >> 1], sel);
          w[1] = __builtin_amdgcn_perm(vreg[it][3][e >> 1], vreg[it][2][e >> 1], sel);
          *reinterpret_cast<u32x2*>(&sm.vt[buf][(8 * dc + e) * Smem::VS + pos0]) = w;
        }
      }
    }
  };

  const f32x16 zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

  // One K/V tile: S^T, running max / sum with exp-shift correction, O^T update.
  auto compute_tile = [&](uint32_t j, int buf, auto masked_tag) {
    constexpr bool MASKED = decltype(masked_tag)::value;
    // ---- S^T = K_tile * Q^T
    f32x16 s[KT];
    const bf16_t* sk = &sm.k[buf][c * Smem::KS + 8 * h];
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) {
        bf16x8 a = *reinterpret_cast<const bf16x8*>(sk + 32 * kt * Smem::KS + 16 * ks);
        s[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[ks], ks == 0 ? zero16 : s[kt], 0, 0, 0);
      }
    }

    // ---- tail guard: keys past nk do not take part in the max
    if constexpr (MASKED) {
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const uint32_t key = j * BN + 32 * kt + 8 * (i >> 2) + 4 * h + (i & 3);
          if (key >= p.nk) s[kt][i] = -INFINITY;
        }
    }

    // ---- running max (snapshot m_old = m_run, then fold this tile)
    float mx = s[0][0];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[kt][i]);
    mx = half_max(mx);
    const float m_new = fmaxf(m_run, mx);
    // exp-shift correction; the first tile (m_run = -inf) contributes nothing to rescale
    const float alpha = m_run == -INFINITY ? 0.0f : fast_exp2((m_run - m_new) * scale_log2);
    const float mb = m_new * scale_log2;
    m_run = m_new;

    // ---- P = exp(S - m), running sum with correction
    float psum = 0.0f;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        float e = fast_exp2(__builtin_fmaf(s[kt][i], scale_log2, -mb));
        if constexpr (MASKED) {
          // spelled out rather than left to exp(-inf): a zero scale turns the masked score into 0 * inf
          const uint32_t key = j * BN + 32 * kt + 8 * (i >> 2) + 4 * h + (i & 3);
          if (key >= p.nk) e = 0.0f;
        }
        s[kt][i] = e;
        psum += e;
      }
    l_run = l_run * alpha + psum;

    // ---- O correction (skipped when no row of this wave moved its max)
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f)) {
#pragma unroll
      for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[t][i] *= alpha;
    }

    // ---- O^T += V_tile^T * P^T
    bf16x8 pb[KT][2];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int e = 0; e < 8; ++e) pb[kt][u][e] = (bf16_t)s[kt][8 * u + e];
    const bf16_t* sv = &sm.vt[buf][c * Smem::VS + 8 * h];
#pragma unroll
    for (int s4 = 0; s4 < BN / 16; ++s4) {
#pragma unroll
      for (int t = 0; t < DT; ++t) {
        bf16x8 a = *reinterpret_cast<const bf16x8*>(sv + 32 * t * Smem::VS + 16 * s4);
        o[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pb[s4 >> 1][s4 & 1], o[t], 0, 0, 0);
      }
    }
  };

  using No = std::integral_constant<bool, false>;
  using Yes = std::integral_constant<bool, true>;
  const uint32_t ntiles = (p.nk + BN - 1) / BN;
  const uint32_t nfull = p.nk / BN;  // tiles that lie entirely inside nk

  if (nfull > 0) load_tile(0, No{});
  else load_tile(0, Yes{});
  store_tile(0);
  __syncthreads();

  // full tiles run unguarded; a trailing partial tile is handled once, after the loop
  for (uint32_t j = 0; j < nfull; ++j) {
    const int buf = j & 1;
    if (j + 1 < nfull) load_tile((j + 1) * BN, No{});
    else if (j + 1 < ntiles) load_tile((j + 1) * BN, Yes{});
    compute_tile(j, buf, No{});
    if (j + 1 < ntiles) store_tile(buf ^ 1);
    __syncthreads();
  }
  if (nfull < ntiles) compute_tile(nfull, nfull & 1, Yes{});

  // ---- normalise and store: lane holds o^T[d][query], d = 32t + 8(i/4) + 4h + i%4
  const float l_tot = half_sum(l_run);
  const float inv = 1.0f / l_tot;
  if (qrow < p.nq) {
    if (p.out_bf16) {
      bf16_t* O = reinterpret_cast<bf16_t*>(p.o) + ((size_t)head * p.nq + qrow) * dv;
#pragma unroll
      for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const uint32_t col = 32 * t + 8 * g + 4 * h;
          if (EXACT || col < dv) {
            bf16x4 w;
#pragma unroll
            for (int e = 0; e < 4; ++e) w[e] = (bf16_t)(o[t][4 * g + e] * inv);
            *reinterpret_cast<bf16x4*>(O + col) = w;
          }
        }
    } else {
      float* O = reinterpret_cast<float*>(p.o) + ((size_t)head * p.nq + qrow) * dv;
#pragma unroll
      for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const uint32_t col = 32 * t + 8 * g + 4 * h;
          if (EXACT || col < dv) {
            f32x4 w;
#pragma unroll
            for (int e = 0; e < 4; ++e) w[e] = o[t][4 * g + e] * inv;
            *reinterpret_cast<f32x4*>(O + col) = w;
          }
        }
    }
  }
}
