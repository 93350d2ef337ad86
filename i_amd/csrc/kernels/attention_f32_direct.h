// FlashAttention forward for f32 inputs (full f32 arithmetic) on gfx950, for d == dv == DPAD:
// K and V tiles go from global memory straight into LDS.
//
// Same fused nest, the same lane mapping and the same arithmetic as attention_f32.h (one query per lane, S^T and
// O^T accumulators of v_mfma_f32_32x32x2_f32, running max and sum with the exp-shift correction applied tile by
// tile, products and sums in IEEE f32 as in the reference C backend, ilang-python/annotated-flashattn.c:52-310).
// What differs is how the tiles reach the matrix cores, which is what that kernel spends its time on:
//
//   global -> LDS   global_load_lds_dwordx4 as in attention_bf16_direct.h: every lane fetches 16 bytes and the
//                   wave deposits them as one contiguous 1 KiB run of LDS, no registers in between.  A tile is
//                   BN = 32 keys of 4 DPAD bytes; two buffers, tile j+1 is requested before tile j is computed and
//                   awaited (vmcnt(0) + barrier) after it: one barrier per tile.
//   swizzle         rows are 512 (DPAD 128) or 256 (DPAD 64) bytes, so unpadded rows would collide in the banks.
//                   The 16-byte chunk index is XOR-ed with a function of the row on the GLOBAL side (a lane chooses
//                   which chunk it fetches for its fixed LDS slot):
//                     K: chunk ^= row % 16            16 consecutive rows, same chunk -> 16 different bank groups
//                     V: chunk ^= 8 ((row / 4) % 2)   the two rows a wave reads at once (4 apart) -> different halves
//                                                     of the 256-byte bank window
//   LDS -> K operand  the instruction's A operand is one f32 per lane, A[row = lane % 32][k = lane / 32].  A lane
//                   reads 16 bytes of its row, chunk 2 ks + h (h = lane / 32), and element e of them feeds MFMA e of
//                   the group: the contraction pairs are {8 ks + e, 8 ks + 4 + e}, a permutation of d that the Q
//                   fragments follow.
//   LDS -> V operand  A[dv = lane % 32][key = lane / 32]: V stays row-major, a lane reads the one f32 at
//                   (key, 32 t + lane % 32); the key of half-wave h for accumulator element i is the key whose
//                   probability that half-wave holds in element i, so the probabilities are the B operand as
//                   they are.
//
// Requires d == dv == DPAD, 16-byte aligned operands and nk * d * 4 < 2^32 (the launcher falls back to
// attention_f32.h otherwise).  4 waves (128 queries) per workgroup, two workgroups per CU.
//
// PADDED: d = p.d and dv = p.dv are any multiples of 4 up to DPAD.  The tiles in LDS keep their DPAD-wide rows: a
// lane whose 16-byte chunk lies past the end of a row fetches nothing, and the tile memory is cleared once before
// the first transfer, so the columns d .. DPAD - 1 of K and dv .. DPAD - 1 of V read as zeros for the whole kernel
// (Q is padded with zeros in its registers; the output columns past dv are not stored).  Global rows of Q and K
// are 4 p.d bytes apart, those of V and O 4 p.dv.
#pragma once
#include <type_traits>

#include "common.h"
#include "params.h"

template <int DPAD, int NWAVES, bool PADDED = false>
__device__ __forceinline__ void attn_fwd_f32_direct_body(const AttnParams& p) {
  constexpr int BN = 32;
  constexpr int BM = 32 * NWAVES;
  constexpr int KG = DPAD / 8;            // groups of 4 MFMAs of the QK^T contraction (8 d each)
  constexpr int DT = DPAD / 32;           // 32-column output tiles
  constexpr int RB = 4 * DPAD;            // bytes per K/V row
  constexpr int CH = RB / 16;             // 16-byte chunks per row (= lanes per row of a wave-load)
  constexpr int RPW = 64 / CH;            // rows per wave-load
  constexpr int TILE_BYTES = BN * RB;
  constexpr int WL = TILE_BYTES / 1024;   // wave-loads per tile
  constexpr int WLW = WL / NWAVES;        // ... per wave
  static_assert(CH == 16 || CH == 32, "row size");
  static_assert(WL % NWAVES == 0 && WLW >= 1, "tile / wave shape");
  __shared__ __attribute__((aligned(1024))) char smem[2][2][TILE_BYTES];  // [buffer][K, V]

  uint32_t head, qt;
  xcd_map(blockIdx.x, p.nqt, p.bh, head, qt);
  if (head >= p.bh) return;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t c = lane & 31;  // query column within the wave / A-operand row
  const uint32_t h = lane >> 5;  // half-wave
  const uint32_t d = PADDED ? p.d : (uint32_t)DPAD;    // elements per row of Q and K in global memory
  const uint32_t dv = PADDED ? p.dv : (uint32_t)DPAD;  // ... of V and O
  const uint32_t RBG = 4 * d, RBGV = 4 * dv;            // bytes per global row of K, of V (RB when not PADDED)
  const uint32_t chunks = d / 4, chunks_v = dv / 4;     // 16-byte chunks per global row

  // The keys of a head split over workgroups (p.kv_splits > 1), as in the bf16 kernels: `head` counts (head, part)
  // pairs, a part runs the keys first_key .. first_key + nk of its head and leaves its normalised result in o[head] (a
  // temporary) and log2 of its row sums of exponentials in p.lse[head] for attn_kv_merge.
  uint32_t qhead = head, first_key = 0, nk = p.nk;
  if (p.kv_splits > 1) {
    qhead = head / p.kv_splits;
    first_key = (head - qhead * p.kv_splits) * p.kv_chunk;
    nk = p.nk - first_key < p.kv_chunk ? p.nk - first_key : p.kv_chunk;
  }
  const float* __restrict__ Q = reinterpret_cast<const float*>(p.q) + (size_t)qhead * p.nq * d;
  const char* __restrict__ K = reinterpret_cast<const char*>(p.k) + ((size_t)qhead * p.nk + first_key) * RBG;
  const char* __restrict__ V = reinterpret_cast<const char*>(p.v) + ((size_t)qhead * p.nk + first_key) * RBGV;

  const float scale_raw = load_scale(p.scale_ptr, p.scale_value);
  const float qsign = scale_raw < 0.0f ? -1.0f : 1.0f;  // negative scale folded into Q (exact)
  const float scale_log2 = fabsf(scale_raw) * I_LOG2_E32;

  // ---- global -> LDS: this lane's slot in wave-load w is tile row w*RPW + lane/CH, chunk lane%CH; rows past nk
  // re-read the last row (their scores are masked)
  const uint32_t ntiles = (nk + BN - 1) / BN;
  const uint32_t lrow = lane / CH, lch = lane % CH;
  const uint32_t smem0 = lds_address(&smem[0][0][0]);
  auto request_tile = [&](uint32_t tile, int buf) {
#pragma unroll
    for (int it = 0; it < WLW; ++it) {
      const uint32_t w = wave + NWAVES * it;
      const uint32_t row = w * RPW + lrow;  // row within the tile
      uint32_t key = tile * BN + row;
      key = key < nk ? key : nk - 1;
      const uint32_t kch = lch ^ (row % 16), vch = lch ^ (8 * ((row >> 2) & 1));
      if (!PADDED || kch < chunks) dma16(K, key * RBG + 16 * kch, smem0 + (2 * buf + 0) * TILE_BYTES + w * 1024);
      if (!PADDED || vch < chunks_v) dma16(V, key * RBGV + 16 * vch, smem0 + (2 * buf + 1) * TILE_BYTES + w * 1024);
    }
  };
  if constexpr (PADDED) {
    // the tile memory, cleared once: what no transfer ever writes (the columns past d) then reads as zero
    for (uint32_t at = 16 * tid; at < 4 * TILE_BYTES; at += 16 * 64 * NWAVES)
      *reinterpret_cast<u32x4*>(&smem[0][0][0] + at) = u32x4{0, 0, 0, 0};
    __syncthreads();
  }
  request_tile(0, 0);

  // Q^T fragments (B operand): lane (c, h) holds q[row][8 g + 4 h + e] in element e of group g
  const uint32_t qrow = qt * BM + wave * 32 + c;
  f32x4 qf[KG];
#pragma unroll
  for (int g = 0; g < KG; ++g) {
    f32x4 z = {0.0f, 0.0f, 0.0f, 0.0f};
    if (qrow < p.nq && (!PADDED || (uint32_t)(8 * g + 4 * h) < d)) z = *reinterpret_cast<const f32x4*>(Q + (size_t)qrow * d + 8 * g + 4 * h);
    qf[g] = z * qsign;
  }

  f32x16 o[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[t][i] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;

  // ---- LDS -> operands: per-lane byte offsets inside a tile
  // K: row c, chunk (2 g + h) ^ (c % 16) = (h ^ (c % 16)) ^ 2 g: the address of group 0 with 32 g XOR-ed in
  // (one instruction per read instead of KG registers; 32 g stays below the row size)
  const uint32_t kaddr0 = c * RB + 16 * (h ^ (c % 16));
  // V: key 8 (i / 4) + 4 h + i % 4 for accumulator element i, column 32 t + c: chunk (8 t + c / 4) ^ 8 h (the key's
  // bit 2 is h), element c % 4
  uint32_t vaddr[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t) vaddr[t] = 4 * h * RB + 16 * ((uint32_t)(8 * t + c / 4) ^ (8 * h)) + 4 * (c % 4);

  dma_wait_all();
  __syncthreads();
  for (uint32_t j = 0; j < ntiles; ++j) {
    const int buf = j & 1;
    const uint32_t key0 = j * BN;
    if (j + 1 < ntiles) request_tile(j + 1, buf ^ 1);
    const char* sk = &smem[buf][0][0];
    const char* sv = &smem[buf][1][0];

    // ---- S^T = K_tile * Q^T
    f32x16 s;
#pragma unroll
    for (int i = 0; i < 16; ++i) s[i] = 0.0f;
#pragma unroll
    for (int g = 0; g < KG; ++g) {
      uint32_t first = kaddr0;
      asm volatile("" : "+v"(first));  // (keeps the KG addresses from being hoisted into registers of their own)
      const f32x4 a = *reinterpret_cast<const f32x4*>(sk + (first ^ (32u * g)));
#pragma unroll
      for (int e = 0; e < 4; ++e) s = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], qf[g][e], s, 0, 0, 0);
    }

    const bool masked = key0 + BN > nk;
    if (masked) {  // tail guard: keys past nk do not take part in the max
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const uint32_t key = key0 + 8 * (i >> 2) + 4 * h + (i & 3);
        if (key >= nk) s[i] = -INFINITY;
      }
    }
    float mx = s[0];
#pragma unroll
    for (int i = 1; i < 16; ++i) mx = fmaxf(mx, s[i]);
    mx = fmaxf(mx, xhalf(mx));
    const float m_new = fmaxf(m_run, mx);
    const float alpha = m_run == -INFINITY ? 0.0f : fast_exp2((m_run - m_new) * scale_log2);
    const float mb = m_new * scale_log2;
    m_run = m_new;

    float psum = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      float e = fast_exp2(__builtin_fmaf(s[i], scale_log2, -mb));
      if (masked) {
        // spelled out rather than left to exp(-inf): a zero scale turns the masked score into 0 * inf
        const uint32_t key = key0 + 8 * (i >> 2) + 4 * h + (i & 3);
        if (key >= nk) e = 0.0f;
      }
      s[i] = e;
      psum += e;
    }
    l_run = l_run * alpha + psum;
    // (a factor of exactly 1 in every lane, the usual case once the row maxima have settled, changes nothing)
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f)) {
#pragma unroll
      for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[t][i] *= alpha;
    }

    // ---- O^T += V^T P^T, one key per half-wave and MFMA
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const uint32_t krow = (8 * (i >> 2) + (i & 3)) * RB;  // (+ 4 h rows inside vaddr)
#pragma unroll
      for (int t = 0; t < DT; ++t) {
        const float a = *reinterpret_cast<const float*>(sv + krow + vaddr[t]);
        o[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, s[i], o[t], 0, 0, 0);
      }
    }
    dma_wait_all();
    __syncthreads();
  }

  // ---- epilogue: normalise and store.  Lane (c, h) holds O[q = c][32 t + 8 g + 4 h + e].
  const float l_tot = l_run + xhalf(l_run);
  const float inv = 1.0f / l_tot;
  if (p.kv_splits > 1 && qrow < p.nq && h == 0) p.lse[(size_t)head * p.nq + qrow] = m_run * scale_log2 + log2f(l_tot);
  if (qrow < p.nq) {
    float* O = reinterpret_cast<float*>(p.o) + ((size_t)head * p.nq + qrow) * dv;
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        f32x4 w;
#pragma unroll
        for (int e = 0; e < 4; ++e) w[e] = o[t][4 * g + e] * inv;
        if (!PADDED || (uint32_t)(32 * t + 8 * g + 4 * h) < dv) *reinterpret_cast<f32x4*>(O + 32 * t + 8 * g + 4 * h) = w;
      }
  }
}
