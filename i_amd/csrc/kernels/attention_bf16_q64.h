// FlashAttention forward, bf16 in / f32 accumulate, for d == dv == 64: 64 queries per wave.
//
// The data path is the one of attention_bf16_direct.h (K and V tiles go from global memory straight into
// swizzled LDS tiles, K operands by ds_read_b128, V operands by the transposing ds_read_b64_tr_b16, scores
// of tile j+1 on the matrix pipe while the softmax of tile j runs on the vector pipe; the steady state takes no
// row max and no reference at all, see below).  What differs: a wave owns QB = 2 blocks of 32 query rows instead of one, so every K or V
// operand that is read from LDS feeds two MFMAs (one per block), which halves the LDS reads per flop.  At
// d = 64 the registers allow that with two waves per SIMD (O 64 + two score tiles of 32 keys 64 + Q 32 + P 16),
// which a wave needs because only about half of an MFMA's 32 cycles can be covered by its own vector work;
// at d = 128 it would take the whole register file of a SIMD for one wave, and that form measured slower.
// Tiles are 32 keys, 8 waves form a workgroup of 512 queries; a 32-key tile of K or V is only 4 wave-loads,
// so waves 0-3 request K and waves 4-7 request V.
#pragma once
#include <type_traits>

#include "common.h"
#include "params.h"

// extra operand-fetch lead of the steady-state loop, in operands (see fast_step)
#ifndef ATTN_Q64_XLEAD
#define ATTN_Q64_XLEAD 0
#endif

template <int DPAD, int BN, int NWAVES>
__device__ __forceinline__ void attn_fwd_bf16_q64_body(const AttnParams& p) {
  constexpr int QB = 2;                   // 32-row query blocks per wave
  constexpr int BM = 32 * QB * NWAVES;
  constexpr int KSTEPS = DPAD / 16;       // k-steps of the QK^T contraction
  constexpr int KT = BN / 32;             // 32-key accumulator tiles
  constexpr int DT = DPAD / 32;           // 32-column output tiles
  constexpr int RB = 2 * DPAD;            // bytes per K/V row
  constexpr int CH = RB / 16;             // 16-byte chunks per row (= lanes per row of a wave-load)
  constexpr int RPB = 256 / RB;           // rows per 256 bytes
  constexpr int RPW = 64 / CH;            // rows per wave-load
  constexpr int TILE_BYTES = BN * RB;
  constexpr int WL = TILE_BYTES / 1024;   // wave-loads per tile
  // Either every wave requests WLW wave-loads of K and WLW of V per tile, or (SPLIT: a tile has fewer wave-loads
  // than the workgroup has waves) waves 0 .. WL-1 request one wave-load of K each and waves WL .. 2 WL-1 one of V.
  constexpr bool SPLIT = WL < NWAVES;
  constexpr int WLW = SPLIT ? 1 : WL / NWAVES;
  static_assert(RB == 128 || RB == 256, "row size");
  static_assert(SPLIT ? 2 * WL == NWAVES : WL % NWAVES == 0, "tile / wave shape");
  __shared__ __attribute__((aligned(1024))) char smem[2][2][TILE_BYTES];  // [buffer][K, V]

  uint32_t head, qt;
  xcd_map(blockIdx.x, p.nqt, p.bh, head, qt);
  if (head >= p.bh) return;
  clock_note(p.clock, false);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 31;  // query column within the wave / A-operand row
  const int h = lane >> 5;  // half-wave
  constexpr uint32_t d = DPAD;

  const bf16_t* __restrict__ Q = reinterpret_cast<const bf16_t*>(p.q) + (size_t)head * p.nq * d;
  const char* __restrict__ K = reinterpret_cast<const char*>(p.k) + (size_t)head * p.nk * RB;
  const char* __restrict__ V = reinterpret_cast<const char*>(p.v) + (size_t)head * p.nk * RB;

  // A negative scale is folded into Q (sign flip is exact), so the running max
  // can be tracked on the raw scores: max_j(s_j * scale) == scale * max_j(s_j).
  const float scale_raw = load_scale(p.scale_ptr, p.scale_value);
  // As in attention_bf16_direct.h for d = 64: the factor scale * log2(e) is folded into Q (one more bf16 rounding),
  // and in the steady state a score tile's first MFMA adds -reference instead of 0, so that scores leave the
  // matrix pipe as arguments of exp2.
  const float scale_log2 = 1.0f;
  const float q_factor = scale_raw * I_LOG2_E32;

  // Q^T fragments (B operand): lane (c, h) holds q[row][16*ks + 8*h .. +8].
  uint32_t qrow[QB];
  bf16x8 qf[QB][KSTEPS];
#pragma unroll
  for (int b = 0; b < QB; ++b) {
    qrow[b] = qt * BM + wave * (32 * QB) + 32 * b + c;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      u32x4 z = {0, 0, 0, 0};
      if (qrow[b] < p.nq) z = ldg128(Q + (size_t)qrow[b] * d + 16 * ks + 8 * h);
      bf16x8 scaled = __builtin_bit_cast(bf16x8, z);
#pragma unroll
      for (int e = 0; e < 8; ++e) scaled[e] = (bf16_t)((float)scaled[e] * q_factor);
      qf[b][ks] = scaled;
    }
  }

  f32x16 o[QB][DT];
  float m_run[QB], l_run[QB];  // running max of the scores; running sum over this half-wave's keys
#pragma unroll
  for (int b = 0; b < QB; ++b) {
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[b][t][i] = 0.0f;
    m_run[b] = -INFINITY;
    l_run[b] = 0.0f;
  }

  const uint32_t nfull_tiles = p.nk / BN;  // tiles that lie entirely inside nk
  // ---- global -> LDS: this lane's slot in wave-load w is tile row w*RPW + lane/CH, chunk lane%CH
  const uint32_t lrow = lane / CH, lch = lane % CH;
  const uint32_t smem0 = lds_address(&smem[0][0][0]);

  // For a full tile the per-lane part of the address is the same for every tile and every wave-load
  // (the swizzle term does not depend on `it` because NWAVES * RPW rows is a multiple of the swizzle
  // period); everything that varies is wave-uniform and is folded into the scalar base address.
  static_assert(SPLIT || (NWAVES * RPW / RPB) % CH == 0, "swizzle period");
  const bool k_wave = !SPLIT || wave < WL;   // this wave takes part in K requests
  const bool v_wave = !SPLIT || wave >= WL;  // ... in V requests
  const uint32_t wave_w = SPLIT ? wave % WL : wave;  // its first wave-load
  const uint32_t lane_row = wave_w * RPW + lrow;
  const uint32_t koff_lane = lrow * RB + 16 * (lch ^ ((lane_row / RPB) % CH));
  const uint32_t voff_lane = lrow * RB + 16 * (lch ^ (4 * ((lane_row / RPB) % (CH / 4))));
  // one wave-load of a full tile: `it` of K (want_k) or of V
  auto request_full_one = [&](uint32_t tile, int buf, int it, auto want_k) {
    const uint32_t w = wave_w + NWAVES * it;
    const size_t byte0 = (size_t)tile * TILE_BYTES + w * 1024;
    if constexpr (decltype(want_k)::value) {
      if (k_wave) dma16(K + byte0, koff_lane, smem0 + (2 * buf + 0) * TILE_BYTES + w * 1024);
    } else {
      if (v_wave) dma16(V + byte0, voff_lane, smem0 + (2 * buf + 1) * TILE_BYTES + w * 1024);
    }
  };

  // one wave-load of K of any tile index: full tile, partial tile (rows past nk re-read the last row), or none
  auto request_k_one = [&](uint32_t tile, int buf, int it) {
    if (!k_wave) return;
    if (tile < nfull_tiles) {
      const uint32_t w = wave_w + NWAVES * it;
      dma16(K + (size_t)tile * TILE_BYTES + w * 1024, koff_lane, smem0 + (2 * buf + 0) * TILE_BYTES + w * 1024);
    } else if (tile * BN < p.nk) {
      const uint32_t w = wave_w + NWAVES * it;
      const uint32_t row = w * RPW + lrow;
      uint32_t key = tile * BN + row;
      key = key < p.nk ? key : p.nk - 1;
      dma16(K, key * RB + 16 * (lch ^ ((row / RPB) % CH)), smem0 + (2 * buf + 0) * TILE_BYTES + w * 1024);
    }
  };

  // PARTIAL: the tile runs past nk; rows past the end re-read the last row (their scores are masked).
  auto request_tile = [&](uint32_t key0, int buf, auto partial_tag, auto want_k, auto want_v) {
    constexpr bool PARTIAL = decltype(partial_tag)::value;
#pragma unroll
    for (int it = 0; it < WLW; ++it) {
      const uint32_t w = wave_w + NWAVES * it;
      const uint32_t row = w * RPW + lrow;  // row within the tile
      const uint32_t kch = lch ^ ((row / RPB) % CH);
      const uint32_t vch = lch ^ (4 * ((row / RPB) % (CH / 4)));
      uint32_t key = key0 + row;
      if constexpr (PARTIAL) key = key < p.nk ? key : p.nk - 1;
      if constexpr (decltype(want_k)::value) {
        if (k_wave) dma16(K, key * RB + 16 * kch, smem0 + (2 * buf + 0) * TILE_BYTES + w * 1024);
      }
      if constexpr (decltype(want_v)::value) {
        if (v_wave) dma16(V, key * RB + 16 * vch, smem0 + (2 * buf + 1) * TILE_BYTES + w * 1024);
      }
    }
  };

  // ---- LDS -> operands: per-lane byte offsets inside a tile
  // K: row c (+ 32 kt), chunk (2 ks + h) ^ fk, where fk depends on c only
  const uint32_t fk = (c / RPB) % CH;
  uint32_t kaddr[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) kaddr[ks] = c * RB + 16 * ((2 * ks + h) ^ fk);
  // V: 16-lane block b = lane / 16 covers columns 16 (b & 1) .. +16 of a 32-column tile; lane 4 jj + q of
  // the block points at key (4 h + jj), columns 4 q .. +4
  const uint32_t blk = lane >> 4, jj = (lane >> 2) & 3, qq = lane & 3;
  const uint32_t gv = 4 * (((4 * h + jj) / RPB) % (CH / 4));
  uint32_t vaddr[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t)
    vaddr[t] = (4 * h + jj) * RB + 16 * (((4 * t) ^ gv) + 2 * (blk & 1) + (qq >> 1)) + 8 * (qq & 1);

  const f32x16 zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  typedef __attribute__((ext_vector_type(4))) short s16x4;
  typedef __attribute__((ext_vector_type(8))) short s16x8;
  typedef __attribute__((address_space(3))) s16x4* lds_s16x4_ptr;
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;

  // ---- S^T = K_tile * Q^T for the K tile in buffer kbuf
  auto qk = [&](f32x16 (&s)[QB][KT], int kbuf) {
    const char* sk = &smem[kbuf][0][0];
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) {
        bf16x8 a = *reinterpret_cast<const bf16x8*>(sk + 32 * kt * RB + kaddr[ks]);
#pragma unroll
        for (int b = 0; b < QB; ++b)
          s[b][kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[b][ks], ks == 0 ? zero16 : s[b][kt], 0, 0, 0);
      }
    }
  };

  // ---- running max / sum with exp-shift correction, then O^T += V_tile^T * P^T (V tile in buffer vbuf).
  // The reference max is moved only when a row's tile max exceeds it by more than 2^RESCALE_LOG2 in the
  // exponent: until then P = exp(S - m_run) is at most 2^RESCALE_LOG2, well inside f32 / bf16 range, and
  // sum and output stay consistently scaled, so the normalised result is the same while the correction
  // pass over the O accumulators is skipped for almost every tile.
  constexpr float RESCALE_LOG2 = 8.0f;
  auto softmax_pv = [&](f32x16 (&s)[QB][KT], uint32_t j, int vbuf, bool masked) {
    bf16x8 pb[QB][KT][2];
    const bf16x2 ones = {(bf16_t)1.0f, (bf16_t)1.0f};
#pragma unroll
    for (int b = 0; b < QB; ++b) {
      if (masked) {  // tail guard: keys past nk do not take part in the max
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const uint32_t key = j * BN + 32 * kt + 8 * (i >> 2) + 4 * h + (i & 3);
            if (key >= p.nk) s[b][kt][i] = -INFINITY;
          }
      }
      float mx = s[b][0][0];
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[b][kt][i]);
      mx = half_max(mx);
      // the first tile (m_run = -inf) always sets the reference; written so that a zero scale (inf * 0) is covered
      const bool first = m_run[b] == -INFINITY;
      const bool move = first || (mx - m_run[b]) * scale_log2 > RESCALE_LOG2;
      const float m_new = move ? mx : m_run[b];
      const float alpha = first ? 0.0f : fast_exp2((m_run[b] - m_new) * scale_log2);  // 1 when the reference stays
      const float mb = m_new * scale_log2;
      m_run[b] = m_new;

      // P = exp(S - m) rounded to bf16 (the PV operand); the row sum is taken over the rounded values
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          float e = fast_exp2(__builtin_fmaf(s[b][kt][i], scale_log2, -mb));
          if (masked) {
            // spelled out rather than left to exp(-inf): a zero scale turns the masked score into 0 * inf
            const uint32_t key = j * BN + 32 * kt + 8 * (i >> 2) + 4 * h + (i & 3);
            if (key >= p.nk) e = 0.0f;
          }
          pb[b][kt][i >> 3][i & 7] = (bf16_t)e;
        }
      float psum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int u = 0; u < 2; ++u) {
#pragma unroll
          for (int w = 0; w < 4; ++w)
            psum[w] = __builtin_amdgcn_fdot2_f32_bf16(bf16x2{pb[b][kt][u][2 * w], pb[b][kt][u][2 * w + 1]}, ones, psum[w],
                                                      false);
        }
      l_run[b] = l_run[b] * alpha + ((psum[0] + psum[1]) + (psum[2] + psum[3]));

      // O correction (skipped unless some row of this block moved its reference)
      if (__builtin_amdgcn_ballot_w64(move)) {
#pragma unroll
        for (int t = 0; t < DT; ++t)
#pragma unroll
          for (int i = 0; i < 16; ++i) o[b][t][i] *= alpha;
      }
    }

    const char* sv = &smem[vbuf][1][0];
#pragma unroll
    for (int s4 = 0; s4 < BN / 16; ++s4) {
#pragma unroll
      for (int t = 0; t < DT; ++t) {
        const char* va = sv + 16 * s4 * RB + vaddr[t];
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(va));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(va + 8 * RB));
        const bf16x8 both = __builtin_bit_cast(bf16x8, (s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
#pragma unroll
        for (int b = 0; b < QB; ++b)
          o[b][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(both, pb[b][s4 >> 1][s4 & 1], o[b][t], 0, 0, 0);
      }
    }
  };

  using No = std::integral_constant<bool, false>;
  using Yes = std::integral_constant<bool, true>;
  const uint32_t ntiles = (p.nk + BN - 1) / BN;
  const uint32_t nfull = p.nk / BN;  // tiles that lie entirely inside nk

  // Software pipeline: the scores of tile j+1 are computed (matrix pipe) in the same iteration as the
  // softmax of tile j (vector pipe).  K is therefore consumed one iteration before V: K(j+2) and V(j+1)
  // are requested at the top of iteration j, into the buffers of K(j) (last read in iteration j-1) and of
  // V(j-1) (last read in iteration j-1); one wait + barrier per iteration publishes both.
  auto request_k = [&](uint32_t t, int buf) {
    if (t < nfull) request_tile(t * BN, buf, No{}, Yes{}, No{});
    else request_tile(t * BN, buf, Yes{}, Yes{}, No{});
  };
  auto request_v = [&](uint32_t t, int buf) {
    if (t < nfull) request_tile(t * BN, buf, No{}, No{}, Yes{});
    else request_tile(t * BN, buf, Yes{}, No{}, Yes{});
  };

  f32x16 sa[QB][KT], sb[QB][KT];
  // tiles 0 and 1 of K and tile 0 of V into LDS, then S(0)
  auto first_tiles = [&]() {
    request_k(0, 0);
    request_v(0, 0);
    if (ntiles > 1) request_k(1, 1);
    dma_wait_all();
    __syncthreads();
    qk(sa, 0);
    __syncthreads();  // K(2) is requested into the buffer of K(0): not before every wave has read K(0)
  };
  first_tiles();

  // Steady state (tiles j and j+1 are full tiles).  One trip runs from barrier to barrier and is written as a
  // sequence of MFMA slots, everything else dealt out between the MFMAs a few vector instructions per slot, so
  // that the matrix pipe and the vector pipe of the SIMD are fed by the same wave at the same time.  A
  // scheduling fence after every slot keeps this order.  The trip uses NOP = NQK + NPV operands (K rows, then
  // transposed V columns); operand k feeds the QB slots QB k .. QB k + QB - 1, one per query block:
  //   QB * DT slots          last 16-key group of O += V(j-1)^T P(j-1)^T, operands and probabilities carried
  //                          in registers across the barrier
  //   QB * NQK slots         S(j+1) = K(j+1) Q^T
  //                          (these slots also carry the global -> LDS requests for K(j+2), V(j+1) and all of
  //                          P(j) = exp(S(j) - reference), its bf16 rounding and the row sums)
  //   QB * (NPV - DT) slots  O += V(j)^T P(j)^T for all but the last 16-key group
  // LDS operands are fetched in operand order, DT + ATTN_Q64_XLEAD operands ahead of their first MFMA; the fetches
  // for the carried group are the last ones before the barrier, so the barrier sits in the middle of a stream of
  // MFMAs instead of at a point where the matrix pipe has drained.
  constexpr int NQK = KSTEPS * KT;      // K operands of the score tile
  constexpr int NPV = (BN / 16) * DT;   // V operands of the output update
  constexpr int NOP = NQK + NPV;
  constexpr int NPAIR = KT * 8;         // score pairs per lane and block; pairs 4 g .. 4 g + 3 are the 16-key group g
  constexpr int NPRE = QB * (DT + NQK); // slots that carry the exponentials (all before the first PV slot of the tile)
  constexpr int NMAIN = NPV - DT;       // V operands of the trip that owns the tile
  constexpr int XLEAD = ATTN_Q64_XLEAD;
  static_assert(NPAIR % 4 == 0 && 2 * WLW <= NPRE && XLEAD >= 0 && XLEAD < NQK, "slot shape");

  // The steady state takes P = exp2(score) as it is, with no reference at all (Q carries scale * log2(e)).  The
  // normalised result does not depend on the reference, and with probabilities rounded to bf16 (same exponent
  // range as f32) neither does its precision, as long as nothing overflows or a whole row underflows.  A wave
  // notes (without branching) whether a tile's row sum reached 2^80 and, at the end, whether a row sum fell below
  // 2^-100; if any wave of the workgroup did, the workgroup throws the pass away and computes the item again
  // with the general loop, which takes the running max tile by tile.
  bool bad = false;
  // The first NEARLY pairs of a tile and block are computed one trip early, one per output slot of the
  // previous tile (those slots carry no other vector work, while every other slot of the trip carries one pair);
  // they wait in `early`, and the row-sum parts live across trips with them
  constexpr int NEARLY = 2;
  uint32_t early[QB][NEARLY];
  float psum[QB][2];
#pragma unroll
  for (int b = 0; b < QB; ++b) psum[b][0] = psum[b][1] = 0.0f;
  const bf16x2 ones = {(bf16_t)1.0f, (bf16_t)1.0f};
  // pair pr of block b of score tile s: two exponentials, their bf16 rounding, the row-sum part
  auto exp_pair_of = [&](const f32x16 (&s)[QB][KT], int b, int pr) -> uint32_t {
    const int pkt = pr / 8, i = 2 * (pr % 8);
    const float e0 = fast_exp2(s[b][pkt][i]);  // relative to the reference already
    const float e1 = fast_exp2(s[b][pkt][i + 1]);
    const bf16x2 pair = {(bf16_t)e0, (bf16_t)e1};
    psum[b][pr & 1] = __builtin_amdgcn_fdot2_f32_bf16(pair, ones, psum[b][pr & 1], false);
    uint32_t packed = __builtin_bit_cast(uint32_t, pair);
    asm volatile("" : "+v"(packed), "+v"(psum[b][pr & 1]));
    return packed;
  };

  struct Carry {
    bf16x8 a[DT];  // V^T operands of the last 16-key group
    u32x4 p[QB];   // its probabilities, per query block
  };

  // any_k_tag: tile j+2 may be partial or absent (the last steady-state trip); otherwise it is a full tile
  auto fast_step = [&](uint32_t j, int buf, f32x16 (&s_cur)[QB][KT], f32x16 (&s_next)[QB][KT], const Carry& cin,
                       Carry& cout, auto any_k_tag) {
    const char* sk = &smem[buf ^ 1][0][0];  // K(j+1)
    const char* sv = &smem[buf][1][0];      // V(j)

    // operand k of this trip: K rows for k < NQK, transposed V columns after that
    bf16x8 opnd[NOP];
    auto fetch = [&](int k) {
      if (k < NQK) {
        const int ks = k / KT, kt = k % KT;
        opnd[k] = *reinterpret_cast<const bf16x8*>(sk + 32 * kt * RB + kaddr[ks]);
      } else {
        const int s4 = (k - NQK) / DT, t = (k - NQK) % DT;
        const char* va = sv + 16 * s4 * RB + vaddr[t];
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(va));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(va + 8 * RB));
        opnd[k] = __builtin_bit_cast(bf16x8, (s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
      }
    };
    // the first slot of operand position g (counted from the start of the trip, carried operands included)
    // issues fetch g + XLEAD (position 0 also issues 0 .. XLEAD - 1)
    auto fetch_for_position = [&](int g) {
      if (g == 0) {
#pragma unroll
        for (int k = 0; k < XLEAD; ++k) fetch(k);
      }
      if (g + XLEAD < NOP) fetch(g + XLEAD);
    };
    // request g of the 2 WLW global -> LDS requests of the trip
    auto request_for_slot = [&](int g) {
      if (g < 2 * WLW) {
        if (g < WLW) {
          if constexpr (decltype(any_k_tag)::value) request_k_one(j + 2, buf, g);
          else request_full_one(j + 2, buf, g, Yes{});
        } else {
          request_full_one(j + 1, buf ^ 1, g - WLW, No{});
        }
      }
    };

    // packed probability pairs: pq[b][g][w] holds scores 2 (4 g + w), + 1 of the lane in (kt, i) order, so
    // pq[b][g] is the B operand of 16-key group g of block b.  The empty asm statements tie each slot's vector
    // work to its slot.
    u32x4 pq[QB][NPAIR / 4];
#pragma unroll
    for (int b = 0; b < QB; ++b)
#pragma unroll
      for (int w = 0; w < NEARLY; ++w) pq[b][0][w] = early[b][w];
    // late pair n of the trip: block n / NLATE, pair NEARLY + n % NLATE
    constexpr int NLATE = NPAIR - NEARLY;
    auto exp_pair = [&](int n) {
      const int b = n / NLATE, pr = NEARLY + n % NLATE;
      pq[b][pr / 4][pr % 4] = exp_pair_of(s_cur, b, pr);
    };
    auto pairs_for_slot = [&](int g) {
#pragma unroll
      for (int n = g * (QB * NLATE) / NPRE; n < (g + 1) * (QB * NLATE) / NPRE; ++n) exp_pair(n);
    };

    // ---- carried slots: last key group of tile j-1
#pragma unroll
    for (int g = 0; g < DT; ++g) {
      fetch_for_position(g);
#pragma unroll
      for (int b = 0; b < QB; ++b) {
        o[b][g] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(cin.a[g], __builtin_bit_cast(bf16x8, cin.p[b]), o[b][g], 0, 0, 0);
        request_for_slot(QB * g + b);
        pairs_for_slot(QB * g + b);
        __builtin_amdgcn_sched_barrier(0);
      }
    }

    // ---- score slots of tile j+1
#pragma unroll
    for (int n = 0; n < NQK; ++n) {
      fetch_for_position(DT + n);
      const int ks = n / KT, kt = n % KT;
#pragma unroll
      for (int b = 0; b < QB; ++b) {
        s_next[b][kt] =
            __builtin_amdgcn_mfma_f32_32x32x16_bf16(opnd[n], qf[b][ks], ks == 0 ? zero16 : s_next[b][kt], 0, 0, 0);
        request_for_slot(QB * (DT + n) + b);
        pairs_for_slot(QB * (DT + n) + b);
        __builtin_amdgcn_sched_barrier(0);
      }
    }

    // ---- the tile's row sums: noted when out of range (acted upon after the pass), then added
#pragma unroll
    for (int b = 0; b < QB; ++b) {
      bad = bad || !(psum[b][0] + psum[b][1] < 0x1p80f);
      l_run[b] += psum[b][0] + psum[b][1];
      psum[b][0] = psum[b][1] = 0.0f;
    }
    __builtin_amdgcn_sched_barrier(0);

    // ---- output slots of tile j, all key groups but the last
#pragma unroll
    for (int m = 0; m < NMAIN; ++m) {
      fetch_for_position(DT + NQK + m);
      const int s4 = m / DT, t = m % DT;
#pragma unroll
      for (int b = 0; b < QB; ++b) {
        o[b][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(opnd[NQK + m], __builtin_bit_cast(bf16x8, pq[b][s4]), o[b][t], 0, 0, 0);
        // early pairs of tile j+1, dealt out over the output slots
#pragma unroll
        for (int n = (QB * m + b) * (QB * NEARLY) / (QB * NMAIN); n < (QB * m + b + 1) * (QB * NEARLY) / (QB * NMAIN); ++n)
          early[n / NEARLY][n % NEARLY] = exp_pair_of(s_next, n / NEARLY, n % NEARLY);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
#pragma unroll
    for (int t = 0; t < DT; ++t) cout.a[t] = opnd[NQK + NMAIN + t];
#pragma unroll
    for (int b = 0; b < QB; ++b) cout.p[b] = pq[b][NPAIR / 4 - 1];
    dma_wait_all();
    __syncthreads();
  };

  uint32_t j = 0;
  const bool steady = nfull >= 4;
  if (steady) {
    // what has been accumulated when the steady state ends is relative to reference 0
#pragma unroll
    for (int b = 0; b < QB; ++b) m_run[b] = 0.0f;
#pragma unroll
    for (int b = 0; b < QB; ++b)
#pragma unroll
      for (int w = 0; w < NEARLY; ++w) early[b][w] = exp_pair_of(sa, b, w);
    // the first trip has no predecessor: its carried slots add zero
    Carry ca, cb;
#pragma unroll
    for (int t = 0; t < DT; ++t) ca.a[t] = __builtin_bit_cast(bf16x8, u32x4{0, 0, 0, 0});
#pragma unroll
    for (int b = 0; b < QB; ++b) ca.p[b] = u32x4{0, 0, 0, 0};
    for (; j + 4 <= nfull; j += 2) {  // j + 3 <= nfull - 1
      fast_step(j, 0, sa, sb, ca, cb, No{});
      fast_step(j + 1, 1, sb, sa, cb, ca, No{});
    }
    // last key group of the last steady-state tile
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int b = 0; b < QB; ++b)
        o[b][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ca.a[t], __builtin_bit_cast(bf16x8, ca.p[b]), o[b][t], 0, 0, 0);
  }
  // the general loop from tile j on (running max per tile, partial tiles): sa holds S(j); S(j+1) is computed
  // after the softmax of tile j, into the same registers
  auto general_loop = [&](uint32_t j) {
    for (; j < ntiles; ++j) {
      const int buf = j & 1;
      if (j + 2 < ntiles) request_k(j + 2, buf);
      if (j + 1 < ntiles) request_v(j + 1, buf ^ 1);
      softmax_pv(sa, j, buf, j >= nfull);
      if (j + 1 < ntiles) qk(sa, buf ^ 1);
      dma_wait_all();
      __syncthreads();
    }
  };
  // the last tiles (no successor, or a partial one)
  general_loop(j);
  {
    if (steady) {
      // did the pass without a reference stay inside the floating-point range, for every wave of the workgroup?
      bool lane_bad = bad;
#pragma unroll
      for (int b = 0; b < QB; ++b) {
        const float row_sum = half_sum(l_run[b]);
        lane_bad = lane_bad || !(row_sum > 0x1p-100f && row_sum < INFINITY);
      }
      // one word per wave in the tile memory, which nobody reads any more after the loop's last barrier
      int* wave_flags = reinterpret_cast<int*>(&smem[0][0][0]);
      if (lane == 0) wave_flags[wave] = __builtin_amdgcn_ballot_w64(lane_bad) != 0;
      __syncthreads();
      int redo = 0;
#pragma unroll
      for (int w = 0; w < NWAVES; ++w) redo |= wave_flags[w];
      if (redo != 0) {
        __syncthreads();  // every wave has read the flags before the tile requests overwrite them
        // throw the pass away and compute the item again, every tile through the general loop
#pragma unroll
        for (int b = 0; b < QB; ++b) {
#pragma unroll
          for (int t = 0; t < DT; ++t)
#pragma unroll
            for (int i = 0; i < 16; ++i) o[b][t][i] = 0.0f;
          m_run[b] = -INFINITY;
          l_run[b] = 0.0f;
        }
        first_tiles();
        general_loop(0);
      }
    }
  }

  // ---- epilogue: normalise and store.  Lane (c, h) holds O[q = c][32 t + 8 g + 4 h + e].
#pragma unroll
  for (int b = 0; b < QB; ++b) {
    const float inv = 1.0f / half_sum(l_run[b]);
    if (qrow[b] < p.nq) {
      if (p.out_bf16) {
        bf16_t* O = reinterpret_cast<bf16_t*>(p.o) + ((size_t)head * p.nq + qrow[b]) * d;
#pragma unroll
        for (int t = 0; t < DT; ++t)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            bf16x4 w;
#pragma unroll
            for (int e = 0; e < 4; ++e) w[e] = (bf16_t)(o[b][t][4 * g + e] * inv);
            *reinterpret_cast<bf16x4*>(O + 32 * t + 8 * g + 4 * h) = w;
          }
      } else {
        float* O = reinterpret_cast<float*>(p.o) + ((size_t)head * p.nq + qrow[b]) * d;
#pragma unroll
        for (int t = 0; t < DT; ++t)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            f32x4 w;
#pragma unroll
            for (int e = 0; e < 4; ++e) w[e] = o[b][t][4 * g + e] * inv;
            *reinterpret_cast<f32x4*>(O + 32 * t + 8 * g + 4 * h) = w;
          }
      }
    }
  }
  clock_note(p.clock, true);
}
