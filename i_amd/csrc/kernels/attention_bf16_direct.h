// FlashAttention forward, bf16 in / f32 accumulate, for d == dv == DPAD:
// K and V tiles go from global memory straight into LDS (no register staging).
//
// Same mapping of work as attention_bf16.h (one query per lane, S^T = K Q^T,
// O^T += V^T P^T, running max / sum with exp-shift corrections).  What differs
// is how the K/V tiles reach the matrix cores:
//
//   global -> LDS   global_load_lds_dwordx4: every lane fetches 16 bytes and
//                   the wave deposits them as one contiguous 1 KiB run of LDS.
//                   A tile is a contiguous BN * 2*DPAD byte piece of K (or V),
//                   so wave-load w of a tile fills LDS bytes [1024 w, 1024 w + 1024).
//   swizzle         rows are 256 (DPAD 128) or 128 (DPAD 64) bytes, so unpadded
//                   rows would collide in the banks.  The 16-byte chunk index is
//                   XOR-ed with a function of the row, applied on the GLOBAL side
//                   (a lane chooses which chunk it fetches for its fixed LDS slot):
//                     K: chunk ^= (row / RPB) % KMOD        16 consecutive rows, same
//                                                           chunk -> 16 different bank groups
//                     V: chunk ^= 4 * ((row / RPB) % VMOD)  4 consecutive rows, same
//                                                           64-byte group -> 4 different groups
//                   (RPB = rows per 256 bytes, at least 1; KMOD = 16 / RPB and VMOD = 4 / RPB: the chunks and the
//                   64-byte groups of the 256-byte bank window that a row can be sent to).
//   LDS -> K operand  ds_read_b128 of row (32 kt + c), chunk (2 ks + h): the A operand of
//                   v_mfma_f32_32x32x16_bf16 exactly as in attention_bf16.h.
//   LDS -> V operand  V stays row-major [key][dv]; ds_read_b64_tr_b16 transposes while
//                   reading.  Within a 16-lane block, lane 4j+q supplies the address of
//                   V[kb + j][dv0 + 4q .. +4) and lane i receives V[kb + 0..3][dv0 + i].
//                   Two such reads (kb = 16 s4 + 4 h and + 8) give the 8 keys that the
//                   P^T B-operand (the S^T accumulator layout) holds in the same lane.
//
// The transfers cost neither vector registers nor LDS-write instructions.  They are
// software-pipelined against the arithmetic: while the softmax of tile j runs on the
// vector pipe, the scores of tile j+1 are computed on the matrix pipe, so K is consumed
// one trip before V.  K(j+2) and V(j+1) are requested early in trip j, into the buffer
// of K(j) and of V(j-1) (both last read before the barrier that opens the trip), and are
// awaited (vmcnt(0) + barrier) at the end of the trip.  One barrier per tile, and one after the
// first score tile (K(2) goes into the buffer of K(0)).
//
// Other differences from attention_bf16.h:
//   * in the steady state no row max is taken at all.  d = 64: probabilities are computed against
//     the reference the row already has and the reference is only moved (with the exp-shift
//     correction of O and l) when a tile's row sum reaches 2^40, checked before that tile's
//     PV product.  d = 128: no reference either (P = exp2 of the score as it is); a workgroup
//     whose rows leave the floating-point range computes its item a second time with the
//     running max.  The remaining tiles move the reference when the tile max exceeds it by 2^8;
//   * scale * log2(e) is folded into Q when it is loaded (one more bf16 rounding), so a score is
//     the argument of its exp2;
//   * the row sum is taken over the bf16-rounded probabilities with v_dot2c_f32_bf16
//     (two terms per instruction), i.e. over exactly the weights the PV product uses.
//
// QB: a wave owns QB blocks of 32 query rows instead of one, so every K or V operand that is read from LDS feeds
// QB MFMAs (one per block), which divides the LDS reads per flop by QB.  At d = 64 the registers allow QB = 2 with
// two waves per SIMD (O 64 + two score tiles of 32 keys 64 + Q 32 + P 16), which a wave needs there because only
// about half of an MFMA's 32 cycles can be covered by its own vector work; at d = 128 it would take the whole
// register file of a SIMD for one wave, and that form measured slower.  With 32-key tiles, 8 waves form a
// workgroup of 512 queries; such a tile of K or V is only 4 wave-loads, so waves 0-3 request K and waves 4-7
// request V (SPLIT below).
#pragma once
#include <type_traits>

#include "common.h"
#include "params.h"

// extra operand-fetch lead of the steady-state loop, in operands (see fast_step): one query block per wave, several
#ifndef ATTN_XLEAD
#define ATTN_XLEAD 1
#endif
#ifndef ATTN_Q64_XLEAD
#define ATTN_Q64_XLEAD 0
#endif
// d = 128: steady state without any reference for the exponentials (see NOREF below)
#ifndef ATTN_NOREF
#define ATTN_NOREF 1
#endif
#ifndef ATTN_STAGED_STORE
#define ATTN_STAGED_STORE 1
#endif

// PRECISE: the score scale is applied in f32 to every score (the reference's arithmetic,
// compiler/src/lower/exec_plan_to_module.rs:605-640) instead of being folded into Q with one more bf16 rounding;
// the steady state then keeps a reference for its exponentials at either head size.  About 5 % slower.
//
// PADDED: d = p.d and dv = p.dv are any multiples of 8 up to DPAD.  The tiles in LDS keep their DPAD-wide rows: a
// lane whose 16-byte chunk lies past the end of a row fetches nothing, and the tile memory is cleared once before
// the first transfer, so the columns d .. DPAD - 1 of K and dv .. DPAD - 1 of V read as zeros for the whole kernel
// (Q is padded with zeros in its registers; the output columns past dv are not stored).  Global rows of Q and K are
// 2 p.d bytes apart, those of V 2 p.dv (and those of O p.dv elements).
template <int DPAD, int BN, int NWAVES, bool PRECISE = false, bool PADDED = false, int QB = 1>
__device__ __forceinline__ void attn_fwd_bf16_direct_body(const AttnParams& p) {
  constexpr int BM = 32 * QB * NWAVES;
  constexpr int KSTEPS = DPAD / 16;       // k-steps of the QK^T contraction
  constexpr int KT = BN / 32;             // 32-key accumulator tiles
  constexpr int DT = DPAD / 32;           // 32-column output tiles
  constexpr int RB = 2 * DPAD;            // bytes per K/V row
  constexpr int CH = RB / 16;             // 16-byte chunks per row (= lanes per row of a wave-load)
  constexpr int RPB = RB >= 256 ? 1 : 256 / RB;  // rows per 256 bytes (1 for longer rows, which start at the same banks)
  constexpr int KMOD = 16 / RPB;          // K swizzle: values of the chunk XOR
  constexpr int VMOD = 4 / RPB;           // V swizzle: values of the 64-byte group XOR
  constexpr int RPW = 64 / CH;            // rows per wave-load
  constexpr int TILE_BYTES = BN * RB;
  constexpr int WL = TILE_BYTES / 1024;   // wave-loads per tile
  // Either every wave requests WLW wave-loads of K and WLW of V per tile, or (SPLIT: a tile has fewer wave-loads
  // than the workgroup has waves) waves 0 .. WL-1 request one wave-load of K each and waves WL .. 2 WL-1 one of V.
  constexpr bool SPLIT = WL < NWAVES;
  constexpr int WLW = SPLIT ? 1 : WL / NWAVES;  // ... per wave
  static_assert(RB == 128 || RB == 256 || RB == 512, "row size");
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
  const uint32_t d = PADDED ? p.d : (uint32_t)DPAD;    // elements per row of Q and K in global memory
  const uint32_t dv = PADDED ? p.dv : (uint32_t)DPAD;  // ... of V and O
  const uint32_t RBG = 2 * d, RBGV = 2 * dv;            // bytes per global row of K, of V (RB when not PADDED)
  const uint32_t chunks = d / 8, chunks_v = dv / 8;     // 16-byte chunks per global row

  // The keys of a head split over workgroups (p.kv_splits > 1): `head` then counts (head, part) pairs.  A part runs
  // the keys first_key .. first_key + nk of its head as if they were all there are and leaves its normalised result in
  // o[head] (a temporary) and, per query row, the base-2 logarithm of its sum of exponentials in p.lse[head];
  // attn_kv_merge puts the parts together.
  uint32_t qhead = head, first_key = 0, nk = p.nk;
  if (p.kv_splits > 1) {
    qhead = head / p.kv_splits;
    first_key = (head - qhead * p.kv_splits) * p.kv_chunk;
    nk = p.nk - first_key < p.kv_chunk ? p.nk - first_key : p.kv_chunk;
  }
  const bf16_t* __restrict__ Q = reinterpret_cast<const bf16_t*>(p.q) + (size_t)qhead * p.nq * d;
  const char* __restrict__ K = reinterpret_cast<const char*>(p.k) + ((size_t)qhead * p.nk + first_key) * RBG;
  const char* __restrict__ V = reinterpret_cast<const char*>(p.v) + ((size_t)qhead * p.nk + first_key) * RBGV;

  // A negative scale is folded into Q (sign flip is exact), so the running max
  // can be tracked on the raw scores: max_j(s_j * scale) == scale * max_j(s_j).
  //
  // PRESCALE (d = 64, where the softmax and not the MFMAs sets the pace: half the MFMA work per exponential): the
  // whole factor scale * log2(e) is folded into Q, rounded to bf16 once more, and in the steady state the score
  // accumulators start at -reference instead of 0 (a 16-register tuple as the MFMA's addend), so that a score
  // comes out of the matrix pipe as the argument of its exp2 and the vector pipe does one instruction less per
  // score.  The extra rounding of Q perturbs a score by about 0.007 in the exponent (0.5 % of a probability,
  // independent from key to key), the size of the bf16 rounding of the probability itself.
  //
  // NOREF (d = 128, where the 16 registers of that tuple do not exist): Q is scaled in the same way and the steady
  // state takes P = exp2(score) as it is, without a reference at all.  The normalised result does not depend on
  // the reference, and with probabilities rounded to bf16 (same exponent range as f32) neither does its precision,
  // as long as nothing overflows or the whole row underflows; scores of attention stay within a few tens.  A
  // wave notes (without branching) whether any tile's row sum reached 2^80 and, at the end, whether a row sum
  // fell below 2^-100; if any wave of the workgroup did, the workgroup throws the pass away and computes the item
  // again with the general loop, which takes the running max tile by tile.
  // (Also the steady state of d = 64 with several query blocks per wave, which has no registers for the tuples either.)
  constexpr bool NOREF = (DPAD >= 128 || QB > 1) && ATTN_NOREF && !PRECISE;
  constexpr bool PRESCALE = DPAD == 64 && !NOREF && !PRECISE;
  constexpr bool QSCALE = PRESCALE || NOREF;
  // f32 output written through LDS (see the epilogue): 8 KiB of tile memory per wave
  constexpr bool STAGED_STORE = ATTN_STAGED_STORE && NWAVES * 8192 <= 4 * TILE_BYTES;
  const float scale_raw = load_scale(p.scale_ptr, p.scale_value);
  const uint32_t sign_flip = scale_raw < 0.0f ? 0x80008000u : 0u;
  const float scale_log2 = QSCALE ? 1.0f : fabsf(scale_raw) * I_LOG2_E32;
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
      if (qrow[b] < p.nq && (!PADDED || (uint32_t)(16 * ks + 8 * h) < d)) z = ldg128(Q + (size_t)qrow[b] * d + 16 * ks + 8 * h);
      if constexpr (QSCALE) {
        bf16x8 scaled = __builtin_bit_cast(bf16x8, z);
#pragma unroll
        for (int e = 0; e < 8; ++e) scaled[e] = (bf16_t)((float)scaled[e] * q_factor);
        qf[b][ks] = scaled;
      } else {
        z ^= sign_flip;
        qf[b][ks] = __builtin_bit_cast(bf16x8, z);
      }
    }
  }

  f32x16 o[QB][DT];
  float m_run[QB];   // running max of the raw scores
  float l_run[QB];   // running sum over this half-wave's keys
  float mb_run[QB];  // m_run * scale_log2, kept while the steady-state loop runs
#pragma unroll
  for (int b = 0; b < QB; ++b) {
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[b][t][i] = 0.0f;
    m_run[b] = -INFINITY;
    l_run[b] = 0.0f;
    mb_run[b] = 0.0f;
  }

  const uint32_t nfull_tiles = nk / BN;  // tiles that lie entirely inside nk
  // ---- global -> LDS: this lane's slot in wave-load w is tile row w*RPW + lane/CH, chunk lane%CH
  const uint32_t lrow = lane / CH, lch = lane % CH;
  const uint32_t smem0 = lds_address(&smem[0][0][0]);

  // For a full tile the per-lane part of the address is the same for every tile, and for every wave-load when
  // the NWAVES * RPW rows between a wave's consecutive wave-loads are a multiple of the swizzle period.  With
  // fewer waves (KSTRIDE < CH) the K swizzle of wave-load `it` differs from that of wave-load 0 in the bits
  // (KSTRIDE * it) % KMOD, which the rows of one wave-load (fewer than KSTRIDE swizzle steps) never reach: one
  // XOR with a constant.  Everything else that varies is wave-uniform and is folded into the scalar base address.
  constexpr int KSTRIDE = NWAVES * RPW / RPB;  // swizzle steps between consecutive wave-loads of a wave
  static_assert((KSTRIDE & (KSTRIDE - 1)) == 0 && (KSTRIDE % KMOD == 0 || KMOD % KSTRIDE == 0), "swizzle period");
  static_assert((NWAVES * RPW / RPB) % VMOD == 0, "V swizzle period");
  const bool k_wave = !SPLIT || wave < WL;   // this wave takes part in K requests
  const bool v_wave = !SPLIT || wave >= WL;  // ... in V requests
  const uint32_t wave_w = SPLIT ? wave % WL : wave;  // its first wave-load
  const uint32_t lane_row = wave_w * RPW + lrow;
  const uint32_t kch_lane = lch ^ ((lane_row / RPB) % KMOD), vch_lane = lch ^ (4 * ((lane_row / RPB) % VMOD));
  const uint32_t koff_lane = lrow * RBG + 16 * kch_lane;
  const uint32_t voff_lane = lrow * RBGV + 16 * vch_lane;
  // K offset of wave-load `it`: the chunk of wave-load 0 with the constant XOR-ed in.  (On the byte offset itself
  // when the row part cannot reach the chunk bits, i.e. when rows are a power of two long: not PADDED.)
  auto koff_of = [&](int it) {
    const uint32_t x = (uint32_t)(KSTRIDE * it) % KMOD;
    if constexpr (PADDED) return lrow * RBG + 16 * (kch_lane ^ x);
    else return koff_lane ^ (16u * x);
  };
  // a transfer of 16 bytes per lane; PADDED: only by the lanes whose chunk exists in the global row
  auto dma16_chunk = [&](bool taking_part, const void* base, uint32_t voff, uint32_t lds_base, uint32_t chunk, uint32_t row_chunks) {
    if (!taking_part) return;
    if constexpr (PADDED) {
      if (chunk < row_chunks) dma16(base, voff, lds_base);
    } else {
      dma16(base, voff, lds_base);
    }
  };
  // one wave-load of a full tile: `it` of K (want_k) or of V
  auto request_full_one = [&](uint32_t tile, int buf, int it, auto want_k) {
    const uint32_t w = wave_w + NWAVES * it;
    const size_t row0 = (size_t)tile * BN + w * RPW;  // PADDED: first row of the wave-load
    if constexpr (decltype(want_k)::value)
      dma16_chunk(k_wave, K + (PADDED ? row0 * RBG : (size_t)tile * TILE_BYTES + w * 1024), koff_of(it),
                  smem0 + (2 * buf + 0) * TILE_BYTES + w * 1024, kch_lane ^ ((uint32_t)(KSTRIDE * it) % KMOD), chunks);
    else
      dma16_chunk(v_wave, V + (PADDED ? row0 * RBGV : (size_t)tile * TILE_BYTES + w * 1024), voff_lane,
                  smem0 + (2 * buf + 1) * TILE_BYTES + w * 1024, vch_lane, chunks_v);
  };

  // one wave-load of K of any tile index: full tile, partial tile (rows past nk re-read the last row), or none
  auto request_k_one = [&](uint32_t tile, int buf, int it) {
    if (tile < nfull_tiles) {
      const uint32_t w = wave_w + NWAVES * it;
      dma16_chunk(k_wave, K + (PADDED ? ((size_t)tile * BN + w * RPW) * RBG : (size_t)tile * TILE_BYTES + w * 1024),
                  koff_of(it), smem0 + (2 * buf + 0) * TILE_BYTES + w * 1024, kch_lane ^ ((uint32_t)(KSTRIDE * it) % KMOD), chunks);
    } else if (tile * BN < nk) {
      const uint32_t w = wave_w + NWAVES * it;
      const uint32_t row = w * RPW + lrow;
      uint32_t key = tile * BN + row;
      key = key < nk ? key : nk - 1;
      const uint32_t kch = lch ^ ((row / RPB) % KMOD);
      dma16_chunk(k_wave, K, key * RBG + 16 * kch, smem0 + (2 * buf + 0) * TILE_BYTES + w * 1024, kch, chunks);
    }
  };

  // PARTIAL: the tile runs past nk; rows past the end re-read the last row (their scores are masked).
  auto request_tile = [&](uint32_t key0, int buf, auto partial_tag, auto want_k, auto want_v) {
    constexpr bool PARTIAL = decltype(partial_tag)::value;
#pragma unroll
    for (int it = 0; it < WLW; ++it) {
      const uint32_t w = wave_w + NWAVES * it;
      const uint32_t row = w * RPW + lrow;  // row within the tile
      const uint32_t kch = lch ^ ((row / RPB) % KMOD);
      const uint32_t vch = lch ^ (4 * ((row / RPB) % VMOD));
      uint32_t key = key0 + row;
      if constexpr (PARTIAL) key = key < nk ? key : nk - 1;
      if constexpr (decltype(want_k)::value) dma16_chunk(k_wave, K, key * RBG + 16 * kch, smem0 + (2 * buf + 0) * TILE_BYTES + w * 1024, kch, chunks);
      if constexpr (decltype(want_v)::value) dma16_chunk(v_wave, V, key * RBGV + 16 * vch, smem0 + (2 * buf + 1) * TILE_BYTES + w * 1024, vch, chunks_v);
    }
  };

  // ---- LDS -> operands: per-lane byte offsets inside a tile
  // K: row c (+ 32 kt), chunk (2 ks + h) ^ fk, where fk depends on c only
  const uint32_t fk = (c / RPB) % KMOD;
  uint32_t kaddr[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) kaddr[ks] = c * RB + 16 * ((2 * ks + h) ^ fk);
  // V: 16-lane block b = lane / 16 covers columns 16 (b & 1) .. +16 of a 32-column tile; lane 4 jj + q of
  // the block points at key (4 h + jj), columns 4 q .. +4
  const uint32_t blk = lane >> 4, jj = (lane >> 2) & 3, qq = lane & 3;
  const uint32_t gv = 4 * (((4 * h + jj) / RPB) % VMOD);
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
            if (key >= nk) s[b][kt][i] = -INFINITY;
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
            if (key >= nk) e = 0.0f;
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
        const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
        for (int b = 0; b < QB; ++b)
          o[b][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, both), pb[b][s4 >> 1][s4 & 1],
                                                            o[b][t], 0, 0, 0);
      }
    }
  };

  using No = std::integral_constant<bool, false>;
  using Yes = std::integral_constant<bool, true>;
  const uint32_t ntiles = (nk + BN - 1) / BN;
  const uint32_t nfull = nk / BN;  // tiles that lie entirely inside nk

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

  // Steady state (tiles j, j+1, j+2 are all full tiles).  One trip runs from barrier to barrier and is
  // written as a sequence of MFMA slots, everything else dealt out between the MFMAs a few vector
  // instructions per slot, so that the matrix pipe and the vector pipe of the SIMD are fed by the same
  // wave at the same time.  A scheduling fence after every slot keeps this order.  The trip uses
  // NOP = NQK + NPV operands (K rows, then transposed V columns); operand k feeds the QB slots
  // QB k .. QB k + QB - 1, one per query block:
  //   QB * DT slots          last 16-key group of O += V(j-1)^T P(j-1)^T, operands and probabilities carried
  //                          in registers across the barrier
  //   QB * NQK slots         S(j+1) = K(j+1) Q^T
  //                          (these QB (DT + NQK) slots also carry the global -> LDS requests for K(j+2), V(j+1)
  //                          and the later part of P(j) = exp(S(j) - reference), its bf16 rounding and the row sum)
  //   QB * (NPV - DT) slots  O += V(j)^T P(j)^T for all but the last 16-key group
  //                          (these slots carry the first pairs of P(j+1): S(j+1) is complete by then)
  // LDS operands are fetched in operand order, DT + XLEAD operands ahead of their first MFMA; the fetches for
  // the carried group are the last ones before the barrier, so the barrier sits in the middle of a
  // stream of MFMAs instead of at a point where the matrix pipe has drained.
  constexpr int NQK = KSTEPS * KT;      // K operands of the score tile
  constexpr int NPV = (BN / 16) * DT;   // V operands of the output update
  constexpr int NOP = NQK + NPV;
  constexpr int NPAIR = KT * 8;         // score pairs per lane and block; pairs 4 g .. 4 g + 3 are the 16-key group g
  constexpr int NPRE = QB * (DT + NQK); // slots that carry the exponentials (all before the first PV slot of the tile)
  constexpr int NMAIN = NPV - DT;       // V operands of the trip that owns the tile
  constexpr int XLEAD = QB > 1 ? ATTN_Q64_XLEAD : ATTN_XLEAD;
  static_assert(NPAIR % 4 == 0 && 2 * WLW <= NPRE && XLEAD >= 0 && XLEAD < NQK, "slot shape");

  struct Carry {
    bf16x8 a[DT];  // V^T operands of the last 16-key group
    u32x4 p[QB];   // its probabilities, per query block
  };

  // No row max is taken in the steady state.  P = exp(S - reference) is computed against the reference the
  // row already has; floating point is scale-free, so any reference gives the same normalised result as long
  // as nothing overflows.  The tile's row sum (a by-product) is checked before the tile's PV product: if it is
  // not below 2^40 (this includes inf and NaN) for any row of the wave, the reference is moved up to the tile
  // max, O and l are corrected by the exp-shift factor, and the tile's probabilities are recomputed.
  constexpr float SUM_GUARD = 1099511627776.0f;  // 2^40

  // packed probability pairs: pq[b][g][w] holds scores 2 (4 g + w), + 1 of the lane in (kt, i) order, so pq[b][g]
  // is the B operand of 16-key group g of block b.  The empty asm statement ties the pair's vector work to the slot
  // it is written in.  The row-sum parts live across trips, because the first NEARLY pairs of a tile and block are
  // computed one trip early, in the output slots of the previous tile, which otherwise carry no vector work at
  // all, while the score slots are the crowded ones:
  //   four or more key groups per tile (IN_PLACE): key groups 0 and 1, written straight into pq, each once the
  //     MFMAs that read the group's old registers have been issued (pq lives across trips);
  //   fewer groups, several query blocks: one pair per output slot, which waits in `early` for its trip;
  //   fewer groups, one query block: none, every pair is computed in the score slots.
  constexpr bool IN_PLACE = BN / 16 >= 4;
  constexpr int NEARLY = IN_PLACE ? 8 : (QB > 1 ? 2 : 0);
  constexpr int NLATE = NPAIR - NEARLY;
  f32x16 negmb16[QB];  // PRESCALE: -reference in every element, the addend of a score tile's first MFMA
  u32x4 pq[QB][NPAIR / 4];
  uint32_t early[QB][NEARLY > 0 ? NEARLY : 1];
  float psum[QB][2];
#pragma unroll
  for (int b = 0; b < QB; ++b) {
    negmb16[b] = zero16;
    psum[b][0] = psum[b][1] = 0.0f;
  }
  bool bad = false;  // NOREF: some tile's row sum left the safe range
  const bf16x2 ones = {(bf16_t)1.0f, (bf16_t)1.0f};
  // pair pr of block b of score tile s: two exponentials, their bf16 rounding, the row-sum part
  auto exp_pair_of = [&](const f32x16 (&s)[QB][KT], int b, int pr, float mb) -> uint32_t {
    const int pkt = pr / 8, i = 2 * (pr % 8);
    // QSCALE: the steady-state scores are already relative to the reference
    const float e0 = QSCALE ? fast_exp2(s[b][pkt][i]) : fast_exp2(__builtin_fmaf(s[b][pkt][i], scale_log2, -mb));
    const float e1 = QSCALE ? fast_exp2(s[b][pkt][i + 1]) : fast_exp2(__builtin_fmaf(s[b][pkt][i + 1], scale_log2, -mb));
    const bf16x2 pair = {(bf16_t)e0, (bf16_t)e1};
    psum[b][pr & 1] = __builtin_amdgcn_fdot2_f32_bf16(pair, ones, psum[b][pr & 1], false);
    uint32_t packed = __builtin_bit_cast(uint32_t, pair);
    asm volatile("" : "+v"(packed), "+v"(psum[b][pr & 1]));
    return packed;
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

    float mb[QB];
#pragma unroll
    for (int b = 0; b < QB; ++b) {
      mb[b] = mb_run[b];
      if constexpr (!IN_PLACE) {
#pragma unroll
        for (int w = 0; w < NEARLY; ++w) pq[b][0][w] = early[b][w];
      }
    }
    // the late pairs of tile j (the early ones were computed during the previous trip): late pair n of the trip is
    // pair NEARLY + n % NLATE of block n / NLATE
    auto pairs_for_slot = [&](int g) {
#pragma unroll
      for (int n = g * (QB * NLATE) / NPRE; n < (g + 1) * (QB * NLATE) / NPRE; ++n) {
        const int b = n / NLATE, pr = NEARLY + n % NLATE;
        pq[b][pr / 4][pr % 4] = exp_pair_of(s_cur, b, pr, mb[b]);
      }
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
        s_next[b][kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
            opnd[n], qf[b][ks], ks == 0 ? (PRESCALE ? negmb16[b] : zero16) : s_next[b][kt], 0, 0, 0);
        request_for_slot(QB * (DT + n) + b);
        pairs_for_slot(QB * (DT + n) + b);
        __builtin_amdgcn_sched_barrier(0);
      }
    }

    // ---- guard (see above); O at this point holds everything up to and including tile j-1
#pragma unroll
    for (int b = 0; b < QB; ++b) {
      if constexpr (NOREF) {
        // noted, acted upon after the pass.  With reference 0 a score may reach 2^80 / 64 as a probability
        // (about 51 nats) before its tile counts as out of range: O then stays below 2^80 nk max|v|.
        bad = bad || !(psum[b][0] + psum[b][1] < 0x1p80f);
      } else if (__builtin_amdgcn_ballot_w64(!(psum[b][0] + psum[b][1] < SUM_GUARD))) {
        float mx = s_cur[b][0][0];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
          for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s_cur[b][kt][i]);
        mx = half_max(mx);
        if constexpr (PRESCALE) mx += mb_run[b];  // the scores are relative to the reference they were computed against
        const bool move = mx * scale_log2 > mb_run[b];  // the reference only moves up
        const float mb_new = move ? mx * scale_log2 : mb_run[b];
        const float alpha = fast_exp2(mb_run[b] - mb_new);
        if constexpr (PRESCALE) {
          // both score tiles in flight were accumulated against the old reference
          const float delta = mb_new - mb_run[b];
#pragma unroll
          for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
              s_cur[b][kt][i] -= delta;
              s_next[b][kt][i] -= delta;
            }
#pragma unroll
          for (int i = 0; i < 16; ++i) negmb16[b][i] = -mb_new;
        }
        m_run[b] = move ? mx : m_run[b];
        mb_run[b] = mb_new;
        l_run[b] *= alpha;
#pragma unroll
        for (int t = 0; t < DT; ++t)
#pragma unroll
          for (int i = 0; i < 16; ++i) o[b][t][i] *= alpha;
        mb[b] = mb_new;
        psum[b][0] = psum[b][1] = 0.0f;
#pragma unroll
        for (int pr = 0; pr < NPAIR; ++pr) pq[b][pr / 4][pr % 4] = exp_pair_of(s_cur, b, pr, mb[b]);
      }
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
        // the early pairs of tile j+1
        if constexpr (IN_PLACE) {
          // key groups 0 and 1, each once the MFMAs that read the group's old registers have been issued
          if (m >= DT && m < 3 * DT) {
#pragma unroll
            for (int pr = (m - DT) * 4 / DT; pr < (m - DT + 1) * 4 / DT; ++pr)
              pq[b][pr / 4][pr % 4] = exp_pair_of(s_next, b, pr, mb[b]);
          }
        } else if constexpr (NEARLY > 0) {
          // dealt out over the output slots
#pragma unroll
          for (int n = (QB * m + b) * (QB * NEARLY) / (QB * NMAIN); n < (QB * m + b + 1) * (QB * NEARLY) / (QB * NMAIN); ++n)
            early[n / NEARLY][n % NEARLY] = exp_pair_of(s_next, n / NEARLY, n % NEARLY, mb[n / NEARLY]);
        }
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

  // tiles 0 and 1 of K and tile 0 of V into LDS, then S(0)
  if constexpr (PADDED) {
    // the tile memory, cleared once: what no transfer ever writes (the columns past d) then reads as zero
    for (uint32_t at = 16 * tid; at < 4 * TILE_BYTES; at += 16 * 64 * NWAVES)
      *reinterpret_cast<u32x4*>(&smem[0][0][0] + at) = u32x4{0, 0, 0, 0};
    __syncthreads();
  }
  auto first_tiles = [&]() {
    request_k(0, 0);
    request_v(0, 0);
    if (ntiles > 1) request_k(1, 1);
    dma_wait_all();
    __syncthreads();
    qk(sa, 0);
    // the first trip of either loop requests K(2) into the buffer of K(0): not before every wave has read K(0).
    // (Without this barrier a wave that leaves qk early can overwrite rows that a late wave has yet to read,
    // once the request is answered from L2 faster than the late wave gets through its 2 KSTEPS reads.)
    __syncthreads();
  };
  // the general loop from tile j on (running max per tile, partial tiles): sa holds S(j).  S(j+1) is computed
  // after the softmax of tile j, into the same registers: this loop runs for the last one to three tiles (and
  // for the second pass of an item), and a second score tile alive next to the softmax's temporaries is what
  // would push the kernel over its register budget.
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
  first_tiles();

  uint32_t j = 0;
  const bool steady = nfull >= 4;
  if (steady) {
#pragma unroll
    for (int b = 0; b < QB; ++b) {
      if constexpr (NOREF) {
        m_run[b] = 0.0f;  // what has been accumulated when the steady state ends is relative to reference 0
        mb_run[b] = 0.0f;
      } else {
        // nothing has been accumulated yet, so the first tile's max becomes the reference without any correction
        float mx_tile = sa[b][0][0];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
          for (int i = 0; i < 16; ++i) mx_tile = fmaxf(mx_tile, sa[b][kt][i]);
        m_run[b] = half_max(mx_tile);
        mb_run[b] = m_run[b] * scale_log2;
      }
      if constexpr (PRESCALE) {
        // from here to the end of the steady state the score tiles are kept relative to the reference
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
          for (int i = 0; i < 16; ++i) sa[b][kt][i] -= mb_run[b];
#pragma unroll
        for (int i = 0; i < 16; ++i) negmb16[b][i] = -mb_run[b];
      }
#pragma unroll
      for (int pr = 0; pr < NEARLY; ++pr) {
        const uint32_t packed = exp_pair_of(sa, b, pr, mb_run[b]);
        if constexpr (IN_PLACE) pq[b][pr / 4][pr % 4] = packed;
        else early[b][pr] = packed;
      }
    }
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
    // one more trip: tile j+1 is still a full tile, tile j+2 may be partial or absent
    {
      fast_step(j, 0, sa, sb, ca, cb, Yes{});
      ++j;
#pragma unroll
      for (int b = 0; b < QB; ++b)
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) sa[b][kt] = sb[b][kt];
      ca = cb;
    }
    // last key group of the last steady-state tile
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int b = 0; b < QB; ++b)
        o[b][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ca.a[t], __builtin_bit_cast(bf16x8, ca.p[b]), o[b][t], 0, 0, 0);
    if constexpr (PRESCALE) {
      // the general loop below works on scores as they are
#pragma unroll
      for (int b = 0; b < QB; ++b)
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
          for (int i = 0; i < 16; ++i) sa[b][kt][i] += mb_run[b];
    }
  }
  // the last tiles (no successor, or a partial one)
  general_loop(j);
  if constexpr (NOREF) {
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
      __syncthreads();  // every wave has read the flags before tile requests or the epilogue overwrite them
      if (redo != 0) {
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

  // ---- epilogue: normalise and store.  Lane (c, h) holds O[q = c][32 t + 8 g + 4 h + e] of each of its blocks.
  float inv[QB];
#pragma unroll
  for (int b = 0; b < QB; ++b) {
    const float row_total = half_sum(l_run[b]);
    inv[b] = 1.0f / row_total;
    if (p.kv_splits > 1 && qrow[b] < p.nq && h == 0)
      p.lse[(size_t)head * p.nq + qrow[b]] = m_run[b] * scale_log2 + log2f(row_total);
    if (qrow[b] < p.nq) {
      if (p.out_bf16) {
        bf16_t* O = reinterpret_cast<bf16_t*>(p.o) + ((size_t)head * p.nq + qrow[b]) * dv;
#pragma unroll
        for (int t = 0; t < DT; ++t)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            bf16x4 w;
#pragma unroll
            for (int e = 0; e < 4; ++e) w[e] = (bf16_t)(o[b][t][4 * g + e] * inv[b]);
            if (!PADDED || (uint32_t)(32 * t + 8 * g + 4 * h) < dv) *reinterpret_cast<bf16x4*>(O + 32 * t + 8 * g + 4 * h) = w;
          }
      } else if constexpr (!STAGED_STORE) {
        float* O = reinterpret_cast<float*>(p.o) + ((size_t)head * p.nq + qrow[b]) * dv;
#pragma unroll
        for (int t = 0; t < DT; ++t)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            f32x4 w;
#pragma unroll
            for (int e = 0; e < 4; ++e) w[e] = o[b][t][4 * g + e] * inv[b];
            if (!PADDED || (uint32_t)(32 * t + 8 * g + 4 * h) < dv) *reinterpret_cast<f32x4*>(O + 32 * t + 8 * g + 4 * h) = w;
          }
      }
    }
  }
  if constexpr (STAGED_STORE) {
    // f32 output through LDS.  In the accumulator layout a lane owns a query row, so a store instruction would
    // touch 32 rows with 32 bytes each (32 cache lines); staged through the tile memory, which nobody reads any
    // more, an instruction writes 4 rows x 256 contiguous bytes (8 lines).  Each wave stages 32 rows x 64 columns
    // of its own at a time in 8 KiB of its own: no workgroup barrier, LDS instructions of a wave execute in order.
    // The 16-byte chunk index of a row is XOR-ed with row % 16, which spreads both the row-per-lane writes and
    // the 4-rows-per-instruction reads over the banks.
    if (!p.out_bf16) {
      // lane coordinates taken afresh (behind an opaque copy), so that nothing computed here is kept in
      // registers through the main loop
      uint32_t tid2 = threadIdx.x;
      asm volatile("" : "+v"(tid2));
      const uint32_t lane = tid2 & 63, c = tid2 & 31, h = (tid2 >> 5) & 1;
      const uint32_t wave = __builtin_amdgcn_readfirstlane(tid2 >> 6);
      char* stage = &smem[0][0][0] + wave * 8192;
#pragma unroll
      for (int b = 0; b < QB; ++b) {
        const uint32_t row0 = qt * BM + wave * (32 * QB) + 32 * b;  // first query row of this block
        const uint32_t rows_valid = row0 < p.nq ? (p.nq - row0 < 32u ? p.nq - row0 : 32u) : 0u;
        float* O = reinterpret_cast<float*>(p.o) + ((size_t)head * p.nq + row0) * dv;
#pragma unroll
        for (int half = 0; half < DT / 2; ++half) {
#pragma unroll
          for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
              f32x4 w;
#pragma unroll
              for (int e = 0; e < 4; ++e) w[e] = o[b][2 * half + tt][4 * g + e] * inv[b];
              *reinterpret_cast<f32x4*>(stage + c * 256 + 16 * ((8 * tt + 2 * g + h) ^ (c & 15))) = w;
            }
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
          for (int it = 0; it < 8; ++it) {
            const uint32_t r = 4 * it + (lane >> 4), q = lane & 15;
            const f32x4 w = *reinterpret_cast<const f32x4*>(stage + r * 256 + 16 * (q ^ (r & 15)));
            if (r < rows_valid && (!PADDED || 64 * half + 4 * q < dv)) *reinterpret_cast<f32x4*>(O + (size_t)r * dv + 64 * half + 4 * q) = w;
          }
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        }
      }
    }
  }
  clock_note(p.clock, true);
}
