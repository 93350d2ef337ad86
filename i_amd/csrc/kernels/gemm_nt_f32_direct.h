// C[m,n] = sum_k A[m,k] * B[n,k]  for f32 operands (the reference's own arithmetic type; products and sums in
// f32, f32 out) on gfx950, large-tile form on v_mfma_f32_32x32x2_f32: a 256 x 256 (or 128 x 128) output tile per
// workgroup, K in slabs of 32, operand slabs moved from global memory straight into LDS.
//
// Device form of the fused 𝚒 nest  i("ik*jk~ijk") >> i("+ijk~ij ... k0")
// (README.md:16; annotated-flashattn.c:57-89 shows the same pair with a tile-local
// output): tile loops i, j -> workgroups, the k loop is sequential per workgroup,
// i', j' -> MFMA lanes, and the product never exists outside a register.  bf16 operands run the same design on
// 16x16x32 MFMAs (gemm_nt_bf16_mfma16.h).
//
//   workgroup   8 waves as 2 (m) x 4 (n); a wave owns 128 x 64 of the tile = 4 x 2 accumulators of 32 x 32
//               (128 registers)
//   slabs       A and B slabs are both [256 rows][32 k] f32 = 128-byte rows.  One
//               global_load_lds_dwordx4 of a wave deposits 8 rows (1 KiB) contiguously
//               in LDS; the 16-byte chunk a lane fetches is XOR-ed with (row / 2) % 8 so
//               that the 16 rows one quarter-wave reads for an MFMA operand fall into
//               16 different bank groups.  Two slab buffers: slab s+1 is requested at the
//               top of iteration s and awaited (vmcnt(0) + barrier) at its end.
//   operands    both A rows and B rows are K-contiguous, so both MFMA operands are plain ds_read_b128 of
//               (row, chunk 2 ks + h).  The instruction's operands are one f32 per lane with k = lane / 32: a
//               16-byte operand read covers k = 4 (2 ks + h) .. + 3, and element e of it feeds MFMA e of the k-step.
//   L2          the workgroup ids that land on one XCD (id % 8) walk blocks of 4 x 8
//               tiles, so at any time an XCD streams 1024 rows of A and 2048 rows of B
//   M, N edges  rows past the end re-read the last valid row and are not stored
// Requires k % 32 == 0, or k % 4 == 0 with KTAIL.
#pragma once

#include "common.h"
#include "params.h"

// BT x BT output tile per workgroup of WM x WN waves: 256 with 2 x 4 waves (one workgroup per CU) for large
// problems, 128 with 2 x 2 waves (two workgroups per CU) for problems with too few 256-tiles to fill the chip.
// KTAIL: k is a multiple of 4 but not of 32, the last slab is partial: a lane whose 16-byte chunk lies past k
// transfers nothing and clears its LDS slot instead, so the slab reads as zeros there.
template <int BT, int WM, int WN, bool KTAIL = false>
__device__ __forceinline__ void gemm_nt_f32_direct_body(const GemmParams& p) {
  constexpr int BMT = BT, BNT = BT;
  constexpr int ELEM = 4;            // bytes per operand element
  constexpr int BK = 128 / ELEM;      // k per slab: 128-byte slab rows
  constexpr int NWAVES = WM * WN;
  constexpr int TM = BMT / WM / 32;  // 32-row accumulator tiles per wave
  constexpr int TN = BNT / WN / 32;
  constexpr int RB = ELEM * BK;      // bytes per slab row
  constexpr int CH = RB / 16;        // chunks per row (= lanes per row of a wave-load)
  constexpr int RPW = 64 / CH;       // rows per wave-load
  constexpr int SLAB = BMT * RB;     // bytes of one operand slab (BMT == BNT)
  constexpr int WL = SLAB / 1024;    // wave-loads per slab
  constexpr int WLW = WL / NWAVES;   // ... per wave
  constexpr int KS = RB / 32;        // k-steps per slab: two 16-byte chunks (one per half-wave) each
  static_assert(BMT == BNT && WL % NWAVES == 0 && NWAVES % 2 == 0, "slab shape");
  __shared__ __attribute__((aligned(1024))) char smem[2][2][SLAB];  // [buffer][A, B]

  // ---- tile of this workgroup
  uint32_t tm, tn;
  if (!gemm_tile_of_workgroup(blockIdx.x, blockIdx.y, p.tiles_m, p.tiles_n, tm, tn)) return;
  // (the k loop split over workgroups, as in the bf16 kernels: blockIdx.y counts (batch, split) pairs, split s
  // contracts k_chunk * s .. + kk and writes its partial products to c[blockIdx.y])
  const uint32_t nsplit = p.splits > 1 ? p.splits : 1;
  const uint32_t batch = blockIdx.y / nsplit, split = blockIdx.y - batch * nsplit;
  const uint32_t k_first = split * p.k_chunk;
  const uint32_t kk = nsplit > 1 ? (p.k - k_first < p.k_chunk ? p.k - k_first : p.k_chunk) : p.k;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave % WM, wn = wave / WM;
  const int c = lane & 31, h = lane >> 5;

  const size_t row_bytes = (size_t)p.k * ELEM;
  const char* __restrict__ A = reinterpret_cast<const char*>(p.a) + (size_t)batch * p.m * row_bytes + (size_t)k_first * ELEM;
  const char* __restrict__ B = reinterpret_cast<const char*>(p.b) + (size_t)batch * p.n * row_bytes + (size_t)k_first * ELEM;
  float* __restrict__ C = reinterpret_cast<float*>(p.c) + (size_t)blockIdx.y * p.m * p.n;
  const uint32_t m0 = tm * BMT, n0 = tn * BNT;

  // ---- global -> LDS.  Wave-load w of a slab covers slab rows 8 w .. 8 w + 7; this lane's LDS slot is
  // (row 8 w + lane / 8, chunk lane % 8) and it fetches chunk (lane % 8) ^ ((row / 2) % 8) of that row.
  // w = wave + 8 it, so (row / 2) % 8 = (4 (wave % 2) + lane / 16) % 8 does not depend on `it`.
  const uint32_t lrow = lane / CH, lch = lane % CH;
  const uint32_t gch = lch ^ ((4 * (wave & 1) + lane / 16) % CH);
  const uint32_t smem0 = lds_address(&smem[0][0][0]);
  // per-lane byte offsets from the slab's first row of this wave-load; edge tiles clamp the row
  uint32_t aoff[WLW], boff[WLW];
#pragma unroll
  for (int it = 0; it < WLW; ++it) {
    const uint32_t r = (wave + NWAVES * it) * RPW + lrow;
    const uint32_t ra = m0 + r < p.m ? m0 + r : p.m - 1;
    const uint32_t rb = n0 + r < p.n ? n0 + r : p.n - 1;
    aoff[it] = (ra - m0) * (uint32_t)row_bytes + 16 * gch;
    boff[it] = (rb - n0) * (uint32_t)row_bytes + 16 * gch;
  }
  const char* a_tile = A + (size_t)m0 * row_bytes;
  const char* b_tile = B + (size_t)n0 * row_bytes;
  const size_t b_slab_step = (size_t)RB;  // bytes from one k slab of B to the next
  const uint32_t nslabs = KTAIL ? (kk + BK - 1) / BK : kk / BK;
  const uint32_t tail_chunks = (kk - (nslabs - 1) * BK) / 4;  // KTAIL: 16-byte chunks per row of the last slab
  // one transfer of 16 bytes per lane of slab s; KTAIL: nothing to fetch for this lane: its slot is cleared
  auto move = [&](const void* base, uint32_t voff, uint32_t lds_base, uint32_t s) {
    if constexpr (KTAIL) {
      if (s + 1 < nslabs || gch < tail_chunks) dma16(base, voff, lds_base);
      else *reinterpret_cast<u32x4*>(&smem[0][0][0] + (lds_base - smem0) + 16 * lane) = u32x4{0, 0, 0, 0};
    } else {
      dma16(base, voff, lds_base);
    }
  };
  auto request_slab = [&](uint32_t s, int buf) {
    const size_t k_byte = (size_t)s * RB;
#pragma unroll
    for (int it = 0; it < WLW; ++it) {
      const uint32_t w = wave + NWAVES * it;
      move(a_tile + k_byte, aoff[it], smem0 + (2 * buf + 0) * SLAB + w * 1024, s);
      move(b_tile + s * b_slab_step, boff[it], smem0 + (2 * buf + 1) * SLAB + w * 1024, s);
    }
  };

  // ---- LDS -> operands: row (32 i + c) of the wave's rows, chunk (2 ks + h) ^ ((row / 2) % 8)
  const uint32_t fr = (c / 2) % CH;
  uint32_t addr[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) addr[ks] = c * RB + 16 * ((2 * ks + h) ^ fr);
  const uint32_t a_rows = wm * TM * 32 * RB, b_rows = wn * TN * 32 * RB;
  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  request_slab(0, 0);
  dma_wait_all();
  __syncthreads();

  // One trip runs from barrier to barrier.  The barrier that publishes slab s sits before the LAST k-step of
  // slab s-1: that k-step's operands are fetched before the barrier and carried across it in registers, so
  // the trip opens with MFMAs that need nothing from LDS while the first operands of slab s are on their
  // way, and the matrix pipe does not drain at the barrier (both waves of a SIMD belong to this workgroup
  // and reach the barrier together).  Within a trip the operands of the next k-step are fetched while the
  // MFMAs of the current one issue; the global -> LDS requests for slab s+1 (into the buffer slab s-1 has
  // just left) ride on the carried MFMAs.  Scheduling fences keep the order.
  struct Frags {
    f32x4 a[TM], b[TN];
  };
  auto fetch = [&](const char* sa, const char* sb, int ks, Frags& f) {
#pragma unroll
    for (int i = 0; i < TM; ++i) f.a[i] = *reinterpret_cast<const f32x4*>(sa + i * 32 * RB + addr[ks]);
#pragma unroll
    for (int j = 0; j < TN; ++j) f.b[j] = *reinterpret_cast<const f32x4*>(sb + j * 32 * RB + addr[ks]);
  };
  auto mfma = [&](const Frags& f, int i, int j) {
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(f.a[i][e], f.b[j][e], acc[i][j], 0, 0, 0);
  };
  constexpr int NREQ = 2 * WLW;  // slab requests per wave and trip, dealt out over the TM * TN carried MFMAs
  // The last trip has no successor; it requests its own slab once more into the other buffer, which nobody
  // reads any more: one redundant slab per workgroup instead of a branch in every slot.
  auto step = [&](uint32_t s, int buf, const Frags& cin, Frags& cout) {
    const char* sa = &smem[buf][0][0] + a_rows;
    const char* sb = &smem[buf][1][0] + b_rows;
    const uint32_t s_req = s + 1 < nslabs ? s + 1 : s;
    const size_t k_byte = (size_t)s_req * RB;
    Frags f[2];
    fetch(sa, sb, 0, f[0]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        mfma(cin, i, j);
        const int slot = i * TN + j;
#pragma unroll
        for (int r = slot * NREQ / (TM * TN); r < (slot + 1) * NREQ / (TM * TN); ++r) {
          const int it = r % WLW;
          const uint32_t w = wave + NWAVES * it;
          if (r < WLW) move(a_tile + k_byte, aoff[it], smem0 + (2 * (buf ^ 1) + 0) * SLAB + w * 1024, s_req);
          else move(b_tile + s_req * b_slab_step, boff[it], smem0 + (2 * (buf ^ 1) + 1) * SLAB + w * 1024, s_req);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
    for (int ks = 0; ks + 1 < KS; ++ks) {
      if (ks + 2 < KS) fetch(sa, sb, ks + 1, f[(ks + 1) & 1]);
      else fetch(sa, sb, ks + 1, cout);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          mfma(f[ks & 1], i, j);
          __builtin_amdgcn_sched_barrier(0);
        }
    }
    dma_wait_all();
    __syncthreads();
  };
  Frags ca, cb;  // the first trip has no predecessor: its carried MFMAs add zero
#pragma unroll
  for (int i = 0; i < TM; ++i) ca.a[i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int j = 0; j < TN; ++j) ca.b[j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  uint32_t s = 0;
  for (; s + 2 <= nslabs; s += 2) {  // two per trip so that the buffer index is a constant
    step(s, 0, ca, cb);
    step(s + 1, 1, cb, ca);
  }
  if (s < nslabs) {
    step(s, 0, ca, cb);
    ca = cb;
  }
  // last k-step of the last slab
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) mfma(ca, i, j);

  // ---- store.  Accumulator layout: column n = c, rows 8 (e / 4) + 4 h + e % 4: every store instruction
  // writes two full 128-byte lines.  C is written once and not read again: non-temporal.
  const bool interior = m0 + BMT <= p.m && n0 + BNT <= p.n;
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const uint32_t col = n0 + (wn * TN + j) * 32 + c;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const uint32_t row = m0 + (wm * TM + i) * 32 + 8 * (e >> 2) + 4 * h + (e & 3);
        if (interior || (row < p.m && col < p.n)) __builtin_nontemporal_store(acc[i][j][e], &C[(size_t)row * p.n + col]);
      }
    }
}
