// C[m,n] = sum_k A[m,k] * B[n,k]  (bf16 in, f32 accumulate, f32 or bf16 out) on gfx950, large-tile form on
// v_mfma_f32_16x16x32_bf16.
//
// Same device form of the fused 𝚒 nest  i("ik*jk~ijk") >> i("+ijk~ij ... k0")  (README.md:16;
// annotated-flashattn.c:57-89) as gemm_nt_f32_direct.h (the f32-operand kernel, on 32 x 32 MFMAs), with the same
// slabs, the same global -> LDS transfers, the same swizzle and the same workgroup -> tile mapping; what differs
// is the matrix instruction and what follows from it.  On operands that toggle the datapath (anything but constants) the chip sustains more
// 16x16x32 MFMAs per second than 32x32x16 ones under its power limit, at the same operand traffic from LDS.
//
//   workgroup   WM x WN waves on a BTM x BTN tile of C (BTM rows of A against BTN rows of B; square but for the
//               192 x 256 and 256 x 192 forms, which are one full round of workgroups where 256 x 256 tiles leave a
//               partly empty one: 3072^3, 6144^3); a wave owns (BTM / WM) x (BTN / WN) of the tile as TM x TN accumulators of
//               16 x 16 (256 x 256 with 2 x 4 waves: 8 x 4 accumulators, 128 registers; with 2 x 2 waves, one per
//               SIMD: 8 x 8 accumulators, the 256 registers of the accumulation file, a third fewer operand
//               reads per matrix instruction; that form's matrix instructions are inline assembly, see kstep)
//   operands    a lane holds 8 consecutive k of one row: row = lane % 16 of the 16-row fragment, 16-byte
//               chunk 4 ks + lane / 16 of the 128-byte slab row (ks = 0, 1: two k-steps of 32 per slab).
//               The 16 rows one quarter-wave reads with one ds_read_b128 fall into 16 different bank groups
//               because the chunk is XOR-ed with (row / 2) % 8 on the way in.
//   roles       the B rows are passed as the instruction's first operand and the A rows as its second, so
//               a lane ends up with C[m = lane % 16][n = 4 (lane / 16) .. + 3] of each accumulator: four
//               consecutive columns, one 16-byte (f32) or 8-byte (bf16) store
//   registers   operand fragments are refilled in place: fragment i of A is reloaded with the next k-step's
//               rows right after its last MFMA of this k-step; the B fragments alternate between two sets
//   trips       as in gemm_nt_f32_direct.h one trip runs from barrier to barrier, opens with the last k-step
//               of the previous slab (operands carried across the barrier in registers) and requests slab
//               s + 1 into the buffer that slab s - 1 has just left
//   edges       a tile that lies wholly inside C (EDGE = false) steps from one wave-load to the next by a scalar
//               add on the base address and keeps one per-lane offset; a tile that overhangs m or n
//               (EDGE = true) re-reads the last valid row for the rows past the end, which makes the offset
//               of every wave-load a per-lane value, recomputed at each request, and checks what it stores
//   store       plain (cached) stores: the tile leaves through L2, and the write-back to memory overlaps
//               whatever runs next
//
// NN = true is the same kernel for a row-major right operand, C[m,n] = sum_k A[m,k] * B[k,n] (the reference's
// test.py matmul  ik*kj~ijk  and the demo's standalone mm  ij*jk~ikj).  A B slab is then [64 k][BT n]: rows of
// 2 BT bytes, of which one wave-load deposits 1 KiB (2 or 4 rows) contiguously, 16 slab rows per round of the
// workgroup's wave-loads.  The instruction wants 8 consecutive k for one n per lane, a column of the slab,
// which ds_read_b64_tr_b16 delivers: within a 16-lane block, lane 4 jj + q supplies the address of slab row
// k0 + jj, columns 4 q .. + 4 of a 16-column fragment, and lane c receives column c of rows k0 .. k0 + 3; two
// such reads (k0 = 32 ks + 8 (lane / 16) and + 4) complete the lane's 8 k.  Two 16-lane blocks read 8 rows x
// 32 bytes at a time (rows 0-3 and 8-11 of a k-step, then 4-7 and 12-15, ...), so the 32-byte unit index of a
// row is XOR-ed, on the global side, with f(row) = row % 4 + 4 ((row / 8) % 2), which sends those 8 rows to 8
// different bank groups.  Requires n % 8 == 0 as well; 16-byte chunks that start past n re-read the row's last
// chunk (their columns are not stored).
//
// KTAIL = true is the same kernel for k that is a multiple of 8 but not of 64: the last slab is partial.  The lanes
// whose 16-byte chunk (NN: whose slab row of B) lies past k transfer nothing and clear their LDS slot instead, so
// the slab reads as zeros there and the k loop runs over whole slabs as before.
// Requires k % 64 == 0, or k % 8 == 0 with KTAIL.
#pragma once
#include <type_traits>

#include "common.h"
#include "params.h"

template <int BTM, int BTN, int WM, int WN, bool EDGE, bool NN, bool KTAIL>
__device__ __forceinline__ void gemm_nt_mfma16_tile(const GemmParams& p, char* smem_base, uint32_t tm, uint32_t tn) {
  constexpr int RB = 128;            // bytes per slab row: 64 k of bf16
  constexpr int BK = 64;
  constexpr int NWAVES = WM * WN;
  constexpr int TM = BTM / WM / 16;  // 16-row fragments of A per wave
  constexpr int TN = BTN / WN / 16;  // 16-row fragments of B per wave
  constexpr int CH = RB / 16;        // 16-byte chunks per row
  constexpr int RPW = 64 / CH;       // rows per wave-load
  constexpr int SLAB_A = BTM * RB, SLAB_B = BTN * RB, SLABS = SLAB_A + SLAB_B;  // a buffer: the A slab, then the B slab
  constexpr int WLW_A = SLAB_A / 1024 / NWAVES;  // wave-loads per slab and wave
  constexpr int WLW_B = SLAB_B / 1024 / NWAVES;
  constexpr int WLW = WLW_A > WLW_B ? WLW_A : WLW_B;
  static_assert(SLAB_A % (1024 * NWAVES) == 0 && SLAB_B % (1024 * NWAVES) == 0 && NWAVES % 2 == 0 && TM >= 2 && TN >= 2, "slab shape");
  static_assert(!NN || BTM == BTN, "the row-major right operand has square tiles only");
  // slab `which` (0: A, 1: B) of buffer `buf`
  auto slab = [&](int buf, int which) { return smem_base + buf * SLABS + which * SLAB_A; };
  // (the k loop split over workgroups: blockIdx.y counts (batch, split) pairs)
  const uint32_t nsplit = p.splits > 1 ? p.splits : 1u;
  const uint32_t batch = blockIdx.y / nsplit, split = blockIdx.y - batch * nsplit;
  const uint32_t k_first = split * p.k_chunk;                                            // first k of this split
  const uint32_t kk = nsplit > 1 ? (p.k - k_first < p.k_chunk ? p.k - k_first : p.k_chunk) : p.k;  // its extent

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave % WM, wn = wave / WM;
  const uint32_t c16 = lane & 15, g = lane >> 4;

  const size_t row_bytes = (size_t)p.k * 2;
  const char* __restrict__ A = reinterpret_cast<const char*>(p.a) + (size_t)batch * p.m * row_bytes + (size_t)k_first * 2;
  const char* __restrict__ B = reinterpret_cast<const char*>(p.b) + (size_t)batch * p.n * row_bytes +
                               (NN ? (size_t)k_first * p.n * 2 : (size_t)k_first * 2);  // (NN: rows of B are k)
  char* __restrict__ C = reinterpret_cast<char*>(p.c) + (size_t)blockIdx.y * p.m * p.n * (p.out_bf16 ? 2 : 4);
  const uint32_t m0 = tm * BTM, n0 = tn * BTN;

  // ---- global -> LDS.  Wave-load w of a slab covers slab rows 8 w .. 8 w + 7; this lane's LDS slot is
  // (row 8 w + lane / 8, chunk lane % 8) and it fetches chunk (lane % 8) ^ ((row / 2) % 8) of that row.
  // w = wave + NWAVES it with NWAVES even, so (row / 2) % 8 = (4 (wave % 2) + lane / 16) % 8 for every `it`.
  const uint32_t lrow = lane / CH, lch = lane % CH;
  const uint32_t gch = lch ^ ((4 * (wave & 1) + lane / 16) % CH);
  const uint32_t smem0 = lds_address(smem_base);
  // Per-lane byte offset of this lane's 16 bytes from the first row of its wave-load.  EDGE: from the tile's
  // first row, with the row clamped, recomputed at every request (held in registers it would cost 2 WLW of
  // them; the empty asm keeps the compiler from hoisting the values back out of the loop).
  const uint32_t rbase = wave * RPW + lrow, ch_bytes = 16 * gch;
  const uint32_t voff0 = rbase * (uint32_t)row_bytes + ch_bytes;
  const size_t it_stride = (size_t)(NWAVES * RPW) * row_bytes;  // bytes from one wave-load of a wave to its next
  const uint32_t lim_a = p.m - 1 - m0, lim_b = p.n - 1 - n0;
  auto row_offset = [&](int it, uint32_t lim) {
    uint32_t r = rbase;
    asm volatile("" : "+v"(r));
    r += NWAVES * RPW * it;
    return (r < lim ? r : lim) * (uint32_t)row_bytes + ch_bytes;
  };
  uint32_t voff_it[WLW];  // (k <= 2^22: 256 rows of 2 k bytes stay below 2^32)
#pragma unroll
  for (int it = 0; it < WLW; ++it) voff_it[it] = voff0 + (uint32_t)it * (uint32_t)it_stride;
  const char* a_tile = A + (size_t)m0 * row_bytes;
  const char* b_tile = NN ? B + (size_t)n0 * 2 : B + (size_t)n0 * row_bytes;
  // NN: wave-load w of a B slab covers slab rows (k) RPWN w .. + RPWN - 1; this lane's LDS slot is (row, chunk
  // lane % CHN) and it fetches chunk (lane % CHN) ^ 2 f(row) of that row.  Rounds of wave-loads are 16 rows apart,
  // which changes neither f(row) nor the clamp, so one per-lane offset serves every request.
  constexpr int RBN = 2 * BTN;        // bytes per row of an NN slab
  constexpr int CHN = RBN / 16;       // chunks per row
  constexpr int RPWN = 1024 / RBN;    // rows per wave-load
  // (with four waves a round of wave-loads is 8 rows, and f(row) of a lane alternates between two values from one
  // round to the next: two offsets, by the parity of the round)
  constexpr int NN_ROUND = NWAVES * RPWN;  // slab rows per round of the workgroup's wave-loads
  static_assert(!NN || NN_ROUND == 16 || NN_ROUND == 8, "NN slab rounds");
  const size_t brow_bytes = (size_t)p.n * 2;  // NN: a row of B is n elements
  uint32_t boff_nn[2] = {0, 0};
  if constexpr (NN) {
    const uint32_t last_chunk = (p.n - n0) / 8 - 1;  // n % 8 == 0 and n0 < n
#pragma unroll
    for (int parity = 0; parity < 2; ++parity) {
      const uint32_t r = wave * RPWN + lane / CHN + (NN_ROUND == 8 ? 8 * parity : 0);
      uint32_t ch = (lane % CHN) ^ (2 * ((r & 3) | (((r >> 3) & 1) << 2)));
      ch = ch < last_chunk ? ch : last_chunk;
      boff_nn[parity] = (wave * RPWN + lane / CHN) * (uint32_t)brow_bytes + 16 * ch;
    }
  }
  const uint32_t nslabs = KTAIL ? (kk + BK - 1) / BK : kk / BK;
  // KTAIL: what exists of the last slab: 16-byte chunks per row (rows of k for an NN slab of B)
  const uint32_t tail_chunks = (kk - (nslabs - 1) * BK) / 8;
  // a transfer of 16 bytes per lane; KTAIL: a lane that has nothing to fetch (`valid` false) clears its slot
  auto move = [&](const void* base, uint32_t voff, uint32_t lds_base, bool valid) {
    if constexpr (KTAIL) {
      if (valid) dma16(base, voff, lds_base);
      else *reinterpret_cast<u32x4*>(smem_base + (lds_base - smem0) + 16 * lane) = u32x4{0, 0, 0, 0};
    } else {
      dma16(base, voff, lds_base);
    }
  };
  // request r of the WLW_A + WLW_B that bring slab s into `buf` (A first); `tail`: slab s may be the partial one (KTAIL)
  auto request = [&](uint32_t s, int buf, int r, auto tail) {
    const int it = r < WLW_A ? r : r - WLW_A;
    const uint32_t w = wave + NWAVES * it;
    const size_t k_byte = (size_t)s * RB;
    const uint32_t to_a = smem0 + buf * SLABS + w * 1024, to_b = smem0 + buf * SLABS + SLAB_A + w * 1024;
    const bool whole = !KTAIL || !decltype(tail)::value || s + 1 < nslabs;  // the slab lies inside k
    const bool valid = whole || gch < tail_chunks;         // ... or this lane's chunk of a K-contiguous row does
    if (r >= WLW_A && NN) {
      const bool valid_row = whole || (w * RPWN + lane / CHN) < 8 * tail_chunks;
      move(b_tile + ((size_t)s * BK + NN_ROUND * it) * brow_bytes, boff_nn[NN_ROUND == 8 ? it % 2 : 0], to_b, valid_row);
    } else if constexpr (EDGE) {
      if (r < WLW_A) move(a_tile + k_byte, row_offset(it, lim_a), to_a, valid);
      else move(b_tile + k_byte, row_offset(it, lim_b), to_b, valid);
    } else if constexpr (TM * TN > 32) {
      // (one wave per SIMD: nothing hides the scalar address arithmetic of a request, so the wave-loads differ in
      // a per-lane offset kept in a register each, and the base moves once per slab)
      if (r < WLW_A) move(a_tile + k_byte, voff_it[it], to_a, valid);
      else move(b_tile + k_byte, voff_it[it], to_b, valid);
    } else {
      if (r < WLW_A) move(a_tile + k_byte + it * it_stride, voff0, to_a, valid);
      else move(b_tile + k_byte + it * it_stride, voff0, to_b, valid);
    }
  };

  // ---- LDS -> operands: row c16 of a 16-row fragment, chunk (4 ks + g) ^ ((row / 2) % 8); fragments start at
  // multiples of 16 rows, which leaves (row / 2) % 8 = c16 / 2
  uint32_t addr[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) addr[ks] = c16 * RB + 16 * ((4 * ks + g) ^ (c16 / 2));
  const uint32_t a_rows = wm * TM * 16 * RB, b_rows = wn * TN * 16 * RB;
  // NN: lane 4 jj + qq of block g points at slab row 8 g + jj (+ 32 ks, + 4), columns 4 qq .. + 4 of fragment j;
  // f(row) = jj + 4 (g % 2) for both reads of a lane
  typedef __attribute__((ext_vector_type(4))) short s16x4;
  typedef __attribute__((ext_vector_type(8))) short s16x8;
  typedef __attribute__((address_space(3))) s16x4* lds_s16x4_ptr;
  const uint32_t jj = (lane >> 2) & 3, qq = lane & 3;
  // (fragment j of the wave is unit wn TN + j = (wn TN) ^ j of the row, TN being a power of two that j stays below:
  // the fragment's address is the first one's with 32 j XOR-ed in, one instruction instead of TN registers)
  static_assert(!NN || (TN & (TN - 1)) == 0, "fragments per wave");
  const uint32_t baddr0 = NN ? (8 * g + jj) * RBN + 32 * ((uint32_t)(wn * TN) ^ (jj | ((g & 1) << 2))) + 8 * qq : 0u;

  f32x4 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  // The matrix instructions of the 256-accumulator form are inline assembly (see kstep), which the compiler's
  // hazard handling does not look into: the wait states between an ordinary write of an accumulator register
  // and the first matrix instruction that reads it, and between the last matrix instruction and the first
  // ordinary read of its result, are spelled out here and after the k loop.
  constexpr bool ASM_MFMA = TM * TN > 32;
  auto settle = [&]() {
    if constexpr (ASM_MFMA) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) asm volatile("" : "+a"(acc[i][j]));
    }
  };
  if constexpr (ASM_MFMA) {
    settle();                         // the zeros are in their registers here ...
    asm volatile("s_nop 7");          // ... and have landed before anything below reads them
  }

#pragma unroll
  for (int r = 0; r < WLW_A + WLW_B; ++r) request(0, 0, r, std::true_type{});
  dma_wait_all();
  __syncthreads();

  bf16x8 a[TM], b0[TN], b1[TN];
  auto load_a = [&](int buf, int ks, int i) {
    a[i] = *reinterpret_cast<const bf16x8*>(slab(buf, 0) + a_rows + i * 16 * RB + addr[ks]);
  };
  auto load_b = [&](int buf, int ks, int j, bf16x8 (&b)[TN]) {
    if constexpr (NN) {
      uint32_t first = baddr0;
      asm volatile("" : "+v"(first));  // (keeps the TN addresses from being hoisted into registers of their own)
      const char* ba = slab(buf, 1) + 32 * ks * RBN + (first ^ (32u * j));
      const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(ba));
      const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(ba + 4 * RBN));
      b[j] = __builtin_bit_cast(bf16x8, (s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    } else {
      b[j] = *reinterpret_cast<const bf16x8*>(slab(buf, 1) + b_rows + j * 16 * RB + addr[ks]);
    }
  };
  // One k-step: TM x TN MFMAs on (a, bc) while a is refilled in place and bn is filled with the operands of
  // k-step `ks` of buffer `buf`; `reqs` says whether the slab requests of this trip ride on it.
  constexpr int NREQ = WLW_A + WLW_B, NSLOT = TM * TN;
  auto kstep = [&](bf16x8 (&bc)[TN], bf16x8 (&bn)[TN], int buf, int ks, bool refill, auto reqs, uint32_t s_req, int req_buf,
                   auto tail) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        if constexpr (ASM_MFMA) {
          // 256 accumulator registers: named as the accumulation file, the operands as the ordinary one (left to
          // itself the register allocator moves values between the two files three times per instruction)
          asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(bc[j]), "v"(a[i]));
        } else {
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bc[j], a[i], acc[i][j], 0, 0, 0);
        }
        const int slot = i * TN + j;
        if (refill) {
          if (i == 0) load_b(buf, ks, j, bn);
          if (j == TN - 1) load_a(buf, ks, i);
        }
        if constexpr (decltype(reqs)::value) {
#pragma unroll
          for (int r = slot * NREQ / NSLOT; r < (slot + 1) * NREQ / NSLOT; ++r) request(s_req, req_buf, r, tail);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
  };
  // Trip for slab s in buffer `buf`: the carried k-step (operands a, b0) while k-step 0 of slab s arrives in
  // (a, b1) and slab s + 1 is requested; then k-step 0 while k-step 1 arrives in (a, b0), carried into the next
  // trip.  The last trip has no successor; it requests its own slab once more into the other buffer, which
  // nobody reads any more: one redundant slab per workgroup instead of a branch in every slot.
  // `tail`: the slab this trip requests may be the partial one (KTAIL), so its requests carry the per-lane test
  auto trip = [&](uint32_t s, int buf, auto tail) {
    const uint32_t s_req = s + 1 < nslabs ? s + 1 : s;
    kstep(b0, b1, buf, 0, true, std::true_type{}, s_req, buf ^ 1, tail);
    kstep(b1, b0, buf, 1, true, std::false_type{}, 0, 0, std::false_type{});
    dma_wait_all();
    __syncthreads();
  };
  // the first trip has no predecessor: its carried MFMAs add zero
#pragma unroll
  for (int i = 0; i < TM; ++i) a[i] = __builtin_bit_cast(bf16x8, u32x4{0, 0, 0, 0});
#pragma unroll
  for (int j = 0; j < TN; ++j) b0[j] = __builtin_bit_cast(bf16x8, u32x4{0, 0, 0, 0});
  if constexpr (ASM_MFMA) {
    // (these zeros are written by ordinary vector instructions, and a matrix instruction may read a register two
    // wait states after such a write at the earliest: a matrix instruction that came sooner multiplied what the
    // registers held before, which is NaN now and then)
#pragma unroll
    for (int i = 0; i < TM; ++i) asm volatile("" : "+v"(a[i]));
#pragma unroll
    for (int j = 0; j < TN; ++j) asm volatile("" : "+v"(b0[j]));
    asm volatile("s_nop 3");
  }
  uint32_t s = 0;
  // KTAIL: trip s requests slab s + 1, so the trips before nslabs - 2 request whole slabs; the two or three that
  // remain after the pairs of them are written out with the per-lane test
  const uint32_t nplain = KTAIL ? (nslabs > 2 ? (nslabs - 2) & ~1u : 0u) : nslabs;
  for (; s + 2 <= nplain; s += 2) {  // two per iteration so that the buffer index is a constant
    trip(s, 0, std::false_type{});
    trip(s + 1, 1, std::false_type{});
  }
  if constexpr (KTAIL) {
    if (s < nslabs) trip(s, 0, std::true_type{});
    if (s + 1 < nslabs) trip(s + 1, 1, std::true_type{});
    if (s + 2 < nslabs) trip(s + 2, 0, std::true_type{});
  } else {
    if (s < nslabs) trip(s, 0, std::false_type{});
  }
  // last k-step of the last slab
  kstep(b0, b1, 0, 0, false, std::false_type{}, 0, 0, std::false_type{});
  if constexpr (ASM_MFMA) {
    // an 8-pass matrix instruction needs 11 wait states before its result may be read by another kind of
    // instruction; the reads below are tied to this point
    asm volatile("s_nop 15\n\ts_nop 15");
    settle();
  }

  // ---- store.  acc[i][j][r] is C[m0 + 16 (wm TM + i) + c16][n0 + 16 (wn TN + j) + 4 g + r]: a lane writes four
  // consecutive columns at once, a quarter-wave 16 rows of them.  Columns come in fours, so a C whose n is not
  // a multiple of 4 (or whose base is not 16-byte aligned) is stored element by element.
  const bool n4 = p.n % 4 == 0 && reinterpret_cast<uintptr_t>(C) % 16 == 0;
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const uint32_t row = m0 + (wm * TM + i) * 16 + c16;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const uint32_t col = n0 + (wn * TN + j) * 16 + 4 * g;
      const size_t at = (size_t)row * p.n + col;
      if (n4 && (!EDGE || (row < p.m && col < p.n))) {
        if (p.out_bf16) {
          bf16x4 v;
#pragma unroll
          for (int r = 0; r < 4; ++r) v[r] = (bf16_t)acc[i][j][r];
          *reinterpret_cast<bf16x4*>(C + 2 * at) = v;
        } else {
          *reinterpret_cast<f32x4*>(C + 4 * at) = acc[i][j];
        }
      } else if (!EDGE || row < p.m) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (!EDGE || col + r < p.n) {
            if (p.out_bf16) reinterpret_cast<bf16_t*>(C + 2 * at)[r] = (bf16_t)acc[i][j][r];
            else reinterpret_cast<float*>(C + 4 * at)[r] = acc[i][j][r];
          }
      }
    }
  }
}

template <int BTM, int WM, int WN, bool NN = false, bool KTAIL = false, int BTN = BTM>
__device__ __forceinline__ void gemm_nt_mfma16_body(const GemmParams& p) {
  __shared__ __attribute__((aligned(1024))) char smem[2 * (BTM + BTN) * 128];  // [buffer][A: BTM rows, B: BTN rows][128 bytes]
  // ---- tile of this workgroup
  uint32_t tm, tn;
  if (!gemm_tile_of_workgroup(blockIdx.x, blockIdx.y, p.tiles_m, p.tiles_n, tm, tn)) return;
  if ((tm + 1) * BTM <= p.m && (tn + 1) * BTN <= p.n) gemm_nt_mfma16_tile<BTM, BTN, WM, WN, false, NN, KTAIL>(p, smem, tm, tn);
  else gemm_nt_mfma16_tile<BTM, BTN, WM, WN, true, NN, KTAIL>(p, smem, tm, tn);
}
