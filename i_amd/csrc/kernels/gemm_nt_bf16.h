// C[m,n] = sum_k A[m,k] * B[n,k]  (bf16 in, f32 accumulate and f32 out) on gfx950.
//
// Device form of the fused 𝚒 nest  i("ik*jk~ijk") >> i("+ijk~ij ... k0"): the
// product is folded to a scalar inside the reduction (README.md:16,
// annotated-flashattn.c:57-89 shows the same pair with a tile-local output).
// Tile loops i, j -> workgroups; the k loop is sequential per workgroup and
// staged through LDS in BK-wide slabs; i', j' -> MFMA lanes.
#pragma once
#include "common.h"
#include "params.h"

template <int BMT, int BNT, int BK>
struct GemmSmem {
  static constexpr int S = BK + 8;
  bf16_t a[2][BMT * S];
  bf16_t b[2][BNT * S];
};

// WM x WN waves, each owning a (BMT/WM) x (BNT/WN) sub-tile of 32x32 MFMA tiles.
template <int BMT, int BNT, int BK, int WM, int WN>
__device__ __forceinline__ void gemm_nt_bf16_body(const GemmParams& p) {
  constexpr int NT = WM * WN * WAVE;
  constexpr int TM = BMT / WM / 32;
  constexpr int TN = BNT / WN / 32;
  constexpr int CH = BK / 8;
  constexpr int A_ITERS = BMT * CH / NT;
  constexpr int B_ITERS = BNT * CH / NT;
  using Smem = GemmSmem<BMT, BNT, BK>;
  __shared__ __attribute__((aligned(16))) Smem sm;

  // XCD-aware tile order: the ids that land on one XCD walk a column of
  // m-tiles for a fixed group of n-tiles, so B slabs stay in that XCD's L2.
  const uint32_t tiles = p.tiles_m * p.tiles_n;
  uint32_t lin = blockIdx.x;
  const uint32_t batch = lin / (((tiles + 7) / 8) * 8);
  lin -= batch * (((tiles + 7) / 8) * 8);
  const uint32_t per_xcd = (tiles + 7) / 8;
  const uint32_t tile = ((lin + batch) & 7u) * per_xcd + (lin >> 3);  // (the runs rotate over the XCDs from batch to batch)
  if (tile >= tiles) return;
  const uint32_t tn = tile / p.tiles_m;
  const uint32_t tm = tile % p.tiles_m;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave % WM, wn = wave / WM;
  const int c = lane & 31, h = lane >> 5;

  const bf16_t* __restrict__ A = reinterpret_cast<const bf16_t*>(p.a) + (size_t)batch * p.m * p.k;
  const bf16_t* __restrict__ B = reinterpret_cast<const bf16_t*>(p.b) + (size_t)batch * p.n * p.k;
  float* __restrict__ C = reinterpret_cast<float*>(reinterpret_cast<char*>(p.c) + (size_t)batch * p.m * p.n * (p.out_bf16 ? 2 : 4));
  const uint32_t m0 = tm * BMT, n0 = tn * BNT;

  u32x4 areg[A_ITERS], breg[B_ITERS];
  auto load_slab = [&](uint32_t k0) {
#pragma unroll
    for (int it = 0; it < A_ITERS; ++it) {
      const int idx = tid + it * NT;
      const int row = idx / CH, ch = idx % CH;
      u32x4 z = {0, 0, 0, 0};
      if (m0 + row < p.m && k0 + 8 * ch < p.k) z = ldg128(A + (size_t)(m0 + row) * p.k + k0 + 8 * ch);
      areg[it] = z;
    }
#pragma unroll
    for (int it = 0; it < B_ITERS; ++it) {
      const int idx = tid + it * NT;
      const int row = idx / CH, ch = idx % CH;
      u32x4 z = {0, 0, 0, 0};
      if (n0 + row < p.n && k0 + 8 * ch < p.k) z = ldg128(B + (size_t)(n0 + row) * p.k + k0 + 8 * ch);
      breg[it] = z;
    }
  };
  auto store_slab = [&](int buf) {
#pragma unroll
    for (int it = 0; it < A_ITERS; ++it) {
      const int idx = tid + it * NT;
      *reinterpret_cast<u32x4*>(&sm.a[buf][(idx / CH) * Smem::S + 8 * (idx % CH)]) = areg[it];
    }
#pragma unroll
    for (int it = 0; it < B_ITERS; ++it) {
      const int idx = tid + it * NT;
      *reinterpret_cast<u32x4*>(&sm.b[buf][(idx / CH) * Smem::S + 8 * (idx % CH)]) = breg[it];
    }
  };

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  const uint32_t nslabs = (p.k + BK - 1) / BK;
  load_slab(0);
  store_slab(0);
  __syncthreads();
  for (uint32_t s = 0; s < nslabs; ++s) {
    const int buf = s & 1;
    if (s + 1 < nslabs) load_slab((s + 1) * BK);
    const bf16_t* sa = &sm.a[buf][(wm * TM * 32 + c) * Smem::S + 8 * h];
    const bf16_t* sb = &sm.b[buf][(wn * TN * 32 + c) * Smem::S + 8 * h];
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      bf16x8 af[TM], bfr[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) af[i] = *reinterpret_cast<const bf16x8*>(sa + i * 32 * Smem::S + 16 * ks);
#pragma unroll
      for (int j = 0; j < TN; ++j) bfr[j] = *reinterpret_cast<const bf16x8*>(sb + j * 32 * Smem::S + 16 * ks);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
    }
    if (s + 1 < nslabs) store_slab(buf ^ 1);
    __syncthreads();
  }

  // accumulator layout: column n = c, rows 8(e/4) + 4h + e%4
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const uint32_t col = n0 + (wn * TN + j) * 32 + c;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const uint32_t row = m0 + (wm * TM + i) * 32 + 8 * (e >> 2) + 4 * h + (e & 3);
        if (row < p.m && col < p.n) {
          if (p.out_bf16) reinterpret_cast<bf16_t*>(C)[(size_t)row * p.n + col] = (bf16_t)acc[i][j][e];
          else C[(size_t)row * p.n + col] = acc[i][j][e];
        }
      }
    }
}
