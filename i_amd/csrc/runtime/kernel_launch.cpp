#include "kernel_launch.h"

#include <cmath>
#include <cstdlib>
#include <initializer_list>
#include <cstdint>
#include <string>

#include "../kernels/params.h"

namespace ihip {
namespace {
constexpr size_t kMaxGrid = 0x7fffffffu;

bool fits_u32(size_t v) { return v <= 0xffffffffull; }
bool aligned16(const void* ptr) { return reinterpret_cast<uintptr_t>(ptr) % 16 == 0; }
}  // namespace

Err set_kernel_option(KernelOptions& o, const std::string& name, int value) {
  auto one_of = [&](std::initializer_list<int> allowed) {
    for (int a : allowed)
      if (a == value) return true;
    return false;
  };
  auto bad = [&](const char* allowed) { return "program option '" + name + "' must be " + allowed + ", not " + std::to_string(value); };
  if (name == "attention.f32_scale") {
    o.attention_f32_scale = value != 0;
  } else if (name == "attention.kv_parts") {
    if (value < 0) return bad("0 (the launcher decides), 1 (never) or a number of parts");
    o.attention_kv_parts = value;
  } else if (name == "attention.waves") {
    if (!one_of({0, 2, 4, 8, 64})) return bad("0, 2, 4 or 8 (or 64: the 64-queries-per-wave kernel for d = 64)");
    o.attention_waves = value;
  } else if (name == "attention.direct") {
    o.attention_direct = value != 0;
  } else if (name == "gemm.k_parts") {
    if (value < 0) return bad("0 (the launcher decides), 1 (never) or a number of parts");
    o.gemm_k_parts = value;
  } else if (name == "gemm.waves") {
    if (!one_of({0, 4, 8})) return bad("0, 4 or 8");
    o.gemm_waves = value;
  } else if (name == "gemm.tile") {
    if (!one_of({0, 128, 192, 256})) return bad("0, 128, 192 (192 x 256) or 256");
    o.gemm_tile = value;
  } else if (name == "gemm.tile_n") {
    if (!one_of({0, 128, 192, 256})) return bad("0 (what goes with gemm.tile), 128, 192 (256 x 192) or 256");
    o.gemm_tile_n = value;
  } else if (name == "gemm.direct") {
    o.gemm_direct = value != 0;
  } else if (name == "generated.only") {
    o.generated_only = value != 0;
  } else if (name == "generated.wave") {
    if (!one_of({-1, 0, 1})) return bad("-1 (the launcher decides), 0 or 1");
    o.generated_wave = value;
  } else if (name == "generated.parts") {
    if (value < 0 || value > 4096) return bad("0 (the launcher decides), 1 (never) or a number of parts up to 4096");
    o.generated_parts = value;
  } else {
    return "unknown program option '" + name +
           "' (known: attention.f32_scale, attention.kv_parts, attention.waves, attention.direct, gemm.k_parts, gemm.waves, "
           "gemm.tile, gemm.tile_n, gemm.direct, generated.only, generated.wave, generated.parts)";
  }
  return {};
}

Err parse_kernel_options(const char* text, KernelOptions* options) {
  if (!text) return {};
  const std::string all(text);
  size_t at = 0;
  auto separator = [](char c) { return c == ' ' || c == ',' || c == ';' || c == '\t' || c == '\n'; };
  while (at < all.size()) {
    while (at < all.size() && separator(all[at])) ++at;
    size_t end = at;
    while (end < all.size() && !separator(all[end])) ++end;
    if (end == at) break;
    const std::string pair = all.substr(at, end - at);
    at = end;
    const size_t eq = pair.find('=');
    if (eq == std::string::npos || eq == 0 || eq + 1 == pair.size()) return "option '" + pair + "' is not of the form name=value";
    char* tail = nullptr;
    const long value = std::strtol(pair.c_str() + eq + 1, &tail, 10);
    if (*tail != '\0') return "option '" + pair + "' has no integer value";
    if (Err e = set_kernel_option(*options, pair.substr(0, eq), (int)value); !e.empty()) return e;
  }
  return {};
}

Err launch_shader_clock_probe(unsigned long long* ticks, unsigned microseconds, hipStream_t stream) {
  if (!ticks) return "clock probe: null device pointer";
  if (reinterpret_cast<uintptr_t>(ticks) % 8 != 0) return "clock probe: the counters must be 8-byte aligned";
  if (microseconds > 2000000u) return "clock probe: at most two seconds";
  ClockProbeParams p{ticks, microseconds * 100u};
  hipFunction_t fn;
  if (Err e = builtin_function("shader_clock_probe", &fn); !e.empty()) return e;
  return launch(fn, 1, 1, 1, 64, &p, sizeof(p), stream);
}

bool attention_supported(DType in_dtype, size_t d, size_t dv, const KernelOptions& knobs) {
  if (d == 0 || dv == 0) return false;
  // head sizes above 128 up to 256: bf16, on the direct kernels only
  if (d > 128 || dv > 128)
    return in_dtype == BF16 && d <= 256 && dv <= 256 && d % 8 == 0 && dv % 8 == 0 && knobs.attention_direct;
  if (in_dtype == BF16) return d % 8 == 0 && dv % 8 == 0;
  return true;
}

Err launch_attention(const void* q, const void* k, const void* v, void* o, DType in_dtype, DType out_dtype, size_t bh,
                     size_t nq, size_t nk, size_t d, size_t dv, const float* scale_ptr, float scale, hipStream_t stream,
                     const AttentionOptions& options, LaunchNote* note) {
  const KernelOptions& knobs = options.knobs;
  if (!attention_supported(in_dtype, d, dv, knobs))
    return "attention kernel: unsupported operands (need 0 < d, dv <= 128, or bf16 with d, dv <= 256; bf16 needs d, dv % 8 == 0)";
  if ((d > 128 || dv > 128) && nk * (d > dv ? d : dv) * 2 >= (size_t(1) << 32))
    return "attention kernel: too many keys for a head size above 128";
  if (!std::isfinite(scale)) return "attention kernel: unsupported scale (must be finite)";
  if (in_dtype == F32 && out_dtype != F32) return "attention kernel: f32 inputs produce f32 output";
  if (bh == 0 || nq == 0) return {};
  if (nk == 0) return "attention kernel: no keys";
  if (!fits_u32(bh) || !fits_u32(nq) || !fits_u32(nk)) return "attention kernel: extent exceeds 32 bits";
  if (!q || !k || !v || !o) return "attention kernel: null device pointer";
  // every bf16 kernel moves 16 bytes per lane (the direct ones straight into LDS) and stores 8 (bf16) or 16 (f32)
  if (in_dtype == BF16 && (!aligned16(q) || !aligned16(k) || !aligned16(v) || reinterpret_cast<uintptr_t>(o) % (out_dtype == BF16 ? 8 : 16) != 0))
    return "attention kernel: bf16 operands must be 16-byte aligned (the output 8-byte for bf16, 16-byte for f32)";

  const size_t dmax = d > dv ? d : dv;
  const size_t query_tile = options.query_tile, key_tile = options.key_tile;
  // Kernel choice for bf16:
  //   d == dv in {64, 128}: direct-to-LDS kernels, templated on the workgroup's query rows (64 / 128 / 256 = 2 / 4 / 8
  //     waves) and on the key tile in LDS (32 / 64).  The schedule's tile decides when such a kernel exists.
  //     Without a usable request: 64-key tiles, and 256 query rows (half the L2 -> LDS traffic per query) on long
  //     key loops when that still leaves at least two workgroups per CU and does not pad nq by much, else 128.
  //     d == 64 on grids with at least two 512-query workgroups per CU (or a schedule tile of 512 x 32): the
  //     64-queries-per-wave kernel, which reads every K/V operand from LDS once for two MFMAs.
  //   any other d, dv that are multiples of 8 up to 128: the 4- and 8-wave kernels with 64-key tiles and their LDS
  //     rows padded to 64 or 128 columns (the larger of d and dv decides).
  //   d or dv above 128 up to 256 (multiples of 8): the kernel for 256-column rows (padded below 256), 4 waves, one
  //     per SIMD, 32-key tiles; nothing else exists above 128, so callers ask attention_supported() first.
  //   otherwise (knobs.attention_direct == 0, key offsets beyond 32 bits): register-staged kernel with guarded
  //     columns (always multiplies the scores in f32)
  // knobs.attention_waves = 2 | 4 | 8 forces the workgroup size of the direct kernel (64: the 64-queries-per-wave
  // kernel, d == 64 only) and knobs.attention_direct = 0 the register-staged kernel; both exist so that tests and
  // searches can reach every kernel with small inputs.
  unsigned bm = 128, bn = 64;
  bool q64 = false;
  const bool exact = in_dtype == BF16 && d == dv && (d == 64 || d == 128);
  const bool wide = in_dtype == BF16 && dmax > 128;  // (supported: d, dv <= 256, multiples of 8)
  const bool padded = in_dtype == BF16 && !exact && d % 8 == 0 && dv % 8 == 0 && !(d == 256 && dv == 256);
  // per-head K/V byte offsets are 32-bit in the direct-to-LDS kernel
  const bool direct = (exact || padded || wide) && nk * dmax * 2 < (size_t(1) << 32) && knobs.attention_direct;
  const bool f32_scale = knobs.attention_f32_scale != 0;
  if (direct && wide) {
    bm = 128;  // 4 waves, one per SIMD
    bn = 32;
  } else if (direct && padded) {
    // 64-key tiles; 256 query rows per workgroup on the grids where the unpadded kernels take them, else 128
    if (query_tile == 256 || (query_tile != 128 && bh * ((nq + 255) / 256) >= 2 * 256 && nk >= 2560 &&
                              10 * ((nq + 255) / 256 * 256) <= 11 * ((nq + 127) / 128 * 128)))
      bm = 256;
    if (const int waves = knobs.attention_waves) {
      if (waves != 4 && waves != 8) return "attention kernel: attention.waves must be 4 or 8 for a padded head size";
      bm = 32u * (unsigned)waves;
    }
  } else if (direct) {
    const bool tile_known = query_tile == 64 || query_tile == 128 || query_tile == 256;
    if (key_tile == 32 && !f32_scale && tile_known && !(d == 64 && query_tile == 256)) bn = 32;
    if (tile_known && !(f32_scale && query_tile == 64)) bm = (unsigned)query_tile;  // the schedule's i split
    else if (d == 64 && !f32_scale &&
             ((query_tile == 512 && (key_tile == 32 || key_tile == 0)) ||
              (query_tile == 0 && bh * ((nq + 511) / 512) >= 2 * 256 &&
               10 * ((nq + 511) / 512 * 512) <= 11 * ((nq + 127) / 128 * 128))))
      q64 = true;
    else if (bh * ((nq + 255) / 256) >= 2 * 256 && nk >= 2560 &&
             10 * ((nq + 255) / 256 * 256) <= 11 * ((nq + 127) / 128 * 128))
      bm = 256;  // ... on long key loops (two resident 4-wave workgroups hide each other's prologue and epilogue,
                 // which wins up to about 2048 keys), and unless rounding nq up to 256 instead of 128 adds more
                 // than 10 % of idle query rows
    if (const int waves = knobs.attention_waves) {
      q64 = waves == 64 && d == 64 && !f32_scale;
      if (!q64) {
        if (waves != 2 && waves != 4 && waves != 8) return "attention kernel: attention.waves must be 2, 4 or 8 (or 64 for d = 64)";
        bm = 32u * (unsigned)waves;
        if (f32_scale && bm == 64) bm = 128;
        if (d == 64 && bm == 256) bn = 64;
      }
    }
    if (q64) { bm = 512; bn = 32; }
  }
  // f32: the direct-to-LDS kernel for d, dv multiples of 4 up to 128, the larger above 32 (16-byte aligned operands,
  // 32-bit byte offsets inside a head; up to 32 the register-staged kernel with 32-column tiles is the faster one), the
  // register-staged kernel with guarded columns otherwise (and with knobs.attention_direct == 0)
  const bool f32_direct = in_dtype == F32 && d % 4 == 0 && dv % 4 == 0 && dmax > 32 && dmax <= 128 &&
                          nk * dmax * 4 < (size_t(1) << 32) && aligned16(q) && aligned16(k) && aligned16(v) && aligned16(o) &&
                          knobs.attention_direct;
  AttnParams p{};
  p.q = q; p.k = k; p.v = v; p.o = o;
  p.bh = (uint32_t)bh; p.nq = (uint32_t)nq; p.nk = (uint32_t)nk; p.d = (uint32_t)d; p.dv = (uint32_t)dv;
  p.nqt = (uint32_t)((nq + bm - 1) / bm);
  p.out_bf16 = out_dtype == BF16 ? 1u : 0u;
  p.scale_ptr = scale_ptr;
  p.scale_value = scale;
  p.clock = knobs.clock_ticks;
  // the keys of a head in several parts: the direct kernels take (head, part) pairs for heads and write to the
  // caller's temporaries; attn_kv_merge follows.  (A request that the kernel chosen above cannot honour, the
  // register-staged ones and the 64-queries-per-wave kernel, is ignored: the result is the same.)
  unsigned splits = 1;
  if (options.kv_splits > 1 && ((in_dtype == BF16 && direct && !q64) || f32_direct)) {
    if (!options.partial_o || !options.partial_lse) return "attention kernel: a split needs its temporaries";
    p.kv_chunk = (uint32_t)(((nk + options.kv_splits - 1) / options.kv_splits + 63) / 64 * 64);
    splits = (unsigned)((nk + p.kv_chunk - 1) / p.kv_chunk);  // (rounding the parts up to whole tiles may leave fewer)
    if (splits > 1) {
      if (!fits_u32(bh * splits)) return "attention kernel: extent exceeds 32 bits";
      p.kv_splits = splits;
      p.bh = (uint32_t)(bh * splits);
      p.o = options.partial_o;
      p.lse = options.partial_lse;
      p.out_bf16 = 0;
    }
  }

  std::string name;
  unsigned threads = 2 * bm;  // one query per lane of a half-wave: 32 queries per wave
  if (in_dtype == BF16) {
    if (direct && q64) {
      name = "attn_fwd_bf16_d64_bn32_q64";
      threads = bm;
    } else if (direct) {
      name = "attn_fwd_bf16_d" + std::to_string(wide ? 256 : padded ? (dmax <= 64 ? 64 : 128) : d) + "_bn" + std::to_string(bn) + "_direct";
      if (bm == 64) name += "_w2";
      if (bm == 256) name += "_w8";
      if (f32_scale) name += "_f32scale";
      if (padded) name += "_pad";
    } else if (exact) name = d == 64 ? "attn_fwd_bf16_d64_bn64" : "attn_fwd_bf16_d128_bn64";
    else name = dmax <= 64 ? "attn_fwd_bf16_d64_bn64_any" : "attn_fwd_bf16_d128_bn64_any";
  } else {
    if (f32_direct) {
      // (head sizes other than d == dv in {64, 128}: the same kernel with its LDS rows padded to 64 or 128 columns)
      name = dmax <= 64 ? "attn_fwd_f32_d64_bn32_direct" : "attn_fwd_f32_d128_bn32_direct";
      if (!(d == dv && (d == 64 || d == 128))) name += "_pad";
    }
    else name = dmax <= 32 ? "attn_fwd_f32_d32_bn32" : dmax <= 64 ? "attn_fwd_f32_d64_bn32" : "attn_fwd_f32_d128_bn32";
    bn = 32;
  }
  if (note) *note = LaunchNote{splits > 1 ? name + " (keys in " + std::to_string(splits) + " parts)" : name, bm, bn};

  const size_t grid = (size_t(p.bh) * p.nqt + 7) / 8 * 8;  // the query tiles of all heads in 8 equal runs, one per XCD
  if (grid > kMaxGrid) return "attention kernel: grid too large";
  hipFunction_t fn;
  if (Err e = builtin_function(name.c_str(), &fn); !e.empty()) return e;
  if (Err e = launch(fn, (unsigned)grid, 1, 1, threads, &p, sizeof(p), stream); !e.empty() || splits == 1) return e;
  AttnMergeParams m{options.partial_o, options.partial_lse, o, (uint32_t)bh, splits, (uint32_t)nq, (uint32_t)dv, out_dtype == BF16 ? 1u : 0u};
  if (Err e = builtin_function("attn_kv_merge", &fn); !e.empty()) return e;
  size_t mgrid = (bh * nq * (dv / 4) + 255) / 256;
  if (mgrid > 65536) mgrid = 65536;
  return launch(fn, (unsigned)mgrid, 1, 1, 256, &m, sizeof(m), stream);
}

// Into how many parts to split the keys of each head (1: do not).  A grid of bh * ceil(nq / 128) workgroups that
// leaves most of the 256 CUs without one (a single head, a few sequences, a few queries against many keys)
// finishes sooner when parts of the key loop run side by side: as many parts as fill the CUs once, of at least 512
// keys each, at most 32, and only for loops of 2048 keys and more (below that the second launch takes what the
// split gains).  Measured, enqueued back to back, d = 128: one head of 8192 x 8192 92 -> 46 us (4 parts), of
// 4096 x 4096 48 -> 27, 128 queries x 8192 keys 91 -> 23 (16 parts), 8 heads of 128 x 16384 176 -> 32; from 256
// workgroups on nothing is gained (16 heads of 4096: 127 -> 146 us with 2 parts).  An f32 workgroup spends four times
// as long on half the keys, so f32 loops are split from 256 keys on, into parts of at least 64: the reference's
// demo, one head of 512 x 64, 45 -> 16 us in 8 parts; 2 heads of 128 queries x 8192 keys of 128, 1136 -> 64 in 32.  Only where the direct kernels run (launch_attention's own
// conditions).
unsigned attention_kv_splits(DType in_dtype, size_t bh, size_t nq, size_t nk, size_t d, size_t dv, const AttentionOptions& options) {
  const KernelOptions& knobs = options.knobs;
  if (bh == 0 || nq == 0 || d == 0 || dv == 0 || !knobs.attention_direct || knobs.attention_kv_parts == 1) return 1;
  const size_t dmax = d > dv ? d : dv;
  if (in_dtype == BF16) {
    if (d % 8 != 0 || dv % 8 != 0 || d > 256 || dv > 256 || !(nk * dmax * 2 < (size_t(1) << 32))) return 1;
    if (knobs.attention_waves == 64) return 1;
    if (options.query_tile == 512) return 1;  // (may select the 64-queries-per-wave kernel)
  } else if (d % 4 != 0 || dv % 4 != 0 || dmax <= 32 || dmax > 128 || !(nk * dmax * 4 < (size_t(1) << 32))) {
    return 1;  // (f32: the direct kernel's head sizes; operands it cannot take for their alignment run unsplit)
  }
  // an f32 workgroup takes about 2.8 us per 32 keys (a bf16 one 0.7 us per 64): much shorter loops are worth parts
  const size_t least_loop = in_dtype == BF16 ? 2048 : 256, least_part = in_dtype == BF16 ? 512 : 64;
  size_t want;
  if (knobs.attention_kv_parts > 1) {
    want = (size_t)knobs.attention_kv_parts;  // forced, still bounded by whole 64-key tiles below
  } else {
    const size_t bm = in_dtype == BF16 && (options.query_tile == 64 || options.query_tile == 256) ? options.query_tile : 128;
    const size_t groups = bh * ((nq + bm - 1) / bm);
    if (nk < least_loop || nk < least_loop / 64 * groups) return 1;  // (half the CUs busy: two parts pay from twice the least loop on)
    want = std::min<size_t>(std::min<size_t>(256 / groups, nk / least_part), 32);
  }
  if (want < 2 || nk < 128) return 1;
  want = std::min<size_t>(want, nk / 64);
  if (want < 2) return 1;
  const size_t chunk = ((nk + want - 1) / want + 63) / 64 * 64;
  return (unsigned)((nk + chunk - 1) / chunk);
}

bool gemm_nt_bf16_supported(size_t k) { return k > 0 && k % 8 == 0; }

// 256 x 256 tiles (one workgroup per CU, 256 at a time) or 128 x 128 tiles (two per CU, 512 at a time) for a
// problem with enough of either?  The larger tile is about 20 % more efficient per flop (1442 against 1237 TFLOP/s
// at 4096^3, whole rounds of either), but its last round of workgroups may leave most of the chip idle: 4608^3 is
// 1.27 rounds of 256-tiles (measured 1061 TFLOP/s) and 2.53 rounds of 128-tiles (1092).  Rounds of the two-per-CU
// kernel count in halves.  A round that leaves part of the chip idle runs its tiles faster (the clock rises when
// fewer CUs draw power): 1600 per filled CU-round against 1460 for full rounds.  (A model, within 3 % of the
// better tile from 1024^3 to 8192^3 in steps of 512.)
static unsigned pick_direct_tile(size_t t256, size_t t128) {
  const double r256 = (double)t256 / 256.0, r128 = (double)t128 / 512.0;
  const double fill256 = r256 / std::ceil(r256);
  const double e256 = (fill256 > 0.95 ? 1460.0 : 1600.0) * fill256;
  const double e128 = (r128 < 1.0 ? 1250.0 : 1150.0) * r128 / (std::ceil(2.0 * r128) / 2.0);
  return e256 >= e128 ? 256 : 128;
}

// A model of a launch's time in us, by which the 192 x 256 tile is weighed against the one chosen above: a fixed
// part (launch, first slab, the store of C), plus the slabs of the k loop times the time of a slab for a full round
// of workgroups (1.5 us on a 256 x 256 tile, 1.154 on 192 x 256, 0.95 on two 128 x 128 tiles per CU), times the
// rounds, a partly empty round counting for 0.55 + half of its fill (fewer busy CUs run a higher clock and share
// L2 and the fabric among fewer); less than one round of 128-tiles is cheaper still (one workgroup per CU).
// Fitted to cubes from 1792 to 8192, where it is within 5 % of the measured times of all three tiles but for the
// 192 x 256 tile from 7168 on, which it flatters by 8 %: that tile has to win by 8 % to be taken.  It is taken at
// 3072^3 (64 against 71 us), 4608^3 (170 against 190) and 6144^3 (344 against 382), and nowhere from 5120 to 5632
// or from 6400 on.
static double direct_tile_time(unsigned tile, size_t tiles, size_t slabs) {
  const double slots = tile == 128 ? 512.0 : 256.0;
  const double slab_us = tile == 128 ? 0.95 : tile == 192 ? 1.154 : 1.5;
  const double r = (double)tiles / slots, whole = std::floor(r), part = r - whole;
  double rounds = whole + (part > 0.0 ? std::min(1.0, 0.55 + 0.5 * part) : 0.0);
  if (tile == 128 && r <= 1.0) rounds = std::min(1.0, 0.25 + 0.85 * r);
  return (tile == 128 ? 9.0 : 12.0) + rounds * (double)slabs * slab_us;
}

Err launch_gemm_nt_bf16(const void* a, const void* b, void* c, size_t bh, size_t m, size_t n, size_t k,
                        hipStream_t stream, size_t tile_m, size_t tile_n, LaunchNote* note, DType out_dtype,
                        const KernelOptions& knobs) {
  if (!gemm_nt_bf16_supported(k)) return "gemm_nt kernel: k must be a positive multiple of 8";
  if (bh == 0 || m == 0 || n == 0) return {};
  if (!fits_u32(m) || !fits_u32(n) || !fits_u32(k) || !fits_u32(bh)) return "gemm_nt kernel: extent exceeds 32 bits";
  if (!a || !b || !c) return "gemm_nt kernel: null device pointer";
  if (!aligned16(a) || !aligned16(b)) return "gemm_nt kernel: operands must be 16-byte aligned";
  GemmParams p{};
  p.a = a; p.b = b; p.c = c;
  p.bh = (uint32_t)bh; p.m = (uint32_t)m; p.n = (uint32_t)n; p.k = (uint32_t)k;
  p.out_bf16 = out_dtype == BF16 ? 1u : 0u;
  // Direct global -> LDS kernels (64-wide k slabs, 32-bit byte offsets inside a tile's rows):
  //   256 x 256 tiles  long k loops on grids that fill at least half of the CUs (its prologue and its
  //                    unoverlapped store only pay off there)
  //   128 x 128 tiles  everything else, two workgroups per CU (down to one tile and one slab it is the faster
  //                    128-tile kernel: 4.3 against 5.9 us at 128 x 128 x 64, 9.4 against 17.0 at 128 x 128 x 1024)
  // (k that is no multiple of 64: their _ktail forms, the last slab partial)
  // and the register-staged 128 x 128 kernel beyond their offset ranges (k > 2^22, more than 65535 batches).
  // The schedule's i, j splits (256 x 256, 192 x 256, 256 x 192 or 128 x 128) decide when given; knobs.gemm_tile
  // = 256 | 192 | 128 (with knobs.gemm_tile_n = 192 for 256 x 192) and
  // knobs.gemm_direct = 0 force a kernel so that tests and searches can reach each of them at small sizes.
  {
    const size_t t256 = ((m + 255) / 256) * ((n + 255) / 256) * bh, t128 = ((m + 127) / 128) * ((n + 127) / 128) * bh;
    // the two rectangular tiles: 192 rows of A against 256 of B, or 256 against 192, whichever leaves fewer tiles
    const size_t t192m = ((m + 191) / 192) * ((n + 255) / 256) * bh, t192n = ((m + 255) / 256) * ((n + 191) / 192) * bh;
    unsigned tile = 128, across = 0;  // rows of A and of B per tile (across 0: as many as of A; tile 0: register-staged kernel)
    if (k >= 512 && t256 >= 64) {
      tile = pick_direct_tile(t256, t128);
      const size_t slabs = (k + 63) / 64;
      if (1.08 * direct_tile_time(192, std::min(t192m, t192n), slabs) < direct_tile_time(tile, tile == 256 ? t256 : t128, slabs)) {
        tile = t192m <= t192n ? 192 : 256;
        across = t192m <= t192n ? 256 : 192;
      }
    }
    if (tile_m == 128 && tile_n == 128) tile = 128, across = 0;
    if ((tile_m == 256 || tile_m == 192) && (tile_n == 256 || tile_n == 192) && tile_m + tile_n >= 448) tile = (unsigned)tile_m, across = (unsigned)tile_n;
    if (knobs.gemm_tile) tile = (unsigned)knobs.gemm_tile, across = (unsigned)knobs.gemm_tile_n;
    if (!across) across = tile == 192 ? 256 : tile;
    if (tile == 192 && across != 256) return "gemm_nt kernel: a 192-row tile goes with 256 columns";
    if (tile == 128 && across != 128) return "gemm_nt kernel: a 128-row tile goes with 128 columns";
    if (tile == 256 && across != 256 && across != 192) return "gemm_nt kernel: a 256-row tile goes with 256 or 192 columns";
    if (!knobs.gemm_direct) tile = 0;
    const bool ktail = k % 64 != 0;
    if (tile && k <= (size_t(1) << 22) && bh <= 65535) {
      p.tiles_m = (uint32_t)((m + tile - 1) / tile);
      p.tiles_n = (uint32_t)((n + across - 1) / across);
      const size_t grid = (size_t(p.tiles_m) * p.tiles_n + 7) / 8 * 8;  // the tiles in 8 equal runs, one per XCD
      if (grid > kMaxGrid) return "gemm_nt kernel: grid too large";
      hipFunction_t fn;
      // the 256 x 256 tile runs with four waves of 128 x 128 (knobs.gemm_waves = 8: the form with eight of 128 x 64,
      // kept for comparison: equal on one round of tiles, 5-10 % behind on several); the rectangular ones with four
      // of 96 x 128 or 128 x 96
      const bool w4 = tile + across == 448 || (tile == 256 && knobs.gemm_waves != 8);
      const std::string name = "gemm_nt_bf16_" + std::to_string(tile) + "x" + std::to_string(across) + "x64_direct" +
                               (ktail ? "_ktail" : "") + (w4 ? "_w4" : "");
      if (note) *note = LaunchNote{name, tile, across};
      if (Err e = builtin_function(name.c_str(), &fn); !e.empty()) return e;
      return launch(fn, (unsigned)grid, (unsigned)bh, 1, w4 || tile == 128 ? 256 : 512, &p, sizeof(p), stream);
    }
  }
  p.tiles_m = (uint32_t)((m + 127) / 128);
  p.tiles_n = (uint32_t)((n + 127) / 128);
  const size_t tiles = (size_t)p.tiles_m * p.tiles_n;
  const size_t grid = ((tiles + 7) / 8 * 8) * bh;
  if (grid > kMaxGrid) return "gemm_nt kernel: grid too large";
  hipFunction_t fn;
  if (note) *note = LaunchNote{"gemm_nt_bf16_128x128x64", 128, 128};
  if (Err e = builtin_function("gemm_nt_bf16_128x128x64", &fn); !e.empty()) return e;
  return launch(fn, (unsigned)grid, 1, 1, 256, &p, sizeof(p), stream);
}

// Tile of a split product: the large tile needs both extents to fill most of it
static unsigned split_k_tile(size_t m, size_t n) { return m >= 192 && n >= 192 ? 256 : 128; }

unsigned gemm_nt_bf16_split_k(size_t bh, size_t m, size_t n, size_t k, const KernelOptions& knobs) {
  if (bh == 0 || m == 0 || n == 0 || k % 8 != 0 || knobs.gemm_k_parts == 1) return 1;
  const unsigned tile = split_k_tile(m, n);
  if (knobs.gemm_k_parts > 1) {  // (tests, searches and measurements: that many parts, whole slabs each)
    const size_t want = std::min<size_t>((size_t)knobs.gemm_k_parts, k / 64);
    if (want < 2 || bh * want > 65535) return 1;
    const size_t chunk = (k / want + 63) / 64 * 64;
    return (unsigned)((k + chunk - 1) / chunk);
  }
  // A model of the time in us, fitted to products from 32 x 4096 x 4096 to 2048 x 2048 x 8192 enqueued back to back
  // (it picks the measured best number of parts, or one within a few per cent of it, on 14 of 16 of them): a
  // workgroup spends 0.7 us per 64-wide slab on a 128 x 128 tile (1.1 us when two share a CU), 1.3 us on a
  // 256 x 256 tile, plus two slabs' worth before and after its loop; the chip holds 512 / 256 of them at a time;
  // the second launch costs 4 us and the pass over the partial products runs at 3 TB/s.  Examples (unsplit ->
  // split): 64 x 8192 x 8192 79 -> 30 us in 8 parts, 512 x 512 x 4096 52 -> 27 in 8, 256 x 4096 x 4096 41 -> 29
  // in 8, 256 x 256 x 65536 576 -> 49 in 32; left whole: 1024^3 (10 us; 25 in 2 parts), 2048^3 (28; 40).
  if (k > (size_t(1) << 22)) return 1;
  const size_t slabs = (k + 63) / 64;
  const size_t t128 = ((m + 127) / 128) * ((n + 127) / 128) * bh, t256 = ((m + 255) / 256) * ((n + 255) / 256) * bh;
  auto time_of = [](unsigned tile_, size_t workgroups, size_t slabs_) {
    const double rounds = (double)((workgroups + (tile_ == 128 ? 511 : 255)) / (tile_ == 128 ? 512 : 256));
    return rounds * (double)(slabs_ + 2) * (tile_ == 128 ? (workgroups <= 256 ? 0.7 : 1.1) : 1.3);
  };
  double best = time_of(128, t128, slabs);
  if (t256 >= 64) best = std::min(best, time_of(256, t256, slabs));
  best *= 0.85;  // a split has to gain at least 15 %
  const size_t tiles = tile == 256 ? t256 : t128;
  size_t splits = 1;
  for (size_t s = 2; s <= 32 && k / s >= 512 && bh * s <= 65535; s *= 2) {
    const double t = time_of(tile, tiles * s, (slabs + s - 1) / s) + 4.0 + (double)(bh * s * m * n * 4) / 3e6;
    if (t < best) {
      best = t;
      splits = s;
    }
  }
  if (splits < 2) return 1;
  const size_t chunk = (k / splits + 63) / 64 * 64;  // what one split contracts: whole 64-wide slabs
  return (unsigned)((k + chunk - 1) / chunk);
}

Err launch_gemm_nt_bf16_split_k(const void* a, const void* b, void* c, float* partial, unsigned splits, size_t bh, size_t m,
                                size_t n, size_t k, hipStream_t stream, LaunchNote* note, DType out_dtype) {
  if (!gemm_nt_bf16_supported(k)) return "gemm_nt kernel: k must be a positive multiple of 8";
  if (splits < 2 || bh * splits > 65535 || !fits_u32(m) || !fits_u32(n) || k > (size_t(1) << 22)) return "gemm_nt kernel: bad split";
  if (!a || !b || !c || !partial) return "gemm_nt kernel: null device pointer";
  if (!aligned16(a) || !aligned16(b)) return "gemm_nt kernel: operands must be 16-byte aligned";
  if ((m * n) % 4 != 0) return "gemm_nt kernel: a split product needs m * n to be a multiple of 4";
  GemmParams p{};
  p.a = a; p.b = b; p.c = partial;
  p.bh = (uint32_t)bh; p.m = (uint32_t)m; p.n = (uint32_t)n; p.k = (uint32_t)k;
  p.k_chunk = (uint32_t)(((k + splits - 1) / splits + 63) / 64 * 64);
  splits = (unsigned)((k + p.k_chunk - 1) / p.k_chunk);  // (rounding the parts up to whole slabs may leave fewer of them)
  if (splits < 2) return "gemm_nt kernel: bad split";
  p.splits = splits;
  const unsigned tile = split_k_tile(m, n);
  p.tiles_m = (uint32_t)((m + tile - 1) / tile);
  p.tiles_n = (uint32_t)((n + tile - 1) / tile);
  const size_t grid = (size_t(p.tiles_m) * p.tiles_n + 7) / 8 * 8;
  if (grid > kMaxGrid) return "gemm_nt kernel: grid too large";
  const bool ktail = k % 64 != 0;  // (only the last split is partial; the others run whole slabs through the same code)
  const std::string name = std::string(tile == 256 ? "gemm_nt_bf16_256x256x64_direct" : "gemm_nt_bf16_128x128x64_direct") +
                           (ktail ? "_ktail" : "") + (tile == 256 ? "_w4" : "");
  if (note) *note = LaunchNote{name + " (k in " + std::to_string(splits) + " parts)", tile, tile};
  hipFunction_t fn;
  if (Err e = builtin_function(name.c_str(), &fn); !e.empty()) return e;
  if (Err e = launch(fn, (unsigned)grid, (unsigned)(bh * splits), 1, 256, &p, sizeof(p), stream); !e.empty()) return e;
  SplitReduceParams r{partial, c, (uint32_t)bh, splits, (uint64_t)m * n, out_dtype == BF16 ? 1u : 0u};
  if (Err e = builtin_function("splitk_reduce", &fn); !e.empty()) return e;
  size_t rgrid = (bh * m * n / 4 + 255) / 256;
  if (rgrid > 65536) rgrid = 65536;
  return launch(fn, (unsigned)rgrid, 1, 1, 256, &r, sizeof(r), stream);
}

static unsigned gemm_nn_tile(size_t bh, size_t m, size_t n, size_t k, size_t tile_m, size_t tile_n, const KernelOptions& knobs) {
  if (k == 0 || k % 8 != 0 || n % 8 != 0 || k > (size_t(1) << 22) || n > (size_t(1) << 24) || bh > 65535) return 0;
  if (!fits_u32(m) || !fits_u32(n)) return 0;
  const size_t t256 = ((m + 255) / 256) * ((n + 255) / 256) * bh, t128 = ((m + 127) / 128) * ((n + 127) / 128) * bh;
  unsigned tile = t256 >= 128 ? pick_direct_tile(t256, t128) : 128;
  if (tile_m == 256 && tile_n == 256) tile = 256;
  if (tile_m == 128 && tile_n == 128) tile = 128;
  if (knobs.gemm_tile) tile = knobs.gemm_tile == 192 ? 256u : (unsigned)knobs.gemm_tile;  // (192 x 256 exists for bf16 NT products only)
  if (!knobs.gemm_direct) tile = 0;  // (no register-staged form of this product: callers transpose and use the NT kernels)
  return tile;
}

bool gemm_nn_bf16_supported(size_t bh, size_t m, size_t n, size_t k, const KernelOptions& knobs) {
  return gemm_nn_tile(bh, m, n, k, 0, 0, knobs) != 0;
}

Err launch_gemm_nn_bf16(const void* a, const void* b, void* c, size_t bh, size_t m, size_t n, size_t k,
                        hipStream_t stream, size_t tile_m, size_t tile_n, LaunchNote* note, DType out_dtype, float* partial,
                        unsigned splits, const KernelOptions& knobs) {
  unsigned tile = gemm_nn_tile(bh, m, n, k, tile_m, tile_n, knobs);
  if (tile == 0) return "gemm_nn kernel: needs k % 8 == 0 and n % 8 == 0 (and extents within its offset range)";
  if (bh == 0 || m == 0 || n == 0) return {};
  if (!a || !b || !c) return "gemm_nn kernel: null device pointer";
  if (!aligned16(a) || !aligned16(b)) return "gemm_nn kernel: operands must be 16-byte aligned";
  GemmParams p{};
  p.a = a; p.b = b; p.c = c;
  p.bh = (uint32_t)bh; p.m = (uint32_t)m; p.n = (uint32_t)n; p.k = (uint32_t)k;
  p.out_bf16 = out_dtype == BF16 ? 1u : 0u;
  // the k loop in parts over workgroups (gemm_nt_bf16_split_k says when, for this form too): f32 partial products
  // in the caller's temporary, added up by splitk_reduce
  if (splits > 1) {
    if (!partial) return "gemm_nn kernel: a split needs its temporary";
    if ((m * n) % 4 != 0) return "gemm_nn kernel: a split product needs m * n to be a multiple of 4";
    p.k_chunk = (uint32_t)(((k + splits - 1) / splits + 63) / 64 * 64);
    splits = (unsigned)((k + p.k_chunk - 1) / p.k_chunk);  // (rounding the parts up to whole slabs may leave fewer of them)
    if (bh * splits > 65535) return "gemm_nn kernel: extent too large";
  }
  if (splits > 1) {
    p.splits = splits;
    p.c = partial;
    p.out_bf16 = 0;
    tile = split_k_tile(m, n);
  }
  p.tiles_m = (uint32_t)((m + tile - 1) / tile);
  p.tiles_n = (uint32_t)((n + tile - 1) / tile);
  const size_t grid = (size_t(p.tiles_m) * p.tiles_n + 7) / 8 * 8;  // the tiles in 8 equal runs, one per XCD
  if (grid > kMaxGrid) return "gemm_nn kernel: grid too large";
  hipFunction_t fn;
  const bool w4 = tile == 256 && knobs.gemm_waves != 8;  // (as for the NT kernels: four waves unless 8 are asked for)
  const std::string name = std::string(tile == 256 ? "gemm_nn_bf16_256x256x64_direct" : "gemm_nn_bf16_128x128x64_direct") +
                           (k % 64 != 0 ? "_ktail" : "") + (w4 ? "_w4" : "");
  if (note) *note = LaunchNote{splits > 1 ? name + " (k in " + std::to_string(splits) + " parts)" : name, tile, tile};
  if (Err e = builtin_function(name.c_str(), &fn); !e.empty()) return e;
  if (Err e = launch(fn, (unsigned)grid, (unsigned)(bh * (splits > 1 ? splits : 1)), 1, tile == 256 && !w4 ? 512 : 256, &p, sizeof(p), stream);
      !e.empty() || splits <= 1)
    return e;
  SplitReduceParams r{partial, c, (uint32_t)bh, splits, (uint64_t)m * n, out_dtype == BF16 ? 1u : 0u};
  if (Err e = builtin_function("splitk_reduce", &fn); !e.empty()) return e;
  size_t rgrid = (bh * m * n / 4 + 255) / 256;
  if (rgrid > 65536) rgrid = 65536;
  return launch(fn, (unsigned)rgrid, 1, 1, 256, &r, sizeof(r), stream);
}

bool gemm_nt_f32_supported(size_t k) { return k > 0 && k % 4 == 0 && k <= (size_t(1) << 21); }

unsigned gemm_nt_f32_split_k(size_t bh, size_t m, size_t n, size_t k, const KernelOptions& knobs) {
  if (bh == 0 || m == 0 || n == 0 || !gemm_nt_f32_supported(k) || knobs.gemm_k_parts == 1) return 1;
  auto parts_of = [&](size_t want) -> unsigned {
    if (want < 2 || bh * want > 65535) return 1;
    const size_t chunk = (k / want + 63) / 64 * 64;  // what one split contracts: whole slabs
    return (unsigned)((k + chunk - 1) / chunk);
  };
  if (knobs.gemm_k_parts > 1) return parts_of(std::min<size_t>((size_t)knobs.gemm_k_parts, k / 64));
  // The model of gemm_nt_bf16_split_k with this kernel's figures: 1.7 us per 32-wide slab for a workgroup on a
  // 128 x 128 tile, 256 of them at a time (the 256 x 256 tile only takes grids that fill the chip), parts of at
  // least 64 of k.  Unsplit -> split, us: 128 x 128 x 8192 444 -> 36 (32 parts), 512 x 512 x 4096 227 -> 31 (16),
  // 1024 x 1024 x 1024 60 -> 27 (4), 8192 x 128 x 8192 (the probabilities times the values of a naive attention)
  // 451 -> 128 (4), 512 x 64 x 512 34 -> 15 (8); left whole: 2048^3 (120 us; 130 in two parts).
  const size_t t128 = ((m + 127) / 128) * ((n + 127) / 128) * bh, t256 = ((m + 255) / 256) * ((n + 255) / 256) * bh;
  if (t256 >= 128) return 1;  // (the large tile's grids fill the chip)
  const size_t slabs = (k + 31) / 32;
  auto time_of = [](size_t workgroups, size_t slabs_) { return (double)((workgroups + 255) / 256) * (double)(slabs_ + 2) * 1.7; };
  double best = 0.85 * time_of(t128, slabs);
  size_t splits = 1;
  for (size_t s = 2; s <= 32 && k / s >= 64 && bh * s <= 65535; s *= 2) {
    const double t = time_of(t128 * s, (slabs + s - 1) / s) + 4.0 + (double)(bh * s * m * n * 4) / 3e6;
    if (t < best) {
      best = t;
      splits = s;
    }
  }
  return parts_of(splits);
}

Err launch_gemm_nt_f32(const float* a, const float* b, float* c, size_t bh, size_t m, size_t n, size_t k,
                       hipStream_t stream, LaunchNote* note, float* partial, unsigned splits, const KernelOptions& knobs) {
  if (!gemm_nt_f32_supported(k)) return "gemm_nt f32 kernel: k must be a positive multiple of 4 (at most 2^21)";
  if (reinterpret_cast<uintptr_t>(a) % 16 != 0 || reinterpret_cast<uintptr_t>(b) % 16 != 0)
    return "gemm_nt f32 kernel: operands must be 16-byte aligned";
  if (bh == 0 || m == 0 || n == 0) return {};
  if (!fits_u32(m) || !fits_u32(n) || bh > 65535) return "gemm_nt f32 kernel: extent too large";
  if (!a || !b || !c) return "gemm_nt f32 kernel: null device pointer";
  GemmParams p{};
  p.a = a; p.b = b; p.c = c;
  p.bh = (uint32_t)bh; p.m = (uint32_t)m; p.n = (uint32_t)n; p.k = (uint32_t)k;
  // 256 x 256 tiles when they fill at least half of the CUs, 128 x 128 tiles otherwise
  const size_t t256 = ((m + 255) / 256) * ((n + 255) / 256) * bh;
  unsigned tile = t256 >= 128 ? 256 : 128;
  if (knobs.gemm_tile) tile = knobs.gemm_tile == 192 ? 256u : (unsigned)knobs.gemm_tile;  // (192 x 256 exists for bf16 NT products only)
  // the k loop in parts over workgroups (gemm_nt_f32_split_k says when): partial products in the caller's temporary
  if (splits > 1) {
    if (!partial) return "gemm_nt f32 kernel: a split needs its temporary";
    if ((m * n) % 4 != 0) return "gemm_nt f32 kernel: a split product needs m * n to be a multiple of 4";
    p.k_chunk = (uint32_t)(((k + splits - 1) / splits + 63) / 64 * 64);
    splits = (unsigned)((k + p.k_chunk - 1) / p.k_chunk);  // (rounding the parts up to whole slabs may leave fewer of them)
    if (bh * splits > 65535) return "gemm_nt f32 kernel: extent too large";
  }
  if (splits > 1) {
    p.splits = splits;
    p.c = partial;
  }
  p.tiles_m = (uint32_t)((m + tile - 1) / tile);
  p.tiles_n = (uint32_t)((n + tile - 1) / tile);
  const size_t grid = (size_t(p.tiles_m) * p.tiles_n + 7) / 8 * 8;  // the tiles in 8 equal runs, one per XCD
  if (grid > kMaxGrid) return "gemm_nt f32 kernel: grid too large";
  hipFunction_t fn;
  const std::string name = std::string(tile == 256 ? "gemm_nt_f32_256x256x32_direct" : "gemm_nt_f32_128x128x32_direct") +
                           (k % 32 != 0 ? "_ktail" : "");  // (a partial last slab of 32 k; of the last part, when split)
  if (note) *note = LaunchNote{splits > 1 ? name + " (k in " + std::to_string(splits) + " parts)" : name, tile, tile};
  if (Err e = builtin_function(name.c_str(), &fn); !e.empty()) return e;
  if (Err e = launch(fn, (unsigned)grid, (unsigned)(bh * (splits > 1 ? splits : 1)), 1, tile == 256 ? 512 : 256, &p, sizeof(p), stream);
      !e.empty() || splits <= 1)
    return e;
  SplitReduceParams r{partial, c, (uint32_t)bh, splits, (uint64_t)m * n, 0u};
  if (Err e = builtin_function("splitk_reduce", &fn); !e.empty()) return e;
  size_t rgrid = (bh * m * n / 4 + 255) / 256;
  if (rgrid > 65536) rgrid = 65536;
  return launch(fn, (unsigned)rgrid, 1, 1, 256, &r, sizeof(r), stream);
}

// Into how many parts to cut each row of a softmax (1: do not): fewer rows than half the CUs, each of 2^17 columns
// and more, which one workgroup per row would leave to a few CUs; parts of at least 2^15 columns, as many as give
// every CU a workgroup.
unsigned row_softmax_parts(size_t rows, size_t cols, int mode) {
  if ((mode != 0 && mode != 4) || rows == 0 || rows > 128 || cols < (size_t(1) << 17)) return 1;
  const size_t parts = std::min<size_t>(std::min<size_t>(256 / rows, cols >> 15), 64);
  return parts < 2 ? 1u : (unsigned)parts;
}

Err launch_row_softmax(const float* x, float* y, size_t rows, size_t cols, hipStream_t stream, int mode,
                       LaunchNote* note, const float* scale_ptr, float scale, float* stats, unsigned parts) {
  if (rows == 0 || cols == 0) return {};
  if (!fits_u32(rows) || !fits_u32(cols)) return "row_softmax kernel: extent exceeds 32 bits";
  if (!x || !y) return "row_softmax kernel: null device pointer";
  if (mode < 0 || mode > 4) return "row_softmax kernel: unknown mode";
  if (mode == 4 && !std::isfinite(scale)) return "row_softmax kernel: unsupported scale (must be finite)";
  static const char* const kOps[5] = {"softmax", "shift", "norm", "exp", "scaled_softmax"};
  SoftmaxParams p{x, y, (uint32_t)rows, (uint32_t)cols, scale_ptr, scale};
  hipFunction_t fn;
  const bool vec = cols % 4 == 0 && (reinterpret_cast<uintptr_t>(x) % 16 == 0) && (reinterpret_cast<uintptr_t>(y) % 16 == 0);
  if (parts > 1 && (mode == 0 || mode == 4)) {
    // every row in parts over workgroups: the parts' (max, sum) pairs into `stats`, then a second launch that
    // combines them and writes
    if (!stats) return "row_softmax kernel: rows in parts need their temporary";
    const size_t chunks = vec ? cols / 4 : cols;
    p.part_chunks = (uint32_t)((chunks + parts - 1) / parts);
    p.parts = (uint32_t)((chunks + p.part_chunks - 1) / p.part_chunks);
    p.stats = stats;
    if (rows * p.parts > kMaxGrid) return "row_softmax kernel: grid too large";
    const std::string base = std::string("row_") + kOps[mode] + "_parts_";
    if (note) *note = LaunchNote{base + "stats" + (vec ? "_v" : "") + " + " + base + "apply" + (vec ? "_v" : "") + " (rows in " + std::to_string(p.parts) + " parts)", 0, 0};
    if (Err e = builtin_function((base + "stats" + (vec ? "_v" : "")).c_str(), &fn); !e.empty()) return e;
    if (Err e = launch(fn, (unsigned)(rows * p.parts), 1, 1, 1024, &p, sizeof(p), stream); !e.empty()) return e;
    if (Err e = builtin_function((base + "apply" + (vec ? "_v" : "")).c_str(), &fn); !e.empty()) return e;
    return launch(fn, (unsigned)(rows * p.parts), 1, 1, 1024, &p, sizeof(p), stream);
  }
  if (cols <= 128) {
    // G lanes per row, one float4 chunk each: 64 / G rows per wavefront
    size_t g = 1;
    while (4 * g < cols) g *= 2;
    const std::string name = std::string("row_") + kOps[mode] + "_sub_" + (vec ? "v" : "s") + std::to_string(g);
    if (note) *note = LaunchNote{name, 0, 0};
    if (Err e = builtin_function(name.c_str(), &fn); !e.empty()) return e;
    const size_t grid = (rows * g + 255) / 256;
    if (grid > kMaxGrid) return "row_softmax kernel: grid too large";
    return launch(fn, (unsigned)grid, 1, 1, 256, &p, sizeof(p), stream);
  }
  if (cols <= 8192) {
    int nv = 1;
    while ((size_t)256 * nv < cols) nv *= 2;
    const std::string name = std::string("row_") + kOps[mode] + "_wave_" + (vec ? "v" : "s") + std::to_string(nv);
    if (note) *note = LaunchNote{name, 0, 0};
    if (Err e = builtin_function(name.c_str(), &fn); !e.empty()) return e;
    const size_t grid = (rows + 3) / 4;  // four wavefronts (rows) per workgroup
    if (grid > kMaxGrid) return "row_softmax kernel: grid too large";
    return launch(fn, (unsigned)grid, 1, 1, 256, &p, sizeof(p), stream);
  }
  if (rows > kMaxGrid) return "row_softmax kernel: grid too large";
  if (cols <= 32768 || (cols <= 65536 && vec)) {
    // the row still fits the registers of one workgroup of 16 wavefronts: one read and one write per element
    const int nv = cols <= 16384 ? 4 : cols <= 32768 ? 8 : 16;
    const std::string name = std::string("row_") + kOps[mode] + "_group_" + (vec ? "v" : "s") + std::to_string(nv);
    if (note) *note = LaunchNote{name, 0, 0};
    if (Err e = builtin_function(name.c_str(), &fn); !e.empty()) return e;
    return launch(fn, (unsigned)rows, 1, 1, 1024, &p, sizeof(p), stream);
  }
  // wider rows: two passes over the row (one for exp, elementwise)
  const std::string name = std::string("row_") + kOps[mode] + (vec ? "_block_v" : "_block");
  if (note) *note = LaunchNote{name, 0, 0};
  if (Err e = builtin_function(name.c_str(), &fn); !e.empty()) return e;
  return launch(fn, (unsigned)rows, 1, 1, 1024, &p, sizeof(p), stream);
}

Err launch_transpose(const void* src, void* dst, size_t bh, size_t rows, size_t cols, size_t elem_bytes,
                     hipStream_t stream) {
  if (elem_bytes != 2 && elem_bytes != 4) return "transpose kernel: element size must be 2 or 4 bytes";
  if (bh == 0 || rows == 0 || cols == 0) return {};
  if (!fits_u32(bh) || !fits_u32(rows) || !fits_u32(cols)) return "transpose kernel: extent exceeds 32 bits";
  if (!src || !dst) return "transpose kernel: null device pointer";
  TransposeParams p{};
  p.src = src; p.dst = dst;
  p.bh = (uint32_t)bh; p.rows = (uint32_t)rows; p.cols = (uint32_t)cols;
  p.tiles_r = (uint32_t)((rows + 63) / 64);
  p.tiles_c = (uint32_t)((cols + 63) / 64);
  const size_t grid = bh * p.tiles_r * p.tiles_c;
  if (grid > kMaxGrid) return "transpose kernel: grid too large";
  hipFunction_t fn;
  if (Err e = builtin_function(elem_bytes == 2 ? "transpose_b16" : "transpose_b32", &fn); !e.empty()) return e;
  return launch(fn, (unsigned)grid, 1, 1, 256, &p, sizeof(p), stream);
}

Err launch_convert(const void* src, void* dst, DType from, DType to, size_t n, hipStream_t stream) {
  if (n == 0) return {};
  if (from == to) return "convert kernel: identical dtypes";
  ConvertParams p{src, dst, (uint64_t)n};
  hipFunction_t fn;
  if (Err e = builtin_function(from == F32 ? "convert_f32_to_bf16" : "convert_bf16_to_f32", &fn); !e.empty()) return e;
  size_t grid = (n + 255) / 256;
  if (grid > 65536) grid = 65536;
  return launch(fn, (unsigned)grid, 1, 1, 256, &p, sizeof(p), stream);
}

Err launch_pad_rows(const void* src, void* dst, size_t rows, size_t cols, size_t cols_padded, size_t elem_bytes,
                    hipStream_t stream) {
  if (elem_bytes != 2 && elem_bytes != 4) return "pad kernel: element size must be 2 or 4 bytes";
  if (rows == 0 || cols_padded == 0) return {};
  if (!fits_u32(cols_padded) || cols > cols_padded) return "pad kernel: bad extents";
  if (!src || !dst) return "pad kernel: null device pointer";
  PadParams p{src, dst, (uint64_t)rows, (uint32_t)cols, (uint32_t)cols_padded};
  hipFunction_t fn;
  if (Err e = builtin_function(elem_bytes == 2 ? "pad_rows_b16" : "pad_rows_b32", &fn); !e.empty()) return e;
  size_t grid = (rows * cols_padded + 255) / 256;
  if (grid > 65536) grid = 65536;
  return launch(fn, (unsigned)grid, 1, 1, 256, &p, sizeof(p), stream);
}

}  // namespace ihip
