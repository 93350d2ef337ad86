// Host-side launchers for the hand-written gfx950 kernels.  They validate the
// operand shapes against what each kernel and its grid assume, pick the
// kernel variant, and enqueue it on `stream`.  All pointers are device memory.
#pragma once
#include <cstddef>
#include <string>

#include "hip_rt.h"

namespace ihip {

enum DType { F32 = 0, BF16 = 1 };

// What a launcher did with a request: the kernel it enqueued and, for tiled kernels, the workgroup tile that kernel
// works on, so that callers can report a schedule tile that no kernel has.
struct LaunchNote {
  std::string kernel;         // name in the code object
  size_t tile_i = 0, tile_j = 0;  // rows x columns (attention: query rows x keys) per workgroup step
};

// Choices that a caller may take from the launchers.  They belong to a compiled program (i_hip_program_option) or to
// one launch (the i_hip_*_opt entry points), never to the process: two programs, or two threads, with different
// wishes do not meet.  The defaults leave every choice to the launcher.
struct KernelOptions {
  int attention_f32_scale = 0;  // 1: apply the score scale in f32 to every score instead of folding it into Q
  int attention_kv_parts = 0;   // keys of a head in parts over workgroups: 0 the launcher decides, 1 never, n that many
  int attention_waves = 0;      // waves per workgroup of the direct kernels: 0 decides; 2, 4, 8; 64 = the 64-queries-per-wave kernel (d = 64)
  int attention_direct = 1;     // 0: the register-staged kernels instead of the direct-to-LDS ones
  int gemm_k_parts = 0;         // k loop of a product in parts over workgroups: 0 the launcher decides, 1 never, n that many
  int gemm_waves = 0;           // waves of the 256 x 256 tile: 0 decides (four), 4, 8
  int gemm_tile = 0;            // workgroup tile of the direct kernels, rows of A: 0 decides, 128, 192 (x 256), 256
  int gemm_tile_n = 0;          // ... rows of B: 0 what goes with gemm_tile, 192 with gemm_tile 256 for 256 x 192
  int gemm_direct = 1;          // 0: the register-staged bf16 kernel instead of the direct-to-LDS ones
  int generated_only = 0;       // 1: every kernel of a program in its generated form
  int generated_wave = -1;      // wavefront-per-iteration form of generated reduction nests: -1 decides, 0 never, 1 wherever a nest has one
  int generated_parts = 0;      // outermost sequential loop of a generated reduction nest in parts over workgroups: 0 decides, 1 never, n that many
  // two 64-bit counters in device memory to which the bf16 direct-to-LDS attention kernels add the time their
  // workgroups were resident, on the shader clock and on the constant 100 MHz clock (AttnParams::clock)
  unsigned long long* clock_ticks = nullptr;
};
// One option by its name ("attention.kv_parts", "gemm.tile", ...); "" or the failure text (unknown name, bad value).
Err set_kernel_option(KernelOptions& options, const std::string& name, int value);
// "name=value name=value" (blanks, commas or semicolons between the pairs); nullptr and "" are no options.
Err parse_kernel_options(const char* text, KernelOptions* options);

// One wavefront that reads the shader clock and the constant 100 MHz clock, sleeps for `microseconds` (at most two
// seconds) and reads them again; the differences are added to ticks[0] and ticks[1] (device memory).  Enqueued on a
// second stream beside other work it tells the shader clock under that work.
Err launch_shader_clock_probe(unsigned long long* ticks, unsigned microseconds, hipStream_t stream);

// o[bh,nq,dv] = softmax(s * q[bh,nq,d] k[bh,nk,d]^T) v[bh,nk,dv],  s = scale * (scale_ptr ? *scale_ptr : 1)
// in_dtype applies to q, k, v; out_dtype to o (F32 or BF16; BF16 only with bf16 inputs).
// scale_ptr, when given, is a rank-0 f32 operand in device memory, read by the kernel.
// query_tile x key_tile is the tile the schedule asks for (the products of the split factors of the row and of
// the key index; 0 = no preference).  The direct-to-LDS kernels (bf16, d == dv in {64, 128}) exist for
// query tiles 64 / 128 / 256 (2, 4, 8 waves) with key tiles 32 / 64 (no 256 x 32 at d = 64), and for 512 x 32 at
// d = 64 (64 queries per wave); any other request leaves the choice to the launcher's size heuristic.
// knobs.attention_f32_scale: apply the score scale in f32 to every score, as the reference does, instead of folding
// it into Q with one more bf16 rounding (direct kernels only; the other kernels always multiply in f32);
// knobs.attention_waves and knobs.attention_direct reach every kernel with small operands (tests, searches).
// kv_splits > 1: the keys of each head in that many parts over workgroups (the direct kernels, bf16 and f32; ask
// attention_kv_splits, which also says when it pays: grids that leave most CUs without a workgroup).  The caller
// provides partial_o, room for bh * kv_splits * nq * dv floats, and partial_lse, for bh * kv_splits * nq.
struct AttentionOptions {
  size_t query_tile = 0, key_tile = 0;
  KernelOptions knobs;
  unsigned kv_splits = 0;
  float* partial_o = nullptr;
  float* partial_lse = nullptr;
};
unsigned attention_kv_splits(DType in_dtype, size_t bh, size_t nq, size_t nk, size_t d, size_t dv, const AttentionOptions& options = {});
Err launch_attention(const void* q, const void* k, const void* v, void* o, DType in_dtype, DType out_dtype, size_t bh,
                     size_t nq, size_t nk, size_t d, size_t dv, const float* scale_ptr, float scale, hipStream_t stream,
                     const AttentionOptions& options = {}, LaunchNote* note = nullptr);
bool attention_supported(DType in_dtype, size_t d, size_t dv, const KernelOptions& knobs = {});

// c[bh,m,n] = a[bh,m,k] b[bh,n,k]^T, a and b bf16, sums in f32; c is f32, or bf16 (out_dtype) with the sums rounded on the way out
// tile_m x tile_n is the output tile the schedule asks for (0 = no preference): 256 x 256 and 128 x 128 select
// the kernel with that workgroup tile (when its requirements hold), anything else leaves the choice to the launcher.
Err launch_gemm_nt_bf16(const void* a, const void* b, void* c, size_t bh, size_t m, size_t n, size_t k,
                        hipStream_t stream, size_t tile_m = 0, size_t tile_n = 0, LaunchNote* note = nullptr,
                        DType out_dtype = F32, const KernelOptions& knobs = {});
bool gemm_nt_bf16_supported(size_t k);

// The same product with its k loop split over workgroups, for products that have few output tiles and a long k loop
// (one small extent against two large ones), which would leave most of the chip idle.  gemm_nt_bf16_split_k says
// into how many parts (1: do not split); the caller provides `partial`, room for bh * splits * m * n floats, which
// the GEMM kernels fill with the partial products of each split and splitk_reduce adds up into c.
unsigned gemm_nt_bf16_split_k(size_t bh, size_t m, size_t n, size_t k, const KernelOptions& knobs = {});
Err launch_gemm_nt_bf16_split_k(const void* a, const void* b, void* c, float* partial, unsigned splits, size_t bh, size_t m,
                                size_t n, size_t k, hipStream_t stream, LaunchNote* note = nullptr, DType out_dtype = F32);

// c[bh,m,n] (f32) = a[bh,m,k] b[bh,k,n], a and b bf16, on the direct kernels with a row-major right operand.
// Needs k % 8 == 0 and n % 8 == 0 (gemm_nn_bf16_supported); callers transpose b and use the NT kernels otherwise.
// (splits > 1: the k loop in that many parts, as launch_gemm_nt_bf16_split_k does it, gemm_nt_bf16_split_k deciding;
// `partial` is room for bh * splits * m * n floats)
Err launch_gemm_nn_bf16(const void* a, const void* b, void* c, size_t bh, size_t m, size_t n, size_t k,
                        hipStream_t stream, size_t tile_m = 0, size_t tile_n = 0, LaunchNote* note = nullptr,
                        DType out_dtype = F32, float* partial = nullptr, unsigned splits = 1, const KernelOptions& knobs = {});
bool gemm_nn_bf16_supported(size_t bh, size_t m, size_t n, size_t k, const KernelOptions& knobs = {});

// c[bh,m,n] = a[bh,m,k] b[bh,n,k]^T, all f32, products and sums in f32 (f32 MFMA); needs k % 4 == 0 and 16-byte aligned operands
Err launch_gemm_nt_f32(const float* a, const float* b, float* c, size_t bh, size_t m, size_t n, size_t k,
                       hipStream_t stream, LaunchNote* note = nullptr, float* partial = nullptr, unsigned splits = 1,
                       const KernelOptions& knobs = {});
// (splits > 1: the k loop in that many parts over workgroups, as launch_gemm_nt_bf16_split_k does it; `partial` is
// room for bh * splits * m * n floats, and gemm_nt_f32_split_k says into how many parts, 1: do not split)
unsigned gemm_nt_f32_split_k(size_t bh, size_t m, size_t n, size_t k, const KernelOptions& knobs = {});
bool gemm_nt_f32_supported(size_t k);

// y[rows,cols] = row softmax of x, f32
// mode 0: softmax; 1: y = x - rowmax(x) (row_max_shift); 2: y = x / rowsum(x) (row_normalize); 3: y = exp(x);
// 4: softmax of s * x with s = scale * (scale_ptr ? *scale_ptr : 1), scale_ptr a rank-0 f32 operand in device memory.
// y may be x: every kernel has read a row's element before it writes it.
Err launch_row_softmax(const float* x, float* y, size_t rows, size_t cols, hipStream_t stream, int mode = 0,
                       LaunchNote* note = nullptr, const float* scale_ptr = nullptr, float scale = 1.0f,
                       float* stats = nullptr, unsigned parts = 1);
// (parts > 1, softmax modes only: every row in that many parts over workgroups, two launches; `stats` is room for
// 2 * rows * parts floats; row_softmax_parts says when it pays: fewer rows than half the CUs, 2^17 columns and more)
unsigned row_softmax_parts(size_t rows, size_t cols, int mode);

// dst[b][c][r] = src[b][r][c]; elem_bytes is 2 or 4.  An NN product that the direct kernels cannot read runs as transpose + NT kernel.
Err launch_transpose(const void* src, void* dst, size_t bh, size_t rows, size_t cols, size_t elem_bytes,
                     hipStream_t stream);

Err launch_convert(const void* src, void* dst, DType from, DType to, size_t n, hipStream_t stream);

// dst[r][c] = c < cols ? src[r][c] : 0 for c < cols_padded; elem_bytes is 2 or 4
Err launch_pad_rows(const void* src, void* dst, size_t rows, size_t cols, size_t cols_padded, size_t elem_bytes,
                    hipStream_t stream);

}  // namespace ihip
