/*
 * Device-side additions of the gfx950 backend to the 𝚒 runtime ABI (i.h).
 *
 * The reference runtime only knows host f32 buffers (core/i.h:8-30) and its
 * generated libraries export their kernels as plain functions
 * `void fK(const View* readonlys, ViewMut* writeables)`
 * (compiler/src/backends/c/stmt.rs:36-41).  The entry points below are the
 * GPU counterparts of those two things and do not change any i.h signature:
 *
 *   i_exec_into_device  run a compiled program on device-resident operands,
 *            f32 or bf16, asynchronously on a stream.
 *   i_hip_*  kernel launchers: the hand-written kernels a compiled program
 *            dispatches to, callable directly on device memory (the `fK`
 *            level of the generated-library ABI, ABI.md:4-9).
 *
 * All pointers are device pointers unless stated; `stream` is a hipStream_t
 * (NULL = the default stream).  Launches are asynchronous on that stream.
 * Return value 0 = enqueued, -1 = failure with the text in i_error().
 */
#pragma once

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#include "i.h"

enum { I_DTYPE_F32 = 0, I_DTYPE_BF16 = 1 };

/* A dense row-major tensor in DEVICE memory: the device-side twin of
 * i_tensor / i_tensor_mut (core/i.h:8-18) plus an element type tag. */
typedef struct {
  void* data;
  const size_t* shape;
  size_t rank;
  int dtype; /* I_DTYPE_* */
} i_device_tensor;

/*
 * i_exec_into for operands that already live on the GPU (reference host form:
 * core/src/lib.rs:200-225).  Enqueues the whole program on `stream` and returns
 * without waiting; temporaries are stream-ordered (a block per stream that the
 * library keeps from call to call, at most ILANG_HIP_ARENA_MB, default 256, and
 * stream-ordered allocations beyond it).  Rank-0 operands
 * (scalars) must be f32.  bf16 operands select the bf16-in / f32-accumulate
 * kernels where a kernel has one and are widened on the device otherwise;
 * each output is written in its own dtype.  Output shapes, when given
 * (rank > 0), are checked against i_output_shapes.
 *
 * Precision of bf16 attention: by default the fused kernels fold scale * log2(e) into Q, rounded to bf16 once
 * more, which saves one multiply per score (about 5 % of the time) and perturbs every score by about
 * 2^-9.5 * |q . k| * scale nats.  At the magnitudes attention has (inputs of unit variance, scores within +-30
 * nats) the result stays within 1e-2 of an f32 computation, relative to max |result|; at scores beyond about
 * +-30 nats (inputs x 3) it leaves the 2e-2 bar of the reference comparison (up to 2.4e-2 measured).  Callers
 * with such scores set i_hip_program_option(program, "attention.f32_scale", 1): the scale is then applied in f32
 * to every score, the reference's own arithmetic (compiler/src/lower/exec_plan_to_module.rs:605-640), and the
 * error stays below 1e-2 at any score magnitude.  f32 operands never fold anything.
 */
int i_exec_into_device(const i_program* program,
                       const i_device_tensor* inputs, size_t input_count,
                       const i_device_tensor* outputs, size_t output_count,
                       void* stream);

/*
 * i_exec_into_device for callers that cannot allocate device memory: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference (whose generated
 * `exec` mallocs its scratch on every call, ilang-python/annotated-flashattn.c:318-386).  Same arguments,
 * same kernels and same results as i_exec_into_device, but the program's temporaries (intermediates of
 * multi-kernel plans, f32 staging of bf16 operands, transposed operands, per-work-item slices of generated
 * kernels) are carved out of one fixed array of I_HIP_STATIC_WORKSPACE_BYTES that the library holds in the
 * memory of every GPU it runs on until the process ends; the call allocates and frees no device memory.
 * Operands whose temporaries add up to more are refused (-1, i_error says how much was needed) before
 * anything is enqueued.  Nothing in the array has to start at zero, and nothing is kept from call to call.
 * All calls on one GPU share that GPU's array: calls that overlap in time on one GPU, from different
 * streams or threads, race; serialise them (one stream, or events).  The first call of a program on a
 * device loads its code objects; make that call before capturing a graph.
 */
#define I_HIP_STATIC_WORKSPACE_BYTES ((size_t)64 << 20)
int i_exec_into_device_noalloc(const i_program* program,
                               const i_device_tensor* inputs, size_t input_count,
                               const i_device_tensor* outputs, size_t output_count,
                               void* stream);

/*
 * FlashAttention forward,  o = softmax(scale * q k^T) v  per (batch*head):
 * the fused kernel for  mm_t >> [scale] >> row_max_shift >> exp >> row_normalize >> mm
 * (reference emission of the same component: ilang-python/annotated-flashattn.c:52-310,
 * `f0`).  q [bh,nq,d], k [bh,nk,d], v [bh,nk,dv], o [bh,nq,dv], row-major.
 * in_dtype applies to q/k/v, out_dtype to o.  Requires a finite scale and 0 < d,dv <= 128
 * (f32), 0 < d,dv <= 256 and multiples of 8 (bf16).  bf16 runs the direct-to-LDS kernels
 * at every such head size (d = dv = 64, 128, 256 exactly, the others with zero-padded LDS
 * rows); f32 with d and dv multiples of 4, the larger from 36 to 128, and 16-byte aligned
 * operands runs the f32 kernel of the same design.  One kernel launch, no temporaries: the key loop
 * of a head is split over workgroups (few heads, long loops) only by programs run through i_exec*.
 */
int i_hip_attention(const void* q, const void* k, const void* v, void* o,
                    int in_dtype, int out_dtype,
                    size_t bh, size_t nq, size_t nk, size_t d, size_t dv,
                    float scale, void* stream);

/*
 * i_hip_attention with the schedule spelled out: query_tile x key_tile is the workgroup tile the schedule's split
 * factors ask for (README.md:139-163; 0 = no preference).  bf16 operands with d == dv in {64, 128} have kernels
 * for query tiles 64 / 128 / 256 with key tiles 32 / 64 (not 256 x 32 at d = 64) and for 512 x 32 at d = 64;
 * any other request leaves the choice to the launcher.  f32_scale != 0 applies the score scale in f32 to every
 * score, the reference's arithmetic (compiler/src/lower/exec_plan_to_module.rs:605-640), instead of folding
 * scale * log2(e) into Q with one more bf16 rounding: about 5 % slower, and the error against an f32 computation
 * no longer grows with the magnitude of the scores.  f32 operands and the other bf16 kernels always multiply in f32.
 */
int i_hip_attention_ex(const void* q, const void* k, const void* v, void* o,
                       int in_dtype, int out_dtype,
                       size_t bh, size_t nq, size_t nk, size_t d, size_t dv,
                       float scale, size_t query_tile, size_t key_tile, int f32_scale, void* stream);

/*
 * i_hip_attention_ex with the launcher's remaining choices by name: `options` is "name=value name=value" with the
 * attention.* names of i_hip_program_option ("attention.waves=8 attention.direct=1"; NULL or "": none), for tests
 * and searches that want a particular kernel on small operands.
 */
int i_hip_attention_opt(const void* q, const void* k, const void* v, void* o,
                        int in_dtype, int out_dtype,
                        size_t bh, size_t nq, size_t nk, size_t d, size_t dv,
                        float scale, size_t query_tile, size_t key_tile, const char* options, void* stream);

/*
 * Options of a compiled program, by name (i_compile has no options argument, core/i.h:44).  The schedule's splits
 * pick the workgroup tile (README.md:139-163); these are the choices a schedule has no spelling for.  They belong
 * to the program, not to the process: two programs (or threads) with different wishes do not meet.  Known:
 *   "attention.f32_scale"  0 (default) / 1: what f32_scale is to i_hip_attention_ex, for the program's attention kernels
 *   "attention.kv_parts"   keys of a head in parts over workgroups: 0 (default) the launcher decides by grid size,
 *                          1 never, n that many (whole 64-key tiles each, so fewer may result)
 *   "attention.waves"      waves per workgroup of the direct bf16 kernels: 0 (default) by schedule tile and size,
 *                          2 / 4 / 8, 64 = the 64-queries-per-wave kernel (d = 64)
 *   "attention.direct"     1 (default) / 0: the register-staged kernels instead of the direct-to-LDS ones
 *   "gemm.k_parts"         k loop of a product in parts over workgroups: 0 (default) by a model of the time, 1 never, n
 *   "gemm.tile"            workgroup tile of the direct product kernels: 0 (default) by schedule tile and size, 128, 256,
 *                          192 (192 x 256: bf16 products with a K-contiguous right operand; the others take 256)
 *   "gemm.tile_n"          columns of that tile when gemm.tile is given: 0 (default) what goes with it, 192 with
 *                          gemm.tile = 256 for the 256 x 192 tile (same products as 192 x 256)
 *   "gemm.waves"           waves of the 256 x 256 tile: 0 (default: four), 4, 8
 *   "gemm.direct"          1 (default) / 0: the register-staged bf16 product kernel
 *   "generated.only"       0 (default) / 1: every kernel in its generated form (no hand-written kernel)
 *   "generated.wave"       wavefront-per-iteration form of generated reduction nests: -1 (default) by extents, 0 never, 1 always
 *   "generated.parts"      outermost sequential loop of a generated reduction nest in parts over workgroups (a sum to one
 *                          element, a column sum of few columns): 0 (default) by extents, 1 never, n that many (at most 4096)
 * Returns 0, or -1 with the text in i_error() for an unknown name or a value the option does not take.  Takes
 * effect from the next i_exec*.
 */
int i_hip_program_option(i_program* program, const char* name, int value);

/*
 * Shader-clock accounting for a program's attention kernels (no counterpart in the reference).  `ticks` is device
 * memory for two 64-bit counters, 8-byte aligned, that the caller clears; from the next i_exec* on every workgroup
 * of the program's bf16 direct-to-LDS attention kernels adds to ticks[0] the shader-clock cycles (s_memtime: the
 * clock the power manager grants at the moment) and to ticks[1] the ticks of the constant 100 MHz clock that passed
 * between its first and its last instruction.  ticks[0] / ticks[1] / 10 is the shader clock in GHz under the
 * kernel, averaged over the time its workgroups were resident: what a measured fraction of the matrix-core peak,
 * quoted at 2.4 GHz, has to be read against.  NULL switches it off.  Costs four atomic adds per workgroup.
 */
int i_hip_program_clock_probe(i_program* program, void* ticks);

/*
 * The same two clocks read by a one-wavefront kernel of its own, for work that cannot count for itself (a vendor
 * library's kernel): reads both clocks, sleeps for `microseconds` (at most 2 000 000), reads them again and adds the
 * differences to ticks[0] (shader clock) and ticks[1] (100 MHz clock).  Enqueue it on a second stream beside the
 * work in question.  It occupies one wave slot of one compute unit while it sleeps.
 */
int i_hip_shader_clock_probe(void* ticks, unsigned microseconds, void* stream);

/*
 * Memory that the library keeps from call to call, so that a call allocates nothing after the first of its kind: per
 * (device, stream), for the 16 pairs used most recently, a block for temporaries (at most ILANG_HIP_ARENA_MB, default
 * 256 MiB each); per device a block for the device copies of host operands (at most ILANG_HIP_STAGING_MB, default
 * 1 GiB) with an 8 MiB page-locked mirror, two rings of four page-locked chunks of 8 MiB for large host operands
 * (one ring per direction), up to 1 GiB of freed temporaries in the library's own memory pool, and the fixed workspace of i_exec_into_device_noalloc
 * (I_HIP_STATIC_WORKSPACE_BYTES, part of the loaded library).  This call frees all of it except the last, as far as
 * no call is using it at the moment, and returns the bytes released; the next calls allocate again.  No counterpart
 * in the reference, whose generated exec mallocs and frees on every call.
 */
size_t i_hip_release_cached_memory(void);

/*
 * What the last i_exec* of this program dispatched, one line per kernel of the plan that i_code prints:
 * "f0: attn_fwd_bf16_d128_bn64_direct_w8 (tile 256 x 64)"; a schedule tile that no hand-written kernel has for
 * the operands is spelled out on that line.  Heap string, free with i_string_free; NULL + i_error on failure.
 */
char* i_hip_program_report(const i_program* program);

/*
 * Whether the program only ever maps over the first index of its outputs: that index is the first dimension of some
 * of the inputs and no other dimension of any, no expression reduces over it, and none uses it under two names.
 * Rows r0 .. r1 of every output are then what the program computes from rows r0 .. r1 of those inputs and all of
 * the others, so the program may be run slice by slice.  Returns the number of the program's inputs (at least 1)
 * and sets sliced[i] to 1 for the inputs that are cut with the outputs and to 0 for those every slice needs whole
 * (sliced may be NULL; else `capacity` entries, at least as many as the program has inputs), 0 if the program has
 * to run whole, -1 + i_error on a bad argument.  i_exec and i_exec_into use it themselves: calls
 * that move 64 MiB and more in such rows go up, run and come down in up to 8 slices, the kernels of one slice under
 * the transfer of the next (i_hip_program_report then says so).  A slice is computed by the kernels the launchers
 * pick for its shape, which may add up sums in another order than the whole would (within the parity bars).  No
 * counterpart in the reference, which runs on the host.
 */
int i_hip_program_row_slices(const i_program* program, unsigned char* sliced, size_t capacity);

/*
 * mm_t,  c[bh,m,n] = sum_k a[bh,m,k] * b[bh,n,k]  with bf16 a, b and f32 c:
 * the fused kernel for  i("ik*jk~ijk") >> i("+ijk~ij ... k0")  (README.md:16;
 * same nest as annotated-flashattn.c:57-89).  Requires k % 8 == 0.
 */
int i_hip_gemm_nt_bf16(const void* a, const void* b, float* c,
                       size_t bh, size_t m, size_t n, size_t k, void* stream);

/*
 * i_hip_gemm_nt_bf16 with the output element type and the schedule's tile spelled out: c is f32 (I_DTYPE_F32) or
 * bf16 (I_DTYPE_BF16: the f32 sums are rounded to nearest-even on the way out, half the bytes written);
 * tile_m x tile_n of 128 x 128 or 256 x 256 selects the kernel with that workgroup tile, 0 leaves the choice to
 * the launcher.
 */
int i_hip_gemm_nt_bf16_ex(const void* a, const void* b, void* c, int out_dtype,
                          size_t bh, size_t m, size_t n, size_t k, size_t tile_m, size_t tile_n, void* stream);

/*
 * The product with a row-major right operand,  c[bh,m,n] = sum_k a[bh,m,k] * b[bh,k,n]  (bf16 a, b, f32 c):
 * the fused kernel for  i("ik*kj~ijk") >> i("+ijk~ij ...")  (ilang-python/test.py:52-56) and for the demo's
 * standalone mm,  i("ij*jk~ikj") >> i("+ikj~ik ...")  (ilang-python/flash-attn.py:51).  Requires k % 8 == 0
 * and n % 8 == 0; other shapes go through a transpose and i_hip_gemm_nt_bf16.
 */
int i_hip_gemm_nn_bf16(const void* a, const void* b, float* c,
                       size_t bh, size_t m, size_t n, size_t k, void* stream);

/*
 * The same mm_t with f32 a, b, c and f32 products and sums (f32 MFMA), the reference's own
 * arithmetic type: what the host f32 ABI of i.h dispatches to.  Requires k % 4 == 0 and 16-byte aligned a, b.
 */
int i_hip_gemm_nt_f32(const float* a, const float* b, float* c,
                      size_t bh, size_t m, size_t n, size_t k, void* stream);

/*
 * Any of the three products above with the launcher's choices by name: in_dtype I_DTYPE_BF16 (b_row_major 0: a b^T,
 * 1: a b; c f32 or bf16) or I_DTYPE_F32 (a b^T, f32 c); `options` is "name=value name=value" with the gemm.* names of
 * i_hip_program_option ("gemm.tile=128 gemm.waves=8"; NULL or "": none).  No temporaries, so gemm.k_parts does not apply.
 */
int i_hip_gemm_opt(const void* a, const void* b, void* c, int in_dtype, int out_dtype, int b_row_major,
                   size_t bh, size_t m, size_t n, size_t k, const char* options, void* stream);

/*
 * Row softmax over the last axis of an f32 [rows, cols] matrix: the fused
 * kernel for  row_max_shift >> exp >> row_normalize  (README.md:19-25).
 * Any cols: up to 65536 columns a row is read once and written once (it lives
 * in the registers of a group of lanes, a wavefront or a workgroup), wider
 * rows are read twice.  16-byte aligned operands with cols % 4 == 0 take the
 * float4 forms.  One launch with a workgroup (or less) per row, no temporaries:
 * a few very long rows are cut into parts over workgroups only by programs run
 * through i_exec*.
 */
int i_hip_row_softmax(const float* x, float* y, size_t rows, size_t cols, void* stream);

/* Element-wise dtype conversion between f32 and bf16 device buffers (n elements). */
int i_hip_convert(const void* src, void* dst, int from_dtype, int to_dtype, size_t n, void* stream);

#ifdef __cplusplus
}
#endif
