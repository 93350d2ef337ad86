/*
 * 𝚒 runtime C ABI, as served by the gfx950 backend's libi_core.so.
 *
 * Symbol names, argument order, struct layouts, ownership and error rules are
 * those of the reference runtime (core/i.h:8-70, implemented in
 * core/src/lib.rs:61-333), so an existing 𝚒 frontend (for example the ctypes
 * binding ilang-python/ilang.py:66-106) drives this library unchanged.  What
 * differs is behind i_compile / i_exec*: components are lowered to gfx950
 * kernels and run on the GPU instead of being rendered to C and built with cc.
 *
 * Conventions (all from the reference):
 *   - handles are opaque, immutable after creation, freed by the caller;
 *   - constructors return NULL, int functions return -1, i_output_count
 *     returns 0 and i_exec returns {NULL, 0} on failure, with the reason
 *     readable through i_error() on the same thread;
 *   - tensors are dense row-major f32 in HOST memory.
 * Device-resident operands and bf16 use the extra entry points in i_hip.h.
 */
#pragma once

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct i_component i_component; /* a combinator tree of 𝚒 expressions */
typedef struct i_program i_program;     /* a compiled, loaded component       */

/* Borrowed read-only input (core/i.h:8-12). */
typedef struct {
  const float* data;
  const size_t* shape;
  size_t rank;
} i_tensor;

/* Borrowed caller-allocated output (core/i.h:14-18). */
typedef struct {
  float* data;
  const size_t* shape;
  size_t rank;
} i_tensor_mut;

/* Library-allocated output of i_exec; len = product of shape (core/i.h:20-25). */
typedef struct {
  float* data;
  size_t* shape;
  size_t rank;
  size_t len;
} i_owned_tensor;

/* Returned by value from i_exec, released with i_outputs_free (core/i.h:27-30). */
typedef struct {
  i_owned_tensor* tensors;
  size_t count;
} i_outputs;

/* Parse one expression "semantic | splits | order" into a leaf component.
 * Parsing only; language rules are checked at compile time (core/src/lib.rs:62-71). */
i_component* i_parse(const char* src);
/* The identity component `I` (core/src/lib.rs:74-78). */
i_component* i_identity(void);
/* Combinators; both operands are cloned and stay owned by the caller
 * (core/src/lib.rs:81-121, 336-351):
 *   chain   (f >> g)(x) = g(f(x))        compose (f << g)(x) = f(g(x))
 *   fanout  (f & g)(x) = (f(x), g(x))    pair    (f | g)(x, y) = (f(x), g(y))
 *   swap    (~f)(x, y) = f(y, x)                                              */
i_component* i_chain(const i_component* left, const i_component* right);
i_component* i_compose(const i_component* left, const i_component* right);
i_component* i_fanout(const i_component* left, const i_component* right);
i_component* i_pair(const i_component* left, const i_component* right);
i_component* i_swap(const i_component* component);

/* Backend source for the component as a heap string (free with i_string_free):
 * the kernel plan and the generated HIP for kernels that are not hand-written
 * (the reference returns its generated C here, core/src/lib.rs:124-139). */
char* i_code(const i_component* component);
/* Validate, lower, select / generate gfx950 kernels and load them
 * (reference: lower -> render C -> cc -> dlopen, core/src/lib.rs:142-151, 353-375). */
i_program* i_compile(const i_component* component);

size_t i_output_count(const i_program* program);                 /* core/src/lib.rs:154-160 */
int i_output_ranks(const i_program* program, size_t* ranks);     /* core/src/lib.rs:163-174 */
/* Caller allocates shapes[o][rank_o]; input_count is only null-checked
 * against `inputs`, as in the reference (core/src/lib.rs:177-197). */
int i_output_shapes(
  const i_program* program,
  const i_tensor* inputs,
  size_t input_count,
  size_t** shapes
);

/* Run with caller-owned host buffers; output_count must equal
 * i_output_count(program) (core/src/lib.rs:200-225).  Inputs are uploaded,
 * the kernels run, outputs are copied back before the call returns. */
int i_exec_into(
  const i_program* program,
  const i_tensor* inputs,
  size_t input_count,
  i_tensor_mut* outputs,
  size_t output_count
);

/* Run with library-allocated, zero-initialised outputs (core/src/lib.rs:228-286). */
i_outputs i_exec(
  const i_program* program,
  const i_tensor* inputs,
  size_t input_count
);

/* Thread-local last error, NULL if none yet; valid until the next failure on
 * this thread; not cleared by successful calls (core/src/lib.rs:327-333). */
const char* i_error(void);
/* All four accept NULL (core/src/lib.rs:289-324). */
void i_component_free(i_component* component);
void i_program_free(i_program* program);
void i_outputs_free(i_outputs outputs);
void i_string_free(char* s);

#ifdef __cplusplus
}
#endif
