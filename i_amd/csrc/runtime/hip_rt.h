// Thin host-side layer over the HIP driver-style API.  This is the only place
// the library touches the GPU: a gfx950 code object built by hipcc is loaded
// with hipModuleLoadData, kernels are looked up by name and launched with
// hipModuleLaunchKernel, memory moves through hipMalloc / hipMemcpy.
// It takes the place of the reference's cc + dlopen/dlsym loader
// (core/src/loader.rs:8-42, core/src/lib.rs:353-415).
#pragma once
#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <string>

namespace ihip {

// Every call returns an empty string on success, else the failure text.
using Err = std::string;

// Loads (once per device) the prebuilt kernel code object that sits beside the
// shared library, or the file named by ILANG_HIP_KERNELS.
Err builtin_function(const char* name, hipFunction_t* fn);

// Loads a code object from memory (generic kernels produced at compile time).
Err load_module(const void* image, hipModule_t* mod);
Err module_function(hipModule_t mod, const char* name, hipFunction_t* fn);
void unload_module(hipModule_t mod);

// Launches `fn` with a single by-value parameter block.
Err launch(hipFunction_t fn, unsigned grid_x, unsigned grid_y, unsigned grid_z, unsigned block_x,
           const void* params, size_t params_size, hipStream_t stream);

// While one of these lives on a thread, launch() on that thread checks nothing in and enqueues nothing: the
// executor walks a program once this way to add up the temporaries it would need.
struct DryRun {
  DryRun();
  ~DryRun();
  DryRun(const DryRun&) = delete;
  DryRun& operator=(const DryRun&) = delete;
};

Err dev_alloc(void** p, size_t bytes);
// a temporary that hipFreeAsync(p, stream) gives back, from the library's own pool of the current device
Err temp_alloc(void** p, size_t bytes, hipStream_t stream);
void dev_free(void* p);
// Hands the freed memory that the library's pools of temporaries hold back to the system; returns the bytes (0 when
// the runtime cannot tell).
size_t trim_temp_pool();
Err h2d(void* dst, const void* src, size_t bytes, hipStream_t stream);
Err d2h(void* dst, const void* src, size_t bytes, hipStream_t stream);
Err sync(hipStream_t stream);
Err check(hipError_t e, const char* what);

}  // namespace ihip
