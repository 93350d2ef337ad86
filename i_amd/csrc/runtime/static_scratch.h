// A fixed device workspace for callers that cannot allocate device memory (code under HIP graph capture,
// serving loops that forbid hipMalloc): one file-scope array in device memory per GPU, held from the moment
// the library's code is loaded on that GPU until the process ends.  The executor carves a program's
// temporaries out of it instead of calling hipMallocAsync.
#pragma once
#include <cstddef>

#include "hip_rt.h"

namespace ihip {

constexpr size_t kStaticScratchBytes = size_t(64) << 20;  // I_HIP_STATIC_WORKSPACE_BYTES in i_hip.h

// Device address of the current device's copy of the array.  The first call on a device resolves it
// (hipGetSymbolAddress) and remembers it; later calls only look it up.
Err static_scratch(void** ptr);

}  // namespace ihip
