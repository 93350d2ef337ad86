// The fixed device workspace behind i_exec_into_device_noalloc: a file-scope array in device memory and the
// per-device lookup of its address.  Compiled by hipcc (host + gfx950) and linked into libi_core.so; the
// kernels that use the memory live in the prebuilt code object and in per-program code objects and receive
// the address as an ordinary pointer argument.
#include <hip/hip_runtime.h>

#include <map>
#include <mutex>

#include "static_scratch.h"

namespace {

// In host code this name is only a handle for hipGetSymbolAddress, never a device address: each GPU has its
// own copy of the array at its own address.  The host-side use below is what makes the compiler export the
// device copy under a name the runtime can look up; do not mark it `used` (the device copy then stays a local
// symbol of the code object and the lookup aborts inside the runtime).
static __device__ __align__(256) unsigned char scratch[ihip::kStaticScratchBytes];

std::mutex g_mu;
std::map<int, void*> g_address;  // device ordinal -> device address of that device's copy

}  // namespace

namespace ihip {

Err static_scratch(void** ptr) {
  *ptr = nullptr;
  int dev = 0;
  if (Err e = check(hipGetDevice(&dev), "hipGetDevice"); !e.empty()) return e;
  std::lock_guard<std::mutex> lock(g_mu);
  auto it = g_address.find(dev);
  if (it == g_address.end()) {
    void* address = nullptr;
    if (Err e = check(hipGetSymbolAddress(&address, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(static workspace)");
        !e.empty())
      return e;
    if (!address) return "static workspace: the runtime returned a null device address";
    it = g_address.emplace(dev, address).first;
  }
  *ptr = it->second;
  return {};
}

}  // namespace ihip
