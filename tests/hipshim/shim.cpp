// A host implementation of the dozen HIP entry points the runtime uses, for CPU tests of the generic
// code generator and the program executor (no GPU, no HIP runtime).
//   memory    every allocation ends exactly at an inaccessible guard page and has one before it, and is
//             filled with NaN bit patterns: an out-of-bounds access faults, a read of unwritten memory shows
//   modules   an "image" is a host shared object (produced by hostcc.py from the generated HIP source);
//             anything else (the prebuilt gfx950 code object) is refused, so only generated kernels run
//   launches  run synchronously, one work-item after the other, with blockIdx / threadIdx set per item; a
//             workgroup of more than 64 work-items runs its work-items as real threads with a working
//             __syncthreads(), one workgroup after the other
#include <dlfcn.h>
#include <elf.h>
#include <hip/hip_runtime_api.h>
#include <pthread.h>

#include <algorithm>
#include <sys/mman.h>
#include <unistd.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "../../i_amd/csrc/runtime/static_scratch.h"

namespace {
std::mutex g_mu;
struct Block {
  void* map;
  size_t map_len;
};
std::map<void*, Block> g_blocks;
const size_t kPage = 4096;

hipError_t guarded_alloc(void** p, size_t bytes) {
  if (bytes == 0) bytes = 4;
  const size_t body = (bytes + kPage - 1) / kPage * kPage;
  const size_t len = body + 2 * kPage;
  char* m = static_cast<char*>(mmap(nullptr, len, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS, -1, 0));
  if (m == MAP_FAILED) return hipErrorOutOfMemory;
  std::memset(m, 0xFF, len);
  mprotect(m, kPage, PROT_NONE);
  mprotect(m + kPage + body, kPage, PROT_NONE);
  char* user = m + kPage + body - ((bytes + 15) / 16 * 16);  // 16-byte aligned, ends within 15 bytes of the guard
  *p = user;
  std::lock_guard<std::mutex> lock(g_mu);
  g_blocks[user] = {m, len};
  return hipSuccess;
}
hipError_t guarded_free(void* p) {
  if (!p) return hipSuccess;
  std::lock_guard<std::mutex> lock(g_mu);
  auto it = g_blocks.find(p);
  if (it == g_blocks.end()) return hipErrorInvalidValue;
  munmap(it->second.map, it->second.map_len);
  g_blocks.erase(it);
  return hipSuccess;
}
struct Module {
  void* handle;
  std::string path;
};
struct BigArgs {
  unsigned char bytes[4096];
};
struct Function {
  void *kernel, *set_ids, *set_barrier, *set_wave;
};
void wait_on(void* barrier) { pthread_barrier_wait(static_cast<pthread_barrier_t*>(barrier)); }
}  // namespace

// The product takes its fixed workspace from a file-scope array in device memory (static_scratch.hip, built by
// hipcc); here it is one guarded host block of the same size, so a temporary carved past its end faults.
namespace ihip {
Err static_scratch(void** ptr) {
  static void* block = nullptr;
  if (!block && guarded_alloc(&block, kStaticScratchBytes) != hipSuccess) return "shim: no memory for the workspace";
  *ptr = block;
  return {};
}
}  // namespace ihip

extern "C" {
hipError_t hipGetDevice(int* dev) {
  *dev = 0;
  return hipSuccess;
}
const char* hipGetErrorString(hipError_t e) { return e == hipSuccess ? "no error" : "emulated HIP error"; }
hipError_t hipMalloc(void** p, size_t bytes) { return guarded_alloc(p, bytes); }
hipError_t hipFree(void* p) { return guarded_free(p); }
hipError_t hipMallocAsync(void** p, size_t bytes, hipStream_t) { return guarded_alloc(p, bytes); }
hipError_t hipFreeAsync(void* p, hipStream_t) { return guarded_free(p); }
// (no pool of its own here: the creation fails and the library allocates without one)
hipError_t hipGetLastError() { return hipSuccess; }
hipError_t hipHostMalloc(void**, size_t, unsigned int) { return hipErrorNotSupported; }
hipError_t hipStreamIsCapturing(hipStream_t, hipStreamCaptureStatus* status) {
  *status = hipStreamCaptureStatusNone;
  return hipSuccess;
}
hipError_t hipMemPoolCreate(hipMemPool_t*, const hipMemPoolProps*) { return hipErrorNotSupported; }
hipError_t hipMemPoolDestroy(hipMemPool_t) { return hipErrorNotSupported; }
hipError_t hipMemPoolSetAttribute(hipMemPool_t, hipMemPoolAttr, void*) { return hipErrorNotSupported; }
hipError_t hipMallocFromPoolAsync(void** p, size_t bytes, hipMemPool_t, hipStream_t) { return guarded_alloc(p, bytes); }
hipError_t hipMemcpyAsync(void* dst, const void* src, size_t bytes, hipMemcpyKind, hipStream_t) {
  std::memcpy(dst, src, bytes);
  return hipSuccess;
}
hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }
// (no page-locked memory here, so the library never gets as far as the events of its chunked host copies)
hipError_t hipSetDevice(int) { return hipSuccess; }
hipError_t hipStreamCreateWithFlags(hipStream_t*, unsigned) { return hipErrorNotSupported; }
hipError_t hipStreamWaitEvent(hipStream_t, hipEvent_t, unsigned) { return hipErrorNotSupported; }
hipError_t hipEventCreateWithFlags(hipEvent_t*, unsigned) { return hipErrorNotSupported; }
hipError_t hipEventRecord(hipEvent_t, hipStream_t) { return hipErrorNotSupported; }
hipError_t hipEventSynchronize(hipEvent_t) { return hipErrorNotSupported; }
hipError_t hipEventDestroy(hipEvent_t) { return hipErrorNotSupported; }
hipError_t hipHostFree(void*) { return hipErrorNotSupported; }
hipError_t hipMemPoolGetAttribute(hipMemPool_t, hipMemPoolAttr, void*) { return hipErrorNotSupported; }
hipError_t hipMemPoolTrimTo(hipMemPool_t, size_t) { return hipErrorNotSupported; }

hipError_t hipModuleLoadData(hipModule_t* mod, const void* image) {
  const auto* eh = static_cast<const Elf64_Ehdr*>(image);
  if (std::memcmp(eh->e_ident, ELFMAG, SELFMAG) != 0 || eh->e_machine != EM_X86_64) return hipErrorInvalidImage;
  const size_t size = eh->e_shoff + size_t(eh->e_shnum) * eh->e_shentsize;
  char path[] = "/tmp/ilang_shim_XXXXXX";
  const int fd = mkstemp(path);
  if (fd < 0) return hipErrorInvalidImage;
  const bool ok = write(fd, image, size) == (ssize_t)size;
  close(fd);
  void* h = ok ? dlopen(path, RTLD_NOW | RTLD_LOCAL) : nullptr;
  unlink(path);
  if (!h) {
    std::fprintf(stderr, "hip shim: dlopen failed: %s\n", dlerror());
    return hipErrorInvalidImage;
  }
  *mod = reinterpret_cast<hipModule_t>(new Module{h, path});
  return hipSuccess;
}
hipError_t hipModuleUnload(hipModule_t mod) {
  auto* m = reinterpret_cast<Module*>(mod);
  dlclose(m->handle);
  delete m;
  return hipSuccess;
}
hipError_t hipModuleGetFunction(hipFunction_t* fn, hipModule_t mod, const char* name) {
  auto* m = reinterpret_cast<Module*>(mod);
  void* f = dlsym(m->handle, name);
  void* set = dlsym(m->handle, "shim_set_ids");
  void* bar = dlsym(m->handle, "shim_set_barrier");
  void* wave = dlsym(m->handle, "shim_set_wave");
  if (!f || !set || !bar || !wave) return hipErrorNotFound;
  // a function handle is the kernel with the setters of its library (ids, workgroup barrier, wavefront context)
  *fn = reinterpret_cast<hipFunction_t>(new Function{f, set, bar, wave});
  return hipSuccess;
}
hipError_t hipModuleLaunchKernel(hipFunction_t fn, unsigned gx, unsigned gy, unsigned gz, unsigned bx, unsigned by,
                                 unsigned bz, unsigned, hipStream_t, void**, void** extra) {
  if (gy != 1 || gz != 1 || by != 1 || bz != 1 || !extra) return hipErrorInvalidValue;
  const void* buf = nullptr;
  size_t size = 0;
  for (void** e = extra; *e != HIP_LAUNCH_PARAM_END; e += 2) {
    if (*e == HIP_LAUNCH_PARAM_BUFFER_POINTER) buf = e[1];
    else if (*e == HIP_LAUNCH_PARAM_BUFFER_SIZE) size = *static_cast<size_t*>(e[1]);
  }
  if (!buf || size > sizeof(BigArgs)) return hipErrorInvalidValue;
  BigArgs args;
  std::memset(&args, 0xEE, sizeof args);
  std::memcpy(&args, buf, size);
  auto* f = reinterpret_cast<Function*>(fn);
  // a by-value struct larger than 16 bytes travels in memory at the start of the argument area, so a kernel
  // that declares a smaller struct reads its prefix of this one
  auto kernel = reinterpret_cast<void (*)(BigArgs)>(f->kernel);
  auto set_ids = reinterpret_cast<void (*)(unsigned, unsigned, unsigned, unsigned)>(f->set_ids);
  auto set_barrier = reinterpret_cast<void (*)(void (*)(void*), void*)>(f->set_barrier);
  auto set_wave = reinterpret_cast<void (*)(void (*)(void*), void*, float*)>(f->set_wave);
  if (bx > 64) {
    // the work-items of a workgroup run as threads, so that a barrier between two loop nests of a kernel means
    // what it means on the device: every work-item has finished the first nest before any starts the second
    for (unsigned block = 0; block < gx; ++block) {
      pthread_barrier_t barrier;
      pthread_barrier_init(&barrier, nullptr, bx);
      // every 64 consecutive work-items are a wavefront with a barrier and exchange slots of its own
      const unsigned waves = (bx + 63) / 64;
      std::vector<pthread_barrier_t> wave_barriers(waves);
      std::vector<float> wave_slots(64 * waves, 0.0f);
      for (unsigned w = 0; w < waves; ++w) pthread_barrier_init(&wave_barriers[w], nullptr, std::min(64u, bx - 64 * w));
      std::vector<std::thread> items;
      for (unsigned t = 0; t < bx; ++t)
        items.emplace_back([&, t] {
          set_ids(block, t, bx, gx);
          set_barrier(wait_on, &barrier);
          set_wave(wait_on, &wave_barriers[t / 64], &wave_slots[64 * (t / 64)]);
          kernel(args);
          set_barrier(nullptr, nullptr);
          set_wave(nullptr, nullptr, nullptr);
        });
      for (auto& th : items) th.join();
      for (unsigned w = 0; w < waves; ++w) pthread_barrier_destroy(&wave_barriers[w]);
      pthread_barrier_destroy(&barrier);
    }
    return hipSuccess;
  }
  // ILANG_SHIM_ORDER=reverse runs the work-items last to first: a result that depends on the order in which
  // work-items run exposes a dependency between them that the parallelisation analysis missed
  const char* order = std::getenv("ILANG_SHIM_ORDER");
  const bool reverse = order && std::strcmp(order, "reverse") == 0;
  const unsigned long total = (unsigned long)gx * bx;
  for (unsigned long n = 0; n < total; ++n) {
    const unsigned long id = reverse ? total - 1 - n : n;
    set_ids((unsigned)(id / bx), (unsigned)(id % bx), bx, gx);
    kernel(args);
  }
  return hipSuccess;
}
}
