#include "hip_rt.h"

#include <dlfcn.h>

#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <map>
#include <mutex>
#include <sstream>
#include <vector>

namespace ihip {

Err check(hipError_t e, const char* what) {
  if (e == hipSuccess) return {};
  std::ostringstream os;
  os << what << " failed: " << hipGetErrorString(e) << " (hip error " << (int)e << ")";
  return os.str();
}

namespace {

struct DeviceModule {
  hipModule_t mod = nullptr;
  std::map<std::string, hipFunction_t> fns;
  bool pool_tried = false;
  hipMemPool_t pool = nullptr;  // stream-ordered temporaries (temp_alloc)
};

thread_local int g_dry_run = 0;
std::mutex g_mu;
std::map<int, DeviceModule> g_builtin;  // keyed by device ordinal
std::vector<char> g_image;

std::string code_object_path() {
  if (const char* env = std::getenv("ILANG_HIP_KERNELS")) return env;
  Dl_info info;
  if (dladdr(reinterpret_cast<void*>(&code_object_path), &info) && info.dli_fname) {
    std::string so = info.dli_fname;
    auto slash = so.find_last_of('/');
    std::string dir = slash == std::string::npos ? "." : so.substr(0, slash);
    return dir + "/i_kernels_gfx950.hsaco";
  }
  return "i_kernels_gfx950.hsaco";
}

Err read_image() {
  if (!g_image.empty()) return {};
  const std::string path = code_object_path();
  std::ifstream f(path, std::ios::binary);
  if (!f) return "cannot open gfx950 code object '" + path + "' (build it with hipcc --genco, or set ILANG_HIP_KERNELS)";
  g_image.assign(std::istreambuf_iterator<char>(f), std::istreambuf_iterator<char>());
  if (g_image.empty()) return "gfx950 code object '" + path + "' is empty";
  return {};
}

}  // namespace

Err builtin_function(const char* name, hipFunction_t* fn) {
  std::lock_guard<std::mutex> lock(g_mu);
  int dev = 0;
  if (Err e = check(hipGetDevice(&dev), "hipGetDevice"); !e.empty()) return e;
  DeviceModule& dm = g_builtin[dev];
  if (!dm.mod) {
    if (Err e = read_image(); !e.empty()) return e;
    if (Err e = check(hipModuleLoadData(&dm.mod, g_image.data()), "hipModuleLoadData"); !e.empty()) {
      dm.mod = nullptr;
      return e;
    }
  }
  auto it = dm.fns.find(name);
  if (it == dm.fns.end()) {
    hipFunction_t f = nullptr;
    if (Err e = check(hipModuleGetFunction(&f, dm.mod, name), "hipModuleGetFunction"); !e.empty())
      return e + " [" + name + "]";
    it = dm.fns.emplace(name, f).first;
  }
  *fn = it->second;
  return {};
}

Err load_module(const void* image, hipModule_t* mod) { return check(hipModuleLoadData(mod, image), "hipModuleLoadData"); }

Err module_function(hipModule_t mod, const char* name, hipFunction_t* fn) {
  Err e = check(hipModuleGetFunction(fn, mod, name), "hipModuleGetFunction");
  if (!e.empty()) e += std::string(" [") + name + "]";
  return e;
}

void unload_module(hipModule_t mod) {
  if (mod) (void)hipModuleUnload(mod);
}

Err launch(hipFunction_t fn, unsigned gx, unsigned gy, unsigned gz, unsigned bx, const void* params,
           size_t params_size, hipStream_t stream) {
  if (gx == 0 || gy == 0 || gz == 0 || g_dry_run) return {};
  size_t size = params_size;
  void* config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, const_cast<void*>(params), HIP_LAUNCH_PARAM_BUFFER_SIZE, &size,
                    HIP_LAUNCH_PARAM_END};
  return check(hipModuleLaunchKernel(fn, gx, gy, gz, bx, 1, 1, 0, stream, nullptr, config), "hipModuleLaunchKernel");
}

DryRun::DryRun() { ++g_dry_run; }
DryRun::~DryRun() { --g_dry_run; }

// Stream-ordered temporaries come from a pool of the library's own, one per device, that keeps up to 1 GiB of
// freed memory instead of handing it back to the system when the stream runs dry, which is what makes a
// temporary cost tens of microseconds from the device's default pool.  The default pool and its settings, which
// belong to the application, are left alone; without a pool of its own (a runtime that has none to give: the
// creation fails) the library allocates from the default one.
Err temp_alloc(void** p, size_t bytes, hipStream_t stream) {
  *p = nullptr;
  if (bytes == 0) bytes = 4;
  hipMemPool_t pool = nullptr;
  {
    std::lock_guard<std::mutex> lock(g_mu);
    int dev = 0;
    if (Err e = check(hipGetDevice(&dev), "hipGetDevice"); !e.empty()) return e;
    DeviceModule& dm = g_builtin[dev];
    if (!dm.pool_tried) {
      dm.pool_tried = true;
      hipMemPoolProps props{};
      props.allocType = hipMemAllocationTypePinned;
      props.handleTypes = hipMemHandleTypeNone;
      props.location.type = hipMemLocationTypeDevice;
      props.location.id = dev;
      uint64_t keep = uint64_t(1) << 30;
      if (hipMemPoolCreate(&dm.pool, &props) != hipSuccess ||
          hipMemPoolSetAttribute(dm.pool, hipMemPoolAttrReleaseThreshold, &keep) != hipSuccess) {
        if (dm.pool) (void)hipMemPoolDestroy(dm.pool);
        dm.pool = nullptr;
        (void)hipGetLastError();
      }
    }
    pool = dm.pool;
  }
  if (pool) return check(hipMallocFromPoolAsync(p, bytes, pool, stream), "hipMallocFromPoolAsync");
  return check(hipMallocAsync(p, bytes, stream), "hipMallocAsync");
}

size_t trim_temp_pool() {
  std::lock_guard<std::mutex> lock(g_mu);
  size_t released = 0;
  for (auto& [dev, dm] : g_builtin) {
    if (!dm.pool) continue;
    uint64_t before = 0, after = 0;
    (void)hipMemPoolGetAttribute(dm.pool, hipMemPoolAttrReservedMemCurrent, &before);
    if (hipMemPoolTrimTo(dm.pool, 0) != hipSuccess) (void)hipGetLastError();
    (void)hipMemPoolGetAttribute(dm.pool, hipMemPoolAttrReservedMemCurrent, &after);
    if (before > after) released += (size_t)(before - after);
  }
  return released;
}

Err dev_alloc(void** p, size_t bytes) {
  *p = nullptr;
  if (bytes == 0) bytes = 4;
  return check(hipMalloc(p, bytes), "hipMalloc");
}
void dev_free(void* p) {
  if (p) (void)hipFree(p);
}
Err h2d(void* dst, const void* src, size_t bytes, hipStream_t stream) {
  if (bytes == 0) return {};
  return check(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, stream), "hipMemcpy H2D");
}
Err d2h(void* dst, const void* src, size_t bytes, hipStream_t stream) {
  if (bytes == 0) return {};
  return check(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, stream), "hipMemcpy D2H");
}
Err sync(hipStream_t stream) { return check(hipStreamSynchronize(stream), "hipStreamSynchronize"); }

}  // namespace ihip
