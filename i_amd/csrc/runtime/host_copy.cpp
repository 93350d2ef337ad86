#include "host_copy.h"

#include <algorithm>
#include <condition_variable>
#include <cstdlib>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <thread>
#include <vector>

namespace ihip {
namespace {

// A few threads that copy slices of one block of host memory at a time (one thread moves 10-15 GB/s, the link
// to the device four times that).  ILANG_HIP_COPY_THREADS sets their number (default 8, the caller included;
// 1: the caller alone).  The threads are started on first use and live until the process ends.
class CopyCrew {
 public:
  static CopyCrew& get() {
    static CopyCrew* crew = new CopyCrew();  // (never destroyed: its threads may outlive static destructors)
    return *crew;
  }
  void copy(void* dst, const void* src, size_t bytes) {
    const size_t slices = std::min<size_t>(workers_.size() + 1, std::max<size_t>(1, bytes >> 20));  // at least 1 MiB each
    if (slices <= 1) {
      std::memcpy(dst, src, bytes);
      return;
    }
    std::lock_guard<std::mutex> one_job(job_mu_);  // one block at a time
    const size_t each = (bytes / slices + 63) / 64 * 64;
    {
      std::lock_guard<std::mutex> lock(mu_);
      dst_ = static_cast<char*>(dst);
      src_ = static_cast<const char*>(src);
      bytes_ = bytes;
      each_ = each;
      next_ = 1;  // slice 0 is the caller's
      pending_ = slices - 1;
      slices_ = slices;
      ++generation_;
    }
    wake_.notify_all();
    std::memcpy(dst, src, std::min(each, bytes));
    std::unique_lock<std::mutex> lock(mu_);
    done_.wait(lock, [&] { return pending_ == 0; });
  }

 private:
  CopyCrew() {
    size_t n = 8;
    if (const char* v = std::getenv("ILANG_HIP_COPY_THREADS")) n = (size_t)std::max(1, std::atoi(v));
    n = std::min<size_t>(n, std::max(1u, std::thread::hardware_concurrency()));
    for (size_t t = 1; t < n; ++t) workers_.emplace_back([this] { work(); }).detach();
  }
  void work() {
    size_t seen = 0;
    std::unique_lock<std::mutex> lock(mu_);
    for (;;) {
      wake_.wait(lock, [&] { return generation_ != seen && next_ < slices_; });
      while (next_ < slices_) {
        const size_t slice = next_++;
        const size_t at = slice * each_, len = at < bytes_ ? std::min(each_, bytes_ - at) : 0;
        char* const d = dst_ + at;
        const char* const s = src_ + at;
        lock.unlock();
        if (len) std::memcpy(d, s, len);
        lock.lock();
        if (--pending_ == 0) done_.notify_all();
      }
      seen = generation_;
    }
  }
  std::vector<std::thread> workers_;
  std::mutex job_mu_, mu_;
  std::condition_variable wake_, done_;
  char* dst_ = nullptr;
  const char* src_ = nullptr;
  size_t bytes_ = 0, each_ = 0, next_ = 0, slices_ = 0, pending_ = 0, generation_ = 0;
};

// A ring of page-locked chunks of one device (one for each direction): four chunks of 8 MiB (small enough that the first chunk's fill and
// the last chunk's transfer, which nothing overlaps, are a small part of a 64 MiB operand), allocated by the first
// large host call on that device and kept until the process ends.  One transfer uses the ring at a time; a chunk
// whose last transfer may still be in flight (in_flight) is awaited before it is touched again, not before: the
// upload of one operand runs into the upload of the next.
constexpr size_t kChunkBytes = size_t(8) << 20;
constexpr int kChunks = 4;
struct Ring {
  void* chunk[kChunks] = {};
  hipEvent_t landed[kChunks] = {};
  bool in_flight[kChunks] = {};
  size_t next = 0;  // the chunk that the next transfer step takes
  bool ready = false, failed = false;
  std::mutex busy;
  Err settle(int slot) {
    if (!in_flight[slot]) return {};
    in_flight[slot] = false;
    return check(hipEventSynchronize(landed[slot]), "hipEventSynchronize");
  }
};

struct RingTable {
  std::mutex mu;
  std::map<int, std::unique_ptr<Ring>> rings;
};
RingTable& ring_table() {
  static RingTable* table = new RingTable();
  return *table;
}
// (a ring for uploads and one for downloads per device, so that a download on one thread can run beside an upload
// on another: the link carries both directions at once)
Ring* ring_of_current_device(bool download) {
  RingTable& t = ring_table();
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return nullptr;
  std::lock_guard<std::mutex> lock(t.mu);
  auto& ring = t.rings[2 * device + (download ? 1 : 0)];
  if (!ring) ring = std::make_unique<Ring>();
  return ring.get();
}

// with ring->busy held
bool prepare(Ring* ring) {
  if (ring->ready) return true;
  if (ring->failed) return false;
  for (int c = 0; c < kChunks; ++c)
    if (hipHostMalloc(&ring->chunk[c], kChunkBytes, hipHostMallocDefault) != hipSuccess ||
        hipEventCreateWithFlags(&ring->landed[c], hipEventDisableTiming) != hipSuccess) {
      (void)hipGetLastError();
      ring->failed = true;  // (no page-locked memory to be had: plain copies from now on)
      return false;
    }
  ring->ready = true;
  return true;
}

}  // namespace

size_t release_copy_chunks() {
  RingTable& t = ring_table();
  std::lock_guard<std::mutex> lock(t.mu);
  size_t released = 0;
  for (auto& [device, ring] : t.rings) {
    std::unique_lock<std::mutex> idle(ring->busy, std::try_to_lock);
    if (!idle.owns_lock() || !ring->ready) continue;
    for (int c = 0; c < kChunks; ++c) {
      (void)ring->settle(c);
      (void)hipHostFree(ring->chunk[c]);
      (void)hipEventDestroy(ring->landed[c]);
      ring->chunk[c] = nullptr;
      ring->landed[c] = nullptr;
      released += kChunkBytes;
    }
    ring->ready = false;
  }
  return released;
}

Err upload_pipelined(void* dst, const void* src, size_t bytes, hipStream_t stream) {
  Ring* ring = bytes >= kPipelinedCopyBytes ? ring_of_current_device(false) : nullptr;
  std::unique_lock<std::mutex> lock;
  if (ring) lock = std::unique_lock<std::mutex>(ring->busy, std::try_to_lock);
  if (!ring || !lock.owns_lock() || !prepare(ring)) return h2d(dst, src, bytes, stream);
  for (size_t at = 0; at < bytes; at += kChunkBytes) {
    const int slot = (int)(ring->next++ % kChunks);
    const size_t len = std::min(kChunkBytes, bytes - at);
    if (Err e = ring->settle(slot); !e.empty()) return e;  // the chunk's last transfer has left it
    CopyCrew::get().copy(ring->chunk[slot], static_cast<const char*>(src) + at, len);
    if (Err e = check(hipMemcpyAsync(static_cast<char*>(dst) + at, ring->chunk[slot], len, hipMemcpyHostToDevice, stream), "hipMemcpy H2D");
        !e.empty())
      return e;
    if (Err e = check(hipEventRecord(ring->landed[slot], stream), "hipEventRecord"); !e.empty()) return e;
    ring->in_flight[slot] = true;
  }
  return {};
}

Err download_pipelined(void* dst, const void* src, size_t bytes, hipStream_t stream) {
  Ring* ring = bytes >= kPipelinedCopyBytes ? ring_of_current_device(true) : nullptr;
  std::unique_lock<std::mutex> lock;
  if (ring) lock = std::unique_lock<std::mutex>(ring->busy, std::try_to_lock);
  if (!ring || !lock.owns_lock() || !prepare(ring)) {
    if (Err e = d2h(dst, src, bytes, stream); !e.empty()) return e;
    return sync(stream);
  }
  const size_t chunks = (bytes + kChunkBytes - 1) / kChunkBytes, first = ring->next;
  ring->next += chunks;
  auto request = [&](size_t c) -> Err {
    const size_t at = c * kChunkBytes, len = std::min(kChunkBytes, bytes - at);
    const int slot = (int)((first + c) % kChunks);
    if (Err e = ring->settle(slot); !e.empty()) return e;
    if (Err e = check(hipMemcpyAsync(ring->chunk[slot], static_cast<const char*>(src) + at, len, hipMemcpyDeviceToHost, stream), "hipMemcpy D2H");
        !e.empty())
      return e;
    if (Err e = check(hipEventRecord(ring->landed[slot], stream), "hipEventRecord"); !e.empty()) return e;
    ring->in_flight[slot] = true;
    return {};
  };
  // transfers in flight ahead of the chunk that the host threads are emptying: all chunks of the ring but one
  for (size_t c = 0; c < std::min<size_t>(chunks, kChunks - 1); ++c)
    if (Err e = request(c); !e.empty()) return e;
  for (size_t c = 0; c < chunks; ++c) {
    const size_t at = c * kChunkBytes, len = std::min(kChunkBytes, bytes - at);
    const int slot = (int)((first + c) % kChunks);
    if (c + kChunks - 1 < chunks)
      if (Err e = request(c + kChunks - 1); !e.empty()) return e;  // (into the chunk emptied in the step before)
    if (Err e = ring->settle(slot); !e.empty()) return e;
    CopyCrew::get().copy(static_cast<char*>(dst) + at, ring->chunk[slot], len);
  }
  return {};
}

}  // namespace ihip
