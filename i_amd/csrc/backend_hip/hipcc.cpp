#include "hipcc.h"

#include <spawn.h>
#include <sys/stat.h>
#include <sys/wait.h>
#include <unistd.h>
#include <fcntl.h>
#include <cerrno>
#include <cstring>

#include <atomic>
#include <chrono>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <iterator>
#include <map>
#include <mutex>
#include <sstream>

extern char** environ;

namespace ihipc {
namespace {

const char* kFlags[] = {"--genco", "--offload-arch=gfx950", "-O3", "-std=c++17",
                        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};

std::mutex g_mu;
std::map<uint64_t, std::vector<char>> g_cache;
std::atomic<unsigned> g_counter{0};

uint64_t fnv1a(const std::string& s) {
  uint64_t h = 1469598103934665603ull;
  for (unsigned char c : s) {
    h ^= c;
    h *= 1099511628211ull;
  }
  return h;
}

std::string tmp_dir() {
  for (const char* name : {"TMPDIR", "TMP", "TEMP"})
    if (const char* v = std::getenv(name))
      if (*v) return v;
  return "/tmp";
}

std::string hipcc_path() {
  if (const char* v = std::getenv("ILANG_HIPCC")) return v;
  if (const char* v = std::getenv("ROCM_PATH")) {
    std::string p = std::string(v) + "/bin/hipcc";
    if (access(p.c_str(), X_OK) == 0) return p;
  }
  if (access("/opt/rocm/bin/hipcc", X_OK) == 0) return "/opt/rocm/bin/hipcc";
  return "hipcc";
}

// The on-disk cache of code objects: a directory that belongs to this user alone ($XDG_CACHE_HOME/ilang_hip or
// ~/.cache/ilang_hip, else <tmp>/ilang_hip_cache-<uid>), created 0700 and refused when somebody else owns it or
// others may write to it: what is found there is loaded and run on the GPU.  "" when no usable directory exists.
std::string private_cache_dir() {
  std::string dir;
  if (const char* x = std::getenv("XDG_CACHE_HOME"); x && *x) dir = std::string(x) + "/ilang_hip";
  else if (const char* h = std::getenv("HOME"); h && *h) {
    const std::string base = std::string(h) + "/.cache";
    mkdir(base.c_str(), 0700);  // may exist
    dir = base + "/ilang_hip";
  } else {
    dir = tmp_dir() + "/ilang_hip_cache-" + std::to_string((unsigned long)getuid());
  }
  if (mkdir(dir.c_str(), 0700) != 0 && errno != EEXIST) {
    dir = tmp_dir() + "/ilang_hip_cache-" + std::to_string((unsigned long)getuid());
    if (mkdir(dir.c_str(), 0700) != 0 && errno != EEXIST) return {};
  }
  struct stat st;
  if (lstat(dir.c_str(), &st) != 0 || !S_ISDIR(st.st_mode) || st.st_uid != getuid() || (st.st_mode & 022) != 0) return {};
  return dir;
}

// A cached image is stored behind its full source text (length, text, image): a 64-bit hash names the file, the
// comparison of the text is what says that the image belongs to this source.
bool read_cached(const std::string& path, const std::string& key_text, std::vector<char>* image) {
  std::ifstream f(path, std::ios::binary);
  if (!f) return false;
  uint64_t n = 0;
  f.read(reinterpret_cast<char*>(&n), sizeof n);
  if (!f || n != key_text.size()) return false;
  std::string text(n, '\0');
  f.read(text.data(), (std::streamsize)n);
  if (!f || text != key_text) return false;
  image->assign(std::istreambuf_iterator<char>(f), std::istreambuf_iterator<char>());
  return !image->empty();
}

bool write_cached(const std::string& path, const std::string& key_text, const std::vector<char>& image) {
  std::ofstream f(path, std::ios::binary | std::ios::trunc);
  const uint64_t n = key_text.size();
  f.write(reinterpret_cast<const char*>(&n), sizeof n);
  f.write(key_text.data(), (std::streamsize)n);
  f.write(image.data(), (std::streamsize)image.size());
  return (bool)f;
}

bool read_file(const std::string& path, std::vector<char>* out) {
  std::ifstream f(path, std::ios::binary);
  if (!f) return false;
  out->assign(std::istreambuf_iterator<char>(f), std::istreambuf_iterator<char>());
  return !out->empty();
}

}  // namespace

std::string hipcc_build(const std::string& source, std::vector<char>* image) {
  std::string key_text = source;
  for (const char* f : kFlags) key_text += std::string("\n") + f;
  const uint64_t key = fnv1a(key_text);
  {
    std::lock_guard<std::mutex> lock(g_mu);
    auto it = g_cache.find(key);
    if (it != g_cache.end()) {
      *image = it->second;
      return {};
    }
  }
  const std::string dir = tmp_dir();
  const std::string cache_dir = std::getenv("ILANG_NO_DISK_CACHE") == nullptr ? private_cache_dir() : std::string();
  char name[64];
  snprintf(name, sizeof name, "%016llx", (unsigned long long)key);
  const std::string cached = cache_dir + "/" + name + ".hsaco.cache";
  if (!cache_dir.empty() && read_cached(cached, key_text, image)) {
    std::lock_guard<std::mutex> lock(g_mu);
    g_cache[key] = *image;
    return {};
  }

  // unique per process, call and instant (the reference's bare nanosecond stamp can collide)
  const auto nanos = std::chrono::duration_cast<std::chrono::nanoseconds>(
                         std::chrono::system_clock::now().time_since_epoch()).count();
  std::ostringstream stem;
  stem << dir << "/ilang_" << getpid() << "_" << g_counter.fetch_add(1) << "_" << nanos;
  const std::string src_path = stem.str() + ".hip", obj_path = stem.str() + ".hsaco", log_path = stem.str() + ".log";
  {
    std::ofstream f(src_path, std::ios::binary);
    f << source;
    if (!f) return "cannot write " + src_path;
  }
  const std::string hipcc = hipcc_path();
  std::vector<std::string> args = {hipcc};
  for (const char* f : kFlags) args.push_back(f);
  args.push_back(src_path);
  args.push_back("-o");
  args.push_back(obj_path);
  std::vector<char*> argv;
  for (auto& a : args) argv.push_back(const_cast<char*>(a.c_str()));
  argv.push_back(nullptr);

  posix_spawn_file_actions_t fa;
  posix_spawn_file_actions_init(&fa);
  posix_spawn_file_actions_addopen(&fa, 1, log_path.c_str(), O_WRONLY | O_CREAT | O_TRUNC, 0600);
  posix_spawn_file_actions_adddup2(&fa, 1, 2);
  pid_t pid = 0;
  const int rc = posix_spawnp(&pid, hipcc.c_str(), &fa, nullptr, argv.data(), environ);
  posix_spawn_file_actions_destroy(&fa);
  std::string err;
  if (rc != 0) {
    err = "cannot run " + hipcc + ": " + std::string(strerror(rc));
  } else {
    int status = 0;
    while (waitpid(pid, &status, 0) < 0 && errno == EINTR) {
    }
    if (!WIFEXITED(status) || WEXITSTATUS(status) != 0) {
      std::ostringstream os;
      if (WIFEXITED(status)) os << "hipcc failed with status exit status: " << WEXITSTATUS(status);
      else os << "hipcc failed with status signal: " << (WIFSIGNALED(status) ? WTERMSIG(status) : -1);
      std::vector<char> log;
      if (read_file(log_path, &log)) os << "\n" << std::string(log.begin(), log.end()).substr(0, 4000);
      err = os.str();
    } else if (!read_file(obj_path, image)) {
      err = "hipcc produced no code object";
    }
  }
  std::remove(src_path.c_str());
  std::remove(log_path.c_str());
  if (err.empty()) {
    if (!cache_dir.empty()) {
      const std::string tmp = cached + "." + std::to_string(getpid()) + "." + std::to_string(g_counter.fetch_add(1));
      if (write_cached(tmp, key_text, *image)) std::rename(tmp.c_str(), cached.c_str());
      else std::remove(tmp.c_str());
    }
    std::lock_guard<std::mutex> lock(g_mu);
    g_cache[key] = *image;
  }
  std::remove(obj_path.c_str());
  return err;
}

}  // namespace ihipc
