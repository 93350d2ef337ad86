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
  const std::string cache_dir = dir + "/ilang_hip_cache";
  char name[64];
  snprintf(name, sizeof name, "%016llx", (unsigned long long)key);
  const std::string cached = cache_dir + "/" + name + ".hsaco";
  if (std::getenv("ILANG_NO_DISK_CACHE") == nullptr && read_file(cached, image)) {
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
    if (std::getenv("ILANG_NO_DISK_CACHE") == nullptr) {
      mkdir(cache_dir.c_str(), 0700);
      const std::string tmp = cached + "." + std::to_string(getpid());
      if (std::rename(obj_path.c_str(), tmp.c_str()) == 0) std::rename(tmp.c_str(), cached.c_str());
    }
    std::lock_guard<std::mutex> lock(g_mu);
    g_cache[key] = *image;
  }
  std::remove(obj_path.c_str());
  return err;
}

}  // namespace ihipc
