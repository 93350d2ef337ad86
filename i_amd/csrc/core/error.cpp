#include "error.h"

#include <algorithm>

namespace icore {
namespace {
thread_local std::string g_error;
thread_local bool g_has_error = false;
}  // namespace

void set_error(std::string message) {
  message.erase(std::remove(message.begin(), message.end(), '\0'), message.end());
  g_error = std::move(message);
  g_has_error = true;
}

const char* last_error() { return g_has_error ? g_error.c_str() : nullptr; }
}  // namespace icore
