// Thread-local last-error slot behind i_error(): set on failure, never cleared
// on success, pointer valid until the next failure on the same thread
// (reference: core/src/lib.rs:57-59, 327-333, 442-446).
#pragma once
#include <string>

namespace icore {
void set_error(std::string message);
const char* last_error();
}  // namespace icore
