// Builds generated HIP source into a gfx950 code object with hipcc
// (the counterpart of the reference's `cc -O3 -shared -fPIC` step,
// core/src/lib.rs:394-415).  Results are cached by source text, in the process
// and under $TMPDIR/ilang_hip_cache, so a component is compiled once per machine.
#pragma once
#include <string>
#include <vector>

namespace ihipc {
// Returns "" on success and fills `image`; otherwise the failure text
// ("hipcc failed with status ..." plus the compiler's diagnostics).
std::string hipcc_build(const std::string& source, std::vector<char>* image);
}
