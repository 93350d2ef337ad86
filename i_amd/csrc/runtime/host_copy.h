// Large host operands on their way to and from the device.
//
// The host entry points of the runtime ABI (i_exec, i_exec_into: core/src/lib.rs:200-286 in the reference) take
// operands in ordinary pageable memory, which the DMA engines cannot read: a plain hipMemcpy stages such data
// through the driver's own bounce buffer with one host thread and runs at a quarter of the link's rate.  Here the
// staging is the library's own: a ring of page-locked chunks per device, filled (or emptied) by a few host threads
// at once while the DMA of the chunk before is in flight.
#pragma once
#include <cstddef>

#include "hip_rt.h"

namespace ihip {

// Copies `bytes` from pageable host memory at `src` to device memory at `dst`, enqueuing the transfers on `stream`;
// the host side of every chunk is finished when the call returns, the last DMAs may still be in flight.
Err upload_pipelined(void* dst, const void* src, size_t bytes, hipStream_t stream);
// Copies `bytes` from device memory at `src` (as `stream` leaves it) to pageable host memory at `dst`; complete when
// the call returns.
Err download_pipelined(void* dst, const void* src, size_t bytes, hipStream_t stream);
// From this size on the two calls above pay (below it one plain copy does)
constexpr size_t kPipelinedCopyBytes = size_t(8) << 20;

// Frees the page-locked chunks of every device (those that no transfer is using at this moment); returns the bytes.
size_t release_copy_chunks();

}  // namespace ihip
