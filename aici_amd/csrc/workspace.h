// The split-K scratch buffer that paged_attention_v1 needs but whose
// reference signature has no argument for.  One buffer per device, owned by
// the library, grown on demand, released by hipattn_shutdown.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>

namespace hipattn {

// Returns at least `bytes` of device memory on the current device.  Growing
// the buffer synchronises `stream` first, since enqueued work may still use
// the old one.  Calls that overlap on one device share the buffer and race.
void *library_workspace(size_t bytes, hipStream_t stream);

}  // namespace hipattn
