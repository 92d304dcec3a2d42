// Scratch memory and tuning switches shared by the ops of the library.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>

namespace hipattn {

// Which op a library-owned scratch buffer belongs to: ops never share one.
enum WorkspaceUser { WS_PAGED_ATTENTION = 0, WS_BIAS_ARGMAX = 1, WS_LINEAR = 2 };

// Returns at least `bytes` of device memory on the current device for `user`,
// private to `stream`: calls on different streams never share a buffer, so
// they may overlap.  A buffer is zero-filled when it is allocated.  Growing allocates a new buffer and
// keeps the old one alive until hipattn_shutdown (work already enqueued, or a
// captured graph, may still point at it); nothing is synchronised.  A stream
// that is being captured cannot grow its buffer: the call fails with a
// message that says so.
void *library_workspace(WorkspaceUser user, size_t bytes, hipStream_t stream);

// Switches for tuning and for tests that want one particular kernel; read
// from the environment (HIPATTN_<NAME in capitals>) once, when the library is
// loaded, and changed afterwards only through hipattn_tuning_set.  Ops read
// plain integers here, never the environment.
struct Tuning {
  int decode_flat;         // -1: the library chooses; 0 / 1: partitioned / flat-split launch
  int decode_flat_wgs;     // 0: what the device holds at once; else workgroups of the flat launch
  int decode_part_blocks;  // 0: chosen per call; else KV blocks per partition (2..64)
  int prefill_kernel;      // 0: the library chooses; 1: eight wavefronts; 2 / 3: four wavefronts, 2 / 1 row tiles each; 4: three groups of four
  int paged_prefill_dma;   // -1: the library chooses; 0: staged tiles; 1: block images where possible
  int cache_move_lds;      // -1: the library chooses; 0: never the LDS-transposing kernels
  int prefill_wg_heads;      // eight-wavefront prefill: query heads of one kv group per workgroup, at most (0: the library chooses -- up to four; 1: one)
  int prefill_rescale_log2;  // prefill: a row's reference maximum moves when outgrown by more than 2^this (0..16, default 8)
  int linear_tiles;          // linear: 16-row tiles of the weight per wavefront (0: the library chooses; 1 or 2)
  int linear_waves;          // linear: wavefronts per workgroup (0: the library chooses; 4 or 8)
  int linear_splits;         // linear: ranges of the inner dimension (0: the library chooses; else 1..32)
};
const Tuning &tuning();

}  // namespace hipattn
