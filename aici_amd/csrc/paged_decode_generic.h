// Interface between paged_attention_v1 / v2's argument checking
// (paged_decode.hip) and the fp32-FMA decode kernel that serves 8- and
// 32-token blocks and fp32 caches (paged_decode_generic.hip).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace hipattn {

struct GenericDecodeParams {
  const void *q;
  int64_t q_stride;  // elements between sequences; heads are head_size apart
  const void *kc;    // [nb, Hkv, d/x, block_size, x], x = 16 / sizeof(T)
  const void *vc;    // [nb, Hkv, d, block_size]
  int64_t k_block_stride, k_head_stride, v_block_stride, v_head_stride;
  int64_t num_blocks;
  const int32_t *block_tables;
  int64_t table_stride;
  int table_cols;  // columns of block_tables: lookups are clamped to them
  const int32_t *context_lens;
  const float *alibi;  // [Hq] or null
  float scale;
  int Hq, G;  // G = Hq / Hkv
  int head_size, block_size;
  int num_seqs;
  int max_ctx;      // context lengths are clamped to this
  int part_tokens;  // tokens per partition, a multiple of block_size (set by paged_decode_generic)
  int num_parts;    // v2: given by the workspaces; v1: set by paged_decode_generic
  float *ws_acc;    // v1 partials [S, Hq, P, d] fp32
  float *ws_m;      // [S, Hq, P] partition maxima (natural-log units)
  float *ws_l;      // [S, Hq, P] partition sums
  void *tmp_out;    // v2 partials [S, Hq, P, d] in T
  void *out;
  int64_t out_stride;
};

// Tokens per partition of the v1 launch.
constexpr int kGenericPartTokens = 512;

// Launches on `stream`.  v2: the workspaces of `p` give the partition count.  v1: `num_parts` partitions of
// kGenericPartTokens tokens; with more than one, `scratch` holds num_seqs * Hq * num_parts * (head_size + 2)
// floats for the partials.
void paged_decode_generic(GenericDecodeParams p, int dtype, bool v2, int max_context_len, int num_parts, float *scratch,
                          hipStream_t stream);

}  // namespace hipattn
