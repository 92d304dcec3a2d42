// What the varlen prefill kernels share: the launch parameters, the MFMA
// wrappers and the few cross-lane and LDS helpers.  Device code; included by
// the translation units that hold the kernels.
#pragma once

#include <type_traits>

#include "common.h"
#include "device_types.h"
#include "workspace.h"

namespace hipattn {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

struct PrefillParams {
  const void *q, *k, *v;
  void *out;
  float *lse;  // [batch, Hq, max_q] or null
  int64_t q_row, q_head, k_row, k_head, v_row, v_head, o_row, o_head;
  const int32_t *cu_q, *cu_k, *seqused_k;
  int batch, Hq, Hkv, G, d;
  int max_q;      // caller's bound on Lq; sizes the grid
  int lse_pitch;  // elements between (batch, head) rows of lse
  int n_qblocks;
  float scale_log2;
  int causal;  // win_left < 0 && win_right == 0
  // Query row i (0-based in its sequence) sees key j iff i + off - win_left <= j <= i + off + win_right,
  // off = Lk - Lq; a negative bound is no bound (flash_attn/softmax.h:142-179, flash_api.cpp:113-120).
  // Only prefill_varlen_kernel reads these; the eight-wavefront kernel takes causal or unmasked launches.
  int win_left, win_right;
  // K/V read straight from the paged cache (prefill_varlen_w8_kernel<..., W8_PAGED or W8_PAGED_DMA>): k and v are
  // the caches, position p of sequence b lives in block block_tables[b][p / 16] at offset p % 16.
  const int32_t *block_tables;
  const int32_t *context_lens;  // keys per sequence
  int64_t table_stride;
  int table_cols;
  int64_t num_blocks;
  int64_t kc_block, kc_head, vc_block, vc_head;  // cache strides in elements
  int64_t total_k;  // rows of k / v (all sequences): bounds the byte offsets inside a sequence
  int block_log2;  // paged forms: log2 of the cache's block size (3, 4 or 5); every kernel but the four-wavefront one needs 4
  // out holds fp32 instead of the input type: the accumulators divided by the row sums, not rounded again
  // (for checking the kernel's arithmetic apart from the rounding of its output; o_row / o_head count floats).
  int out_f32;
  float rescale_thr;  // a row's reference maximum moves when the row outgrows it by more than this (log2 units)
  // A workgroup of W wavefronts covers 2^wg_heads_log2 query heads of one kv group and 32 W >> wg_heads_log2
  // query rows of each (wavefront w: head w % heads, row group w / heads).
  int wg_heads_log2;
};

template <typename T>
struct Mfma32;
template <>
struct Mfma32<half_t> {
  __device__ static __forceinline__ f32x16_t run(half8_t a, half8_t b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};
template <>
struct Mfma32<bf16_t> {
  __device__ static __forceinline__ f32x16_t run(bf16x8_t a, bf16x8_t b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// A pointer that is the same in every lane, as the scalar it is: an "s" operand of inline asm is not made one
// when the compiler holds the value in vector registers.
template <typename P>
__device__ __forceinline__ const P *uniform_ptr(const P *ptr) {
  const uint64_t v = reinterpret_cast<uint64_t>(ptr);
  return reinterpret_cast<const P *>(((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32)) << 32) |
                                     (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v));
}

// Workgroup barrier for LDS hand-offs: waits for this wavefront's LDS
// operations only.  __syncthreads() also drains the vector-memory counter,
// which would make every tile wait for the global loads of later tiles
// that were just issued.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Maximum of a value and its counterpart in the other half of the wavefront
// (lane ^ 32), through the gfx950 half-swap instead of an LDS permute.
__device__ __forceinline__ float max_across_halves(float x) {
  const unsigned u = bit_cast<unsigned>(x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(bit_cast<float>((unsigned)r[0]), bit_cast<float>((unsigned)r[1]));
}

// max(a, b, c) in one instruction.  Scores are never NaN here, so the
// canonicalising copies fmaxf would add to every MFMA result are not needed.
__device__ __forceinline__ float max3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}

// Launches the kernel that rotates three groups of wavefronts through the matrix pipe (prefill_r3.hip) when it
// covers the shapes in p; returns false, having done nothing, when it does not.
bool launch_prefill_r3(const PrefillParams &p, int dtype, hipStream_t stream);
// Whether that kernel is the faster one for the launch in p (measured against the eight-wavefront kernel).
bool prefer_prefill_r3(const PrefillParams &p);

}  // namespace hipattn
