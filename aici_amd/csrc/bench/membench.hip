// Yardsticks for the benchmark: what this device delivers for a plain read, a copy, a fill and a read of
// shuffled fixed-size chunks -- the figures the decode kernels' bandwidth is held against -- and what its matrix
// pipes deliver to a wavefront that does nothing but issue MFMAs, which the prefill kernels' rate is held
// against.  Built into a library of its own (libmembench.so); nothing in the attention library links or calls it.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <algorithm>

namespace {
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// NT: loads and stores carry the non-temporal hint (data touched once: not kept in the caches).
template <bool NT>
__device__ __forceinline__ u32x4 ld(const u32x4 *p) {
  if constexpr (NT) return __builtin_nontemporal_load(p);
  return *p;
}
template <bool NT>
__device__ __forceinline__ void st(u32x4 *p, u32x4 v) {
  if constexpr (NT)
    __builtin_nontemporal_store(v, p);
  else
    *p = v;
}

// Reads `n` 16-byte words once; the xor is stored only if it hits a value it cannot have by chance, so the
// loads stay and no traffic is written.
template <bool NT>
__global__ __launch_bounds__(256) void read_kernel(const u32x4 *__restrict__ src, unsigned int *sink, int64_t n) {
  unsigned int acc = 0;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const u32x4 v = ld<NT>(src + i);
    acc ^= v[0] ^ v[1] ^ v[2] ^ v[3];
  }
  if (acc == 0x9e3779b9u && sink) sink[0] = acc;
}
template <bool NT>
__global__ __launch_bounds__(256) void copy_kernel(const u32x4 *__restrict__ src, u32x4 *__restrict__ dst, int64_t n) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    st<NT>(dst + i, ld<NT>(src + i));
}
template <bool NT>
__global__ __launch_bounds__(256) void fill_kernel(u32x4 *__restrict__ dst, int64_t n) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    st<NT>(dst + i, u32x4{1u, 2u, 3u, 4u});
}
// One workgroup per entry of `chunks`: reads the chunk with that number, `words` 16-byte words long (256 for
// the 4 KiB in which the paged caches are read: one block of one kv head at head size 128, 16-bit).
template <bool NT>
__global__ __launch_bounds__(256) void read_chunks_kernel(const u32x4 *__restrict__ src, const int32_t *__restrict__ chunks,
                                                           unsigned int *sink, int64_t n_chunks, int words) {
  unsigned int acc = 0;
  for (int64_t k = blockIdx.x; k < n_chunks; k += gridDim.x) {
    const u32x4 *c = src + (int64_t)chunks[k] * words;
    for (int i = threadIdx.x; i < words; i += 256) {
      const u32x4 v = ld<NT>(c + i);
      acc ^= v[0] ^ v[1] ^ v[2] ^ v[3];
    }
  }
  if (acc == 0x9e3779b9u && sink) sink[0] = acc;
}

// Every wavefront streams v_mfma_f32_32x32x16_bf16 into four independent accumulators: 16 x iters MFMAs per
// wavefront, two wavefronts per SIMD, no memory traffic inside the loop.  The operands -- four A and four B
// registers per lane, used in rotation -- come from `ops` (8 x 512 x 16 bytes), because what the card's power
// management lets the pipes do depends on the values that flow through them.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
__global__ __launch_bounds__(512, 2) void mfma_stream_kernel(const u32x4 *__restrict__ ops, float *sink, int iters) {
  bf16x8 a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    a[i] = __builtin_bit_cast(bf16x8, ops[(2 * i) * 512 + threadIdx.x]);
    b[i] = __builtin_bit_cast(bf16x8, ops[(2 * i + 1) * 512 + threadIdx.x]);
  }
  f32x16 c0 = {}, c1 = {}, c2 = {}, c3 = {};
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[i], c0, 0, 0, 0);
      c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(i + 1) & 3], b[i], c1, 0, 0, 0);
      c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(i + 2) & 3], b[i], c2, 0, 0, 0);
      c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(i + 3) & 3], b[i], c3, 0, 0, 0);
    }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 16; i++) s += c0[i] + c1[i] + c2[i] + c3[i];
  if (s == 12345.678f && sink) sink[threadIdx.x] = s;  // (keeps the loop; never true by chance)
}
}  // namespace

// One launch of the MFMA stream on `workgroups` workgroups of eight wavefronts: 16 * iters MFMAs of 32768 flop
// per wavefront.  ops: 8 * 512 * 16 bytes of bf16 operands; sink may be null.  Returns 0, a hipError_t, or -1.
extern "C" int membench_mfma_stream(const void *ops, void *sink, int workgroups, int iters, void *stream_arg) {
  if (!ops || workgroups <= 0 || iters <= 0) return -1;
  mfma_stream_kernel<<<workgroups, 512, 0, static_cast<hipStream_t>(stream_arg)>>>(static_cast<const u32x4 *>(ops),
                                                                                  static_cast<float *>(sink), iters);
  return (int)hipGetLastError();
}

// mode 0 reads src once (dst may be null), 1 copies src to dst, 2 fills dst, 3 reads the chunks of src that
// chunks[0..n_chunks) number (each 0 <= chunks[k] < bytes / chunk_bytes; chunk_bytes a multiple of 4096);
// mode + 8: the same with non-temporal loads and stores.  Returns 0, a hipError_t, or -1 for bad arguments.
extern "C" int membench_probe(int mode, void *dst, const void *src, int64_t bytes, const int32_t *chunks, int64_t n_chunks,
                              int chunk_bytes, void *stream_arg) {
  hipStream_t stream = static_cast<hipStream_t>(stream_arg);
  if (bytes < 0 || bytes % 16 != 0) return -1;
  const int64_t n = bytes / 16;
  if (n == 0) return 0;
  const unsigned grid = (unsigned)std::min<int64_t>((n + 255) / 256, 65536);
  const bool nt = (mode & 8) != 0;
  switch (mode & ~8) {
    case 0:
      if (!src) return -1;
      if (nt) read_kernel<true><<<grid, 256, 0, stream>>>(static_cast<const u32x4 *>(src), static_cast<unsigned int *>(dst), n);
      else read_kernel<false><<<grid, 256, 0, stream>>>(static_cast<const u32x4 *>(src), static_cast<unsigned int *>(dst), n);
      break;
    case 1:
      if (!src || !dst) return -1;
      if (nt) copy_kernel<true><<<grid, 256, 0, stream>>>(static_cast<const u32x4 *>(src), static_cast<u32x4 *>(dst), n);
      else copy_kernel<false><<<grid, 256, 0, stream>>>(static_cast<const u32x4 *>(src), static_cast<u32x4 *>(dst), n);
      break;
    case 2:
      if (!dst) return -1;
      if (nt) fill_kernel<true><<<grid, 256, 0, stream>>>(static_cast<u32x4 *>(dst), n);
      else fill_kernel<false><<<grid, 256, 0, stream>>>(static_cast<u32x4 *>(dst), n);
      break;
    case 3: {
      if (!src || !chunks || n_chunks <= 0 || chunk_bytes <= 0 || chunk_bytes % 4096 != 0 || bytes % chunk_bytes != 0) return -1;
      const unsigned g = (unsigned)std::min<int64_t>(n_chunks, 16384);
      if (nt)
        read_chunks_kernel<true><<<g, 256, 0, stream>>>(static_cast<const u32x4 *>(src), chunks, static_cast<unsigned int *>(dst),
                                                        n_chunks, chunk_bytes / 16);
      else
        read_chunks_kernel<false><<<g, 256, 0, stream>>>(static_cast<const u32x4 *>(src), chunks, static_cast<unsigned int *>(dst),
                                                         n_chunks, chunk_bytes / 16);
      break;
    }
    default: return -1;
  }
  return (int)hipGetLastError();
}
