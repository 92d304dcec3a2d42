// Rotary embedding, RMS norm, activations and the AICI bias+argmax step.
// All are HBM-bound streaming kernels: one workgroup per token (row), 16-byte
// accesses where alignment allows, reductions through wave shuffles and LDS.
#include "common.h"
#include "device_types.h"
#include "workspace.h"

namespace hipattn {

namespace {

// ---------------------------------------------------------------------------
// rotary_embedding (pos_encoding_kernels.cu:9-77).  Every product and the
// final sum are rounded to T, which is what the reference's per-operator
// half/bfloat16 arithmetic does and what torch's CPU ops do in the oracle.
// ---------------------------------------------------------------------------
template <typename T, typename Pos, bool NEOX>
__global__ __launch_bounds__(512) void rotary_kernel(const Pos *__restrict__ positions, T *__restrict__ query,
                                                     T *__restrict__ key, const T *__restrict__ cos_sin,
                                                     int rot_dim, int64_t q_stride, int64_t k_stride,
                                                     int num_heads, int num_kv_heads, int head_size,
                                                     int64_t max_pos) {
  const int64_t token = blockIdx.x;
  int64_t pos = (int64_t)positions[token];
  if (pos < 0 || pos >= max_pos) return;  // outside the table: leave the row untouched
  const int embed = rot_dim / 2;
  const T *cos_ptr = cos_sin + pos * rot_dim;
  const T *sin_ptr = cos_ptr + embed;
  const int nq = num_heads * embed;
  const int n = nq + num_kv_heads * embed;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    T *arr;
    int r;
    if (i < nq) {
      arr = query + token * q_stride + (int64_t)(i / embed) * head_size;
      r = i % embed;
    } else {
      const int j = i - nq;
      arr = key + token * k_stride + (int64_t)(j / embed) * head_size;
      r = j % embed;
    }
    const int xi = NEOX ? r : 2 * r;
    const int yi = NEOX ? embed + r : 2 * r + 1;
    const T c = cos_ptr[r], s = sin_ptr[r];
    const T x = arr[xi], y = arr[yi];
    arr[xi] = sub_t(mul_t(x, c), mul_t(y, s));
    arr[yi] = add_t(mul_t(y, c), mul_t(x, s));
  }
}

// NeoX layout, 2-byte types, in 16-byte steps: a thread rotates 8 pairs
// (x at r..r+7, y at rot/2 + r..) of one head.  Same per-operation rounding.
template <typename T, typename Pos>
__global__ __launch_bounds__(512) void rotary_neox_vec8_kernel(const Pos *__restrict__ positions, T *__restrict__ query,
                                                               T *__restrict__ key, const T *__restrict__ cos_sin,
                                                               int rot_dim, int64_t q_stride, int64_t k_stride,
                                                               int num_heads, int num_kv_heads, int head_size,
                                                               int64_t max_pos) {
  const int64_t token = blockIdx.x;
  const int64_t pos = (int64_t)positions[token];
  if (pos < 0 || pos >= max_pos) return;
  const int embed = rot_dim / 2;
  const int per_head = embed / 8;
  const int n = (num_heads + num_kv_heads) * per_head;
  const T *cos_ptr = cos_sin + pos * rot_dim;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const int hd = i / per_head;
    const int r = (i % per_head) * 8;
    T *arr = hd < num_heads ? query + token * q_stride + (int64_t)hd * head_size
                            : key + token * k_stride + (int64_t)(hd - num_heads) * head_size;
    const uint4 xr = load16_once(arr + r);
    const uint4 yr = load16_once(arr + embed + r);
    const uint4 cr = *reinterpret_cast<const uint4 *>(cos_ptr + r);
    const uint4 sr = *reinterpret_cast<const uint4 *>(cos_ptr + embed + r);
    const T *x = reinterpret_cast<const T *>(&xr), *y = reinterpret_cast<const T *>(&yr);
    const T *c = reinterpret_cast<const T *>(&cr), *sn = reinterpret_cast<const T *>(&sr);
    uint4 xo, yo;
    T *xe = reinterpret_cast<T *>(&xo), *ye = reinterpret_cast<T *>(&yo);
#pragma unroll
    for (int j = 0; j < 8; j++) {
      xe[j] = sub_t(mul_t(x[j], c[j]), mul_t(y[j], sn[j]));
      ye[j] = add_t(mul_t(y[j], c[j]), mul_t(x[j], sn[j]));
    }
    *reinterpret_cast<uint4 *>(arr + r) = xo;
    *reinterpret_cast<uint4 *>(arr + embed + r) = yo;
  }
}

// ---------------------------------------------------------------------------
// rms_norm / fused_add_rms_norm (layernorm_kernels.cu:10-65):
//   out = T(x * rsqrt(mean(x^2) + eps)) * w, the product again rounded to T.
// ---------------------------------------------------------------------------
template <typename T, bool FUSED_ADD>
__global__ __launch_bounds__(1024) void rms_norm_kernel(T *__restrict__ out, T *__restrict__ input,
                                                        T *__restrict__ residual,
                                                        const T *__restrict__ weight, float eps,
                                                        int hidden, int64_t in_stride,
                                                        int64_t out_stride) {
  __shared__ float smem[17];
  const int64_t row = blockIdx.x;
  T *x = input + row * in_stride;
  T *res = FUSED_ADD ? residual + row * in_stride : nullptr;
  T *o = FUSED_ADD ? x : out + row * out_stride;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float v = to_float(x[i]);
    if (FUSED_ADD) {
      // The variance uses the un-rounded sum, the second pass the rounded one
      // (layernorm_kernels.cu:48-63).
      v += to_float(res[i]);
      res[i] = from_float<T>(v);
    }
    ss += v * v;
  }
  const float total = block_sum(ss, smem);
  const float inv = rsqrtf(total / (float)hidden + eps);
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float v = to_float(FUSED_ADD ? res[i] : x[i]);
    const T normed = from_float<T>(v * inv);
    o[i] = from_float<T>(to_float(normed) * to_float(weight[i]));
  }
}

// 16-byte variant for 2-byte types: a thread keeps its 8 elements in registers
// between the reduction and the scaling, so every byte crosses once.
template <typename T, bool FUSED_ADD>
__global__ __launch_bounds__(1024) void rms_norm_vec8_kernel(T *__restrict__ out, T *__restrict__ input,
                                                             T *__restrict__ residual,
                                                             const T *__restrict__ weight, float eps, int hidden) {
  __shared__ float smem[17];
  const int64_t row = blockIdx.x;
  const int i = threadIdx.x * 8;
  const bool active = i < hidden;
  T *x = input + row * (int64_t)hidden + i;
  float v[8];
  float ss = 0.f;
  if (active) {
    // (read-once hint only where the row is not written back in place: with the residual update it measured
    // 2 % slower, without it 6 % faster, 32768 x 4096)
    const uint4 raw = FUSED_ADD ? *reinterpret_cast<const uint4 *>(x) : load16_once(x);
    const T *e = reinterpret_cast<const T *>(&raw);
#pragma unroll
    for (int j = 0; j < 8; j++) v[j] = to_float(e[j]);
    if (FUSED_ADD) {
      T *res = residual + row * (int64_t)hidden + i;
      const uint4 rr = *reinterpret_cast<const uint4 *>(res);
      const T *re = reinterpret_cast<const T *>(&rr);
      uint4 ro;
      T *oe = reinterpret_cast<T *>(&ro);
#pragma unroll
      for (int j = 0; j < 8; j++) {
        v[j] += to_float(re[j]);
        oe[j] = from_float<T>(v[j]);
      }
      *reinterpret_cast<uint4 *>(res) = ro;
#pragma unroll
      for (int j = 0; j < 8; j++) {
        ss += v[j] * v[j];            // variance from the un-rounded sum,
        v[j] = to_float(oe[j]);       // scaling from the rounded one (layernorm_kernels.cu:48-63)
      }
    } else {
#pragma unroll
      for (int j = 0; j < 8; j++) ss += v[j] * v[j];
    }
  }
  const float total = block_sum(ss, smem);
  const float inv = rsqrtf(total / (float)hidden + eps);
  if (active) {
    const uint4 wr = *reinterpret_cast<const uint4 *>(weight + i);
    const T *we = reinterpret_cast<const T *>(&wr);
    uint4 o;
    T *oe = reinterpret_cast<T *>(&o);
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const T normed = from_float<T>(v[j] * inv);
      oe[j] = from_float<T>(to_float(normed) * to_float(we[j]));
    }
    T *op = FUSED_ADD ? x : out + row * (int64_t)hidden + i;
    *reinterpret_cast<uint4 *>(op) = o;
  }
}

// ---------------------------------------------------------------------------
// Activations (activation_kernels.cu:15-115).
// ---------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ T silu_t(T x) {
  const float f = to_float(x);
  return from_float<T>(f / (1.0f + expf(-f)));
}

template <typename T>
__global__ __launch_bounds__(1024) void silu_and_mul_kernel(T *__restrict__ out, const T *__restrict__ in, int d) {
  const int64_t row = blockIdx.x;
  for (int i = threadIdx.x; i < d; i += blockDim.x) {
    const T x = in[row * 2 * d + i];
    const T y = in[row * 2 * d + d + i];
    out[row * d + i] = mul_t(silu_t(x), y);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void silu_and_mul_vec8_kernel(T *__restrict__ out, const T *__restrict__ in, int d) {
  const int64_t row = blockIdx.y;
  const int i = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (i >= d) return;
  const uint4 xr = load16_once(in + row * 2 * d + i);
  const uint4 yr = load16_once(in + row * 2 * d + d + i);
  const T *xe = reinterpret_cast<const T *>(&xr);
  const T *ye = reinterpret_cast<const T *>(&yr);
  uint4 o;
  T *oe = reinterpret_cast<T *>(&o);
#pragma unroll
  for (int j = 0; j < 8; j++) oe[j] = mul_t(silu_t(xe[j]), ye[j]);
  *reinterpret_cast<uint4 *>(out + row * d + i) = o;
}

template <typename T>
__device__ __forceinline__ T gelu_new_t(T x) {
  // 0.5*x*(1+tanh(sqrt(2/pi)*(x+0.044715*x^3))), rounded where the reference rounds.
  const T x3t = mul_t(mul_t(x, x), x);
  const float x3 = to_float(x3t);
  const T inner = add_t(x, from_float<T>(0.044715f * x3));
  const T arg = from_float<T>(0.79788456f * to_float(inner));
  const T t = from_float<T>(tanhf(to_float(arg)));
  return mul_t(mul_t(from_float<T>(0.5f), x), add_t(from_float<T>(1.0f), t));
}

template <typename T>
__device__ __forceinline__ T gelu_fast_t(T x) {
  const float f = to_float(x);
  const T a = from_float<T>(f * 0.79788456f);
  const T b = add_t(from_float<T>(1.0f), mul_t(from_float<T>(0.044715f * f), x));
  const T t = from_float<T>(tanhf(to_float(mul_t(a, b))));
  return mul_t(mul_t(from_float<T>(0.5f), x), add_t(from_float<T>(1.0f), t));
}

template <typename T, int KIND>
__global__ __launch_bounds__(1024) void activation_kernel(T *__restrict__ out, const T *__restrict__ in, int d) {
  const int64_t row = blockIdx.x;
  for (int i = threadIdx.x; i < d; i += blockDim.x) {
    const T x = in[row * d + i];
    out[row * d + i] = KIND == 0 ? gelu_new_t(x) : gelu_fast_t(x);
  }
}

// ---------------------------------------------------------------------------
// AICI step: biased logits -> greedy token, one workgroup per sequence.
// ---------------------------------------------------------------------------
template <typename T, int MODE /*0 = f32 bias rows, 1 = packed allow-bits*/>
__global__ __launch_bounds__(1024) void bias_argmax_kernel(const T *__restrict__ logits, int64_t logit_stride,
                                                           const float *__restrict__ bias, int64_t bias_stride,
                                                           const uint8_t *__restrict__ mask, int64_t mask_stride,
                                                           int64_t mask_bytes, const int32_t *__restrict__ rows, int64_t nrows,
                                                           int vocab, int32_t *__restrict__ out_tokens,
                                                           float *__restrict__ out_logits) {
  __shared__ float s_val[16];
  __shared__ int s_idx[16];
  const int64_t seq = blockIdx.x;
  int64_t row = rows ? (int64_t)rows[seq] : seq;
  row = row < 0 ? 0 : (row >= nrows ? nrows - 1 : row);  // a bad row index reads a wrong row, never outside
  const T *lg = logits + seq * logit_stride;
  float best = -INFINITY;
  int best_i = 0x7fffffff;
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
    float v = to_float(lg[i]);
    if (MODE == 0) {
      v += bias[row * bias_stride + i];
    } else {
      const int64_t byte = i >> 3;
      const bool allowed = byte < mask_bytes && ((mask[row * mask_stride + byte] >> (i & 7)) & 1);
      if (!allowed) v = -INFINITY;
    }
    if (v > best) {  // strided order is increasing in i, so ties keep the lowest id
      best = v;
      best_i = i;
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best, o, 64);
    const int oi = __shfl_xor(best_i, o, 64);
    if (ov > best || (ov == best && oi < best_i)) {
      best = ov;
      best_i = oi;
    }
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nwaves = (blockDim.x + 63) >> 6;
  if (lane == 0) {
    s_val[wave] = best;
    s_idx[wave] = best_i;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < nwaves; w++) {
      if (s_val[w] > best || (s_val[w] == best && s_idx[w] < best_i)) {
        best = s_val[w];
        best_i = s_idx[w];
      }
    }
    // Every token disallowed (or vocab == 0): torch's argmax over a row of
    // equal -inf values yields index 0.
    if (best_i == 0x7fffffff) best_i = 0;
    out_tokens[seq] = best_i;
    if (out_logits) out_logits[seq] = best;
  }
}

// Wide variant: each row is cut into slices handled by separate workgroups (a
// step has far fewer sequences than the chip has CUs), 8 logits and one mask
// byte per thread and load.  Same order rule: the largest value, the lowest id
// among equals.  A slice's winner is one 64-bit key -- the value's bits made
// monotonic above, the complement of the id below -- so the best slice of a
// row is a device-wide atomic maximum; the workgroup that counts in last reads
// it and writes the row's result (row_state: {key, counter} per row, cleared by
// a small fill kernel in front of every launch, so that whatever an overlapping
// or interrupted call left there cannot reach a later one).
struct ArgmaxRowState {
  unsigned long long key;
  unsigned int arrived;
  unsigned int pad;
};

// (a kernel, not hipMemsetAsync: the call may be recorded into a graph)
__global__ void argmax_state_clear_kernel(ArgmaxRowState *__restrict__ st, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) st[i] = ArgmaxRowState{0ull, 0u, 0u};
}

__device__ __forceinline__ unsigned long long argmax_key(float v, int idx) {
  const unsigned int b = __float_as_uint(v);
  const unsigned int mono = (b & 0x80000000u) ? ~b : (b | 0x80000000u);
  return ((unsigned long long)mono << 32) | (unsigned int)(0xffffffffu - (unsigned int)idx);
}

template <typename T, int MODE>
__global__ __launch_bounds__(256) void bias_argmax_slice_kernel(const T *__restrict__ logits, int64_t logit_stride,
                                                                const float *__restrict__ bias, int64_t bias_stride,
                                                                const uint8_t *__restrict__ mask, int64_t mask_stride,
                                                                int64_t mask_bytes, const int32_t *__restrict__ rows, int64_t nrows,
                                                                int vocab, int per_slice /* multiple of 8 */,
                                                                ArgmaxRowState *__restrict__ row_state,
                                                                int32_t *__restrict__ out_tokens,
                                                                float *__restrict__ out_logits) {
  __shared__ float s_val[4];
  __shared__ int s_idx[4];
  const int64_t seq = blockIdx.y;
  const int slice = blockIdx.x;
  int64_t row = rows ? (int64_t)rows[seq] : seq;
  row = row < 0 ? 0 : (row >= nrows ? nrows - 1 : row);  // a bad row index reads a wrong row, never outside
  const T *lg = logits + seq * logit_stride;
  const int begin = slice * per_slice;
  const int end = min(begin + per_slice, vocab);
  float best = -INFINITY;
  int best_i = 0x7fffffff;
  for (int i = begin + threadIdx.x * 8; i < end; i += blockDim.x * 8) {
    const uint4 raw = *reinterpret_cast<const uint4 *>(lg + i);
    const T *e = reinterpret_cast<const T *>(&raw);
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; j++) v[j] = to_float(e[j]);
    if (MODE == 0) {
      const float4 b0 = *reinterpret_cast<const float4 *>(bias + row * bias_stride + i);
      const float4 b1 = *reinterpret_cast<const float4 *>(bias + row * bias_stride + i + 4);
      v[0] += b0.x; v[1] += b0.y; v[2] += b0.z; v[3] += b0.w;
      v[4] += b1.x; v[5] += b1.y; v[6] += b1.z; v[7] += b1.w;
    } else {
      const int64_t byte = i >> 3;
      const unsigned m = byte < mask_bytes ? mask[row * mask_stride + byte] : 0u;
#pragma unroll
      for (int j = 0; j < 8; j++)
        if (!((m >> j) & 1)) v[j] = -INFINITY;
    }
#pragma unroll
    for (int j = 0; j < 8; j++)
      if (v[j] > best) {  // increasing ids within a thread: ties keep the lowest
        best = v[j];
        best_i = i + j;
      }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best, o, 64);
    const int oi = __shfl_xor(best_i, o, 64);
    if (ov > best || (ov == best && oi < best_i)) {
      best = ov;
      best_i = oi;
    }
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) {
    s_val[wave] = best;
    s_idx[wave] = best_i;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < (int)(blockDim.x >> 6); w++)
      if (s_val[w] > best || (s_val[w] == best && s_idx[w] < best_i)) {
        best = s_val[w];
        best_i = s_idx[w];
      }
    ArgmaxRowState *st = row_state + seq;
    // Key and counter are only ever touched by device-scope read-modify-writes, which are performed where every XCD
    // sees them.  The count depends on what the maximum returned, so it is issued only once the maximum has been
    // performed, and the workgroup whose count comes back last takes the key with one more read-modify-write.
    // Fences instead (release before the count: the XCD's L2 written back by every workgroup; acquire in the last
    // workgroup: that L2 invalidated under the others) were measured at 29 and 17 us per call against 12.
    const unsigned long long old =
        __hip_atomic_fetch_max(&st->key, argmax_key(best, best_i), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned int one = old == ~0ull ? 2u : 1u;  // always 1: no key is all ones
    const unsigned int before = __hip_atomic_fetch_add(&st->arrived, one, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (before == gridDim.x - 1) {
      const unsigned long long key = __hip_atomic_exchange(&st->key, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const unsigned int mono = (unsigned int)(key >> 32);
      int token = (int)(0xffffffffu - (unsigned int)key);
      if (token == 0x7fffffff) token = 0;  // every token disallowed: torch's argmax of equal -inf is 0
      out_tokens[seq] = token;
      if (out_logits) out_logits[seq] = __uint_as_float((mono & 0x80000000u) ? (mono & 0x7fffffffu) : ~mono);
    }
  }
}

int round_threads(int64_t n, int cap) {
  int64_t t = ((n + 63) / 64) * 64;
  if (t < 64) t = 64;
  if (t > cap) t = cap;
  return (int)t;
}

void rotary_impl(const hipattn_tensor *positions, hipattn_tensor *query, hipattn_tensor *key, int head_size,
                 const hipattn_tensor *cos_sin, bool is_neox, void *stream_arg) {
  check_index_tensor(positions, "positions", 1);
  check_tensor(query, "query", 2);
  check_tensor(key, "key", 2);
  check_tensor(cos_sin, "cos_sin_cache", 2);
  HA_CHECK(is_float_dtype(query->dtype), "rotary_embedding: query must be f32/f16/bf16");
  HA_CHECK(key->dtype == query->dtype && cos_sin->dtype == query->dtype,
           "rotary_embedding: query, key and cos_sin_cache must share a dtype");
  HA_CHECK(head_size > 0, "rotary_embedding: head_size must be positive");
  const int64_t T = query->sizes[0];
  HA_CHECK(key->sizes[0] == T && positions->sizes[0] == T,
           "rotary_embedding: positions/query/key disagree on the token count");
  HA_CHECK(query->sizes[1] % head_size == 0 && key->sizes[1] % head_size == 0,
           "rotary_embedding: row width is not a multiple of head_size %d", head_size);
  const int rot_dim = (int)cos_sin->sizes[1];
  HA_CHECK(rot_dim % 2 == 0 && rot_dim <= head_size, "rotary_embedding: rot_dim %d invalid for head_size %d",
           rot_dim, head_size);
  HA_CHECK((query->sizes[1] <= 1 || query->strides[1] == 1) && (key->sizes[1] <= 1 || key->strides[1] == 1),
           "rotary_embedding: query/key rows must be contiguous");
  check_contiguous(cos_sin, "cos_sin_cache");
  check_data(query, "query");
  check_data(key, "key");
  check_data(cos_sin, "cos_sin_cache");
  if (T == 0 || rot_dim == 0) return;
  const int Hq = (int)(query->sizes[1] / head_size), Hkv = (int)(key->sizes[1] / head_size);
  hipStream_t stream = resolve_stream(stream_arg);
  const int threads = round_threads((int64_t)(Hq + Hkv) * rot_dim / 2, 512);
  const int64_t max_pos = cos_sin->sizes[0];
  auto a16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  if (is_neox && dtype_size(query->dtype) == 2 && rot_dim % 16 == 0 && head_size % 8 == 0 &&
      query->strides[0] % 8 == 0 && key->strides[0] % 8 == 0 && a16(query->data) && a16(key->data) &&
      a16(cos_sin->data)) {
    const int vthreads = round_threads((int64_t)(Hq + Hkv) * rot_dim / 16, 512);
#define HA_ROTV(TT, PP)                                                                                       \
  rotary_neox_vec8_kernel<TT, PP><<<dim3((unsigned)T), vthreads, 0, stream>>>(                                 \
      static_cast<const PP *>(positions->data), static_cast<TT *>(query->data), static_cast<TT *>(key->data), \
      static_cast<const TT *>(cos_sin->data), rot_dim, query->strides[0], key->strides[0], Hq, Hkv, head_size, \
      max_pos)
    if (query->dtype == HIPATTN_F16) {
      if (positions->dtype == HIPATTN_I64) HA_ROTV(half_t, int64_t);
      else HA_ROTV(half_t, int32_t);
    } else {
      if (positions->dtype == HIPATTN_I64) HA_ROTV(bf16_t, int64_t);
      else HA_ROTV(bf16_t, int32_t);
    }
#undef HA_ROTV
    check_launch("rotary_embedding");
    return;
  }
#define HA_ROT(TT, PP, NX)                                                                              \
  rotary_kernel<TT, PP, NX><<<dim3((unsigned)T), threads, 0, stream>>>(                                  \
      static_cast<const PP *>(positions->data), static_cast<TT *>(query->data), static_cast<TT *>(key->data), \
      static_cast<const TT *>(cos_sin->data), rot_dim, query->strides[0], key->strides[0], Hq, Hkv, head_size, \
      max_pos)
#define HA_ROT_P(TT, NX)                           \
  if (positions->dtype == HIPATTN_I64) HA_ROT(TT, int64_t, NX); \
  else HA_ROT(TT, int32_t, NX)
#define HA_ROT_T(TT)          \
  if (is_neox) { HA_ROT_P(TT, true); } \
  else { HA_ROT_P(TT, false); }
  switch (query->dtype) {
    case HIPATTN_F32: HA_ROT_T(float); break;
    case HIPATTN_F16: HA_ROT_T(half_t); break;
    default: HA_ROT_T(bf16_t); break;
  }
#undef HA_ROT_T
#undef HA_ROT_P
#undef HA_ROT
  check_launch("rotary_embedding");
}

void rms_norm_impl(hipattn_tensor *out, hipattn_tensor *input, hipattn_tensor *residual,
                   const hipattn_tensor *weight, float eps, bool fused, void *stream_arg) {
  const char *op = fused ? "fused_add_rms_norm" : "rms_norm";
  HA_CHECK(input != nullptr && input->ndim >= 1 && input->ndim <= HIPATTN_MAX_DIMS, "%s: bad input rank", op);
  check_tensor(weight, "weight", 1);
  HA_CHECK(is_float_dtype(input->dtype) && weight->dtype == input->dtype, "%s: input/weight dtype mismatch", op);
  const int64_t hidden = input->sizes[input->ndim - 1];
  HA_CHECK(weight->sizes[0] == hidden, "%s: weight has %lld elements, hidden size is %lld", op,
           (long long)weight->sizes[0], (long long)hidden);
  check_contiguous(input, "input");
  check_contiguous(weight, "weight");
  hipattn_tensor *other = fused ? residual : out;
  HA_CHECK(other != nullptr && other->ndim == input->ndim && other->dtype == input->dtype, "%s: %s mismatch", op,
           fused ? "residual" : "out");
  for (int i = 0; i < input->ndim; i++)
    HA_CHECK(other->sizes[i] == input->sizes[i], "%s: shape mismatch in dim %d", op, i);
  check_contiguous(other, fused ? "residual" : "out");
  const int64_t rows = hidden == 0 ? 0 : numel(input) / hidden;
  if (rows == 0) return;
  check_data(input, "input");
  check_data(other, fused ? "residual" : "out");
  check_data(weight, "weight");
  hipStream_t stream = resolve_stream(stream_arg);
  auto al16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  if (dtype_size(input->dtype) == 2 && hidden % 8 == 0 && hidden <= 8192 && al16(input->data) &&
      al16(other->data) && al16(weight->data)) {
    const int vthreads = round_threads(hidden / 8, 1024);
#define HA_RMSV(TT)                                                                                         \
  if (fused)                                                                                                \
    rms_norm_vec8_kernel<TT, true><<<dim3((unsigned)rows), vthreads, 0, stream>>>(                           \
        nullptr, static_cast<TT *>(input->data), static_cast<TT *>(residual->data),                         \
        static_cast<const TT *>(weight->data), eps, (int)hidden);                                           \
  else                                                                                                      \
    rms_norm_vec8_kernel<TT, false><<<dim3((unsigned)rows), vthreads, 0, stream>>>(                          \
        static_cast<TT *>(out->data), static_cast<TT *>(input->data), nullptr,                              \
        static_cast<const TT *>(weight->data), eps, (int)hidden)
    if (input->dtype == HIPATTN_F16) {
      HA_RMSV(half_t);
    } else {
      HA_RMSV(bf16_t);
    }
#undef HA_RMSV
    check_launch(op);
    return;
  }
  const int threads = round_threads(hidden, 1024);
#define HA_RMS(TT)                                                                                          \
  if (fused)                                                                                                \
    rms_norm_kernel<TT, true><<<dim3((unsigned)rows), threads, 0, stream>>>(                                 \
        nullptr, static_cast<TT *>(input->data), static_cast<TT *>(residual->data),                         \
        static_cast<const TT *>(weight->data), eps, (int)hidden, hidden, hidden);                           \
  else                                                                                                      \
    rms_norm_kernel<TT, false><<<dim3((unsigned)rows), threads, 0, stream>>>(                                \
        static_cast<TT *>(out->data), static_cast<TT *>(input->data), nullptr,                              \
        static_cast<const TT *>(weight->data), eps, (int)hidden, hidden, hidden)
  switch (input->dtype) {
    case HIPATTN_F32: HA_RMS(float); break;
    case HIPATTN_F16: HA_RMS(half_t); break;
    default: HA_RMS(bf16_t); break;
  }
#undef HA_RMS
  check_launch(op);
}

void activation_impl(hipattn_tensor *out, const hipattn_tensor *input, int kind, void *stream_arg) {
  static const char *names[] = {"silu_and_mul", "gelu_new", "gelu_fast"};
  const char *op = names[kind];
  HA_CHECK(input != nullptr && out != nullptr && input->ndim >= 1 && out->ndim == input->ndim, "%s: rank mismatch", op);
  HA_CHECK(is_float_dtype(input->dtype) && out->dtype == input->dtype, "%s: dtype mismatch", op);
  const int64_t in_w = input->sizes[input->ndim - 1];
  const int64_t d = kind == 0 ? in_w / 2 : in_w;
  HA_CHECK(kind != 0 || in_w % 2 == 0, "%s: input width must be even", op);
  HA_CHECK(out->sizes[out->ndim - 1] == d, "%s: out width %lld, expected %lld", op,
           (long long)out->sizes[out->ndim - 1], (long long)d);
  for (int i = 0; i + 1 < input->ndim; i++)
    HA_CHECK(out->sizes[i] == input->sizes[i], "%s: shape mismatch in dim %d", op, i);
  check_contiguous(input, "input");
  check_contiguous(out, "out");
  const int64_t rows = in_w == 0 ? 0 : numel(input) / in_w;
  if (rows == 0 || d == 0) return;
  check_data(input, "input");
  check_data(out, "out");
  hipStream_t stream = resolve_stream(stream_arg);
  if (kind == 0 && dtype_size(input->dtype) == 2 && d % 8 == 0 && rows <= 65535 &&
      (reinterpret_cast<uintptr_t>(input->data) & 15) == 0 && (reinterpret_cast<uintptr_t>(out->data) & 15) == 0) {
    const dim3 grid((unsigned)((d / 8 + 255) / 256), (unsigned)rows);
    if (input->dtype == HIPATTN_F16)
      silu_and_mul_vec8_kernel<half_t><<<grid, 256, 0, stream>>>(static_cast<half_t *>(out->data),
                                                                 static_cast<const half_t *>(input->data), (int)d);
    else
      silu_and_mul_vec8_kernel<bf16_t><<<grid, 256, 0, stream>>>(static_cast<bf16_t *>(out->data),
                                                                 static_cast<const bf16_t *>(input->data), (int)d);
    check_launch(op);
    return;
  }
  const int threads = round_threads(d, 1024);
#define HA_ACT(TT)                                                                                     \
  if (kind == 0)                                                                                       \
    silu_and_mul_kernel<TT><<<dim3((unsigned)rows), threads, 0, stream>>>(static_cast<TT *>(out->data), \
                                                                          static_cast<const TT *>(input->data), (int)d); \
  else if (kind == 1)                                                                                  \
    activation_kernel<TT, 0><<<dim3((unsigned)rows), threads, 0, stream>>>(static_cast<TT *>(out->data), \
                                                                           static_cast<const TT *>(input->data), (int)d); \
  else                                                                                                 \
    activation_kernel<TT, 1><<<dim3((unsigned)rows), threads, 0, stream>>>(static_cast<TT *>(out->data), \
                                                                           static_cast<const TT *>(input->data), (int)d)
  switch (input->dtype) {
    case HIPATTN_F32: HA_ACT(float); break;
    case HIPATTN_F16: HA_ACT(half_t); break;
    default: HA_ACT(bf16_t); break;
  }
#undef HA_ACT
  check_launch(op);
}

void bias_argmax_impl(const hipattn_tensor *logits, const hipattn_tensor *bias, const hipattn_tensor *mask,
                      const hipattn_tensor *rows, hipattn_tensor *out_tokens, hipattn_tensor *out_logits,
                      void *stream_arg) {
  check_tensor(logits, "logits", 2);
  HA_CHECK(is_float_dtype(logits->dtype), "bias_argmax: logits must be f32/f16/bf16");
  HA_CHECK((bias != nullptr) != (mask != nullptr), "bias_argmax: pass exactly one of bias and mask");
  const int64_t S = logits->sizes[0], V = logits->sizes[1];
  HA_CHECK(V <= 0x7ffffff0, "bias_argmax: vocabulary too large");
  HA_CHECK(V <= 1 || logits->strides[1] == 1, "bias_argmax: logits rows must be contiguous");
  check_tensor(out_tokens, "out_tokens", 1);
  HA_CHECK(out_tokens->dtype == HIPATTN_I32 && out_tokens->sizes[0] == S, "bias_argmax: out_tokens must be int32 [S]");
  check_contiguous(out_tokens, "out_tokens");
  if (out_logits) {
    check_tensor(out_logits, "out_logits", 1);
    HA_CHECK(out_logits->dtype == HIPATTN_F32 && out_logits->sizes[0] == S, "bias_argmax: out_logits must be f32 [S]");
    check_contiguous(out_logits, "out_logits");
  }
  int64_t nrows;
  if (bias) {
    check_tensor(bias, "bias", 2);
    HA_CHECK(bias->dtype == HIPATTN_F32, "bias_argmax: bias must be f32");
    HA_CHECK(bias->sizes[1] >= V, "bias_argmax: bias rows have %lld entries, vocabulary is %lld",
             (long long)bias->sizes[1], (long long)V);
    HA_CHECK(bias->sizes[1] <= 1 || bias->strides[1] == 1, "bias_argmax: bias rows must be contiguous");
    check_data(bias, "bias");
    nrows = bias->sizes[0];
  } else {
    check_tensor(mask, "mask", 2);
    HA_CHECK(mask->dtype == HIPATTN_U8, "bias_argmax: mask must be u8");
    HA_CHECK(mask->sizes[1] <= 1 || mask->strides[1] == 1, "bias_argmax: mask rows must be contiguous");
    check_data(mask, "mask");
    nrows = mask->sizes[0];
  }
  if (rows) {
    check_tensor(rows, "bias_rows", 1);
    HA_CHECK(rows->dtype == HIPATTN_I32 && rows->sizes[0] == S, "bias_argmax: bias_rows must be int32 [S]");
    check_contiguous(rows, "bias_rows");
    check_data(rows, "bias_rows");
  } else {
    HA_CHECK(nrows >= S, "bias_argmax: %lld bias rows for %lld sequences", (long long)nrows, (long long)S);
  }
  if (S == 0) return;
  check_data(logits, "logits");
  check_data(out_tokens, "out_tokens");
  hipStream_t stream = resolve_stream(stream_arg);
  const int threads = round_threads(V, 1024);
  const int32_t *rp = rows ? static_cast<const int32_t *>(rows->data) : nullptr;
  float *ol = out_logits ? static_cast<float *>(out_logits->data) : nullptr;
  // Wide path: 2-byte logits in 16-byte steps, rows cut into slices so that about a thousand workgroups run.
  const bool wide = dtype_size(logits->dtype) == 2 && V % 8 == 0 && V >= 16384 && S <= 65535 &&
                    logits->strides[0] % 8 == 0 && (reinterpret_cast<uintptr_t>(logits->data) & 15) == 0 &&
                    (!bias || (bias->strides[0] % 4 == 0 && (reinterpret_cast<uintptr_t>(bias->data) & 15) == 0));
  if (wide) {
    int64_t chunks = (1024 + S - 1) / S;
    const int64_t max_chunks = V / 4096;
    if (chunks > max_chunks) chunks = max_chunks;
    if (chunks < 1) chunks = 1;
    const int per_slice = (int)((((V + chunks - 1) / chunks) + 7) / 8 * 8);
    chunks = (V + per_slice - 1) / per_slice;
    // The row states are cleared on the stream in front of every launch: a call never depends on what the
    // one before it (or a replay of a captured graph overlapping it on another stream) left behind.
    ArgmaxRowState *st =
        static_cast<ArgmaxRowState *>(library_workspace(WS_BIAS_ARGMAX, (size_t)S * sizeof(ArgmaxRowState), stream));
    argmax_state_clear_kernel<<<dim3((unsigned)((S + 255) / 256)), 256, 0, stream>>>(st, (int)S);
    int32_t *ot = static_cast<int32_t *>(out_tokens->data);
    const dim3 grid((unsigned)chunks, (unsigned)S);
#define HA_BAW(TT)                                                                                               \
  if (bias)                                                                                                     \
    bias_argmax_slice_kernel<TT, 0><<<grid, 256, 0, stream>>>(                                                   \
        static_cast<const TT *>(logits->data), logits->strides[0], static_cast<const float *>(bias->data),      \
        bias->strides[0], nullptr, 0, 0, rp, nrows, (int)V, per_slice, st, ot, ol);                                      \
  else                                                                                                          \
    bias_argmax_slice_kernel<TT, 1><<<grid, 256, 0, stream>>>(                                                   \
        static_cast<const TT *>(logits->data), logits->strides[0], nullptr, 0,                                  \
        static_cast<const uint8_t *>(mask->data), mask->strides[0], mask->sizes[1], rp, nrows, (int)V, per_slice, st, ot, ol)
    if (logits->dtype == HIPATTN_F16) {
      HA_BAW(half_t);
    } else {
      HA_BAW(bf16_t);
    }
#undef HA_BAW
    check_launch("bias_argmax");
    return;
  }
#define HA_BA(TT)                                                                                               \
  if (bias)                                                                                                     \
    bias_argmax_kernel<TT, 0><<<dim3((unsigned)S), threads, 0, stream>>>(                                        \
        static_cast<const TT *>(logits->data), logits->strides[0], static_cast<const float *>(bias->data),      \
        bias->strides[0], nullptr, 0, 0, rp, nrows, (int)V, static_cast<int32_t *>(out_tokens->data), ol);             \
  else                                                                                                          \
    bias_argmax_kernel<TT, 1><<<dim3((unsigned)S), threads, 0, stream>>>(                                        \
        static_cast<const TT *>(logits->data), logits->strides[0], nullptr, 0,                                  \
        static_cast<const uint8_t *>(mask->data), mask->strides[0], mask->sizes[1], rp, nrows, (int)V,                 \
        static_cast<int32_t *>(out_tokens->data), ol)
  switch (logits->dtype) {
    case HIPATTN_F32: HA_BA(float); break;
    case HIPATTN_F16: HA_BA(half_t); break;
    default: HA_BA(bf16_t); break;
  }
#undef HA_BA
  check_launch("bias_argmax");
}

}  // namespace
}  // namespace hipattn

using namespace hipattn;

extern "C" char *hipattn_rotary_embedding(const hipattn_tensor *positions, hipattn_tensor *query,
                                          hipattn_tensor *key, int head_size, const hipattn_tensor *cos_sin_cache,
                                          bool is_neox, void *stream) {
  HA_PROTECT(rotary_impl(positions, query, key, head_size, cos_sin_cache, is_neox, stream));
}

extern "C" char *hipattn_rms_norm(hipattn_tensor *out, const hipattn_tensor *input, const hipattn_tensor *weight,
                                  float epsilon, void *stream) {
  HA_PROTECT(rms_norm_impl(out, const_cast<hipattn_tensor *>(input), nullptr, weight, epsilon, false, stream));
}

extern "C" char *hipattn_fused_add_rms_norm(hipattn_tensor *input, hipattn_tensor *residual,
                                            const hipattn_tensor *weight, float epsilon, void *stream) {
  HA_PROTECT(rms_norm_impl(nullptr, input, residual, weight, epsilon, true, stream));
}

extern "C" char *hipattn_silu_and_mul(hipattn_tensor *out, const hipattn_tensor *input, void *stream) {
  HA_PROTECT(activation_impl(out, input, 0, stream));
}
extern "C" char *hipattn_gelu_new(hipattn_tensor *out, const hipattn_tensor *input, void *stream) {
  HA_PROTECT(activation_impl(out, input, 1, stream));
}
extern "C" char *hipattn_gelu_fast(hipattn_tensor *out, const hipattn_tensor *input, void *stream) {
  HA_PROTECT(activation_impl(out, input, 2, stream));
}

extern "C" char *hipattn_bias_argmax(const hipattn_tensor *logits, const hipattn_tensor *bias,
                                     const hipattn_tensor *mask, const hipattn_tensor *bias_rows,
                                     hipattn_tensor *out_tokens, hipattn_tensor *out_logits, void *stream) {
  HA_PROTECT(bias_argmax_impl(logits, bias, mask, bias_rows, out_tokens, out_logits, stream));
}
