// Row-wise kernels of layers that normalise a sublayer's output before the residual sum:
//
//   group norm    dst[r] (+)= w * x_g / sqrt(mean(x_g^2) + eps) for each of `groups` equal consecutive parts x_g of
//                 the row x = sum_p src[p][row] (* silu(gate[row]) if a gate is given), float32 arithmetic.
//                 One entry point serves the norm of chosen rows into a fresh tensor, the norm of rows where they
//                 lie (dst == src; the rows may be columns of a wider tensor) and the norm that adds into the
//                 float32 residual stream (accumulate); the rows as they then stand can be left in a second tensor of
//                 another type as well (the next sublayer's input).
//   token shift   s_t = h_t + (h_(t-1) - h_t) * mu on the float32 stream, the previous token of a portion's first
//                 token coming from the sequence's state, which receives the portion's last h.
//   sigmoid gate  out = a * sigmoid(g).
//
// A block serves one (row, group) resp. one token; sums run in a fixed order that depends on the row's own
// length only.
#include "common.h"

CWM_DEFINE_ERROR_API

__device__ __forceinline__ float load_as_f32(const void* p, int dtype, size_t i) {
  return dtype == CWM_F32 ? ((const float*)p)[i] : bf16_to_f32(((const bf16_t*)p)[i]);
}

__device__ __forceinline__ void store_from_f32(void* p, int dtype, size_t i, float v) {
  if (dtype == CWM_F32)
    ((float*)p)[i] = v;
  else
    ((bf16_t*)p)[i] = f32_to_bf16(v);
}

__device__ __forceinline__ float silu_f32(float z) { return z / (1.f + expf(-z)); }

#define GN_KEEP 8  // elements of a part that a thread keeps in registers between the two passes

__global__ void __launch_bounds__(256) group_norm_kernel(const void* src, int src_dtype, long src_ld, int n_partials,
                                                         long partial_stride, const void* gate, int gate_dtype,
                                                         long gate_ld, const void* __restrict__ weight, int w_dtype, void* dst,
                                                         int dst_dtype, long dst_ld, const int* __restrict__ rows, int part,
                                                         float eps, int accumulate, void* __restrict__ copy, int copy_dtype, long copy_ld) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const int g = blockIdx.y;
  const size_t row = rows ? (size_t)rows[r] : (size_t)r;
  const size_t s0 = row * src_ld + (size_t)g * part;
  const size_t g0 = row * gate_ld + (size_t)g * part;
  const size_t d0 = (size_t)r * dst_ld + (size_t)g * part;
  float keep[GN_KEEP];
  float ss = 0.f;
  int n = 0;
  for (int i = threadIdx.x; i < part; i += blockDim.x, ++n) {
    float v = 0.f;
    for (int p = 0; p < n_partials; ++p) v += load_as_f32(src, src_dtype, (size_t)p * partial_stride + s0 + i);
    if (gate) v *= silu_f32(load_as_f32(gate, gate_dtype, g0 + i));
    if (n < GN_KEEP) keep[n] = v;
    ss += v * v;
  }
  const float total = block_sum(ss, scratch);
  const float inv = 1.f / sqrtf(total / (float)part + eps);
  n = 0;
  for (int i = threadIdx.x; i < part; i += blockDim.x, ++n) {
    float v;
    if (n < GN_KEEP) {
      v = keep[n];
    } else {
      v = 0.f;
      for (int p = 0; p < n_partials; ++p) v += load_as_f32(src, src_dtype, (size_t)p * partial_stride + s0 + i);
      if (gate) v *= silu_f32(load_as_f32(gate, gate_dtype, g0 + i));
    }
    float y = v * inv * load_as_f32(weight, w_dtype, (size_t)g * part + i);
    if (accumulate) y += load_as_f32(dst, dst_dtype, d0 + i);
    store_from_f32(dst, dst_dtype, d0 + i, y);
    if (copy) store_from_f32(copy, copy_dtype, (size_t)r * copy_ld + (size_t)g * part + i, y);  // what dst now holds, in another type
  }
}

// src: [n_partials][.][src_ld] (rows `rows[r]` or r), dst: [n_rows][dst_ld]; dim = groups * part elements of a row.
extern "C" int cwm_group_norm(const void* src, int src_dtype, long src_ld, int n_partials, long partial_stride, const void* gate,
                              int gate_dtype, long gate_ld, const void* weight, int w_dtype, void* dst, int dst_dtype, long dst_ld,
                              const int* rows, int n_rows, int dim, int groups, float eps, int accumulate, void* copy, int copy_dtype,
                              long copy_ld, hipStream_t stream) {
  CWM_REQUIRE(src && weight && dst, "group_norm: arguments missing");
  CWM_REQUIRE(n_rows >= 0 && dim > 0 && groups > 0 && dim % groups == 0, "group_norm: %d elements do not divide into %d groups", dim, groups);
  CWM_REQUIRE(n_partials >= 1 && src_ld >= dim && dst_ld >= dim && (!gate || gate_ld >= dim), "group_norm: rows shorter than %d", dim);
  CWM_REQUIRE(groups <= 65535, "group_norm: too many groups");
  // a thread re-reads what it has not kept after it has written its own elements only: in place is safe
  if (n_rows == 0) return 0;
  hipLaunchKernelGGL(group_norm_kernel, dim3(n_rows, groups), dim3(256), 0, stream, src, src_dtype, src_ld, n_partials, partial_stride,
                     gate, gate_dtype, gate_ld, weight, w_dtype, dst, dst_dtype, dst_ld, rows, dim / groups, eps, accumulate, copy, copy_dtype, copy_ld);
  return cwm_launch_status("group_norm");
}

__global__ void __launch_bounds__(256) token_shift_kernel(const float* __restrict__ h, const float* __restrict__ mu, float* state,
                                                          const int* __restrict__ slots, const int* __restrict__ cu_q,
                                                          const int* __restrict__ seq_of_token, const int* __restrict__ positions,
                                                          void* __restrict__ out, int out_dtype, int dim, int n_slots, int write_state) {
  const int t = blockIdx.x;
  const int b = seq_of_token[t];
  const int first = cu_q[b];
  const bool head = t == first;
  const int slot = slots[b];
  const bool slot_ok = slot >= 0 && slot < n_slots;
  const bool fresh = positions[t] == 0;
  const size_t last = (size_t)(cu_q[b + 1] - 1) * dim;
  for (int i = threadIdx.x; i < dim; i += blockDim.x) {
    const float x = h[(size_t)t * dim + i];
    float prev;
    if (head) {
      prev = (fresh || !slot_ok) ? 0.f : state[(size_t)slot * dim + i];
      // the block of a portion's first token is the only one that touches the sequence's state: it reads what
      // the step before left and then leaves the portion's last row, element by element in one thread
      if (write_state && slot_ok) state[(size_t)slot * dim + i] = h[last + i];
    } else {
      prev = h[(size_t)(t - 1) * dim + i];
    }
    store_from_f32(out, out_dtype, (size_t)t * dim + i, x + (prev - x) * mu[i]);
  }
}

extern "C" int cwm_token_shift(const float* h, const float* mu, float* state, const int* slots, const int* cu_q,
                               const int* seq_of_token, const int* positions, void* out, int out_dtype, int n_tokens, int dim,
                               int n_slots, int write_state, hipStream_t stream) {
  CWM_REQUIRE(h && mu && state && slots && cu_q && seq_of_token && positions && out, "token_shift: arguments missing");
  CWM_REQUIRE(n_tokens >= 0 && dim > 0 && n_slots > 0, "token_shift: bad sizes");
  if (n_tokens == 0) return 0;
  hipLaunchKernelGGL(token_shift_kernel, dim3(n_tokens), dim3(256), 0, stream, h, mu, state, slots, cu_q, seq_of_token, positions, out,
                     out_dtype, dim, n_slots, write_state);
  return cwm_launch_status("token_shift");
}

__global__ void __launch_bounds__(256) sigmoid_mul_kernel(const void* __restrict__ a, long a_ld, const void* __restrict__ g, long g_ld,
                                                          void* __restrict__ out, long out_ld, int dtype, int width) {
  const size_t t = blockIdx.x;
  for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < width; i += gridDim.y * blockDim.x) {
    const float z = load_as_f32(g, dtype, t * g_ld + i);
    store_from_f32(out, dtype, t * out_ld + i, load_as_f32(a, dtype, t * a_ld + i) / (1.f + expf(-z)));
  }
}

extern "C" int cwm_sigmoid_mul(const void* a, long a_ld, const void* g, long g_ld, void* out, long out_ld, int dtype, int n_rows,
                               int width, hipStream_t stream) {
  CWM_REQUIRE(a && g && out && n_rows >= 0 && width > 0, "sigmoid_mul: bad arguments");
  if (n_rows == 0) return 0;
  int gy = (width + 1023) / 1024;
  hipLaunchKernelGGL(sigmoid_mul_kernel, dim3(n_rows, gy), dim3(256), 0, stream, a, a_ld, g, g_ld, out, out_ld, dtype, width);
  return cwm_launch_status("sigmoid_mul");
}

// out[r][0..width) = src[r][0..width) for rows of `src_ld` and `out_ld` elements of 2 or 4 bytes (columns of one
// tensor into columns of another).
template <typename T>
__global__ void __launch_bounds__(256) copy_columns_kernel(const T* __restrict__ src, long src_ld, T* __restrict__ out, long out_ld, int width) {
  const size_t r = blockIdx.x;
  for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < width; i += gridDim.y * blockDim.x) out[r * out_ld + i] = src[r * src_ld + i];
}

extern "C" int cwm_copy_columns(const void* src, long src_ld, void* out, long out_ld, int dtype, long n_rows, int width, hipStream_t stream) {
  CWM_REQUIRE(src && out && n_rows >= 0 && width > 0 && n_rows <= 2147483647L, "copy_columns: bad arguments");
  if (n_rows == 0) return 0;
  dim3 grid((unsigned)n_rows, (width + 1023) / 1024);
  if (dtype == CWM_BF16)
    hipLaunchKernelGGL(copy_columns_kernel<bf16_t>, grid, dim3(256), 0, stream, (const bf16_t*)src, src_ld, (bf16_t*)out, out_ld, width);
  else
    hipLaunchKernelGGL(copy_columns_kernel<float>, grid, dim3(256), 0, stream, (const float*)src, src_ld, (float*)out, out_ld, width);
  return cwm_launch_status("copy_columns");
}
