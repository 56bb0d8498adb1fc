// A residual kept as several streams (hyper-connections): a token's row of the residual is S vectors
// x_0 .. x_(S-1) of D float32 values, [T][S][D].
//
// A sublayer reads u = sum_s a[s] x_s, normalised; its result y then changes all streams at once,
//   x_t <- sum_s M[s][t] x_s + b[t] y          (M indexed [from][to]).
// The kernel below does the pending change of the sublayer before (if there is one) and the read of the
// next sublayer in one pass over the row, as the norm of a single residual adds the pending update and
// normalises:
//   x   <- M^T x + b y                         written back unless only chosen rows are read
//   out  = u / sqrt(mean(u^2) + eps) * w,      u = sum_t a[t] x_t
// all in float32, every sum in the order of the stream index; y may be float32 partial sums [P][T][D] of
// a product whose K was split, added in order first.  S = 1 with M = b = a = 1 is the single residual.
// One block a row; u is kept in LDS between the two passes over the row.
#include "common.h"

CWM_DEFINE_ERROR_API

#define STREAMS_MAX 8

extern "C" int cwm_streams_max() { return STREAMS_MAX; }

// four consecutive elements
template <typename T> struct Four;
template <> struct Four<float> {
  static __device__ __forceinline__ void add(const float* p, float (&v)[4]) {
    const float4 x = *(const float4*)p;
    v[0] += x.x, v[1] += x.y, v[2] += x.z, v[3] += x.w;
  }
  static __device__ __forceinline__ void store(float* p, const float (&v)[4]) { *(float4*)p = make_float4(v[0], v[1], v[2], v[3]); }
};
template <> struct Four<bf16_t> {
  static __device__ __forceinline__ void add(const bf16_t* p, float (&v)[4]) {
    const uint2 x = *(const uint2*)p;
    v[0] += __uint_as_float(x.x << 16), v[1] += __uint_as_float(x.x & 0xffff0000u);
    v[2] += __uint_as_float(x.y << 16), v[3] += __uint_as_float(x.y & 0xffff0000u);
  }
  static __device__ __forceinline__ void store(bf16_t* p, const float (&v)[4]) {
    uint2 x;
    x.x = pack2_bf16(v[0], v[1]);
    x.y = pack2_bf16(v[2], v[3]);
    *(uint2*)p = x;
  }
};

// W: elements a thread takes at a time (4 where the row's length is a multiple of 4 and every row starts at a
// multiple of 16 bytes, else 1).  A row's sum of squares is added up in the same order for every W.
template <typename TY, typename TO, int S, int W>
__global__ void stream_mix_norm_kernel(float* __restrict__ x, const TY* __restrict__ y, int n_partials, long partial_stride,
                                       const float* __restrict__ mix, const float* __restrict__ out_coef,
                                       const float* __restrict__ in_coef, const float* __restrict__ weight,
                                       TO* __restrict__ out, const int* __restrict__ rows, int dim, float eps,
                                       const int* __restrict__ pair_row, const float* __restrict__ pair_weight, int top) {
  extern __shared__ __attribute__((aligned(16))) float u_row[];  // [dim], then 16 floats of scratch
  float* scratch = u_row + dim;
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  float* xrow = x + (size_t)src * S * dim;
  // with pair_row, y holds rows of which the token's result is a weighted sum: sum_k pair_weight[t][k] * y[pair_row[t][k]]
  const TY* yrow = y ? (pair_row ? y : y + (size_t)src * dim) : nullptr;
  const bool write_back = (y != nullptr) && (rows == nullptr);
  float m[S][S], b[S], a[S];
#pragma unroll
  for (int s = 0; s < S; ++s) {
    a[s] = in_coef ? in_coef[s] : 1.f;
    b[s] = out_coef ? out_coef[s] : 1.f;
#pragma unroll
    for (int t = 0; t < S; ++t) m[s][t] = mix ? mix[s * S + t] : (s == t ? 1.f : 0.f);
  }
  float ss = 0.f;
  for (int i = W * threadIdx.x; i < dim; i += W * blockDim.x) {
    float xs[S][W];
#pragma unroll
    for (int s = 0; s < S; ++s) {
      if constexpr (W == 4) {
        const float4 v = *(const float4*)(xrow + (size_t)s * dim + i);
        xs[s][0] = v.x, xs[s][1] = v.y, xs[s][2] = v.z, xs[s][3] = v.w;
      } else {
        xs[s][0] = xrow[(size_t)s * dim + i];
      }
    }
    float u[W];
#pragma unroll
    for (int e = 0; e < W; ++e) u[e] = 0.f;
    if (yrow) {
      float yv[W];
#pragma unroll
      for (int e = 0; e < W; ++e) yv[e] = 0.f;
      if (pair_row) {
        for (int k = 0; k < top; ++k) {  // in the order of the token's choices, as the kernel that only adds them up does
          const int row = pair_row[(size_t)src * top + k];
          if (row < 0) continue;
          const float wk = pair_weight[(size_t)src * top + k];
          float part[W];
#pragma unroll
          for (int e = 0; e < W; ++e) part[e] = 0.f;
          if constexpr (W == 4)
            Four<TY>::add(yrow + (size_t)row * dim + i, (float(&)[4])part);
          else
            part[0] = Elem<TY>::load(yrow + (size_t)row * dim + i);
#pragma unroll
          for (int e = 0; e < W; ++e) yv[e] += wk * part[e];
        }
      } else {
        for (int p = 0; p < n_partials; ++p) {
          if constexpr (W == 4)
            Four<TY>::add(yrow + (size_t)p * partial_stride + i, (float(&)[4])yv);
          else
            yv[0] += Elem<TY>::load(yrow + (size_t)p * partial_stride + i);
        }
      }
#pragma unroll
      for (int t = 0; t < S; ++t) {
        float v[W];
#pragma unroll
        for (int e = 0; e < W; ++e) {
          v[e] = 0.f;
#pragma unroll
          for (int s = 0; s < S; ++s) v[e] += m[s][t] * xs[s][e];
          v[e] += b[t] * yv[e];
          u[e] += a[t] * v[e];
        }
        if (write_back) {
          if constexpr (W == 4)
            *(float4*)(xrow + (size_t)t * dim + i) = make_float4(v[0], v[1], v[2], v[3]);
          else
            xrow[(size_t)t * dim + i] = v[0];
        }
      }
    } else {
#pragma unroll
      for (int t = 0; t < S; ++t)
#pragma unroll
        for (int e = 0; e < W; ++e) u[e] += a[t] * xs[t][e];
    }
#pragma unroll
    for (int e = 0; e < W; ++e) u_row[i + e] = u[e];
  }
  __syncthreads();
  // the sum of squares in one order whatever W was: thread j adds the elements j, j + threads, ...
  for (int i = threadIdx.x; i < dim; i += blockDim.x) ss += u_row[i] * u_row[i];
  ss = block_sum(ss, scratch);
  const float rstd = 1.0f / sqrtf(ss / (float)dim + eps);
  TO* orow = out + (size_t)r * dim;
  if constexpr (W == 4) {
    for (int i = 4 * threadIdx.x; i < dim; i += 4 * blockDim.x) {
      const float4 uu = *(const float4*)(u_row + i), ww = *(const float4*)(weight + i);
      const float o[4] = {uu.x * rstd * ww.x, uu.y * rstd * ww.y, uu.z * rstd * ww.z, uu.w * rstd * ww.w};
      Four<TO>::store(orow + i, o);
    }
  } else {
    for (int i = threadIdx.x; i < dim; i += blockDim.x) Elem<TO>::store(orow + i, u_row[i] * rstd * weight[i]);
  }
}

template <typename TY, typename TO>
static int launch_stream_mix_norm(bool vec, int streams, int n_out, int threads, size_t lds, hipStream_t stream, float* x, const void* y,
                                  int n_partials, long partial_stride, const float* mix, const float* out_coef,
                                  const float* in_coef, const float* weight, void* out, const int* rows, int dim, float eps,
                                  const int* pair_row, const float* pair_weight, int top) {
#define CWM_STREAMS_CASE(S)                                                                                                  \
  case S:                                                                                                                   \
    if (vec)                                                                                                                \
      hipLaunchKernelGGL((stream_mix_norm_kernel<TY, TO, S, 4>), dim3(n_out), dim3(threads), lds, stream, x, (const TY*)y,   \
                         n_partials, partial_stride, mix, out_coef, in_coef, weight, (TO*)out, rows, dim, eps, pair_row,     \
                         pair_weight, top);                                                                                  \
    else                                                                                                                    \
      hipLaunchKernelGGL((stream_mix_norm_kernel<TY, TO, S, 1>), dim3(n_out), dim3(threads), lds, stream, x, (const TY*)y,   \
                         n_partials, partial_stride, mix, out_coef, in_coef, weight, (TO*)out, rows, dim, eps, pair_row,     \
                         pair_weight, top);                                                                                  \
    break
  switch (streams) {
    CWM_STREAMS_CASE(1);
    CWM_STREAMS_CASE(2);
    CWM_STREAMS_CASE(3);
    CWM_STREAMS_CASE(4);
    CWM_STREAMS_CASE(5);
    CWM_STREAMS_CASE(6);
    CWM_STREAMS_CASE(7);
    CWM_STREAMS_CASE(8);
    default:
      return cwm_fail("stream_mix_norm: %d streams, the kernel takes 1..%d", streams, STREAMS_MAX);
  }
#undef CWM_STREAMS_CASE
  return 0;
}

// x: float32 [n_tokens][streams][dim].  y: null (nothing pending), or [n_tokens][dim] of type y_dtype, or n_partials
// float32 slabs partial_stride apart.  mix [streams * streams], out_coef [streams], in_coef [streams]: float32, null
// for the identity / ones.  weight: float32 [dim].  rows: null, or n_out indices of the rows to read (x then stays
// as it is; what is normalised is still the row after the pending change).  pair_row (int32 [n_tokens][top], -1: none)
// and pair_weight (float32 [n_tokens][top]): y is then float32 [any][dim] and token t's pending result is
// sum_k pair_weight[t][k] * y[pair_row[t][k]], added in the order of k (the weighted sum of a token's experts).
extern "C" int cwm_stream_mix_norm(void* x, int streams, const void* y, int y_dtype, int n_partials, long partial_stride,
                                   const float* mix, const float* out_coef, const float* in_coef, const float* weight,
                                   void* out, int out_dtype, const int* rows, int n_out, int dim, float eps,
                                   const int* pair_row, const float* pair_weight, int top, hipStream_t stream) {
  CWM_REQUIRE(n_out >= 0 && dim > 0, "stream_mix_norm: bad sizes rows=%d D=%d", n_out, dim);
  CWM_REQUIRE(streams >= 1 && streams <= STREAMS_MAX, "stream_mix_norm: %d streams, the kernel takes 1..%d", streams, STREAMS_MAX);
  CWM_REQUIRE(n_partials >= 1 && (n_partials == 1 || y_dtype == CWM_F32), "stream_mix_norm: partial sums must be float32");
  CWM_REQUIRE(eps > 0.f, "stream_mix_norm: eps must be positive");
  CWM_REQUIRE(x && weight && out, "stream_mix_norm: arguments missing");
  CWM_REQUIRE(!pair_row || (y && pair_weight && top >= 1 && y_dtype == CWM_F32 && n_partials == 1),
              "stream_mix_norm: a weighted sum of rows needs float32 rows, weights and the number of rows a token");
  CWM_REQUIRE(dim <= 15360, "stream_mix_norm: rows of %d elements do not fit the block's LDS", dim);
  if (n_out == 0) return 0;
  if (!y) y_dtype = CWM_F32;
  const bool vec = dim % 4 == 0 && partial_stride % 4 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)y % 16) == 0 &&
                   ((uintptr_t)weight % 16) == 0 && ((uintptr_t)out % 16) == 0;
  const int threads = dim >= 4096 ? 512 : (dim >= 512 ? 256 : (dim >= 128 ? 128 : 64));
  const size_t lds = ((size_t)dim + 16) * sizeof(float);
  int status;
  const int key = (y_dtype << 1) | out_dtype;
  switch (key) {
    case 0: status = launch_stream_mix_norm<float, float>(vec, streams, n_out, threads, lds, stream, (float*)x, y, n_partials, partial_stride, mix, out_coef, in_coef, weight, out, rows, dim, eps, pair_row, pair_weight, top); break;
    case 1: status = launch_stream_mix_norm<float, bf16_t>(vec, streams, n_out, threads, lds, stream, (float*)x, y, n_partials, partial_stride, mix, out_coef, in_coef, weight, out, rows, dim, eps, pair_row, pair_weight, top); break;
    case 2: status = launch_stream_mix_norm<bf16_t, float>(vec, streams, n_out, threads, lds, stream, (float*)x, y, n_partials, partial_stride, mix, out_coef, in_coef, weight, out, rows, dim, eps, pair_row, pair_weight, top); break;
    case 3: status = launch_stream_mix_norm<bf16_t, bf16_t>(vec, streams, n_out, threads, lds, stream, (float*)x, y, n_partials, partial_stride, mix, out_coef, in_coef, weight, out, rows, dim, eps, pair_row, pair_weight, top); break;
    default: return cwm_fail("stream_mix_norm: unknown dtypes y=%d out=%d", y_dtype, out_dtype);
  }
  if (status) return status;
  return cwm_launch_status("stream_mix_norm");
}

// out[t][s][:] = scale * table[tokens[t]][:] for every stream s: the embedding's row as the start of all streams.
template <typename TW>
__global__ void embedding_streams_kernel(float* __restrict__ out, const TW* __restrict__ table, const int* __restrict__ tokens,
                                         int dim, int vocab, int streams, float scale) {
  const int t = blockIdx.x;
  const int token = tokens[t];
  const bool known = token >= 0 && token < vocab;
  const TW* row = table + (size_t)(known ? token : 0) * dim;
  for (int i = threadIdx.x; i < dim; i += blockDim.x) {
    const float v = known ? Elem<TW>::load(row + i) * scale : __uint_as_float(0x7fc00000u);
    for (int s = 0; s < streams; ++s) out[((size_t)t * streams + s) * dim + i] = v;
  }
}

extern "C" int cwm_embedding_streams(void* out, const void* table, int table_dtype, const int* tokens, int n_tokens, int dim,
                                     int vocab, int streams, float scale, hipStream_t stream) {
  CWM_REQUIRE(n_tokens >= 0 && dim > 0 && vocab > 0 && streams >= 1, "embedding_streams: bad sizes");
  if (n_tokens == 0) return 0;
  const int threads = dim >= 512 ? 256 : (dim >= 128 ? 128 : 64);
  if (table_dtype == CWM_F32)
    hipLaunchKernelGGL(embedding_streams_kernel<float>, dim3(n_tokens), dim3(threads), 0, stream, (float*)out, (const float*)table,
                       tokens, dim, vocab, streams, scale);
  else if (table_dtype == CWM_BF16)
    hipLaunchKernelGGL(embedding_streams_kernel<bf16_t>, dim3(n_tokens), dim3(threads), 0, stream, (float*)out, (const bf16_t*)table,
                       tokens, dim, vocab, streams, scale);
  else
    return cwm_fail("embedding_streams: unknown dtype %d", table_dtype);
  return cwm_launch_status("embedding_streams");
}
