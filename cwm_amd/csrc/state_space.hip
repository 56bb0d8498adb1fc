// The two sequential pieces of a selective state-space mixer, each going on from a per-request state.
//
//   causal convolution + SiLU, per channel c of a token t at place j of its sequence:
//       out[t][c] = silu(bias[c] + sum_k w[c][k] * in[j - (taps - 1 - k)][c]),   inputs before the sequence's start are 0;
//     a portion's first taps - 1 tokens read the inputs that the step before left in the state (oldest first),
//     and the portion leaves its own last taps - 1 inputs there.
//   the recurrence, per head h (group g = h / (heads / groups)), state S [N][P] in float32:
//       dt = softplus(dt_raw + dt_bias[h]);  a = exp(-exp(A_log[h]) * dt)
//       S <- a S + dt B_t x_t^T;   y_t = S^T C_t + D[h] x_t
//     with x_t [P], B_t and C_t [N] from the convolution's output row [x: heads * P | B: groups * N | C: groups * N].
//
// Both are exact under any cut of a sequence into portions: a portion starts from the state as the previous one
// left it and performs the same operations in the same order as the whole sequence would.
#include "common.h"

CWM_DEFINE_ERROR_API

#define CONV_MAX_TAPS 8
#define SCAN_ROWS 16  // rows of the state that one thread holds

extern "C" int cwm_conv_max_taps() { return CONV_MAX_TAPS; }
extern "C" int cwm_scan_max_state() { return SCAN_ROWS * 16; }

__device__ __forceinline__ float silu_f32(float z) { return z / (1.f + expf(-z)); }

// The block of a sequence's first token in this step computes the first taps - 1 tokens of the portion (all that
// read the state) and then writes the new state, so reads and writes of one sequence's state stay in one thread
// per channel.  Blocks of the other tokens read inputs of this step only.
template <typename T>
__global__ void __launch_bounds__(256) conv_silu_kernel(const T* __restrict__ in, long in_ld, const float* __restrict__ w,
                                                        const float* __restrict__ bias, float* state, long state_ld, long state_off,
                                                        const int* __restrict__ slots, const int* __restrict__ cu_q,
                                                        const int* __restrict__ seq_of_token, T* __restrict__ out, int channels,
                                                        int taps, int n_slots) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int t = blockIdx.x;
  const int b = seq_of_token[t];
  const int first = cu_q[b];
  const int j = t - first;
  const int q = cu_q[b + 1] - first;
  const int hist = taps - 1;
  float wk[CONV_MAX_TAPS];
#pragma unroll
  for (int k = 0; k < CONV_MAX_TAPS; ++k) wk[k] = k < taps ? w[(size_t)c * taps + k] : 0.f;
  const float bc = bias[c];
  if (j >= hist) {
    float acc = bc;
#pragma unroll
    for (int k = 0; k < CONV_MAX_TAPS; ++k)
      if (k < taps) acc += wk[k] * Elem<T>::load(in + (size_t)(t - (hist - k)) * in_ld + c);
    Elem<T>::store(out + (size_t)t * channels + c, silu_f32(acc));
    return;
  }
  if (j != 0) return;
  const int slot = slots[b];
  float* st = (slot >= 0 && slot < n_slots) ? state + (size_t)slot * state_ld + state_off : nullptr;
  float old[CONV_MAX_TAPS];  // old[m]: the input m places after the oldest one kept, m < hist
#pragma unroll
  for (int m = 0; m < CONV_MAX_TAPS; ++m) old[m] = (st && m < hist) ? st[(size_t)m * channels + c] : 0.f;
  // input at place i of the sequence as this step sees it: i < 0 lies in the state
  auto input = [&](int i) -> float {
    if (i >= 0) return Elem<T>::load(in + (size_t)(first + i) * in_ld + c);
    float v = 0.f;
#pragma unroll
    for (int m = 0; m < CONV_MAX_TAPS; ++m)
      if (m == hist + i) v = old[m];
    return v;
  };
  const int n_head = q < hist ? q : hist;
  for (int jj = 0; jj < n_head; ++jj) {
    float acc = bc;
#pragma unroll
    for (int k = 0; k < CONV_MAX_TAPS; ++k)
      if (k < taps) acc += wk[k] * input(jj - (hist - k));
    Elem<T>::store(out + (size_t)(first + jj) * channels + c, silu_f32(acc));
  }
  if (st) {
    float fresh[CONV_MAX_TAPS];
#pragma unroll
    for (int m = 0; m < CONV_MAX_TAPS; ++m) fresh[m] = m < hist ? input(q - hist + m) : 0.f;
#pragma unroll
    for (int m = 0; m < CONV_MAX_TAPS; ++m)
      if (m < hist) st[(size_t)m * channels + c] = fresh[m];
  }
}

extern "C" int cwm_conv_silu(const void* in, long in_ld, int dtype, const float* w, const float* bias, float* state, long state_ld,
                             long state_off, const int* slots, const int* cu_q, const int* seq_of_token, void* out, int n_tokens,
                             int channels, int taps, int n_slots, hipStream_t stream) {
  CWM_REQUIRE(in && w && bias && state && slots && cu_q && seq_of_token && out, "conv_silu: arguments missing");
  CWM_REQUIRE(taps >= 1 && taps <= CONV_MAX_TAPS, "conv_silu: %d taps, the kernel takes 1..%d", taps, CONV_MAX_TAPS);
  CWM_REQUIRE(channels > 0 && in_ld >= channels && n_tokens >= 0, "conv_silu: bad sizes");
  CWM_REQUIRE(state_off >= 0 && state_off + (long)(taps - 1) * channels <= state_ld, "conv_silu: the state row is too short");
  if (n_tokens == 0) return 0;
  dim3 grid(n_tokens, (channels + 255) / 256);
  if (dtype == CWM_BF16)
    hipLaunchKernelGGL(conv_silu_kernel<bf16_t>, grid, dim3(256), 0, stream, (const bf16_t*)in, in_ld, w, bias, state, state_ld, state_off,
                       slots, cu_q, seq_of_token, (bf16_t*)out, channels, taps, n_slots);
  else if (dtype == CWM_F32)
    hipLaunchKernelGGL(conv_silu_kernel<float>, grid, dim3(256), 0, stream, (const float*)in, in_ld, w, bias, state, state_ld, state_off,
                       slots, cu_q, seq_of_token, (float*)out, channels, taps, n_slots);
  else
    return cwm_fail("conv_silu: unknown dtype %d", dtype);
  return cwm_launch_status("conv_silu");
}

// One block per (tile of P, head, sequence).  Thread (p, s) holds 16 rows of column p of the head's state: with
// `split` lanes a column (a power of two, adjacent in a wavefront), lane s has rows 4 (s + q split) + j, q, j < 4,
// so that its B and C values are four 16-byte pieces of LDS.  The block walks the sequence's tokens of this step in
// order, SCAN_TC at a time: while it computes on one chunk from LDS (B, C and the tile's x as float32, the step
// sizes and decays computed once a token), the next chunk's values are already on their way into registers.  The
// split lanes add their parts of y_t[p] by shuffles in a fixed order.  The state is read once before and written
// once after the walk; what a token's result is made of, and in which order, does not depend on how the
// sequence is cut into steps.
#define SCAN_TC 16  // tokens of a chunk
#define SCAN_PF 36  // most values of a chunk that one thread fetches

template <typename T>
__global__ void __launch_bounds__(256) selective_scan_kernel(const T* __restrict__ xbc, long xbc_ld, const T* __restrict__ dt_raw,
                                                             long dt_ld, const float* __restrict__ dt_bias,
                                                             const float* __restrict__ a_log, const float* __restrict__ d_skip,
                                                             float* state, long state_ld, const int* __restrict__ slots,
                                                             const int* __restrict__ cu_q, float* __restrict__ y, int heads, int P,
                                                             int N, int groups, int split, int n_slots) {
  extern __shared__ float lds[];
  const int h = blockIdx.y;
  const int b = blockIdx.z;
  const int cols = blockDim.x / split;
  const int s = threadIdx.x % split;
  const int col = threadIdx.x / split;
  const int p0 = blockIdx.x * cols;
  const int p = p0 + col;
  const bool live = p < P;
  const int g = h / (heads / groups);
  const int inner = heads * P;
  const int NB = SCAN_ROWS * split;      // rows of B (and of C) in LDS, zeros from N on
  const int row = 2 * NB + cols;         // a token's values in LDS: B, C, the tile's x
  float* dtv = lds + SCAN_TC * row;      // the chunk's step sizes
  float* av = dtv + SCAN_TC;             // and decays
  const int slot = slots[b];
  float* st = (slot >= 0 && slot < n_slots) ? state + (size_t)slot * state_ld + (size_t)h * N * P : nullptr;
  float S[SCAN_ROWS];
#pragma unroll
  for (int i = 0; i < SCAN_ROWS; ++i) {
    const int n = 4 * (s + (i >> 2) * split) + (i & 3);
    S[i] = (st && live && n < N) ? st[(size_t)n * P + p] : 0.f;
  }
  const float bias = dt_bias[h];
  const float rate = -expf(a_log[h]);
  const float skip = d_skip[h];
  const int t0 = cu_q[b], t1 = cu_q[b + 1];
  const int total = SCAN_TC * row;

  float pf[SCAN_PF];
  float pf_dt = 0.f, pf_a = 0.f;
  auto fetch = [&](int start) {  // the chunk that starts at token `start`, into registers
#pragma unroll
    for (int k = 0; k < SCAN_PF; ++k) {
      const int idx = threadIdx.x + k * 256;
      float v = 0.f;
      if (idx < total) {
        const int tc = idx / row, e = idx - tc * row;
        const int t = start + tc;
        if (t < t1) {
          const T* src = xbc + (size_t)t * xbc_ld;
          if (e < NB) {
            if (e < N) v = Elem<T>::load(src + inner + (size_t)g * N + e);
          } else if (e < 2 * NB) {
            if (e - NB < N) v = Elem<T>::load(src + inner + (size_t)(groups + g) * N + (e - NB));
          } else if (p0 + e - 2 * NB < P) {
            v = Elem<T>::load(src + (size_t)h * P + p0 + (e - 2 * NB));
          }
        }
      }
      pf[k] = v;
    }
    if (threadIdx.x < SCAN_TC) {
      const int t = start + threadIdx.x;
      if (t < t1) {
        const float z = Elem<T>::load(dt_raw + (size_t)t * dt_ld + h) + bias;
        pf_dt = z > 20.f ? z : log1pf(expf(z));
        pf_a = expf(rate * pf_dt);
      }
    }
  };
  auto stage = [&]() {  // registers -> LDS
#pragma unroll
    for (int k = 0; k < SCAN_PF; ++k) {
      const int idx = threadIdx.x + k * 256;
      if (idx < total) lds[idx] = pf[k];
    }
    if (threadIdx.x < SCAN_TC) {
      dtv[threadIdx.x] = pf_dt;
      av[threadIdx.x] = pf_a;
    }
  };

  fetch(t0);
  stage();
  __syncthreads();
  for (int start = t0; start < t1; start += SCAN_TC) {
    const bool more = start + SCAN_TC < t1;
    if (more) fetch(start + SCAN_TC);
    const int n_here = min(SCAN_TC, t1 - start);
    for (int tc = 0; tc < n_here; ++tc) {
      const float* tok = lds + tc * row;
      const float dt = dtv[tc], a = av[tc];
      const float x = tok[2 * NB + col];
      const float dx = dt * x;
      float acc = 0.f;
#pragma unroll
      for (int q = 0; q < SCAN_ROWS / 4; ++q) {
        const float4 Bq = *(const float4*)(tok + 4 * (s + q * split));
        const float4 Cq = *(const float4*)(tok + NB + 4 * (s + q * split));
        S[4 * q + 0] = a * S[4 * q + 0] + Bq.x * dx;
        S[4 * q + 1] = a * S[4 * q + 1] + Bq.y * dx;
        S[4 * q + 2] = a * S[4 * q + 2] + Bq.z * dx;
        S[4 * q + 3] = a * S[4 * q + 3] + Bq.w * dx;
        acc += S[4 * q + 0] * Cq.x;
        acc += S[4 * q + 1] * Cq.y;
        acc += S[4 * q + 2] * Cq.z;
        acc += S[4 * q + 3] * Cq.w;
      }
      for (int off = 1; off < split; off <<= 1) acc += __shfl_xor(acc, off, CWM_WAVE);
      if (live && s == 0) y[(size_t)(start + tc) * inner + (size_t)h * P + p] = acc + skip * x;
    }
    __syncthreads();
    if (more) {
      stage();
      __syncthreads();
    }
  }
  if (st && live) {
#pragma unroll
    for (int i = 0; i < SCAN_ROWS; ++i) {
      const int n = 4 * (s + (i >> 2) * split) + (i & 3);
      if (n < N) st[(size_t)n * P + p] = S[i];
    }
  }
}

extern "C" int cwm_selective_scan(const void* xbc, long xbc_ld, const void* dt_raw, long dt_ld, int dtype, const float* dt_bias,
                                  const float* a_log, const float* d_skip, float* state, long state_ld, const int* slots,
                                  const int* cu_q, float* y, int n_tokens, int n_seqs, int heads, int P, int N, int groups, int n_slots,
                                  hipStream_t stream) {
  CWM_REQUIRE(xbc && dt_raw && dt_bias && a_log && d_skip && state && slots && cu_q && y, "selective_scan: arguments missing");
  CWM_REQUIRE(heads > 0 && P > 0 && N > 0 && groups > 0 && heads % groups == 0, "selective_scan: bad sizes");
  CWM_REQUIRE(N <= SCAN_ROWS * 16, "selective_scan: a state of %d rows, the kernel takes up to %d", N, SCAN_ROWS * 16);
  CWM_REQUIRE(xbc_ld >= (long)heads * P + 2L * groups * N && dt_ld >= heads, "selective_scan: rows too short");
  CWM_REQUIRE((long)heads * N * P <= state_ld, "selective_scan: the state row is too short");
  CWM_REQUIRE(heads <= 65535 && n_seqs <= 65535, "selective_scan: too many heads or sequences for one launch");
  if (n_tokens == 0 || n_seqs == 0) return 0;
  int split = 1;
  while (split * SCAN_ROWS < N) split <<= 1;  // 1, 2, 4, 8 or 16 lanes a column
  const int cols = 256 / split;
  dim3 grid((P + cols - 1) / cols, heads, n_seqs);
  const int row = 2 * SCAN_ROWS * split + cols;
  const size_t lds_bytes = (size_t)(SCAN_TC * row + 2 * SCAN_TC) * sizeof(float);
  CWM_REQUIRE(SCAN_TC * row <= SCAN_PF * 256, "selective_scan: a chunk of %d values is more than the threads fetch", SCAN_TC * row);
  if (dtype == CWM_BF16)
    hipLaunchKernelGGL(selective_scan_kernel<bf16_t>, grid, dim3(256), lds_bytes, stream, (const bf16_t*)xbc, xbc_ld, (const bf16_t*)dt_raw, dt_ld,
                       dt_bias, a_log, d_skip, state, state_ld, slots, cu_q, y, heads, P, N, groups, split, n_slots);
  else if (dtype == CWM_F32)
    hipLaunchKernelGGL(selective_scan_kernel<float>, grid, dim3(256), lds_bytes, stream, (const float*)xbc, xbc_ld, (const float*)dt_raw, dt_ld,
                       dt_bias, a_log, d_skip, state, state_ld, slots, cu_q, y, heads, P, N, groups, split, n_slots);
  else
    return cwm_fail("selective_scan: unknown dtype %d", dtype);
  return cwm_launch_status("selective_scan");
}
