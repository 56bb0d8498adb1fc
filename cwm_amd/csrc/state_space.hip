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
//     A head's state lies in memory in the order its threads hold it (see the kernel), padded to 16 * split rows.
//
// Both are exact under any cut of a sequence into portions: a portion starts from the state as the previous one
// left it and performs the same operations in the same order as the whole sequence would.
#include "common.h"
#include <type_traits>

CWM_DEFINE_ERROR_API

#define CONV_MAX_TAPS 8
#define SCAN_ROWS 16  // rows of the state that one thread holds

extern "C" int cwm_conv_max_taps() { return CONV_MAX_TAPS; }
extern "C" int cwm_scan_max_state() { return SCAN_ROWS * 16; }
// lanes that share a column of a head's state of N rows: 1, 2, 4, 8 or 16; the head's state takes SCAN_ROWS * split * P floats
extern "C" int cwm_scan_split(int N) {
  int split = 1;
  while (split * SCAN_ROWS < N) split <<= 1;
  return split;
}

__device__ __forceinline__ float silu_f32(float z) { return z / (1.f + expf(-z)); }

// The block of a sequence's first token in this step computes the first taps - 1 tokens of the portion (all that
// read the state) and then writes the new state, so reads and writes of one sequence's state stay in one thread
// per channel.  Blocks of the other tokens read inputs of this step only.
template <typename T>
__global__ void __launch_bounds__(256) conv_silu_kernel(const T* __restrict__ in, long in_ld, const float* __restrict__ w,
                                                        const float* __restrict__ bias, float* state, long state_ld, long state_off,
                                                        const int* __restrict__ slots, const int* __restrict__ cu_q,
                                                        const int* __restrict__ seq_of_token, T* __restrict__ out, int channels,
                                                        int taps, int n_slots, int by_sequence) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  // a block a token; or (by_sequence) a block a sequence, for its first tokens and its state alone, the other
  // tokens being the other kernel's
  const int b = by_sequence ? blockIdx.x : seq_of_token[blockIdx.x];
  const int t = by_sequence ? cu_q[b] : blockIdx.x;
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
      if (k < taps) acc = fmaf(wk[k], Elem<T>::load(in + (size_t)(t - (hist - k)) * in_ld + c), acc);
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
      if (k < taps) acc = fmaf(wk[k], input(jj - (hist - k)), acc);
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

// The tokens that read no state (place >= taps - 1 in their portion), bfloat16, eight channels a thread: a tap's eight
// inputs are one load of 16 bytes.  The sums run in the order of the kernel above.
__global__ void __launch_bounds__(256) conv_silu_body_kernel(const bf16_t* __restrict__ in, long in_ld, const float* __restrict__ w_by_tap,
                                                             const float* __restrict__ bias, const int* __restrict__ cu_q,
                                                             const int* __restrict__ seq_of_token, bf16_t* __restrict__ out, int channels,
                                                             int taps) {
  const int c = 8 * (blockIdx.y * blockDim.x + threadIdx.x);
  if (c >= channels) return;
  const int t = blockIdx.x;
  const int hist = taps - 1;
  if (t - cu_q[seq_of_token[t]] < hist) return;
  float acc[8];
  {
    const float4 b0 = *(const float4*)(bias + c), b1 = *(const float4*)(bias + c + 4);
    acc[0] = b0.x, acc[1] = b0.y, acc[2] = b0.z, acc[3] = b0.w, acc[4] = b1.x, acc[5] = b1.y, acc[6] = b1.z, acc[7] = b1.w;
  }
#pragma unroll
  for (int k = 0; k < CONV_MAX_TAPS; ++k) {
    if (k < taps) {
      Frag8 x;
      x.u = *(const uint4*)(in + (size_t)(t - (hist - k)) * in_ld + c);
      // the weights tap by tap ([taps][channels]): a thread's eight are 32 bytes, the threads' side by side
      const float4 w0 = *(const float4*)(w_by_tap + (size_t)k * channels + c), w1 = *(const float4*)(w_by_tap + (size_t)k * channels + c + 4);
      const float wv[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] = fmaf(wv[e], bf16_to_f32(x.h[e]), acc[e]);
    }
  }
  uint4 o;
  o.x = pack2_bf16(silu_f32(acc[0]), silu_f32(acc[1]));
  o.y = pack2_bf16(silu_f32(acc[2]), silu_f32(acc[3]));
  o.z = pack2_bf16(silu_f32(acc[4]), silu_f32(acc[5]));
  o.w = pack2_bf16(silu_f32(acc[6]), silu_f32(acc[7]));
  *(uint4*)(out + (size_t)t * channels + c) = o;
}

// w_by_tap: the same weights as [taps][channels], or null (then every token goes through the kernel of a thread a channel)
extern "C" int cwm_conv_silu(const void* in, long in_ld, int dtype, const float* w, const float* w_by_tap, const float* bias, float* state, long state_ld,
                             long state_off, const int* slots, const int* cu_q, const int* seq_of_token, void* out, int n_tokens,
                             int n_seqs, int channels, int taps, int n_slots, hipStream_t stream) {
  CWM_REQUIRE(in && w && bias && state && slots && cu_q && seq_of_token && out, "conv_silu: arguments missing");
  CWM_REQUIRE(taps >= 1 && taps <= CONV_MAX_TAPS, "conv_silu: %d taps, the kernel takes 1..%d", taps, CONV_MAX_TAPS);
  CWM_REQUIRE(channels > 0 && in_ld >= channels && n_tokens >= 0, "conv_silu: bad sizes");
  CWM_REQUIRE(state_off >= 0 && state_off + (long)(taps - 1) * channels <= state_ld, "conv_silu: the state row is too short");
  if (n_tokens == 0) return 0;
  dim3 grid(n_tokens, (channels + 255) / 256);
  if (dtype == CWM_BF16 && w_by_tap && n_seqs > 0 && n_tokens > n_seqs && channels % 8 == 0 && in_ld % 8 == 0 && ((uintptr_t)in % 16) == 0 &&
      ((uintptr_t)out % 16) == 0 && ((uintptr_t)w_by_tap % 16) == 0 && ((uintptr_t)bias % 16) == 0) {
    // portions of a prompt: the tokens that read no state in pieces of 16 bytes, then a block a sequence for the rest
    hipLaunchKernelGGL(conv_silu_body_kernel, dim3(n_tokens, (channels / 8 + 255) / 256), dim3(256), 0, stream, (const bf16_t*)in, in_ld, w_by_tap,
                       bias, cu_q, seq_of_token, (bf16_t*)out, channels, taps);
    hipLaunchKernelGGL(conv_silu_kernel<bf16_t>, dim3(n_seqs, (channels + 255) / 256), dim3(256), 0, stream, (const bf16_t*)in, in_ld, w, bias,
                       state, state_ld, state_off, slots, cu_q, seq_of_token, (bf16_t*)out, channels, taps, n_slots, 1);
  } else if (dtype == CWM_BF16)
    hipLaunchKernelGGL(conv_silu_kernel<bf16_t>, grid, dim3(256), 0, stream, (const bf16_t*)in, in_ld, w, bias, state, state_ld, state_off,
                       slots, cu_q, seq_of_token, (bf16_t*)out, channels, taps, n_slots, 0);
  else if (dtype == CWM_F32)
    hipLaunchKernelGGL(conv_silu_kernel<float>, grid, dim3(256), 0, stream, (const float*)in, in_ld, w, bias, state, state_ld, state_off,
                       slots, cu_q, seq_of_token, (float*)out, channels, taps, n_slots, 0);
  else
    return cwm_fail("conv_silu: unknown dtype %d", dtype);
  return cwm_launch_status("conv_silu");
}

// One block per (tile of P, head, sequence).  Thread (p, s) holds 16 rows of column p of the head's state: with
// `split` lanes a column (a power of two, adjacent in a wavefront), lane s has rows 4 (s + q split) + j, q, j < 4,
// so that its B and C values are four 16-byte pieces of LDS.  The block walks the sequence's tokens of this step in
// order, a chunk of up to 16 at a time: while it computes on one chunk from LDS (B, C and the tile's x as float32, the step
// sizes and decays computed once a token), the next chunk's values are already on their way into registers.  The
// split lanes add their parts of y_t[p] by shuffles in a fixed order.  The state is read once before and written
// once after the walk; what a token's result is made of, and in which order, does not depend on how the
// sequence is cut into steps.
#define SCAN_PF 36  // most values of a chunk that one thread fetches

// THREADS a block, TC tokens a chunk.  VEC: the rows of xbc start at multiples of 16 bytes and N and P are multiples
// of the values in 16 bytes, so a chunk is fetched in pieces of 16 bytes; otherwise value by value.
#define SCAN_PFV 6  // most 16-byte pieces of a chunk that one thread fetches

//
// Long portions are cut into segments that run side by side (PHASE 1 and 2; PHASE 0 is the walk of whole portions):
// `segments` holds, for every block z, {sequence, first token, end token, number j of the segment in its sequence,
// the sequence's first entry in the scratch lists, segments of the sequence}.  PHASE 1: segment j < last walks its
// tokens from a zero state and leaves that state and the product of its decays in entry 1 + j; the last segment's
// block copies the sequence's state into entry 0.  PHASE 2: segment j starts from entry 0 carried through the
// entries 1 .. j (S <- decay_i S + state_i), walks its tokens and writes y; the last one leaves the sequence's state.
// No block reads a state that another block of the same launch writes.
template <typename T, int THREADS, int TC, bool VEC, int PHASE>
__global__ void __launch_bounds__(THREADS) selective_scan_kernel(const T* __restrict__ xbc, long xbc_ld, const T* __restrict__ dt_raw,
                                                                 long dt_ld, const float* __restrict__ dt_bias,
                                                                 const float* __restrict__ a_log, const float* __restrict__ d_skip,
                                                                 float* state, long state_ld, const int* __restrict__ slots,
                                                                 const int* __restrict__ cu_q, float* __restrict__ y, int heads, int P,
                                                                 int N, int groups, int split, int n_slots,
                                                                 const int* __restrict__ segments, float* seg_state, float* seg_decay) {
  extern __shared__ float lds[];
  const int h = blockIdx.y;
  int b = blockIdx.z, t0, t1, seg = 0, seg_base = 0, n_segs = 1;
  if (PHASE == 0) {
    t0 = cu_q[b], t1 = cu_q[b + 1];
  } else {
    const int* entry = segments + 6 * blockIdx.z;
    b = entry[0], t0 = entry[1], t1 = entry[2], seg = entry[3], seg_base = entry[4], n_segs = entry[5];
  }
  const int cols = THREADS / split;
  const int s = threadIdx.x % split;
  const int col = threadIdx.x / split;
  const int p0 = blockIdx.x * cols;
  const int p = p0 + col;
  const bool live = p < P;
  const int g = h / (heads / groups);
  const int inner = heads * P;
  const int NB = SCAN_ROWS * split;  // rows of B (and of C) in LDS, zeros from N on
  const int row = 2 * NB + cols;     // a token's values in LDS: B, C, the tile's x
  float* dtv = lds + TC * row;       // the chunk's step sizes
  float* av = dtv + TC;              // and decays
  const int slot = slots[b];
  // A head's state in memory, as its threads hold it: [q][p][s][j] for row 4 (s + q split) + j of column p, so that a
  // thread's four rows are 16 bytes and the split lanes of a column lie side by side (rows from N on stay zero).
  float* st = (slot >= 0 && slot < n_slots) ? state + (size_t)slot * state_ld + (size_t)h * SCAN_ROWS * split * P : nullptr;
  float S[SCAN_ROWS];
  const size_t head_elems = (size_t)SCAN_ROWS * split * P;
  auto load_state = [&](const float* from) {  // null: zeros
#pragma unroll
    for (int q = 0; q < SCAN_ROWS / 4; ++q) {
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (from && live) v = *(const float4*)(from + (((size_t)q * P + p) * split + s) * 4);
      S[4 * q + 0] = v.x, S[4 * q + 1] = v.y, S[4 * q + 2] = v.z, S[4 * q + 3] = v.w;
    }
  };
  auto store_state = [&](float* to) {
    if (to && live) {
#pragma unroll
      for (int q = 0; q < SCAN_ROWS / 4; ++q)
        *(float4*)(to + (((size_t)q * P + p) * split + s) * 4) = make_float4(S[4 * q + 0], S[4 * q + 1], S[4 * q + 2], S[4 * q + 3]);
    }
  };
  auto entry_state = [&](int k) { return seg_state + ((size_t)(seg_base + k) * heads + h) * head_elems; };
  if (PHASE == 0) {
    load_state(st);
  } else if (PHASE == 1) {
    if (seg == n_segs - 1) {  // the whole block: the sequence's state as it is, for the segments of the next launch
      load_state(st);
      store_state(entry_state(0));
      return;
    }
    load_state(nullptr);
  } else {
    load_state(entry_state(0));
    for (int i = 0; i < seg; ++i) {
      const float d = seg_decay[(size_t)(seg_base + 1 + i) * heads + h];
      const float* local = entry_state(1 + i);
#pragma unroll
      for (int q = 0; q < SCAN_ROWS / 4; ++q) {
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (live) v = *(const float4*)(local + (((size_t)q * P + p) * split + s) * 4);
        S[4 * q + 0] = d * S[4 * q + 0] + v.x, S[4 * q + 1] = d * S[4 * q + 1] + v.y;
        S[4 * q + 2] = d * S[4 * q + 2] + v.z, S[4 * q + 3] = d * S[4 * q + 3] + v.w;
      }
    }
  }
  const float bias = dt_bias[h];
  const float rate = -expf(a_log[h]);
  const float skip = d_skip[h];
  float decays = 1.f;  // PHASE 1: the product of the segment's decays

  constexpr int U = 16 / sizeof(T);  // values in 16 bytes
  float pf[VEC ? 1 : SCAN_PF];
  uint4 pfv[VEC ? SCAN_PFV : 1];
  int pfv_at[VEC ? SCAN_PFV : 1];  // where in LDS each piece goes (-1: nowhere)
  float pf_dt = 0.f, pf_a = 0.f;
  auto fetch = [&](int start) {  // the chunk that starts at token `start`, into registers
    const int n_tok = min(TC, t1 - start);  // what lies behind the sequence's end is not read (nor used)
    if constexpr (VEC) {
      const int pieces = row / U;  // of one token
      int tc = threadIdx.x / pieces, e = threadIdx.x - tc * pieces;
      const int step_tc = THREADS / pieces, step_e = THREADS - step_tc * pieces;
#pragma unroll
      for (int k = 0; k < SCAN_PFV; ++k) {
        uint4 v = make_uint4(0, 0, 0, 0);
        pfv_at[k] = tc < TC ? tc * row + e * U : -1;
        if (tc < n_tok) {
          const T* src = xbc + (size_t)(start + tc) * xbc_ld;
          const int at = e * U;
          if (at < NB) {
            if (at < N) v = *(const uint4*)(src + inner + (size_t)g * N + at);
          } else if (at < 2 * NB) {
            if (at - NB < N) v = *(const uint4*)(src + inner + (size_t)(groups + g) * N + (at - NB));
          } else if (p0 + at - 2 * NB < P) {
            v = *(const uint4*)(src + (size_t)h * P + p0 + (at - 2 * NB));
          }
        }
        pfv[k] = v;
        tc += step_tc;
        e += step_e;
        if (e >= pieces) e -= pieces, ++tc;
      }
    } else {
      const int total = n_tok * row;
      int tc = 0, e = threadIdx.x;  // this thread's k-th value, number threadIdx.x + k * THREADS of the chunk, is value e of token tc
      while (e >= row) e -= row, ++tc;
#pragma unroll
      for (int k = 0; k < SCAN_PF; ++k) {
        float v = 0.f;
        if (tc * row + e < total) {
          const T* src = xbc + (size_t)(start + tc) * xbc_ld;
          if (e < NB) {
            if (e < N) v = Elem<T>::load(src + inner + (size_t)g * N + e);
          } else if (e < 2 * NB) {
            if (e - NB < N) v = Elem<T>::load(src + inner + (size_t)(groups + g) * N + (e - NB));
          } else if (p0 + e - 2 * NB < P) {
            v = Elem<T>::load(src + (size_t)h * P + p0 + (e - 2 * NB));
          }
        }
        pf[k] = v;
        e += THREADS;
        while (e >= row) e -= row, ++tc;
      }
    }
    if (threadIdx.x < TC) {
      const int t = start + threadIdx.x;
      if (t < t1) {
        const float z = Elem<T>::load(dt_raw + (size_t)t * dt_ld + h) + bias;
        pf_dt = z > 20.f ? z : log1pf(expf(z));
        pf_a = expf(rate * pf_dt);
      }
    }
  };
  auto stage = [&]() {  // registers -> LDS
    if constexpr (VEC) {
#pragma unroll
      for (int k = 0; k < SCAN_PFV; ++k) {
        if (pfv_at[k] < 0) continue;
        float* dst = lds + pfv_at[k];
        if constexpr (sizeof(T) == 4) {
          *(uint4*)dst = pfv[k];
        } else {
          const uint32_t w[4] = {pfv[k].x, pfv[k].y, pfv[k].z, pfv[k].w};
          *(float4*)dst = make_float4(__uint_as_float(w[0] << 16), __uint_as_float(w[0] & 0xffff0000u), __uint_as_float(w[1] << 16),
                                      __uint_as_float(w[1] & 0xffff0000u));
          *(float4*)(dst + 4) = make_float4(__uint_as_float(w[2] << 16), __uint_as_float(w[2] & 0xffff0000u), __uint_as_float(w[3] << 16),
                                            __uint_as_float(w[3] & 0xffff0000u));
        }
      }
    } else {
#pragma unroll
      for (int k = 0; k < SCAN_PF; ++k) {
        const int idx = threadIdx.x + k * THREADS;
        if (idx < TC * row) lds[idx] = pf[k];
      }
    }
    if (threadIdx.x < TC) {
      dtv[threadIdx.x] = pf_dt;
      av[threadIdx.x] = pf_a;
    }
  };
  // One chunk from LDS.  The walk itself holds no wait on another lane: every token leaves its lane's part of y in
  // a register, and the parts of the whole chunk are added across the split lanes afterwards, side by side.  A full
  // chunk runs without a condition in it, so that a token's reads from LDS can start while the one before computes.
  auto walk = [&](auto full_tag, int start, int n_here) {
    constexpr bool FULL = decltype(full_tag)::value;
    float part[TC], xs[TC];
#pragma unroll
    for (int tc = 0; tc < TC; ++tc) {
      part[tc] = 0.f;
      xs[tc] = 0.f;
      if (FULL || tc < n_here) {
        const float* tok = lds + tc * row;
        const float a = av[tc];
        if (PHASE == 1) decays *= a;
        const float x = tok[2 * NB + col];
        const float dx = dtv[tc] * x;
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int q = 0; q < SCAN_ROWS / 4; ++q) {
          const float4 Bq = *(const float4*)(tok + 4 * (s + q * split));
          const float4 Cq = *(const float4*)(tok + NB + 4 * (s + q * split));
          S[4 * q + 0] = fmaf(a, S[4 * q + 0], Bq.x * dx);
          S[4 * q + 1] = fmaf(a, S[4 * q + 1], Bq.y * dx);
          S[4 * q + 2] = fmaf(a, S[4 * q + 2], Bq.z * dx);
          S[4 * q + 3] = fmaf(a, S[4 * q + 3], Bq.w * dx);
          acc[0] = fmaf(S[4 * q + 0], Cq.x, acc[0]);
          acc[1] = fmaf(S[4 * q + 1], Cq.y, acc[1]);
          acc[2] = fmaf(S[4 * q + 2], Cq.z, acc[2]);
          acc[3] = fmaf(S[4 * q + 3], Cq.w, acc[3]);
        }
        part[tc] = (acc[0] + acc[1]) + (acc[2] + acc[3]);
        xs[tc] = x;
      }
    }
    if (PHASE == 1) return;  // only the state is wanted
    for (int off = 1; off < split; off <<= 1) {
#pragma unroll
      for (int tc = 0; tc < TC; ++tc)
        if (FULL || tc < n_here) part[tc] += __shfl_xor(part[tc], off, CWM_WAVE);
    }
    if (live && s == 0) {
#pragma unroll
      for (int tc = 0; tc < TC; ++tc)
        if (FULL || tc < n_here) y[(size_t)(start + tc) * inner + (size_t)h * P + p] = part[tc] + skip * xs[tc];
    }
  };

  fetch(t0);
  stage();
  __syncthreads();
  for (int start = t0; start < t1; start += TC) {
    const bool more = start + TC < t1;
    if (more) fetch(start + TC);
    const int n_here = min(TC, t1 - start);
    if (n_here == TC)
      walk(std::true_type{}, start, TC);
    else
      walk(std::false_type{}, start, n_here);
    __syncthreads();
    if (more) {
      stage();
      __syncthreads();
    }
  }
  if (PHASE == 0) {
    store_state(st);
  } else if (PHASE == 1) {
    store_state(entry_state(1 + seg));
    if (threadIdx.x == 0) seg_decay[(size_t)(seg_base + 1 + seg) * heads + h] = decays;
  } else if (seg == n_segs - 1) {
    store_state(st);
  }
}

// A step in which every sequence brings one token (decoding): no chunk, no LDS.  Thread (p, s) as above; its 16 values
// of B and of C, x, dt and its 16 state values are all asked for at once, so the step waits for memory once.
template <typename T>
__global__ void __launch_bounds__(256) selective_scan_single_kernel(const T* __restrict__ xbc, long xbc_ld, const T* __restrict__ dt_raw,
                                                                    long dt_ld, const float* __restrict__ dt_bias,
                                                                    const float* __restrict__ a_log, const float* __restrict__ d_skip,
                                                                    float* state, long state_ld, const int* __restrict__ slots,
                                                                    float* __restrict__ y, int heads, int P, int N, int groups, int split,
                                                                    int n_slots) {
  const int h = blockIdx.y;
  const int t = blockIdx.z;  // the sequence, and its one token
  const int cols = 256 / split;
  const int s = threadIdx.x % split;
  const int p = blockIdx.x * cols + threadIdx.x / split;
  const bool live = p < P;
  const int pc = live ? p : P - 1;
  const int g = h / (heads / groups);
  const int inner = heads * P;
  const int slot = slots[t];
  float* st = (slot >= 0 && slot < n_slots) ? state + (size_t)slot * state_ld + (size_t)h * SCAN_ROWS * split * P : nullptr;
  const T* row = xbc + (size_t)t * xbc_ld;
  const T* Bt = row + inner + (size_t)g * N;
  const T* Ct = Bt + (size_t)groups * N;
  float S[SCAN_ROWS], Bv[SCAN_ROWS], Cv[SCAN_ROWS];
#pragma unroll
  for (int q = 0; q < SCAN_ROWS / 4; ++q) {
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (st && live) v = *(const float4*)(st + (((size_t)q * P + p) * split + s) * 4);
    S[4 * q + 0] = v.x, S[4 * q + 1] = v.y, S[4 * q + 2] = v.z, S[4 * q + 3] = v.w;
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      const int n = 4 * (s + q * split) + jj;
      Bv[4 * q + jj] = n < N ? Elem<T>::load(Bt + n) : 0.f;
      Cv[4 * q + jj] = n < N ? Elem<T>::load(Ct + n) : 0.f;
    }
  }
  const float x = Elem<T>::load(row + (size_t)h * P + pc);
  const float z = Elem<T>::load(dt_raw + (size_t)t * dt_ld + h) + dt_bias[h];
  const float dt = z > 20.f ? z : log1pf(expf(z));
  const float a = expf(-expf(a_log[h]) * dt);
  const float dx = dt * x;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < SCAN_ROWS; ++i) {  // the same operations in the same order as the walk of a chunk
    S[i] = fmaf(a, S[i], Bv[i] * dx);
    acc[i & 3] = fmaf(S[i], Cv[i], acc[i & 3]);
  }
  float part = (acc[0] + acc[1]) + (acc[2] + acc[3]);
  for (int off = 1; off < split; off <<= 1) part += __shfl_xor(part, off, CWM_WAVE);
  if (live && s == 0) y[(size_t)t * inner + (size_t)h * P + p] = part + d_skip[h] * x;
  if (st && live) {
#pragma unroll
    for (int q = 0; q < SCAN_ROWS / 4; ++q)
      *(float4*)(st + (((size_t)q * P + p) * split + s) * 4) = make_float4(S[4 * q + 0], S[4 * q + 1], S[4 * q + 2], S[4 * q + 3]);
  }
}

template <typename T, bool VEC>
static void launch_scan(dim3 grid, int split, hipStream_t stream, const void* xbc, long xbc_ld, const void* dt_raw, long dt_ld,
                        const float* dt_bias, const float* a_log, const float* d_skip, float* state, long state_ld, const int* slots,
                        const int* cu_q, float* y, int heads, int P, int N, int groups, int n_slots, const int* segments, float* seg_state,
                        float* seg_decay) {
  constexpr int THREADS = 256, TC = 16;
  const int row = 2 * SCAN_ROWS * split + THREADS / split;
  const size_t lds_bytes = (size_t)(TC * row + 2 * TC) * sizeof(float);
#define CWM_SCAN_PHASE(PHASE)                                                                                                              \
  hipLaunchKernelGGL((selective_scan_kernel<T, THREADS, TC, VEC, PHASE>), grid, dim3(THREADS), lds_bytes, stream, (const T*)xbc, xbc_ld,     \
                     (const T*)dt_raw, dt_ld, dt_bias, a_log, d_skip, state, state_ld, slots, cu_q, y, heads, P, N, groups, split, n_slots, \
                     segments, seg_state, seg_decay)
  if (!segments) {
    CWM_SCAN_PHASE(0);
  } else {
    CWM_SCAN_PHASE(1);
    CWM_SCAN_PHASE(2);
  }
#undef CWM_SCAN_PHASE
}

extern "C" int cwm_selective_scan(const void* xbc, long xbc_ld, const void* dt_raw, long dt_ld, int dtype, const float* dt_bias,
                                  const float* a_log, const float* d_skip, float* state, long state_ld, const int* slots,
                                  const int* cu_q, float* y, int n_tokens, int n_seqs, int heads, int P, int N, int groups, int n_slots,
                                  const int* segments, int n_segments, float* seg_state, float* seg_decay, hipStream_t stream) {
  CWM_REQUIRE(xbc && dt_raw && dt_bias && a_log && d_skip && state && slots && cu_q && y, "selective_scan: arguments missing");
  CWM_REQUIRE(heads > 0 && P > 0 && N > 0 && groups > 0 && heads % groups == 0, "selective_scan: bad sizes");
  CWM_REQUIRE(N <= SCAN_ROWS * 16, "selective_scan: a state of %d rows, the kernel takes up to %d", N, SCAN_ROWS * 16);
  CWM_REQUIRE(xbc_ld >= (long)heads * P + 2L * groups * N && dt_ld >= heads, "selective_scan: rows too short");
  CWM_REQUIRE(heads <= 65535 && n_seqs <= 65535, "selective_scan: too many heads or sequences for one launch");
  const int split = cwm_scan_split(N);
  CWM_REQUIRE((long)heads * SCAN_ROWS * split * P <= state_ld && state_ld % 4 == 0 && ((uintptr_t)state % 16) == 0,
              "selective_scan: the state row is too short or not a multiple of 16 bytes");
  if (n_tokens == 0 || n_seqs == 0) return 0;
  const int cols = 256 / split;
  const int row = 2 * SCAN_ROWS * split + cols;
  CWM_REQUIRE(16 * row <= SCAN_PF * 256, "selective_scan: a chunk of tokens does not fit the threads' registers");
  // with a list of segments (6 numbers each; its scratch lists have an entry for every segment) the blocks' z counts those
  CWM_REQUIRE(!segments || (n_segments > 0 && n_segments <= 65535 && seg_state && seg_decay && ((uintptr_t)seg_state % 16) == 0),
              "selective_scan: a list of segments needs its scratch lists and at most 65535 entries");
  dim3 grid((P + cols - 1) / cols, heads, segments ? n_segments : n_seqs);
  if (!segments && n_tokens == n_seqs) {  // one token a sequence
    dim3 single((P + cols - 1) / cols, heads, n_seqs);
    if (dtype == CWM_BF16)
      hipLaunchKernelGGL(selective_scan_single_kernel<bf16_t>, single, dim3(256), 0, stream, (const bf16_t*)xbc, xbc_ld, (const bf16_t*)dt_raw, dt_ld,
                         dt_bias, a_log, d_skip, state, state_ld, slots, y, heads, P, N, groups, split, n_slots);
    else if (dtype == CWM_F32)
      hipLaunchKernelGGL(selective_scan_single_kernel<float>, single, dim3(256), 0, stream, (const float*)xbc, xbc_ld, (const float*)dt_raw, dt_ld,
                         dt_bias, a_log, d_skip, state, state_ld, slots, y, heads, P, N, groups, split, n_slots);
    else
      return cwm_fail("selective_scan: unknown dtype %d", dtype);
    return cwm_launch_status("selective_scan");
  }
  const int unit = dtype == CWM_BF16 ? 8 : 4;
  const bool vec = N % unit == 0 && P % unit == 0 && xbc_ld % unit == 0 && ((uintptr_t)xbc % 16) == 0 && 16 * row / unit <= SCAN_PFV * 256;
#define CWM_SCAN(T, VEC) \
  launch_scan<T, VEC>(grid, split, stream, xbc, xbc_ld, dt_raw, dt_ld, dt_bias, a_log, d_skip, state, state_ld, slots, cu_q, y, heads, P, N, groups, n_slots, \
                      segments, seg_state, seg_decay)
  if (dtype == CWM_BF16) {
    if (vec) CWM_SCAN(bf16_t, true); else CWM_SCAN(bf16_t, false);
  } else if (dtype == CWM_F32) {
    if (vec) CWM_SCAN(float, true); else CWM_SCAN(float, false);
  } else {
    return cwm_fail("selective_scan: unknown dtype %d", dtype);
  }
#undef CWM_SCAN
  return cwm_launch_status("selective_scan");
}
