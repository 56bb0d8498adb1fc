// Routed experts and other products in which every row has a weight matrix of its own choosing.
//
//   route_top        per token: the `top` largest of its router logits (the lower index wins a tie) and the softmax
//                    over those alone, float32; or, mode 1, the softmax over all experts, a choice by score plus a
//                    correction per expert, and weights that are the chosen scores times a scale.
//   group_by_expert  the step's (token, choice) pairs grouped by expert, each group padded to whole tiles of 16
//                    rows: row_token[row] (-1 in the padding), pair_row[pair], tile_expert[tile] (-1 beyond the
//                    last tile).  One block; no count leaves the device.  The order of a group's rows is whatever
//                    the block's atomic counters give: a row's result does not depend on its place.
//   grouped product  out[row] = W[e(row)] a[row] on the matrix cores, e from tile_expert (16 rows a tile share it)
//                    or, for a batch of independent products (one weight per head, say), from the block's z.
//                    bfloat16 operands on v_mfma_f32_16x16x32_bf16, float32 operands on v_mfma_f32_16x16x4_f32
//                    (exact products); float32 sums in the order of k either way, whatever else is in the step.
//                    With two weights the epilogue forms silu(W0 a) * (W1 a), or the clamped form of `GateAct`.
//   combine          out[t] = sum_k weight[t][k] * rows[pair_row[t][k]] in the order of k, float32.
//
// Matrix-core layout as in the other products of this package: operand A = the weight tile (lane 16 j + r: row
// n0 + r, 8 values of k from 32 s + 8 j), operand B = the rows (lane 16 j + r: row r, the same k), result lane
// 16 j + r holds out[r][n0 + 4 j + i], i = 0..3.
#include "common.h"

CWM_DEFINE_ERROR_API

#define ROUTE_MAX_TOP 16
#define ROUTE_MAX_EXPERTS 256
#define TILE_ROWS 16

extern "C" int cwm_route_max_top() { return ROUTE_MAX_TOP; }
extern "C" int cwm_route_max_experts() { return ROUTE_MAX_EXPERTS; }
extern "C" int cwm_route_tile_rows() { return TILE_ROWS; }

// mode 0: the `top` largest logits, weights = softmax over those alone.
// mode 1: scores s = softmax over all experts; the `top` largest of s + correction (correction: null for none) are
//         chosen; weights = scale * s of the chosen, divided by their sum first if `renormalize`.
// One wavefront a token: lane l holds the experts l, l + 64, ...; a choice is a vote of the lanes (the larger value, the
// lower index among equals), so a token's router costs `top` rounds of shuffles whatever the number of experts.
#define ROUTE_PER_LANE (ROUTE_MAX_EXPERTS / CWM_WAVE)
// One token's router, by one wavefront: score[i] holds the logit of expert lane + 64 i (-inf beyond the last expert) on
// entry; the chosen experts and their weights are written by lane 0, to chosen_out / weights_out (`top` entries each)
// and, if given, to chosen_lds.
__device__ __forceinline__ void route_wave(float (&score)[ROUTE_MAX_EXPERTS / CWM_WAVE], int lane, int n_experts, int top, int mode,
                                           const float* __restrict__ correction, float scale, int renormalize,
                                           int* __restrict__ chosen_out, float* __restrict__ weights_out, int* chosen_lds) {
  const float neg_inf = -__builtin_inff();
  float choice[ROUTE_PER_LANE];  // what an expert is chosen by; score: what a weight is made of
#pragma unroll
  for (int i = 0; i < ROUTE_PER_LANE; ++i) choice[i] = score[i];
  if (mode == 1) {
    float largest = score[0];
#pragma unroll
    for (int i = 1; i < ROUTE_PER_LANE; ++i) largest = fmaxf(largest, score[i]);
    largest = wave_max(largest);
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < ROUTE_PER_LANE; ++i) {
      score[i] = lane + CWM_WAVE * i < n_experts ? expf(score[i] - largest) : 0.f;
      sum += score[i];
    }
    const float inv = 1.f / wave_sum(sum);
#pragma unroll
    for (int i = 0; i < ROUTE_PER_LANE; ++i) {
      const int e = lane + CWM_WAVE * i;
      score[i] *= inv;
      choice[i] = e < n_experts ? (correction ? score[i] + correction[e] : score[i]) : neg_inf;
    }
  }
  int idx[ROUTE_MAX_TOP];
  float val[ROUTE_MAX_TOP];
#pragma unroll
  for (int k = 0; k < ROUTE_MAX_TOP; ++k) {
    idx[k] = -1;
    val[k] = 0.f;
  }
#pragma unroll
  for (int k = 0; k < ROUTE_MAX_TOP; ++k) {
    if (k < top) {
      // this lane's best expert that is not taken yet, then the wavefront's
      float bv = neg_inf, bs = 0.f;
      int be = 0x7fffffff;
#pragma unroll
      for (int i = 0; i < ROUTE_PER_LANE; ++i) {
        const int e = lane + CWM_WAVE * i;
        if (e < n_experts && (be == 0x7fffffff || choice[i] > bv)) {  // taken experts have left the vote (below)
          bool taken = false;
#pragma unroll
          for (int m = 0; m < ROUTE_MAX_TOP; ++m) taken |= (m < k && idx[m] == e);
          if (!taken) {
            bv = choice[i];
            bs = score[i];
            be = e;
          }
        }
      }
#pragma unroll
      for (int off = CWM_WAVE / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, CWM_WAVE), os = __shfl_xor(bs, off, CWM_WAVE);
        const int oe = __shfl_xor(be, off, CWM_WAVE);
        const bool theirs = oe != 0x7fffffff && (be == 0x7fffffff || ov > bv || (ov == bv && oe < be));
        if (theirs) {
          bv = ov;
          bs = os;
          be = oe;
        }
      }
      idx[k] = be;
      val[k] = bs;
    }
  }
  if (lane != 0) return;
  float sum = 0.f;
  if (mode == 0) {
    const float largest = val[0];  // the first chosen is the largest
#pragma unroll
    for (int k = 0; k < ROUTE_MAX_TOP; ++k)
      if (k < top) {
        val[k] = expf(val[k] - largest);
        sum += val[k];
      }
  } else {
#pragma unroll
    for (int k = 0; k < ROUTE_MAX_TOP; ++k)
      if (k < top) sum += val[k];
    if (!renormalize) sum = 1.f;
  }
#pragma unroll
  for (int k = 0; k < ROUTE_MAX_TOP; ++k)
    if (k < top) {
      chosen_out[k] = idx[k];
      if (chosen_lds) chosen_lds[k] = idx[k];
      weights_out[k] = mode == 0 ? val[k] / sum : scale * (val[k] / sum);
    }
}

__global__ void __launch_bounds__(256) route_top_kernel(const float* __restrict__ logits, int* __restrict__ chosen,
                                                        float* __restrict__ weights, int n_tokens, int n_experts, int top, int mode,
                                                        const float* __restrict__ correction, float scale, int renormalize) {
  const int lane = threadIdx.x & (CWM_WAVE - 1);
  const int t = blockIdx.x * (blockDim.x / CWM_WAVE) + threadIdx.x / CWM_WAVE;
  if (t >= n_tokens) return;
  const float* z = logits + (size_t)t * n_experts;
  float score[ROUTE_PER_LANE];
#pragma unroll
  for (int i = 0; i < ROUTE_PER_LANE; ++i) {
    const int e = lane + CWM_WAVE * i;
    score[i] = e < n_experts ? z[e] : -__builtin_inff();
  }
  route_wave(score, lane, n_experts, top, mode, correction, scale, renormalize, chosen + (size_t)t * top, weights + (size_t)t * top, nullptr);
}

extern "C" int cwm_route_top(const float* logits, int* chosen, float* weights, int n_tokens, int n_experts, int top, int mode,
                             const float* correction, float scale, int renormalize, hipStream_t stream) {
  CWM_REQUIRE(logits && chosen && weights, "route_top: arguments missing");
  CWM_REQUIRE(top >= 1 && top <= ROUTE_MAX_TOP && top <= n_experts, "route_top: %d of %d experts, the kernel takes up to %d", top, n_experts,
              ROUTE_MAX_TOP);
  CWM_REQUIRE(n_experts <= ROUTE_MAX_EXPERTS, "route_top: %d experts, the kernel takes up to %d", n_experts, ROUTE_MAX_EXPERTS);
  CWM_REQUIRE(mode == 0 || mode == 1, "route_top: unknown mode %d", mode);
  if (n_tokens <= 0) return 0;
  hipLaunchKernelGGL(route_top_kernel, dim3((n_tokens + 3) / 4), dim3(256), 0, stream, logits, chosen, weights, n_tokens, n_experts, top,
                     mode, correction, scale, renormalize);
  return cwm_launch_status("route_top");
}

// The grouping, by one block; `chosen` may lie in global memory or in LDS.
__device__ __forceinline__ void group_pairs(const int* chosen, int n_pairs, int n_experts, int* __restrict__ row_token,
                                            int* __restrict__ pair_row, int* __restrict__ tile_expert, int n_tiles, int top,
                                            int tile_align, int* count, int* start) {
  for (int e = threadIdx.x; e < n_experts; e += blockDim.x) count[e] = 0;
  for (int i = threadIdx.x; i < n_tiles * TILE_ROWS; i += blockDim.x) row_token[i] = -1;
  for (int i = threadIdx.x; i < n_tiles; i += blockDim.x) tile_expert[i] = -1;
  __syncthreads();
  for (int i = threadIdx.x; i < n_pairs; i += blockDim.x) {
    const int e = chosen[i];
    if (e >= 0 && e < n_experts) atomicAdd(&count[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int tile = 0;
    for (int e = 0; e < n_experts; ++e) {
      start[e] = tile * TILE_ROWS;
      const int tiles = (count[e] + TILE_ROWS - 1) / TILE_ROWS;
      for (int k = 0; k < tiles && tile + k < n_tiles; ++k) tile_expert[tile + k] = e;
      tile += (tiles + tile_align - 1) / tile_align * tile_align;  // an expert's tiles start at a multiple of tile_align
      count[e] = 0;
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < n_pairs; i += blockDim.x) {
    const int e = chosen[i];
    int row = -1;
    if (e >= 0 && e < n_experts) {
      row = start[e] + atomicAdd(&count[e], 1);
      if (row < n_tiles * TILE_ROWS)
        row_token[row] = i / top;
      else
        row = -1;
    }
    pair_row[i] = row;
  }
}

__global__ void __launch_bounds__(1024) group_by_expert_kernel(const int* __restrict__ chosen, int n_pairs, int n_experts,
                                                               int* __restrict__ row_token, int* __restrict__ pair_row,
                                                               int* __restrict__ tile_expert, int n_tiles, int top, int tile_align) {
  __shared__ int count[ROUTE_MAX_EXPERTS];
  __shared__ int start[ROUTE_MAX_EXPERTS];
  group_pairs(chosen, n_pairs, n_experts, row_token, pair_row, tile_expert, n_tiles, top, tile_align, count, start);
}

// tile_align: an expert's first tile lies at a multiple of so many tiles (the tiles that one block of the product takes).
extern "C" int cwm_group_by_expert(const int* chosen, int n_tokens, int top, int n_experts, int* row_token, int* pair_row,
                                   int* tile_expert, int n_tiles, int tile_align, hipStream_t stream) {
  CWM_REQUIRE(chosen && row_token && pair_row && tile_expert, "group_by_expert: arguments missing");
  CWM_REQUIRE(n_experts >= 1 && n_experts <= ROUTE_MAX_EXPERTS && top >= 1, "group_by_expert: %d experts, the kernel takes up to %d", n_experts,
              ROUTE_MAX_EXPERTS);
  const long n_pairs = (long)n_tokens * top;
  CWM_REQUIRE(tile_align >= 1 && (long)n_tiles >= (n_pairs + TILE_ROWS - 1) / TILE_ROWS + (long)n_experts * tile_align,
              "group_by_expert: %d tiles do not hold %ld pairs of %d experts", n_tiles, n_pairs, n_experts);
  if (n_tokens <= 0) return 0;
  hipLaunchKernelGGL(group_by_expert_kernel, dim3(1), dim3(1024), 0, stream, chosen, (int)n_pairs, n_experts, row_token, pair_row, tile_expert,
                     n_tiles, top, tile_align);
  return cwm_launch_status("group_by_expert");
}

// ---- the grouped product ------------------------------------------------------------------------------------- //
// What the epilogue of a product with two weights makes of g = W0 a and u = W1 a:
//   kind 0: silu(g) * u
//   kind 1: g' * sigmoid(alpha g') * (u' + 1) with g' = min(g, limit), u' = clamp(u, -limit, limit)
struct GateAct {
  int kind;
  float alpha, limit;
};
__device__ __forceinline__ float gated_value(float g, float u, const GateAct act) {
  if (act.kind == 1) {
    g = fminf(g, act.limit);
    u = fminf(fmaxf(u, -act.limit), act.limit);
    return g / (1.f + expf(-act.alpha * g)) * (u + 1.f);
  }
  return g / (1.f + expf(-g)) * u;
}

template <typename T> struct Frag;
template <> struct Frag<bf16_t> {
  static constexpr int K_STEP = 32;  // values of k one matrix instruction takes
  static constexpr int PER_LANE = 8;
  Frag8 f;
  __device__ __forceinline__ void zero() { f.u = make_uint4(0, 0, 0, 0); }
  __device__ __forceinline__ void load16(const bf16_t* p) { f.u = *(const uint4*)p; }
  __device__ __forceinline__ void load_some(const bf16_t* p, int n) {
    zero();
    for (int i = 0; i < PER_LANE; ++i)
      if (i < n) f.h[i] = p[i];
  }
  static __device__ __forceinline__ float4v mma(const Frag& w, const Frag& a, float4v acc) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(w.f.v, a.f.v, acc, 0, 0, 0);
  }
};
template <> struct Frag<float> {
  static constexpr int K_STEP = 16;  // four instructions of 4: lane group j supplies k = 4 j + e to instruction e
  static constexpr int PER_LANE = 4;
  float4 f;
  __device__ __forceinline__ void zero() { f = make_float4(0.f, 0.f, 0.f, 0.f); }
  __device__ __forceinline__ void load16(const float* p) { f = *(const float4*)p; }
  __device__ __forceinline__ void load_some(const float* p, int n) {
    f.x = n > 0 ? p[0] : 0.f;
    f.y = n > 1 ? p[1] : 0.f;
    f.z = n > 2 ? p[2] : 0.f;
    f.w = n > 3 ? p[3] : 0.f;
  }
  static __device__ __forceinline__ float4v mma(const Frag& w, const Frag& a, float4v acc) {
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(w.f.x, a.f.x, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(w.f.y, a.f.y, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(w.f.z, a.f.z, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(w.f.w, a.f.w, acc, 0, 0, 0);
    return acc;
  }
};

// A block of four wavefronts, WR of them down the rows and 4 / WR along the columns, takes WR * RT row tiles of one
// expert (they follow one another in the list, and an expert's tiles start at a multiple of that many) and
// (4 / WR) * CT * 16 columns; a wavefront multiplies RT row tiles by CT column tiles, so each piece of a weight tile
// it loads serves RT tiles of rows and each piece of rows CT tiles of columns.  Shapes in use: 1 x 1 tiles a
// wavefront, four wavefronts along the columns (few rows an expert: many blocks stream the weights); 4 x 1 likewise;
// 4 x 4 (4 x 2 with two weights) with the wavefronts 2 x 2 (many rows an expert).
// VEC: rows of a and W start at multiples of 16 bytes and K is a multiple of a lane's piece.
template <typename T, int RT, int CT, int WR, bool GATED, bool VEC>
__global__ void __launch_bounds__(256) grouped_product_kernel(const T* __restrict__ a, long a_ld, long a_batch, const int* __restrict__ row_token,
                                                              const T* __restrict__ w0, const T* __restrict__ w1, long w_stride,
                                                              const int* __restrict__ tile_expert, int n_tiles, void* __restrict__ out,
                                                              int out_dtype, long out_ld, long out_batch, int n_rows, int N, int K, GateAct act) {
  constexpr int WC = 4 / WR;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wave_r = wave / WC, wave_c = wave % WC;
  const int r = lane & 15, j = lane >> 4;
  const int block_tile0 = blockIdx.x * (WR * RT);
  const int tile0 = block_tile0 + wave_r * RT;
  int expert;
  if (tile_expert) {
    expert = block_tile0 < n_tiles ? tile_expert[block_tile0] : -1;
    if (expert < 0) return;
  } else {
    expert = blockIdx.z;
  }
  const int n0 = (blockIdx.y * WC + wave_c) * CT * 16;
  if (n0 >= N) return;
  const T* wrow0[CT];
  const T* wrow1[CT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int col = n0 + ct * 16 + r;
    const size_t at = (size_t)expert * w_stride + (size_t)(col < N ? col : N - 1) * K;
    wrow0[ct] = w0 + at;
    wrow1[ct] = GATED ? w1 + at : nullptr;
  }
  const T* arow[RT];
  bool tile_live[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int tile = tile0 + rt;
    // a tile of another expert, or beyond the rows, is left out
    tile_live[rt] = tile_expert ? (tile < n_tiles && tile_expert[tile] == expert) : tile * TILE_ROWS < n_rows;
    const int row = tile * TILE_ROWS + r;
    long src = -1;
    if (tile_live[rt]) src = row_token ? row_token[row] : (row < n_rows ? row : -1);
    arow[rt] = src >= 0 ? a + (size_t)blockIdx.z * a_batch + (size_t)src * a_ld : nullptr;
  }
  float4v acc0[RT][CT], acc1[RT][CT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) acc0[rt][ct] = acc1[rt][ct] = (float4v){0.f, 0.f, 0.f, 0.f};
  constexpr int STEP = Frag<T>::K_STEP, PIECE = Frag<T>::PER_LANE;
  // two sets of operands: while one is multiplied, the loads of the next step are in flight
  auto load_set = [&](Frag<T> (&fw0)[CT], Frag<T> (&fw1)[CT], Frag<T> (&fa)[RT], int k0) {
    const int k = k0 + j * PIECE;
    const int left = K - k;  // values of this lane's piece inside K
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      if (VEC) {
        if (left > 0) {
          fw0[ct].load16(wrow0[ct] + k);
          if (GATED) fw1[ct].load16(wrow1[ct] + k);
        } else {
          fw0[ct].zero();
          if (GATED) fw1[ct].zero();
        }
      } else {
        fw0[ct].load_some(wrow0[ct] + k, left);
        if (GATED) fw1[ct].load_some(wrow1[ct] + k, left);
      }
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      if (!arow[rt] || left <= 0)
        fa[rt].zero();
      else if (VEC)
        fa[rt].load16(arow[rt] + k);
      else
        fa[rt].load_some(arow[rt] + k, left);
    }
  };
  auto multiply = [&](const Frag<T> (&fw0)[CT], const Frag<T> (&fw1)[CT], const Frag<T> (&fa)[RT]) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) {
        acc0[rt][ct] = Frag<T>::mma(fw0[ct], fa[rt], acc0[rt][ct]);
        if (GATED) acc1[rt][ct] = Frag<T>::mma(fw1[ct], fa[rt], acc1[rt][ct]);
      }
  };
  Frag<T> w0a[CT], w1a[CT], ra[RT], w0b[CT], w1b[CT], rb[RT];
  load_set(w0a, w1a, ra, 0);
  for (int k0 = 0; k0 < K; k0 += 2 * STEP) {
    load_set(w0b, w1b, rb, k0 + STEP);  // beyond K: zeros
    multiply(w0a, w1a, ra);
    load_set(w0a, w1a, ra, k0 + 2 * STEP);
    multiply(w0b, w1b, rb);
  }
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    if (!tile_live[rt]) continue;
    const int row = (tile0 + rt) * TILE_ROWS + r;
    if (!tile_expert && row >= n_rows) continue;
    const size_t base = (size_t)blockIdx.z * out_batch + (size_t)row * out_ld;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = n0 + ct * 16 + 4 * j + i;
        if (c >= N) continue;
        float v = acc0[rt][ct][i];
        if (GATED) v = gated_value(v, acc1[rt][ct][i], act);
        if (out_dtype == CWM_F32)
          ((float*)out)[base + c] = v;
        else
          ((bf16_t*)out)[base + c] = f32_to_bf16(v);
      }
  }
}

// Few rows an expert (a decode step): the product is bound by streaming the chosen experts' weights once.  A block
// takes one row tile and 16 columns; its four wavefronts split K (wavefront w the steps w, w + 4, ...: together they
// read whole lines of a weight row), each with STREAM_DEPTH steps of operands in flight while the ones before are
// multiplied, and add their sums through LDS in the order of w.  Rows of a and W start at multiples of 16 bytes.
#define STREAM_DEPTH 4

template <typename T, bool GATED>
__global__ void __launch_bounds__(256) grouped_stream_kernel(const T* __restrict__ a, long a_ld, long a_batch, const int* __restrict__ row_token,
                                                             const T* __restrict__ w0, const T* __restrict__ w1, long w_stride,
                                                             const int* __restrict__ tile_expert, int n_tiles, void* __restrict__ out,
                                                             int out_dtype, long out_ld, long out_batch, int n_rows, int N, int K, GateAct act) {
  __shared__ float sums[4][GATED ? 2 : 1][64][4];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int r = lane & 15, j = lane >> 4;
  const int tile = blockIdx.x;
  int expert;
  if (tile_expert) {
    expert = tile < n_tiles ? tile_expert[tile] : -1;
    if (expert < 0) return;
  } else {
    expert = blockIdx.z;
  }
  const int n0 = blockIdx.y * 16;
  const int col = n0 + r;
  const size_t at = (size_t)expert * w_stride + (size_t)(col < N ? col : N - 1) * K;
  const T* wrow0 = w0 + at;
  const T* wrow1 = GATED ? w1 + at : nullptr;
  const int row = tile * TILE_ROWS + r;
  long src = row_token ? row_token[row] : (row < n_rows ? row : -1);
  const T* arow = src >= 0 ? a + (size_t)blockIdx.z * a_batch + (size_t)src * a_ld : nullptr;
  constexpr int STEP = Frag<T>::K_STEP, PIECE = Frag<T>::PER_LANE;
  const int steps = (K + STEP - 1) / STEP;
  float4v acc0 = (float4v){0.f, 0.f, 0.f, 0.f}, acc1 = acc0;
  auto load_group = [&](Frag<T> (&fw0)[STREAM_DEPTH], Frag<T> (&fw1)[STREAM_DEPTH], Frag<T> (&fa)[STREAM_DEPTH], int first) {
#pragma unroll
    for (int d = 0; d < STREAM_DEPTH; ++d) {
      const int step = wave + 4 * (first + d);
      const int k = step * STEP + j * PIECE;
      if (step < steps && k < K) {
        fw0[d].load16(wrow0 + k);
        if (GATED) fw1[d].load16(wrow1 + k);
        if (arow) fa[d].load16(arow + k); else fa[d].zero();
      } else {
        fw0[d].zero();
        if (GATED) fw1[d].zero();
        fa[d].zero();
      }
    }
  };
  auto multiply_group = [&](const Frag<T> (&fw0)[STREAM_DEPTH], const Frag<T> (&fw1)[STREAM_DEPTH], const Frag<T> (&fa)[STREAM_DEPTH]) {
#pragma unroll
    for (int d = 0; d < STREAM_DEPTH; ++d) {
      acc0 = Frag<T>::mma(fw0[d], fa[d], acc0);
      if (GATED) acc1 = Frag<T>::mma(fw1[d], fa[d], acc1);
    }
  };
  Frag<T> w0a[STREAM_DEPTH], w1a[STREAM_DEPTH], ra[STREAM_DEPTH], w0b[STREAM_DEPTH], w1b[STREAM_DEPTH], rb[STREAM_DEPTH];
  const int groups = (steps + 4 * STREAM_DEPTH - 1) / (4 * STREAM_DEPTH);  // of STREAM_DEPTH steps a wavefront
  load_group(w0a, w1a, ra, 0);
  for (int g = 0; g < groups; g += 2) {
    load_group(w0b, w1b, rb, (g + 1) * STREAM_DEPTH);  // beyond K: zeros
    multiply_group(w0a, w1a, ra);
    load_group(w0a, w1a, ra, (g + 2) * STREAM_DEPTH);
    multiply_group(w0b, w1b, rb);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    sums[wave][0][lane][i] = acc0[i];
    if (GATED) sums[wave][GATED ? 1 : 0][lane][i] = acc1[i];
  }
  __syncthreads();
  if (wave != 0) return;
  if (!tile_expert && row >= n_rows) return;
  const size_t base = (size_t)blockIdx.z * out_batch + (size_t)row * out_ld;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int c = n0 + 4 * j + i;
    if (c >= N) continue;
    float v = ((sums[0][0][lane][i] + sums[1][0][lane][i]) + sums[2][0][lane][i]) + sums[3][0][lane][i];
    if (GATED) {
      const float u = ((sums[0][GATED ? 1 : 0][lane][i] + sums[1][GATED ? 1 : 0][lane][i]) + sums[2][GATED ? 1 : 0][lane][i]) + sums[3][GATED ? 1 : 0][lane][i];
      v = gated_value(v, u, act);
    }
    if (out_dtype == CWM_F32)
      ((float*)out)[base + c] = v;
    else
      ((bf16_t*)out)[base + c] = f32_to_bf16(v);
  }
}

// Many rows an expert, bfloat16, K a multiple of 64: a block of four wavefronts (2 x 2) takes 8 row tiles of one expert
// and 128 rows of weights (128 columns of the result; with two weights 64 columns of each), 64 values of k a step.
// The step's 16 KB of rows and 16 KB of weights go from global memory to registers while the step before is
// multiplied, then into the other of two LDS buffers (16-byte pieces, a row's pieces XOR-swizzled by the row so that
// the lanes of a matrix operand read different banks); every wavefront multiplies 64 rows by 64 weight rows from there.
template <bool GATED>
__global__ void __launch_bounds__(256) grouped_tiled_kernel(const bf16_t* __restrict__ a, long a_ld, long a_batch, const int* __restrict__ row_token,
                                                            const bf16_t* __restrict__ w0, const bf16_t* __restrict__ w1, long w_stride,
                                                            const int* __restrict__ tile_expert, int n_tiles, void* __restrict__ out,
                                                            int out_dtype, long out_ld, long out_batch, int n_rows, int N, int K, GateAct act) {
  extern __shared__ uint4 tiled_lds[];  // [2 buffers][rows: 128 x 8 pieces | weights: 128 x 8 pieces]
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wr = wave >> 1, wc = wave & 1;
  const int r = lane & 15, j = lane >> 4;
  const int block_tile0 = blockIdx.x * 8;
  int expert;
  if (tile_expert) {
    expert = block_tile0 < n_tiles ? tile_expert[block_tile0] : -1;
    if (expert < 0) return;
  } else {
    expert = blockIdx.z;
  }
  constexpr int OUT_COLS = GATED ? 64 : 128;  // columns of the result a block makes
  const int n0 = blockIdx.y * OUT_COLS;
  // what this thread fetches every step: pieces id = threadIdx.x + 256 i, i < 4, of the rows and of the weights
  const bf16_t* src_a[4];
  const bf16_t* src_w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int id = threadIdx.x + 256 * i;
    const int row = id >> 3, piece = id & 7;
    const int tile = block_tile0 + (row >> 4);
    const bool live = tile_expert ? (tile < n_tiles && tile_expert[tile] == expert) : tile * TILE_ROWS < n_rows;
    const int list_row = tile * TILE_ROWS + (row & 15);
    long src = -1;
    if (live) src = row_token ? row_token[list_row] : (list_row < n_rows ? list_row : -1);
    src_a[i] = src >= 0 ? a + (size_t)blockIdx.z * a_batch + (size_t)src * a_ld + piece * 8 : nullptr;
    int col;  // the weight row: with two weights rows 0..63 are the first one's, 64..127 the second one's
    const bf16_t* w = w0;
    if (GATED) {
      col = n0 + (row & 63);
      if (row >= 64) w = w1;
    } else {
      col = n0 + row;
    }
    src_w[i] = w + (size_t)expert * w_stride + (size_t)(col < N ? col : N - 1) * K + piece * 8;
  }
  // three steps of operands on their way: what is fetched at the start of step k is put into LDS at the end of step k + 2
  uint4 ra[3][4], rw[3][4];
  auto fetch = [&](uint4 (&fa)[4], uint4 (&fw)[4], int k0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool inside = k0 < K;
      fa[i] = (inside && src_a[i]) ? *(const uint4*)(src_a[i] + k0) : make_uint4(0, 0, 0, 0);
      fw[i] = inside ? *(const uint4*)(src_w[i] + k0) : make_uint4(0, 0, 0, 0);
    }
  };
  auto stage = [&](const uint4 (&fa)[4], const uint4 (&fw)[4], int buf) {
    uint4* rows = tiled_lds + buf * 2048;
    uint4* weights = rows + 1024;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int id = threadIdx.x + 256 * i;
      const int row = id >> 3, piece = id & 7;
      rows[row * 8 + (piece ^ (row & 7))] = fa[i];
      weights[row * 8 + (piece ^ (row & 7))] = fw[i];
    }
  };
  float4v acc0[4][GATED ? 2 : 4], acc1[4][GATED ? 2 : 1];
#pragma unroll
  for (int rt = 0; rt < 4; ++rt) {
#pragma unroll
    for (int ct = 0; ct < (GATED ? 2 : 4); ++ct) acc0[rt][ct] = (float4v){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ct = 0; ct < (GATED ? 2 : 1); ++ct) acc1[rt][ct] = (float4v){0.f, 0.f, 0.f, 0.f};
  }
  auto multiply = [&](int buf) {
    const uint4* rows = tiled_lds + buf * 2048;
    const uint4* weights = rows + 1024;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int piece = half * 4 + j;
      Frag8 fa[4], fw[4];
#pragma unroll
      for (int rt = 0; rt < 4; ++rt) {
        const int row = wr * 64 + rt * 16 + r;
        fa[rt].u = rows[row * 8 + (piece ^ (row & 7))];
      }
#pragma unroll
      for (int ct = 0; ct < 4; ++ct) {
        // weight rows of this wavefront: 64 in a row, or (two weights) 32 of each
        const int row = GATED ? (ct < 2 ? wc * 32 + ct * 16 + r : 64 + wc * 32 + (ct - 2) * 16 + r) : wc * 64 + ct * 16 + r;
        fw[ct].u = weights[row * 8 + (piece ^ (row & 7))];
      }
#pragma unroll
      for (int rt = 0; rt < 4; ++rt) {
        if (GATED) {
#pragma unroll
          for (int ct = 0; ct < 2; ++ct) {
            acc0[rt][ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw[ct].v, fa[rt].v, acc0[rt][ct], 0, 0, 0);
            acc1[rt][ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw[2 + ct].v, fa[rt].v, acc1[rt][ct], 0, 0, 0);
          }
        } else {
#pragma unroll
          for (int ct = 0; ct < 4; ++ct) acc0[rt][ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw[ct].v, fa[rt].v, acc0[rt][ct], 0, 0, 0);
        }
      }
    }
  };
  const int steps = K / 64;
  fetch(ra[0], rw[0], 0);
  stage(ra[0], rw[0], 0);
  fetch(ra[1], rw[1], 64);
  fetch(ra[2], rw[2], 128);
  __syncthreads();
  for (int base = 0; base < steps; base += 6) {  // six steps a turn: register set step % 3 and buffer step % 2 keep their names
#pragma unroll
    for (int u = 0; u < 6; ++u) {
      const int step = base + u;
      if (step >= steps) break;
      fetch(ra[u % 3], rw[u % 3], (step + 3) * 64);  // this set's step went into LDS a step ago
      multiply(u % 2);
      stage(ra[(u + 1) % 3], rw[(u + 1) % 3], (u + 1) % 2);
      __syncthreads();
    }
  }
#pragma unroll
  for (int rt = 0; rt < 4; ++rt) {
    const int tile = block_tile0 + wr * 4 + rt;
    const bool live = tile_expert ? (tile < n_tiles && tile_expert[tile] == expert) : tile * TILE_ROWS < n_rows;
    if (!live) continue;
    const int row = tile * TILE_ROWS + r;
    if (!tile_expert && row >= n_rows) continue;
    const size_t base = (size_t)blockIdx.z * out_batch + (size_t)row * out_ld;
#pragma unroll
    for (int ct = 0; ct < (GATED ? 2 : 4); ++ct)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = n0 + (GATED ? wc * 32 : wc * 64) + ct * 16 + 4 * j + i;
        if (c >= N) continue;
        float v = acc0[rt][ct][i];
        if (GATED) v = gated_value(v, acc1[rt][ct][i], act);
        if (out_dtype == CWM_F32)
          ((float*)out)[base + c] = v;
        else
          ((bf16_t*)out)[base + c] = f32_to_bf16(v);
      }
  }
}

template <typename T, int RT, int CT, int WR, bool GATED>
static void launch_grouped(bool vec, int tiles, int n_batch, hipStream_t stream, const T* a, long a_ld, long a_batch, const int* row_token,
                           const T* w0, const T* w1, long w_stride, const int* tile_expert, int n_tiles, void* out, int out_dtype,
                           long out_ld, long out_batch, int n_rows, int N, int K, GateAct act) {
  constexpr int block_tiles = WR * RT, block_cols = (4 / WR) * CT * 16;
  dim3 grid((tiles + block_tiles - 1) / block_tiles, (N + block_cols - 1) / block_cols, n_batch);
  if (vec)
    hipLaunchKernelGGL((grouped_product_kernel<T, RT, CT, WR, GATED, true>), grid, dim3(256), 0, stream, a, a_ld, a_batch, row_token, w0, w1,
                       w_stride, tile_expert, n_tiles, out, out_dtype, out_ld, out_batch, n_rows, N, K, act);
  else
    hipLaunchKernelGGL((grouped_product_kernel<T, RT, CT, WR, GATED, false>), grid, dim3(256), 0, stream, a, a_ld, a_batch, row_token, w0, w1,
                       w_stride, tile_expert, n_tiles, out, out_dtype, out_ld, out_batch, n_rows, N, K, act);
}

// a: rows of K values, `a_ld` apart (row `row_token[row]` for list row `row` if a list is given; batch z starts
// `a_batch` further).  w0 (and w1 for the gated form): [experts or batches][N][K], `w_stride` apart.  With
// `tile_expert` the rows are the list's n_tiles * 16 and out is [rows][out_ld]; without, every batch z < n_batch
// multiplies the same n_rows rows by its own weight into out + z * out_batch.  tiles_a_block: 1, 4 or 8 row tiles
// a block (with a list, an expert's tiles start at a multiple of it).  act_kind, act_alpha, act_limit: the gated
// form's activation (`GateAct`).
extern "C" int cwm_grouped_product(const void* a, long a_ld, long a_batch, int dtype, const int* row_token, const void* w0, const void* w1,
                                   long w_stride, const int* tile_expert, int n_tiles, int n_batch, void* out, int out_dtype, long out_ld,
                                   long out_batch, int n_rows, int N, int K, int tiles_a_block, int act_kind, float act_alpha,
                                   float act_limit, hipStream_t stream) {
  CWM_REQUIRE(a && w0 && out, "grouped_product: arguments missing");
  CWM_REQUIRE(act_kind == 0 || act_kind == 1, "grouped_product: unknown gated activation %d", act_kind);
  const GateAct act = {act_kind, act_alpha, act_limit};
  CWM_REQUIRE(N > 0 && K > 0 && a_ld >= K && out_ld >= 0, "grouped_product: bad sizes");
  CWM_REQUIRE(tile_expert ? (n_tiles >= 0 && n_batch == 1 && row_token) : (n_batch >= 1 && n_batch <= 65535), "grouped_product: give a tile list or a number of batches");
  const int tiles = tile_expert ? n_tiles : (n_rows + TILE_ROWS - 1) / TILE_ROWS;
  if (tiles <= 0) return 0;
  const int esize = dtype == CWM_BF16 ? 2 : 4;
  const int piece = dtype == CWM_BF16 ? 8 : 4;
  const bool vec = K % piece == 0 && (a_ld * esize) % 16 == 0 && (a_batch * esize) % 16 == 0 && (w_stride * esize) % 16 == 0 &&
                   ((uintptr_t)a % 16) == 0 && ((uintptr_t)w0 % 16) == 0 && (!w1 || ((uintptr_t)w1 % 16) == 0);
  CWM_REQUIRE(tiles_a_block == 1 || tiles_a_block == 4 || tiles_a_block == 8, "grouped_product: a block takes 1, 4 or 8 row tiles");
  CWM_REQUIRE((N + 15) / 16 <= 65535, "grouped_product: too many columns");
  const int nb = tile_expert ? 1 : n_batch;
#define CWM_GROUPED(T, RT, CT, WR, GATED)                                                                                                 \
  launch_grouped<T, RT, CT, WR, GATED>(vec, tiles, nb, stream, (const T*)a, a_ld, a_batch, row_token, (const T*)w0, (const T*)w1, w_stride, \
                                       tile_expert, n_tiles, out, out_dtype, out_ld, out_batch, n_rows, N, K, act)
#define CWM_GROUPED_SHAPES(T)                                                   \
  do {                                                                          \
    if (w1) {                                                                   \
      if (tiles_a_block == 8) CWM_GROUPED(T, 4, 2, 2, true);                    \
      else if (tiles_a_block == 4) CWM_GROUPED(T, 4, 1, 1, true);               \
      else CWM_GROUPED(T, 1, 1, 1, true);                                       \
    } else {                                                                    \
      if (tiles_a_block == 8) CWM_GROUPED(T, 4, 4, 2, false);                   \
      else if (tiles_a_block == 4) CWM_GROUPED(T, 4, 1, 1, false);              \
      else CWM_GROUPED(T, 1, 1, 1, false);                                      \
    }                                                                           \
  } while (0)
  if (tiles_a_block == 1 && vec && (dtype == CWM_BF16 || dtype == CWM_F32)) {
    // the weight-streaming shape
    dim3 grid(tiles, (N + 15) / 16, nb);
#define CWM_STREAMED(T, GATED)                                                                                                             \
  hipLaunchKernelGGL((grouped_stream_kernel<T, GATED>), grid, dim3(256), 0, stream, (const T*)a, a_ld, a_batch, row_token, (const T*)w0,     \
                     (const T*)w1, w_stride, tile_expert, n_tiles, out, out_dtype, out_ld, out_batch, n_rows, N, K, act)
    if (dtype == CWM_BF16) {
      if (w1) CWM_STREAMED(bf16_t, true); else CWM_STREAMED(bf16_t, false);
    } else {
      if (w1) CWM_STREAMED(float, true); else CWM_STREAMED(float, false);
    }
#undef CWM_STREAMED
    return cwm_launch_status("grouped_product");
  }
  if (tiles_a_block == 8 && vec && dtype == CWM_BF16 && K % 64 == 0) {
    // the shape that goes through LDS
    const size_t lds_bytes = 2 * 2048 * sizeof(uint4);
    dim3 grid((tiles + 7) / 8, w1 ? (N + 63) / 64 : (N + 127) / 128, nb);
    if (w1)
      hipLaunchKernelGGL(grouped_tiled_kernel<true>, grid, dim3(256), lds_bytes, stream, (const bf16_t*)a, a_ld, a_batch, row_token,
                         (const bf16_t*)w0, (const bf16_t*)w1, w_stride, tile_expert, n_tiles, out, out_dtype, out_ld, out_batch, n_rows, N, K, act);
    else
      hipLaunchKernelGGL(grouped_tiled_kernel<false>, grid, dim3(256), lds_bytes, stream, (const bf16_t*)a, a_ld, a_batch, row_token,
                         (const bf16_t*)w0, (const bf16_t*)w1, w_stride, tile_expert, n_tiles, out, out_dtype, out_ld, out_batch, n_rows, N, K, act);
    return cwm_launch_status("grouped_product");
  }
  if (dtype == CWM_BF16)
    CWM_GROUPED_SHAPES(bf16_t);
  else if (dtype == CWM_F32)
    CWM_GROUPED_SHAPES(float);
  else
    return cwm_fail("grouped_product: unknown dtype %d", dtype);
#undef CWM_GROUPED_SHAPES
#undef CWM_GROUPED
  return cwm_launch_status("grouped_product");
}

__global__ void __launch_bounds__(256) combine_routed_kernel(const float* __restrict__ rows, long rows_ld, const int* __restrict__ pair_row,
                                                             const float* __restrict__ weights, float* __restrict__ out, int top, int dim) {
  const size_t t = blockIdx.x;
  for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < dim; i += gridDim.y * blockDim.x) {
    float acc = 0.f;
    for (int k = 0; k < top; ++k) {
      const int row = pair_row[t * top + k];
      if (row >= 0) acc += weights[t * top + k] * rows[(size_t)row * rows_ld + i];
    }
    out[t * dim + i] = acc;
  }
}

extern "C" int cwm_combine_routed(const float* rows, long rows_ld, const int* pair_row, const float* weights, float* out, int n_tokens,
                                  int top, int dim, hipStream_t stream) {
  CWM_REQUIRE(rows && pair_row && weights && out && top >= 1 && dim > 0, "combine_routed: bad arguments");
  if (n_tokens <= 0) return 0;
  hipLaunchKernelGGL(combine_routed_kernel, dim3(n_tokens, (dim + 1023) / 1024), dim3(256), 0, stream, rows, rows_ld, pair_row, weights, out, top, dim);
  return cwm_launch_status("combine_routed");
}
