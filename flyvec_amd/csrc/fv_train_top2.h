// The two largest |W| of every row, carried from step to step (device code of fv_train.hip).
#pragma once

#include "fv_train_state.h"

// ---- the two largest weights of every row ------------------------------------------------------------

// The two largest of a multiset of non-negative values, kept as (m1 >= m2): one more value, and the
// union with another pair.
__device__ __forceinline__ void fv_top2_insert(float &m1, float &m2, float a) {
  m2 = fmaxf(m2, fminf(m1, a));
  m1 = fmaxf(m1, a);
}
// The same with |w| of a weight known not to be a NaN, in two instructions with |w| as an operand modifier:
// the median of (m1, m2, |w|) is the new second value, max(m1, |w|) the new first. The maximum is written as
// the instruction itself: from fmaxf the compiler makes three, two of them to quieten signalling NaNs that
// cannot be there.
__device__ __forceinline__ void fv_top2_insert_abs(float &m1, float &m2, float w) {
  m2 = __builtin_amdgcn_fmed3f(m1, m2, __builtin_fabsf(w));
  asm("v_max_f32_e64 %0, %1, |%2|" : "=v"(m1) : "v"(m1), "v"(w));
}
__device__ __forceinline__ void fv_top2_merge(float &m1, float &m2, float b1, float b2) {
  const float lo = fminf(m1, b1);
  m1 = fmaxf(m1, b1);
  m2 = fmaxf(lo, fmaxf(m2, b2));
}

// The shares of every row's two largest weights that the blocks of the last dense launches left
// (top2_part[block][neuron], a block's pairs side by side) are merged into row_top2[neuron] for the step that
// begins: one 256-thread block per 32 neurons and per chunk of FV_MERGE_CHUNK shares, eight threads per
// neuron sharing the chunk's blocks among them, eight loads in flight each. A single dense launch leaves
// one chunk, which the first blocks of the next winner kernel's launch merge. Separate dense launches
// leave a share per block of a large grid: two small launches behind them merge first every chunk into a
// staging array, then the staged pairs (fv_merge_shares_kernel, fv_merge_stage_kernel).
#define FV_MERGE_NEURONS 32
#define FV_MERGE_CHUNK 256
struct fv_merge_args {
  const float2 *part;  // top2_part
  uint32_t stride;     // pairs per share (ldk)
  uint32_t n_part;     // shares
  uint32_t K;
  float2 *row_top2;    // out
  float2 *stage;       // [chunk][ldk], used with more than one chunk
};

__device__ __forceinline__ void fv_merge_row_top2(const fv_merge_args &a, uint32_t block) {
  __shared__ float2 sh_pair[8][FV_MERGE_NEURONS];
  const uint32_t groups = (a.K + FV_MERGE_NEURONS - 1) / FV_MERGE_NEURONS;
  const uint32_t chunks = (a.n_part + FV_MERGE_CHUNK - 1) / FV_MERGE_CHUNK;
  const uint32_t group = block % groups, chunk = block / groups;
  const uint32_t first = chunk * FV_MERGE_CHUNK, last = min(first + FV_MERGE_CHUNK, a.n_part);  // shares [first, last)
  const uint32_t hh = threadIdx.x & (FV_MERGE_NEURONS - 1), bl = threadIdx.x / FV_MERGE_NEURONS;
  const bool real = group * FV_MERGE_NEURONS + hh < a.K;
  const uint32_t h = min(group * FV_MERGE_NEURONS + hh, a.K - 1);  // past K: the last neuron once more, not stored
  float m1 = 0.0f, m2 = 0.0f;
  for (uint32_t b0 = first + bl; b0 < last; b0 += 64) {
    float2 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = a.part[(uint64_t)min(b0 + 8u * u, last - 1) * a.stride + h];
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (b0 + 8u * u < last) fv_top2_merge(m1, m2, v[u].x, v[u].y);
  }
  sh_pair[bl][hh] = make_float2(m1, m2);
  __syncthreads();
  if (bl == 0 && real) {
    for (int i = 1; i < 8; ++i) fv_top2_merge(m1, m2, sh_pair[i][hh].x, sh_pair[i][hh].y);
    float2 *out = chunks == 1 ? a.row_top2 : a.stage + (uint64_t)chunk * a.stride;
    out[h] = make_float2(m1, m2);
  }
}

__global__ __launch_bounds__(256) void fv_merge_shares_kernel(fv_merge_args a) { fv_merge_row_top2(a, blockIdx.x); }

__global__ __launch_bounds__(256) void fv_merge_stage_kernel(fv_merge_args a) {
  const uint32_t h = blockIdx.x * 256 + threadIdx.x;
  if (h >= a.K) return;
  const uint32_t chunks = (a.n_part + FV_MERGE_CHUNK - 1) / FV_MERGE_CHUNK;
  float m1 = 0.0f, m2 = 0.0f;
  for (uint32_t c = 0; c < chunks; ++c) {
    const float2 b = a.stage[(uint64_t)c * a.stride + h];
    fv_top2_merge(m1, m2, b.x, b.y);
  }
  a.row_top2[h] = make_float2(m1, m2);
}
