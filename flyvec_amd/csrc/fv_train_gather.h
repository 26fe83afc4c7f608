// Kernel 1 of the training step (device code of fv_train.hip).
#pragma once

#include "fv_train_top2.h"

// ---- kernel 1: sampler + gather-sum + winner ----------------------------------------------------

struct fv_gather_args {
  const float *Wt;
  const int32_t *corpus;
  const uint64_t *pstart;  // start of every window, in the current order
  const float *invf;
  int32_t *idx;
  int32_t *win;
  uint16_t *win16;  // the same winners as 16-bit values, for the grouping kernel
  uint32_t *won;        // not null: bit r of row hstar is set (atomic OR; the rows are zero before)
  uint32_t *won2;       // not null (anti-Hebbian form): the same for the window's second neuron
  uint32_t won_words;
  float *sc;
  // anti-Hebbian form only: the second neuron of every window and its scaled activation
  int32_t *win2;
  uint16_t *win2_16;
  float *sc2;
  uint64_t first;
  uint32_t n, K, ldk, w, V, tie_rule;
  uint32_t stride;   // entries per row of idx: w rounded up to 4, the ones past w hold -1
  uint32_t sampled;  // idx already holds this minibatch
  uint32_t n_fresh;  // windows the sampler fills (not sampled): the rows from there on keep what idx holds
  uint32_t prune;    // in-window duplicate pruning while sampling
  float lmid, lbase; // weight of a window's centre position and of the others (WEIGHTED kernels)
  // the first merge_rows blocks of the launch merge the shares of the rows' two largest weights that the
  // last dense launches left (fv_merge_row_top2: a block per 32 neurons and chunk of shares); 0: none
  uint32_t merge_rows;
  fv_merge_args merge;
};

// FV_GATHER_WINDOWS windows per wavefront, one after the other: the grid then fits the machine in
// one round (a second round of waves cost more than the longer life of each wave). The tokens of
// all the wave's windows are fetched up front.
#ifndef FV_GATHER_WINDOWS
#define FV_GATHER_WINDOWS 1
#endif

template <int NV, bool DELTA, bool WEIGHTED>
__device__ __forceinline__ void fv_gather_one_window(const fv_gather_args &a, uint32_t r, int32_t idx, int lane);

// In-window duplicate pruning of the reference's switched-off sampler variant
// (flyvec/src/cuda_funcs.cu:938-979): for i = 1 .. w-1 every position >= i holding the current value
// of position i-1 becomes -1, then the centre gets its token back. A first occurrence is never
// pruned, so that is: a position other than the centre loses its token if an earlier position holds
// the same one. Lane c holds the token of position c; called by the lanes below w together.
__device__ __forceinline__ int32_t fv_prune_token(int32_t tok, int lane, int w) {
  bool dup = false;
  for (int j = 0; j + 1 < w; ++j) {
    const int32_t earlier = (int32_t)fv_readlane((uint32_t)tok, j);
    dup = dup || (lane > j && earlier == tok);
  }
  return (dup && lane != w / 2) ? -1 : tok;
}

// Column index of position c of a window from its token: a masked token stays -1, the centre token
// addresses the target block (flyvec/src/cuda_funcs.cu:915-936).
__device__ __forceinline__ int32_t fv_column_index(int32_t tok, uint32_t c, uint32_t w, uint32_t V) {
  return tok < 0 ? -1 : (c == w / 2 ? tok + (int32_t)V : tok);
}

// DELTA: also the window's second neuron (flyvec/src/cuda_funcs.cu:495-548 with num_m = 2), which
// receives the anti-Hebbian terms. WEIGHTED: position weights other than 1 (:266-286, :307-327).
template <int NV, bool DELTA, bool WEIGHTED>
__global__ __launch_bounds__(256) void fv_gather_winner_kernel(fv_gather_args a) {
  // The arguments of the usual path are asked for here, together: the compiler fetches an argument where it is first
  // used, and three or four of those scalar loads, each behind a branch, stood one after the other in front of the
  // first load of a window's ids.
  asm volatile("" ::"s"(a.Wt), "s"(a.idx), "s"(a.invf), "s"(a.win), "s"(a.win16), "s"(a.won), "s"(a.sc), "s"(a.n),
               "s"(a.K), "s"(a.ldk), "s"(a.w), "s"(a.V), "s"(a.tie_rule), "s"(a.stride), "s"(a.sampled),
               "s"(a.n_fresh), "s"(a.won_words), "s"(a.merge_rows));
  if (blockIdx.x < a.merge_rows) {
    fv_merge_row_top2(a.merge, blockIdx.x);
    return;
  }
  const int lane = threadIdx.x & 63;
  const uint32_t g = (blockIdx.x - a.merge_rows) * 4 + (threadIdx.x >> 6);
  const uint32_t per = (a.n + FV_GATHER_WINDOWS - 1) / FV_GATHER_WINDOWS;  // wave g takes windows g, g + per, ...
  if (g >= per) return;

  // sampler: lane c holds column index c of the window (flyvec/src/cuda_funcs.cu:915-936)
  int32_t idx[FV_GATHER_WINDOWS];
#pragma unroll
  for (int k = 0; k < FV_GATHER_WINDOWS; ++k) {
    const uint32_t r = g + k * per;
    idx[k] = -1;
    const bool kept = a.sampled || r >= a.n_fresh;
    if (lane < (int)a.w && r < a.n) {
      if (kept) {
        idx[k] = a.idx[(uint64_t)r * a.stride + lane];
      } else {
        const uint64_t s = a.pstart[a.first + r];
        int32_t tok = a.corpus[s + lane];
        if (a.prune) tok = fv_prune_token(tok, lane, (int)a.w);
        idx[k] = fv_column_index(tok, (uint32_t)lane, a.w, a.V);
      }
    }
    if (!kept && lane < (int)a.stride && r < a.n) a.idx[(uint64_t)r * a.stride + lane] = idx[k];
  }
#pragma unroll
  for (int k = 0; k < FV_GATHER_WINDOWS; ++k) {
    const uint32_t r = g + k * per;
    if (r < a.n) fv_gather_one_window<NV, DELTA, WEIGHTED>(a, r, idx[k], lane);
  }
}

// Argmax over the wave's K values, given as order-preserving keys (neuron h = lane + 64 j in key[j];
// entries past K hold 0 and are never chosen). The largest key is found first (one 32-bit maximum
// per register, one wave reduction); among the neurons that hold it the smaller tie key wins. Tie
// key = neuron index (lowest index wins: the first set bit of a ballot per register), or the position
// of the neuron in the reference's reduction order: its 64 threads each scan a stride-64 class (= this
// lane's values, ascending), warp 0 beats warp 1, and inside a warp the shuffle-down tree prefers
// lanes in bit-reversed order (flyvec/src/cuda_funcs.cu:488-561).
template <int NV>
__device__ __forceinline__ uint32_t fv_wave_argmax(const uint32_t (&key)[NV], uint32_t K, uint32_t tie_rule, int lane) {
  uint32_t m = key[0];
#pragma unroll
  for (int j = 1; j < NV; ++j) m = max(m, key[j]);
  const uint32_t top = fv_wave_max_u32(m);
  const bool last_valid = (uint32_t)lane + 64u * (NV - 1) < K;
  if (tie_rule == 0) {
    uint32_t best = 0xffffffffu;
#pragma unroll
    for (int j = NV - 1; j >= 0; --j) {
      const uint64_t hits = __ballot(key[j] == top && (j < NV - 1 || last_valid));
      if (hits) best = 64u * j + (uint32_t)__ffsll((long long)hits) - 1u;  // lower registers overwrite higher ones
    }
    return best;
  }
  const uint32_t lane_rank = ((uint32_t)lane & 32u) | (__brev((uint32_t)lane & 31u) >> 27);
  uint32_t tie = 0xffffffffu;
#pragma unroll
  for (int j = NV - 1; j >= 0; --j)
    if (key[j] == top && (j < NV - 1 || last_valid)) tie = (lane_rank << 16) | (uint32_t)j;
  const uint32_t bkey = fv_wave_min_u32(tie);
  const uint32_t rank = bkey >> 16;
  return (bkey & 0xffffu) * 64 + ((rank & 32u) | (__brev(rank & 31u) >> 27));
}

// Frequency-scaled activation of neuron h for the window whose column index c sits in lane c:
// fp32 products, double sum in window order, one rounding (flyvec/src/cuda_funcs.cu:289-305).
template <bool WEIGHTED>
__device__ __forceinline__ float fv_scaled_activation(const fv_gather_args &a, int32_t idx, uint32_t h) {
  double pd = 0.0;
  if ((uint32_t)idx < 2 * a.V) {
    float wv = a.Wt[(uint64_t)idx * a.ldk + h];
    const float f = a.invf[(uint32_t)idx >= a.V ? (uint32_t)idx - a.V : (uint32_t)idx];
    if (WEIGHTED) wv = __fmul_rn(wv, (uint32_t)idx >= a.V ? a.lmid : a.lbase);  // (W * L) * 1/f, :307-327
    pd = (double)__fmul_rn(wv, f);
  }
  double s = 0.0;
  for (int c = 0; c < (int)a.w; ++c) {
    const uint64_t bits = (uint64_t)__double_as_longlong(pd);
    const uint64_t got = ((uint64_t)fv_readlane((uint32_t)(bits >> 32), c) << 32) |
                         fv_readlane((uint32_t)bits, c);
    s = s + __longlong_as_double((long long)got);
  }
  return (float)s;
}

template <int NV, bool DELTA, bool WEIGHTED>
__device__ __forceinline__ void fv_gather_one_window(const fv_gather_args &a, uint32_t r, int32_t idx, int lane) {
  double acc[NV];
#pragma unroll
  for (int j = 0; j < NV; ++j) acc[j] = 0.0;
  fv_gather_accumulate<NV, fv_rows_per_batch<NV>::value, double, WEIGHTED>(a.Wt, a.ldk, a.K, 2 * a.V, lane,
                                                                           (int)a.w, idx, acc, a.lmid, a.lbase);
  // the search runs on order-preserving keys of the fp32 activations; entries past K sort lowest
  uint32_t key[NV];
#pragma unroll
  for (int j = 0; j < NV; ++j)
    key[j] = (j < NV - 1 || (uint32_t)lane + 64u * j < a.K) ? fv_ord_key((float)acc[j]) : 0u;
  const uint32_t hstar = fv_wave_argmax<NV>(key, a.K, a.tie_rule, lane);
  // the scaled activation is only ever read at the chosen neurons (flyvec/src/cuda_funcs.cu:731)
  const float s = fv_scaled_activation<WEIGHTED>(a, idx, hstar);
  if (lane == 0) {
    a.win[r] = (int32_t)hstar;
    a.win16[r] = (uint16_t)hstar;
    a.sc[r] = s;
    // The window's bit in the winner's row, last: behind a branch the compiler waits for everything in flight,
    // and issued before the scaled activation the atomic's trip to memory stood in front of that one's loads.
    if (a.won && hstar < a.K) atomicOr(&a.won[(uint64_t)hstar * a.won_words + (r >> 5)], 1u << (r & 31u));
  }
  // the wave of the step's last window fills the 16-bit winners up to the next multiple of 64 with a
  // value no neuron has
  if (r == a.n - 1 && r + 1 + lane < ((a.n + 63) & ~63u)) a.win16[r + 1 + lane] = 0x7fffu;
  if (DELTA) {
    // flyvec/src/cuda_funcs.cu:495-548: the winner's activation becomes -9999.9999, the search repeats
    const uint32_t lost = fv_ord_key((float)-9999.9999);
#pragma unroll
    for (int j = 0; j < NV; ++j)
      if ((uint32_t)lane + 64u * j == hstar) key[j] = lost;
    const uint32_t second = fv_wave_argmax<NV>(key, a.K, a.tie_rule, lane);
    const float s2 = fv_scaled_activation<WEIGHTED>(a, idx, second);
    if (lane == 0) {
      a.win2[r] = (int32_t)second;
      a.win2_16[r] = (uint16_t)second;
      a.sc2[r] = s2;
      if (a.won2 && second < a.K) atomicOr(&a.won2[(uint64_t)second * a.won_words + (r >> 5)], 1u << (r & 31u));
    }
  }
}
