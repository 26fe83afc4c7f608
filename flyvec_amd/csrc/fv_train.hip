// The FlyVec training minibatch step on one MI355X.
//
// Replaces the kernel chain of flyvec/src/cuda_funcs.cu:1662-1803 (sparse input, frequency
// scaling, Lmid = Lbase = 1, delta = 0, p = 2).  The reference materialises ds (K x N) and
// walks it five times per step; here ds is never stored and nothing uses global atomics:
//
//   1. gather+winner   one wavefront per window: sampler (cuda_funcs.cu:915-936), raw
//                      activation = sum of ~w token rows of the token-major matrix with the K
//                      neurons spread over lanes (:248-263, double accumulators, one rounding),
//                      argmax by a wave reduction (:488-561) and the winner's frequency-scaled
//                      activation (:289-305; it is only ever read at the winner, :731).
//   2. neuron owners   one block per neuron h: the ordered list of windows h won; xx[h] = sum of
//                      their scaled activations in window order (:722-744 -- the reference's
//                      atomic order is undefined, this one is fixed, so a step is reproducible
//                      bit for bit); then the sparse Hebbian term of row h (:657-672): the block
//                      alone owns elements (h, token), so it counts repeated tokens in LDS, and
//                      for each distinct token saves the true weight and the count in a slot
//                      record, evaluates ds there, and plants a sentinel in W.
//   3. max|ds|         dense pass: ds = -xx[h] * W (:394-406), sentinel elements skipped; block
//                      maxima (cu_special_reduction.cu:26-99, 153-189).
//   4. update          W += s * ds where |s * ds| > 1e-10, s = eps / max(prec, max|ds|), rows
//                      with xx == 0 untouched (cuda_funcs.cu:1797-1799,
//                      cu_special_reduction.cu:316-354); dense blocks leave sentinels alone,
//                      slot blocks of the same launch write the final value over each sentinel.
//
// Every one of the n additions of 1/f onto ds[h][i] adds the same value, so the reference's
// result for that element depends only on n; replaying n sequential fp32 adds reproduces it
// exactly whatever order its atomics ran in.
#include <math.h>
#include <string.h>

#include <vector>

#include "fv_internal.h"
#include "fv_repeat_add.h"

// Written over W[p] while the true weight of a sparse element waits in its slot record. A quiet
// NaN with a payload no arithmetic produces.
#define FV_SENTINEL 0x7fc5ca1eu
#define FV_SLOT_INVALID 0xffffffffu

struct fv_slot {
  uint32_t p;  // element index i * ldk + h, or FV_SLOT_INVALID
  uint32_t n;  // pending additions of 1/f
  float wv;    // the weight the sentinel replaced
};

struct fv_trainer {
  fv_train_config cfg;
  uint32_t K, ldk, w, B;
  uint64_t V, N;
  uint32_t total4;  // N * ldk / 4 (float4 elements of the matrix)
  hipStream_t stream;
  float *Wt;
  int32_t *corpus;
  uint64_t n_tokens;
  uint64_t *starts, *perm;
  uint64_t n_windows;
  float *invf;
  int32_t *idx;     // B x w column indices of the current minibatch
  int32_t *win;     // B winners
  float *sc;        // B scaled activations at the winner
  uint32_t *order;  // B window ids grouped by winner, ascending inside a group
  uint32_t nb_chunk;  // column counters per LDS pass of the neuron kernel
  fv_slot *slots;   // B x w slot records
  float *xx;        // ldk
  float *emax;      // K: max|ds| over the sparse elements of each neuron
  float *bmax;      // dense_blocks: max|ds| of each dense block
  float *scalars;   // [0] max|ds| of the last step
  uint32_t last_n;
  uint64_t shuffle_calls;
  bool have_corpus, have_weights;
  unsigned dense_blocks;
  float update_cut;  // largest fp32 <= 1e-10
};

// ---- kernel 1: sampler + gather-sum + winner ----------------------------------------------------

struct fv_gather_args {
  const float *Wt;
  const int32_t *corpus;
  const uint64_t *starts;
  const uint64_t *perm;
  const float *invf;
  int32_t *idx;
  int32_t *win;
  float *sc;
  uint64_t first;
  uint32_t n, K, ldk, w, V, tie_rule;
};

// acc[j] += W[idx_c][lane + 64 j] for every window position c, in order; positions are taken
// RB at a time so RB * NV independent loads are in flight per lane.
template <int NV, int RB, typename Acc>
__device__ __forceinline__ void fv_gather_accumulate(const float *__restrict__ Wt, uint32_t ldk,
                                                     uint32_t K, uint32_t n_cols, int lane, int w,
                                                     int32_t idx_lane, Acc (&acc)[NV]) {
  for (int c0 = 0; c0 < w; c0 += RB) {
    float v[RB][NV];
#pragma unroll
    for (int b = 0; b < RB; ++b) {
      const int c = c0 + b;
      const int32_t i = (int32_t)fv_readlane((uint32_t)idx_lane, c < 63 ? c : 63);
      const bool ok = (c < w) && ((uint32_t)i < n_cols);
      const float *row = Wt + (uint64_t)(ok ? i : 0) * ldk + lane;
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        const bool in = ok && (j < NV - 1 || (uint32_t)(lane + 64 * j) < K);
        v[b][j] = in ? row[64 * j] : 0.0f;
      }
    }
#pragma unroll
    for (int b = 0; b < RB; ++b)
#pragma unroll
      for (int j = 0; j < NV; ++j) acc[j] = acc[j] + (Acc)v[b][j];
  }
}

template <int NV>
struct fv_rows_per_batch {
  static constexpr int value = NV <= 2 ? 16 : NV <= 4 ? 8 : NV <= 8 ? 4 : NV <= 16 ? 2 : 1;
};

template <int NV>
__global__ __launch_bounds__(256) void fv_gather_winner_kernel(fv_gather_args a) {
  const int lane = threadIdx.x & 63;
  const uint32_t r = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= a.n) return;

  // sampler: lane c holds column index c of the window (flyvec/src/cuda_funcs.cu:915-936)
  int32_t idx = -1;
  if (lane < (int)a.w) {
    const uint64_t s = a.starts[a.perm[a.first + r]];
    const int32_t tok = a.corpus[s + lane];
    idx = tok < 0 ? -1 : (lane == (int)(a.w / 2) ? tok + (int32_t)a.V : tok);
    a.idx[(uint64_t)r * a.w + lane] = idx;
  }

  double acc[NV];
#pragma unroll
  for (int j = 0; j < NV; ++j) acc[j] = 0.0;
  fv_gather_accumulate<NV, fv_rows_per_batch<NV>::value, double>(a.Wt, a.ldk, a.K, 2 * a.V, lane,
                                                                 (int)a.w, idx, acc);

  // argmax of the raw activation. Ties: the smaller tie key wins. Key = neuron index (lowest
  // index wins), or the position of the neuron in the reference's reduction order: its 64
  // threads each scan a stride-64 class (= this lane's values, ascending), warp 0 beats warp 1,
  // and inside a warp the shuffle-down tree prefers lanes in bit-reversed order.
  const uint32_t lane_rank = ((uint32_t)lane & 32u) | (__brev((uint32_t)lane & 31u) >> 27);
  uint64_t best = 0;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const uint32_t h = lane + 64 * j;
    const bool valid = (j < NV - 1) || h < a.K;
    const uint32_t key = a.tie_rule ? ((lane_rank << 16) | (uint32_t)j) : h;
    const uint64_t pk = ((uint64_t)fv_ord_key((float)acc[j]) << 32) | (0xffffffffu - key);
    best = (valid && pk > best) ? pk : best;
  }
  best = fv_wave_max_u64(best);
  const uint32_t bkey = 0xffffffffu - (uint32_t)best;
  uint32_t hstar;
  if (a.tie_rule) {
    const uint32_t rank = bkey >> 16;
    hstar = (bkey & 0xffffu) * 64 + ((rank & 32u) | (__brev(rank & 31u) >> 27));
  } else {
    hstar = bkey;
  }

  // frequency-scaled activation of the winner: fp32 products, double sum in window order
  double pd = 0.0;
  if ((uint32_t)idx < 2 * a.V) {
    const float wv = a.Wt[(uint64_t)idx * a.ldk + hstar];
    const float f = a.invf[(uint32_t)idx >= a.V ? (uint32_t)idx - a.V : (uint32_t)idx];
    pd = (double)__fmul_rn(wv, f);
  }
  double s = 0.0;
  for (int c = 0; c < (int)a.w; ++c) {
    const uint64_t bits = (uint64_t)__double_as_longlong(pd);
    const uint64_t got = ((uint64_t)fv_readlane((uint32_t)(bits >> 32), c) << 32) |
                         fv_readlane((uint32_t)bits, c);
    s = s + __longlong_as_double((long long)got);
  }
  if (lane == 0) {
    a.win[r] = (int32_t)hstar;
    a.sc[r] = (float)s;
  }
}

// ---- kernel 2: one block per neuron -- its windows, xx, and its sparse elements --------------------

#define FV_NB_THREADS 1024
#define FV_NB_WAVES (FV_NB_THREADS / 64)
#define FV_NB_MAX_CHUNK 32768  // column counters per LDS pass (128 KB of the CU's 160 KB)
#define FV_NB_SC_CACHE 2048

struct fv_neuron_args {
  const int32_t *win;
  const float *sc;
  const int32_t *idx;
  const float *invf;
  float *Wt;
  float *xx;
  float *emax;
  uint32_t *order;
  fv_slot *slots;
  uint32_t n, K, ldk, w, V, chunk;
};

// ds of one sparse element: the dense term, then n sequential additions of 1/f.
__device__ __forceinline__ float fv_sparse_ds(float xx, float wv, float f, uint32_t n) {
  return fv_add_repeat(__fmul_rn(-xx, wv), f, n);
}

__device__ __forceinline__ float fv_absmax_keep(float m, float v) {
  const float a = fabsf(v);
  return a > m ? a : m;  // a NaN never replaces m, as in the reference's comparison
}

// Exclusive prefix sum of one value per thread over the block, and the block total.
__device__ __forceinline__ uint32_t fv_block_exclusive_scan(uint32_t v, uint32_t *wave_tot /*FV_NB_WAVES+1*/,
                                                            uint32_t *total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  uint32_t incl = v;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const uint32_t o = __shfl_up(incl, d, 64);
    if (lane >= d) incl += o;
  }
  __syncthreads();
  if (lane == 63) wave_tot[wave] = incl;
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t run = 0;
    for (int i = 0; i < FV_NB_WAVES; ++i) {
      const uint32_t t = wave_tot[i];
      wave_tot[i] = run;
      run += t;
    }
    wave_tot[FV_NB_WAVES] = run;
  }
  __syncthreads();
  *total = wave_tot[FV_NB_WAVES];
  return wave_tot[wave] + incl - v;
}

__global__ __launch_bounds__(FV_NB_THREADS) void fv_neuron_kernel(fv_neuron_args a) {
  extern __shared__ uint32_t cnt[];  // a.chunk counters, one per column index of the current pass
  __shared__ float scbuf[FV_NB_SC_CACHE];
  __shared__ uint32_t wave_tot[FV_NB_WAVES + 1];
  __shared__ uint32_t sh_lt, sh_pos;
  __shared__ float sh_xx, sh_wmax[FV_NB_WAVES];

  const uint32_t h = blockIdx.x;
  const uint32_t tid = threadIdx.x;
  const uint32_t n = a.n;
  const int32_t *__restrict__ win = a.win;
  const int32_t *__restrict__ idx = a.idx;

  if (tid == 0) {
    sh_lt = 0;
    sh_pos = 0;
  }
  for (uint32_t i = tid; i < a.chunk / 4; i += FV_NB_THREADS) ((uint4 *)cnt)[i] = make_uint4(0, 0, 0, 0);

  // (1) windows won by lower neurons / by this one. Each thread takes a contiguous segment, so the
  // per-thread match counts scan into window order; matches of the first 64 windows of a segment
  // are remembered as a bit mask so the second walk needs no reload.
  const uint32_t seg = (n + FV_NB_THREADS - 1) / FV_NB_THREADS;
  const uint32_t r0 = min(tid * seg, n), r1 = min(r0 + seg, n);
  uint32_t lt = 0, eq = 0;
  uint64_t mask = 0;
#pragma unroll 8
  for (uint32_t r = r0; r < r1; ++r) {
    const uint32_t wv = (uint32_t)win[r];
    lt += wv < h;
    const bool hit = wv == h;
    eq += hit;
    if (hit && r - r0 < 64) mask |= 1ull << (r - r0);
  }
  __syncthreads();
  {
    uint32_t wl = lt;  // wave-reduce before touching the shared counter
    for (int d = 32; d >= 1; d >>= 1) wl += __shfl_down(wl, d, 64);
    if ((tid & 63) == 0 && wl) atomicAdd(&sh_lt, wl);
  }
  uint32_t c_h;
  const uint32_t my_off = fv_block_exclusive_scan(eq, wave_tot, &c_h);
  const uint32_t base = sh_lt;  // start of this neuron's group in order[]
  {
    uint32_t pos = base + my_off;
    while (mask) {
      a.order[pos++] = r0 + (uint32_t)__ffsll((long long)mask) - 1;
      mask &= mask - 1;
    }
    for (uint32_t r = r0 + 64; r < r1; ++r)
      if ((uint32_t)win[r] == h) a.order[pos++] = r;
  }
  __syncthreads();  // order[base .. base + c_h) is now readable by the whole block
  const uint32_t *__restrict__ order = a.order + base;

  // (2) xx[h]: fp32 adds in window order
  float xx = 0.0f;
  for (uint32_t j0 = 0; j0 < c_h; j0 += FV_NB_SC_CACHE) {
    const uint32_t m = min(c_h - j0, (uint32_t)FV_NB_SC_CACHE);
    for (uint32_t j = tid; j < m; j += FV_NB_THREADS) scbuf[j] = a.sc[order[j0 + j]];
    __syncthreads();
    if (tid == 0) {
#pragma unroll 8
      for (uint32_t j = 0; j < m; ++j) xx = __fadd_rn(xx, scbuf[j]);
    }
    __syncthreads();
  }
  if (tid == 0) {
    sh_xx = xx;
    a.xx[h] = xx;
  }
  __syncthreads();
  xx = sh_xx;

  // (3) sparse elements of row h. The neuron's windows own the slot records [base*w, (base+c_h)*w).
  const uint32_t m_ent = c_h * a.w;
  fv_slot *slots = a.slots + (uint64_t)base * a.w;
  float m = 0.0f;
  uint32_t n_emitted = 0;
  if (xx != 0.0f) {  // (the reference zero-fills ds of a row with xx == 0: no sparse term, no update)
    const uint32_t n_cols = 2 * a.V;
    for (uint32_t lo = 0; lo < n_cols; lo += a.chunk) {
      // count the occurrences of every column index of this pass: one window per thread at a time
      for (uint32_t j = tid; j < c_h; j += FV_NB_THREADS) {
        const int32_t *row = idx + (uint64_t)order[j] * a.w;
        for (uint32_t c = 0; c < a.w; ++c) {
          const int32_t i = row[c];
          const uint32_t k = (uint32_t)i - lo;
          if ((uint32_t)i < n_cols && k < a.chunk) atomicAdd(&cnt[k], 1u);
        }
      }
      __syncthreads();
      // every non-zero counter is one distinct element (h, column): save its weight and count in
      // a slot record, evaluate ds, plant the sentinel; reset the counter for the next pass
      for (uint32_t k4 = tid; k4 < a.chunk / 4; k4 += FV_NB_THREADS) {
        const uint4 c4 = ((const uint4 *)cnt)[k4];
        if ((c4.x | c4.y | c4.z | c4.w) == 0) continue;
        ((uint4 *)cnt)[k4] = make_uint4(0, 0, 0, 0);
        const uint32_t cc[4] = {c4.x, c4.y, c4.z, c4.w};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          if (cc[q] == 0) continue;
          const uint32_t i = lo + k4 * 4 + q;
          fv_slot sl;
          sl.p = i * a.ldk + h;
          sl.n = cc[q];
          sl.wv = a.Wt[sl.p];
          const float f = a.invf[i >= a.V ? i - a.V : i];
          m = fv_absmax_keep(m, fv_sparse_ds(xx, sl.wv, f, sl.n));
          a.Wt[sl.p] = __uint_as_float(FV_SENTINEL);
          slots[atomicAdd(&sh_pos, 1u)] = sl;
        }
      }
      __syncthreads();
    }
    n_emitted = sh_pos;
  }
  for (uint32_t e = n_emitted + tid; e < m_ent; e += FV_NB_THREADS) slots[e].p = FV_SLOT_INVALID;
  const uint32_t wm = fv_wave_max_u32(__float_as_uint(m));  // m >= 0: bit order == value order
  if ((tid & 63) == 0) sh_wmax[tid >> 6] = __uint_as_float(wm);
  __syncthreads();
  if (tid == 0) {
    float bm = 0.0f;
    for (int i = 0; i < FV_NB_WAVES; ++i) bm = fmaxf(bm, sh_wmax[i]);
    a.emax[h] = bm;
  }
}

// ---- kernels 3 and 4: dense passes over the matrix ------------------------------------------------

struct fv_dense_args {
  float4 *Wt4;
  const float *xx;
  const float *invf;
  const fv_slot *slots;
  const float *emax;
  float *bmax;
  float *scalars;
  uint32_t total4, ldk4, ldk, V, K, n_slots, slot_blocks, n_bmax;
  float eps, prec, update_cut;
};

__device__ __forceinline__ bool fv_is_sentinel(float w) { return __float_as_uint(w) == FV_SENTINEL; }

__device__ __forceinline__ float fv_dense_ds(float x, float w) {
  return (x != 0.0f && !fv_is_sentinel(w)) ? __fmul_rn(-x, w) : 0.0f;
}

// Block-wide maximum of non-negative floats; result valid in thread 0.
__device__ __forceinline__ float fv_block_max_nonneg(float m, float *smem4) {
  const uint32_t wm = fv_wave_max_u32(__float_as_uint(m));
  __syncthreads();
  if ((threadIdx.x & 63) == 0) smem4[threadIdx.x >> 6] = __uint_as_float(wm);
  __syncthreads();
  return fmaxf(fmaxf(smem4[0], smem4[1]), fmaxf(smem4[2], smem4[3]));
}

__global__ __launch_bounds__(256) void fv_absmax_kernel(fv_dense_args a) {
  extern __shared__ float4 xs4[];  // xx, ldk4 float4
  __shared__ float smem4[4];
  for (uint32_t q = threadIdx.x; q < a.ldk4; q += 256) xs4[q] = ((const float4 *)a.xx)[q];
  __syncthreads();
  const uint32_t stride = gridDim.x * 256;
  const uint32_t dq = stride % a.ldk4;
  uint32_t q = (blockIdx.x * 256 + threadIdx.x) % a.ldk4;
  float m = 0.0f;
  for (uint32_t p4 = blockIdx.x * 256 + threadIdx.x; p4 < a.total4; p4 += stride) {
    const float4 w = a.Wt4[p4];
    const float4 x = xs4[q];
    m = fv_absmax_keep(m, fv_dense_ds(x.x, w.x));
    m = fv_absmax_keep(m, fv_dense_ds(x.y, w.y));
    m = fv_absmax_keep(m, fv_dense_ds(x.z, w.z));
    m = fv_absmax_keep(m, fv_dense_ds(x.w, w.w));
    q += dq;
    if (q >= a.ldk4) q -= a.ldk4;
  }
  const float bm = fv_block_max_nonneg(m, smem4);
  if (threadIdx.x == 0) a.bmax[blockIdx.x] = bm;
}

__global__ __launch_bounds__(256) void fv_update_kernel(fv_dense_args a) {
  extern __shared__ float4 xs4[];
  __shared__ float smem4[4];
  __shared__ float sh_s;
  for (uint32_t q = threadIdx.x; q < a.ldk4; q += 256) xs4[q] = ((const float4 *)a.xx)[q];
  // max|ds| = max over the dense block maxima and the per-neuron sparse maxima
  float nc = 0.0f;
  for (uint32_t i = threadIdx.x; i < a.n_bmax; i += 256) nc = fmaxf(nc, a.bmax[i]);
  for (uint32_t i = threadIdx.x; i < a.K; i += 256) nc = fmaxf(nc, a.emax[i]);
  nc = fv_block_max_nonneg(nc, smem4);
  if (threadIdx.x == 0) {
    sh_s = a.prec > nc ? a.eps / a.prec : a.eps / nc;  // flyvec/src/cuda_funcs.cu:1797-1799
    if (blockIdx.x == 0) a.scalars[0] = nc;
  }
  __syncthreads();
  const float s = sh_s;

  const uint32_t bid = blockIdx.x;
  const uint32_t stride = gridDim.x * 256;
  const uint32_t dq = stride % a.ldk4;
  uint32_t q = (bid * 256 + threadIdx.x) % a.ldk4;
  for (uint32_t p4 = bid * 256 + threadIdx.x; p4 < a.total4; p4 += stride) {
    float4 w = a.Wt4[p4];
    const float4 x = xs4[q];
    const bool s0 = fv_is_sentinel(w.x), s1 = fv_is_sentinel(w.y), s2 = fv_is_sentinel(w.z),
               s3 = fv_is_sentinel(w.w);
    bool c0 = false, c1 = false, c2 = false, c3 = false;
    float d;
    d = __fmul_rn(s, fv_dense_ds(x.x, w.x)); if (fabsf(d) > a.update_cut) { w.x = __fadd_rn(w.x, d); c0 = true; }
    d = __fmul_rn(s, fv_dense_ds(x.y, w.y)); if (fabsf(d) > a.update_cut) { w.y = __fadd_rn(w.y, d); c1 = true; }
    d = __fmul_rn(s, fv_dense_ds(x.z, w.z)); if (fabsf(d) > a.update_cut) { w.z = __fadd_rn(w.z, d); c2 = true; }
    d = __fmul_rn(s, fv_dense_ds(x.w, w.w)); if (fabsf(d) > a.update_cut) { w.w = __fadd_rn(w.w, d); c3 = true; }
    if (s0 | s1 | s2 | s3) {
      // the slot kernel writes the sentinel positions; store the other components one by one
      float *wp = (float *)&a.Wt4[p4];
      if (c0) wp[0] = w.x;
      if (c1) wp[1] = w.y;
      if (c2) wp[2] = w.z;
      if (c3) wp[3] = w.w;
    } else if (c0 | c1 | c2 | c3) {
      a.Wt4[p4] = w;
    }
    q += dq;
    if (q >= a.ldk4) q -= a.ldk4;
  }
}

// Kernel 5: the final value of every sparse element goes over its sentinel. Runs after the dense
// update so no dense thread can mistake a finished element for an ordinary weight.
__global__ __launch_bounds__(256) void fv_slot_update_kernel(fv_dense_args a) {
  const uint32_t e = blockIdx.x * 256 + threadIdx.x;
  if (e >= a.n_slots) return;
  const fv_slot sl = a.slots[e];
  if (sl.p == FV_SLOT_INVALID) return;
  const float nc = a.scalars[0];
  const float s = a.prec > nc ? a.eps / a.prec : a.eps / nc;
  const uint32_t i = sl.p / a.ldk, h = sl.p - i * a.ldk;
  const float f = a.invf[i >= a.V ? i - a.V : i];
  const float v = fv_sparse_ds(a.xx[h], sl.wv, f, sl.n);
  const float d = __fmul_rn(s, v);
  ((float *)a.Wt4)[sl.p] = fabsf(d) > a.update_cut ? __fadd_rn(sl.wv, d) : sl.wv;
}

// ---- row norms (log line of flyvec/src/cuda_funcs.cu:1234-1242) -------------------------------

__global__ __launch_bounds__(256) void fv_row_norm_kernel(const float *__restrict__ Wt, uint64_t N,
                                                          uint32_t ldk, double *__restrict__ out) {
  __shared__ double part[4];
  const uint32_t h = blockIdx.x;
  double acc = 0.0;
  for (uint64_t i = threadIdx.x; i < N; i += 256) {
    const double v = (double)Wt[i * ldk + h];
    acc += v * v;
  }
  for (int d = 32; d >= 1; d >>= 1) acc += __shfl_down(acc, d, 64);
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) out[h] = sqrt(part[0] + part[1] + part[2] + part[3]);
}

// ---- host side ------------------------------------------------------------------------------

static void fv_trainer_free_corpus(fv_trainer *t) {
  (void)hipFree(t->corpus);
  (void)hipFree(t->starts);
  (void)hipFree(t->perm);
  (void)hipFree(t->invf);
  t->corpus = nullptr;
  t->starts = t->perm = nullptr;
  t->invf = nullptr;
  t->n_tokens = t->n_windows = 0;
  t->have_corpus = false;
}

extern "C" int fv_trainer_destroy(fv_trainer *t) {
  if (!t) return FV_OK;
  if (t->stream) (void)hipStreamSynchronize(t->stream);
  fv_trainer_free_corpus(t);
  (void)hipFree(t->Wt);
  (void)hipFree(t->idx);
  (void)hipFree(t->order);
  (void)hipFree(t->slots);
  (void)hipFree(t->emax);
  (void)hipFree(t->bmax);
  (void)hipFree(t->win);
  (void)hipFree(t->sc);
  (void)hipFree(t->xx);
  (void)hipFree(t->scalars);
  if (t->stream) (void)hipStreamDestroy(t->stream);
  delete t;
  return FV_OK;
}

static int fv_trainer_alloc(fv_trainer *t) {
  const size_t elems = (size_t)t->N * t->ldk;
  FV_HIP(hipStreamCreate(&t->stream));
  FV_HIP(hipMalloc((void **)&t->Wt, elems * sizeof(float)));
  FV_HIP(hipMalloc((void **)&t->idx, (size_t)t->B * t->w * sizeof(int32_t)));
  FV_HIP(hipMalloc((void **)&t->win, (size_t)t->B * sizeof(int32_t)));
  FV_HIP(hipMalloc((void **)&t->sc, (size_t)t->B * sizeof(float)));
  FV_HIP(hipMalloc((void **)&t->order, (size_t)t->B * sizeof(uint32_t)));
  FV_HIP(hipMalloc((void **)&t->slots, (size_t)t->B * t->w * sizeof(fv_slot)));
  FV_HIP(hipMalloc((void **)&t->xx, (size_t)t->ldk * sizeof(float)));
  FV_HIP(hipMalloc((void **)&t->emax, (size_t)t->K * sizeof(float)));
  FV_HIP(hipMalloc((void **)&t->bmax, (size_t)t->dense_blocks * sizeof(float)));
  FV_HIP(hipMalloc((void **)&t->scalars, 16 * sizeof(float)));
  FV_HIP(hipMemsetAsync(t->Wt, 0, elems * sizeof(float), t->stream));
  FV_HIP(hipMemsetAsync(t->xx, 0, (size_t)t->ldk * sizeof(float), t->stream));
  FV_HIP(hipMemsetAsync(t->scalars, 0, 16 * sizeof(float), t->stream));
  FV_HIP(hipStreamSynchronize(t->stream));
  // the neuron kernel counts column indices in LDS: as much of the column range per pass as fits
  uint32_t chunk = (uint32_t)((t->N + 255) / 256 * 256);
  if (chunk > FV_NB_MAX_CHUNK) chunk = FV_NB_MAX_CHUNK;
  t->nb_chunk = chunk;
  FV_HIP(hipFuncSetAttribute((const void *)fv_neuron_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                             (int)(chunk * sizeof(uint32_t))));
  return FV_OK;
}

extern "C" int fv_trainer_create(const fv_train_config *cfg, fv_trainer **out_trainer) {
  FV_REQUIRE(cfg && out_trainer, FV_ERR_INVALID, "fv_trainer_create: null argument");
  *out_trainer = nullptr;
  FV_REQUIRE(cfg->hid >= 1 && cfg->hid <= FV_MAX_HID, FV_ERR_INVALID,
             "hid = %u is outside 1..%d", cfg->hid, FV_MAX_HID);
  FV_REQUIRE(cfg->window >= 1 && cfg->window <= FV_MAX_WINDOW, FV_ERR_INVALID,
             "window = %u is outside 1..%d", cfg->window, FV_MAX_WINDOW);
  FV_REQUIRE(cfg->batch >= 1 && cfg->batch <= (1u << 30), FV_ERR_INVALID, "batch = %u is out of range",
             cfg->batch);
  FV_REQUIRE(cfg->vocab >= 1 && cfg->vocab < (1ull << 30), FV_ERR_INVALID,
             "vocab = %llu is out of range", (unsigned long long)cfg->vocab);
  FV_REQUIRE(cfg->tie_rule <= 1, FV_ERR_INVALID, "tie_rule must be 0 or 1");
  FV_REQUIRE(cfg->delta == 0.0f, FV_ERR_INVALID,
             "delta != 0 (anti-Hebbian term on the m-th winner) is not implemented");
  const uint32_t ldk = fv_ldk(cfg->hid);
  const uint64_t N = 2 * cfg->vocab;
  FV_REQUIRE(N * ldk < 0xffffffffull - (1u << 24), FV_ERR_INVALID,
             "synapse matrix of %llu x %u floats exceeds 2^32 elements", (unsigned long long)N, ldk);
  FV_REQUIRE((uint64_t)cfg->batch * cfg->window < (1ull << 31), FV_ERR_INVALID,
             "batch x window = %llu is out of range", (unsigned long long)cfg->batch * cfg->window);
  fv_trainer *t = new fv_trainer();
  memset(t, 0, sizeof *t);
  t->cfg = *cfg;
  t->K = cfg->hid;
  t->ldk = ldk;
  t->w = cfg->window;
  t->B = cfg->batch;
  t->V = cfg->vocab;
  t->N = N;
  t->total4 = (uint32_t)(N * ldk / 4);
  float cut = (float)1.e-10;  // the reference compares fabs(fp32) > 1.e-10 in double
  if ((double)cut > 1.e-10) cut = nextafterf(cut, 0.0f);
  t->update_cut = cut;
  int cus = 0;
  int rc = fv_device_info(nullptr, 0, &cus, nullptr);
  if (rc == FV_OK) {
    uint64_t want = ((uint64_t)t->total4 + 255) / 256;
    uint64_t cap = (uint64_t)(cus > 0 ? cus : 256) * 8;
    t->dense_blocks = (unsigned)(want < cap ? (want ? want : 1) : cap);
    rc = fv_trainer_alloc(t);
  }
  if (rc != FV_OK) {
    fv_trainer_destroy(t);
    return rc;
  }
  *out_trainer = t;
  return FV_OK;
}

extern "C" int fv_trainer_set_corpus(fv_trainer *t, const int32_t *tokens, uint64_t n_tokens,
                                     const uint64_t *offsets, uint64_t n_offsets) {
  FV_REQUIRE(t, FV_ERR_INVALID, "null trainer");
  FV_REQUIRE(tokens && n_tokens > 0, FV_ERR_INVALID, "empty corpus");
  FV_REQUIRE(offsets && n_offsets >= 1, FV_ERR_INVALID, "empty offsets");
  FV_HIP(hipStreamSynchronize(t->stream));
  fv_trainer_free_corpus(t);
  const uint64_t n_chunks = n_offsets - 1;
  uint64_t *off_dev = nullptr;
  int rc = FV_OK;
  hipError_t e = hipMalloc((void **)&t->corpus, n_tokens * sizeof(int32_t));
  if (e == hipSuccess) e = hipMalloc((void **)&t->invf, t->V * sizeof(float));
  if (e == hipSuccess) e = hipMalloc((void **)&off_dev, n_offsets * sizeof(uint64_t));
  if (e == hipSuccess)
    e = hipMemcpyAsync(t->corpus, tokens, n_tokens * sizeof(int32_t), hipMemcpyHostToDevice, t->stream);
  if (e == hipSuccess)
    e = hipMemcpyAsync(off_dev, offsets, n_offsets * sizeof(uint64_t), hipMemcpyHostToDevice, t->stream);
  if (e != hipSuccess) rc = fv_fail(FV_ERR_HIP, "corpus upload failed: %s", hipGetErrorString(e));

  int32_t lo = 0, hi = 0;
  if (rc == FV_OK) rc = fv_dev_inverse_frequency(t->corpus, n_tokens, t->V, t->invf, &lo, &hi, t->stream);
  if (rc == FV_OK && (lo < -1 || (hi >= 0 && (uint64_t)hi >= t->V)))
    rc = fv_fail(FV_ERR_DATA, "token ids span [%d, %d]; allowed are -1 (masked) and 0..%llu", lo, hi,
                 (unsigned long long)(t->V - 1));
  uint64_t nwin = 0;
  if (rc == FV_OK) rc = fv_dev_count_windows(off_dev, n_chunks, t->w, &nwin, t->stream);
  if (rc == FV_OK && nwin) {
    e = hipMalloc((void **)&t->starts, nwin * sizeof(uint64_t));
    if (e == hipSuccess) e = hipMalloc((void **)&t->perm, nwin * sizeof(uint64_t));
    if (e != hipSuccess) rc = fv_fail(FV_ERR_HIP, "window table allocation failed: %s", hipGetErrorString(e));
    if (rc == FV_OK) {
      // Starts are sums of chunk lengths: with non-decreasing offsets that span no more than the
      // corpus, every window lies inside it (the kernels never read past n_tokens).
      const uint64_t span = offsets[n_chunks] - offsets[0];
      bool monotone = true;
      for (uint64_t s = 0; s < n_chunks && monotone; ++s) monotone = offsets[s + 1] >= offsets[s];
      if (!monotone || span > n_tokens)
        rc = fv_fail(FV_ERR_DATA,
                     "offsets are not non-decreasing or describe %llu tokens but the corpus holds %llu",
                     (unsigned long long)span, (unsigned long long)n_tokens);
    }
    if (rc == FV_OK) rc = fv_dev_build_window_starts(off_dev, n_chunks, t->w, t->starts, nwin, t->stream);
    if (rc == FV_OK) {
      std::vector<uint64_t> ident(nwin);
      for (uint64_t i = 0; i < nwin; ++i) ident[i] = i;
      e = hipMemcpy(t->perm, ident.data(), nwin * sizeof(uint64_t), hipMemcpyHostToDevice);
      if (e != hipSuccess) rc = fv_fail(FV_ERR_HIP, "permutation upload failed: %s", hipGetErrorString(e));
    }
  }
  (void)hipFree(off_dev);
  if (rc != FV_OK) {
    fv_trainer_free_corpus(t);
    return rc;
  }
  t->n_tokens = n_tokens;
  t->n_windows = nwin;
  t->have_corpus = true;
  return FV_OK;
}

extern "C" int fv_trainer_num_windows(fv_trainer *t, uint64_t *out_count) {
  FV_REQUIRE(t && out_count, FV_ERR_INVALID, "null argument");
  FV_REQUIRE(t->have_corpus, FV_ERR_STATE, "no corpus set");
  *out_count = t->n_windows;
  return FV_OK;
}

extern "C" int fv_trainer_get_window_starts(fv_trainer *t, uint64_t *out_starts, uint64_t capacity) {
  FV_REQUIRE(t, FV_ERR_INVALID, "null trainer");
  FV_REQUIRE(t->have_corpus, FV_ERR_STATE, "no corpus set");
  FV_REQUIRE(capacity >= t->n_windows, FV_ERR_INVALID, "capacity %llu < %llu windows",
             (unsigned long long)capacity, (unsigned long long)t->n_windows);
  if (t->n_windows) {
    FV_REQUIRE(out_starts, FV_ERR_INVALID, "null output");
    FV_HIP(hipStreamSynchronize(t->stream));
    FV_HIP(hipMemcpy(out_starts, t->starts, t->n_windows * sizeof(uint64_t), hipMemcpyDeviceToHost));
  }
  return FV_OK;
}

extern "C" int fv_trainer_get_inverse_frequency(fv_trainer *t, float *out_invf) {
  FV_REQUIRE(t && out_invf, FV_ERR_INVALID, "null argument");
  FV_REQUIRE(t->have_corpus, FV_ERR_STATE, "no corpus set");
  FV_HIP(hipStreamSynchronize(t->stream));
  FV_HIP(hipMemcpy(out_invf, t->invf, t->V * sizeof(float), hipMemcpyDeviceToHost));
  return FV_OK;
}

extern "C" int fv_trainer_set_weights(fv_trainer *t, const float *W) {
  FV_REQUIRE(t && W, FV_ERR_INVALID, "null argument");
  FV_TRY(fv_upload_weights(W, t->Wt, t->K, t->N, t->ldk, t->stream));
  t->have_weights = true;
  return FV_OK;
}

extern "C" int fv_trainer_get_weights(fv_trainer *t, float *out_W) {
  FV_REQUIRE(t && out_W, FV_ERR_INVALID, "null argument");
  FV_REQUIRE(t->have_weights, FV_ERR_STATE, "no weights set");
  return fv_download_weights(t->Wt, out_W, t->K, t->N, t->ldk, t->stream);
}

static inline uint64_t fv_splitmix64(uint64_t *state) {
  uint64_t z = (*state += 0x9E3779B97F4A7C15ull);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

extern "C" int fv_trainer_shuffle(fv_trainer *t, uint64_t seed) {
  FV_REQUIRE(t, FV_ERR_INVALID, "null trainer");
  FV_REQUIRE(t->have_corpus, FV_ERR_STATE, "no corpus set");
  const uint64_t n = t->n_windows;
  if (n == 0) return FV_OK;
  FV_HIP(hipStreamSynchronize(t->stream));
  std::vector<uint64_t> perm(n);
  FV_HIP(hipMemcpy(perm.data(), t->perm, n * sizeof(uint64_t), hipMemcpyDeviceToHost));
  uint64_t state = seed ^ (0xD1B54A32D192ED03ull * (t->shuffle_calls + 1));
  for (uint64_t i = 0; i < n; ++i) {  // flyvec/src/model_arrays.cu:458-463
    const uint64_t j = fv_splitmix64(&state) % n;
    const uint64_t tmp = perm[i];
    perm[i] = perm[j];
    perm[j] = tmp;
  }
  t->shuffle_calls++;
  FV_HIP(hipMemcpy(t->perm, perm.data(), n * sizeof(uint64_t), hipMemcpyHostToDevice));
  return FV_OK;
}

extern "C" int fv_trainer_set_permutation(fv_trainer *t, const uint64_t *perm, uint64_t n) {
  FV_REQUIRE(t, FV_ERR_INVALID, "null trainer");
  FV_REQUIRE(t->have_corpus, FV_ERR_STATE, "no corpus set");
  FV_REQUIRE(n == t->n_windows, FV_ERR_INVALID, "permutation has %llu entries, the corpus %llu windows",
             (unsigned long long)n, (unsigned long long)t->n_windows);
  if (n == 0) return FV_OK;
  FV_REQUIRE(perm, FV_ERR_INVALID, "null permutation");
  for (uint64_t i = 0; i < n; ++i)
    FV_REQUIRE(perm[i] < n, FV_ERR_DATA, "permutation entry %llu = %llu is not a window index",
               (unsigned long long)i, (unsigned long long)perm[i]);
  FV_HIP(hipStreamSynchronize(t->stream));
  FV_HIP(hipMemcpy(t->perm, perm, n * sizeof(uint64_t), hipMemcpyHostToDevice));
  return FV_OK;
}

extern "C" int fv_trainer_get_permutation(fv_trainer *t, uint64_t *out_perm, uint64_t capacity) {
  FV_REQUIRE(t, FV_ERR_INVALID, "null trainer");
  FV_REQUIRE(t->have_corpus, FV_ERR_STATE, "no corpus set");
  FV_REQUIRE(capacity >= t->n_windows, FV_ERR_INVALID, "capacity too small");
  if (t->n_windows) {
    FV_REQUIRE(out_perm, FV_ERR_INVALID, "null output");
    FV_HIP(hipStreamSynchronize(t->stream));
    FV_HIP(hipMemcpy(out_perm, t->perm, t->n_windows * sizeof(uint64_t), hipMemcpyDeviceToHost));
  }
  return FV_OK;
}

template <int NV>
static void fv_launch_gather(const fv_gather_args &a, hipStream_t stream) {
  hipLaunchKernelGGL(fv_gather_winner_kernel<NV>, dim3((a.n + 3) / 4), dim3(256), 0, stream, a);
}

// Enqueues the kernels of one step; ev (nullable) receives FV_TRAIN_KERNELS + 1 events recorded
// around them.
static int fv_enqueue_step(fv_trainer *t, uint64_t first, uint32_t n, float eps, hipEvent_t *ev) {
  fv_gather_args g;
  g.Wt = t->Wt;
  g.corpus = t->corpus;
  g.starts = t->starts;
  g.perm = t->perm;
  g.invf = t->invf;
  g.idx = t->idx;
  g.win = t->win;
  g.sc = t->sc;
  g.first = first;
  g.n = n;
  g.K = t->K;
  g.ldk = t->ldk;
  g.w = t->w;
  g.V = (uint32_t)t->V;
  g.tie_rule = t->cfg.tie_rule;
  if (ev) FV_HIP(hipEventRecord(ev[0], t->stream));
  switch ((t->K + 63) / 64) {
#define FV_CASE(NV) case NV: fv_launch_gather<NV>(g, t->stream); break;
    FV_CASE(1) FV_CASE(2) FV_CASE(3) FV_CASE(4) FV_CASE(5) FV_CASE(6) FV_CASE(7) FV_CASE(8)
    FV_CASE(9) FV_CASE(10) FV_CASE(11) FV_CASE(12) FV_CASE(13) FV_CASE(14) FV_CASE(15) FV_CASE(16)
    FV_CASE(17) FV_CASE(18) FV_CASE(19) FV_CASE(20) FV_CASE(21) FV_CASE(22) FV_CASE(23) FV_CASE(24)
    FV_CASE(25) FV_CASE(26) FV_CASE(27) FV_CASE(28) FV_CASE(29) FV_CASE(30) FV_CASE(31) FV_CASE(32)
#undef FV_CASE
    default:
      return fv_fail(FV_ERR_INVALID, "hid = %u not supported", t->K);
  }
  if (ev) FV_HIP(hipEventRecord(ev[1], t->stream));
  fv_neuron_args nb;
  nb.win = t->win;
  nb.sc = t->sc;
  nb.idx = t->idx;
  nb.invf = t->invf;
  nb.Wt = t->Wt;
  nb.xx = t->xx;
  nb.emax = t->emax;
  nb.order = t->order;
  nb.slots = t->slots;
  nb.chunk = t->nb_chunk;
  nb.n = n;
  nb.K = t->K;
  nb.ldk = t->ldk;
  nb.w = t->w;
  nb.V = (uint32_t)t->V;
  hipLaunchKernelGGL(fv_neuron_kernel, dim3(t->K), dim3(FV_NB_THREADS), t->nb_chunk * sizeof(uint32_t),
                     t->stream, nb);
  if (ev) FV_HIP(hipEventRecord(ev[2], t->stream));
  fv_dense_args d;
  d.Wt4 = (float4 *)t->Wt;
  d.xx = t->xx;
  d.invf = t->invf;
  d.slots = t->slots;
  d.emax = t->emax;
  d.bmax = t->bmax;
  d.scalars = t->scalars;
  d.total4 = t->total4;
  d.ldk4 = t->ldk / 4;
  d.ldk = t->ldk;
  d.V = (uint32_t)t->V;
  d.K = t->K;
  d.n_slots = n * t->w;
  d.slot_blocks = (d.n_slots + 255) / 256;
  d.n_bmax = t->dense_blocks;
  d.eps = eps;
  d.prec = t->cfg.prec;
  d.update_cut = t->update_cut;
  const size_t smem = (size_t)t->ldk * sizeof(float);
  hipLaunchKernelGGL(fv_absmax_kernel, dim3(t->dense_blocks), dim3(256), smem, t->stream, d);
  if (ev) FV_HIP(hipEventRecord(ev[3], t->stream));
  hipLaunchKernelGGL(fv_update_kernel, dim3(t->dense_blocks), dim3(256), smem, t->stream, d);
  if (ev) FV_HIP(hipEventRecord(ev[4], t->stream));
  hipLaunchKernelGGL(fv_slot_update_kernel, dim3(d.slot_blocks), dim3(256), 0, t->stream, d);
  if (ev) FV_HIP(hipEventRecord(ev[5], t->stream));
  FV_HIP(hipGetLastError());
  t->last_n = n;
  return FV_OK;
}

static int fv_check_step(fv_trainer *t, uint64_t first, uint64_t n) {
  FV_REQUIRE(t, FV_ERR_INVALID, "null trainer");
  FV_REQUIRE(t->have_corpus, FV_ERR_STATE, "no corpus set");
  FV_REQUIRE(t->have_weights, FV_ERR_STATE, "no weights set");
  FV_REQUIRE(n >= 1 && n <= t->B, FV_ERR_INVALID, "step of %llu windows; batch is %u",
             (unsigned long long)n, t->B);
  FV_REQUIRE(first + n <= t->n_windows, FV_ERR_INVALID, "windows [%llu, %llu) exceed the %llu available",
             (unsigned long long)first, (unsigned long long)(first + n),
             (unsigned long long)t->n_windows);
  return FV_OK;
}

extern "C" int fv_trainer_step(fv_trainer *t, uint64_t first_window, uint32_t n_windows, float eps) {
  FV_TRY(fv_check_step(t, first_window, n_windows));
  return fv_enqueue_step(t, first_window, n_windows, eps, nullptr);
}

extern "C" int fv_trainer_epoch_eps(fv_trainer *t, uint64_t epoch_id, uint64_t n_epochs, float *out_eps) {
  FV_REQUIRE(t && out_eps, FV_ERR_INVALID, "null argument");
  // flyvec/src/cuda_funcs.cu:1229: the ratio is fp32, the rest double, rounded to fp32 once
  *out_eps = (float)(t->cfg.initial_learning_rate * (1.0 - ((float)epoch_id) / ((float)n_epochs)));
  return FV_OK;
}

extern "C" int fv_trainer_run_epoch(fv_trainer *t, uint64_t epoch_id, uint64_t n_epochs) {
  FV_REQUIRE(t, FV_ERR_INVALID, "null trainer");
  FV_REQUIRE(t->have_corpus, FV_ERR_STATE, "no corpus set");
  FV_REQUIRE(t->have_weights, FV_ERR_STATE, "no weights set");
  FV_REQUIRE(n_epochs > 0, FV_ERR_INVALID, "n_epochs must be positive");
  float eps = 0.0f;
  FV_TRY(fv_trainer_epoch_eps(t, epoch_id, n_epochs, &eps));
  for (uint64_t k = 0; k < t->n_windows; k += t->B) {
    const uint64_t n = t->n_windows - k < t->B ? t->n_windows - k : t->B;
    FV_TRY(fv_enqueue_step(t, k, (uint32_t)n, eps, nullptr));
  }
  FV_HIP(hipStreamSynchronize(t->stream));
  return FV_OK;
}

extern "C" int fv_trainer_sync(fv_trainer *t) {
  FV_REQUIRE(t, FV_ERR_INVALID, "null trainer");
  FV_HIP(hipStreamSynchronize(t->stream));
  return FV_OK;
}

extern "C" int fv_trainer_get_winners(fv_trainer *t, int32_t *out_winners, uint32_t capacity) {
  FV_REQUIRE(t && out_winners, FV_ERR_INVALID, "null argument");
  FV_REQUIRE(capacity >= t->last_n, FV_ERR_INVALID, "capacity %u < %u windows of the last step", capacity,
             t->last_n);
  FV_HIP(hipStreamSynchronize(t->stream));
  if (t->last_n)
    FV_HIP(hipMemcpy(out_winners, t->win, (size_t)t->last_n * sizeof(int32_t), hipMemcpyDeviceToHost));
  return FV_OK;
}

extern "C" int fv_trainer_get_step_stats(fv_trainer *t, float *out_xx, float *out_max_abs_ds) {
  FV_REQUIRE(t, FV_ERR_INVALID, "null trainer");
  FV_HIP(hipStreamSynchronize(t->stream));
  if (out_xx) FV_HIP(hipMemcpy(out_xx, t->xx, (size_t)t->K * sizeof(float), hipMemcpyDeviceToHost));
  if (out_max_abs_ds) {
    FV_HIP(hipMemcpy(out_max_abs_ds, t->scalars, sizeof(float), hipMemcpyDeviceToHost));
  }
  return FV_OK;
}

extern "C" int fv_trainer_row_norms(fv_trainer *t, uint32_t n_rows, double *out_norms) {
  FV_REQUIRE(t && out_norms, FV_ERR_INVALID, "null argument");
  FV_REQUIRE(t->have_weights, FV_ERR_STATE, "no weights set");
  if (n_rows > t->K) n_rows = t->K;
  if (n_rows == 0) return FV_OK;
  double *d = nullptr;
  FV_HIP(hipMalloc((void **)&d, n_rows * sizeof(double)));
  hipLaunchKernelGGL(fv_row_norm_kernel, dim3(n_rows), dim3(256), 0, t->stream, t->Wt, t->N, t->ldk, d);
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) e = hipMemcpyAsync(out_norms, d, n_rows * sizeof(double), hipMemcpyDeviceToHost, t->stream);
  if (e == hipSuccess) e = hipStreamSynchronize(t->stream);
  (void)hipFree(d);
  if (e != hipSuccess) return fv_fail(FV_ERR_HIP, "row norms failed: %s", hipGetErrorString(e));
  return FV_OK;
}

extern "C" int fv_trainer_time_steps(fv_trainer *t, uint64_t first_window, uint32_t n_steps, float eps,
                                     float *out_total_ms, float *out_kernel_ms) {
  FV_REQUIRE(t && out_total_ms, FV_ERR_INVALID, "null argument");
  FV_REQUIRE(n_steps >= 1, FV_ERR_INVALID, "n_steps must be >= 1");
  FV_TRY(fv_check_step(t, first_window, t->B));
  FV_REQUIRE(first_window + (uint64_t)n_steps * t->B <= t->n_windows, FV_ERR_INVALID,
             "%u steps of %u windows from %llu exceed the %llu available", n_steps, t->B,
             (unsigned long long)first_window, (unsigned long long)t->n_windows);
  hipEvent_t e0, e1;
  FV_HIP(hipEventCreate(&e0));
  FV_HIP(hipEventCreate(&e1));
  int rc = FV_OK;
  FV_HIP(hipStreamSynchronize(t->stream));
  FV_HIP(hipEventRecord(e0, t->stream));
  for (uint32_t s = 0; s < n_steps && rc == FV_OK; ++s)
    rc = fv_enqueue_step(t, first_window + (uint64_t)s * t->B, t->B, eps, nullptr);
  FV_HIP(hipEventRecord(e1, t->stream));
  FV_HIP(hipStreamSynchronize(t->stream));
  FV_HIP(hipEventElapsedTime(out_total_ms, e0, e1));
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (rc != FV_OK || !out_kernel_ms) return rc;

  const int per = FV_TRAIN_KERNELS + 1;
  std::vector<hipEvent_t> ev((size_t)n_steps * per);
  for (auto &e : ev) FV_HIP(hipEventCreate(&e));
  for (uint32_t s = 0; s < n_steps && rc == FV_OK; ++s)
    rc = fv_enqueue_step(t, first_window + (uint64_t)s * t->B, t->B, eps, &ev[(size_t)s * per]);
  FV_HIP(hipStreamSynchronize(t->stream));
  for (int k = 0; k < FV_TRAIN_KERNELS; ++k) out_kernel_ms[k] = 0.0f;
  if (rc == FV_OK) {
    for (uint32_t s = 0; s < n_steps; ++s)
      for (int k = 0; k < FV_TRAIN_KERNELS; ++k) {
        float ms = 0.0f;
        FV_HIP(hipEventElapsedTime(&ms, ev[(size_t)s * per + k], ev[(size_t)s * per + k + 1]));
        out_kernel_ms[k] += ms / (float)n_steps;
      }
  }
  for (auto &e : ev) (void)hipEventDestroy(e);
  return rc;
}
