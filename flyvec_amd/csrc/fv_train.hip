// The FlyVec training minibatch step on one MI355X.
//
// Replaces the kernel chain of flyvec/src/cuda_funcs.cu:1662-1803 (sparse input, frequency
// scaling, Lmid = Lbase = 1, delta = 0, p = 2).  The reference materialises ds (K x N) and
// walks it five times per step; here ds is never stored:
//
//   1. gather+winner   one wavefront per window: sampler (cuda_funcs.cu:915-936), raw
//                      activation = sum of ~w token rows of the token-major matrix with the K
//                      neurons spread over lanes (:248-263, double accumulators, one rounding),
//                      argmax by a wave reduction (:488-561), the winner's frequency-scaled
//                      activation (:289-305, needed only at the winner, :731), and the sparse
//                      Hebbian term recorded as integer counts per (winner, token) plus one
//                      flag bit per 4 matrix elements (:657-672).
//   2. xx totals       xx[h] = sum of the scaled activations of the windows h won, added in
//                      window order (:722-744; the reference's atomic order is undefined, this
//                      one is fixed so a step is reproducible bit for bit).
//   3. max|ds|         ds = -xx[h] * W + count * (1/f) re-derived on the fly from W, xx and the
//                      flagged counts; grid-wide maximum of |ds| (:394-406,
//                      cu_special_reduction.cu:26-99, 153-189).
//   4. update          W += s * ds where |s * ds| > 1e-10, s = eps / max(prec, max|ds|), rows
//                      with xx == 0 untouched (cuda_funcs.cu:1797-1799,
//                      cu_special_reduction.cu:316-354); clears the counts and flags it consumed.
//
// Because every one of the n additions of 1/f onto ds[h][i] adds the same value, the
// reference's result for that element depends only on n; replaying n sequential fp32 adds
// reproduces it exactly whatever order its atomics ran in.
#include <math.h>
#include <string.h>

#include <vector>

#include "fv_internal.h"

struct fv_trainer {
  fv_train_config cfg;
  uint32_t K, ldk, w, B;
  uint64_t V, N;
  uint32_t total4;  // N * ldk / 4 (float4 elements of the matrix)
  hipStream_t stream;
  float *Wt;
  uint32_t *cnt;    // per matrix element: additions of 1/f pending for the current step
  uint32_t *flags;  // bit g set <=> some cnt in float4 group g is non-zero
  int32_t *corpus;
  uint64_t n_tokens;
  uint64_t *starts, *perm;
  uint64_t n_windows;
  float *invf;
  int32_t *win;
  float *sc;
  float *xx;
  uint32_t *scalars;  // [0] bits of max|ds| of the current step
  uint32_t last_n;
  uint64_t shuffle_calls;
  bool have_corpus, have_weights;
  unsigned dense_blocks;
  float update_cut;  // largest fp32 <= 1e-10
};

// ---- kernel 1: sampler + gather-sum + winner + sparse counts ---------------------------------

struct fv_gather_args {
  const float *Wt;
  const int32_t *corpus;
  const uint64_t *starts;
  const uint64_t *perm;
  const float *invf;
  uint32_t *cnt;
  uint32_t *flags;
  int32_t *win;
  float *sc;
  uint32_t *scalars;
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
  if (blockIdx.x == 0 && threadIdx.x == 0) a.scalars[0] = 0;  // max|ds| of this step starts at 0
  if (r >= a.n) return;

  // sampler: lane c holds column index c of the window (flyvec/src/cuda_funcs.cu:915-936)
  int32_t idx = -1;
  if (lane < (int)a.w) {
    const uint64_t s = a.starts[a.perm[a.first + r]];
    const int32_t tok = a.corpus[s + lane];
    idx = tok < 0 ? -1 : (lane == (int)(a.w / 2) ? tok + (int32_t)a.V : tok);
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
  const bool ok = (uint32_t)idx < 2 * a.V;
  double pd = 0.0;
  uint64_t p = 0;
  if (ok) {
    p = (uint64_t)idx * a.ldk + hstar;
    const float wv = a.Wt[p];
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

  // sparse Hebbian term: one more pending addition of 1/f at (winner, token)
  if (ok) {
    atomicAdd(&a.cnt[p], 1u);
    atomicOr(&a.flags[p >> 7], 1u << ((p >> 2) & 31));
  }
}

// ---- kernel 2: xx[h] = sum over the windows h won, in window order ------------------------------

__global__ __launch_bounds__(256) void fv_xx_totals_kernel(const int32_t *__restrict__ win,
                                                           const float *__restrict__ sc, uint32_t n,
                                                           uint32_t K, uint32_t ldk,
                                                           float *__restrict__ xx) {
  const int lane = threadIdx.x & 63;
  const uint32_t h = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (h >= ldk) return;
  float acc = 0.0f;
  if (h < K) {
    for (uint32_t base = 0; base < n; base += 64) {
      const uint32_t r = base + lane;
      const int32_t wv = r < n ? win[r] : -1;
      uint64_t m = __ballot(wv == (int32_t)h);
      if (m) {
        const float sv = r < n ? sc[r] : 0.0f;
        while (m) {
          const int l = __ffsll((long long)m) - 1;
          acc = __fadd_rn(acc, __uint_as_float(fv_readlane(__float_as_uint(sv), l)));
          m &= m - 1;
        }
      }
    }
  }
  if (lane == 0) xx[h] = acc;
}

// ---- kernels 3 and 4: dense passes over the matrix ------------------------------------------------

struct fv_dense_args {
  float4 *Wt4;
  uint4 *cnt4;
  uint64_t *flags64;
  const float *xx;
  const float *invf;
  uint32_t *scalars;
  uint32_t total4, ldk4, V;
  float eps, prec, update_cut;
};

// ds for the 4 consecutive neurons of one token held by this lane.
__device__ __forceinline__ float4 fv_ds_value(const float4 w, const float4 x, bool flagged,
                                              const uint4 *__restrict__ cnt4, uint32_t p4,
                                              uint32_t ldk4, const float *__restrict__ invf,
                                              uint32_t V) {
  float4 v;
  v.x = x.x != 0.0f ? __fmul_rn(-x.x, w.x) : 0.0f;
  v.y = x.y != 0.0f ? __fmul_rn(-x.y, w.y) : 0.0f;
  v.z = x.z != 0.0f ? __fmul_rn(-x.z, w.z) : 0.0f;
  v.w = x.w != 0.0f ? __fmul_rn(-x.w, w.w) : 0.0f;
  if (flagged) {
    const uint4 n = cnt4[p4];
    const uint32_t i = p4 / ldk4;  // token row; the target block repeats the frequencies
    const float f = invf[i >= V ? i - V : i];
    if (x.x != 0.0f) for (uint32_t t = 0; t < n.x; ++t) v.x = __fadd_rn(v.x, f);
    if (x.y != 0.0f) for (uint32_t t = 0; t < n.y; ++t) v.y = __fadd_rn(v.y, f);
    if (x.z != 0.0f) for (uint32_t t = 0; t < n.z; ++t) v.z = __fadd_rn(v.z, f);
    if (x.w != 0.0f) for (uint32_t t = 0; t < n.w; ++t) v.w = __fadd_rn(v.w, f);
  }
  return v;
}

__device__ __forceinline__ float fv_absmax_keep(float m, float v) {
  const float a = fabsf(v);
  return a > m ? a : m;  // a NaN never replaces m, as in the reference's comparison
}

template <bool UPDATE>
__global__ __launch_bounds__(256) void fv_dense_kernel(fv_dense_args a) {
  extern __shared__ float4 xs4[];  // xx, ldk4 float4
  for (uint32_t q = threadIdx.x; q < a.ldk4; q += 256) xs4[q] = ((const float4 *)a.xx)[q];
  __syncthreads();

  float s = 0.0f;
  if (UPDATE) {
    const float nc = __uint_as_float(a.scalars[0]);
    s = a.prec > nc ? a.eps / a.prec : a.eps / nc;  // flyvec/src/cuda_funcs.cu:1797-1799
  }

  const int lane = threadIdx.x & 63;
  const uint32_t stride = gridDim.x * 256;
  const uint32_t dq = stride % a.ldk4;
  uint32_t p4 = blockIdx.x * 256 + threadIdx.x;
  uint32_t q = p4 % a.ldk4;
  float m = 0.0f;
  // The loop bound is taken on the wave's first element so the whole wave iterates together.
  for (uint32_t base = p4 - lane; base < a.total4; base += stride, p4 += stride) {
    const uint64_t fw = a.flags64[__builtin_amdgcn_readfirstlane(base >> 6)];
    if (p4 < a.total4) {
      float4 w = a.Wt4[p4];
      const float4 x = xs4[q];
      const bool flagged = (fw >> lane) & 1;
      const float4 v = fv_ds_value(w, x, flagged, a.cnt4, p4, a.ldk4, a.invf, a.V);
      if (!UPDATE) {
        m = fv_absmax_keep(m, v.x);
        m = fv_absmax_keep(m, v.y);
        m = fv_absmax_keep(m, v.z);
        m = fv_absmax_keep(m, v.w);
      } else {
        bool changed = false;
        float d;
        d = __fmul_rn(s, v.x); if (fabsf(d) > a.update_cut) { w.x = __fadd_rn(w.x, d); changed = true; }
        d = __fmul_rn(s, v.y); if (fabsf(d) > a.update_cut) { w.y = __fadd_rn(w.y, d); changed = true; }
        d = __fmul_rn(s, v.z); if (fabsf(d) > a.update_cut) { w.z = __fadd_rn(w.z, d); changed = true; }
        d = __fmul_rn(s, v.w); if (fabsf(d) > a.update_cut) { w.w = __fadd_rn(w.w, d); changed = true; }
        if (changed) a.Wt4[p4] = w;
        if (flagged) a.cnt4[p4] = make_uint4(0, 0, 0, 0);
      }
    }
    if (UPDATE && fw != 0 && lane == 0) a.flags64[base >> 6] = 0;
    q += dq;
    if (q >= a.ldk4) q -= a.ldk4;
  }

  if (!UPDATE) {
    __shared__ uint32_t wave_max[4];
    const uint32_t wm = fv_wave_max_u32(__float_as_uint(m));  // m >= 0: bit order == value order
    if (lane == 0) wave_max[threadIdx.x >> 6] = wm;
    __syncthreads();
    if (threadIdx.x == 0) {
      uint32_t b = wave_max[0];
      b = wave_max[1] > b ? wave_max[1] : b;
      b = wave_max[2] > b ? wave_max[2] : b;
      b = wave_max[3] > b ? wave_max[3] : b;
      if (b) atomicMax(&a.scalars[0], b);
    }
  }
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
  (void)hipFree(t->cnt);
  (void)hipFree(t->flags);
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
  const size_t flag_words64 = ((size_t)t->total4 + 63) / 64;
  FV_HIP(hipStreamCreate(&t->stream));
  FV_HIP(hipMalloc((void **)&t->Wt, elems * sizeof(float)));
  FV_HIP(hipMalloc((void **)&t->cnt, elems * sizeof(uint32_t)));
  FV_HIP(hipMalloc((void **)&t->flags, flag_words64 * sizeof(uint64_t)));
  FV_HIP(hipMalloc((void **)&t->win, (size_t)t->B * sizeof(int32_t)));
  FV_HIP(hipMalloc((void **)&t->sc, (size_t)t->B * sizeof(float)));
  FV_HIP(hipMalloc((void **)&t->xx, (size_t)t->ldk * sizeof(float)));
  FV_HIP(hipMalloc((void **)&t->scalars, 16 * sizeof(uint32_t)));
  FV_HIP(hipMemsetAsync(t->Wt, 0, elems * sizeof(float), t->stream));
  FV_HIP(hipMemsetAsync(t->cnt, 0, elems * sizeof(uint32_t), t->stream));
  FV_HIP(hipMemsetAsync(t->flags, 0, flag_words64 * sizeof(uint64_t), t->stream));
  FV_HIP(hipMemsetAsync(t->xx, 0, (size_t)t->ldk * sizeof(float), t->stream));
  FV_HIP(hipMemsetAsync(t->scalars, 0, 16 * sizeof(uint32_t), t->stream));
  FV_HIP(hipStreamSynchronize(t->stream));
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
  FV_REQUIRE(N * ldk / 4 < (1ull << 31), FV_ERR_INVALID,
             "synapse matrix of %llu x %u floats exceeds 2^33 elements", (unsigned long long)N, ldk);
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
  g.cnt = t->cnt;
  g.flags = t->flags;
  g.win = t->win;
  g.sc = t->sc;
  g.scalars = t->scalars;
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
  hipLaunchKernelGGL(fv_xx_totals_kernel, dim3((t->ldk + 3) / 4), dim3(256), 0, t->stream, t->win,
                     t->sc, n, t->K, t->ldk, t->xx);
  if (ev) FV_HIP(hipEventRecord(ev[2], t->stream));
  fv_dense_args d;
  d.Wt4 = (float4 *)t->Wt;
  d.cnt4 = (uint4 *)t->cnt;
  d.flags64 = (uint64_t *)t->flags;
  d.xx = t->xx;
  d.invf = t->invf;
  d.scalars = t->scalars;
  d.total4 = t->total4;
  d.ldk4 = t->ldk / 4;
  d.V = (uint32_t)t->V;
  d.eps = eps;
  d.prec = t->cfg.prec;
  d.update_cut = t->update_cut;
  const size_t smem = (size_t)t->ldk * sizeof(float);
  hipLaunchKernelGGL(fv_dense_kernel<false>, dim3(t->dense_blocks), dim3(256), smem, t->stream, d);
  if (ev) FV_HIP(hipEventRecord(ev[3], t->stream));
  hipLaunchKernelGGL(fv_dense_kernel<true>, dim3(t->dense_blocks), dim3(256), smem, t->stream, d);
  if (ev) FV_HIP(hipEventRecord(ev[4], t->stream));
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
    uint32_t bits = 0;
    FV_HIP(hipMemcpy(&bits, t->scalars, sizeof bits, hipMemcpyDeviceToHost));
    memcpy(out_max_abs_ds, &bits, sizeof bits);
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
