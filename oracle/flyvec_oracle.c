/*
 * CPU restatement of the FlyVec training minibatch step and its host set-up.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the HIP library is
 * compared against; nothing in the shipped package may link or call it.
 * It follows the reference sources statement by statement (citations are
 * path:line inside the reference tree) and keeps the reference's data layout
 * (W is K x N row-major, N = 2V) and arithmetic (fp32 products, double
 * accumulation of the window sums, one rounding to fp32; fp32 everywhere
 * else).  Build with -ffp-contract=off so no multiply-add is fused.
 *
 * Pinned by (see tests/test_oracle_*.py):
 *   fvo_count_windows / fvo_window_starts : the reference's own prune_input.cpp
 *       compiled into oracle/_ref (bit-exact on random and edge-case offsets).
 *   fvo_inverse_frequency, fvo_inflate, fvo_activations, fvo_argmax_*,
 *   fvo_train_step, fvo_train_step_delta (the anti-Hebbian term), fvo_epoch_delta : closed forms (one-window batch, W = 0 fixed point,
 *       invariance to a global rescale of 1/frequency by a power of two,
 *       max|dW| == eps), a from-scratch brute force in Python floats on tiny
 *       shapes, and numpy restatements of each stage.
 *   fvo_train_step_weighted (position weights Lmid / Lbase) : the brute force
 *       with weights, and closed forms (a weight of 0 is a masked position; a
 *       common power of two changes no bit of the update; weights under which
 *       centre and context elect different winners).
 *   fvo_prune_windows : the reference's own prune_input_data (oracle/_ref).
 *   fvo_inflate_prune : a set-based first-occurrence formulation in Python.
 *   fvo_train_steps_tail (the reference's re-use of the previous minibatch's
 *       rows on a final partial minibatch) : the single step on an index
 *       matrix assembled by hand from two inflate calls.
 *
 * Order-dependent fp32 sums (the reference uses atomics whose order is not
 * defined) are given a fixed order here.  The sparse term of ds: increasing
 * window order, then increasing position inside the window.  The per-neuron
 * totals xx: see fvo_xx_sums (the minibatch's rows in groups of 64: a
 * neuron's values of a group are added in row order, the groups' sums over the
 * balanced binary tree on the group number).  fvo_xx_sums is pinned by a numpy
 * restatement of that order (halving an array of group sums), by the cases in
 * which it is the plain sum in row order (one group; two groups; one value per
 * group and a power-of-two alignment) and by its agreement with plain row
 * order to rounding, in tests/test_oracle_train.py.
 *
 * Parity unpinned against the reference BINARY in one rounding: the update
 * W += (eps / max|ds|) * ds is written as a multiply and then an add in
 * flyvec/src/cu_special_reduction.cu:341-344, and that is what this file does.
 * The reference is built with plain nvcc -O3, which is allowed to contract the
 * two into one fused multiply-add; without nvcc its choice cannot be read
 * off, so the binary's W may differ from this file's by one ulp per updated
 * element and step.  No fixture of the reference settles it.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define FVO_MAXLEN 214 /* flyvec/src/prune_input.cpp:7 */

int fvo_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* flyvec/src/prune_input.cpp:64-84 (getnum_samples) */
uint64_t fvo_count_windows(const uint64_t *offsets, uint64_t n_chunks, uint64_t w) {
  uint64_t total = 0;
  for (uint64_t s = 0; s < n_chunks; ++s) {
    uint64_t len = offsets[s + 1] - offsets[s];
    if (len >= w && len < FVO_MAXLEN) total += len - w + 1;
  }
  return total;
}

/* flyvec/src/prune_input.cpp:88-122 (compute_offset_phrases): the start of a
 * window is the running sum of ALL previous chunk lengths plus the position
 * inside the chunk; offsets[s] itself is never used as a position. */
void fvo_window_starts(const uint64_t *offsets, uint64_t n_chunks, uint64_t w, uint64_t *starts) {
  uint64_t running = 0, cnt = 0;
  for (uint64_t s = 0; s < n_chunks; ++s) {
    uint64_t len = offsets[s + 1] - offsets[s];
    if (len >= w && len < FVO_MAXLEN)
      for (uint64_t i = 0; i < len - w + 1; ++i) starts[cnt++] = running + i;
    running += len;
  }
}

/* flyvec/src/model_arrays.cu:396-424: counts are accumulated IN FP32 (they stop
 * growing at 2^24), negative ids are ignored, 1/count is formed in double and
 * rounded once, absent ids get 0. */
void fvo_inverse_frequency(const int32_t *corpus, uint64_t n_tok, uint64_t V, float *invf) {
  for (uint64_t i = 0; i < V; ++i) invf[i] = 0.0f;
  for (uint64_t i = 0; i < n_tok; ++i)
    if (corpus[i] >= 0) invf[corpus[i]] = (float)((double)invf[corpus[i]] + 1.0);
  for (uint64_t i = 0; i < V; ++i)
    invf[i] = (invf[i] != 0) ? (float)(1.0 / (double)invf[i]) : 0.0f;
}

/* flyvec/src/cuda_funcs.cu:915-936 (inflate_from_M_kernel_4): window r of the
 * minibatch is the corpus slice at starts[perm[first + r]]; the centre column
 * (c == w/2) is shifted into the target block, masked ids (-1) stay -1. */
void fvo_inflate(const int32_t *corpus, const uint64_t *starts, const uint64_t *perm,
                 uint64_t first, uint64_t n, int w, uint64_t V, int32_t *idx) {
  const int mid = w / 2;
  for (uint64_t r = 0; r < n; ++r) {
    const int32_t *src = corpus + starts[perm[first + r]];
    for (int c = 0; c < w; ++c) {
      int32_t val = src[c];
      idx[r * (uint64_t)w + c] = (val == -1) ? -1 : (c == mid ? (int32_t)(val + (int64_t)V) : val);
    }
  }
}

/* flyvec/src/cuda_funcs.cu:938-979 (inflate_from_M_kernel_4_and_prune, switched off in the reference
 * at :1681): for i = 1 .. w-1 every position c >= i that holds the CURRENT value of position i-1
 * becomes -1; afterwards the centre gets its original token back; then the indices are formed as in
 * fvo_inflate. */
void fvo_inflate_prune(const int32_t *corpus, const uint64_t *starts, const uint64_t *perm,
                       uint64_t first, uint64_t n, int w, uint64_t V, int32_t *idx) {
  const int mid = w / 2;
  int32_t tmp[256];
  for (uint64_t r = 0; r < n; ++r) {
    const int32_t *src = corpus + starts[perm[first + r]];
    for (int c = 0; c < w; ++c) tmp[c] = src[c];
    for (int i = 1; i < w; ++i) {
      int32_t val = tmp[i - 1];
      for (int c = i; c < w; ++c)
        if (tmp[c] == val) tmp[c] = -1;
    }
    tmp[mid] = src[mid];
    for (int c = 0; c < w; ++c)
      idx[r * (uint64_t)w + c] = (tmp[c] == -1) ? -1 : (c == mid ? (int32_t)(tmp[c] + (int64_t)V) : tmp[c]);
  }
}

/* flyvec/src/prune_input.cpp:14-60 (prune_input_data, exported by the reference but never called):
 * rows x cols window matrix in place; scanning a row left to right, a value already kept at an
 * earlier position becomes -1; the centre column takes no part (it counts as -1 while the row is
 * scanned) and keeps its value. */
void fvo_prune_windows(int32_t *data, uint64_t rows, uint64_t cols) {
  const uint64_t mid = cols / 2;
  int32_t *tmp = (int32_t *)malloc(sizeof(int32_t) * (cols ? cols : 1));
  for (uint64_t r = 0; r < rows; ++r) {
    int32_t *row = data + r * cols;
    if (cols == 0) continue;
    tmp[0] = row[0];
    for (uint64_t c = 1; c < cols; ++c) {
      if (c == mid) {
        tmp[c] = -1;
        continue;
      }
      int dup = 0;
      for (uint64_t cc = 0; cc < c && !dup; ++cc) dup = tmp[cc] == row[c];
      tmp[c] = dup ? -1 : row[c];
    }
    tmp[mid] = row[mid];
    for (uint64_t c = 0; c < cols; ++c) row[c] = tmp[c];
  }
  free(tmp);
}

/* flyvec/src/cuda_funcs.cu:248-263 (raw) and :289-305 (scaled by 1/frequency):
 * per window and neuron a double accumulator over the window positions in
 * order, skipping -1; the scaled product is formed in fp32 first. */
void fvo_activations(const float *W, int K, uint64_t N, const int32_t *idx, uint64_t n, int w,
                     const float *invf, uint64_t V, float *raw, float *scaled) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < (int64_t)n; ++r) {
    const int32_t *ix = idx + (uint64_t)r * w;
    for (int h = 0; h < K; ++h) {
      const float *row = W + (uint64_t)h * N;
      double sr = 0.0, ss = 0.0;
      for (int c = 0; c < w; ++c) {
        int32_t i = ix[c];
        if (i != -1) {
          float f = invf[(uint64_t)i % V];
          float prod = row[i] * f; /* fp32 product, cuda_funcs.cu:298-299 */
          ss += (double)prod;
          sr += (double)row[i];
        }
      }
      if (raw) raw[(uint64_t)r * K + h] = (float)sr;
      if (scaled) scaled[(uint64_t)r * K + h] = (float)ss;
    }
  }
}

/* flyvec/src/cuda_funcs.cu:488-561 (get_max_and_m_max_kernel_2, first pass):
 * a literal simulation of the 64 threads: each scans its stride-64 class
 * keeping strictly greater values, seeded with (data[0], 0); a shuffle-down
 * tree inside each 32-lane warp keeps the lower lane on ties; warp 1 replaces
 * warp 0 only when strictly greater. */
int fvo_argmax_reference(const float *data, int K) {
  float val[64];
  int ind[64];
  for (int t = 0; t < 64; ++t) {
    float best = data[0];
    int bi = 0;
    for (int i = t; i < K; i += 64)
      if (data[i] > best) { best = data[i]; bi = i; }
    val[t] = best;
    ind[t] = bi;
  }
  for (int wp = 0; wp < 2; ++wp) {
    float *v = val + 32 * wp;
    int *x = ind + 32 * wp;
    for (int d = 16; d >= 1; d /= 2) {
      float nv[32];
      int nx[32];
      for (int l = 0; l < 32; ++l) {
        /* __shfl_down_sync returns the caller's own value past the warp end */
        float ov = (l + d < 32) ? v[l + d] : v[l];
        int ox = (l + d < 32) ? x[l + d] : x[l];
        if (ov > v[l]) { nv[l] = ov; nx[l] = ox; } else { nv[l] = v[l]; nx[l] = x[l]; }
      }
      memcpy(v, nv, sizeof nv);
      memcpy(x, nx, sizeof nx);
    }
  }
  float best = val[0];
  int bi = ind[0];
  if (val[32] > best) { best = val[32]; bi = ind[32]; }
  return bi;
}

/* Plain argmax, lowest index on ties. */
int fvo_argmax_lowest(const float *data, int K) {
  int bi = 0;
  for (int i = 1; i < K; ++i)
    if (data[i] > data[bi]) bi = i;
  return bi;
}

/* flyvec/src/cuda_funcs.cu:1229 */
float fvo_epoch_eps(float lr0, uint64_t epoch, uint64_t n_epochs) {
  return (float)(lr0 * (1.0 - ((float)epoch) / ((float)n_epochs)));
}

/*
 * xx[h] = sum of sc[r] over the windows r won by h (flyvec/src/cuda_funcs.cu:722-744, fp32 atomics
 * there: the reference's order of additions is not defined).  order_kind 0, the step's order: the rows
 * of the minibatch are taken in groups of 64 consecutive rows; P_g is the sum, onto 0 and in row order,
 * of sc[r] over the rows of group g that h won (0 if none); xx[h] is the sum of P_0, P_1, ... over the
 * balanced binary tree on the group number: node(0, g) = P_g, node(k, i) = node(k-1, 2i) + node(k-1, 2i+1),
 * groups past the last one counting as 0 (a sum onto +0 is never -0, so adding such a 0 changes no bit and
 * the result does not depend on how far the tree is padded).  order_kind 1: every window added onto xx[h]
 * in increasing row order.
 */
#define FVO_XX_GROUP 64
#define FVO_XX_LEVELS 64
void fvo_xx_sums(const int32_t *win, const float *sc, uint64_t n, int K, int order_kind, float *xx) {
  for (int h = 0; h < K; ++h) xx[h] = 0.0f;
  if (order_kind == 1) {
    for (uint64_t r = 0; r < n; ++r) xx[win[r]] = xx[win[r]] + sc[r];
    return;
  }
  /* the tree is evaluated as the groups arrive: stack[h][k] holds a finished node of level k that waits for
   * its right sibling; a neuron's stack after G groups holds the nodes the set bits of G name */
  float *stack = (float *)calloc((size_t)K * FVO_XX_LEVELS, sizeof(float));
  float *part = (float *)calloc((size_t)K, sizeof(float));
  const uint64_t G = (n + FVO_XX_GROUP - 1) / FVO_XX_GROUP;
  for (uint64_t g = 0; g < G; ++g) {
    const uint64_t r1 = (g + 1) * FVO_XX_GROUP < n ? (g + 1) * FVO_XX_GROUP : n;
    for (int h = 0; h < K; ++h) part[h] = 0.0f;
    for (uint64_t r = g * FVO_XX_GROUP; r < r1; ++r) part[win[r]] = part[win[r]] + sc[r];
    for (int h = 0; h < K; ++h) {
      float carry = part[h];
      int level = 0;
      for (uint64_t i = g; i & 1; i >>= 1, ++level) carry = stack[(size_t)h * FVO_XX_LEVELS + level] + carry;
      stack[(size_t)h * FVO_XX_LEVELS + level] = carry;
    }
  }
  for (int h = 0; h < K; ++h) {
    /* the groups from G on are 0: what is left on the stack is added from the lowest level up, each node
     * as the left operand of the partial node to its right */
    float acc = 0.0f;
    int level = 0;
    for (uint64_t i = G; i; i >>= 1, ++level)
      if (i & 1) acc = stack[(size_t)h * FVO_XX_LEVELS + level] + acc;
    xx[h] = acc;
  }
  free(stack);
  free(part);
}

/*
 * One minibatch step on already inflated indices (idx is n x w).
 * Order follows flyvec/src/cuda_funcs.cu:1662-1803 for sparse_input = 1,
 * frequency_scaling = 1, Lmid = Lbase = 1, delta = 0, p = 2:
 *   :1688        ds <- W                      (cuda_func1_odd, p-1 = 1: a copy)
 *   :1700-1701   scaled and raw activations   (from that copy, i.e. from W)
 *   :1715        xx <- 0
 *   :1719        winner = argmax of RAW
 *   :1721        xx[winner] += SCALED[r][winner]              (:722-744; order: fvo_xx_sums kind 0)
 *   :1722        ds[h][:] = xx[h] != 0 ? -xx[h]*W[h][:] : 0   (:394-406)
 *   :1732        ds[winner][idx] += invf[idx % V]             (:657-672)
 *   :1792        rows with xx == 0 zero-filled; nc = max|ds|  (cu_special_reduction.cu:26-99)
 *   :1797-1799   s = eps / max(prec, nc)
 *   :1803        rows with xx != 0: v = s*ds; |v| > 1e-10 ? W += v   (cu_special_reduction.cu:316-354)
 * tie_rule: 0 = lowest index, 1 = the reference's lane-tree order.
 * Outputs (any may be NULL): winners[n], sc_at_winner[n], xx[K], *nc_out.
 * ds_scratch must hold K*N floats.
 */
void fvo_train_step_weighted(float *W, int K, uint64_t N, uint64_t V, const int32_t *idx, uint64_t n, int w,
                             const float *invf, float eps, float prec, int tie_rule, float delta, float lmid,
                             float lbase, float *ds_scratch, int32_t *winners, float *sc_at_winner,
                             int32_t *seconds, float *sc_at_second, float *xx_out, float *nc_out) {
  const int mid = w / 2;
  int32_t *win = (int32_t *)malloc(sizeof(int32_t) * (n ? n : 1));
  float *scw = (float *)malloc(sizeof(float) * (n ? n : 1));
  int32_t *win2 = (int32_t *)malloc(sizeof(int32_t) * (n ? n : 1));
  float *scw2 = (float *)malloc(sizeof(float) * (n ? n : 1));
  float *xx = (float *)calloc((size_t)(K > 0 ? K : 1), sizeof(float));
  float *ds = ds_scratch;

#pragma omp parallel
  {
    float *raw = (float *)malloc(sizeof(float) * (size_t)K);
#pragma omp for schedule(static)
    for (int64_t r = 0; r < (int64_t)n; ++r) {
      const int32_t *ix = idx + (uint64_t)r * w;
      for (int h = 0; h < K; ++h) {
        const float *row = W + (uint64_t)h * N;
        double sr = 0.0;
        for (int c = 0; c < w; ++c)
          if (ix[c] != -1) {
            /* flyvec/src/cuda_funcs.cu:266-286: the fp32 product with the position's weight is what is summed */
            float wl = row[ix[c]] * (c == mid ? lmid : lbase);
            sr += (double)wl;
          }
        raw[h] = (float)sr;
      }
      int best = tie_rule ? fvo_argmax_reference(raw, K) : fvo_argmax_lowest(raw, K);
      const float *row = W + (uint64_t)best * N;
      double ss = 0.0;
      for (int c = 0; c < w; ++c)
        if (ix[c] != -1) {
          /* flyvec/src/cuda_funcs.cu:307-327: (W * L) * 1/f, both products in fp32 */
          float wl = row[ix[c]] * (c == mid ? lmid : lbase);
          float prod = wl * invf[(uint64_t)ix[c] % V];
          ss += (double)prod;
        }
      win[r] = best;
      scw[r] = (float)ss;
      win2[r] = best;
      scw2[r] = 0.0f;
      if (delta != 0) {
        /* flyvec/src/cuda_funcs.cu:495-548 with num_m = 2: the winner's entry is overwritten with
         * -9999.9999 and the same search runs again on the row */
        raw[best] = (float)-9999.9999;
        int second = tie_rule ? fvo_argmax_reference(raw, K) : fvo_argmax_lowest(raw, K);
        const float *row2 = W + (uint64_t)second * N;
        double s2 = 0.0;
        for (int c = 0; c < w; ++c)
          if (ix[c] != -1) {
            float wl = row2[ix[c]] * (c == mid ? lmid : lbase);
            float prod = wl * invf[(uint64_t)ix[c] % V];
            s2 += (double)prod;
          }
        win2[r] = second;
        scw2[r] = (float)s2;
      }
    }
    free(raw);
  }

  fvo_xx_sums(win, scw, n, K, 0, xx);
  if (delta != 0) {
    /* flyvec/src/cuda_funcs.cu:726-734: xx[second] += -delta * scaled[second]. Fixed order: the
     * anti-Hebbian contributions of a neuron are summed like the Hebbian ones (fvo_xx_sums), and the
     * two totals are then added. */
    float *neg = (float *)malloc(sizeof(float) * (n ? n : 1));
    float *xx2 = (float *)calloc((size_t)(K > 0 ? K : 1), sizeof(float));
    for (uint64_t r = 0; r < n; ++r) neg[r] = -delta * scw2[r];
    fvo_xx_sums(win2, neg, n, K, 0, xx2);
    for (int h = 0; h < K; ++h) xx[h] = xx[h] + xx2[h];
    free(neg);
    free(xx2);
  }

  /* ds = -xx*W or 0 */
#pragma omp parallel for schedule(static)
  for (int h = 0; h < K; ++h) {
    float *d = ds + (uint64_t)h * N;
    const float *row = W + (uint64_t)h * N;
    if (xx[h] != 0) {
      float nx = -xx[h];
      for (uint64_t c = 0; c < N; ++c) d[c] = nx * row[c];
    } else {
      for (uint64_t c = 0; c < N; ++c) d[c] = 0.0f;
    }
  }

  /* sparse Hebbian term, increasing (window, position) order */
  for (uint64_t r = 0; r < n; ++r) {
    float *d = ds + (uint64_t)win[r] * N;
    const int32_t *ix = idx + r * (uint64_t)w;
    for (int c = 0; c < w; ++c)
      if (ix[c] != -1) {
        /* flyvec/src/cuda_funcs.cu:675-697: 1.0 * L * 1/f is a double product, rounded to fp32 by the add */
        float add = (float)((double)(c == mid ? lmid : lbase) * (double)invf[(uint64_t)ix[c] % V]);
        d[ix[c]] = d[ix[c]] + add;
      }
  }
  if (delta != 0) {
    /* flyvec/src/cuda_funcs.cu:668: ds[second][idx] += -delta * 1/f. Fixed order: after every
     * Hebbian addition, in increasing (window, position) order. */
    for (uint64_t r = 0; r < n; ++r) {
      float *d = ds + (uint64_t)win2[r] * N;
      const int32_t *ix = idx + r * (uint64_t)w;
      for (int c = 0; c < w; ++c)
        if (ix[c] != -1) {
          /* (-delta * L) * 1/f, both products in fp32 (flyvec/src/cuda_funcs.cu:689, 693) */
          float dl = -delta * (c == mid ? lmid : lbase);
          float g = dl * invf[(uint64_t)ix[c] % V];
          d[ix[c]] = d[ix[c]] + g;
        }
    }
  }

  /* rows with xx == 0 are zero-filled (drops their sparse term); nc = max|ds| */
  float nc = 0.0f;
#pragma omp parallel for schedule(static) reduction(max : nc)
  for (int h = 0; h < K; ++h) {
    float *d = ds + (uint64_t)h * N;
    if (xx[h] != 0) {
      float m = 0.0f;
      for (uint64_t c = 0; c < N; ++c) {
        float a = fabsf(d[c]);
        m = a > m ? a : m;
      }
      nc = m > nc ? m : nc;
    } else {
      for (uint64_t c = 0; c < N; ++c) d[c] = 0.0f;
    }
  }

  float s = (prec > nc) ? eps / prec : eps / nc;

#pragma omp parallel for schedule(static)
  for (int h = 0; h < K; ++h) {
    if (xx[h] == 0) continue;
    float *row = W + (uint64_t)h * N;
    const float *d = ds + (uint64_t)h * N;
    for (uint64_t c = 0; c < N; ++c) {
      float v = s * d[c];
      if (fabs((double)v) > 1.e-10) row[c] = row[c] + v;
    }
  }

  if (winners) memcpy(winners, win, sizeof(int32_t) * n);
  if (sc_at_winner) memcpy(sc_at_winner, scw, sizeof(float) * n);
  if (seconds) memcpy(seconds, win2, sizeof(int32_t) * n);
  if (sc_at_second) memcpy(sc_at_second, scw2, sizeof(float) * n);
  if (xx_out) memcpy(xx_out, xx, sizeof(float) * (size_t)K);
  if (nc_out) *nc_out = nc;
  free(win);
  free(scw);
  free(win2);
  free(scw2);
  free(xx);
}

/* The step with unit position weights (Lmid = Lbase = 1, all the reference's command line reaches). */
void fvo_train_step_delta(float *W, int K, uint64_t N, uint64_t V, const int32_t *idx, uint64_t n, int w,
                          const float *invf, float eps, float prec, int tie_rule, float delta, float *ds_scratch,
                          int32_t *winners, float *sc_at_winner, int32_t *seconds, float *sc_at_second,
                          float *xx_out, float *nc_out) {
  fvo_train_step_weighted(W, K, N, V, idx, n, w, invf, eps, prec, tie_rule, delta, 1.0f, 1.0f, ds_scratch, winners,
                          sc_at_winner, seconds, sc_at_second, xx_out, nc_out);
}

/* The step without the anti-Hebbian term (delta = 0, the trainer's default). */
void fvo_train_step(float *W, int K, uint64_t N, uint64_t V, const int32_t *idx, uint64_t n, int w,
                    const float *invf, float eps, float prec, int tie_rule, float *ds_scratch,
                    int32_t *winners, float *sc_at_winner, float *xx_out, float *nc_out) {
  fvo_train_step_delta(W, K, N, V, idx, n, w, invf, eps, prec, tie_rule, 0.0f, ds_scratch, winners, sc_at_winner,
                       NULL, NULL, xx_out, nc_out);
}

/* flyvec/src/cuda_funcs.cu:1230: the anti-Hebbian strength of an epoch */
float fvo_epoch_delta(float delta, uint64_t epoch, uint64_t n_epochs) {
  return (float)(delta * 0.5 * (1.0 + tanh((((float)epoch) - (0.125 * n_epochs)) / 10.0)));
}

/*
 * n_steps consecutive minibatches of one epoch, as the loop at
 * flyvec/src/cuda_funcs.cu:1662 walks them: step j takes windows
 * perm[first + j*B .. first + (j+1)*B), the last one only its remainder
 * (the reference re-uses stale rows there; this restatement processes the
 * remainder only).  winners (if given) receives the winners of every step
 * back to back.  Returns the number of windows processed.
 *
 * stale_tail != 0 mirrors what the reference does on a final partial
 * minibatch: only the sampler is launched with the remainder
 * (flyvec/src/cuda_funcs.cu:1679 passes input_end - input_start), every other
 * kernel with the full Num (:1700-1732), so the rows from the remainder on
 * still hold the previous minibatch's windows and are trained on once more.
 * The index matrix below is kept from step to step exactly like the
 * reference's input_sparse_indx; a partial step that no full one precedes in
 * this call takes its remainder only (the reference would read rows nobody
 * has written).  The winners of re-used rows are not returned.
 * Pinned in tests/test_oracle_train.py by building that index matrix by hand
 * and running the (separately pinned) single step on it.
 */
uint64_t fvo_train_steps_tail(float *W, int K, uint64_t V, const int32_t *corpus, const uint64_t *starts,
                              const uint64_t *perm, uint64_t n_windows, uint64_t first, uint64_t B,
                              uint64_t n_steps, int w, const float *invf, float eps, float prec,
                              int tie_rule, float delta, float lmid, float lbase, int prune, int stale_tail,
                              int32_t *winners) {
  const uint64_t N = 2 * V;
  float *ds = (float *)malloc(sizeof(float) * (size_t)K * N);
  int32_t *idx = (int32_t *)malloc(sizeof(int32_t) * B * (uint64_t)w);
  int32_t *win_all = (int32_t *)malloc(sizeof(int32_t) * B);
  uint64_t done = 0;
  int full_before = 0;
  for (uint64_t j = 0; j < n_steps; ++j) {
    uint64_t k0 = first + j * B;
    if (k0 >= n_windows) break;
    uint64_t n = (k0 + B <= n_windows) ? B : n_windows - k0;
    if (prune)
      fvo_inflate_prune(corpus, starts, perm, k0, n, w, V, idx);
    else
      fvo_inflate(corpus, starts, perm, k0, n, w, V, idx);
    const uint64_t rows = (stale_tail && n < B && full_before) ? B : n;
    fvo_train_step_weighted(W, K, N, V, idx, rows, w, invf, eps, prec, tie_rule, delta, lmid, lbase, ds, win_all,
                            NULL, NULL, NULL, NULL, NULL);
    if (winners) memcpy(winners + done, win_all, sizeof(int32_t) * n);
    done += n;
    if (n == B) full_before = 1;
  }
  free(ds);
  free(idx);
  free(win_all);
  return done;
}

uint64_t fvo_train_steps_weighted(float *W, int K, uint64_t V, const int32_t *corpus, const uint64_t *starts,
                                  const uint64_t *perm, uint64_t n_windows, uint64_t first, uint64_t B,
                                  uint64_t n_steps, int w, const float *invf, float eps, float prec,
                                  int tie_rule, float delta, float lmid, float lbase, int prune,
                                  int32_t *winners) {
  return fvo_train_steps_tail(W, K, V, corpus, starts, perm, n_windows, first, B, n_steps, w, invf, eps, prec,
                              tie_rule, delta, lmid, lbase, prune, 0, winners);
}

uint64_t fvo_train_steps_delta(float *W, int K, uint64_t V, const int32_t *corpus, const uint64_t *starts,
                               const uint64_t *perm, uint64_t n_windows, uint64_t first, uint64_t B,
                               uint64_t n_steps, int w, const float *invf, float eps, float prec,
                               int tie_rule, float delta, int32_t *winners) {
  return fvo_train_steps_weighted(W, K, V, corpus, starts, perm, n_windows, first, B, n_steps, w, invf, eps, prec,
                                  tie_rule, delta, 1.0f, 1.0f, 0, winners);
}

uint64_t fvo_train_steps(float *W, int K, uint64_t V, const int32_t *corpus, const uint64_t *starts,
                         const uint64_t *perm, uint64_t n_windows, uint64_t first, uint64_t B,
                         uint64_t n_steps, int w, const float *invf, float eps, float prec,
                         int tie_rule, int32_t *winners) {
  return fvo_train_steps_delta(W, K, V, corpus, starts, perm, n_windows, first, B, n_steps, w, invf, eps, prec,
                               tie_rule, 0.0f, winners);
}
