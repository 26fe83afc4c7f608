// Kernels 4 to 6 of the training step: the dense passes over the matrix in their launch forms (device code of
// fv_train.hip).
#pragma once

#include "fv_train_top2.h"

// ---- kernel 4: dense passes over the matrix (one launch, or 4a + 5 + 6) ---------------------------

struct fv_dense_args {
  float4 *Wt4;
  const float *xx;
  const float *invf;
  const fv_slot *slots;  // FV_NB_CLASSES regions of slot_stride records
  uint64_t slot_stride;
  const uint32_t *slot_count;  // records of each block of the sparse launch
  const uint32_t *group_base;
  const uint32_t *group_base2;  // anti-Hebbian form only, like slot_n2 and delta
  const uint32_t *slot_n2;
  float delta;
  float *bmax;           // n_bmax block maxima of |ds|: dense blocks, then the sparse kernel's blocks
  float *scalars;
  uint32_t total4, ldk4, ldk, V, K, w, n_bmax, dense_blocks;
  float eps, prec, update_cut;
  // single-launch form only
  unsigned long long *arrive;  // one word per block, then the launch's decision word
  uint32_t *status;
  uint32_t epoch, spin_limit;
  uint32_t step_tag;  // what a launch that gives up leaves in *status (not 0)
  float lmid, lbase;  // weight of a window's centre position (elements p >= V * ldk) and of the others
  // the minibatch sampled ahead (ahead_n = 0: none)
  const int32_t *corpus;
  const uint64_t *pstart;
  int32_t *idx_ahead;
  uint64_t ahead_first;
  uint32_t ahead_n;
  uint32_t idx_stride;  // entries per row of idx_ahead
  uint32_t sparse_base;  // index in bmax of the sparse launch's first block maximum (a multiple of 4)
  // single-launch form: the rows of the token-major matrix are dealt over the blocks in turn, and of a
  // block's threads the first `active` (the largest multiple of ldk4 it holds) own elements, so that a
  // thread keeps the same four neurons in every round
  uint32_t n_rows, active;
  uint32_t n_slots;  // records the slot regions hold (what a sentinel can name)
  uint32_t slot_region;  // not 0: records per block of the sparse launch, which has a region of its own (fv_sparse_args)
  uint32_t hit_cap;      // sentinels a block of the single launch notes in its LDS list (no more than the list holds)
  // the two largest |W[h][i]| of every row before this step (v1 >= v2), when known, and for every block of
  // the sparse launch how many of its elements hold them (fv_sparse_args.row_hits)
  const float2 *row_top2;
  const uint32_t *row_hits;
  uint32_t top2_known;
  float2 *top2_part;     // out: the same of the matrix this launch leaves, over each block's share: [block][ldk]
  uint32_t part_base;    // separate launches: the update launch's blocks come first, then the slot launch's four
  uint32_t *path_count;  // [0] launches that knew max|ds| when they started, [1] launches that made the pass for it
  // Single-launch form without any wait between blocks, for a device the launch may have to share (a process with
  // more than one trainer): the step enqueues the kernel twice with the same launch number. phase 1 does the
  // whole step when max|ds| is known beforehand; otherwise it only makes the pass for the maximum and leaves
  // every block's maximum in its arrival word. phase 2 ends at once in the first case (every block evaluates the
  // same rule on the same inputs) and in the second reads the words, all written when it starts, and makes the
  // update. phase 0: one launch, the blocks exchange their maxima inside it (they must be resident together).
  uint32_t phase;
};

// ds of a dense element is -xx[h] * W (flyvec/src/cuda_funcs.cu:657-672 without the sparse term). No
// test for a sentinel or for xx == 0 is needed in the two passes: a sentinel is a NaN and so are
// its products, which neither replace a maximum nor pass the update's comparison, and a row with
// xx == 0 has ds = 0, which changes nothing either.
__device__ __forceinline__ float fv_absmax_four(float m, const float4 x, const float4 w) {
  // |x * w| = |-x * w| bit for bit; fmaxf returns the other operand when one is a NaN
  m = fmaxf(m, fabsf(__fmul_rn(x.x, w.x)));
  m = fmaxf(m, fabsf(__fmul_rn(x.y, w.y)));
  m = fmaxf(m, fabsf(__fmul_rn(x.z, w.z)));
  return fmaxf(m, fabsf(__fmul_rn(x.w, w.w)));
}

// W += s * ds on four consecutive elements (flyvec/src/cuda_funcs.cu:1800-1803): an element changes
// only where |s * ds| exceeds the cut. Returns whether any did.
__device__ __forceinline__ bool fv_apply_four(float4 &w, const float4 x, const float s, const float cut) {
  bool changed = false;
  float d;
  d = __fmul_rn(s, __fmul_rn(-x.x, w.x)); if (fabsf(d) > cut) { w.x = __fadd_rn(w.x, d); changed = true; }
  d = __fmul_rn(s, __fmul_rn(-x.y, w.y)); if (fabsf(d) > cut) { w.y = __fadd_rn(w.y, d); changed = true; }
  d = __fmul_rn(s, __fmul_rn(-x.z, w.z)); if (fabsf(d) > cut) { w.z = __fadd_rn(w.z, d); changed = true; }
  d = __fmul_rn(s, __fmul_rn(-x.w, w.w)); if (fabsf(d) > cut) { w.w = __fadd_rn(w.w, d); changed = true; }
  return changed;
}

// The update of the two-launch form: a sentinel goes back as it came, the slot kernel, a later
// launch, replaces it.
__device__ __forceinline__ void fv_update_four(const fv_dense_args &a, uint32_t p4, float4 w, const float4 x,
                                               const float s) {
  if (fv_apply_four(w, x, s, a.update_cut)) a.Wt4[p4] = w;
}

// 16-byte loads a thread of a dense pass has in flight, and the blocks per compute unit of its launch
#ifndef FV_ABSMAX_UNROLL
#define FV_ABSMAX_UNROLL 2
#endif
#ifndef FV_UPDATE_UNROLL
#define FV_UPDATE_UNROLL 8
#endif
#ifndef FV_ABSMAX_BLOCKS_PER_CU
#define FV_ABSMAX_BLOCKS_PER_CU 8
#endif
#ifndef FV_UPDATE_BLOCKS_PER_CU
#define FV_UPDATE_BLOCKS_PER_CU 8
#endif

// Batch u of a thread's elements: 16-byte group p4 + u * stride. Every load is unconditional; one
// past the end reads the thread's first group again and is not used (one common address for all
// of them would queue thousands of wavefronts on a single cache line).
template <int U>
__device__ __forceinline__ void fv_dense_load(const fv_dense_args &a, uint32_t p4, uint32_t stride, float4 (&w)[U]) {
  const uint32_t inside = min(p4, a.total4 - 1);
#pragma unroll
  for (int u = 0; u < U; ++u) w[u] = a.Wt4[p4 + u * stride < a.total4 ? p4 + u * stride : inside];
}

// |w| for the bookkeeping of a row's largest weights; a NaN (a sentinel) counts as 0
__device__ __forceinline__ float fv_abs_or_zero(float w) { return w == w ? fabsf(w) : 0.0f; }

// A 16-byte group's four weights into the four neurons' pairs of largest weights; has_nan says whether any of
// the four is a sentinel (the usual group has none and takes the short form).
__device__ __forceinline__ void fv_top2_insert_four(float (&t1)[4], float (&t2)[4], const float4 &v, bool has_nan) {
  if (!has_nan) {
    fv_top2_insert_abs(t1[0], t2[0], v.x);
    fv_top2_insert_abs(t1[1], t2[1], v.y);
    fv_top2_insert_abs(t1[2], t2[2], v.z);
    fv_top2_insert_abs(t1[3], t2[3], v.w);
  } else {
    fv_top2_insert(t1[0], t2[0], fv_abs_or_zero(v.x));
    fv_top2_insert(t1[1], t2[1], fv_abs_or_zero(v.y));
    fv_top2_insert(t1[2], t2[2], fv_abs_or_zero(v.z));
    fv_top2_insert(t1[3], t2[3], fv_abs_or_zero(v.w));
  }
}

// What one row adds to what is known of max|ds| before the matrix is seen (all three as bit patterns of
// non-negative floats): S, the largest |ds| of a sparse element; E, the largest, over the rows whose largest
// dense weight is known, of fl(|xx| * that weight); F, the same over the other rows with an upper bound of
// that weight. x is the row's xx, top2 its two largest |W| (v1 >= v2), hit4 the counts of the row's sparse
// elements that hold them, one word per block of the sparse launch, smx those blocks' largest |ds|.
__device__ __forceinline__ void fv_row_candidate(float x, float2 top2, uint4 hit4, float4 smx, uint32_t &S, uint32_t &E,
                                                 uint32_t &F) {
  const uint32_t n1 = (hit4.x & 3u) + (hit4.y & 3u) + (hit4.z & 3u) + (hit4.w & 3u);
  const uint32_t n2 = ((hit4.x >> 2) & 3u) + ((hit4.y >> 2) & 3u) + ((hit4.z >> 2) & 3u) + ((hit4.w >> 2) & 3u);
  const float v1 = top2.x, v2 = top2.y;
  // v1 == v2: two elements hold the largest value, one of them is dense unless two sparse ones hold it.
  // v1 > v2: one element holds v1; if it is sparse, v2 bounds the rest, and is reached unless a
  // sparse element holds it.
  const bool first = v1 == v2 ? n1 <= 1 : n1 == 0;
  const bool exact = first || (v1 != v2 && n2 == 0);
  const uint32_t cand = __float_as_uint(__fmul_rn(fabsf(x), first ? v1 : v2));
  // both maxima updated, one of them with 0: a store to whichever of the two the row chooses would keep them
  // in memory, behind the loads of the matrix already in flight
  E = max(E, exact ? cand : 0u);
  F = max(F, exact ? 0u : cand);
  S = max(S, __float_as_uint(fmaxf(fmaxf(smx.x, smx.y), fmaxf(smx.z, smx.w))));
}

// Before the separate dense launches: one block looks at what is known of max|ds| (fv_row_candidate) and
// leaves scalars[2] != 0 and max|ds| in scalars[3] when that settles it; the launch for the maximum then
// ends at once and the update takes the figure from there.
__global__ __launch_bounds__(1024) void fv_decide_kernel(fv_dense_args a) {
  __shared__ uint32_t red3[16][3];
  const uint32_t tid = threadIdx.x;
  uint32_t S = 0, E = 0, F = 0;
  for (uint32_t h = tid; h < a.K; h += 1024)
    fv_row_candidate(a.xx[h], a.row_top2[h], ((const uint4 *)a.row_hits)[h],
                     ((const float4 *)(a.bmax + a.sparse_base))[h], S, E, F);
  const uint32_t ws = fv_wave_max_u32(S), we = fv_wave_max_u32(E), wf = fv_wave_max_u32(F);
  if ((tid & 63) == 0) {
    red3[tid >> 6][0] = ws;
    red3[tid >> 6][1] = we;
    red3[tid >> 6][2] = wf;
  }
  __syncthreads();
  if (tid == 0) {
    S = E = F = 0;
    for (int i = 0; i < 16; ++i) {
      S = max(S, red3[i][0]);
      E = max(E, red3[i][1]);
      F = max(F, red3[i][2]);
    }
    const bool known = a.top2_known && F <= max(S, E);
    a.scalars[2] = known ? 1.0f : 0.0f;
    a.scalars[3] = __uint_as_float(max(S, E));
    a.path_count[known ? 0 : 1] += 1;
  }
}

// Kernel 4a: block maxima of |ds| over the dense elements. A thread's first loads of W
// are issued before the block stages xx in LDS.
__global__ __launch_bounds__(256) void fv_absmax_kernel(fv_dense_args a) {
  extern __shared__ float4 xs4[];  // xx, ldk4 float4
  __shared__ float smem4[4];
  if (a.scalars[2] != 0.0f) return;  // max|ds| is known without the pass (fv_decide_kernel)
  const uint32_t stride = gridDim.x * 256;
  const uint32_t dq = stride % a.ldk4;
  uint32_t p4 = blockIdx.x * 256 + threadIdx.x;
  uint32_t q = p4 % a.ldk4;
  float4 w[FV_ABSMAX_UNROLL];
  fv_dense_load(a, p4, stride, w);
  for (uint32_t i = threadIdx.x; i < a.ldk4; i += 256) xs4[i] = ((const float4 *)a.xx)[i];
  __syncthreads();
  float m = 0.0f;
  while (p4 < a.total4) {
#pragma unroll
    for (int u = 0; u < FV_ABSMAX_UNROLL; ++u) {
      if (p4 + u * stride < a.total4) {
        m = fv_absmax_four(m, xs4[q], w[u]);
      }
      q += dq;
      if (q >= a.ldk4) q -= a.ldk4;
    }
    p4 += FV_ABSMAX_UNROLL * stride;
    if (p4 < a.total4) fv_dense_load(a, p4, stride, w);
  }
  const float bm = fv_block_max_nonneg<4>(m, smem4);
  if (threadIdx.x == 0) a.bmax[blockIdx.x] = bm;
}

// Kernel 5: max|ds| -- from fv_decide_kernel, else from the block maxima -- then W += (eps / max|ds|) * ds over
// the dense elements. The first loads of W are in flight while the block finds the maximum. A block takes
// whole rows of the token-major matrix, TB / ldk4 at a time, so that a thread keeps the same four neurons
// throughout and can keep the two largest |W| it leaves behind for each of them; the block's share of every
// row's two largest weights goes to top2_part[neuron][block] (the slot launch adds the sparse elements').
template <int TB>
__global__ __launch_bounds__(TB) void fv_update_kernel(fv_dense_args a) {
  extern __shared__ float4 dyn4[];  // xx (ldk4 groups), then the threads' pairs (4 x TB)
  float4 *xs4 = dyn4;
  float2 *pairs = (float2 *)(dyn4 + a.ldk4);
  __shared__ float smem16[16];
  __shared__ float sh_s;
  const uint32_t tid = threadIdx.x;
  const uint32_t rows_per_round = TB / a.ldk4;  // the launch is sized so that this is at least 1
  const bool active = tid < rows_per_round * a.ldk4;
  const uint32_t q = tid % a.ldk4, r = tid / a.ldk4;
  const uint32_t row_step = gridDim.x * rows_per_round;
  const uint32_t row0 = blockIdx.x * rows_per_round + r;
  const uint32_t row_inside = min(row0, a.n_rows - 1);  // read again, and not used, by a load past the end
  uint32_t row = active ? row0 : a.n_rows;
  float4 w[FV_UPDATE_UNROLL];
#define FV_UPDATE_LOADS                                                              \
  _Pragma("unroll") for (int u = 0; u < FV_UPDATE_UNROLL; ++u) {                     \
    const uint32_t rr = row + u * row_step;                                          \
    w[u] = a.Wt4[(rr < a.n_rows ? rr : row_inside) * a.ldk4 + q];                    \
  }
  FV_UPDATE_LOADS
  for (uint32_t i = tid; i < a.ldk4; i += TB) xs4[i] = ((const float4 *)a.xx)[i];
  float nc = 0.0f;
  const bool known = a.scalars[2] != 0.0f;
  if (known) {
    nc = a.scalars[3];
  } else {
    const uint32_t n4 = a.n_bmax / 4;
    const float4 *b4 = (const float4 *)a.bmax;
    for (uint32_t i = tid; i < n4; i += 4 * TB) {  // four 16-byte loads together
      float4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) v[u] = b4[min(i + u * TB, n4 - 1)];
#pragma unroll
      for (int u = 0; u < 4; ++u) nc = fmaxf(nc, fmaxf(fmaxf(v[u].x, v[u].y), fmaxf(v[u].z, v[u].w)));
    }
    for (uint32_t i = 4 * n4 + tid; i < a.n_bmax; i += TB) nc = fmaxf(nc, a.bmax[i]);
  }
  nc = fv_block_max_nonneg<TB / 64>(nc, smem16);
  if (tid == 0) {
    sh_s = a.prec > nc ? a.eps / a.prec : a.eps / nc;  // flyvec/src/cuda_funcs.cu:1797-1799
    if (blockIdx.x == 0) a.scalars[0] = nc;
  }
  __syncthreads();
  const float s = sh_s;
  const float4 xq = xs4[q];
  float t1[4] = {0.0f, 0.0f, 0.0f, 0.0f}, t2[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  while (row < a.n_rows) {
#pragma unroll
    for (int u = 0; u < FV_UPDATE_UNROLL; ++u) {
      const uint32_t rr = row + u * row_step;
      if (rr < a.n_rows) {
        float4 v = w[u];
        const bool has_nan = __builtin_isunordered(v.x, v.y) || __builtin_isunordered(v.z, v.w);
        // a sentinel goes back as it came; the slot launch replaces it
        if (fv_apply_four(v, xq, s, a.update_cut)) a.Wt4[rr * a.ldk4 + q] = v;
        fv_top2_insert_four(t1, t2, v, has_nan);
      }
    }
    row += FV_UPDATE_UNROLL * row_step;
    if (row < a.n_rows) {
      FV_UPDATE_LOADS
    }
  }
#undef FV_UPDATE_LOADS
  if (active) {
#pragma unroll
    for (int e = 0; e < 4; ++e) pairs[(e * rows_per_round + r) * a.ldk4 + q] = make_float2(t1[e], t2[e]);
  }
  __syncthreads();
  for (uint32_t h = tid; h < a.K; h += TB) {
    const uint32_t e = h & 3u, qq = h >> 2;
    float m1 = 0.0f, m2 = 0.0f;
    for (uint32_t rr = 0; rr < rows_per_round; ++rr) {
      const float2 b = pairs[(e * rows_per_round + rr) * a.ldk4 + qq];
      fv_top2_merge(m1, m2, b.x, b.y);
    }
    a.top2_part[(uint64_t)blockIdx.x * a.ldk + h] = make_float2(m1, m2);
  }
}

// Kernels 4, 5 and 6 as ONE launch, for a matrix that fits the register file of the machine: one
// block per compute unit.
//
// max|ds| without a pass over the matrix. A dense element has ds = -xx[h] * W[h][i], and fp32
// rounding is monotone, so the largest |ds| of the dense elements of row h is fl(|xx[h]| * m) with m
// the largest |W[h][i]| over the row's dense elements. Every launch leaves, for every row, the two
// largest |W| of the matrix it has written (each block over its share; the winner kernel of the next
// step merges the shares). The sparse launch reports how many of a row's sparse elements hold those two
// values, so this launch knows for every row either m exactly (the largest value, or the second
// largest when the largest is sparse and the second is not) or an upper bound of it. When the largest
// exact figure (the sparse elements' own |ds| included) is at least every upper bound, it is max|ds|:
// s = eps / max(prec, max|ds|) is known before the first weight arrives and the launch is one streaming
// read-modify-write of the matrix, with no exchange between the blocks and nothing to wait for.
// Otherwise (or when the largest weights are not known: the first step on a new matrix, or after a step
// in another launch form) the launch makes the pass: every thread keeps its U 16-byte groups of W in
// registers from the maximum pass to the update, so W is still read once and written once. Between
// the passes every block publishes its maximum of |ds| as (launch number, value) in one 64-bit word and
// one wave of it reads the words of all blocks until each carries this launch's number; the values it
// read are the maxima, no second look-up follows. The wait is bounded: a block that does not see
// the others within spin_limit rounds (they are not resident together: the launch was given fewer
// compute units than it was sized for) marks its word as abandoned, so that blocks arriving later
// give up as well, sets the status word and leaves its part of W as it is.
//
// The sparse elements are finished here as well, by the block that owns them: a thread that meets a
// sentinel leaves it alone and notes (sentinel, element) in its wave's LDS list; when the wave has updated its
// dense elements it deals its list over its lanes, each of which finds the record through the sentinel's
// number, forms ds and writes the element. No other block ever reads or writes that element in this launch.
// (A list per wave, not per block: the wave asks for its records as soon as its own last store is issued,
// without a barrier, so the records travel while the stores drain -- a wave's loads and stores share one
// counter, and a load asked for behind the block's barrier would begin its trip only when the drain is over.)
#ifndef FV_ONEPASS_THREADS
#define FV_ONEPASS_THREADS 1024
#endif
#define FV_ONEPASS_BLOCKS_PER_CU (1024 / FV_ONEPASS_THREADS)
#define FV_ONEPASS_MAX_UNROLL 16
// 16-byte loads of W a thread has in flight at a time: with all 16 issued at once the first pass
// took 2 us longer (10 or 12 in flight measured best; 8 and 14 lie between)
#ifndef FV_ONEPASS_DEPTH
#define FV_ONEPASS_DEPTH 12
#endif
#define FV_ONEPASS_SPIN_LIMIT (1u << 14)  // rounds of a few microseconds each: tens of milliseconds
#define FV_ONEPASS_ABANDONED 0xffffffffu  // in place of a block's maximum (no maximum is a NaN): it gave up
#define FV_ONEPASS_HIT_CAP 4096           // sentinels a block notes in LDS, a list of its own for every wave; one
                                          // that finds its wave's list full is finished by its thread, from memory
#define FV_ONEPASS_WAVE_HITS (FV_ONEPASS_HIT_CAP / (FV_ONEPASS_THREADS / 64))

// The same on two LDS words per neuron, from many threads at once: the value that loses at the first
// word -- the newcomer, or the value it displaced -- goes on to the second; every value but the
// largest is handed on exactly once. Non-negative floats order like their bit patterns.
__device__ __forceinline__ void fv_top2_insert_lds(uint32_t *s1, uint32_t *s2, uint32_t h, float a) {
  const uint32_t b = __float_as_uint(a);
  const uint32_t old = atomicMax(&s1[h], b);
  atomicMax(&s2[h], min(old, b));
}

// The element p holds the sentinel `bits`: its final value from the record the sentinel names. The saved
// weight goes back where the row is not updated (xx == 0) or the launch gave up, else the updated one.
template <bool DELTA>
__device__ __forceinline__ void fv_finish_sparse_element(const fv_dense_args &a, uint32_t bits, uint32_t p, float s,
                                                         bool ok, const float *xs, uint32_t *sp1, uint32_t *sp2) {
  const uint32_t number = (bits & FV_SENTINEL_MAX) - 1u;
  if (number >= a.n_slots) return;  // a NaN of another origin stays what it is
  const uint32_t col = p / a.ldk, h = p - col * a.ldk;
  // the sentinel's number counts from the start of the slots, or of the region of the sparse launch's block
  // that owns the element
  const uint64_t at = a.slot_region ? fv_slot_place((h << FV_NB_CLASS_SHIFT) | (col & (FV_NB_CLASSES - 1)), number,
                                                    a.slot_region, a.K * FV_NB_CLASSES)
                                    : number;
  const fv_slot sl = a.slots[at];
  if (sl.p != p) return;
  const float x = xs[h];
  float out = sl.wv;
  if (ok && x != 0.0f) {
    const float l = p >= a.V * a.ldk ? a.lmid : a.lbase;
    const float ds = DELTA ? fv_sparse_ds2(x, sl.wv, sl.f, sl.n, a.delta, a.slot_n2[at], l)
                           : fv_sparse_ds(x, sl.wv, sl.f, sl.n, l);
    const float d = __fmul_rn(s, ds);
    if (fabsf(d) > a.update_cut) out = __fadd_rn(sl.wv, d);
  }
  ((float *)a.Wt4)[p] = out;
  fv_top2_insert_lds(sp1, sp2, h, fv_abs_or_zero(out));
}

// The sentinels of a list, dealt over `width` threads (this one is number `me` of them), four records in flight per
// thread: a wave that has met a row of a frequent token holds a few hundred of them, and one after the other each
// would be a trip to memory of its own.
template <bool DELTA>
__device__ __forceinline__ void fv_finish_sparse_elements(const fv_dense_args &a, const uint2 *list, uint32_t n, uint32_t me,
                                                          uint32_t width, float s, bool ok, const float *xs, uint32_t *sp1,
                                                          uint32_t *sp2) {
  for (uint32_t i0 = me; i0 < n; i0 += 4 * width) {
    uint2 hit[4];
    fv_slot sl[4];
    uint32_t n2[4];
    bool mine[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      hit[u] = list[min(i0 + u * width, n - 1)];
      const uint32_t number = (hit[u].x & FV_SENTINEL_MAX) - 1u;
      mine[u] = i0 + u * width < n && number < a.n_slots;  // a NaN of another origin stays what it is
      const uint32_t p = hit[u].y, col = p / a.ldk, h = p - col * a.ldk;
      const uint64_t at = a.slot_region ? fv_slot_place((h << FV_NB_CLASS_SHIFT) | (col & (FV_NB_CLASSES - 1)), number,
                                                        a.slot_region, a.K * FV_NB_CLASSES)
                                        : number;
      sl[u] = a.slots[mine[u] ? at : 0];
      n2[u] = DELTA ? a.slot_n2[mine[u] ? at : 0] : 0u;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const uint32_t p = hit[u].y;
      if (!mine[u] || sl[u].p != p) continue;
      const uint32_t h = p % a.ldk;
      const float x = xs[h];
      float out = sl[u].wv;
      if (ok && x != 0.0f) {
        const float l = p >= a.V * a.ldk ? a.lmid : a.lbase;
        const float ds = DELTA ? fv_sparse_ds2(x, sl[u].wv, sl[u].f, sl[u].n, a.delta, n2[u], l)
                               : fv_sparse_ds(x, sl[u].wv, sl[u].f, sl[u].n, l);
        const float d = __fmul_rn(s, ds);
        if (fabsf(d) > a.update_cut) out = __fadd_rn(sl[u].wv, d);
      }
      ((float *)a.Wt4)[p] = out;
      fv_top2_insert_lds(sp1, sp2, h, fv_abs_or_zero(out));
    }
  }
}

// s_setprio takes its level as an immediate.
__device__ __forceinline__ void fv_set_wave_priority(uint32_t level) {
  if (level == 0) __builtin_amdgcn_s_setprio(0);
  else if (level == 1) __builtin_amdgcn_s_setprio(1);
  else if (level == 2) __builtin_amdgcn_s_setprio(2);
  else __builtin_amdgcn_s_setprio(3);
}

// The next minibatch's column indices, by all waves but the first (which polls in the exchange): the
// window's start was fetched behind the loads of W, the token follows here; then, for a minibatch with more
// positions than the launch has sampling threads, the rest.
__device__ __forceinline__ void fv_sample_ahead(const fv_dense_args &a, bool samples0, uint32_t e0, uint32_t er0,
                                                uint64_t start0, uint32_t ahead_entries, uint32_t TS) {
  if (samples0) {
    const uint32_t c = e0 - er0 * a.idx_stride;
    a.idx_ahead[e0] = c < a.w ? fv_column_index(a.corpus[start0 + c], c, a.w, a.V) : -1;
  }
  if (threadIdx.x >= 64) {
    // four entries at a time: their window starts travel together, then their tokens
    const uint32_t step = gridDim.x * TS;
    for (uint32_t e = e0 + step; e < ahead_entries; e += 4 * step) {
      uint32_t c[4];
      uint64_t at[4];
      int32_t tok[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const uint32_t ek = e + k * step < ahead_entries ? e + k * step : e;
        const uint32_t r = ek / a.idx_stride;
        c[k] = ek - r * a.idx_stride;
        at[k] = a.pstart[a.ahead_first + r];
      }
#pragma unroll
      for (int k = 0; k < 4; ++k) tok[k] = a.corpus[at[k] + (c[k] < a.w ? c[k] : 0u)];
#pragma unroll
      for (int k = 0; k < 4; ++k)
        if (e + k * step < ahead_entries)
          a.idx_ahead[e + k * step] = c[k] < a.w ? fv_column_index(tok[k], c[k], a.w, a.V) : -1;
    }
  }
}

// The one decision of a launch that makes the pass for max|ds|: whether all its blocks go on to the update,
// and with which maximum. The word carries (launch number, value); whoever writes this launch's number
// first -- block 0 with the maximum once every block has arrived, or any block that has run out of patience
// with FV_ONEPASS_ABANDONED -- has decided for all, and everybody, the writer included, follows what the
// word says. Returns the decision.
__device__ __forceinline__ uint32_t fv_onepass_decide(unsigned long long *word, uint32_t epoch, uint32_t value) {
  unsigned long long old = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const unsigned long long mine = ((unsigned long long)epoch << 32) | value;
  while ((uint32_t)(old >> 32) != epoch) {
    if (__hip_atomic_compare_exchange_strong(word, &old, mine, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                             __HIP_MEMORY_SCOPE_AGENT))
      return value;
  }
  return (uint32_t)old;
}

// Between the pass for the maximum and the update of a single dense launch: the block publishes its maximum m
// of |ds|, its first wave waits (bounded) for the launch's decision, and its first thread leaves the step's scale
// in *sh_s and whether the update goes ahead in *sh_ok (read behind the caller's next barrier).
__device__ __forceinline__ void fv_onepass_exchange(const fv_dense_args &a, float m, uint32_t limit, bool dead,
                                                    float *smem16, float *sh_s_out, uint32_t *sh_ok_out) {
  constexpr uint32_t T = FV_ONEPASS_THREADS;
  const uint32_t tid = threadIdx.x;
  float &sh_s = *sh_s_out;
  uint32_t &sh_ok = *sh_ok_out;
  // the block's maximum, needed by its first wave only: one barrier
  {
    const uint32_t wm = fv_wave_max_u32(__float_as_uint(m));
    if ((tid & 63) == 0) smem16[tid >> 6] = __uint_as_float(wm);
  }
  __syncthreads();
  if (tid < 64) {
    float bm = tid < T / 64 ? smem16[tid] : 0.0f;
    bm = __uint_as_float(fv_wave_max_u32(__float_as_uint(bm)));
    if (tid == 0)
      __hip_atomic_store(&a.arrive[blockIdx.x], ((unsigned long long)a.epoch << 32) | __float_as_uint(bm),
                         __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // Block 0 waits for every block's word and decides; the others wait for the decision. Both waits are
    // bounded, and a block that gives up decides "abandoned" unless the decision has already been made.
    unsigned long long *decision = a.arrive + gridDim.x;
    uint32_t verdict = FV_ONEPASS_ABANDONED;
    bool decided = false;
    if (blockIdx.x == 0) {
      uint32_t mx = 0;
      bool done = false;
      for (uint32_t spin = 0; spin < limit && !done; ++spin) {
        bool all = true;
        mx = 0;
        for (uint32_t i = tid; i < gridDim.x; i += 64) {
          const unsigned long long v = __hip_atomic_load(&a.arrive[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          all = all && (uint32_t)(v >> 32) == a.epoch;
          mx = max(mx, (uint32_t)v);  // non-negative floats order like their bit patterns
        }
        done = __all(all);
        if (!done) __builtin_amdgcn_s_sleep(2);
      }
      mx = fv_wave_max_u32(mx);
      if (done) verdict = mx;
    } else {
      for (uint32_t spin = 0; spin < limit && !decided; ++spin) {
        const unsigned long long v = __hip_atomic_load(decision, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        decided = (uint32_t)(v >> 32) == a.epoch;
        if (decided) verdict = (uint32_t)v; else __builtin_amdgcn_s_sleep(2);
      }
    }
    if (tid == 0) {
      if (!decided) verdict = fv_onepass_decide(decision, a.epoch, verdict);
      const bool go = verdict != FV_ONEPASS_ABANDONED;
      const float nc = __uint_as_float(verdict);
      sh_s = a.prec > nc ? a.eps / a.prec : a.eps / nc;  // flyvec/src/cuda_funcs.cu:1797-1799
      sh_ok = go;
      if (!go) {
        if (!dead) *a.status = a.step_tag;  // the launches behind this one are dead and leave the word alone
        a.scalars[0] = __uint_as_float(0x7fc00000u);
        a.scalars[1] = 1.0f;
      } else if (blockIdx.x == 0) {
        a.scalars[0] = nc;
        a.path_count[1] += 1;
      }
    }
  }
}

// Phase 1 of the launch that waits for nobody: the block's maximum m of |ds| into its arrival word, for phase 2.
__device__ __forceinline__ void fv_onepass_publish(const fv_dense_args &a, float m, float *smem16) {
  constexpr uint32_t T = FV_ONEPASS_THREADS;
  const uint32_t tid = threadIdx.x;
  const uint32_t wm = fv_wave_max_u32(__float_as_uint(m));
  if ((tid & 63) == 0) smem16[tid >> 6] = __uint_as_float(wm);
  __syncthreads();
  if (tid < 64) {
    float bm = tid < T / 64 ? smem16[tid] : 0.0f;
    bm = __uint_as_float(fv_wave_max_u32(__float_as_uint(bm)));
    if (tid == 0) {
      __hip_atomic_store(&a.arrive[blockIdx.x], ((unsigned long long)a.epoch << 32) | __float_as_uint(bm),
                         __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (blockIdx.x == 0) a.path_count[1] += 1;
    }
  }
}

// Phase 2: the maxima phase 1 left, one word per block, all of this launch number (the launch that wrote them has
// ended); the step's scale into *sh_s_out (read behind the caller's next barrier). A word of another number can
// only mean that phase 1 did not run: the update is then withheld (*sh_ok_out = 0).
__device__ __forceinline__ void fv_onepass_collect(const fv_dense_args &a, float *sh_s_out, uint32_t *sh_ok_out) {
  const uint32_t tid = threadIdx.x;
  if (tid < 64) {
    uint32_t mx = 0;
    bool all = true;
    for (uint32_t i = tid; i < gridDim.x; i += 64) {
      const unsigned long long v = __hip_atomic_load(&a.arrive[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      all = all && (uint32_t)(v >> 32) == a.epoch;
      mx = max(mx, (uint32_t)v);
    }
    mx = fv_wave_max_u32(mx);
    const bool go = __all(all);
    if (tid == 0) {
      const float nc = __uint_as_float(mx);
      *sh_s_out = a.prec > nc ? a.eps / a.prec : a.eps / nc;  // flyvec/src/cuda_funcs.cu:1797-1799
      *sh_ok_out = go;
      if (blockIdx.x == 0) a.scalars[0] = go ? nc : __uint_as_float(0x7fc00000u);
    }
  }
}

static_assert(FV_MAX_HID <= 2 * FV_ONEPASS_THREADS, "two neurons per thread cover every row");
static_assert(FV_NB_CLASSES == 4, "a neuron's block maxima and hit counts are read as one 16-byte word each");

// PHASE: fv_dense_args.phase, fixed at compile time (the branches of the other phases cost the register form
// its last registers).
template <int U, bool DELTA, int PHASE = 0>
__global__ __launch_bounds__(FV_ONEPASS_THREADS) void fv_dense_onepass_kernel(fv_dense_args a) {
  constexpr uint32_t T = FV_ONEPASS_THREADS;
  constexpr int DEPTH = FV_ONEPASS_DEPTH < U ? FV_ONEPASS_DEPTH : U;
  // xx (ldk floats); the two largest finished sparse elements of every neuron (2 x ldk words); the
  // sentinels met (FV_ONEPASS_WAVE_HITS pairs per wave); the threads' two largest weights (4 x active pairs)
  extern __shared__ float4 dyn4[];
  float *xs = (float *)dyn4;
  uint32_t *sp1 = (uint32_t *)(xs + a.ldk);
  uint32_t *sp2 = sp1 + a.ldk;
  uint2 *hit_list = (uint2 *)(sp2 + a.ldk);
  float2 *pairs = (float2 *)(hit_list + FV_ONEPASS_HIT_CAP);
  __shared__ uint32_t red3[T / 64][3];
  __shared__ float smem16[16];
  __shared__ float sh_s;
  __shared__ uint32_t sh_ok, sh_hits[T / 64];
  uint2 *wave_list = hit_list + (threadIdx.x >> 6) * FV_ONEPASS_WAVE_HITS;
  uint32_t *wave_hits = &sh_hits[threadIdx.x >> 6];
  const uint32_t tid = threadIdx.x;
  const bool active = tid < a.active;
  const uint32_t q = tid % a.ldk4, r = tid / a.ldk4;
  const uint32_t rows_per_round = a.active / a.ldk4;
  const uint32_t row0 = blockIdx.x + gridDim.x * r;  // the thread's row in round 0
  const uint32_t row_step = gridDim.x * rows_per_round;
  const uint32_t row_inside = min(row0, a.n_rows - 1);  // read again, and not used, by a load past the end
  // The small loads first, every one unconditional, then this thread's W: loads return in the order
  // of issue, so what is issued here is in hand while W is in flight.
  float xh[2];
  float2 rm[2];
  uint4 hit4[2];
  float4 smx[2];  // the sparse launch's block maxima of |ds|
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const uint32_t h = min(tid + T * j, a.K - 1);
    xh[j] = a.xx[min(tid + T * j, a.ldk - 1)];
    rm[j] = a.row_top2[h];
    hit4[j] = ((const uint4 *)a.row_hits)[h];
    smx[j] = ((const float4 *)(a.bmax + a.sparse_base))[h];
  }
  // after one launch has given up, the launches already enqueued behind it neither wait nor update
  const bool dead = a.scalars[1] != 0.0f;
  const uint32_t limit = dead ? 0u : a.spin_limit;
  float4 w[U];
  __builtin_amdgcn_sched_barrier(0);  // nothing that uses a small load moves up between the loads of W
  // (phase 2 usually ends behind the decision: it asks for the matrix only once it knows that it goes on)
#define FV_ONEPASS_FIRST_LOADS                                            \
  _Pragma("unroll") for (int u = 0; u < DEPTH; ++u) {                     \
    const uint32_t row = row0 + u * row_step;                             \
    w[u] = a.Wt4[(row < a.n_rows ? row : row_inside) * a.ldk4 + q];       \
  }
  if (PHASE != 2) {
    FV_ONEPASS_FIRST_LOADS
  }
  __builtin_amdgcn_sched_barrier(0);
  // the next minibatch's column indices, by all waves but the first: the window's start now
  constexpr uint32_t TS = T - 64;
  const uint32_t ahead_entries = a.ahead_n * a.idx_stride;  // the entries past w of a row get -1
  const uint32_t e0 = blockIdx.x * TS + (tid - 64);
  const bool samples0 = tid >= 64 && e0 < ahead_entries;
  const uint32_t er0 = samples0 ? e0 / a.idx_stride : 0u;
  const uint64_t start0 = a.ahead_n ? a.pstart[a.ahead_first + er0] : 0ull;

  // what is known of max|ds| before the matrix is seen (fv_row_candidate)
  uint32_t S = 0, E = 0, F = 0;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const uint32_t h = tid + T * j;
    if (h < a.ldk) {
      xs[h] = xh[j];
      sp1[h] = 0;
      sp2[h] = 0;
    }
    if (h < a.K) fv_row_candidate(xh[j], rm[j], hit4[j], smx[j], S, E, F);
  }
  if (tid < T / 64) sh_hits[tid] = 0;
  {
    const uint32_t ws = fv_wave_max_u32(S), we = fv_wave_max_u32(E), wf = fv_wave_max_u32(F);
    if ((tid & 63) == 0) {
      red3[tid >> 6][0] = ws;
      red3[tid >> 6][1] = we;
      red3[tid >> 6][2] = wf;
    }
  }
  __syncthreads();
  S = E = F = 0;
#pragma unroll
  for (uint32_t i = 0; i < T / 64; ++i) {
    S = max(S, red3[i][0]);
    E = max(E, red3[i][1]);
    F = max(F, red3[i][2]);
  }
  const bool fast = a.top2_known && F <= max(S, E);  // the same answer in every thread of every block
  const float4 xq = ((const float4 *)xs)[q];
  if (PHASE == 2 && fast) return;  // phase 1 has made the whole step
  // the rows are streamed (loaded as their turn comes, updated, stored) rather than held from a pass for the maximum
  const bool streams = fast || PHASE == 2;

  float s;
  bool ok = true;
  if (fast) {
    const float nc = __uint_as_float(max(S, E));
    s = a.prec > nc ? a.eps / a.prec : a.eps / nc;  // flyvec/src/cuda_funcs.cu:1797-1799
    ok = !dead;
    if (blockIdx.x == 0 && tid == 0 && ok) {
      a.scalars[0] = nc;
      a.path_count[0] += 1;
    }
  } else if (PHASE == 2) {
    FV_ONEPASS_FIRST_LOADS
    fv_onepass_collect(a, &sh_s, &sh_ok);
    __syncthreads();
    ok = sh_ok != 0 && !dead;
    s = sh_s;
  } else {
    // the pass for the maximum, on registers; the loads not yet issued take the places of those used
    float m = __uint_as_float(S);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t row = row0 + u * row_step;
      if (active && row < a.n_rows) m = fv_absmax_four(m, xq, w[u]);
      if (u + DEPTH < U) {
        const uint32_t rown = row0 + (u + DEPTH) * row_step;
        w[u + DEPTH] = a.Wt4[(rown < a.n_rows ? rown : row_inside) * a.ldk4 + q];
      }
    }
    if (PHASE == 1) {  // the update is phase 2's
      fv_onepass_publish(a, m, smem16);
      return;
    }
    fv_onepass_exchange(a, m, limit, dead, smem16, &sh_s, &sh_ok);
    fv_sample_ahead(a, samples0, e0, er0, start0, ahead_entries, TS);  // while the first wave waits
    __syncthreads();
    ok = sh_ok != 0;
    s = sh_s;
  }
#undef FV_ONEPASS_FIRST_LOADS

  // The update. A group without a sentinel is stored whole where something changed; in a group with
  // one the other elements are stored one by one and the sentinel is noted for later. The two largest
  // |W| of what the thread leaves behind are kept per neuron.
  // the token of the thread's first entry of the minibatch sampled ahead: fetched before the stream over the
  // rows, so that a corpus too large for the Infinity Cache does not lengthen the launch's tail
  const uint32_t c0 = e0 - er0 * a.idx_stride;
  int32_t tok0 = -1;
  if (streams && samples0 && c0 < a.w) tok0 = a.corpus[start0 + c0];
  float t1[4] = {0.0f, 0.0f, 0.0f, 0.0f}, t2[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  // A sentinel that finds the block's list full is finished by its own thread behind the stream (bit 4 u + e:
  // element e of the thread's group u), from memory, where it still stands.
  static_assert(4 * U <= 64, "one bit per element of a thread");
  uint64_t beyond_list = 0;
#define FV_ONEPASS_ELEMENT(member, lane4)                                                      \
  if (v.member == v.member) {                                                                  \
    if (changed) e[lane4] = v.member;                                                          \
  } else {                                                                                     \
    const uint32_t k = atomicAdd(wave_hits, 1u);                                               \
    if (k < a.hit_cap)                                                                         \
      wave_list[k] = make_uint2(__float_as_uint(v.member), 4u * p4 + lane4);                   \
    else                                                                                       \
      beyond_list |= 1ull << (4 * u + lane4);                                                  \
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const uint32_t row = row0 + u * row_step;
    // The four waves that share a SIMD take turns at going first. Left to the age of the waves, the youngest ones
    // of every block are served last throughout and end their stream 3 to 4 us behind the median wave, and the
    // block ends with them.
    fv_set_wave_priority(((tid >> 8) + (uint32_t)u) & 3u);
    if (active && row < a.n_rows) {
      const uint32_t p4 = row * a.ldk4 + q;
      float4 v = w[u];
      const bool has_nan = __builtin_isunordered(v.x, v.y) || __builtin_isunordered(v.z, v.w);
      const bool changed = ok && fv_apply_four(v, xq, s, a.update_cut);
      if (!has_nan) {
        if (changed) a.Wt4[p4] = v;
      } else {
        float *e = (float *)&a.Wt4[p4];
        FV_ONEPASS_ELEMENT(x, 0)
        FV_ONEPASS_ELEMENT(y, 1)
        FV_ONEPASS_ELEMENT(z, 2)
        FV_ONEPASS_ELEMENT(w, 3)
      }
      fv_top2_insert_four(t1, t2, v, has_nan);
    }
    if (streams && u + DEPTH < U) {  // the next load takes the place of the one just used
      const uint32_t rown = row0 + (u + DEPTH) * row_step;
      w[u + DEPTH] = a.Wt4[(rown < a.n_rows ? rown : row_inside) * a.ldk4 + q];
    }
  }
#undef FV_ONEPASS_ELEMENT
  if (streams) {
    if (samples0) a.idx_ahead[e0] = c0 < a.w ? fv_column_index(tok0, c0, a.w, a.V) : -1;
    fv_sample_ahead(a, false, e0, er0, start0, ahead_entries, TS);  // the entries beyond the first, if any
  }
  // the sentinels the wave has met, dealt over its lanes (the list and its count are the wave's own: no barrier)
  __builtin_amdgcn_s_setprio(0);
  {
    const uint32_t n_hits = min(*wave_hits, a.hit_cap);
    fv_finish_sparse_elements<DELTA>(a, wave_list, n_hits, tid & 63u, 64u, s, ok, xs, sp1, sp2);
  }
  while (beyond_list) {
    const uint32_t b = (uint32_t)__ffsll((long long)beyond_list) - 1u;
    beyond_list &= beyond_list - 1;
    const uint32_t at = 4u * ((row0 + (b >> 2) * row_step) * a.ldk4 + q) + (b & 3u);
    fv_finish_sparse_element<DELTA>(a, __float_as_uint(((const float *)a.Wt4)[at]), at, s, ok, xs, sp1, sp2);
  }
  if (active) {
#pragma unroll
    for (int e = 0; e < 4; ++e) pairs[(e * rows_per_round + r) * a.ldk4 + q] = make_float2(t1[e], t2[e]);
  }
  __syncthreads();
  // the block's share of every row's two largest weights: its threads' pairs and the finished sparse elements
  for (uint32_t h = tid; h < a.K; h += T) {
    const uint32_t e = h & 3u, qq = h >> 2;
    float m1 = __uint_as_float(sp1[h]), m2 = __uint_as_float(sp2[h]);
    for (uint32_t rr = 0; rr < rows_per_round; ++rr) {
      const float2 b = pairs[(e * rows_per_round + rr) * a.ldk4 + qq];
      fv_top2_merge(m1, m2, b.x, b.y);
    }
    a.top2_part[(uint64_t)blockIdx.x * a.ldk + h] = make_float2(m1, m2);
  }
}

// The same launch for a matrix of any size: nothing is kept in registers between the passes, the block's rows
// go through FV_STREAM_DEPTH 16-byte groups per thread in rounds. When max|ds| is known from the rows' largest
// weights (the usual case) it is one streaming read-modify-write; otherwise the rows are streamed once for the
// maximum, the blocks exchange their maxima as above, and the rows are streamed again for the update: the
// traffic of the separate launches, without their launches. Rows, ownership of the sparse elements, the shares of
// the rows' largest weights and the minibatch sampled ahead are those of fv_dense_onepass_kernel.
#ifndef FV_STREAM_DEPTH
#define FV_STREAM_DEPTH 2
#endif
#define FV_STREAM_HIT_CAP 8192  // sentinels a block notes in LDS (64 KB)

template <bool DELTA, int PHASE = 0>
__global__ __launch_bounds__(FV_ONEPASS_THREADS) void fv_dense_stream_kernel(fv_dense_args a) {
  constexpr uint32_t T = FV_ONEPASS_THREADS;
  constexpr int D = FV_STREAM_DEPTH;
  extern __shared__ float4 dyn4[];
  float *xs = (float *)dyn4;
  uint32_t *sp1 = (uint32_t *)(xs + a.ldk);
  uint32_t *sp2 = sp1 + a.ldk;
  uint2 *hit_list = (uint2 *)(sp2 + a.ldk);
  float2 *pairs = (float2 *)(hit_list + FV_STREAM_HIT_CAP);
  __shared__ uint32_t red3[T / 64][3];
  __shared__ float smem16[16];
  __shared__ float sh_s;
  __shared__ uint32_t sh_ok, sh_hits;
  const uint32_t tid = threadIdx.x;
  const bool active = tid < a.active;
  const uint32_t q = tid % a.ldk4, r = tid / a.ldk4;
  const uint32_t rows_per_round = a.active / a.ldk4;
  const uint32_t row0 = blockIdx.x + gridDim.x * r;
  const uint32_t row_step = gridDim.x * rows_per_round;
  const uint32_t rounds = (a.n_rows + row_step - 1) / row_step;
  const uint32_t row_inside = min(row0, a.n_rows - 1);
  float xh[2];
  float2 rm[2];
  uint4 hit4[2];
  float4 smx[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const uint32_t h = min(tid + T * j, a.K - 1);
    xh[j] = a.xx[min(tid + T * j, a.ldk - 1)];
    rm[j] = a.row_top2[h];
    hit4[j] = ((const uint4 *)a.row_hits)[h];
    smx[j] = ((const float4 *)(a.bmax + a.sparse_base))[h];
  }
  const bool dead = a.scalars[1] != 0.0f;
  const uint32_t limit = dead ? 0u : a.spin_limit;
  float4 w[D];
  auto group_of = [&](uint32_t row) { return (row < a.n_rows ? row : row_inside) * a.ldk4 + q; };
  // (phase 2 usually ends behind the decision: it asks for the matrix only once it knows that it goes on)
  if (PHASE != 2) {
#pragma unroll
    for (int u = 0; u < D; ++u) w[u] = a.Wt4[group_of(row0 + u * row_step)];
  }
  constexpr uint32_t TS = T - 64;
  const uint32_t ahead_entries = a.ahead_n * a.idx_stride;
  const uint32_t e0 = blockIdx.x * TS + (tid - 64);
  const bool samples0 = tid >= 64 && e0 < ahead_entries;
  const uint32_t er0 = samples0 ? e0 / a.idx_stride : 0u;
  const uint64_t start0 = a.ahead_n ? a.pstart[a.ahead_first + er0] : 0ull;

  uint32_t S = 0, E = 0, F = 0;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const uint32_t h = tid + T * j;
    if (h < a.ldk) {
      xs[h] = xh[j];
      sp1[h] = 0;
      sp2[h] = 0;
    }
    if (h < a.K) fv_row_candidate(xh[j], rm[j], hit4[j], smx[j], S, E, F);
  }
  if (tid == 0) sh_hits = 0;
  {
    const uint32_t ws = fv_wave_max_u32(S), we = fv_wave_max_u32(E), wf = fv_wave_max_u32(F);
    if ((tid & 63) == 0) {
      red3[tid >> 6][0] = ws;
      red3[tid >> 6][1] = we;
      red3[tid >> 6][2] = wf;
    }
  }
  __syncthreads();
  S = E = F = 0;
#pragma unroll
  for (uint32_t i = 0; i < T / 64; ++i) {
    S = max(S, red3[i][0]);
    E = max(E, red3[i][1]);
    F = max(F, red3[i][2]);
  }
  const bool fast = a.top2_known && F <= max(S, E);
  const float4 xq = ((const float4 *)xs)[q];
  if (PHASE == 2 && fast) return;  // phase 1 has made the whole step
  // the next minibatch is sampled beside the update's stream rather than during a wait
  const bool streams = fast || PHASE == 2;

  float s;
  bool ok = true;
  if (fast) {
    const float nc = __uint_as_float(max(S, E));
    s = a.prec > nc ? a.eps / a.prec : a.eps / nc;  // flyvec/src/cuda_funcs.cu:1797-1799
    ok = !dead;
    if (blockIdx.x == 0 && tid == 0 && ok) {
      a.scalars[0] = nc;
      a.path_count[0] += 1;
    }
  } else if (PHASE == 2) {
#pragma unroll
    for (int u = 0; u < D; ++u) w[u] = a.Wt4[group_of(row0 + u * row_step)];
    fv_onepass_collect(a, &sh_s, &sh_ok);
    __syncthreads();
    ok = sh_ok != 0 && !dead;
    s = sh_s;
  } else {
    float m = __uint_as_float(S);
    for (uint32_t c = 0; c < rounds; c += D) {
#pragma unroll
      for (int u = 0; u < D; ++u) {
        const uint32_t row = row0 + (c + u) * row_step;
        if (active && row < a.n_rows) m = fv_absmax_four(m, xq, w[u]);
        w[u] = a.Wt4[group_of(row + D * row_step)];
      }
    }
    if (PHASE == 1) {  // the update is phase 2's
      fv_onepass_publish(a, m, smem16);
      return;
    }
    fv_onepass_exchange(a, m, limit, dead, smem16, &sh_s, &sh_ok);
    fv_sample_ahead(a, samples0, e0, er0, start0, ahead_entries, TS);  // while the first wave waits
    __syncthreads();
    ok = sh_ok != 0;
    s = sh_s;
#pragma unroll
    for (int u = 0; u < D; ++u) w[u] = a.Wt4[group_of(row0 + u * row_step)];  // the stream starts again
  }

  // (as in fv_dense_onepass_kernel: the first token of the minibatch sampled ahead travels during the stream)
  const uint32_t c0 = e0 - er0 * a.idx_stride;
  int32_t tok0 = -1;
  if (streams && samples0 && c0 < a.w) tok0 = a.corpus[start0 + c0];
  float t1[4] = {0.0f, 0.0f, 0.0f, 0.0f}, t2[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#define FV_STREAM_ELEMENT(member, lane4)                                                       \
  if (v.member == v.member) {                                                                  \
    if (changed) e[lane4] = v.member;                                                          \
  } else {                                                                                     \
    const uint32_t k = atomicAdd(&sh_hits, 1u);                                                \
    if (k < a.hit_cap)                                                                         \
      hit_list[k] = make_uint2(__float_as_uint(v.member), 4u * p4 + lane4);                    \
    else                                                                                       \
      fv_finish_sparse_element<DELTA>(a, __float_as_uint(v.member), 4u * p4 + lane4, s, ok, xs, sp1, sp2); \
  }
  for (uint32_t c = 0; c < rounds; c += D) {
#pragma unroll
    for (int u = 0; u < D; ++u) {
      const uint32_t row = row0 + (c + u) * row_step;
      if (active && row < a.n_rows) {
        const uint32_t p4 = row * a.ldk4 + q;
        float4 v = w[u];
        const bool has_nan = __builtin_isunordered(v.x, v.y) || __builtin_isunordered(v.z, v.w);
        const bool changed = ok && fv_apply_four(v, xq, s, a.update_cut);
        if (!has_nan) {
          if (changed) a.Wt4[p4] = v;
        } else {
          float *e = (float *)&a.Wt4[p4];
          FV_STREAM_ELEMENT(x, 0)
          FV_STREAM_ELEMENT(y, 1)
          FV_STREAM_ELEMENT(z, 2)
          FV_STREAM_ELEMENT(w, 3)
        }
        fv_top2_insert_four(t1, t2, v, has_nan);
      }
      w[u] = a.Wt4[group_of(row + D * row_step)];  // the round that takes this one's place
    }
  }
#undef FV_STREAM_ELEMENT
  if (streams) {
    if (samples0) a.idx_ahead[e0] = c0 < a.w ? fv_column_index(tok0, c0, a.w, a.V) : -1;
    fv_sample_ahead(a, false, e0, er0, start0, ahead_entries, TS);
  }
  if (active) {
#pragma unroll
    for (int e = 0; e < 4; ++e) pairs[(e * rows_per_round + r) * a.ldk4 + q] = make_float2(t1[e], t2[e]);
  }
  __syncthreads();
  const uint32_t n_hits = min(sh_hits, a.hit_cap);
  for (uint32_t i = tid; i < n_hits; i += T) {
    const uint2 hit = hit_list[i];
    fv_finish_sparse_element<DELTA>(a, hit.x, hit.y, s, ok, xs, sp1, sp2);
  }
  __syncthreads();
  for (uint32_t h = tid; h < a.K; h += T) {
    const uint32_t e = h & 3u, qq = h >> 2;
    float m1 = __uint_as_float(sp1[h]), m2 = __uint_as_float(sp2[h]);
    for (uint32_t rr = 0; rr < rows_per_round; ++rr) {
      const float2 b = pairs[(e * rows_per_round + rr) * a.ldk4 + qq];
      fv_top2_merge(m1, m2, b.x, b.y);
    }
    a.top2_part[(uint64_t)blockIdx.x * a.ldk + h] = make_float2(m1, m2);
  }
}

static int fv_stream_fits(size_t smem) {
  int nb = 0, nb2 = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, (fv_dense_stream_kernel<false, 0>), FV_ONEPASS_THREADS, smem) !=
          hipSuccess ||
      hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb2, (fv_dense_stream_kernel<true, 0>), FV_ONEPASS_THREADS, smem) !=
          hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return nb >= 1 && nb2 >= 1;
}

template <int U, bool DELTA>
static void fv_launch_onepass(const fv_dense_args &d, unsigned blocks, size_t smem, hipStream_t stream) {
  const dim3 grid(blocks), block(FV_ONEPASS_THREADS);
  if (d.phase == 0)
    hipLaunchKernelGGL((fv_dense_onepass_kernel<U, DELTA, 0>), grid, block, smem, stream, d);
  else if (d.phase == 1)
    hipLaunchKernelGGL((fv_dense_onepass_kernel<U, DELTA, 1>), grid, block, smem, stream, d);
  else
    hipLaunchKernelGGL((fv_dense_onepass_kernel<U, DELTA, 2>), grid, block, smem, stream, d);
}

template <bool DELTA>
static void fv_launch_stream(const fv_dense_args &d, unsigned blocks, size_t smem, hipStream_t stream) {
  const dim3 grid(blocks), block(FV_ONEPASS_THREADS);
  if (d.phase == 0)
    hipLaunchKernelGGL((fv_dense_stream_kernel<DELTA, 0>), grid, block, smem, stream, d);
  else if (d.phase == 1)
    hipLaunchKernelGGL((fv_dense_stream_kernel<DELTA, 1>), grid, block, smem, stream, d);
  else
    hipLaunchKernelGGL((fv_dense_stream_kernel<DELTA, 2>), grid, block, smem, stream, d);
}

template <int U>
static int fv_onepass_fits(size_t smem) {
  int nb = 0, nb2 = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, (fv_dense_onepass_kernel<U, false, 0>), FV_ONEPASS_THREADS,
                                                   smem) != hipSuccess ||
      hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb2, (fv_dense_onepass_kernel<U, true, 0>), FV_ONEPASS_THREADS,
                                                   smem) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return nb >= FV_ONEPASS_BLOCKS_PER_CU && nb2 >= FV_ONEPASS_BLOCKS_PER_CU;
}

// Kernel 6: the final value of every sparse element goes over its sentinel. Runs after the dense
// update so no dense thread can mistake a finished element for an ordinary weight.
template <bool DELTA>
__global__ __launch_bounds__(256) void fv_slot_update_kernel(fv_dense_args a) {
  // block (h, q) of the sparse launch wrote slot_count records at the start of its part of region q
  __shared__ float2 wave_pair[4];
  const uint32_t count = a.slot_count[blockIdx.x];
  const uint32_t h = blockIdx.x >> FV_NB_CLASS_SHIFT, q = blockIdx.x & (FV_NB_CLASSES - 1);
  // the two largest of what the block writes: its share of the row's two largest weights, behind the
  // update launch's shares
  float2 *share = a.top2_part + (uint64_t)(a.part_base + q) * a.ldk + h;
  if (count == 0) {
    if (threadIdx.x == 0) *share = make_float2(0.0f, 0.0f);
    return;
  }
  float m1 = 0.0f, m2 = 0.0f;
  const uint64_t slot_first =
      a.slot_region ? 0ull
                    : (uint64_t)q * a.slot_stride + (uint64_t)(a.group_base[h] + (DELTA ? a.group_base2[h] : 0u)) * a.w;
  // record `number` of the block
  auto place_of = [&](uint32_t number) {
    return a.slot_region ? fv_slot_place(blockIdx.x, number, a.slot_region, gridDim.x) : slot_first + number;
  };
  const float x = a.xx[h];
  const float nc = a.scalars[0];
  const float s = a.prec > nc ? a.eps / a.prec : a.eps / nc;
  for (uint32_t eb = threadIdx.x; eb < count; eb += 4 * 256) {  // four records in flight per thread
    fv_slot sl[4];
    uint32_t n2[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const uint64_t place = place_of(min(eb + u * 256, count - 1));
      sl[u] = a.slots[place];
      n2[u] = DELTA ? a.slot_n2[place] : 0u;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (eb + u * 256 >= count) break;
      float out = sl[u].wv;  // a row with xx == 0 is not updated: the saved weight goes back
      if (x != 0.0f) {
        const float l = sl[u].p >= a.V * a.ldk ? a.lmid : a.lbase;
        const float ds = DELTA ? fv_sparse_ds2(x, sl[u].wv, sl[u].f, sl[u].n, a.delta, n2[u], l)
                               : fv_sparse_ds(x, sl[u].wv, sl[u].f, sl[u].n, l);
        const float d = __fmul_rn(s, ds);
        if (fabsf(d) > a.update_cut) out = __fadd_rn(sl[u].wv, d);
      }
      ((float *)a.Wt4)[sl[u].p] = out;
      fv_top2_insert(m1, m2, fv_abs_or_zero(out));
    }
  }
  for (int d = 32; d >= 1; d >>= 1) {  // the partner's pair covers other elements: no value is counted twice
    const float b1 = __shfl_xor(m1, d, 64), b2 = __shfl_xor(m2, d, 64);
    fv_top2_merge(m1, m2, b1, b2);
  }
  if ((threadIdx.x & 63) == 0) wave_pair[threadIdx.x >> 6] = make_float2(m1, m2);
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int i = 1; i < 4; ++i) fv_top2_merge(m1, m2, wave_pair[i].x, wave_pair[i].y);
    *share = make_float2(m1, m2);
  }
}
