// Kernel 3 of the training step (device code of fv_train.hip).
#pragma once

#include "fv_train_group.h"

// ---- kernel 3: sparse elements -----------------------------------------------------------------------
//
// FV_NB_CLASSES blocks per neuron h; block q owns the elements (h, column i) with
// i mod FV_NB_CLASSES == q, so a neuron that won a large share of the minibatch is spread over
// several blocks and no two blocks share an element.  A block counts the occurrences of each of
// its columns over the neuron's windows in LDS, and for every distinct one saves
// (element, count, weight) in a slot record and plants the sentinel in W.

struct fv_sparse_args {
  const uint32_t *order;
  const uint32_t *group_base;
  const uint32_t *group_count;
  const int32_t *idx;  // followed by FV_IDX_PAD entries of -1
  float *Wt;
  fv_slot *slots;  // FV_NB_CLASSES regions of slot_stride records
  uint64_t slot_stride;
  // Not 0 (grouping form only): every block has a region of slot_region records of its own in slots[]
  // (fv_slot_place), and a sentinel names a record by its number in the block's region. A block has no
  // more records than its class has columns, so no block needs to know what the others write.
  uint32_t slot_region;
  uint32_t n_blocks;  // blocks of the launch (what fv_slot_place needs; read from the arguments, not from the dispatch packet)
  const float *xx;
  const float *invf;
  float *bmax_sparse;    // one maximum of |ds| per block
  uint32_t *slot_count;  // records written per block
  uint32_t ldk, w, V, pad_row;  // pad_row: the row index just behind the index matrix
  uint32_t stride;              // entries per row of idx (a multiple of 4)
  // anti-Hebbian form only: the windows in which the neuron came second, grouped like the others;
  // the count of those occurrences of an element goes to slot_n2 beside its record
  const uint32_t *order2;
  const uint32_t *group_base2;
  const uint32_t *group_count2;
  uint32_t *slot_n2;
  float delta;
  float lmid, lbase;  // weight of a window's centre position (columns >= V) and of the others
  // grouping form only: the block finds the neuron's windows in the winner array itself
  const uint32_t *won;        // row h: bit r set where neuron h won window r (won_words words, an even number)
  const uint16_t *win;        // 16-bit winners; behind the last one, up to a multiple of 64 entries, 0x7fff
  uint32_t won_words;
  uint32_t *won_clear;  // the other buffer: the class-0 block of neuron h clears row h
  // anti-Hebbian form that groups for itself: the same pair of bit rows for the second neurons, their scaled
  // activations, and where the class-0 block leaves the second count
  const uint32_t *won2;
  uint32_t *won2_clear;
  const float *sc2;
  uint32_t *group_base2_out, *group_count2_out;
  const float *sc;      // scaled activations of the windows
  uint32_t n;           // windows of the step
  uint32_t *order_out;  // a neuron's window ids beyond what LDS stages go through here
  uint32_t *group_base_out, *group_count_out;
  float *xx_out;
  // The two largest |W[h][i]| of every row as the step finds the matrix (row_top2[h] = (v1, v2), v1 >= v2),
  // when known: the block reports in row_hits how many of its elements hold v1 and, where v2 < v1, how
  // many hold v2 (bits 0-1 and 2-3, each saturated at 3). The dense launch then knows whether the
  // largest weight of a row is one of the step's sparse elements.
  const float2 *row_top2;
  uint32_t *row_hits;
  uint32_t top2_known;
  // grouping form with a slot region per block: a neuron whose window positions are no more than the block has
  // threads is finished by its class-0 block alone, an entry per thread (fv_sparse_light); 0 switches that off
  uint32_t light;
};

// Counting pass of one class block over the windows whose ids are staged in LDS: ord[0 .. n_staged),
// followed up to the next multiple of the windows a batch of loads takes by the id of the padding row behind the
// index matrix (all -1). A row of idx is `stride` entries, a multiple of 4, those past w holding -1; a lane
// reads four positions of one window, 16 bytes, and a window takes as many neighbouring lanes as its row has
// such pieces, up to four (fv_sparse_lanes: three for the eleven positions of the reference's window, so that a
// block's load covers 85 windows, not 64; a longer row is read in chunks of sixteen positions). A lane issues
// LOADS loads back to back with no branch between them (the compiler waits for every load in flight at a
// branch target), then counts. With the class in the top bits and the column of the class below, one
// subtraction and one comparison tell whether an entry is this block's: of class q, inside [lo, lo + span),
// not masked, not padding.
#define FV_SLOT_REGIONS_MAX_BYTES (1ull << 30)  // most memory spent on slot regions per block
template <bool NARROW>
__device__ __forceinline__ void fv_sparse_count_entry(uint32_t *cnt, int32_t iv, uint32_t drop, uint32_t origin,
                                                      uint32_t span) {
  const uint32_t t = __builtin_rotateright32((uint32_t)iv | drop, FV_NB_CLASS_SHIFT) - origin;
  if (t < span) {
    if (NARROW)
      atomicAdd(&cnt[t >> 1], 1u << (16 * (t & 1)));
    else
      atomicAdd(&cnt[t], 1u);
  }
}

// Lanes that share a window in the counting pass, and the windows a block of FV_SP_THREADS then takes per load.
__host__ __device__ __forceinline__ uint32_t fv_sparse_lanes(uint32_t stride) { return stride >= 16 ? 4u : stride >> 2; }
__host__ __device__ __forceinline__ uint32_t fv_sparse_wps(uint32_t stride) { return FV_SP_THREADS / fv_sparse_lanes(stride); }
// Window ids staged in LDS at a time: whole batches of FV_SP_LOADS loads, so that the padding stays inside ord[].
__host__ __device__ __forceinline__ uint32_t fv_sparse_stage_cap(uint32_t stride) {
  const uint32_t per = fv_sparse_wps(stride) * FV_SP_LOADS;
  return FV_SP_STAGE / per * per;
}

// behind_first_loads() runs once, between the issue of the first loads and the counting of what they bring: the
// place for work on values whose own loads were issued earlier and so have returned by then.
template <bool NARROW, int LOADS, typename Ord, typename Hook>
__device__ __forceinline__ void fv_sparse_count(uint32_t *cnt, const Ord *ord, uint32_t n_staged,
                                                const int32_t *__restrict__ idx, uint32_t stride, uint32_t q,
                                                uint32_t lo, uint32_t span, uint32_t tid, Hook &behind_first_loads) {
  const uint32_t lanes = fv_sparse_lanes(stride), wps = FV_SP_THREADS / lanes;
  // tid / lanes without a division: exact for tid < 2^16 / lanes
  const uint32_t slot_of = (tid * ((65536u + lanes - 1) / lanes)) >> 16;
  const bool alive = slot_of < wps;  // (255 of 256 threads with three lanes per window)
  const uint32_t slot = alive ? slot_of : 0u;
  const uint32_t c4 = 4u * (tid - slot_of * lanes);
  const uint32_t steps = (n_staged + wps - 1) / wps;
  const uint32_t origin = (q << (32 - FV_NB_CLASS_SHIFT)) | lo;
  for (uint32_t c0 = 0; c0 < stride; c0 += FV_SP_CHUNK) {
    const bool live = alive && c0 + c4 < stride;  // a row shorter than the chunk: the lanes past its end read its start again
    const uint32_t cc = live ? c0 + c4 : 0u;
    const uint32_t drop = live ? 0u : 0xffffffffu;
    for (uint32_t s0 = 0; s0 < steps; s0 += LOADS) {
      int4 iv[LOADS];
#pragma unroll
      for (int b = 0; b < LOADS; ++b)
        iv[b] = *(const int4 *)(idx + (uint64_t)ord[(s0 + b) * wps + slot] * stride + cc);
      if (c0 == 0 && s0 == 0) behind_first_loads();
#pragma unroll
      for (int b = 0; b < LOADS; ++b) {
        fv_sparse_count_entry<NARROW>(cnt, iv[b].x, drop, origin, span);
        fv_sparse_count_entry<NARROW>(cnt, iv[b].y, drop, origin, span);
        fv_sparse_count_entry<NARROW>(cnt, iv[b].z, drop, origin, span);
        fv_sparse_count_entry<NARROW>(cnt, iv[b].w, drop, origin, span);
      }
    }
  }
}

// The same with the number of loads in flight fitted to the number of windows; pads ord[] (n_staged is at most
// fv_sparse_stage_cap).
template <bool NARROW, typename Ord, typename Hook>
__device__ __forceinline__ void fv_sparse_count_any(uint32_t *cnt, Ord *ord, uint32_t n_staged, uint32_t pad_row,
                                                    const int32_t *__restrict__ idx, uint32_t stride, uint32_t q,
                                                    uint32_t lo, uint32_t span, uint32_t tid, Hook &behind_first_loads) {
  static_assert(FV_SP_LOADS % 4 == 0 && FV_SP_STAGE >= FV_SP_THREADS * FV_SP_LOADS, "padding of ord[] stays inside it");
  const uint32_t wps = fv_sparse_wps(stride);
  const uint32_t per = wps * (n_staged <= wps ? 1 : n_staged <= wps * 4 ? 4 : FV_SP_LOADS);
  const uint32_t padded = (n_staged + per - 1) / per * per;
  for (uint32_t i = n_staged + tid; i < padded; i += FV_SP_THREADS) ord[i] = (Ord)pad_row;
  fv_lds_barrier();
  if (per == wps)
    fv_sparse_count<NARROW, 1, Ord>(cnt, ord, n_staged, idx, stride, q, lo, span, tid, behind_first_loads);
  else if (per == wps * 4)
    fv_sparse_count<NARROW, 4, Ord>(cnt, ord, n_staged, idx, stride, q, lo, span, tid, behind_first_loads);
  else
    fv_sparse_count<NARROW, FV_SP_LOADS, Ord>(cnt, ord, n_staged, idx, stride, q, lo, span, tid, behind_first_loads);
}

// A neuron with few windows (grouping form, a slot region per block): one of its four blocks takes all four column
// classes, one window position per thread, and the other three end at once. The counter array and a pass over
// 5120 words to find the few counters that are not zero would be most of such a block's time; here the thread
// whose addition finds a counter at zero owns the element, reads the final count behind a barrier and clears the
// counter again, so nothing is scanned. The classes share the counter array and are taken one after the other.
// Every thread asks for its element's weight and 1/f as soon as it has the column, before ownership is settled: the
// loads of the threads that turn out not to own an element are wasted, the owners' have arrived by the time they
// are needed (one trip less in the chain). Records go to the region of the element's class, numbered in the order
// the owners arrive; the results do not depend on that order.
// Called by the whole block with the neuron's window ids staged by rank in ord[0 .. c_h) (c_h * stride <= the
// block's threads), cnt[] zero and x_h = xx[h].
// DELTA: ord[c_h .. c_h + c2_h) holds the windows in which the neuron came second; a column's two counts share a
// 32-bit counter (cnt[] then has a word for every column of a class), the first in the low half.
template <bool DELTA, typename Ord>
__device__ __forceinline__ void fv_sparse_light(const fv_sparse_args &a, uint32_t h, uint32_t blk, uint32_t c_h, uint32_t c2_h,
                                                float x_h, uint32_t *cnt, const Ord *ord, uint32_t *cls_n, uint32_t *sh_hits,
                                                float *wave_max) {
  const uint32_t tid = threadIdx.x;
  const uint32_t n_cols = 2 * a.V;
  if (tid < FV_NB_CLASSES) cls_n[tid] = 0;
  if (tid == 0) sh_hits[0] = sh_hits[1] = 0;
  fv_lds_barrier();
  // the thread's window position: entry tid of the neuron's c_h rows of the index matrix
  const uint32_t j = tid / a.stride, c = tid - j * a.stride;
  const bool inside = j < c_h + c2_h;
  const bool second = DELTA && j >= c_h;  // a position of a window in which the neuron came second
  const int32_t iv = a.idx[(uint64_t)ord[inside ? j : 0u] * a.stride + c];
  const bool real = inside && (uint32_t)iv < n_cols;
  const uint32_t col = real ? (uint32_t)iv : 0u;
  const uint32_t p = col * a.ldk + h;
  const float wv = a.Wt[p];
  const float f = a.invf[col >= a.V ? col - a.V : col];
  const float l = col >= a.V ? a.lmid : a.lbase;
  const float2 top2 = a.top2_known ? a.row_top2[h] : make_float2(0.0f, 0.0f);
  const uint32_t cls = col & (FV_NB_CLASSES - 1), t = col >> FV_NB_CLASS_SHIFT;
  // the element's counter: half of word t / 2, or, with two counts to keep, word t
  const uint32_t shift = DELTA ? 0u : 16u * (t & 1u), at = DELTA ? t : t >> 1;
  uint32_t hits1 = 0, hits2 = 0;  // the same in all lanes of a wave
  float ds_max = 0.0f;
  for (uint32_t q = 0; q < FV_NB_CLASSES; ++q) {
    const bool mine = real && cls == q;
    bool owner = false;
    if (mine) {
      const uint32_t old = atomicAdd(&cnt[at], second ? 0x10000u : 1u << shift);
      owner = DELTA ? old == 0u : ((old >> shift) & 0xffffu) == 0u;
    }
    fv_lds_barrier();  // every occurrence of the class is counted
    uint32_t n = 0, n2 = 0, number = 0;
    if (owner) {
      const uint32_t word = cnt[at];
      n = (word >> shift) & 0xffffu;
      n2 = DELTA ? word >> 16 : 0u;
      number = atomicAdd(&cls_n[q], 1u);
    }
    fv_lds_barrier();  // the counts are read
    if (owner) {
      if (DELTA)
        cnt[at] = 0;  // zero again for the next class
      else
        atomicAnd(&cnt[at], 0xffff0000u >> shift);
      fv_slot rec;
      rec.p = p;
      rec.n = n;
      rec.wv = wv;
      rec.f = f;
      // (fv_slot_place for a number below the block's threads, which is below FV_SLOT_PRIMARY or below the region)
      const uint64_t place = ((h << FV_NB_CLASS_SHIFT) | q) * min(a.slot_region, FV_SLOT_PRIMARY) + number;
      a.slots[place] = rec;
      if (DELTA) a.slot_n2[place] = n2;
      a.Wt[p] = fv_sentinel(number);
      if (x_h != 0.0f)
        ds_max = fv_absmax_keep(ds_max, DELTA ? fv_sparse_ds2(x_h, wv, f, n, a.delta, n2, l) : fv_sparse_ds(x_h, wv, f, n, l));
    }
    const float aw = fabsf(wv);
    hits1 += (uint32_t)__popcll(__ballot(owner && aw == top2.x));
    hits2 += (uint32_t)__popcll(__ballot(owner && aw == top2.y && top2.y < top2.x));
    fv_lds_barrier();  // the class's counters are zero again
  }
  if ((tid & 63u) == 0 && (hits1 | hits2)) {
    atomicAdd(&sh_hits[0], hits1);
    atomicAdd(&sh_hits[1], hits2);
  }
  const float bm = fv_block_max_nonneg<FV_SP_THREADS / 64>(ds_max, wave_max);  // behind its barriers every wave's hits are counted
  if (tid == 0) {
    a.bmax_sparse[blk] = bm;
    a.row_hits[blk] = min(sh_hits[0], 3u) | (min(sh_hits[1], 3u) << 2);
  }
  if (tid < FV_NB_CLASSES) a.slot_count[(h << FV_NB_CLASS_SHIFT) | tid] = cls_n[tid];
}

// DELTA: the neuron's elements are counted over two lists of windows, those it won and those in
// which it came second, into two counter arrays; a record carries both counts.
// GROUPING: no grouping launch has run. Every class block takes its neuron's windows from the bit row
// the winner kernel has filled (a thread's two words are one group of 64 windows: the step has no more than
// 64 * FV_SP_THREADS), stages the window ids in LDS by rank, and adds the neuron's scaled activations in the
// grouping kernel's order: every thread those of its group, in row order, then the threads' sums over the balanced
// tree on the thread number (fv_block_tree_sum). The block of class 0 leaves xx[h], the neuron's count and its base
// for the dense launch and clears the neuron's row of the other bit-row buffer. The blocks of this form go to the
// device's eight XCDs in turn, so the class a block takes rotates with the neuron: every XCD gets its share of each
// class (the class-0 blocks are the ones that finish a neuron with few windows alone, fv_sparse_light).
// IDS16: the window ids staged in LDS are 16 bits wide (a batch below 65535 windows, so that the id of the padding
// row behind the index matrix fits too): the smaller array lets one more block share a compute unit.
// NW (GROUPING): 64-bit words of the neuron's bit row per thread; a step has up to 64 * NW * FV_SP_THREADS windows.
// (Four words per thread, for steps of up to 65534 windows, were built and measured at K = 1000, B = 50000: the
// four class blocks of a neuron then each fetch and add its activations, and the launch takes as much longer
// as the grouping launch it replaces lasts; only the one-word form is instantiated.)
template <bool DELTA, bool GROUPING, int CW, bool IDS16 = GROUPING, int NW = 1>
__device__ __forceinline__ void fv_sparse_block(const fv_sparse_args &a) {
  __shared__ uint32_t cnt_all[DELTA ? 2 * CW : CW];  // (one array: the form for neurons with few windows uses all of it)
  uint32_t *const cnt = cnt_all, *const cnt2 = cnt_all + (DELTA ? CW : 0);
  __shared__ uint16_t list[FV_SP_LIST_CAP];
  // window ids of a grouping step (at most 64 * FV_SP_THREADS windows, and the padding row behind them)
  // fit 16 bits: the smaller array lets one more block share a compute unit
  static_assert(NW == 1 || NW == 4, "one or four words of the bit row per thread");
  static_assert(64 * FV_SP_THREADS < 65536, "ids of a grouping step fit 16 bits (the host keeps a step below 65535 windows)");
  static_assert(IDS16 || !GROUPING, "a grouping step's ids are 16 bits wide");
  typedef typename std::conditional<IDS16, uint16_t, uint32_t>::type ord_t;
  __shared__ ord_t ord[FV_SP_STAGE];
  __shared__ uint32_t sh_pos;
  __shared__ uint32_t sh_hits[2];
  __shared__ float wave_max[16];
  __shared__ uint32_t red[17];
  constexpr uint32_t T = FV_SP_THREADS;
  const uint32_t h = blockIdx.x >> FV_NB_CLASS_SHIFT;
  const uint32_t q = GROUPING ? ((blockIdx.x & (FV_NB_CLASSES - 1)) + (blockIdx.x >> (FV_NB_CLASS_SHIFT + 1))) & (FV_NB_CLASSES - 1)
                              : blockIdx.x & (FV_NB_CLASSES - 1);
  const uint32_t blk = (h << FV_NB_CLASS_SHIFT) | q;  // the block's number in the arrays the other launches read
  const uint32_t tid = threadIdx.x;
  __shared__ uint32_t red2[GROUPING ? 17 : 1];
  uint32_t c_h, base, my_off = 0, r0 = 0;
  uint64_t mask[NW];
#pragma unroll
  for (int i = 0; i < NW; ++i) mask[i] = 0;
  uint32_t eq = 0;  // the thread's matches
  // anti-Hebbian form: the windows in which the neuron came second, likewise
  uint64_t mask2 = 0;
  uint32_t eq2 = 0, my_off2 = 0, c2_grouped = 0;
  // scaled activations a thread fetches before it knows how many it needs: four, or sixteen in a wave with a
  // thread that has more than four matches (a neuron that won a tenth of the minibatch has seven per thread)
  constexpr int PF = 4, PF_BIG = 16;
  float pf[PF_BIG];
  float x_h = 0.0f;
  if (GROUPING) {
    static_assert(NW == 1, "a thread's words are one group of 64 windows of the order of the totals xx");
    const uint32_t n = a.n;
    // (the counters are cleared while the bit row travels)
    for (uint32_t i = tid; i < CW / 4; i += T) ((uint4 *)cnt)[i] = make_uint4(0, 0, 0, 0);
    if (DELTA)
      for (uint32_t i = tid; i < CW / 4; i += T) ((uint4 *)cnt2)[i] = make_uint4(0, 0, 0, 0);
    // thread t takes windows 64 NW t .. 64 NW (t + 1) - 1: 2 NW words of the neuron's row
    r0 = 64 * NW * tid;
#pragma unroll
    for (int i = 0; i < NW; ++i) {
      const uint32_t word = 2 * (NW * tid + i);
      uint2 mw = make_uint2(0u, 0u);
      if (word < a.won_words) mw = *(const uint2 *)(a.won + (uint64_t)h * a.won_words + word);
      mask[i] = (uint64_t)mw.x | ((uint64_t)mw.y << 32);
    }
#pragma unroll
    for (int i = 0; i < NW; ++i) eq += (uint32_t)__popcll(mask[i]);
    if (DELTA) {
      const uint32_t word = 2 * tid;
      uint2 mw = make_uint2(0u, 0u);
      if (word < a.won_words) mw = *(const uint2 *)(a.won2 + (uint64_t)h * a.won_words + word);
      mask2 = (uint64_t)mw.x | ((uint64_t)mw.y << 32);
      eq2 = (uint32_t)__popcll(mask2);
    }
    if (q == 0) {
#pragma unroll
      for (int i = 0; i < NW; ++i) {
        const uint32_t word = 2 * (NW * tid + i);
        if (word < a.won_words) {
          *(uint2 *)(a.won_clear + (uint64_t)h * a.won_words + word) = make_uint2(0u, 0u);
          if (DELTA) *(uint2 *)(a.won2_clear + (uint64_t)h * a.won_words + word) = make_uint2(0u, 0u);
        }
      }
    }
    // the scaled activations of a thread's matches travel while the scan runs
    {
      const bool wave_big = __ballot(eq > (uint32_t)PF) != 0ull;
      // such a wave belongs to one of the few blocks the launch waits for: it goes first from here on wherever
      // it shares a SIMD with the waves of other blocks
      if (wave_big) __builtin_amdgcn_s_setprio(3);
      uint64_t left = mask[0];
#pragma unroll
      for (int e = 0; e < PF_BIG; ++e) pf[e] = 0.0f;
      // the lowest bit left (none left: the thread's first window, whose value is not used)
#define FV_SP_FETCH(e)                                                                    \
  {                                                                                       \
    const uint32_t r = left ? r0 + (uint32_t)__ffsll((long long)left) - 1 : r0;           \
    left &= left - 1;                                                                     \
    pf[e] = a.sc[min(r, n - 1)];                                                          \
  }
      if (wave_big) {
#pragma unroll
        for (int e = 0; e < PF_BIG; ++e) FV_SP_FETCH(e)
      } else {
#pragma unroll
        for (int e = 0; e < PF; ++e) FV_SP_FETCH(e)
      }
#undef FV_SP_FETCH
    }
    // anti-Hebbian form: the second neurons' activations, times -delta (flyvec/src/cuda_funcs.cu:726-734), summed
    // like the others; a thread's group in row order, eight loads in flight
    float part2 = 0.0f;
    if (DELTA) {
      uint64_t left = mask2;
      while (__ballot(left != 0ull)) {
        float v[8];
        uint64_t l2 = left;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const uint32_t r = l2 ? r0 + (uint32_t)__ffsll((long long)l2) - 1 : r0;
          l2 &= l2 - 1;
          v[e] = a.sc2[min(r, n - 1)];
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          if (left) part2 = __fadd_rn(part2, __fmul_rn(-a.delta, v[e]));
          left &= left - 1;
        }
      }
    }
    // one block scan gives the ranks and the neuron's count (both lists' as the halves of a word: a step of this
    // form has fewer than 2^16 windows)
    const uint32_t both = eq | (eq2 << 16);
    const uint32_t incl = fv_wave_inclusive_scan_u32(both);
    if ((tid & 63u) == 63u) red[tid >> 6] = incl;
    fv_lds_barrier();
    uint32_t before = 0, total = 0;
#pragma unroll
    for (uint32_t i = 0; i < T / 64; ++i) {
      const uint32_t t = red[i];
      before += i < (tid >> 6) ? t : 0u;
      total += t;
    }
    c_h = total & 0xffffu;
    c2_grouped = total >> 16;
    my_off = ((before + incl - both) & 0xffffu);
    my_off2 = (before + incl - both) >> 16;
    // The launch lasts as long as its few heaviest blocks: their waves go first wherever they share a
    // SIMD with the waves of light blocks.
    if (c_h > FV_SP_HEAVY) __builtin_amdgcn_s_setprio(3);
    // xx[h]: the thread's group first, in row order onto +0 (what was fetched, then, for a thread with more matches
    // than that, the rest one by one), then the tree over the threads
    {
      float part = 0.0f;
#pragma unroll
      for (int e = 0; e < PF_BIG; ++e)
        if ((uint32_t)e < eq) part = __fadd_rn(part, pf[e]);
      if (__ballot(eq > (uint32_t)PF_BIG)) {  // (a neuron that won more than a quarter of some group of 64 windows)
        uint64_t left = eq > (uint32_t)PF_BIG ? mask[0] : 0ull;
        for (int e = 0; e < PF_BIG; ++e) left &= left - 1;
        while (__ballot(left != 0ull)) {  // eight loads in flight, then their additions in row order
          float v[8];
          uint64_t l2 = left;
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const uint32_t r = l2 ? r0 + (uint32_t)__ffsll((long long)l2) - 1 : r0;
            l2 &= l2 - 1;
            v[e] = a.sc[min(r, n - 1)];
          }
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            if (left) part = __fadd_rn(part, v[e]);
            left &= left - 1;
          }
        }
      }
      x_h = fv_block_tree_sum<T / 64>(part, wave_max);
      // the second neurons' total is added to the winners' (the checker's order)
      if (DELTA) x_h = __fadd_rn(x_h, fv_block_tree_sum<T / 64>(part2, wave_max));
    }
    base = 0;
    if (c_h != 0 && a.slot_region == 0) {
      // The number of windows won by lower neurons is the neuron's place in a class's slot region where the
      // blocks have no regions of their own. It is counted in the 16-bit winner array: 16-byte pieces dealt over the threads, two winners
      // compared per operation (winner - h is negative in a 16-bit half exactly where the winner is lower;
      // both are below 2^15). The entries behind the step's last window, up to the end of its piece, hold
      // 0x7fff.
      const uint32_t n8 = (n + 7) / 8;
      const fv_short2 hh = {(short)h, (short)h};
      fv_short2 below = {0, 0};
      // n <= 8 * 8 * NW * T: up to 8 NW pieces per thread, in batches of four loads with no branch between them (a
      // piece past the end reads the last one again and counts as 0x7fff)
#pragma unroll
      for (int g0 = 0; g0 < 8 * NW; g0 += 4) {
        if (g0 * T < n8) {  // the same answer in the whole block
          int4 v4[4];
#pragma unroll
          for (int g = 0; g < 4; ++g) v4[g] = ((const int4 *)a.win)[min(tid + (g0 + g) * T, n8 - 1)];
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            int4 v = v4[g];
            if (tid + (g0 + g) * T >= n8) v = make_int4(0x7fff7fff, 0x7fff7fff, 0x7fff7fff, 0x7fff7fff);
            below += (__builtin_bit_cast(fv_short2, v.x) - hh) >> 15;
            below += (__builtin_bit_cast(fv_short2, v.y) - hh) >> 15;
            below += (__builtin_bit_cast(fv_short2, v.z) - hh) >> 15;
            below += (__builtin_bit_cast(fv_short2, v.w) - hh) >> 15;
          }
        }
      }
      base = fv_block_sum_u32<T / 64>((uint32_t)(-((int)below.x + (int)below.y)), red2);
    }
    if (q == 0 && tid == 0) {
      a.group_base_out[h] = base;  // used where it was counted
      a.group_count_out[h] = c_h;
      a.xx_out[h] = x_h;  // (+0 for a neuron without a window)
      if (DELTA) {
        a.group_base2_out[h] = 0;
        a.group_count2_out[h] = c2_grouped;
      }
    }
  } else {
    c_h = a.group_count[h];
  }
  const uint32_t c2_h = DELTA ? (GROUPING ? c2_grouped : a.group_count2[h]) : 0u;
  if (c_h == 0 && c2_h == 0) {
    if (tid == 0) {
      a.bmax_sparse[blk] = 0.0f;
      a.slot_count[blk] = 0;
      a.row_hits[blk] = 0;
    }
    return;
  }
  if (GROUPING) {
    // a neuron with no more window positions than the block has threads: all of it in the class-0 block
    const uint32_t class_cols0 = (2 * a.V + FV_NB_CLASSES - 1) >> FV_NB_CLASS_SHIFT;
    // (the same answer in the neuron's four blocks; both forms have a counter for every column of a class: halves
    // of CW words, or, with two counts per column, 2 CW words)
    const bool light = a.light && a.slot_region != 0 && (c_h + c2_h) * a.stride <= T && class_cols0 <= 2u * CW;
    if (light) {
      if (q != 0) {
        if (tid == 0) {
          a.bmax_sparse[blk] = 0.0f;  // the neuron's records are counted by its class-0 block
          a.row_hits[blk] = 0;
        }
        return;
      }
      {
        uint32_t at = my_off;  // the window ids by rank
#pragma unroll
        for (int i = 0; i < NW; ++i)
          for (uint64_t mm = mask[i]; mm; mm &= mm - 1) ord[at++] = (ord_t)(r0 + 64 * i + (uint32_t)__ffsll((long long)mm) - 1);
        if (DELTA) {
          at = c_h + my_off2;  // behind them those in which the neuron came second
          for (uint64_t mm = mask2; mm; mm &= mm - 1) ord[at++] = (ord_t)(r0 + (uint32_t)__ffsll((long long)mm) - 1);
        }
      }
      fv_sparse_light<DELTA, ord_t>(a, h, blk, c_h, c2_h, x_h, cnt, ord, red2, sh_hits, wave_max);
      return;
    }
  }
  // counts of the block's elements that hold the row's largest / second largest weight (every path to the
  // elements passes a barrier)
  if (tid == 0) sh_hits[0] = sh_hits[1] = 0;
  uint32_t hits1 = 0, hits2 = 0;  // the same in all lanes of a wave
  // (GROUPING: done as soon as the count was known) the waves of the few heaviest blocks go first
  if (!GROUPING && c_h > FV_SP_HEAVY) __builtin_amdgcn_s_setprio(3);
  if (!GROUPING) base = a.group_base[h];
  const uint32_t base2 = DELTA && !GROUPING ? a.group_base2[h] : 0u;
  if (!GROUPING) x_h = a.xx[h];
  float ds_max = 0.0f;
  const uint32_t *order = (GROUPING ? a.order_out : a.order) + base;  // GROUPING: also written here, through order_out
  const uint32_t n_cols = 2 * a.V;
  const uint32_t m_ent = max(c_h, c2_h) * a.w;
  // the block's records: no more than (c_h + c2_h) * w of them, behind those of the lower neurons
  const bool regions = GROUPING && a.slot_region != 0;
  // (without regions of their own: behind the records of the lower neurons in the class's part)
  const uint64_t slot_first = regions ? 0ull : (uint64_t)q * a.slot_stride + (uint64_t)(base + base2) * a.w;
  // where the block's records lie (fv_slot_place, the block's part of it formed once)
  const uint32_t slot_primary = min(a.slot_region, FV_SLOT_PRIMARY);
  const uint64_t place_low = regions ? (uint64_t)blk * slot_primary : slot_first;
  const uint64_t place_high = regions ? fv_slot_place(blk, slot_primary, a.slot_region, a.n_blocks) - slot_primary : slot_first;

  const uint32_t stage_cap = fv_sparse_stage_cap(a.stride);  // window ids staged in LDS at a time
  const bool staged_once = !DELTA && c_h <= stage_cap;  // the usual case: the neuron's window ids are staged here
  if (!GROUPING) {
    for (uint32_t i = tid; i < CW / 4; i += T) ((uint4 *)cnt)[i] = make_uint4(0, 0, 0, 0);
    if (DELTA)
      for (uint32_t i = tid; i < CW / 4; i += T) ((uint4 *)cnt2)[i] = make_uint4(0, 0, 0, 0);
  }
  // GROUPING: the window ids of ranks [j0, j0 + FV_SP_STAGE) into LDS, every thread those of its own matches (its
  // ranks start at my_off; a neuron with more windows than LDS stages is staged part by part, each time
  // from the bit row's words in registers)
  auto stage_ids = [&](uint32_t j0, int second = 0) {
    uint32_t at = (second ? my_off2 : my_off) - j0;  // wraps below 0 for the ranks in front of the part
    // the two halves of a word one after the other, four matches between two branches, as many rounds as the
    // wave's busiest thread needs (a taken branch costs a lone wave as much as four or five instructions)
#pragma unroll
    for (int half = 0; half < 2 * NW; ++half) {
      uint32_t mm = (uint32_t)((second ? mask2 : mask[half >> 1]) >> (32 * (half & 1)));
      const uint32_t first = r0 + 32u * half;
      const uint32_t rounds = (fv_wave_max_u32((uint32_t)__popc(mm)) + 3u) >> 2;
      for (uint32_t it = 0; it < rounds; ++it) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          // (no branch around a match: one masked store, the rest by selects; a thread out of matches adds nothing)
          const bool more = mm != 0;
          if (more && at < stage_cap) ord[at] = (ord_t)(first + (uint32_t)__ffs((int)mm) - 1u);
          at += more ? 1u : 0u;
          mm &= mm - 1;
        }
      }
    }
  };
  if (GROUPING) {
    if (staged_once) stage_ids(0);
    // the counting pass starts behind a barrier
  } else {
    if (staged_once)
      for (uint32_t i = tid; i < c_h; i += T) ord[i] = (ord_t)order[i];
    fv_lds_barrier();
  }

  // No counter can exceed the neuron's number of window positions: below 2^16 of them, two 16-bit
  // counters share a word and one pass covers twice as many columns.
  const bool narrow = m_ent < 65536u;
  const uint32_t span = narrow ? 2 * CW : CW;          // class columns per pass
  const uint32_t class_cols = (n_cols + FV_NB_CLASSES - 1) >> FV_NB_CLASS_SHIFT;  // columns of a class
  uint32_t emitted = 0;

  auto nothing = []() {};

  for (uint32_t lo = 0; lo < class_cols; lo += span) {
    for (int l = 0; l < (DELTA ? 2 : 1); ++l) {
      const uint32_t *ids = l == 0 ? order : a.order2 + base2;
      const uint32_t n_ids = l == 0 ? c_h : c2_h;
      uint32_t *counters = l == 0 ? cnt : cnt2;
      for (uint32_t j0 = 0; j0 < n_ids; j0 += stage_cap) {
        const uint32_t n_staged = min(n_ids - j0, stage_cap);
        if (!staged_once) {
          fv_lds_barrier();  // the previous part has been counted
          if (GROUPING) {
            stage_ids(j0, l);
          } else {
            for (uint32_t i = tid; i < n_staged; i += T) ord[i] = (ord_t)ids[j0 + i];
          }
          fv_lds_barrier();
        }
        if (narrow)
          fv_sparse_count_any<true, ord_t>(counters, ord, n_staged, a.pad_row, a.idx, a.stride, q, lo, span, tid, nothing);
        else
          fv_sparse_count_any<false, ord_t>(counters, ord, n_staged, a.pad_row, a.idx, a.stride, q, lo, span, tid, nothing);
      }
    }
    // Every non-zero counter is one distinct element. Their positions are collected in LDS, up to
    // FV_SP_LIST_CAP at a time; a counter is cleared when its element is taken, so what did not fit
    // is found again by the next round.
    uint32_t found;
    do {
      if (tid == 0) sh_pos = 0;
      fv_lds_barrier();
      {
        // bit 8 * i + u of `mine`: counter u of the thread's i-th group of four words is non-zero
        constexpr int n_groups = (CW / 4 + T - 1) / T;
        static_assert(n_groups <= 8, "a 64-bit mask holds eight groups");
        uint64_t mine = 0;
#pragma unroll
        for (int i = 0; i < n_groups; ++i) {
          const uint32_t g4 = min(tid + i * T, (uint32_t)CW / 4 - 1);
          uint4 c4 = ((const uint4 *)cnt)[g4];
          if (DELTA) {
            const uint4 d4 = ((const uint4 *)cnt2)[g4];
            if (narrow) {
              // a 16-bit half is non-zero in the union if it is in either word: OR keeps that
              c4.x |= d4.x; c4.y |= d4.y; c4.z |= d4.z; c4.w |= d4.w;
            } else {
              c4.x |= d4.x; c4.y |= d4.y; c4.z |= d4.z; c4.w |= d4.w;
            }
          }
          if (tid + i * T >= CW / 4) c4 = make_uint4(0, 0, 0, 0);
          const uint32_t cw[4] = {c4.x, c4.y, c4.z, c4.w};
          uint32_t bits = 0;
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            if (narrow) {
              bits |= ((cw[u] & 0xffffu) ? 1u : 0u) << (2 * u);
              bits |= ((cw[u] >> 16) ? 1u : 0u) << (2 * u + 1);
            } else {
              bits |= (cw[u] ? 1u : 0u) << u;
            }
          }
          mine |= (uint64_t)bits << (8 * i);
        }
        // list positions: prefix sum inside the wave, one LDS atomic per wave
        const uint32_t my = (uint32_t)__popcll(mine);
        const int lane = tid & 63;
        const uint32_t incl = fv_wave_inclusive_scan_u32(my);
        uint32_t wave_base = 0;
        if (lane == 63 && incl) wave_base = atomicAdd(&sh_pos, incl);
        wave_base = fv_readlane(wave_base, 63);
        uint32_t e = wave_base + incl - my;
        while (mine) {
          const uint32_t b = (uint32_t)__ffsll((long long)mine) - 1;
          mine &= mine - 1;
          if (e < FV_SP_LIST_CAP) list[e] = (uint16_t)((tid + (b >> 3) * T) * (narrow ? 8u : 4u) + (b & 7u));
          ++e;
        }
      }
      fv_lds_barrier();
      found = sh_pos;
      const uint32_t take = min(found, (uint32_t)FV_SP_LIST_CAP);
      // one element per thread (four in flight): save its weight and its count in a slot record,
      // plant the sentinel, take |ds| (the dense term plus count additions of 1/f; a row with
      // xx == 0 has ds == 0)
      // number of the round's first record, for the sentinels (saturated: a step with more records than a
      // sentinel can name is not finished by the launch that reads the numbers)
      const uint32_t record0 = (uint32_t)min((regions ? 0ull : slot_first) + emitted, (uint64_t)FV_SENTINEL_MAX);
      // a round's records are numbered from a multiple of the list's length: all in the first part of the block's
      // region or all in the second (fv_slot_place)
      static_assert(FV_SLOT_PRIMARY % FV_SP_LIST_CAP == 0, "a round of records does not straddle the two parts of a region");
      const uint64_t round_place = emitted < slot_primary ? place_low : place_high;
      // the row's two largest weights: the same address in the whole block, fetched where they are used
      const float2 top2 = a.top2_known ? a.row_top2[h] : make_float2(0.0f, 0.0f);
      for (uint32_t eb = tid; eb < take; eb += 4 * T) {
        uint32_t pe[4], ne[4], n2e[4];
        float wv[4], fe[4], le[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const uint32_t k = list[min(eb + u * T, take - 1)];
          const uint32_t word = narrow ? cnt[k >> 1] : cnt[k];
          ne[u] = narrow ? (word >> (16 * (k & 1))) & 0xffffu : word;
          n2e[u] = 0;
          if (DELTA) {
            const uint32_t word2 = narrow ? cnt2[k >> 1] : cnt2[k];
            n2e[u] = narrow ? (word2 >> (16 * (k & 1))) & 0xffffu : word2;
          }
          const uint32_t col = ((lo + k) << FV_NB_CLASS_SHIFT) | q;
          pe[u] = col * a.ldk + h;
          wv[u] = a.Wt[pe[u]];
          fe[u] = a.invf[col >= a.V ? col - a.V : col];
          le[u] = col >= a.V ? a.lmid : a.lbase;
          if (eb + u * T < take) {
            if (narrow) {
              atomicAnd(&cnt[k >> 1], 0xffff0000u >> (16 * (k & 1)));
              if (DELTA) atomicAnd(&cnt2[k >> 1], 0xffff0000u >> (16 * (k & 1)));
            } else {
              cnt[k] = 0;
              if (DELTA) cnt2[k] = 0;
            }
          }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
          if (eb + u * T < take) {
            fv_slot rec;
            rec.p = pe[u];
            rec.n = ne[u];
            rec.wv = wv[u];
            rec.f = fe[u];
            const uint32_t number = emitted + eb + u * T;
            const uint64_t place = round_place + number;
            a.slots[place] = rec;
            if (DELTA) a.slot_n2[place] = n2e[u];
            a.Wt[pe[u]] = fv_sentinel(record0 + eb + u * T);
            // counted per wave from lane masks: the counts stay in scalar registers
            const float aw = fabsf(wv[u]);
            hits1 += (uint32_t)__popcll(__ballot(aw == top2.x));
            hits2 += (uint32_t)__popcll(__ballot(aw == top2.y && top2.y < top2.x));
            if (x_h != 0.0f)
              ds_max = fv_absmax_keep(ds_max, DELTA ? fv_sparse_ds2(x_h, wv[u], fe[u], ne[u], a.delta, n2e[u], le[u])
                                                    : fv_sparse_ds(x_h, wv[u], fe[u], ne[u], le[u]));
          }
      }
      emitted += take;
      fv_lds_barrier();
    } while (found > FV_SP_LIST_CAP);
  }
  if ((tid & 63u) == 0 && (hits1 | hits2)) {
    atomicAdd(&sh_hits[0], hits1);
    atomicAdd(&sh_hits[1], hits2);
  }
  const float bm = fv_block_max_nonneg<FV_SP_THREADS / 64>(ds_max, wave_max);  // behind its barriers every wave's hits are counted
  if (tid == 0) {
    a.bmax_sparse[blk] = bm;
    a.slot_count[blk] = emitted;
    a.row_hits[blk] = min(sh_hits[0], 3u) | (min(sh_hits[1], 3u) << 2);
  }
}

// CW: words of the block's LDS counter array (two 16-bit counters each while a neuron has fewer than 2^16
// window positions). FV_NB_CNT_WORDS, six blocks per compute unit, covers the 10000 columns per class of the
// headline shape in one pass; FV_NB_CNT_WORDS_WIDE, five blocks per compute unit, is taken where it saves a pass
// (25000 columns per class at V = 50000: two passes instead of three).
template <bool DELTA, int CW, bool IDS16 = false>
__global__ __launch_bounds__(FV_SP_THREADS) void fv_sparse_kernel(fv_sparse_args a) {
  fv_sparse_block<DELTA, false, CW, IDS16>(a);
}

// The form that groups for itself: with its 16-bit window ids six blocks fit a compute unit's LDS, and
// the register count is held to what six waves per SIMD allow.
__global__ __launch_bounds__(FV_SP_THREADS) __attribute__((amdgpu_waves_per_eu(6))) void fv_sparse_grouping_kernel(
    fv_sparse_args a) {
  fv_sparse_block<false, true, FV_NB_CNT_WORDS>(a);
}

__global__ __launch_bounds__(FV_SP_THREADS) void fv_sparse_grouping_wide_kernel(fv_sparse_args a) {
  fv_sparse_block<false, true, FV_NB_CNT_WORDS_WIDE>(a);
}

// The anti-Hebbian form that groups for itself: both of a neuron's window lists from bit rows. With two counter
// arrays of full length it takes 47 KB of LDS and three blocks share a compute unit (arrays of half the length, six
// blocks, two counting passes per class measured 3 us slower at 10000 windows of 11 over 400 neurons).
template <int CW>
__global__ __launch_bounds__(FV_SP_THREADS) void fv_sparse_grouping_delta_kernel(fv_sparse_args a) {
  fv_sparse_block<true, true, CW>(a);
}
