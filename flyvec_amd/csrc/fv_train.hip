// The FlyVec training minibatch step on one MI355X.
//
// Replaces the kernel chain of flyvec/src/cuda_funcs.cu:1662-1803 (sparse input, frequency
// scaling, p = 2; delta, Lmid / Lbase and the pruning sampler included).  The reference
// materialises ds (K x N) and walks it five times per step; here ds is never stored and the only
// global atomic is the OR that marks a window in its winner's bit row:
//
//   1. gather+winner   one wavefront per window: sampler (cuda_funcs.cu:915-936), raw
//                      activation = sum of ~w token rows of the token-major matrix with the K
//                      neurons spread over lanes (:248-263, double accumulators, one rounding),
//                      argmax by a wave reduction (:488-561) and the winner's frequency-scaled
//                      activation (:289-305; it is only ever read at the winner, :731).
//   2. group + xx      one block per neuron h: the ordered list of the windows h won and xx[h], the
//                      sum of their scaled activations (:722-744 -- the reference's atomic order
//                      is undefined, this one is fixed, so a step is reproducible bit for bit).
//                      A launch of its own only for batches beyond 16384 windows and for steps
//                      with the anti-Hebbian term: otherwise the blocks of launch 3 do it
//                      themselves, from the bit rows launch 1 leaves.
//   3. sparse owners   four blocks per neuron, one per column class: the sparse Hebbian term of
//                      row h (:657-672). A block alone owns its elements (h, column), so it counts
//                      repeated columns in LDS and for each distinct one saves the true weight and
//                      the count in a slot record, evaluates ds there, and plants a sentinel in W.
//   4. dense passes    max|ds| with ds = -xx[h] * W (:394-406; cu_special_reduction.cu:26-99,
//                      153-189), then W += s * ds where |s * ds| > 1e-10, s = eps / max(prec,
//                      max|ds|) (cuda_funcs.cu:1797-1803, cu_special_reduction.cu:316-354), then the
//                      final value of every sparse element over its sentinel. One launch that keeps
//                      W in registers between the passes when the matrix fits the register file of
//                      the machine, otherwise three launches (4a max, 5 update, 6 slot update).
//
// Every one of the n additions of 1/f onto ds[h][i] adds the same value, so the reference's
// result for that element depends only on n; replaying n sequential fp32 adds reproduces it
// exactly whatever order its atomics ran in.
#include <math.h>
#include <string.h>

#include <atomic>
#include <type_traits>
#include <utility>
#include <vector>

#include "fv_internal.h"
#include "fv_permute.h"
#include "fv_repeat_add.h"

// Written over W[p] while the true weight of a sparse element waits in its slot record: a NaN whose
// 23 mantissa bits hold the number of that record plus one (so they are never all zero, which would
// be an infinity), saturated at the largest value. A step whose record numbers all fit takes the
// single dense launch, where the thread that meets the NaN finds the record through it; the other
// launch forms only rely on it being a NaN.
#define FV_SENTINEL_EXP 0x7f800000u
#define FV_SENTINEL_MAX 0x007fffffu
__device__ __forceinline__ float fv_sentinel(uint32_t record) {
  return __uint_as_float(FV_SENTINEL_EXP | min(record + 1u, FV_SENTINEL_MAX));
}

struct __attribute__((aligned(16))) fv_slot {
  uint32_t p;  // element index i * ldk + h
  uint32_t n;  // pending additions of 1/f
  float wv;    // the weight the sentinel replaced
  float f;     // 1/f of the element's token
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
  uint64_t *pstart;    // starts[perm[i]]: where the i-th window of the current order begins
  uint64_t *perm_alt;  // second permutation buffer, allocated by the first shuffle
  uint64_t n_windows;
  float *invf;
  int32_t *idx;     // B rows of idx_stride column indices of the current minibatch (w used, the rest -1)
  uint32_t idx_stride;  // w rounded up to 4: rows are read 16 bytes at a time
  // the single dense launch samples the column indices of the minibatch expected next (the windows
  // that follow, a full batch or what is left) into idx_ahead while it waits between its passes;
  // a step that finds its own windows there swaps the buffers and skips the sampler's look-ups
  int32_t *idx_ahead;
  bool ahead_valid;
  uint64_t ahead_first;
  uint32_t ahead_n;
  int32_t *win;     // B winners
  uint16_t *win16;  // the same, 16 bits each (padded by 64)
  // Steps whose sparse launch groups for itself: the winner kernel sets bit r of the winner's row of
  // won[parity]; the sparse launch reads the rows and clears the other parity's, which the next such
  // step fills. Null when the batch is too large.
  uint32_t *won[2];        // K rows of won_words words each
  uint32_t won_words;      // words per row (even)
  uint32_t won_parity;     // the pair the last such step used
  // anti-Hebbian form (delta != 0), allocated with the first such step: the second neuron of every
  // window, its scaled activation, the windows grouped by it, the second count of every slot record
  int32_t *win2;
  uint16_t *win2_16;
  float *sc2;
  uint32_t *order2, *group_base2, *group_count2;
  uint32_t *slot_n2;
  fv_slot *slots2;  // records of a step with delta != 0: twice the room
  float last_delta;
  float *sc;        // B scaled activations at the winner
  uint32_t *order;  // B window ids grouped by winner, ascending inside a group
  uint32_t *group_base, *group_count;  // K each
  fv_slot *slots;   // FV_NB_CLASSES regions of B x w slot records
  // a region of slot_region records for every block of the sparse launch that groups for itself (0: none, the
  // blocks share the class regions of slots[])
  fv_slot *slots_blocks;
  uint32_t slot_region;
  bool no_block_regions;  // fv_trainer_set_slot_regions(0): the class regions are used all the same
  uint32_t *slot_count;  // K * FV_NB_CLASSES
  float *xx;        // ldk
  float *bmax;      // max|ds| of each block of the absmax launch, then of each block of the sparse launch
  float *scalars;   // [0] max|ds| of the last step, [1] non-zero once a single-launch dense pass has given up
  uint32_t last_n;
  uint64_t last_first;
  float last_eps;
  uint64_t shuffle_calls;
  bool have_corpus, have_weights;
  unsigned dense_blocks;   // blocks of the absmax launch
  unsigned update_blocks;  // blocks of the dense update launch
  // one launch for both dense passes (a matrix that fits the machine's registers): blocks, 16-byte
  // groups per thread (0 = two launches), the arrival word of every block, launches so far, and a
  // host-visible word a block sets when it gave up waiting for the others
  unsigned onepass_blocks, onepass_unroll;
  unsigned onepass_active;  // threads of a block of that launch that own elements (a multiple of ldk / 4)
  bool onepass;  // in use (fv_trainer_set_dense_launches)
  // the same launch with the rows streamed through the registers (any matrix size): available, in use
  bool stream_ok, onepass_stream;
  uint32_t hit_cap_limit;  // fv_trainer_set_sentinel_list: 0, or fewer entries than the launches' LDS lists hold
  // The two largest |W| of every row, kept by the single dense launch so that it knows max|ds| without
  // a pass over the matrix: each block's share after a launch (top2_part), merged by the next step's
  // winner kernel (row_top2); what the sparse launch reports on them (row_hits); whether top2_part
  // describes the matrix as it is (top2_valid: set by a single dense launch, cleared by every other
  // write of the matrix), and whether the last whole step used them.
  float2 *row_top2, *top2_part;
  float2 *top2_stage;  // inside row_top2's allocation
  bool top2_merged;    // row_top2 already holds the merged pairs (separate dense launches merge behind themselves)
  uint32_t *row_hits;
  uint32_t *path_count;  // device: launches that took max|ds| from them / that made the pass
  bool top2_valid, last_top2_known;
  uint32_t top2_n_part;  // shares per row that the last dense launches left (their number of blocks)
  unsigned update_threads;  // 256, or 512 when a row has more than 256 groups of four neurons
  unsigned sparse_base;  // index in bmax of the sparse launch's first block maximum
  bool stale_tail;  // run_epoch trains a final partial minibatch with the previous one's rows behind its own
  bool separate_grouping;  // the grouping kernel always runs as a launch of its own (fv_trainer_set_grouping_launch)
  bool last_grouped_in_sparse;  // the form the last whole step took: a launch on its own repeats that form
  unsigned long long *arrive;
  uint32_t onepass_epoch;
  uint32_t onepass_spin_limit;
  uint32_t *onepass_status;  // pinned host word: 0, or the tag of the first launch that gave up
  uint32_t step_tag;         // tag of the step being enqueued: run_epoch numbers its steps from 1, else 0
  uint64_t giveups_recovered;  // epochs in which run_epoch took up again behind a launch that gave up
  float update_cut;  // largest fp32 <= 1e-10
};

// ---- the two largest weights of every row ------------------------------------------------------------

// The two largest of a multiset of non-negative values, kept as (m1 >= m2): one more value, and the
// union with another pair.
__device__ __forceinline__ void fv_top2_insert(float &m1, float &m2, float a) {
  m2 = fmaxf(m2, fminf(m1, a));
  m1 = fmaxf(m1, a);
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
  // the window's bit in the winner's row: issued first, it travels while the scaled activation is formed
  if (lane == 0 && a.won && hstar < a.K)
    atomicOr(&a.won[(uint64_t)hstar * a.won_words + (r >> 5)], 1u << (r & 31u));
  // the scaled activation is only ever read at the chosen neurons (flyvec/src/cuda_funcs.cu:731)
  const float s = fv_scaled_activation<WEIGHTED>(a, idx, hstar);
  if (lane == 0) {
    a.win[r] = (int32_t)hstar;
    a.win16[r] = (uint16_t)hstar;
    a.sc[r] = s;
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
    }
  }
}

// ---- kernel 2: group the windows by winner, xx ----------------------------------------------------
//
// One block per neuron h scans the winner array once (every thread a contiguous run, so per-thread
// match counts are in window order) and writes the neuron's windows, ascending, to
// order[group_base[h] .. +group_count[h]); it then adds their scaled activations in that order: xx[h].

#define FV_NB_MAX_THREADS 1024
#ifndef FV_NB_CLASS_SHIFT
#define FV_NB_CLASS_SHIFT 2
#endif
#define FV_NB_CLASSES (1 << FV_NB_CLASS_SHIFT)  // column classes per neuron (kernel 3)
#define FV_NB_CNT_WORDS 5120    // LDS counter words per class block (20 KB)
#define FV_NB_CNT_WORDS_WIDE 6272  // or 24.5 KB, where that saves a pass
#define FV_SP_LIST_CAP 1024     // positions of non-zero counters collected in LDS at a time
#define FV_SP_CHUNK 16          // window positions read by 4 neighbouring lanes, 16 bytes each
#define FV_IDX_PAD 80            // entries of -1 behind the index matrix: a padding row (up to 64 entries) and spare
#define FV_SP_STAGE 2048        // window ids staged in LDS at a time
#ifndef FV_SP_THREADS
#define FV_SP_THREADS 256       // threads of a class block
#endif
#ifndef FV_SP_LOADS
#define FV_SP_LOADS 8           // most 16-byte loads a lane has in flight in the counting pass
#endif
#define FV_SP_HEAVY 128         // a class block of a neuron with more windows than this runs at raised wave priority
#define FV_NB_ROUND 2048        // scaled activations staged in LDS at a time
#define FV_NB_LOADS 32          // winners a thread of the grouping kernel fetches together

struct fv_group_args {
  const uint16_t *win;  // 16-bit winners, padded: readable up to n rounded up to 64
  const float *sc;
  uint32_t *order;
  uint32_t *group_base;
  uint32_t *group_count;
  float *xx;
  uint32_t n;
  float scale;          // every scaled activation is multiplied by this first (1, or -delta for the second neurons)
  uint32_t accumulate;  // add the total to xx[h] instead of storing it
};

// ds of one sparse element: the dense term, then n sequential additions of l * 1/f, l the weight of
// the element's window position (flyvec/src/cuda_funcs.cu:675-697: a double product of two floats
// rounded once is their fp32 product; l = 1 leaves 1/f as it is).
__device__ __forceinline__ float fv_sparse_ds(float xx, float wv, float f, uint32_t n, float l) {
  return fv_add_repeat(__fmul_rn(-xx, wv), __fmul_rn(l, f), n);
}

__device__ __forceinline__ float fv_absmax_keep(float m, float v) {
  const float a = fabsf(v);
  return a > m ? a : m;  // a NaN never replaces m, as in the reference's comparison
}

// ds of one sparse element with the anti-Hebbian term: after the n additions of l * 1/f, n2 additions
// of (-delta * l) * 1/f (flyvec/src/cuda_funcs.cu:667-668, 689, 693; this order of the additions is
// the checker's).
__device__ __forceinline__ float fv_sparse_ds2(float xx, float wv, float f, uint32_t n, float delta, uint32_t n2,
                                               float l) {
  return fv_add_repeat(fv_sparse_ds(xx, wv, f, n, l), __fmul_rn(__fmul_rn(-delta, l), f), n2);
}

// Block-wide maximum of non-negative floats (blocks of up to 16 waves; smem holds one float per wave).
__device__ __forceinline__ float fv_block_max_nonneg(float m, float *smem) {
  const uint32_t wm = fv_wave_max_u32(__float_as_uint(m));
  __syncthreads();
  if ((threadIdx.x & 63) == 0) smem[threadIdx.x >> 6] = __uint_as_float(wm);
  __syncthreads();
  float r = smem[0];
  for (uint32_t i = 1; i < (blockDim.x >> 6); ++i) r = fmaxf(r, smem[i]);
  return r;
}

// Sum over the block of one value per thread (result in every thread).
__device__ __forceinline__ uint32_t fv_block_sum_u32(uint32_t v, uint32_t *smem /*17*/) {
  v = fv_wave_sum_u32(v);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n_waves = blockDim.x >> 6;
  __syncthreads();
  if (lane == 0) smem[wave] = v;
  __syncthreads();
  uint32_t t = 0;
  for (int i = 0; i < n_waves; ++i) t += smem[i];
  return t;
}

// Exclusive prefix sum of one value per thread over the block.
__device__ __forceinline__ uint32_t fv_block_exclusive_scan(uint32_t v, uint32_t *smem /*17*/) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t incl = fv_wave_inclusive_scan_u32(v);
  __syncthreads();
  if (lane == 63) smem[wave] = incl;
  __syncthreads();
  uint32_t before = 0;
  for (int i = 0; i < wave; ++i) before += smem[i];
  return before + incl - v;
}

// Barrier for data exchanged through LDS only: waits for the wave's LDS operations, not for its
// global loads and stores still in flight.
__device__ __forceinline__ void fv_lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Exclusive prefix sum and total of one value per thread over the block, in one pass. LDS_ONLY: the
// barriers do not wait for the caller's global loads in flight.
template <bool LDS_ONLY = false>
__device__ __forceinline__ uint32_t fv_block_scan_total(uint32_t v, uint32_t *smem /*17*/, uint32_t *total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n_waves = blockDim.x >> 6;
  const uint32_t incl = fv_wave_inclusive_scan_u32(v);
  if (LDS_ONLY) fv_lds_barrier(); else __syncthreads();
  if (lane == 63) smem[wave] = incl;
  if (LDS_ONLY) fv_lds_barrier(); else __syncthreads();
  uint32_t before = 0, all = 0;
  for (int i = 0; i < n_waves; ++i) {
    const uint32_t t = smem[i];
    before += i < wave ? t : 0u;
    all += t;
  }
  *total = all;
  return before + incl - v;
}

// SMALL: a thread's run is at most 64 windows and the minibatch has fewer than 2^16. The run is then
// fetched in one trip to memory (16 loads of 16 bytes in flight), the two counts travel through
// one block scan as the halves of a word, and the scaled activations of a thread's first matches
// are fetched while that scan runs.
// Winner number q (0 .. 7) of a 16-byte load of 16-bit winners.
__device__ __forceinline__ uint32_t fv_winner_of(const int4 &v, int q) {
  const uint32_t word = (uint32_t)((q >> 1) == 0 ? v.x : (q >> 1) == 1 ? v.y : (q >> 1) == 2 ? v.z : v.w);
  return (q & 1) ? word >> 16 : word & 0xffffu;
}

typedef short fv_short2 __attribute__((ext_vector_type(2)));

template <bool SMALL>
__global__ __launch_bounds__(FV_NB_MAX_THREADS) void fv_group_kernel(fv_group_args a) {
  __shared__ float scbuf[FV_NB_ROUND];
  __shared__ uint32_t red[17];

  const uint32_t h = blockIdx.x;
  const uint32_t tid = threadIdx.x, T = blockDim.x;
  const uint32_t n = a.n;
  const uint16_t *__restrict__ win = a.win;

  // A thread's run is a multiple of 8 windows, read as 16-byte loads of 8 winners; matches among
  // its first 64 windows are kept as a bit mask.
  const uint32_t seg = ((n + T - 1) / T + 7) & ~7u;
  const uint32_t r0 = min(tid * seg, n), r1 = min(r0 + seg, n);
  const uint32_t n_pad = (n + 63) & ~63u;
  uint32_t lt = 0, eq = 0;
  uint64_t mask = 0;
  uint32_t base, my_off, c_h;
  constexpr int PF = 8;
  float pf[PF];
  if (SMALL) {
    int4 wv4[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) wv4[q] = *(const int4 *)(win + min(r0 + 8 * q, n_pad - 8));
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      if (g * 16 < (int)seg) {  // the same answer in the whole block
#pragma unroll
        for (int q = 16 * g; q < 16 * g + 16; ++q) {
          const uint32_t wv = fv_winner_of(wv4[q >> 3], q & 7);
          const bool in = r0 + q < r1;
          lt += in && wv < h;
          const bool hit = in && wv == h;
          eq += hit;
          mask |= (uint64_t)hit << q;
        }
      }
    }
    uint64_t mm = mask;
#pragma unroll
    for (int q = 0; q < PF; ++q) {
      const uint32_t r = mm ? r0 + (uint32_t)__ffsll((long long)mm) - 1 : r0;
      pf[q] = __fmul_rn(a.scale, a.sc[min(r, n - 1)]);
      mm &= mm - 1;
    }
    uint32_t total;
    const uint32_t before = fv_block_scan_total(lt | (eq << 16), red, &total);
    base = total & 0xffffu;
    c_h = total >> 16;
    my_off = before >> 16;
  } else {
    for (uint32_t rb = r0; rb < r1; rb += FV_NB_LOADS) {
      int4 wv4[FV_NB_LOADS / 8];
#pragma unroll
      for (int q = 0; q < FV_NB_LOADS / 8; ++q) wv4[q] = *(const int4 *)(win + min(rb + 8 * q, n_pad - 8));
#pragma unroll
      for (int q = 0; q < FV_NB_LOADS; ++q) {
        const uint32_t wv = fv_winner_of(wv4[q >> 3], q & 7);
        const bool in = rb + q < r1;
        lt += in && wv < h;
        const bool hit = in && wv == h;
        eq += hit;
        const uint32_t o = rb + q - r0;
        mask |= o < 64 ? (uint64_t)hit << o : 0ull;
      }
    }
    base = fv_block_sum_u32(lt, red);  // windows won by lower neurons
    my_off = fv_block_exclusive_scan(eq, red);
    c_h = fv_block_sum_u32(eq, red);
  }
  if (tid == 0) {
    a.group_base[h] = base;
    a.group_count[h] = c_h;
  }
  // SMALL and the neuron's values fit scbuf: they are placed by rank here, without a trip through order[]
  const bool staged = SMALL && c_h <= FV_NB_ROUND;
  uint32_t *order = a.order + base;
  {
    uint32_t rank = my_off;
    uint64_t mm = mask;
    if (SMALL) {
#pragma unroll
      for (int q = 0; q < PF; ++q) {
        if (mm) {
          order[rank] = r0 + (uint32_t)__ffsll((long long)mm) - 1;
          if (staged) scbuf[rank] = pf[q];
          ++rank;
          mm &= mm - 1;
        }
      }
    }
    while (mm) {
      const uint32_t r = r0 + (uint32_t)__ffsll((long long)mm) - 1;
      order[rank] = r;
      if (staged) scbuf[rank] = __fmul_rn(a.scale, a.sc[r]);
      ++rank;
      mm &= mm - 1;
    }
    for (uint32_t r = r0 + 64; r < r1; ++r)
      if ((uint32_t)win[r] == h) order[rank++] = r;
  }
  __syncthreads();  // the neuron's part of order[] (and of scbuf) is now readable by the whole block

  // xx[h]: lane l of the first wave adds the neuron's scaled activations number l, l + 64, l + 128, ...
  // (window order) onto 0, then the 64 partial sums are added onto 0 in lane order. For up to 64
  // windows that is the plain sum in window order.
  float part = 0.0f;
  if (staged) {
    if (tid < 64) {
      // four values fetched together, added one after the other
      uint32_t j = tid;
      for (; j + 192 < c_h; j += 256) {
        const float v0 = scbuf[j], v1 = scbuf[j + 64], v2 = scbuf[j + 128], v3 = scbuf[j + 192];
        part = __fadd_rn(__fadd_rn(__fadd_rn(__fadd_rn(part, v0), v1), v2), v3);
      }
      for (; j < c_h; j += 64) part = __fadd_rn(part, scbuf[j]);
    }
  } else {
    for (uint32_t j0 = 0; j0 < c_h; j0 += FV_NB_ROUND) {
      const uint32_t mr = min(c_h - j0, (uint32_t)FV_NB_ROUND);
      for (uint32_t jb = tid; jb < mr; jb += 4 * T) {  // up to 4 independent loads per thread
        uint32_t r[4];
        float v[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) r[q] = order[j0 + min(jb + q * T, mr - 1)];
#pragma unroll
        for (int q = 0; q < 4; ++q) v[q] = __fmul_rn(a.scale, a.sc[r[q]]);
#pragma unroll
        for (int q = 0; q < 4; ++q)
          if (jb + q * T < mr) scbuf[jb + q * T] = v[q];
      }
      __syncthreads();
      if (tid < 64)
        for (uint32_t j = tid; j < mr; j += 64) part = __fadd_rn(part, scbuf[j]);  // FV_NB_ROUND % 64 == 0
      __syncthreads();
    }
  }
  // The partial sums in lane order, read straight from the lanes of the first wave (a partial sum
  // without values is +0, which changes nothing: the running total starts at +0 and so is never -0).
  if (tid < 64) {
    float xx = 0.0f;
#pragma unroll
    for (int l = 0; l < 64; ++l) xx = __fadd_rn(xx, __uint_as_float(fv_readlane(__float_as_uint(part), l)));
    if (tid == 0) a.xx[h] = a.accumulate ? __fadd_rn(a.xx[h], xx) : xx;
  }
}

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
  // Not 0 (grouping form only): every block has a region of slot_region records of its own in slots[], at
  // blockIdx * slot_region, and a sentinel names a record by its place in the block's region. A block has no
  // more records than its class has columns, so no block needs to know what the others write.
  uint32_t slot_region;
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
};

// Counting pass of one class block over the windows whose ids are staged in LDS: ord[0 .. n_staged),
// followed up to the next multiple of FV_SP_WPS * LOADS by the id of the padding row behind the
// index matrix (all -1). A row of idx is `stride` entries, a multiple of 4, those past w holding -1;
// four consecutive lanes read the sixteen positions of a chunk of one window 16 bytes each, so a
// wave's load covers sixteen windows. A lane issues LOADS loads back to back with no branch between
// them (the compiler waits for every load in flight at a branch target), then counts. With the
// class in the top bits and the column of the class below, one subtraction and one comparison tell
// whether an entry is this block's: of class q, inside [lo, lo + span), not masked, not padding.
#define FV_SP_WPS (FV_SP_THREADS / 4)  // windows the block takes per step
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

template <bool NARROW, int LOADS, typename Ord>
__device__ __forceinline__ void fv_sparse_count(uint32_t *cnt, const Ord *ord, uint32_t n_staged,
                                                const int32_t *__restrict__ idx, uint32_t stride, uint32_t q,
                                                uint32_t lo, uint32_t span, uint32_t tid) {
  const uint32_t c4 = 4u * (tid & 3u), slot = tid >> 2;
  const uint32_t steps = (n_staged + FV_SP_WPS - 1) / FV_SP_WPS;
  const uint32_t origin = (q << (32 - FV_NB_CLASS_SHIFT)) | lo;
  for (uint32_t c0 = 0; c0 < stride; c0 += FV_SP_CHUNK) {
    const bool live = c0 + c4 < stride;  // a row shorter than the chunk: the lanes past its end read its start again
    const uint32_t cc = live ? c0 + c4 : 0u;
    const uint32_t drop = live ? 0u : 0xffffffffu;
    for (uint32_t s0 = 0; s0 < steps; s0 += LOADS) {
      int4 iv[LOADS];
#pragma unroll
      for (int b = 0; b < LOADS; ++b)
        iv[b] = *(const int4 *)(idx + (uint64_t)ord[(s0 + b) * FV_SP_WPS + slot] * stride + cc);
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

// The same with the number of loads in flight fitted to the number of windows; pads ord[].
template <bool NARROW, typename Ord>
__device__ __forceinline__ void fv_sparse_count_any(uint32_t *cnt, Ord *ord, uint32_t n_staged, uint32_t pad_row,
                                                    const int32_t *__restrict__ idx, uint32_t stride, uint32_t q,
                                                    uint32_t lo, uint32_t span, uint32_t tid) {
  static_assert(FV_SP_STAGE % (FV_SP_WPS * FV_SP_LOADS) == 0 && FV_SP_LOADS % 4 == 0, "padding of ord[] stays inside it");
  const uint32_t per = FV_SP_WPS * (n_staged <= FV_SP_WPS ? 1 : n_staged <= FV_SP_WPS * 4 ? 4 : FV_SP_LOADS);
  const uint32_t padded = (n_staged + per - 1) / per * per;
  for (uint32_t i = n_staged + tid; i < padded; i += FV_SP_THREADS) ord[i] = (Ord)pad_row;
  fv_lds_barrier();
  if (per == FV_SP_WPS)
    fv_sparse_count<NARROW, 1, Ord>(cnt, ord, n_staged, idx, stride, q, lo, span, tid);
  else if (per == FV_SP_WPS * 4)
    fv_sparse_count<NARROW, 4, Ord>(cnt, ord, n_staged, idx, stride, q, lo, span, tid);
  else
    fv_sparse_count<NARROW, FV_SP_LOADS, Ord>(cnt, ord, n_staged, idx, stride, q, lo, span, tid);
}

// DELTA: the neuron's elements are counted over two lists of windows, those it won and those in
// which it came second, into two counter arrays; a record carries both counts.
// GROUPING: no grouping launch has run. Every class block takes its neuron's windows from the bit row
// the winner kernel has filled (a thread's two words are 64 windows: the step has no more than
// 64 * FV_SP_THREADS), counts the windows of lower neurons in the 16-bit winner array, stages the
// window ids in LDS by rank, and adds the neuron's scaled activations in the grouping kernel's order;
// the block of class 0 leaves xx[h], the neuron's count and its base for the dense launch and clears
// the neuron's row of the other bit-row buffer.
template <bool DELTA, bool GROUPING, int CW>
__device__ __forceinline__ void fv_sparse_block(const fv_sparse_args &a) {
  static_assert(!(DELTA && GROUPING), "the anti-Hebbian form has its two lists grouped by launches of their own");
  __shared__ uint32_t cnt[CW];
  __shared__ uint32_t cnt2[DELTA ? CW : 4];
  __shared__ uint16_t list[FV_SP_LIST_CAP];
  // window ids of a grouping step (at most 64 * FV_SP_THREADS windows, and the padding row behind them)
  // fit 16 bits: the smaller array lets one more block share a compute unit
  static_assert(64 * FV_SP_THREADS < 65536, "ids of a grouping step fit 16 bits");
  typedef typename std::conditional<GROUPING, uint16_t, uint32_t>::type ord_t;
  __shared__ ord_t ord[FV_SP_STAGE];
  __shared__ uint32_t sh_pos;
  __shared__ float sh_xx;
  __shared__ uint32_t sh_hits[2];
  __shared__ float sc64[GROUPING ? 64 : 1];  // activations of a neuron with up to 64 windows, by rank
  __shared__ float wave_max[16];
  __shared__ uint32_t red[17];
  constexpr uint32_t T = FV_SP_THREADS;
  const uint32_t h = blockIdx.x >> FV_NB_CLASS_SHIFT;
  const uint32_t q = blockIdx.x & (FV_NB_CLASSES - 1);
  const uint32_t tid = threadIdx.x;
  __shared__ uint32_t red2[GROUPING ? 17 : 1];
  uint32_t c_h, base, my_off = 0, r0 = 0;
  bool sc_complete = true;  // every thread's matches have their activations in pf[]
  uint64_t mask = 0;
  constexpr int PF = 4;
  float pf[PF];
  if (GROUPING) {
    const uint32_t n = a.n;
    // thread t takes windows 64 t .. 64 t + 63: two words of the neuron's row
    r0 = 64 * tid;
    uint2 mw = make_uint2(0u, 0u);
    if (2 * tid < a.won_words) mw = *(const uint2 *)(a.won + (uint64_t)h * a.won_words + 2 * tid);
    mask = (uint64_t)mw.x | ((uint64_t)mw.y << 32);
    const uint32_t eq = (uint32_t)__popcll(mask);
    if (q == 0) {
      if (2 * tid < a.won_words) *(uint2 *)(a.won_clear + (uint64_t)h * a.won_words + 2 * tid) = make_uint2(0u, 0u);
    }
    // the scaled activations of a thread's first matches travel while the scan runs
    uint64_t mm = mask;
#pragma unroll
    for (int e = 0; e < PF; ++e) {
      const uint32_t r = mm ? r0 + (uint32_t)__ffsll((long long)mm) - 1 : r0;
      pf[e] = a.sc[min(r, n - 1)];
      mm &= mm - 1;
    }
    // one block scan gives the ranks and the neuron's count, and tells whether any thread has more matches
    // than it has fetched activations for
    const bool wave_more = __ballot(eq > (uint32_t)PF) != 0ull;
    const uint32_t incl = fv_wave_inclusive_scan_u32(eq);
    if ((tid & 63u) == 63u) red[tid >> 6] = incl, red[8 + (tid >> 6)] = wave_more;
    fv_lds_barrier();
    uint32_t before = 0, total = 0;
    bool more = false;
#pragma unroll
    for (uint32_t i = 0; i < T / 64; ++i) {
      const uint32_t t = red[i];
      before += i < (tid >> 6) ? t : 0u;
      total += t;
      more = more || red[8 + i] != 0;
    }
    c_h = total;
    my_off = before + incl - eq;
    sc_complete = !more;
    base = 0;
    if (c_h != 0 && (a.slot_region == 0 || c_h > FV_SP_STAGE)) {
      // The number of windows won by lower neurons is the neuron's place in order[] (more windows than LDS
      // stages go through there) and in a class's slot region (where the blocks have no regions of their
      // own). It is counted in the 16-bit winner array: 16-byte pieces dealt over the threads, two winners
      // compared per operation (winner - h is negative in a 16-bit half exactly where the winner is lower;
      // both are below 2^15). The entries behind the step's last window, up to the end of its piece, hold
      // 0x7fff.
      const uint32_t n8 = (n + 7) / 8;
      const fv_short2 hh = {(short)h, (short)h};
      fv_short2 below = {0, 0};
#pragma unroll
      for (int g = 0; g < 8; ++g) {  // n <= 8 * 8 * T
        if (g * T < n8) {            // the same answer in the whole block
          const uint32_t i4 = tid + g * T;
          int4 v = ((const int4 *)a.win)[min(i4, n8 - 1)];
          if (i4 >= n8) v = make_int4(0x7fff7fff, 0x7fff7fff, 0x7fff7fff, 0x7fff7fff);
          below += (__builtin_bit_cast(fv_short2, v.x) - hh) >> 15;
          below += (__builtin_bit_cast(fv_short2, v.y) - hh) >> 15;
          below += (__builtin_bit_cast(fv_short2, v.z) - hh) >> 15;
          below += (__builtin_bit_cast(fv_short2, v.w) - hh) >> 15;
        }
      }
      base = fv_block_sum_u32((uint32_t)(-((int)below.x + (int)below.y)), red2);
    }
    for (uint32_t i = tid; i < CW / 4; i += T) ((uint4 *)cnt)[i] = make_uint4(0, 0, 0, 0);
    if (q == 0 && tid == 0) {
      a.group_base_out[h] = base;  // used where it was counted
      a.group_count_out[h] = c_h;
      if (c_h == 0) a.xx_out[h] = 0.0f;
    }
  } else {
    c_h = a.group_count[h];
  }
  const uint32_t c2_h = DELTA ? a.group_count2[h] : 0u;
  if (c_h == 0 && c2_h == 0) {
    if (tid == 0) {
      a.bmax_sparse[blockIdx.x] = 0.0f;
      a.slot_count[blockIdx.x] = 0;
      a.row_hits[blockIdx.x] = 0;
    }
    return;
  }
  // counts of the block's elements that hold the row's largest / second largest weight (every path to the
  // elements passes a barrier)
  if (tid == 0) sh_hits[0] = sh_hits[1] = 0;
  uint32_t hits1 = 0, hits2 = 0;  // the same in all lanes of a wave
  // The launch lasts as long as its few heaviest blocks: their waves go first wherever they share a
  // SIMD with the waves of light blocks.
  if (c_h > FV_SP_HEAVY) __builtin_amdgcn_s_setprio(3);
  if (!GROUPING) base = a.group_base[h];
  const uint32_t base2 = DELTA ? a.group_base2[h] : 0u;
  float x_h = GROUPING ? 0.0f : a.xx[h];
  float ds_max = 0.0f;
  const uint32_t *order = (GROUPING ? a.order_out : a.order) + base;  // GROUPING: also written here, through order_out
  const uint32_t n_cols = 2 * a.V;
  const uint32_t m_ent = max(c_h, c2_h) * a.w;
  // the block's records: no more than (c_h + c2_h) * w of them, behind those of the lower neurons
  const bool regions = GROUPING && a.slot_region != 0;
  const uint64_t slot_first = regions ? (uint64_t)blockIdx.x * a.slot_region
                                      : (uint64_t)q * a.slot_stride + (uint64_t)(base + base2) * a.w;
  fv_slot *slots = a.slots + slot_first;

  const bool staged_once = !DELTA && c_h <= FV_SP_STAGE;  // the usual case: the neuron's window ids are staged here
  if (!GROUPING) {
    for (uint32_t i = tid; i < CW / 4; i += T) ((uint4 *)cnt)[i] = make_uint4(0, 0, 0, 0);
    if (DELTA)
      for (uint32_t i = tid; i < CW / 4; i += T) ((uint4 *)cnt2)[i] = make_uint4(0, 0, 0, 0);
  }
  // xx[h] is added up in the grouping kernel's order: lane l of the first wave adds the values number
  // l, l + 64, ... onto 0, then the partial sums are added onto 0 in lane order (those of the lanes
  // from c_h on are +0 and change nothing). A neuron with up to 64 windows, each thread holding the
  // activations of all its matches, does that behind the counting pass, where the value is first
  // needed and the loads have long returned.
  bool xx_pending = GROUPING && staged_once && sc_complete && c_h <= 64;
  if (GROUPING) {
    // Window ids by rank: into LDS, or (more than LDS stages) to the neuron's part of order[], where
    // the neuron's four blocks write the same values.
    uint32_t rank = my_off;
    for (uint64_t mm = mask; mm; mm &= mm - 1) {
      const uint32_t r = r0 + (uint32_t)__ffsll((long long)mm) - 1;
      if (staged_once)
        ord[rank++] = (ord_t)r;
      else
        a.order_out[base + rank++] = r;
    }
    if (!xx_pending) {
      // A neuron with many windows: the activations are fetched by rank into the counter array
      // (cleared behind the block scan, and again by the first wave once it has added them).
      static_assert(FV_SP_STAGE <= CW && FV_SP_STAGE % 64 == 0 && FV_SP_STAGE <= 8 * T,
                    "a stage of activations fits the counters and one trip to memory");
      float *scbuf = (float *)cnt;
      float part = 0.0f;
      if (staged_once)
        fv_lds_barrier();  // the ids are in LDS
      else
        __syncthreads();  // the ids are in memory
      for (uint32_t j0 = 0; j0 < c_h; j0 += FV_SP_STAGE) {
        const uint32_t mr = min(c_h - j0, (uint32_t)FV_SP_STAGE);
        float v8[8];  // eight loads in flight per thread
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const uint32_t j = j0 + min(tid + u * T, mr - 1);
          v8[u] = a.sc[staged_once ? (uint32_t)ord[j] : order[j]];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (tid + u * T < mr) scbuf[tid + u * T] = v8[u];
        fv_lds_barrier();
        if (tid < 64) {
          uint32_t j = tid;
          for (; j + 192 < mr; j += 256) {  // four values fetched together, added one after the other
            const float v0 = scbuf[j], v1 = scbuf[j + 64], v2 = scbuf[j + 128], v3 = scbuf[j + 192];
            part = __fadd_rn(__fadd_rn(__fadd_rn(__fadd_rn(part, v0), v1), v2), v3);
          }
          for (; j < mr; j += 64) part = __fadd_rn(part, scbuf[j]);
        }
        if (j0 + FV_SP_STAGE < c_h) fv_lds_barrier();  // before the next stage overwrites this one
      }
      if (tid < 64) {
        float xx = 0.0f;
        if (c_h >= 64) {
#pragma unroll
          for (int l = 0; l < 64; ++l) xx = __fadd_rn(xx, __uint_as_float(fv_readlane(__float_as_uint(part), l)));
        } else {
          for (uint32_t l = 0; l < c_h; ++l)
            xx = __fadd_rn(xx, __uint_as_float(fv_readlane(__float_as_uint(part), (int)l)));
        }
        if (tid == 0) {
          sh_xx = xx;
          if (q == 0) a.xx_out[h] = xx;
        }
        const uint32_t used = (min(c_h, (uint32_t)FV_SP_STAGE) + 3) / 4;
        for (uint32_t i = tid; i < used; i += 64) ((uint4 *)cnt)[i] = make_uint4(0, 0, 0, 0);
      }
    }
    // the counting pass starts behind a barrier; sh_xx is read behind that pass
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

  for (uint32_t lo = 0; lo < class_cols; lo += span) {
    for (int l = 0; l < (DELTA ? 2 : 1); ++l) {
      const uint32_t *ids = l == 0 ? order : a.order2 + base2;
      const uint32_t n_ids = l == 0 ? c_h : c2_h;
      uint32_t *counters = l == 0 ? cnt : cnt2;
      for (uint32_t j0 = 0; j0 < n_ids; j0 += FV_SP_STAGE) {
        const uint32_t n_staged = min(n_ids - j0, (uint32_t)FV_SP_STAGE);
        if (!staged_once) {
          fv_lds_barrier();  // the previous part has been counted
          for (uint32_t i = tid; i < n_staged; i += T) ord[i] = (ord_t)ids[j0 + i];
          fv_lds_barrier();
        }
        if (narrow)
          fv_sparse_count_any<true, ord_t>(counters, ord, n_staged, a.pad_row, a.idx, a.stride, q, lo, span, tid);
        else
          fv_sparse_count_any<false, ord_t>(counters, ord, n_staged, a.pad_row, a.idx, a.stride, q, lo, span, tid);
      }
    }
    // Every non-zero counter is one distinct element. Their positions are collected in LDS, up to
    // FV_SP_LIST_CAP at a time; a counter is cleared when its element is taken, so what did not fit
    // is found again by the next round.
    uint32_t found;
    do {
      if (tid == 0) sh_pos = 0;
      if (GROUPING && xx_pending) {
        uint32_t rk = my_off;
        uint64_t mm = mask;
#pragma unroll
        for (int e = 0; e < PF; ++e)
          if (mm) {
            sc64[rk++] = pf[e];
            mm &= mm - 1;
          }
      }
      fv_lds_barrier();
      if (GROUPING && xx_pending) {
        if (tid < 64) {
          const float part = tid < c_h ? __fadd_rn(0.0f, sc64[tid]) : 0.0f;
          float xx = 0.0f;
          for (uint32_t l = 0; l < c_h; ++l)
            xx = __fadd_rn(xx, __uint_as_float(fv_readlane(__float_as_uint(part), (int)l)));
          if (tid == 0) {
            sh_xx = xx;
            if (q == 0) a.xx_out[h] = xx;
          }
        }
        xx_pending = false;
      }
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
      if (GROUPING) x_h = sh_xx;
      const uint32_t take = min(found, (uint32_t)FV_SP_LIST_CAP);
      // one element per thread (four in flight): save its weight and its count in a slot record,
      // plant the sentinel, take |ds| (the dense term plus count additions of 1/f; a row with
      // xx == 0 has ds == 0)
      // number of the round's first record, for the sentinels (saturated: a step with more records than a
      // sentinel can name is not finished by the launch that reads the numbers)
      const uint32_t record0 = (uint32_t)min((regions ? 0ull : slot_first) + emitted, (uint64_t)FV_SENTINEL_MAX);
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
            slots[emitted + eb + u * T] = rec;
            if (DELTA) a.slot_n2[slot_first + emitted + eb + u * T] = n2e[u];
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
  const float bm = fv_block_max_nonneg(ds_max, wave_max);  // behind its barriers every wave's hits are counted
  if (tid == 0) {
    a.bmax_sparse[blockIdx.x] = bm;
    a.slot_count[blockIdx.x] = emitted;
    a.row_hits[blockIdx.x] = min(sh_hits[0], 3u) | (min(sh_hits[1], 3u) << 2);
  }
}

// CW: words of the block's LDS counter array (two 16-bit counters each while a neuron has fewer than 2^16
// window positions). FV_NB_CNT_WORDS, six blocks per compute unit, covers the 10000 columns per class of the
// headline shape in one pass; FV_NB_CNT_WORDS_WIDE, five blocks per compute unit, is taken where it saves a pass
// (25000 columns per class at V = 50000: two passes instead of three).
template <bool DELTA, int CW>
__global__ __launch_bounds__(FV_SP_THREADS) void fv_sparse_kernel(fv_sparse_args a) {
  fv_sparse_block<DELTA, false, CW>(a);
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
  if (exact) E = max(E, cand); else F = max(F, cand);
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
  const float bm = fv_block_max_nonneg(m, smem4);
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
  nc = fv_block_max_nonneg(nc, smem16);
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
        // a sentinel goes back as it came; the slot launch replaces it
        if (fv_apply_four(v, xq, s, a.update_cut)) a.Wt4[rr * a.ldk4 + q] = v;
        fv_top2_insert(t1[0], t2[0], fv_abs_or_zero(v.x));
        fv_top2_insert(t1[1], t2[1], fv_abs_or_zero(v.y));
        fv_top2_insert(t1[2], t2[2], fv_abs_or_zero(v.z));
        fv_top2_insert(t1[3], t2[3], fv_abs_or_zero(v.w));
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
// sentinel leaves it alone and notes (sentinel, element) in an LDS list; when the block has updated its
// dense elements the list is dealt over its threads, each of which finds the record through the
// sentinel's number, forms ds and writes the element. No other block ever reads or writes that element
// in this launch.
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
#define FV_ONEPASS_HIT_CAP 2048           // sentinels a block notes in LDS; one beyond that is finished on the spot

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
  const uint64_t at = a.slot_region
                          ? (uint64_t)((h << FV_NB_CLASS_SHIFT) | (col & (FV_NB_CLASSES - 1))) * a.slot_region + number
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

// The next minibatch's column indices, by all waves but the first (which polls in the exchange): the
// window's start was fetched behind the loads of W, the token follows here; then, for a minibatch with more
// positions than the launch has sampling threads, the rest.
__device__ __forceinline__ void fv_sample_ahead(const fv_dense_args &a, bool samples0, uint32_t e0, uint32_t er0,
                                                uint64_t start0, uint32_t ahead_entries, uint32_t TS) {
  if (samples0) {
    const uint32_t c = e0 - er0 * a.idx_stride;
    a.idx_ahead[e0] = c < a.w ? fv_column_index(a.corpus[start0 + c], c, a.w, a.V) : -1;
  }
  if (threadIdx.x >= 64)
    for (uint32_t e = e0 + gridDim.x * TS; e < ahead_entries; e += gridDim.x * TS) {
      const uint32_t r = e / a.idx_stride, c = e - r * a.idx_stride;
      a.idx_ahead[e] = c < a.w ? fv_column_index(a.corpus[a.pstart[a.ahead_first + r] + c], c, a.w, a.V) : -1;
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

static_assert(FV_MAX_HID <= 2 * FV_ONEPASS_THREADS, "two neurons per thread cover every row");
static_assert(FV_NB_CLASSES == 4, "a neuron's block maxima and hit counts are read as one 16-byte word each");

template <int U, bool DELTA>
__global__ __launch_bounds__(FV_ONEPASS_THREADS) void fv_dense_onepass_kernel(fv_dense_args a) {
  constexpr uint32_t T = FV_ONEPASS_THREADS;
  constexpr int DEPTH = FV_ONEPASS_DEPTH < U ? FV_ONEPASS_DEPTH : U;
  // xx (ldk floats); the two largest finished sparse elements of every neuron (2 x ldk words); the
  // sentinels met (FV_ONEPASS_HIT_CAP pairs); the threads' two largest weights (4 x active pairs)
  extern __shared__ float4 dyn4[];
  float *xs = (float *)dyn4;
  uint32_t *sp1 = (uint32_t *)(xs + a.ldk);
  uint32_t *sp2 = sp1 + a.ldk;
  uint2 *hit_list = (uint2 *)(sp2 + a.ldk);
  float2 *pairs = (float2 *)(hit_list + FV_ONEPASS_HIT_CAP);
  __shared__ uint32_t red3[T / 64][3];
  __shared__ float smem16[16];
  __shared__ float sh_s;
  __shared__ uint32_t sh_ok, sh_hits;
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
#pragma unroll
  for (int u = 0; u < DEPTH; ++u) {
    const uint32_t row = row0 + u * row_step;
    w[u] = a.Wt4[(row < a.n_rows ? row : row_inside) * a.ldk4 + q];
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
  const bool fast = a.top2_known && F <= max(S, E);  // the same answer in every thread of every block
  const float4 xq = ((const float4 *)xs)[q];

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
    fv_onepass_exchange(a, m, limit, dead, smem16, &sh_s, &sh_ok);
    fv_sample_ahead(a, samples0, e0, er0, start0, ahead_entries, TS);  // while the first wave waits
    __syncthreads();
    ok = sh_ok != 0;
    s = sh_s;
  }

  // The update. A group without a sentinel is stored whole where something changed; in a group with
  // one the other elements are stored one by one and the sentinel is noted for later. The two largest
  // |W| of what the thread leaves behind are kept per neuron.
  float t1[4] = {0.0f, 0.0f, 0.0f, 0.0f}, t2[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#define FV_ONEPASS_ELEMENT(member, lane4)                                                      \
  if (v.member == v.member) {                                                                  \
    if (changed) e[lane4] = v.member;                                                          \
  } else {                                                                                     \
    const uint32_t k = atomicAdd(&sh_hits, 1u);                                                \
    if (k < a.hit_cap)                                                                         \
      hit_list[k] = make_uint2(__float_as_uint(v.member), 4u * p4 + lane4);                    \
    else                                                                                       \
      fv_finish_sparse_element<DELTA>(a, __float_as_uint(v.member), 4u * p4 + lane4, s, ok, xs, sp1, sp2); \
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const uint32_t row = row0 + u * row_step;
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
      fv_top2_insert(t1[0], t2[0], fv_abs_or_zero(v.x));
      fv_top2_insert(t1[1], t2[1], fv_abs_or_zero(v.y));
      fv_top2_insert(t1[2], t2[2], fv_abs_or_zero(v.z));
      fv_top2_insert(t1[3], t2[3], fv_abs_or_zero(v.w));
    }
    if (fast && u + DEPTH < U) {  // the next load takes the place of the one just used
      const uint32_t rown = row0 + (u + DEPTH) * row_step;
      w[u + DEPTH] = a.Wt4[(rown < a.n_rows ? rown : row_inside) * a.ldk4 + q];
    }
  }
#undef FV_ONEPASS_ELEMENT
  if (fast) fv_sample_ahead(a, samples0, e0, er0, start0, ahead_entries, TS);
  if (active) {
#pragma unroll
    for (int e = 0; e < 4; ++e) pairs[(e * rows_per_round + r) * a.ldk4 + q] = make_float2(t1[e], t2[e]);
  }
  __syncthreads();
  // the sentinels the block has met, dealt over its threads
  const uint32_t n_hits = min(sh_hits, a.hit_cap);
  for (uint32_t i = tid; i < n_hits; i += T) {
    const uint2 hit = hit_list[i];
    fv_finish_sparse_element<DELTA>(a, hit.x, hit.y, s, ok, xs, sp1, sp2);
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

template <bool DELTA>
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
#pragma unroll
  for (int u = 0; u < D; ++u) w[u] = a.Wt4[group_of(row0 + u * row_step)];
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
    fv_onepass_exchange(a, m, limit, dead, smem16, &sh_s, &sh_ok);
    fv_sample_ahead(a, samples0, e0, er0, start0, ahead_entries, TS);  // while the first wave waits
    __syncthreads();
    ok = sh_ok != 0;
    s = sh_s;
#pragma unroll
    for (int u = 0; u < D; ++u) w[u] = a.Wt4[group_of(row0 + u * row_step)];  // the stream starts again
  }

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
        fv_top2_insert(t1[0], t2[0], fv_abs_or_zero(v.x));
        fv_top2_insert(t1[1], t2[1], fv_abs_or_zero(v.y));
        fv_top2_insert(t1[2], t2[2], fv_abs_or_zero(v.z));
        fv_top2_insert(t1[3], t2[3], fv_abs_or_zero(v.w));
      }
      w[u] = a.Wt4[group_of(row + D * row_step)];  // the round that takes this one's place
    }
  }
#undef FV_STREAM_ELEMENT
  if (fast) fv_sample_ahead(a, samples0, e0, er0, start0, ahead_entries, TS);
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
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, fv_dense_stream_kernel<false>, FV_ONEPASS_THREADS, smem) !=
          hipSuccess ||
      hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb2, fv_dense_stream_kernel<true>, FV_ONEPASS_THREADS, smem) !=
          hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return nb >= 1 && nb2 >= 1;
}

template <int U, bool DELTA>
static void fv_launch_onepass(const fv_dense_args &d, unsigned blocks, size_t smem, hipStream_t stream) {
  hipLaunchKernelGGL((fv_dense_onepass_kernel<U, DELTA>), dim3(blocks), dim3(FV_ONEPASS_THREADS), smem, stream, d);
}

template <int U>
static int fv_onepass_fits(size_t smem) {
  int nb = 0, nb2 = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, fv_dense_onepass_kernel<U, false>, FV_ONEPASS_THREADS,
                                                   smem) != hipSuccess ||
      hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb2, fv_dense_onepass_kernel<U, true>, FV_ONEPASS_THREADS,
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
      a.slot_region ? (uint64_t)blockIdx.x * a.slot_region
                    : (uint64_t)q * a.slot_stride + (uint64_t)(a.group_base[h] + (DELTA ? a.group_base2[h] : 0u)) * a.w;
  const fv_slot *slots = a.slots + slot_first;
  const float x = a.xx[h];
  const float nc = a.scalars[0];
  const float s = a.prec > nc ? a.eps / a.prec : a.eps / nc;
  for (uint32_t eb = threadIdx.x; eb < count; eb += 4 * 256) {  // four records in flight per thread
    fv_slot sl[4];
    uint32_t n2[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      sl[u] = slots[min(eb + u * 256, count - 1)];
      n2[u] = DELTA ? a.slot_n2[slot_first + min(eb + u * 256, count - 1)] : 0u;
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

// ---- window order ------------------------------------------------------------------------------

__global__ __launch_bounds__(256) void fv_identity_kernel(uint64_t *__restrict__ perm, uint64_t n) {
  for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (uint64_t)gridDim.x * 256) perm[i] = i;
}

// The reshuffle of flyvec/src/model_arrays.cu:451-465 rearranges the current order, cumulatively
// over the epochs; here out[i] = in[sigma(i)] with sigma a keyed bijection computed per index.
__global__ __launch_bounds__(256) void fv_shuffle_kernel(const uint64_t *__restrict__ in, uint64_t *__restrict__ out,
                                                         uint64_t n, fv_feistel f) {
  for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (uint64_t)gridDim.x * 256)
    out[i] = in[fv_permute_index(&f, i, n)];
}

// The sampler's two look-ups (order -> window -> start) folded into one table whenever the order changes.
__global__ __launch_bounds__(256) void fv_order_starts_kernel(const uint64_t *__restrict__ perm,
                                                              const uint64_t *__restrict__ starts,
                                                              uint64_t *__restrict__ pstart, uint64_t n) {
  for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (uint64_t)gridDim.x * 256)
    pstart[i] = starts[perm[i]];
}

static unsigned fv_perm_blocks(uint64_t n) {
  const uint64_t want = (n + 255) / 256;
  return (unsigned)(want < 8192 ? want : 8192);
}

// ---- host side ------------------------------------------------------------------------------

static void fv_trainer_free_delta(fv_trainer *t);

static void fv_trainer_free_corpus(fv_trainer *t) {
  (void)hipFree(t->corpus);
  (void)hipFree(t->starts);
  (void)hipFree(t->perm);
  (void)hipFree(t->perm_alt);
  (void)hipFree(t->pstart);
  (void)hipFree(t->invf);
  t->corpus = nullptr;
  t->starts = t->perm = t->perm_alt = t->pstart = nullptr;
  t->invf = nullptr;
  t->n_tokens = t->n_windows = 0;
  t->have_corpus = false;
  t->ahead_valid = false;
}

// Trainers alive in this process. The single dense launch needs every compute unit for itself: two
// of them in flight at once, from two trainers' streams, could each hold half the machine and wait
// for the other half, so the form is only used while one trainer exists.
static std::atomic<int> fv_trainers_alive{0};

// After a single dense launch has given up: the trainer goes on with two launches per step, and the marks
// the launch left (status word, "dead" flag for the launches behind it) are cleared. Returns the tag.
static int fv_trainer_take_giveup(fv_trainer *t, uint32_t *out_tag) {
  *out_tag = 0;
  if (!t->onepass_status || !*(volatile uint32_t *)t->onepass_status) return FV_OK;
  *out_tag = *(volatile uint32_t *)t->onepass_status;
  *t->onepass_status = 0;
  t->onepass = false;
  t->top2_valid = false;
  t->ahead_valid = false;
  FV_HIP(hipMemsetAsync(t->scalars + 1, 0, sizeof(float), t->stream));
  FV_HIP(hipStreamSynchronize(t->stream));
  return FV_OK;
}

// Waits for the trainer's stream; reports a single dense launch that gave up waiting for its other blocks.
static int fv_trainer_wait(fv_trainer *t) {
  FV_HIP(hipStreamSynchronize(t->stream));
  uint32_t tag = 0;
  FV_TRY(fv_trainer_take_giveup(t, &tag));
  if (tag)
    return fv_fail(FV_ERR_STATE, "a single dense launch gave up waiting for its blocks (not resident together): neither "
                                 "that step nor the steps enqueued behind it have changed the matrix; later steps use "
                                 "two launches");
  return FV_OK;
}

extern "C" int fv_trainer_destroy(fv_trainer *t) {
  if (!t) return FV_OK;
  if (t->stream) (void)hipStreamSynchronize(t->stream);
  fv_trainer_free_corpus(t);
  (void)hipFree(t->Wt);
  (void)hipFree(t->idx);
  (void)hipFree(t->idx_ahead);
  (void)hipFree(t->slots);
  (void)hipFree(t->slots_blocks);
  (void)hipFree(t->slot_count);
  (void)hipFree(t->order);
  (void)hipFree(t->group_base);
  (void)hipFree(t->group_count);
  (void)hipFree(t->bmax);
  (void)hipFree(t->win);
  (void)hipFree(t->win16);
  (void)hipFree(t->won[0]);
  fv_trainer_free_delta(t);
  (void)hipFree(t->sc);
  (void)hipFree(t->xx);
  (void)hipFree(t->scalars);
  (void)hipFree(t->arrive);
  (void)hipFree(t->row_top2);
  (void)hipFree(t->top2_part);
  (void)hipFree(t->row_hits);
  (void)hipFree(t->path_count);
  if (t->onepass_status) (void)hipHostFree(t->onepass_status);
  if (t->stream) (void)hipStreamDestroy(t->stream);
  fv_trainers_alive.fetch_sub(1);
  delete t;
  return FV_OK;
}

static int fv_trainer_alloc(fv_trainer *t) {
  // zeros behind the matrix: what the gather reads for masked positions and in its lanes past K
  const size_t elems = (size_t)fv_matrix_alloc_elems(t->K, t->N);
  FV_REQUIRE(fv_matrix_gather_reach(t->K, t->N) <= elems, FV_ERR_INVALID,
             "a gather of a %u x %llu matrix would read past its allocation", t->K, (unsigned long long)t->N);
  FV_HIP(hipStreamCreate(&t->stream));
  FV_HIP(hipMalloc((void **)&t->Wt, elems * sizeof(float)));
  t->idx_stride = (t->w + 3u) & ~3u;
  const size_t idx_entries = (size_t)t->B * t->idx_stride + FV_IDX_PAD;
  FV_HIP(hipMalloc((void **)&t->idx, idx_entries * sizeof(int32_t)));
  FV_HIP(hipMemsetAsync(t->idx, 0xff, idx_entries * sizeof(int32_t), t->stream));
  if (t->onepass_blocks) {
    FV_HIP(hipMalloc((void **)&t->idx_ahead, idx_entries * sizeof(int32_t)));
    FV_HIP(hipMemsetAsync(t->idx_ahead, 0xff, idx_entries * sizeof(int32_t), t->stream));
  }
  FV_HIP(hipMalloc((void **)&t->win, ((size_t)t->B + 16) * sizeof(int32_t)));  // read in 16-byte pieces
  FV_HIP(hipMalloc((void **)&t->sc, (size_t)t->B * sizeof(float)));
  FV_HIP(hipMalloc((void **)&t->order, (size_t)t->B * sizeof(uint32_t)));
  FV_HIP(hipMalloc((void **)&t->group_base, (size_t)t->K * sizeof(uint32_t)));
  FV_HIP(hipMalloc((void **)&t->group_count, (size_t)t->K * sizeof(uint32_t)));
  FV_HIP(hipMalloc((void **)&t->slots, (size_t)FV_NB_CLASSES * t->B * t->w * sizeof(fv_slot)));
  FV_HIP(hipMalloc((void **)&t->slot_count, (size_t)FV_NB_CLASSES * t->K * sizeof(uint32_t)));
  FV_HIP(hipMalloc((void **)&t->xx, (size_t)t->ldk * sizeof(float)));
  // a neuron's four sparse block maxima are read as one 16-byte word: they start at a multiple of 4
  t->sparse_base = (t->dense_blocks + 3u) & ~3u;
  const size_t n_bmax = (size_t)t->sparse_base + (size_t)FV_NB_CLASSES * t->K;
  FV_HIP(hipMalloc((void **)&t->bmax, n_bmax * sizeof(float)));
  FV_HIP(hipMemsetAsync(t->bmax, 0, n_bmax * sizeof(float), t->stream));
  FV_HIP(hipMalloc((void **)&t->row_hits, (size_t)FV_NB_CLASSES * t->K * sizeof(uint32_t)));
  FV_HIP(hipMemsetAsync(t->row_hits, 0, (size_t)FV_NB_CLASSES * t->K * sizeof(uint32_t), t->stream));
  {
    const size_t shares = t->onepass_blocks > t->update_blocks + FV_NB_CLASSES ? t->onepass_blocks
                                                                               : t->update_blocks + FV_NB_CLASSES;
    const size_t chunks = (shares + FV_MERGE_CHUNK - 1) / FV_MERGE_CHUNK;
    // row_top2, then the staging array of the merge
    const size_t bytes = (1 + chunks) * t->ldk * sizeof(float2);
    FV_HIP(hipMalloc((void **)&t->row_top2, bytes));
    FV_HIP(hipMemsetAsync(t->row_top2, 0, bytes, t->stream));
    t->top2_stage = t->row_top2 + t->ldk;
  }
  FV_HIP(hipMalloc((void **)&t->path_count, 2 * sizeof(uint32_t)));
  FV_HIP(hipMemsetAsync(t->path_count, 0, 2 * sizeof(uint32_t), t->stream));
  {
    // shares per row: the single launch's blocks, or the update launch's blocks and the slot launch's four
    const size_t per_row = t->onepass_blocks > t->update_blocks + FV_NB_CLASSES ? t->onepass_blocks
                                                                                : t->update_blocks + FV_NB_CLASSES;
    FV_HIP(hipMalloc((void **)&t->top2_part, (size_t)t->ldk * per_row * sizeof(float2)));
    FV_HIP(hipMemsetAsync(t->top2_part, 0, (size_t)t->ldk * per_row * sizeof(float2), t->stream));
  }
  FV_HIP(hipMemsetAsync(t->win, 0, ((size_t)t->B + 16) * sizeof(int32_t), t->stream));
  FV_HIP(hipMalloc((void **)&t->win16, ((size_t)t->B + 64) * sizeof(uint16_t)));  // read in 16-byte pieces
  FV_HIP(hipMemsetAsync(t->win16, 0, ((size_t)t->B + 64) * sizeof(uint16_t), t->stream));
  if (t->B <= 64 * FV_SP_THREADS) {  // steps of such a trainer can be grouped inside the sparse launch
    t->won_words = 2 * ((t->B + 63) / 64);
    const size_t row_words = (size_t)t->K * t->won_words;
    FV_HIP(hipMalloc((void **)&t->won[0], 2 * row_words * sizeof(uint32_t)));
    t->won[1] = t->won[0] + row_words;
    FV_HIP(hipMemsetAsync(t->won[0], 0, 2 * row_words * sizeof(uint32_t), t->stream));
    // A block of that launch writes no more records than its class has columns, nor more than the step has
    // window positions: with that much room of its own per block, no block has to count the windows of the
    // neurons before it to find its place. Left out where the regions would take more than a gigabyte.
    const uint64_t class_cols = (t->N + FV_NB_CLASSES - 1) / FV_NB_CLASSES, positions = (uint64_t)t->B * t->w;
    const uint64_t region = class_cols < positions ? class_cols : positions;
    if (region * t->K * FV_NB_CLASSES * sizeof(fv_slot) <= FV_SLOT_REGIONS_MAX_BYTES && region + 1 < FV_SENTINEL_MAX) {
      t->slot_region = (uint32_t)region;
      FV_HIP(hipMalloc((void **)&t->slots_blocks, region * t->K * FV_NB_CLASSES * sizeof(fv_slot)));
    }
  }
  FV_HIP(hipMalloc((void **)&t->scalars, 16 * sizeof(float)));
  FV_HIP(hipMemsetAsync(t->Wt, 0, elems * sizeof(float), t->stream));
  FV_HIP(hipMemsetAsync(t->xx, 0, (size_t)t->ldk * sizeof(float), t->stream));
  FV_HIP(hipMemsetAsync(t->scalars, 0, 16 * sizeof(float), t->stream));
  if (t->onepass_blocks) {
    FV_HIP(hipMalloc((void **)&t->arrive, ((size_t)t->onepass_blocks + 1) * sizeof(unsigned long long)));
    FV_HIP(hipMemsetAsync(t->arrive, 0, ((size_t)t->onepass_blocks + 1) * sizeof(unsigned long long), t->stream));
    FV_HIP(hipHostMalloc((void **)&t->onepass_status, sizeof(uint32_t), hipHostMallocDefault));
    *t->onepass_status = 0;
  }
  FV_HIP(hipStreamSynchronize(t->stream));
  return FV_OK;
}

// One launch for both dense passes when every compute unit can hold a block whose threads keep the
// whole matrix in registers between them; otherwise (onepass_unroll = 0) the two launches.
// Dynamic LDS of that launch: xx and two words per neuron, the list of sentinels, four pairs per thread.
static size_t fv_onepass_smem(const fv_trainer *t) {
  return (size_t)t->ldk * 3 * sizeof(float) + (size_t)FV_ONEPASS_HIT_CAP * sizeof(uint2) +
         (size_t)FV_ONEPASS_THREADS * 4 * sizeof(float2);
}

static size_t fv_stream_smem(const fv_trainer *t) {
  return (size_t)t->ldk * 3 * sizeof(float) + (size_t)FV_STREAM_HIT_CAP * sizeof(uint2) +
         (size_t)FV_ONEPASS_THREADS * 4 * sizeof(float2);
}

static void fv_choose_onepass(fv_trainer *t, uint64_t cu) {
  t->onepass_blocks = t->onepass_unroll = t->onepass_active = 0;
  t->stream_ok = t->onepass_stream = t->onepass = false;
  t->onepass_spin_limit = FV_ONEPASS_SPIN_LIMIT;
  const uint32_t ldk4 = t->ldk / 4;
  if (ldk4 > FV_ONEPASS_THREADS) return;
  // a block takes whole rows: rows_per_round of them at a time, one 16-byte group per thread
  const uint32_t rows_per_round = FV_ONEPASS_THREADS / ldk4;
  uint64_t blocks = (t->N + rows_per_round - 1) / rows_per_round;
  if (blocks > cu * FV_ONEPASS_BLOCKS_PER_CU) blocks = cu * FV_ONEPASS_BLOCKS_PER_CU;
  const uint64_t need = (t->N + blocks * rows_per_round - 1) / (blocks * rows_per_round);
  {
    // the streaming form: its sentinel list takes more LDS than a launch may have without asking
    const size_t smem = fv_stream_smem(t);
    if (hipFuncSetAttribute((const void *)fv_dense_stream_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)smem) == hipSuccess &&
        hipFuncSetAttribute((const void *)fv_dense_stream_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)smem) == hipSuccess)
      t->stream_ok = fv_stream_fits(smem) != 0;
    else
      (void)hipGetLastError();
  }
  unsigned unroll = 0;
  if (need <= FV_ONEPASS_MAX_UNROLL) {
    unroll = need <= 8 ? 8 : 16;
    const size_t smem = fv_onepass_smem(t);
    if (!(unroll == 8 ? fv_onepass_fits<8>(smem) : fv_onepass_fits<16>(smem))) unroll = 0;
  }
  if (!unroll && !t->stream_ok) return;
  t->onepass_blocks = (unsigned)blocks;
  t->onepass_unroll = unroll;
  t->onepass_active = rows_per_round * ldk4;
  t->onepass = true;
  t->onepass_stream = unroll == 0;
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
  FV_REQUIRE(cfg->prune_duplicates <= 1, FV_ERR_INVALID, "prune_duplicates must be 0 or 1");
  FV_REQUIRE(fabsf(cfg->lmid) <= 1.0e6f && fabsf(cfg->lbase) <= 1.0e6f, FV_ERR_INVALID,
             "Lmid = %g, Lbase = %g: out of range (1 and 1 are the reference's values)", (double)cfg->lmid,
             (double)cfg->lbase);
  FV_REQUIRE(cfg->delta == cfg->delta && fabsf(cfg->delta) <= 1.0e6f, FV_ERR_INVALID, "delta = %g is out of range",
             (double)cfg->delta);
  // the slot regions of a step with delta != 0 hold twice as many records
  FV_REQUIRE(cfg->delta == 0.0f || (uint64_t)cfg->batch * cfg->window < (1ull << 30), FV_ERR_INVALID,
             "batch x window = %llu is out of range for delta != 0", (unsigned long long)cfg->batch * cfg->window);
  const uint32_t ldk = fv_ldk(cfg->hid);
  const uint64_t N = 2 * cfg->vocab;
  FV_REQUIRE(N * ldk < 0xffffffffull - (1u << 24), FV_ERR_INVALID,
             "synapse matrix of %llu x %u floats exceeds 2^32 elements", (unsigned long long)N, ldk);
  FV_REQUIRE((uint64_t)cfg->batch * cfg->window < (1ull << 31), FV_ERR_INVALID,
             "batch x window = %llu is out of range", (unsigned long long)cfg->batch * cfg->window);
  fv_trainer *t = new fv_trainer();
  memset(t, 0, sizeof *t);
  fv_trainers_alive.fetch_add(1);
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
    if (want == 0) want = 1;
    const uint64_t cu = (uint64_t)(cus > 0 ? cus : 256);
    t->dense_blocks = (unsigned)(want < cu * FV_ABSMAX_BLOCKS_PER_CU ? want : cu * FV_ABSMAX_BLOCKS_PER_CU);
    {
      // the update launch takes whole rows: 256-thread blocks, 512 when a row has more groups than that
      const uint32_t ldk4 = t->ldk / 4;
      t->update_threads = ldk4 <= 256 ? 256 : 512;
      const uint64_t rows_per_round = t->update_threads / ldk4;
      const uint64_t want_rows = (t->N + rows_per_round - 1) / rows_per_round;
      const uint64_t cap = cu * FV_UPDATE_BLOCKS_PER_CU * 256 / t->update_threads;
      t->update_blocks = (unsigned)(want_rows < cap ? want_rows : cap);
    }
    fv_choose_onepass(t, cu);
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
    if (e == hipSuccess) e = hipMalloc((void **)&t->pstart, nwin * sizeof(uint64_t));
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
      hipLaunchKernelGGL(fv_identity_kernel, dim3(fv_perm_blocks(nwin)), dim3(256), 0, t->stream, t->perm, nwin);
      hipLaunchKernelGGL(fv_order_starts_kernel, dim3(fv_perm_blocks(nwin)), dim3(256), 0, t->stream, t->perm,
                         t->starts, t->pstart, nwin);
      e = hipStreamSynchronize(t->stream);
      if (e != hipSuccess) rc = fv_fail(FV_ERR_HIP, "permutation fill failed: %s", hipGetErrorString(e));
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

// The same with the window table given instead of built: what the reference's driver hands over
// (flyvec/src/model_arrays.cu:358 set_up_INPUT_pointer takes the corpus and the table that
// compute_offset_phrases wrote; :396 compute_inverse_word_frequency the corpus length).
extern "C" int fv_trainer_set_corpus_starts(fv_trainer *t, const int32_t *tokens, uint64_t n_tokens,
                                            const uint64_t *starts, uint64_t n_windows) {
  FV_REQUIRE(t, FV_ERR_INVALID, "null trainer");
  FV_REQUIRE(tokens && n_tokens > 0, FV_ERR_INVALID, "empty corpus");
  FV_REQUIRE(starts || n_windows == 0, FV_ERR_INVALID, "null window table");
  for (uint64_t i = 0; i < n_windows; ++i)
    FV_REQUIRE(starts[i] <= n_tokens && t->w <= n_tokens - starts[i], FV_ERR_DATA,
               "window %llu starts at token %llu: it does not fit the corpus of %llu", (unsigned long long)i,
               (unsigned long long)starts[i], (unsigned long long)n_tokens);
  FV_HIP(hipStreamSynchronize(t->stream));
  fv_trainer_free_corpus(t);
  int rc = FV_OK;
  hipError_t e = hipMalloc((void **)&t->corpus, n_tokens * sizeof(int32_t));
  if (e == hipSuccess) e = hipMalloc((void **)&t->invf, t->V * sizeof(float));
  if (e == hipSuccess)
    e = hipMemcpyAsync(t->corpus, tokens, n_tokens * sizeof(int32_t), hipMemcpyHostToDevice, t->stream);
  if (e != hipSuccess) rc = fv_fail(FV_ERR_HIP, "corpus upload failed: %s", hipGetErrorString(e));
  int32_t lo = 0, hi = 0;
  if (rc == FV_OK) rc = fv_dev_inverse_frequency(t->corpus, n_tokens, t->V, t->invf, &lo, &hi, t->stream);
  if (rc == FV_OK && (lo < -1 || (hi >= 0 && (uint64_t)hi >= t->V)))
    rc = fv_fail(FV_ERR_DATA, "token ids span [%d, %d]; allowed are -1 (masked) and 0..%llu", lo, hi,
                 (unsigned long long)(t->V - 1));
  if (rc == FV_OK && n_windows) {
    e = hipMalloc((void **)&t->starts, n_windows * sizeof(uint64_t));
    if (e == hipSuccess) e = hipMalloc((void **)&t->perm, n_windows * sizeof(uint64_t));
    if (e == hipSuccess) e = hipMalloc((void **)&t->pstart, n_windows * sizeof(uint64_t));
    if (e == hipSuccess)
      e = hipMemcpyAsync(t->starts, starts, n_windows * sizeof(uint64_t), hipMemcpyHostToDevice, t->stream);
    if (e != hipSuccess) rc = fv_fail(FV_ERR_HIP, "window table upload failed: %s", hipGetErrorString(e));
    if (rc == FV_OK) {
      hipLaunchKernelGGL(fv_identity_kernel, dim3(fv_perm_blocks(n_windows)), dim3(256), 0, t->stream, t->perm, n_windows);
      hipLaunchKernelGGL(fv_order_starts_kernel, dim3(fv_perm_blocks(n_windows)), dim3(256), 0, t->stream, t->perm,
                         t->starts, t->pstart, n_windows);
      e = hipStreamSynchronize(t->stream);
      if (e != hipSuccess) rc = fv_fail(FV_ERR_HIP, "permutation fill failed: %s", hipGetErrorString(e));
    }
  }
  if (rc != FV_OK) {
    fv_trainer_free_corpus(t);
    return rc;
  }
  t->n_tokens = n_tokens;
  t->n_windows = n_windows;
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
  t->top2_valid = false;  // the first single dense launch on the new matrix makes the pass for max|ds|
  return FV_OK;
}

extern "C" int fv_trainer_get_weights(fv_trainer *t, float *out_W) {
  FV_REQUIRE(t && out_W, FV_ERR_INVALID, "null argument");
  FV_REQUIRE(t->have_weights, FV_ERR_STATE, "no weights set");
  FV_TRY(fv_trainer_wait(t));
  return fv_download_weights(t->Wt, out_W, t->K, t->N, t->ldk, t->stream);
}

extern "C" int fv_trainer_shuffle(fv_trainer *t, uint64_t seed) {
  FV_REQUIRE(t, FV_ERR_INVALID, "null trainer");
  FV_REQUIRE(t->have_corpus, FV_ERR_STATE, "no corpus set");
  const uint64_t n = t->n_windows;
  if (n == 0) return FV_OK;
  if (!t->perm_alt) FV_HIP(hipMalloc((void **)&t->perm_alt, n * sizeof(uint64_t)));
  // every call draws a different bijection, also under one seed
  const fv_feistel f = fv_feistel_make(n, seed ^ (0xD1B54A32D192ED03ull * (t->shuffle_calls + 1)));
  hipLaunchKernelGGL(fv_shuffle_kernel, dim3(fv_perm_blocks(n)), dim3(256), 0, t->stream, t->perm, t->perm_alt, n, f);
  FV_HIP(hipGetLastError());
  std::swap(t->perm, t->perm_alt);
  t->ahead_valid = false;  // sampled in the old order
  hipLaunchKernelGGL(fv_order_starts_kernel, dim3(fv_perm_blocks(n)), dim3(256), 0, t->stream, t->perm, t->starts,
                     t->pstart, n);
  FV_HIP(hipGetLastError());
  t->shuffle_calls++;
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
  t->ahead_valid = false;  // sampled in the old order
  hipLaunchKernelGGL(fv_order_starts_kernel, dim3(fv_perm_blocks(n)), dim3(256), 0, t->stream, t->perm, t->starts,
                     t->pstart, n);
  FV_HIP(hipGetLastError());
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
static void fv_launch_gather(const fv_gather_args &a, bool with_second, bool weighted, hipStream_t stream) {
  const uint32_t waves = (a.n + FV_GATHER_WINDOWS - 1) / FV_GATHER_WINDOWS;
  const dim3 grid((waves + 3) / 4 + a.merge_rows), block(256);
  if (weighted) {
    if (with_second)
      hipLaunchKernelGGL((fv_gather_winner_kernel<NV, true, true>), grid, block, 0, stream, a);
    else
      hipLaunchKernelGGL((fv_gather_winner_kernel<NV, false, true>), grid, block, 0, stream, a);
  } else {
    if (with_second)
      hipLaunchKernelGGL((fv_gather_winner_kernel<NV, true, false>), grid, block, 0, stream, a);
    else
      hipLaunchKernelGGL((fv_gather_winner_kernel<NV, false, false>), grid, block, 0, stream, a);
  }
}

// Enqueues the kernels of one step (those whose bit is set in `which`); ev (nullable) receives
// FV_TRAIN_KERNELS + 1 events recorded around them.
// Buffers of the anti-Hebbian form, on first use.
static void fv_trainer_free_delta(fv_trainer *t) {
  (void)hipFree(t->win2);
  (void)hipFree(t->win2_16);
  (void)hipFree(t->sc2);
  (void)hipFree(t->order2);
  (void)hipFree(t->group_base2);
  (void)hipFree(t->group_count2);
  (void)hipFree(t->slots2);
  (void)hipFree(t->slot_n2);
  t->win2 = nullptr;
  t->win2_16 = nullptr;
  t->sc2 = nullptr;
  t->order2 = t->group_base2 = t->group_count2 = t->slot_n2 = nullptr;
  t->slots2 = nullptr;
}

static int fv_trainer_alloc_delta(fv_trainer *t) {
  if (t->slot_n2) return FV_OK;  // the last one allocated: all are there
  fv_trainer_free_delta(t);      // what an earlier, failed attempt left
  const size_t B = t->B, bw = (size_t)t->B * t->w;
  FV_HIP(hipMalloc((void **)&t->win2, B * sizeof(int32_t)));
  FV_HIP(hipMalloc((void **)&t->win2_16, (B + 64) * sizeof(uint16_t)));
  FV_HIP(hipMemsetAsync(t->win2_16, 0, (B + 64) * sizeof(uint16_t), t->stream));
  FV_HIP(hipMalloc((void **)&t->sc2, B * sizeof(float)));
  FV_HIP(hipMalloc((void **)&t->order2, B * sizeof(uint32_t)));
  FV_HIP(hipMalloc((void **)&t->group_base2, (size_t)t->K * sizeof(uint32_t)));
  FV_HIP(hipMalloc((void **)&t->group_count2, (size_t)t->K * sizeof(uint32_t)));
  FV_HIP(hipMalloc((void **)&t->slots2, 2 * FV_NB_CLASSES * bw * sizeof(fv_slot)));
  FV_HIP(hipMalloc((void **)&t->slot_n2, 2 * FV_NB_CLASSES * bw * sizeof(uint32_t)));
  return FV_OK;
}

// n_fresh < n: only the first n_fresh windows are sampled (from `first` on), the rows behind them are what
// the index buffer of the previous step holds.
static int fv_enqueue_step(fv_trainer *t, uint64_t first, uint32_t n, float eps, float delta, hipEvent_t *ev,
                           unsigned which = 0x3f, bool repeated = false, uint32_t n_fresh = 0xffffffffu) {
  const bool anti = delta != 0.0f;  // the second neuron of every window takes part (flyvec/src/cuda_funcs.cu:726-734)
  if (anti) FV_TRY(fv_trainer_alloc_delta(t));
  const bool whole = which == 0x3f;
  // records the slot regions of this step hold; the single dense launch finds a record through the number in
  // its sentinel, so it is only taken when every record number fits one
  uint64_t n_slots = (uint64_t)FV_NB_CLASSES * t->B * t->w * (anti ? 2 : 1);
  // the rows' two largest weights are in hand if the last write of the matrix was a single dense launch
  const bool top2_known = whole ? t->top2_valid : t->last_top2_known;
  if (whole) t->last_top2_known = top2_known;
  fv_gather_args g;
  const uint32_t merge_groups = (t->K + FV_MERGE_NEURONS - 1) / FV_MERGE_NEURONS;
  g.merge_rows = (top2_known && !t->top2_merged && (whole || (which & 1u))) ? merge_groups : 0u;  // one chunk
  g.merge.part = t->top2_part;
  g.merge.stride = t->ldk;
  g.merge.n_part = t->top2_n_part;  // the shares the last dense launches left
  g.merge.K = t->K;
  g.merge.row_top2 = t->row_top2;
  g.merge.stage = t->top2_stage;
  g.Wt = t->Wt;
  g.corpus = t->corpus;
  g.pstart = t->pstart;
  g.invf = t->invf;
  g.idx = t->idx;
  g.stride = t->idx_stride;
  g.win = t->win;
  g.win16 = t->win16;
  g.sc = t->sc;
  g.win2 = t->win2;
  g.win2_16 = t->win2_16;
  g.sc2 = t->sc2;
  g.first = first;
  g.n = n;
  g.n_fresh = n_fresh < n ? n_fresh : n;
  g.K = t->K;
  g.ldk = t->ldk;
  g.w = t->w;
  g.V = (uint32_t)t->V;
  g.tie_rule = t->cfg.tie_rule;
  g.prune = t->cfg.prune_duplicates;
  g.lmid = t->cfg.lmid;
  g.lbase = t->cfg.lbase;
  const bool weighted = t->cfg.lmid != 1.0f || t->cfg.lbase != 1.0f;
  // A step of a trainer with up to 64 windows per thread of a class block, without the anti-Hebbian
  // term, has no grouping launch: the winner kernel marks every window in its winner's bit row, and
  // the sparse launch's blocks group for themselves from those rows. A whole step takes the pair of
  // buffers the last such step's sparse launch has cleared; a launch on its own (measurement) stays
  // on the last step's pair, cleared here first unless it repeats the launch before it.
  const bool grouping_in_sparse =
      which == 0x3f ? !anti && t->won[0] && !t->separate_grouping : t->last_grouped_in_sparse;
  if (which == 0x3f) t->last_grouped_in_sparse = grouping_in_sparse;
  // the blocks of a sparse launch that groups for itself write their records to regions of their own, where
  // the trainer has them, and a sentinel names a record inside its block's region
  const uint32_t slot_region = grouping_in_sparse && !t->no_block_regions ? t->slot_region : 0u;
  if (slot_region) n_slots = slot_region;
  const bool onepass = t->onepass && fv_trainers_alive.load() == 1 && n_slots + 1 < FV_SENTINEL_MAX;
  g.won = nullptr;
  g.won_words = t->won_words;
  if (grouping_in_sparse) {
    if (which == 0x3f) {
      t->won_parity ^= 1u;
    } else if ((which & 1u) && !repeated) {
      FV_HIP(hipMemsetAsync(t->won[t->won_parity], 0, (size_t)t->K * t->won_words * sizeof(uint32_t), t->stream));
    }
    g.won = t->won[t->won_parity];
  }
  // a whole step whose windows the previous one has sampled ahead takes that buffer
  g.sampled = 0;
  if (whole) {
    if (t->ahead_valid && t->ahead_first == first && t->ahead_n == n && n_fresh >= n) {
      std::swap(t->idx, t->idx_ahead);
      g.idx = t->idx;
      g.sampled = 1;
    }
    t->ahead_valid = false;
  }
  if (ev) FV_HIP(hipEventRecord(ev[0], t->stream));
  if (which & 1u) switch ((t->K + 63) / 64) {
#define FV_CASE(NV) case NV: fv_launch_gather<NV>(g, anti, weighted, t->stream); break;
    FV_CASE(1) FV_CASE(2) FV_CASE(3) FV_CASE(4) FV_CASE(5) FV_CASE(6) FV_CASE(7) FV_CASE(8)
    FV_CASE(9) FV_CASE(10) FV_CASE(11) FV_CASE(12) FV_CASE(13) FV_CASE(14) FV_CASE(15) FV_CASE(16)
    FV_CASE(17) FV_CASE(18) FV_CASE(19) FV_CASE(20) FV_CASE(21) FV_CASE(22) FV_CASE(23) FV_CASE(24)
    FV_CASE(25) FV_CASE(26) FV_CASE(27) FV_CASE(28) FV_CASE(29) FV_CASE(30) FV_CASE(31) FV_CASE(32)
#undef FV_CASE
    default:
      return fv_fail(FV_ERR_INVALID, "hid = %u not supported", t->K);
  }
  if (ev) FV_HIP(hipEventRecord(ev[1], t->stream));
  fv_group_args gr;
  gr.win = t->win16;
  gr.sc = t->sc;
  gr.order = t->order;
  gr.group_base = t->group_base;
  gr.group_count = t->group_count;
  gr.xx = t->xx;
  gr.n = n;
  gr.scale = 1.0f;
  gr.accumulate = 0;
  // a thread's run of the winner array should fit its 64-bit match mask
  const unsigned gr_threads = n <= 16384 ? 256 : FV_NB_MAX_THREADS;
  // with delta != 0 a second launch groups the windows by their second neuron and adds
  // -delta * (their scaled activations) to xx
  for (int l = 0; l < (anti ? 2 : 1); ++l) {
    if (l == 1) {
      gr.win = t->win2_16;
      gr.sc = t->sc2;
      gr.order = t->order2;
      gr.group_base = t->group_base2;
      gr.group_count = t->group_count2;
      gr.scale = -delta;
      gr.accumulate = 1;
    }
    if ((which & 2u) && !grouping_in_sparse) {
      if (n <= 64 * gr_threads && n < 65536)
        hipLaunchKernelGGL(fv_group_kernel<true>, dim3(t->K), dim3(gr_threads), 0, t->stream, gr);
      else
        hipLaunchKernelGGL(fv_group_kernel<false>, dim3(t->K), dim3(gr_threads), 0, t->stream, gr);
    }
  }
  if (ev) FV_HIP(hipEventRecord(ev[2], t->stream));
  fv_sparse_args sp;
  sp.order = t->order;
  sp.group_base = t->group_base;
  sp.group_count = t->group_count;
  sp.idx = t->idx;
  sp.Wt = t->Wt;
  sp.slots = anti ? t->slots2 : slot_region ? t->slots_blocks : t->slots;
  sp.slot_region = slot_region;
  sp.slot_stride = (uint64_t)t->B * t->w * (anti ? 2 : 1);
  sp.order2 = t->order2;
  sp.group_base2 = t->group_base2;
  sp.group_count2 = t->group_count2;
  sp.slot_n2 = t->slot_n2;
  sp.delta = delta;
  sp.lmid = t->cfg.lmid;
  sp.lbase = t->cfg.lbase;
  sp.xx = t->xx;
  sp.invf = t->invf;
  sp.bmax_sparse = t->bmax + t->sparse_base;
  sp.row_top2 = t->row_top2;
  sp.row_hits = t->row_hits;
  sp.top2_known = top2_known ? 1u : 0u;
  sp.slot_count = t->slot_count;
  sp.pad_row = t->B;
  sp.stride = t->idx_stride;
  sp.ldk = t->ldk;
  sp.w = t->w;
  sp.V = (uint32_t)t->V;
  sp.won = t->won[t->won_parity];
  sp.win = t->win16;
  sp.won_words = t->won_words;
  sp.won_clear = t->won[t->won_parity ^ 1u];
  sp.sc = t->sc;
  sp.n = n;
  sp.order_out = t->order;
  sp.group_base_out = t->group_base;
  sp.group_count_out = t->group_count;
  sp.xx_out = t->xx;
  if (which & 4u) {
    const dim3 sp_grid(t->K * FV_NB_CLASSES), sp_block(FV_SP_THREADS);
    // the wider counter array where it saves a pass over the neuron's windows
    const uint32_t class_cols = (uint32_t)((t->N + FV_NB_CLASSES - 1) / FV_NB_CLASSES);
    // (counted for 16-bit counters, two to a word: what all but the heaviest neurons of a large minibatch use)
    const auto passes = [&](uint32_t words) { return (class_cols + 2 * words - 1) / (2 * words); };
    const bool wide = passes(FV_NB_CNT_WORDS_WIDE) < passes(FV_NB_CNT_WORDS);
#define FV_LAUNCH_SPARSE(CW, GROUPING_KERNEL)                                                       \
  if (anti)                                                                                         \
    hipLaunchKernelGGL((fv_sparse_kernel<true, CW>), sp_grid, sp_block, 0, t->stream, sp);          \
  else if (grouping_in_sparse)                                                                      \
    hipLaunchKernelGGL(GROUPING_KERNEL, sp_grid, sp_block, 0, t->stream, sp);                       \
  else                                                                                              \
    hipLaunchKernelGGL((fv_sparse_kernel<false, CW>), sp_grid, sp_block, 0, t->stream, sp);
    if (wide) {
      FV_LAUNCH_SPARSE(FV_NB_CNT_WORDS_WIDE, fv_sparse_grouping_wide_kernel)
    } else {
      FV_LAUNCH_SPARSE(FV_NB_CNT_WORDS, fv_sparse_grouping_kernel)
    }
#undef FV_LAUNCH_SPARSE
  }
  if (ev) FV_HIP(hipEventRecord(ev[3], t->stream));
  fv_dense_args d;
  d.Wt4 = (float4 *)t->Wt;
  d.xx = t->xx;
  d.invf = t->invf;
  d.slots = anti ? t->slots2 : slot_region ? t->slots_blocks : t->slots;
  d.slot_region = slot_region;
  {
    const uint32_t holds = t->onepass_stream ? FV_STREAM_HIT_CAP : FV_ONEPASS_HIT_CAP;
    d.hit_cap = t->hit_cap_limit && t->hit_cap_limit < holds ? t->hit_cap_limit : holds;
  }
  d.slot_count = t->slot_count;
  d.group_base = t->group_base;
  d.group_base2 = t->group_base2;
  d.slot_n2 = t->slot_n2;
  d.delta = delta;
  d.w = t->w;
  d.arrive = nullptr;
  d.status = nullptr;
  d.epoch = d.spin_limit = d.step_tag = 0;
  d.lmid = t->cfg.lmid;
  d.lbase = t->cfg.lbase;
  d.corpus = t->corpus;
  d.pstart = t->pstart;
  d.idx_ahead = nullptr;
  d.idx_stride = t->idx_stride;
  d.ahead_first = 0;
  d.ahead_n = 0;
  d.slot_stride = (uint64_t)t->B * t->w * (anti ? 2 : 1);
  d.bmax = t->bmax;
  d.scalars = t->scalars;
  d.total4 = t->total4;
  d.ldk4 = t->ldk / 4;
  d.ldk = t->ldk;
  d.V = (uint32_t)t->V;
  d.K = t->K;
  d.n_bmax = t->sparse_base + t->K * FV_NB_CLASSES;
  d.dense_blocks = t->dense_blocks;
  d.sparse_base = t->sparse_base;
  d.n_rows = (uint32_t)t->N;
  d.active = t->onepass_active;
  d.n_slots = (uint32_t)n_slots;
  d.row_top2 = t->row_top2;
  d.row_hits = t->row_hits;
  d.top2_known = top2_known ? 1u : 0u;
  d.top2_part = t->top2_part;
  d.part_base = onepass ? 0u : t->update_blocks;
  d.path_count = t->path_count;
  d.eps = eps;
  d.prec = t->cfg.prec;
  d.update_cut = t->update_cut;
  const size_t smem = (size_t)t->ldk * sizeof(float);
  if (onepass) {
    // both dense passes in the launch that takes the place of the first one
    if (which & 8u) {
      if (++t->onepass_epoch == 0) t->onepass_epoch = 1;
      d.arrive = t->arrive;
      d.status = t->onepass_status;
      d.epoch = t->onepass_epoch;
      d.spin_limit = t->onepass_spin_limit;
      d.step_tag = t->step_tag ? t->step_tag : 0xffffffffu;
      // the windows that follow this step's, a full batch or what is left of the order
      const uint64_t next_first = first + n;
      if (whole && next_first < t->n_windows && !t->cfg.prune_duplicates) {  // the ahead sampler does not prune
        d.ahead_first = next_first;
        d.ahead_n = (uint32_t)(t->n_windows - next_first < t->B ? t->n_windows - next_first : t->B);
        d.idx_ahead = t->idx_ahead;
        t->ahead_valid = true;
        t->ahead_first = next_first;
        t->ahead_n = d.ahead_n;
      }
      const size_t smem1 = fv_onepass_smem(t);
#define FV_CASE(U)                                                                     \
  if (anti) fv_launch_onepass<U, true>(d, t->onepass_blocks, smem1, t->stream);        \
  else fv_launch_onepass<U, false>(d, t->onepass_blocks, smem1, t->stream);
      if (t->onepass_stream) {
        const dim3 grid(t->onepass_blocks), block(FV_ONEPASS_THREADS);
        if (anti)
          hipLaunchKernelGGL(fv_dense_stream_kernel<true>, grid, block, fv_stream_smem(t), t->stream, d);
        else
          hipLaunchKernelGGL(fv_dense_stream_kernel<false>, grid, block, fv_stream_smem(t), t->stream, d);
      } else if (t->onepass_unroll == 8) { FV_CASE(8) } else { FV_CASE(16) }
#undef FV_CASE
      t->top2_valid = true;  // this launch leaves the shares of the matrix it writes
      t->top2_n_part = t->onepass_blocks;
      t->top2_merged = false;  // the next winner kernel's first blocks merge them
      static_assert(FV_ONEPASS_BLOCKS_PER_CU == 1, "a single dense launch leaves no more shares than one chunk holds");
    }
    if (ev) FV_HIP(hipEventRecord(ev[4], t->stream));
  } else {
    if (which & 8u) {
      // one block settles whether max|ds| is known from the rows' largest weights; the pass ends at once if so
      hipLaunchKernelGGL(fv_decide_kernel, dim3(1), dim3(1024), 0, t->stream, d);
      hipLaunchKernelGGL(fv_absmax_kernel, dim3(t->dense_blocks), dim3(256), smem, t->stream, d);
    }
    if (ev) FV_HIP(hipEventRecord(ev[4], t->stream));
    if (which & 16u) {
      const size_t smem_u = smem + (size_t)t->update_threads * 4 * sizeof(float2);
      if (t->update_threads == 256)
        hipLaunchKernelGGL(fv_update_kernel<256>, dim3(t->update_blocks), dim3(256), smem_u, t->stream, d);
      else
        hipLaunchKernelGGL(fv_update_kernel<512>, dim3(t->update_blocks), dim3(512), smem_u, t->stream, d);
      // with the slot launch behind it, the two leave the shares of the matrix they write
      t->top2_valid = whole;
      t->top2_n_part = t->update_blocks + FV_NB_CLASSES;
    }
  }
  if (ev) FV_HIP(hipEventRecord(ev[5], t->stream));
  if ((which & 32u) && !onepass) {  // the single launch has finished the sparse elements as well
    if (anti)
      hipLaunchKernelGGL(fv_slot_update_kernel<true>, dim3(t->K * FV_NB_CLASSES), dim3(256), 0, t->stream, d);
    else
      hipLaunchKernelGGL(fv_slot_update_kernel<false>, dim3(t->K * FV_NB_CLASSES), dim3(256), 0, t->stream, d);
    if (whole) {
      // the shares the update and slot launches have left, merged here: a share per block of a large grid is
      // more than the next winner kernel's first blocks should be kept busy with
      fv_merge_args m = g.merge;
      m.n_part = t->top2_n_part;
      const uint32_t chunks = (m.n_part + FV_MERGE_CHUNK - 1) / FV_MERGE_CHUNK;
      hipLaunchKernelGGL(fv_merge_shares_kernel, dim3(merge_groups * chunks), dim3(256), 0, t->stream, m);
      if (chunks > 1)
        hipLaunchKernelGGL(fv_merge_stage_kernel, dim3((t->K + 255) / 256), dim3(256), 0, t->stream, m);
      t->top2_merged = true;
    }
  }
  if (ev) FV_HIP(hipEventRecord(ev[6], t->stream));
  FV_HIP(hipGetLastError());
  t->last_n = n;
  t->last_first = first;
  t->last_eps = eps;
  t->last_delta = delta;
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
  return fv_enqueue_step(t, first_window, n_windows, eps, 0.0f, nullptr);
}

extern "C" int fv_trainer_step_delta(fv_trainer *t, uint64_t first_window, uint32_t n_windows, float eps,
                                     float delta) {
  FV_TRY(fv_check_step(t, first_window, n_windows));
  return fv_enqueue_step(t, first_window, n_windows, eps, delta, nullptr);
}

extern "C" int fv_trainer_epoch_delta(fv_trainer *t, uint64_t epoch_id, uint64_t n_epochs, float *out_delta) {
  FV_REQUIRE(t && out_delta, FV_ERR_INVALID, "null argument");
  // flyvec/src/cuda_funcs.cu:1230: double arithmetic on the fp32 epoch, rounded to fp32 once
  *out_delta = (float)(t->cfg.delta * 0.5 * (1.0 + tanh((((float)epoch_id) - (0.125 * n_epochs)) / 10.0)));
  return FV_OK;
}

extern "C" int fv_trainer_get_second_winners(fv_trainer *t, int32_t *out_seconds, uint32_t capacity) {
  FV_REQUIRE(t && out_seconds, FV_ERR_INVALID, "null argument");
  FV_REQUIRE(t->win2 && t->last_delta != 0.0f, FV_ERR_STATE, "the last step had no anti-Hebbian term");
  FV_REQUIRE(capacity >= t->last_n, FV_ERR_INVALID, "capacity %u below the %u windows of the last step", capacity,
             t->last_n);
  FV_HIP(hipStreamSynchronize(t->stream));
  FV_HIP(hipMemcpy(out_seconds, t->win2, (size_t)t->last_n * sizeof(int32_t), hipMemcpyDeviceToHost));
  return FV_OK;
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
  float eps = 0.0f, delta = 0.0f;
  FV_TRY(fv_trainer_epoch_eps(t, epoch_id, n_epochs, &eps));
  FV_TRY(fv_trainer_epoch_delta(t, epoch_id, n_epochs, &delta));
  // The reference's loop never skips a minibatch (flyvec/src/cuda_funcs.cu:1662-1812). A single dense launch
  // that gives up leaves the matrix as the step before it left it, and so do all launches behind it; the loop
  // is then taken up again at that step, with two launches per step.
  uint64_t k_first = 0;
  for (int attempt = 0; attempt < 2; ++attempt) {
    int rc = FV_OK;
    for (uint64_t k = k_first; k < t->n_windows && rc == FV_OK; k += t->B) {
      const uint64_t n = t->n_windows - k < t->B ? t->n_windows - k : t->B;
      t->step_tag = (uint32_t)(k / t->B) + 1u;
      if (n < t->B && k > 0 && t->stale_tail)
        // flyvec/src/cuda_funcs.cu:1679 against :1700-1732: only the sampler sees the remainder, the other
        // kernels run on all Num rows, those behind the remainder being the previous minibatch's
        rc = fv_enqueue_step(t, k, t->B, eps, delta, nullptr, 0x3f, false, (uint32_t)n);
      else
        rc = fv_enqueue_step(t, k, (uint32_t)n, eps, delta, nullptr);
    }
    t->step_tag = 0;
    FV_TRY(rc);
    FV_HIP(hipStreamSynchronize(t->stream));
    uint32_t tag = 0;
    FV_TRY(fv_trainer_take_giveup(t, &tag));
    if (!tag) return FV_OK;
    FV_REQUIRE(attempt == 0 && tag != 0xffffffffu, FV_ERR_STATE,
               "a dense launch gave up although the epoch was already being redone with two launches per step");
    k_first = (uint64_t)(tag - 1u) * t->B;
    t->giveups_recovered++;
  }
  return FV_OK;
}

extern "C" int fv_trainer_get_giveups_recovered(fv_trainer *t, uint64_t *out_count) {
  FV_REQUIRE(t && out_count, FV_ERR_INVALID, "null argument");
  *out_count = t->giveups_recovered;
  return FV_OK;
}

extern "C" int fv_trainer_set_stale_tail(fv_trainer *t, uint32_t on) {
  FV_REQUIRE(t, FV_ERR_INVALID, "null trainer");
  FV_REQUIRE(on <= 1, FV_ERR_INVALID, "on must be 0 or 1");
  t->stale_tail = on != 0;
  return FV_OK;
}

extern "C" int fv_trainer_set_dense_launches(fv_trainer *t, uint32_t launches) {
  FV_REQUIRE(t, FV_ERR_INVALID, "null trainer");
  FV_REQUIRE(launches <= 3, FV_ERR_INVALID, "launches must be 0 (choose), 1, 2 or 3 (one launch, rows streamed)");
  FV_REQUIRE(launches != 1 || t->onepass_blocks, FV_ERR_INVALID,
             "a row of %u neurons does not fit a block of this device: the dense passes need separate launches", t->K);
  FV_REQUIRE(launches != 3 || t->stream_ok, FV_ERR_INVALID,
             "the streaming dense launch does not fit this device: the dense passes need separate launches");
  t->onepass = launches == 2 ? false : t->onepass_blocks != 0;
  t->onepass_stream = launches == 3 || t->onepass_unroll == 0;
  FV_HIP(hipMemsetAsync(t->scalars + 1, 0, sizeof(float), t->stream));  // "a launch has given up"
  return FV_OK;
}

extern "C" int fv_trainer_set_grouping_launch(fv_trainer *t, uint32_t separate) {
  FV_REQUIRE(t, FV_ERR_INVALID, "null trainer");
  FV_REQUIRE(separate <= 1, FV_ERR_INVALID, "separate must be 0 or 1");
  t->separate_grouping = separate != 0;
  return FV_OK;
}

extern "C" int fv_trainer_set_sentinel_list(fv_trainer *t, uint32_t entries) {
  FV_REQUIRE(t, FV_ERR_INVALID, "null trainer");
  t->hit_cap_limit = entries;
  return FV_OK;
}

extern "C" int fv_trainer_set_slot_regions(fv_trainer *t, uint32_t per_block) {
  FV_REQUIRE(t, FV_ERR_INVALID, "null trainer");
  t->no_block_regions = per_block == 0;
  return FV_OK;
}

extern "C" int fv_trainer_get_grouping_launch(fv_trainer *t, uint32_t *out_separate) {
  FV_REQUIRE(t && out_separate, FV_ERR_INVALID, "null argument");
  *out_separate = (t->won[0] && !t->separate_grouping) ? 0u : 1u;
  return FV_OK;
}

extern "C" int fv_trainer_get_dense_launches(fv_trainer *t, uint32_t *out_launches) {
  FV_REQUIRE(t && out_launches, FV_ERR_INVALID, "null argument");
  // what a sentinel has to number in a step without the anti-Hebbian term
  const bool regions = t->won[0] && !t->separate_grouping && t->slot_region && !t->no_block_regions;
  const uint64_t n_slots = regions ? t->slot_region : (uint64_t)FV_NB_CLASSES * t->B * t->w;
  *out_launches = t->onepass && fv_trainers_alive.load() == 1 && n_slots + 1 < FV_SENTINEL_MAX ? 1u : 2u;
  return FV_OK;
}

extern "C" int fv_trainer_get_dense_path_counts(fv_trainer *t, uint64_t *out_known, uint64_t *out_pass) {
  FV_REQUIRE(t && out_known && out_pass, FV_ERR_INVALID, "null argument");
  uint32_t c[2] = {0, 0};
  FV_HIP(hipStreamSynchronize(t->stream));
  FV_HIP(hipMemcpy(c, t->path_count, sizeof c, hipMemcpyDeviceToHost));
  *out_known = c[0];
  *out_pass = c[1];
  return FV_OK;
}

extern "C" int fv_trainer_set_wait_limit(fv_trainer *t, uint32_t rounds) {
  FV_REQUIRE(t, FV_ERR_INVALID, "null trainer");
  t->onepass_spin_limit = rounds;
  return FV_OK;
}

extern "C" int fv_trainer_sync(fv_trainer *t) {
  FV_REQUIRE(t, FV_ERR_INVALID, "null trainer");
  return fv_trainer_wait(t);
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
    rc = fv_enqueue_step(t, first_window + (uint64_t)s * t->B, t->B, eps, 0.0f, nullptr);
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
    rc = fv_enqueue_step(t, first_window + (uint64_t)s * t->B, t->B, eps, 0.0f, &ev[(size_t)s * per]);
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

// The same steps as fv_trainer_time_steps, enqueued as HIP graphs: the launches of steps_per_graph consecutive
// steps are captured from the trainer's stream into one graph (every launch with the arguments it would have
// had), all graphs are instantiated first, and the timed region holds their launches only. The steps train
// like any others. No launch of a whole step is a memset, so the graphs hold kernel nodes only.
extern "C" int fv_trainer_time_steps_graph(fv_trainer *t, uint64_t first_window, uint32_t n_steps, float eps,
                                           uint32_t steps_per_graph, float *out_total_ms) {
  FV_REQUIRE(t && out_total_ms, FV_ERR_INVALID, "null argument");
  FV_REQUIRE(n_steps >= 1 && steps_per_graph >= 1, FV_ERR_INVALID, "n_steps and steps_per_graph must be >= 1");
  FV_TRY(fv_check_step(t, first_window, t->B));
  FV_REQUIRE(first_window + (uint64_t)n_steps * t->B <= t->n_windows, FV_ERR_INVALID,
             "%u steps of %u windows from %llu exceed the %llu available", n_steps, t->B,
             (unsigned long long)first_window, (unsigned long long)t->n_windows);
  FV_HIP(hipStreamSynchronize(t->stream));
  std::vector<hipGraphExec_t> execs;
  int rc = FV_OK;
  hipError_t e = hipSuccess;
  for (uint32_t s = 0; s < n_steps && rc == FV_OK && e == hipSuccess; s += steps_per_graph) {
    const uint32_t last = s + steps_per_graph < n_steps ? s + steps_per_graph : n_steps;
    hipGraph_t graph = nullptr;
    e = hipStreamBeginCapture(t->stream, hipStreamCaptureModeRelaxed);
    if (e != hipSuccess) break;
    for (uint32_t i = s; i < last && rc == FV_OK; ++i)
      rc = fv_enqueue_step(t, first_window + (uint64_t)i * t->B, t->B, eps, 0.0f, nullptr);
    e = hipStreamEndCapture(t->stream, &graph);
    if (e == hipSuccess && rc == FV_OK) {
      hipGraphExec_t exec = nullptr;
      e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
      if (e == hipSuccess) execs.push_back(exec);
    }
    if (graph) (void)hipGraphDestroy(graph);
  }
  hipEvent_t e0 = nullptr, e1 = nullptr;
  if (rc == FV_OK && e == hipSuccess) e = hipEventCreate(&e0);
  if (rc == FV_OK && e == hipSuccess) e = hipEventCreate(&e1);
  if (rc == FV_OK && e == hipSuccess) {
    e = hipEventRecord(e0, t->stream);
    for (size_t i = 0; i < execs.size() && e == hipSuccess; ++i) e = hipGraphLaunch(execs[i], t->stream);
    if (e == hipSuccess) e = hipEventRecord(e1, t->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(t->stream);
    if (e == hipSuccess) e = hipEventElapsedTime(out_total_ms, e0, e1);
  }
  for (hipGraphExec_t x : execs) (void)hipGraphExecDestroy(x);
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  if (rc != FV_OK) return rc;
  if (e != hipSuccess) return fv_fail(FV_ERR_HIP, "steps as graphs failed: %s", hipGetErrorString(e));
  return FV_OK;
}

extern "C" int fv_trainer_time_kernel(fv_trainer *t, uint32_t kernel_index, uint32_t reps, float *out_mean_ms) {
  FV_REQUIRE(t && out_mean_ms, FV_ERR_INVALID, "null argument");
  FV_REQUIRE(kernel_index < FV_TRAIN_KERNELS && reps >= 1, FV_ERR_INVALID, "bad kernel index or repetition count");
  FV_REQUIRE(t->last_n > 0, FV_ERR_STATE, "no step has run yet");
  hipEvent_t e0, e1;
  FV_HIP(hipEventCreate(&e0));
  FV_HIP(hipEventCreate(&e1));
  FV_HIP(hipStreamSynchronize(t->stream));
  int rc = fv_enqueue_step(t, t->last_first, t->last_n, t->last_eps, t->last_delta, nullptr, 1u << kernel_index);  // warm-up
  FV_HIP(hipEventRecord(e0, t->stream));
  for (uint32_t r = 0; r < reps && rc == FV_OK; ++r)
    rc = fv_enqueue_step(t, t->last_first, t->last_n, t->last_eps, t->last_delta, nullptr, 1u << kernel_index, true);
  FV_HIP(hipEventRecord(e1, t->stream));
  // the repeated winner launches have counted every window many times: once more from cleared buffers
  if (kernel_index == 0 && rc == FV_OK)
    rc = fv_enqueue_step(t, t->last_first, t->last_n, t->last_eps, t->last_delta, nullptr, 1u);
  FV_HIP(hipStreamSynchronize(t->stream));
  float ms = 0.0f;
  FV_HIP(hipEventElapsedTime(&ms, e0, e1));
  *out_mean_ms = ms / (float)reps;
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  return rc;
}
