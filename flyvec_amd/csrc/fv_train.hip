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
//                      final value of every sparse element over its sentinel. One launch: max|ds|
//                      is usually known from the two largest |W| of every row, carried from step to
//                      step, and the launch is a single read-modify-write of the matrix; otherwise it
//                      makes the pass for the maximum first (on registers where the matrix fits the
//                      register file of the machine, by streaming the rows twice where it does not).
//                      As separate launches (4a max, 5 update, 6 slot update) on request or while the
//                      process holds more than one trainer.
//
// The device code is in fv_train_gather.h (1), fv_train_group.h (2), fv_train_sparse.h (3),
// fv_train_dense.h (4 to 6) and fv_train_top2.h (the carried largest weights); fv_train_state.h holds
// the trainer's state. This file has the small kernels of the window order and the host side.
//
// Every one of the n additions of 1/f onto ds[h][i] adds the same value, so the reference's
// result for that element depends only on n; replaying n sequential fp32 adds reproduces it
// exactly whatever order its atomics ran in.
#include "fv_train_state.h"
#include "fv_train_top2.h"
#include "fv_train_gather.h"
#include "fv_train_group.h"
#include "fv_train_sparse.h"
#include "fv_train_dense.h"

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

// Trainers alive in this process. The single dense launch, where it has to make the pass for max|ds|, exchanges
// the blocks' maxima inside the launch and so needs every compute unit for itself: two of them in flight at
// once, from two trainers' streams, could each hold half the machine and wait for the other half. While more
// than one trainer exists a step therefore enqueues the launch twice, in the form that waits for nobody
// (fv_dense_args.phase): the first does the whole step whenever max|ds| is known beforehand, the second then
// ends at once.
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
  // every block leaves a share of the rows' largest weights, and the next winner kernel merges one chunk of them
  if (blocks > FV_MERGE_CHUNK) blocks = FV_MERGE_CHUNK;
  const uint64_t need = (t->N + blocks * rows_per_round - 1) / (blocks * rows_per_round);
  {
    // the streaming form: its sentinel list takes more LDS than a launch may have without asking
    const size_t smem = fv_stream_smem(t);
    bool set = true;
#define FV_SET(KERNEL)                                                                                              \
  set = set && hipFuncSetAttribute((const void *)KERNEL, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) == hipSuccess;
    FV_SET((fv_dense_stream_kernel<false, 0>)) FV_SET((fv_dense_stream_kernel<true, 0>))
    FV_SET((fv_dense_stream_kernel<false, 1>)) FV_SET((fv_dense_stream_kernel<true, 1>))
    FV_SET((fv_dense_stream_kernel<false, 2>)) FV_SET((fv_dense_stream_kernel<true, 2>))
#undef FV_SET
    if (set)
      t->stream_ok = fv_stream_fits(smem) != 0;
    else
      (void)hipGetLastError();
  }
  unsigned unroll = 0;
  if (need <= FV_ONEPASS_MAX_UNROLL) {
    unroll = need <= 8 ? 8 : 16;
    const size_t smem = fv_onepass_smem(t);
    {
      // its sentinel lists take more LDS than a launch may have without asking
      bool set = true;
#define FV_SET(KERNEL)                                                                                              \
  set = set && hipFuncSetAttribute((const void *)KERNEL, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) == hipSuccess;
#define FV_SET_PHASES(U, DELTA) \
  FV_SET((fv_dense_onepass_kernel<U, DELTA, 0>)) FV_SET((fv_dense_onepass_kernel<U, DELTA, 1>)) FV_SET((fv_dense_onepass_kernel<U, DELTA, 2>))
      if (unroll == 8) { FV_SET_PHASES(8, false) FV_SET_PHASES(8, true) } else { FV_SET_PHASES(16, false) FV_SET_PHASES(16, true) }
#undef FV_SET_PHASES
#undef FV_SET
      if (!set) {
        (void)hipGetLastError();
        unroll = 0;
      }
    }
    if (unroll)
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
  (void)hipFree(t->won2[0]);
  (void)hipFree(t->slots2_blocks);
  (void)hipFree(t->slot_n2_blocks);
  t->won2[0] = t->won2[1] = nullptr;
  t->slots2_blocks = nullptr;
  t->slot_n2_blocks = nullptr;
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
  // The form that groups inside the sparse launch: bit rows for the second neurons, and a slot region per block. A
  // block writes at most one record per column of its class; the regions are that long only where a class has no
  // more columns than the minibatch has window positions (fv_trainer_alloc), else this form is not taken.
  const uint64_t class_cols = (t->N + FV_NB_CLASSES - 1) / FV_NB_CLASSES;
  if (t->won[0] && t->slot_region && t->slot_region == class_cols) {
    const size_t row_words = (size_t)t->K * t->won_words;
    const size_t records = (size_t)t->slot_region * t->K * FV_NB_CLASSES;
    FV_HIP(hipMalloc((void **)&t->won2[0], 2 * row_words * sizeof(uint32_t)));
    t->won2[1] = t->won2[0] + row_words;
    FV_HIP(hipMemsetAsync(t->won2[0], 0, 2 * row_words * sizeof(uint32_t), t->stream));
    FV_HIP(hipMalloc((void **)&t->slots2_blocks, records * sizeof(fv_slot)));
    FV_HIP(hipMalloc((void **)&t->slot_n2_blocks, records * sizeof(uint32_t)));
  }
  FV_HIP(hipMalloc((void **)&t->slot_n2, 2 * FV_NB_CLASSES * bw * sizeof(uint32_t)));
  return FV_OK;
}

// Whether the sparse launch of a step without the anti-Hebbian term groups for itself: the trainer has the bit rows
// (a minibatch of up to 64 windows per thread of a class block).
static bool fv_groups_in_sparse(const fv_trainer *t) { return t->won[0] && !t->separate_grouping; }

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
  // (beyond 64 windows per thread of a class block only with a slot region per block: without one every block
  // would count the lower neurons' windows in the whole winner array)
  const bool can_group = fv_groups_in_sparse(t) && (!anti || (t->slot_n2_blocks && !t->no_block_regions));
  const bool grouping_in_sparse = which == 0x3f ? can_group : (anti ? t->last_delta_grouped : t->last_grouped_in_sparse);
  if (which == 0x3f) (anti ? t->last_delta_grouped : t->last_grouped_in_sparse) = grouping_in_sparse;
  // the blocks of a sparse launch that groups for itself write their records to regions of their own, where
  // the trainer has them, and a sentinel names a record inside its block's region
  const uint32_t slot_region = grouping_in_sparse && !t->no_block_regions ? t->slot_region : 0u;
  if (slot_region) n_slots = slot_region;
  const bool onepass = t->onepass && n_slots + 1 < FV_SENTINEL_MAX;
  const bool alone = fv_trainers_alive.load() == 1;
  g.won = nullptr;
  g.won2 = nullptr;
  g.won_words = t->won_words;
  if (grouping_in_sparse) {
    if (which == 0x3f) {
      t->won_parity ^= 1u;
      if (anti) t->won2_parity ^= 1u;
    } else if ((which & 1u) && !repeated) {
      FV_HIP(hipMemsetAsync(t->won[t->won_parity], 0, (size_t)t->K * t->won_words * sizeof(uint32_t), t->stream));
      if (anti)
        FV_HIP(hipMemsetAsync(t->won2[t->won2_parity], 0, (size_t)t->K * t->won_words * sizeof(uint32_t), t->stream));
    }
    g.won = t->won[t->won_parity];
    if (anti) g.won2 = t->won2[t->won2_parity];
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
  sp.slots = anti ? (slot_region ? t->slots2_blocks : t->slots2) : slot_region ? t->slots_blocks : t->slots;
  sp.slot_region = slot_region;
  sp.n_blocks = t->K * FV_NB_CLASSES;
  sp.slot_stride = (uint64_t)t->B * t->w * (anti ? 2 : 1);
  sp.order2 = t->order2;
  sp.group_base2 = t->group_base2;
  sp.group_count2 = t->group_count2;
  sp.slot_n2 = anti && slot_region ? t->slot_n2_blocks : t->slot_n2;
  sp.delta = delta;
  sp.lmid = t->cfg.lmid;
  sp.lbase = t->cfg.lbase;
  sp.xx = t->xx;
  sp.invf = t->invf;
  sp.bmax_sparse = t->bmax + t->sparse_base;
  sp.row_top2 = t->row_top2;
  sp.row_hits = t->row_hits;
  sp.top2_known = top2_known ? 1u : 0u;
  sp.light = t->no_light_blocks ? 0u : 1u;
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
  sp.won2 = anti && grouping_in_sparse ? t->won2[t->won2_parity] : nullptr;
  sp.won2_clear = anti && grouping_in_sparse ? t->won2[t->won2_parity ^ 1u] : nullptr;
  sp.sc2 = t->sc2;
  sp.group_base2_out = t->group_base2;
  sp.group_count2_out = t->group_count2;
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
  if (anti && grouping_in_sparse)                                                                   \
    hipLaunchKernelGGL((fv_sparse_grouping_delta_kernel<CW>), sp_grid, sp_block, 0, t->stream, sp); \
  else if (anti)                                                                                    \
    hipLaunchKernelGGL((fv_sparse_kernel<true, CW>), sp_grid, sp_block, 0, t->stream, sp);          \
  else if (grouping_in_sparse)                                                                      \
    hipLaunchKernelGGL(GROUPING_KERNEL, sp_grid, sp_block, 0, t->stream, sp);                       \
  else if (t->B < 65535u)                                                                           \
    hipLaunchKernelGGL((fv_sparse_kernel<false, CW, true>), sp_grid, sp_block, 0, t->stream, sp);   \
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
  d.slots = anti ? (slot_region ? t->slots2_blocks : t->slots2) : slot_region ? t->slots_blocks : t->slots;
  d.slot_region = slot_region;
  {
    // (the register form keeps a list per wave, the streaming form one per block)
    const uint32_t holds = t->onepass_stream ? FV_STREAM_HIT_CAP : FV_ONEPASS_WAVE_HITS;
    d.hit_cap = t->hit_cap_limit && t->hit_cap_limit < holds ? t->hit_cap_limit : holds;
  }
  d.slot_count = t->slot_count;
  d.group_base = t->group_base;
  d.group_base2 = t->group_base2;
  d.slot_n2 = anti && slot_region ? t->slot_n2_blocks : t->slot_n2;
  d.delta = delta;
  d.w = t->w;
  d.arrive = nullptr;
  d.status = nullptr;
  d.phase = 0;
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
      // alone on the device: one launch that exchanges the blocks' maxima itself where it needs them; else the
      // launch twice, in the form that waits for nobody (both with this step's launch number)
      for (uint32_t phase = alone ? 0u : 1u; phase <= (alone ? 0u : 2u); ++phase) {
        d.phase = phase;
        if (t->onepass_stream) {
          if (anti) fv_launch_stream<true>(d, t->onepass_blocks, fv_stream_smem(t), t->stream);
          else fv_launch_stream<false>(d, t->onepass_blocks, fv_stream_smem(t), t->stream);
        } else if (t->onepass_unroll == 8) { FV_CASE(8) } else { FV_CASE(16) }
      }
#undef FV_CASE
      t->top2_valid = true;  // this launch leaves the shares of the matrix it writes
      t->top2_n_part = t->onepass_blocks;
      t->top2_merged = false;  // the next winner kernel's first blocks merge them
      FV_REQUIRE(t->top2_n_part <= FV_MERGE_CHUNK, FV_ERR_STATE, "a single dense launch of %u blocks leaves more shares "
                 "than the %d one chunk holds", t->top2_n_part, FV_MERGE_CHUNK);
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
    FV_REQUIRE(tag != 0xffffffffu, FV_ERR_STATE,
               "a single dense launch of a step enqueued before this epoch (fv_trainer_step without a fv_trainer_sync "
               "behind it) had given up: neither that step nor the epoch's steps have changed the matrix");
    FV_REQUIRE(attempt == 0, FV_ERR_STATE,
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

extern "C" int fv_trainer_set_light_blocks(fv_trainer *t, uint32_t on) {
  FV_REQUIRE(t, FV_ERR_INVALID, "null trainer");
  FV_REQUIRE(on <= 1, FV_ERR_INVALID, "on must be 0 or 1");
  t->no_light_blocks = on == 0;
  return FV_OK;
}

extern "C" int fv_trainer_get_grouping_launch(fv_trainer *t, uint32_t *out_separate) {
  FV_REQUIRE(t && out_separate, FV_ERR_INVALID, "null argument");
  *out_separate = fv_groups_in_sparse(t) ? 0u : 1u;
  return FV_OK;
}

extern "C" int fv_trainer_get_dense_launches(fv_trainer *t, uint32_t *out_launches) {
  FV_REQUIRE(t && out_launches, FV_ERR_INVALID, "null argument");
  // what a sentinel has to number in a step without the anti-Hebbian term
  const bool regions = fv_groups_in_sparse(t) && t->slot_region && !t->no_block_regions;
  const uint64_t n_slots = regions ? t->slot_region : (uint64_t)FV_NB_CLASSES * t->B * t->w;
  *out_launches = t->onepass && n_slots + 1 < FV_SENTINEL_MAX ? 1u : 2u;
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
  if (rc != FV_OK) return rc;
  FV_TRY(fv_trainer_wait(t));  // a launch that gave up makes the figure one of dead launches: FV_ERR_STATE
  if (!out_kernel_ms) return FV_OK;

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
  if (rc != FV_OK) return rc;
  return fv_trainer_wait(t);
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
  return fv_trainer_wait(t);  // FV_ERR_STATE if a launch gave up: the figure would be one of dead launches
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
