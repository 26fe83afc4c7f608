/*
 * flyvec_hip.h -- C ABI of libflyvec_hip.so: the FlyVec training minibatch step and
 * the top-k hashing path on one AMD MI355X (gfx950).
 *
 * One shared library replaces the five CUDA shared objects the reference's Python
 * driver loads with ctypes (flyvec/train_flyvec.py:62-66) and adds the batched form
 * of FlyVec.get_sparse_embedding (flyvec/core.py:139-163).  Every entry point cites
 * the reference interface it stands in for.  Unlike the reference (void returns,
 * exit() on error, flyvec/src/cuda_funcs.cu:36-54) every function returns a status
 * and leaves a message for fv_last_error(); nothing here terminates the process.
 *
 * Conventions: plain pointers and sizes only.  Unless a name ends in _dev, pointer
 * arguments are HOST memory owned by the caller.  The synapse matrix crosses this
 * boundary exactly as the reference's checkpoint stores it: fp32, K x 2V, row-major
 * (flyvec/train_flyvec.py:245-263; context block = columns [0,V), target block =
 * [V,2V), flyvec/src/cuda_funcs.cu:929-932).  Handles are thread-compatible, not
 * thread-safe.  The library uses device 0 unless fv_set_device() is called first.
 */
#ifndef FLYVEC_HIP_H
#define FLYVEC_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FV_OK 0
#define FV_ERR_INVALID 1 /* bad argument or shape */
#define FV_ERR_HIP 2     /* a HIP runtime call failed */
#define FV_ERR_STATE 3   /* call order: corpus / weights / permutation not set */
#define FV_ERR_DATA 4    /* input data violates the contract (token id out of range, ...) */

/* ---- runtime ------------------------------------------------------------------ */

/* Message of the last failing call on this thread ("" if none). */
const char *fv_last_error(void);

/* flyvec/src/cuda_helpers.cu:31 get_cuda_num_devices */
int fv_device_count(int *out_count);
int fv_set_device(int device);
/* Name, compute units and HBM bytes of the current device (for logs and the bench). */
int fv_device_info(char *name, size_t name_cap, int *out_compute_units, uint64_t *out_hbm_bytes);
/* Free and total memory of the current device as the runtime reports them (either may be NULL). */
int fv_device_memory(uint64_t *out_free_bytes, uint64_t *out_total_bytes);

/* flyvec/src/cuda_helpers.cu:22 do_gpu_cudaHostAlloc (pinned host staging memory) */
int fv_host_alloc_pinned(size_t bytes, void **out_ptr);
int fv_host_free_pinned(void *ptr);

/* flyvec/src/cuda_helpers.cu:8 do_gpu_cudaMallocManaged -- the reference keeps every
 * buffer in managed memory; here device buffers are explicit.  Used by callers that
 * keep hash inputs / outputs resident in HBM (the *_dev entry points). */
int fv_dev_alloc(size_t bytes, void **out_dev_ptr);
int fv_dev_free(void *dev_ptr);
int fv_dev_upload(void *dst_dev, const void *src_host, size_t bytes);
int fv_dev_download(void *dst_host, const void *src_dev, size_t bytes);

/* Measurement: `reps` launches of a plain device-to-device copy kernel moving `bytes` (read) +
 * `bytes` (written); mean duration by HIP events. The yardstick for hardware byte counters. No
 * counterpart in the reference. */
int fv_calibration_copy(size_t bytes, uint32_t reps, float *out_mean_ms);

/* ---- window sampler, host half ------------------------------------------------ */

/* flyvec/src/prune_input.cpp:64 getnum_samples: number of length-w windows that do not
 * cross a chunk boundary, over chunks with w <= length < 214. offsets has n_chunks+1
 * entries. */
int fv_count_windows(const uint64_t *offsets, uint64_t n_chunks, uint64_t w, uint64_t *out_count);

/* flyvec/src/prune_input.cpp:88 compute_offset_phrases: corpus position of every window,
 * in chunk order; a start is the sum of all previous chunk LENGTHS plus the position in
 * the chunk (offsets[0] is assumed 0, as the reference does). out_starts must hold
 * `capacity` >= fv_count_windows entries. */
int fv_build_window_starts(const uint64_t *offsets, uint64_t n_chunks, uint64_t w,
                           uint64_t *out_starts, uint64_t capacity);

/* flyvec/src/model_arrays.cu:396 compute_inverse_word_frequency: out[t] = 1/count(t) over
 * the whole corpus, 0 for absent ids, negative ids ignored; counts saturate at 2^24 as the
 * reference's fp32 counter does. */
int fv_inverse_frequency(const int32_t *corpus, uint64_t n_tokens, uint64_t vocab, float *out_invf);

/* fv_inverse_frequency for callers that cannot allocate device memory (tight serving loops, harnesses
 * that forbid hipMalloc, a process whose device memory is all spoken for). It has no counterpart in the
 * reference. Corpus and output are DEVICE memory of the caller (fv_dev_alloc or any other device
 * allocation); the occurrence counters live in an array built into the library (4 MiB on every device
 * the library runs on, kept until the process ends), so vocab is at most 2^20 = 1,048,576 ids and a
 * larger one is refused with FV_ERR_INVALID. Calls nothing that allocates or frees. It runs on the
 * default stream and ends with a blocking copy of the id range to the host: it returns when the result
 * is in out_invf_dev, and is not itself a sequence a HIP graph could capture. FV_ERR_DATA on an id >= vocab (the output then ignores
 * such ids). All calls on one device share that device's array: calls that overlap on one device
 * race, results of calls made one after the other do not depend on earlier ones. */
int fv_inverse_frequency_static(const int32_t *corpus_dev, uint64_t n_tokens, uint64_t vocab,
                                float *out_invf_dev);

/* Test hook. The token histogram behind 1/frequency keeps 32-bit counters in HBM. A corpus of fewer than 2^31
 * tokens cannot bring one to 2^31 and is counted with plain additions; a longer one is counted by a form whose
 * counters stop at 2^31 instead of wrapping (the result is clamped to 2^24 either way). n_tokens > 0: corpora of
 * at least that many tokens take the second form; 0 restores 2^31. Process-wide. No counterpart in the reference. */
int fv_histogram_stops_from(uint64_t n_tokens);

/* flyvec/src/remove_words.cpp:28-37 (an off-line tool of the reference: for every id of a stop list,
 * data[w] == id ? -1): rewrites `tokens` in place, every occurrence of an id of `remove_ids`
 * becomes -1 (masked: such a position contributes nothing to a window). One pass on the device,
 * whatever the length of the list; ids must lie in [0, vocab). */
int fv_mask_tokens(int32_t *tokens, uint64_t n_tokens, const int32_t *remove_ids, uint64_t n_remove,
                   uint64_t vocab);

/* flyvec/src/prune_input.cpp:14 prune_input_data (exported by the reference, bound at
 * flyvec/train_flyvec.py:79, never called): in every row of a rows x cols int32 window matrix a value
 * that an earlier column holds becomes -1; the centre column (cols / 2) takes no part and keeps its
 * value. In place, one pass on the device; cols <= 64. */
int fv_prune_windows(int32_t *data, uint64_t rows, uint64_t cols);

/* ---- trainer ------------------------------------------------------------------ */

typedef struct fv_trainer fv_trainer;

/* The hyper-parameters flyvec/train_flyvec.py:191-213 pushes through set_model_param_int /
 * set_model_param_float (flyvec/src/model_descriptor.cu:51-87). */
typedef struct fv_train_config {
  uint64_t vocab;              /* V ("vocabulary_size"); W is hid x 2V */
  uint32_t hid;                /* K ("hid"), 1..2048 */
  uint32_t window;             /* w ("W"), 1..64 */
  uint32_t batch;              /* B ("Num"), windows per minibatch */
  uint32_t tie_rule;           /* argmax ties: 0 lowest index, 1 the reference's lane-tree order
                                  (flyvec/src/cuda_funcs.cu:488-561) */
  float initial_learning_rate; /* "initial_learning_rate" */
  float delta;                 /* "delta": strength of the anti-Hebbian term on the second neuron (0 = none) */
  float prec;                  /* "prec" */
  float lmid;                  /* "Lmid": weight of a window's centre position (flyvec/src/cuda_funcs.cu:266-327,
                                  675-697); 1 is all the reference's command line reaches */
  float lbase;                 /* "Lbase": weight of the other positions; 1 likewise */
  uint32_t prune_duplicates;   /* 1: the sampler drops a token that an earlier position of its window holds
                                  (not the centre's): flyvec/src/cuda_funcs.cu:938-979, switched off in the
                                  reference (:1681); 0 is the reference's behaviour */
} fv_train_config;

/* flyvec/src/model_descriptor.cu:18 model_create_descriptor + flyvec/src/model_arrays.cu:15,22
 * model_create_arrays / model_arrays_allocate_memory */
int fv_trainer_create(const fv_train_config *cfg, fv_trainer **out_trainer);
int fv_trainer_destroy(fv_trainer *t);

/* flyvec/src/model_arrays.cu:358 set_up_INPUT_pointer + :396 compute_inverse_word_frequency
 * + flyvec/src/prune_input.cpp:88: uploads the corpus (int32 ids in [0,V) or -1) and builds
 * the window-start table, 1/frequency and the identity permutation in HBM. offsets has
 * n_offsets entries (n_offsets-1 chunks). Fails with FV_ERR_DATA on ids outside [-1, V). */
int fv_trainer_set_corpus(fv_trainer *t, const int32_t *tokens, uint64_t n_tokens,
                          const uint64_t *offsets, uint64_t n_offsets);
/* flyvec/src/model_arrays.cu:358 set_up_INPUT_pointer as the reference's driver calls it: the corpus and
 * the window-start table that compute_offset_phrases wrote (every start + window <= n_tokens, else
 * FV_ERR_DATA); builds 1/frequency and the identity permutation like fv_trainer_set_corpus. */
int fv_trainer_set_corpus_starts(fv_trainer *t, const int32_t *tokens, uint64_t n_tokens,
                                 const uint64_t *starts, uint64_t n_windows);
int fv_trainer_num_windows(fv_trainer *t, uint64_t *out_count);
/* Read-back of what set_corpus built (parity hooks). */
int fv_trainer_get_window_starts(fv_trainer *t, uint64_t *out_starts, uint64_t capacity);
int fv_trainer_get_inverse_frequency(fv_trainer *t, float *out_invf);

/* flyvec/src/model_arrays.cu:305 get_data_pointer("synapses"): the reference hands Python a
 * pointer into managed memory; here the matrix is copied in / out (K x 2V fp32 row-major). */
int fv_trainer_set_weights(fv_trainer *t, const float *W);
int fv_trainer_get_weights(fv_trainer *t, float *out_W);

/* flyvec/src/model_arrays.cu:442 do_reshuffle_indices: rearranges the current window order,
 * cumulatively across calls.  The reference runs a serial swap loop on the host fed by cuRAND's
 * scrambled Sobol64; here the order becomes perm[sigma(i)] on the device, sigma a bijection of
 * [0, Nwin) keyed by `seed` and the number of earlier calls.  Asynchronous. */
int fv_trainer_shuffle(fv_trainer *t, uint64_t seed);
/* Test hook replacing the random stream: install / read the window permutation. */
int fv_trainer_set_permutation(fv_trainer *t, const uint64_t *perm, uint64_t n);
int fv_trainer_get_permutation(fv_trainer *t, uint64_t *out_perm, uint64_t capacity);

/* One pass of the minibatch loop body, flyvec/src/cuda_funcs.cu:1662-1803, on windows
 * perm[first_window .. first_window + n_windows) with n_windows <= batch. Asynchronous. */
int fv_trainer_step(fv_trainer *t, uint64_t first_window, uint32_t n_windows, float eps);

/* The same step with the anti-Hebbian term of strength `delta` (flyvec/src/cuda_funcs.cu:495-548,
 * 667-668, 726-734): the second neuron of every window -- the winner search repeated with the
 * winner's activation overwritten by -9999.9999 -- receives -delta times what the winner receives.
 * fv_trainer_step is this with delta = 0. */
int fv_trainer_step_delta(fv_trainer *t, uint64_t first_window, uint32_t n_windows, float eps, float delta);
/* flyvec/src/cuda_funcs.cu:1230: delta_epoch = delta * 0.5 * (1 + tanh((epoch - 0.125 n_epochs) / 10))
 * with delta from the configuration; fv_trainer_run_epoch uses it. */
int fv_trainer_epoch_delta(fv_trainer *t, uint64_t epoch_id, uint64_t n_epochs, float *out_delta);
/* Test hook: the second neurons of the last step (only after a step with delta != 0). */
int fv_trainer_get_second_winners(fv_trainer *t, int32_t *out_seconds, uint32_t capacity);

/* flyvec/src/cuda_funcs.cu:1220 launch_epoch_INPUT_AS_INT: eps = lr0 * (1 - epoch/n_epochs),
 * then every minibatch of the current permutation (the last one takes the remainder only, unless
 * fv_trainer_set_stale_tail says otherwise).
 * Returns after the device has finished. */
int fv_trainer_run_epoch(fv_trainer *t, uint64_t epoch_id, uint64_t n_epochs);
/* The reference's treatment of a final partial minibatch: flyvec/src/cuda_funcs.cu:1679 launches only the
 * sampler with the remainder, every other kernel with the full minibatch (:1700-1732), so the rows behind
 * the remainder still hold the previous minibatch's windows and are trained on once more. on = 1 makes
 * fv_trainer_run_epoch do the same (when a full minibatch precedes the partial one in the epoch);
 * 0, the default, trains the remainder only. */
int fv_trainer_set_stale_tail(fv_trainer *t, uint32_t on);
/* eps of flyvec/src/cuda_funcs.cu:1229 for this trainer's learning rate. */
int fv_trainer_epoch_eps(fv_trainer *t, uint64_t epoch_id, uint64_t n_epochs, float *out_eps);

/* Waits for the trainer's stream. FV_ERR_STATE if a single dense launch (below) gave up waiting for
 * its other blocks: neither that step nor the steps enqueued behind it have changed the matrix.
 * fv_trainer_run_epoch does not return that error: it takes the epoch up again at the step that gave up,
 * with two launches per step, and counts the event (fv_trainer_get_giveups_recovered). */
int fv_trainer_sync(fv_trainer *t);
int fv_trainer_get_giveups_recovered(fv_trainer *t, uint64_t *out_count);

/* The two passes over the matrix of a step (max|ds|, flyvec/src/cu_special_reduction.cu:241, and
 * the update, flyvec/src/cuda_funcs.cu:1787-1806) run as ONE launch wherever a block of the device holds a row
 * of the matrix (every hid this library takes) and a sentinel can number the step's slot records (fewer than 2^23): with
 * the matrix kept in registers between the passes where it fits them (64 MiB on 256 compute units), with its
 * rows streamed through the registers otherwise. launches = 1 asks for the single launch (FV_ERR_INVALID where
 * there is none), 3 for its streaming form whatever the matrix size, 2 for separate launches (maximum, update,
 * sparse elements), 0 returns to the choice made at creation. Results are bit-identical in all forms. Where the
 * single launch has to make the pass for max|ds| its blocks exchange their maxima inside the launch and need the
 * whole device for themselves; while a process holds more than one trainer a step therefore enqueues the launch
 * twice in a form that waits for nobody: the first does the whole step when max|ds| is known beforehand (the
 * usual case) and the second ends at once, else the first makes the pass and the second the update. */
int fv_trainer_set_dense_launches(fv_trainer *t, uint32_t launches);
/* The single launch carries the two largest |W| of every row from step to step; from them and from what
 * the sparse-element launch reports it usually knows max|ds| (flyvec/src/cu_special_reduction.cu:241) before
 * it reads the matrix and is then one streaming read-modify-write; otherwise it makes the pass for the
 * maximum first, on registers. Counts of single launches so far that knew it / that made the pass (the
 * first step on a new matrix always makes it). Same results either way. No counterpart in the reference. */
int fv_trainer_get_dense_path_counts(fv_trainer *t, uint64_t *out_known, uint64_t *out_pass);
/* The form the next step takes: 1 = the single launch (after fv_trainer_set_dense_launches(1) or (3), its
 * register or its streaming form, as the matrix size and that call decide), 2 = separate launches. */
int fv_trainer_get_dense_launches(fv_trainer *t, uint32_t *out_launches);
/* Grouping the windows of a step by winner (what flyvec/src/cuda_funcs.cu:1719-1721 leaves in
 * max_IDs and xx) runs inside the sparse-element launch when the trainer's batch is at most 16384
 * windows and the step has no anti-Hebbian term, as a launch of its own otherwise. separate = 1 forces the launch of its
 * own, 0 returns to that rule. Results are bit-identical either way. */
int fv_trainer_set_grouping_launch(fv_trainer *t, uint32_t separate);
int fv_trainer_get_grouping_launch(fv_trainer *t, uint32_t *out_separate); /* the form a step without the anti-Hebbian term takes */
/* Where the sparse-element launch that groups for itself keeps a step's records of sparse elements (the
 * weight, count and 1/frequency of each element the minibatch touches: the sparse operand of
 * flyvec/src/cuda_funcs.cu:657-672). per_block = 1, the default: every block of that launch has room of its own
 * for as many records as its class has columns (or the minibatch positions, if fewer), where that takes no more
 * than a gigabyte in all, so no block has to count the windows of the neurons before it; per_block = 0: the
 * blocks share one region per class, each behind the records of the neurons before it, as the other launch
 * forms do. Results are bit-identical either way. No counterpart in the reference. */
int fv_trainer_set_slot_regions(fv_trainer *t, uint32_t per_block);
/* In that launch form (blocks with regions of their own) a neuron that won so few windows that a block has a thread
 * for each of their positions (21 windows of 11 at 256 threads) is finished by one of its four blocks alone, an
 * entry per thread, and the other three end at once: most neurons of a Zipf minibatch are such. on = 1, the
 * default; 0 keeps the four class blocks for every neuron. Results are bit-identical either way. No counterpart
 * in the reference. */
int fv_trainer_set_light_blocks(fv_trainer *t, uint32_t on);
/* Test hook. The single dense launch notes the sparse elements it meets (their sentinels) in LDS lists, one of
 * 256 entries per wave in the register form, one of 8192 per block in the streaming form, and finishes them when
 * its dense elements are done; an element that finds its list full is finished by its own thread. entries > 0
 * makes a list count as full after that many (no more than it holds), 0 restores its size. Results are
 * bit-identical. No counterpart in the reference. */
int fv_trainer_set_sentinel_list(fv_trainer *t, uint32_t entries);
/* Test hook: between its two passes a single-launch dense pass waits for all its blocks, at most
 * `rounds` polling rounds (2^14 by default, tens of milliseconds); 0 makes every block give up at once, which
 * is how the error path of fv_trainer_sync is exercised. No counterpart in the reference. */
int fv_trainer_set_wait_limit(fv_trainer *t, uint32_t rounds);

/* Parity hooks on the last step: winner per window (max_IDs[r][0], flyvec/src/cuda_funcs.cu:
 * 1719), per-neuron totals xx (:1721) and max|ds| (flyvec/src/cu_special_reduction.cu:241). */
int fv_trainer_get_winners(fv_trainer *t, int32_t *out_winners, uint32_t capacity);
int fv_trainer_get_step_stats(fv_trainer *t, float *out_xx /* hid */, float *out_max_abs_ds);

/* flyvec/src/cuda_funcs.cu:1234-1242: L2 norm of the first n_rows rows of W (the reference
 * prints them for 10 rows before every epoch). */
int fv_trainer_row_norms(fv_trainer *t, uint32_t n_rows, double *out_norms);

/* Measurement: n_steps consecutive full minibatches starting at first_window, timed with HIP
 * events on the trainer's stream. out_total_ms covers all steps; out_kernel_ms[FV_TRAIN_KERNELS]
 * (nullable) receives the mean duration of each kernel of the step, measured in a second,
 * separately instrumented run of the same steps. */
#define FV_TRAIN_KERNELS 6 /* gather+winner, group by winner + xx, sparse owners, max|ds|, update, sparse update;
                              as a single dense launch (fv_trainer_set_dense_launches) the last three are
                              one kernel, timed under the first of them, and the other two read ~0 */
int fv_trainer_time_steps(fv_trainer *t, uint64_t first_window, uint32_t n_steps, float eps,
                          float *out_total_ms, float *out_kernel_ms);

/* Measurement: the same n_steps minibatches enqueued as HIP graphs. The launches of steps_per_graph
 * consecutive steps are captured from the trainer's stream into one graph, each with the arguments an
 * ordinary step would give it; all graphs are instantiated before the clock starts, and out_total_ms covers
 * their launches. The steps train like any others (same bits in W). No counterpart in the reference. */
int fv_trainer_time_steps_graph(fv_trainer *t, uint64_t first_window, uint32_t n_steps, float eps,
                                uint32_t steps_per_graph, float *out_total_ms);

/* Measurement: launches kernel `kernel_index` (0 .. FV_TRAIN_KERNELS-1) of the last step `reps`
 * times back to back on its buffers and returns the mean duration between two HIP events on the
 * trainer's stream. The kernels that write W are not idempotent: the matrix is left in a state
 * that is only good for timing, so install weights again before training on. */
int fv_trainer_time_kernel(fv_trainer *t, uint32_t kernel_index, uint32_t reps, float *out_mean_ms);

/* ---- hashing ------------------------------------------------------------------ */

typedef struct fv_hasher fv_hasher;

/* flyvec/core.py:82-88 (FlyVec.synapses): takes the checkpoint matrix (K x N fp32 row-major,
 * N = 2V) and keeps it resident in HBM. */
int fv_hasher_create(const float *W, uint32_t hid, uint64_t n_columns, fv_hasher **out_hasher);
int fv_hasher_destroy(fv_hasher *h);

/* flyvec/core.py:23-36 normalize_synapses, p = 2: each row divided by (sqrt(sum of squares)
 * + prec), sum taken in numpy's pairwise fp32 order. In place on the resident matrix. */
int fv_hasher_normalize(fv_hasher *h, float prec);
/* The two device passes of that normalisation, for callers that take the p-th root themselves
 * (numpy's power(x, 1/p) is what the reference calls): out_sums[r] = sum_i W[r][i]^2 in numpy's
 * pairwise fp32 order; then W[r][:] /= divisors[r]. */
int fv_hasher_row_sumsq(fv_hasher *h, float *out_sums /* hid */);
/* The same for another integer exponent of the norm (flyvec/core.py:23 takes p): out_sums[r] = sum_i W[r][i]^p in the
 * same order. p = 1 and p = 2 restate numpy exactly (the value, the fp32 product); from p = 3 on numpy's float32
 * power is the C library's powf, and the power taken here -- the product in double, rounded to fp32 once -- can
 * differ from it in the last bit of an element. 1 <= p <= 64. */
int fv_hasher_row_sum_pow(fv_hasher *h, uint32_t p, float *out_sums /* hid */);
int fv_hasher_scale_rows(fv_hasher *h, const float *divisors /* hid */);
/* Current resident matrix, K x N row-major. */
int fv_hasher_get_weights(fv_hasher *h, float *out_W);

/* flyvec/core.py:153-158 get_sparse_embedding for n token ids at once: activation = column
 * V + id; thr = fl32(a[k-1] + a[k]) / 2 over the descending order statistics; code = act > thr.
 * out_codes is n x hid int8. Requires 0 < k < hid (the reference raises IndexError otherwise). */
int fv_hash_targets(fv_hasher *h, const int32_t *ids, uint64_t n, uint32_t k, int8_t *out_codes);

/* Windowed form: activation = fp32 sum, in window order, of the columns idx[r][0..w) (-1
 * skipped), then the same threshold rule. Either output may be NULL: out_bits is
 * n x ceil(hid/64) uint64 (neuron h -> word h>>6, bit h&63), out_codes is n x hid int8. */
int fv_hash_windows(fv_hasher *h, const int32_t *idx, uint64_t n, uint32_t w, uint32_t k,
                    uint64_t *out_bits, int8_t *out_codes);

/* Same with idx and outputs already in HBM (fv_dev_alloc); asynchronous on the hasher's stream. */
int fv_hash_windows_dev(fv_hasher *h, const int32_t *idx_dev, uint64_t n, uint32_t w, uint32_t k,
                        uint64_t *out_bits_dev, int8_t *out_codes_dev);
/* Waits for the stream; FV_ERR_DATA if any launched batch met a column index outside [-1, N). */
int fv_hasher_sync(fv_hasher *h);
/* Measurement: `reps` launches of fv_hash_windows_dev, mean kernel duration by HIP events. */
int fv_hasher_time_windows(fv_hasher *h, const int32_t *idx_dev, uint64_t n, uint32_t w, uint32_t k,
                           uint64_t *out_bits_dev, int8_t *out_codes_dev, uint32_t reps,
                           float *out_mean_ms);

#ifdef __cplusplus
}
#endif
#endif /* FLYVEC_HIP_H */
