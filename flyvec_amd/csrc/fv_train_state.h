// State of a trainer and what its kernels share: the sentinel that stands in W for a sparse element, the
// slot record that holds the element meanwhile, and the trainer itself.
#pragma once

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
  // the same for the second neurons of the anti-Hebbian form (allocated with its other buffers; its own parity: it
  // changes only with the steps that use the rows)
  uint32_t *won2[2];
  uint32_t won2_parity;
  // records per block of the sparse launch when that form groups for itself (like slots_blocks) and their second counts
  fv_slot *slots2_blocks;
  uint32_t *slot_n2_blocks;
  bool last_delta_grouped;  // the form the last whole anti-Hebbian step took
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
  bool no_light_blocks;   // fv_trainer_set_light_blocks(0): a neuron with few windows keeps its four class blocks
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
