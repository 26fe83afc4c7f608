// Size of the device allocation that holds the token-major synapse matrix, and the farthest element
// a window gather reads from it. Plain C: the kernels' host code and the CPU test-suite both use it.
//
// The matrix is N rows (one per column of the K x N checkpoint matrix) of ldk floats, ldk = K rounded
// up to 4. A window gather (fv_gather_batch) loads, for every row it touches, the floats
// row * ldk + lane + 64 * j for all 64 lanes and j < NV = ceil(K / 64), with no bound on the lane: the
// values past K are accumulated and never used. The rows it touches are 0 .. N, row N being the row
// of zeros that a masked position reads. So the farthest element read is N * ldk + 64 * NV - 1, and
// the allocation holds N * ldk + max(FV_PAD_ROWS * ldk, 64 * NV) floats; everything behind the N real
// rows is zero and no pass writes it. (Two rows cover the overrun only while 64 * NV <= 2 * ldk,
// which fails for K <= 28.)
#pragma once

#include <stdint.h>

#define FV_PAD_ROWS 2

#if defined(__HIPCC__)
#define FV_LAYOUT_HD __host__ __device__ __forceinline__
#else
#define FV_LAYOUT_HD static inline
#endif

static inline uint32_t fv_ldk(uint32_t K) { return (K + 3u) & ~3u; }

// 64-float registers per lane of a wave that holds K values.
static inline uint32_t fv_lane_values(uint32_t K) { return (K + 63u) / 64u; }

// Floats behind the N real rows.
static inline uint64_t fv_matrix_pad_elems(uint32_t K) {
  const uint64_t rows = (uint64_t)FV_PAD_ROWS * fv_ldk(K), reach = 64ull * fv_lane_values(K);
  return rows > reach ? rows : reach;
}

// Floats of the whole allocation.
static inline uint64_t fv_matrix_alloc_elems(uint32_t K, uint64_t N) {
  return N * fv_ldk(K) + fv_matrix_pad_elems(K);
}

// One past the farthest element index a gather of rows 0 .. N reads.
static inline uint64_t fv_matrix_gather_reach(uint32_t K, uint64_t N) {
  return N * fv_ldk(K) + 64ull * fv_lane_values(K);
}

// Where record `number` of block `blk` of the sparse launch lies when every block has a region of `region` records
// of its own (n_blocks blocks): the first FV_SLOT_PRIMARY records of all blocks side by side, the others in a second
// part with the rest of every region. Nearly every block has fewer records than that, so a step's records lie
// within n_blocks * FV_SLOT_PRIMARY records (26 MB at 1600 blocks) instead of being strewn over all regions (256 MB at
// 10000 records each; with that layout the sparse launch was measured at 16.8 us instead of 14.8 in some processes
// and not in others), and only the few heaviest neurons' blocks touch the second part.
#ifndef FV_SLOT_PRIMARY
#define FV_SLOT_PRIMARY 1024u
#endif
FV_LAYOUT_HD uint64_t fv_slot_place(uint32_t blk, uint32_t number, uint32_t region, uint32_t n_blocks) {
  const uint32_t first = region < FV_SLOT_PRIMARY ? region : FV_SLOT_PRIMARY;
  // (the usual case in 32 bits: n_blocks * first is at most 2^13 * 2^10; on the device the other case is a branch
  // the wave takes only if one of its lanes has such a record, so that the usual one stays one instruction)
  const uint32_t low = blk * first + number;
#if defined(__HIP_DEVICE_COMPILE__)
  if (!__any(number >= first)) return low;
#endif
  return number < first ? (uint64_t)low
                        : (uint64_t)n_blocks * first + (uint64_t)blk * (region - first) + (number - first);
}

// Records the regions of n_blocks blocks take together.
static inline uint64_t fv_slot_regions_records(uint32_t region, uint32_t n_blocks) { return (uint64_t)region * n_blocks; }
