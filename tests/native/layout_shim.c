/* Host build of flyvec_amd/csrc/fv_layout.h for the CPU test-suite. */
#include "fv_layout.h"

uint32_t fvt_ldk(uint32_t K) { return fv_ldk(K); }
uint64_t fvt_alloc_elems(uint32_t K, uint64_t N) { return fv_matrix_alloc_elems(K, N); }
uint64_t fvt_gather_reach(uint32_t K, uint64_t N) { return fv_matrix_gather_reach(K, N); }
uint64_t fvt_pad_elems(uint32_t K) { return fv_matrix_pad_elems(K); }
uint64_t fvt_slot_place(uint32_t blk, uint32_t number, uint32_t region, uint32_t n_blocks) {
  return fv_slot_place(blk, number, region, n_blocks);
}
uint64_t fvt_slot_regions_records(uint32_t region, uint32_t n_blocks) { return fv_slot_regions_records(region, n_blocks); }
uint32_t fvt_slot_primary(void) { return FV_SLOT_PRIMARY; }
