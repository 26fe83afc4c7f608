/* Host build of flyvec_amd/csrc/fv_layout.h for the CPU test-suite. */
#include "fv_layout.h"

uint32_t fvt_ldk(uint32_t K) { return fv_ldk(K); }
uint64_t fvt_alloc_elems(uint32_t K, uint64_t N) { return fv_matrix_alloc_elems(K, N); }
uint64_t fvt_gather_reach(uint32_t K, uint64_t N) { return fv_matrix_gather_reach(K, N); }
uint64_t fvt_pad_elems(uint32_t K) { return fv_matrix_pad_elems(K); }
