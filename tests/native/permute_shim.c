/* Host build of flyvec_amd/csrc/fv_permute.h for the CPU test-suite. */
#include "fv_permute.h"

/* out[i] = sigma(i) for i < n under `seed`. */
void fvt_permutation(uint64_t n, uint64_t seed, uint64_t *out) {
  fv_feistel f = fv_feistel_make(n, seed);
  for (uint64_t i = 0; i < n; ++i) out[i] = fv_permute_index(&f, i, n);
}

uint32_t fvt_half_bits(uint64_t n) { return fv_feistel_make(n, 0).half_bits; }
