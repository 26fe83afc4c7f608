/* Host build of flyvec_amd/csrc/fv_histogram.h for the CPU test-suite. */
#include "fv_histogram.h"

uint32_t fvt_hist_blocks(uint64_t n_tokens) { return fv_hist_blocks(n_tokens); }
uint64_t fvt_hist_block_tokens(uint64_t n_tokens, uint32_t blocks) { return fv_hist_block_tokens(n_tokens, blocks); }
uint32_t fvt_hist_saturated_sum(uint32_t seen, uint32_t add) { return fv_hist_saturated_sum(seen, add); }
float fvt_hist_invert(uint32_t count) { return fv_hist_invert(count); }
uint64_t fvt_hist_max_tokens(void) { return FV_HIST_MAX_TOKENS; }

/* The token indices one thread of the launch visits, as the kernel's loop forms them (64-bit throughout):
 * returns how many, leaves the first and the last in out[0], out[1]. */
uint64_t fvt_hist_thread_span(uint64_t n_tokens, uint32_t blocks, uint32_t block, uint32_t thread, uint64_t *out) {
  const uint64_t stride = (uint64_t)blocks * FV_HIST_THREADS;
  const uint64_t first = (uint64_t)block * FV_HIST_THREADS + thread;
  if (first >= n_tokens) return 0;
  const uint64_t count = (n_tokens - first + stride - 1) / stride;
  out[0] = first;
  out[1] = first + (count - 1) * stride;
  return count;
}
