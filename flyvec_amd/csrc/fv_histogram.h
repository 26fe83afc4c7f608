// Arithmetic of the token histogram behind 1/frequency (flyvec/src/model_arrays.cu:396-424), shared by the
// kernel's host and device code and by the CPU test-suite. Plain C.
//
// The reference counts every token of a corpus indexed with uint64_t into an fp32 counter, which stops at
// 2^24. Here a grid of blocks strides over the corpus with 64-bit indices; a block counts the frequent ids
// in 32-bit LDS counters and adds them to 32-bit counters in HBM that saturate instead of wrapping, and
// the result is clamped to 2^24. Nothing in it depends on the corpus being shorter than 2^32 tokens.
#pragma once

#include <stdint.h>

#ifndef FV_HD
#if defined(__HIPCC__)
#define FV_HD __host__ __device__ __forceinline__
#else
#define FV_HD static inline
#endif
#endif

#define FV_HIST_THREADS 256u
#define FV_HIST_MAX_BLOCKS 2048u
#define FV_HIST_SATURATED 0x80000000u   /* where a counter in HBM stops: far above the 2^24 of the result */
#define FV_HIST_MAX_TOKENS (1ull << 42) /* a block's LDS counters stay below 2^32 up to here */
#define FV_HIST_CLAMP (1u << 24)        /* where the reference's fp32 counter stops */

/* Blocks of the histogram launch: one per 4096 tokens, at most FV_HIST_MAX_BLOCKS. */
FV_HD uint32_t fv_hist_blocks(uint64_t n_tokens) {
  const uint64_t want = (n_tokens + FV_HIST_THREADS * 16 - 1) / (FV_HIST_THREADS * 16);
  return (uint32_t)(want < 1 ? 1 : (want > FV_HIST_MAX_BLOCKS ? FV_HIST_MAX_BLOCKS : want));
}

/* Most tokens one block of that launch visits: its threads take the indices block * 256 + thread,
 * + blocks * 256, ... below n_tokens. */
FV_HD uint64_t fv_hist_block_tokens(uint64_t n_tokens, uint32_t blocks) {
  const uint64_t stride = (uint64_t)blocks * FV_HIST_THREADS;
  return (n_tokens + stride - 1) / stride * FV_HIST_THREADS;
}

/* A counter that holds `seen` after `add` more occurrences. */
FV_HD uint32_t fv_hist_saturated_sum(uint32_t seen, uint32_t add) {
  const uint64_t sum = (uint64_t)seen + add;
  return sum < FV_HIST_SATURATED ? (uint32_t)sum : FV_HIST_SATURATED;
}

/* 1 / count as the reference forms it: the count as the fp32 counter would hold it, the quotient in
 * double, rounded to fp32 (flyvec/src/model_arrays.cu:418-421). */
FV_HD float fv_hist_invert(uint32_t count) {
  const uint32_t c = count > FV_HIST_CLAMP ? FV_HIST_CLAMP : count;
  return c ? (float)(1.0 / (double)(float)c) : 0.0f;
}
