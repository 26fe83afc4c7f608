// A keyed bijection of [0, n) computed per index, for shuffling the window order on the device.
//
// The reference reshuffles with a serial swap loop over the whole index array on the host
// (flyvec/src/model_arrays.cu:451-465). Here sigma(i) is a balanced Feistel network on
// 2 * half_bits bits (the smallest even width that covers n - 1), iterated until the value falls
// below n ("cycle walking"): a Feistel network is a bijection of its whole domain whatever the
// round function is, and walking a bijection's cycle back into a subset is a bijection of the
// subset. The domain holds fewer than 4 n values, so an index takes fewer than 4 walks on average.
// Compiles for the host too, where the tests check the bijection.
#pragma once

#include <stdint.h>

#ifndef FV_HD
#if defined(__HIPCC__)
#define FV_HD __host__ __device__ __forceinline__
#else
#define FV_HD static inline
#endif
#endif

#define FV_FEISTEL_ROUNDS 8

typedef struct fv_feistel {
  uint32_t half_bits;  // 1 .. 32
  uint32_t half_mask;
  uint32_t keys[FV_FEISTEL_ROUNDS];
} fv_feistel;

FV_HD uint64_t fv_mix64(uint64_t z) {  // splitmix64 finaliser
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

FV_HD uint32_t fv_mix32(uint32_t h) {  // murmur3 finaliser
  h ^= h >> 16;
  h *= 0x85ebca6bu;
  h ^= h >> 13;
  h *= 0xc2b2ae35u;
  return h ^ (h >> 16);
}

// Network for indices below n (n >= 1) under the given seed.
FV_HD fv_feistel fv_feistel_make(uint64_t n, uint64_t seed) {
  fv_feistel f;
  uint32_t bits = 0;
  while (bits < 64 && ((n - 1) >> bits) != 0) ++bits;
  f.half_bits = bits < 2 ? 1u : (bits + 1) / 2;
  f.half_mask = f.half_bits == 32 ? 0xffffffffu : (1u << f.half_bits) - 1u;
  uint64_t s = seed;
  for (int r = 0; r < FV_FEISTEL_ROUNDS; r += 2) {
    s += 0x9E3779B97F4A7C15ull;
    const uint64_t k = fv_mix64(s);
    f.keys[r] = (uint32_t)k;
    f.keys[r + 1] = (uint32_t)(k >> 32);
  }
  return f;
}

// One pass through the network: a bijection of [0, 2^(2 * half_bits)).
FV_HD uint64_t fv_feistel_apply(const fv_feistel *f, uint64_t x) {
  uint32_t l = (uint32_t)(x >> f->half_bits) & f->half_mask, r = (uint32_t)x & f->half_mask;
  for (int i = 0; i < FV_FEISTEL_ROUNDS; ++i) {
    const uint32_t t = l ^ (fv_mix32(r * 0x9E3779B1u + f->keys[i]) & f->half_mask);
    l = r;
    r = t;
  }
  return ((uint64_t)l << f->half_bits) | r;
}

// sigma(i) for i < n.
FV_HD uint64_t fv_permute_index(const fv_feistel *f, uint64_t i, uint64_t n) {
  uint64_t x = i;
  do {
    x = fv_feistel_apply(f, x);
  } while (x >= n);
  return x;
}
