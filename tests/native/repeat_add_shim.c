/* Host build of flyvec_amd/csrc/fv_repeat_add.h for the CPU test-suite: the accelerated
 * repeated addition next to the plain loop it must equal bit for bit. */
#include "fv_repeat_add.h"

float fvt_add_repeat(float v, float f, uint32_t n) { return fv_add_repeat(v, f, n); }

float fvt_add_naive(float v, float f, uint32_t n) {
  for (uint32_t t = 0; t < n; ++t) v = fv_add1(v, f);
  return v;
}

/* Number of (v, f, n) triples on which the two disagree. */
uint64_t fvt_count_mismatches(const float *v, const float *f, const uint32_t *n, uint64_t count) {
  uint64_t bad = 0;
  for (uint64_t i = 0; i < count; ++i) {
    float a = fv_add_repeat(v[i], f[i], n[i]), b = fvt_add_naive(v[i], f[i], n[i]);
    if (fv_f2u(a) != fv_f2u(b)) ++bad;
  }
  return bad;
}
