// n sequential fp32 additions of the same value, in fewer than n steps, bit for bit.
//
// The reference adds 1/f onto ds[h][i] once per occurrence of token i in the windows neuron h
// won (flyvec/src/cuda_funcs.cu:657-672); for a frequent token that is thousands of additions
// onto one element.  The result v_n of  v_{k+1} = fl(v_k + f)  is reproduced exactly by noting
// that while v stays inside one binade (same sign and exponent) its bit pattern moves by a
// constant number of ulps per addition: the exact sum is (m + q + r) ulps with m the integer
// significand of v and q + r = f / ulp, and round-to-nearest turns the fraction r into the same
// 0 or 1 every time.  The one exception, r = 1/2 exactly (ties-to-even looks at the parity of
// m + q), settles after one addition, because every tie result is even.  So: take three real
// additions; if all three results share a binade and the two differences are equal, the state
// is steady and the remaining additions inside the binade are one integer multiply-add on the
// bit pattern (stopping short of the binade's ends); binade crossings, including the passage
// through zero, are taken with real additions.  Compiles for the host too, where the tests
// check it against the plain loop.
#pragma once

#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#define FV_HD __host__ __device__ __forceinline__
#else
#define FV_HD static inline
#endif

FV_HD uint32_t fv_f2u(float x) {
  uint32_t u;
  memcpy(&u, &x, sizeof u);
  return u;
}

FV_HD float fv_u2f(uint32_t u) {
  float x;
  memcpy(&x, &u, sizeof x);
  return x;
}

// One rounded addition; never fused with a neighbouring multiply.
FV_HD float fv_add1(float a, float b) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __fadd_rn(a, b);
#else
  volatile float r = a + b;
  return r;
#endif
}

FV_HD float fv_add_repeat(float v, float f, uint32_t n) {
  while (n >= 4) {
    const float v1 = fv_add1(v, f), v2 = fv_add1(v1, f), v3 = fv_add1(v2, f);
    n -= 3;
    v = v3;
    const uint32_t b1 = fv_f2u(v1), b2 = fv_f2u(v2);
    uint32_t b3 = fv_f2u(v3);
    if (b3 == b2) return v;  // f is absorbed: every further addition returns v again
    const uint32_t se = b1 >> 23;  // sign and exponent
    if (se == (b2 >> 23) && se == (b3 >> 23) && (se & 0xffu) != 0u && (se & 0xffu) != 0xffu) {
      const int32_t d1 = (int32_t)(b2 - b1), d2 = (int32_t)(b3 - b2);
      if (d1 == d2) {
        // the bit pattern grows when the magnitude grows, whatever the sign
        const uint32_t mant = b3 & 0x7fffffu;
        // ulps left inside the binade. Shrinking magnitudes stop one ulp short of the binade's
        // lowest value: a sum that rounds onto it may lie below it, where the spacing is finer.
        const uint32_t room = d1 > 0 ? 0x7fffffu - mant : (mant ? mant - 1u : 0u);
        const uint32_t step = d1 > 0 ? (uint32_t)d1 : (uint32_t)(-d1);
        uint32_t k = room / step;
        if (k > n) k = n;
        b3 = d1 > 0 ? b3 + k * step : b3 - k * step;
        v = fv_u2f(b3);
        n -= k;
      }
    }
  }
  while (n > 0) {
    v = fv_add1(v, f);
    --n;
  }
  return v;
}
