// Kernel 2 of the training step and the block-level helpers kernel 3 shares with it (device code of fv_train.hip).
#pragma once

#include "fv_train_state.h"

// ---- kernel 2: group the windows by winner, xx ----------------------------------------------------
//
// One block per neuron h scans the winner array once (every thread a contiguous run, so per-thread
// match counts are in window order) and writes the neuron's windows, ascending, to
// order[group_base[h] .. +group_count[h]); it then adds their scaled activations in that order: xx[h].

#define FV_NB_MAX_THREADS 1024
#ifndef FV_NB_CLASS_SHIFT
#define FV_NB_CLASS_SHIFT 2
#endif
#define FV_NB_CLASSES (1 << FV_NB_CLASS_SHIFT)  // column classes per neuron (kernel 3)
#define FV_NB_CNT_WORDS 5120    // LDS counter words per class block (20 KB)
#define FV_NB_CNT_WORDS_WIDE 6272  // or 24.5 KB, where that saves a pass
#define FV_SP_LIST_CAP 1024     // positions of non-zero counters collected in LDS at a time
#define FV_SP_CHUNK 16          // window positions read by 4 neighbouring lanes, 16 bytes each
#define FV_IDX_PAD 80            // entries of -1 behind the index matrix: a padding row (up to 64 entries) and spare
#define FV_SP_STAGE 2048        // window ids staged in LDS at a time
#ifndef FV_SP_THREADS
#define FV_SP_THREADS 256       // threads of a class block
#endif
#ifndef FV_SP_LOADS
#define FV_SP_LOADS 8           // most 16-byte loads a lane has in flight in the counting pass
#endif
#define FV_SP_HEAVY 128         // a class block of a neuron with more windows than this runs at raised wave priority
#define FV_NB_ROUND 2048        // scaled activations staged in LDS at a time
#define FV_NB_LOADS 32          // winners a thread of the grouping kernel fetches together

struct fv_group_args {
  const uint16_t *win;  // 16-bit winners, padded: readable up to n rounded up to 64
  const float *sc;
  uint32_t *order;
  uint32_t *group_base;
  uint32_t *group_count;
  float *xx;
  uint32_t n;
  float scale;          // every scaled activation is multiplied by this first (1, or -delta for the second neurons)
  uint32_t accumulate;  // add the total to xx[h] instead of storing it
};

// ds of one sparse element: the dense term, then n sequential additions of l * 1/f, l the weight of
// the element's window position (flyvec/src/cuda_funcs.cu:675-697: a double product of two floats
// rounded once is their fp32 product; l = 1 leaves 1/f as it is).
__device__ __forceinline__ float fv_sparse_ds(float xx, float wv, float f, uint32_t n, float l) {
  return fv_add_repeat(__fmul_rn(-xx, wv), __fmul_rn(l, f), n);
}

__device__ __forceinline__ float fv_absmax_keep(float m, float v) {
  const float a = fabsf(v);
  return a > m ? a : m;  // a NaN never replaces m, as in the reference's comparison
}

// ds of one sparse element with the anti-Hebbian term: after the n additions of l * 1/f, n2 additions
// of (-delta * l) * 1/f (flyvec/src/cuda_funcs.cu:667-668, 689, 693; this order of the additions is
// the checker's).
__device__ __forceinline__ float fv_sparse_ds2(float xx, float wv, float f, uint32_t n, float delta, uint32_t n2,
                                               float l) {
  return fv_add_repeat(fv_sparse_ds(xx, wv, f, n, l), __fmul_rn(__fmul_rn(-delta, l), f), n2);
}

// Block-wide maximum of non-negative floats (blocks of up to 16 waves; smem holds one float per wave).
__device__ __forceinline__ float fv_block_max_nonneg(float m, float *smem) {
  const uint32_t wm = fv_wave_max_u32(__float_as_uint(m));
  __syncthreads();
  if ((threadIdx.x & 63) == 0) smem[threadIdx.x >> 6] = __uint_as_float(wm);
  __syncthreads();
  float r = smem[0];
  for (uint32_t i = 1; i < (blockDim.x >> 6); ++i) r = fmaxf(r, smem[i]);
  return r;
}

// Sum over the block of one value per thread (result in every thread).
__device__ __forceinline__ uint32_t fv_block_sum_u32(uint32_t v, uint32_t *smem /*17*/) {
  v = fv_wave_sum_u32(v);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n_waves = blockDim.x >> 6;
  __syncthreads();
  if (lane == 0) smem[wave] = v;
  __syncthreads();
  uint32_t t = 0;
  for (int i = 0; i < n_waves; ++i) t += smem[i];
  return t;
}

// Exclusive prefix sum of one value per thread over the block.
__device__ __forceinline__ uint32_t fv_block_exclusive_scan(uint32_t v, uint32_t *smem /*17*/) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t incl = fv_wave_inclusive_scan_u32(v);
  __syncthreads();
  if (lane == 63) smem[wave] = incl;
  __syncthreads();
  uint32_t before = 0;
  for (int i = 0; i < wave; ++i) before += smem[i];
  return before + incl - v;
}

// Barrier for data exchanged through LDS only: waits for the wave's LDS operations, not for its
// global loads and stores still in flight.
__device__ __forceinline__ void fv_lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Exclusive prefix sum and total of one value per thread over the block, in one pass. LDS_ONLY: the
// barriers do not wait for the caller's global loads in flight.
template <bool LDS_ONLY = false>
__device__ __forceinline__ uint32_t fv_block_scan_total(uint32_t v, uint32_t *smem /*17*/, uint32_t *total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n_waves = blockDim.x >> 6;
  const uint32_t incl = fv_wave_inclusive_scan_u32(v);
  if (LDS_ONLY) fv_lds_barrier(); else __syncthreads();
  if (lane == 63) smem[wave] = incl;
  if (LDS_ONLY) fv_lds_barrier(); else __syncthreads();
  uint32_t before = 0, all = 0;
  for (int i = 0; i < n_waves; ++i) {
    const uint32_t t = smem[i];
    before += i < wave ? t : 0u;
    all += t;
  }
  *total = all;
  return before + incl - v;
}

// SMALL: a thread's run is at most 64 windows and the minibatch has fewer than 2^16. The run is then
// fetched in one trip to memory (16 loads of 16 bytes in flight), the two counts travel through
// one block scan as the halves of a word, and the scaled activations of a thread's first matches
// are fetched while that scan runs.
// Winner number q (0 .. 7) of a 16-byte load of 16-bit winners.
__device__ __forceinline__ uint32_t fv_winner_of(const int4 &v, int q) {
  const uint32_t word = (uint32_t)((q >> 1) == 0 ? v.x : (q >> 1) == 1 ? v.y : (q >> 1) == 2 ? v.z : v.w);
  return (q & 1) ? word >> 16 : word & 0xffffu;
}

typedef short fv_short2 __attribute__((ext_vector_type(2)));

template <bool SMALL>
__global__ __launch_bounds__(FV_NB_MAX_THREADS) void fv_group_kernel(fv_group_args a) {
  __shared__ float scbuf[FV_NB_ROUND];
  __shared__ uint32_t red[17];

  const uint32_t h = blockIdx.x;
  const uint32_t tid = threadIdx.x, T = blockDim.x;
  const uint32_t n = a.n;
  const uint16_t *__restrict__ win = a.win;

  // A thread's run is a multiple of 8 windows, read as 16-byte loads of 8 winners; matches among
  // its first 64 windows are kept as a bit mask.
  const uint32_t seg = ((n + T - 1) / T + 7) & ~7u;
  const uint32_t r0 = min(tid * seg, n), r1 = min(r0 + seg, n);
  const uint32_t n_pad = (n + 63) & ~63u;
  uint32_t lt = 0, eq = 0;
  uint64_t mask = 0;
  uint32_t base, my_off, c_h;
  constexpr int PF = 8;
  float pf[PF];
  if (SMALL) {
    int4 wv4[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) wv4[q] = *(const int4 *)(win + min(r0 + 8 * q, n_pad - 8));
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      if (g * 16 < (int)seg) {  // the same answer in the whole block
#pragma unroll
        for (int q = 16 * g; q < 16 * g + 16; ++q) {
          const uint32_t wv = fv_winner_of(wv4[q >> 3], q & 7);
          const bool in = r0 + q < r1;
          lt += in && wv < h;
          const bool hit = in && wv == h;
          eq += hit;
          mask |= (uint64_t)hit << q;
        }
      }
    }
    uint64_t mm = mask;
#pragma unroll
    for (int q = 0; q < PF; ++q) {
      const uint32_t r = mm ? r0 + (uint32_t)__ffsll((long long)mm) - 1 : r0;
      pf[q] = __fmul_rn(a.scale, a.sc[min(r, n - 1)]);
      mm &= mm - 1;
    }
    uint32_t total;
    const uint32_t before = fv_block_scan_total(lt | (eq << 16), red, &total);
    base = total & 0xffffu;
    c_h = total >> 16;
    my_off = before >> 16;
  } else {
    for (uint32_t rb = r0; rb < r1; rb += FV_NB_LOADS) {
      int4 wv4[FV_NB_LOADS / 8];
#pragma unroll
      for (int q = 0; q < FV_NB_LOADS / 8; ++q) wv4[q] = *(const int4 *)(win + min(rb + 8 * q, n_pad - 8));
#pragma unroll
      for (int q = 0; q < FV_NB_LOADS; ++q) {
        const uint32_t wv = fv_winner_of(wv4[q >> 3], q & 7);
        const bool in = rb + q < r1;
        lt += in && wv < h;
        const bool hit = in && wv == h;
        eq += hit;
        const uint32_t o = rb + q - r0;
        mask |= o < 64 ? (uint64_t)hit << o : 0ull;
      }
    }
    base = fv_block_sum_u32(lt, red);  // windows won by lower neurons
    my_off = fv_block_exclusive_scan(eq, red);
    c_h = fv_block_sum_u32(eq, red);
  }
  if (tid == 0) {
    a.group_base[h] = base;
    a.group_count[h] = c_h;
  }
  // SMALL and the neuron's values fit scbuf: they are placed by rank here, without a trip through order[]
  const bool staged = SMALL && c_h <= FV_NB_ROUND;
  uint32_t *order = a.order + base;
  {
    uint32_t rank = my_off;
    uint64_t mm = mask;
    if (SMALL) {
#pragma unroll
      for (int q = 0; q < PF; ++q) {
        if (mm) {
          order[rank] = r0 + (uint32_t)__ffsll((long long)mm) - 1;
          if (staged) scbuf[rank] = pf[q];
          ++rank;
          mm &= mm - 1;
        }
      }
    }
    while (mm) {
      const uint32_t r = r0 + (uint32_t)__ffsll((long long)mm) - 1;
      order[rank] = r;
      if (staged) scbuf[rank] = __fmul_rn(a.scale, a.sc[r]);
      ++rank;
      mm &= mm - 1;
    }
    for (uint32_t r = r0 + 64; r < r1; ++r)
      if ((uint32_t)win[r] == h) order[rank++] = r;
  }
  __syncthreads();  // the neuron's part of order[] (and of scbuf) is now readable by the whole block

  // xx[h]: lane l of the first wave adds the neuron's scaled activations number l, l + 64, l + 128, ...
  // (window order) onto 0, then the 64 partial sums are added onto 0 in lane order. For up to 64
  // windows that is the plain sum in window order.
  float part = 0.0f;
  if (staged) {
    if (tid < 64) {
      // four values fetched together, added one after the other
      uint32_t j = tid;
      for (; j + 192 < c_h; j += 256) {
        const float v0 = scbuf[j], v1 = scbuf[j + 64], v2 = scbuf[j + 128], v3 = scbuf[j + 192];
        part = __fadd_rn(__fadd_rn(__fadd_rn(__fadd_rn(part, v0), v1), v2), v3);
      }
      for (; j < c_h; j += 64) part = __fadd_rn(part, scbuf[j]);
    }
  } else {
    for (uint32_t j0 = 0; j0 < c_h; j0 += FV_NB_ROUND) {
      const uint32_t mr = min(c_h - j0, (uint32_t)FV_NB_ROUND);
      for (uint32_t jb = tid; jb < mr; jb += 4 * T) {  // up to 4 independent loads per thread
        uint32_t r[4];
        float v[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) r[q] = order[j0 + min(jb + q * T, mr - 1)];
#pragma unroll
        for (int q = 0; q < 4; ++q) v[q] = __fmul_rn(a.scale, a.sc[r[q]]);
#pragma unroll
        for (int q = 0; q < 4; ++q)
          if (jb + q * T < mr) scbuf[jb + q * T] = v[q];
      }
      __syncthreads();
      if (tid < 64)
        for (uint32_t j = tid; j < mr; j += 64) part = __fadd_rn(part, scbuf[j]);  // FV_NB_ROUND % 64 == 0
      __syncthreads();
    }
  }
  // The partial sums in lane order, read straight from the lanes of the first wave (a partial sum
  // without values is +0, which changes nothing: the running total starts at +0 and so is never -0).
  if (tid < 64) {
    float xx = 0.0f;
#pragma unroll
    for (int l = 0; l < 64; ++l) xx = __fadd_rn(xx, __uint_as_float(fv_readlane(__float_as_uint(part), l)));
    if (tid == 0) a.xx[h] = a.accumulate ? __fadd_rn(a.xx[h], xx) : xx;
  }
}
