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
// WAVES: the block's waves where the caller knows them at compile time. blockDim.x is one of the launch's hidden
// arguments: the compiler fetches it where it is first used, and that first use then waits for a trip to memory
// in the middle of the kernel (0: read it).
template <uint32_t WAVES = 0>
__device__ __forceinline__ float fv_block_max_nonneg(float m, float *smem) {
  const uint32_t wm = fv_wave_max_u32(__float_as_uint(m));
  __syncthreads();
  if ((threadIdx.x & 63) == 0) smem[threadIdx.x >> 6] = __uint_as_float(wm);
  __syncthreads();
  float r = smem[0];
  const uint32_t n_waves = WAVES ? WAVES : blockDim.x >> 6;
  for (uint32_t i = 1; i < n_waves; ++i) r = fmaxf(r, smem[i]);
  return r;
}

// Sum over the block of one value per thread (result in every thread).
template <uint32_t WAVES = 0>
__device__ __forceinline__ uint32_t fv_block_sum_u32(uint32_t v, uint32_t *smem /*17*/) {
  v = fv_wave_sum_u32(v);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n_waves = WAVES ? (int)WAVES : (int)(blockDim.x >> 6);
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

// The sum of one value per lane over the balanced binary tree on the lane number: lanes 2i and 2i + 1 first, then
// the pairs, ... The partner's value arrives by a DPP lane pattern inside a row of 16 lanes (addition is commutative,
// so both partners form the same bits and every lane of an aligned group holds the group's sum), the four rows' sums
// through v_readlane. All 64 lanes must be active. This is the order of the per-neuron totals xx: a lane's value is the
// total of one group of 64 windows, and flyvec/src/cuda_funcs.cu:722-744 leaves the order to its atomics.
__device__ __forceinline__ float fv_wave_tree_sum(float v) {
#define FV_TREE_STEP(CTRL) v = __fadd_rn(v, __uint_as_float(fv_dpp<CTRL>(__float_as_uint(v))));
  FV_TREE_STEP(FV_DPP_QUAD_XOR1)  // lane ^ 1
  FV_TREE_STEP(FV_DPP_QUAD_XOR2)  // lane ^ 2
  FV_TREE_STEP(0x141)             // row_half_mirror: lane 7 - i of each 8, which holds the other quad's sum
  FV_TREE_STEP(0x140)             // row_mirror: lane 15 - i, which holds the other half's sum
#undef FV_TREE_STEP
  const float r0 = __uint_as_float(fv_readlane(__float_as_uint(v), 0)), r1 = __uint_as_float(fv_readlane(__float_as_uint(v), 16));
  const float r2 = __uint_as_float(fv_readlane(__float_as_uint(v), 32)), r3 = __uint_as_float(fv_readlane(__float_as_uint(v), 48));
  return __fadd_rn(__fadd_rn(r0, r1), __fadd_rn(r2, r3));
}

// The same tree continued over the waves of a block (wave w holds the lanes 64 w .. 64 w + 63 of the tree): the wave
// sums meet in smem (16 floats) and every thread adds them up, the waves a block does not have counting as +0
// (no value here is -0, so that changes no bit). LDS-only barriers.
__device__ __forceinline__ void fv_lds_barrier();
template <uint32_t WAVES = 0>
__device__ __forceinline__ float fv_block_tree_sum(float v, float *smem /*16*/) {
  const float ws = fv_wave_tree_sum(v);
  const uint32_t wave = threadIdx.x >> 6, n_waves = WAVES ? WAVES : blockDim.x >> 6;
  fv_lds_barrier();  // whoever still reads smem from an earlier use has done so
  if ((threadIdx.x & 63u) == 0) smem[wave] = ws;
  fv_lds_barrier();
  float t[16];
#pragma unroll
  for (uint32_t i = 0; i < 16; ++i) t[i] = i < n_waves ? smem[i] : 0.0f;
#pragma unroll
  for (uint32_t stride = 1; stride < 16; stride <<= 1)
#pragma unroll
    for (uint32_t i = 0; i < 16; i += 2 * stride) t[i] = __fadd_rn(t[i], t[i + stride]);
  return t[0];
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

// The order of the additions behind xx[h] (the reference leaves it to its atomics, flyvec/src/cuda_funcs.cu:731): the
// minibatch's rows in groups of 64; a neuron's values of a group are added in row order onto +0; the groups' sums
// over the balanced binary tree on the group number (fv_wave_tree_sum, fv_block_tree_sum). A thread's run is one
// group, or a power of two of them (its own subtree, which it adds up itself), so the thread number continues the
// tree. The CPU checker states the same order.
//
// SMALL: a thread's run is one group and the minibatch has fewer than 2^16 windows. The run is then
// fetched in one trip to memory (8 loads of 16 bytes in flight), the two counts travel through
// one block scan as the halves of a word, and the scaled activations of a thread's first matches
// are fetched while that scan runs.
// Winner number q (0 .. 7) of a 16-byte load of 16-bit winners.
__device__ __forceinline__ uint32_t fv_winner_of(const int4 &v, int q) {
  const uint32_t word = (uint32_t)((q >> 1) == 0 ? v.x : (q >> 1) == 1 ? v.y : (q >> 1) == 2 ? v.z : v.w);
  return (q & 1) ? word >> 16 : word & 0xffffu;
}

typedef short fv_short2 __attribute__((ext_vector_type(2)));

// Groups of 64 windows per thread of a block of T threads that takes n windows: the smallest power of two that covers them.
__host__ __device__ __forceinline__ uint32_t fv_group_run_groups(uint32_t n, uint32_t T) {
  uint32_t m = 1;
  while ((uint64_t)64 * m * T < n) m <<= 1;
  return m;
}

template <bool SMALL>
__global__ __launch_bounds__(FV_NB_MAX_THREADS) void fv_group_kernel(fv_group_args a) {
  __shared__ uint32_t red[17];
  __shared__ float tree[16];

  const uint32_t h = blockIdx.x;
  const uint32_t tid = threadIdx.x, T = blockDim.x;
  const uint32_t n = a.n;
  const uint16_t *__restrict__ win = a.win;

  // A thread's run is m groups of 64 windows (SMALL: one), read as 16-byte loads of 8 winners; matches among
  // its first 64 windows are kept as a bit mask.
  const uint32_t m_groups = SMALL ? 1u : fv_group_run_groups(n, T);
  const uint32_t seg = 64u * m_groups;
  const uint32_t r0 = (uint32_t)min((uint64_t)tid * seg, (uint64_t)n), r1 = (uint32_t)min((uint64_t)r0 + seg, (uint64_t)n);
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
    for (int q = 0; q < 64; ++q) {
      const uint32_t wv = fv_winner_of(wv4[q >> 3], q & 7);
      const bool in = r0 + q < r1;
      lt += in && wv < h;
      const bool hit = in && wv == h;
      eq += hit;
      mask |= (uint64_t)hit << q;
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
  // the neuron's windows, ascending, into order[]; the thread's own part of xx beside it
  uint32_t *order = a.order + base;
  float part = 0.0f;
  if (SMALL) {
    uint32_t rank = my_off;
    uint64_t mm = mask;
#pragma unroll
    for (int q = 0; q < PF; ++q) {
      if (mm) {
        order[rank++] = r0 + (uint32_t)__ffsll((long long)mm) - 1;
        part = __fadd_rn(part, pf[q]);
        mm &= mm - 1;
      }
    }
    // a thread with more matches than it has fetched values for: the rest, eight loads at a time
    while (__ballot(mm != 0ull)) {
      uint32_t r[8];
      float v[8];
      uint64_t m2 = mm;
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        r[q] = m2 ? r0 + (uint32_t)__ffsll((long long)m2) - 1 : r0;
        m2 &= m2 - 1;
        v[q] = __fmul_rn(a.scale, a.sc[min(r[q], n - 1)]);
      }
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        if (mm) {
          order[rank++] = r[q];
          part = __fadd_rn(part, v[q]);
          mm &= mm - 1;
        }
      }
    }
  } else {
    // the matches of the thread's first 64 windows are in the mask, the others are found again in the winner array
    uint32_t rank = my_off;
    for (uint64_t mm = mask; mm; mm &= mm - 1) order[rank++] = r0 + (uint32_t)__ffsll((long long)mm) - 1;
    for (uint32_t r = r0 + 64; r < r1; ++r)
      if ((uint32_t)win[r] == h) order[rank++] = r;
    // the thread's groups one after the other; their sums meet on a stack that is the thread's subtree: a finished
    // node of level k waits in stack[k] for its right sibling (static indices: the stack stays in registers)
    float stack[16];  // n < 2^30 windows and 1024 threads: at most 2^14 groups per thread
#pragma unroll
    for (int k = 0; k < 16; ++k) stack[k] = 0.0f;
    uint32_t j = my_off;  // next match of the thread, by rank (its own writes to order[] above)
    const uint32_t j_end = my_off + eq;
    for (uint32_t g = 0; g < m_groups; ++g) {
      const uint32_t g_end = r0 + 64u * (g + 1);
      float p_g = 0.0f;
      while (j < j_end) {  // up to four values of the group fetched together
        uint32_t r[4];
        float v[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) r[q] = order[min(j + q, j_end - 1)];
#pragma unroll
        for (int q = 0; q < 4; ++q) v[q] = __fmul_rn(a.scale, a.sc[r[q]]);
        uint32_t took = 0;
#pragma unroll
        for (int q = 0; q < 4; ++q)
          if (took == (uint32_t)q && j + q < j_end && r[q] < g_end) {
            p_g = __fadd_rn(p_g, v[q]);
            ++took;
          }
        j += took;
        if (took < 4) break;
      }
      float carry = p_g;
      bool placed = false;
      uint32_t i = g;
#pragma unroll
      for (int k = 0; k < 16; ++k) {
        if (!placed) {
          if (i & 1u) {
            carry = __fadd_rn(stack[k], carry);
          } else {
            stack[k] = carry;
            placed = true;
          }
        }
        i >>= 1;
      }
    }
    // m_groups = 2^k: the last group's carry ended in stack[k], the root of the thread's subtree
#pragma unroll
    for (int k = 0; k < 16; ++k)
      if (m_groups == (1u << k)) part = stack[k];
  }
  const float xx = fv_block_tree_sum(part, tree);
  if (tid == 0) a.xx[h] = a.accumulate ? __fadd_rn(a.xx[h], xx) : xx;
}
