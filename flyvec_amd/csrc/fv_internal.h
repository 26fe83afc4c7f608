// Internal declarations shared by the translation units of libflyvec_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "flyvec_hip.h"
#include "fv_layout.h"

#define FV_WAVE 64
#define FV_MAX_HID 2048   // 32 values per lane in the wave-per-window kernels
#define FV_MAX_WINDOW 64  // one lane per window position

// ---- error plumbing -------------------------------------------------------------
int fv_fail(int code, const char *fmt, ...);
void fv_clear_error();

#define FV_HIP(call)                                                                          \
  do {                                                                                        \
    hipError_t e__ = (call);                                                                  \
    if (e__ != hipSuccess)                                                                    \
      return fv_fail(FV_ERR_HIP, "%s failed: %s (%s:%d)", #call, hipGetErrorString(e__),      \
                     __FILE__, __LINE__);                                                     \
  } while (0)

#define FV_TRY(call)          \
  do {                        \
    int rc__ = (call);        \
    if (rc__ != FV_OK) return rc__; \
  } while (0)

#define FV_REQUIRE(cond, code, ...)              \
  do {                                           \
    if (!(cond)) return fv_fail(code, __VA_ARGS__); \
  } while (0)

// ---- device layout of the synapse matrix -----------------------------------------
// Token-major: column i of the K x N checkpoint matrix is the contiguous row
// Wt[i * ldk .. i * ldk + K), ldk = K rounded up to a multiple of 4 floats (fv_ldk) so every
// row starts 16-byte aligned; the pad is kept at zero. fv_layout.h sizes the allocation.

// K x N row-major (staging, device) <-> token-major N x ldk (device). Asynchronous.
int fv_launch_to_token_major(const float *W_rowmajor_dev, float *Wt_dev, uint32_t K, uint64_t N,
                             uint32_t ldk, hipStream_t stream);
int fv_launch_to_row_major(const float *Wt_dev, float *W_rowmajor_dev, uint32_t K, uint64_t N,
                           uint32_t ldk, hipStream_t stream);
// Upload / download a K x N host matrix through a temporary device staging buffer.
int fv_upload_weights(const float *W_host, float *Wt_dev, uint32_t K, uint64_t N, uint32_t ldk,
                      hipStream_t stream);
int fv_download_weights(const float *Wt_dev, float *W_host, uint32_t K, uint64_t N, uint32_t ldk,
                        hipStream_t stream);

// ---- corpus kernels (fv_corpus.hip) ----------------------------------------------
// All pointers are device memory.
int fv_dev_count_windows(const uint64_t *offsets_dev, uint64_t n_chunks, uint64_t w,
                         uint64_t *out_count_host, hipStream_t stream);
int fv_dev_build_window_starts(const uint64_t *offsets_dev, uint64_t n_chunks, uint64_t w,
                               uint64_t *starts_dev, uint64_t n_windows, hipStream_t stream);
int fv_dev_inverse_frequency(const int32_t *corpus_dev, uint64_t n_tokens, uint64_t vocab,
                             float *invf_dev, int32_t *out_min_host, int32_t *out_max_host,
                             hipStream_t stream);

// ---- wave-level helpers used by the window kernels --------------------------------
// Order-preserving map fp32 -> uint32 (a < b  <=>  key(a) < key(b) for non-NaN a, b).
__device__ __forceinline__ uint32_t fv_ord_key(float f) {
  uint32_t u = __float_as_uint(f);
  return u ^ (uint32_t)(((int32_t)u >> 31) | 0x80000000);
}
__device__ __forceinline__ float fv_ord_unkey(uint32_t k) {
  uint32_t u = (k & 0x80000000u) ? (k ^ 0x80000000u) : ~k;
  return __uint_as_float(u);
}

template <int CTRL>
__device__ __forceinline__ uint32_t fv_dpp(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, CTRL, 0xf, 0xf, false);
}

// Lane patterns that, applied in sequence with an idempotent commutative operator, leave
// the reduction over each 16-lane row in every lane of that row.
#define FV_DPP_QUAD_XOR1 0xB1  // quad_perm [1,0,3,2]
#define FV_DPP_QUAD_XOR2 0x4E  // quad_perm [2,3,0,1]
#define FV_DPP_ROW_ROR4 0x124
#define FV_DPP_ROW_ROR8 0x128

__device__ __forceinline__ uint32_t fv_readlane(uint32_t v, int lane) {
  return (uint32_t)__builtin_amdgcn_readlane((int)v, lane);
}

// Wave-uniform maximum of a 64-bit key over all 64 lanes (all lanes must be active).
__device__ __forceinline__ uint64_t fv_wave_max_u64(uint64_t v) {
#define FV_STEP64(CTRL)                                                 \
  {                                                                     \
    uint32_t lo = fv_dpp<CTRL>((uint32_t)v), hi = fv_dpp<CTRL>((uint32_t)(v >> 32)); \
    uint64_t o = ((uint64_t)hi << 32) | lo;                             \
    v = o > v ? o : v;                                                  \
  }
  FV_STEP64(FV_DPP_QUAD_XOR1)
  FV_STEP64(FV_DPP_QUAD_XOR2)
  FV_STEP64(FV_DPP_ROW_ROR4)
  FV_STEP64(FV_DPP_ROW_ROR8)
#undef FV_STEP64
  uint64_t r = 0;
#pragma unroll
  for (int row = 0; row < 4; ++row) {
    uint64_t x = ((uint64_t)fv_readlane((uint32_t)(v >> 32), row * 16) << 32) |
                 fv_readlane((uint32_t)v, row * 16);
    r = x > r ? x : r;
  }
  return r;
}

__device__ __forceinline__ uint32_t fv_wave_max_u32(uint32_t v) {
  // old = 0 with bound_ctrl: every lane of these patterns has a source, and 0 is the identity of an unsigned
  // maximum, which lets the compiler fold the lane move into the maximum (one instruction per step)
#define FV_STEP32(CTRL)                                                                    \
  {                                                                                        \
    const uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, true); \
    v = o > v ? o : v;                                                                     \
  }
  FV_STEP32(FV_DPP_QUAD_XOR1)
  FV_STEP32(FV_DPP_QUAD_XOR2)
  FV_STEP32(FV_DPP_ROW_ROR4)
  FV_STEP32(FV_DPP_ROW_ROR8)
#undef FV_STEP32
  uint32_t r = 0;
#pragma unroll
  for (int row = 0; row < 4; ++row) {
    uint32_t x = fv_readlane(v, row * 16);
    r = x > r ? x : r;
  }
  return r;
}

__device__ __forceinline__ uint32_t fv_wave_min_u32(uint32_t v) { return ~fv_wave_max_u32(~v); }

// Inclusive prefix sum over the 64 lanes (all must be active) in six DPP additions: shifts by 1, 2,
// 4, 8 inside each row of 16 lanes (a lane without a source adds 0), then the last lane of row 0 / 2
// onto rows 1 / 3, then the last lane of row 1 onto rows 2 and 3. A cross-lane shuffle costs an LDS
// round trip per step; these are ordinary vector instructions.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t fv_dpp_or_zero(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, ROW_MASK, 0xf, true);
}
__device__ __forceinline__ uint32_t fv_wave_inclusive_scan_u32(uint32_t v) {
  v += fv_dpp_or_zero<0x111, 0xf>(v);  // row_shr:1
  v += fv_dpp_or_zero<0x112, 0xf>(v);  // row_shr:2
  v += fv_dpp_or_zero<0x114, 0xf>(v);  // row_shr:4
  v += fv_dpp_or_zero<0x118, 0xf>(v);  // row_shr:8
  v += fv_dpp_or_zero<0x142, 0xa>(v);  // row_bcast:15 into rows 1 and 3
  v += fv_dpp_or_zero<0x143, 0xc>(v);  // row_bcast:31 into rows 2 and 3
  return v;
}
// Sum over the 64 lanes, the same in every lane.
__device__ __forceinline__ uint32_t fv_wave_sum_u32(uint32_t v) {
  return fv_readlane(fv_wave_inclusive_scan_u32(v), 63);
}


// ---- gather-sum of one window, shared by the training and the hashing kernel ----------------
// Lane l holds neurons l, l + 64, ... of the window's activation. acc[j] += W[idx_c][l + 64 j]
// for every window position c in order (idx_c is held by lane c of idx_lane). The allocation
// carries zeros behind its n_cols real rows (fv_matrix_alloc_elems): row n_cols is all zeros and is
// what a position whose index is outside [0, n_cols) reads (adding +0 leaves a sum that started at
// +0 unchanged), and lanes past K read on into what follows, up to fv_matrix_gather_reach, and
// accumulate values nobody uses. So every load is unconditional and no value is selected afterwards: a
// batch of RB rows is RB * NV independent loads in flight per lane with no branch between them,
// and one conversion and one addition per element.
// WEIGHTED: every weight is first multiplied, in fp32, by the weight of its window position --
// l_mid for the centre, whose column lies in the second half of the columns, l_base for the others
// (flyvec/src/cuda_funcs.cu:266-286).
template <int NV, int RB, typename Acc, bool WEIGHTED = false, bool MASK_TAIL = false>
__device__ __forceinline__ void fv_gather_batch(const float *__restrict__ Wt, uint32_t ldk, uint32_t n_cols, int lane,
                                                int c0, int32_t idx_lane, Acc (&acc)[NV], float l_mid = 1.0f,
                                                float l_base = 1.0f, int tail = 64) {
  float v[RB][NV];
  float l[RB];
  const float *rows[RB];
#pragma unroll
  for (int b = 0; b < RB; ++b) {
    const uint32_t i = fv_readlane((uint32_t)idx_lane, c0 + b);
    l[b] = i >= n_cols / 2 ? l_mid : l_base;
    rows[b] = Wt + (uint64_t)(i < n_cols ? i : n_cols) * ldk;  // the same in every lane
#pragma unroll
    for (int j = 0; j < NV - 1; ++j) v[b][j] = rows[b][lane + 64 * j];
    if (MASK_TAIL)
      v[b][NV - 1] = 0.0f;
    else
      v[b][NV - 1] = rows[b][lane + 64 * (NV - 1)];
  }
  // MASK_TAIL: the last register holds neurons in its first `tail` lanes only, and the other lanes stay out of its
  // loads, which then fetch the end of the row and not the start of the next one (3 % on the hashing kernel,
  // nothing on the training kernel, which does without). These loads come last in the batch, so the wait the
  // compiler puts behind the branch is the wait for the batch.
  if (MASK_TAIL && lane < tail) {
#pragma unroll
    for (int b = 0; b < RB; ++b) v[b][NV - 1] = rows[b][lane + 64 * (NV - 1)];
  }
#pragma unroll
  for (int b = 0; b < RB; ++b) {
#pragma unroll
    for (int j = 0; j < NV; ++j) acc[j] = acc[j] + (Acc)(WEIGHTED ? __fmul_rn(v[b][j], l[b]) : v[b][j]);
  }
}

template <int NV, int RB, typename Acc, bool WEIGHTED = false, bool MASK_TAIL = false>
__device__ __forceinline__ void fv_gather_accumulate(const float *__restrict__ Wt, uint32_t ldk, uint32_t K,
                                                     uint32_t n_cols, int lane, int w, int32_t idx_lane,
                                                     Acc (&acc)[NV], float l_mid = 1.0f, float l_base = 1.0f) {
  const int tail = (int)K - 64 * (NV - 1);  // lanes of the last register that hold neurons
  int c0 = 0;
  for (; c0 + RB <= w; c0 += RB)
    fv_gather_batch<NV, RB, Acc, WEIGHTED, MASK_TAIL>(Wt, ldk, n_cols, lane, c0, idx_lane, acc, l_mid, l_base, tail);
  // the rows left over, in batches of 8, 4, 2, 1 rather than one at a time: fewer dependent trips
#define FV_TAIL(R)                                                                                    \
  if (RB > R && (w - c0) >= R) {                                                                      \
    fv_gather_batch<NV, (R < RB ? R : 1), Acc, WEIGHTED, MASK_TAIL>(Wt, ldk, n_cols, lane, c0, idx_lane, acc, l_mid,     \
                                                                    l_base, tail);                                   \
    c0 += R;                                                                                          \
  }
  FV_TAIL(8) FV_TAIL(4) FV_TAIL(2) FV_TAIL(1)
#undef FV_TAIL
}

template <int NV>
struct fv_rows_per_batch {
  static constexpr int value = NV <= 2 ? 16 : NV <= 4 ? 8 : NV <= 8 ? 4 : NV <= 16 ? 2 : 1;
};
