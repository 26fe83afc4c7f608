// Host half of the window sampler, done on the device: window count, window-start table and
// inverse unigram frequency.  Restates flyvec/src/prune_input.cpp:64-122 and
// flyvec/src/model_arrays.cu:396-424 as data-parallel passes:
//   * the running sum of chunk lengths the reference keeps (prune_input.cpp:103-115) telescopes
//     to offsets[s] - offsets[0] (uint64 arithmetic, wrap-around included), so a window start
//     is offsets[s] - offsets[0] + i;
//   * the output slot of a chunk's first window is an exclusive prefix sum of per-chunk window
//     counts (three-pass scan: block totals, scan of totals, rescan + expansion);
//   * the reference counts occurrences in an fp32 accumulator, which stops at 2^24; an integer
//     histogram clamped to 2^24 gives the same value. The counters saturate (at 2^31) instead of wrapping,
//     so a corpus of any length is counted right: the reference indexes its corpus with uint64_t
//     (flyvec/src/model_arrays.cu:396-424) and was run on 5.8 G tokens (flyvec/src/test_inv.cpp:10-11).
#include <atomic>

#include "fv_internal.h"
#include "fv_histogram.h"

#define FV_MAXLEN 214ull  // flyvec/src/prune_input.cpp:7
#define FV_SCAN_THREADS 256
#define FV_SCAN_ITEMS 8
#define FV_SCAN_TILE (FV_SCAN_THREADS * FV_SCAN_ITEMS)

__device__ __forceinline__ uint64_t fv_chunk_windows(const uint64_t *__restrict__ off, uint64_t s,
                                                     uint64_t n_chunks, uint64_t w) {
  if (s >= n_chunks) return 0;
  uint64_t len = off[s + 1] - off[s];
  return (len >= w && len < FV_MAXLEN) ? len - w + 1 : 0;
}

__device__ __forceinline__ uint64_t fv_block_sum_u64(uint64_t v, uint64_t *smem /*4*/) {
  for (int d = 32; d >= 1; d >>= 1) v += __shfl_down(v, d, 64);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  __syncthreads();
  if (lane == 0) smem[wave] = v;
  __syncthreads();
  return smem[0] + smem[1] + smem[2] + smem[3];
}

// Pass 1: total number of windows of each tile of FV_SCAN_TILE chunks.
__global__ __launch_bounds__(FV_SCAN_THREADS) void fv_tile_totals_kernel(
    const uint64_t *__restrict__ off, uint64_t n_chunks, uint64_t w, uint64_t *__restrict__ totals) {
  __shared__ uint64_t smem[4];
  const uint64_t base = (uint64_t)blockIdx.x * FV_SCAN_TILE + (uint64_t)threadIdx.x * FV_SCAN_ITEMS;
  uint64_t v = 0;
#pragma unroll
  for (int j = 0; j < FV_SCAN_ITEMS; ++j) v += fv_chunk_windows(off, base + j, n_chunks, w);
  uint64_t t = fv_block_sum_u64(v, smem);
  if (threadIdx.x == 0) totals[blockIdx.x] = t;
}

// Pass 2: exclusive scan of the tile totals by one block; totals[n_tiles] receives the sum.
__global__ __launch_bounds__(FV_SCAN_THREADS) void fv_scan_totals_kernel(uint64_t *totals,
                                                                         uint64_t n_tiles) {
  __shared__ uint64_t part[FV_SCAN_THREADS];
  __shared__ uint64_t carry;
  if (threadIdx.x == 0) carry = 0;
  __syncthreads();
  for (uint64_t b0 = 0; b0 < n_tiles; b0 += FV_SCAN_THREADS) {
    uint64_t i = b0 + threadIdx.x;
    uint64_t v = i < n_tiles ? totals[i] : 0;
    part[threadIdx.x] = v;
    __syncthreads();
    for (int d = 1; d < FV_SCAN_THREADS; d <<= 1) {  // Hillis-Steele inclusive scan
      uint64_t add = threadIdx.x >= (unsigned)d ? part[threadIdx.x - d] : 0;
      __syncthreads();
      part[threadIdx.x] += add;
      __syncthreads();
    }
    uint64_t incl = part[threadIdx.x];
    uint64_t c = carry;
    if (i < n_tiles) totals[i] = c + incl - v;
    __syncthreads();
    if (threadIdx.x == FV_SCAN_THREADS - 1) carry = c + incl;
    __syncthreads();
  }
  if (threadIdx.x == 0) totals[n_tiles] = carry;
}

// Pass 3: each thread rescans its FV_SCAN_ITEMS chunks and writes their window starts.
__global__ __launch_bounds__(FV_SCAN_THREADS) void fv_expand_starts_kernel(
    const uint64_t *__restrict__ off, uint64_t n_chunks, uint64_t w,
    const uint64_t *__restrict__ tile_base, uint64_t *__restrict__ starts, uint64_t n_windows) {
  __shared__ uint64_t part[FV_SCAN_THREADS];
  const uint64_t base = (uint64_t)blockIdx.x * FV_SCAN_TILE + (uint64_t)threadIdx.x * FV_SCAN_ITEMS;
  uint64_t cnt[FV_SCAN_ITEMS];
  uint64_t mine = 0;
#pragma unroll
  for (int j = 0; j < FV_SCAN_ITEMS; ++j) {
    cnt[j] = fv_chunk_windows(off, base + j, n_chunks, w);
    mine += cnt[j];
  }
  part[threadIdx.x] = mine;
  __syncthreads();
  for (int d = 1; d < FV_SCAN_THREADS; d <<= 1) {
    uint64_t add = threadIdx.x >= (unsigned)d ? part[threadIdx.x - d] : 0;
    __syncthreads();
    part[threadIdx.x] += add;
    __syncthreads();
  }
  uint64_t out = tile_base[blockIdx.x] + part[threadIdx.x] - mine;
  const uint64_t off0 = off[0];
#pragma unroll
  for (int j = 0; j < FV_SCAN_ITEMS; ++j) {
    if (cnt[j]) {
      uint64_t first = off[base + j] - off0;
      for (uint64_t i = 0; i < cnt[j]; ++i)
        if (out + i < n_windows) starts[out + i] = first + i;
      out += cnt[j];
    }
  }
}

static int fv_scan_windows(const uint64_t *offsets_dev, uint64_t n_chunks, uint64_t w,
                           uint64_t **out_tile_base, uint64_t *out_total, hipStream_t stream) {
  const uint64_t n_tiles = (n_chunks + FV_SCAN_TILE - 1) / FV_SCAN_TILE;
  FV_REQUIRE(n_tiles < (1ull << 31), FV_ERR_INVALID, "too many chunks (%llu)",
             (unsigned long long)n_chunks);
  uint64_t *totals = nullptr;
  FV_HIP(hipMalloc((void **)&totals, (n_tiles + 1) * sizeof(uint64_t)));
  if (n_tiles)
    hipLaunchKernelGGL(fv_tile_totals_kernel, dim3((unsigned)n_tiles), dim3(FV_SCAN_THREADS), 0,
                       stream, offsets_dev, n_chunks, w, totals);
  hipLaunchKernelGGL(fv_scan_totals_kernel, dim3(1), dim3(FV_SCAN_THREADS), 0, stream, totals,
                     n_tiles);
  hipError_t e = hipGetLastError();
  if (e == hipSuccess)
    e = hipMemcpyAsync(out_total, totals + n_tiles, sizeof(uint64_t), hipMemcpyDeviceToHost, stream);
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  if (e != hipSuccess) {
    (void)hipFree(totals);
    return fv_fail(FV_ERR_HIP, "window scan failed: %s", hipGetErrorString(e));
  }
  if (out_tile_base)
    *out_tile_base = totals;
  else
    (void)hipFree(totals);
  return FV_OK;
}

int fv_dev_count_windows(const uint64_t *offsets_dev, uint64_t n_chunks, uint64_t w,
                         uint64_t *out_count_host, hipStream_t stream) {
  return fv_scan_windows(offsets_dev, n_chunks, w, nullptr, out_count_host, stream);
}

int fv_dev_build_window_starts(const uint64_t *offsets_dev, uint64_t n_chunks, uint64_t w,
                               uint64_t *starts_dev, uint64_t n_windows, hipStream_t stream) {
  uint64_t *tile_base = nullptr;
  uint64_t total = 0;
  FV_TRY(fv_scan_windows(offsets_dev, n_chunks, w, &tile_base, &total, stream));
  int rc = FV_OK;
  if (total != n_windows) {
    rc = fv_fail(FV_ERR_INVALID, "window table capacity %llu does not match the %llu windows found",
                 (unsigned long long)n_windows, (unsigned long long)total);
  } else if (n_chunks) {
    const uint64_t n_tiles = (n_chunks + FV_SCAN_TILE - 1) / FV_SCAN_TILE;
    hipLaunchKernelGGL(fv_expand_starts_kernel, dim3((unsigned)n_tiles), dim3(FV_SCAN_THREADS), 0,
                       stream, offsets_dev, n_chunks, w, tile_base, starts_dev, n_windows);
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) e = hipStreamSynchronize(stream);
    if (e != hipSuccess) rc = fv_fail(FV_ERR_HIP, "window expansion failed: %s", hipGetErrorString(e));
  }
  (void)hipFree(tile_base);
  return rc;
}

// ---- inverse unigram frequency ---------------------------------------------------------
#define FV_HIST_LDS 12288  // ids below this are counted in LDS first (Zipf head), the rest in HBM

// counts[i] = min(counts[i] + add, FV_HIST_SATURATED), whatever the other blocks add meanwhile
__device__ __forceinline__ void fv_saturating_add(uint32_t *counter, uint32_t add) {
  uint32_t seen = *counter;
  for (;;) {
    const uint32_t want = fv_hist_saturated_sum(seen, add);
    if (want == seen) return;
    const uint32_t old = atomicCAS(counter, seen, want);
    if (old == seen) return;
    seen = old;
  }
}

// STOPS: the counters in HBM stop at FV_HIST_SATURATED instead of wrapping, for a corpus long enough that one could
// get there; the block's additions are then compare-and-swap loops, which under the contention of 2048 blocks on the
// same few thousand counters take some 10 ms in all, against 0.2 ms for the plain additions of the other form.
template <bool STOPS>
__global__ __launch_bounds__(256) void fv_histogram_kernel(const int32_t *__restrict__ corpus,
                                                           uint64_t n_tokens, uint32_t vocab,
                                                           uint32_t *__restrict__ counts,
                                                           int32_t *__restrict__ minmax) {
  __shared__ uint32_t hist[FV_HIST_LDS];
  for (int i = threadIdx.x; i < FV_HIST_LDS; i += 256) hist[i] = 0;
  __syncthreads();
  int32_t lo = 0x7fffffff, hi = -0x7fffffff - 1;
  const uint64_t stride = (uint64_t)gridDim.x * 256;
  for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n_tokens; i += stride) {
    int32_t t = corpus[i];
    lo = t < lo ? t : lo;
    hi = t > hi ? t : hi;
    if (t >= 0 && (uint32_t)t < vocab) {
      if (t < FV_HIST_LDS) {
        atomicAdd(&hist[t], 1u);
      } else if (!STOPS) {
        atomicAdd(&counts[t], 1u);
      } else if (atomicAdd(&counts[t], 1u) >= FV_HIST_SATURATED + (1u << 30)) {
        // far beyond the stop: back to it. Every thread that sees this writes the same value, and between the
        // stop and the wrap lie 2^30 more additions than there are threads in flight.
        atomicExch(&counts[t], FV_HIST_SATURATED);
      }
    }
  }
  __syncthreads();
  const uint32_t lim = vocab < FV_HIST_LDS ? vocab : FV_HIST_LDS;
  for (uint32_t i = threadIdx.x; i < lim; i += 256)
    if (hist[i]) {
      if (STOPS)
        fv_saturating_add(&counts[i], hist[i]);
      else
        atomicAdd(&counts[i], hist[i]);
    }
  for (int d = 32; d >= 1; d >>= 1) {
    int32_t ol = __shfl_down(lo, d, 64), oh = __shfl_down(hi, d, 64);
    lo = ol < lo ? ol : lo;
    hi = oh > hi ? oh : hi;
  }
  if ((threadIdx.x & 63) == 0 && lo <= hi) {
    atomicMin(&minmax[0], lo);
    atomicMax(&minmax[1], hi);
  }
}

// A corpus shorter than the stop cannot bring a counter there: plain additions. fv_histogram_stops_from (a test
// hook) lowers the length from which the other form is taken.
static std::atomic<uint64_t> fv_hist_stops_from{FV_HIST_SATURATED};

extern "C" int fv_histogram_stops_from(uint64_t n_tokens) {
  fv_hist_stops_from.store(n_tokens ? n_tokens : (uint64_t)FV_HIST_SATURATED);
  return FV_OK;
}

static void fv_launch_histogram(unsigned blocks, hipStream_t stream, const int32_t *corpus_dev, uint64_t n_tokens,
                                uint32_t vocab, uint32_t *counts, int32_t *minmax) {
  if (n_tokens >= fv_hist_stops_from.load())
    hipLaunchKernelGGL(fv_histogram_kernel<true>, dim3(blocks), dim3(256), 0, stream, corpus_dev, n_tokens, vocab, counts,
                       minmax);
  else
    hipLaunchKernelGGL(fv_histogram_kernel<false>, dim3(blocks), dim3(256), 0, stream, corpus_dev, n_tokens, vocab, counts,
                       minmax);
}

__global__ void fv_invert_counts_kernel(const uint32_t *__restrict__ counts, uint32_t vocab,
                                        float *__restrict__ invf) {
  uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= vocab) return;
  invf[i] = fv_hist_invert(counts[i]);
}

int fv_dev_inverse_frequency(const int32_t *corpus_dev, uint64_t n_tokens, uint64_t vocab,
                             float *invf_dev, int32_t *out_min_host, int32_t *out_max_host,
                             hipStream_t stream) {
  FV_REQUIRE(vocab > 0 && vocab < (1ull << 30), FV_ERR_INVALID, "vocabulary size %llu out of range",
             (unsigned long long)vocab);
  FV_REQUIRE(n_tokens < FV_HIST_MAX_TOKENS, FV_ERR_INVALID, "corpus of %llu tokens exceeds 2^42",
             (unsigned long long)n_tokens);
  uint32_t *counts = nullptr;
  FV_HIP(hipMalloc((void **)&counts, vocab * sizeof(uint32_t) + 2 * sizeof(int32_t)));
  int32_t *minmax = (int32_t *)(counts + vocab);
  int32_t init[2] = {0x7fffffff, -0x7fffffff - 1};
  hipError_t e = hipMemsetAsync(counts, 0, vocab * sizeof(uint32_t), stream);
  if (e == hipSuccess)
    e = hipMemcpyAsync(minmax, init, sizeof init, hipMemcpyHostToDevice, stream);
  if (e == hipSuccess && n_tokens) {
    const unsigned blocks = fv_hist_blocks(n_tokens);
    fv_launch_histogram(blocks, stream, corpus_dev, n_tokens, (uint32_t)vocab, counts, minmax);
    e = hipGetLastError();
  }
  if (e == hipSuccess) {
    hipLaunchKernelGGL(fv_invert_counts_kernel, dim3((unsigned)((vocab + 255) / 256)), dim3(256), 0,
                       stream, counts, (uint32_t)vocab, invf_dev);
    e = hipGetLastError();
  }
  int32_t mm[2] = {0, 0};
  if (e == hipSuccess) e = hipMemcpyAsync(mm, minmax, sizeof mm, hipMemcpyDeviceToHost, stream);
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  (void)hipFree(counts);
  if (e != hipSuccess) return fv_fail(FV_ERR_HIP, "inverse frequency failed: %s", hipGetErrorString(e));
  if (out_min_host) *out_min_host = mm[0];
  if (out_max_host) *out_max_host = mm[1];
  return FV_OK;
}

// ---- C ABI on host buffers ---------------------------------------------------------------

static int fv_upload_offsets(const uint64_t *offsets, uint64_t n_chunks, uint64_t **out_dev) {
  FV_HIP(hipMalloc((void **)out_dev, (n_chunks + 1) * sizeof(uint64_t)));
  hipError_t e = hipMemcpy(*out_dev, offsets, (n_chunks + 1) * sizeof(uint64_t), hipMemcpyHostToDevice);
  if (e != hipSuccess) {
    (void)hipFree(*out_dev);
    *out_dev = nullptr;
    return fv_fail(FV_ERR_HIP, "offset upload failed: %s", hipGetErrorString(e));
  }
  return FV_OK;
}

extern "C" int fv_count_windows(const uint64_t *offsets, uint64_t n_chunks, uint64_t w,
                                uint64_t *out_count) {
  FV_REQUIRE(out_count, FV_ERR_INVALID, "fv_count_windows: null output");
  *out_count = 0;
  if (n_chunks == 0) return FV_OK;
  FV_REQUIRE(offsets, FV_ERR_INVALID, "fv_count_windows: null offsets");
  FV_REQUIRE(w >= 1, FV_ERR_INVALID, "fv_count_windows: window length must be >= 1");
  uint64_t *d = nullptr;
  FV_TRY(fv_upload_offsets(offsets, n_chunks, &d));
  int rc = fv_dev_count_windows(d, n_chunks, w, out_count, 0);
  (void)hipFree(d);
  return rc;
}

extern "C" int fv_build_window_starts(const uint64_t *offsets, uint64_t n_chunks, uint64_t w,
                                      uint64_t *out_starts, uint64_t capacity) {
  if (n_chunks == 0) return FV_OK;
  FV_REQUIRE(offsets, FV_ERR_INVALID, "fv_build_window_starts: null offsets");
  FV_REQUIRE(w >= 1, FV_ERR_INVALID, "fv_build_window_starts: window length must be >= 1");
  uint64_t *d = nullptr, *s = nullptr;
  FV_TRY(fv_upload_offsets(offsets, n_chunks, &d));
  uint64_t total = 0;
  int rc = fv_dev_count_windows(d, n_chunks, w, &total, 0);
  if (rc == FV_OK && total > capacity)
    rc = fv_fail(FV_ERR_INVALID, "fv_build_window_starts: %llu windows do not fit capacity %llu",
                 (unsigned long long)total, (unsigned long long)capacity);
  if (rc == FV_OK && total) {
    FV_REQUIRE(out_starts, FV_ERR_INVALID, "fv_build_window_starts: null output");
    hipError_t e = hipMalloc((void **)&s, total * sizeof(uint64_t));
    if (e != hipSuccess) rc = fv_fail(FV_ERR_HIP, "hipMalloc failed: %s", hipGetErrorString(e));
    if (rc == FV_OK) rc = fv_dev_build_window_starts(d, n_chunks, w, s, total, 0);
    if (rc == FV_OK) {
      e = hipMemcpy(out_starts, s, total * sizeof(uint64_t), hipMemcpyDeviceToHost);
      if (e != hipSuccess) rc = fv_fail(FV_ERR_HIP, "download failed: %s", hipGetErrorString(e));
    }
  }
  (void)hipFree(d);
  (void)hipFree(s);
  return rc;
}

extern "C" int fv_inverse_frequency(const int32_t *corpus, uint64_t n_tokens, uint64_t vocab,
                                    float *out_invf) {
  FV_REQUIRE(out_invf, FV_ERR_INVALID, "fv_inverse_frequency: null output");
  FV_REQUIRE(corpus || n_tokens == 0, FV_ERR_INVALID, "fv_inverse_frequency: null corpus");
  int32_t *dc = nullptr;
  float *df = nullptr;
  FV_HIP(hipMalloc((void **)&df, vocab * sizeof(float)));
  int rc = FV_OK;
  hipError_t e = hipSuccess;
  if (n_tokens) {
    e = hipMalloc((void **)&dc, n_tokens * sizeof(int32_t));
    if (e == hipSuccess) e = hipMemcpy(dc, corpus, n_tokens * sizeof(int32_t), hipMemcpyHostToDevice);
    if (e != hipSuccess) rc = fv_fail(FV_ERR_HIP, "corpus upload failed: %s", hipGetErrorString(e));
  }
  int32_t lo = 0, hi = 0;
  if (rc == FV_OK) rc = fv_dev_inverse_frequency(dc, n_tokens, vocab, df, &lo, &hi, 0);
  if (rc == FV_OK && n_tokens && hi >= 0 && (uint64_t)hi >= vocab)
    rc = fv_fail(FV_ERR_DATA, "token id %d is outside the vocabulary of %llu", hi,
                 (unsigned long long)vocab);
  if (rc == FV_OK) {
    e = hipMemcpy(out_invf, df, vocab * sizeof(float), hipMemcpyDeviceToHost);
    if (e != hipSuccess) rc = fv_fail(FV_ERR_HIP, "download failed: %s", hipGetErrorString(e));
  }
  (void)hipFree(dc);
  (void)hipFree(df);
  return rc;
}

// ---- inverse unigram frequency without any allocation -------------------------------------------------
// For callers that cannot allocate device memory (tight serving loops, harnesses that forbid hipMalloc,
// a process whose memory is all spoken for): the occurrence counters and the id range live in a file-scope
// device array instead of a buffer from hipMalloc. The call itself runs on the null stream and ends with a
// blocking copy of the id range to the host, so it cannot be captured into a graph as it is. Every device the library runs on holds its own
// copy of the array, at its own address, until the process ends; host code reaches it only through
// the address hipGetSymbolAddress returns for the device that is current.
#define FV_STATIC_MAX_VOCAB (1u << 20)  // counters of the array: 4 MiB
#define FV_STATIC_MAX_DEVICES 64

static __device__ __align__(256) uint32_t fv_static_scratch[FV_STATIC_MAX_VOCAB + 64];  // counters, then {min, max} of the ids
static uint32_t *fv_static_scratch_addr[FV_STATIC_MAX_DEVICES];  // per device, filled on first use

// The array's address on the current device.
static int fv_static_scratch_on_device(uint32_t **out) {
  int dev = -1;
  FV_HIP(hipGetDevice(&dev));
  FV_REQUIRE(dev >= 0 && dev < FV_STATIC_MAX_DEVICES, FV_ERR_INVALID, "device %d is beyond the %d this entry point serves",
             dev, FV_STATIC_MAX_DEVICES);
  if (!fv_static_scratch_addr[dev]) {
    void *p = nullptr;
    FV_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(fv_static_scratch)));
    FV_REQUIRE(p, FV_ERR_HIP, "hipGetSymbolAddress returned no address for the scratch array");
    fv_static_scratch_addr[dev] = (uint32_t *)p;
  }
  *out = fv_static_scratch_addr[dev];
  return FV_OK;
}

// counters[0 .. vocab) = 0 and the id range to (INT_MAX, INT_MIN), by a kernel.
__global__ __launch_bounds__(256) void fv_static_clear_kernel(uint32_t *__restrict__ counts, uint32_t vocab,
                                                              int32_t *__restrict__ minmax) {
  for (uint32_t i = blockIdx.x * 256 + threadIdx.x; i < vocab; i += gridDim.x * 256) counts[i] = 0;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    minmax[0] = 0x7fffffff;
    minmax[1] = -0x7fffffff - 1;
  }
}

extern "C" int fv_inverse_frequency_static(const int32_t *corpus_dev, uint64_t n_tokens, uint64_t vocab,
                                           float *out_invf_dev) {
  FV_REQUIRE(out_invf_dev, FV_ERR_INVALID, "fv_inverse_frequency_static: null output");
  FV_REQUIRE(corpus_dev || n_tokens == 0, FV_ERR_INVALID, "fv_inverse_frequency_static: null corpus");
  FV_REQUIRE(vocab >= 1 && vocab <= FV_STATIC_MAX_VOCAB, FV_ERR_INVALID,
             "fv_inverse_frequency_static: vocabulary of %llu ids; the built-in scratch array holds counters for at "
             "most %u (use fv_inverse_frequency, which allocates)",
             (unsigned long long)vocab, FV_STATIC_MAX_VOCAB);
  FV_REQUIRE(n_tokens < FV_HIST_MAX_TOKENS, FV_ERR_INVALID, "fv_inverse_frequency_static: corpus of %llu tokens exceeds 2^42",
             (unsigned long long)n_tokens);
  uint32_t *counts = nullptr;
  FV_TRY(fv_static_scratch_on_device(&counts));
  int32_t *minmax = (int32_t *)(counts + FV_STATIC_MAX_VOCAB);
  hipStream_t stream = 0;
  // the array keeps the last call's counts: clear what this call uses
  const unsigned clear_blocks = (unsigned)((vocab + 255) / 256 < 1024 ? (vocab + 255) / 256 : 1024);
  hipLaunchKernelGGL(fv_static_clear_kernel, dim3(clear_blocks), dim3(256), 0, stream, counts, (uint32_t)vocab, minmax);
  if (n_tokens) {
    const unsigned blocks = fv_hist_blocks(n_tokens);
    fv_launch_histogram(blocks, stream, corpus_dev, n_tokens, (uint32_t)vocab, counts, minmax);
  }
  hipLaunchKernelGGL(fv_invert_counts_kernel, dim3((unsigned)((vocab + 255) / 256)), dim3(256), 0, stream, counts,
                     (uint32_t)vocab, out_invf_dev);
  FV_HIP(hipGetLastError());
  int32_t mm[2] = {0, 0};
  FV_HIP(hipMemcpy(mm, minmax, sizeof mm, hipMemcpyDeviceToHost));  // waits for the kernels above
  if (n_tokens && mm[1] >= 0 && (uint64_t)mm[1] >= vocab)
    return fv_fail(FV_ERR_DATA, "token id %d is outside the vocabulary of %llu", mm[1], (unsigned long long)vocab);
  return FV_OK;
}

// ---- masking of token ids ---------------------------------------------------------------------------
// The reference removes stop words from an encoded corpus off line, one pass over the whole corpus
// per id (flyvec/src/remove_words.cpp:28-37: data[w] == id ? -1). Here a bit per vocabulary id
// marks the ids to remove and one pass rewrites the corpus, a part of bounded size at a time so that a
// corpus larger than the device's free memory streams through.

__global__ __launch_bounds__(256) void fv_mark_ids_kernel(const int32_t *__restrict__ remove, uint64_t n_remove,
                                                          uint64_t vocab, uint32_t *__restrict__ bits) {
  for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n_remove; i += (uint64_t)gridDim.x * 256) {
    const int32_t id = remove[i];
    if (id >= 0 && (uint64_t)id < vocab) atomicOr(&bits[id >> 5], 1u << (id & 31));
  }
}

__global__ __launch_bounds__(256) void fv_mask_tokens_kernel(int32_t *__restrict__ tokens, uint64_t n,
                                                             const uint32_t *__restrict__ bits, uint64_t vocab) {
  for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (uint64_t)gridDim.x * 256) {
    const int32_t t = tokens[i];
    if (t >= 0 && (uint64_t)t < vocab && ((bits[t >> 5] >> (t & 31)) & 1u)) tokens[i] = -1;
  }
}

#define FV_MASK_PART (64ull << 20)  // tokens per part (256 MB)

extern "C" int fv_mask_tokens(int32_t *tokens, uint64_t n_tokens, const int32_t *remove_ids, uint64_t n_remove,
                              uint64_t vocab) {
  FV_REQUIRE(tokens || n_tokens == 0, FV_ERR_INVALID, "fv_mask_tokens: null corpus");
  FV_REQUIRE(remove_ids || n_remove == 0, FV_ERR_INVALID, "fv_mask_tokens: null id list");
  FV_REQUIRE(vocab >= 1 && vocab <= (1ull << 31), FV_ERR_INVALID, "fv_mask_tokens: vocabulary of %llu ids",
             (unsigned long long)vocab);
  if (n_tokens == 0 || n_remove == 0) return FV_OK;
  for (uint64_t i = 0; i < n_remove; ++i)
    FV_REQUIRE(remove_ids[i] >= 0 && (uint64_t)remove_ids[i] < vocab, FV_ERR_DATA,
               "fv_mask_tokens: id %d is outside the vocabulary of %llu", remove_ids[i], (unsigned long long)vocab);
  const uint64_t words = (vocab + 31) / 32;
  const uint64_t part = n_tokens < FV_MASK_PART ? n_tokens : FV_MASK_PART;
  uint32_t *bits = nullptr;
  int32_t *rem = nullptr, *buf = nullptr;
  hipError_t e = hipMalloc((void **)&bits, words * sizeof(uint32_t));
  if (e == hipSuccess) e = hipMalloc((void **)&rem, n_remove * sizeof(int32_t));
  if (e == hipSuccess) e = hipMalloc((void **)&buf, part * sizeof(int32_t));
  if (e == hipSuccess) e = hipMemset(bits, 0, words * sizeof(uint32_t));
  if (e == hipSuccess) e = hipMemcpy(rem, remove_ids, n_remove * sizeof(int32_t), hipMemcpyHostToDevice);
  if (e == hipSuccess) {
    const unsigned blocks = (unsigned)((n_remove + 255) / 256 < 1024 ? (n_remove + 255) / 256 : 1024);
    hipLaunchKernelGGL(fv_mark_ids_kernel, dim3(blocks), dim3(256), 0, 0, rem, n_remove, vocab, bits);
    e = hipGetLastError();
  }
  for (uint64_t first = 0; e == hipSuccess && first < n_tokens; first += part) {
    const uint64_t n = n_tokens - first < part ? n_tokens - first : part;
    e = hipMemcpy(buf, tokens + first, n * sizeof(int32_t), hipMemcpyHostToDevice);
    if (e != hipSuccess) break;
    const unsigned blocks = (unsigned)((n + 255) / 256 < 8192 ? (n + 255) / 256 : 8192);
    hipLaunchKernelGGL(fv_mask_tokens_kernel, dim3(blocks), dim3(256), 0, 0, buf, n, bits, vocab);
    e = hipGetLastError();
    if (e == hipSuccess) e = hipMemcpy(tokens + first, buf, n * sizeof(int32_t), hipMemcpyDeviceToHost);
  }
  (void)hipFree(bits);
  (void)hipFree(rem);
  (void)hipFree(buf);
  if (e != hipSuccess) return fv_fail(FV_ERR_HIP, "fv_mask_tokens failed: %s", hipGetErrorString(e));
  return FV_OK;
}

// ---- in-window duplicate pruning of a window matrix (an off-line tool of the reference) ---------------

// One wavefront per row, lane c holds the value of column c. flyvec/src/prune_input.cpp:14-60 scans a
// row left to right and replaces a value already kept at an earlier position by -1; the centre column
// takes no part (it counts as -1 during the scan) and keeps its value. A first occurrence is always
// kept, so: a column other than the centre loses its value if an earlier column other than the centre
// holds the same one.
__global__ __launch_bounds__(256) void fv_prune_windows_kernel(int32_t *__restrict__ data, uint64_t rows,
                                                               uint32_t cols) {
  const int lane = threadIdx.x & 63;
  const int mid = (int)(cols / 2);
  for (uint64_t r = (uint64_t)blockIdx.x * 4 + (threadIdx.x >> 6); r < rows; r += (uint64_t)gridDim.x * 4) {
    const int32_t val = lane < (int)cols ? data[r * cols + lane] : -1;
    bool dup = false;
    for (int j = 0; j + 1 < (int)cols; ++j) {
      const int32_t earlier = (int32_t)fv_readlane((uint32_t)val, j);
      dup = dup || (lane > j && j != mid && earlier == val);
    }
    if (lane < (int)cols && lane != mid && dup) data[r * cols + lane] = -1;
  }
}

#define FV_PRUNE_PART (1ull << 26)  // matrix entries per trip through the device

extern "C" int fv_prune_windows(int32_t *data, uint64_t rows, uint64_t cols) {
  FV_REQUIRE(data || rows == 0 || cols == 0, FV_ERR_INVALID, "fv_prune_windows: null matrix");
  FV_REQUIRE(cols <= FV_MAX_WINDOW, FV_ERR_INVALID, "fv_prune_windows: %llu columns, at most %d are supported",
             (unsigned long long)cols, FV_MAX_WINDOW);
  if (rows == 0 || cols <= 1) return FV_OK;
  const uint64_t part_rows = FV_PRUNE_PART / cols < rows ? FV_PRUNE_PART / cols : rows;
  int32_t *buf = nullptr;
  hipError_t e = hipMalloc((void **)&buf, part_rows * cols * sizeof(int32_t));
  for (uint64_t first = 0; e == hipSuccess && first < rows; first += part_rows) {
    const uint64_t n = rows - first < part_rows ? rows - first : part_rows;
    e = hipMemcpy(buf, data + first * cols, n * cols * sizeof(int32_t), hipMemcpyHostToDevice);
    if (e != hipSuccess) break;
    const unsigned blocks = (unsigned)((n + 3) / 4 < 16384 ? (n + 3) / 4 : 16384);
    hipLaunchKernelGGL(fv_prune_windows_kernel, dim3(blocks), dim3(256), 0, 0, buf, n, (uint32_t)cols);
    e = hipGetLastError();
    if (e == hipSuccess) e = hipMemcpy(data + first * cols, buf, n * cols * sizeof(int32_t), hipMemcpyDeviceToHost);
  }
  (void)hipFree(buf);
  if (e != hipSuccess) return fv_fail(FV_ERR_HIP, "fv_prune_windows failed: %s", hipGetErrorString(e));
  return FV_OK;
}
