// Batched top-k hashing: FlyVec.get_sparse_embedding (flyvec/core.py:139-163) for many target
// ids or many context windows at once.
//
// One wavefront per window.  The activation (fp32 sum of the window's token rows, in window
// order) lives in registers, neuron h = lane + 64 j in register j of its lane.  The reference
// sorts all K activations (core.py:155) but only uses the k-th and (k+1)-th largest:
//     thr = fl32(a[k-1] + a[k]) / 2;  code = act > thr            (core.py:157-158)
// so the kernel selects instead of sorting: a bit-by-bit search from the most significant bit of
// an order-preserving integer key finds the largest threshold with at least k keys at or above
// it; each probe is one compare per register and a population count of the resulting lane mask.
// The search stops as soon as exactly k keys pass (the top-k set is then known; its minimum and
// the maximum of the rest are the two order statistics) and otherwise ends on the exact k-th key,
// with ties at the boundary counted with multiplicity as the sort does.  A compare's lane mask is
// also exactly one 64-bit word of the packed code, so bit packing costs nothing.
#include <math.h>
#include <string.h>

#include <atomic>
#include <memory>
#include <thread>
#include <vector>

#include "fv_internal.h"

// Host-buffer batches go through the device in chunks on two streams of equal priority, so that one
// chunk's copies run while the other's kernel does: per stream a device buffer for the chunk's indices and
// one for each kind of output, kept from call to call (grown when a call needs more).
#define FV_HASH_LANES 2
#define FV_HASH_CHUNK (1u << 17)  // windows per chunk

struct fv_hash_lane {
  hipStream_t stream;
  int32_t *idx;
  uint64_t *bits;
  int8_t *codes;
  size_t idx_cap, bits_cap, codes_cap;  // bytes
  // page-locked staging for outputs that go to pageable host memory, and the event behind a chunk's copies
  char *stage_bits, *stage_codes;
  size_t stage_bits_cap, stage_codes_cap;
  hipEvent_t done;
};

struct fv_hasher {
  uint32_t K, ldk;
  uint64_t N;
  hipStream_t stream;
  float *Wt;
  uint32_t *err;  // device flag: a column index outside [-1, N) was met
  unsigned max_blocks;
  fv_hash_lane lane[FV_HASH_LANES];  // lane 0 runs on `stream`
};

struct fv_hash_args {
  const float *Wt;
  const int32_t *idx;
  uint64_t n;
  uint32_t w, k, K, ldk, n_cols;
  int32_t shift;  // added to every index (V for target ids, 0 for window columns)
  uint64_t *out_bits;
  int8_t *out_codes;
  uint32_t *err;
};

template <int NV>
__global__ __launch_bounds__(256) void fv_hash_kernel(fv_hash_args a) {
  const int lane = threadIdx.x & 63;
  const uint64_t n_waves = (uint64_t)gridDim.x * 4;
  const uint64_t r_first = (uint64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  // a window's ids are fetched one window ahead: the load is on its way while the rows of the window before are
  // gathered, and the wave's chain of dependent trips is one shorter per window
  int32_t raw_ahead = -1;
  if (r_first < a.n && lane < (int)a.w) raw_ahead = a.idx[r_first * a.w + lane];
  for (uint64_t r = r_first; r < a.n; r += n_waves) {
    int32_t idx = -1;
    const int32_t raw = raw_ahead;
    if (r + n_waves < a.n && lane < (int)a.w) raw_ahead = a.idx[(r + n_waves) * a.w + lane];
    if (lane < (int)a.w) {
      if (raw != -1 || a.shift != 0) {
        const int64_t col = (int64_t)raw + a.shift;
        if (raw >= 0 && col < (int64_t)a.n_cols)
          idx = (int32_t)col;
        else
          atomicOr(a.err, 1u);
      }
    }

    float acc[NV];
#pragma unroll
    for (int j = 0; j < NV; ++j) acc[j] = 0.0f;
    fv_gather_accumulate<NV, fv_rows_per_batch<NV>::value, float, false, true>(a.Wt, a.ldk, a.K, a.n_cols, lane, (int)a.w,
                                                                               idx, acc);

    uint32_t key[NV];
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const bool valid = (j < NV - 1) || (uint32_t)(lane + 64 * j) < a.K;
      key[j] = valid ? fv_ord_key(acc[j]) : 0u;  // pads sort below every real value
    }

    // largest cand with count(key >= cand) >= k, built from the top bit down. The sign and exponent bits are
    // usually settled in two steps instead of nine: the largest key M bounds cand from above, so if at least
    // k keys reach the start t of M's binade, cand lies in [t, t + 2^23) -- nothing reaches t + 2^23 -- and only
    // its mantissa bits are open; else the binade below is tried, where the count at t + 2^23 is known to be
    // short of k. Past three binades of positive values the search runs over all 32 bits.
    uint32_t cand = 0, c_at = 0;
    int bit = 31;
    {
      uint32_t m = key[0];
#pragma unroll
      for (int j = 1; j < NV; ++j) m = max(m, key[j]);
      // (the maximum is the same in every lane: said to the compiler, so that the search runs on scalar registers)
      uint32_t t = (uint32_t)__builtin_amdgcn_readfirstlane((int)fv_wave_max_u32(m)) & 0xff800000u;
      for (int tries = 0; tries < 3 && t > 0x80000000u; ++tries, t -= 0x00800000u) {  // keys of positive floats
        uint32_t c = 0;
#pragma unroll
        for (int j = 0; j < NV; ++j) c += (uint32_t)__popcll(__ballot(key[j] >= t));
        if (c >= a.k) {
          cand = t;
          c_at = c;
          bit = c == a.k ? -1 : 22;
          break;
        }
      }
    }
    while (bit >= 0) {
      // the threshold, the count and the decision are the same in every lane: kept in scalar registers
      const uint32_t t = (uint32_t)__builtin_amdgcn_readfirstlane((int)(cand | (1u << bit)));
      uint32_t c = 0;
#pragma unroll
      for (int j = 0; j < NV; ++j) c += (uint32_t)__popcll(__ballot(key[j] >= t));
      const bool take = c >= a.k;
      cand = take ? t : cand;
      c_at = take ? c : c_at;
      bit = c == a.k ? -1 : bit - 1;
    }
    // The k-th largest is the smallest key >= cand, the (k+1)-th the largest key below it (or the k-th again
    // where more than k keys reach cand). As unsigned differences both are minima without a comparison: key -
    // cand is smallest for the smallest key >= cand (a key below cand wraps around to more than any such
    // difference), and cand - 1 - key likewise for the largest key below cand (a pad, key 0, if nothing else).
    uint32_t up = 0xffffffffu, down = 0xffffffffu;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      up = min(up, key[j] - cand);
      down = min(down, cand - 1u - key[j]);
    }
    const float a_k = fv_ord_unkey(cand + fv_wave_min_u32(up));  // k-th largest
    const float a_k1 = c_at > a.k ? a_k : fv_ord_unkey(cand - 1u - fv_wave_min_u32(down));  // (k+1)-th largest
    const float thr = __fmul_rn(__fadd_rn(a_k, a_k1), 0.5f);

    uint64_t mine = 0;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const bool valid = (j < NV - 1) || (uint32_t)(lane + 64 * j) < a.K;
      const bool on = valid && acc[j] > thr;
      const uint64_t m = __ballot(on);
      if (lane == j) mine = m;
      if (a.out_codes && valid) a.out_codes[r * a.K + lane + 64 * j] = on ? 1 : 0;
    }
    if (a.out_bits && lane < NV) a.out_bits[r * NV + lane] = mine;
  }
}

template <int NV>
static void fv_launch_hash(const fv_hash_args &a, unsigned blocks, hipStream_t stream) {
  hipLaunchKernelGGL(fv_hash_kernel<NV>, dim3(blocks), dim3(256), 0, stream, a);
}

static int fv_enqueue_hash(fv_hasher *h, const int32_t *idx_dev, uint64_t n, uint32_t w, uint32_t k,
                           int32_t shift, uint64_t *bits_dev, int8_t *codes_dev, hipStream_t stream = nullptr) {
  if (n == 0) return FV_OK;
  if (!stream) stream = h->stream;
  fv_hash_args a;
  a.Wt = h->Wt;
  a.idx = idx_dev;
  a.n = n;
  a.w = w;
  a.k = k;
  a.K = h->K;
  a.ldk = h->ldk;
  a.n_cols = (uint32_t)h->N;
  a.shift = shift;
  a.out_bits = bits_dev;
  a.out_codes = codes_dev;
  a.err = h->err;
  uint64_t want = (n + 3) / 4;
  unsigned blocks = (unsigned)(want < h->max_blocks ? want : h->max_blocks);
  switch ((h->K + 63) / 64) {
#define FV_CASE(NV) case NV: fv_launch_hash<NV>(a, blocks, stream); break;
    FV_CASE(1) FV_CASE(2) FV_CASE(3) FV_CASE(4) FV_CASE(5) FV_CASE(6) FV_CASE(7) FV_CASE(8)
    FV_CASE(9) FV_CASE(10) FV_CASE(11) FV_CASE(12) FV_CASE(13) FV_CASE(14) FV_CASE(15) FV_CASE(16)
    FV_CASE(17) FV_CASE(18) FV_CASE(19) FV_CASE(20) FV_CASE(21) FV_CASE(22) FV_CASE(23) FV_CASE(24)
    FV_CASE(25) FV_CASE(26) FV_CASE(27) FV_CASE(28) FV_CASE(29) FV_CASE(30) FV_CASE(31) FV_CASE(32)
#undef FV_CASE
    default:
      return fv_fail(FV_ERR_INVALID, "hid = %u not supported", h->K);
  }
  FV_HIP(hipGetLastError());
  return FV_OK;
}

static int fv_check_hash_args(fv_hasher *h, uint32_t w, uint32_t k) {
  FV_REQUIRE(h, FV_ERR_INVALID, "null hasher");
  FV_REQUIRE(w >= 1 && w <= FV_MAX_WINDOW, FV_ERR_INVALID, "window = %u is outside 1..%d", w,
             FV_MAX_WINDOW);
  FV_REQUIRE(k >= 1 && k < h->K, FV_ERR_INVALID,
             "hash length k = %u must satisfy 0 < k < %u (the k-th and (k+1)-th largest are read)", k,
             h->K);
  return FV_OK;
}

extern "C" int fv_hasher_destroy(fv_hasher *h) {
  if (!h) return FV_OK;
  if (h->stream) (void)hipStreamSynchronize(h->stream);
  for (int l = 0; l < FV_HASH_LANES; ++l) {
    fv_hash_lane &ln = h->lane[l];
    if (ln.stream && ln.stream != h->stream) {
      (void)hipStreamSynchronize(ln.stream);
      (void)hipStreamDestroy(ln.stream);
    }
    (void)hipFree(ln.idx);
    (void)hipFree(ln.bits);
    (void)hipFree(ln.codes);
    if (ln.stage_bits) (void)hipHostFree(ln.stage_bits);
    if (ln.stage_codes) (void)hipHostFree(ln.stage_codes);
    if (ln.done) (void)hipEventDestroy(ln.done);
  }
  (void)hipFree(h->Wt);
  (void)hipFree(h->err);
  if (h->stream) (void)hipStreamDestroy(h->stream);
  delete h;
  return FV_OK;
}

extern "C" int fv_hasher_create(const float *W, uint32_t hid, uint64_t n_columns, fv_hasher **out_hasher) {
  FV_REQUIRE(W && out_hasher, FV_ERR_INVALID, "fv_hasher_create: null argument");
  *out_hasher = nullptr;
  FV_REQUIRE(hid >= 2 && hid <= FV_MAX_HID, FV_ERR_INVALID, "hid = %u is outside 2..%d", hid, FV_MAX_HID);
  FV_REQUIRE(n_columns >= 1 && n_columns < (1ull << 31), FV_ERR_INVALID, "n_columns = %llu out of range",
             (unsigned long long)n_columns);
  fv_hasher *h = new fv_hasher();
  memset(h, 0, sizeof *h);
  h->K = hid;
  h->ldk = fv_ldk(hid);
  h->N = n_columns;
  if (fv_matrix_gather_reach(h->K, h->N) > fv_matrix_alloc_elems(h->K, h->N)) {
    delete h;
    return fv_fail(FV_ERR_INVALID, "a gather of a %u x %llu matrix would read past its allocation", hid,
                   (unsigned long long)n_columns);
  }
  int cus = 0;
  int rc = fv_device_info(nullptr, 0, &cus, nullptr);
  h->max_blocks = (unsigned)(cus > 0 ? cus : 256) * 8;
  hipError_t e = hipSuccess;
  if (rc == FV_OK) {
    e = hipStreamCreate(&h->stream);
    // behind the matrix, what the gather reads for masked positions and in its lanes past K: zeros
    if (e == hipSuccess) e = hipMalloc((void **)&h->Wt, (size_t)fv_matrix_alloc_elems(h->K, h->N) * sizeof(float));
    if (e == hipSuccess)
      e = hipMemsetAsync(h->Wt + (size_t)h->N * h->ldk, 0, (size_t)fv_matrix_pad_elems(h->K) * sizeof(float), h->stream);
    if (e == hipSuccess) e = hipMalloc((void **)&h->err, sizeof(uint32_t));
    if (e == hipSuccess) e = hipMemsetAsync(h->err, 0, sizeof(uint32_t), h->stream);
    if (e != hipSuccess) rc = fv_fail(FV_ERR_HIP, "hasher allocation failed: %s", hipGetErrorString(e));
  }
  if (rc == FV_OK) rc = fv_upload_weights(W, h->Wt, h->K, h->N, h->ldk, h->stream);
  if (rc != FV_OK) {
    fv_hasher_destroy(h);
    return rc;
  }
  *out_hasher = h;
  return FV_OK;
}

extern "C" int fv_hasher_get_weights(fv_hasher *h, float *out_W) {
  FV_REQUIRE(h && out_W, FV_ERR_INVALID, "null argument");
  return fv_download_weights(h->Wt, out_W, h->K, h->N, h->ldk, h->stream);
}

extern "C" int fv_hasher_sync(fv_hasher *h) {
  FV_REQUIRE(h, FV_ERR_INVALID, "null hasher");
  FV_HIP(hipStreamSynchronize(h->stream));
  uint32_t err = 0;
  FV_HIP(hipMemcpy(&err, h->err, sizeof err, hipMemcpyDeviceToHost));
  if (err) {
    FV_HIP(hipMemset(h->err, 0, sizeof err));
    return fv_fail(FV_ERR_DATA, "a column index outside [-1, %llu) was met; its position was skipped",
                   (unsigned long long)h->N);
  }
  return FV_OK;
}

extern "C" int fv_hash_windows_dev(fv_hasher *h, const int32_t *idx_dev, uint64_t n, uint32_t w, uint32_t k,
                                   uint64_t *out_bits_dev, int8_t *out_codes_dev) {
  FV_TRY(fv_check_hash_args(h, w, k));
  FV_REQUIRE(idx_dev || n == 0, FV_ERR_INVALID, "null index buffer");
  return fv_enqueue_hash(h, idx_dev, n, w, k, 0, out_bits_dev, out_codes_dev);
}

// Makes a lane's buffer hold at least `bytes` (freed and allocated anew when it does not).
template <typename P>
static int fv_hash_reserve(P **buf, size_t *cap, size_t bytes) {
  if (*cap >= bytes) return FV_OK;
  (void)hipFree(*buf);
  *buf = nullptr;
  *cap = 0;
  FV_HIP(hipMalloc((void **)buf, bytes));
  *cap = bytes;
  return FV_OK;
}

static int fv_hash_reserve_pinned(char **buf, size_t *cap, size_t bytes) {
  if (*cap >= bytes) return FV_OK;
  if (*buf) (void)hipHostFree(*buf);
  *buf = nullptr;
  *cap = 0;
  FV_HIP(hipHostMalloc((void **)buf, bytes, hipHostMallocDefault));
  *cap = bytes;
  return FV_OK;
}

// Ordinary (pageable) host memory, which the device cannot write by DMA?
static bool fv_is_pageable(const void *p) {
  hipPointerAttribute_t at;
  if (hipPointerGetAttributes(&at, p) != hipSuccess) {
    (void)hipGetLastError();
    return true;
  }
  return at.type == hipMemoryTypeUnregistered;
}

// Copies from page-locked staging to the caller's pageable buffers, done by a few host threads while the
// device works on the next chunks: one thread copies ~10 GB/s, less than the link delivers. Items are
// published in order; every worker copies its slice of every item.
#define FV_HASH_COPY_THREADS 4
struct fv_copy_ring {
  struct item {
    const char *src;
    char *dst;
    size_t bytes;
  };
  std::vector<item> items;
  std::unique_ptr<std::atomic<uint32_t>[]> finished;  // workers done with item i
  std::atomic<uint32_t> published{0};
  std::atomic<bool> quit{false};
  std::vector<std::thread> workers;

  explicit fv_copy_ring(size_t max_items) : items(max_items), finished(new std::atomic<uint32_t>[max_items]) {
    for (size_t i = 0; i < max_items; ++i) finished[i].store(0);
    for (int p = 0; p < FV_HASH_COPY_THREADS; ++p) workers.emplace_back([this, p] { run(p); });
  }
  void run(int p) {
    for (uint32_t i = 0;; ++i) {
      while (published.load(std::memory_order_acquire) <= i) {
        if (quit.load(std::memory_order_acquire)) return;
        std::this_thread::yield();
      }
      const item &it = items[i];
      const size_t per = (it.bytes + FV_HASH_COPY_THREADS - 1) / FV_HASH_COPY_THREADS;
      const size_t lo = per * p < it.bytes ? per * p : it.bytes, hi = lo + per < it.bytes ? lo + per : it.bytes;
      if (hi > lo) memcpy(it.dst + lo, it.src + lo, hi - lo);
      finished[i].fetch_add(1, std::memory_order_release);
    }
  }
  uint32_t publish(const char *src, char *dst, size_t bytes) {
    const uint32_t i = published.load(std::memory_order_relaxed);
    items[i] = {src, dst, bytes};
    published.store(i + 1, std::memory_order_release);
    return i;
  }
  void wait(uint32_t i) {
    while (finished[i].load(std::memory_order_acquire) < FV_HASH_COPY_THREADS) std::this_thread::yield();
  }
  ~fv_copy_ring() {
    for (uint32_t i = 0; i < published.load(); ++i) wait(i);
    quit.store(true, std::memory_order_release);
    for (auto &t : workers) t.join();
  }
};

// A batch in host memory: chunks of FV_HASH_CHUNK windows alternate between the lanes; on its lane a
// chunk is copied in, hashed and copied out in stream order, so the copies of one chunk overlap the kernel
// of the other. Host buffers from fv_host_alloc_pinned are copied by DMA as they are. Outputs that go to
// pageable memory are copied by DMA into the lane's page-locked staging and from there by host threads
// (fv_copy_ring) while the device goes on; pageable inputs go through the runtime's staging. Nothing is
// allocated once the lanes' buffers have reached the chunk size.
static int fv_hash_host(fv_hasher *h, const int32_t *idx, uint64_t n, uint32_t w, uint32_t k, int32_t shift,
                        uint64_t *out_bits, int8_t *out_codes) {
  if (n == 0) return FV_OK;
  FV_REQUIRE(idx, FV_ERR_INVALID, "null index buffer");
  const uint32_t words = (h->K + 63) / 64;
  const uint64_t chunk = n < FV_HASH_CHUNK ? n : FV_HASH_CHUNK;
  const int lanes = n > chunk ? FV_HASH_LANES : 1;
  const size_t bits_row = words * sizeof(uint64_t), codes_row = h->K;
  // staging pays off for outputs of some size that the device cannot reach by DMA
  const bool stage_bits = out_bits && lanes > 1 && fv_is_pageable(out_bits);
  const bool stage_codes = out_codes && lanes > 1 && fv_is_pageable(out_codes);
  FV_HIP(hipStreamSynchronize(h->stream));  // what the caller enqueued on the hasher's stream comes first
  for (int l = 0; l < lanes; ++l) {
    fv_hash_lane &ln = h->lane[l];
    if (!ln.stream) {
      if (l == 0)
        ln.stream = h->stream;
      else
        FV_HIP(hipStreamCreate(&ln.stream));
    }
    if (!ln.done) FV_HIP(hipEventCreateWithFlags(&ln.done, hipEventDisableTiming));
    FV_TRY(fv_hash_reserve(&ln.idx, &ln.idx_cap, chunk * w * sizeof(int32_t)));
    if (out_bits) FV_TRY(fv_hash_reserve(&ln.bits, &ln.bits_cap, chunk * bits_row));
    if (out_codes) FV_TRY(fv_hash_reserve(&ln.codes, &ln.codes_cap, chunk * codes_row));
    if (stage_bits) FV_TRY(fv_hash_reserve_pinned(&ln.stage_bits, &ln.stage_bits_cap, chunk * bits_row));
    if (stage_codes) FV_TRY(fv_hash_reserve_pinned(&ln.stage_codes, &ln.stage_codes_cap, chunk * codes_row));
  }
  const uint64_t n_chunks = (n + chunk - 1) / chunk;
  std::unique_ptr<fv_copy_ring> ring;
  if (stage_bits || stage_codes) ring.reset(new fv_copy_ring(2 * n_chunks));
  std::vector<uint32_t> last_item(n_chunks, 0xffffffffu);  // the last copy item of every chunk
  int rc = FV_OK;
  // chunk c's staged outputs are handed to the host threads once its copies have landed (one iteration later,
  // while the device works on chunk c + 1), and have left the staging before chunk c + 2 is copied into it
  auto hand_over = [&](uint64_t c) -> int {
    fv_hash_lane &ln = h->lane[c % lanes];
    FV_HIP(hipEventSynchronize(ln.done));
    const uint64_t first = c * chunk, m = n - first < chunk ? n - first : chunk;
    if (stage_bits) last_item[c] = ring->publish(ln.stage_bits, (char *)out_bits + first * bits_row, m * bits_row);
    if (stage_codes) last_item[c] = ring->publish(ln.stage_codes, (char *)out_codes + first * codes_row, m * codes_row);
    return FV_OK;
  };
  for (uint64_t c = 0; c < n_chunks && rc == FV_OK; ++c) {
    fv_hash_lane &ln = h->lane[c % lanes];
    const uint64_t first = c * chunk, m = n - first < chunk ? n - first : chunk;
    if (ring && c >= (uint64_t)lanes && last_item[c - lanes] != 0xffffffffu) ring->wait(last_item[c - lanes]);
    hipError_t e = hipMemcpyAsync(ln.idx, idx + first * w, m * w * sizeof(int32_t), hipMemcpyHostToDevice, ln.stream);
    if (e != hipSuccess) {
      rc = fv_fail(FV_ERR_HIP, "hash upload failed: %s", hipGetErrorString(e));
      break;
    }
    rc = fv_enqueue_hash(h, ln.idx, m, w, k, shift, out_bits ? ln.bits : nullptr, out_codes ? ln.codes : nullptr,
                         ln.stream);
    if (rc == FV_OK && out_bits) {
      void *dst = stage_bits ? (void *)ln.stage_bits : (void *)((char *)out_bits + first * bits_row);
      e = hipMemcpyAsync(dst, ln.bits, m * bits_row, hipMemcpyDeviceToHost, ln.stream);
      if (e != hipSuccess) rc = fv_fail(FV_ERR_HIP, "download failed: %s", hipGetErrorString(e));
    }
    if (rc == FV_OK && out_codes) {
      void *dst = stage_codes ? (void *)ln.stage_codes : (void *)((char *)out_codes + first * codes_row);
      e = hipMemcpyAsync(dst, ln.codes, m * codes_row, hipMemcpyDeviceToHost, ln.stream);
      if (e != hipSuccess) rc = fv_fail(FV_ERR_HIP, "download failed: %s", hipGetErrorString(e));
    }
    if (rc == FV_OK && ring) {
      e = hipEventRecord(ln.done, ln.stream);
      if (e != hipSuccess) rc = fv_fail(FV_ERR_HIP, "event record failed: %s", hipGetErrorString(e));
      if (rc == FV_OK && c >= 1) rc = hand_over(c - 1);
    }
  }
  if (rc == FV_OK && ring) rc = hand_over(n_chunks - 1);
  ring.reset();  // waits for the host threads' copies
  for (int l = 1; l < lanes; ++l) {
    const hipError_t e = hipStreamSynchronize(h->lane[l].stream);
    if (e != hipSuccess && rc == FV_OK) rc = fv_fail(FV_ERR_HIP, "hash stream failed: %s", hipGetErrorString(e));
  }
  const int rs = fv_hasher_sync(h);  // lane 0, and the flag for indices out of range
  return rc == FV_OK ? rs : rc;
}

extern "C" int fv_hash_windows(fv_hasher *h, const int32_t *idx, uint64_t n, uint32_t w, uint32_t k,
                               uint64_t *out_bits, int8_t *out_codes) {
  FV_TRY(fv_check_hash_args(h, w, k));
  return fv_hash_host(h, idx, n, w, k, 0, out_bits, out_codes);
}

extern "C" int fv_hash_targets(fv_hasher *h, const int32_t *ids, uint64_t n, uint32_t k, int8_t *out_codes) {
  FV_TRY(fv_check_hash_args(h, 1, k));
  FV_REQUIRE(h->N % 2 == 0, FV_ERR_INVALID, "the matrix has %llu columns; targets need 2V",
             (unsigned long long)h->N);
  FV_REQUIRE(out_codes || n == 0, FV_ERR_INVALID, "null output");
  // target block = columns [V, 2V) (flyvec/core.py:179); ids outside [0, V) are reported
  const uint64_t V = h->N / 2;
  for (uint64_t i = 0; i < n; ++i)
    FV_REQUIRE(ids && ids[i] >= 0 && (uint64_t)ids[i] < V, FV_ERR_DATA,
               "token id %d at position %llu is outside [0, %llu)", ids ? ids[i] : 0,
               (unsigned long long)i, (unsigned long long)V);
  return fv_hash_host(h, ids, n, 1, k, (int32_t)V, nullptr, out_codes);
}

extern "C" int fv_hasher_time_windows(fv_hasher *h, const int32_t *idx_dev, uint64_t n, uint32_t w, uint32_t k,
                                      uint64_t *out_bits_dev, int8_t *out_codes_dev, uint32_t reps,
                                      float *out_mean_ms) {
  FV_TRY(fv_check_hash_args(h, w, k));
  FV_REQUIRE(out_mean_ms && reps >= 1, FV_ERR_INVALID, "bad timing arguments");
  hipEvent_t e0, e1;
  FV_HIP(hipEventCreate(&e0));
  FV_HIP(hipEventCreate(&e1));
  FV_HIP(hipStreamSynchronize(h->stream));
  FV_HIP(hipEventRecord(e0, h->stream));
  int rc = FV_OK;
  for (uint32_t i = 0; i < reps && rc == FV_OK; ++i)
    rc = fv_enqueue_hash(h, idx_dev, n, w, k, 0, out_bits_dev, out_codes_dev);
  FV_HIP(hipEventRecord(e1, h->stream));
  FV_HIP(hipStreamSynchronize(h->stream));
  float ms = 0.0f;
  FV_HIP(hipEventElapsedTime(&ms, e0, e1));
  *out_mean_ms = ms / (float)reps;
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  return rc;
}

// ---- normalisation (flyvec/core.py:23-36) ------------------------------------------------------
// numpy sums each row of syn**p in runs of 8192 elements (its buffer size), added in order onto 0;
// each run is summed with its pairwise scheme: blocks of at most 128 elements with 8 interleaved
// accumulators combined as ((r0+r1)+(r2+r3))+((r4+r5)+(r6+r7)) plus a sequential tail; longer
// ranges split at n/2 rounded down to a multiple of 8. The leaves of that recursion are
// independent (first kernel); their combination order is a fixed tree replayed by a small stack
// program (second kernel).
#define FV_NUMPY_BUFSIZE 8192u

struct fv_leaf {
  uint32_t start, len;
};

static void fv_pairwise_plan(uint32_t start, uint32_t n, std::vector<fv_leaf> &leaves,
                             std::vector<int32_t> &prog) {
  if (n <= 128) {
    prog.push_back((int32_t)leaves.size());
    leaves.push_back({start, n});
    return;
  }
  uint32_t n2 = n / 2;
  n2 -= n2 % 8;
  fv_pairwise_plan(start, n2, leaves, prog);
  fv_pairwise_plan(start + n2, n - n2, leaves, prog);
  prog.push_back(-1);  // pop two, push their sum
}

// x**p as numpy forms it for a float32 array and a Python integer p: p = 1 is the value itself, p = 2 the fp32
// product x * x (numpy's fast paths, exact restatements). For p >= 3 numpy calls the platform's powf, whose last
// bit is the C library's choice; here that case is the product x * x * ... * x taken in double and rounded to
// fp32 once, which agrees with a correctly rounded powf except for double-rounding cases.
template <int P>
__device__ __forceinline__ float fv_elem_pow(float x, uint32_t p) {
  if (P == 1) return x;
  if (P == 2) return __fmul_rn(x, x);
  double r = (double)x;
  for (uint32_t i = 1; i < p; ++i) r *= (double)x;
  return (float)r;
}

template <int P>
__global__ __launch_bounds__(256) void fv_leaf_sumsq_kernel(const float *__restrict__ Wt, uint32_t K,
                                                            uint32_t ldk, const fv_leaf *__restrict__ leaves,
                                                            float *__restrict__ leaf_sums, uint32_t p) {
  const uint32_t h = blockIdx.y * 256 + threadIdx.x;
  if (h >= K) return;
  const fv_leaf lf = leaves[blockIdx.x];
  const float *col = Wt + (uint64_t)lf.start * ldk + h;
#define FV_SQ(i) fv_elem_pow<P>(col[(uint64_t)(i) * ldk], p)
  float res;
  if (lf.len < 8) {
    res = -0.0f;
    for (uint32_t i = 0; i < lf.len; ++i) res = __fadd_rn(res, FV_SQ(i));
  } else {
    float r[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) r[k] = FV_SQ(k);
    uint32_t i = 8;
    for (; i < lf.len - (lf.len % 8); i += 8) {
#pragma unroll
      for (int k = 0; k < 8; ++k) r[k] = __fadd_rn(r[k], FV_SQ(i + k));
    }
    res = __fadd_rn(__fadd_rn(__fadd_rn(r[0], r[1]), __fadd_rn(r[2], r[3])),
                    __fadd_rn(__fadd_rn(r[4], r[5]), __fadd_rn(r[6], r[7])));
    for (; i < lf.len; ++i) res = __fadd_rn(res, FV_SQ(i));
  }
#undef FV_SQ
  leaf_sums[(uint64_t)blockIdx.x * K + h] = res;
}

__global__ void fv_combine_leaves_kernel(const float *__restrict__ leaf_sums, uint32_t K,
                                         const int32_t *__restrict__ prog, uint32_t prog_len,
                                         float *__restrict__ out) {
  const uint32_t h = blockIdx.x * blockDim.x + threadIdx.x;
  if (h >= K) return;
  float stack[40];
  int sp = 0;
  for (uint32_t i = 0; i < prog_len; ++i) {
    const int32_t op = prog[i];
    if (op >= 0) {
      stack[sp++] = leaf_sums[(uint64_t)op * K + h];
    } else if (op == -2) {
      stack[sp++] = 0.0f;
    } else {
      const float b = stack[--sp];
      const float a = stack[--sp];
      stack[sp++] = __fadd_rn(a, b);
    }
  }
  out[h] = stack[0];
}

__global__ __launch_bounds__(256) void fv_scale_rows_kernel(float *__restrict__ Wt, uint64_t N, uint32_t K,
                                                            uint32_t ldk, const float *__restrict__ div) {
  const uint64_t total = N * ldk;
  for (uint64_t p = (uint64_t)blockIdx.x * 256 + threadIdx.x; p < total; p += (uint64_t)gridDim.x * 256) {
    const uint32_t h = (uint32_t)(p % ldk);
    if (h < K) Wt[p] = Wt[p] / div[h];
  }
}

extern "C" int fv_hasher_row_sumsq(fv_hasher *h, float *out_sums) { return fv_hasher_row_sum_pow(h, 2, out_sums); }

// out_sums[h] = numpy.sum(W[h]**p) in numpy's fp32 pairwise order
extern "C" int fv_hasher_row_sum_pow(fv_hasher *h, uint32_t p, float *out_sums) {
  FV_REQUIRE(h && out_sums, FV_ERR_INVALID, "null argument");
  FV_REQUIRE(p >= 1 && p <= 64, FV_ERR_INVALID, "p = %u: the norm's exponent must be an integer from 1 to 64", p);
  std::vector<fv_leaf> leaves;
  std::vector<int32_t> prog;
  prog.push_back(-2);  // push 0: the reduction starts from add's identity
  for (uint32_t s0 = 0; s0 < (uint32_t)h->N; s0 += FV_NUMPY_BUFSIZE) {
    const uint32_t len = (uint32_t)h->N - s0 < FV_NUMPY_BUFSIZE ? (uint32_t)h->N - s0 : FV_NUMPY_BUFSIZE;
    fv_pairwise_plan(s0, len, leaves, prog);
    prog.push_back(-1);
  }
  fv_leaf *d_leaves = nullptr;
  int32_t *d_prog = nullptr;
  float *d_leaf = nullptr, *d_out = nullptr;
  hipError_t e = hipMalloc((void **)&d_leaves, leaves.size() * sizeof(fv_leaf));
  if (e == hipSuccess) e = hipMalloc((void **)&d_prog, prog.size() * sizeof(int32_t));
  if (e == hipSuccess) e = hipMalloc((void **)&d_leaf, leaves.size() * (size_t)h->K * sizeof(float));
  if (e == hipSuccess) e = hipMalloc((void **)&d_out, (size_t)h->K * sizeof(float));
  if (e == hipSuccess)
    e = hipMemcpyAsync(d_leaves, leaves.data(), leaves.size() * sizeof(fv_leaf), hipMemcpyHostToDevice, h->stream);
  if (e == hipSuccess)
    e = hipMemcpyAsync(d_prog, prog.data(), prog.size() * sizeof(int32_t), hipMemcpyHostToDevice, h->stream);
  if (e == hipSuccess) {
    const dim3 grid((unsigned)leaves.size(), (h->K + 255) / 256);
    if (p == 1)
      hipLaunchKernelGGL(fv_leaf_sumsq_kernel<1>, grid, dim3(256), 0, h->stream, h->Wt, h->K, h->ldk, d_leaves, d_leaf, p);
    else if (p == 2)
      hipLaunchKernelGGL(fv_leaf_sumsq_kernel<2>, grid, dim3(256), 0, h->stream, h->Wt, h->K, h->ldk, d_leaves, d_leaf, p);
    else
      hipLaunchKernelGGL(fv_leaf_sumsq_kernel<0>, grid, dim3(256), 0, h->stream, h->Wt, h->K, h->ldk, d_leaves, d_leaf, p);
    hipLaunchKernelGGL(fv_combine_leaves_kernel, dim3((h->K + 63) / 64), dim3(64), 0, h->stream, d_leaf, h->K,
                       d_prog, (uint32_t)prog.size(), d_out);
    e = hipGetLastError();
  }
  if (e == hipSuccess)
    e = hipMemcpyAsync(out_sums, d_out, (size_t)h->K * sizeof(float), hipMemcpyDeviceToHost, h->stream);
  if (e == hipSuccess) e = hipStreamSynchronize(h->stream);
  (void)hipFree(d_leaves);
  (void)hipFree(d_prog);
  (void)hipFree(d_leaf);
  (void)hipFree(d_out);
  if (e != hipSuccess) return fv_fail(FV_ERR_HIP, "row sums failed: %s", hipGetErrorString(e));
  return FV_OK;
}

// W[h][:] /= divisors[h] (fp32 division, correctly rounded)
extern "C" int fv_hasher_scale_rows(fv_hasher *h, const float *divisors) {
  FV_REQUIRE(h && divisors, FV_ERR_INVALID, "null argument");
  float *d = nullptr;
  FV_HIP(hipMalloc((void **)&d, (size_t)h->K * sizeof(float)));
  hipError_t e = hipMemcpyAsync(d, divisors, (size_t)h->K * sizeof(float), hipMemcpyHostToDevice, h->stream);
  if (e == hipSuccess) {
    hipLaunchKernelGGL(fv_scale_rows_kernel, dim3(h->max_blocks), dim3(256), 0, h->stream, h->Wt, h->N, h->K,
                       h->ldk, d);
    e = hipGetLastError();
  }
  if (e == hipSuccess) e = hipStreamSynchronize(h->stream);
  (void)hipFree(d);
  if (e != hipSuccess) return fv_fail(FV_ERR_HIP, "row scaling failed: %s", hipGetErrorString(e));
  return FV_OK;
}

extern "C" int fv_hasher_normalize(fv_hasher *h, float prec) {
  FV_REQUIRE(h, FV_ERR_INVALID, "null hasher");
  std::vector<float> sums(h->K);
  FV_TRY(fv_hasher_row_sumsq(h, sums.data()));
  // power(x, 1/2) taken as the correctly rounded square root
  for (auto &v : sums) v = sqrtf(v) + prec;
  return fv_hasher_scale_rows(h, sums.data());
}
