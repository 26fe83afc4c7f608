// Runtime plumbing of libflyvec_hip.so: error reporting, device queries, pinned / device
// memory helpers, and the layout change between the checkpoint matrix (K x N row-major) and
// the token-major matrix the kernels read.
#include <string.h>

#include <string>

#include "fv_internal.h"

static thread_local std::string g_last_error;

int fv_fail(int code, const char *fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  g_last_error = buf;
  return code;
}

void fv_clear_error() { g_last_error.clear(); }

extern "C" const char *fv_last_error(void) { return g_last_error.c_str(); }

extern "C" int fv_device_count(int *out_count) {
  FV_REQUIRE(out_count, FV_ERR_INVALID, "fv_device_count: null output");
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess) {
    *out_count = 0;
    return fv_fail(FV_ERR_HIP, "hipGetDeviceCount failed: %s", hipGetErrorString(e));
  }
  *out_count = n;
  return FV_OK;
}

extern "C" int fv_set_device(int device) {
  FV_HIP(hipSetDevice(device));
  return FV_OK;
}

extern "C" int fv_device_info(char *name, size_t name_cap, int *out_compute_units,
                              uint64_t *out_hbm_bytes) {
  int dev = 0;
  FV_HIP(hipGetDevice(&dev));
  hipDeviceProp_t prop;
  FV_HIP(hipGetDeviceProperties(&prop, dev));
  if (name && name_cap) {
    snprintf(name, name_cap, "%s (%s)", prop.name, prop.gcnArchName);
  }
  if (out_compute_units) *out_compute_units = prop.multiProcessorCount;
  if (out_hbm_bytes) *out_hbm_bytes = (uint64_t)prop.totalGlobalMem;
  return FV_OK;
}

extern "C" int fv_device_memory(uint64_t *out_free_bytes, uint64_t *out_total_bytes) {
  size_t free_b = 0, total_b = 0;
  FV_HIP(hipMemGetInfo(&free_b, &total_b));
  if (out_free_bytes) *out_free_bytes = (uint64_t)free_b;
  if (out_total_bytes) *out_total_bytes = (uint64_t)total_b;
  return FV_OK;
}

extern "C" int fv_host_alloc_pinned(size_t bytes, void **out_ptr) {
  FV_REQUIRE(out_ptr, FV_ERR_INVALID, "fv_host_alloc_pinned: null output");
  *out_ptr = nullptr;
  if (bytes == 0) return FV_OK;
  FV_HIP(hipHostMalloc(out_ptr, bytes, hipHostMallocDefault));
  return FV_OK;
}

extern "C" int fv_host_free_pinned(void *ptr) {
  if (ptr) FV_HIP(hipHostFree(ptr));
  return FV_OK;
}

extern "C" int fv_dev_alloc(size_t bytes, void **out_dev_ptr) {
  FV_REQUIRE(out_dev_ptr, FV_ERR_INVALID, "fv_dev_alloc: null output");
  *out_dev_ptr = nullptr;
  if (bytes == 0) return FV_OK;
  FV_HIP(hipMalloc(out_dev_ptr, bytes));
  return FV_OK;
}

extern "C" int fv_dev_free(void *dev_ptr) {
  if (dev_ptr) FV_HIP(hipFree(dev_ptr));
  return FV_OK;
}

extern "C" int fv_dev_upload(void *dst_dev, const void *src_host, size_t bytes) {
  if (bytes == 0) return FV_OK;
  FV_REQUIRE(dst_dev && src_host, FV_ERR_INVALID, "fv_dev_upload: null pointer");
  FV_HIP(hipMemcpy(dst_dev, src_host, bytes, hipMemcpyHostToDevice));
  return FV_OK;
}

extern "C" int fv_dev_download(void *dst_host, const void *src_dev, size_t bytes) {
  if (bytes == 0) return FV_OK;
  FV_REQUIRE(dst_host && src_dev, FV_ERR_INVALID, "fv_dev_download: null pointer");
  FV_HIP(hipMemcpy(dst_host, src_dev, bytes, hipMemcpyDeviceToHost));
  return FV_OK;
}

// ---- layout change ------------------------------------------------------------------
// 64 x 64 tiles through LDS (+1 padding column against bank conflicts): reads are coalesced
// along N of the row-major matrix, writes along K of the token-major one (and vice versa).

#define FV_TT 64

__global__ __launch_bounds__(256) void fv_to_token_major_kernel(const float *__restrict__ W,
                                                                float *__restrict__ Wt, uint32_t K,
                                                                uint64_t N, uint32_t ldk) {
  __shared__ float tile[FV_TT][FV_TT + 1];
  const uint64_t i0 = (uint64_t)blockIdx.x * FV_TT;  // token (column of W)
  const uint32_t h0 = blockIdx.y * FV_TT;            // neuron (row of W)
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int r = ty; r < FV_TT; r += 4) {
    uint32_t h = h0 + r;
    uint64_t i = i0 + tx;
    tile[r][tx] = (h < K && i < N) ? W[(uint64_t)h * N + i] : 0.0f;
  }
  __syncthreads();
  for (int r = ty; r < FV_TT; r += 4) {
    uint64_t i = i0 + r;
    uint32_t h = h0 + tx;
    if (i < N && h < ldk) Wt[i * ldk + h] = tile[tx][r];  // pad columns (h >= K) receive 0
  }
}

__global__ __launch_bounds__(256) void fv_to_row_major_kernel(const float *__restrict__ Wt,
                                                              float *__restrict__ W, uint32_t K,
                                                              uint64_t N, uint32_t ldk) {
  __shared__ float tile[FV_TT][FV_TT + 1];
  const uint64_t i0 = (uint64_t)blockIdx.x * FV_TT;
  const uint32_t h0 = blockIdx.y * FV_TT;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int r = ty; r < FV_TT; r += 4) {
    uint64_t i = i0 + r;
    uint32_t h = h0 + tx;
    tile[r][tx] = (i < N && h < K) ? Wt[i * ldk + h] : 0.0f;
  }
  __syncthreads();
  for (int r = ty; r < FV_TT; r += 4) {
    uint32_t h = h0 + r;
    uint64_t i = i0 + tx;
    if (h < K && i < N) W[(uint64_t)h * N + i] = tile[tx][r];
  }
}

int fv_launch_to_token_major(const float *W, float *Wt, uint32_t K, uint64_t N, uint32_t ldk,
                             hipStream_t stream) {
  dim3 grid((unsigned)((N + FV_TT - 1) / FV_TT), (ldk + FV_TT - 1) / FV_TT);
  hipLaunchKernelGGL(fv_to_token_major_kernel, grid, dim3(256), 0, stream, W, Wt, K, N, ldk);
  FV_HIP(hipGetLastError());
  return FV_OK;
}

int fv_launch_to_row_major(const float *Wt, float *W, uint32_t K, uint64_t N, uint32_t ldk,
                           hipStream_t stream) {
  dim3 grid((unsigned)((N + FV_TT - 1) / FV_TT), (K + FV_TT - 1) / FV_TT);
  hipLaunchKernelGGL(fv_to_row_major_kernel, grid, dim3(256), 0, stream, Wt, W, K, N, ldk);
  FV_HIP(hipGetLastError());
  return FV_OK;
}

int fv_upload_weights(const float *W_host, float *Wt_dev, uint32_t K, uint64_t N, uint32_t ldk,
                      hipStream_t stream) {
  float *stage = nullptr;
  size_t bytes = (size_t)K * N * sizeof(float);
  FV_HIP(hipMalloc((void **)&stage, bytes));
  hipError_t e = hipMemcpyAsync(stage, W_host, bytes, hipMemcpyHostToDevice, stream);
  int rc = FV_OK;
  if (e != hipSuccess) rc = fv_fail(FV_ERR_HIP, "weight upload failed: %s", hipGetErrorString(e));
  if (rc == FV_OK) rc = fv_launch_to_token_major(stage, Wt_dev, K, N, ldk, stream);
  e = hipStreamSynchronize(stream);
  if (rc == FV_OK && e != hipSuccess)
    rc = fv_fail(FV_ERR_HIP, "weight upload failed: %s", hipGetErrorString(e));
  (void)hipFree(stage);
  return rc;
}

int fv_download_weights(const float *Wt_dev, float *W_host, uint32_t K, uint64_t N, uint32_t ldk,
                        hipStream_t stream) {
  float *stage = nullptr;
  size_t bytes = (size_t)K * N * sizeof(float);
  FV_HIP(hipMalloc((void **)&stage, bytes));
  int rc = fv_launch_to_row_major(Wt_dev, stage, K, N, ldk, stream);
  hipError_t e = hipSuccess;
  if (rc == FV_OK) {
    e = hipMemcpyAsync(W_host, stage, bytes, hipMemcpyDeviceToHost, stream);
    if (e != hipSuccess) rc = fv_fail(FV_ERR_HIP, "weight download failed: %s", hipGetErrorString(e));
  }
  e = hipStreamSynchronize(stream);
  if (rc == FV_OK && e != hipSuccess)
    rc = fv_fail(FV_ERR_HIP, "weight download failed: %s", hipGetErrorString(e));
  (void)hipFree(stage);
  return rc;
}

// ---- calibration copy -------------------------------------------------------------------------------
// A plain streaming copy of known size: the yardstick hardware byte counters are scaled by, and a
// measured ceiling for this machine's copy bandwidth.

__global__ __launch_bounds__(256) void fv_calibration_copy_kernel(const float4 *__restrict__ src,
                                                                  float4 *__restrict__ dst, uint64_t n4) {
  for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += (uint64_t)gridDim.x * 256)
    dst[i] = src[i];
}

extern "C" int fv_calibration_copy(size_t bytes, uint32_t reps, float *out_mean_ms) {
  FV_REQUIRE(bytes >= 16 && reps >= 1 && out_mean_ms, FV_ERR_INVALID, "fv_calibration_copy: bad arguments");
  const uint64_t n4 = bytes / 16;
  float4 *src = nullptr, *dst = nullptr;
  FV_HIP(hipMalloc((void **)&src, n4 * 16));
  hipError_t e = hipMalloc((void **)&dst, n4 * 16);
  hipEvent_t e0 = nullptr, e1 = nullptr;
  if (e == hipSuccess) e = hipMemset(src, 1, n4 * 16);
  if (e == hipSuccess) e = hipEventCreate(&e0);
  if (e == hipSuccess) e = hipEventCreate(&e1);
  if (e == hipSuccess) {
    const unsigned blocks = 256 * 8;
    hipLaunchKernelGGL(fv_calibration_copy_kernel, dim3(blocks), dim3(256), 0, 0, src, dst, n4);  // warm-up
    e = hipEventRecord(e0, 0);
    for (uint32_t r = 0; r < reps; ++r)
      hipLaunchKernelGGL(fv_calibration_copy_kernel, dim3(blocks), dim3(256), 0, 0, src, dst, n4);
    if (e == hipSuccess) e = hipEventRecord(e1, 0);
    if (e == hipSuccess) e = hipEventSynchronize(e1);
    float ms = 0.0f;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    *out_mean_ms = ms / (float)reps;
  }
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  (void)hipFree(src);
  (void)hipFree(dst);
  if (e != hipSuccess) return fv_fail(FV_ERR_HIP, "calibration copy failed: %s", hipGetErrorString(e));
  return FV_OK;
}
