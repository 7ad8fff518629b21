// Library-level entry points: version, error text, device probe, flag helpers, the producer-side
// chunk push, and the calibration copy kernel.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <mutex>

#include "common.h"

namespace tdist {

static thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int launch_status(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(TDIST_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return TDIST_OK;
}

static DeviceInfo g_info = {0, 0, 0};
static std::mutex g_info_mu;

const DeviceInfo& device_info() {
  std::lock_guard<std::mutex> lk(g_info_mu);
  if (!g_info.ok) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) {
      g_info.num_cus = prop.multiProcessorCount;
      g_info.num_xcds = 8;  // MI355X: 8 XCDs x 32 CUs
      if (g_info.num_cus % g_info.num_xcds != 0) g_info.num_xcds = 1;
      g_info.ok = strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? 1 : -1;
    } else {
      (void)hipGetLastError();
      g_info.ok = -1;
    }
  }
  return g_info;
}

__global__ void flag_fill_kernel(int32_t* flags, int n, int value) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) __hip_atomic_store(flags + i, value, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

__global__ __launch_bounds__(256) void copy_bytes_kernel(int4v* __restrict__ dst, const int4v* __restrict__ src,
                                                         int64_t n16) {
  int64_t i = (int64_t)blockIdx.x * 1024 + threadIdx.x;
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    int64_t j = i + u * 256;
    if (j < n16) __builtin_nontemporal_store(__builtin_nontemporal_load(src + j), dst + j);
  }
}

}  // namespace tdist

using namespace tdist;

extern "C" {

int tdist_version(void) { return 100; }

const char* tdist_last_error_string(void) { return g_err; }

int tdist_init(void) {
  const DeviceInfo& di = device_info();
  if (di.ok != 1) return fail(TDIST_ERR_DEVICE, "tdist_init: current device is not a gfx950 GPU");
  return TDIST_OK;
}

int tdist_num_cus(void) {
  const DeviceInfo& di = device_info();
  return di.ok == 1 ? di.num_cus : 0;
}

int tdist_flag_fill(int32_t* flags, int n, int value, void* stream) {
  if (!flags || n < 0) return fail(TDIST_ERR_INVALID, "tdist_flag_fill: null flags or negative n");
  if (n == 0) return TDIST_OK;
  hipLaunchKernelGGL(flag_fill_kernel, dim3((n + 255) / 256), dim3(256), 0, (hipStream_t)stream, flags, n, value);
  return launch_status("tdist_flag_fill");
}

int tdist_flag_set(int32_t* flag, int value, void* stream) {
  if (!flag) return fail(TDIST_ERR_INVALID, "tdist_flag_set: null flag");
  hipLaunchKernelGGL(flag_fill_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, flag, 1, value);
  return launch_status("tdist_flag_set");
}

int tdist_producer_push_chunk(void* dst, const void* src, int64_t nbytes, int32_t* flag, const int32_t* one,
                              int use_sdma, void* stream) {
  if (!dst || !src || !flag || !one || nbytes < 0)
    return fail(TDIST_ERR_INVALID, "tdist_producer_push_chunk: null pointer or negative size");
  hipStream_t s = (hipStream_t)stream;
  hipMemcpyKind kind = use_sdma ? hipMemcpyDeviceToDeviceNoCU : hipMemcpyDeviceToDevice;
  if (nbytes > 0) {
    hipError_t e = hipMemcpyAsync(dst, src, (size_t)nbytes, kind, s);
    if (e != hipSuccess) return fail(TDIST_ERR_LAUNCH, "tdist_producer_push_chunk(data): %s", hipGetErrorString(e));
  }
  // Same stream, so the 4-byte copy that publishes the flag is ordered after the data copy.
  hipError_t e = hipMemcpyAsync(flag, one, sizeof(int32_t), kind, s);
  if (e != hipSuccess) return fail(TDIST_ERR_LAUNCH, "tdist_producer_push_chunk(flag): %s", hipGetErrorString(e));
  return TDIST_OK;
}

int tdist_copy_bytes(void* dst, const void* src, int64_t nbytes, void* stream) {
  if (!dst || !src || nbytes < 0 || (nbytes & 15) || !aligned16(dst) || !aligned16(src))
    return fail(TDIST_ERR_INVALID, "tdist_copy_bytes: pointers and size must be 16-byte aligned");
  if (nbytes == 0) return TDIST_OK;
  int64_t n16 = nbytes / 16;
  int64_t blocks = ceil_div(n16, 1024);
  if (blocks > 0x7fffffff) return fail(TDIST_ERR_UNSUPPORTED, "tdist_copy_bytes: too large");
  hipLaunchKernelGGL(copy_bytes_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (int4v*)dst,
                     (const int4v*)src, n16);
  return launch_status("tdist_copy_bytes");
}

}  // extern "C"
