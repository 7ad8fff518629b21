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

// MFMA-only loop for the rate yardstick: no memory traffic at all, eight independent accumulators, and operand
// fragments that change from one MFMA to the next (eight A and eight B fragments in registers, paired differently
// every time). kRandom fills them with hashed bit patterns (random sign, mantissa and low exponent bits), else with 1.0.
__device__ __forceinline__ uint32_t probe_hash(uint32_t x) {
  x ^= x >> 16;
  x *= 0x7feb352dU;
  x ^= x >> 15;
  x *= 0x846ca68bU;
  x ^= x >> 16;
  return x;
}

template <bool kFp8, bool kRandom>
__global__ __launch_bounds__(256, 1) void mfma_rate_kernel(float* __restrict__ sink, int iters) {
  typedef __bf16 bf16x8v __attribute__((ext_vector_type(8)));
  typedef int int8v_ __attribute__((ext_vector_type(8)));
  int8v_ a[8], b[8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint32_t h1 = probe_hash(threadIdx.x * 131u + i * 17u + e), h2 = probe_hash(threadIdx.x * 71u + i * 29u + e + 1000u);
      if (kFp8) {  // e4m3 bytes: random sign, exponent 4..7, random mantissa
        a[i][e] = kRandom ? (int)((h1 & 0x9f9f9f9fu) | 0x20202020u) : 0x38383838;
        b[i][e] = kRandom ? (int)((h2 & 0x9f9f9f9fu) | 0x20202020u) : 0x38383838;
      } else {     // bf16 pairs: random sign, exponent 124..127, random mantissa
        a[i][e] = kRandom ? (int)((h1 & 0x81ff81ffu) | 0x3e003e00u) : 0x3f803f80;
        b[i][e] = kRandom ? (int)((h2 & 0x81ff81ffu) | 0x3e003e00u) : 0x3f803f80;
      }
    }
  float16v acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;
  for (int it = 0; it < iters; it += 4) {
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int8v_ av = a[(i + u) & 7], bv = b[(i * 3 + u) & 7];
        if (kFp8) {
          acc[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, bv, acc[i], 0, 0, 0, 0, 0, 0);
        } else {
          const int4v a4 = __builtin_shufflevector(av, av, 0, 1, 2, 3), b4 = __builtin_shufflevector(bv, bv, 0, 1, 2, 3);
          acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8v, a4), __builtin_bit_cast(bf16x8v, b4),
                                                           acc[i], 0, 0, 0);
        }
      }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) s += acc[i][0];
  sink[blockIdx.x * 256 + threadIdx.x] = s;
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

int tdist_mfma_rate_probe(int dtype, int random_operands, int iters, float* sink, void* stream) {
  if (!sink || iters <= 0 || iters % 4 != 0) return fail(TDIST_ERR_INVALID, "tdist_mfma_rate_probe: sink, iters (multiple of 4)");
  if (dtype != TDIST_BF16 && dtype != TDIST_F8E4M3) return fail(TDIST_ERR_UNSUPPORTED, "tdist_mfma_rate_probe: bf16 or e4m3");
  const DeviceInfo& di = device_info();
  if (di.ok != 1) return fail(TDIST_ERR_DEVICE, "tdist_mfma_rate_probe: current device is not gfx950");
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid(di.num_cus), block(256);
  if (dtype == TDIST_BF16) {
    if (random_operands) hipLaunchKernelGGL((mfma_rate_kernel<false, true>), grid, block, 0, st, sink, iters);
    else hipLaunchKernelGGL((mfma_rate_kernel<false, false>), grid, block, 0, st, sink, iters);
  } else {
    if (random_operands) hipLaunchKernelGGL((mfma_rate_kernel<true, true>), grid, block, 0, st, sink, iters);
    else hipLaunchKernelGGL((mfma_rate_kernel<true, false>), grid, block, 0, st, sink, iters);
  }
  return launch_status("tdist_mfma_rate_probe");
}

}  // extern "C"
