// Measurement helpers for bench.py, built into their own shared object (libtdist_bench.so): a plain 16-byte-vector
// device copy (the HBM streaming yardstick, and the calibration of rocprof's FETCH_SIZE / WRITE_SIZE readings) and
// an MFMA-only loop (the rate the matrix cores sustain with no memory traffic). None of this is on the hot path, and
// the product library does not carry it.
#include <stdarg.h>
#include <stdio.h>

#include "common.h"
#include "tdist_bench.h"

namespace tdist {

// this object has its own error text: it does not link against the product library
static thread_local char g_bench_err[256] = "";
int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_bench_err, sizeof(g_bench_err), fmt, ap);
  va_end(ap);
  return code;
}
int launch_status(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(TDIST_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return TDIST_OK;
}
static int num_cus() {
  int dev = 0;
  hipDeviceProp_t prop;
  if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return 0;
  return prop.multiProcessorCount;
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

// one-directional streams: a fill (writes only) and a sum (reads only; every lane's partial sum goes to sink)
__global__ __launch_bounds__(256) void fill_bytes_kernel(int4v* __restrict__ dst, int64_t n16) {
  int64_t i = (int64_t)blockIdx.x * 1024 + threadIdx.x;
  const int4v v = {(int)threadIdx.x, (int)blockIdx.x, 3, 4};
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    int64_t j = i + u * 256;
    if (j < n16) __builtin_nontemporal_store(v, dst + j);
  }
}
__global__ __launch_bounds__(256) void read_bytes_kernel(const int4v* __restrict__ src, int64_t n16, int* __restrict__ sink) {
  int64_t i = (int64_t)blockIdx.x * 4096 + threadIdx.x;
  int4v v[16];
#pragma unroll
  for (int u = 0; u < 16; ++u) {
    int64_t j = i + u * 256;
    v[u] = j < n16 ? __builtin_nontemporal_load(src + j) : int4v{0, 0, 0, 0};
  }
  int acc = 0;
#pragma unroll
  for (int u = 0; u < 16; ++u) acc += v[u][0] ^ v[u][1] ^ v[u][2] ^ v[u][3];
  if (acc == 0x5a5a5a5a) sink[threadIdx.x] = acc;   // (keeps the loads alive; practically never taken)
}

// MFMA-only loop for the rate yardstick: the K loop of a 128 x 128 wave tile with no memory traffic at all. 256
// accumulators, eight A and eight B operand fragments in registers, and the GEMM kernel's order of use: a B fragment
// serves a row of MFMAs against every A fragment in turn. kRandom fills the fragments with hashed bit patterns (random
// sign, mantissa and low exponent bits), else with 1.0. kRows = 32: 4 x 4 blocks of 32x32x16 (bf16) / 32x32x64 (e4m3);
// kRows = 16: 8 x 8 blocks of 16x16x32 / 16x16x128, i.e. twice the K per round.
__device__ __forceinline__ uint32_t probe_hash(uint32_t x) {
  x ^= x >> 16;
  x *= 0x7feb352dU;
  x ^= x >> 15;
  x *= 0x846ca68bU;
  x ^= x >> 16;
  return x;
}

template <bool kFp8, bool kRandom, int kRows>
__global__ __launch_bounds__(256, 1) void mfma_rate_kernel(float* __restrict__ sink, int iters) {
  typedef __bf16 bf16x8v __attribute__((ext_vector_type(8)));
  typedef int int8v_ __attribute__((ext_vector_type(8)));
  constexpr int kT = 128 / kRows;            // blocks per side of the wave tile
  constexpr int kAcc = kRows * kRows / 64;   // accumulators per lane and block
  typedef float acc_t __attribute__((ext_vector_type(kAcc)));
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
  acc_t acc[kT][kT];
#pragma unroll
  for (int j = 0; j < kT; ++j)
#pragma unroll
    for (int i = 0; i < kT; ++i)
#pragma unroll
      for (int e = 0; e < kAcc; ++e) acc[j][i][e] = 0.f;
  for (int it = 0; it < iters; it += 2) {
#pragma unroll
    for (int u = 0; u < 2; ++u)  // (two rounds with the fragments paired differently, as two K steps would be)
#pragma unroll
      for (int j = 0; j < kT; ++j)
#pragma unroll
        for (int i = 0; i < kT; ++i) {
          const int8v_ av = a[(i + 4 * u) & 7], bv = b[(j + 4 * u) & 7];
          if constexpr (kFp8) {
            if constexpr (kRows == 32) acc[j][i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bv, av, acc[j][i], 0, 0, 0, 0, 0, 0);
            else acc[j][i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bv, av, acc[j][i], 0, 0, 0, 0, 0, 0);
          } else {
            const int4v a4 = __builtin_shufflevector(av, av, 0, 1, 2, 3), b4 = __builtin_shufflevector(bv, bv, 0, 1, 2, 3);
            if constexpr (kRows == 32)
              acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8v, b4), __builtin_bit_cast(bf16x8v, a4), acc[j][i], 0, 0, 0);
            else
              acc[j][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8v, b4), __builtin_bit_cast(bf16x8v, a4), acc[j][i], 0, 0, 0);
          }
        }
  }
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < kT; ++j)
#pragma unroll
    for (int i = 0; i < kT; ++i) s += acc[j][i][0];
  sink[blockIdx.x * 256 + threadIdx.x] = s;
}

}  // namespace tdist

using namespace tdist;

extern "C" {

const char* tdist_bench_last_error_string(void) { return g_bench_err; }

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

int tdist_fill_bytes(void* dst, int64_t nbytes, void* stream) {
  if (!dst || nbytes < 0 || (nbytes & 15) || !aligned16(dst))
    return fail(TDIST_ERR_INVALID, "tdist_fill_bytes: pointer and size must be 16-byte aligned");
  if (nbytes == 0) return TDIST_OK;
  const int64_t n16 = nbytes / 16, blocks = ceil_div(n16, 1024);
  if (blocks > 0x7fffffff) return fail(TDIST_ERR_UNSUPPORTED, "tdist_fill_bytes: too large");
  hipLaunchKernelGGL(fill_bytes_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (int4v*)dst, n16);
  return launch_status("tdist_fill_bytes");
}

int tdist_read_bytes(const void* src, int64_t nbytes, int32_t* sink, void* stream) {
  if (!src || !sink || nbytes < 0 || (nbytes & 15) || !aligned16(src))
    return fail(TDIST_ERR_INVALID, "tdist_read_bytes: pointer and size must be 16-byte aligned, sink of 256 words");
  if (nbytes == 0) return TDIST_OK;
  const int64_t n16 = nbytes / 16, blocks = ceil_div(n16, 4096);
  if (blocks > 0x7fffffff) return fail(TDIST_ERR_UNSUPPORTED, "tdist_read_bytes: too large");
  hipLaunchKernelGGL(read_bytes_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const int4v*)src, n16, sink);
  return launch_status("tdist_read_bytes");
}

static int mfma_rate_probe(const char* who, bool narrow, int dtype, int random_operands, int iters, float* sink, void* stream) {
  if (!sink || iters <= 0 || iters % 2 != 0) return fail(TDIST_ERR_INVALID, "%s: sink, iters (even)", who);
  if (dtype != TDIST_BF16 && dtype != TDIST_F8E4M3) return fail(TDIST_ERR_UNSUPPORTED, "%s: bf16 or e4m3", who);
  const int cus = num_cus();
  if (cus <= 0) return fail(TDIST_ERR_DEVICE, "%s: no device", who);
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid(cus), block(256);
  const int which = (narrow ? 4 : 0) + (dtype == TDIST_F8E4M3 ? 2 : 0) + (random_operands ? 1 : 0);
  switch (which) {
    case 0: hipLaunchKernelGGL((mfma_rate_kernel<false, false, 32>), grid, block, 0, st, sink, iters); break;
    case 1: hipLaunchKernelGGL((mfma_rate_kernel<false, true, 32>), grid, block, 0, st, sink, iters); break;
    case 2: hipLaunchKernelGGL((mfma_rate_kernel<true, false, 32>), grid, block, 0, st, sink, iters); break;
    case 3: hipLaunchKernelGGL((mfma_rate_kernel<true, true, 32>), grid, block, 0, st, sink, iters); break;
    case 4: hipLaunchKernelGGL((mfma_rate_kernel<false, false, 16>), grid, block, 0, st, sink, iters); break;
    case 5: hipLaunchKernelGGL((mfma_rate_kernel<false, true, 16>), grid, block, 0, st, sink, iters); break;
    case 6: hipLaunchKernelGGL((mfma_rate_kernel<true, false, 16>), grid, block, 0, st, sink, iters); break;
    default: hipLaunchKernelGGL((mfma_rate_kernel<true, true, 16>), grid, block, 0, st, sink, iters); break;
  }
  return launch_status(who);
}

int tdist_mfma_rate_probe(int dtype, int random_operands, int iters, float* sink, void* stream) {
  return mfma_rate_probe("tdist_mfma_rate_probe", false, dtype, random_operands, iters, sink, stream);
}

int tdist_mfma_rate_probe_16row(int dtype, int random_operands, int iters, float* sink, void* stream) {
  return mfma_rate_probe("tdist_mfma_rate_probe_16row", true, dtype, random_operands, iters, sink, stream);
}

}  // extern "C"
