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

static int wall_clock_khz() {
  static int rate_khz = 0;   // constant-rate wall clock of the device (100 MHz on gfx950)
  if (rate_khz == 0) {
    int dev = 0, khz = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess ||
        khz <= 0) {
      (void)hipGetLastError();
      return 0;
    }
    rate_khz = khz;
  }
  return rate_khz;
}

__global__ void flag_fill_kernel(int32_t* flags, int n, int value) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) __hip_atomic_store(flags + i, value, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

// Link pacing of the one-GPU producer: a time stamp of the constant-rate wall clock, and a one-wave kernel that
// holds its stream until that clock has moved `ticks` past the stamp. The loop ends by itself: the clock only
// moves forward, a stamp from the future makes the unsigned difference huge, and `ticks` is capped by the host.
__global__ void producer_mark_kernel(unsigned long long* stamp) {
  if (threadIdx.x == 0) *stamp = wall_clock64();
}
__global__ void producer_wait_until_kernel(const unsigned long long* stamp, unsigned long long ticks) {
  if (threadIdx.x != 0) return;
  const unsigned long long t0 = *stamp;
  const unsigned long long begin = wall_clock64();
  while (true) {
    const unsigned long long now = wall_clock64();
    if (now - t0 >= ticks || now - begin >= ticks) break;
    __builtin_amdgcn_s_sleep(16);
  }
}

// The peers' copy engines of an all-gather, played by one small kernel on the GPU that consumes the rows: block
// row y stands for peer (rank + 1 + y) % world and pushes that peer's chunks into the workspace one after the
// other, each no earlier than its link time, and releases the chunk's flag when the last of its workgroups has
// stored its part. Nothing in it waits for another workgroup, and the pacing wait is bounded by the clock.
// It is written to need few registers and no LDS so that its waves fit beside a resident GEMM wave on the same
// SIMD: the consumer then needs no compute units set aside for the producer.
struct PushParams {
  unsigned char* workspace;
  const unsigned char* const* peer_src;  // [world] device pointers; the entry of `rank` is not read
  int32_t* flags;
  int32_t* counters;                     // [world * chunks_per_rank], zero on entry, left zero
  const int32_t* held;                   // optional [world * chunks_per_rank]: non-zero = never deliver (test hook)
  const unsigned long long* stamp;       // optional: wall-clock stamp of the op's start
  unsigned long long ticks_per_chunk;
  long long chunk_bytes, rank_bytes;
  int world, rank, chunks_per_rank, flag_value;
};

__global__ __launch_bounds__(256) void producer_push_kernel(const PushParams p) {
  const int r = (p.rank + 1 + (int)blockIdx.y) % p.world;
  const unsigned char* src = p.peer_src[r];
  unsigned char* dst = p.workspace + (long long)r * p.rank_bytes;
  unsigned long long t0 = 0, begin = 0;
  if (p.stamp != nullptr && threadIdx.x == 0) {
    t0 = *p.stamp;
    begin = wall_clock64();
  }
  for (int c = 0; c < p.chunks_per_rank; ++c) {
    const int chunk_pos = r * p.chunks_per_rank + c;
    if (p.held != nullptr && p.held[chunk_pos] != 0) continue;
    if (p.stamp != nullptr) {
      if (threadIdx.x == 0) {
        const unsigned long long due = (unsigned long long)(c + 1) * p.ticks_per_chunk;
        while (true) {
          const unsigned long long now = wall_clock64();
          if (now - t0 >= due || now - begin >= due) break;
          __builtin_amdgcn_s_sleep(16);
        }
      }
      __syncthreads();
    }
    // Four loads in flight per lane: more would cost the registers that let these waves sit beside a GEMM wave.
    // Addresses are a wave-uniform chunk base plus a 32-bit byte offset (chunks are below 4 GiB): one register
    // per lane instead of a 64-bit pointer per load.
    const unsigned char* const sbase = (const unsigned char*)src + (long long)c * p.chunk_bytes;
    unsigned char* const dbase = (unsigned char*)dst + (long long)c * p.chunk_bytes;
    const uint32_t nbytes = (uint32_t)p.chunk_bytes;
    const uint32_t stride = gridDim.x * 256u * 16u;
    auto put = [&](uint32_t off, const int4v v) { __builtin_nontemporal_store(v, (int4v*)(dbase + off)); };
    uint32_t off = (blockIdx.x * 256u + threadIdx.x) * 16u;
    // (the host keeps chunk_bytes + 4 * stride below 2^32, so the offsets cannot wrap)
    for (; off + 3 * stride < nbytes; off += 4 * stride) {
      const int4v v0 = __builtin_nontemporal_load((const int4v*)(sbase + off));
      const int4v v1 = __builtin_nontemporal_load((const int4v*)(sbase + off + stride));
      const int4v v2 = __builtin_nontemporal_load((const int4v*)(sbase + off + 2 * stride));
      const int4v v3 = __builtin_nontemporal_load((const int4v*)(sbase + off + 3 * stride));
      put(off, v0);
      put(off + stride, v1);
      put(off + 2 * stride, v2);
      put(off + 3 * stride, v3);
    }
    for (; off < nbytes; off += stride) put(off, __builtin_nontemporal_load((const int4v*)(sbase + off)));
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
      // one release per workgroup and chunk: writes this XCD's dirty lines (the workgroup's rows among them) back
      // to memory before the counter says that this part is in place
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "");
      int32_t* ctr = p.counters + chunk_pos;
      const int old = __hip_atomic_fetch_add(ctr, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (old == (int)gridDim.x - 1) {
        __hip_atomic_store(ctr, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(p.flags + chunk_pos, p.flag_value, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
      }
    }
  }
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

int tdist_producer_mark(uint64_t* stamp, void* stream) {
  if (!stamp) return fail(TDIST_ERR_INVALID, "tdist_producer_mark: null stamp");
  hipLaunchKernelGGL(producer_mark_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, (unsigned long long*)stamp);
  return launch_status("tdist_producer_mark");
}

int tdist_producer_wait_until(const uint64_t* stamp, int64_t offset_ns, void* stream) {
  if (!stamp) return fail(TDIST_ERR_INVALID, "tdist_producer_wait_until: null stamp");
  if (offset_ns < 0 || offset_ns > 100000000)
    return fail(TDIST_ERR_INVALID, "tdist_producer_wait_until: offset %lld ns outside [0, 100 ms]", (long long)offset_ns);
  const int rate_khz = wall_clock_khz();
  if (rate_khz <= 0) return fail(TDIST_ERR_DEVICE, "tdist_producer_wait_until: cannot read the wall clock rate");
  const unsigned long long ticks = (unsigned long long)((double)offset_ns * 1e-6 * (double)rate_khz);
  hipLaunchKernelGGL(producer_wait_until_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream,
                     (const unsigned long long*)stamp, ticks);
  return launch_status("tdist_producer_wait_until");
}

int tdist_producer_push_peers(void* workspace, const void* const* peer_src, int world_size, int rank,
                              int64_t rank_bytes, int64_t chunk_bytes, int32_t* flags, int flag_value,
                              int32_t* counters, const int32_t* held, const uint64_t* stamp, int64_t ns_per_chunk,
                              int workgroups_per_peer, void* stream) {
  const char* who = "tdist_producer_push_peers";
  if (!workspace || !peer_src || !flags || !counters) return fail(TDIST_ERR_INVALID, "%s: null pointer", who);
  if (world_size < 1 || rank < 0 || rank >= world_size) return fail(TDIST_ERR_INVALID, "%s: rank %d / world_size %d", who, rank, world_size);
  if (chunk_bytes <= 0 || rank_bytes <= 0 || rank_bytes % chunk_bytes != 0 || chunk_bytes % 16 != 0)
    return fail(TDIST_ERR_INVALID, "%s: rank_bytes %lld must be a multiple of chunk_bytes %lld, itself a multiple of 16",
                who, (long long)rank_bytes, (long long)chunk_bytes);
  if (!aligned16(workspace)) return fail(TDIST_ERR_UNSUPPORTED, "%s: workspace must be 16-byte aligned", who);
  if (workgroups_per_peer < 1 || workgroups_per_peer > 64) return fail(TDIST_ERR_INVALID, "%s: workgroups_per_peer in 1..64", who);
  const int64_t cpr = rank_bytes / chunk_bytes;
  if (cpr > 65535) return fail(TDIST_ERR_UNSUPPORTED, "%s: too many chunks per rank", who);
  if (chunk_bytes > (1ll << 31)) return fail(TDIST_ERR_UNSUPPORTED, "%s: chunks above 2 GiB are not supported", who);
  if (world_size == 1) return TDIST_OK;
  PushParams p;
  p.workspace = (unsigned char*)workspace;
  p.peer_src = (const unsigned char* const*)peer_src;
  p.flags = flags;
  p.counters = counters;
  p.held = held;
  p.stamp = nullptr;
  p.ticks_per_chunk = 0;
  if (stamp != nullptr && ns_per_chunk > 0) {
    if (ns_per_chunk * cpr > 100000000)
      return fail(TDIST_ERR_INVALID, "%s: %lld ns per chunk x %lld chunks is beyond the 100 ms the pacing may hold a kernel", who,
                  (long long)ns_per_chunk, (long long)cpr);
    const int khz = wall_clock_khz();
    if (khz <= 0) return fail(TDIST_ERR_DEVICE, "%s: cannot read the wall clock rate", who);
    p.stamp = (const unsigned long long*)stamp;
    p.ticks_per_chunk = (unsigned long long)((double)ns_per_chunk * 1e-6 * (double)khz);
  }
  p.chunk_bytes = chunk_bytes;
  p.rank_bytes = rank_bytes;
  p.world = world_size;
  p.rank = rank;
  p.chunks_per_rank = (int)cpr;
  p.flag_value = flag_value;
  hipLaunchKernelGGL(producer_push_kernel, dim3(workgroups_per_peer, world_size - 1), dim3(256), 0, (hipStream_t)stream, p);
  return launch_status(who);
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

static int mfma_rate_probe(const char* who, bool narrow, int dtype, int random_operands, int iters, float* sink, void* stream) {
  if (!sink || iters <= 0 || iters % 2 != 0) return fail(TDIST_ERR_INVALID, "%s: sink, iters (even)", who);
  if (dtype != TDIST_BF16 && dtype != TDIST_F8E4M3) return fail(TDIST_ERR_UNSUPPORTED, "%s: bf16 or e4m3", who);
  const DeviceInfo& di = device_info();
  if (di.ok != 1) return fail(TDIST_ERR_DEVICE, "%s: current device is not gfx950", who);
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid(di.num_cus), block(256);
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
