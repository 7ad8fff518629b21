// Library-level entry points: version, error text, device probe, flag helpers, the producer-side
// chunk push, and the calibration copy kernel.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <atomic>
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

static DeviceInfo g_info = {0, 0, 0, 0};
static std::mutex g_info_mu;

// Test and measurement switches: -1 = the library decides. Set through tdist_debug_set only (nothing is read from the
// environment), read by the host side of the entry points at call time.
static std::atomic<int> g_debug[TDIST_DEBUG_NUM_KEYS];
static std::once_flag g_debug_once;
static void debug_init() {
  std::call_once(g_debug_once, [] {
    for (auto& v : g_debug) v.store(-1, std::memory_order_relaxed);
  });
}
int debug_get(int key) {
  debug_init();
  return key >= 0 && key < TDIST_DEBUG_NUM_KEYS ? g_debug[key].load(std::memory_order_relaxed) : -1;
}

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

// Every workgroup of a grid writes down the XCD it runs on. The ids land in a small array of the library's own (one
// copy per GPU; its device address comes from hipGetSymbolAddress), so the check allocates nothing.
constexpr int kProbeMaxWorkgroups = 4096;
static __device__ int32_t g_probe_ids[kProbeMaxWorkgroups];
__global__ void xcd_probe_kernel(int32_t* out) {
  if (threadIdx.x == 0) out[blockIdx.x] = xcc_id();
}

int probe_xcd_round_robin() {
  const DeviceInfo& di = device_info();
  if (di.ok != 1) return fail(TDIST_ERR_DEVICE, "tdist_init: current device is not a gfx950 GPU");
  {
    std::lock_guard<std::mutex> lk(g_info_mu);
    if (g_info.xcd_round_robin != 0) return TDIST_OK;   // checked before (1 = holds, -1 = does not)
  }
  if (di.num_xcds <= 1) return TDIST_OK;
  // four workgroups per compute unit: workgroups i and j must share an XCD exactly when i = j (mod num_xcds)
  const int n = 4 * di.num_cus < kProbeMaxWorkgroups ? 4 * di.num_cus : kProbeMaxWorkgroups;
  int32_t* dev_ids = nullptr;
  bool ok = hipGetSymbolAddress((void**)&dev_ids, HIP_SYMBOL(g_probe_ids)) == hipSuccess && dev_ids != nullptr;
  int32_t* ids = new int32_t[n];
  if (ok) {
    hipLaunchKernelGGL(xcd_probe_kernel, dim3(n), dim3(256), 0, (hipStream_t) nullptr, dev_ids);
    ok = hipMemcpy(ids, dev_ids, (size_t)n * 4, hipMemcpyDeviceToHost) == hipSuccess;
  }
  if (!ok) (void)hipGetLastError();   // not verified: the kernels keep to device-coherent exchanges
  for (int i = 0; ok && i < n; ++i) ok = ids[i] == ids[i % di.num_xcds];
  for (int i = 0; ok && i < di.num_xcds; ++i)
    for (int j = 0; ok && j < i; ++j) ok = ids[i] != ids[j];
  delete[] ids;
  std::lock_guard<std::mutex> lk(g_info_mu);
  g_info.xcd_round_robin = ok ? 1 : -1;
  return TDIST_OK;
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

// status[0..1] of the launch before → first_error[0..1] if that is still clear; status cleared for the next launch
__global__ void status_retire_kernel(int32_t* status, int32_t* first_error) {
  if (threadIdx.x != 0) return;
  const int32_t code = status[0];
  if (code != 0 && first_error != nullptr && first_error[0] == 0) {
    first_error[1] = status[1];
    first_error[0] = code;
  }
  status[1] = 0;
  status[0] = 0;
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
  const int32_t* held;                   // optional [world * chunks_per_rank]: > 0 = never deliver, < 0 = deliver that many
                                         // microseconds late (test and measurement hooks)
  const unsigned long long* stamp;       // optional: wall-clock stamp of the op's start
  unsigned long long ticks_per_chunk;
  unsigned long long max_delay_ticks;    // > 0: seeded random extra delay per (peer, chunk), see producer_delay_ticks
  unsigned long long ticks_per_us;       // wall-clock ticks per microsecond (for the per-chunk delays in `held`)
  uint32_t delay_seed;
  long long chunk_bytes, rank_bytes;
  int world, rank, chunks_per_rank, flag_value;
};

// Race provocation (the reference sleeps in front of its producer with probability 0.7 when it runs "for
// correctness", kernels/nvidia/allgather.py:72-77,118-121): chunk `chunk_pos` is held back by a pseudo-random time
// below max_ticks in about 7 of 10 cases, by none otherwise. A function of (seed, chunk) alone, so every workgroup of a
// peer's block row holds the chunk for the same time and a run can be repeated.
__device__ __forceinline__ unsigned long long producer_delay_ticks(uint32_t seed, int chunk_pos, unsigned long long max_ticks) {
  uint32_t h = seed ^ (0x9e3779b9u * (uint32_t)(chunk_pos + 1));
  h ^= h >> 16; h *= 0x7feb352du; h ^= h >> 15; h *= 0x846ca68bu; h ^= h >> 16;
  if ((h & 1023u) >= 717u) return 0;
  return (unsigned long long)(h >> 10) % max_ticks;
}

__global__ __launch_bounds__(256) __attribute__((amdgpu_num_vgpr(24))) void producer_push_kernel(const PushParams p) {
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
    const int hold = p.held != nullptr ? p.held[chunk_pos] : 0;
    if (hold > 0) continue;
    // Pacing: over a link the last byte of the peer's chunk c lands (c+1) chunk times after the start. The rows
    // are therefore copied when their turn comes (they are "on the wire" once chunk c-1 is through) and the flag is
    // held back until the chunk's arrival time: what the consumer sees is a chunk that is complete at that time.
    if (p.stamp != nullptr && c > 0) {
      if (threadIdx.x == 0) {
        const unsigned long long due = (unsigned long long)c * p.ticks_per_chunk;
        while (true) {
          const unsigned long long now = wall_clock64();
          if (now - t0 >= due || now - begin >= due) break;
          __builtin_amdgcn_s_sleep(16);
        }
      }
      __syncthreads();
    }
    if (p.max_delay_ticks != 0 || hold < 0) {
      if (threadIdx.x == 0) {
        unsigned long long wait = p.max_delay_ticks != 0 ? producer_delay_ticks(p.delay_seed, chunk_pos, p.max_delay_ticks) : 0;
        if (hold < 0) wait += (unsigned long long)(-(long long)hold) * p.ticks_per_us;   // a straggler: this chunk is late by -hold us
        const unsigned long long from = wall_clock64();
        while (wall_clock64() - from < wait) __builtin_amdgcn_s_sleep(16);   // (ends by itself: the clock only moves forward)
      }
      __syncthreads();
    }
    // Two loads in flight per lane: more would cost the registers that let these waves sit beside a GEMM wave
    // (the kernel is held to 24 registers per lane; the GEMM's wave takes up to 488 of the SIMD's 512).
    // Addresses are a wave-uniform chunk base plus a 32-bit byte offset (chunks are below 4 GiB): one register
    // per lane instead of a 64-bit pointer per load.
    const unsigned char* const sbase = (const unsigned char*)src + (long long)c * p.chunk_bytes;
    unsigned char* const dbase = (unsigned char*)dst + (long long)c * p.chunk_bytes;
    const uint32_t nbytes = (uint32_t)p.chunk_bytes;
    const uint32_t stride = gridDim.x * 256u * 16u;
    auto put = [&](uint32_t off, const int4v v) { __builtin_nontemporal_store(v, (int4v*)(dbase + off)); };
    uint32_t off = (blockIdx.x * 256u + threadIdx.x) * 16u;
    // (the host keeps chunk_bytes + 4 * stride below 2^32, so the offsets cannot wrap)
    for (; off + stride < nbytes; off += 2 * stride) {
      const int4v v0 = __builtin_nontemporal_load((const int4v*)(sbase + off));
      const int4v v1 = __builtin_nontemporal_load((const int4v*)(sbase + off + stride));
      put(off, v0);
      put(off + stride, v1);
    }
    for (; off < nbytes; off += stride) put(off, __builtin_nontemporal_load((const int4v*)(sbase + off)));
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
      if (p.stamp != nullptr) {
        const unsigned long long due = (unsigned long long)(c + 1) * p.ticks_per_chunk;
        while (true) {
          const unsigned long long now = wall_clock64();
          if (now - t0 >= due || now - begin >= due) break;
          __builtin_amdgcn_s_sleep(8);
        }
      }
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

}  // namespace tdist

using namespace tdist;

extern "C" {

int tdist_version(void) { return 100; }

const char* tdist_last_error_string(void) { return g_err; }

int tdist_init(void) {
  const DeviceInfo& di = device_info();
  if (di.ok != 1) return fail(TDIST_ERR_DEVICE, "tdist_init: current device is not a gfx950 GPU");
  // where the workgroups of a grid land (the split-round exchange of the GEMMs stays within one XCD's L2 only when
  // this has been seen to hold on this device)
  if (int rc = probe_xcd_round_robin()) return rc;
  // the address of the current device's copy of the library's built-in scratch (tdist_moe_scatter_index_static), so
  // that a caller that may not run set-up work later (under graph capture) finds it ready
  return moe_static_scratch_init();
}

int tdist_debug_set(int key, int value) {
  if (key < 0 || key >= TDIST_DEBUG_NUM_KEYS) return fail(TDIST_ERR_INVALID, "tdist_debug_set: key %d outside [0, %d)", key, TDIST_DEBUG_NUM_KEYS);
  debug_init();
  g_debug[key].store(value < 0 ? -1 : value, std::memory_order_relaxed);
  return TDIST_OK;
}

int tdist_debug_get(int key) { return debug_get(key); }

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

int tdist_status_retire(int32_t* status, int32_t* first_error, void* stream) {
  if (!status) return fail(TDIST_ERR_INVALID, "tdist_status_retire: null status");
  hipLaunchKernelGGL(status_retire_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, status, first_error);
  return launch_status("tdist_status_retire");
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
                              uint32_t delay_seed, int64_t max_delay_ns, int workgroups_per_peer, void* stream) {
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
  p.max_delay_ticks = 0;
  p.ticks_per_us = 0;
  if (held != nullptr) {
    const int khz = wall_clock_khz();
    if (khz <= 0) return fail(TDIST_ERR_DEVICE, "%s: cannot read the wall clock rate", who);
    p.ticks_per_us = (unsigned long long)khz / 1000ull;
  }
  p.delay_seed = delay_seed;
  if (max_delay_ns < 0 || max_delay_ns * cpr > 100000000)
    return fail(TDIST_ERR_INVALID, "%s: max_delay_ns %lld x %lld chunks outside [0, 100 ms]", who, (long long)max_delay_ns, (long long)cpr);
  if (max_delay_ns > 0) {
    const int khz = wall_clock_khz();
    if (khz <= 0) return fail(TDIST_ERR_DEVICE, "%s: cannot read the wall clock rate", who);
    p.max_delay_ticks = (unsigned long long)((double)max_delay_ns * 1e-6 * (double)khz);
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

}  // extern "C"
