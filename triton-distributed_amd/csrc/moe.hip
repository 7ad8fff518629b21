// (c) MoE low-latency dispatch / combine permute on one GPU.
//
// Index construction (splits, cumsum, stable scatter index, gather index) is a stable counting sort
// of the flat [T*topk] expert ids, restating in parallel form what the reference does with
//   torch.bincount / cumsum / argsort(stable).argsort()      test/nvidia/test_all_to_all.py:42-46,95-96,314
//   calc_gather_index                                         test/nvidia/test_all_to_all.py:49-92
// One launch when the ids fit one co-resident grid (moe_index_fused_kernel: per-block histograms, a grid-wide
// rendezvous, then every block derives its own prefixes and ranks its ids), else three launches (per-block
// histograms, scan, per-block ranking). Inside a wave the rank of an entry among equal ids is found with ballots
// (one per id bit), so no sort is involved and the order of equal ids is their flat order (stability).
//
// Row movement restates all_to_all_kernel (kernels/nvidia/low_latency_all_to_all.py:56-103): the rows
// of destination d are contiguous in the sorted order, and land in that destination's receive slot.
#include <stdlib.h>

#include <mutex>

#include "common.h"

namespace tdist {

constexpr int kMoeThreads = 256;              // 4 waves
constexpr int kMoeItemsPerBlock = 256;        // ids ranked by one block (64 per wave: one pass)
constexpr int kMoeMaxExperts = 4096;          // LDS: 4 waves * G * 4 B
constexpr int kScanThreads = 1024;

__host__ __device__ static inline int id_bits(int g) {
  int b = 1;
  while ((1 << b) < g) ++b;
  return b;
}

// hist[b][g] = #ids equal to g among block b's items.
__global__ __launch_bounds__(kMoeThreads) void moe_hist_kernel(const int32_t* __restrict__ ids, int64_t n, int G,
                                                              int32_t* __restrict__ hist,
                                                              int32_t* __restrict__ scan_counter) {
  extern __shared__ int32_t s_hist[];
  if (blockIdx.x == 0 && threadIdx.x == 0) *scan_counter = 0;  // arrival counter of the scan that follows
  for (int g = threadIdx.x; g < G; g += kMoeThreads) s_hist[g] = 0;
  __syncthreads();
  const int64_t base = (int64_t)blockIdx.x * kMoeItemsPerBlock;
#pragma unroll
  for (int u = 0; u < kMoeItemsPerBlock / kMoeThreads; ++u) {
    const int64_t i = base + u * kMoeThreads + threadIdx.x;
    if (i < n) {
      const int e = ids[i];
      if (e >= 0 && e < G) atomicAdd(&s_hist[e], 1);
    }
  }
  __syncthreads();
  int32_t* out = hist + (int64_t)blockIdx.x * G;
  for (int g = threadIdx.x; g < G; g += kMoeThreads) out[g] = s_hist[g];
}

// Turns hist[b][g] into the exclusive prefix over b, writes splits[g] and cumsum[0..G]. One workgroup per 256
// columns (a single workgroup would move the whole table through one compute unit: 19 us for 2048 groups x 32
// blocks), four row ranges per column; the workgroup that finishes last adds up the column totals. `counter` is zero
// on entry (the histogram kernel clears it) and zero again on exit.
// splits is never NULL here: the host substitutes a row of the workspace when the caller has none.
constexpr int kScanCols = 256, kScanParts = kScanThreads / kScanCols;
__global__ __launch_bounds__(kScanThreads) void moe_scan_kernel(int32_t* __restrict__ hist, int num_blocks, int G,
                                                               int32_t* __restrict__ splits,
                                                               int32_t* __restrict__ cumsum,
                                                               int32_t* __restrict__ counter) {
  __shared__ int32_t s_tot[kScanParts][kScanCols];
  __shared__ int32_t s_part[kScanThreads];
  __shared__ int s_last;
  const int c = threadIdx.x % kScanCols, q = threadIdx.x / kScanCols;
  const int g = blockIdx.x * kScanCols + c;
  const int rows_per = (num_blocks + kScanParts - 1) / kScanParts;
  const int b_begin = min(q * rows_per, num_blocks), b_end = min(b_begin + rows_per, num_blocks);
  constexpr int kDepth = 32;  // loads in flight per thread and round
  int32_t h[kDepth];
  int32_t total = 0;
  if (g < G) {
    for (int b0 = b_begin; b0 < b_end; b0 += kDepth) {
#pragma unroll
      for (int u = 0; u < kDepth; ++u) h[u] = b0 + u < b_end ? hist[(int64_t)(b0 + u) * G + g] : 0;
#pragma unroll
      for (int u = 0; u < kDepth; ++u) total += h[u];
    }
  }
  s_tot[q][c] = total;
  __syncthreads();
  int32_t run = 0, column = 0;
#pragma unroll
  for (int p = 0; p < kScanParts; ++p) {
    if (p < q) run += s_tot[p][c];
    column += s_tot[p][c];
  }
  if (g < G) {
    if (q == 0) splits[g] = column;
    const bool kept = b_end - b_begin <= kDepth;  // the only round's values are still in registers
    for (int b0 = b_begin; b0 < b_end; b0 += kDepth) {
      if (!kept) {
#pragma unroll
        for (int u = 0; u < kDepth; ++u) h[u] = b0 + u < b_end ? hist[(int64_t)(b0 + u) * G + g] : 0;
      }
#pragma unroll
      for (int u = 0; u < kDepth; ++u) {
        if (b0 + u < b_end) hist[(int64_t)(b0 + u) * G + g] = run;
        run += h[u];
      }
    }
  }
  // ---- the last workgroup: cumsum over all columns -------------------------------------------
  if (gridDim.x > 1) {
    __syncthreads();
    if (threadIdx.x == 0) {
      __threadfence();  // this workgroup's splits are visible before its arrival is
      const int arrived = atomicAdd(counter, 1);
      s_last = arrived == (int)gridDim.x - 1;
      if (s_last) {
        *counter = 0;
        __threadfence();
      }
    }
    __syncthreads();
    if (!s_last) return;
  }
  const int per = (G + kScanThreads - 1) / kScanThreads;  // consecutive columns per thread
  const int g0 = threadIdx.x * per;
  int32_t local_total = 0;
  for (int j = 0; j < per; ++j)
    if (g0 + j < G) local_total += __hip_atomic_load(splits + g0 + j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  s_part[threadIdx.x] = local_total;
  __syncthreads();
  // Hillis-Steele inclusive scan over the per-thread totals.
  for (int off = 1; off < kScanThreads; off <<= 1) {
    int32_t v = (threadIdx.x >= off) ? s_part[threadIdx.x - off] : 0;
    __syncthreads();
    s_part[threadIdx.x] += v;
    __syncthreads();
  }
  int32_t acc = s_part[threadIdx.x] - local_total;  // exclusive prefix of this thread's first column
  if (threadIdx.x == 0) cumsum[0] = 0;
  for (int j = 0; j < per; ++j) {
    const int gg = g0 + j;
    if (gg < G) {
      acc += __hip_atomic_load(splits + gg, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      cumsum[gg + 1] = acc;
    }
  }
}

// Ranks block b's items. base position of expert g for wave w of block b =
//   cumsum[g] + hist[b][g] (items of earlier blocks) + items of earlier waves of this block.
__global__ __launch_bounds__(kMoeThreads) void moe_rank_kernel(const int32_t* __restrict__ ids, int64_t n, int topk,
                                                              int G, int nbits, const int32_t* __restrict__ hist,
                                                              const int32_t* __restrict__ cumsum,
                                                              int32_t* __restrict__ scatter_idx,
                                                              int32_t* __restrict__ gather_idx,
                                                              int32_t* __restrict__ topk_idx) {
  extern __shared__ int32_t s_cnt[];  // [4][G]
  constexpr int kWaves = kMoeThreads / 64;
  constexpr int kPerWave = kMoeItemsPerBlock / kWaves;
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  for (int g = threadIdx.x; g < kWaves * G; g += kMoeThreads) s_cnt[g] = 0;
  __syncthreads();
  const int64_t wbase = (int64_t)blockIdx.x * kMoeItemsPerBlock + wave * kPerWave;
  int32_t* my_cnt = s_cnt + wave * G;
  // Pass 1: per-wave counts.
#pragma unroll
  for (int u = 0; u < kPerWave / 64; ++u) {
    const int64_t i = wbase + u * 64 + lane;
    if (i < n) {
      const int e = ids[i];
      if (e >= 0 && e < G) atomicAdd(&my_cnt[e], 1);
    }
  }
  __syncthreads();
  // Pass 2: counts → base positions (exclusive over waves, plus the block and expert offsets).
  const int32_t* bh = hist + (int64_t)blockIdx.x * G;
  for (int g = threadIdx.x; g < G; g += kMoeThreads) {
    int32_t run = cumsum[g] + bh[g];
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      const int32_t c = s_cnt[w * G + g];
      s_cnt[w * G + g] = run;
      run += c;
    }
  }
  __syncthreads();
  // Pass 3: walk the wave's items in flat order, 64 at a time.
  volatile int32_t* pos = my_cnt;
  const uint64_t lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  for (int u = 0; u < kPerWave / 64; ++u) {
    const int64_t i = wbase + u * 64 + lane;
    int e = -1;
    if (i < n) {
      e = ids[i];
      if (e < 0 || e >= G) e = -1;
    }
    const bool valid = e >= 0;
    uint64_t peers = __ballot(valid);
    for (int b = 0; b < nbits; ++b) {
      const bool bit = (e >> b) & 1;
      const uint64_t m = __ballot(valid && bit);
      peers &= bit ? m : ~m;
    }
    if (valid) {
      const int32_t start = pos[e];
      const int rank_in = __popcll(peers & lt_mask);
      const int32_t p = start + rank_in;
      scatter_idx[i] = p;
      gather_idx[p] = (int32_t)(i / topk);
      if (topk_idx) topk_idx[p] = (int32_t)(i % topk);
    } else if (i < n) {
      scatter_idx[i] = -1;
    }
    // every lane of the wave has read pos[] before the leaders advance it
    __builtin_amdgcn_wave_barrier();
    if (valid && (peers & lt_mask) == 0) pos[e] = pos[e] + __popcll(peers);
    __builtin_amdgcn_wave_barrier();
  }
}

// ---- the same in one launch ---------------------------------------------------------------------
// Block b owns ids [b * kItems, (b+1) * kItems), kPerWave consecutive ones per wave, in flat order.
//   1. every wave counts its ids per expert in its own row of LDS counters; the block's sum goes to hist[b][.];
//   2. rendezvous: every block needs every other block's histogram (cumsum is a prefix over ALL ids), so the blocks
//      wait for each other. That is safe because the host only takes this path when the grid is at most one block per
//      compute unit, i.e. co-resident (ctrl[0] counts arrivals and is put back to zero by the last one, ctrl[1] is a
//      generation number that the last arrival bumps; the wait is bounded all the same: if it ran out, the block leaves
//      without writing, cumsum[0] is set to -1 instead of 0 and ctrl[2] to 1, where it stays). Co-residency is the
//      caller's to guarantee (nothing else on the GPU may hold compute units for good, e.g. a persistent GEMM that
//      waits for flags), so the host takes this form only on request (TDIST_DEBUG_MOE_INDEX_FORM = 2);
//   3. every block adds up the histogram columns (all rows: the split of the expert; rows before its own: its offset
//      within the expert), scans the splits into cumsum, and turns its waves' counters into start positions;
//   4. ranking as in moe_rank_kernel.
// ctrl[0] must be zero on entry and is zero again on exit.
// A block is 8 waves x 256 ids. (One block of 16 waves x 2048 ids for all of a decode step's 32768 ids, with no
// rendezvous at all, was measured 4 x slower: a wave ranks its ids 64 at a time, each pass behind the previous one's
// counter update, and 32 such passes in a row cost more than the trips through memory they save.) A single block
// (up to 2048 ids) skips the rendezvous.
constexpr int kFusedSpinLimit = 1 << 22;
constexpr int kFusedThreads = 512, kFusedPerWave = 256, kFusedItems = kFusedThreads / 64 * kFusedPerWave;

// kRecount (few ids): no rendezvous and no histogram rows in memory at all. Every block counts, beside its own ids,
// everybody else's (the ids in front of its range and those behind it, into two more rows of LDS counters): reading
// all the ids once more per block (131 KB out of the L2 for a decode step's 32768) is cheaper than the three trips
// through memory of the rendezvous, and with nothing to wait for the blocks can be small (512 or 1024 ids: one or two
// ranking passes per wave). Measured for 32768 ids, launch to launch: 8.7 us with 64 blocks of 512 ids (10.5 with 16
// blocks of 2048) against 12.3 with the rendezvous, of which 2.2 us are the first trip to memory, 2.4 the counting
// (64 LDS atomics per thread), 1.9 column sums and scan, 1.0 the ranking; an empty launch is 3.3 us of the total.
// The work grows with blocks x ids, so the host takes this form up to kRecountMaxBlocks blocks of 1024 ids only.
constexpr int kRecountMaxBlocks = 64;

template <int kThreads, int kPerWave, bool kRecount>
__global__ __launch_bounds__(kThreads) void moe_index_fused_kernel(const int32_t* __restrict__ ids, int64_t n, int topk,
                                                                  int G, int nbits, int32_t* hist, int32_t* ctrl,
                                                                  int32_t* __restrict__ splits,
                                                                  int32_t* __restrict__ cumsum,
                                                                  int32_t* __restrict__ scatter_idx,
                                                                  int32_t* __restrict__ gather_idx,
                                                                  int32_t* __restrict__ topk_idx) {
  constexpr int kWaves = kThreads / 64, kItems = kWaves * kPerWave, kPasses = kPerWave / 64;
  extern __shared__ int32_t s_mem[];  // [kWaves][G] wave counters, [G] column sums, kRecount: [2][G] ids before / behind
  int32_t* const s_cnt = s_mem;
  int32_t* const s_col = s_mem + kWaves * G;
  int32_t* const s_out = s_col + G;
  __shared__ int32_t s_part[kWaves];
  __shared__ int s_flag;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int B = gridDim.x, b = blockIdx.x;
  int gen0 = 0;
  if (!kRecount && B > 1 && threadIdx.x == 0) gen0 = __hip_atomic_load(ctrl + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  // the wave's ids first: the loads are in flight while the counters are cleared
  const int64_t wbase = (int64_t)b * kItems + (int64_t)wave * kPerWave;
  int e_of[kPasses];
#pragma unroll
  for (int u = 0; u < kPasses; ++u) {
    const int64_t i = wbase + u * 64 + lane;
    e_of[u] = i < n ? ids[i] : -1;
  }
  // kRecount: the other blocks' ids, four per load, kVecBatch loads in flight (the ranges are multiples of four ids,
  // so a vector lies on one side of this block's range or inside it). The first batch (all of a decode step's ids)
  // goes out here, together with the block's own ids, so that there is one wait for memory and not two.
  constexpr int kVecBatch = kRecount ? 16 : 1;
  const int64_t own_lo = (int64_t)b * kItems, own_hi = own_lo + kItems;
  const int64_t n_vec = (n + 3) / 4;
  int4v q[kVecBatch];
  auto load_others = [&](int64_t v0) {
#pragma unroll
    for (int u = 0; u < kVecBatch; ++u) {
      const int64_t vi = v0 + (int64_t)u * kThreads;
      const bool mine = vi * 4 >= own_lo && vi * 4 < own_hi;
      q[u] = int4v{-1, -1, -1, -1};
      if (vi < n_vec && !mine) {
        if (vi * 4 + 3 < n) q[u] = ((const int4v*)ids)[vi];
        else
          for (int j = 0; j < 4; ++j) q[u][j] = vi * 4 + j < n ? ids[vi * 4 + j] : -1;
      }
    }
  };
  // (no branch per id: one unsigned compare, and an id out of range counts into a word of its own lane behind the
  // counters; with 64 ids per lane every instruction per id is a quarter of a microsecond per launch)
  int32_t* const s_trash = s_mem + (kWaves + 3) * G + lane;
  auto count_others = [&](int64_t v0) {
#pragma unroll
    for (int u = 0; u < kVecBatch; ++u) {
      const int64_t vi = v0 + (int64_t)u * kThreads;
      int32_t* const row = s_out + (vi * 4 < own_lo ? 0 : G);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t x = (uint32_t)q[u][j];
        atomicAdd(x < (uint32_t)G ? row + x : s_trash, 1);
      }
    }
  };
  if constexpr (kRecount) {
    if (B > 1) load_others(threadIdx.x);
  }
  for (int g = threadIdx.x; g < (kWaves + (kRecount ? 3 : 0)) * G; g += kThreads) s_cnt[g] = 0;
  __syncthreads();
  // 1. per-wave counts
  int32_t* const my_cnt = s_cnt + wave * G;
#pragma unroll
  for (int u = 0; u < kPasses; ++u) {
    if (e_of[u] < 0 || e_of[u] >= G) e_of[u] = -1;
    if (e_of[u] >= 0) atomicAdd(&my_cnt[e_of[u]], 1);
  }
  if constexpr (kRecount) {
    if (B > 1) {
      count_others(threadIdx.x);
      for (int64_t v0 = threadIdx.x + (int64_t)kVecBatch * kThreads; v0 < n_vec; v0 += (int64_t)kVecBatch * kThreads) {
        load_others(v0);
        count_others(v0);
      }
    }
  }
  __syncthreads();
  if (!kRecount && B > 1) {
    for (int g = threadIdx.x; g < G; g += kThreads) {
      int32_t t = 0;
#pragma unroll
      for (int w = 0; w < kWaves; ++w) t += s_cnt[w * G + g];
      // (device-coherent store: it goes through to memory, so no cache has to be written back before the arrival)
      __hip_atomic_store(hist + (int64_t)b * G + g, t, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    // 2. rendezvous. No fence on either side (a release or acquire fence at device scope writes back or invalidates
    // the whole L2 of this XCD, microseconds after a kernel that left it full of dirty lines): every wave waits for
    // its own coherent stores, then the arrival is counted; the histograms are read back with coherent loads.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
      int ok = 1;
      if (__hip_atomic_fetch_add(ctrl, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == B - 1) {
        __hip_atomic_store(ctrl, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(ctrl + 1, gen0 + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      } else {
        ok = 0;
        for (int it = 0; it < kFusedSpinLimit; ++it) {
          if (__hip_atomic_load(ctrl + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != gen0) {
            ok = 1;
            break;
          }
          __builtin_amdgcn_s_sleep(1);
        }
      }
      s_flag = ok;
    }
    __syncthreads();
    if (!s_flag) {
      // Reported in a word nobody else writes (block 0, if it gets through later, puts cumsum[0] back to 0): ctrl[2]
      // stays non-zero from the first expiry on until the caller clears it.
      if (threadIdx.x == 0) {
        __hip_atomic_store(ctrl + 2, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        cumsum[0] = -1;
      }
      return;
    }
  }
  // 3. column sums: s_col[g] = ids of expert g in all blocks; the blocks before this one go into wave 0's start
  for (int g = threadIdx.x; g < G; g += kThreads) {
    int32_t total = 0, before = 0;
    if (kRecount && B > 1) {
      before = s_out[g];
      total = before + s_out[G + g];
#pragma unroll
      for (int w = 0; w < kWaves; ++w) total += s_cnt[w * G + g];
    } else if (B > 1) {
      for (int r = 0; r < B; ++r) {
        const int32_t h = __hip_atomic_load(hist + (int64_t)r * G + g, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        total += h;
        before += r < b ? h : 0;
      }
    }
    // wave starts within the expert: blocks before, then the earlier waves of this block
    int32_t run = before;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      const int32_t c = s_cnt[w * G + g];
      s_cnt[w * G + g] = run;
      run += c;
    }
    s_col[g] = B > 1 ? total : run;
  }
  __syncthreads();
  // exclusive scan of s_col over the experts: consecutive experts per thread, an inclusive scan of the threads' totals
  // within the wave by shuffles, then the waves' totals through LDS
  const int per = (G + kThreads - 1) / kThreads;
  const int g0 = threadIdx.x * per;
  int32_t local_total = 0;
  for (int j = 0; j < per; ++j)
    if (g0 + j < G) local_total += s_col[g0 + j];
  int32_t incl = local_total;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int32_t t = __shfl_up(incl, off);
    if (lane >= off) incl += t;
  }
  if (lane == 63) s_part[wave] = incl;
  __syncthreads();
  int32_t acc = incl - local_total;  // ids of the experts before this thread's first one
#pragma unroll
  for (int w = 0; w < kWaves; ++w) acc += w < wave ? s_part[w] : 0;
  if (b == 0 && threadIdx.x == 0) cumsum[0] = 0;
  for (int j = 0; j < per; ++j) {
    const int g = g0 + j;
    if (g < G) {
      const int32_t c = s_col[g];
      if (b == 0) {
        if (splits) splits[g] = c;
        cumsum[g + 1] = acc + c;
      }
      // the expert's first position goes into every wave's start
#pragma unroll
      for (int w = 0; w < kWaves; ++w) s_cnt[w * G + g] += acc;
      acc += c;
    }
  }
  __syncthreads();
  if (scatter_idx == nullptr) return;  // splits and cumsum only
  // 4. walk the wave's ids in flat order, 64 at a time
  volatile int32_t* pos = my_cnt;
  const uint64_t lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
#pragma unroll
  for (int u = 0; u < kPasses; ++u) {
    if (wbase + u * 64 >= n) break;  // (the whole wave is past the end)
    const int64_t i = wbase + u * 64 + lane;
    const int e = e_of[u];
    const bool valid = e >= 0;
    uint64_t peers = __ballot(valid);
    for (int bit = 0; bit < nbits; ++bit) {
      const bool one = (e >> bit) & 1;
      const uint64_t m = __ballot(valid && one);
      peers &= one ? m : ~m;
    }
    if (valid) {
      const int32_t p = pos[e] + __popcll(peers & lt_mask);
      scatter_idx[i] = p;
      gather_idx[p] = (int32_t)(i / topk);
      if (topk_idx) topk_idx[p] = (int32_t)(i % topk);
    } else if (i < n) {
      scatter_idx[i] = -1;
    }
    // every lane of the wave has read pos[] before the leaders advance it
    __builtin_amdgcn_wave_barrier();
    if (valid && (peers & lt_mask) == 0) pos[e] = pos[e] + __popcll(peers);
    __builtin_amdgcn_wave_barrier();
  }
}

// ---- row movement ------------------------------------------------------------------------------

// Finds d with bound[d] <= p < bound[d+1] in a non-decreasing bound[0..W] with bound[W] > p.
__device__ __forceinline__ int find_dest(const int32_t* bound, int stride, int W, int32_t p) {
  int lo = 0, hi = W;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (bound[mid * stride] <= p) lo = mid; else hi = mid;
  }
  return lo;
}

constexpr int kRowsPerWave = 2;
constexpr int kRowsPerBlock = 4 * kRowsPerWave;  // 4 waves

// Copies up to kRowsPerWave rows of n16 16-byte chunks; all loads of a 512-chunk window are issued
// before its stores so each lane keeps up to 16 vectors in flight.
__device__ __forceinline__ void copy_rows_vec(const int4v* const* src, int4v* const* dst, const bool* has, int n16,
                                              int lane) {
  for (int base = 0; base < n16; base += 8 * 64) {
    int4v v[kRowsPerWave][8];
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r) {
      if (has[r]) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int c = base + j * 64 + lane;
          if (c < n16) v[r][j] = __builtin_nontemporal_load(src[r] + c);
        }
      }
    }
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r) {
      if (has[r]) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int c = base + j * 64 + lane;
          if (c < n16) __builtin_nontemporal_store(v[r][j], dst[r] + c);
        }
      }
    }
  }
}

// kFromSlots = false: dispatch (sorted/gathered rows → slots); true: post-process (slots → compact).
// s_bound[d] = first sorted row of destination d, s_bound[W] = total.
template <bool kVec16, bool kFromSlots>
__global__ __launch_bounds__(256) void moe_rows_kernel(const unsigned char* __restrict__ in_rows, int64_t row_bytes,
                                                       const float* __restrict__ in_scales,
                                                       const int32_t* __restrict__ gather_idx,
                                                       const int32_t* __restrict__ counts, int64_t n_rows, int W,
                                                       int Er, int max_m, unsigned char* __restrict__ out_rows,
                                                       float* __restrict__ out_scales,
                                                       int32_t* __restrict__ splits_out) {
  extern __shared__ int32_t s_bound[];  // [W+1]
  if (kFromSlots) {
    // counts = splits[G]: per-destination totals, then a serial prefix (W is small).
    for (int d = threadIdx.x; d < W; d += 256) {
      int32_t t = 0;
      for (int j = 0; j < Er; ++j) t += counts[d * Er + j];
      s_bound[d + 1] = t;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      s_bound[0] = 0;
      for (int d = 0; d < W; ++d) s_bound[d + 1] += s_bound[d];
    }
  } else {
    // counts = cumsum[G+1]
    for (int d = threadIdx.x; d <= W; d += 256) s_bound[d] = counts[d * Er];
    if (splits_out && blockIdx.x == 0) {
      const int G = W * Er;
      for (int g = threadIdx.x; g < G; g += 256) splits_out[g] = counts[g + 1] - counts[g];
    }
  }
  __syncthreads();
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int32_t total = s_bound[W];
  const unsigned char* src[kRowsPerWave];
  unsigned char* dst[kRowsPerWave];
  bool has[kRowsPerWave];
#pragma unroll
  for (int r = 0; r < kRowsPerWave; ++r) {
    const int64_t p = (int64_t)blockIdx.x * kRowsPerBlock + wave * kRowsPerWave + r;
    has[r] = false;
    src[r] = in_rows;
    dst[r] = out_rows;
    if (p >= n_rows || p >= total) continue;
    const int d = find_dest(s_bound, 1, W, (int32_t)p);
    const int64_t in_slot = p - s_bound[d];
    if (in_slot >= max_m) continue;
    const int64_t slot_row = (int64_t)d * max_m + in_slot;
    int64_t src_row, dst_row;
    if (kFromSlots) {
      src_row = slot_row;
      dst_row = p;
    } else {
      src_row = gather_idx ? (int64_t)gather_idx[p] : p;
      dst_row = slot_row;
    }
    has[r] = true;
    src[r] = in_rows + src_row * row_bytes;
    dst[r] = out_rows + dst_row * row_bytes;
    if (in_scales && out_scales && lane == 0) out_scales[dst_row] = in_scales[src_row];
  }
  if (kVec16) {
    copy_rows_vec((const int4v* const*)src, (int4v* const*)dst, has, (int)(row_bytes >> 4), lane);
  } else {
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r)
      if (has[r])
        for (int64_t c = lane; c < row_bytes; c += 64) dst[r][c] = src[r][c];
  }
}

// Token-major dispatch: the row of token t is read once and written to the slot rows of its topk sorted
// positions p = scatter_idx[t*topk + k]. One wave per (token, window of 512 16-byte chunks).
template <bool kVec16>
__global__ __launch_bounds__(256) void moe_dispatch_tokens_kernel(const unsigned char* __restrict__ tokens,
                                                                  int64_t row_bytes, const float* __restrict__ scales,
                                                                  const int32_t* __restrict__ scatter_idx, int topk,
                                                                  const int32_t* __restrict__ cumsum, int64_t n_tokens,
                                                                  int W, int Er, int max_m,
                                                                  unsigned char* __restrict__ slot_rows,
                                                                  float* __restrict__ slot_scales,
                                                                  int32_t* __restrict__ splits_out, int windows) {
  if (splits_out && blockIdx.x == 0) {
    const int G = W * Er;
    for (int g = threadIdx.x; g < G; g += 256) splits_out[g] = cumsum[g + 1] - cumsum[g];
  }
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int64_t unit = (int64_t)blockIdx.x * 4 + wave;
  const int64_t t = unit / windows;
  const int win = (int)(unit - t * windows);
  if (t >= n_tokens) return;
  const unsigned char* src = tokens + t * row_bytes;
  // the row's loads go out first: they do not depend on where the copies land
  const int n16 = (int)(row_bytes >> 4);
  const int base = win * 512;
  int4v v[8];
  if (kVec16) {
    const int4v* s16 = (const int4v*)src;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int c = base + j * 64 + lane;
      if (c < n16) v[j] = s16[c];
    }
  }
  // lane k < topk resolves the slot row of copy k; the W+1 slot boundaries sit one per lane, so the search is
  // register work behind a single load
  int32_t my_dst = -1;
  {
    const int32_t p = lane < topk ? scatter_idx[t * topk + lane] : -1;
    if (W < 64) {
      const int32_t bound = lane <= W ? cumsum[lane * Er] : 0x7fffffff;
      const int32_t total = __builtin_amdgcn_readlane(bound, W);
      int d = 0;
      int32_t first = __builtin_amdgcn_readlane(bound, 0);
      for (int i = 1; i < W; ++i) {
        const int32_t b = __builtin_amdgcn_readlane(bound, i);
        if (b <= p) {
          d = i;
          first = b;
        }
      }
      if (p >= 0 && p < total && p - first < max_m) my_dst = d * max_m + (p - first);
    } else if (p >= 0 && p < cumsum[W * Er]) {
      const int d = find_dest(cumsum, Er, W, p);
      const int32_t in_slot = p - cumsum[d * Er];
      if (in_slot < max_m) my_dst = d * max_m + in_slot;
    }
    if (win == 0 && my_dst >= 0 && scales) slot_scales[my_dst] = scales[t];
  }
  if (kVec16) {
    for (int k = 0; k < topk; ++k) {
      const int32_t dst_row = __shfl(my_dst, k);
      if (dst_row < 0) continue;
      int4v* d16 = (int4v*)(slot_rows + (int64_t)dst_row * row_bytes);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int c = base + j * 64 + lane;
        if (c < n16) __builtin_nontemporal_store(v[j], d16 + c);
      }
    }
  } else {
    for (int k = 0; k < topk; ++k) {
      const int32_t dst_row = __shfl(my_dst, k);
      if (dst_row < 0) continue;
      unsigned char* dst = slot_rows + (int64_t)dst_row * row_bytes;
      for (int64_t c = (int64_t)win * 8192 + lane; c < row_bytes && c < (int64_t)(win + 1) * 8192; c += 64) dst[c] = src[c];
    }
  }
}

// ---- dispatch straight from the expert ids: index build and row movement in one launch ---------------------------
// For a decode step's worth of ids (up to kFusedDispatchMaxIds) the index build is cheaper redone by everybody than
// waited for: as in the recounting form of moe_index_fused_kernel, every workgroup counts ALL ids itself (its own
// tokens' per wave, the ids in front of its range and behind it into two more rows of LDS counters), so it knows the
// splits, their prefix sums and the rank of each of its own (token, k) entries without any exchange, and can place its
// rows at once. The row loads go out before the counting starts, so the counting runs while they are in flight. As
// by-products the workgroups write what tdist_moe_scatter_index writes: scatter_idx and gather_idx for their own
// entries, workgroup 0 the splits and cumsum.
// A workgroup is kFdWaves waves; wave w stands for (token, 8 KB window) unit w of the workgroup, as in
// moe_dispatch_tokens_kernel. The window-0 wave of a token counts and ranks that token's ids.
constexpr int kFdWaves = 16, kFdThreads = kFdWaves * 64;
constexpr int64_t kFusedDispatchMaxIds = 65536;

template <bool kVec16>
__global__ __launch_bounds__(kFdThreads) void moe_dispatch_fused_kernel(
    const unsigned char* __restrict__ tokens, int64_t row_bytes, const float* __restrict__ scales,
    const int32_t* __restrict__ ids, int topk, int64_t n_tokens, int G, int nbits, int W, int Er, int max_m, int windows,
    unsigned char* __restrict__ slot_rows, float* __restrict__ slot_scales, int32_t* __restrict__ splits_out,
    int32_t* __restrict__ splits, int32_t* __restrict__ cumsum, int32_t* __restrict__ scatter_idx,
    int32_t* __restrict__ gather_idx) {
  // [3][G] counters: ids in front of this workgroup's range, its own, ids behind it; [G + 1] expert starts (cumsum);
  // then this workgroup's own ids in flat order, padded to a multiple of four with -1
  extern __shared__ int32_t s_fd[];
  int32_t* const s_before = s_fd;
  int32_t* const s_own = s_fd + G;
  int32_t* const s_behind = s_fd + 2 * G;
  int32_t* const s_start = s_fd + 3 * G;
  int32_t* const s_ids = s_start + ((G + 1 + 3) & ~3);
  __shared__ int32_t s_part[kFdWaves];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int tokens_per_block = kFdWaves / windows;
  const int64_t unit = (int64_t)blockIdx.x * kFdWaves + wave;
  const int64_t t = unit / windows;
  const int win = (int)(unit - t * windows);
  const bool live = t < n_tokens;
  // 1. this token's ids, and everybody else's four at a time
  const int64_t n = n_tokens * topk;
  const int own_n = tokens_per_block * topk;
  const int64_t own_lo = (int64_t)blockIdx.x * own_n, own_hi = own_lo + own_n;
  const int own_f = (wave / windows) * topk + lane;   // this lane's entry among the workgroup's own, in flat order
  int e = -1;
  if (live && lane < topk) e = ids[t * topk + lane];
  if (e < 0 || e >= G) e = -1;
  constexpr int kBatch = 8;
  const int64_t n_vec = (n + 3) / 4;
  const bool vec_ok = (reinterpret_cast<uintptr_t>(ids) & 15u) == 0;
  int4v q[kBatch];
  auto load_others = [&](int64_t v0) {
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int64_t vi = v0 + (int64_t)u * kFdThreads;
      q[u] = int4v{-1, -1, -1, -1};
      if (vi < n_vec) {
        if (vec_ok && vi * 4 + 3 < n) q[u] = ((const int4v*)ids)[vi];
        else
          for (int j = 0; j < 4; ++j) q[u][j] = vi * 4 + j < n ? ids[vi * 4 + j] : -1;
      }
    }
  };
  // (no branch per id: a vector that lies wholly in front of the workgroup's range or behind it, as all but one or
  // two do, takes one unsigned compare per id, and what is not counted goes into a word of the lane's own)
  int32_t* const s_trash = s_ids + ((own_n + 4 + 3) & ~3) + lane;
  auto count_others = [&](int64_t v0) {
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int64_t vi = v0 + (int64_t)u * kFdThreads;
      const int64_t i0 = vi * 4;
      if (i0 + 3 < own_lo || i0 >= own_hi) {
        int32_t* const row = i0 < own_lo ? s_before : s_behind;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t x = (uint32_t)q[u][j];
          atomicAdd(x < (uint32_t)G ? row + x : s_trash, 1);
        }
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int64_t i = i0 + j;
          const int x = q[u][j];
          if (x >= 0 && x < G && (i < own_lo || i >= own_hi)) atomicAdd(i < own_lo ? &s_before[x] : &s_behind[x], 1);
        }
      }
    }
  };
  load_others(threadIdx.x);
  // the row's loads go out behind the ids' (loads return in order, and the counting only needs the ids: it runs while
  // the row is on its way)
  const int n16 = (int)(row_bytes >> 4);
  const int base = win * 512;
  int4v v[8];
  if (kVec16 && live) {
    const int4v* s16 = (const int4v*)(tokens + t * row_bytes);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int c = base + j * 64 + lane;
      if (c < n16) v[j] = s16[c];
    }
  }
  for (int g = threadIdx.x; g < 3 * G; g += kFdThreads) s_fd[g] = 0;
  if (win == 0 && lane < topk) s_ids[own_f] = e;
  if (threadIdx.x < 4) s_ids[own_n + threadIdx.x] = -1;
  __syncthreads();
  if (e >= 0 && win == 0) atomicAdd(&s_own[e], 1);
  count_others(threadIdx.x);
  for (int64_t v0 = threadIdx.x + (int64_t)kBatch * kFdThreads; v0 < n_vec; v0 += (int64_t)kBatch * kFdThreads) {
    load_others(v0);
    count_others(v0);
  }
  __syncthreads();
  // 3. the splits (ids in front + own + behind) and their exclusive scan over the experts: consecutive experts per
  // thread, the threads' totals within the wave by shuffles, the waves' through LDS
  const int per = (G + kFdThreads - 1) / kFdThreads;
  const int g0 = threadIdx.x * per;
  int32_t local_total = 0;
  for (int j = 0; j < per; ++j)
    if (g0 + j < G) local_total += s_before[g0 + j] + s_own[g0 + j] + s_behind[g0 + j];
  int32_t incl = local_total;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int32_t up = __shfl_up(incl, off);
    if (lane >= off) incl += up;
  }
  if (lane == 63) s_part[wave] = incl;
  __syncthreads();
  int32_t acc = incl - local_total;
#pragma unroll
  for (int w = 0; w < kFdWaves; ++w) acc += w < wave ? s_part[w] : 0;
  if (threadIdx.x == 0 && blockIdx.x == 0) cumsum[0] = 0;
  for (int j = 0; j < per; ++j) {
    const int g = g0 + j;
    if (g < G) {
      const int32_t c = s_before[g] + s_own[g] + s_behind[g];
      if (blockIdx.x == 0) {
        if (splits) splits[g] = c;
        if (splits_out) splits_out[g] = c;
        cumsum[g + 1] = acc + c;
      }
      s_start[g] = acc;
      acc += c;
    }
  }
  __syncthreads();
  if (!live) return;
  // 4. the sorted position of this token's k-th entry (lane k): the expert's start, the ids in front of the workgroup's
  // range, and the workgroup's own entries before this one in flat order; then its slot row
  int32_t my_dst = -1;
  if (e >= 0) {
    int32_t earlier = 0;
    for (int f = 0; f < own_f; f += 4) {
      const int4v o = *(const int4v*)(s_ids + f);
#pragma unroll
      for (int j = 0; j < 4; ++j) earlier += (f + j < own_f && o[j] == e) ? 1 : 0;
    }
    const int32_t p = s_start[e] + s_before[e] + earlier;
    if (win == 0) {
      scatter_idx[t * topk + lane] = p;
      gather_idx[p] = (int32_t)t;
    }
    const int d = e / Er;
    const int32_t in_slot = p - s_start[d * Er];
    if (in_slot < max_m) my_dst = d * max_m + in_slot;
    if (win == 0 && my_dst >= 0 && scales) slot_scales[my_dst] = scales[t];
  } else if (lane < topk && win == 0) {
    scatter_idx[t * topk + lane] = -1;
  }
  // 5. the copies
  if (kVec16) {
    for (int k = 0; k < topk; ++k) {
      const int32_t dst_row = __shfl(my_dst, k);
      if (dst_row < 0) continue;
      int4v* d16 = (int4v*)(slot_rows + (int64_t)dst_row * row_bytes);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int c = base + j * 64 + lane;
        if (c < n16) __builtin_nontemporal_store(v[j], d16 + c);
      }
    }
  } else {
    const unsigned char* src = tokens + t * row_bytes;
    for (int k = 0; k < topk; ++k) {
      const int32_t dst_row = __shfl(my_dst, k);
      if (dst_row < 0) continue;
      unsigned char* dst = slot_rows + (int64_t)dst_row * row_bytes;
      for (int64_t c = (int64_t)win * 8192 + lane; c < row_bytes && c < (int64_t)(win + 1) * 8192; c += 64) dst[c] = src[c];
    }
  }
}

// ---- online e4m3 quantisation in groups of 128 columns -----------------------------------------------------
// Follows _quant_kernel of the reference's tutorials/04-deepseek-infer-all2all.py (:309-329) and its fused form in
// the dispatch kernel (:180-200): per group, scale = max|x| (as fp32) * fp32(1/448), q = e4m3(float(x) / scale).
// A group whose values are all zero divides 0 by 0 there and so it does here (NaN bytes, scale 0).
constexpr int kQuantGroup = 128;

// One lane's 16 consecutive bf16 columns (two 16-byte vectors) → 16 e4m3 bytes; the 8 lanes of a group share the scale.
__device__ __forceinline__ int4v quant16_bf16_e4m3(const int4v& x0, const int4v& x1, float* scale_out) {
  float f[16];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    f[2 * j] = BF16::lo((uint32_t)x0[j]);
    f[2 * j + 1] = BF16::hi((uint32_t)x0[j]);
    f[8 + 2 * j] = BF16::lo((uint32_t)x1[j]);
    f[8 + 2 * j + 1] = BF16::hi((uint32_t)x1[j]);
  }
  float amax = 0.f;
#pragma unroll
  for (int j = 0; j < 16; ++j) amax = fmaxf(amax, fabsf(f[j]));
  amax = fmaxf(amax, __shfl_xor(amax, 1));
  amax = fmaxf(amax, __shfl_xor(amax, 2));
  amax = fmaxf(amax, __shfl_xor(amax, 4));
  const float scale = amax * (float)(1.0 / 448.0);
  *scale_out = scale;
  int4v q;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    int w = 0;
    w = __builtin_amdgcn_cvt_pk_fp8_f32(f[4 * j] / scale, f[4 * j + 1] / scale, w, false);
    w = __builtin_amdgcn_cvt_pk_fp8_f32(f[4 * j + 2] / scale, f[4 * j + 3] / scale, w, true);
    q[j] = w;
  }
  return q;
}

// Stand-alone quantiser: one wave per (row, window of 1024 columns).
__global__ __launch_bounds__(256) void quant_groups_kernel(const unsigned short* __restrict__ x, int64_t n_rows, int hidden,
                                                          int windows, unsigned char* __restrict__ q,
                                                          float* __restrict__ scales) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t unit = (int64_t)blockIdx.x * 4 + wave;
  const int64_t r = unit / windows;
  const int win = (int)(unit - r * windows);
  if (r >= n_rows) return;
  const int col = win * 1024 + lane * 16;
  const bool active = col < hidden;
  int4v x0 = {0, 0, 0, 0}, x1 = {0, 0, 0, 0};
  if (active) {
    const int4v* src = (const int4v*)(x + r * hidden + col);
    x0 = src[0];
    x1 = src[1];
  }
  float scale;
  const int4v v = quant16_bf16_e4m3(x0, x1, &scale);
  if (active) {
    *(int4v*)(q + r * hidden + col) = v;
    if ((lane & 7) == 0) scales[r * (hidden / kQuantGroup) + col / kQuantGroup] = scale;
  }
}

// Token-major dispatch with the quantisation fused in: bf16 token rows in, e4m3 slot rows + one fp32 scale per
// group of 128 columns out. One wave per (token, window of 1024 columns).
__global__ __launch_bounds__(256) void moe_dispatch_quant_kernel(const unsigned short* __restrict__ tokens, int hidden,
                                                                const int32_t* __restrict__ scatter_idx, int topk,
                                                                const int32_t* __restrict__ cumsum, int64_t n_tokens,
                                                                int W, int Er, int max_m,
                                                                unsigned char* __restrict__ slot_rows,
                                                                float* __restrict__ slot_scales,
                                                                int32_t* __restrict__ splits_out, int windows) {
  if (splits_out && blockIdx.x == 0) {
    const int G = W * Er;
    for (int g = threadIdx.x; g < G; g += 256) splits_out[g] = cumsum[g + 1] - cumsum[g];
  }
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t unit = (int64_t)blockIdx.x * 4 + wave;
  const int64_t t = unit / windows;
  const int win = (int)(unit - t * windows);
  if (t >= n_tokens) return;
  const int col = win * 1024 + lane * 16;
  const bool active = col < hidden;
  int4v x0 = {0, 0, 0, 0}, x1 = {0, 0, 0, 0};
  if (active) {
    const int4v* src = (const int4v*)(tokens + t * hidden + col);
    x0 = src[0];
    x1 = src[1];
  }
  // lane k < topk resolves the slot row of copy k (slot boundaries one per lane, as in the unquantised dispatch)
  int32_t my_dst = -1;
  {
    const int32_t p = lane < topk ? scatter_idx[t * topk + lane] : -1;
    if (W < 64) {
      const int32_t bound = lane <= W ? cumsum[lane * Er] : 0x7fffffff;
      const int32_t total = __builtin_amdgcn_readlane(bound, W);
      int d = 0;
      int32_t first = __builtin_amdgcn_readlane(bound, 0);
      for (int i = 1; i < W; ++i) {
        const int32_t b = __builtin_amdgcn_readlane(bound, i);
        if (b <= p) {
          d = i;
          first = b;
        }
      }
      if (p >= 0 && p < total && p - first < max_m) my_dst = d * max_m + (p - first);
    } else if (p >= 0 && p < cumsum[W * Er]) {
      const int d = find_dest(cumsum, Er, W, p);
      const int32_t in_slot = p - cumsum[d * Er];
      if (in_slot < max_m) my_dst = d * max_m + in_slot;
    }
  }
  float scale;
  const int4v v = quant16_bf16_e4m3(x0, x1, &scale);
  const int ng = hidden / kQuantGroup;
  for (int k = 0; k < topk; ++k) {
    const int32_t dst_row = __builtin_amdgcn_readlane(my_dst, k);
    if (dst_row < 0) continue;
    if (active) {
      __builtin_nontemporal_store(v, (int4v*)(slot_rows + (int64_t)dst_row * hidden + col));
      if ((lane & 7) == 0) slot_scales[(int64_t)dst_row * ng + col / kQuantGroup] = scale;
    }
  }
}

// Weighted combine: one wave per (token, window of 64 16-byte column chunks). Lane k < topk resolves the k-th
// source row and its coefficient w[t,k] * scale[row]; the wave then reads the rows eight at a time (all loads
// of a batch in flight before the first add) and accumulates in k order.
// kFp8: rows are e4m3 bytes (16 elements per chunk), else bf16 (8 elements per chunk).
constexpr int kCombineMaxTopk = 32;
constexpr int kCombineWaves = 4;

template <bool kFp8>
__global__ __launch_bounds__(kCombineWaves * 64) void moe_combine_kernel(
    const unsigned char* __restrict__ slot_rows, const float* __restrict__ slot_scales,
    const int32_t* __restrict__ scatter_idx, const float* __restrict__ topk_w, const int32_t* __restrict__ cumsum,
    int64_t n_tokens, int topk, int hidden, int W, int Er, int max_m, int scale_group, int n_windows,
    unsigned short* __restrict__ out) {
  // e4m3 rows: a lane ends up with 32 bytes of output; they go through LDS so that each store instruction of the
  // wave writes one contiguous KiB (16 bytes per lane) instead of every other 16 bytes of two
  __shared__ __attribute__((aligned(16))) unsigned char s_tr[kCombineWaves][kFp8 ? 2048 : 16];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int64_t gw = (int64_t)blockIdx.x * kCombineWaves + wave;
  if (gw >= n_tokens * n_windows) return;
  const int64_t t = gw / n_windows;
  const int win = (int)(gw - t * n_windows);

  // Lane k resolves source row k. The W+1 slot boundaries sit one per lane (a single load, issued together with
  // the index and weight loads), so the search for the destination is register work, not a chain of loads.
  int64_t row = -1;  // source row of the lane's k, -1 = skip
  const int32_t p = lane < topk ? scatter_idx[t * topk + lane] : -1;
  float coef = (lane < topk && topk_w) ? topk_w[t * topk + lane] : 1.0f;
  if (max_m > 0) {
    if (W < 64) {
      const int32_t bound = lane <= W ? cumsum[lane * Er] : 0x7fffffff;
      const int32_t total = __builtin_amdgcn_readlane(bound, W);
      int d = 0;
      int32_t base = __builtin_amdgcn_readlane(bound, 0);
      for (int i = 1; i < W; ++i) {
        const int32_t b = __builtin_amdgcn_readlane(bound, i);
        if (b <= p) {
          d = i;
          base = b;
        }
      }
      if (p >= 0 && p < total && p - base < max_m) row = (int64_t)d * max_m + (p - base);
    } else if (p >= 0 && p < cumsum[W * Er]) {
      const int d = find_dest(cumsum, Er, W, p);
      const int64_t in_slot = p - cumsum[d * Er];
      if (in_slot < max_m) row = (int64_t)d * max_m + in_slot;
    }
  } else if (p >= 0) {
    row = p;
  }
  // scale_group == 0: one scale per row, folded into the coefficient; else one per 128 columns, read per lane below
  if (row >= 0 && slot_scales && scale_group == 0) coef *= slot_scales[row];
  if (row < 0) coef = 0.f;
  constexpr int kElems = kFp8 ? 16 : 8;
  const int64_t row_bytes = (int64_t)hidden * (kFp8 ? 1 : 2);
  const int n16 = hidden / kElems;
  const int c = win * 64 + lane;
  const bool active = c < n16;
  float acc[kElems];
#pragma unroll
  for (int j = 0; j < kElems; ++j) acc[j] = 0.f;
  const int row_lo = (int)(uint32_t)row, row_hi = (int)(row >> 32);
  const bool grouped = kFp8 && slot_scales != nullptr && scale_group > 0;
  const int ng = grouped ? hidden / scale_group : 0;
  const int my_group = grouped ? (c * kElems) / scale_group : 0;
  for (int k0 = 0; k0 < topk; k0 += 8) {
    int4v v[8];
    float cf[8], gs[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int k = min(k0 + j, topk - 1);
      const int64_t r = (int64_t)(((uint64_t)(uint32_t)__builtin_amdgcn_readlane(row_hi, k) << 32) |
                                  (uint32_t)__builtin_amdgcn_readlane(row_lo, k));
      const bool use = (k0 + j < topk) && r >= 0;
      v[j] = (use && active) ? __builtin_nontemporal_load((const int4v*)(slot_rows + r * row_bytes) + c)
                             : int4v{0, 0, 0, 0};
      gs[j] = (grouped && use && active) ? slot_scales[r * ng + my_group] : 1.f;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int k = min(k0 + j, topk - 1);
      cf[j] = (k0 + j < topk) ? __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, coef), k)) : 0.f;
      cf[j] *= gs[j];
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (kFp8) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          float f[4];
          e4m3x4_to_f32((uint32_t)v[j][q], f);
#pragma unroll
          for (int r = 0; r < 4; ++r) acc[4 * q + r] += cf[j] * f[r];
        }
      } else {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          acc[2 * q] += cf[j] * BF16::lo((uint32_t)v[j][q]);
          acc[2 * q + 1] += cf[j] * BF16::hi((uint32_t)v[j][q]);
        }
      }
    }
  }
  int4v w[kElems / 8];
#pragma unroll
  for (int q = 0; q < kElems / 8; ++q)
#pragma unroll
    for (int j = 0; j < 4; ++j) w[q][j] = (int)pack_bf16x2(acc[8 * q + 2 * j], acc[8 * q + 2 * j + 1]);
  unsigned short* const orow = out + t * hidden + (int64_t)win * 64 * kElems;  // first output element of the window
  if (kFp8) {
    TDIST_AS3 unsigned char* tr = (TDIST_AS3 unsigned char*)s_tr[wave];
    *(TDIST_AS3 int4v*)(tr + lane * 32) = w[0];
    *(TDIST_AS3 int4v*)(tr + lane * 32 + 16) = w[kElems / 8 - 1];
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int piece = h * 64 + lane;  // 16-byte piece of the window's 2 KiB of output
      const int4v o = *(TDIST_AS3 int4v*)(tr + piece * 16);
      if (win * 64 + piece / 2 < n16) __builtin_nontemporal_store(o, (int4v*)orow + piece);
    }
  } else {
    if (active) __builtin_nontemporal_store(w[0], (int4v*)orow + lane);
  }
}

// ---- align / sort for the grouped GEMM ------------------------------------------------------------------
// Follows moe_ag_scatter_align_block_size_kernel (csrc/lib/moe_utils.cu:60-165): per rank segment, entries grouped
// by expert in flat order, every group padded to a multiple of block_size, groups and segments laid end to end.
// Built on the stable index of this file with the composite key segment * E + expert: the position of an entry in
// the padded layout is its position in the unpadded sorted order moved by the padding in front of its group.

// keys[i] = (i / per_iter) * E + ids[i], or -1 for an id outside [0, E)
// Also pre-fills sorted_ids[0 .. fill_n) with n (the value padding positions keep; fill_n = 0: the caller has done it).
__global__ __launch_bounds__(256) void moe_align_keys_kernel(const void* __restrict__ ids, int ids_int64, int64_t n,
                                                            int64_t per_iter, int E, int32_t* __restrict__ keys,
                                                            int32_t* __restrict__ sorted_ids, int64_t fill_n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < fill_n) sorted_ids[i] = (int32_t)n;
  if (i >= n) return;
  const int64_t id = ids_int64 ? ((const int64_t*)ids)[i] : (int64_t)((const int32_t*)ids)[i];
  keys[i] = (id >= 0 && id < E) ? (int32_t)((i / per_iter) * E + id) : -1;
}

// Padding and placement in one launch. Every workgroup works out the padded exclusive prefix over the G = R * E group
// sizes for itself (G <= 4096 values through LDS: cheaper than a launch of its own and the wait for it), then places
// its 256 entries: an entry's position in the padded layout is its position in the unpadded sorted order moved by the
// padding in front of its group. Workgroup 0 also writes the per-block expert / segment ids, the blocks per segment
// and the padded total.
constexpr int kPlaceThreads = 256;
__global__ __launch_bounds__(kPlaceThreads) void moe_align_place_kernel(
    const int32_t* __restrict__ keys, const int32_t* __restrict__ scatter_idx, const int32_t* __restrict__ splits,
    const int32_t* __restrict__ cumsum, int64_t n, int G, int E, int R, int block_size, int32_t* __restrict__ sorted_ids,
    int32_t* __restrict__ expert_ids, int32_t* __restrict__ block_barrier_ids, int32_t* __restrict__ rank_block_num,
    int32_t* __restrict__ total_post_pad) {
  extern __shared__ int32_t s_pad[];  // [G + 1] padded exclusive prefix
  __shared__ int32_t s_part[kPlaceThreads];
  // the entry's own loads first: they do not depend on the prefix
  const int64_t i = (int64_t)blockIdx.x * kPlaceThreads + threadIdx.x;
  const int32_t k = i < n ? keys[i] : -1;
  const int32_t rank_in_group = k >= 0 ? scatter_idx[i] - cumsum[k] : 0;
  const int per = (G + kPlaceThreads - 1) / kPlaceThreads;  // consecutive groups per thread
  const int g0 = threadIdx.x * per;
  int32_t local_total = 0;
  for (int j = 0; j < per; ++j) {
    const int g = g0 + j;
    if (g < G) local_total += (splits[g] + block_size - 1) / block_size * block_size;
  }
  s_part[threadIdx.x] = local_total;
  __syncthreads();
  for (int off = 1; off < kPlaceThreads; off <<= 1) {
    const int32_t v = (threadIdx.x >= off) ? s_part[threadIdx.x - off] : 0;
    __syncthreads();
    s_part[threadIdx.x] += v;
    __syncthreads();
  }
  int32_t run = s_part[threadIdx.x] - local_total;
  if (threadIdx.x == 0) s_pad[0] = 0;
  for (int j = 0; j < per; ++j) {
    const int g = g0 + j;
    if (g < G) {
      const int32_t padded = (splits[g] + block_size - 1) / block_size * block_size;
      if (blockIdx.x == 0) {
        for (int32_t b = run / block_size; b < (run + padded) / block_size; ++b) {
          expert_ids[b] = g % E;
          block_barrier_ids[b] = g / E;
        }
      }
      run += padded;
      s_pad[g + 1] = run;
    }
  }
  __syncthreads();
  if (blockIdx.x == 0) {
    for (int r = threadIdx.x; r < R; r += kPlaceThreads) rank_block_num[r] = (s_pad[(r + 1) * E] - s_pad[r * E]) / block_size;
    if (threadIdx.x == 0) *total_post_pad = s_pad[G];
  }
  if (k >= 0) sorted_ids[s_pad[k] + rank_in_group] = (int32_t)i;
}

// Align / sort in ONE launch for few entries (up to kRecountMaxBlocks blocks of 1024): the recounting index build above
// with the composite keys formed on the way in and the groups' starts taken from the PADDED prefix, so that an entry's
// rank is its place in the padded layout at once. Every block counts all entries (those in front of its range, its
// own, those behind), works out the padded prefix over the G = R * E groups for itself and places its own entries;
// the padding positions, the per-block expert / segment ids and the positions behind the padded total (up to fill_n)
// are shared out among the blocks, groups in turn; block 0 writes the blocks per segment and the padded total.
template <int kThreads, int kPerWave, bool kIds64>
__global__ __launch_bounds__(kThreads) void moe_align_fused_kernel(
    const void* __restrict__ ids_v, int64_t n, int per_iter, int E, int R, int nbits, int block_size,
    int32_t* __restrict__ sorted_ids, int64_t fill_n, int32_t* __restrict__ expert_ids,
    int32_t* __restrict__ block_barrier_ids, int32_t* __restrict__ rank_block_num, int32_t* __restrict__ total_post_pad,
    uint32_t seg_magic) {
  constexpr int kWaves = kThreads / 64, kItems = kWaves * kPerWave, kPasses = kPerWave / 64;
  typedef __attribute__((__vector_size__(2 * sizeof(long long)))) long long long2v;
  const int G = E * R;
  extern __shared__ int32_t s_mem[];  // [kWaves][G] wave counters, [G] group sizes, [2][G] before / behind, then starts
  int32_t* const s_cnt = s_mem;
  int32_t* const s_col = s_mem + kWaves * G;
  int32_t* const s_out = s_col + G;
  int32_t* const s_start = s_out;     // [G + 1] padded exclusive prefix, once the two rows have been summed
  __shared__ int32_t s_part[kWaves];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int B = gridDim.x, b = blockIdx.x;
  const int32_t* const ids32 = (const int32_t*)ids_v;
  const long long* const ids64 = (const long long*)ids_v;
  const uint32_t per = (uint32_t)per_iter;
  auto key_of = [&](uint32_t i, long long id) -> int {
    return (id >= 0 && id < E) ? (int)__umulhi(i, seg_magic) * E + (int)id : -1;
  };
  // the wave's own entries first
  const int64_t wbase = (int64_t)b * kItems + (int64_t)wave * kPerWave;
  long long id_own[kPasses];
#pragma unroll
  for (int u = 0; u < kPasses; ++u) {
    const int64_t i = wbase + u * 64 + lane;
    id_own[u] = i < n ? (kIds64 ? ids64[i] : (long long)ids32[i]) : -1;
  }
  // everybody else's, four per lane and load, all of a batch in flight
  constexpr int kVecBatch = 16;
  const int64_t own_lo = (int64_t)b * kItems, own_hi = own_lo + kItems;
  const int64_t n_vec = (n + 3) / 4;
  int4v q32[kIds64 ? 1 : kVecBatch];
  long2v q64[kIds64 ? 2 * kVecBatch : 1];
  auto load_others = [&](int64_t v0) {
#pragma unroll
    for (int u = 0; u < kVecBatch; ++u) {
      const int64_t vi = v0 + (int64_t)u * kThreads;
      const bool take = vi < n_vec && !(vi * 4 >= own_lo && vi * 4 < own_hi);
      const bool whole = vi * 4 + 3 < n;
      if constexpr (kIds64) {
        q64[2 * u] = long2v{-1, -1};
        q64[2 * u + 1] = long2v{-1, -1};
        if (take && whole) {
          q64[2 * u] = ((const long2v*)ids64)[2 * vi];
          q64[2 * u + 1] = ((const long2v*)ids64)[2 * vi + 1];
        } else if (take) {
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (vi * 4 + j < n) q64[2 * u + j / 2][j % 2] = ids64[vi * 4 + j];
        }
      } else {
        q32[u] = int4v{-1, -1, -1, -1};
        if (take && whole) q32[u] = ((const int4v*)ids32)[vi];
        else if (take) {
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (vi * 4 + j < n) q32[u][j] = ids32[vi * 4 + j];
        }
      }
    }
  };
  // Counting is the kernel's longest phase (every lane counts n / kThreads entries), so an entry costs as few
  // instructions as can be: the segment of a vector's first entry by a multiplication (seg_magic = ceil(2^32 / per),
  // exact below 65536 entries), at most one segment boundary inside a vector (per >= 4), one unsigned compare for the
  // id's range, and no branch: an id out of range counts into a word of its own lane behind the counters.
  int32_t* const s_trash = s_mem + (kWaves + 3) * G + lane;
  auto count_others = [&](int64_t v0) {
#pragma unroll
    for (int u = 0; u < kVecBatch; ++u) {
      const int64_t vi = v0 + (int64_t)u * kThreads;
      int32_t* const row = s_out + (vi * 4 < own_lo ? 0 : G);
      const uint32_t i0 = (uint32_t)(vi * 4);
      const uint32_t seg = __umulhi(i0, seg_magic);
      const uint32_t to_next = (seg + 1) * per - i0;   // entries of this vector that are still in segment `seg`
      int32_t* const row_seg = row + seg * (uint32_t)E;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        uint32_t lo;
        bool ok;
        if constexpr (kIds64) {
          const long long id = q64[2 * u + j / 2][j % 2];
          lo = (uint32_t)id;
          ok = (uint32_t)(id >> 32) == 0u && lo < (uint32_t)E;
        } else {
          lo = (uint32_t)q32[u][j];
          ok = lo < (uint32_t)E;
        }
        int32_t* const at = row_seg + (j > 0 && (uint32_t)j >= to_next ? E : 0) + lo;
        atomicAdd(ok ? at : s_trash, 1);
      }
    }
  };
  if (B > 1) load_others(threadIdx.x);
  for (int g = threadIdx.x; g < (kWaves + 3) * G; g += kThreads) s_cnt[g] = 0;
  __syncthreads();
  int32_t* const my_cnt = s_cnt + wave * G;
  int e_of[kPasses];
#pragma unroll
  for (int u = 0; u < kPasses; ++u) {
    e_of[u] = key_of((uint32_t)(wbase + u * 64 + lane), id_own[u]);
    if (e_of[u] >= 0) atomicAdd(&my_cnt[e_of[u]], 1);
  }
  if (B > 1) {
    count_others(threadIdx.x);
    for (int64_t v0 = threadIdx.x + (int64_t)kVecBatch * kThreads; v0 < n_vec; v0 += (int64_t)kVecBatch * kThreads) {
      load_others(v0);
      count_others(v0);
    }
  }
  __syncthreads();
  // group sizes; the waves' starts within their group (entries of the blocks in front, then of the earlier waves)
  for (int g = threadIdx.x; g < G; g += kThreads) {
    int32_t run = s_out[g], total = s_out[g] + s_out[G + g];
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      const int32_t c = s_cnt[w * G + g];
      s_cnt[w * G + g] = run;
      run += c;
      total += c;
    }
    s_col[g] = total;
  }
  __syncthreads();
  // exclusive scan of the PADDED group sizes: consecutive groups per thread, then across threads and waves
  const int per_thread = (G + kThreads - 1) / kThreads;
  const int g0 = threadIdx.x * per_thread;
  auto padded = [&](int32_t c) { return (c + block_size - 1) / block_size * block_size; };
  int32_t local_total = 0;
  for (int j = 0; j < per_thread; ++j)
    if (g0 + j < G) local_total += padded(s_col[g0 + j]);
  int32_t incl = local_total;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int32_t t = __shfl_up(incl, off);
    if (lane >= off) incl += t;
  }
  if (lane == 63) s_part[wave] = incl;
  __syncthreads();
  int32_t acc = incl - local_total;
#pragma unroll
  for (int w = 0; w < kWaves; ++w) acc += w < wave ? s_part[w] : 0;
  for (int j = 0; j < per_thread; ++j) {
    const int g = g0 + j;
    if (g < G) {
      s_start[g] = acc;
#pragma unroll
      for (int w = 0; w < kWaves; ++w) s_cnt[w * G + g] += acc;
      acc += padded(s_col[g]);
      if (g == G - 1) s_start[G] = acc;
    }
  }
  __syncthreads();
  const int32_t total = s_start[G];
  if (b == 0) {
    for (int r = threadIdx.x; r < R; r += kThreads) rank_block_num[r] = (s_start[(r + 1) * E] - s_start[r * E]) / block_size;
    if (threadIdx.x == 0) *total_post_pad = total;
  }
  // the groups this block looks after (a wave each, in turn): their padding positions and their blocks' ids
  for (int g = b + B * wave; g < G; g += B * kWaves) {
    const int32_t st = s_start[g], c = s_col[g], pc = padded(c);
    for (int32_t o = c + lane; o < pc; o += 64) sorted_ids[st + o] = (int32_t)n;
    for (int32_t k = st / block_size + lane; k < (st + pc) / block_size; k += 64) {
      expert_ids[k] = g % E;
      block_barrier_ids[k] = g / E;
    }
  }
  // and its share of the positions behind the padded total
  if (fill_n > total) {
    const int64_t share = (fill_n - total + B - 1) / B;
    const int64_t lo = total + share * b, hi = lo + share < fill_n ? lo + share : fill_n;
    for (int64_t i = lo + threadIdx.x; i < hi; i += kThreads) sorted_ids[i] = (int32_t)n;
  }
  // the wave's entries in flat order, 64 at a time (as in moe_rank_kernel)
  volatile int32_t* pos = my_cnt;
  const uint64_t lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
#pragma unroll
  for (int u = 0; u < kPasses; ++u) {
    if (wbase + u * 64 >= n) break;
    const int64_t i = wbase + u * 64 + lane;
    const int e = e_of[u];
    const bool valid = e >= 0;
    uint64_t peers = __ballot(valid);
    for (int bit = 0; bit < nbits; ++bit) {
      const bool one = (e >> bit) & 1;
      const uint64_t m = __ballot(valid && one);
      peers &= one ? m : ~m;
    }
    if (valid) sorted_ids[pos[e] + __popcll(peers & lt_mask)] = (int32_t)i;
    __builtin_amdgcn_wave_barrier();
    if (valid && (peers & lt_mask) == 0) pos[e] = pos[e] + __popcll(peers);
    __builtin_amdgcn_wave_barrier();
  }
}

static int moe_index_common(const int32_t* ids, int64_t n_ids, int topk, int G, int32_t* splits, int32_t* cumsum,
                            int32_t* scatter_idx, int32_t* gather_idx, int32_t* topk_idx, void* workspace,
                            int64_t workspace_bytes, hipStream_t stream, bool want_index, const char* who) {
  if (!ids || !cumsum) return fail(TDIST_ERR_INVALID, "%s: null ids or cumsum", who);
  if (want_index && (!scatter_idx || !gather_idx)) return fail(TDIST_ERR_INVALID, "%s: null index output", who);
  if (n_ids < 0 || G <= 0 || (want_index && topk <= 0)) return fail(TDIST_ERR_INVALID, "%s: bad sizes", who);
  if (G > kMoeMaxExperts) return fail(TDIST_ERR_UNSUPPORTED, "%s: num_experts %d > %d", who, G, kMoeMaxExperts);
  if (n_ids > 0x7fffffffll) return fail(TDIST_ERR_UNSUPPORTED, "%s: more than 2^31-1 ids", who);
  const int64_t need = tdist_moe_workspace_bytes(n_ids, G);
  if (!workspace || workspace_bytes < need)
    return fail(TDIST_ERR_WORKSPACE, "%s: workspace %lld B < %lld B", who, (long long)workspace_bytes, (long long)need);
  const int num_blocks = (int)ceil_div(n_ids > 0 ? n_ids : 1, kMoeItemsPerBlock);
  // workspace: 256 bytes of control words (always at the start, whatever the sizes of the call), the block
  // histograms, one row for the splits
  int32_t* scan_counter = (int32_t*)workspace;
  int32_t* hist = scan_counter + 64;
  int32_t* splits_buf = splits ? splits : hist + (int64_t)num_blocks * G;
  // One launch for few ids (up to 65536): every block counts all of them itself and nothing is exchanged. Beyond
  // that, three launches. A one-launch form whose blocks (2048 ids each, at most one per compute unit) wait for each
  // other's histograms exists too, but its wait only ends if every block is resident at once, which the library
  // cannot know when other streams hold compute units: it is taken on request only (TDIST_DEBUG_MOE_INDEX_FORM = 2,
  // for tests and measurements; 3 = always three launches). Its histogram rows (one per 2048 ids) fit the rows the
  // workspace holds (one per 256 ids).
  const DeviceInfo& di = device_info();
  const int64_t fused_blocks = ceil_div(n_ids > 0 ? n_ids : 1, kFusedItems);
  const int form_dbg = debug_get(TDIST_DEBUG_MOE_INDEX_FORM);
  constexpr int kLdsLimit = 160 * 1024 - 256;          // (the kernel has a few static words of its own)
  constexpr int kRowsPlain = kFusedThreads / 64 + 1;   // wave counters, column sums
  constexpr int kRowsRecount = kRowsPlain + 2;         // and the ids before / behind the block
  constexpr int kSmall = kFusedThreads;                // ids per block of the recounting forms: 512, or 1024
  const int64_t n1 = n_ids > 0 ? n_ids : 1;
  const bool can_recount = form_dbg != 2 && kRowsRecount * G * 4 + 256 <= kLdsLimit && aligned16(ids);
  // 0: blocks of 2048 ids that exchange their histograms; 1 / 2: blocks of 512 / 1024 ids that count everything
  const int form = !can_recount ? 0 : ceil_div(n1, kSmall) <= kRecountMaxBlocks ? 1 : ceil_div(n1, 2 * kSmall) <= kRecountMaxBlocks ? 2 : 0;
  if (di.ok == 1 && fused_blocks <= di.num_cus && form_dbg != 3 && (form != 0 || form_dbg == 2)) {
    auto kern = form == 1 ? moe_index_fused_kernel<kFusedThreads, kSmall / 8, true>
              : form == 2 ? moe_index_fused_kernel<kFusedThreads, kSmall / 4, true>
                          : moe_index_fused_kernel<kFusedThreads, kFusedPerWave, false>;
    const int64_t blocks = form == 1 ? ceil_div(n1, kSmall) : form == 2 ? ceil_div(n1, 2 * kSmall) : fused_blocks;
    const int rows = form != 0 ? kRowsRecount : kRowsPlain;
    static bool attr_set[3] = {false, false, false};
    if (!attr_set[form]) {
      const int most = rows * kMoeMaxExperts * 4 < kLdsLimit ? rows * kMoeMaxExperts * 4 : kLdsLimit;
      if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, most) != hipSuccess)
        return fail(TDIST_ERR_LAUNCH, "%s: cannot reserve LDS for the index kernel", who);
      attr_set[form] = true;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(kFusedThreads), (size_t)rows * G * 4 + (form != 0 ? 256 : 0), stream,
                       ids, n_ids, want_index ? topk : 1, G, id_bits(G), hist, scan_counter, splits, cumsum,
                       want_index ? scatter_idx : nullptr, gather_idx, topk_idx);
    return launch_status(who);
  }
  hipLaunchKernelGGL(moe_hist_kernel, dim3(num_blocks), dim3(kMoeThreads), (size_t)G * 4, stream, ids, n_ids, G, hist,
                     scan_counter);
  hipLaunchKernelGGL(moe_scan_kernel, dim3((G + kScanCols - 1) / kScanCols), dim3(kScanThreads), 0, stream, hist, num_blocks,
                     G, splits_buf, cumsum, scan_counter);
  if (want_index && n_ids > 0) {
    hipLaunchKernelGGL(moe_rank_kernel, dim3(num_blocks), dim3(kMoeThreads), (size_t)G * 4 * (kMoeThreads / 64), stream,
                       ids, n_ids, topk, G, id_bits(G), hist, cumsum, scatter_idx, gather_idx, topk_idx);
  }
  return launch_status(who);
}

// ---- the index build without a caller's workspace ---------------------------------------------------------
// Scratch for tdist_moe_scatter_index_static: every GPU the library runs on holds its own copy of this array until the
// process ends. Host code never uses the array's name as an address: the per-device address comes from
// hipGetSymbolAddress, once per device, and is what the kernels are given.
constexpr int64_t kMoeStaticScratchBytes = 1 << 20;
static __device__ __align__(256) unsigned char scratch[kMoeStaticScratchBytes];

constexpr int kMoeMaxDevices = 64;
static void* g_scratch_ptr[kMoeMaxDevices];   // device address of `scratch` per device, NULL until looked up
static std::mutex g_scratch_mutex;

// Device address of the current device's copy of `scratch` (looked up on first use, with that device current).
static int moe_static_scratch(void** out, const char* who) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMoeMaxDevices)
    return fail(TDIST_ERR_DEVICE, "%s: no current device (or more than %d devices)", who, kMoeMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr)
      return fail(TDIST_ERR_DEVICE, "%s: hipGetSymbolAddress(scratch) failed on device %d: %s", who, dev, hipGetErrorString(e));
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return TDIST_OK;
}

int moe_static_scratch_init() {
  void* ptr = nullptr;
  return moe_static_scratch(&ptr, "tdist_init");
}

}  // namespace tdist

using namespace tdist;

extern "C" {

int tdist_moe_scatter_index_static(const int32_t* ids, int64_t n_ids, int topk, int num_experts, int32_t* splits,
                                   int32_t* cumsum, int32_t* scatter_idx, int32_t* gather_idx, int32_t* topk_idx,
                                   void* stream) {
  const char* who = "tdist_moe_scatter_index_static";
  const int64_t need = tdist_moe_workspace_bytes(n_ids, num_experts);
  if (need <= 0) return fail(TDIST_ERR_INVALID, "%s: bad sizes", who);
  if (need > kMoeStaticScratchBytes)
    return fail(TDIST_ERR_UNSUPPORTED, "%s: %lld ids over %d experts need %lld bytes of scratch, the built-in buffer holds "
                "%lld (use tdist_moe_scatter_index with a workspace)", who, (long long)n_ids, num_experts, (long long)need,
                (long long)kMoeStaticScratchBytes);
  void* ws = nullptr;
  if (int rc = moe_static_scratch(&ws, who)) return rc;
  // (the control words are the array's first 256 bytes whatever the call's sizes; they are zero between calls: the
  // kernels leave them so, and the array starts out zero. The rest needs no clearing, every word is written before it
  // is read, so a call after a larger one is not disturbed by what that one left behind.)
  return moe_index_common(ids, n_ids, topk, num_experts, splits, cumsum, scatter_idx, gather_idx, topk_idx, ws, need,
                          (hipStream_t)stream, true, who);
}

int64_t tdist_moe_workspace_bytes(int64_t n_ids, int num_experts) {
  if (n_ids < 0 || num_experts <= 0) return 0;
  const int64_t num_blocks = ceil_div(n_ids > 0 ? n_ids : 1, kMoeItemsPerBlock);
  return 256 + (num_blocks + 1) * (int64_t)num_experts * 4;  // control words + block histograms + one splits row
}

int tdist_moe_splits_cumsum(const int32_t* ids, int64_t n_ids, int num_experts, int32_t* splits, int32_t* cumsum,
                            void* workspace, int64_t workspace_bytes, void* stream) {
  return moe_index_common(ids, n_ids, 1, num_experts, splits, cumsum, nullptr, nullptr, nullptr, workspace,
                          workspace_bytes, (hipStream_t)stream, false, "tdist_moe_splits_cumsum");
}

int tdist_moe_scatter_index(const int32_t* ids, int64_t n_ids, int topk, int num_experts, int32_t* splits,
                            int32_t* cumsum, int32_t* scatter_idx, int32_t* gather_idx, int32_t* topk_idx,
                            void* workspace, int64_t workspace_bytes, void* stream) {
  return moe_index_common(ids, n_ids, topk, num_experts, splits, cumsum, scatter_idx, gather_idx, topk_idx, workspace,
                          workspace_bytes, (hipStream_t)stream, true, "tdist_moe_scatter_index");
}

int tdist_moe_dispatch(const void* rows, int64_t row_bytes, const float* scales, const int32_t* gather_idx,
                       const int32_t* cumsum, int64_t n_rows, int world_size, int experts_per_rank, int max_m,
                       void* slot_rows, float* slot_scales, int32_t* splits_out, void* stream) {
  if (!rows || !cumsum || !slot_rows) return fail(TDIST_ERR_INVALID, "tdist_moe_dispatch: null pointer");
  if ((scales != nullptr) != (slot_scales != nullptr))
    return fail(TDIST_ERR_INVALID, "tdist_moe_dispatch: scales and slot_scales must both be given or both NULL");
  if (row_bytes <= 0 || n_rows < 0 || world_size <= 0 || experts_per_rank <= 0 || max_m <= 0)
    return fail(TDIST_ERR_INVALID, "tdist_moe_dispatch: bad sizes");
  if (world_size > 8192) return fail(TDIST_ERR_UNSUPPORTED, "tdist_moe_dispatch: world_size > 8192");
  const int64_t blocks = ceil_div(n_rows > 0 ? n_rows : 1, kRowsPerBlock);
  if (blocks > 0x7fffffff) return fail(TDIST_ERR_UNSUPPORTED, "tdist_moe_dispatch: too many rows");
  const bool vec = (row_bytes % 16 == 0) && aligned16(rows) && aligned16(slot_rows);
  auto kern = vec ? moe_rows_kernel<true, false> : moe_rows_kernel<false, false>;
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(256), (size_t)(world_size + 1) * 4, (hipStream_t)stream,
                     (const unsigned char*)rows, row_bytes, scales, gather_idx, cumsum, n_rows, world_size,
                     experts_per_rank, max_m, (unsigned char*)slot_rows, slot_scales, splits_out);
  return launch_status("tdist_moe_dispatch");
}

int tdist_moe_dispatch_tokens(const void* tokens, int64_t row_bytes, const float* token_scales,
                              const int32_t* scatter_idx, int topk, const int32_t* cumsum, int64_t n_tokens,
                              int world_size, int experts_per_rank, int max_m, void* slot_rows, float* slot_scales,
                              int32_t* splits_out, void* stream) {
  if (!tokens || !scatter_idx || !cumsum || !slot_rows)
    return fail(TDIST_ERR_INVALID, "tdist_moe_dispatch_tokens: null pointer");
  if ((token_scales != nullptr) != (slot_scales != nullptr))
    return fail(TDIST_ERR_INVALID, "tdist_moe_dispatch_tokens: token_scales and slot_scales go together");
  if (row_bytes <= 0 || n_tokens < 0 || world_size <= 0 || experts_per_rank <= 0 || max_m <= 0 || topk <= 0)
    return fail(TDIST_ERR_INVALID, "tdist_moe_dispatch_tokens: bad sizes");
  if (topk > 64) return fail(TDIST_ERR_UNSUPPORTED, "tdist_moe_dispatch_tokens: topk > 64");
  if (world_size > 8192 || (int64_t)world_size * max_m > 0x7fffffff)
    return fail(TDIST_ERR_UNSUPPORTED, "tdist_moe_dispatch_tokens: world_size * max_m too large");
  const int windows = (int)ceil_div(row_bytes, 8192);
  const int64_t units = (n_tokens > 0 ? n_tokens : 1) * windows;
  const int64_t blocks = ceil_div(units, 4);
  if (blocks > 0x7fffffff) return fail(TDIST_ERR_UNSUPPORTED, "tdist_moe_dispatch_tokens: too many tokens");
  const bool vec = (row_bytes % 16 == 0) && aligned16(tokens) && aligned16(slot_rows);
  auto kern = vec ? moe_dispatch_tokens_kernel<true> : moe_dispatch_tokens_kernel<false>;
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                     (const unsigned char*)tokens, row_bytes, token_scales, scatter_idx, topk, cumsum, n_tokens,
                     world_size, experts_per_rank, max_m, (unsigned char*)slot_rows, slot_scales, splits_out, windows);
  return launch_status("tdist_moe_dispatch_tokens");
}

int tdist_moe_dispatch_tokens_from_ids(const void* tokens, int64_t row_bytes, const float* token_scales,
                                       const int32_t* ids, int topk, int64_t n_tokens, int world_size,
                                       int experts_per_rank, int max_m, void* slot_rows, float* slot_scales,
                                       int32_t* splits_out, int32_t* splits, int32_t* cumsum, int32_t* scatter_idx,
                                       int32_t* gather_idx, void* stream) {
  const char* who = "tdist_moe_dispatch_tokens_from_ids";
  if (!tokens || !ids || !slot_rows || !cumsum || !scatter_idx || !gather_idx) return fail(TDIST_ERR_INVALID, "%s: null pointer", who);
  if ((token_scales != nullptr) != (slot_scales != nullptr))
    return fail(TDIST_ERR_INVALID, "%s: token_scales and slot_scales go together", who);
  if (row_bytes <= 0 || n_tokens < 0 || world_size <= 0 || experts_per_rank <= 0 || max_m <= 0 || topk <= 0)
    return fail(TDIST_ERR_INVALID, "%s: bad sizes", who);
  if (topk > 64) return fail(TDIST_ERR_UNSUPPORTED, "%s: topk > 64", who);
  const int64_t G64 = (int64_t)world_size * experts_per_rank;
  if (G64 > kMoeMaxExperts) return fail(TDIST_ERR_UNSUPPORTED, "%s: num_experts %lld > %d", who, (long long)G64, kMoeMaxExperts);
  if ((int64_t)world_size * max_m > 0x7fffffff) return fail(TDIST_ERR_UNSUPPORTED, "%s: world_size * max_m too large", who);
  const int G = (int)G64;
  const int windows = (int)ceil_div(row_bytes, 8192);
  const int64_t lds = ((int64_t)3 * G + ((G + 1 + 3) & ~3) + kFdWaves * topk + 8 + 64) * 4;   // (+ a word per lane for what is not counted)
  if (n_tokens * topk > kFusedDispatchMaxIds || windows > kFdWaves || kFdWaves % windows != 0 || lds > 160 * 1024 - 256)
    return fail(TDIST_ERR_UNSUPPORTED, "%s: more than %lld ids, rows above %d bytes (or no power-of-two number of 8 KB windows), or too "
                "many experts for one workgroup's counters: use tdist_moe_scatter_index + tdist_moe_dispatch_tokens", who,
                (long long)kFusedDispatchMaxIds, kFdWaves * 8192);
  const int64_t units = (n_tokens > 0 ? n_tokens : 1) * windows;
  const int64_t blocks = ceil_div(units, kFdWaves);
  const bool vec = (row_bytes % 16 == 0) && aligned16(tokens) && aligned16(slot_rows);
  auto kern = vec ? moe_dispatch_fused_kernel<true> : moe_dispatch_fused_kernel<false>;
  static bool attr_set[2] = {false, false};
  if (!attr_set[vec]) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 256) != hipSuccess)
      return fail(TDIST_ERR_LAUNCH, "%s: cannot reserve LDS", who);
    attr_set[vec] = true;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(kFdThreads), (size_t)lds, (hipStream_t)stream,
                     (const unsigned char*)tokens, row_bytes, token_scales, ids, topk, n_tokens, G, id_bits(G), world_size,
                     experts_per_rank, max_m, windows, (unsigned char*)slot_rows, slot_scales, splits_out, splits, cumsum,
                     scatter_idx, gather_idx);
  return launch_status(who);
}

int tdist_moe_post_process(const void* slot_rows, int64_t row_bytes, const float* slot_scales, const int32_t* splits,
                           int64_t n_rows, int world_size, int experts_per_rank, int max_m, void* out_rows,
                           float* out_scales, void* stream) {
  if (!slot_rows || !splits || (!out_rows && n_rows > 0))
    return fail(TDIST_ERR_INVALID, "tdist_moe_post_process: null pointer");
  if (row_bytes <= 0 || n_rows < 0 || world_size <= 0 || experts_per_rank <= 0 || max_m <= 0)
    return fail(TDIST_ERR_INVALID, "tdist_moe_post_process: bad sizes");
  if (world_size > 8192) return fail(TDIST_ERR_UNSUPPORTED, "tdist_moe_post_process: world_size > 8192");
  if (n_rows == 0) return TDIST_OK;
  const int64_t blocks = ceil_div(n_rows, kRowsPerBlock);
  if (blocks > 0x7fffffff) return fail(TDIST_ERR_UNSUPPORTED, "tdist_moe_post_process: too many rows");
  const bool vec = (row_bytes % 16 == 0) && aligned16(out_rows) && aligned16(slot_rows);
  auto kern = vec ? moe_rows_kernel<true, true> : moe_rows_kernel<false, true>;
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(256), (size_t)(world_size + 1) * 4, (hipStream_t)stream,
                     (const unsigned char*)slot_rows, row_bytes, slot_scales, (const int32_t*)nullptr, splits, n_rows,
                     world_size, experts_per_rank, max_m, (unsigned char*)out_rows, out_scales, (int32_t*)nullptr);
  return launch_status("tdist_moe_post_process");
}

int tdist_moe_combine(const void* slot_rows, int row_dtype, const float* slot_scales, const int32_t* scatter_idx,
                      const float* topk_w, const int32_t* cumsum, int64_t n_tokens, int topk, int hidden,
                      int world_size, int experts_per_rank, int max_m, int scale_group_size, void* out_bf16,
                      void* stream) {
  if (!slot_rows || !scatter_idx || !out_bf16) return fail(TDIST_ERR_INVALID, "tdist_moe_combine: null pointer");
  if (max_m > 0 && (!cumsum || world_size <= 0 || experts_per_rank <= 0))
    return fail(TDIST_ERR_INVALID, "tdist_moe_combine: slot layout needs cumsum, world_size, experts_per_rank");
  if (n_tokens < 0 || topk <= 0 || topk > kCombineMaxTopk || hidden <= 0)
    return fail(TDIST_ERR_INVALID, "tdist_moe_combine: bad sizes (topk <= %d)", kCombineMaxTopk);
  if (row_dtype != TDIST_F8E4M3 && row_dtype != TDIST_BF16)
    return fail(TDIST_ERR_UNSUPPORTED, "tdist_moe_combine: row dtype %d (e4m3 and bf16 only)", row_dtype);
  if (scale_group_size != 0 && (row_dtype != TDIST_F8E4M3 || scale_group_size < 16 || scale_group_size % 16 != 0 ||
                                hidden % scale_group_size != 0))
    return fail(TDIST_ERR_UNSUPPORTED, "tdist_moe_combine: grouped scales need e4m3 rows and a group size that is a "
                "multiple of 16 and divides hidden");
  const int elems = row_dtype == TDIST_F8E4M3 ? 16 : 8;
  if (hidden % elems != 0 || !aligned16(slot_rows) || !aligned16(out_bf16))
    return fail(TDIST_ERR_UNSUPPORTED, "tdist_moe_combine: hidden must be a multiple of %d and buffers 16-byte aligned", elems);
  if (n_tokens == 0) return TDIST_OK;
  if (n_tokens > 0x7fffffff) return fail(TDIST_ERR_UNSUPPORTED, "tdist_moe_combine: too many tokens");
  const int n_windows = (hidden / elems + 63) / 64;
  const int64_t waves = n_tokens * n_windows;
  const int64_t blocks = ceil_div(waves, kCombineWaves);
  if (blocks > 0x7fffffff) return fail(TDIST_ERR_UNSUPPORTED, "tdist_moe_combine: too many tokens");
  auto kern = row_dtype == TDIST_F8E4M3 ? moe_combine_kernel<true> : moe_combine_kernel<false>;
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(kCombineWaves * 64), 0, (hipStream_t)stream,
                     (const unsigned char*)slot_rows, slot_scales, scatter_idx, topk_w, cumsum, n_tokens, topk, hidden,
                     world_size, experts_per_rank, max_m, scale_group_size, n_windows, (unsigned short*)out_bf16);
  return launch_status("tdist_moe_combine");
}

int tdist_quant_e4m3_groups(const void* x_bf16, int64_t n_rows, int hidden, int group_size, void* q_out,
                            float* scales_out, void* stream) {
  if (!x_bf16 || !q_out || !scales_out) return fail(TDIST_ERR_INVALID, "tdist_quant_e4m3_groups: null pointer");
  if (n_rows < 0 || hidden <= 0) return fail(TDIST_ERR_INVALID, "tdist_quant_e4m3_groups: bad sizes");
  if (group_size != kQuantGroup || hidden % kQuantGroup != 0 || !aligned16(x_bf16) || !aligned16(q_out))
    return fail(TDIST_ERR_UNSUPPORTED, "tdist_quant_e4m3_groups: group size %d, hidden a multiple of it, 16-byte aligned buffers",
                kQuantGroup);
  if (n_rows == 0) return TDIST_OK;
  const int windows = (hidden + 1023) / 1024;
  const int64_t blocks = ceil_div(n_rows * windows, 4);
  if (blocks > 0x7fffffff) return fail(TDIST_ERR_UNSUPPORTED, "tdist_quant_e4m3_groups: too many rows");
  hipLaunchKernelGGL(quant_groups_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                     (const unsigned short*)x_bf16, n_rows, hidden, windows, (unsigned char*)q_out, scales_out);
  return launch_status("tdist_quant_e4m3_groups");
}

int tdist_moe_dispatch_tokens_quant(const void* tokens_bf16, int hidden, int group_size, const int32_t* scatter_idx,
                                    int topk, const int32_t* cumsum, int64_t n_tokens, int world_size,
                                    int experts_per_rank, int max_m, void* slot_rows, float* slot_scales,
                                    int32_t* splits_out, void* stream) {
  const char* who = "tdist_moe_dispatch_tokens_quant";
  if (!tokens_bf16 || !scatter_idx || !cumsum || !slot_rows || !slot_scales) return fail(TDIST_ERR_INVALID, "%s: null pointer", who);
  if (n_tokens < 0 || hidden <= 0 || world_size <= 0 || experts_per_rank <= 0 || max_m <= 0 || topk <= 0)
    return fail(TDIST_ERR_INVALID, "%s: bad sizes", who);
  if (topk > 64) return fail(TDIST_ERR_UNSUPPORTED, "%s: topk > 64", who);
  if (group_size != kQuantGroup || hidden % kQuantGroup != 0 || !aligned16(tokens_bf16) || !aligned16(slot_rows))
    return fail(TDIST_ERR_UNSUPPORTED, "%s: group size %d, hidden a multiple of it, 16-byte aligned buffers", who, kQuantGroup);
  if (world_size > 8192 || (int64_t)world_size * max_m > 0x7fffffff)
    return fail(TDIST_ERR_UNSUPPORTED, "%s: world_size * max_m too large", who);
  const int windows = (hidden + 1023) / 1024;
  const int64_t blocks = ceil_div((n_tokens > 0 ? n_tokens : 1) * windows, 4);
  if (blocks > 0x7fffffff) return fail(TDIST_ERR_UNSUPPORTED, "%s: too many tokens", who);
  hipLaunchKernelGGL(moe_dispatch_quant_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                     (const unsigned short*)tokens_bf16, hidden, scatter_idx, topk, cumsum, n_tokens, world_size,
                     experts_per_rank, max_m, (unsigned char*)slot_rows, slot_scales, splits_out, windows);
  return launch_status(who);
}

int64_t tdist_moe_align_workspace_bytes(int64_t n_total, int num_experts, int num_iterations) {
  if (n_total < 0 || num_experts <= 0 || num_iterations <= 0) return 0;
  const int64_t G = (int64_t)num_experts * num_iterations;
  if (G > kMoeMaxExperts) return 0;
  // the index build's own scratch; then keys, scatter index, gather index, group sizes and their prefix
  return (3 * n_total + 3 * (G + 1)) * 4 + tdist_moe_workspace_bytes(n_total, (int)G);
}

int tdist_moe_align_block_size(const void* topk_ids, int ids_int64, int64_t n_total, int num_experts,
                               int num_iterations, int64_t n_per_iteration, int block_size, int32_t* sorted_token_ids,
                               int64_t sorted_fill, int32_t* expert_ids, int32_t* block_barrier_ids,
                               int32_t* rank_block_num, int32_t* total_tokens_post_pad, void* workspace,
                               int64_t workspace_bytes, void* stream) {
  const char* who = "tdist_moe_align_block_size";
  if (!topk_ids || !sorted_token_ids || !expert_ids || !block_barrier_ids || !rank_block_num || !total_tokens_post_pad)
    return fail(TDIST_ERR_INVALID, "%s: null pointer", who);
  if (num_experts <= 0 || num_iterations <= 0 || block_size <= 0 || n_per_iteration < 0 ||
      n_total != n_per_iteration * num_iterations)
    return fail(TDIST_ERR_INVALID, "%s: bad sizes (n_total must be num_iterations * n_per_iteration)", who);
  const int64_t G = (int64_t)num_experts * num_iterations;
  if (G > kMoeMaxExperts)
    return fail(TDIST_ERR_UNSUPPORTED, "%s: num_experts * num_iterations = %lld > %d", who, (long long)G, kMoeMaxExperts);
  if (n_total + G * (int64_t)(block_size - 1) > 0x7fffffffll) return fail(TDIST_ERR_UNSUPPORTED, "%s: too many entries", who);
  if (sorted_fill < 0 || sorted_fill > 0x7fffffffll) return fail(TDIST_ERR_INVALID, "%s: sorted_fill %lld", who, (long long)sorted_fill);
  const int64_t need = tdist_moe_align_workspace_bytes(n_total, num_experts, num_iterations);
  if (!workspace || workspace_bytes < need)
    return fail(TDIST_ERR_WORKSPACE, "%s: workspace %lld B < %lld B", who, (long long)workspace_bytes, (long long)need);
  hipStream_t st = (hipStream_t)stream;
  // the index build's own scratch first, so that its control words are the workspace's first 256 bytes whatever the
  // sizes; then keys, scatter index, gather index, group sizes and two prefix rows
  void* index_ws = workspace;
  int32_t* keys = (int32_t*)((unsigned char*)workspace + tdist_moe_workspace_bytes(n_total, (int)G));
  int32_t* scatter = keys + n_total;
  int32_t* gather = scatter + n_total;
  int32_t* splits = gather + n_total;
  int32_t* cumsum = splits + (G + 1);
  const int64_t blocks = ceil_div(n_total > 0 ? n_total : 1, 256);
  // Few entries: one launch in which every block counts all of them (see moe_align_fused_kernel).
  {
    constexpr int kLdsLimit = 160 * 1024 - 256;
    constexpr int kRows = kFusedThreads / 64 + 3;
    const int64_t n1 = n_total > 0 ? n_total : 1;
    const int form = ceil_div(n1, kFusedThreads) <= kRecountMaxBlocks ? 1 : ceil_div(n1, 2 * kFusedThreads) <= kRecountMaxBlocks ? 2 : 0;
    const int64_t per_iter = n_per_iteration > 0 ? n_per_iteration : 1;
    // (a vector of four entries may cross one segment boundary, not two; the segment of an entry by multiplication)
    const uint32_t seg_magic = per_iter >= 65536 ? 0u : (uint32_t)(((1ull << 32) + per_iter - 1) / per_iter);
    if (form != 0 && device_info().ok == 1 && kRows * G * 4 + 256 <= kLdsLimit && aligned16(topk_ids) &&
        (per_iter >= 4 || num_iterations == 1) && debug_get(TDIST_DEBUG_MOE_INDEX_FORM) != 3) {
      auto kern = form == 1 ? (ids_int64 ? moe_align_fused_kernel<kFusedThreads, kFusedThreads / 8, true>
                                         : moe_align_fused_kernel<kFusedThreads, kFusedThreads / 8, false>)
                            : (ids_int64 ? moe_align_fused_kernel<kFusedThreads, kFusedThreads / 4, true>
                                         : moe_align_fused_kernel<kFusedThreads, kFusedThreads / 4, false>);
      static bool attr_set[4] = {false, false, false, false};
      const int which = (form - 1) * 2 + (ids_int64 ? 1 : 0);
      if (!attr_set[which]) {
        if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, kLdsLimit) != hipSuccess)
          return fail(TDIST_ERR_LAUNCH, "%s: cannot reserve LDS for the align kernel", who);
        attr_set[which] = true;
      }
      const int64_t nblk = ceil_div(n1, form == 1 ? kFusedThreads : 2 * kFusedThreads);
      hipLaunchKernelGGL(kern, dim3((unsigned)nblk), dim3(kFusedThreads), (size_t)kRows * G * 4 + 256, st, topk_ids, n_total,
                         (int)per_iter, num_experts, num_iterations, id_bits((int)G), block_size, sorted_token_ids, sorted_fill,
                         expert_ids, block_barrier_ids, rank_block_num, total_tokens_post_pad, seg_magic);
      return launch_status(who);
    }
  }
  // three launches: keys (and the pre-fill of the padding positions), the stable index on the keys, padding + placement
  const int64_t key_items = n_total > sorted_fill ? n_total : sorted_fill;
  if (key_items > 0)
    hipLaunchKernelGGL(moe_align_keys_kernel, dim3((unsigned)ceil_div(key_items, 256)), dim3(256), 0, st, topk_ids, ids_int64,
                       n_total, n_per_iteration > 0 ? n_per_iteration : 1, num_experts, keys, sorted_token_ids, sorted_fill);
  int rc = moe_index_common(keys, n_total, 1, (int)G, splits, cumsum, scatter, gather, nullptr, index_ws,
                            tdist_moe_workspace_bytes(n_total, (int)G), st, true, who);
  if (rc != TDIST_OK) return rc;
  hipLaunchKernelGGL(moe_align_place_kernel, dim3((unsigned)blocks), dim3(kPlaceThreads), (size_t)(G + 1) * 4, st, keys, scatter,
                     splits, cumsum, n_total, (int)G, num_experts, num_iterations, block_size, sorted_token_ids, expert_ids,
                     block_barrier_ids, rank_block_num, total_tokens_post_pad);
  return launch_status(who);
}

}  // extern "C"
