// (d) split-KV GQA flash decode and the LSE-weighted combine.
//
// Restates kernel_gqa_fwd_batch_decode_split_kv (kernels/nvidia/flash_decode.py:129-239) and the
// combine kernels (:392-449, :481-532) for CDNA4:
//
//  * one workgroup per (split, kv head [x block of 16 query heads], sequence); its NW waves each stream
//    an interleaved subset of the split's 16-key blocks and keep a private online-softmax state, merged
//    through LDS at the end, so the main loop has no workgroup barrier;
//  * K and V rows go HBM → LDS with asynchronous 16-byte-per-lane LDS-DMA loads into a per-wave ring of
//    NST stages (P = NST-1 stages in flight), so the only synchronisation is the wave's own vmcnt;
//    the page-table entries a stage needs travel the same way, two rounds ahead of the rows;
//  * scores:  S^T[key, head] = K[16 keys, D] . Q^T[D, 16 heads]   v_mfma_f32_16x16x32 (D/32 steps) per group
//    of 16 keys; the result layout (lane = head, 4 keys per lane) is exactly the B operand of
//    O^T[dv, head] += V^T[16 dv, keys] . P^T[keys, 16 heads]  (v_mfma 16x16x32 over two key groups, or
//    16x16x16 over one), so probabilities never leave registers; the V^T fragments come from the
//    row-major V rows in LDS with the transposing read ds_read_b64_tr_b16, one instruction per 4 keys;
//  * probabilities enter the PV product as a hi+lo pair of 16-bit values, which keeps the product at
//    fp32-level accuracy for the cost of a second (idle anyway) MFMA.
//
//  * heads whose key dimension is not a power of two (192 = 128 + 64, 576 = 512 + 64: flash_decode.py:771-772,
//    BLOCK_DPE) are handled as the reference does: the power-of-two part DM (= the value dimension) and the
//    extra DPE key dimensions are two row sets of the stage, each with its own DMA layout and swizzle;
//  * the fused entry point replaces the reference's persistent kernel (split-KV, grid barrier, combine:
//    flash_decode.py:586-760) by "the last workgroup to arrive merges": every workgroup publishes its partial
//    result, bumps a counter of its (sequence, head block), and the one that finds the counter at S-1 merges the S
//    partials. No workgroup ever waits for another, so nothing depends on the grid being co-resident.
//
// HBM traffic per launch: every K and V row of the split once (len * Hkv * (Dk + Dv) * 2 B per sequence).
#include <stdlib.h>

#include "common.h"

// Cache policy of the K/V stream: non-temporal (every byte is used once; the hint lets it pass through the
// caches without displacing anything and measurably raises the HBM streaming rate).
#ifndef TDIST_KV_AUX
#define TDIST_KV_AUX 2
#endif

namespace tdist {

struct DecodeParams {
  const unsigned char* q;
  const unsigned char* k;
  const unsigned char* v;
  float* out;  // [B,Hq,S,D]
  float* lse;  // [B,Hq,S]
  const int32_t* table;
  const int32_t* lens;
  float sm_scale;
  float soft_cap;
  int B, Hq, Hkv, S;
  int when_lens;        // 0: run; 1: run only if the sequence lengths are even (decode_lens_even), 2: only if not
  int splits_per_team;  // kWaveHeads: consecutive splits of a sequence that one workgroup streams through (>= 1)
  int d_valid;  // kernels compiled for a padded head dimension: the real one (a multiple of 8), else unused
  int page_size;
  // n / page_size for 0 <= n < 2^31 as (n * page_magic) >> page_shift with
  // page_shift = 31 + ceil(log2 page_size), page_magic = ceil(2^page_shift / page_size)  (exact, Granlund-Montgomery)
  int page_shift;
  uint64_t page_magic;
  // byte strides
  int64_t q_sb, q_sh;
  int64_t k_sp, k_st, k_sh;
  int64_t v_sp, v_st, v_sh;
  int64_t t_s;  // table stride in entries
  // fused merge (null counters = plain split-KV launch)
  int32_t* counters;         // one per (sequence, head block), zero on entry, left zero on exit
  unsigned char* final_out;  // [B,Hq,Dv] of final_dtype
  float* final_lse;          // [B,Hq] or null
  int final_dtype;
  int64_t fo_sb, fo_sh;      // element strides of final_out
};

struct MmaBF16 {
  typedef bf16x8v frag8;
  typedef short4v frag4;
  __device__ static __forceinline__ float4v mma32(frag8 a, frag8 b, float4v c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  __device__ static __forceinline__ float4v mma16(frag4 a, frag4 b, float4v c) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, b, c, 0, 0, 0);
  }
  // p → (hi, lo) 16-bit patterns with hi + lo ≈ p to ~16 mantissa bits
  __device__ static __forceinline__ void split(float p0, float p1, uint32_t& hi, uint32_t& lo) {
    hi = pack_bf16x2(p0, p1);
    lo = pack_bf16x2(p0 - BF16::lo(hi), p1 - BF16::hi(hi));
  }
};
struct MmaF16 {
  typedef f16x8v frag8;
  typedef f16x4v frag4;
  __device__ static __forceinline__ float4v mma32(frag8 a, frag8 b, float4v c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  __device__ static __forceinline__ float4v mma16(frag4 a, frag4 b, float4v c) {
    return __builtin_amdgcn_mfma_f32_16x16x16f16(a, b, c, 0, 0, 0);
  }
  __device__ static __forceinline__ void split(float p0, float p1, uint32_t& hi, uint32_t& lo) {
    hi = pack_f16x2(p0, p1);
    lo = pack_f16x2(p0 - F16::lo(hi), p1 - F16::hi(hi));
  }
};

// kWaveHeads: splits one workgroup may stream through (the results of all but the last wait in registers: D / 4 each).
// `heavy`: the instances that already fill their registers (soft cap, fused merge, padded rows).
constexpr int decode_max_splits_per_team(int d, bool heavy) { return d <= 64 ? 4 : d <= 128 ? (heavy ? 3 : 4) : 2; }
constexpr int kTableSlots = 8;  // ring of page-table rows per wave (>= 2P+2)

// what the DMA lanes of a padded head dimension read for the dimensions that do not exist
static __device__ __align__(16) const unsigned char kZeroChunk[16] = {0};

// KEYS = keys per block (16 or 32): one or two groups of 16 keys, a group being one MFMA tile of scores.
// DM = value dimension = power-of-two part of the key dimension; DPE = the extra key dimensions (0 or 64).
template <int DM, int DPE, int KEYS, int NST>
struct DecodeCfg {
  static constexpr int kGroups = KEYS / 16;
  static constexpr int kRowBytes = DM * 2;
  static constexpr int kLanesPerRow = kRowBytes / 16;       // 16-byte chunks per row
  static constexpr int kRowsPerInstr = 64 / kLanesPerRow;   // rows one wave-wide DMA covers
  static constexpr int kInstrPerTensor = KEYS / kRowsPerInstr;
  static constexpr int kTensorBytes = KEYS * kRowBytes;
  // the extra key dimensions: rows of DPE * 2 bytes behind the K and V rows of the stage
  static constexpr int kPeRowBytes = DPE * 2;
  static constexpr int kPeLanesPerRow = DPE > 0 ? kPeRowBytes / 16 : 1;
  static constexpr int kPeRowsPerInstr = 64 / kPeLanesPerRow;
  static constexpr int kPeInstr = DPE > 0 ? KEYS / kPeRowsPerInstr : 0;
  static constexpr int kPeBytes = KEYS * kPeRowBytes;
  static constexpr int kPeBase = 2 * kTensorBytes;
  static constexpr int kStageBytes = 2 * kTensorBytes + kPeBytes;
  static constexpr int kLoadsPerGroup = 1 + 2 * kInstrPerTensor + kPeInstr;  // table row + K + V (+ extra K)
  static constexpr int kP = NST - 1;
  // LDS position of 16-byte chunk c of a row: K rows c ^ kswz(key), V rows c ^ vswz(key).
  // K operand reads: 16 lanes = 16 keys, same chunk      → spread over 16 positions: key & 15.
  // V transposed reads: 32 lanes = 8 keys x 2 adjacent chunks → spread the chunk pairs: (key & 7) << 1.
  static constexpr int kSwzMask = (kLanesPerRow < 16 ? kLanesPerRow : 16) - 1;
  static constexpr int kPeSwzMask = kPeLanesPerRow - 1;
  static constexpr int kTableSlotBytes = KEYS * 4;
  static constexpr int kWaveBytes = NST * kStageBytes + kTableSlots * kTableSlotBytes;
  static_assert(KEYS == 16 || KEYS == 32, "one or two key groups");
  static_assert(kP >= 1 && kP <= 3, "1..3 stages in flight");
  // vmcnt is a 6-bit counter. When a new group is issued, up to kP older ones may still be in flight; where
  // kP + 1 groups do not fit the counter (the 576-dimension heads: 35 loads per group), the loop waits for the
  // block it is about to use BEFORE it issues the next one, so only one group is ever outstanding.
  static constexpr bool kWaitFirst = (kP + 1) * kLoadsPerGroup >= 64;
  static_assert(kLoadsPerGroup < 64 && (!kWaitFirst || kP == 1), "vmcnt is 6 bits");
  static_assert(2 * kP + 2 <= kTableSlots, "table ring too small");
  static_assert(DM % 32 == 0 && DM >= 64 && DM <= 512, "head dim");
  static_assert(DPE == 0 || DPE == 64, "extra key dimensions: none or 64");
  static_assert(DPE == 0 || KEYS % kPeRowsPerInstr == 0, "whole DMA instructions for the extra key rows");
  // Rows shorter than the 256-byte bank window already differ in their row offset: only every kRowsPerWindow-th
  // key needs a new XOR term.
  static constexpr int kRowsPerWindow = kRowBytes >= 256 ? 1 : 256 / kRowBytes;
  static constexpr int kPeRowsPerWindow = DPE > 0 ? 256 / kPeRowBytes : 1;
  __device__ static __forceinline__ int kswz(int key) { return (key / kRowsPerWindow) & kSwzMask; }
  __device__ static __forceinline__ int vswz(int key) { return (((key / kRowsPerWindow) & 7) << 1) & kSwzMask; }
  __device__ static __forceinline__ int peswz(int key) { return (key / kPeRowsPerWindow) & kPeSwzMask; }
};

template <int N>
__device__ __forceinline__ void wait_groups(int rem) {
  // rem in [0, P]: number of younger load groups allowed to stay in flight
  if (rem >= 3) wait_vmcnt<(3 * N < 64 ? 3 * N : 63)>();
  else if (rem == 2) wait_vmcnt<(2 * N < 64 ? 2 * N : 63)>();
  else if (rem == 1) wait_vmcnt<N>();
  else wait_vmcnt<0>();
}

// One workgroup's split: streams its keys and writes the partial result and LSE of its 16 heads.
// Partial results that another workgroup of the same launch will read (fused merge) are written through to where
// every XCD sees them (agent-scope store: the L2 caches of the 8 XCDs are not coherent with each other); with that,
// publishing them needs no cache write-back, only the wait for the stores themselves.
template <bool kCoherent>
__device__ __forceinline__ void store_partial(float* p, float v) {
  if constexpr (kCoherent) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  else *p = v;
}
// Four consecutive floats (16-byte aligned) the same way: one 16-byte vector store, written through at agent scope
// (the sc1 bit, which is what the 4-byte atomic store above carries) where the merge reads them in the same launch.
// A store of more than 8 bytes reads its data registers one cycle after it issues: the s_nop keeps the next
// instruction, which the compiler may let write those registers, out of that cycle (for its own stores the compiler
// does this itself; it does not look into the asm).
template <bool kCoherent>
__device__ __forceinline__ void store_partial4(float* p, float4v v) {
  if constexpr (kCoherent) asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 0" ::"v"(p), "v"(v) : "memory");
  else *(float4v*)p = v;
}

// Are the B sequence lengths even enough for the form that hands a workgroup 8 kv heads of one (sequence, split)?
// Its time goes with the longest sequence, the other form's (eight times as many, smaller workgroups) with the
// sum: even means mean >= 0.8 max (measured: the one form is 7-11 % faster from mean = 0.9 max on, the other 11 % at
// 0.57 and 6 x with one long sequence among short ones). Every wave computes the same answer from the same loads, so
// two launches, one of each form, can each ask and exactly one of them does the work.
__device__ __forceinline__ bool decode_lens_even(const int32_t* lens, int B) {
  const int lane = threadIdx.x & 63;
  long long sum = 0;
  int mx = 0;
  // sixteen loads in flight per lane: one round trip for up to 1024 sequences
  for (int i0 = 0; i0 < B; i0 += 64 * 16) {
    int l[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      const int i = i0 + u * 64 + lane;
      l[u] = i < B ? lens[i] : 0;
    }
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      sum += max(l[u], 0);
      mx = max(mx, l[u]);
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const unsigned int lo = __shfl_xor((unsigned int)sum, o), hi = __shfl_xor((unsigned int)(sum >> 32), o);
    sum += (long long)(((unsigned long long)hi << 32) | lo);
    mx = max(mx, __shfl_xor(mx, o));
  }
  return sum * 5 >= (long long)mx * B * 4;
}

// kPadded: the head dimension is prm.d_valid <= D (key and value alike, a multiple of 8): the rows in the LDS are D
// wide, the 16-byte pieces beyond the real row are fetched from a page of zeros (so that the MFMA blocks see exact
// zeros there: the reference masks the same dimensions, kernels/nvidia/flash_decode.py:771-772 with BLOCK_DPE), and
// results are stored d_valid wide.
// kWaveHeads: the NW waves of a workgroup take NW neighbouring kv heads (one each, all keys of the split) instead of
// sharing one kv head's keys: together they read whole stretches of the token rows (NW * 2 * D bytes of every row) at
// the same time, and no wave waits for another: each writes its own heads' results. For at most 16 query heads per kv
// head and a number of kv heads that is a multiple of NW.
template <typename MMA, int D, int DPE, int KEYS, int NW, int NST, bool kSoftCap, bool kFuse, bool kPadded, bool kWaveHeads>
__device__ __forceinline__ void decode_split_body(const DecodeParams& prm) {
  typedef DecodeCfg<D, DPE, KEYS, NST> C;
  constexpr int G = C::kGroups;
  constexpr int DK = D + DPE;  // key (and query) dimensions; D is the value dimension
  static_assert(!kPadded || DPE == 0, "padded rows have no extra key dimensions");
  const int Dout = kPadded ? prm.d_valid : D;          // width of the stored results
  const int valid_chunks = kPadded ? prm.d_valid >> 3 : D / 8;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

  // kv heads vary fastest over the grid: workgroups that run together then read the neighbouring 2*D-byte
  // pieces of the same token rows
  const int group = prm.Hq / prm.Hkv;
  const int head_blocks = (group + 15) >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform for the compiler too
  const int lane = threadIdx.x & 63;
  const int kvh = kWaveHeads ? blockIdx.x * NW + wave : blockIdx.x / head_blocks;
  const int hb = kWaveHeads ? 0 : blockIdx.x - kvh * head_blocks;
  const int b = blockIdx.z;
  const int h0 = kvh * group + hb * 16;
  const int nvalid = min(16, group - hb * 16);
  // threads that share the work of one (kv head, head block): the workgroup, or the wave
  const int team_tid = kWaveHeads ? lane : (int)threadIdx.x;
  constexpr int kTeam = kWaveHeads ? 64 : NW * 64;
  const int g = lane >> 4;   // lane group 0..3
  const int x = lane & 15;   // head (score column) / dv within tile (V^T row) / key (K row)

  const int len = prm.lens[b];
  const int per = (len + prm.S - 1) / prm.S;
  // kWaveHeads: the team streams through splits split .. split + n_splits - 1 of its sequence, one after the other
  const int split = kWaveHeads ? blockIdx.y * prm.splits_per_team : blockIdx.y;
  const int n_splits = kWaveHeads ? min(prm.splits_per_team, prm.S - split) : 1;
  const int start = per * split;
  const int end = min(start + per, len);

  float* out_base = prm.out + (((int64_t)b * prm.Hq + h0) * prm.S + split) * Dout;
  float* lse_base = prm.lse + ((int64_t)b * prm.Hq + h0) * prm.S + split;
  if (end <= start) {
    // empty split (and with it every later one): zeros and LSE = -inf so that any merge gives it weight 0
    for (int sp = 0; sp < n_splits; ++sp) {
      for (int i = team_tid; i < nvalid * Dout; i += kTeam) {
        const int h = i / Dout, d = i - h * Dout;
        store_partial<kFuse>(out_base + ((int64_t)h * prm.S + sp) * Dout + d, 0.f);
      }
      if (team_tid < nvalid) store_partial<kFuse>(lse_base + (int64_t)team_tid * prm.S + sp, -INFINITY);
    }
    return;
  }

  typedef TDIST_AS3 unsigned char* lds_u8;  // explicit LDS pointers: a generic pointer would turn reads into
                                            // flat loads, which count on vmcnt and break the DMA accounting
  lds_u8 const smem3 = (lds_u8)smem;
  lds_u8 const wbase = smem3 + wave * C::kWaveBytes;
  lds_u8 const tbl_base = wbase + NST * C::kStageBytes;

  const int nb_total = (end - start + KEYS - 1) / KEYS;
  // this wave's blocks: every NW-th one of the kv head's; or all of its own kv head's, split after split (an empty
  // split at the sequence's end runs one block with every key masked, which writes its zeros)
  auto blocks_of = [&](int lo, int hi) { return max(1, (hi - lo + KEYS - 1) / KEYS); };
  int n_w = nb_total > wave ? (nb_total - wave + NW - 1) / NW : 0;
  if constexpr (kWaveHeads) {
    n_w = 0;
    for (int sp = 0; sp < n_splits; ++sp) n_w += blocks_of(start + sp * per, min(start + (sp + 1) * per, len));
  }

  // ---- Q fragments (B operand of the score MFMA): head x, dims 32s + 8g .. +8 -------------------
  typename MMA::frag8 qf[DK / 32];
  {
    const unsigned char* qrow = prm.q + (int64_t)b * prm.q_sb + (int64_t)(h0 + x) * prm.q_sh;
#pragma unroll
    for (int s = 0; s < DK / 32; ++s) {
      int4v raw = {0, 0, 0, 0};
      if (x < nvalid && (!kPadded || 4 * s + g < valid_chunks)) raw = *(const int4v*)(qrow + (32 * s + 8 * g) * 2);
      qf[s] = __builtin_bit_cast(typename MMA::frag8, raw);
    }
  }

  constexpr float kLog2e = 1.4426950408889634f;
  const float scale_log2 = prm.sm_scale * kLog2e;

  float m_run = -INFINITY;  // running max (log2 domain) of head x, identical in the 4 lane groups
  float l_run = 0.f;        // this lane group's share of the running sum
  float4v acc[D / 16];
#pragma unroll
  for (int d = 0; d < D / 16; ++d) acc[d] = float4v{0.f, 0.f, 0.f, 0.f};

  // Loop-invariant LDS offsets (relative to the stage) of this lane's operand reads.
  // K (A operand of the scores): row = key x of group q, logical chunk 4s+g.
  // The extra key dimensions D + 32s' + 8g live in their own rows behind the K and V rows.
  int koff[G][DK / 32];
#pragma unroll
  for (int q = 0; q < G; ++q)
#pragma unroll
    for (int s = 0; s < DK / 32; ++s) {
      const int key = 16 * q + x;
      if (s < D / 32) koff[q][s] = key * C::kRowBytes + (((4 * s + g) ^ C::kswz(key)) << 4);
      else koff[q][s] = C::kPeBase + key * C::kPeRowBytes + (((4 * (s - D / 32) + g) ^ C::peswz(key)) << 4);
    }
  // V^T (A operand of the output MFMA) through the transposing LDS read: within a 16-lane block, lane x ends
  // up with elements x, 16+x, 32+x, 48+x of the 64 the block loads (lane s loads 4 consecutive ones), so lane s
  // supplies V[key 4g + s/4 of group q][dv 16d + 4(s%4) .. +3] and lane x receives V[4g+j][16d+x], j = 0..3.
  int voff[G][D / 16];
#pragma unroll
  for (int q = 0; q < G; ++q)
#pragma unroll
    for (int d = 0; d < D / 16; ++d) {
      const int key = 16 * q + 4 * g + (x >> 2);
      const int chunk = 2 * d + ((x & 3) >> 1);
      voff[q][d] = C::kTensorBytes + key * C::kRowBytes + ((chunk ^ C::vswz(key)) << 4) + (x & 1) * 8;
    }

  // A block: its first key and the key range [lo, hi) of its split. Keys outside the range are read as the nearest
  // key inside (and, for a split that is empty, as the sequence's last key) and masked in the scores.
  struct Block { int key0, lo, hi; };
  auto clamp_key = [&](int n, const Block& blk) {
    n = max(min(n, blk.hi - 1), blk.lo);
    if constexpr (kWaveHeads) n = min(n, len - 1);
    return n;
  };
  // first key of the wave's j-th block where the workgroup shares one split
  auto shared_block = [&](int j) { return Block{start + (wave + j * NW) * KEYS, start, end}; };
  // kWaveHeads: a cursor over the team's blocks in order
  struct Cursor { Block blk; int left; };   // left: blocks of this split still to come, this one included
  auto cursor_begin = [&]() { return Cursor{Block{start, start, end}, blocks_of(start, end)}; };
  auto cursor_next = [&](Cursor& c) {
    c.blk.key0 += KEYS;
    if (--c.left == 0) {
      c.blk.lo += per;
      c.blk.hi = min(c.blk.lo + per, len);
      c.blk.key0 = c.blk.lo;
      c.left = blocks_of(c.blk.lo, c.blk.hi);
    }
  };

  // page-table row of block j → table ring slot j % kTableSlots (one entry per key)
  auto issue_table = [&](int j, const Block& blk) {
    if (lane < KEYS) {
      const int n = clamp_key(blk.key0 + lane, blk);
      const int e = (int)(((uint64_t)(uint32_t)n * prm.page_magic) >> prm.page_shift);
      const int32_t* src = prm.table + (int64_t)b * prm.t_s + e;
      __builtin_amdgcn_global_load_lds((const TDIST_AS1 void*)src,
                                       (TDIST_AS3 void*)(tbl_base + (j % kTableSlots) * C::kTableSlotBytes), 4, 0, 0);
    }
  };

  // K and V rows of block j → stage j % NST
  auto issue_rows = [&](int j, const Block& blk) {
    const int key0 = blk.key0;
    const volatile TDIST_AS3 int32_t* tbl =
        (const volatile TDIST_AS3 int32_t*)(tbl_base + (j % kTableSlots) * C::kTableSlotBytes);
    lds_u8 const kst = wbase + (j % NST) * C::kStageBytes;
    lds_u8 const vst = kst + C::kTensorBytes;
    const int chunk = lane % C::kLanesPerRow;
#pragma unroll
    for (int i = 0; i < C::kInstrPerTensor; ++i) {
      const int key = i * C::kRowsPerInstr + lane / C::kLanesPerRow;
      const int n = clamp_key(key0 + key, blk);
      const uint32_t page = (uint32_t)tbl[key];
      const uint32_t in_page = (uint32_t)n - (uint32_t)(((uint64_t)(uint32_t)n * prm.page_magic) >> prm.page_shift) * (uint32_t)prm.page_size;
      const unsigned char* ksrc = prm.k + (uint64_t)page * (uint64_t)prm.k_sp +
                                  (in_page * (uint32_t)prm.k_st + (uint32_t)kvh * (uint32_t)prm.k_sh + ((chunk ^ C::kswz(key)) << 4));
      const unsigned char* vsrc = prm.v + (uint64_t)page * (uint64_t)prm.v_sp +
                                  (in_page * (uint32_t)prm.v_st + (uint32_t)kvh * (uint32_t)prm.v_sh + ((chunk ^ C::vswz(key)) << 4));
      if constexpr (kPadded) {
        if ((chunk ^ C::kswz(key)) >= valid_chunks) ksrc = kZeroChunk;
        if ((chunk ^ C::vswz(key)) >= valid_chunks) vsrc = kZeroChunk;
      }
      __builtin_amdgcn_global_load_lds((const TDIST_AS1 void*)ksrc, (TDIST_AS3 void*)(kst + i * 1024), 16, 0, TDIST_KV_AUX);
      __builtin_amdgcn_global_load_lds((const TDIST_AS1 void*)vsrc, (TDIST_AS3 void*)(vst + i * 1024), 16, 0, TDIST_KV_AUX);
    }
    if constexpr (DPE > 0) {
      lds_u8 const pst = kst + C::kPeBase;
      const int pchunk = lane % C::kPeLanesPerRow;
#pragma unroll
      for (int i = 0; i < C::kPeInstr; ++i) {
        const int key = i * C::kPeRowsPerInstr + lane / C::kPeLanesPerRow;
        const int n = clamp_key(key0 + key, blk);
        const uint32_t page = (uint32_t)tbl[key];
        const uint32_t in_page = (uint32_t)n - (uint32_t)(((uint64_t)(uint32_t)n * prm.page_magic) >> prm.page_shift) * (uint32_t)prm.page_size;
        const unsigned char* psrc = prm.k + (uint64_t)page * (uint64_t)prm.k_sp +
                                    (in_page * (uint32_t)prm.k_st + (uint32_t)kvh * (uint32_t)prm.k_sh +
                                     (uint32_t)(C::kRowBytes + ((pchunk ^ C::peswz(key)) << 4)));
        __builtin_amdgcn_global_load_lds((const TDIST_AS1 void*)psrc, (TDIST_AS3 void*)(pst + i * 1024), 16, 0, TDIST_KV_AUX);
      }
    }
  };

  auto compute = [&](int j, const Block& blk) {
    const int key0 = blk.key0;
    lds_u8 const st = wbase + (j % NST) * C::kStageBytes;
    // scores: A = K rows (key x of group q, dims 32s+8g..), B = Q  →  sc[q][i]: key 16q+4g+i, head x
    float4v sc[G];
#pragma unroll
    for (int q = 0; q < G; ++q) {
      sc[q] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < DK / 32; ++s) {
        const int4v raw = *(const TDIST_AS3 int4v*)(st + koff[q][s]);
        sc[q] = MMA::mma32(__builtin_bit_cast(typename MMA::frag8, raw), qf[s], sc[q]);
      }
    }
    float t[G][4];
    float mx = -INFINITY;
#pragma unroll
    for (int q = 0; q < G; ++q)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v;
        if (kSoftCap) {
          v = prm.soft_cap * tanhf(sc[q][i] * prm.sm_scale / prm.soft_cap) * kLog2e;
        } else {
          v = sc[q][i] * scale_log2;
        }
        const bool valid = key0 + 16 * q + 4 * g + i < blk.hi;
        t[q][i] = valid ? v : -INFINITY;
        mx = fmaxf(mx, t[q][i]);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16));
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float m_new = fmaxf(m_run, mx);
    if (__any(m_new > m_run)) {
      const float alpha = (m_run == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m_run - m_new);
      l_run *= alpha;
#pragma unroll
      for (int d = 0; d < D / 16; ++d) acc[d] *= alpha;
      m_run = m_new;
    }
    const float m_safe = (m_run == -INFINITY) ? 0.f : m_run;
    // probabilities as the B operand: k slots 4q..4q+3 of lane group g ↔ keys 16q+4g .. +3
    uint32_t hi[G][2], lo[G][2];
#pragma unroll
    for (int q = 0; q < G; ++q) {
      float p[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        p[i] = __builtin_amdgcn_exp2f(t[q][i] - m_safe);
        l_run += p[i];
      }
      MMA::split(p[0], p[1], hi[q][0], lo[q][0]);
      MMA::split(p[2], p[3], hi[q][1], lo[q][1]);
    }
    // O^T tiles: A = V^T (dv 16d+x; k slots as above), B = P^T
#pragma unroll
    for (int d = 0; d < D / 16; ++d) {
      if (G == 2) {
        const short4v v0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((TDIST_AS3 short4v*)(st + voff[0][d]));
        const short4v v1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((TDIST_AS3 short4v*)(st + voff[G - 1][d]));
        const int2v a0 = __builtin_bit_cast(int2v, v0), a1 = __builtin_bit_cast(int2v, v1);
        const int4v vt = {a0[0], a0[1], a1[0], a1[1]};
        const int4v ph = {(int)hi[0][0], (int)hi[0][1], (int)hi[G - 1][0], (int)hi[G - 1][1]};
        const int4v pl = {(int)lo[0][0], (int)lo[0][1], (int)lo[G - 1][0], (int)lo[G - 1][1]};
        const typename MMA::frag8 vf = __builtin_bit_cast(typename MMA::frag8, vt);
        acc[d] = MMA::mma32(vf, __builtin_bit_cast(typename MMA::frag8, ph), acc[d]);
        acc[d] = MMA::mma32(vf, __builtin_bit_cast(typename MMA::frag8, pl), acc[d]);
      } else {
        const short4v v0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((TDIST_AS3 short4v*)(st + voff[0][d]));
        const int2v ph = {(int)hi[0][0], (int)hi[0][1]};
        const int2v pl = {(int)lo[0][0], (int)lo[0][1]};
        const typename MMA::frag4 vf = __builtin_bit_cast(typename MMA::frag4, v0);
        acc[d] = MMA::mma16(vf, __builtin_bit_cast(typename MMA::frag4, ph), acc[d]);
        acc[d] = MMA::mma16(vf, __builtin_bit_cast(typename MMA::frag4, pl), acc[d]);
      }
    }
  };

  constexpr float kLn2 = 0.6931471805599453f;
  if constexpr (kWaveHeads) {
    static_assert(!C::kWaitFirst, "a kv head per wave: several groups in flight");
    // One pipeline over all blocks of the team's splits: the loads of the next split's first blocks are in flight
    // while the last blocks of this one are computed. The results go out of the registers (no LDS: the ring belongs
    // to the loads in flight) when the stream has ended.
    Cursor c_tbl = cursor_begin(), c_rows = cursor_begin(), c_cmp = cursor_begin();
    int j_tbl = 0;
    for (; j_tbl <= C::kP; ++j_tbl) {
      issue_table(j_tbl, c_tbl.blk);
      cursor_next(c_tbl);
    }
    wait_vmcnt<0>();
    for (int gi = 0; gi < C::kP; ++gi) {
      if (gi < n_w) {
        issue_table(j_tbl++, c_tbl.blk);
        cursor_next(c_tbl);
        issue_rows(gi, c_rows.blk);
        cursor_next(c_rows);
      }
    }
    // results of the splits before the team's last one, held until the stream ends
    constexpr int kMaxHeld = decode_max_splits_per_team(D, kSoftCap || kFuse || kPadded) - 1;
    float4v held[kMaxHeld][D / 16];
    float held_lse[kMaxHeld];
#pragma unroll
    for (int u = 0; u < kMaxHeld; ++u) {
      held_lse[u] = 0.f;
#pragma unroll
      for (int d = 0; d < D / 16; ++d) held[u][d] = float4v{0.f, 0.f, 0.f, 0.f};
    }
    int sp = 0;
    for (int i = 0; i < n_w; ++i) {
      if (i + C::kP < n_w) {
        issue_table(j_tbl++, c_tbl.blk);
        cursor_next(c_tbl);
        issue_rows(i + C::kP, c_rows.blk);
        cursor_next(c_rows);
      }
      wait_groups<C::kLoadsPerGroup>(min(C::kP, n_w - 1 - i));
      compute(i, c_cmp.blk);
      if (c_cmp.left == 1) {
        // the split's last block: this lane holds dimensions 16d + 4g .. + 3 of head x
        float L = l_run + __shfl_xor(l_run, 16);
        L += __shfl_xor(L, 32);
        float4v r[D / 16];
#pragma unroll
        for (int d = 0; d < D / 16; ++d)
#pragma unroll
          for (int e = 0; e < 4; ++e) r[d][e] = L > 0.f ? acc[d][e] / L : 0.f;
        const float r_lse = L > 0.f ? (m_run + log2f(L)) * kLn2 : -INFINITY;
        auto store_split = [&](int which, const float4v(&val)[D / 16], float val_lse) {
          if (x < nvalid) {
            float* o = out_base + ((int64_t)x * prm.S + which) * Dout + 4 * g;
#pragma unroll
            for (int d = 0; d < D / 16; ++d)
              if (!kPadded || 16 * d + 4 * g < Dout) store_partial4<kFuse>(o + 16 * d, val[d]);
            if (g == 0) store_partial<kFuse>(lse_base + (int64_t)x * prm.S + which, val_lse);
          }
        };
        if (i == n_w - 1) {
          // the team's last split: everything goes out now
#pragma unroll
          for (int u = 0; u < kMaxHeld; ++u)
            if (u < sp) store_split(u, held[u], held_lse[u]);
          store_split(sp, r, r_lse);
        } else {
          // Not yet: stores count on the same counter as the loads, so the next wait for a block would also wait for
          // these stores, which take tens of microseconds to be acknowledged while the read stream runs (measured:
          // 40 us per launch at 8 stores per wave). The result waits in registers for the end of the stream.
#pragma unroll
          for (int u = 0; u < kMaxHeld; ++u)
            if (sp == u) {
#pragma unroll
              for (int d = 0; d < D / 16; ++d) held[u][d] = r[d];
              held_lse[u] = r_lse;
            }
        }
        ++sp;
        m_run = -INFINITY;
        l_run = 0.f;
#pragma unroll
        for (int d = 0; d < D / 16; ++d) acc[d] = float4v{0.f, 0.f, 0.f, 0.f};
      }
      cursor_next(c_cmp);
    }
    return;
  }

  if (n_w > 0) {
    // page-table rows of the first P+1 blocks, then the first P row groups
    for (int j = 0; j <= C::kP; ++j) issue_table(j, shared_block(j));
    wait_vmcnt<0>();
    for (int gi = -C::kP; gi < 0; ++gi) {
      if (gi + C::kP < n_w) {
        issue_table(gi + 2 * C::kP + 1, shared_block(gi + 2 * C::kP + 1));
        issue_rows(gi + C::kP, shared_block(gi + C::kP));
      }
    }
    for (int i = 0; i < n_w; ++i) {
      if constexpr (C::kWaitFirst) wait_vmcnt<0>();
      if (i + C::kP < n_w) {
        issue_table(i + 2 * C::kP + 1, shared_block(i + 2 * C::kP + 1));
        issue_rows(i + C::kP, shared_block(i + C::kP));
      }
      if constexpr (!C::kWaitFirst) wait_groups<C::kLoadsPerGroup>(min(C::kP, n_w - 1 - i));
      compute(i, shared_block(i));
    }
  }

  // ---- merge the waves' partial states ---------------------------------------------------------
  l_run += __shfl_xor(l_run, 16);
  l_run += __shfl_xor(l_run, 32);
  wait_vmcnt<0>();
  __syncthreads();  // every wave is done with its ring; reuse it
  TDIST_AS3 float* s_m = (TDIST_AS3 float*)(wbase);  // [16]
  TDIST_AS3 float* s_l = s_m + 16;                   // [16]
  TDIST_AS3 float* s_acc = s_l + 16;                 // [D][16]
  if (lane < 16) {
    s_m[lane] = m_run;
    s_l[lane] = l_run;
  }
#pragma unroll
  for (int d = 0; d < D / 16; ++d)
#pragma unroll
    for (int i = 0; i < 4; ++i) s_acc[(16 * d + 4 * g + i) * 16 + x] = acc[d][i];
  __syncthreads();
  for (int idx = threadIdx.x; idx < nvalid * Dout; idx += NW * 64) {
    const int h = idx / Dout, dv = idx - h * Dout;
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < NW; ++w) M = fmaxf(M, ((const TDIST_AS3 float*)(smem3 + w * C::kWaveBytes))[h]);
    float L = 0.f, O = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const TDIST_AS3 float* wm = (const TDIST_AS3 float*)(smem3 + w * C::kWaveBytes);
      const float mw = wm[h];
      const float sc = (mw == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(mw - M);
      L += wm[16 + h] * sc;
      O += wm[32 + dv * 16 + h] * sc;
    }
    store_partial<kFuse>(out_base + (int64_t)h * prm.S * Dout + dv, O / L);
    if (dv == 0) store_partial<kFuse>(lse_base + (int64_t)h * prm.S, (M + log2f(L)) * kLn2);
  }
}

// ---- combine --------------------------------------------------------------------------------------
struct CombineParams {
  const unsigned char* part;
  const float* lse;
  const int32_t* lens;
  unsigned char* out;
  float* lse_out;
  int P, mode, B, Hq, Dv;
  int part_dtype, out_dtype;
  int64_t p_sp, p_sb, p_sh;  // element strides
  int64_t l_sp, l_sb, l_sh;
  int64_t o_sb, o_sh;
};

__device__ __forceinline__ float load_elem(const unsigned char* base, int64_t idx, int dtype) {
  if (dtype == TDIST_F32) return ((const float*)base)[idx];
  const uint32_t bits = ((const unsigned short*)base)[idx];
  return dtype == TDIST_BF16 ? bf16_bits_to_f32(bits) : f16_bits_to_f32(bits);
}
__device__ __forceinline__ void store_elem(unsigned char* base, int64_t idx, int dtype, float v) {
  if (dtype == TDIST_F32) ((float*)base)[idx] = v;
  else if (dtype == TDIST_BF16) ((unsigned short*)base)[idx] = (unsigned short)f32_to_bf16_bits(v);
  else ((unsigned short*)base)[idx] = (unsigned short)(pack_f16x2(v, 0.f) & 0xffffu);
}

// One wave per (b,h); lanes stride over Dv. Partial j is weighted by exp(lse_j - max).
// Lane j holds the LSE of partial j (one load per lane instead of a loop of loads in every lane; -inf where the
// partial is skipped), the maximum is a wave reduction, and the partial rows of up to 32 / kPerLane partials are in
// flight together: two round trips to memory for a merge of 16 partials. The sums run over the partials in index
// order, whatever the batching.
template <int kPerLane>
__global__ __launch_bounds__(256) void decode_combine_kernel(const CombineParams prm) {
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int64_t bh = (int64_t)blockIdx.x * 4 + wave;
  if (bh >= (int64_t)prm.B * prm.Hq) return;
  const int b = (int)(bh / prm.Hq);
  const int h = (int)(bh - (int64_t)b * prm.Hq);
  auto skipped = [&](int j) -> bool {
    if (prm.mode == 1) {
      const int len = prm.lens[b];
      const int per = (len + prm.P - 1) / prm.P;
      const int st = per * j;
      return min(st + per, len) <= st;
    }
    if (prm.mode == 2) return prm.lens[(int64_t)j * prm.B + b] == 0;
    return false;
  };
  const float* lse = prm.lse + (int64_t)b * prm.l_sb + (int64_t)h * prm.l_sh;
  // LSE of partial j0 + lane
  auto lse_of_lane = [&](int j0) -> float {
    const int j = j0 + lane;
    return (j < prm.P && !skipped(j)) ? lse[(int64_t)j * prm.l_sp] : -INFINITY;
  };
  float M = -INFINITY;
  for (int j0 = 0; j0 < prm.P; j0 += 64) M = fmaxf(M, lse_of_lane(j0));
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) M = fmaxf(M, __shfl_xor(M, o));
  float L = 0.f;
  float acc[kPerLane];
#pragma unroll
  for (int q = 0; q < kPerLane; ++q) acc[q] = 0.f;
  if (M != -INFINITY) {
    constexpr int kBatch = 32 / kPerLane;
    for (int c0 = 0; c0 < prm.P; c0 += 64) {
      const float l_lane = lse_of_lane(c0);
      const int n_here = min(64, prm.P - c0);
      for (int j0 = 0; j0 < n_here; j0 += kBatch) {
        float w[kBatch];
        float x[kBatch][kPerLane];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
          const int jj = j0 + u;   // (within the chunk; lanes beyond it hold -inf)
          const float lj = jj < 64 ? __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, l_lane), jj & 63)) : -INFINITY;
          w[u] = lj == -INFINITY ? 0.f : __expf(lj - M);
          const int64_t base = (int64_t)min(c0 + jj, prm.P - 1) * prm.p_sp + (int64_t)b * prm.p_sb + (int64_t)h * prm.p_sh;
#pragma unroll
          for (int q = 0; q < kPerLane; ++q) {
            const int d = lane + q * 64;
            x[u][q] = (d < prm.Dv && lj != -INFINITY) ? load_elem(prm.part, base + d, prm.part_dtype) : 0.f;
          }
        }
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
          L += w[u];   // a skipped, empty or out-of-range partial has w = 0 and x = 0: it adds nothing
#pragma unroll
          for (int q = 0; q < kPerLane; ++q) acc[q] += w[u] * x[u][q];
        }
      }
    }
  }
  const int64_t obase = (int64_t)b * prm.o_sb + (int64_t)h * prm.o_sh;
#pragma unroll
  for (int u = 0; u < kPerLane; ++u) {
    const int d = lane + u * 64;
    if (d < prm.Dv) store_elem(prm.out, obase + d, prm.out_dtype, L > 0.f ? acc[u] / L : 0.f);
  }
  if (prm.lse_out && lane == 0) prm.lse_out[bh] = L > 0.f ? M + logf(L) : -INFINITY;
}

// Fused tail: publishes this team's partial result (the workgroup's, or with kWaveHeads the wave's); the last of the
// S teams of a (sequence, head block) to get here merges their partials (same arithmetic, in the same order, as
// decode_combine_kernel in mode 1) and puts the counter back to zero for the next launch.
template <int DM, int NW, bool kPadded, bool kWaveHeads>
__device__ __forceinline__ void decode_fused_merge(const DecodeParams& prm) {
  const int D = kPadded ? prm.d_valid : DM;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  TDIST_AS3 int* const s_last = (TDIST_AS3 int*)smem;
  const int group = prm.Hq / prm.Hkv;
  const int head_blocks = (group + 15) >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int kvh = kWaveHeads ? blockIdx.x * NW + wave : blockIdx.x / head_blocks;
  const int hb = kWaveHeads ? 0 : blockIdx.x - kvh * head_blocks;
  const int b = blockIdx.z;
  const int h0 = kvh * group + hb * 16;
  const int nvalid = min(16, group - hb * 16);
  const int team_tid = kWaveHeads ? (int)(threadIdx.x & 63) : (int)threadIdx.x;
  constexpr int kTeam = kWaveHeads ? 64 : NW * 64;
  // one counter per (sequence, kv head, head block)
  int32_t* const ctr = prm.counters + ((int64_t)b * prm.Hkv + kvh) * head_blocks + hb;

  // This thread's partial results were stored write-through (store_partial): once the stores have completed they
  // are visible to every XCD. (A release fence here would write back the whole L2 once per wave: measured at 2x the
  // kernel time.)
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  if constexpr (kWaveHeads) {
    // the wave's stores are complete: its first lane counts, and tells the others
    // (its team brought n_mine of the S splits)
    const int n_mine = min(prm.splits_per_team, prm.S - (int)blockIdx.y * prm.splits_per_team);
    int last = 0;
    if (team_tid == 0) {
      const int old = __hip_atomic_fetch_add(ctr, n_mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      last = old + n_mine == prm.S;
      if (last) __hip_atomic_store(ctr, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (!__builtin_amdgcn_readfirstlane(last)) return;
  } else {
    // the barrier orders all of the workgroup's stores before thread 0's counter update
    __syncthreads();   // (also: every wave is done with the merge scratch that s_last overlays)
    if (threadIdx.x == 0) {
      const int old = __hip_atomic_fetch_add(ctr, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const int last = old == prm.S - 1;
      if (last) __hip_atomic_store(ctr, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      *s_last = last;
    }
    __syncthreads();
    if (!*s_last) return;
  }
  // The counter has reached S: every other team's stores completed before its increment. Only the merging team pays
  // for an acquire (it drops this CU's and this XCD's possibly stale lines; the K/V stream is non-temporal and
  // loses nothing by it), after which plain vector loads may read the partial results.
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");

  const float* lse_p = prm.lse + ((int64_t)b * prm.Hq + h0) * prm.S;
  const float* out_p = prm.out + ((int64_t)b * prm.Hq + h0) * prm.S * D;
  const int kVecs = D / 4;
  for (int idx = team_tid; idx < nvalid * kVecs; idx += kTeam) {
    const int h = idx / kVecs, dv = (idx - h * kVecs) * 4;
    const float* l = lse_p + (int64_t)h * prm.S;
    // sixteen splits at a time: their LSEs, then their rows, are in flight together (two round trips for 16 splits);
    // the sums run over the splits in order
    constexpr int kBatch = 16;
    float M = -INFINITY;
    for (int j0 = 0; j0 < prm.S; j0 += kBatch) {
      float lj[kBatch];
#pragma unroll
      for (int u = 0; u < kBatch; ++u) lj[u] = j0 + u < prm.S ? l[j0 + u] : -INFINITY;
#pragma unroll
      for (int u = 0; u < kBatch; ++u) M = fmaxf(M, lj[u]);
    }
    float L = 0.f;
    float4v acc = {0.f, 0.f, 0.f, 0.f};
    if (M != -INFINITY) {
      // an empty split has LSE = -inf and zeros: weight exp(-inf) = 0 adds nothing, as skipping it would
      for (int j0 = 0; j0 < prm.S; j0 += kBatch) {
        float lj[kBatch];
        float4v x[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
          const int j = min(j0 + u, prm.S - 1);
          lj[u] = l[j];
          x[u] = *(const float4v*)(out_p + ((int64_t)h * prm.S + j) * D + dv);
        }
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
          if (j0 + u < prm.S) {
            const float w = __expf(lj[u] - M);
            L += w;
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] += w * x[u][e];
          }
        }
      }
    }
    const int64_t o = (int64_t)b * prm.fo_sb + (int64_t)(h0 + h) * prm.fo_sh + dv;
#pragma unroll
    for (int e = 0; e < 4; ++e) store_elem(prm.final_out, o + e, prm.final_dtype, L > 0.f ? acc[e] / L : 0.f);
    if (dv == 0 && prm.final_lse) prm.final_lse[(int64_t)b * prm.Hq + h0 + h] = L > 0.f ? M + logf(L) : -INFINITY;
  }
}

template <typename MMA, int D, int DPE, int KEYS, int NW, int NST, bool kSoftCap, bool kFuse, bool kPadded, bool kWaveHeads = false>
__global__ __launch_bounds__(NW * 64) void decode_split_kv_kernel(const DecodeParams prm) {
  if (prm.when_lens != 0 && decode_lens_even(prm.lens, prm.B) != (prm.when_lens == 1)) return;
  decode_split_body<MMA, D, DPE, KEYS, NW, NST, kSoftCap, kFuse, kPadded, kWaveHeads>(prm);
  if constexpr (kFuse) decode_fused_merge<D, NW, kPadded, kWaveHeads>(prm);
}

template <typename MMA, int D, int DPE, int KEYS, int NW, int NST, bool kSoftCap, bool kFuse, bool kPadded, bool kWaveHeads = false>
static int launch_decode_cfg(const DecodeParams& prm, int head_blocks, hipStream_t stream) {
  typedef DecodeCfg<D, DPE, KEYS, NST> C;
  static_assert((32 + D * 16) * 4 <= C::kWaveBytes, "merge scratch must fit in a wave's ring");
  const size_t lds = (size_t)NW * C::kWaveBytes;
  static_assert((size_t)NW * C::kWaveBytes <= 160 * 1024, "LDS of one CU");
  auto kern = decode_split_kv_kernel<MMA, D, DPE, KEYS, NW, NST, kSoftCap, kFuse, kPadded, kWaveHeads>;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return fail(TDIST_ERR_LAUNCH, "decode: cannot reserve %zu B of LDS: %s", lds, hipGetErrorString(e));
    attr_set = true;
  }
  dim3 grid(kWaveHeads ? prm.Hkv / NW : prm.Hkv * head_blocks,
            kWaveHeads ? (prm.S + prm.splits_per_team - 1) / prm.splits_per_team : prm.S, prm.B);
  hipLaunchKernelGGL(kern, grid, dim3(NW * 64), lds, stream, prm);
  return launch_status(kFuse ? "tdist_decode_fused" : "tdist_decode_split_kv");
}

template <typename MMA, int D, int DPE, int KEYS, int NW, int NST, bool kPadded = false>
static int launch_decode(const DecodeParams& prm, int head_blocks, hipStream_t stream) {
  const bool fuse = prm.counters != nullptr;
  if (prm.soft_cap > 0.f)
    return fuse ? launch_decode_cfg<MMA, D, DPE, KEYS, NW, NST, true, true, kPadded>(prm, head_blocks, stream)
                : launch_decode_cfg<MMA, D, DPE, KEYS, NW, NST, true, false, kPadded>(prm, head_blocks, stream);
  return fuse ? launch_decode_cfg<MMA, D, DPE, KEYS, NW, NST, false, true, kPadded>(prm, head_blocks, stream)
              : launch_decode_cfg<MMA, D, DPE, KEYS, NW, NST, false, false, kPadded>(prm, head_blocks, stream);
}

}  // namespace tdist

using namespace tdist;

namespace tdist {

struct DecodeCall {
  const void *q, *k_cache, *v_cache;
  float *out_split, *lse_split;
  float sm_scale, soft_cap;
  const int32_t *block_table, *kv_lens;
  int batch, q_heads, kv_heads, head_dim, head_dim_v, page_size, num_splits;
  int64_t q_stride_b, q_stride_h, k_stride_page, k_stride_token, k_stride_head, v_stride_page, v_stride_token,
      v_stride_head, table_stride;
  int dtype;
  // fused merge
  int32_t* counters;
  int64_t n_counters;
  void* out;
  int out_dtype;
  int64_t out_stride_b, out_stride_h;
  float* lse_out;
  void* stream;
  const char* who;
};

static int64_t decode_fused_counters(int batch, int q_heads, int kv_heads) {
  if (batch <= 0 || q_heads <= 0 || kv_heads <= 0 || q_heads % kv_heads != 0) return -1;
  const int group = q_heads / kv_heads;
  return (int64_t)batch * kv_heads * ((group + 15) / 16);
}

static int run_decode(const DecodeCall& c, bool fuse) {
  const char* who = c.who;
  if (!c.q || !c.k_cache || !c.v_cache || !c.out_split || !c.lse_split || !c.block_table || !c.kv_lens)
    return fail(TDIST_ERR_INVALID, "%s: null pointer", who);
  if (c.batch <= 0 || c.q_heads <= 0 || c.kv_heads <= 0 || c.page_size <= 0 || c.num_splits <= 0)
    return fail(TDIST_ERR_INVALID, "%s: sizes must be positive", who);
  if (c.q_heads % c.kv_heads != 0)
    return fail(TDIST_ERR_INVALID, "%s: q_heads %d not a multiple of kv_heads %d", who, c.q_heads, c.kv_heads);
  if (c.dtype != TDIST_BF16 && c.dtype != TDIST_F16)
    return fail(TDIST_ERR_UNSUPPORTED, "%s: dtype %d (bf16 and f16 only)", who, c.dtype);
  const int dk = c.head_dim, dv = c.head_dim_v;
  const bool padded = dk == dv && dk > 0 && dk < 256 && dk % 8 == 0 && dk != 64 && dk != 128;
  const bool dims_ok = (dk == dv && (dk == 64 || dk == 128 || dk == 256)) || (dk == 192 && dv == 128) ||
                       (dk == 576 && dv == 512) || padded;
  if (!dims_ok)
    return fail(TDIST_ERR_UNSUPPORTED, "%s: head dims (%d, %d): equal ones that are a multiple of 8 up to 256, (192,128) "
                "and (576,512) only", who, dk, dv);
  if (!aligned16(c.q) || !aligned16(c.k_cache) || !aligned16(c.v_cache) || (c.q_stride_b % 8) || (c.q_stride_h % 8) ||
      (c.k_stride_page % 8) || (c.k_stride_token % 8) || (c.k_stride_head % 8) || (c.v_stride_page % 8) ||
      (c.v_stride_token % 8) || (c.v_stride_head % 8))
    return fail(TDIST_ERR_UNSUPPORTED, "%s: q/k/v rows must be 16-byte aligned", who);
  if (c.num_splits > 65535 || c.batch > 65535) return fail(TDIST_ERR_UNSUPPORTED, "%s: grid too large", who);
  DecodeParams prm;
  prm.q = (const unsigned char*)c.q;
  prm.k = (const unsigned char*)c.k_cache;
  prm.v = (const unsigned char*)c.v_cache;
  prm.out = c.out_split;
  prm.lse = c.lse_split;
  prm.table = c.block_table;
  prm.lens = c.kv_lens;
  prm.sm_scale = c.sm_scale;
  prm.soft_cap = c.soft_cap;
  prm.B = c.batch;
  prm.Hq = c.q_heads;
  prm.Hkv = c.kv_heads;
  prm.S = c.num_splits;
  prm.d_valid = dk;
  prm.splits_per_team = 1;
  prm.when_lens = 0;
  prm.page_size = c.page_size;
  int lg = 0;
  while ((1ll << lg) < c.page_size) ++lg;
  prm.page_shift = 31 + lg;
  prm.page_magic = ((1ull << prm.page_shift) + (uint64_t)c.page_size - 1) / (uint64_t)c.page_size;
  prm.q_sb = c.q_stride_b * 2;
  prm.q_sh = c.q_stride_h * 2;
  prm.k_sp = c.k_stride_page * 2;
  prm.k_st = c.k_stride_token * 2;
  prm.k_sh = c.k_stride_head * 2;
  prm.v_sp = c.v_stride_page * 2;
  prm.v_st = c.v_stride_token * 2;
  prm.v_sh = c.v_stride_head * 2;
  prm.t_s = c.table_stride;
  prm.counters = nullptr;
  prm.final_out = nullptr;
  prm.final_lse = nullptr;
  prm.final_dtype = TDIST_F32;
  prm.fo_sb = prm.fo_sh = 0;
  if (fuse) {
    if (!c.counters || !c.out) return fail(TDIST_ERR_INVALID, "%s: null counters or output", who);
    if (!aligned16(c.out_split)) return fail(TDIST_ERR_UNSUPPORTED, "%s: out_split must be 16-byte aligned", who);
    if (c.out_dtype != TDIST_F32 && c.out_dtype != TDIST_BF16 && c.out_dtype != TDIST_F16)
      return fail(TDIST_ERR_UNSUPPORTED, "%s: output dtype %d", who, c.out_dtype);
    const int64_t need = decode_fused_counters(c.batch, c.q_heads, c.kv_heads);
    if (c.n_counters < need)
      return fail(TDIST_ERR_WORKSPACE, "%s: %lld counters given, %lld needed", who, (long long)c.n_counters, (long long)need);
    prm.counters = c.counters;
    prm.final_out = (unsigned char*)c.out;
    prm.final_lse = c.lse_out;
    prm.final_dtype = c.out_dtype;
    prm.fo_sb = c.out_stride_b;
    prm.fo_sh = c.out_stride_h;
  }
  const int group = c.q_heads / c.kv_heads;
  const int head_blocks = (group + 15) / 16;
  if ((int64_t)c.kv_heads * head_blocks > 65535) return fail(TDIST_ERR_UNSUPPORTED, "%s: too many heads", who);
  hipStream_t st = (hipStream_t)c.stream;
  const bool bf = c.dtype == TDIST_BF16;
  // <dtype, Dv, extra key dims, keys per block, waves, stages>:
  // LDS = waves * (stages * keys * (Dk + Dv) * 2 B + tables) <= 160 KB
#define TDIST_DEC(D_, DPE_, KEYS_, NW_, NST_)                                             \
  return bf ? launch_decode<MmaBF16, D_, DPE_, KEYS_, NW_, NST_>(prm, head_blocks, st)   \
            : launch_decode<MmaF16, D_, DPE_, KEYS_, NW_, NST_>(prm, head_blocks, st);
#define TDIST_DEC_PADDED(D_, KEYS_, NW_, NST_)                                                 \
  return bf ? launch_decode<MmaBF16, D_, 0, KEYS_, NW_, NST_, true>(prm, head_blocks, st)     \
            : launch_decode<MmaF16, D_, 0, KEYS_, NW_, NST_, true>(prm, head_blocks, st);
  // A kv head per wave (8 waves of 2 stages or 4 waves of 4, 130-136 KB: one workgroup per CU) where the heads allow
  // it, the grid fills the CUs in whole rounds or in many (such a workgroup is NW_ times the work of one of the other
  // form, whose small workgroups fill a small grid's CUs better) and the cache is large enough for a tenth of the
  // kernel's time to outweigh a second launch: the form's time goes with the longest sequence, so the other form is
  // launched behind it and the kernels decide by the sequence lengths which of the two runs (decode_lens_even).
  // tdist_debug_set(TDIST_DEBUG_DECODE_WAVE_HEADS, 0) never takes this form; 2 takes it wherever the heads allow it,
  // alone and whatever the lengths; 4 likewise but only its 4-wave workgroups.
  const int wh_dbg = debug_get(TDIST_DEBUG_DECODE_WAVE_HEADS);
  const int wh_mode = wh_dbg >= 0 ? wh_dbg : 1;
  auto wave_heads = [&](int nw) {
    if (wh_mode == 0 || head_blocks != 1 || c.kv_heads % nw != 0 || (wh_mode == 4 && nw != 4)) return false;
    if (!aligned16(c.out_split)) return false;   // its partial results go out as 16-byte vectors
    // Splits per workgroup: the count that needs the least time in units of (one split on every CU): rounds of
    // workgroups x splits in each; of equal ones the larger, which starts fewer workgroups.
    const int64_t heads_seqs = (int64_t)(c.kv_heads / nw) * c.batch;
    const int cus = device_info().num_cus > 0 ? device_info().num_cus : 256;
    int64_t best_cost = 0;
    int best_w = 1;
    const int max_w = std::min(c.num_splits, decode_max_splits_per_team(dv, c.soft_cap > 0.f || fuse || padded));
    for (int w = 1; w <= max_w; ++w) {
      const int64_t teams = heads_seqs * ((c.num_splits + w - 1) / w);
      const int64_t cost = ((teams + cus - 1) / cus) * w;
      if (w == 1 || cost <= best_cost) best_cost = cost, best_w = w;
    }
    const int spt = debug_get(TDIST_DEBUG_DECODE_SPLITS_PER_TEAM);
    if (spt >= 1) best_w = std::min(spt, max_w);
    prm.splits_per_team = best_w;
    if (wh_mode > 1) return true;
    // the most that the block table lets the call read: below 256 MB (40 us) the form's gain is less than a launch
    const double cap_bytes = (double)c.batch * c.kv_heads * (double)c.table_stride * c.page_size * (dk + dv) * 2.0;
    if (cap_bytes < 256e6) return false;
    // against the time that work spread evenly over the CUs would need: at most a third more
    return best_cost * cus * 3 <= heads_seqs * c.num_splits * 4;
  };
#define TDIST_DEC_WH_(MMA_, D_, KEYS_, NW_, NST_, CAP_, FUSE_, PAD_) \
  launch_decode_cfg<MMA_, D_, 0, KEYS_, NW_, NST_, CAP_, FUSE_, PAD_, true>(prm, head_blocks, st)
#define TDIST_DEC_WH(D_, KEYS_, NW_, NST_) TDIST_DEC_WH_P(D_, KEYS_, NW_, NST_, false)
#define TDIST_DEC_WH_P(D_, KEYS_, NW_, NST_, PAD_)                                                                      \
  if (prm.when_lens == 0 && wave_heads(NW_)) {                                                                       \
    /* chosen for the grid: it runs if the sequence lengths are even, and the other form, launched behind it, if   \
       they are not (forced by the environment: unconditionally, alone) */                                          \
    prm.when_lens = (wh_mode > 1 || c.batch == 1) ? 0 : 1;   /* (one sequence: even by definition) */               \
    int rc_;                                                                                                         \
    if (prm.soft_cap > 0.f) {                                                                                        \
      if (fuse) rc_ = bf ? TDIST_DEC_WH_(MmaBF16, D_, KEYS_, NW_, NST_, true, true, PAD_) : TDIST_DEC_WH_(MmaF16, D_, KEYS_, NW_, NST_, true, true, PAD_);     \
      else rc_ = bf ? TDIST_DEC_WH_(MmaBF16, D_, KEYS_, NW_, NST_, true, false, PAD_) : TDIST_DEC_WH_(MmaF16, D_, KEYS_, NW_, NST_, true, false, PAD_);         \
    } else {                                                                                                         \
      if (fuse) rc_ = bf ? TDIST_DEC_WH_(MmaBF16, D_, KEYS_, NW_, NST_, false, true, PAD_) : TDIST_DEC_WH_(MmaF16, D_, KEYS_, NW_, NST_, false, true, PAD_);   \
      else rc_ = bf ? TDIST_DEC_WH_(MmaBF16, D_, KEYS_, NW_, NST_, false, false, PAD_) : TDIST_DEC_WH_(MmaF16, D_, KEYS_, NW_, NST_, false, false, PAD_);       \
    }                                                                                                                \
    if (rc_ != TDIST_OK || prm.when_lens == 0) return rc_;                                                           \
    prm.when_lens = 2;                                                                                               \
  }
  if (padded) {
    // any other head dimension: the shape of the next power of two, rows filled up with zeros on their way in
    if (dk < 64) TDIST_DEC_PADDED(64, 32, 4, 4)
    if (dk < 128) {
      TDIST_DEC_WH_P(128, 16, 8, 2, true)
      TDIST_DEC_PADDED(128, 16, 3, 3)
    }
    TDIST_DEC_PADDED(256, 16, 2, 3)
  }
  switch (dk) {
    case 64:
      TDIST_DEC_WH(64, 32, 8, 2)
      TDIST_DEC_WH(64, 32, 4, 4)
      TDIST_DEC(64, 0, 32, 4, 4)
    // 16-key blocks, 3 waves, 3 stages = 72 KB of LDS: two workgroups share a CU and two thirds of the ring are
    // in flight
    case 128:
      TDIST_DEC_WH(128, 16, 8, 2)   // (four waves of four stages: no faster than the form below)
      TDIST_DEC(128, 0, 16, 3, 3)
    case 192: TDIST_DEC(128, 64, 16, 2, 3)   // 61 KB: two workgroups per CU
    case 256:
      TDIST_DEC_WH(256, 16, 4, 2)
      TDIST_DEC(256, 0, 16, 2, 3)
    default: TDIST_DEC(512, 64, 16, 2, 2)    // 576 = 512 + 64: 136 KB
  }
#undef TDIST_DEC
#undef TDIST_DEC_WH
#undef TDIST_DEC_WH_P
#undef TDIST_DEC_WH_
#undef TDIST_DEC_PADDED
}

}  // namespace tdist

extern "C" {

int tdist_decode_split_kv(const void* q, const void* k_cache, const void* v_cache, float* out_split, float* lse_split,
                          float sm_scale, float soft_cap, const int32_t* block_table, const int32_t* kv_lens, int batch,
                          int q_heads, int kv_heads, int head_dim, int head_dim_v, int page_size, int num_splits,
                          int64_t q_stride_b, int64_t q_stride_h, int64_t k_stride_page, int64_t k_stride_token,
                          int64_t k_stride_head, int64_t v_stride_page, int64_t v_stride_token, int64_t v_stride_head,
                          int64_t table_stride, int dtype, void* stream) {
  DecodeCall c = {q, k_cache, v_cache, out_split, lse_split, sm_scale, soft_cap, block_table, kv_lens, batch, q_heads,
                  kv_heads, head_dim, head_dim_v, page_size, num_splits, q_stride_b, q_stride_h, k_stride_page,
                  k_stride_token, k_stride_head, v_stride_page, v_stride_token, v_stride_head, table_stride, dtype,
                  nullptr, 0, nullptr, TDIST_F32, 0, 0, nullptr, stream, "tdist_decode_split_kv"};
  return run_decode(c, false);
}

int64_t tdist_decode_fused_counters(int batch, int q_heads, int kv_heads) {
  return decode_fused_counters(batch, q_heads, kv_heads);
}

int tdist_decode_fused(const void* q, const void* k_cache, const void* v_cache, float* out_split, float* lse_split,
                       float sm_scale, float soft_cap, const int32_t* block_table, const int32_t* kv_lens, int batch,
                       int q_heads, int kv_heads, int head_dim, int head_dim_v, int page_size, int num_splits,
                       int64_t q_stride_b, int64_t q_stride_h, int64_t k_stride_page, int64_t k_stride_token,
                       int64_t k_stride_head, int64_t v_stride_page, int64_t v_stride_token, int64_t v_stride_head,
                       int64_t table_stride, int dtype, int32_t* counters, int64_t n_counters, void* out, int out_dtype,
                       int64_t out_stride_b, int64_t out_stride_h, float* lse_out, void* stream) {
  DecodeCall c = {q, k_cache, v_cache, out_split, lse_split, sm_scale, soft_cap, block_table, kv_lens, batch, q_heads,
                  kv_heads, head_dim, head_dim_v, page_size, num_splits, q_stride_b, q_stride_h, k_stride_page,
                  k_stride_token, k_stride_head, v_stride_page, v_stride_token, v_stride_head, table_stride, dtype,
                  counters, n_counters, out, out_dtype, out_stride_b, out_stride_h, lse_out, stream,
                  "tdist_decode_fused"};
  return run_decode(c, true);
}

int tdist_decode_combine(const void* part, int part_dtype, const float* lse, int num_partials, int mode,
                         const int32_t* lens, int batch, int q_heads, int head_dim_v, int64_t part_stride_p,
                         int64_t part_stride_b, int64_t part_stride_h, int64_t lse_stride_p, int64_t lse_stride_b,
                         int64_t lse_stride_h, void* out, int out_dtype, int64_t out_stride_b, int64_t out_stride_h,
                         float* lse_out, void* stream) {
  if (!part || !lse || !out) return fail(TDIST_ERR_INVALID, "tdist_decode_combine: null pointer");
  if (num_partials <= 0 || batch <= 0 || q_heads <= 0 || head_dim_v <= 0)
    return fail(TDIST_ERR_INVALID, "tdist_decode_combine: sizes must be positive");
  if (head_dim_v > 512) return fail(TDIST_ERR_UNSUPPORTED, "tdist_decode_combine: head_dim_v %d > 512", head_dim_v);
  if (mode < 0 || mode > 2 || (mode != 0 && !lens))
    return fail(TDIST_ERR_INVALID, "tdist_decode_combine: mode %d needs lens", mode);
  if ((part_dtype != TDIST_F32 && part_dtype != TDIST_BF16 && part_dtype != TDIST_F16) ||
      (out_dtype != TDIST_F32 && out_dtype != TDIST_BF16 && out_dtype != TDIST_F16))
    return fail(TDIST_ERR_UNSUPPORTED, "tdist_decode_combine: dtype");
  CombineParams prm;
  prm.part = (const unsigned char*)part;
  prm.lse = lse;
  prm.lens = lens;
  prm.out = (unsigned char*)out;
  prm.lse_out = lse_out;
  prm.P = num_partials;
  prm.mode = mode;
  prm.B = batch;
  prm.Hq = q_heads;
  prm.Dv = head_dim_v;
  prm.part_dtype = part_dtype;
  prm.out_dtype = out_dtype;
  prm.p_sp = part_stride_p;
  prm.p_sb = part_stride_b;
  prm.p_sh = part_stride_h;
  prm.l_sp = lse_stride_p;
  prm.l_sb = lse_stride_b;
  prm.l_sh = lse_stride_h;
  prm.o_sb = out_stride_b;
  prm.o_sh = out_stride_h;
  const int64_t blocks = ceil_div((int64_t)batch * q_heads, 4);
  if (blocks > 0x7fffffff) return fail(TDIST_ERR_UNSUPPORTED, "tdist_decode_combine: grid too large");
  auto kern = head_dim_v <= 128 ? decode_combine_kernel<2> : head_dim_v <= 256 ? decode_combine_kernel<4> : decode_combine_kernel<8>;
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, prm);
  return launch_status("tdist_decode_combine");
}

}  // extern "C"
