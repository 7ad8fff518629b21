// (a)/(b1) Persistent MFMA tile GEMM for gfx950: C[M,N] = A[M,K] * B[N,K]^T with
//   - per-chunk gating of A rows on HBM flag words (the AG-GEMM consumer), and/or
//   - an epilogue that scatters row blocks to per-rank buffers (the GEMM-RS producer), or
//   - the grouped form of the MoE tensor-parallel path: gathered A rows, per-block expert weights, scattered C rows.
//
// Restates kernel_consumer_gemm_persistent (kernels/amd/all_gather_gemm.py:140-254), wait_eq_sys
// (kernels/amd/common_ops.py:39-46), kernel_gemm_rs_producer_fuse_scatter
// (kernels/amd/gemm_reduce_scatter.py:125-229) and kernel_consumer_m_parallel_scatter_group_gemm
// (kernels/nvidia/allgather_group_gemm.py:238-314) as one hand-scheduled kernel:
//
//  * workgroup = WM x WN waves, macro tile BM x BN, each wave owns (BM/WM) x (BN/WN) of it as MFMA blocks with
//    fp32 accumulators: on the 256-row tiles 16 x 16 blocks (v_mfma_f32_16x16x32_{bf16,f16}, 16 B of K per lane,
//    and v_mfma_f32_16x16x128_f8f6f4, 32 B per lane), which spend the least power per flop and so hold the highest
//    clock on real data; elsewhere 32 x 32 blocks (v_mfma_f32_32x32x16_{bf16,f16}, v_mfma_f32_32x32x64_f8f6f4);
//  * A and B tiles go HBM/L2 → LDS with asynchronous 16-byte-per-lane LDS-DMA loads into a ring of NST
//    stages, P = NST-1 tiles in flight (NST == 5: a split ring of three A and two B half stages whose refill is
//    spread over the K steps); rows are stored with an XOR swizzle of the 16-byte chunk index
//    so that the ds_read_b128 operand reads are bank-conflict free; the swizzle is applied on the global
//    side (which chunk a lane fetches) because the DMA writes lanes to consecutive LDS addresses;
//  * one s_barrier per K tile, placed before the MFMAs of the tile's last K step, so the first operand
//    reads of the next tile and the DMA refill overlap those MFMAs;
//  * the MFMA is issued as D^T = B_tile * A_tile^T so that a lane ends up with 4 consecutive columns
//    of one row; the epilogue stages the tile through LDS and writes full 16-byte vectors per lane;
//  * persistent grid (one workgroup per CU). The tile schedule is chunk-major in arrival order, and
//    within a round of concurrently running tiles the workgroups of one XCD (workgroup id mod 8) get a
//    compact block of tiles so they share A rows and B rows in that XCD's L2.
#include <stdlib.h>

#include <mutex>
#include <utility>

#include "common.h"

namespace tdist {

struct GemmParams {
  const unsigned char* A;        // gathered workspace
  const unsigned char* A_local;  // own shard or NULL
  const unsigned char* B;
  unsigned char* C;              // plain output (scatter_bufs == NULL)
  void* const* scatter_bufs;     // GEMM-RS: per-owner buffers
  const float* row_scale;
  const float* col_scale;
  const int32_t* flags;
  const int32_t* chunk_order;
  int32_t* status;
  int64_t lda_b, lda_local_b, ldb_b;  // byte strides
  int64_t ldc;                         // elements
  int M, N, K;
  int local_row_begin, local_rows;
  int m_per_chunk;   // rows per schedule chunk (multiple of BM)
  int n_chunks;      // ceil(M / m_per_chunk)
  int gate_rows;     // rows per flag word: m_per_chunk, or (ragged chunks, walked in row order) any positive number:
                     // a tile then waits for every flag its rows touch
  int k_tail_bytes;  // bytes of K in the last K tile when K is not a whole number of them (128 x 128 tile only), else 0
  int chunks_per_rank;
  int wait_value;
  int rank, world_size;
  int order_mode;    // 0 identity, 1 reference AG order, 2 reference RS order (owner = oc+rank+1), 3 explicit
  int spin_limit;
  int m_per_rank;    // GEMM-RS: rows per owner; grouped mode: token rows per rank segment
  int num_xcds;
  // Grouped (MoE) mode, kernel instances with kGrouped: row r of row block m is the token sorted_ids[m*BM + r] / topk
  // (an id >= num_valid is padding), the block multiplies by the weights of expert block_expert[m], waits for the
  // flag of rank segment block_segment[m], and writes its rows to C at row sorted_ids[m*BM + r].
  const int32_t* sorted_ids;
  const int32_t* block_expert;
  const int32_t* block_segment;
  const int32_t* post_pad;       // device scalar: rows of the sorted space in use (a multiple of BM)
  int64_t b_expert_stride_b;     // bytes between the experts' weight matrices
  int num_valid, topk, first_block, a_rows;
  // Split rounds (sk_ctrl != NULL: the caller handed in a workspace). A tile may be cut along K into s = 2, 4 or 8
  // equal pieces (at least kSkMinPiece K tiles each), one per workgroup: workgroups s*t .. s*t+s-1 of the round share
  // tile t. Every piece writes its fp32 accumulators (register order) to slot [workgroup] of sk_partials and raises
  // flag [workgroup] to the round's tag; then each of the s workgroups adds up 1/s of the tile from the s slots, in
  // slot order (so the sum does not depend on timing), and stores that part of C. A slot is written again only after
  // its s readers have acknowledged (ack [workgroup] counts them). Tags are unique per launch and round: the header
  // word kSkCtrlEpoch is read at the start and advanced by the last workgroup to leave, so nothing has to be cleared
  // between launches, a launch that ran into a timeout included. Launches that share a workspace must not overlap.
  // Only a last round that fills at most half of the grid is split (sk_mode 1; 0 = no workspace in use).
  // (Cutting every tile of the schedule into equal shares of K tiles, "stream-K", was measured slower than whole
  // tiles: workgroups that share an operand panel are then at different K positions, and the panel is fetched once
  // per workgroup instead of once per XCD.)
  int32_t* sk_ctrl;
  float* sk_partials;
  int sk_mode;
  int sk_l2_local;   // 1: workgroup i has been seen to run on XCD i mod num_xcds (tdist_init), so pieces that the
                     // schedule puts on one XCD may exchange through that XCD's L2 alone
  // Tiles in arrival order (sched_rounds > 0; gated calls with whole-tile chunks, at most kSchedMaxChunks of them, and
  // 2 .. 64 rounds of tiles). The static schedule parks a workgroup on the flag of the chunk its position names, also
  // while rows of other chunks have long arrived (the reference orders its tiles by expected arrival for the same
  // reason, kernels/amd/all_gather_gemm.py:193-206). Here a workgroup keeps the tiles the static schedule gives it
  // (position w + r G of the static order in round r: the workgroups of an XCD still work on neighbouring tiles and
  // share operand panels in that XCD's L2) but takes them in the order in which their chunks arrive: when it has
  // finished a tile it takes the earliest round whose chunk has arrived; only with none of its tiles ready does it
  // wait, polling the flags, bounded as the static order's flag wait is. The look at the flags (wave 0, one lane per
  // chunk) is issued when the current tile's epilogue begins and used when it ends, so in a call whose rows are all
  // there the schedule costs no waiting at all (the static order pays a trip to memory for the flag of every tile).
  // Every tile is computed whole and by the workgroup the static schedule names, so neither the result nor the
  // balance of the work depends on the arrival order; nothing is shared between workgroups and no workspace is used.
  // (An earlier form let the workgroups of an XCD draw tiles from a common list with an atomic add per tile: with 32
  // workgroups drawing at the same moment the draws queued up behind each other for 2-5 us per tile.)
  int sched_rounds;
  // (host-side constants of that schedule, so that the kernel divides by multiplying: ceil(2^32 / d) for d = tiles
  // per chunk and d = world_size; the host takes the schedule only while positions x d stay below 2^31, where the
  // product's high word is the quotient)
  uint32_t sched_tpc_magic, sched_ws_magic;
  // Chunks of few row tiles (1, 2 or 4) are scheduled group_s at a time (a power of two; 1: chunk by chunk): the
  // positions of a group run down the rows of all its chunks before they move on to the next column of tiles, so that
  // the block of tiles an XCD's workgroups work on is 8 rows x 4 columns (or 4 x 8) instead of 2 x 16 or 1 x 32, and
  // fetches 12 operand panels instead of 18 or 33 (16384 x 7168 x 8192 e4m3 in chunks of 512 rows: 615 -> 597 us).
  // Every tile is still gated by the flag of its own chunk. The sched_tpc_magic is then that of a group's tiles.
  int group_s, group_rows_shift, cm_shift;
};

// Workspace header, in int32 words
constexpr int kSkCtrlEpoch = 0;          // tag base of the next launch
constexpr int kSkCtrlDone = 1;           // workgroups of the running launch that have left
constexpr int kSkMaxWorkgroups = 1024;
constexpr int kSkFlagsOff = 1024;        // [kSkMaxWorkgroups] tag of the partial in the slot
constexpr int kSkAcksOff = 2048;         // [kSkMaxWorkgroups] readers that are done with the slot, ever
constexpr int kSkHeaderWords = 3072;
constexpr int64_t kSkHeaderBytes = (int64_t)kSkHeaderWords * 4;
constexpr int kSchedMaxChunks = 64;      // one lane of the deciding wave per chunk
constexpr int kSchedMaxRounds = 64;      // and per round of this workgroup's tiles
constexpr int kSkTagStride = 16;         // tags per launch (rounds that may be split)
// a flag word is the tag (low 27 bits) with the XCD the piece ran on above it
constexpr int kSkTagBits = 27, kSkTagMask = (1 << kSkTagBits) - 1, kSkTagWrap = kSkTagMask - 0x10000;
static_assert(kSkHeaderBytes % 256 == 0, "the partial slots start 256-byte aligned");

// Operand fragment of one lane: K bytes [0, kLaneBytes) of one row; chunk0 / chunk1 are LDS addresses of its
// 16-byte pieces.
struct ElemBF16 {
  static constexpr int kBytes = 2;
  static constexpr int kLaneBytes = 16;  // K bytes one lane feeds to one MFMA
  static constexpr int kRows = 32;       // rows (and columns) of one MFMA block
  typedef float16v acc_t;                // its accumulators in one lane
  typedef int4v frag;
  __device__ static __forceinline__ frag load(const TDIST_AS3 unsigned char* c0, const TDIST_AS3 unsigned char*) {
    return *(const TDIST_AS3 int4v*)c0;
  }
  __device__ static __forceinline__ float16v mma(frag a, frag b, float16v c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8v, a), __builtin_bit_cast(bf16x8v, b), c, 0,
                                                   0, 0);
  }
  __device__ static __forceinline__ uint32_t pack(float a, float b) { return pack_bf16x2(a, b); }
};
struct ElemF16 {
  static constexpr int kBytes = 2;
  static constexpr int kLaneBytes = 16;
  static constexpr int kRows = 32;
  typedef float16v acc_t;
  typedef int4v frag;
  __device__ static __forceinline__ frag load(const TDIST_AS3 unsigned char* c0, const TDIST_AS3 unsigned char*) {
    return *(const TDIST_AS3 int4v*)c0;
  }
  __device__ static __forceinline__ float16v mma(frag a, frag b, float16v c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8v, a), __builtin_bit_cast(f16x8v, b), c, 0, 0,
                                                  0);
  }
  __device__ static __forceinline__ uint32_t pack(float a, float b) { return pack_f16x2(a, b); }
};
// The same element types on the 16x16x32 MFMA: four lane groups along K instead of two, sixteen rows per block.
// Per flop it draws less power than the 32x32x16 form, which is what the clock of a long GEMM on real data
// is limited by.
// Its four-register result is not tied to its accumulator input in the compiler's instruction model, and with all 256
// accumulation registers in use the register allocator, left to place the accumulators itself, has shuffled them
// between registers and spilled them inside the K loop, after edits far from the loop. The kernels on these blocks
// therefore keep their accumulators in FIXED accumulation registers: block (j, i) of the wave tile lives in
// a[4*(j*kTM+i) .. +3], the instruction is written as assembly that names those registers, and the compiler never
// allocates an accumulation register in these kernels (see acc_reserve). (The compiler then knows none of the
// instruction's hazards: the K loop never reads an accumulator, and the code after it waits out the last MFMA
// before it does.)
struct ElemBF16N : ElemBF16 {
  static constexpr int kRows = 16;
  typedef float4v acc_t;
  template <int kBase>
  __device__ static __forceinline__ void mma_at(frag a, frag b) {
    asm volatile("v_mfma_f32_16x16x32_bf16 a[%2:%3], %0, %1, a[%2:%3]" ::"v"(a), "v"(b), "n"(kBase), "n"(kBase + 3));
  }
};
struct ElemF16N : ElemF16 {
  static constexpr int kRows = 16;
  typedef float4v acc_t;
  template <int kBase>
  __device__ static __forceinline__ void mma_at(frag a, frag b) {
    asm volatile("v_mfma_f32_16x16x32_f16 a[%2:%3], %0, %1, a[%2:%3]" ::"v"(a), "v"(b), "n"(kBase), "n"(kBase + 3));
  }
};
struct ElemFP8 {
  static constexpr int kBytes = 1;
  static constexpr int kLaneBytes = 32;
  static constexpr int kRows = 32;
  typedef float16v acc_t;
  typedef int8v frag;
  __device__ static __forceinline__ frag load(const TDIST_AS3 unsigned char* c0, const TDIST_AS3 unsigned char* c1) {
    const int4v lo = *(const TDIST_AS3 int4v*)c0;
    const int4v hi = *(const TDIST_AS3 int4v*)c1;
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  }
  __device__ static __forceinline__ float16v mma(frag a, frag b, float16v c) {
    // cbsz = 0 / blgp = 0 select e4m3 for both operands; scales are 2^0
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
  }
  __device__ static __forceinline__ uint32_t pack(float a, float b) { return pack_bf16x2(a, b); }  // bf16 output
};

// KB = bytes of K per tile row. Chunk c (16 B) of row r is stored at position c ^ swz(r).
// A ds_read_b128 is served 16 lanes at a time (16 x 16 B = 256 B = one pass over the 64 banks), and the 16
// lanes of a pass read the same logical chunk of 16 consecutive rows. Those rows cover 256 B / KB positions
// "for free" through their row offset; the XOR term has to spread the rest, i.e. change every (256 / KB) rows.
// e4m3 on the 16x16x128 MFMA: a lane feeds the same 32 bytes of K, four lane groups cover a whole 128-byte tile row
struct ElemFP8N : ElemFP8 {
  static constexpr int kRows = 16;
  typedef float4v acc_t;
  template <int kBase>
  __device__ static __forceinline__ void mma_at(frag a, frag b) {
    asm volatile("v_mfma_f32_16x16x128_f8f6f4 a[%2:%3], %0, %1, a[%2:%3]" ::"v"(a), "v"(b), "n"(kBase), "n"(kBase + 3));
  }
};

template <int KB>
__host__ __device__ constexpr int swz(int r) {
  return KB >= 128 ? ((r >> 1) & 7) : ((r >> 2) & 3);
}

template <typename E, int BM, int BN, int KB, int WM, int WN, int NST>
struct GemmCfg {
  static constexpr int kWaves = WM * WN;
  static constexpr int kThreads = kWaves * 64;
  static constexpr int kChunksPerRow = KB / 16;
  static constexpr int kRowsPerInstr = 64 / kChunksPerRow;
  static constexpr int kAInstr = BM / kRowsPerInstr / kWaves;  // DMA instructions per wave per tile
  static constexpr int kBInstr = BN / kRowsPerInstr / kWaves;
  static constexpr int kLoadsPerTile = kAInstr + kBInstr;
  static constexpr int kABytes = BM * KB;
  static constexpr int kBBytes = BN * KB;
  static constexpr int kStageBytes = kABytes + kBBytes;
  static constexpr int kP = NST - 1;
  static constexpr int kLaneGroups = 64 / E::kRows;  // lane groups along K within one MFMA
  static constexpr int kAccLen = E::kRows * E::kRows / 64;  // accumulators per lane and MFMA block
  static constexpr int kKSteps = KB / (kLaneGroups * E::kLaneBytes);
  static constexpr int kFragVecs = E::kLaneBytes / 16;  // 16-byte pieces per operand fragment (1 or 2)
  static constexpr int kWaveM = BM / WM, kWaveN = BN / WN;
  static constexpr int kTM = kWaveM / E::kRows, kTN = kWaveN / E::kRows;
  // NST == 5 selects the split ring: three stages of A rows and two of B rows (five half stages, exactly the
  // 160 KB of LDS at 256x256x128). A freed B stage is refilled at once; the A refill then has a whole K tile of
  // time, so the DMA issue can be spread evenly over the K steps instead of bunching up behind the barrier.
  static constexpr bool kSplit = NST == 5;
  static constexpr int kAStages = kSplit ? 3 : NST, kBStages = kSplit ? 2 : NST;
  static constexpr int kLdsBytes = kSplit ? kAStages * kABytes + kBStages * kBBytes : NST * kStageBytes;
  // split ring: byte offset of A stage s / B stage s (taken modulo the ring's length)
  static constexpr int a_stage_off(int s) { return (s % kAStages) * kABytes; }
  static constexpr int b_stage_off(int s) { return kAStages * kABytes + (s % kBStages) * kBBytes; }
  // split ring: DMA instructions issued per K step (list of one K tile: the B rows, then the A rows)
  static constexpr int kDmaPerStep = (kLoadsPerTile + kKSteps - 1) / kKSteps;
  // epilogue staging: per wave kWaveM rows of kWaveN 16-bit outputs; 16-byte chunk c of row r sits at
  // position c ^ (r & kEpiSwz) so that the 32 rows one store instruction touches spread over the banks
  // (a row of 16-byte pieces whose number is no power of two, the 96 columns of the 128 x 192 tile's waves, is
  // staged at the pitch of the next power of two, so that the XOR stays inside the row)
  static constexpr int kRowPieces = kWaveN * 2 / 16;
  static constexpr int kEpiChunks = kRowPieces <= 4 ? 4 : kRowPieces <= 8 ? 8 : kRowPieces <= 16 ? 16 : 32;
  static constexpr int kEpiPitch = kEpiChunks * 16;
  static constexpr int kEpiBytes = kWaveM * kEpiPitch;
  static constexpr int kEpiSwz = (kEpiChunks < 16 ? kEpiChunks : 16) - 1;
  // MFMAs of a tile's last K step issued before the barrier
  static constexpr int kLeadMfma = (kTM * kTN >= 8) ? 2 : 1;
  // n-th operand fragment (A fragments are 0..kTM-1, B fragments kTM..) in the order in which the MFMA sequence
  // (idx -> B fragment idx / kTM, A fragment idx % kTM) first needs them
  static constexpr int frag_order(int n) {
    int c = 0;
    for (int u = 0; u < kTM * kTN; ++u) {
      if (u % kTM == 0) {
        if (c == n) return kTM + u / kTM;
        ++c;
      }
      if (u < kTM) {
        if (c == n) return u;
        ++c;
      }
    }
    return -1;
  }
  static_assert(KB == 64 || KB == 128, "tile rows of 64 or 128 bytes");
  static_assert(BM % (kRowsPerInstr * kWaves) == 0 && BN % (kRowsPerInstr * kWaves) == 0, "tile/wave split");
  static_assert(kSplit || (kP >= 1 && kP <= 3 && kP * kLoadsPerTile < 64), "vmcnt budget");
  static_assert(!kSplit || (kTM + kTN <= kTM * kTN - kLeadMfma && kLoadsPerTile % kKSteps == 0),
                "split ring: one fragment read per MFMA slot, whole DMA groups per K step");
  static_assert(kEpiBytes * kWaves <= kLdsBytes, "epilogue staging must fit in the stage ring");
  static_assert(kWaveM % 32 == 0 && kWaveN % 32 == 0, "wave tile");
};

// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>): a loop whose index is a constant in every trip
// without leaning on the unroller (which gives up on bodies as long as a K step's schedule)
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// Waits until at most `kOutstanding` of this wave's DMA loads are in flight and for its LDS reads, then joins
// the workgroup barrier.
template <int kOutstanding>
__device__ __forceinline__ void wait_tiles_and_barrier() {
  static_assert(kOutstanding >= 0 && kOutstanding < 64, "vmcnt is a 6-bit counter");
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(kOutstanding) : "memory");
}

// Split rounds: most pieces per tile, fewest K tiles per piece
constexpr int kSkMaxSplit = 8, kSkMinPiece = 4;
// pieces per tile when `tiles` tiles are all that `workgroups` workgroups have to do: the largest power of two that
// the workgroups and the K tiles allow (1 = whole tiles)
__host__ __device__ inline int sk_split_for(int workgroups, int tiles, int k_tiles) {
  int s = 1;
  while (2 * s <= kSkMaxSplit && (int64_t)2 * s * tiles <= workgroups && k_tiles / (2 * s) >= kSkMinPiece) s *= 2;
  return s;
}

// Instruction classes for __builtin_amdgcn_sched_group_barrier
constexpr int kSchedMfma = 0x008, kSchedDsRead = 0x100;

// Kernels with fixed accumulators: declares a[0 .. kN) in use, so that the kernel is given them and the compiler
// neither parks spilled vector registers in them nor counts them as free; nothing else in such a kernel is ever of
// the accumulation register class. Then clears them.
#define TDIST_A10(n) "a" #n "0", "a" #n "1", "a" #n "2", "a" #n "3", "a" #n "4", "a" #n "5", "a" #n "6", "a" #n "7", "a" #n "8", "a" #n "9"
#define TDIST_A_0_99 "a0", "a1", "a2", "a3", "a4", "a5", "a6", "a7", "a8", "a9", TDIST_A10(1), TDIST_A10(2), TDIST_A10(3), TDIST_A10(4), \
    TDIST_A10(5), TDIST_A10(6), TDIST_A10(7), TDIST_A10(8), TDIST_A10(9)
#define TDIST_A_100_127 TDIST_A10(10), TDIST_A10(11), "a120", "a121", "a122", "a123", "a124", "a125", "a126", "a127"
#define TDIST_A_128_255 "a128", "a129", TDIST_A10(13), TDIST_A10(14), TDIST_A10(15), TDIST_A10(16), TDIST_A10(17), TDIST_A10(18), \
    TDIST_A10(19), TDIST_A10(20), TDIST_A10(21), TDIST_A10(22), TDIST_A10(23), TDIST_A10(24), "a250", "a251", "a252", "a253", "a254", "a255"
template <int kN>
__device__ __forceinline__ void acc_reserve() {
  static_assert(kN == 96 || kN == 128 || kN == 256, "accumulators of a 64 x 96, a 128 x 64 or a 128 x 128 wave tile");
  if constexpr (kN == 256) asm volatile("" ::: TDIST_A_0_99, TDIST_A_100_127, TDIST_A_128_255);
  else if constexpr (kN == 128) asm volatile("" ::: TDIST_A_0_99, TDIST_A_100_127);
  else asm volatile("" ::: TDIST_A_0_99);   // (a96 .. a99 go unused)
}
template <int kN>
__device__ __forceinline__ void acc_clear() {
  static_for<kN>([&](auto r_c) { asm volatile("v_accvgpr_write_b32 a[%0], 0" ::"n"(decltype(r_c)::value)); });
}

// what the DMA lanes of a ragged last K tile read for the bytes of K that do not exist
static __device__ __align__(16) const unsigned char kZeroChunk[16] = {0};

// schedule position → chunk id
__device__ __forceinline__ int chunk_of(const GemmParams& p, int oc) {
  switch (p.order_mode) {
    case 1: {  // own rank's chunks first, then rank+1, ... one chunk of every rank per sweep
      const int sweep = oc / p.world_size;
      const int r = (oc % p.world_size + p.rank) % p.world_size;
      return r * p.chunks_per_rank + sweep;
    }
    case 2:  // row blocks of rank+1 first
      return (oc + p.rank + 1) % p.world_size;
    case 3:
      return p.chunk_order[oc];
    case 4:  // grouped: row blocks starting at the own rank segment's first one
      return (oc + p.first_block) % p.n_chunks;
    default:
      return oc;
  }
}

// kPlain: an instance for calls without flags and without a local shard (the GEMM-RS producer, plain GEMMs): no gating
// code at all, and the next tile's first loads go out before the current tile's epilogue (see kEarly).
template <typename E, int BM, int BN, int KB, int WM, int WN, int NST, bool kScales, bool kGrouped = false, bool kPlain = false>
__global__ __launch_bounds__(WM * WN * 64, 1) void gemm_kernel(const GemmParams p) {
  typedef GemmCfg<E, BM, BN, KB, WM, WN, NST> C;
  typedef TDIST_AS3 unsigned char* lds_u8;
  constexpr bool kFixedAcc = E::kRows == 16;
  constexpr int kAccRegs = C::kTM * C::kTN * C::kAccLen;
  if constexpr (kFixedAcc) acc_reserve<kAccRegs>();
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem_generic[];
  lds_u8 const smem = (lds_u8)smem_generic;
  // gate result (1 = tile may proceed, 0 = wait expired) lives in the first word of the ring, which is idle
  // between tiles
  TDIST_AS3 int* const s_gate = (TDIST_AS3 int*)smem;

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int wm = wave / WN, wn = wave % WN;
  const int lrow = lane % E::kRows, lgrp = lane / E::kRows;

  // Per-lane parts of the operand fragment reads (16-row MFMA blocks: 16-byte piece lgrp or lgrp + 4 of row lrow of the
  // wave's rows; the swizzle term does not depend on the 16-row block): A rows, A rows + 64 KB (the offset field of
  // an LDS read ends at 64 KB), B rows with the start of the B stages folded in. Opaque to the compiler, which would
  // otherwise re-associate them with the constants of the K loop.
  uint32_t frag_lane_a[2] = {0, 0}, frag_lane_a_hi[2] = {0, 0}, frag_lane_b[2] = {0, 0};
  if constexpr (E::kRows == 16) {
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const int ra = wm * C::kWaveM + lrow, rb = wn * C::kWaveN + lrow;
      frag_lane_a[q] = ra * KB + (((lgrp + 4 * q) ^ swz<KB>(ra)) << 4);
      frag_lane_a_hi[q] = frag_lane_a[q] + 65536;
      frag_lane_b[q] = C::kAStages * C::kABytes + rb * KB + (((lgrp + 4 * q) ^ swz<KB>(rb)) << 4);
      asm volatile("" : "+v"(frag_lane_a[q]), "+v"(frag_lane_a_hi[q]), "+v"(frag_lane_b[q]));
    }
  }
  const int num_pid_m = (p.M + BM - 1) / BM;
  const int num_pid_n = (p.N + BN - 1) / BN;
  const int cm = p.m_per_chunk / BM;                 // row tiles per chunk
  const int tiles_per_chunk = cm * num_pid_n;
  // grouped: only the row blocks in use are scheduled (their count is written by an earlier kernel of the stream)
  int n_chunks = p.n_chunks;
  if constexpr (kGrouped) n_chunks = min(n_chunks, __builtin_nontemporal_load(p.post_pad) / BM);
  const int total_sched = n_chunks * tiles_per_chunk;
  const int G = gridDim.x;
  const int KT = (p.K * E::kBytes + KB - 1) / KB;   // (a ragged last K tile only on the plain ring: see k_tail_bytes)

  // DMA lane roles: row within an instruction's row group, and the LDS chunk position it fills
  const int dma_row = lane / C::kChunksPerRow;
  const int dma_pos = lane % C::kChunksPerRow;

  // XCD-aware position within a round: workgroups of XCD x take a contiguous range
  int wg_pos = blockIdx.x;
  if (p.num_xcds > 1 && G % p.num_xcds == 0) wg_pos = (wg_pos % p.num_xcds) * (G / p.num_xcds) + wg_pos / p.num_xcds;
  // ---- workspace state of this launch ---------------------------------------------------------------------
  int32_t* const sk_flags = p.sk_ctrl + kSkFlagsOff;
  int32_t* const sk_acks = p.sk_ctrl + kSkAcksOff;
  // the workgroups of one XCD hold a contiguous range of positions (see wg_pos): pieces of a tile share an XCD when
  // the pieces per tile (2, 4 or 8) divide the workgroups per XCD
  // (only where that dispatch order has been checked on this device; each piece also publishes the XCD it really ran
  // on and the readers compare, so a launch that lands differently reports it instead of summing stale slots)
  const bool sk_xcd_local = p.sk_l2_local != 0 && p.num_xcds > 1 && G % p.num_xcds == 0 && (G / p.num_xcds) % kSkMaxSplit == 0;
  const int my_xcc = p.sk_mode != 0 ? __builtin_amdgcn_readfirstlane(xcc_id()) : 0;
  int tag_base = 0;   // tags of this launch are tag_base + 1 + round
  int sk_need = 0;    // value of this workgroup's ack word once every reader of its last partial is done
  if (p.sk_mode != 0) {
    if (threadIdx.x == 0) {
      s_gate[0] = __hip_atomic_load(p.sk_ctrl + kSkCtrlEpoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      s_gate[1] = __hip_atomic_load(sk_acks + wg_pos, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    tag_base = __builtin_amdgcn_readfirstlane(s_gate[0]);
    sk_need = __builtin_amdgcn_readfirstlane(s_gate[1]);
    __syncthreads();
  }
  // static schedule: the last round is cut into s pieces per tile (1 = not split)
  const int sk_tail_tiles = total_sched % G;
  int sk_split = 1;
  if (p.sk_mode == 1 && sk_tail_tiles > 0) sk_split = sk_split_for(G, sk_tail_tiles, KT);

  // ---- tiles in arrival order (see GemmParams::sched_rounds); everything here is wave 0's ------------------------------
  const bool arrival = !kGrouped && !kPlain && p.sched_rounds > 0;
  bool arr_decided = false;
  // The schedule's state lives in ONE vector register, a word per lane (wave 0's copy), read and written with
  // v_readlane / v_writelane where a tile is chosen, so that nothing of it is held in scalar registers across the K
  // loop: the rounds of this workgroup that are done with (taken or given up; 64 bits in two lanes), the looks a wait
  // may take (1 once any wait of the launch has expired) and the chunks whose rows this workgroup has acquired.
  enum { kArrDoneLo = 0, kArrDoneHi = 1, kArrLimit = 2, kArrSeenLo = 3, kArrSeenHi = 4 };
  int arr_v = 0;
  asm volatile("" : "+v"(arr_v));
  auto arr_get = [&](int i) { return __builtin_amdgcn_readlane(arr_v, i); };
  // (the lane is an immediate: a second scalar operand would be one too many for the instruction)
#define TDIST_ARR_SET(LANE, VAL) \
  asm volatile("v_writelane_b32 %0, %1, %2" : "+v"(arr_v) : "s"(__builtin_amdgcn_readfirstlane(VAL)), "n"(LANE))
  if (arrival) TDIST_ARR_SET(kArrLimit, p.spin_limit);
  // chunk of the tile at position sidx of the static order (chunk_of with its divisions as multiplications)
  // position sidx of the static order -> the chunk's place in the chunk order and the tile within the chunk (column *
  // cm + row), with the divisions as multiplications and shifts (see GemmParams::group_s)
  auto arr_locate = [&](int sidx, int& oc, int& within) {
    const int og = (int)__umulhi((uint32_t)sidx, p.sched_tpc_magic);
    const int win = sidx - og * (p.group_s * tiles_per_chunk);
    if (p.group_s > 1) {
      const int pn = win >> p.group_rows_shift, j = win & ((1 << p.group_rows_shift) - 1);
      oc = og * p.group_s + (j >> p.cm_shift);
      within = pn * cm + (j & (cm - 1));
    } else {
      oc = og;
      within = win;
    }
  };
  auto arr_chunk_at = [&](int sidx) {
    int oc, within_unused;
    arr_locate(sidx, oc, within_unused);
    if (p.order_mode == 1) {
      const int sweep = (int)__umulhi((uint32_t)oc, p.sched_ws_magic);
      int r = oc - sweep * p.world_size + p.rank;
      r -= r >= p.world_size ? p.world_size : 0;
      return r * p.chunks_per_rank + sweep;
    }
    return chunk_of(p, oc);
  };
  auto arr_is_local = [&](int ch) {
    const int cm0 = ch * p.m_per_chunk;
    return p.A_local != nullptr && cm0 >= p.local_row_begin && cm0 < p.local_row_begin + p.local_rows;
  };
  // One look: lane c loads chunk c's flag (system scope); issued at once, waited for at its first use.
  auto arr_look = [&]() {
    int l = lane;
    asm volatile("" : "+v"(l));   // (nothing of this is computed ahead and held across the K loop)
    return __hip_atomic_load(p.flags + min(l, n_chunks - 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  };
  // The next tile of this workgroup given a look (lane c: chunk c's flag): its position in the static order with its
  // chunk in the low six bits, or -1 when there is nothing left to do. Lane r stands for round r of this workgroup.
  auto arr_next = [&](int flag) -> int {
    int l = lane;
    asm volatile("" : "+v"(l));
    uint64_t done = ((uint64_t)(uint32_t)arr_get(kArrDoneHi) << 32) | (uint32_t)arr_get(kArrDoneLo);
    uint64_t seen = ((uint64_t)(uint32_t)arr_get(kArrSeenHi) << 32) | (uint32_t)arr_get(kArrSeenLo);
    int arr_limit = arr_get(kArrLimit);
    // this lane's round: its position, whether there is a tile there, its chunk
    const int sidx = l * G + wg_pos;
    const bool exists = l < p.sched_rounds && sidx < total_sched;
    const int ch = exists ? arr_chunk_at(sidx) : 0;
    const bool local = arr_is_local(ch);
    int looks = 0, next = -1;
    for (;;) {
      const uint64_t open = __ballot(exists) & ~done;          // rounds still to be done
      if (open == 0) break;                                      // nothing left (next = -1)
      // the chunk of this lane's round has arrived (its flag is lane ch's)
      const int flag_ch = __shfl(flag, ch);   // (by every lane: a lane that sits out answers nobody)
      const bool arrived = local || flag_ch == p.wait_value;
      const uint64_t ready = __ballot(exists && arrived) & open;
      if (ready != 0) {
        const int r = __builtin_amdgcn_readfirstlane(__builtin_ctzll(ready));   // the earliest round that can be done
        done |= 1ull << r;
        const int c_next = __builtin_amdgcn_readlane(ch, r);
        next = ((r * G + wg_pos) << 6) | c_next;
        // Acquire, once per chunk and workgroup at most: an invalidate drops every line the XCD's L2 holds for the
        // other workgroups too, operand panels included, so it is issued only for a chunk whose rows this workgroup
        // has not acquired yet, and it then covers every chunk whose flag this look has seen (with all rows there at
        // the start: once per launch, where the static order invalidates once per tile). The wait behind it also
        // waits for the last tile's stores, which is why it must be rare.
        if (!__builtin_amdgcn_readlane((int)local, r) && ((seen >> c_next) & 1) == 0) {
          seen |= __ballot(l < n_chunks && flag == p.wait_value);
          asm volatile("buffer_inv sc0 sc1\n\ts_waitcnt vmcnt(0)" ::: "memory");
        }
        break;
      }
      // every tile left waits for a flag: look again, as the static order's flag wait does (bounded; once any wait of
      // the launch has expired, one look is all the others get)
      if (looks == 0 && p.status != nullptr && __hip_atomic_load(p.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) arr_limit = 1;
      if (++looks >= arr_limit) {
        // expired: the earliest round is given up (skipped, as a tile whose flag wait expires is) and reported
        const int r = __builtin_amdgcn_readfirstlane(__builtin_ctzll(open));
        done |= 1ull << r;
        if (l == 0 && p.status != nullptr) {
          if (atomicCAS(p.status, 0, TDIST_ERR_TIMEOUT) == 0) p.status[1] = __builtin_amdgcn_readlane(ch, r);
        }
        arr_limit = 1;
        looks = 0;
        continue;
      }
      __builtin_amdgcn_s_sleep(4);
      flag = arr_look();
    }
    TDIST_ARR_SET(kArrDoneLo, (int)(uint32_t)done);
    TDIST_ARR_SET(kArrDoneHi, (int)(uint32_t)(done >> 32));
    TDIST_ARR_SET(kArrLimit, arr_limit);
    TDIST_ARR_SET(kArrSeenLo, (int)(uint32_t)seen);
    TDIST_ARR_SET(kArrSeenHi, (int)(uint32_t)(seen >> 32));
    return next;
  };

  // ---- the next tile's first loads issued before this tile's epilogue ------------------------------------------------
  // Plain tiles (whole, ungated, unsplit) followed by another plain tile of the same workgroup, on the 256 x 256 split
  // ring: A(0), B(0) and B(1) of the next tile go out before this tile's epilogue, which then stages through the A
  // stages 1 and 2 only (two 32-row blocks per wave, used in turn). The next tile's prologue has A(1) left to issue
  // and waits for A(0) and B(0) alone: the epilogue's stores, issued behind those loads, are still on their way then
  // and have the whole first K tile to be acknowledged (loads and stores retire in order through one counter, so a
  // prologue that issues its loads behind the stores waits for every store of the tile before it).
  constexpr bool kEarly = kPlain && C::kSplit && !kGrouped && kFixedAcc && C::kWaves <= 4 && C::kRowPieces == C::kEpiChunks &&
                          2 * C::kABytes >= C::kWaves * 64 * C::kEpiPitch && C::kAInstr == C::kBInstr;
  constexpr int kEpiStores = (C::kWaveM / 32) * 32 * C::kEpiChunks / 64;   // 16-byte stores per wave and tile
  static_assert(!kEarly || C::kBInstr + kEpiStores + C::kAInstr < 64, "vmcnt is a 6-bit counter");
  bool prefetched = false;   // this tile's A(0), B(0), B(1) were issued by the tile before
  // tile of C behind schedule index sidx (ungated calls)
  auto locate = [&](int sidx, int& tm0, int& tn0) -> bool {
    const int toc = sidx / tiles_per_chunk, twithin = sidx - toc * tiles_per_chunk;
    const int tpid_m = chunk_of(p, toc) * cm + twithin % cm;
    tm0 = tpid_m * BM;
    tn0 = (twithin / cm) * BN;
    return tpid_m < num_pid_m;
  };

  int sbase = 0;
  for (;;) {
    // ---- next piece of work: K tiles [ka, kb) of tile `within` of chunk position oc, as piece sk_j of sk_s -----
    int oc, within, ka = 0, kb = KT, sk_s = 1, sk_j = 0, sk_tag = 0;
    int arr_chunk = -1;   // arrival order: the chunk of the tile taken (its flag has been seen and acquired)
    if (arrival) {
      if (!arr_decided && wave == 0) {
        // not decided while the last tile was stored: the first tile, or a position that turned out to hold no tile
        const int next = arr_next(arr_look());
        if (lane == 0) s_gate[0] = next;
      }
      arr_decided = false;
      // (barriers that wait for LDS only: the last tile's stores stay in flight)
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      const int next = __builtin_amdgcn_readfirstlane(s_gate[0]);
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      if (next < 0) break;
      arr_locate(next >> 6, oc, within);
      arr_chunk = next & 63;
    } else {
      int sidx;
      if (sbase >= total_sched) break;
      const int round_base = sbase;
      sbase += G;
      if (sk_split > 1 && round_base + G > total_sched) {
        // the last round, split: workgroup s*t + j takes piece j of the round's tile t
        const int t = wg_pos / sk_split, j = wg_pos - t * sk_split;
        if (t >= sk_tail_tiles) break;
        sidx = __builtin_amdgcn_readfirstlane(round_base + t);
        sk_s = sk_split;
        sk_j = __builtin_amdgcn_readfirstlane(j);
        sk_tag = tag_base + 1;
        ka = __builtin_amdgcn_readfirstlane(KT * j / sk_split);  // (KT < 2^20 and j < 8: 32-bit scalar arithmetic)
        kb = __builtin_amdgcn_readfirstlane(KT * (j + 1) / sk_split);
      } else {
        sidx = round_base + wg_pos;
        if (sidx >= total_sched) continue;
      }
      if (!kGrouped && p.group_s > 1) {
        const int rows_g = p.group_s * cm, tpg = rows_g * num_pid_n;
        const int og = sidx / tpg, win = sidx - og * tpg;
        const int pn = win >> p.group_rows_shift, j = win & (rows_g - 1);
        oc = og * p.group_s + (j >> p.cm_shift);
        within = pn * cm + (j & (cm - 1));
      } else {
        oc = sidx / tiles_per_chunk;
        within = sidx - oc * tiles_per_chunk;
      }
    }
    const int KTp = kb - ka;
    const int chunk = kGrouped ? (oc + p.first_block) % n_chunks : arr_chunk >= 0 ? arr_chunk : chunk_of(p, oc);
    const int pid_m = chunk * cm + within % cm;
    const int pid_n = within / cm;
    if (pid_m >= num_pid_m) continue;
    const int m0 = pid_m * BM, n0 = pid_n * BN;
    int segment = 0;  // grouped: rank segment of this row block
    if constexpr (kGrouped) {
      if (m0 >= __builtin_nontemporal_load(p.post_pad)) continue;  // (written by an earlier kernel of the stream)
      segment = p.block_segment[pid_m];
    }

    // ---- gate ---------------------------------------------------------------------------------
    const bool is_local = kPlain ? false : kGrouped ? (p.A_local != nullptr && segment == p.rank)
                                   : (p.A_local != nullptr && m0 >= p.local_row_begin && m0 < p.local_row_begin + p.local_rows);
    if (!kPlain && p.flags != nullptr && !is_local && arr_chunk < 0) {
      if (threadIdx.x == 0) {
        // the flags of the tile's rows: one (the tile lies inside a chunk), or, with ragged chunks, every flag from
        // the first row's to the last row's (the reference's NVIDIA-side kernel waits for a range of rank segments
        // in the same way, kernels/nvidia/allgather_gemm.py:222-224)
        int f_lo = kGrouped ? segment : chunk, f_hi = f_lo;
        if (!kGrouped && p.gate_rows != p.m_per_chunk) {
          f_lo = m0 / p.gate_rows;
          f_hi = min(m0 + BM - 1, p.M - 1) / p.gate_rows;
        }
        int ok = 1;
        int limit = p.spin_limit;
        if (p.status != nullptr && __hip_atomic_load(p.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) limit = 1;
        // poll with plain coherent loads and acquire once, after the flags have been seen: an acquiring load
        // invalidates this CU's and this XCD's caches every time it is executed
        for (int f = f_lo; f <= f_hi && ok; ++f) {
          ok = 0;
          for (int it = 0; it < limit; ++it) {
            if (__hip_atomic_load(p.flags + f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) == p.wait_value) {
              ok = 1;
              break;
            }
            __builtin_amdgcn_s_sleep(4);
          }
          if (!ok && p.status != nullptr) {
            if (atomicCAS(p.status, 0, TDIST_ERR_TIMEOUT) == 0) p.status[1] = f;
          }
        }
        if (ok) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "");
        *s_gate = ok;
      }
      __syncthreads();
      const int ok = *s_gate;
      __syncthreads();
      if (!ok) continue;
    }

    const unsigned char* Arows = is_local ? p.A_local : p.A;
    const int64_t a_ld = is_local ? p.lda_local_b : p.lda_b;
    const int a_row_off = is_local ? p.local_row_begin : 0;
    const int a_row_max = is_local ? p.local_rows - 1 : p.M - 1;

    // DMA sources: a wave-uniform base (first row of the tile, advanced along K in scalar registers) plus a
    // 32-bit per-lane offset, so that the load takes its address as SGPR base + VGPR offset and the K loop
    // carries no vector address arithmetic for it
    const int a_g0 = kGrouped ? 0 : min(m0 - a_row_off, a_row_max), b_g0 = min(n0, p.N - 1);
    const unsigned char* const a_base = Arows + (int64_t)a_g0 * a_ld + (int64_t)ka * KB;
    const unsigned char* b_base_ = p.B + (int64_t)b_g0 * p.ldb_b + (int64_t)ka * KB;
    if constexpr (kGrouped) b_base_ += (int64_t)p.block_expert[pid_m] * p.b_expert_stride_b;
    const unsigned char* const b_base = b_base_;
    uint32_t a_off[C::kAInstr], b_off[C::kBInstr];
#pragma unroll
    for (int t = 0; t < C::kAInstr; ++t) {
      const int r = (wave * C::kAInstr + t) * C::kRowsPerInstr + dma_row;  // row within the tile
      int gr;
      if constexpr (kGrouped) {
        // the token this row stands for; padding reads the first token of the block's segment (never stored)
        const int sid = p.sorted_ids[m0 + r];
        const int tok = sid < p.num_valid ? sid / p.topk : segment * p.m_per_rank;
        gr = min(max(tok - a_row_off, 0), is_local ? p.local_rows - 1 : p.a_rows - 1);
      } else {
        gr = min(m0 + r - a_row_off, a_row_max);
      }
      a_off[t] = (uint32_t)(gr - a_g0) * (uint32_t)a_ld + (uint32_t)((dma_pos ^ swz<KB>(r)) << 4);
    }
#pragma unroll
    for (int t = 0; t < C::kBInstr; ++t) {
      const int r = (wave * C::kBInstr + t) * C::kRowsPerInstr + dma_row;
      const int gr = min(n0 + r, p.N - 1);
      b_off[t] = (uint32_t)(gr - b_g0) * (uint32_t)p.ldb_b + (uint32_t)((dma_pos ^ swz<KB>(r)) << 4);
    }


    // DMA of K tile kt into stage kt % NST, one instruction at a time (kLoadsPerTile of them: A rows first, then
    // B rows). Past the last tile the last one is fetched again (into a stage nobody reads any more): every trip
    // of the main loop then issues the same number of loads, which keeps the loop free of branches and the vmcnt
    // bookkeeping constant.
    auto a_stage = [&](int kt) -> lds_u8 {
      return C::kSplit ? smem + (kt % C::kAStages) * C::kABytes : smem + (kt % NST) * C::kStageBytes;
    };
    auto b_stage = [&](int kt) -> lds_u8 {
      return C::kSplit ? smem + C::kAStages * C::kABytes + (kt % C::kBStages) * C::kBBytes
                       : smem + (kt % NST) * C::kStageBytes + C::kABytes;
    };
    // global_load_lds_dwordx4 in its SGPR-base + 32-bit-VGPR-offset form (the builtin only produces the 64-bit
    // VGPR address form, which costs a 64-bit vector add per load, and with one wave per SIMD every vector ALU
    // instruction in the K loop is time the MFMA pipe stands idle): M0 carries the wave-uniform LDS address.
    auto dma16 = [&](const unsigned char* sbase, uint32_t voff, lds_u8 dst) {
      const uint32_t lds_addr = (uint32_t)(uintptr_t)dst;
      // (M0 is a reserved register the compiler never allocates and nothing else in this kernel uses)
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "s"(lds_addr)
                   : "memory");
    };
    // A ragged last K tile (plain ring only): the lanes whose 16 bytes of K lie beyond the row's end fetch zeros from
    // kZeroChunk instead, through the load's 64-bit address form (the zero page is not within reach of a 32-bit
    // offset from the operand). Only the tile that holds the end of K takes this path.
    auto dma16_tail = [&](const unsigned char* sbase, uint32_t voff, int r, lds_u8 dst) {
      const int chunk = dma_pos ^ swz<KB>(r);   // which 16 bytes of the K tile this lane fetches
      const unsigned char* src = chunk * 16 < p.k_tail_bytes ? sbase + voff : kZeroChunk;
      __builtin_amdgcn_global_load_lds((const TDIST_AS1 void*)src, (TDIST_AS3 void*)dst, 16, 0, 0);
    };
    auto issue_a = [&](int kt, int t) {
      lds_u8 const dst = a_stage(kt) + (wave * C::kAInstr + t) * 1024;
      if constexpr (!C::kSplit) {
        if (p.k_tail_bytes != 0 && kb == KT && kt >= KTp - 1) {
          dma16_tail(a_base + (int64_t)(KTp - 1) * KB, a_off[t], (wave * C::kAInstr + t) * C::kRowsPerInstr + dma_row, dst);
          return;
        }
      }
      dma16(a_base + (int64_t)min(kt, KTp - 1) * KB, a_off[t], dst);
    };
    auto issue_b = [&](int kt, int u) {
      lds_u8 const dst = b_stage(kt) + (wave * C::kBInstr + u) * 1024;
      if constexpr (!C::kSplit) {
        if (p.k_tail_bytes != 0 && kb == KT && kt >= KTp - 1) {
          dma16_tail(b_base + (int64_t)(KTp - 1) * KB, b_off[u], (wave * C::kBInstr + u) * C::kRowsPerInstr + dma_row, dst);
          return;
        }
      }
      dma16(b_base + (int64_t)min(kt, KTp - 1) * KB, b_off[u], dst);
    };
    auto issue_dma = [&](int kt, int t) {
      if (t < C::kAInstr) issue_a(kt, t);
      else issue_b(kt, t - C::kAInstr);
    };
    auto issue_tile = [&](int kt) {
#pragma unroll
      for (int t = 0; t < C::kLoadsPerTile; ++t) issue_dma(kt, t);
    };

    // operand fragments of the K step being multiplied (cur) and of the one after it (nxt)
    typename E::frag a_cur[C::kTM], b_cur[C::kTN], a_nxt[C::kTM], b_nxt[C::kTN];
    // f-th operand fragment (A fragments first) of K step ks of tile kt
    // (a_st, b_st: the stages that hold the K tile's A and B rows)
    auto load_frag_from = [&](lds_u8 a_st, lds_u8 b_st, int ks, int f, typename E::frag* af, typename E::frag* bf) {
      // 16-byte chunks of this lane's K bytes (c1 == c0 for 16-byte fragments). With four lane groups and two chunks
      // per lane, group g takes chunks g and g + 4 rather than 2g and 2g + 1: any assignment of K bytes to lanes gives
      // the same product as long as A and B share it, and only with the four groups of one read on consecutive chunks
      // is the swizzle free of bank conflicts (every other chunk per read: half of the LDS cycles were conflicts).
      constexpr bool kStridedPieces = C::kLaneGroups == 4 && C::kFragVecs == 2;
      const int c0 = kStridedPieces ? lgrp : (ks * C::kLaneGroups + lgrp) * C::kFragVecs;
      const int c1 = kStridedPieces ? lgrp + 4 : c0 + C::kFragVecs - 1;
      if (f < C::kTM) {
        const int r = wm * C::kWaveM + f * E::kRows + lrow;
        lds_u8 const row = a_st + r * KB;
        af[f] = E::load(row + ((c0 ^ swz<KB>(r)) << 4), row + ((c1 ^ swz<KB>(r)) << 4));
      } else {
        const int j = f - C::kTM;
        const int r = wn * C::kWaveN + j * E::kRows + lrow;
        lds_u8 const row = b_st + r * KB;
        bf[j] = E::load(row + ((c0 ^ swz<KB>(r)) << 4), row + ((c1 ^ swz<KB>(r)) << 4));
      }
    };
    auto load_frag = [&](int kt, int ks, int f, typename E::frag* af, typename E::frag* bf) {
      load_frag_from(a_stage(kt), b_stage(kt), ks, f, af, bf);
    };
    // The same read with the stages as constants (split ring, 16-row MFMA blocks): the address is one of a few per-lane
    // bases (frag_lane_*, set up once per kernel: everything that depends on the lane) plus a constant that fits the
    // instruction's 16-bit offset field, so the K loop holds no address arithmetic for its LDS reads.
    auto load_frag_c = [&](auto sa_c, auto sb_c, auto ks_c, auto f_c, typename E::frag* af, typename E::frag* bf) {
      constexpr int SA = decltype(sa_c)::value % C::kAStages, SB = decltype(sb_c)::value % C::kBStages;
      constexpr int ks = decltype(ks_c)::value, f = decltype(f_c)::value;
      constexpr bool kStridedPieces = C::kLaneGroups == 4 && C::kFragVecs == 2;
      static_assert(kStridedPieces || (C::kLaneGroups == 4 && C::kFragVecs == 1 && C::kKSteps == 2), "pieces lgrp and lgrp + 4");
      constexpr int q0 = kStridedPieces ? 0 : ks, q1 = kStridedPieces ? 1 : ks;
      if constexpr (f < C::kTM) {
        constexpr int off = SA * C::kABytes + f * E::kRows * KB;
        constexpr bool hi = off >= 65536;
        lds_u8 const p0 = smem + (hi ? frag_lane_a_hi[q0] : frag_lane_a[q0]) + (hi ? off - 65536 : off);
        lds_u8 const p1 = smem + (hi ? frag_lane_a_hi[q1] : frag_lane_a[q1]) + (hi ? off - 65536 : off);
        af[f] = E::load(p0, p1);
      } else {
        constexpr int j = f - C::kTM;
        constexpr int off = SB * C::kBBytes + j * E::kRows * KB;
        static_assert(off < 65536, "B stages within reach of the offset field");
        bf[j] = E::load(smem + frag_lane_b[q0] + off, smem + frag_lane_b[q1] + off);
      }
    };
    // Split ring, K loop unrolled over the six (A stage, B stage) pairs: stage S of either ring as a constant address
    auto a_stage_c = [&](auto s_c) -> lds_u8 { return smem + (decltype(s_c)::value % C::kAStages) * C::kABytes; };
    // (the same as byte offsets into the ring: C::a_stage_off(S), C::b_stage_off(S))
    auto b_stage_c = [&](auto s_c) -> lds_u8 {
      return smem + C::kAStages * C::kABytes + (decltype(s_c)::value % C::kBStages) * C::kBBytes;
    };
    // The LDS address of such a load is a constant plus the wave's share of the stage; added inside the assembly, so
    // that the compiler does not keep the sum of every (stage, instruction) pair in a scalar register of its own
    // (there are more pairs than registers, and a spilled one comes back through the vector ALU).
    auto dma16_at = [&](const unsigned char* sbase, uint32_t voff, int dst_const, uint32_t dst_wave) {
      // (the constant as a literal of the instruction: held in scalar registers, the forty of them are hoisted out of
      // the K loop, spilled, and reloaded through the vector ALU inside it)
      asm volatile("s_add_u32 m0, %3, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "n"(dst_const),
                   "s"(dst_wave)
                   : "memory", "scc");
    };
    // start of the ring plus the wave's share of a stage
    const uint32_t a_wave_off = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)smem + wave * C::kAInstr * 1024);
    const uint32_t b_wave_off = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)smem + wave * C::kBInstr * 1024);
    // K tile kt_src's rows into the stage at byte `st` of the ring
    auto issue_a_to = [&](int st, int kt_src, int t) {
      dma16_at(a_base + (int64_t)min(kt_src, KTp - 1) * KB, a_off[t], st + t * 1024, a_wave_off);
    };
    auto issue_b_to = [&](int st, int kt_src, int u) {
      dma16_at(b_base + (int64_t)min(kt_src, KTp - 1) * KB, b_off[u], st + u * 1024, b_wave_off);
    };
    auto load_frags = [&](int kt, int ks, typename E::frag* af, typename E::frag* bf) {
#pragma unroll
      for (int f = 0; f < C::kTM + C::kTN; ++f) load_frag(kt, ks, f, af, bf);
    };

    // accumulators: fixed registers a[0 .. kAccRegs) for the 16-row MFMA blocks, else the compiler's
    typename E::acc_t acc[kFixedAcc ? 1 : C::kTN][kFixedAcc ? 1 : C::kTM];
    if constexpr (kFixedAcc) {
      // (the split ring's K loops clear them behind the first loads' issue: 256 register writes that the loads' round
      // trip hides there)
      if constexpr (!(C::kSplit && E::kRows == 16)) acc_clear<kAccRegs>();
    } else {
#pragma unroll
      for (int j = 0; j < C::kTN; ++j)
#pragma unroll
        for (int i = 0; i < C::kTM; ++i)
#pragma unroll
          for (int e = 0; e < C::kAccLen; ++e) acc[j][i][e] = 0.f;
    }

    constexpr int kMfmaPerStep = C::kTM * C::kTN;
    static_assert(!C::kSplit || E::kRows == 16, "the split ring's K loops are written for the 16-row MFMA blocks");
    if constexpr (C::kSplit && E::kRows == 16 && C::kKSteps == 1) {
      // ---- split ring, 16-row MFMA blocks, the whole K tile in one MFMA depth (e4m3) --------------------
      // The MFMAs of a tile run as four quarters: the lower half of the A fragments against one half of the B
      // fragments, then against the other half, then the upper A half against that other half and against the first
      // one again (128 x 128 wave tile: 4 x 4 blocks per quarter). Every quarter reads the fragments whose registers
      // have just fallen idle:
      //   quarter 0: the B half that quarter 1 needs;     quarter 1: the upper A half of this tile;
      //   quarter 2: the lower A half of the next tile;   quarter 3: the B half quarter 2 has finished with, for the
      //                                                    next tile, which therefore starts with that half.
      // So the B halves swap roles from one tile to the next, the fragment registers are never doubled, and the LDS
      // reads are spread evenly over the tile. The barrier (tile kt+1 has landed everywhere, nobody reads tile kt's
      // stages any more) stands in front of quarter 2; the refill DMA ([B(kt+2) rows, A(kt+3) rows], as in the other
      // split-ring loops) goes out evenly spaced from there to the next barrier.
      constexpr int kHA = C::kTM / 2, kHB = C::kTN / 2, kQuarter = kHA * kHB;
      static_assert(C::kTM % 2 == 0 && C::kTN % 2 == 0 && kQuarter - 2 >= kHA && kQuarter - 2 >= kHB,
                    "a quarter has a slot for each of its fragment reads");
      constexpr int kBar = 2 * kQuarter + 1;           // the barrier sits in front of this slot's MFMA
      // list entry q goes out ceil(q * slots / entries) slots after the barrier
      auto dma_due = [](int since) constexpr {
        for (int q = 0; q < C::kLoadsPerTile; ++q)
          if ((q * kMfmaPerStep + C::kLoadsPerTile - 1) / C::kLoadsPerTile == since) return q;
        return -1;
      };
      constexpr int kProDma = [&]() constexpr {        // entries that fall between a barrier and the tile's end
        int n = 0;
        for (int since = 0; since < kMfmaPerStep - kBar; ++since) n += dma_due(since) >= 0 ? 1 : 0;
        return n;
      }();
      auto issue_list = [&](int cyc, int q) {
        if (q < C::kBInstr) issue_b(cyc + 2, q);
        else issue_a(cyc + 3, q - C::kBInstr);
      };
      static_assert(!kEarly || kProDma == C::kBInstr, "the prologue's share of the first list is B(1)");
      if (kEarly && prefetched) {
        // A(0), B(0) and B(1) went out before the last tile's epilogue; its stores are allowed to be still on their way
#pragma unroll
        for (int t = 0; t < C::kAInstr; ++t) issue_a(1, t);
        acc_clear<kAccRegs>();
        wait_tiles_and_barrier<kEarly ? C::kBInstr + kEpiStores + C::kAInstr : 0>();
      } else {
#pragma unroll
        for (int t = 0; t < C::kAInstr; ++t) issue_a(0, t);
#pragma unroll
        for (int u = 0; u < C::kBInstr; ++u) issue_b(0, u);
#pragma unroll
        for (int t = 0; t < C::kAInstr; ++t) issue_a(1, t);
#pragma unroll
        for (int q = 0; q < kProDma; ++q) issue_list(-1, q);
        acc_clear<kAccRegs>();
        wait_tiles_and_barrier<C::kAInstr + kProDma>();
      }
#pragma unroll
      for (int f = 0; f < kHA; ++f) load_frag(0, 0, f, a_cur, b_cur);            // lower A half
#pragma unroll
      for (int f = 0; f < kHB; ++f) load_frag(0, 0, C::kTM + f, a_cur, b_cur);   // lower B half
      __builtin_amdgcn_sched_barrier(0);
      // one tile; kOdd: the B halves in the order (upper, lower); SA, SB: the stages of its A and B rows (the tile
      // after it sits in the next stage of either ring: behind the last K tile that is a stage nobody needs, read all
      // the same, so that every trip runs the same instructions)
      auto tile = [&](auto odd_c, auto sa_c, auto sb_c, int kt) {
        constexpr int kOdd = decltype(odd_c)::value, SA = decltype(sa_c)::value, SB = decltype(sb_c)::value;
        constexpr int a_now = C::a_stage_off(SA);
        constexpr int b_now = C::b_stage_off(SB), b_nx = C::b_stage_off(SB + 1);
        // entry q of the list begun at this tile's barrier ([B(kt+2), A(kt+3)]: the stages of this tile's own rows) or
        // of the one before ([B(kt+1), A(kt+2)])
        auto issue_entry = [&](auto own_c, int q) {
          constexpr bool own = decltype(own_c)::value;
          if (q < C::kBInstr) issue_b_to(own ? b_now : b_nx, own ? kt + 2 : kt + 1, q);
          else issue_a_to(own ? a_now : C::a_stage_off(SA + 2), own ? kt + 3 : kt + 2, q - C::kBInstr);
        };
        static_for<kMfmaPerStep>([&](auto u_c) {
          constexpr int u = decltype(u_c)::value;
          constexpr int quarter = u / kQuarter, w = u % kQuarter;
          constexpr int a_half = quarter / 2;
          constexpr int b_half = ((quarter == 1 || quarter == 2) ? 1 : 0) ^ kOdd;
          constexpr int j = kHB * b_half + w / kHA, i = kHA * a_half + w % kHA;
          if constexpr (u == kBar) {
            __builtin_amdgcn_sched_barrier(0);
            wait_tiles_and_barrier<C::kAInstr>();
            __builtin_amdgcn_sched_barrier(0);
          }
          E::template mma_at<(j * C::kTM + i) * C::kAccLen>(b_cur[j], a_cur[i]);
          // the quarter's fragment reads, from its slot 2 on (128 x 128 wave tile: slots 2, 5, 8, 11)
          constexpr int n_reads = (quarter == 0 || quarter == 3) ? kHB : kHA;
          constexpr int stride = (kQuarter - 2) / n_reads;
          if constexpr (w >= 2 && (w - 2) % stride == 0 && (w - 2) / stride < n_reads) {
            constexpr int f = (w - 2) / stride;
            using Z = std::integral_constant<int, 0>;
            using NowA = std::integral_constant<int, SA>; using NowB = std::integral_constant<int, SB>;
            using NxA = std::integral_constant<int, SA + 1>; using NxB = std::integral_constant<int, SB + 1>;
            if constexpr (quarter == 0) load_frag_c(NowA{}, NowB{}, Z{}, std::integral_constant<int, C::kTM + kHB * (1 ^ kOdd) + f>{}, a_cur, b_cur);
            if constexpr (quarter == 1) load_frag_c(NowA{}, NowB{}, Z{}, std::integral_constant<int, kHA + f>{}, a_cur, b_cur);
            if constexpr (quarter == 2) load_frag_c(NxA{}, NxB{}, Z{}, std::integral_constant<int, f>{}, a_cur, b_cur);
            if constexpr (quarter == 3) load_frag_c(NxA{}, NxB{}, Z{}, std::integral_constant<int, C::kTM + kHB * (1 ^ kOdd) + f>{}, a_cur, b_cur);
          }
          constexpr int since = (u - kBar + kMfmaPerStep) % kMfmaPerStep;  // slots since the last barrier
          constexpr int due = dma_due(since);
          if constexpr (due >= 0) issue_entry(std::integral_constant<bool, (u >= kBar)>{}, due);
          __builtin_amdgcn_sched_barrier(0);
        });
      };
      for (int kt = 0; kt < KTp; kt += 6) {
        static_for<6>([&](auto n_c) {
          constexpr int n = decltype(n_c)::value;
          if (kt + n < KTp)
            tile(std::integral_constant<int, n % 2>{}, std::integral_constant<int, n % 3>{}, std::integral_constant<int, n % 2>{}, kt + n);
        });
      }
      asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");  // the last MFMAs' results: 8 passes + 3 cycles after issue
    } else if constexpr (C::kSplit && E::kRows == 16) {
      // ---- split ring, 16-row MFMA blocks ------------------------------------------------------------
      // The MFMAs of a K step run in B-fragment-major order: a B fragment serves kTM MFMAs in a row and is then dead,
      // so the next step's B fragment is read into the same registers right behind them; only the A fragments, which
      // the whole step uses, are double-buffered. No read sits in the first kLead slots: the last step of a tile holds
      // its barrier there (the reads before it come from the stages the barrier releases, and the last of them,
      // issued behind the previous step's final MFMA, has those slots to come back).
      static_assert(C::kKSteps == 2 && C::kTM >= 4, "schedule written for two K steps per tile");
      constexpr int kLead = C::kTM - 1 < 4 ? C::kTM - 1 : 4;
      constexpr int kAStride = (kMfmaPerStep - kLead - 2) / C::kTM;  // slots between two A fragment reads
      auto issue_list = [&](int cyc, int q) {
        if (q < C::kBInstr) issue_b(cyc + 2, q);
        else issue_a(cyc + 3, q - C::kBInstr);
      };
      static_assert(!kEarly || C::kDmaPerStep == C::kBInstr, "the prologue's share of the first list is B(1)");
      if (kEarly && prefetched) {
        // A(0), B(0) and B(1) went out before the last tile's epilogue; its stores are allowed to be still on their way
#pragma unroll
        for (int t = 0; t < C::kAInstr; ++t) issue_a(1, t);
        acc_clear<kAccRegs>();
        wait_tiles_and_barrier<kEarly ? C::kBInstr + kEpiStores + C::kAInstr : 0>();
      } else {
#pragma unroll
        for (int t = 0; t < C::kAInstr; ++t) issue_a(0, t);
#pragma unroll
        for (int u = 0; u < C::kBInstr; ++u) issue_b(0, u);
#pragma unroll
        for (int t = 0; t < C::kAInstr; ++t) issue_a(1, t);
#pragma unroll
        for (int q = 0; q < C::kDmaPerStep; ++q) issue_list(-1, q);
        acc_clear<kAccRegs>();
        wait_tiles_and_barrier<C::kAInstr + C::kDmaPerStep>();
      }
      load_frags(0, 0, a_cur, b_cur);
      __builtin_amdgcn_sched_barrier(0);
      // K tile kt, its A rows in stage SA and its B rows in stage SB (the tile after it sits in the next stage of either
      // ring: behind the last K tile that is a stage nobody needs, read all the same, so that every trip runs the same
      // instructions)
      auto k_tile = [&](auto sa_c, auto sb_c, int kt) {
        constexpr int SA = decltype(sa_c)::value, SB = decltype(sb_c)::value;
        constexpr int st_a = C::a_stage_off(SA);
        constexpr int st_b = C::b_stage_off(SB), st_b_nx = C::b_stage_off(SB + 1);
        // entry q of this tile's own refill list ([B(kt+2), A(kt+3)]: into the stages of its own rows) or of the one
        // before ([B(kt+1), A(kt+2)])
        auto issue_entry = [&](auto own_c, int q) {
          constexpr bool own = decltype(own_c)::value;
          if (q < C::kBInstr) issue_b_to(own ? st_b : st_b_nx, own ? kt + 2 : kt + 1, q);
          else issue_a_to(own ? st_a : C::a_stage_off(SA + 2), own ? kt + 3 : kt + 2, q - C::kBInstr);
        };
        auto step = [&](auto ks_c, typename E::frag* a_now, typename E::frag* a_new) {
          constexpr int ks = decltype(ks_c)::value;
          constexpr bool last = ks == C::kKSteps - 1;
          constexpr int first = last ? kLead : 0;
          constexpr int nslots = kMfmaPerStep - first;
          constexpr int pos = (ks + 1) % C::kKSteps;
          // stages and K step the reads of this step fetch
          using RA = std::integral_constant<int, last ? SA + 1 : SA>;
          using RB = std::integral_constant<int, last ? SB + 1 : SB>;
          using RKs = std::integral_constant<int, last ? 0 : ks + 1>;
          static_for<kMfmaPerStep>([&](auto idx_c) {
            constexpr int idx = decltype(idx_c)::value;
            constexpr int j = idx / C::kTM, i = idx % C::kTM;
            E::template mma_at<(j * C::kTM + i) * C::kAccLen>(b_cur[j], a_now[i]);
            if constexpr (last && idx == kLead - 1) {
              __builtin_amdgcn_sched_barrier(0);
              wait_tiles_and_barrier<C::kAInstr>();
              __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (i == C::kTM - 1) load_frag_c(RA{}, RB{}, RKs{}, std::integral_constant<int, C::kTM + j>{}, a_new, b_cur);  // B fragment j, in place
            if constexpr (idx > kLead && (idx - kLead - 1) % kAStride == 0 && (idx - kLead - 1) / kAStride < C::kTM)
              load_frag_c(RA{}, RB{}, RKs{}, std::integral_constant<int, (idx - kLead - 1) / kAStride>{}, a_new, b_cur);
            if constexpr (idx >= first) {
              constexpr int slot = idx - first;
#pragma unroll
              for (int d = 0; d < C::kDmaPerStep; ++d)
                if (slot == (d * nslots) / C::kDmaPerStep) issue_entry(std::integral_constant<bool, last>{}, pos * C::kDmaPerStep + d);
            }
            __builtin_amdgcn_sched_barrier(0);
          });
        };
        step(std::integral_constant<int, 0>{}, a_cur, a_nxt);
        step(std::integral_constant<int, 1>{}, a_nxt, a_cur);
      };
      // unrolled over the six (A stage, B stage) pairs: every LDS address in the loop is a constant
      for (int kt = 0; kt < KTp; kt += 6) {
        static_for<6>([&](auto n_c) {
          constexpr int n = decltype(n_c)::value;
          if (kt + n < KTp) k_tile(std::integral_constant<int, n % 3>{}, std::integral_constant<int, n % 2>{}, kt + n);
        });
      }
      // the last MFMAs' results are readable 4 passes + 3 cycles after issue
      asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
    } else {
    // ---- prologue: P tiles in flight, wait for tile 0 ------------------------------------------
#pragma unroll
    for (int t = 0; t < C::kP; ++t) issue_tile(t);
    wait_tiles_and_barrier<(C::kP - 1) * C::kLoadsPerTile>();
    issue_tile(C::kP);
    load_frags(0, 0, a_cur, b_cur);

    // ---- main loop over K tiles -----------------------------------------------------------------
    // Every K step multiplies the fragments read during the previous step while it reads the next ones, one
    // LDS read slotted behind each of the first MFMAs so that neither pipe waits for the other. The last
    // step of a tile first joins the barrier (tile kt+1 has landed everywhere, tile kt is no longer read),
    // then also refills the freed stage.
    constexpr int kReadsPerStep = (C::kTM + C::kTN) * C::kFragVecs;
    for (int kt = 0; kt < KTp; ++kt) {
#pragma unroll
      for (int ks = 0; ks < C::kKSteps; ++ks) {
        if (ks + 1 < C::kKSteps) {
          load_frags(kt, ks + 1, a_nxt, b_nxt);
#pragma unroll
          for (int idx = 0; idx < kMfmaPerStep; ++idx) {
            const int j = idx / C::kTM, i = idx % C::kTM;
            acc[j][i] = E::mma(b_cur[j], a_cur[i], acc[j][i]);
          }
#pragma unroll
          for (int r = 0; r < kReadsPerStep; ++r) {
            __builtin_amdgcn_sched_group_barrier(kSchedMfma, 1, 0);
            __builtin_amdgcn_sched_group_barrier(kSchedDsRead, 1, 0);
          }
          __builtin_amdgcn_sched_group_barrier(kSchedMfma, kMfmaPerStep - kReadsPerStep, 0);
        } else {
#pragma unroll
          for (int idx = 0; idx < C::kLeadMfma; ++idx) {
            const int j = idx / C::kTM, i = idx % C::kTM;
            acc[j][i] = E::mma(b_cur[j], a_cur[i], acc[j][i]);
          }
          __builtin_amdgcn_sched_barrier(0);
          wait_tiles_and_barrier<(C::kP - 1) * C::kLoadsPerTile>();
          __builtin_amdgcn_sched_barrier(0);
          // the rest of the step's MFMAs, each followed by its share of the refill DMA and of the next tile's
          // first fragment reads; the fences pin this order
          constexpr int kTail = kMfmaPerStep - C::kLeadMfma;
          constexpr int kFrags = C::kTM + C::kTN;
          constexpr int kSlots = kFrags < kTail ? kFrags : kTail;
          constexpr int kDmaPerSlot = (C::kLoadsPerTile + kSlots - 1) / kSlots;
          constexpr int kFragPerSlot = (kFrags + kSlots - 1) / kSlots;
          const int kt_next = min(kt + 1, KTp - 1);
#pragma unroll
          for (int idx = C::kLeadMfma; idx < kMfmaPerStep; ++idx) {
            const int j = idx / C::kTM, i = idx % C::kTM;
            acc[j][i] = E::mma(b_cur[j], a_cur[i], acc[j][i]);
            const int slot = idx - C::kLeadMfma;
            if (slot < kSlots) {
#pragma unroll
              for (int d = 0; d < kDmaPerSlot; ++d)
                if (slot * kDmaPerSlot + d < C::kLoadsPerTile) issue_dma(kt + 1 + C::kP, slot * kDmaPerSlot + d);
#pragma unroll
              for (int f = 0; f < kFragPerSlot; ++f)
                if (slot * kFragPerSlot + f < kFrags) load_frag(kt_next, 0, slot * kFragPerSlot + f, a_nxt, b_nxt);
              __builtin_amdgcn_sched_barrier(0);
            }
          }
        }
#pragma unroll
        for (int i = 0; i < C::kTM; ++i) a_cur[i] = a_nxt[i];
#pragma unroll
        for (int j = 0; j < C::kTN; ++j) b_cur[j] = b_nxt[j];
      }
    }

    }

    // ---- epilogue ---------------------------------------------------------------------------------
    // A lane's accumulators, seen as kRowBlocks blocks of 32 rows of the wave tile times kGroups groups of four
    // consecutive columns of one row. Group g of row block ib is
    //   32-row MFMA blocks: acc[g/4][ib][4*(g%4) ...],   row 32*ib + lrow,              column 8*g + 4*lgrp
    //   16-row MFMA blocks: acc[g/2][2*ib + g%2][0 ...], row 32*ib + 16*(g%2) + lrow,   column 16*(g/2) + 4*lgrp
    constexpr int kRowBlocks = C::kWaveM / 32, kGroups = C::kWaveN / 8;
    constexpr bool kWide = E::kRows == 32;
    // Is the next tile's start issued before this tile's epilogue? Both tiles whole and ungated, this one stored by
    // the vector epilogue (the per-lane offsets of the operand loads are then the same for both, only the uniform bases differ). Decided here,
    // behind the K loop, so that nothing of it is held in registers across the loop.
    bool early = false;
    const unsigned char* a_base_n = a_base;
    const unsigned char* b_base_n = b_base;
    if constexpr (kEarly) {
      int nm0 = 0, nn0 = 0;
      const bool next_whole_round = !arrival && sbase < total_sched && !(sk_split > 1 && sbase + G > total_sched) && sbase + wg_pos < total_sched;
      if (p.flags == nullptr && p.A_local == nullptr && sk_s == 1 && KT >= 2 && next_whole_round && m0 + BM <= p.M &&
          n0 + BN <= p.N && p.ldc % 8 == 0 && locate(sbase + wg_pos, nm0, nn0) && nm0 + BM <= p.M && nn0 + BN <= p.N) {
        bool c_aligned = (reinterpret_cast<uintptr_t>(p.C) & 15) == 0;
        if (p.scatter_bufs != nullptr) c_aligned = (reinterpret_cast<uintptr_t>(p.scatter_bufs[m0 / p.m_per_rank]) & 15) == 0;
        if (c_aligned) {
          early = true;
          a_base_n = p.A + (int64_t)nm0 * p.lda_b;
          b_base_n = p.B + (int64_t)nn0 * p.ldb_b;
        }
      }
      // (wave-uniform by construction; said so to the compiler, which otherwise carries them in vector registers)
      auto uniform_ptr = [](const unsigned char* q) {
        const uint64_t v = reinterpret_cast<uint64_t>(q);
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
        return reinterpret_cast<const unsigned char*>(((uint64_t)hi << 32) | lo);
      };
      a_base_n = uniform_ptr(a_base_n);
      b_base_n = uniform_ptr(b_base_n);
    }
    if (kEarly && early) {
      // nobody reads the ring any more; then the next tile's A(0), B(0), B(1) go out into A stage 0 and the B stages,
      // and once everything older than them has landed (the loads the K loop issued beyond the tile's end, which may
      // point anywhere in the ring) the A stages 1 and 2 are free for staging
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
#pragma unroll
      for (int t = 0; t < C::kAInstr; ++t) dma16(a_base_n, a_off[t], smem + (wave * C::kAInstr + t) * 1024);
#pragma unroll
      for (int u = 0; u < C::kBInstr; ++u)
        dma16(b_base_n, b_off[u], smem + C::kAStages * C::kABytes + (wave * C::kBInstr + u) * 1024);
#pragma unroll
      for (int u = 0; u < C::kBInstr; ++u)
        dma16(b_base_n + KB, b_off[u], smem + C::kAStages * C::kABytes + C::kBBytes + (wave * C::kBInstr + u) * 1024);
      wait_tiles_and_barrier<C::kAInstr + 2 * C::kBInstr>();
    } else {
      wait_tiles_and_barrier<0>();  // every DMA has landed and no wave reads the ring any more: reuse it
    }
    // arrival order: the look for the next tile goes out while this tile is being stored and is used when it has been.
    // Issued behind the epilogue's own loads (the scales), not in front of them: loads retire in order, so the wait
    // for the scales would otherwise be a wait for the look's round trip as well.
    int arr_flag = 0;
    int arr_behind = 0;
    bool arr_issued = false;
    // stores_behind: the 16-byte stores this wave still issues behind the look (all of them, or none)
    auto arr_issue = [&](int stores_behind) {
      if (arrival && wave == 0 && !arr_issued) {
        if constexpr (kFixedAcc) {
          // The look lands in an accumulator register of the row block that has just been staged (a0: nothing uses
          // it before the next tile clears it) and is fetched from there when the tile is chosen, behind a wait that
          // leaves this wave's stores in flight. Left to the compiler, the wait for a load's result is a wait for
          // everything the wave has issued, stores included: it does not count on loads and stores retiring in order
          // through the one counter, as they do here. The register is first set to a value that is no chunk's
          // go-ahead: should the wait ever let go with the load still out, the choice sees "not arrived" and polls.
          int l = lane;
          asm volatile("" : "+v"(l));
          const uint32_t flag_off = (uint32_t)min(l, n_chunks - 1) * 4u;
          const int not_yet = p.wait_value ^ 0x40000000;
          asm volatile("v_accvgpr_write_b32 a0, %2\n\tglobal_load_dword a0, %0, %1 sc0 sc1" : : "v"(flag_off), "s"(p.flags), "v"(not_yet) : "memory");
          arr_behind = stores_behind;
        } else {
          arr_flag = arr_look();
        }
      }
      arr_issued = true;
    };
    lds_u8 const epi = (kEarly && early) ? smem + C::kABytes + wave * (64 * C::kEpiPitch) : smem + wave * C::kEpiBytes;
    // The epilogue's lane-dependent addresses are the same for every tile; computed from these opaque copies they are
    // rebuilt per tile (a few dozen instructions) instead of being held in ~100 registers across the K loop.
    int e_lane = lane;
    asm volatile("" : "+v"(e_lane));
    const int e_lrow = e_lane % E::kRows, e_lgrp = e_lane / E::kRows;
    // row (within its 32-row block) and first column of this lane's group g
    auto group_row = [&](int g) { return kWide ? e_lrow : 16 * (g % 2) + e_lrow; };
    auto group_col = [&](int g) { return kWide ? 8 * g + 4 * e_lgrp : 16 * (g / 2) + 4 * e_lgrp; };
    // index of group g's row among the row scales held per MFMA row block
    auto scale_slot = [&](int ib, int g) { return kWide ? ib : 2 * ib + g % 2; };
    // the four accumulators of group g of row block ib (fixed accumulators: read out of their registers here, one
    // by one where they are used, so that no copy of the whole set is ever held in vector registers)
    auto acc4 = [&](auto ib_c, auto g_c) -> float4v {
      constexpr int ib = decltype(ib_c)::value, g = decltype(g_c)::value;
      constexpr int j = kWide ? g / 4 : g / 2, i = kWide ? ib : 2 * ib + g % 2, e0 = kWide ? 4 * (g % 4) : 0;
      if constexpr (kFixedAcc) {
        constexpr int r = (j * C::kTM + i) * C::kAccLen + e0;
        float v0, v1, v2, v3;
        asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(v0) : "n"(r));
        asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(v1) : "n"(r + 1));
        asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(v2) : "n"(r + 2));
        asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(v3) : "n"(r + 3));
        return float4v{v0, v1, v2, v3};
      } else {
        return float4v{acc[j][i][e0], acc[j][i][e0 + 1], acc[j][i][e0 + 2], acc[j][i][e0 + 3]};
      }
    };
    // destination of this tile's rows
    unsigned char* Cbase;
    int64_t crow0;
    if (p.scatter_bufs != nullptr) {
      const int owner = m0 / p.m_per_rank;
      Cbase = (unsigned char*)p.scatter_bufs[owner];
      crow0 = (int64_t)p.rank * p.m_per_rank + (m0 - owner * p.m_per_rank);
    } else {
      Cbase = p.C;
      crow0 = m0;
    }
    constexpr int kLanesPerRow = C::kEpiChunks;  // lanes per staged row: one per 16-byte piece, the last ones idle
                                                 // where the row is no power of two wide
    constexpr bool kFullRows = C::kRowPieces == C::kEpiChunks;
    constexpr int kRowsPerPass = 64 / kLanesPerRow;
    const int er = e_lane / kLanesPerRow, ec = e_lane % kLanesPerRow;
    const bool n_vec_ok = (p.ldc % 8 == 0) && ((reinterpret_cast<uintptr_t>(Cbase) & 15) == 0);

    // scales and packs four columns of one row (row scale rsi, column scales csg) and writes them to `where` in the
    // staging rows
    auto stage_vals = [&](float4v v, float rsi, const float4v csg, lds_u8 where) {
      if constexpr (kScales) {
        v[0] *= rsi * csg[0];
        v[1] *= rsi * csg[1];
        v[2] *= rsi * csg[2];
        v[3] *= rsi * csg[3];
      }
      const int2v w = {(int)E::pack(v[0], v[1]), (int)E::pack(v[2], v[3])};
      *(TDIST_AS3 int2v*)where = w;
    };
    // staging address of this lane's group g in row block ib
    auto stage_addr = [&](int ib, int g) -> lds_u8 {
      const int mrow = 32 * ib + group_row(g), ncol = group_col(g);
      return epi + mrow * C::kEpiPitch + ((((ncol >> 3) ^ (mrow & C::kEpiSwz))) << 4) + (ncol & 7) * 2;
    };
    // group g of row block ib (`rs` holds the row scales by scale_slot, `csg` the group's four column scales)
    auto stage_group = [&](auto ib_c, auto g_c, const float* rs, const float4v csg) {
      constexpr int ib = decltype(ib_c)::value, g = decltype(g_c)::value;
      stage_vals(acc4(ib_c, g_c), kScales ? rs[scale_slot(ib, g)] : 1.f, csg, stage_addr(ib, g));
    };
    // the same for the four groups of the 32 x 32 block (ib, jb); cs4[g % 4] are their column scales
    auto stage_block = [&](auto ib_c, auto jb_c, const float* rs, const float4v* cs4) {
      constexpr int jb = decltype(jb_c)::value;
      static_for<4>([&](auto q_c) {
        constexpr int q = decltype(q_c)::value;
        stage_group(ib_c, std::integral_constant<int, 4 * jb + q>{}, rs, kScales ? cs4[q] : float4v{1.f, 1.f, 1.f, 1.f});
      });
      __builtin_amdgcn_sched_barrier(0);  // keep the accumulator read-out block by block (register pressure)
    };
    // one staged 16-byte piece → global memory
    auto store_piece_at = [&](int mrow, int piece, const int4v v) {
      const int gm = m0 + wm * C::kWaveM + mrow;
      const int gn = n0 + wn * C::kWaveN + piece * 8;
      int64_t crow = crow0 + wm * C::kWaveM + mrow;
      bool row_ok = gm < p.M;
      if constexpr (kGrouped) {
        const int sid = p.sorted_ids[gm];  // the row's place in C; padding is dropped
        crow = sid;
        row_ok = sid < p.num_valid;
      }
      if (row_ok && gn < p.N) {
        TDIST_AS1 unsigned short* dst = (TDIST_AS1 unsigned short*)Cbase + crow * p.ldc + gn;  // device memory: global stores
        if (gn + 8 <= p.N && n_vec_ok) {
          if (p.scatter_bufs == nullptr) __builtin_nontemporal_store(v, (TDIST_AS1 int4v*)dst);  // written once, not read back here
          else *(TDIST_AS1 int4v*)dst = v;
        } else {
          for (int e = 0; e < 8; ++e)
            if (gn + e < p.N) dst[e] = (unsigned short)(((uint32_t)v[e >> 1] >> ((e & 1) * 16)) & 0xffffu);
        }
      }
    };
    auto staged_piece_at = [&](int mrow, int piece) -> int4v {
      return *(const TDIST_AS3 int4v*)(epi + mrow * C::kEpiPitch + ((piece ^ (mrow & C::kEpiSwz)) << 4));
    };
    // staged rows [row0, row0 + nrows) of the wave tile → global memory, 16 bytes per lane
    auto store_rows = [&](int row0, int nrows) {
#pragma unroll 4
      for (int pass = 0; pass < nrows / kRowsPerPass; ++pass) {
        const int mrow = row0 + pass * kRowsPerPass + er;
        if (kFullRows || ec < C::kRowPieces) store_piece_at(mrow, ec, staged_piece_at(mrow, ec));
      }
    };
    static_assert(32 % kRowsPerPass == 0, "a 32-row block is a whole number of store passes");

    if (sk_s > 1) {
      // ---- this piece is 1/sk_s of the tile's K range: exchange through the workspace --------------------------
      constexpr int kThreads = C::kWaves * 64;
      constexpr int kQuads = kRowBlocks * kGroups;  // float4 groups of accumulators per lane
      const int w0 = wg_pos - sk_j;                 // first workgroup of this tile's pieces
      // slot addresses: a uniform base per float4 group plus one 32-bit lane offset (from an opaque copy of the
      // thread id, so that nothing of this is computed ahead and held across the K loop)
      uint32_t sk_voff = threadIdx.x;
      asm volatile("" : "+v"(sk_voff));
      sk_voff *= 16u;
      // (1) the slot is free once the readers of this workgroup's previous partial are done with it
      if (threadIdx.x == 0) {
        int ok = 0;
        for (int it = 0; it < p.spin_limit; ++it) {
          if (__hip_atomic_load(sk_acks + wg_pos, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == sk_need) {
            ok = 1;
            break;
          }
          __builtin_amdgcn_s_sleep(2);
        }
        *s_gate = ok;
      }
      __syncthreads();
      const int slot_ok = *s_gate;
      __syncthreads();
      sk_need += sk_s;

      if (slot_ok) {
        // (2) the partial, every store instruction a contiguous KiB. The pieces of a tile sit on workgroups s*t ..
        // s*t+s-1 of the round, which the XCD-aware order puts on ONE XCD whenever s divides the workgroups per XCD:
        // the partials then need to go no further than that XCD's L2 (plain stores; the readers invalidate their
        // own first-level cache and find the lines in the L2 they share with the writers). Otherwise the stores are
        // coherent at device scope (written through to memory).
        // The store sits in inline assembly (the cache-policy bit has no builtin), where the compiler sees neither
        // a memory instruction nor its hazards. Hence: a vector address (a scalar base that the compiler happened
        // to reload from a spill lane with v_readlane would need five wait states before the store), and a wait
        // state after the store before anything may overwrite its data registers.
        unsigned char* slot = (unsigned char*)(p.sk_partials + (int64_t)wg_pos * (BM * BN)) + sk_voff;
        static_for<kQuads>([&](auto r_c) {
          constexpr int r = decltype(r_c)::value;
          const float4v t = acc4(std::integral_constant<int, r / kGroups>{}, std::integral_constant<int, r % kGroups>{});
          if (sk_xcd_local) asm volatile("s_nop 1\n\tglobal_store_dwordx4 %0, %1, off\n\ts_nop 1" ::"v"(slot), "v"(t) : "memory");
          else asm volatile("s_nop 1\n\tglobal_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" ::"v"(slot), "v"(t) : "memory");
          slot += kThreads * 16;
          asm volatile("" : "+v"(slot));  // one running address, not sixty-four precomputed ones
          if constexpr (r % 4 == 3) __builtin_amdgcn_sched_barrier(0);
        });
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (threadIdx.x == 0)
          __hip_atomic_store(sk_flags + wg_pos, sk_tag | (my_xcc << kSkTagBits), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }

      // (3) all pieces of the tile: thread i waits for the flag of piece i. (The full limit even after an error
      // elsewhere: these pieces are being computed, not awaited from outside; if a workgroup gave its piece up at a
      // chunk flag, the wait runs out and the tile is not stored.)
      if (threadIdx.x < 64) {
        int ok = 1, same_xcd = 1;
        if ((int)threadIdx.x < sk_s) {
          ok = 0;
          for (int it = 0; it < p.spin_limit; ++it) {
            const int f = __hip_atomic_load(sk_flags + w0 + threadIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if ((f & kSkTagMask) == sk_tag) {
              ok = 1;
              same_xcd = (f >> kSkTagBits) == my_xcc;
              break;
            }
            __builtin_amdgcn_s_sleep(2);
          }
        }
        const int all_ok = __ballot(ok != 0) == ~0ull;
        // partials that stayed in another XCD's L2 cannot be read from here
        const int reach_ok = !sk_xcd_local || __ballot(same_xcd != 0) == ~0ull;
        if (threadIdx.x == 0) {
          if (!(all_ok && slot_ok && reach_ok) && p.status != nullptr) {
            if (atomicCAS(p.status, 0, all_ok && slot_ok ? TDIST_ERR_DEVICE : TDIST_ERR_TIMEOUT) == 0) p.status[1] = -1 - wg_pos;
          }
          *s_gate = all_ok && slot_ok && reach_ok;
        }
      }
      __syncthreads();
      const int pieces_ok = *s_gate;
      __syncthreads();
      if (!pieces_ok) continue;
      // acquire: pieces from this XCD are in its L2 once their flags are up, so dropping this compute unit's own
      // first-level lines is all it takes (a device-scope acquire would also sweep the whole L2, once per wave)
      if (sk_xcd_local) asm volatile("buffer_inv sc0" ::: "memory");
      else __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");

      // (4) this workgroup's share of the sum: float4 groups [q0, q0 + nq) of every lane, over the sk_s slots in slot
      // order, packed into the staging rows as the plain epilogue packs them
      const int nq = kQuads / sk_s, q0 = sk_j * nq;
      const TDIST_AS1 unsigned char* const part0 =
          (const TDIST_AS1 unsigned char*)(p.sk_partials + (int64_t)w0 * (BM * BN)) + sk_voff;
      auto reduce_share = [&](auto s_c) {
        constexpr int kS = decltype(s_c)::value;
        constexpr int kBatch = 16 / kS < kQuads / kS ? 16 / kS : kQuads / kS;  // float4 groups per round of loads
        for (int qb = 0; qb < nq; qb += kBatch) {
          float4v t[kBatch][kS];
#pragma unroll
          for (int u = 0; u < kBatch; ++u)
#pragma unroll
            for (int i = 0; i < kS; ++i)
              t[u][i] = *(const TDIST_AS1 float4v*)(part0 + (size_t)i * (BM * BN * 4) + (size_t)(q0 + qb + u) * (kThreads * 16));
#pragma unroll
          for (int u = 0; u < kBatch; ++u) {
            float4v v = t[u][0];
#pragma unroll
            for (int i = 1; i < kS; ++i) v += t[u][i];
            const int r = q0 + qb + u;
            const int ib = r / kGroups, g = r % kGroups;
            float rsi = 1.f;
            float4v csg = {1.f, 1.f, 1.f, 1.f};
            if constexpr (kScales) {
              if (p.row_scale) rsi = p.row_scale[min(m0 + wm * C::kWaveM + 32 * ib + group_row(g), p.M - 1)];
              if (p.col_scale) {
                const int gn = n0 + wn * C::kWaveN + group_col(g);
                for (int e = 0; e < 4; ++e) csg[e] = p.col_scale[min(gn + e, p.N - 1)];
              }
            }
            stage_vals(v, rsi, csg, stage_addr(ib, g));
          }
        }
      };
      if (sk_s == 2) reduce_share(std::integral_constant<int, 2>{});
      else if (sk_s == 4) reduce_share(std::integral_constant<int, 4>{});
      else reduce_share(std::integral_constant<int, 8>{});
      // the slots have been read: acknowledge to their writers
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();

      if ((int)threadIdx.x < sk_s) __hip_atomic_fetch_add(sk_acks + w0 + threadIdx.x, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      // (5) the staged share → C. It is whole 32-row blocks of the wave tile, or a column range of one block:
      // float4 groups [g0, g0 + n) of a row block are its 16-byte pieces [g0, g0 + n).
      {
        const int ib0 = q0 / kGroups;
        const int n_rows = nq >= kGroups ? 32 * (nq / kGroups) : 32;
        const int p0 = nq >= kGroups ? 0 : q0 % kGroups;
        const int np = nq >= kGroups ? kGroups : nq;          // pieces per row: a power of two, 2 .. 16
        const int rows_per_pass = 64 / np;
        const int s_er = e_lane / np, s_ec = p0 + e_lane % np;
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_wave_barrier();
        for (int row = 0; row < n_rows; row += rows_per_pass) {
          const int mrow = 32 * ib0 + row + s_er;
          store_piece_at(mrow, s_ec, staged_piece_at(mrow, s_ec));
        }
      }

      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      continue;
    }

    // A tile that lies inside C with 16-byte-aligned rows. Row block by row block, software-pipelined: the staged rows
    // of block i are read back (LDS serves one wave's instructions in order, so the reads see the writes before them
    // without a wait), block i+1 is packed while those reads are in flight, then block i is stored, with one address
    // per lane for the whole tile (uniform base + constant row step) and no per-store bounds arithmetic. The scales
    // of the whole wave tile are fetched up front, in one round trip.
    bool stored = false;
    if constexpr (C::kWaves <= 4 && !kGrouped && kFullRows) {
      if (m0 + BM <= p.M && n0 + BN <= p.N && n_vec_ok) {
        stored = true;
        constexpr int kPasses = 32 / kRowsPerPass;
        static_assert(2 * kPasses == kGroups, "one read or store per column group of a row block");
        const int64_t row_bytes = p.ldc * 2;
        unsigned char* const tile_dst = Cbase + ((crow0 + wm * C::kWaveM) * p.ldc + n0 + wn * C::kWaveN) * 2;
        const uint32_t lane_off = (uint32_t)er * (uint32_t)row_bytes + (uint32_t)ec * 16u;
        const bool streaming = p.scatter_bufs == nullptr;
        const bool blocks_in_turn = kEarly && early;   // two staging blocks per wave instead of one per row block
        float rs[kScales ? C::kTM : 1] = {1.f};
        // (the two groups of a 16-column block share their column scales)
        constexpr int kColSlots = kWide ? kGroups : kGroups / 2;
        float4v cs[kScales ? kColSlots : 1] = {float4v{1.f, 1.f, 1.f, 1.f}};
        if constexpr (kScales) {
#pragma unroll
          for (int i = 0; i < C::kTM; ++i) {
            rs[i] = 1.f;
            if (p.row_scale) rs[i] = p.row_scale[m0 + wm * C::kWaveM + E::kRows * i + e_lrow];
          }
#pragma unroll
          for (int c = 0; c < kColSlots; ++c) {  // the four column scales of each of this lane's column groups
            cs[c] = float4v{1.f, 1.f, 1.f, 1.f};
            if (p.col_scale) cs[c] = *(const float4v*)(p.col_scale + n0 + wn * C::kWaveN + group_col(kWide ? c : 2 * c));
          }
        }
        // Staging addresses: a row block adds a constant to them (32 rows leave the swizzle term alone), so one
        // address per column group and one per swizzle phase of the read-back serve the whole tile, with the row
        // block in the instruction's offset field.
        constexpr int kReadPhases = (C::kEpiSwz + 1) / kRowsPerPass > 1 ? (C::kEpiSwz + 1) / kRowsPerPass : 1;
        static_assert(kPasses % kReadPhases == 0 && (C::kEpiSwz + 1) <= 32, "swizzle period within a row block");
        lds_u8 wbase[kGroups], rbase[kReadPhases];
#pragma unroll
        for (int g = 0; g < kGroups; ++g) wbase[g] = stage_addr(0, g);
#pragma unroll
        for (int ph = 0; ph < kReadPhases; ++ph)
          rbase[ph] = epi + er * C::kEpiPitch + ((ec ^ ((ph * kRowsPerPass + er) & C::kEpiSwz)) << 4);
        auto stage_fast = [&](auto i_c, auto g_c) {
          constexpr int i = decltype(i_c)::value, g = decltype(g_c)::value;
          stage_vals(acc4(i_c, g_c), kScales ? rs[scale_slot(i, g)] : 1.f, cs[kScales ? (kWide ? g : g / 2) : 0],
                     wbase[g] + (blocks_in_turn ? i % 2 : i) * 32 * C::kEpiPitch);
        };
        static_for<kGroups>([&](auto g_c) { stage_fast(std::integral_constant<int, 0>{}, g_c); });
        __builtin_amdgcn_sched_barrier(0);
        arr_issue(kRowBlocks * kPasses);
        __builtin_amdgcn_sched_barrier(0);
        int4v v[kPasses];
        auto read_piece = [&](int i, int u) {
          v[u] = *(const TDIST_AS3 int4v*)(rbase[u % kReadPhases] + (32 * (blocks_in_turn ? i % 2 : i) + u * kRowsPerPass) * C::kEpiPitch);
        };
        auto store_fast = [&](int i, int u) {
          TDIST_AS1 int4v* dst = (TDIST_AS1 int4v*)(tile_dst + (int64_t)(32 * i + u * kRowsPerPass) * row_bytes + lane_off);
          if (streaming) __builtin_nontemporal_store(v[u], dst);
          else *dst = v[u];
        };
        // One LDS read or one store behind every column group of the next block's packing, so that the three pipes
        // (vector ALU, LDS, vector memory) work at the same time. A wave issues in order and the four waves share one
        // path to memory, so a burst of stores would hold each wave for the whole burst: spread out, a store costs
        // its wave one issue. Piece u of block i is read behind group 2u and stored kLag reads later; the last
        // kLag stores of a block go behind the first groups of the next one.
        constexpr int kLag = 2;
        static_assert(kPasses >= 2 * kLag, "the store of a piece follows its read by kLag reads");
        static_for<kRowBlocks - 1>([&](auto i_c) {
          constexpr int i = decltype(i_c)::value;
          __builtin_amdgcn_wave_barrier();
          static_for<kGroups>([&](auto g_c) {
            constexpr int g = decltype(g_c)::value;
            stage_fast(std::integral_constant<int, i + 1>{}, g_c);
            if constexpr (g % 2 == 0) {
              read_piece(i, g / 2);
            } else {
              constexpr int u = (g - 1) / 2 - kLag;
              if constexpr (u >= 0) store_fast(i, u);
              else if constexpr (i > 0) store_fast(i - 1, u + kPasses);
            }
            __builtin_amdgcn_sched_barrier(0);
          });
        });
        {
          constexpr int i = kRowBlocks - 1;  // nothing left to pack behind the last block
          __builtin_amdgcn_wave_barrier();
#pragma unroll
          for (int u = 0; u < kPasses - kLag; ++u) read_piece(i, u);
          if (i > 0) {
#pragma unroll
            for (int u = kPasses - kLag; u < kPasses; ++u) store_fast(i - 1, u);
          }
#pragma unroll
          for (int u = kPasses - kLag; u < kPasses; ++u) read_piece(i, u);
#pragma unroll
          for (int u = 0; u < kPasses; ++u) store_fast(i, u);
        }
      }
    }
    if (stored) {
    } else if constexpr (!kScales && kFixedAcc) {
      // row block by row block: the stores of block i drain while block i+1 is being packed
      static_for<kRowBlocks>([&](auto i_c) {
        constexpr int i = decltype(i_c)::value;
        static_for<kGroups / 4>([&](auto j_c) { stage_block(i_c, j_c, nullptr, nullptr); });
        __builtin_amdgcn_wave_barrier();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        store_rows(32 * i, 32);
      });
    } else {
      float rs[C::kTM];
#pragma unroll
      for (int i = 0; i < C::kTM; ++i) {
        rs[i] = 1.f;
        if (kScales && p.row_scale) rs[i] = p.row_scale[min(m0 + wm * C::kWaveM + E::kRows * i + e_lrow, p.M - 1)];
      }
      static_for<kGroups / 4>([&](auto j_c) {
        constexpr int j = decltype(j_c)::value;
        // the four column scales of each of this lane's four column groups in this 32-column block
        float4v cs[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          cs[q] = float4v{1.f, 1.f, 1.f, 1.f};
          if (kScales && p.col_scale) {
            const int gn = n0 + wn * C::kWaveN + group_col(4 * j + q);
            if (gn + 3 < p.N) cs[q] = *(const float4v*)(p.col_scale + gn);
            else
              for (int e = 0; e < 4; ++e) cs[q][e] = p.col_scale[min(gn + e, p.N - 1)];
          }
        }
        static_for<kRowBlocks>([&](auto i_c) { stage_block(i_c, j_c, rs, cs); });
      });
      __builtin_amdgcn_wave_barrier();
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      store_rows(0, C::kWaveM);
    }
    arr_issue(0);   // (the epilogue forms that did not issue the look themselves)
    if (arrival) {
      // the next tile, by the look taken while the epilogue ran (wave 0 is done reading its staging rows, which is
      // where the gate words lie)
      if (wave == 0) {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if constexpr (kFixedAcc) {
          constexpr int kBehind = kRowBlocks * (32 / kRowsPerPass);   // the fast epilogue's stores per wave
          static_assert(kBehind > 0 && kBehind < 60, "vmcnt is a 6-bit counter");
          if (arr_behind != 0) {
            asm volatile("s_waitcnt vmcnt(%1)\n\tv_accvgpr_read_b32 %0, a0" : "=v"(arr_flag) : "n"(kBehind) : "memory");
          } else {
            asm volatile("s_waitcnt vmcnt(0)\n\tv_accvgpr_read_b32 %0, a0" : "=v"(arr_flag) : : "memory");
          }
        }
        const int next = arr_next(arr_flag);
        if (lane == 0) s_gate[0] = next;
      }
      arr_decided = true;
    }
    // the next tile's prologue overwrites the ring: every wave must be done reading its staging area
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    if constexpr (kEarly) prefetched = early;
  }
  // ---- the last workgroup out advances the workspace's tag base for the next launch --------------------------
  if (p.sk_mode != 0 && threadIdx.x == 0) {
    int32_t* const done = p.sk_ctrl + kSkCtrlDone;
    if (__hip_atomic_fetch_add(done, 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT) == G - 1) {
      __hip_atomic_store(done, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      int next = tag_base + kSkTagStride;
      if (next > kSkTagWrap) {
        // tags start over: no word may still hold a value that a tag will take again
        next = 0;
        for (int i = 0; i < kSkMaxWorkgroups; ++i) __hip_atomic_store(sk_flags + i, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      __hip_atomic_store(p.sk_ctrl + kSkCtrlEpoch, next, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

// ---- host side ------------------------------------------------------------------------------------
enum GemmElem { kElemBF16, kElemF16, kElemFP8 };

struct GemmCall {
  const void* A;
  int64_t lda;
  const void* A_local;
  int64_t lda_local;
  int local_row_begin, local_rows;
  const void* B;
  int64_t ldb;
  void* C;
  void* const* scatter_bufs;
  int64_t ldc;
  int M, N, K;
  const float* row_scale;
  const float* col_scale;
  const int32_t* flags;
  int m_per_chunk, wait_value;
  const int32_t* chunk_order;
  int rank, world_size, spin_limit;
  int32_t* status;
  int max_workgroups;
  void* sk_workspace;
  int64_t sk_workspace_bytes;
  hipStream_t stream;
  const char* who;
};

template <typename E, int BM, int BN, int KB, int WM, int WN, int NST, bool kScales, bool kGrouped = false, bool kPlain = false>
static int launch_gemm_cfg(const GemmParams& prm, int grid, hipStream_t stream, const char* who) {
  typedef GemmCfg<E, BM, BN, KB, WM, WN, NST> C;
  auto kern = gemm_kernel<E, BM, BN, KB, WM, WN, NST, kScales, kGrouped, kPlain>;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, C::kLdsBytes);
    if (e != hipSuccess) return fail(TDIST_ERR_LAUNCH, "%s: cannot reserve %d B of LDS: %s", who, C::kLdsBytes, hipGetErrorString(e));
    attr_set = true;
  }
  hipLaunchKernelGGL(kern, dim3(grid), dim3(C::kThreads), C::kLdsBytes, stream, prm);
  return launch_status(who);
}

// ---- split-K workspace (the caller's, per call) ------------------------------------------------------------
// [0, kSkHeaderBytes): control words (epoch, done counter), one flag and one acknowledgement word per workgroup; then
// one fp32 tile per workgroup. The memory must be zero when it is first used; the kernels keep it consistent from then
// on (tags, never cleared flags).

// 0 = off, 1 = on wherever the workspace allows, -1 = by the cost estimate
static int sk_env() {
  const int v = debug_get(TDIST_DEBUG_GEMM_SPLIT_K);
  return v < 0 ? -1 : (v != 0 ? 1 : 0);
}

static bool sk_workspace_fits(const void* ws, int64_t bytes, int workgroups, int bm, int bn) {
  return ws != nullptr && workgroups <= kSkMaxWorkgroups && bytes >= kSkHeaderBytes + (int64_t)workgroups * bm * bn * 4;
}

// a workspace that is handed in must be usable at least for the smallest tile
static int sk_workspace_check(const void* ws, int64_t bytes, const char* who) {
  if (ws == nullptr) return TDIST_OK;
  if ((reinterpret_cast<uintptr_t>(ws) & 255u) != 0 || bytes < kSkHeaderBytes + 128 * 128 * 4)
    return fail(TDIST_ERR_WORKSPACE, "%s: sk_workspace of %lld bytes at %p (256-byte aligned, at least %lld bytes; see "
                "tdist_gemm_split_k_workspace_bytes)", who, (long long)bytes, ws, (long long)(kSkHeaderBytes + 128 * 128 * 4));
  return TDIST_OK;
}

static void sk_attach(GemmParams& p, void* ws, int mode) {
  p.sk_ctrl = (int32_t*)ws;
  p.sk_partials = (float*)((unsigned char*)ws + kSkHeaderBytes);
  p.sk_mode = mode;
  p.sk_l2_local = device_info().xcd_round_robin == 1 && debug_get(TDIST_DEBUG_GEMM_SK_COHERENT) != 1;
}

// cost of handing a tile's pieces through the workspace, in K tiles of that tile's work (one compute unit writes the
// tile's fp32 accumulators and reads as much back)
static double sk_handover_k_tiles(int bm, int bn) { return 2.0 + 6.0 * bm * bn / 65536.0; }

static int run_gemm(const GemmCall& c, GemmElem elem) {
  const char* who = c.who;
  const int esz = elem == kElemFP8 ? 1 : 2;
  if (!c.A || !c.B || (!c.C && !c.scatter_bufs)) return fail(TDIST_ERR_INVALID, "%s: null pointer", who);
  if (c.M <= 0 || c.N <= 0 || c.K <= 0) return fail(TDIST_ERR_INVALID, "%s: M, N, K must be positive", who);
  if (((int64_t)c.K * esz) % 16 != 0)
    return fail(TDIST_ERR_UNSUPPORTED, "%s: K*elem_size = %lld must be a multiple of 16 bytes", who, (long long)c.K * esz);
  if (!aligned16(c.A) || !aligned16(c.B) || (c.A_local && !aligned16(c.A_local)) || (c.lda * esz) % 16 ||
      (c.ldb * esz) % 16 || (c.A_local && (c.lda_local * esz) % 16))
    return fail(TDIST_ERR_UNSUPPORTED, "%s: A/B bases and row strides must be 16-byte aligned", who);
  // a K that ends inside a 64-byte K tile: the 128 x 128 tile fetches zeros for the rest of its last K tile
  const int k_tail_bytes = (int)(((int64_t)c.K * esz) % 64);
  // chunks that are not whole 128-row tiles: tiles are walked in row order from the own rank's rows on, and each
  // waits for every flag its rows touch
  const bool ragged = !c.scatter_bufs && c.flags && c.m_per_chunk > 0 && c.m_per_chunk % 128 != 0;
  if (ragged && c.chunk_order)
    return fail(TDIST_ERR_UNSUPPORTED, "%s: chunk_order needs m_per_chunk (%d) to be a multiple of 128 rows", who, c.m_per_chunk);
  if (c.lda < c.K || c.ldb < c.K || c.ldc < c.N) return fail(TDIST_ERR_INVALID, "%s: leading dimension smaller than row", who);
  if (c.lda * esz > (1 << 22) || c.ldb * esz > (1 << 22) || (c.A_local && c.lda_local * esz > (1 << 22)))
    return fail(TDIST_ERR_UNSUPPORTED, "%s: row strides above 4 MiB are not supported", who);
  if (int rc = sk_workspace_check(c.sk_workspace, c.sk_workspace_bytes, who)) return rc;
  const DeviceInfo& di = device_info();
  if (di.ok != 1) return fail(TDIST_ERR_DEVICE, "%s: current device is not gfx950", who);

  // Tile configuration. The 256-row tiles (256x256 and 256x128, both on the split ring) need the call's row blocks
  // (chunks, rank slices, the local shard) to be multiples of 256 rows and K to be a multiple of 128 bytes; the
  // 128x256 and 128x192 tiles (split ring as well, waves of 64 x 128 and 64 x 96: for row blocks of 128·odd rows, and
  // three quarters of a 256x128 tile's work for shapes whose larger tiles would leave a quarter of the chip without
  // one) need whole 128-byte K tiles; the 128x128 tile takes everything else. Among the admissible ones the cheapest estimate wins: rounds of the grid times the tile's work
  // over its measured relative efficiency.
  bool rows256 = true;
  if (c.scatter_bufs && c.world_size > 0 && (c.M % c.world_size != 0 || (c.M / c.world_size) % 256 != 0)) rows256 = false;
  if (!c.scatter_bufs && c.flags && c.m_per_chunk % 256 != 0) rows256 = false;
  if (k_tail_bytes != 0) rows256 = false;
  if (c.A_local && (c.local_row_begin % 256 != 0 || c.local_rows % 256 != 0)) rows256 = false;
  if (((int64_t)c.K * esz) % 128 != 0) rows256 = false;  // the split ring steps through K 128 bytes at a time
  int cap_wgs = di.num_cus;
  if (c.max_workgroups > 0 && c.max_workgroups < cap_wgs) cap_wgs = c.max_workgroups;
  struct TileChoice { int bm, bn; double eff; };
  constexpr int kNumChoices = 5;
  // (rates relative to the 256x256 tile, measured on 8192 x 6144 x 3584 bf16: 1425, 1255, 774, 1078 and 1178
  // TFLOP/s; the 128x192 tile is entered below its multi-round rate because a tile's prologue and epilogue weigh
  // more the smaller it is: one round of 256 of them takes 50.5 us on 4096 x 1536 x 4096 where 192 tiles of 256x128
  // take 48.3 and 192 tiles of 128x256 53.1)
  static const TileChoice kChoices[kNumChoices] = {{256, 256, 1.0}, {256, 128, 0.88}, {128, 128, 0.54}, {128, 192, 0.65}, {128, 256, 0.8}};
  const bool k128 = ((int64_t)c.K * esz) % 128 == 0;
  auto admissible = [&](int t) { return kChoices[t].bm == 256 ? rows256 : (kChoices[t].bn == 128 || k128); };
  auto k_tile_bytes = [&](int t) { return kChoices[t].bm == 256 || kChoices[t].bn != 128 ? 128 : 64; };
  // With a workspace, a last round that fills at most half of the grid is split along K (see GemmParams): it then
  // costs 1/s of a round plus one exchange of the tile's accumulators, and that form is taken where it beats whole
  // tiles by a margin.
  const int sk_mode = sk_env();
  int pick = 2;
  bool use_sk = false;
  double best = 0;
  for (int t = 0; t < kNumChoices; ++t) {
    if (!admissible(t)) continue;
    const int bm = kChoices[t].bm, bn = kChoices[t].bn;
    const int64_t tiles = ceil_div(c.M, bm) * ceil_div(c.N, bn);
    const int64_t kt = ceil_div((int64_t)c.K * esz, k_tile_bytes(t));
    const double per_k_tile = (double)bm * bn / kChoices[t].eff;
    const double cost = (double)ceil_div(tiles, cap_wgs) * kt * per_k_tile;
    if (best == 0 || cost < best) best = cost, pick = t, use_sk = false;
    const int64_t tail = tiles % cap_wgs;
    const int split = tail > 0 ? sk_split_for(cap_wgs, (int)tail, (int)(kt < 0x7fffffff ? kt : 0x7fffffff)) : 1;
    // (the exchange of the split form is written for staged rows of a power-of-two width: not for the 128x192 tile)
    if (sk_mode != 0 && split >= 2 && bn != 192 && sk_workspace_fits(c.sk_workspace, c.sk_workspace_bytes, cap_wgs, bm, bn)) {
      const double cost_sk = ((double)(tiles / cap_wgs) * kt + (double)kt / split + sk_handover_k_tiles(bm, bn)) * per_k_tile;
      if (cost_sk < 0.95 * best || (sk_mode == 1 && (!use_sk || cost_sk < best))) best = cost_sk, pick = t, use_sk = true;
    }
  }
  // TDIST_DEBUG_GEMM_TILE forces a tile (test and measurement aid): 0 = 256x256, 1 = 256x128, 2 = 128x128, 3 = 128x192,
  // 4 = 128x256; a tile that the call's row blocks or K do not admit is not taken.
  {
    const int t = debug_get(TDIST_DEBUG_GEMM_TILE);
    if (t >= 0 && t < kNumChoices && admissible(t)) {
      pick = t;
      // (the split is re-derived for the forced tile)
      const int64_t tiles = ceil_div(c.M, kChoices[t].bm) * ceil_div(c.N, kChoices[t].bn);
      const int64_t kt = ceil_div((int64_t)c.K * esz, k_tile_bytes(t));
      const int64_t tail = tiles % cap_wgs;
      use_sk = sk_mode != 0 && use_sk && kChoices[t].bn != 192 && tail > 0 && sk_split_for(cap_wgs, (int)tail, (int)kt) >= 2 &&
               sk_workspace_fits(c.sk_workspace, c.sk_workspace_bytes, cap_wgs, kChoices[t].bm, kChoices[t].bn);
    }
  }
  const int BM = kChoices[pick].bm;
  const int BN = kChoices[pick].bn;
  // An XCD's workgroups (one in num_xcds of the grid) work on a block of rows x cols tiles at a time and fetch the
  // operand rows of rows + cols panels for it: the bytes of such a block per tile, a little more where a side does not
  // divide the tile count (the blocks then wrap around the matrix's edge and their panels are shared by fewer tiles);
  // 0 if the XCD's workgroups do not make whole rows.
  auto xcd_block_cost = [&](int rows) -> double {
    const int per_xcd = di.num_xcds > 0 && cap_wgs % di.num_xcds == 0 ? cap_wgs / di.num_xcds : cap_wgs;
    if (rows <= 0 || per_xcd % rows != 0) return 0;
    const int cols = per_xcd / rows;
    const int tiles_m = (int)ceil_div(c.M, BM), tiles_n = (int)ceil_div(c.N, BN);
    return ((double)rows * BM + (double)cols * BN) * (1.0 + (tiles_n % cols != 0 ? 0.125 : 0.0) + (tiles_m % rows != 0 ? 0.125 : 0.0));
  };

  GemmParams p;
  p.A = (const unsigned char*)c.A;
  p.A_local = (const unsigned char*)c.A_local;
  p.B = (const unsigned char*)c.B;
  p.C = (unsigned char*)c.C;
  p.scatter_bufs = c.scatter_bufs;
  p.row_scale = c.row_scale;
  p.col_scale = c.col_scale;
  p.flags = c.flags;
  p.chunk_order = c.chunk_order;
  p.status = c.status;
  p.lda_b = c.lda * esz;
  p.lda_local_b = c.lda_local * esz;
  p.ldb_b = c.ldb * esz;
  p.ldc = c.ldc;
  p.M = c.M;
  p.N = c.N;
  p.K = c.K;
  p.local_row_begin = c.A_local ? c.local_row_begin : 0;
  p.local_rows = c.A_local ? c.local_rows : 0;
  p.wait_value = c.wait_value;
  p.rank = c.rank;
  p.world_size = c.world_size;
  p.spin_limit = c.spin_limit > 0 ? c.spin_limit : (1 << 22);  // ~seconds of polling
  p.num_xcds = di.num_xcds;
  p.m_per_rank = 0;
  p.chunks_per_rank = 1;
  p.sorted_ids = p.block_expert = p.block_segment = p.post_pad = nullptr;
  p.b_expert_stride_b = 0;
  p.num_valid = p.topk = p.first_block = p.a_rows = 0;
  p.sk_ctrl = nullptr;
  p.sk_partials = nullptr;
  p.sk_mode = 0;
  p.sk_l2_local = 0;
  p.sched_rounds = 0; p.sched_tpc_magic = 0; p.sched_ws_magic = 0;
  p.group_s = 1; p.group_rows_shift = 0; p.cm_shift = 0;
  p.k_tail_bytes = k_tail_bytes;

  if (c.scatter_bufs) {
    if (c.world_size <= 0 || c.rank < 0 || c.rank >= c.world_size)
      return fail(TDIST_ERR_INVALID, "%s: rank %d / world_size %d", who, c.rank, c.world_size);
    if (c.M % c.world_size != 0 || (c.M / c.world_size) % BM != 0)
      return fail(TDIST_ERR_UNSUPPORTED, "%s: M/world_size = %d must be a multiple of the %d-row tile", who,
                  c.M / c.world_size, BM);
    p.m_per_rank = c.M / c.world_size;
    p.m_per_chunk = p.m_per_rank;
    p.n_chunks = c.world_size;
    p.order_mode = 2;
    p.flags = nullptr;
  } else if (ragged) {
    if (c.A_local && (c.local_row_begin % BM != 0 || c.local_rows % BM != 0))
      return fail(TDIST_ERR_UNSUPPORTED, "%s: with m_per_chunk %d (not a multiple of %d rows) the local shard must start and end "
                  "on a %d-row tile, or be copied into A with its flag set", who, c.m_per_chunk, BM, BM);
    p.m_per_chunk = BM;
    p.n_chunks = (int)ceil_div(c.M, BM);
    p.order_mode = 0;
    if (c.world_size > 1 && c.rank >= 0 && c.rank < c.world_size) {
      // start with the first tile that lies inside the own rank's rows
      p.order_mode = 4;
      p.first_block = (int)(ceil_div((int64_t)c.rank * c.M / c.world_size, BM) % p.n_chunks);
    }
  } else if (c.flags) {
    if (c.m_per_chunk <= 0 || c.m_per_chunk % BM != 0)
      return fail(TDIST_ERR_UNSUPPORTED, "%s: m_per_chunk %d must be a positive multiple of the %d-row tile", who,
                  c.m_per_chunk, BM);
    p.m_per_chunk = c.m_per_chunk;
    p.n_chunks = (int)ceil_div(c.M, c.m_per_chunk);
    if (c.A_local && (c.local_row_begin % BM != 0 || c.local_rows % BM != 0))
      return fail(TDIST_ERR_UNSUPPORTED, "%s: the local shard must start and end on a %d-row tile", who, BM);
    if (c.chunk_order) {
      p.order_mode = 3;
    } else if (c.world_size > 1 && c.M % c.world_size == 0 && (c.M / c.world_size) % c.m_per_chunk == 0 &&
               c.rank >= 0 && c.rank < c.world_size) {
      p.order_mode = 1;
      p.chunks_per_rank = (c.M / c.world_size) / c.m_per_chunk;
    } else {
      p.order_mode = 0;
    }
    // chunks of 1, 2 or 4 row tiles: scheduled several at a time, so that an XCD's block of tiles is 8 (or 4) rows
    // high (see GemmParams::group_s); the chunks of a group are neighbours in the expected order of arrival
    const int cmh = c.m_per_chunk / BM;
    if (cmh == 1 || cmh == 2 || cmh == 4) {
      int gs = 1;
      double best = 0;
      for (int cand = 1; cand * cmh <= 16; cand *= 2) {
        if (p.n_chunks % cand != 0 || (cand > 1 && p.order_mode == 1 && c.world_size % cand != 0)) continue;
        const double cost = xcd_block_cost(cand * cmh);
        if (cost > 0 && (best == 0 || cost < best)) {
          best = cost;
          gs = cand;
        }
      }
      if (gs > 1) {
        auto log2i = [](int v) { int n = 0; while ((1 << n) < v) ++n; return n; };
        p.group_s = gs;
        p.cm_shift = log2i(cmh);
        p.group_rows_shift = log2i(gs * cmh);
      }
    }
  } else {
    // ungated GEMM: scheduled in groups of row tiles, of the size that gives an XCD's block of tiles its best shape
    // (16384 x 7168 x 8192 e4m3, 28 column tiles, constant operands: 472 us in blocks of 4 x 8, 455 in blocks of 8 x 4)
    int rows_per_group = 4;
    {
      double best = 0;
      for (int rows : {4, 8, 2, 16}) {
        const double cost = xcd_block_cost(rows);
        if (cost > 0 && (best == 0 || cost < best)) {
          best = cost;
          rows_per_group = rows;
        }
      }
    }
    p.m_per_chunk = BM * rows_per_group;
    p.n_chunks = (int)ceil_div(c.M, p.m_per_chunk);
    p.order_mode = 0;
    if (c.A_local && (c.local_row_begin % BM != 0 || c.local_rows % BM != 0))
      return fail(TDIST_ERR_UNSUPPORTED, "%s: the local shard must start and end on a %d-row tile", who, BM);
  }
  p.gate_rows = ragged ? c.m_per_chunk : p.m_per_chunk;
  const int64_t sched = (int64_t)p.n_chunks * (p.m_per_chunk / BM) * ceil_div(c.N, BN);
  if (sched > 0x7fffffff) return fail(TDIST_ERR_UNSUPPORTED, "%s: too many tiles", who);
  int grid = (int)(sched < cap_wgs ? sched : cap_wgs);
  if (use_sk) {
    grid = cap_wgs;
    sk_attach(p, c.sk_workspace, 1);
  } else if (c.flags && !c.scatter_bufs && !ragged && p.n_chunks <= kSchedMaxChunks && sched > grid &&
             sched <= (int64_t)kSchedMaxRounds * grid && debug_get(TDIST_DEBUG_GEMM_SCHEDULE) != 0) {
    // gated, whole-tile chunks, 2 .. 64 rounds of tiles: every workgroup takes its tiles in arrival order (a single
    // round is static either way: every workgroup owns its one tile)
    const int64_t tpc = (int64_t)p.group_s * (p.m_per_chunk / BM) * ceil_div(c.N, BN);   // tiles of a group of chunks
    if (sched * tpc < 0x7fffffffll && sched < (1 << 25)) {
      p.sched_rounds = (int)ceil_div(sched, grid);
      p.sched_tpc_magic = (uint32_t)(((1ull << 32) + tpc - 1) / tpc);
      const int64_t wsz = c.world_size > 0 ? c.world_size : 1;
      p.sched_ws_magic = (uint32_t)(((1ull << 32) + wsz - 1) / wsz);   // (positions of chunks: at most 64)
    }
  }
  const bool scales = elem == kElemFP8 && (c.row_scale || c.col_scale);

  // 256-row tiles: 2 x 2 waves on the split ring (3 A stages + 2 B stages), 16-row MFMA blocks
  if (BM == 256 && BN == 256 && p.flags == nullptr && p.A_local == nullptr) {
    // no flags, no local shard: the instances without gating code (the GEMM-RS producer's, the headline shape's)
    switch (elem) {
      case kElemBF16: return launch_gemm_cfg<ElemBF16N, 256, 256, 128, 2, 2, 5, false, false, true>(p, grid, c.stream, who);
      case kElemF16: return launch_gemm_cfg<ElemF16N, 256, 256, 128, 2, 2, 5, false, false, true>(p, grid, c.stream, who);
      default:
        return scales ? launch_gemm_cfg<ElemFP8N, 256, 256, 128, 2, 2, 5, true, false, true>(p, grid, c.stream, who)
                      : launch_gemm_cfg<ElemFP8N, 256, 256, 128, 2, 2, 5, false, false, true>(p, grid, c.stream, who);
    }
  }
  if (BM == 256 && BN == 256) {
    switch (elem) {
      case kElemBF16: return launch_gemm_cfg<ElemBF16N, 256, 256, 128, 2, 2, 5, false>(p, grid, c.stream, who);
      case kElemF16: return launch_gemm_cfg<ElemF16N, 256, 256, 128, 2, 2, 5, false>(p, grid, c.stream, who);
      default:
        return scales ? launch_gemm_cfg<ElemFP8N, 256, 256, 128, 2, 2, 5, true>(p, grid, c.stream, who)
                      : launch_gemm_cfg<ElemFP8N, 256, 256, 128, 2, 2, 5, false>(p, grid, c.stream, who);
    }
  }
  if (BM == 256) {
    switch (elem) {
      case kElemBF16: return launch_gemm_cfg<ElemBF16N, 256, 128, 128, 2, 2, 5, false>(p, grid, c.stream, who);
      case kElemF16: return launch_gemm_cfg<ElemF16N, 256, 128, 128, 2, 2, 5, false>(p, grid, c.stream, who);
      default:
        return scales ? launch_gemm_cfg<ElemFP8N, 256, 128, 128, 2, 2, 5, true>(p, grid, c.stream, who)
                      : launch_gemm_cfg<ElemFP8N, 256, 128, 128, 2, 2, 5, false>(p, grid, c.stream, who);
    }
  }
  if (BM == 128 && BN == 256) {  // 128 x 256: waves of 64 x 128 on the split ring
    switch (elem) {
      case kElemBF16: return launch_gemm_cfg<ElemBF16N, 128, 256, 128, 2, 2, 5, false>(p, grid, c.stream, who);
      case kElemF16: return launch_gemm_cfg<ElemF16N, 128, 256, 128, 2, 2, 5, false>(p, grid, c.stream, who);
      default:
        return scales ? launch_gemm_cfg<ElemFP8N, 128, 256, 128, 2, 2, 5, true>(p, grid, c.stream, who)
                      : launch_gemm_cfg<ElemFP8N, 128, 256, 128, 2, 2, 5, false>(p, grid, c.stream, who);
    }
  }
  if (BN == 192) {  // 128 x 192: waves of 64 x 96 on the split ring
    switch (elem) {
      case kElemBF16: return launch_gemm_cfg<ElemBF16N, 128, 192, 128, 2, 2, 5, false>(p, grid, c.stream, who);
      case kElemF16: return launch_gemm_cfg<ElemF16N, 128, 192, 128, 2, 2, 5, false>(p, grid, c.stream, who);
      default:
        return scales ? launch_gemm_cfg<ElemFP8N, 128, 192, 128, 2, 2, 5, true>(p, grid, c.stream, who)
                      : launch_gemm_cfg<ElemFP8N, 128, 192, 128, 2, 2, 5, false>(p, grid, c.stream, who);
    }
  }
  // the 128 x 128 tile on a four-stage ring of 64-byte K tiles, 32-row MFMA blocks: every shape
  switch (elem) {
    case kElemBF16: return launch_gemm_cfg<ElemBF16, 128, 128, 64, 2, 2, 4, false>(p, grid, c.stream, who);
    case kElemF16: return launch_gemm_cfg<ElemF16, 128, 128, 64, 2, 2, 4, false>(p, grid, c.stream, who);
    default:
      return scales ? launch_gemm_cfg<ElemFP8, 128, 128, 64, 2, 2, 4, true>(p, grid, c.stream, who)
                    : launch_gemm_cfg<ElemFP8, 128, 128, 64, 2, 2, 4, false>(p, grid, c.stream, who);
  }
}

struct GroupGemmCall {
  const void* A;
  int64_t lda;
  const void* A_local;
  int64_t lda_local;
  int local_row_begin, local_rows;
  const void* B;
  int64_t ldb, expert_stride;
  void* C;
  int64_t ldc;
  int a_rows, N, K;
  const int32_t *sorted_ids, *expert_ids, *block_segment, *post_pad;
  int num_blocks, block_size, num_valid, topk, tokens_per_rank, first_block;
  const int32_t* flags;
  int wait_value, rank, spin_limit;
  int32_t* status;
  int max_workgroups;
  void* sk_workspace;
  int64_t sk_workspace_bytes;
  hipStream_t stream;
  const char* who;
};

static int run_group_gemm(const GroupGemmCall& c, GemmElem elem) {
  const char* who = c.who;
  const int esz = elem == kElemFP8 ? 1 : 2;
  if (!c.A || !c.B || !c.C || !c.sorted_ids || !c.expert_ids || !c.block_segment || !c.post_pad)
    return fail(TDIST_ERR_INVALID, "%s: null pointer", who);
  if (c.a_rows <= 0 || c.N <= 0 || c.K <= 0 || c.num_blocks <= 0 || c.topk <= 0 || c.num_valid < 0 || c.tokens_per_rank <= 0)
    return fail(TDIST_ERR_INVALID, "%s: sizes must be positive", who);
  if (c.block_size != 128 && c.block_size != 256)
    return fail(TDIST_ERR_UNSUPPORTED, "%s: block_size %d (the row blocks of the align / sort step must be 128 or 256 rows)", who, c.block_size);
  if (((int64_t)c.K * esz) % 64 != 0)
    return fail(TDIST_ERR_UNSUPPORTED, "%s: K*elem_size = %lld must be a multiple of 64 bytes", who, (long long)c.K * esz);
  if (!aligned16(c.A) || !aligned16(c.B) || (c.A_local && !aligned16(c.A_local)) || (c.lda * esz) % 16 || (c.ldb * esz) % 16 ||
      (c.expert_stride * esz) % 16 || (c.A_local && (c.lda_local * esz) % 16))
    return fail(TDIST_ERR_UNSUPPORTED, "%s: A/B bases and strides must be 16-byte aligned", who);
  if (c.lda < c.K || c.ldb < c.K || c.ldc < c.N) return fail(TDIST_ERR_INVALID, "%s: leading dimension smaller than row", who);
  // rows are addressed as a scalar base plus a 32-bit byte offset: the gathered A (and the own shard) must stay
  // below 4 GiB, as must one expert's B panel
  if ((int64_t)c.a_rows * c.lda * esz >= (1ll << 32) || (c.A_local && (int64_t)c.local_rows * c.lda_local * esz >= (1ll << 32)) ||
      c.ldb * esz > (1 << 22))
    return fail(TDIST_ERR_UNSUPPORTED, "%s: A above 4 GiB or B row stride above 4 MiB", who);
  if ((int64_t)c.num_blocks * c.block_size > 0x7fffffff) return fail(TDIST_ERR_UNSUPPORTED, "%s: too many rows", who);
  if (c.first_block < 0 || c.first_block >= c.num_blocks) return fail(TDIST_ERR_INVALID, "%s: first_block %d", who, c.first_block);
  if (c.A_local && (c.rank < 0 || c.local_rows <= 0)) return fail(TDIST_ERR_INVALID, "%s: local shard without rank / rows", who);
  if (int rc = sk_workspace_check(c.sk_workspace, c.sk_workspace_bytes, who)) return rc;
  const DeviceInfo& di = device_info();
  if (di.ok != 1) return fail(TDIST_ERR_DEVICE, "%s: current device is not gfx950", who);

  GemmParams p;
  p.A = (const unsigned char*)c.A;
  p.A_local = (const unsigned char*)c.A_local;
  p.B = (const unsigned char*)c.B;
  p.C = (unsigned char*)c.C;
  p.scatter_bufs = nullptr;
  p.row_scale = p.col_scale = nullptr;
  p.flags = c.flags;
  p.chunk_order = nullptr;
  p.status = c.status;
  p.lda_b = c.lda * esz;
  p.lda_local_b = c.lda_local * esz;
  p.ldb_b = c.ldb * esz;
  p.ldc = c.ldc;
  p.M = c.num_blocks * c.block_size;  // rows of the sorted space
  p.N = c.N;
  p.K = c.K;
  p.local_row_begin = c.A_local ? c.local_row_begin : 0;
  p.local_rows = c.A_local ? c.local_rows : 0;
  p.m_per_chunk = c.block_size;
  p.n_chunks = c.num_blocks;
  p.chunks_per_rank = 1;
  p.wait_value = c.wait_value;
  p.rank = c.rank;
  p.world_size = 1;
  p.order_mode = 4;
  p.spin_limit = c.spin_limit > 0 ? c.spin_limit : (1 << 22);
  p.m_per_rank = c.tokens_per_rank;
  p.num_xcds = di.num_xcds;
  p.sorted_ids = c.sorted_ids;
  p.block_expert = c.expert_ids;
  p.block_segment = c.block_segment;
  p.post_pad = c.post_pad;
  p.b_expert_stride_b = c.expert_stride * esz;
  p.num_valid = c.num_valid;
  p.topk = c.topk;
  p.first_block = c.first_block;
  p.a_rows = c.a_rows;
  p.sk_ctrl = nullptr;
  p.sk_partials = nullptr;
  p.sk_mode = 0;
  p.sk_l2_local = 0;
  p.sched_rounds = 0; p.sched_tpc_magic = 0; p.sched_ws_magic = 0;
  p.group_s = 1; p.group_rows_shift = 0; p.cm_shift = 0;
  p.gate_rows = p.m_per_chunk;
  p.k_tail_bytes = 0;

  const bool k128 = ((int64_t)c.K * esz) % 128 == 0;
  const int BN = (c.block_size == 256 || k128) ? 256 : 128;
  const int64_t sched = (int64_t)c.num_blocks * ceil_div(c.N, BN);
  if (sched > 0x7fffffff) return fail(TDIST_ERR_UNSUPPORTED, "%s: too many tiles", who);
  int cap_wgs = di.num_cus;
  if (c.max_workgroups > 0 && c.max_workgroups < cap_wgs) cap_wgs = c.max_workgroups;
  int grid = (int)(sched < cap_wgs ? sched : cap_wgs);
  // The number of row blocks in use is only known on the device and is seldom a multiple of the grid: with a
  // workspace at hand the kernel splits the last round along K whenever it fills at most half of the grid.
  {
    const int bm = c.block_size == 256 ? 256 : 128;
    const int64_t kt = (int64_t)c.K * esz / (c.block_size == 256 || k128 ? 128 : 64);
    if (sk_env() != 0 && kt >= 2 * kSkMinPiece && sk_workspace_fits(c.sk_workspace, c.sk_workspace_bytes, cap_wgs, bm, BN)) {
      grid = cap_wgs;
      sk_attach(p, c.sk_workspace, 1);
    }
  }
#define TDIST_GROUPED(EB, EH, E8, BM_, BN_, KB_, NST_)                                                          \
  switch (elem) {                                                                                               \
    case kElemBF16: return launch_gemm_cfg<EB, BM_, BN_, KB_, 2, 2, NST_, false, true>(p, grid, c.stream, who); \
    case kElemF16: return launch_gemm_cfg<EH, BM_, BN_, KB_, 2, 2, NST_, false, true>(p, grid, c.stream, who);  \
    default: return launch_gemm_cfg<E8, BM_, BN_, KB_, 2, 2, NST_, false, true>(p, grid, c.stream, who);        \
  }
  if (c.block_size == 256) {
    if (!k128) return fail(TDIST_ERR_UNSUPPORTED, "%s: 256-row blocks need K*elem_size to be a multiple of 128 bytes", who);
    TDIST_GROUPED(ElemBF16N, ElemF16N, ElemFP8N, 256, 256, 128, 5)
  }
  if (k128) {  // 64 x 128 per wave on the split ring
    TDIST_GROUPED(ElemBF16N, ElemF16N, ElemFP8N, 128, 256, 128, 5)
  }
  TDIST_GROUPED(ElemBF16, ElemF16, ElemFP8, 128, 128, 64, 4)
#undef TDIST_GROUPED
}

}  // namespace tdist

using namespace tdist;

#define TDIST_GATED_BODY(ELEM, RS, CS, WHO)                                                                         \
  GemmCall c;                                                                                                       \
  c.A = A; c.lda = lda; c.A_local = A_local; c.lda_local = lda_local;                                               \
  c.local_row_begin = local_row_begin; c.local_rows = local_rows;                                                   \
  c.B = B; c.ldb = ldb; c.C = C; c.scatter_bufs = nullptr; c.ldc = ldc; c.M = M; c.N = N; c.K = K;                  \
  c.row_scale = RS; c.col_scale = CS; c.flags = flags; c.m_per_chunk = m_per_chunk; c.wait_value = wait_value;      \
  c.chunk_order = chunk_order; c.rank = rank; c.world_size = world_size; c.spin_limit = spin_limit;                 \
  c.status = status; c.max_workgroups = max_workgroups; c.sk_workspace = sk_workspace;                              \
  c.sk_workspace_bytes = sk_workspace_bytes; c.stream = (hipStream_t)stream; c.who = WHO;                           \
  return run_gemm(c, ELEM);

extern "C" {

int64_t tdist_gemm_split_k_workspace_bytes(void) {
  const tdist::DeviceInfo& di = tdist::device_info();
  if (di.ok != 1) return 0;
  return tdist::kSkHeaderBytes + (int64_t)di.num_cus * 256 * 256 * 4;
}

int tdist_gemm_chunk_gated_bf16(const void* A, int64_t lda, const void* A_local, int64_t lda_local,
                                int local_row_begin, int local_rows, const void* B, int64_t ldb, void* C, int64_t ldc,
                                int M, int N, int K, const int32_t* flags, int m_per_chunk, int wait_value,
                                const int32_t* chunk_order, int rank, int world_size, int spin_limit, int32_t* status,
                                int max_workgroups, void* sk_workspace, int64_t sk_workspace_bytes, void* stream) {
  TDIST_GATED_BODY(kElemBF16, nullptr, nullptr, "tdist_gemm_chunk_gated_bf16")
}

int tdist_gemm_chunk_gated_f16(const void* A, int64_t lda, const void* A_local, int64_t lda_local, int local_row_begin,
                               int local_rows, const void* B, int64_t ldb, void* C, int64_t ldc, int M, int N, int K,
                               const int32_t* flags, int m_per_chunk, int wait_value, const int32_t* chunk_order,
                               int rank, int world_size, int spin_limit, int32_t* status, int max_workgroups,
                               void* sk_workspace, int64_t sk_workspace_bytes, void* stream) {
  TDIST_GATED_BODY(kElemF16, nullptr, nullptr, "tdist_gemm_chunk_gated_f16")
}

int tdist_gemm_chunk_gated_fp8e4m3(const void* A, int64_t lda, const void* A_local, int64_t lda_local,
                                   int local_row_begin, int local_rows, const void* B, int64_t ldb, void* C,
                                   int64_t ldc, int M, int N, int K, const float* row_scale, const float* col_scale,
                                   const int32_t* flags, int m_per_chunk, int wait_value, const int32_t* chunk_order,
                                   int rank, int world_size, int spin_limit, int32_t* status, int max_workgroups,
                                   void* sk_workspace, int64_t sk_workspace_bytes, void* stream) {
  TDIST_GATED_BODY(kElemFP8, row_scale, col_scale, "tdist_gemm_chunk_gated_fp8e4m3")
}

static int gemm_rs_scatter(GemmElem elem, const void* A, int64_t lda, const void* B, int64_t ldb,
                           void* const* scatter_bufs, int64_t ldc, int M, int N, int K, int rank, int world_size,
                           void* sk_workspace, int64_t sk_workspace_bytes, void* stream, const char* who,
                           const float* row_scale = nullptr, const float* col_scale = nullptr) {
  if (!scatter_bufs) return fail(TDIST_ERR_INVALID, "%s: null scatter_bufs", who);
  GemmCall c;
  c.A = A; c.lda = lda; c.A_local = nullptr; c.lda_local = 0; c.local_row_begin = 0; c.local_rows = 0;
  c.B = B; c.ldb = ldb; c.C = nullptr; c.scatter_bufs = scatter_bufs; c.ldc = ldc; c.M = M; c.N = N; c.K = K;
  c.row_scale = row_scale; c.col_scale = col_scale; c.flags = nullptr; c.m_per_chunk = 0; c.wait_value = 0;
  c.chunk_order = nullptr; c.rank = rank; c.world_size = world_size; c.spin_limit = 0; c.status = nullptr;
  c.max_workgroups = 0; c.sk_workspace = sk_workspace; c.sk_workspace_bytes = sk_workspace_bytes;
  c.stream = (hipStream_t)stream; c.who = who;
  return run_gemm(c, elem);
}

int tdist_gemm_rs_scatter_bf16(const void* A, int64_t lda, const void* B, int64_t ldb, void* const* scatter_bufs,
                               int64_t ldc, int M, int N, int K, int rank, int world_size, void* sk_workspace,
                               int64_t sk_workspace_bytes, void* stream) {
  return gemm_rs_scatter(kElemBF16, A, lda, B, ldb, scatter_bufs, ldc, M, N, K, rank, world_size, sk_workspace,
                         sk_workspace_bytes, stream, "tdist_gemm_rs_scatter_bf16");
}

int tdist_gemm_rs_scatter_f16(const void* A, int64_t lda, const void* B, int64_t ldb, void* const* scatter_bufs,
                              int64_t ldc, int M, int N, int K, int rank, int world_size, void* sk_workspace,
                              int64_t sk_workspace_bytes, void* stream) {
  return gemm_rs_scatter(kElemF16, A, lda, B, ldb, scatter_bufs, ldc, M, N, K, rank, world_size, sk_workspace,
                         sk_workspace_bytes, stream, "tdist_gemm_rs_scatter_f16");
}

int tdist_gemm_rs_scatter_fp8e4m3(const void* A, int64_t lda, const void* B, int64_t ldb, void* const* scatter_bufs,
                                  int64_t ldc, int M, int N, int K, const float* row_scale, const float* col_scale,
                                  int rank, int world_size, void* sk_workspace, int64_t sk_workspace_bytes, void* stream) {
  return gemm_rs_scatter(kElemFP8, A, lda, B, ldb, scatter_bufs, ldc, M, N, K, rank, world_size, sk_workspace,
                         sk_workspace_bytes, stream, "tdist_gemm_rs_scatter_fp8e4m3", row_scale, col_scale);
}

#define TDIST_GROUP_GEMM_BODY(ELEM, WHO)                                                                              \
  GroupGemmCall c;                                                                                                    \
  c.A = A; c.lda = lda; c.A_local = A_local; c.lda_local = lda_local; c.local_row_begin = local_row_begin;            \
  c.local_rows = local_rows; c.B = B; c.ldb = ldb; c.expert_stride = expert_stride; c.C = C; c.ldc = ldc;             \
  c.a_rows = a_rows; c.N = N; c.K = K; c.sorted_ids = sorted_token_ids; c.expert_ids = expert_ids;                    \
  c.block_segment = block_barrier_ids; c.post_pad = num_tokens_post_padded; c.num_blocks = num_blocks;                \
  c.block_size = block_size; c.num_valid = num_valid_tokens; c.topk = topk; c.tokens_per_rank = tokens_per_rank;      \
  c.first_block = first_block; c.flags = flags; c.wait_value = wait_value; c.rank = rank; c.spin_limit = spin_limit;  \
  c.status = status; c.max_workgroups = max_workgroups; c.sk_workspace = sk_workspace;                                \
  c.sk_workspace_bytes = sk_workspace_bytes; c.stream = (hipStream_t)stream; c.who = WHO;                             \
  return run_group_gemm(c, ELEM);

#define TDIST_GROUP_GEMM_ARGS                                                                                         \
  const void *A, int64_t lda, const void *A_local, int64_t lda_local, int local_row_begin, int local_rows,            \
      const void *B, int64_t ldb, int64_t expert_stride, void *C, int64_t ldc, int a_rows, int N, int K,              \
      const int32_t *sorted_token_ids, const int32_t *expert_ids, const int32_t *block_barrier_ids,                   \
      const int32_t *num_tokens_post_padded, int num_blocks, int block_size, int num_valid_tokens, int topk,          \
      int tokens_per_rank, int first_block, const int32_t *flags, int wait_value, int rank, int spin_limit,           \
      int32_t *status, int max_workgroups, void *sk_workspace, int64_t sk_workspace_bytes, void *stream

int tdist_group_gemm_gated_bf16(TDIST_GROUP_GEMM_ARGS) { TDIST_GROUP_GEMM_BODY(kElemBF16, "tdist_group_gemm_gated_bf16") }
int tdist_group_gemm_gated_f16(TDIST_GROUP_GEMM_ARGS) { TDIST_GROUP_GEMM_BODY(kElemF16, "tdist_group_gemm_gated_f16") }
int tdist_group_gemm_gated_fp8e4m3(TDIST_GROUP_GEMM_ARGS) {
  TDIST_GROUP_GEMM_BODY(kElemFP8, "tdist_group_gemm_gated_fp8e4m3")
}

}  // extern "C"
