/*
 * tdist.h — C ABI of libtdist_hip.so: hand-written gfx950 (MI355X) kernels for the per-GPU compute
 * half of Triton-distributed's overlapped ops.
 *
 * Conventions
 *   - every entry point is extern "C", returns 0 (TDIST_OK) or a negative tdist_status, never aborts;
 *     tdist_last_error_string() gives the text of the calling thread's last failure;
 *   - pointers are DEVICE pointers unless the parameter name ends in _host;
 *   - `stream` is a hipStream_t passed as void* (NULL = the legacy default stream);
 *   - no entry point allocates or frees memory; scratch comes from the caller (see *_workspace_bytes);
 *   - nothing is read from the environment; the only process-wide state is the cached device properties
 *     (tdist_init) and the test switches of tdist_debug_set, which default to "the library decides";
 *   - leading dimensions (lda, ldb, ...) are in ELEMENTS, sizes in elements unless named *_bytes;
 *   - launches are asynchronous on `stream`; a non-zero return means nothing was launched.
 *
 * Each declaration cites the reference interface (file:line under python/triton_dist of
 * Triton-distributed) whose device work it replaces.
 */
#ifndef TDIST_H_
#define TDIST_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum tdist_status {
  TDIST_OK = 0,
  TDIST_ERR_INVALID = -1,     /* bad argument (null pointer, misaligned, non-positive size) */
  TDIST_ERR_UNSUPPORTED = -2, /* shape / dtype outside what the kernels implement */
  TDIST_ERR_LAUNCH = -3,      /* HIP reported an error at launch */
  TDIST_ERR_TIMEOUT = -4,     /* a bounded flag wait expired (reported through a status word) */
  TDIST_ERR_WORKSPACE = -5,   /* caller's scratch buffer is too small */
  TDIST_ERR_DEVICE = -6       /* not a gfx950 device / no device */
} tdist_status;

typedef enum tdist_dtype {
  TDIST_BF16 = 0,
  TDIST_F16 = 1,
  TDIST_F8E4M3 = 2, /* OCP e4m3fn, the gfx950 hardware format */
  TDIST_F32 = 3
} tdist_dtype;

/* ---------------------------------------------------------------------------------------------
 * Library
 * ------------------------------------------------------------------------------------------- */
int tdist_version(void);
const char* tdist_last_error_string(void);
/* Caches properties of the current device (CU count, XCD count) and the device address of the library's built-in
 * scratch (tdist_moe_scatter_index_static), and checks once, with a small grid whose workgroups read their XCD id from
 * the hardware (one launch on the NULL stream and a synchronous 4 KiB copy back; no allocation), that workgroup i
 * of a grid runs on XCD i mod 8. Optional: every entry point does the first two lazily. Without the call, or when the
 * check does not hold (another partition mode, a CU mask), the GEMMs' split-round exchange (sk_workspace) goes through
 * device-coherent stores instead of staying within one XCD's L2: slower by a few microseconds, never wrong.
 * Returns TDIST_ERR_DEVICE when the current device is not gfx950. */
int tdist_init(void);
int tdist_num_cus(void);

/* Test and measurement switches. Process-wide, read by the host side of the entry points at call time; every key
 * starts at -1 = "the library decides" and a negative value puts it back. They select among kernels that all give
 * the documented results; a serving process has no reason to touch them. No counterpart in the reference (its
 * kernels take their variants from autotune configs, e.g. kernels/amd/all_gather_gemm.py:103-137). */
typedef enum tdist_debug_key {
  TDIST_DEBUG_GEMM_TILE = 0,       /* 0..4: force the 256x256, 256x128, 128x128, 128x192 or 128x256 tile where the
                                      call's row blocks and K admit it */
  TDIST_DEBUG_GEMM_SPLIT_K = 1,    /* 0: whole tiles only; 1: split a last round wherever the workspace allows */
  TDIST_DEBUG_GEMM_SK_COHERENT = 2,/* 1: the split-round exchange always through device-coherent stores */
  TDIST_DEBUG_GEMM_SCHEDULE = 3,   /* 0: every workgroup takes its tiles in the static order; 1: in arrival
                                      order (the default for gated calls, see tdist_gemm_chunk_gated_bf16) */
  TDIST_DEBUG_DECODE_WAVE_HEADS = 4,      /* 0: never the kv-head-per-wave form; 2: wherever the heads allow it, whatever
                                             the lengths; 4: likewise, its 4-wave workgroups only */
  TDIST_DEBUG_DECODE_SPLITS_PER_TEAM = 5, /* >= 1: splits one workgroup of that form streams through */
  TDIST_DEBUG_MOE_INDEX_FORM = 6,  /* 2: one launch whose blocks exchange histograms (needs every block resident at
                                      once: see tdist_moe_scatter_index); 3: always three launches */
  TDIST_DEBUG_NUM_KEYS = 8
} tdist_debug_key;
int tdist_debug_set(int key, int value);
int tdist_debug_get(int key);

/* ---------------------------------------------------------------------------------------------
 * (a) chunk-gated tile GEMM — the AG-GEMM consumer.
 *   replaces kernel_consumer_gemm_persistent      kernels/amd/all_gather_gemm.py:140-254
 *            wait_eq_sys                          kernels/amd/common_ops.py:39-46
 *
 * C[M,N] = A[M,K] * B[N,K]^T, fp32 accumulate, output bf16 (or f16 for f16 inputs).
 *   A     gathered workspace, row-major, lda elements between rows (K contiguous)
 *   A_local / local_row_begin / local_rows
 *         rows [local_row_begin, local_row_begin+local_rows) are the caller's own shard: they are read
 *         from A_local (row 0 of A_local = row local_row_begin) and are never gated
 *         (all_gather_gemm.py:201-218). Pass A_local = NULL, local_rows = 0 to gate every row.
 *   B     [N,K] row-major (K contiguous), the reference's non-transposed weight layout (:308-309)
 *   flags int32[ceil(M/m_per_chunk)]: rows of chunk c may be read only once flags[c] == wait_value
 *         (acquire, system scope). flags = NULL disables gating (plain GEMM).
 *   chunk_order  device int32[n_chunks] permutation giving the order in which chunks are consumed,
 *         or NULL for the reference's order (own rank's chunks first, then rank+1, ... :193-199,
 *         which needs rank / world_size).
 *   spin_limit   > 0: polls per wait before giving up; <= 0: library default (seconds of polling).
 *         On expiry the tile is skipped (its C rows are left untouched) and status[0] is set to
 *         TDIST_ERR_TIMEOUT, status[1] to the chunk index. status may be NULL.
 *   max_workgroups  upper bound on the persistent grid; <= 0: one workgroup per compute unit. A producer
 *         whose copies run on this same GPU needs compute units of its own while the GEMM spins on a flag:
 *         leave it 32 (pass tdist_num_cus() - 32). Not needed when the rows arrive from a peer's copy engine.
 * Requirements: K, lda and ldb multiples of 8 (16 for fp8) elements and 16-byte aligned bases. The large tiles are
 * taken when K * element size is a multiple of 128 bytes and the row blocks (m_per_chunk, the local shard) are
 * multiples of 256 rows; a K that ends inside a 64-byte K tile is filled up with zeros on its way in.
 * m_per_chunk may be any positive number of rows: when it is not a multiple of 128, a tile waits for every chunk its
 * rows touch (the reference's per-segment wait, kernels/nvidia/allgather_gemm.py:222-224), tiles are visited in row
 * order starting inside the own rank's rows, chunk_order must be NULL and the local shard must either start and end
 * on a multiple of 128 rows or be copied into A with its flags set (A_local = NULL).
 * Tile order. Every workgroup owns a fixed list of tiles, one per round of the grid, in the order above. With
 * whole-tile chunks (m_per_chunk a multiple of the tile's rows, at most 64 chunks) and 2 to 64 rounds it takes them in
 * the order in which their chunks arrive: when it has finished a tile it takes the earliest of its rounds whose
 * chunk's flag is up, and only with none of them up does it wait, bounded by spin_limit as above; the look at the
 * flags is taken while the tile before is being stored, so a call whose rows are all there pays nothing for it, and
 * the rows of a chunk are acquired once per workgroup, not once per tile. Rows that arrive late or out of order
 * therefore delay only their own tiles. Every tile is computed whole by the workgroup that owns it, so C is bit for
 * bit the same whatever the arrival order is. Otherwise (a single round, ragged chunks, more chunks or rounds) a
 * workgroup waits at the flag of each of its tiles in turn. chunk_order, when given, is the order of the rounds.
 * The reference fixes the order by expected arrival instead (:193-206).
 * ------------------------------------------------------------------------------------------- */
int tdist_gemm_chunk_gated_bf16(const void* A, int64_t lda, const void* A_local, int64_t lda_local,
                                int local_row_begin, int local_rows, const void* B, int64_t ldb, void* C,
                                int64_t ldc, int M, int N, int K, const int32_t* flags, int m_per_chunk,
                                int wait_value, const int32_t* chunk_order, int rank, int world_size,
                                int spin_limit, int32_t* status, int max_workgroups,
    void* sk_workspace, int64_t sk_workspace_bytes, void* stream);

int tdist_gemm_chunk_gated_f16(const void* A, int64_t lda, const void* A_local, int64_t lda_local,
                               int local_row_begin, int local_rows, const void* B, int64_t ldb, void* C,
                               int64_t ldc, int M, int N, int K, const int32_t* flags, int m_per_chunk,
                               int wait_value, const int32_t* chunk_order, int rank, int world_size,
                               int spin_limit, int32_t* status, int max_workgroups,
    void* sk_workspace, int64_t sk_workspace_bytes, void* stream);

/* fp8-e4m3 inputs, bf16 output, C = (sum_k A8*B8) * row_scale[m] * col_scale[n].
 * The scale epilogue has no counterpart in the reference (fp8 is a dtype passthrough there,
 * kernels/nvidia/allgather_gemm.py:313); row_scale / col_scale may be NULL (= 1.0). */
int tdist_gemm_chunk_gated_fp8e4m3(const void* A, int64_t lda, const void* A_local, int64_t lda_local,
                                   int local_row_begin, int local_rows, const void* B, int64_t ldb,
                                   void* C, int64_t ldc, int M, int N, int K, const float* row_scale,
                                   const float* col_scale, const int32_t* flags, int m_per_chunk,
                                   int wait_value, const int32_t* chunk_order, int rank, int world_size,
                                   int spin_limit, int32_t* status, int max_workgroups,
    void* sk_workspace, int64_t sk_workspace_bytes, void* stream);

/* Producer side of the gate on the same GPU: copy one chunk, then release its flag, both ordered on
 * `stream`.   replaces cp_engine_producer_all_gather_full_mesh_push_multi_stream
 *             kernels/amd/all_gather_gemm.py:41-100 (data copy + 4-byte flag copy per chunk).
 * `one` is a device int32 holding the value to publish (the reference copies from a tensor of ones
 * because a stream write-value disturbs the GEMM, :88-100). use_sdma != 0 requests the copy-engine
 * path (hipMemcpyDeviceToDeviceNoCU) so the copy takes no compute unit. */
int tdist_producer_push_chunk(void* dst, const void* src, int64_t nbytes, int32_t* flag, const int32_t* one,
                              int use_sdma, void* stream);

/* All peers of an all-gather in ONE launch (no counterpart in the reference, where every peer's copy engine pushes
 * its own rows: this stands for those engines on a box with one GPU). Block row y plays peer
 * (rank + 1 + y) % world_size: it copies that peer's rows peer_src[r][0 .. rank_bytes) into
 * workspace + r*rank_bytes chunk by chunk (chunk_bytes each) with workgroups_per_peer workgroups, and when the
 * last of them has stored its part of chunk c it stores flag_value into flags[r*chunks_per_rank + c] (release,
 * system scope) — the data-then-flag protocol of kernels/amd/all_gather_gemm.py:80-100.
 * peer_src: device array of world_size device pointers (entry `rank` unused). counters: int32
 * [world_size*chunks_per_rank], zero on entry, left zero. held: optional int32 per chunk: > 0 = never deliver
 * (test hook for the consumer's bounded wait), < 0 = copy it that many microseconds late, at most 100 000 (a straggler;
 * the peer's later chunks follow behind it). stamp + ns_per_chunk > 0: the pace of one link per peer: chunk c of
 * every peer is copied from c*ns_per_chunk after the stamp (tdist_producer_mark) on and its flag is released no
 * earlier than (c+1)*ns_per_chunk after it, when a link of that rate would have delivered the chunk's last byte; the
 * total must stay within 100 ms. max_delay_ns > 0: race provocation, as the reference's producer sleeps with probability
 * 0.7 when run "for correctness" (kernels/nvidia/allgather.py:72-77,118-121): about 7 of 10 (peer, chunk) pairs,
 * chosen by a hash of delay_seed and the chunk, are held back by a pseudo-random time below max_delay_ns before they
 * are copied (max_delay_ns x chunks per rank within 100 ms). The kernel is held to 24 registers per lane and uses no
 * LDS, so its waves fit on a SIMD beside a resident wave of the consumer GEMM; nothing in it waits for another
 * workgroup, and every wait in it is bounded by the device's wall clock. */
int tdist_producer_push_peers(void* workspace, const void* const* peer_src, int world_size, int rank,
                              int64_t rank_bytes, int64_t chunk_bytes, int32_t* flags, int flag_value,
                              int32_t* counters, const int32_t* held, const uint64_t* stamp, int64_t ns_per_chunk,
                              uint32_t delay_seed, int64_t max_delay_ns, int workgroups_per_peer, void* stream);

/* Link pacing for the one-GPU producer (no counterpart in the reference, whose chunks arrive over xGMI at the
 * link's rate: ~153 GB/s per peer). tdist_producer_mark stores the device's constant-rate wall clock into *stamp
 * (device uint64); tdist_producer_wait_until holds `stream` until that clock is offset_ns (0 .. 100 ms) past the
 * stamp, with one idle wave. Queued before a chunk's copy, it makes the chunk arrive no earlier than a link of
 * the given rate would have delivered it. */
int tdist_producer_mark(uint64_t* stamp, void* stream);
int tdist_producer_wait_until(const uint64_t* stamp, int64_t offset_ns, void* stream);

/* A gated GEMM whose bounded flag wait expires writes TDIST_ERR_TIMEOUT and the chunk into its status words, and
 * while status[0] is non-zero every later wait of a launch on the same words gives up after one poll: that is what
 * lets all workgroups of the failing launch leave quickly, and it would make the next launch skip its gated tiles as
 * well. This call, queued in front of the next launch, confines it to one launch: it moves a non-zero status into
 * first_error[0..1] (unless that already holds an earlier one; NULL: dropped) and clears status. No counterpart in
 * the reference, whose waits are unbounded. Safe to record into a HIP graph. */
int tdist_status_retire(int32_t* status, int32_t* first_error, void* stream);

/* Stream-ordered store of `value` into *flag by a one-thread kernel (release, system scope).
 *   replaces set_signal  kernels/amd/common_ops.py:97-112 */
int tdist_flag_set(int32_t* flag, int value, void* stream);
/* Stream-ordered fill of n int32 flags (the reference resets with barrier_ptr.fill_(0),
 * kernels/amd/all_gather_gemm.py:460-461). Safe to record into a HIP graph. */
int tdist_flag_fill(int32_t* flags, int n, int value, void* stream);

/* ---------------------------------------------------------------------------------------------
 * (b) GEMM-RS: GEMM whose epilogue scatters each row block to its owner's buffer, then the
 *     reduction of the per-rank slices.
 *   replaces kernel_gemm_rs_producer_fuse_scatter  kernels/amd/gemm_reduce_scatter.py:125-229
 *            kernel_consumer_reduce                kernels/amd/gemm_reduce_scatter.py:232-258
 * ------------------------------------------------------------------------------------------- */
/* P = A[M,K] * B[N,K]^T (fp32 accumulate) rounded to the input dtype; the rows of P that belong to
 * rank o (rows [o*M/world, (o+1)*M/world)) are stored into scatter_bufs[o] at rows
 * [rank*M/world, (rank+1)*M/world) (gemm_reduce_scatter.py:222-229), every buffer [M, ldc].
 * scatter_bufs is a DEVICE array of world_size device pointers (the reference's scatter_bufs_ptr).
 * Tiles are visited starting with the rows of rank+1 (:171-180).
 * Requirements: M / world_size a multiple of 128 rows (of 256 for the large tiles), K and the row strides
 * multiples of 8 elements (16 for fp8). */
int tdist_gemm_rs_scatter_bf16(const void* A, int64_t lda, const void* B, int64_t ldb,
                               void* const* scatter_bufs, int64_t ldc, int M, int N, int K, int rank,
                               int world_size,
    void* sk_workspace, int64_t sk_workspace_bytes, void* stream);
int tdist_gemm_rs_scatter_f16(const void* A, int64_t lda, const void* B, int64_t ldb,
                              void* const* scatter_bufs, int64_t ldc, int M, int N, int K, int rank,
                              int world_size,
    void* sk_workspace, int64_t sk_workspace_bytes, void* stream);

/* fp8-e4m3 inputs, bf16 partial results: P = (sum_k A8*B8) * row_scale[m] * col_scale[n], scattered as above
 * (row_scale fp32 [M], col_scale fp32 [N], either may be NULL = 1). The reference's kernel takes its output type from
 * its input (gemm_reduce_scatter.py:217-218), which for e4m3 inputs would round the partial sums to e4m3 before they
 * are added up; here they stay bf16, as in the fp8 AG-GEMM above, and go through tdist_reduce_slices like the others. */
int tdist_gemm_rs_scatter_fp8e4m3(const void* A, int64_t lda, const void* B, int64_t ldb,
                                  void* const* scatter_bufs, int64_t ldc, int M, int N, int K,
                                  const float* row_scale, const float* col_scale, int rank, int world_size,
                                  void* sk_workspace, int64_t sk_workspace_bytes, void* stream);

/* out[e] = round( sum_{i=0..n_slices-1} float(c[((i + first_slice) % n_slices) * slice_stride + e]) )
 * for e in [0, n_elems): fp32 accumulation in exactly that order (the reference's order is
 * first_slice = rank+1, gemm_reduce_scatter.py:252-256; it accumulates in the output dtype, this
 * kernel in fp32). dtype: TDIST_BF16 or TDIST_F16 for both c and out. */
int tdist_reduce_slices(const void* c, int64_t slice_stride, int n_slices, int first_slice, int64_t n_elems,
                        void* out, int dtype, void* stream);

/* ---------------------------------------------------------------------------------------------
 * (c) MoE low-latency dispatch / combine permute.
 *   replaces the test-side preprocessing  test/nvidia/test_all_to_all.py:42-96,314-329
 *            all_to_all_kernel            kernels/nvidia/low_latency_all_to_all.py:35-118
 *            all_to_all_post_process      kernels/nvidia/low_latency_all_to_all.py:251-270
 *            combine + index_add_         test/nvidia/test_all_to_all.py:360-370
 *            weighted top-k reduce        test/nvidia/test_moe_reduce_rs.py:103-129
 * ------------------------------------------------------------------------------------------- */
/* Scratch bytes needed by tdist_moe_scatter_index / tdist_moe_splits_cumsum for n_ids ids. The first 256 bytes of the
 * workspace are control words: they must be ZERO when the workspace is first used and are left zero by every call
 * (so one zero-initialised buffer serves all later calls; calls that share it must not overlap). The rest is plain
 * scratch. */
int64_t tdist_moe_workspace_bytes(int64_t n_ids, int num_experts);

/* splits[g] = #{i : ids[i] == g} (torch.bincount(..., minlength=G), test_all_to_all.py:314);
 * cumsum[0] = 0, cumsum[g+1] = splits[0] + ... + splits[g] (splits_to_cumsum, :42-46).
 * ids int32[n_ids] with values in [0, G); splits int32[G]; cumsum int32[G+1]. */
int tdist_moe_splits_cumsum(const int32_t* ids, int64_t n_ids, int num_experts, int32_t* splits,
                            int32_t* cumsum, void* workspace, int64_t workspace_bytes, void* stream);

/* Everything tdist_moe_splits_cumsum writes, plus
 *   scatter_idx[i] = position of flat entry i in the stable sort of ids by expert
 *                    (argsort(stable).argsort(), calc_scatter_index_stable, test_all_to_all.py:95-96)
 *   gather_idx[p]  = token (i / topk) of the entry sorted to position p (calc_gather_index, :49-92)
 *   topk_idx[p]    = i % topk of that entry (may be NULL)
 * all int32; splits may be NULL.
 * Up to 65536 ids: one launch in which every workgroup counts all ids itself; beyond: three launches. No workgroup of
 * either form waits for another one, so both are safe beside kernels that hold compute units (a persistent GEMM
 * spinning on flags). A third form (one launch, workgroups of 2048 ids that exchange histograms and wait for each
 * other) runs only when tdist_debug_set(TDIST_DEBUG_MOE_INDEX_FORM, 2) asks for it: its wait ends only if all its
 * workgroups are resident at once, which is the caller's to guarantee. If that bounded wait expires, the workgroup
 * writes no index rows, cumsum[0] reads -1 unless workgroup 0 got through later, and word 2 of the workspace's
 * control words is set to 1 and stays so until the caller clears it. */
int tdist_moe_scatter_index(const int32_t* ids, int64_t n_ids, int topk, int num_experts, int32_t* splits,
                            int32_t* cumsum, int32_t* scatter_idx, int32_t* gather_idx, int32_t* topk_idx,
                            void* workspace, int64_t workspace_bytes, void* stream);

/* tdist_moe_scatter_index for callers that cannot allocate (code under HIP graph capture, serving loops, harnesses
 * that forbid hipMalloc). It has no counterpart in the reference. Same arguments and same results, without the
 * workspace: the scratch is a 1 MiB array inside the library (one copy per GPU, held until the process ends), so the
 * call allocates nothing. Sizes whose scratch (tdist_moe_workspace_bytes) exceeds 1 MiB are rejected with
 * TDIST_ERR_UNSUPPORTED: e.g. 256 experts take up to 261 632 ids. All calls on one GPU share that GPU's array: calls
 * that overlap on one GPU (different streams without an ordering) race. */
int tdist_moe_scatter_index_static(const int32_t* ids, int64_t n_ids, int topk, int num_experts, int32_t* splits,
                                   int32_t* cumsum, int32_t* scatter_idx, int32_t* gather_idx, int32_t* topk_idx,
                                   void* stream);

/* Dispatch: sorted row p (0 <= p < cumsum[G]) of expert e goes to destination d = e / experts_per_rank,
 * slot row d*max_m + (p - cumsum[d*experts_per_rank]) of slot_rows / slot_scales
 * (low_latency_all_to_all.py:59-103 with every destination's receive slot for this sender kept on the
 * one GPU). Row p is read from rows[gather_idx[p]] (gather_idx = NULL: rows[p], i.e. already sorted
 * input as fast_all_to_all takes it, :189-215). Rows are row_bytes bytes (any dtype); scales fp32 per
 * row or NULL. splits_out int32[G] receives cumsum[g+1]-cumsum[g] (:70-74), or may be NULL.
 * n_rows is the caller's count of sorted rows (T*topk); rows p >= cumsum[G] and rows that would land
 * beyond max_m in their destination slot are not written (the reference asserts the latter away). */
int tdist_moe_dispatch(const void* rows, int64_t row_bytes, const float* scales, const int32_t* gather_idx,
                       const int32_t* cumsum, int64_t n_rows, int world_size, int experts_per_rank,
                       int max_m, void* slot_rows, float* slot_scales, int32_t* splits_out, void* stream);

/* Token-major form of the dispatch, fusing the reference's index_select (test/nvidia/test_all_to_all.py:
 * 328-329) into it: tokens [n_tokens, row_bytes] unsorted, token_scales fp32[n_tokens] or NULL, scatter_idx
 * int32[n_tokens*topk]; the row of token t is read once and written to the slot rows of its topk sorted
 * positions scatter_idx[t*topk + k] (same slot layout and skipping rules as tdist_moe_dispatch). */
int tdist_moe_dispatch_tokens(const void* tokens, int64_t row_bytes, const float* token_scales,
                              const int32_t* scatter_idx, int topk, const int32_t* cumsum, int64_t n_tokens,
                              int world_size, int experts_per_rank, int max_m, void* slot_rows, float* slot_scales,
                              int32_t* splits_out, void* stream);

/* tdist_moe_scatter_index and tdist_moe_dispatch_tokens in ONE launch, for a decode step's worth of tokens: the
 * reference prepares the index tensors with several torch calls and then launches its kernel
 * (test/nvidia/test_all_to_all.py:314-329, kernels/nvidia/low_latency_all_to_all.py:189-248); here every workgroup of
 * the dispatch counts all ids itself while its rows are being fetched, so the rows are placed without a separate
 * index launch and without a workspace. ids int32[n_tokens*topk] (values outside [0, G) take no place: scatter index
 * -1, row not sent). Outputs: the slots as tdist_moe_dispatch_tokens writes them, splits_out (may be NULL), and the
 * index tensors as tdist_moe_scatter_index writes them: splits int32[G] (may be NULL), cumsum int32[G+1], scatter_idx
 * int32[n_tokens*topk], gather_idx int32[n_tokens*topk]. Limits (TDIST_ERR_UNSUPPORTED beyond them: use the two calls):
 * n_tokens*topk <= 65536, rows of 1, 2, 4, 8 or 16 windows of 8 KB. */
int tdist_moe_dispatch_tokens_from_ids(const void* tokens, int64_t row_bytes, const float* token_scales,
                                       const int32_t* ids, int topk, int64_t n_tokens, int world_size,
                                       int experts_per_rank, int max_m, void* slot_rows, float* slot_scales,
                                       int32_t* splits_out, int32_t* splits, int32_t* cumsum, int32_t* scatter_idx,
                                       int32_t* gather_idx, void* stream);

/* Compaction of the slots into one [sum, row_bytes] tensor in destination order
 * (all_to_all_post_process, low_latency_all_to_all.py:251-270): output row p comes from slot row
 * d*max_m + (p - start_d) where start_d = sum of splits of destinations < d.
 * splits int32[world_size*experts_per_rank]; n_rows = number of output rows (the caller knows the
 * total, as the reference does when it slices). out_scales / slot_scales may be NULL. */
int tdist_moe_post_process(const void* slot_rows, int64_t row_bytes, const float* slot_scales,
                           const int32_t* splits, int64_t n_rows, int world_size, int experts_per_rank,
                           int max_m, void* out_rows, float* out_scales, void* stream);

/* Weighted combine back to token order:
 *   y[t, :] = sum_{k=0..topk-1} w[t,k] * scale[p] * float(row[p]),  p = scatter_idx[t*topk + k],
 * fp32 accumulation in k order, output bf16 [T, hidden]. Rows are read from the slot layout written by
 * tdist_moe_dispatch (max_m > 0) or from a compact sorted [n, hidden] tensor (max_m == 0, cumsum
 * ignored). row_dtype: TDIST_F8E4M3 (scales required unless NULL = 1.0) or TDIST_BF16.
 * topk_w fp32 [T, topk] or NULL (= 1.0, the index_add_ form of test_all_to_all.py:366-367).
 * scale_group_size 0: slot_scales holds one scale per row; > 0 (e4m3 rows only): one per group of that many columns,
 * [rows, hidden/scale_group_size], as tdist_moe_dispatch_tokens_quant writes them. */
int tdist_moe_combine(const void* slot_rows, int row_dtype, const float* slot_scales, const int32_t* scatter_idx,
                      const float* topk_w, const int32_t* cumsum, int64_t n_tokens, int topk, int hidden,
                      int world_size, int experts_per_rank, int max_m, int scale_group_size, void* out_bf16,
                      void* stream);

/* Online e4m3 quantisation in groups of group_size = 128 columns.
 *   replaces _quant_kernel / quant_bf16_fp8   tutorials/04-deepseek-infer-all2all.py:309-360
 *   and the fused form in its dispatch kernel  tutorials/04-deepseek-infer-all2all.py:180-200
 * x bf16 [n_rows, hidden] → q e4m3 [n_rows, hidden], scales fp32 [n_rows, hidden/group_size]:
 *   scale = max|x| over the group (as fp32) * fp32(1/448),  q = e4m3(float(x) / scale), round to nearest even.
 * (A group of zeros divides 0 by 0, as the reference does: NaN bytes, scale 0.) */
int tdist_quant_e4m3_groups(const void* x_bf16, int64_t n_rows, int hidden, int group_size, void* q_out,
                            float* scales_out, void* stream);
/* tdist_moe_dispatch_tokens with that quantisation fused in: bf16 token rows [n_tokens, hidden] in, e4m3 slot rows
 * [world_size*max_m, hidden] and slot_scales fp32 [world_size*max_m, hidden/group_size] out; every token row is read
 * and quantised once and written to its topk slot rows. */
int tdist_moe_dispatch_tokens_quant(const void* tokens_bf16, int hidden, int group_size, const int32_t* scatter_idx,
                                    int topk, const int32_t* cumsum, int64_t n_tokens, int world_size,
                                    int experts_per_rank, int max_m, void* slot_rows, float* slot_scales,
                                    int32_t* splits_out, void* stream);

/* Align / sort for the grouped GEMM that follows the dispatch.
 *   replaces moe_ag_scatter_align_block_size_op / _kernel   csrc/lib/moe_utils.cu:60-186
 *   as called by sort_topk_ids_align_block_size              kernels/nvidia/allgather_group_gemm.py:54-135
 * topk_ids: n_total = num_iterations * n_per_iteration flat expert ids (int32, or int64 when ids_int64 != 0, the
 * reference's dtype), one segment of n_per_iteration entries per rank ("iteration"). Per segment, in order, the
 * entries are grouped by expert keeping their flat order, every group is padded to a multiple of block_size, and the
 * padded groups are laid end to end, segment after segment:
 *   sorted_token_ids[pos] = flat index of the entry; capacity n_total + num_experts*num_iterations*(block_size-1).
 *                           Positions of padding keep what was there before: with sorted_fill > 0 the call itself first
 *                           stores n_total into sorted_token_ids[0 .. sorted_fill) (the reference's
 *                           sorted_ids.fill_(numel) in front of its op, allgather_group_gemm.py:103), with 0 the caller
 *                           has pre-filled the array
 *   expert_ids[b], block_barrier_ids[b] = expert and segment of block b; at most
 *                           n_total / block_size + num_experts * num_iterations blocks are written (the reference
 *                           allocates n_total + num_experts * num_iterations entries)
 *   rank_block_num[r]     = blocks of segment r;  *total_tokens_post_pad = padded total.
 * Needs num_experts * num_iterations <= 4096. Workspace: tdist_moe_align_workspace_bytes (0 = unsupported sizes); its
 * first 256 bytes are control words, ZERO on first use and left zero by every call (see tdist_moe_workspace_bytes). */
int64_t tdist_moe_align_workspace_bytes(int64_t n_total, int num_experts, int num_iterations);
int tdist_moe_align_block_size(const void* topk_ids, int ids_int64, int64_t n_total, int num_experts,
                               int num_iterations, int64_t n_per_iteration, int block_size,
                               int32_t* sorted_token_ids, int64_t sorted_fill, int32_t* expert_ids,
                               int32_t* block_barrier_ids, int32_t* rank_block_num, int32_t* total_tokens_post_pad,
                               void* workspace, int64_t workspace_bytes, void* stream);

/* Chunk-gated grouped GEMM of the MoE tensor-parallel path: the consumer of the align / sort step.
 *   replaces kernel_consumer_m_parallel_scatter_group_gemm   kernels/nvidia/allgather_group_gemm.py:238-314
 *   as launched by rowise_intranode_ag_scatter_group_gemm    kernels/nvidia/allgather_group_gemm.py:317-403
 * Row block m (block_size rows of the sorted space, one expert, one rank segment):
 *   C[sorted_token_ids[m*bs + r], :] = A[sorted_token_ids[m*bs + r] / topk, :] . B[expert_ids[m]]^T
 * for the rows whose id is < num_valid_tokens (the rest is padding: read as some valid row, never stored), after
 * flags[block_barrier_ids[m]] == wait_value (dl.wait on block_barrier_ptr, :285-287); blocks at or beyond
 * *num_tokens_post_padded (device int32) are skipped (:274-277). Blocks are taken from first_block on, wrapping
 * (the reference rotates by rank, :263-270): pass the own segment's first block.
 * A [a_rows, K] gathered tokens (lda), A_local optional own shard (tokens [local_row_begin, +local_rows), never
 * waited for); B: expert e's weights at B + e*expert_stride, [N, K] with K contiguous and row stride ldb (the
 * reference takes [E, K, N] with explicit strides: pass a K-contiguous copy or view); C [num_valid_tokens, N]
 * (ldc), of the input dtype (bf16 for e4m3). block_size 128 or 256 = the block_size given to the align / sort;
 * num_blocks = capacity of expert_ids / block_barrier_ids (sorted_token_ids holds num_blocks*block_size ids).
 * tokens_per_rank: tokens of one rank segment. spin_limit / status / max_workgroups as for the gated GEMM;
 * status[1] is the rank segment whose flag did not arrive. */
int tdist_group_gemm_gated_bf16(const void* A, int64_t lda, const void* A_local, int64_t lda_local, int local_row_begin,
                                int local_rows, const void* B, int64_t ldb, int64_t expert_stride, void* C, int64_t ldc,
                                int a_rows, int N, int K, const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                const int32_t* block_barrier_ids, const int32_t* num_tokens_post_padded, int num_blocks,
                                int block_size, int num_valid_tokens, int topk, int tokens_per_rank, int first_block,
                                const int32_t* flags, int wait_value, int rank, int spin_limit, int32_t* status,
                                int max_workgroups,
    void* sk_workspace, int64_t sk_workspace_bytes, void* stream);
int tdist_group_gemm_gated_f16(const void* A, int64_t lda, const void* A_local, int64_t lda_local, int local_row_begin,
                               int local_rows, const void* B, int64_t ldb, int64_t expert_stride, void* C, int64_t ldc,
                               int a_rows, int N, int K, const int32_t* sorted_token_ids, const int32_t* expert_ids,
                               const int32_t* block_barrier_ids, const int32_t* num_tokens_post_padded, int num_blocks,
                               int block_size, int num_valid_tokens, int topk, int tokens_per_rank, int first_block,
                               const int32_t* flags, int wait_value, int rank, int spin_limit, int32_t* status,
                               int max_workgroups,
    void* sk_workspace, int64_t sk_workspace_bytes, void* stream);
int tdist_group_gemm_gated_fp8e4m3(const void* A, int64_t lda, const void* A_local, int64_t lda_local,
                                   int local_row_begin, int local_rows, const void* B, int64_t ldb,
                                   int64_t expert_stride, void* C, int64_t ldc, int a_rows, int N, int K,
                                   const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                   const int32_t* block_barrier_ids, const int32_t* num_tokens_post_padded,
                                   int num_blocks, int block_size, int num_valid_tokens, int topk, int tokens_per_rank,
                                   int first_block, const int32_t* flags, int wait_value, int rank, int spin_limit,
                                   int32_t* status, int max_workgroups,
    void* sk_workspace, int64_t sk_workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Workspace of the GEMM entry points above (tdist_gemm_chunk_gated_*, tdist_gemm_rs_scatter_*,
 * tdist_group_gemm_gated_*): their sk_workspace / sk_workspace_bytes arguments. Optional (NULL, 0). The reference's
 * kernels run whole tiles per program in a fixed order and leave a last round that does not fill the grid to the
 * autotuner's tile choice (kernels/amd/all_gather_gemm.py:151-246 persistent loop;
 * kernels/nvidia/allgather_group_gemm.py:238-314). With a workspace,
 * a last round of tiles that fills at most half of the grid is cut along K: each of its tiles goes to s = 2, 4 or 8
 * workgroups (pieces of at least 4 K tiles); every piece's fp32 accumulators go through the workspace, and each of the
 * s workgroups adds up and stores 1/s of the tile, the pieces in their K order (same products, another order of the
 * sums than a whole tile's: results stay within the stated tolerance, are exact on integer-valued inputs and do not
 * depend on timing). Whole rounds run as before.
 * Bounded waits as for the chunk flags: an exchange that does not complete sets status to
 * {TDIST_ERR_TIMEOUT, -1 - workgroup} and the tile is not stored.
 * The workspace is plain device memory, 256-byte aligned, of at least tdist_gemm_split_k_workspace_bytes() bytes (one
 * fp32 256 x 256 tile per compute unit + a 12 KiB header: 64 MiB + 12 KiB on MI355X; 0 if the device is not gfx950),
 * ZERO when it is first used; the kernels keep it consistent from then on (also across a launch that timed out). It
 * carries no state that the library holds: any number of workspaces may be in use, one per launch in flight —
 * launches that share one must be ordered (same stream, or events). A workspace that is misaligned or smaller than
 * the header plus one 128 x 128 tile is rejected (TDIST_ERR_WORKSPACE); one too small for the call's tiles and grid
 * is left unused.
 * Where the s workgroups of a tile are expected on one XCD (s divides the workgroups per XCD) and tdist_init has
 * seen the dispatch order hold, the partials stay in that XCD's L2 (plain stores, first-level invalidate on the
 * reading side). Every piece also publishes the XCD it ran on, and a reader that finds a partner on another XCD
 * reports {TDIST_ERR_DEVICE, -1 - workgroup} through status and does not store the tile, rather than sum stale slots.
 * tdist_debug_set(TDIST_DEBUG_GEMM_SPLIT_K, 0) turns the split off, 1 takes it wherever a last round can be split;
 * TDIST_DEBUG_GEMM_SK_COHERENT = 1 keeps the exchange device-coherent. */
int64_t tdist_gemm_split_k_workspace_bytes(void);

/* ---------------------------------------------------------------------------------------------
 * (d) split-KV GQA flash decode + LSE combine.
 *   replaces kernel_gqa_fwd_batch_decode_split_kv               kernels/nvidia/flash_decode.py:129-239
 *            kernel_intra_rank_gqa_fwd_batch_decode_combine_kv  kernels/nvidia/flash_decode.py:392-449
 *            kernel_inter_rank_gqa_fwd_batch_decode_combine_kv  kernels/nvidia/flash_decode.py:481-532
 *            kernel_gqa_fwd_batch_decode_split_kv_persistent    kernels/nvidia/flash_decode.py:586-760
 * ------------------------------------------------------------------------------------------- */
/* One query token per sequence. For split s of sequence b (keys [s*per, min((s+1)*per, len)),
 * per = ceil(len/num_splits), flash_decode.py:193-195) and every query head h:
 *   out_split[b,h,s,:] = softmax(q.k*sm_scale [soft-capped]) . v   over the split's keys (fp32)
 *   lse_split[b,h,s]   = log(sum exp(scores))  (natural log, fp32; -inf for an empty split)
 * q [B,Hq,D] (strides q_stride_b, q_stride_h, last dim contiguous); k_cache [num_pages, page_size, Hkv, D] and
 * v_cache [num_pages, page_size, Hkv, Dv] with element strides k_/v_stride_page (between pages), _token, _head;
 * block_table int32 [B, table_stride]; kv_lens int32 [B].
 * out_split fp32 [B,Hq,S,Dv] contiguous; lse_split fp32 [B,Hq,S] contiguous.
 * The reference keeps LSE in-band in the q dtype (column Dv of its [.., Dv+1] buffer, :235-239);
 * here it is a separate fp32 tensor. Supported (head_dim, head_dim_v): every equal pair that is a multiple of 8 up
 * to 256 ((64,64), (128,128) and (256,256) on shapes of their own, the others, e.g. 80, 96 and 160, on the shape of
 * the next power of two with the missing dimensions read as zeros: the reference's BLOCK_DMODEL + BLOCK_DPE split
 * with masks, flash_decode.py:771-772), and the heads whose keys carry 64 dimensions more than their values:
 * (192,128), (576,512); dtype bf16 / f16.
 * A call is one kernel launch, or two where the grid is large enough for the form that gives every wave a kv head of
 * its own: that form runs if the sequence lengths are even (mean >= 0.8 max), the other one, launched behind it, if
 * not; the kernels decide from kv_lens on the device, and the one that does not run returns at once. Kernels only:
 * the call can be captured into a HIP graph. */
int tdist_decode_split_kv(const void* q, const void* k_cache, const void* v_cache, float* out_split,
                          float* lse_split, float sm_scale, float soft_cap, const int32_t* block_table,
                          const int32_t* kv_lens, int batch, int q_heads, int kv_heads, int head_dim,
                          int head_dim_v, int page_size, int num_splits, int64_t q_stride_b, int64_t q_stride_h,
                          int64_t k_stride_page, int64_t k_stride_token, int64_t k_stride_head,
                          int64_t v_stride_page, int64_t v_stride_token, int64_t v_stride_head,
                          int64_t table_stride, int dtype, void* stream);

/* Split-KV decode and the merge of the splits in ONE launch.
 *   replaces kernel_gqa_fwd_batch_decode_split_kv_persistent + barrier_on_this_grid
 *            kernels/nvidia/flash_decode.py:586-760, kernels/nvidia/common_ops.py:62-85
 * Same arguments and partial outputs as tdist_decode_split_kv, plus the merged result of
 * tdist_decode_combine(mode 1): out [B,Hq,Dv] of out_dtype (strides out_stride_b, out_stride_h) and lse_out fp32
 * [B,Hq] or NULL, bit-identical to the two-launch path. Instead of the reference's grid-wide barrier, the last
 * workgroup to finish a (sequence, block of 16 query heads) merges its S partials, so no workgroup waits.
 * counters: int32 [n_counters >= tdist_decode_fused_counters(batch, q_heads, kv_heads)], ALL ZERO on entry; the
 * kernel leaves them zero again, so one zero-initialised buffer serves every later call (calls that share it
 * must not overlap). out_split / lse_split are still written (they are the exchange buffer of the merge). */
int64_t tdist_decode_fused_counters(int batch, int q_heads, int kv_heads);
int tdist_decode_fused(const void* q, const void* k_cache, const void* v_cache, float* out_split, float* lse_split,
                       float sm_scale, float soft_cap, const int32_t* block_table, const int32_t* kv_lens, int batch,
                       int q_heads, int kv_heads, int head_dim, int head_dim_v, int page_size, int num_splits,
                       int64_t q_stride_b, int64_t q_stride_h, int64_t k_stride_page, int64_t k_stride_token,
                       int64_t k_stride_head, int64_t v_stride_page, int64_t v_stride_token, int64_t v_stride_head,
                       int64_t table_stride, int dtype, int32_t* counters, int64_t n_counters, void* out,
                       int out_dtype, int64_t out_stride_b, int64_t out_stride_h, float* lse_out, void* stream);

/* LSE-weighted merge of P partial results per (b,h) — used for the splits of one shard and for the
 * shards of several ranks:
 *   m = max_j lse[j];  w_j = exp(lse[j]-m);  out = sum_j w_j*part[j] / sum_j w_j;  lse_out = m + log(sum_j w_j)
 * over the partials j that are not skipped. part_dtype TDIST_F32 / TDIST_BF16 / TDIST_F16.
 * Partial j of (b,h) lives at part + j*part_stride_p + b*part_stride_b + h*part_stride_h (+ d), its
 * LSE at lse + j*lse_stride_p + b*lse_stride_b + h*lse_stride_h (fp32).
 * Skipping (mode): 0 = none; 1 = split ranges: partial j is skipped when split j of a sequence of
 * lens[b] keys is empty (flash_decode.py:423-428); 2 = shard lengths: lens is int32 [P, B] and partial j
 * is skipped when lens[j*B+b] == 0 (:512-515). A (b,h) whose partials are all skipped gets out = 0,
 * lse_out = -inf. out has out_dtype (TDIST_BF16 / TDIST_F16 / TDIST_F32), [B,Hq,Dv] with strides
 * out_stride_b, out_stride_h; lse_out fp32 [B,Hq] or NULL. */
int tdist_decode_combine(const void* part, int part_dtype, const float* lse, int num_partials, int mode,
                         const int32_t* lens, int batch, int q_heads, int head_dim_v, int64_t part_stride_p,
                         int64_t part_stride_b, int64_t part_stride_h, int64_t lse_stride_p,
                         int64_t lse_stride_b, int64_t lse_stride_h, void* out, int out_dtype,
                         int64_t out_stride_b, int64_t out_stride_h, float* lse_out, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TDIST_H_ */
