/*
 * tdist_bench.h — C ABI of libtdist_bench.so: measurement helpers used by bench.py only. They are kept out of
 * libtdist_hip.so (the product library) and have no counterpart in the reference. Status codes are tdist.h's.
 */
#ifndef TDIST_BENCH_H_
#define TDIST_BENCH_H_

#include <stdint.h>

#include "tdist.h"

#ifdef __cplusplus
extern "C" {
#endif

const char* tdist_bench_last_error_string(void);

/* ---------------------------------------------------------------------------------------------
 * Measurement helper: plain 16-byte-vector device copy of nbytes (multiple of 16). Used to calibrate
 * rocprof FETCH_SIZE / WRITE_SIZE readings and as the HBM streaming yardstick; not on the hot path.
 * ------------------------------------------------------------------------------------------- */
int tdist_copy_bytes(void* dst, const void* src, int64_t nbytes, void* stream);

/* Measurement helpers: the one-directional streams. tdist_fill_bytes writes nbytes (16-byte vectors, non-temporal
 * stores, no reads); tdist_read_bytes reads nbytes (non-temporal loads) and writes nothing unless the XOR of a lane's
 * words hits one magic value (sink: 256 words). On buffers larger than the 256 MB memory-side cache they give the
 * rates HBM sustains for writes and for reads alone: the ceilings of a write-dominated kernel (the MoE dispatch:
 * 8 bytes written per byte read) and of a read-dominated one (the combine, the decode). */
int tdist_fill_bytes(void* dst, int64_t nbytes, void* stream);
int tdist_read_bytes(const void* src, int64_t nbytes, int32_t* sink, void* stream);

/* Measurement helper: the MFMA rate this chip sustains with no memory traffic at all. One workgroup of four waves per
 * compute unit runs iters (even) K steps of a 128 x 128 wave tile on register operands, in the GEMM kernel's order (a B
 * fragment against every A fragment in turn, 256 accumulators per lane): 4 x 4 MFMAs of 32x32x16 (bf16, K step 16) or
 * 32x32x64 (e4m3, K step 64) per K step. random_operands != 0 fills the fragments with random bit patterns, else with
 * 1.0. FLOP per launch = compute units * 4 * iters * 2 * 128 * 128 * K step. sink: compute units * 256 floats.
 * With random operands the chip is power-limited well below its nominal rate: this is the ceiling any GEMM on random
 * data sits under. Not on the hot path. */
int tdist_mfma_rate_probe(int dtype, int random_operands, int iters, float* sink, void* stream);

/* The same on the 16-row MFMA blocks the 256-row GEMM tiles use: 8 x 8 MFMAs of 16x16x32 (bf16, K step 32) or
 * 16x16x128 (e4m3, K step 128) per K step. They move a quarter of the accumulator registers per FLOP and sustain a
 * higher rate under the power limit. */
int tdist_mfma_rate_probe_16row(int dtype, int random_operands, int iters, float* sink, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TDIST_BENCH_H_ */
