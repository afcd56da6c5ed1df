/*
 * Measurement and test hooks of libringattn_hip.so: entry points that run ONE part of what an entry point of
 * ringattn_hip.h runs, so that a benchmark can time a kernel alone and a test can reach every tile kernel.
 * They are not part of the drop-in boundary; a caller of the hot path needs none of them.
 */
#ifndef RINGATTN_HIP_MEASURE_H_
#define RINGATTN_HIP_MEASURE_H_

#include "ringattn_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ra_attn_bwd_block (ringattention_jax.py:181-270) launches two kernels: the key-stationary one that adds into
 * dk and dv, and the query-stationary one that adds into dq.  This launches one of them (MFMA kernels only): what
 * the other one would have written is left untouched, and may be null. */
enum { RA_BWD_PART_DQ = 1, RA_BWD_PART_DKV = 2 };
int ra_attn_bwd_block_part(const ra_attn_bwd_params* p, int32_t part, ra_stream_t stream);
/* The same for ra_attn_bwd_ring_step: one of its two kernels for every device of the ring. */
int ra_attn_bwd_ring_step_part(const ra_attn_bwd_params* p, const ra_ring_step* ring, int32_t part, ra_stream_t stream);

/* ra_gemm_bf16 with the tile kernel named: tile -1 = the library's choice, 0: 256 x 256 over four wavefronts,
 * 1: 256 x 128 over eight, 2: 128 x 128, 3: 256 x 128 over four (a forced tile still gives way to another one where
 * the shape does not divide). */
int ra_gemm_bf16_tile(const void* A, const void* Bm, void* C, int32_t M, int32_t N, int32_t K, int32_t trans_a,
                      int32_t trans_b, int32_t c_dtype, int32_t beta_one, int32_t tile, ra_stream_t stream);

/* C1 = A B1 and C2 = A B2 (all row-major bf16, C (M, N)) as ONE launch over the tile columns of both products: how
 * ra_swiglu_fwd / ra_swiglu_bwd compute a = x w1 and b = x w3 (ringattention_jax.py:340-350 scans a feed-forward
 * whose first two products share their input).  tile as in ra_gemm_bf16_tile; shapes the four-wavefront tile
 * kernels do not take run as two launches. */
int ra_gemm_bf16_pair(const void* A, const void* B1, const void* B2, void* C1, void* C2, int32_t M, int32_t N,
                      int32_t K, int32_t tile, ra_stream_t stream);

/* What the matrix pipes sustain on bf16 MFMAs alone (v_mfma_f32_32x32x16_bf16, four independent accumulators per
 * wavefront, four wavefronts per workgroup): every wavefront issues 64 * iters instructions of 32768 FLOP each.
 * operands 0: one value everywhere; 1: a value per lane, the same in every instruction; 2: random values, consecutive
 * instructions see different operand pairs.  sink: workgroups * 256 floats of device memory (written once).  The rate
 * depends on the operands because the clock is set by a power / current limit, not by the instruction stream. */
int ra_mfma_rate_probe(float* sink, int32_t workgroups, int32_t iters, int32_t operands, ra_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* RINGATTN_HIP_MEASURE_H_ */
