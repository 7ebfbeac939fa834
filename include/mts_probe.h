/* Measurement aid of libmts_moe: not part of the operator boundary and without a counterpart in the
 * reference.  The benchmark prints the rate this probe reaches beside the expert-GEMM figures. */
#ifndef MTS_PROBE_H
#define MTS_PROBE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Bytes of device memory the probe writes its per-thread sums to (so the loop cannot be removed). */
int64_t mts_probe_mfma_sink_bytes(int blocks);

/* Launches `blocks` blocks of four waves (two blocks fit a CU), each wave issuing rounds * 64 bf16
 * 32x32x16 MFMAs on registers only: no LDS, no memory traffic besides one store per thread at the end.
 * random_operands != 0 fills the eight operand register sets with pseudo-random values, 0 with constants;
 * consecutive instructions use them the way a 4x2 register tile of a GEMM does.
 * *flops (host memory, optional) receives the floating-point operations of the launch; the caller times
 * it with events on `stream`.  Returns MTS_OK or a negative MTS_ERR_* code. */
int mts_probe_mfma_rate(int random_operands, int blocks, int rounds, void* sink, int64_t sink_bytes,
                        double* flops, void* stream);

#ifdef __cplusplus
}
#endif
#endif
