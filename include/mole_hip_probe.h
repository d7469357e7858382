/* Measurement aids of the MI355X MoE hot path: NOT part of the drop-in boundary (that is mole_hip.h).
 * Exported by the same library for the benchmark script (`bench.py --probe`), which uses them to show what
 * bounds the grouped products; nothing in the reference corresponds to them and no product code calls them. */
#ifndef MOLE_HIP_PROBE_H
#define MOLE_HIP_PROBE_H

#include "mole_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* timing id (see mole_kernel_timing_read) under which every probe launch is timed */
#define MOLE_K_PROBE MOLE_K_RESERVED_17

/* mole_probe_mfma: `blocks` blocks of eight waves issue v_mfma_f32_32x32x16_bf16 back to
 * back for `iters` rounds of 8 on operands taken once from `operands` (mole_probe_mfma_operand_bytes() bytes: zeros
 * show the published peak, random bf16 data what the chip sustains); sink: blocks * 512 floats; *flop_out: flop of
 * the launch.  mole_probe_kloop: the product kernel at the shape of h = xd . w1^T (a [rows,K], b [E,N,K], experts
 * by offsets / kept_rows) with its epilogue left out - prologue, K loop and launch only; sink: 512 floats.
 * mole_probe_kloop_part: the same with one ingredient of the K loop taken out, to see what the loop waits for
 * (part 0: nothing, 1: the loads of the operand tiles into LDS, 2: the fragment reads from LDS, 3: the barriers, 4: all three);
 * what the accumulators then hold is meaningless.  All are timed under MOLE_K_PROBE. */
size_t mole_probe_mfma_operand_bytes(void);
int mole_probe_mfma(const void *operands, int blocks, int iters, float *sink, double *flop_out, mole_stream_t stream);
int mole_probe_kloop(const void *a, const void *b, const int32_t *offsets, const int32_t *kept_rows, int E,
                     int max_rows, int N, int K, float *sink, mole_stream_t stream);
int mole_probe_kloop_part(const void *a, const void *b, const int32_t *offsets, const int32_t *kept_rows, int E,
                          int max_rows, int N, int K, int part, float *sink, mole_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* MOLE_HIP_PROBE_H */
