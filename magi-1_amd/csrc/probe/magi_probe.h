/* libmagi_probe: measurement only (loaded by bench.py, never by the product path): the rate of an MFMA-only loop
 * and of plain streaming kernels on the current GPU, the per-box ceilings the kernels' rates are reported against. */
#ifndef MAGI_PROBE_H
#define MAGI_PROBE_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif
#define MAGI_PROBE_WORKGROUPS 256   /* one wave per SIMD on 256 CUs */
#define MAGI_PROBE_SINK_FLOATS (MAGI_PROBE_WORKGROUPS * 256)
/* kind 0: bf16 32x32x16, 1: bf16 16x16x32, 2: fp8 (e4m3) 32x32x64, 3: fp8 (e4m3) 16x16x128.
 * operands: DEVICE array of 2^20 32-bit words the MFMA operands are drawn from (random bit patterns of the
 *           operand type), or NULL for all-zero operands.  sink: DEVICE float[MAGI_PROBE_SINK_FLOATS].
 * Runs one warm-up launch and `launches` timed launches of `rounds` loop rounds back to back on `stream`, waits for
 * them and returns the average milliseconds per launch and the FLOPs of one launch.  0 on success. */
int magi_probe_mfma_only(int kind, const uint32_t* operands, float* sink, int rounds, int launches, void* stream,
                         float* ms_per_launch, double* flop_per_launch);
/* kind 0: copy `bytes` from src to dst; 1: read src only (dst: at least 16 bytes, not written in practice);
 * 2: write dst only (src unused).  DEVICE pointers, 16-byte aligned, bytes a multiple of 16, 16 bytes per lane.
 * One warm-up launch and `launches` timed ones back to back on `stream`; average milliseconds per launch.  0 on
 * success. */
int magi_probe_stream(int kind, const void* src, void* dst, size_t bytes, int launches, void* stream,
                      float* ms_per_launch);
#ifdef __cplusplus
}
#endif
#endif
