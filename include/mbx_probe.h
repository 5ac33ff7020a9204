/*
 * mbx_probe.h — C ABI of libmbx_probe.so: measurement aids for bench.py.  Not part of the dropless-MoE path and
 * without a counterpart in databricks/megablocks; nothing in the product library calls them.
 */
#ifndef MBX_PROBE_H_
#define MBX_PROBE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* A loop of matrix-core instructions and nothing else: every wave keeps 4 + 4 operand fragments (read once from
 * `operands`, n_vec16 16-byte vectors, indexed modulo) and 16 accumulator tiles in registers and issues
 * `iters` x 16 MFMAs of 32x32x16 (kind 1: 8 + 8 fragments, 64 tiles, `iters` x 64 MFMAs of 16x16x32) on them; no
 * LDS, no memory traffic inside the loop.  What this reaches on given operand values
 * is the most any kernel built on that instruction can reach on such values (the power limit lowers the clock when
 * the operands switch many bits).
 *   kind 0: v_mfma_f32_32x32x16_bf16 (the instruction of the grouped GEMM), 1: v_mfma_f32_16x16x32_bf16.
 *   blocks x 256 threads are launched (4 waves per block, one per SIMD of a compute unit).
 *   sink: blocks * 256 floats (keeps the results alive).  clocks: 2 int64 — shader-clock cycles and 100 MHz
 *   wall-clock ticks spent in the loop by wave 0 of block 0 (their ratio x 100 MHz = the shader clock).
 * Returns 0 or a hipError_t.  FLOPs of a launch: blocks * 4 * iters * 16 * 32768 (kind 1: ... * 64 * 16384). */
int mbx_probe_mfma(const void* operands, int64_t n_vec16, int kind, int blocks, int iters, float* sink,
                   int64_t* clocks, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MBX_PROBE_H_ */
