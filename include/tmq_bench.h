/*
 * tmq_bench -- measurement helpers for bench.py (libtmq_bench.so).  Not part of
 * the operator boundary in tmq.h and not linked into libtmq.so: nothing here
 * has a counterpart in the reference, and unlike the operators these calls
 * synchronise the device.
 */
#ifndef TMQ_BENCH_H_
#define TMQ_BENCH_H_

#include <stdint.h>

#include "tmq.h" /* tmq_linear_desc, status codes */

#ifdef __cplusplus
extern "C" {
#endif

/* ---------------------------------------------------------------------------
 * Measurement probe.
 * Runs v_mfma_i32_32x32x32_i8 from registers on `blocks` workgroups of four
 * waves and reports the sustained rate in TOP/s and the shader clock in GHz.
 * data_mode 0: zero operands, 1: uniform random bytes, 2: Gaussian int8 (all
 * held in registers), 3: Gaussian int8 operands read afresh from LDS for every
 * instruction, eight waves per workgroup (the GEMM's loop without its copies),
 * 4: as 2 with the sign bits of the second operand cleared (what the part
 * sustains depends on how much the operands toggle, sign extension included),
 * 5: as 2 on v_mfma_i32_16x16x64_i8.
 * The call synchronises (default stream) and creates two HIP events; status
 * codes are tmq.h's; `scratch` is >= 2 KiB of device memory.
 * ------------------------------------------------------------------------- */
int tmq_probe_mfma_i8(int data_mode, int blocks, int iters, void* scratch, double* tops,
                      double* shader_ghz);

/* Floors for the weight-streaming linear kernel, asynchronous on `stream` (a
 * hipStream_t as in tmq.h) so that they can be captured into a HIP graph like
 * the operator: a kernel that only reads `bytes` (a multiple of 65536) with the
 * decode kernel's shape (one block of eight waves per 64 KiB, all loads in
 * flight at once) and an empty kernel on `blocks` workgroups of eight waves.
 * `sink` is >= 2 KiB of device memory that is never written for real data. */
int tmq_bench_stream_read(const void* src, int64_t bytes, void* sink, void* stream);
int tmq_bench_empty_kernel(int blocks, void* sink, void* stream);

/* Where a launch of the persistent int8 GEMM (quantized::linear on more than one
 * round of 256 x 256 tiles) spends its time: launches the kernel's instrumented
 * instantiation on `desc` (tmq.h's descriptor; quint8 output, the shapes the
 * library sends to that kernel) with `stamps` = device memory for
 * blocks x 2 x 16 uint64 (blocks = min(tiles, compute units rounded down to a
 * multiple of 8)): [block][0][i] the 100 MHz wall clock, [block][1][i] the
 * shader cycle counter, i = 0 at the block's start, then per tile 1 + 4t: main
 * loop starts, 2 + 4t: main loop ends, 3 + 4t: behind the barrier after it,
 * 4 + 4t: epilogue ends.  flags & 1 leaves out the activation copies, flags & 2
 * the weight copies (stale operands: the output is wrong, for timing only).
 * Bits 8..15 of flags: some blocks start that many microseconds late (a schedule
 * experiment; same output) -- with bit 4 clear the blocks that have one tile
 * fewer than the others, with bit 4 set every second compute unit of each XCD.
 * Asynchronous on `stream`. */
int tmq_bench_linear_stamps(const tmq_linear_desc* desc, uint64_t* stamps, int flags, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TMQ_BENCH_H_ */
