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

#ifdef __cplusplus
}
#endif
#endif /* TMQ_BENCH_H_ */
