// Shared helpers of the tmq kernel library (device code for gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "tmq.h"

#define TMQ_EXPORT extern "C" __attribute__((visibility("default")))

namespace tmq {

constexpr int kWave = 64;  // CDNA wavefront width

static inline hipStream_t as_stream(tmq_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

// Status of the launch that was just enqueued (no device synchronisation).
static inline int launch_status() {
  return hipGetLastError() == hipSuccess ? TMQ_OK : TMQ_ERR_LAUNCH;
}

static inline bool aligned(const void* p, uintptr_t a) {
  return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0;
}

__host__ __device__ static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
__host__ __device__ static inline int64_t round_up(int64_t a, int64_t b) { return ceil_div(a, b) * b; }

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

}  // namespace tmq
