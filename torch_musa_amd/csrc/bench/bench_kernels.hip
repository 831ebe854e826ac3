// Measurement probe: what the int8 matrix pipe sustains on this device when it
// is fed from registers only, as a function of the operand data.  MI355X is
// power-limited on this instruction: the shader clock, and with it the
// throughput, depends on how much the operands toggle.  bench.py reports the
// probe next to the GEMM figure so that the GEMM can be read against the
// ceiling the silicon actually reaches, not only against the nominal peak.
// Built into libtmq_bench.so, a measurement library of its own: the operator
// library libtmq.so carries no probe.
#include "common.h"
#include "tmq_bench.h"

namespace tmq {
namespace {

__device__ __forceinline__ unsigned mix(unsigned x) {
  x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
  return x;
}

// four bytes ~ N(0, 37) clamped to int8 (sum of four uniform bytes, scaled)
__device__ __forceinline__ unsigned gaussian_bytes(unsigned seed) {
  unsigned out = 0;
  for (int b = 0; b < 4; ++b) {
    const unsigned h = mix(seed + 77u * b);
    int g = 0;
    for (int u = 0; u < 4; ++u) g += static_cast<int>((h >> (8 * u)) & 0xff) - 128;
    g >>= 2;
    g = g > 127 ? 127 : (g < -128 ? -128 : g);
    out |= static_cast<unsigned>(g & 0xff) << (8 * b);
  }
  return out;
}

// data_mode 0: zeros, 1: uniform random bytes, 2: Gaussian int8 (sigma ~37),
// 4: Gaussian int8 with the second operand's sign bits cleared (non-negative
// values), all held in registers for the whole run
__global__ __launch_bounds__(256) void mfma_probe_kernel(int iters, int data_mode, int* sink,
                                                         long long* stamps) {
  v16i acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0;
  v4i a[4], b[4];
  const unsigned seed = threadIdx.x * 977u + blockIdx.x * 131071u;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      unsigned ra = mix(seed + i * 8 + j), rb = mix(seed + 1000 + i * 8 + j);
      if (data_mode == 0) ra = rb = 0;
      if (data_mode == 2 || data_mode == 4) {
        ra = gaussian_bytes(ra);
        rb = gaussian_bytes(rb);
      }
      if (data_mode == 4) rb &= 0x7f7f7f7fu;
      a[i][j] = static_cast<int>(ra);
      b[i][j] = static_cast<int>(rb);
    }
  const long long c0 = __builtin_readcyclecounter(), w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
      acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i & 3], b[(i >> 1) & 3], acc[i], 0, 0, 0);
  }
  const long long c1 = __builtin_readcyclecounter(), w1 = wall_clock64();
  int s = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) s += acc[i][r];
  if (s == 0x7fffffff) sink[threadIdx.x] = s;  // keeps the loop alive
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    stamps[0] = c1 - c0;  // shader clock cycles
    stamps[1] = w1 - w0;  // 100 MHz ticks
  }
}

// data_mode 5: the same register-only loop on v_mfma_i32_16x16x64_i8, Gaussian int8
__global__ __launch_bounds__(256) void mfma_probe_16x16_kernel(int iters, int* sink, long long* stamps) {
  v4i acc[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = v4i{0, 0, 0, 0};
  v4i a[4], b[4];
  const unsigned seed = threadIdx.x * 977u + blockIdx.x * 131071u;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      a[i][j] = static_cast<int>(gaussian_bytes(mix(seed + i * 8 + j)));
      b[i][j] = static_cast<int>(gaussian_bytes(mix(seed + 1000 + i * 8 + j)));
    }
  const long long c0 = __builtin_readcyclecounter(), w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 16; ++i)
      acc[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[i & 3], b[(i >> 2) & 3], acc[i], 0, 0, 0);
  }
  const long long c1 = __builtin_readcyclecounter(), w1 = wall_clock64();
  int s = 0;
#pragma unroll
  for (int i = 0; i < 16; ++i) s += acc[i].x + acc[i].y + acc[i].z + acc[i].w;
  if (s == 0x7fffffff) sink[threadIdx.x] = s;
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    stamps[0] = c1 - c0;
    stamps[1] = w1 - w0;
  }
}

// data_mode 3: the operands of every MFMA are fresh Gaussian bytes read from
// LDS (12 ds_read_b128 per 16 MFMAs and one barrier per 16, the ratios of the
// GEMM's main loop; eight waves per block, two per SIMD), nothing else: no
// global traffic, no address arithmetic.  What this sustains is the ceiling for
// a GEMM whose matrix pipe never waits, on operands that change every
// instruction the way real data does.
__global__ __launch_bounds__(512) void mfma_probe_lds_kernel(int iters, int* sink, long long* stamps) {
  __shared__ __attribute__((aligned(16))) unsigned char smem[65536];
  const int t = threadIdx.x;
  for (int i = t; i < 65536 / 4; i += 512)
    reinterpret_cast<unsigned*>(smem)[i] = gaussian_bytes(mix(i * 2654435761u + blockIdx.x * 977u));
  __syncthreads();
  v16i acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0;
  v4i f0[6], f1[6];
  const int rd = (t & 63) * 16 + (t >> 6) * 4096;  // consecutive 16-byte slots per wave
#pragma unroll
  for (int i = 0; i < 6; ++i) f0[i] = *reinterpret_cast<const v4i*>(&smem[(rd + i * 1024) & 0xffff]);
  const long long c0 = __builtin_readcyclecounter(), w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
    const int base = rd + it * 208;  // a different 16-byte-aligned window every iteration
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (i < 6) f1[i] = *reinterpret_cast<const v4i*>(&smem[(base + i * 1024 + 8192) & 0xffff]);
      acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f0[i & 1], f0[2 + (i >> 1)], acc[i], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (i < 6) f0[i] = *reinterpret_cast<const v4i*>(&smem[(base + i * 1024 + 24576) & 0xffff]);
      acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f1[i & 1], f1[2 + (i >> 1)], acc[i], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  const long long c1 = __builtin_readcyclecounter(), w1 = wall_clock64();
  int s = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) s += acc[i][r];
  if (s == 0x7fffffff) sink[threadIdx.x & 255] = s;
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    stamps[0] = c1 - c0;
    stamps[1] = w1 - w0;
  }
}

}  // namespace
}  // namespace tmq

using namespace tmq;

// Synchronous by design (it is a measurement, not an operator): launches one
// block of 4 waves per `blocks`, times the second of two launches with HIP
// events, and reads back the clock counters.  `scratch` is device memory of at
// least 2 KiB owned by the caller.
TMQ_EXPORT int tmq_probe_mfma_i8(int data_mode, int blocks, int iters, void* scratch, double* tops,
                                 double* shader_ghz) {
  if (data_mode < 0 || data_mode > 5 || blocks <= 0 || iters <= 0 || scratch == nullptr ||
      tops == nullptr || shader_ghz == nullptr)
    return TMQ_ERR_INVALID_ARGUMENT;
  int* sink = static_cast<int*>(scratch);
  long long* stamps = reinterpret_cast<long long*>(static_cast<char*>(scratch) + 1024);
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return TMQ_ERR_LAUNCH;
  // mode 3: eight waves per block and 16 MFMAs per wave and iteration: half the
  // iterations give the same number of operations per block as the other modes
  const int it3 = iters / 4 > 0 ? iters / 4 : 1;
  auto launch = [&]() {
    if (data_mode == 3) mfma_probe_lds_kernel<<<dim3(blocks), dim3(512), 0, nullptr>>>(it3, sink, stamps);
    else if (data_mode == 5) mfma_probe_16x16_kernel<<<dim3(blocks), dim3(256), 0, nullptr>>>(iters, sink, stamps);
    else mfma_probe_kernel<<<dim3(blocks), dim3(256), 0, nullptr>>>(iters, data_mode, sink, stamps);
  };
  launch();
  hipEventRecord(e0, nullptr);
  launch();
  hipEventRecord(e1, nullptr);
  int rc = hipEventSynchronize(e1) == hipSuccess ? TMQ_OK : TMQ_ERR_LAUNCH;
  float ms = 0.f;
  long long host[2] = {0, 1};
  if (rc == TMQ_OK && (hipEventElapsedTime(&ms, e0, e1) != hipSuccess ||
                       hipMemcpy(host, stamps, sizeof(host), hipMemcpyDeviceToHost) != hipSuccess))
    rc = TMQ_ERR_LAUNCH;
  hipEventDestroy(e0);
  hipEventDestroy(e1);
  if (rc != TMQ_OK) return rc;
  // (mode 5: 16 instructions of 16 x 16 x 64 per iteration are the operations of 8 of 32 x 32 x 32)
  const double ops = data_mode == 3 ? 2.0 * 32 * 32 * 32 * 16 * static_cast<double>(it3) * 8 * blocks
                                    : 2.0 * 32 * 32 * 32 * 8 * static_cast<double>(iters) * 4 * blocks;
  *tops = ops / (ms * 1e-3) / 1e12;
  *shader_ghz = static_cast<double>(host[0]) / (static_cast<double>(host[1]) / 100e6) / 1e9;
  return TMQ_OK;
}

// ---------------------------------------------------------------------------
// Floors for the weight-streaming (decode) kernel: a kernel that only reads
// `bytes` (a multiple of 64 KiB) with that kernel's shape -- one block of eight
// waves per 64 KiB, eight 16-byte loads per thread, all in flight at once -- and
// an empty kernel of the same grid.  Both are asynchronous on `stream`, so that
// bench.py can replay them from a HIP graph exactly as it replays the operator.
// ---------------------------------------------------------------------------
namespace tmq {
namespace {
__global__ __launch_bounds__(512) void stream_read_kernel(const v4i* __restrict__ src, int* sink) {
  const v4i* p = src + static_cast<int64_t>(blockIdx.x) * 4096 + threadIdx.x;
  v4i v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = __builtin_nontemporal_load(p + i * 512);
  int s = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) s ^= v[i].x ^ v[i].y ^ v[i].z ^ v[i].w;
  if (s == 0x5a17c0de) sink[threadIdx.x] = s;  // never true for the benchmark's data; keeps the loads alive
}
__global__ __launch_bounds__(512) void empty_kernel(int* sink) {
  if (sink == nullptr) sink[0] = 0;
}
}  // namespace
}  // namespace tmq

TMQ_EXPORT int tmq_bench_stream_read(const void* src, int64_t bytes, void* sink, tmq_stream_t stream) {
  if (src == nullptr || sink == nullptr || bytes <= 0 || bytes % 65536 != 0 || bytes / 65536 > 0x7fffffff)
    return TMQ_ERR_INVALID_ARGUMENT;
  stream_read_kernel<<<dim3(static_cast<unsigned>(bytes / 65536)), dim3(512), 0, as_stream(stream)>>>(
      static_cast<const v4i*>(src), static_cast<int*>(sink));
  return launch_status();
}

TMQ_EXPORT int tmq_bench_empty_kernel(int blocks, void* sink, tmq_stream_t stream) {
  if (blocks <= 0 || sink == nullptr) return TMQ_ERR_INVALID_ARGUMENT;
  empty_kernel<<<dim3(blocks), dim3(512), 0, as_stream(stream)>>>(static_cast<int*>(sink));
  return launch_status();
}
