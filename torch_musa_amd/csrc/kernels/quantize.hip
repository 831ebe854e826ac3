// Affine quantize / dequantize / range calibration for gfx950.
//
// All of these are HBM-streaming kernels: 5 bytes of traffic per element for
// quantize and dequantize (4 + 1), 4 for min/max.  Every wave instruction
// touches one dense run of memory: a lane moves 16 bytes of fp32 and the
// matching 4 bytes of codes, so loads and stores are both fully coalesced, and
// each thread keeps several independent 16-byte accesses in flight.
//
// Numerics follow PyTorch's CPU quantizer (fbgemm/QuantUtils.h:67-101,155-158):
// multiply by the fp32 reciprocal of the fp32 scale, round half to even, add
// the zero point, clamp.  Compiled with -ffp-contract=off.
#include <cmath>
#include <limits>
#include <type_traits>

#include "common.h"
#include "qparams.h"

namespace tmq {
namespace {

constexpr int kThreads = 256;
constexpr int kUnroll = 8;    // independent 16-byte loads per thread, min/max pass
// quantize / dequantize: 2 accesses per thread measured fastest on MI355X at
// 2**28 elements (6.7 and 7.2 TB/s of algorithmic traffic; 8 per thread: 6.0 / 5.3)
constexpr int kUnrollQD = 2;

// FUSED = false: q = clamp(rne(fl(x * inv)) + zp), the arithmetic of
// quantize_per_tensor.  FUSED = true: q = clamp(rne(fl(x * inv + zp))), one
// rounding of product and zero point together, which is how PyTorch's CPU
// quantized::linear_dynamic quantizes its activations while it packs them
// (fbgemm PackAWithQuantRowOffset: fmadd, clip, cvtps); the two differ for
// about one value in 10^5 whose product lies next to a half.
template <bool SIGNED, bool FUSED = false>
__device__ __forceinline__ int quantize_one(float x, float inv, float zp_f) {
  constexpr float lo = SIGNED ? -128.f : 0.f;
  constexpr float hi = SIGNED ? 127.f : 255.f;
  float r;
  if constexpr (FUSED) {
    r = __builtin_rintf(__builtin_fmaf(x, inv, zp_f));
  } else {
    float t = x * inv;
    r = __builtin_rintf(t);  // v_rndne_f32: ties to even
    // zp_f and every in-range r are small integers, so the sum is exact whenever
    // it can land inside [lo, hi]; larger magnitudes clamp either way.
    r = r + zp_f;
  }
  r = fminf(fmaxf(r, lo), hi);
  return static_cast<int>(r);
}

// Four values into one word.  v_cvt_pk_u8_f32 rounds to nearest even, saturates to [0, 255] (NaN -> 0,
// as the clamp of quantize_one has it) and writes its byte into the word: it stands for the clamp, the
// conversion and the packing -- and, where product and zero point are rounded together, for the rounding
// as well.  Signed bytes are the unsigned ones for a zero point 128 higher with the sign bits flipped.
template <bool SIGNED, bool FUSED = false>
__device__ __forceinline__ uint32_t quantize_four(v4f v, float inv, float zp_f) {
  const float zp_u = SIGNED ? zp_f + 128.f : zp_f;
  uint32_t packed = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    float r;
    if constexpr (FUSED && SIGNED)  // (the one rounding of product and zero point is that of the signed zero point)
      r = __builtin_rintf(__builtin_fmaf(v[j], inv, zp_f)) + 128.f;
    else if constexpr (FUSED)
      r = __builtin_fmaf(v[j], inv, zp_u);
    else
      r = __builtin_rintf(v[j] * inv) + zp_u;
    packed = __builtin_amdgcn_cvt_pk_u8_f32(r, j, packed);
  }
  return SIGNED ? packed ^ 0x80808080u : packed;
}

template <bool SIGNED>
__device__ __forceinline__ float dequantize_one(uint32_t byte, int zp, float scale) {
  int v = SIGNED ? static_cast<int>(static_cast<int8_t>(byte)) : static_cast<int>(byte);
  return scale * static_cast<float>(v - zp);
}

// Four bytes of one word.  Byte to float is one instruction (v_cvt_f32_ubyte0..3); the zero point is
// subtracted in fp32, where both terms are small integers and the difference is the exact float(q - zp);
// signed bytes are read as unsigned with the sign bits flipped, against a zero point 128 higher.
template <bool SIGNED>
__device__ __forceinline__ v4f dequantize_four(uint32_t w, int zp, float scale) {
  const uint32_t u = SIGNED ? w ^ 0x80808080u : w;
  const float zp_f = static_cast<float>(SIGNED ? zp + 128 : zp);
  v4f r;
  r.x = scale * (static_cast<float>(u & 0xffu) - zp_f);
  r.y = scale * (static_cast<float>((u >> 8) & 0xffu) - zp_f);
  r.z = scale * (static_cast<float>((u >> 16) & 0xffu) - zp_f);
  r.w = scale * (static_cast<float>(u >> 24) - zp_f);
  return r;
}

// Where the scale / zero point come from: kernel arguments, or device memory
// written earlier on the stream by choose_qparams_kernel.
struct QParamsArg {
  float inv;
  float zp_f;
  const tmq_qparams* dev;
};

__device__ __forceinline__ void resolve(const QParamsArg& a, float& inv, float& zp_f) {
  if (a.dev != nullptr) {
    inv = 1.0f / static_cast<float>(a.dev->scale);  // IEEE division
    zp_f = static_cast<float>(a.dev->zero_point);
  } else {
    inv = a.inv;
    zp_f = a.zp_f;
  }
}

// x4/q4 view the first 4*n4 elements; the block with index 0 also converts the
// n - 4*n4 (< 4) trailing elements one by one.
// The fp32 input is read once and never again: non-temporal loads keep it out of
// the caches.  The codes are written with ordinary stores, so a consumer that
// follows on the stream (dequantize, a GEMM) finds them in the last-level cache --
// unless there are more of them than that cache holds (STREAM_OUT, 128 MiB and
// up): then they leave with non-temporal stores as well (2**28 elements into a
// different output buffer every launch: 211 -> 205.5 us).
// Blocks of two waves, as for the dequantizer below: of 128 / 256 / 512 threads with two
// or four accesses each, two waves x two accesses moved 2**28 elements fastest (213 us
// against 219-225 us in one run).
constexpr int kQThreads = 128;

constexpr int64_t kStreamOutCodes = int64_t{1} << 27;
template <bool SIGNED, bool FUSED = false, bool STREAM_OUT = false>
__global__ __launch_bounds__(kQThreads) void quantize_vec_kernel(
    const v4f* __restrict__ x4, uint32_t* __restrict__ q4, int64_t n4,
    const float* __restrict__ x, uint8_t* __restrict__ q, int64_t n, QParamsArg qp) {
  float inv, zp_f;
  resolve(qp, inv, zp_f);
  const int64_t base = static_cast<int64_t>(blockIdx.x) * (kQThreads * kUnrollQD) + threadIdx.x;
  v4f v[kUnrollQD];
  if (base - threadIdx.x + kQThreads * kUnrollQD <= n4) {
#pragma unroll
    for (int u = 0; u < kUnrollQD; ++u) v[u] = __builtin_nontemporal_load(&x4[base + u * kQThreads]);
#pragma unroll
    for (int u = 0; u < kUnrollQD; ++u) {
      const uint32_t codes = quantize_four<SIGNED, FUSED>(v[u], inv, zp_f);
      if constexpr (STREAM_OUT) __builtin_nontemporal_store(codes, &q4[base + u * kQThreads]);
      else q4[base + u * kQThreads] = codes;
    }
  } else {
#pragma unroll
    for (int u = 0; u < kUnrollQD; ++u) {
      const int64_t i = base + u * kQThreads;
      if (i < n4) v[u] = x4[i];
    }
#pragma unroll
    for (int u = 0; u < kUnrollQD; ++u) {
      const int64_t i = base + u * kQThreads;
      if (i < n4) q4[i] = quantize_four<SIGNED, FUSED>(v[u], inv, zp_f);
    }
  }
  if (blockIdx.x == 0) {
    const int64_t i = 4 * n4 + threadIdx.x;
    if (i < n) q[i] = static_cast<uint8_t>(quantize_one<SIGNED, FUSED>(x[i], inv, zp_f));
  }
}

// Fallback for pointers that are not 16-byte (x) / 4-byte (q) aligned.
template <bool SIGNED, bool FUSED = false>
__global__ __launch_bounds__(kThreads) void quantize_scalar_kernel(
    const float* __restrict__ x, uint8_t* __restrict__ q, int64_t n, QParamsArg qp) {
  float inv, zp_f;
  resolve(qp, inv, zp_f);
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < n; i += stride)
    q[i] = static_cast<uint8_t>(quantize_one<SIGNED, FUSED>(x[i], inv, zp_f));
}

// The codes are read with ordinary loads (they are small and usually still in
// the last-level cache from the kernel that produced them); the fp32 output is
// four times larger and streams out with non-temporal stores so that it does
// not evict them.
// Blocks of two waves: the kernel is bound by the write stream (four of every
// five bytes; a plain 1 GiB fill reaches 4.5-5 TB/s on this part), and of the
// block sizes 64 ... 1024 two waves with two accesses per thread sustained the
// most over 2**28 elements (204.8 us against 210-240 us for the others).
constexpr int kDqThreads = 128;

template <bool SIGNED>
__global__ __launch_bounds__(kDqThreads) void dequantize_vec_kernel(
    const uint32_t* __restrict__ q4, v4f* __restrict__ r4, int64_t n4,
    const uint8_t* __restrict__ q, float* __restrict__ r, int64_t n, float scale, int zp) {
  const int64_t base = static_cast<int64_t>(blockIdx.x) * (kDqThreads * kUnrollQD) + threadIdx.x;
  uint32_t w[kUnrollQD];
  if (base - threadIdx.x + kDqThreads * kUnrollQD <= n4) {
#pragma unroll
    for (int u = 0; u < kUnrollQD; ++u) w[u] = q4[base + u * kDqThreads];
#pragma unroll
    for (int u = 0; u < kUnrollQD; ++u)
      __builtin_nontemporal_store(dequantize_four<SIGNED>(w[u], zp, scale), &r4[base + u * kDqThreads]);
  } else {
#pragma unroll
    for (int u = 0; u < kUnrollQD; ++u) {
      const int64_t i = base + u * kDqThreads;
      if (i < n4) w[u] = q4[i];
    }
#pragma unroll
    for (int u = 0; u < kUnrollQD; ++u) {
      const int64_t i = base + u * kDqThreads;
      if (i < n4) r4[i] = dequantize_four<SIGNED>(w[u], zp, scale);
    }
  }
  if (blockIdx.x == 0) {
    const int64_t i = 4 * n4 + threadIdx.x;
    if (i < n) r[i] = dequantize_one<SIGNED>(q[i], zp, scale);
  }
}

template <bool SIGNED>
__global__ __launch_bounds__(kThreads) void dequantize_scalar_kernel(
    const uint8_t* __restrict__ q, float* __restrict__ r, int64_t n, float scale, int zp) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < n; i += stride)
    r[i] = dequantize_one<SIGNED>(q[i], zp, scale);
}

// ---------------------------------------------------------------------------
// min / max: persistent grid, 16-byte loads, wavefront butterfly reduction,
// one {min,max} pair per block, then a one-block second stage.
// ---------------------------------------------------------------------------
constexpr int kMinMaxMaxBlocks = 2048;  // (1024 ... 4096 blocks and 4 ... 8 loads per thread measure alike)

__device__ __forceinline__ void wave_minmax(float& mn, float& mx) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) {
    mn = fminf(mn, __shfl_xor(mn, off, kWave));
    mx = fmaxf(mx, __shfl_xor(mx, off, kWave));
  }
}

__device__ __forceinline__ void block_minmax_store(float mn, float mx, float* out) {
  __shared__ float s_mn[kThreads / kWave];
  __shared__ float s_mx[kThreads / kWave];
  wave_minmax(mn, mx);
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  if (lane == 0) {
    s_mn[wave] = mn;
    s_mx[wave] = mx;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
#pragma unroll
    for (int w = 1; w < kThreads / kWave; ++w) {
      mn = fminf(mn, s_mn[w]);
      mx = fmaxf(mx, s_mx[w]);
    }
    out[0] = mn;
    out[1] = mx;
  }
}

// KEEP: ordinary loads instead of non-temporal ones, for an input that a second pass on
// the stream reads again while the last-level cache still holds it.
template <bool KEEP = false>
__global__ __launch_bounds__(kThreads) void minmax_partial_kernel(
    const v4f* __restrict__ x4, int64_t n4, const float* __restrict__ x, int64_t head,
    int64_t n, float* __restrict__ partials) {
  auto ld = [](const v4f* p) { return KEEP ? *p : __builtin_nontemporal_load(p); };
  float mn = std::numeric_limits<float>::infinity();
  float mx = -std::numeric_limits<float>::infinity();
  const int64_t step = static_cast<int64_t>(gridDim.x) * (kThreads * kUnroll);
  for (int64_t base = static_cast<int64_t>(blockIdx.x) * (kThreads * kUnroll) + threadIdx.x;
       base - threadIdx.x < n4; base += step) {
    v4f v[kUnroll];
    if (base - threadIdx.x + kThreads * kUnroll <= n4) {
      // a whole chunk: unconditional loads, all in flight before the first comparison
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) v[u] = ld(&x4[base + u * kThreads]);
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        mn = fminf(fminf(mn, v[u].x), fminf(v[u].y, fminf(v[u].z, v[u].w)));
        mx = fmaxf(fmaxf(mx, v[u].x), fmaxf(v[u].y, fmaxf(v[u].z, v[u].w)));
      }
      continue;
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int64_t i = base + u * kThreads;
      if (i < n4) v[u] = ld(&x4[i]);
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int64_t i = base + u * kThreads;
      if (i < n4) {
        mn = fminf(fminf(mn, v[u].x), fminf(v[u].y, fminf(v[u].z, v[u].w)));
        mx = fmaxf(fmaxf(mx, v[u].x), fmaxf(v[u].y, fmaxf(v[u].z, v[u].w)));
      }
    }
  }
  if (blockIdx.x == 0) {
    // elements before the first 16-byte boundary and after the last full group
    const int64_t tail0 = head + 4 * n4;
    const int64_t extra = head + (n - tail0);
    for (int64_t j = threadIdx.x; j < extra; j += kThreads) {
      const float v = j < head ? x[j] : x[tail0 + (j - head)];
      mn = fminf(mn, v);
      mx = fmaxf(mx, v);
    }
  }
  block_minmax_store(mn, mx, partials + 2 * blockIdx.x);
}

__global__ __launch_bounds__(kThreads) void minmax_final_kernel(
    const float* __restrict__ partials, int count, float* __restrict__ out) {
  float mn = std::numeric_limits<float>::infinity();
  float mx = -std::numeric_limits<float>::infinity();
  for (int i = threadIdx.x; i < count; i += kThreads) {
    mn = fminf(mn, partials[2 * i]);
    mx = fmaxf(mx, partials[2 * i + 1]);
  }
  block_minmax_store(mn, mx, out);
}

__global__ void choose_qparams_kernel(const float* __restrict__ minmax, int qmin, int qmax,
                                      int reduce_range, tmq_qparams* __restrict__ out) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    double s;
    int32_t z;
    choose_qparams(minmax[0], minmax[1], qmin, qmax, reduce_range != 0, &s, &z);
    out->scale = s;
    out->zero_point = z;
    out->reserved = 0;
  }
}

// Last stage of the min/max reduction and ChooseQuantizationParams in one block.
__global__ __launch_bounds__(kThreads) void minmax_final_choose_kernel(
    const float* __restrict__ partials, int count, int qmin, int qmax, int reduce_range,
    float* __restrict__ minmax_out, tmq_qparams* __restrict__ out) {
  __shared__ float s_mm[2];
  float mn = std::numeric_limits<float>::infinity();
  float mx = -std::numeric_limits<float>::infinity();
  for (int i = threadIdx.x; i < count; i += kThreads) {
    mn = fminf(mn, partials[2 * i]);
    mx = fmaxf(mx, partials[2 * i + 1]);
  }
  block_minmax_store(mn, mx, s_mm);
  if (threadIdx.x == 0) {
    double s;
    int32_t z;
    choose_qparams(s_mm[0], s_mm[1], qmin, qmax, reduce_range != 0, &s, &z);
    out->scale = s;
    out->zero_point = z;
    out->reserved = 0;
    if (minmax_out != nullptr) {
      minmax_out[0] = s_mm[0];
      minmax_out[1] = s_mm[1];
    }
  }
}

// Second launch of a dynamic quantization: every block first finishes the range
// reduction for itself -- the partial {min, max} pairs of the pass before it (at most
// kDynPartials of them, 4 KB from the L2s), ChooseQuantizationParams in one thread --
// while the loads of its first elements are already in flight, then quantizes its
// share of the input in a grid-stride loop with the next chunk requested before the
// current one is converted.  Block 0 also publishes the parameters.  This replaces a
// one-block launch between the two passes (5 us of a 32 us chain at 2**24 elements:
// launch, 16 KB through one block, the double-precision divisions) by a few hundred
// cycles under each block's first loads.  Same arithmetic in the same order as the
// three launches: min and max do not depend on the order of the reduction.
constexpr int kDynPartials = 512;
constexpr int kDynQBlocks = 2048;
constexpr int64_t kDynKeepMax = int64_t{1} << 25;  // 128 MiB of fp32: half the last-level cache
template <bool SIGNED, bool FUSED>
__global__ __launch_bounds__(kThreads) void quantize_after_minmax_kernel(
    const v4f* __restrict__ x4, uint32_t* __restrict__ q4, int64_t n4, const float* __restrict__ x,
    uint8_t* __restrict__ q, int64_t n, const float* __restrict__ partials, int count, int qmin, int qmax,
    int reduce_range, tmq_qparams* __restrict__ out) {
  __shared__ float s_mm[2];
  __shared__ float s_inv, s_zp;
  constexpr int U = kUnrollQD;
  const int64_t step = static_cast<int64_t>(gridDim.x) * (kThreads * U);
  int64_t base = static_cast<int64_t>(blockIdx.x) * (kThreads * U) + threadIdx.x;
  // (loads are unconditional -- indices clamped into the input -- so that they can be
  // counted: a load under a condition would be waited for before anything else is requested)
  auto request = [&](int64_t b, v4f(&v)[U]) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t i = b + u * kThreads;
      v[u] = x4[i < n4 ? i : (n4 > 0 ? n4 - 1 : 0)];
    }
  };
  v4f cur[U], nxt[U];
  if (n4 > 0) request(base, cur);
  float mn = std::numeric_limits<float>::infinity();
  float mx = -std::numeric_limits<float>::infinity();
  for (int i = threadIdx.x; i < count; i += kThreads) {
    const float2 p = *reinterpret_cast<const float2*>(partials + 2 * i);
    mn = fminf(mn, p.x);
    mx = fmaxf(mx, p.y);
  }
  block_minmax_store(mn, mx, s_mm);  // (ends with thread 0 holding the block's result)
  if (threadIdx.x == 0) {
    double sc;
    int32_t z;
    choose_qparams(s_mm[0], s_mm[1], qmin, qmax, reduce_range != 0, &sc, &z);
    s_inv = 1.0f / static_cast<float>(sc);  // IEEE division, as resolve()
    s_zp = static_cast<float>(z);
    if (blockIdx.x == 0) {
      out->scale = sc;
      out->zero_point = z;
      out->reserved = 0;
    }
  }
  __syncthreads();
  const float inv = s_inv, zp_f = s_zp;
  for (; base - threadIdx.x < n4; base += step) {
    const bool more = base - threadIdx.x + step < n4;
    if (more) request(base + step, nxt);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t i = base + u * kThreads;
      if (i < n4) q4[i] = quantize_four<SIGNED, FUSED>(cur[u], inv, zp_f);
    }
    if (more) {
#pragma unroll
      for (int u = 0; u < U; ++u) cur[u] = nxt[u];
    }
  }
  if (blockIdx.x == 0) {
    const int64_t i = 4 * n4 + threadIdx.x;
    if (i < n) q[i] = static_cast<uint8_t>(quantize_one<SIGNED, FUSED>(x[i], inv, zp_f));
  }
}

// Dynamic quantization of a small tensor in one launch: one block finds the
// range, chooses the parameters and converts.  A decode-sized activation
// ([1..16, 4096] floats) is a few tens of KB: three dependent launches would
// cost several times what the work does.
constexpr int kDynSmallThreads = 1024;
// (elements.  From 32 Ki on the two-launch chain below is faster than one block pulling the
// whole input: a dynamically quantized linear of 16 x 4096 values takes 11.1 instead of 12.6 us.)
constexpr int64_t kDynSmallMax = 32768;
template <bool SIGNED, bool FUSED>
__global__ __launch_bounds__(kDynSmallThreads) void dynamic_quantize_small_kernel(
    const float* __restrict__ x, uint8_t* __restrict__ q, int64_t n, int qmin, int qmax,
    int reduce_range, bool vec, tmq_qparams* __restrict__ out) {
  __shared__ float s_mn[kDynSmallThreads / kWave], s_mx[kDynSmallThreads / kWave];
  __shared__ float s_inv, s_zp;
  const int t = threadIdx.x;
  const int64_t n4 = vec ? n / 4 : 0;
  const v4f* x4 = reinterpret_cast<const v4f*>(x);
  // the whole input fits the block's registers (kDynSmallMax / 4 / threads = 8
  // groups of four per thread): memory is read once, all loads in flight together
  constexpr int kHeld = static_cast<int>(kDynSmallMax / 4 / kDynSmallThreads);
  v4f held[kHeld];
#pragma unroll
  for (int u = 0; u < kHeld; ++u) {
    const int64_t i = t + static_cast<int64_t>(u) * kDynSmallThreads;
    if (i < n4) held[u] = x4[i];
  }
  float mn = std::numeric_limits<float>::infinity();
  float mx = -std::numeric_limits<float>::infinity();
#pragma unroll
  for (int u = 0; u < kHeld; ++u) {
    const int64_t i = t + static_cast<int64_t>(u) * kDynSmallThreads;
    if (i < n4) {
      const v4f v = held[u];
      mn = fminf(fminf(mn, v.x), fminf(v.y, fminf(v.z, v.w)));
      mx = fmaxf(fmaxf(mx, v.x), fmaxf(v.y, fmaxf(v.z, v.w)));
    }
  }
  for (int64_t i = 4 * n4 + t; i < n; i += kDynSmallThreads) {
    mn = fminf(mn, x[i]);
    mx = fmaxf(mx, x[i]);
  }
  wave_minmax(mn, mx);
  if (t % kWave == 0) {
    s_mn[t / kWave] = mn;
    s_mx[t / kWave] = mx;
  }
  __syncthreads();
  if (t == 0) {
#pragma unroll
    for (int w = 1; w < kDynSmallThreads / kWave; ++w) {
      mn = fminf(mn, s_mn[w]);
      mx = fmaxf(mx, s_mx[w]);
    }
    double s;
    int32_t z;
    choose_qparams(mn, mx, qmin, qmax, reduce_range != 0, &s, &z);
    out->scale = s;
    out->zero_point = z;
    out->reserved = 0;
    s_inv = 1.0f / static_cast<float>(s);  // IEEE division, as in resolve()
    s_zp = static_cast<float>(z);
  }
  __syncthreads();
  const float inv = s_inv, zp_f = s_zp;
  uint32_t* q4 = reinterpret_cast<uint32_t*>(q);
#pragma unroll
  for (int u = 0; u < kHeld; ++u) {
    const int64_t i = t + static_cast<int64_t>(u) * kDynSmallThreads;
    if (i < n4) q4[i] = quantize_four<SIGNED, FUSED>(held[u], inv, zp_f);
  }
  for (int64_t i = 4 * n4 + t; i < n; i += kDynSmallThreads)
    q[i] = static_cast<uint8_t>(quantize_one<SIGNED, FUSED>(x[i], inv, zp_f));
}

// ---------------------------------------------------------------------------
// Per-channel kernels over [outer, C, inner], element-indexed: the channel of
// an element comes from its flat index.  They serve short rows (inner < 64,
// e.g. a channel axis that is the last dimension); longer rows take
// pc_rows_kernel below.  VEC = 4 when inner % 4 == 0 and the pointers are
// 16-byte aligned (a group of 4 never straddles a channel).
// ---------------------------------------------------------------------------
template <bool SIGNED, int VEC>
__global__ __launch_bounds__(kThreads) void quantize_pc_kernel(
    const float* __restrict__ x, uint8_t* __restrict__ q, int64_t n, int64_t C, int64_t inner,
    const double* __restrict__ scales, const int64_t* __restrict__ zps) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads * VEC;
  for (int64_t i = (static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x) * VEC; i < n;
       i += stride) {
    const int64_t c = (i / inner) % C;
    const float inv = 1.0f / static_cast<float>(scales[c]);
    const float zp_f = static_cast<float>(zps[c]);
    if constexpr (VEC == 4) {
      const v4f v = *reinterpret_cast<const v4f*>(x + i);
      *reinterpret_cast<uint32_t*>(q + i) = quantize_four<SIGNED>(v, inv, zp_f);
    } else {
      q[i] = static_cast<uint8_t>(quantize_one<SIGNED>(x[i], inv, zp_f));
    }
  }
}

template <bool SIGNED>
__device__ __forceinline__ float dequantize_pc_one(uint32_t byte, float zp_f, double scale) {
  const int v = SIGNED ? static_cast<int>(static_cast<int8_t>(byte)) : static_cast<int>(byte);
  const float d = static_cast<float>(v) - zp_f;
  return static_cast<float>(static_cast<double>(d) * scale);
}

template <bool SIGNED, int VEC>
__global__ __launch_bounds__(kThreads) void dequantize_pc_kernel(
    const uint8_t* __restrict__ q, float* __restrict__ r, int64_t n, int64_t C, int64_t inner,
    const double* __restrict__ scales, const int64_t* __restrict__ zps) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads * VEC;
  for (int64_t i = (static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x) * VEC; i < n;
       i += stride) {
    const int64_t c = (i / inner) % C;
    const double scale = scales[c];
    const float zp_f = static_cast<float>(zps[c]);
    if constexpr (VEC == 4) {
      const uint32_t w = *reinterpret_cast<const uint32_t*>(q + i);
      v4f o;
      o.x = dequantize_pc_one<SIGNED>(w & 0xffu, zp_f, scale);
      o.y = dequantize_pc_one<SIGNED>((w >> 8) & 0xffu, zp_f, scale);
      o.z = dequantize_pc_one<SIGNED>((w >> 16) & 0xffu, zp_f, scale);
      o.w = dequantize_pc_one<SIGNED>(w >> 24, zp_f, scale);
      *reinterpret_cast<v4f*>(r + i) = o;
    } else {
      r[i] = dequantize_pc_one<SIGNED>(q[i], zp_f, scale);
    }
  }
}

// Per-channel quantizer with float scales and float zero points
// (qscheme per_channel_affine_float_qparams): q = clamp(lrintf(x * inv + zp)),
// inv = 1 / scale (1 when the scale is 0), r = (float(q) - zp) * scale, all fp32.
template <bool SIGNED>
__device__ __forceinline__ uint32_t quantize_fq_one(float x, float inv, float zp) {
  const float t = x * inv;
  float r = __builtin_rintf(t + zp);
  r = __builtin_amdgcn_fmed3f(r, SIGNED ? -128.f : 0.f, SIGNED ? 127.f : 255.f);
  return static_cast<uint32_t>(static_cast<int>(r)) & 0xffu;
}

template <bool SIGNED, int VEC>
__global__ __launch_bounds__(kThreads) void quantize_pcf_kernel(
    const float* __restrict__ x, uint8_t* __restrict__ q, int64_t n, int64_t C, int64_t inner,
    const float* __restrict__ scales, const float* __restrict__ zps) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads * VEC;
  for (int64_t i = (static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x) * VEC; i < n;
       i += stride) {
    const int64_t c = (i / inner) % C;
    const float sc = scales[c];
    const float inv = sc == 0.f ? 1.0f : 1.0f / sc;
    const float zp = zps[c];
    if constexpr (VEC == 4) {
      const v4f v = *reinterpret_cast<const v4f*>(x + i);
      *reinterpret_cast<uint32_t*>(q + i) =
          quantize_fq_one<SIGNED>(v.x, inv, zp) | (quantize_fq_one<SIGNED>(v.y, inv, zp) << 8) |
          (quantize_fq_one<SIGNED>(v.z, inv, zp) << 16) | (quantize_fq_one<SIGNED>(v.w, inv, zp) << 24);
    } else {
      q[i] = static_cast<uint8_t>(quantize_fq_one<SIGNED>(x[i], inv, zp));
    }
  }
}

template <bool SIGNED>
__device__ __forceinline__ float dequantize_fq_one(uint32_t byte, float zp, float scale) {
  const int v = SIGNED ? static_cast<int>(static_cast<int8_t>(byte)) : static_cast<int>(byte);
  const float d = static_cast<float>(v) - zp;
  return d * scale;
}

template <bool SIGNED, int VEC>
__global__ __launch_bounds__(kThreads) void dequantize_pcf_kernel(
    const uint8_t* __restrict__ q, float* __restrict__ r, int64_t n, int64_t C, int64_t inner,
    const float* __restrict__ scales, const float* __restrict__ zps) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads * VEC;
  for (int64_t i = (static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x) * VEC; i < n;
       i += stride) {
    const int64_t c = (i / inner) % C;
    const float scale = scales[c], zp = zps[c];
    if constexpr (VEC == 4) {
      const uint32_t w = *reinterpret_cast<const uint32_t*>(q + i);
      v4f o;
      o.x = dequantize_fq_one<SIGNED>(w & 0xffu, zp, scale);
      o.y = dequantize_fq_one<SIGNED>((w >> 8) & 0xffu, zp, scale);
      o.z = dequantize_fq_one<SIGNED>((w >> 16) & 0xffu, zp, scale);
      o.w = dequantize_fq_one<SIGNED>(w >> 24, zp, scale);
      *reinterpret_cast<v4f*>(r + i) = o;
    } else {
      r[i] = dequantize_fq_one<SIGNED>(q[i], zp, scale);
    }
  }
}

// ---------------------------------------------------------------------------
// Per-channel kernels for inner >= kPcRowsMinInner: the channel is a property of
// the block, not of the element.  The tensor is `rows` = outer * C rows of
// `inner` elements; a block takes RB = A >> lg_us consecutive rows (A accesses per thread) x one
// segment of US = 1 << lg_us runs of 256 lanes x VEC elements, i.e. eight
// accesses per thread whatever the row length (a row of 4096 floats is four
// 16-byte accesses per thread, so a quantizing block takes two rows).  Row and channel come
// from blockIdx with one division per block; the parameters of a row are
// wave-uniform (scalar loads); the element loop has no division at all.
// Loads are batched ahead of the stores and carry the same cache hints as the
// per-tensor kernels.
// ---------------------------------------------------------------------------
constexpr int kPcRowsMinInner = 64;

template <bool SIGNED>
struct PcQuantize {
  // fp32 -> codes, double scales, int64 zero points
  static constexpr int kAccesses = 4;
  const float* x;
  uint8_t* q;
  const double* scales;
  const int64_t* zps;
  struct P { float inv, zp; };
  using In4 = v4f;
  using In1 = float;
  __device__ __forceinline__ P params(int64_t c) const {
    return {1.0f / static_cast<float>(scales[c]), static_cast<float>(zps[c])};
  }
  __device__ __forceinline__ In4 load4(int64_t i) const {
    return __builtin_nontemporal_load(reinterpret_cast<const v4f*>(x + i));
  }
  __device__ __forceinline__ In1 load1(int64_t i) const { return x[i]; }
  __device__ __forceinline__ void store4(int64_t i, In4 v, P p) const {
    *reinterpret_cast<uint32_t*>(q + i) = quantize_four<SIGNED>(v, p.inv, p.zp);
  }
  __device__ __forceinline__ void store1(int64_t i, In1 v, P p) const {
    q[i] = static_cast<uint8_t>(quantize_one<SIGNED>(v, p.inv, p.zp));
  }
};

template <bool SIGNED>
struct PcDequantize {
  // codes -> fp32, double scales, int64 zero points
  static constexpr int kAccesses = 2;
  const uint8_t* q;
  float* r;
  const double* scales;
  const int64_t* zps;
  struct P { double scale; float zp; };
  using In4 = uint32_t;
  using In1 = uint32_t;
  __device__ __forceinline__ P params(int64_t c) const { return {scales[c], static_cast<float>(zps[c])}; }
  __device__ __forceinline__ In4 load4(int64_t i) const { return *reinterpret_cast<const uint32_t*>(q + i); }
  __device__ __forceinline__ In1 load1(int64_t i) const { return q[i]; }
  __device__ __forceinline__ void store4(int64_t i, In4 w, P p) const {
    v4f o;
    o.x = dequantize_pc_one<SIGNED>(w & 0xffu, p.zp, p.scale);
    o.y = dequantize_pc_one<SIGNED>((w >> 8) & 0xffu, p.zp, p.scale);
    o.z = dequantize_pc_one<SIGNED>((w >> 16) & 0xffu, p.zp, p.scale);
    o.w = dequantize_pc_one<SIGNED>(w >> 24, p.zp, p.scale);
    __builtin_nontemporal_store(o, reinterpret_cast<v4f*>(r + i));
  }
  __device__ __forceinline__ void store1(int64_t i, In1 b, P p) const {
    r[i] = dequantize_pc_one<SIGNED>(b, p.zp, p.scale);
  }
};

template <bool SIGNED>
struct PcfQuantize {
  // fp32 -> codes, float scales and float zero points
  static constexpr int kAccesses = 4;
  const float* x;
  uint8_t* q;
  const float* scales;
  const float* zps;
  struct P { float inv, zp; };
  using In4 = v4f;
  using In1 = float;
  __device__ __forceinline__ P params(int64_t c) const {
    const float sc = scales[c];
    return {sc == 0.f ? 1.0f : 1.0f / sc, zps[c]};
  }
  __device__ __forceinline__ In4 load4(int64_t i) const {
    return __builtin_nontemporal_load(reinterpret_cast<const v4f*>(x + i));
  }
  __device__ __forceinline__ In1 load1(int64_t i) const { return x[i]; }
  __device__ __forceinline__ void store4(int64_t i, In4 v, P p) const {
    *reinterpret_cast<uint32_t*>(q + i) =
        quantize_fq_one<SIGNED>(v.x, p.inv, p.zp) | (quantize_fq_one<SIGNED>(v.y, p.inv, p.zp) << 8) |
        (quantize_fq_one<SIGNED>(v.z, p.inv, p.zp) << 16) | (quantize_fq_one<SIGNED>(v.w, p.inv, p.zp) << 24);
  }
  __device__ __forceinline__ void store1(int64_t i, In1 v, P p) const {
    q[i] = static_cast<uint8_t>(quantize_fq_one<SIGNED>(v, p.inv, p.zp));
  }
};

template <bool SIGNED>
struct PcfDequantize {
  // codes -> fp32, float scales and float zero points
  static constexpr int kAccesses = 2;
  const uint8_t* q;
  float* r;
  const float* scales;
  const float* zps;
  struct P { float scale, zp; };
  using In4 = uint32_t;
  using In1 = uint32_t;
  __device__ __forceinline__ P params(int64_t c) const { return {scales[c], zps[c]}; }
  __device__ __forceinline__ In4 load4(int64_t i) const { return *reinterpret_cast<const uint32_t*>(q + i); }
  __device__ __forceinline__ In1 load1(int64_t i) const { return q[i]; }
  __device__ __forceinline__ void store4(int64_t i, In4 w, P p) const {
    v4f o;
    o.x = dequantize_fq_one<SIGNED>(w & 0xffu, p.zp, p.scale);
    o.y = dequantize_fq_one<SIGNED>((w >> 8) & 0xffu, p.zp, p.scale);
    o.z = dequantize_fq_one<SIGNED>((w >> 16) & 0xffu, p.zp, p.scale);
    o.w = dequantize_fq_one<SIGNED>(w >> 24, p.zp, p.scale);
    __builtin_nontemporal_store(o, reinterpret_cast<v4f*>(r + i));
  }
  __device__ __forceinline__ void store1(int64_t i, In1 b, P p) const {
    r[i] = dequantize_fq_one<SIGNED>(b, p.zp, p.scale);
  }
};

// Accesses per thread (Op::kAccesses), all in flight before the first store: four for
// the quantizers, two for the dequantizers, in blocks of two waves -- the shape the
// per-tensor kernels settled on as well.  At fp32 [11008, 4096], axis 0, inputs and
// outputs rotating over more bytes than the last-level cache holds: quantize 39.8 us
// (per-tensor kernel on as many elements: 38.4 us), dequantize 37.6 us (35.4 us);
// the dequantizer took 42.2 us with a parameter request per access, each waiting for
// the one before it, 39.4 us with one per row in blocks of four waves x four accesses.
constexpr int kPcThreads = 128;
template <class Op, int VEC>
__global__ __launch_bounds__(kPcThreads) void pc_rows_kernel(Op op, int64_t rows, int64_t C, int64_t inner,
                                                           int lg_us, uint32_t segs) {
  using In = std::conditional_t<VEC == 4, typename Op::In4, typename Op::In1>;
  constexpr int kPcAccesses = Op::kAccesses;
  const uint32_t rg = blockIdx.x / segs, seg = blockIdx.x - rg * segs;
  const int us_mask = (1 << lg_us) - 1;
  const int64_t row0 = static_cast<int64_t>(rg) * (kPcAccesses >> lg_us);
  const int64_t c0 = row0 % C;  // once per block, wave-uniform
  const int64_t col0 = (static_cast<int64_t>(seg) << lg_us) * (kPcThreads * VEC) + threadIdx.x * VEC;
  In held[kPcAccesses];
  bool live[kPcAccesses];
  // a block that lies inside the tensor as a whole (all but the last row group and the
  // last segment of a row) loads and stores without a condition per access
  const bool whole = row0 + (kPcAccesses >> lg_us) <= rows &&
                     ((static_cast<int64_t>(seg) + 1) << lg_us) * (kPcThreads * VEC) <= inner;
  if (whole) {
    // with the number of runs per row as a constant, every index below is one: the
    // parameters of the block's rows are requested together, once per row (not once
    // per access, each request waiting for the one before it)
    auto run = [&](auto lg_tag) {
      constexpr int LG = decltype(lg_tag)::value;
      if constexpr ((1 << LG) <= kPcAccesses) {
        constexpr int kRows = kPcAccesses >> LG, kRuns = 1 << LG;
#pragma unroll
        for (int r = 0; r < kRows; ++r)
#pragma unroll
          for (int k = 0; k < kRuns; ++k) {
            const int64_t at = (row0 + r) * inner + col0 + static_cast<int64_t>(k) * (kPcThreads * VEC);
            if constexpr (VEC == 4) held[r * kRuns + k] = op.load4(at);
            else held[r * kRuns + k] = op.load1(at);
          }
        typename Op::P prm[kRows];
#pragma unroll
        for (int r = 0; r < kRows; ++r) {
          int64_t c = c0 + r;
          while (c >= C) c -= C;   // at most kRows - 1 rows past c0: uniform, a few scalar steps
          prm[r] = op.params(c);
        }
#pragma unroll
        for (int r = 0; r < kRows; ++r)
#pragma unroll
          for (int k = 0; k < kRuns; ++k) {
            const int64_t at = (row0 + r) * inner + col0 + static_cast<int64_t>(k) * (kPcThreads * VEC);
            if constexpr (VEC == 4) op.store4(at, held[r * kRuns + k], prm[r]);
            else op.store1(at, held[r * kRuns + k], prm[r]);
          }
      }
    };
    switch (lg_us) {
      case 0: run(std::integral_constant<int, 0>{}); break;
      case 1: run(std::integral_constant<int, 1>{}); break;
      case 2: run(std::integral_constant<int, 2>{}); break;
      default: run(std::integral_constant<int, 3>{}); break;
    }
    return;
  }
#pragma unroll
  for (int u = 0; u < kPcAccesses; ++u) {
    const int64_t row = row0 + (u >> lg_us);
    const int64_t col = col0 + static_cast<int64_t>(u & us_mask) * (kPcThreads * VEC);
    live[u] = row < rows && col < inner;
    if (live[u]) {
      if constexpr (VEC == 4) held[u] = op.load4(row * inner + col);
      else held[u] = op.load1(row * inner + col);
    }
  }
#pragma unroll
  for (int u = 0; u < kPcAccesses; ++u) {
    const int64_t row = row0 + (u >> lg_us);
    if (row >= rows) break;  // uniform
    int64_t c = c0 + (u >> lg_us);
    while (c >= C) c -= C;   // at most A - 1 rows past c0: uniform, a few scalar steps
    const typename Op::P p = op.params(c);
    const int64_t col = col0 + static_cast<int64_t>(u & us_mask) * (kPcThreads * VEC);
    if (live[u]) {
      if constexpr (VEC == 4) op.store4(row * inner + col, held[u], p);
      else op.store1(row * inner + col, held[u], p);
    }
  }
}

// Launches pc_rows_kernel if the shape suits it; returns false if the caller
// should use the element-indexed kernels (short rows, or a grid beyond 2**31).
template <class Op>
bool launch_pc_rows(const Op& op, int64_t outer, int64_t C, int64_t inner, bool vec, hipStream_t s) {
  if (inner < kPcRowsMinInner) return false;
  constexpr int kPcAccesses = Op::kAccesses;
  const int64_t per_run = kPcThreads * (vec ? 4 : 1);
  int lg_us = 0;
  while ((2 << lg_us) <= kPcAccesses && (per_run << lg_us) < inner) ++lg_us;
  const int64_t rows = outer * C;
  const int64_t segs = ceil_div(inner, per_run << lg_us);
  const int64_t row_groups = ceil_div(rows, kPcAccesses >> lg_us);
  if (segs > 0x7fffffff || row_groups > 0x7fffffff / segs) return false;
  const dim3 grid(static_cast<unsigned>(row_groups * segs));
  if (vec)
    pc_rows_kernel<Op, 4><<<grid, dim3(kPcThreads), 0, s>>>(op, rows, C, inner, lg_us, static_cast<uint32_t>(segs));
  else
    pc_rows_kernel<Op, 1><<<grid, dim3(kPcThreads), 0, s>>>(op, rows, C, inner, lg_us, static_cast<uint32_t>(segs));
  return true;
}

inline unsigned grid_for(int64_t work_items, int64_t per_block, int64_t cap) {
  int64_t g = ceil_div(work_items, per_block);
  if (g < 1) g = 1;
  if (g > cap) g = cap;
  return static_cast<unsigned>(g);
}

template <bool SIGNED, bool FUSED>
int quantize_launch_as(const float* x, void* q, int64_t n, QParamsArg qp, hipStream_t s) {
  uint8_t* qb = static_cast<uint8_t*>(q);
  if (aligned(x, 16) && aligned(q, 4)) {
    const int64_t n4 = n / 4;
    const int64_t blocks = n4 == 0 ? 1 : ceil_div(n4, kQThreads * kUnrollQD);
    if (blocks > 0x7fffffff) return TMQ_ERR_UNSUPPORTED;
    if (n >= kStreamOutCodes)
      quantize_vec_kernel<SIGNED, FUSED, true><<<dim3(blocks), dim3(kQThreads), 0, s>>>(
          reinterpret_cast<const v4f*>(x), reinterpret_cast<uint32_t*>(q), n4, x, qb, n, qp);
    else
      quantize_vec_kernel<SIGNED, FUSED><<<dim3(blocks), dim3(kQThreads), 0, s>>>(
          reinterpret_cast<const v4f*>(x), reinterpret_cast<uint32_t*>(q), n4, x, qb, n, qp);
  } else {
    const unsigned g = grid_for(n, kThreads, 65536);
    quantize_scalar_kernel<SIGNED, FUSED><<<dim3(g), dim3(kThreads), 0, s>>>(x, qb, n, qp);
  }
  return launch_status();
}

int quantize_launch(const float* x, void* q, int64_t n, QParamsArg qp, int q_signed, hipStream_t s,
                    bool fused = false) {
  if (n == 0) return TMQ_OK;
  if (fused)
    return q_signed ? quantize_launch_as<true, true>(x, q, n, qp, s) : quantize_launch_as<false, true>(x, q, n, qp, s);
  return q_signed ? quantize_launch_as<true, false>(x, q, n, qp, s) : quantize_launch_as<false, false>(x, q, n, qp, s);
}

bool zp_in_range(int64_t zp, int q_signed) {
  return q_signed ? (zp >= -128 && zp <= 127) : (zp >= 0 && zp <= 255);
}

}  // namespace
}  // namespace tmq

using namespace tmq;

TMQ_EXPORT int tmq_quantize_per_tensor(const float* x, void* q, int64_t n, double scale,
                                       int64_t zero_point, int q_signed, tmq_stream_t stream) {
  if (n < 0 || (n > 0 && (x == nullptr || q == nullptr))) return TMQ_ERR_INVALID_ARGUMENT;
  if (!zp_in_range(zero_point, q_signed)) return TMQ_ERR_INVALID_ARGUMENT;
  QParamsArg qp;
  qp.inv = 1.0f / static_cast<float>(scale);
  qp.zp_f = static_cast<float>(zero_point);
  qp.dev = nullptr;
  return quantize_launch(x, q, n, qp, q_signed, as_stream(stream));
}

TMQ_EXPORT int tmq_quantize_per_tensor_dev(const float* x, void* q, int64_t n,
                                           const tmq_qparams* qparams, int q_signed,
                                           tmq_stream_t stream) {
  if (n < 0 || qparams == nullptr || (n > 0 && (x == nullptr || q == nullptr)))
    return TMQ_ERR_INVALID_ARGUMENT;
  QParamsArg qp;
  qp.inv = 0.f;
  qp.zp_f = 0.f;
  qp.dev = qparams;
  return quantize_launch(x, q, n, qp, q_signed, as_stream(stream));
}

TMQ_EXPORT int tmq_dequantize_per_tensor(const void* q, float* r, int64_t n, double scale,
                                         int64_t zero_point, int q_signed, tmq_stream_t stream) {
  if (n < 0 || (n > 0 && (r == nullptr || q == nullptr))) return TMQ_ERR_INVALID_ARGUMENT;
  if (!zp_in_range(zero_point, q_signed)) return TMQ_ERR_INVALID_ARGUMENT;
  if (n == 0) return TMQ_OK;
  hipStream_t s = as_stream(stream);
  const float scale_f = static_cast<float>(scale);
  const int zp = static_cast<int>(zero_point);
  const uint8_t* qb = static_cast<const uint8_t*>(q);
  if (aligned(r, 16) && aligned(q, 4)) {
    const int64_t n4 = n / 4;
    const int64_t blocks = n4 == 0 ? 1 : ceil_div(n4, kDqThreads * kUnrollQD);
    if (blocks > 0x7fffffff) return TMQ_ERR_UNSUPPORTED;
    auto* q4 = reinterpret_cast<const uint32_t*>(q);
    auto* r4 = reinterpret_cast<v4f*>(r);
    if (q_signed)
      dequantize_vec_kernel<true><<<dim3(blocks), dim3(kDqThreads), 0, s>>>(q4, r4, n4, qb, r, n, scale_f, zp);
    else
      dequantize_vec_kernel<false><<<dim3(blocks), dim3(kDqThreads), 0, s>>>(q4, r4, n4, qb, r, n, scale_f, zp);
  } else {
    const unsigned g = grid_for(n, kThreads, 65536);
    if (q_signed)
      dequantize_scalar_kernel<true><<<dim3(g), dim3(kThreads), 0, s>>>(qb, r, n, scale_f, zp);
    else
      dequantize_scalar_kernel<false><<<dim3(g), dim3(kThreads), 0, s>>>(qb, r, n, scale_f, zp);
  }
  return launch_status();
}

TMQ_EXPORT size_t tmq_minmax_workspace_bytes(int64_t n) {
  (void)n;
  return static_cast<size_t>(kMinMaxMaxBlocks) * 2 * sizeof(float);
}

TMQ_EXPORT int tmq_minmax(const float* x, int64_t n, float* minmax, void* workspace,
                          size_t workspace_bytes, tmq_stream_t stream) {
  if (n < 0 || minmax == nullptr || (n > 0 && x == nullptr)) return TMQ_ERR_INVALID_ARGUMENT;
  if (workspace == nullptr || workspace_bytes < tmq_minmax_workspace_bytes(n) ||
      !aligned(workspace, 4))
    return TMQ_ERR_WORKSPACE;
  if (!aligned(x, 4)) return TMQ_ERR_ALIGNMENT;
  hipStream_t s = as_stream(stream);
  float* partials = static_cast<float*>(workspace);
  // elements before the first 16-byte boundary are handled one by one
  int64_t head = 0;
  if (n > 0) {
    const uintptr_t mis = reinterpret_cast<uintptr_t>(x) & 15u;
    head = mis == 0 ? 0 : static_cast<int64_t>((16 - mis) / 4);
    if (head > n) head = n;
  }
  const int64_t n4 = (n - head) / 4;
  const unsigned g = grid_for(n4, kThreads * kUnroll, kMinMaxMaxBlocks);
  minmax_partial_kernel<false><<<dim3(g), dim3(kThreads), 0, s>>>(
      reinterpret_cast<const v4f*>(x + head), n4, x, head, n, partials);
  if (launch_status() != TMQ_OK) return TMQ_ERR_LAUNCH;
  minmax_final_kernel<<<dim3(1), dim3(kThreads), 0, s>>>(partials, static_cast<int>(g), minmax);
  return launch_status();
}

TMQ_EXPORT int tmq_choose_qparams_dev(const float* minmax, int q_signed, int reduce_range,
                                      tmq_qparams* qparams, tmq_stream_t stream) {
  if (minmax == nullptr || qparams == nullptr) return TMQ_ERR_INVALID_ARGUMENT;
  choose_qparams_kernel<<<dim3(1), dim3(kWave), 0, as_stream(stream)>>>(
      minmax, q_signed ? -128 : 0, q_signed ? 127 : 255, reduce_range, qparams);
  return launch_status();
}

TMQ_EXPORT int tmq_quantize_per_tensor_dynamic_dev(const float* x, void* q, int64_t n, int q_signed,
                                                   int reduce_range, int rounding, tmq_qparams* qparams,
                                                   void* workspace, size_t workspace_bytes, tmq_stream_t stream) {
  if (n < 0 || qparams == nullptr || (n > 0 && (x == nullptr || q == nullptr))) return TMQ_ERR_INVALID_ARGUMENT;
  if (rounding != TMQ_ROUND_PRODUCT && rounding != TMQ_ROUND_FUSED) return TMQ_ERR_INVALID_ARGUMENT;
  const bool fused = rounding == TMQ_ROUND_FUSED;
  if (!aligned(x, 4)) return TMQ_ERR_ALIGNMENT;
  hipStream_t s = as_stream(stream);
  const int qmin = q_signed ? -128 : 0, qmax = q_signed ? 127 : 255;
  if (n <= kDynSmallMax) {
    const bool vec = aligned(x, 16) && aligned(q, 4);
    uint8_t* qb = static_cast<uint8_t*>(q);
    const dim3 one(1), block(kDynSmallThreads);
    if (q_signed && fused)
      dynamic_quantize_small_kernel<true, true><<<one, block, 0, s>>>(x, qb, n, qmin, qmax, reduce_range, vec, qparams);
    else if (q_signed)
      dynamic_quantize_small_kernel<true, false><<<one, block, 0, s>>>(x, qb, n, qmin, qmax, reduce_range, vec, qparams);
    else if (fused)
      dynamic_quantize_small_kernel<false, true><<<one, block, 0, s>>>(x, qb, n, qmin, qmax, reduce_range, vec, qparams);
    else
      dynamic_quantize_small_kernel<false, false><<<one, block, 0, s>>>(x, qb, n, qmin, qmax, reduce_range, vec, qparams);
    return launch_status();
  }
  if (workspace == nullptr || workspace_bytes < tmq_minmax_workspace_bytes(n) || !aligned(workspace, 4))
    return TMQ_ERR_WORKSPACE;
  float* partials = static_cast<float*>(workspace);
  if (n <= kDynKeepMax && aligned(x, 16) && aligned(q, 4) && aligned(workspace, 8)) {
    // Inputs that fit the last-level cache with room to spare (where the launches, not the
    // bytes, are what counts): two launches -- partial ranges, read with ordinary loads so
    // that the second pass finds the input cached, then the quantizer whose blocks finish
    // the reduction themselves.
    const int64_t n4 = n / 4;
    const unsigned g = grid_for(n4, kThreads * kUnroll, kDynPartials);
    const v4f* x4 = reinterpret_cast<const v4f*>(x);
    minmax_partial_kernel<true><<<dim3(g), dim3(kThreads), 0, s>>>(x4, n4, x, 0, n, partials);
    if (launch_status() != TMQ_OK) return TMQ_ERR_LAUNCH;
    const dim3 grid(grid_for(n4, kThreads * kUnrollQD, kDynQBlocks)), block(kThreads);
    uint32_t* q4 = static_cast<uint32_t*>(q);
    uint8_t* qb = static_cast<uint8_t*>(q);
    const int cnt = static_cast<int>(g);
    if (q_signed && fused)
      quantize_after_minmax_kernel<true, true><<<grid, block, 0, s>>>(x4, q4, n4, x, qb, n, partials, cnt, qmin, qmax, reduce_range, qparams);
    else if (q_signed)
      quantize_after_minmax_kernel<true, false><<<grid, block, 0, s>>>(x4, q4, n4, x, qb, n, partials, cnt, qmin, qmax, reduce_range, qparams);
    else if (fused)
      quantize_after_minmax_kernel<false, true><<<grid, block, 0, s>>>(x4, q4, n4, x, qb, n, partials, cnt, qmin, qmax, reduce_range, qparams);
    else
      quantize_after_minmax_kernel<false, false><<<grid, block, 0, s>>>(x4, q4, n4, x, qb, n, partials, cnt, qmin, qmax, reduce_range, qparams);
    return launch_status();
  }
  // larger inputs (streamed past the caches) and unaligned buffers: range, parameters and
  // codes in three launches
  const uintptr_t mis = reinterpret_cast<uintptr_t>(x) & 15u;
  int64_t head = mis == 0 ? 0 : static_cast<int64_t>((16 - mis) / 4);
  if (head > n) head = n;
  const int64_t n4 = (n - head) / 4;
  const unsigned g = grid_for(n4, kThreads * kUnroll, kMinMaxMaxBlocks);
  minmax_partial_kernel<false><<<dim3(g), dim3(kThreads), 0, s>>>(reinterpret_cast<const v4f*>(x + head), n4, x, head,
                                                           n, partials);
  if (launch_status() != TMQ_OK) return TMQ_ERR_LAUNCH;
  minmax_final_choose_kernel<<<dim3(1), dim3(kThreads), 0, s>>>(partials, static_cast<int>(g), qmin, qmax,
                                                                reduce_range, nullptr, qparams);
  if (launch_status() != TMQ_OK) return TMQ_ERR_LAUNCH;
  QParamsArg qp;
  qp.inv = 0.f;
  qp.zp_f = 0.f;
  qp.dev = qparams;
  return quantize_launch(x, q, n, qp, q_signed, s, fused);
}

TMQ_EXPORT int tmq_choose_qparams_host(float min, float max, int q_signed, int reduce_range,
                                       double* scale, int32_t* zero_point) {
  if (scale == nullptr || zero_point == nullptr || !(min <= max)) return TMQ_ERR_INVALID_ARGUMENT;
  choose_qparams(min, max, q_signed ? -128 : 0, q_signed ? 127 : 255, reduce_range != 0, scale,
                 zero_point);
  return TMQ_OK;
}

namespace {
bool pc_args_ok(const void* a, const void* b, int64_t outer, int64_t C, int64_t inner,
                const double* scales, const int64_t* zps) {
  if (outer < 0 || C < 0 || inner < 0) return false;
  const bool empty = outer == 0 || C == 0 || inner == 0;
  if (!empty && (a == nullptr || b == nullptr || scales == nullptr || zps == nullptr)) return false;
  return true;
}
}  // namespace

TMQ_EXPORT int tmq_quantize_per_channel(const float* x, void* q, int64_t outer, int64_t channels,
                                        int64_t inner, const double* scales,
                                        const int64_t* zero_points, int q_signed,
                                        tmq_stream_t stream) {
  if (!pc_args_ok(x, q, outer, channels, inner, scales, zero_points))
    return TMQ_ERR_INVALID_ARGUMENT;
  const int64_t n = outer * channels * inner;
  if (n == 0) return TMQ_OK;
  hipStream_t s = as_stream(stream);
  uint8_t* qb = static_cast<uint8_t*>(q);
  const bool vec = inner % 4 == 0 && aligned(x, 16) && aligned(q, 4);
  if (q_signed ? launch_pc_rows(PcQuantize<true>{x, qb, scales, zero_points}, outer, channels, inner, vec, s)
               : launch_pc_rows(PcQuantize<false>{x, qb, scales, zero_points}, outer, channels, inner, vec, s))
    return launch_status();
  const unsigned g = grid_for(n, kThreads * (vec ? 4 : 1), 1 << 20);
  if (vec) {
    if (q_signed)
      quantize_pc_kernel<true, 4><<<dim3(g), dim3(kThreads), 0, s>>>(x, qb, n, channels, inner, scales, zero_points);
    else
      quantize_pc_kernel<false, 4><<<dim3(g), dim3(kThreads), 0, s>>>(x, qb, n, channels, inner, scales, zero_points);
  } else {
    if (q_signed)
      quantize_pc_kernel<true, 1><<<dim3(g), dim3(kThreads), 0, s>>>(x, qb, n, channels, inner, scales, zero_points);
    else
      quantize_pc_kernel<false, 1><<<dim3(g), dim3(kThreads), 0, s>>>(x, qb, n, channels, inner, scales, zero_points);
  }
  return launch_status();
}

TMQ_EXPORT int tmq_dequantize_per_channel(const void* q, float* r, int64_t outer, int64_t channels,
                                          int64_t inner, const double* scales,
                                          const int64_t* zero_points, int q_signed,
                                          tmq_stream_t stream) {
  if (!pc_args_ok(q, r, outer, channels, inner, scales, zero_points))
    return TMQ_ERR_INVALID_ARGUMENT;
  const int64_t n = outer * channels * inner;
  if (n == 0) return TMQ_OK;
  hipStream_t s = as_stream(stream);
  const uint8_t* qb = static_cast<const uint8_t*>(q);
  const bool vec = inner % 4 == 0 && aligned(r, 16) && aligned(q, 4);
  if (q_signed ? launch_pc_rows(PcDequantize<true>{qb, r, scales, zero_points}, outer, channels, inner, vec, s)
               : launch_pc_rows(PcDequantize<false>{qb, r, scales, zero_points}, outer, channels, inner, vec, s))
    return launch_status();
  const unsigned g = grid_for(n, kThreads * (vec ? 4 : 1), 1 << 20);
  if (vec) {
    if (q_signed)
      dequantize_pc_kernel<true, 4><<<dim3(g), dim3(kThreads), 0, s>>>(qb, r, n, channels, inner, scales, zero_points);
    else
      dequantize_pc_kernel<false, 4><<<dim3(g), dim3(kThreads), 0, s>>>(qb, r, n, channels, inner, scales, zero_points);
  } else {
    if (q_signed)
      dequantize_pc_kernel<true, 1><<<dim3(g), dim3(kThreads), 0, s>>>(qb, r, n, channels, inner, scales, zero_points);
    else
      dequantize_pc_kernel<false, 1><<<dim3(g), dim3(kThreads), 0, s>>>(qb, r, n, channels, inner, scales, zero_points);
  }
  return launch_status();
}

TMQ_EXPORT int tmq_quantize_per_channel_float_qparams(const float* x, void* q, int64_t outer,
                                                      int64_t channels, int64_t inner,
                                                      const float* scales, const float* zero_points,
                                                      int q_signed, tmq_stream_t stream) {
  if (outer < 0 || channels < 0 || inner < 0) return TMQ_ERR_INVALID_ARGUMENT;
  const int64_t n = outer * channels * inner;
  if (n == 0) return TMQ_OK;
  if (x == nullptr || q == nullptr || scales == nullptr || zero_points == nullptr)
    return TMQ_ERR_INVALID_ARGUMENT;
  hipStream_t s = as_stream(stream);
  uint8_t* qb = static_cast<uint8_t*>(q);
  const bool vec = inner % 4 == 0 && aligned(x, 16) && aligned(q, 4);
  if (q_signed ? launch_pc_rows(PcfQuantize<true>{x, qb, scales, zero_points}, outer, channels, inner, vec, s)
               : launch_pc_rows(PcfQuantize<false>{x, qb, scales, zero_points}, outer, channels, inner, vec, s))
    return launch_status();
  const unsigned g = grid_for(n, kThreads * (vec ? 4 : 1), 1 << 20);
  if (vec) {
    if (q_signed)
      quantize_pcf_kernel<true, 4><<<dim3(g), dim3(kThreads), 0, s>>>(x, qb, n, channels, inner, scales, zero_points);
    else
      quantize_pcf_kernel<false, 4><<<dim3(g), dim3(kThreads), 0, s>>>(x, qb, n, channels, inner, scales, zero_points);
  } else {
    if (q_signed)
      quantize_pcf_kernel<true, 1><<<dim3(g), dim3(kThreads), 0, s>>>(x, qb, n, channels, inner, scales, zero_points);
    else
      quantize_pcf_kernel<false, 1><<<dim3(g), dim3(kThreads), 0, s>>>(x, qb, n, channels, inner, scales, zero_points);
  }
  return launch_status();
}

TMQ_EXPORT int tmq_dequantize_per_channel_float_qparams(const void* q, float* r, int64_t outer,
                                                        int64_t channels, int64_t inner,
                                                        const float* scales, const float* zero_points,
                                                        int q_signed, tmq_stream_t stream) {
  if (outer < 0 || channels < 0 || inner < 0) return TMQ_ERR_INVALID_ARGUMENT;
  const int64_t n = outer * channels * inner;
  if (n == 0) return TMQ_OK;
  if (r == nullptr || q == nullptr || scales == nullptr || zero_points == nullptr)
    return TMQ_ERR_INVALID_ARGUMENT;
  hipStream_t s = as_stream(stream);
  const uint8_t* qb = static_cast<const uint8_t*>(q);
  const bool vec = inner % 4 == 0 && aligned(r, 16) && aligned(q, 4);
  if (q_signed ? launch_pc_rows(PcfDequantize<true>{qb, r, scales, zero_points}, outer, channels, inner, vec, s)
               : launch_pc_rows(PcfDequantize<false>{qb, r, scales, zero_points}, outer, channels, inner, vec, s))
    return launch_status();
  const unsigned g = grid_for(n, kThreads * (vec ? 4 : 1), 1 << 20);
  if (vec) {
    if (q_signed)
      dequantize_pcf_kernel<true, 4><<<dim3(g), dim3(kThreads), 0, s>>>(qb, r, n, channels, inner, scales, zero_points);
    else
      dequantize_pcf_kernel<false, 4><<<dim3(g), dim3(kThreads), 0, s>>>(qb, r, n, channels, inner, scales, zero_points);
  } else {
    if (q_signed)
      dequantize_pcf_kernel<true, 1><<<dim3(g), dim3(kThreads), 0, s>>>(qb, r, n, channels, inner, scales, zero_points);
    else
      dequantize_pcf_kernel<false, 1><<<dim3(g), dim3(kThreads), 0, s>>>(qb, r, n, channels, inner, scales, zero_points);
  }
  return launch_status();
}

TMQ_EXPORT const char* tmq_status_string(int status) {
  switch (status) {
    case TMQ_OK: return "ok";
    case TMQ_ERR_INVALID_ARGUMENT: return "invalid argument";
    case TMQ_ERR_UNSUPPORTED: return "unsupported configuration";
    case TMQ_ERR_WORKSPACE: return "workspace missing or too small";
    case TMQ_ERR_LAUNCH: return "HIP launch failed";
    case TMQ_ERR_ALIGNMENT: return "pointer or leading dimension not aligned";
    default: return "unknown status";
  }
}

TMQ_EXPORT int tmq_version(void) { return TMQ_VERSION; }
