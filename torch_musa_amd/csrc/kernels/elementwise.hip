// Elementwise kernels on quantized tensors for gfx950: quantized::add /
// add_relu and relu of a per-tensor quantized tensor.  HBM streaming kernels:
// a lane moves 16 bytes (16 codes) per access, consecutive lanes touch
// consecutive addresses, a few independent accesses per thread.
//
// quantized::add follows the arithmetic of PyTorch's CPU kernel (the vector
// body of qadd_kernel in ATen/native/quantized/cpu/kernels/QuantizedOpKernels.cpp):
//   a = fma(float(qa), a_scale, fl(-a_zp * a_scale))      (dequantize with a premultiplied zero point)
//   b = fma(float(qb), b_scale, fl(-b_zp * b_scale))
//   c = a + b;   relu: c = max(c, 0)
//   q = clamp(rne(c * fl(1 / out_scale)) + out_zp)
// every step in fp32.
#include "common.h"

namespace tmq {
namespace {

constexpr int kEwThreads = 256;
constexpr int kEwUnroll = 2;  // 16-byte accesses in flight per thread and operand

struct AddParams {
  float a_scale, a_premul, b_scale, b_premul, inv_out, out_zp_f;
};

template <bool SIGNED>
__device__ __forceinline__ float code_to_float(uint32_t word, int j) {
  if constexpr (SIGNED) {
    return static_cast<float>(static_cast<int>(static_cast<int8_t>((word >> (8 * j)) & 0xffu)));
  } else {
    // one v_cvt_f32_ubyteN instruction
    return static_cast<float>((word >> (8 * j)) & 0xffu);
  }
}

template <bool SIGNED, bool RELU>
__device__ __forceinline__ uint32_t add_four(uint32_t wa, uint32_t wb, const AddParams& p) {
  uint32_t packed = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float a = __builtin_fmaf(code_to_float<SIGNED>(wa, j), p.a_scale, p.a_premul);
    const float b = __builtin_fmaf(code_to_float<SIGNED>(wb, j), p.b_scale, p.b_premul);
    float c = a + b;
    if (RELU) c = __builtin_fmaxf(c, 0.f);
    const float t = c * p.inv_out;
    float r = __builtin_rintf(t) + p.out_zp_f;
    if constexpr (SIGNED) {
      r = __builtin_amdgcn_fmed3f(r, -128.f, 127.f);
      packed |= (static_cast<uint32_t>(static_cast<int>(r)) & 0xffu) << (8 * j);
    } else {
      // the conversion rounds an integral value exactly and saturates to [0, 255]
      packed = __builtin_amdgcn_cvt_pk_u8_f32(r, j, packed);
    }
  }
  return packed;
}

template <bool SIGNED, bool RELU>
__device__ __forceinline__ v4i add_sixteen(v4i a, v4i b, const AddParams& p) {
  return v4i{static_cast<int>(add_four<SIGNED, RELU>(a.x, b.x, p)),
             static_cast<int>(add_four<SIGNED, RELU>(a.y, b.y, p)),
             static_cast<int>(add_four<SIGNED, RELU>(a.z, b.z, p)),
             static_cast<int>(add_four<SIGNED, RELU>(a.w, b.w, p))};
}

// n16 full 16-byte groups through the vector path, the n - 16*n16 (< 16)
// trailing codes one by one in block 0.
template <bool SIGNED, bool RELU>
__global__ __launch_bounds__(kEwThreads) void qadd_vec_kernel(const v4i* __restrict__ a16,
                                                              const v4i* __restrict__ b16,
                                                              v4i* __restrict__ o16, int64_t n16,
                                                              const uint8_t* __restrict__ a,
                                                              const uint8_t* __restrict__ b,
                                                              uint8_t* __restrict__ o, int64_t n,
                                                              AddParams p) {
  const int64_t base = static_cast<int64_t>(blockIdx.x) * (kEwThreads * kEwUnroll) + threadIdx.x;
  v4i va[kEwUnroll], vb[kEwUnroll];
  if (base - threadIdx.x + kEwThreads * kEwUnroll <= n16) {
#pragma unroll
    for (int u = 0; u < kEwUnroll; ++u) {
      va[u] = __builtin_nontemporal_load(&a16[base + u * kEwThreads]);
      vb[u] = __builtin_nontemporal_load(&b16[base + u * kEwThreads]);
    }
#pragma unroll
    for (int u = 0; u < kEwUnroll; ++u) o16[base + u * kEwThreads] = add_sixteen<SIGNED, RELU>(va[u], vb[u], p);
  } else {
#pragma unroll
    for (int u = 0; u < kEwUnroll; ++u) {
      const int64_t i = base + u * kEwThreads;
      if (i < n16) o16[i] = add_sixteen<SIGNED, RELU>(a16[i], b16[i], p);
    }
  }
  if (blockIdx.x == 0) {
    const int64_t i = 16 * n16 + threadIdx.x;
    if (i < n) o[i] = static_cast<uint8_t>(add_four<SIGNED, RELU>(a[i], b[i], p) & 0xffu);
  }
}

template <bool SIGNED, bool RELU>
__global__ __launch_bounds__(kEwThreads) void qadd_scalar_kernel(const uint8_t* __restrict__ a,
                                                                 const uint8_t* __restrict__ b,
                                                                 uint8_t* __restrict__ o, int64_t n,
                                                                 AddParams p) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kEwThreads;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kEwThreads + threadIdx.x; i < n; i += stride)
    o[i] = static_cast<uint8_t>(add_four<SIGNED, RELU>(a[i], b[i], p) & 0xffu);
}

// relu of a quantized tensor keeps scale and zero point: q = max(q, zero_point).
// Four codes per dword: even and odd bytes are spread into two pairs of 16-bit
// lanes and clamped with the packed 16-bit integer maximum; signed codes are
// mapped to unsigned order with x ^ 0x80 first (zp likewise) and back after.
typedef unsigned short us2 __attribute__((ext_vector_type(2)));
template <bool SIGNED>
__device__ __forceinline__ uint32_t relu_four(uint32_t w, int zp) {
  const uint32_t bias = SIGNED ? 0x80808080u : 0u;
  const uint32_t z = static_cast<uint32_t>(SIGNED ? zp + 128 : zp);
  const uint32_t z2 = z | (z << 16);
  const uint32_t u = w ^ bias;
  const uint32_t even = u & 0x00ff00ffu, odd = (u >> 8) & 0x00ff00ffu;
  const us2 me = __builtin_elementwise_max(__builtin_bit_cast(us2, even), __builtin_bit_cast(us2, z2));
  const us2 mo = __builtin_elementwise_max(__builtin_bit_cast(us2, odd), __builtin_bit_cast(us2, z2));
  return (__builtin_bit_cast(uint32_t, me) | (__builtin_bit_cast(uint32_t, mo) << 8)) ^ bias;
}

template <bool SIGNED>
__global__ __launch_bounds__(kEwThreads) void qrelu_vec_kernel(const v4i* __restrict__ x16,
                                                               v4i* __restrict__ y16, int64_t n16,
                                                               const uint8_t* __restrict__ x,
                                                               uint8_t* __restrict__ y, int64_t n, int zp) {
  const int64_t base = static_cast<int64_t>(blockIdx.x) * (kEwThreads * kEwUnroll) + threadIdx.x;
#pragma unroll
  for (int u = 0; u < kEwUnroll; ++u) {
    const int64_t i = base + u * kEwThreads;
    if (i < n16) {
      const v4i v = x16[i];
      y16[i] = v4i{static_cast<int>(relu_four<SIGNED>(v.x, zp)), static_cast<int>(relu_four<SIGNED>(v.y, zp)),
                   static_cast<int>(relu_four<SIGNED>(v.z, zp)), static_cast<int>(relu_four<SIGNED>(v.w, zp))};
    }
  }
  if (blockIdx.x == 0) {
    const int64_t i = 16 * n16 + threadIdx.x;
    if (i < n) y[i] = static_cast<uint8_t>(relu_four<SIGNED>(x[i], zp) & 0xffu);
  }
}

template <bool SIGNED>
__global__ __launch_bounds__(kEwThreads) void qrelu_scalar_kernel(const uint8_t* __restrict__ x,
                                                                  uint8_t* __restrict__ y, int64_t n, int zp) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kEwThreads;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kEwThreads + threadIdx.x; i < n; i += stride)
    y[i] = static_cast<uint8_t>(relu_four<SIGNED>(x[i], zp) & 0xffu);
}

bool zp_ok(int32_t zp, int q_signed) { return q_signed ? (zp >= -128 && zp <= 127) : (zp >= 0 && zp <= 255); }

template <bool SIGNED, bool RELU>
int launch_add(const void* a, const void* b, void* out, int64_t n, const AddParams& p, hipStream_t s) {
  const uint8_t* ab = static_cast<const uint8_t*>(a);
  const uint8_t* bb = static_cast<const uint8_t*>(b);
  uint8_t* ob = static_cast<uint8_t*>(out);
  if (aligned(a, 16) && aligned(b, 16) && aligned(out, 16)) {
    const int64_t n16 = n / 16;
    const int64_t blocks = n16 == 0 ? 1 : ceil_div(n16, kEwThreads * kEwUnroll);
    if (blocks > 0x7fffffff) return TMQ_ERR_UNSUPPORTED;
    qadd_vec_kernel<SIGNED, RELU><<<dim3(static_cast<unsigned>(blocks)), dim3(kEwThreads), 0, s>>>(
        static_cast<const v4i*>(a), static_cast<const v4i*>(b), static_cast<v4i*>(out), n16, ab, bb, ob, n, p);
  } else {
    int64_t g = ceil_div(n, kEwThreads);
    g = g > 65536 ? 65536 : g;
    qadd_scalar_kernel<SIGNED, RELU><<<dim3(static_cast<unsigned>(g)), dim3(kEwThreads), 0, s>>>(ab, bb, ob, n, p);
  }
  return launch_status();
}

}  // namespace
}  // namespace tmq

using namespace tmq;

TMQ_EXPORT int tmq_qadd(const void* a, const void* b, void* out, int64_t n, float a_scale,
                        int32_t a_zero_point, float b_scale, int32_t b_zero_point, float out_scale,
                        int32_t out_zero_point, int q_signed, int relu, tmq_stream_t stream) {
  if (n < 0 || (n > 0 && (a == nullptr || b == nullptr || out == nullptr))) return TMQ_ERR_INVALID_ARGUMENT;
  if (!zp_ok(a_zero_point, q_signed) || !zp_ok(b_zero_point, q_signed) || !zp_ok(out_zero_point, q_signed))
    return TMQ_ERR_INVALID_ARGUMENT;
  if (!(out_scale > 0.f)) return TMQ_ERR_INVALID_ARGUMENT;
  if (n == 0) return TMQ_OK;
  AddParams p;
  p.a_scale = a_scale;
  p.a_premul = -static_cast<float>(a_zero_point) * a_scale;
  p.b_scale = b_scale;
  p.b_premul = -static_cast<float>(b_zero_point) * b_scale;
  p.inv_out = 1.0f / out_scale;
  p.out_zp_f = static_cast<float>(out_zero_point);
  hipStream_t s = as_stream(stream);
  if (q_signed) return relu ? launch_add<true, true>(a, b, out, n, p, s) : launch_add<true, false>(a, b, out, n, p, s);
  return relu ? launch_add<false, true>(a, b, out, n, p, s) : launch_add<false, false>(a, b, out, n, p, s);
}

TMQ_EXPORT int tmq_qrelu(const void* x, void* y, int64_t n, int32_t zero_point, int q_signed,
                         tmq_stream_t stream) {
  if (n < 0 || (n > 0 && (x == nullptr || y == nullptr))) return TMQ_ERR_INVALID_ARGUMENT;
  if (!zp_ok(zero_point, q_signed)) return TMQ_ERR_INVALID_ARGUMENT;
  if (n == 0) return TMQ_OK;
  hipStream_t s = as_stream(stream);
  const uint8_t* xb = static_cast<const uint8_t*>(x);
  uint8_t* yb = static_cast<uint8_t*>(y);
  if (aligned(x, 16) && aligned(y, 16)) {
    const int64_t n16 = n / 16;
    const int64_t blocks = n16 == 0 ? 1 : ceil_div(n16, kEwThreads * kEwUnroll);
    if (blocks > 0x7fffffff) return TMQ_ERR_UNSUPPORTED;
    const dim3 grid(static_cast<unsigned>(blocks)), block(kEwThreads);
    if (q_signed)
      qrelu_vec_kernel<true><<<grid, block, 0, s>>>(static_cast<const v4i*>(x), static_cast<v4i*>(y), n16, xb, yb, n, zero_point);
    else
      qrelu_vec_kernel<false><<<grid, block, 0, s>>>(static_cast<const v4i*>(x), static_cast<v4i*>(y), n16, xb, yb, n, zero_point);
  } else {
    int64_t g = ceil_div(n, kEwThreads);
    g = g > 65536 ? 65536 : g;
    const dim3 grid(static_cast<unsigned>(g)), block(kEwThreads);
    if (q_signed)
      qrelu_scalar_kernel<true><<<grid, block, 0, s>>>(xb, yb, n, zero_point);
    else
      qrelu_scalar_kernel<false><<<grid, block, 0, s>>>(xb, yb, n, zero_point);
  }
  return launch_status();
}
