// Elementwise and data-movement kernels on quantized tensors for gfx950:
// quantized::add / add_relu, relu, the row requantiser behind quantized::cat
// and max pooling over NHWC codes.  HBM streaming kernels:
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
constexpr int kReluUnroll = 4;  // one operand only: twice as many per thread

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
  const int64_t base = static_cast<int64_t>(blockIdx.x) * (kEwThreads * kReluUnroll) + threadIdx.x;
  auto relu16 = [&](v4i v) {
    return v4i{static_cast<int>(relu_four<SIGNED>(v.x, zp)), static_cast<int>(relu_four<SIGNED>(v.y, zp)),
               static_cast<int>(relu_four<SIGNED>(v.z, zp)), static_cast<int>(relu_four<SIGNED>(v.w, zp))};
  };
  v4i v[kReluUnroll];
  if (base - threadIdx.x + kEwThreads * kReluUnroll <= n16) {
    // whole block inside the array: all loads first (read once: non-temporal), then all stores
#pragma unroll
    for (int u = 0; u < kReluUnroll; ++u) v[u] = __builtin_nontemporal_load(&x16[base + u * kEwThreads]);
#pragma unroll
    for (int u = 0; u < kReluUnroll; ++u) y16[base + u * kEwThreads] = relu16(v[u]);
  } else {
#pragma unroll
    for (int u = 0; u < kReluUnroll; ++u) {
      const int64_t i = base + u * kEwThreads;
      if (i < n16) y16[i] = relu16(x16[i]);
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

// ---------------------------------------------------------------------------
// quantized::cat building block: rows of `in_row` codes are requantised (or
// copied, when the quantization parameters agree) into a wider output row at a
// column offset:  y[o][off + j] = Q_out(DQ_in(x[o][j])).
//   DQ: r = fl(in_scale) * float(q - in_zp)          (the per-tensor dequantizer)
//   Q : q' = clamp(rne(r * fl(1/out_scale)) + out_zp)  (the per-tensor quantizer)
// ---------------------------------------------------------------------------
struct RequantParams {
  float in_scale, inv_out, out_zp_f;
  int in_zp;
  int identity;
};

template <bool SIGNED>
__device__ __forceinline__ uint32_t requant_codes4(uint32_t w, const RequantParams& p) {
  if (p.identity) return w;
  uint32_t packed = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint32_t byte = (w >> (8 * j)) & 0xffu;
    const int v = SIGNED ? static_cast<int>(static_cast<int8_t>(byte)) : static_cast<int>(byte);
    const float r = p.in_scale * static_cast<float>(v - p.in_zp);
    const float t = r * p.inv_out;
    float q = __builtin_rintf(t) + p.out_zp_f;
    if constexpr (SIGNED) {
      q = __builtin_amdgcn_fmed3f(q, -128.f, 127.f);
      packed |= (static_cast<uint32_t>(static_cast<int>(q)) & 0xffu) << (8 * j);
    } else {
      packed = __builtin_amdgcn_cvt_pk_u8_f32(q, j, packed);
    }
  }
  return packed;
}

// VEC = 16: rows, offset and pointers are multiples of 16 bytes; VEC = 1 otherwise.
template <bool SIGNED, int VEC>
__global__ __launch_bounds__(kEwThreads) void qcat_rows_kernel(const uint8_t* __restrict__ x,
                                                               uint8_t* __restrict__ y, int64_t outer,
                                                               int64_t in_row, int64_t out_row, int64_t off,
                                                               RequantParams p) {
  const int64_t per_row = in_row / VEC;
  const int64_t total = outer * per_row;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kEwThreads;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kEwThreads + threadIdx.x; i < total; i += stride) {
    const int64_t o = i / per_row, j = (i - o * per_row) * VEC;
    const uint8_t* src = x + o * in_row + j;
    uint8_t* dst = y + o * out_row + off + j;
    if constexpr (VEC == 16) {
      const v4i v = *reinterpret_cast<const v4i*>(src);
      *reinterpret_cast<v4i*>(dst) =
          v4i{static_cast<int>(requant_codes4<SIGNED>(v.x, p)), static_cast<int>(requant_codes4<SIGNED>(v.y, p)),
              static_cast<int>(requant_codes4<SIGNED>(v.z, p)), static_cast<int>(requant_codes4<SIGNED>(v.w, p))};
    } else {
      *dst = static_cast<uint8_t>(requant_codes4<SIGNED>(*src, p) & 0xffu);
    }
  }
}

// ---------------------------------------------------------------------------
// max pooling over NHWC codes: the maximum of the window's codes (the scale
// and zero point carry over; positions outside the image do not take part).
// VEC = 16: one thread per (output pixel, 16 channels), C % 16 == 0.
// ---------------------------------------------------------------------------
struct PoolShape {
  int64_t B, H, W, C, OH, OW;
  int kh, kw, sh, sw, ph, pw, dh, dw;
};

template <bool SIGNED>
__device__ __forceinline__ uint32_t max_codes4(uint32_t a, uint32_t b) {
  const uint32_t bias = SIGNED ? 0x80808080u : 0u;
  const uint32_t ua = a ^ bias, ub = b ^ bias;
  const us2 me = __builtin_elementwise_max(__builtin_bit_cast(us2, ua & 0x00ff00ffu),
                                           __builtin_bit_cast(us2, ub & 0x00ff00ffu));
  const us2 mo = __builtin_elementwise_max(__builtin_bit_cast(us2, (ua >> 8) & 0x00ff00ffu),
                                           __builtin_bit_cast(us2, (ub >> 8) & 0x00ff00ffu));
  return (__builtin_bit_cast(uint32_t, me) | (__builtin_bit_cast(uint32_t, mo) << 8)) ^ bias;
}

// Running maximum of 16 codes (four words) over many taps at three vector
// operations per word and tap.  The bytes of a word are compared as the two
// 16-bit lanes of a packed maximum: the even bytes masked into the lanes' low
// halves; the odd bytes as they are -- a lane whose high byte is larger wins
// whatever its low byte holds, and only the high byte of that result is used.
// Signed codes are compared as code ^ 0x80 (flipped when the result is read).
template <bool SIGNED>
struct CodeMax16 {
  uint32_t even[4] = {0, 0, 0, 0}, odd[4] = {0, 0, 0, 0};
  // `take` false: the tap is outside the image and does not take part
  __device__ __forceinline__ void add(const v4i& v, bool take) {
    const uint32_t w[4] = {static_cast<uint32_t>(v.x), static_cast<uint32_t>(v.y), static_cast<uint32_t>(v.z),
                           static_cast<uint32_t>(v.w)};
    const uint32_t lowest = SIGNED ? 0x80808080u : 0u;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      uint32_t u = take ? w[j] : lowest;
      if (SIGNED) u ^= 0x80808080u;
      even[j] = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(us2, even[j]),
                                                                       __builtin_bit_cast(us2, u & 0x00ff00ffu)));
      odd[j] = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(us2, odd[j]),
                                                                      __builtin_bit_cast(us2, u)));
    }
  }
  __device__ __forceinline__ v4i result() const {
    uint32_t r[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) r[j] = ((odd[j] & 0xff00ff00u) | even[j]) ^ (SIGNED ? 0x80808080u : 0u);
    return v4i{static_cast<int>(r[0]), static_cast<int>(r[1]), static_cast<int>(r[2]), static_cast<int>(r[3])};
  }
};

template <bool SIGNED, int VEC>
__global__ __launch_bounds__(kEwThreads) void qmaxpool_kernel(const uint8_t* __restrict__ x,
                                                              uint8_t* __restrict__ y, PoolShape s) {
  const int64_t cv = s.C / VEC;
  const int64_t total = s.B * s.OH * s.OW * cv;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kEwThreads;
  const uint32_t lowest = SIGNED ? 0x80808080u : 0u;  // the smallest code in every byte
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kEwThreads + threadIdx.x; i < total; i += stride) {
    const int64_t c = (i % cv) * VEC;
    int64_t t = i / cv;
    const int64_t ow = t % s.OW;
    t /= s.OW;
    const int64_t oh = t % s.OH, b = t / s.OH;
    v4i m = {static_cast<int>(lowest), static_cast<int>(lowest), static_cast<int>(lowest), static_cast<int>(lowest)};
    for (int kh = 0; kh < s.kh; ++kh) {
      const int64_t ih = oh * s.sh - s.ph + static_cast<int64_t>(kh) * s.dh;
      if (ih < 0 || ih >= s.H) continue;
      for (int kw = 0; kw < s.kw; ++kw) {
        const int64_t iw = ow * s.sw - s.pw + static_cast<int64_t>(kw) * s.dw;
        if (iw < 0 || iw >= s.W) continue;
        const uint8_t* src = x + ((b * s.H + ih) * s.W + iw) * s.C + c;
        if constexpr (VEC == 16) {
          const v4i v = *reinterpret_cast<const v4i*>(src);
          m = v4i{static_cast<int>(max_codes4<SIGNED>(m.x, v.x)), static_cast<int>(max_codes4<SIGNED>(m.y, v.y)),
                  static_cast<int>(max_codes4<SIGNED>(m.z, v.z)), static_cast<int>(max_codes4<SIGNED>(m.w, v.w))};
        } else {
          m.x = static_cast<int>(max_codes4<SIGNED>(m.x, *src) & 0xffu) | (m.x & ~0xff);
        }
      }
    }
    uint8_t* dst = y + ((b * s.OH + oh) * s.OW + ow) * s.C + c;
    if constexpr (VEC == 16)
      *reinterpret_cast<v4i*>(dst) = m;
    else
      *dst = static_cast<uint8_t>(m.x & 0xff);
  }
}

// The common 3x3 window (any stride and padding, dilation 1), 16 channels per
// thread: all nine loads are issued before the first maximum is taken (taps
// outside the image load a clamped address and are then replaced by the lowest
// code), where the general kernel's tap loop waits for each load in turn.
template <bool SIGNED>
__global__ __launch_bounds__(kEwThreads) void qmaxpool_k3_kernel(const uint8_t* __restrict__ x,
                                                                 uint8_t* __restrict__ y, PoolShape s) {
  const int64_t cv = s.C / 16;
  const int64_t total = s.B * s.OH * s.OW * cv;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kEwThreads;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kEwThreads + threadIdx.x; i < total; i += stride) {
    const int64_t c = (i % cv) * 16;
    int64_t t = i / cv;
    const int64_t ow = t % s.OW;
    t /= s.OW;
    const int64_t oh = t % s.OH, b = t / s.OH;
    const int64_t ih0 = oh * s.sh - s.ph, iw0 = ow * s.sw - s.pw;
    const uint8_t* img = x + b * s.H * s.W * s.C + c;
    v4i v[9];
    bool ok[9];
#pragma unroll
    for (int k = 0; k < 9; ++k) {
      const int64_t ih = ih0 + k / 3, iw = iw0 + k % 3;
      ok[k] = ih >= 0 && ih < s.H && iw >= 0 && iw < s.W;
      const int64_t ihc = ih < 0 ? 0 : (ih >= s.H ? s.H - 1 : ih), iwc = iw < 0 ? 0 : (iw >= s.W ? s.W - 1 : iw);
      v[k] = *reinterpret_cast<const v4i*>(img + (ihc * s.W + iwc) * s.C);
    }
    CodeMax16<SIGNED> m;
#pragma unroll
    for (int k = 0; k < 9; ++k) m.add(v[k], ok[k]);
    *reinterpret_cast<v4i*>(y + ((b * s.OH + oh) * s.OW + ow) * s.C + c) = m.result();
  }
}

// The same 3x3 window with the output row in the block index: blockIdx.y = oh,
// blockIdx.z = image, threads over (ow, group of 16 channels), 32-bit arithmetic
// and one division per thread -- the flat kernel above spends most of its
// instructions on five 64-bit divisions per output.  The host sends shapes here
// whose byte offsets inside one image fit 31 bits.
template <bool SIGNED>
__global__ __launch_bounds__(kEwThreads) void qmaxpool_k3_rows_kernel(const uint8_t* __restrict__ x,
                                                                      uint8_t* __restrict__ y, int H, int W, int C,
                                                                      int OH, int OW, int sh, int sw, int ph, int pw) {
  const int cv = C >> 4;
  const int idx = static_cast<int>(blockIdx.x) * kEwThreads + threadIdx.x;
  if (idx >= OW * cv) return;
  const int ow = idx / cv, c = (idx - ow * cv) << 4;
  const int oh = blockIdx.y;
  const int64_t b = blockIdx.z;
  const int ih0 = oh * sh - ph, iw0 = ow * sw - pw;
  const uint8_t* img = x + b * (static_cast<int64_t>(H) * W * C) + c;
  v4i v[9];
  bool ok[9];
#pragma unroll
  for (int k = 0; k < 9; ++k) {
    const int ih = ih0 + k / 3, iw = iw0 + k % 3;
    ok[k] = ih >= 0 && ih < H && iw >= 0 && iw < W;
    const int ihc = ih < 0 ? 0 : (ih >= H ? H - 1 : ih), iwc = iw < 0 ? 0 : (iw >= W ? W - 1 : iw);
    v[k] = *reinterpret_cast<const v4i*>(img + (ihc * W + iwc) * C);
  }
  CodeMax16<SIGNED> m;
#pragma unroll
  for (int k = 0; k < 9; ++k) m.add(v[k], ok[k]);
  *reinterpret_cast<v4i*>(y + ((b * OH + oh) * OW + ow) * static_cast<int64_t>(C) + c) = m.result();
}

// Adaptive average pooling: output pixel (oh, ow) averages the input window
// rows floor(oh*H/OH) .. ceil((oh+1)*H/OH)-1 (likewise columns).  VEC = 4: a
// thread owns four consecutive channels (one 32-bit word per input pixel).
template <bool SIGNED, int VEC>
__global__ __launch_bounds__(kEwThreads) void qadaptive_avgpool_kernel(const uint8_t* __restrict__ x,
                                                                       uint8_t* __restrict__ y, PoolShape s,
                                                                       int32_t zp) {
  const int64_t cv = ceil_div(s.C, static_cast<int64_t>(VEC));
  const int64_t total = s.B * s.OH * s.OW * cv;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kEwThreads;
  const float lo = SIGNED ? -128.f : 0.f, hi = SIGNED ? 127.f : 255.f;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kEwThreads + threadIdx.x; i < total; i += stride) {
    const int64_t c = (i % cv) * VEC;
    int64_t t = i / cv;
    const int64_t ow = t % s.OW;
    t /= s.OW;
    const int64_t oh = t % s.OH, b = t / s.OH;
    const int64_t h0 = (oh * s.H) / s.OH, h1 = ceil_div((oh + 1) * s.H, s.OH);
    const int64_t w0 = (ow * s.W) / s.OW, w1 = ceil_div((ow + 1) * s.W, s.OW);
    int32_t acc[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[j] = 0;
    for (int64_t ih = h0; ih < h1; ++ih) {
      const uint8_t* row = x + ((b * s.H + ih) * s.W) * s.C + c;
      for (int64_t iw = w0; iw < w1; ++iw) {
        if constexpr (VEC == 4) {
          const uint32_t w = *reinterpret_cast<const uint32_t*>(row + iw * s.C);
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const uint32_t bte = (w >> (8 * j)) & 0xffu;
            acc[j] += SIGNED ? static_cast<int32_t>(static_cast<int8_t>(bte)) : static_cast<int32_t>(bte);
          }
        } else {
          const uint8_t bte = row[iw * s.C];
          acc[0] += SIGNED ? static_cast<int32_t>(static_cast<int8_t>(bte)) : static_cast<int32_t>(bte);
        }
      }
    }
    const int32_t size = static_cast<int32_t>((h1 - h0) * (w1 - w0));
    const float mult = 1.0f / static_cast<float>(size);
    uint32_t packed = 0;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float v = static_cast<float>(acc[j] - zp * size) * mult;
      float r = __builtin_rintf(v) + static_cast<float>(zp);
      r = __builtin_amdgcn_fmed3f(r, lo, hi);
      packed |= (static_cast<uint32_t>(static_cast<int32_t>(r)) & 0xffu) << (8 * j);
    }
    uint8_t* dst = y + ((b * s.OH + oh) * s.OW + ow) * s.C + c;
    if constexpr (VEC == 4)
      *reinterpret_cast<uint32_t*>(dst) = packed;
    else
      *dst = static_cast<uint8_t>(packed);
  }
}

// Unary activations of a per-tensor quantized tensor through a 256-entry table:
// the input has 256 codes, so every block first computes f for each of them
// (one per thread, in double precision: y = f((c - zp_in) * s_in),
// q = clamp(rne(y / s_out) + zp_out)) into LDS and then maps the bytes, 16 per
// lane per access.  kind 0: gelu (erf), 1: gelu (tanh approximation), 2: sigmoid.
struct UnaryParams {
  double in_scale, out_scale;
  int in_zp, out_zp;
  int kind;
};
constexpr int kLutBlocksMax = 4096;
template <bool SIGNED>
__global__ __launch_bounds__(kEwThreads) void qunary_lut_kernel(const v4i* __restrict__ x16,
                                                                v4i* __restrict__ y16, int64_t n16,
                                                                const uint8_t* __restrict__ x,
                                                                uint8_t* __restrict__ y, int64_t n,
                                                                UnaryParams p) {
  __shared__ uint8_t lut[256];
  static_assert(kEwThreads == 256, "one table entry per thread");
  {
    const int code = SIGNED ? static_cast<int>(static_cast<int8_t>(threadIdx.x)) : static_cast<int>(threadIdx.x);
    const double r = static_cast<double>(code - p.in_zp) * p.in_scale;
    double f;
    if (p.kind == 0) {
      f = 0.5 * r * (1.0 + erf(r * 0.70710678118654752440));
    } else if (p.kind == 1) {
      f = 0.5 * r * (1.0 + tanh(0.79788456080286535588 * (r + 0.044715 * r * r * r)));
    } else {
      f = 1.0 / (1.0 + exp(-r));
    }
    double q = rint(f / p.out_scale) + static_cast<double>(p.out_zp);
    const double lo = SIGNED ? -128.0 : 0.0, hi = SIGNED ? 127.0 : 255.0;
    q = q < lo ? lo : (q > hi ? hi : q);
    lut[threadIdx.x] = static_cast<uint8_t>(static_cast<int>(q));
  }
  __syncthreads();
  auto map4 = [&](uint32_t w) {
    return static_cast<uint32_t>(lut[w & 0xffu]) | (static_cast<uint32_t>(lut[(w >> 8) & 0xffu]) << 8) |
           (static_cast<uint32_t>(lut[(w >> 16) & 0xffu]) << 16) | (static_cast<uint32_t>(lut[w >> 24]) << 24);
  };
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kEwThreads;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kEwThreads + threadIdx.x; i < n16; i += stride) {
    const v4i v = __builtin_nontemporal_load(&x16[i]);
    y16[i] = v4i{static_cast<int>(map4(static_cast<uint32_t>(v.x))), static_cast<int>(map4(static_cast<uint32_t>(v.y))),
                 static_cast<int>(map4(static_cast<uint32_t>(v.z))), static_cast<int>(map4(static_cast<uint32_t>(v.w)))};
  }
  // bytes outside the 16-byte groups (unaligned buffers: all of them)
  const int64_t done = x16 == nullptr ? 0 : 16 * n16;
  for (int64_t i = done + static_cast<int64_t>(blockIdx.x) * kEwThreads + threadIdx.x; i < n; i += stride)
    y[i] = lut[x[i]];
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
    const int64_t blocks = n16 == 0 ? 1 : ceil_div(n16, kEwThreads * kReluUnroll);
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

TMQ_EXPORT int tmq_qcat_rows(const void* x, void* y, int64_t outer, int64_t in_row, int64_t out_row,
                             int64_t out_col_offset, float in_scale, int32_t in_zero_point,
                             float out_scale, int32_t out_zero_point, int q_signed, tmq_stream_t stream) {
  if (outer < 0 || in_row < 0 || out_row < in_row || out_col_offset < 0 || out_col_offset + in_row > out_row)
    return TMQ_ERR_INVALID_ARGUMENT;
  if (!zp_ok(in_zero_point, q_signed) || !zp_ok(out_zero_point, q_signed) || !(out_scale > 0.f))
    return TMQ_ERR_INVALID_ARGUMENT;
  if (outer == 0 || in_row == 0) return TMQ_OK;
  if (x == nullptr || y == nullptr) return TMQ_ERR_INVALID_ARGUMENT;
  RequantParams p;
  p.in_scale = in_scale;
  p.inv_out = 1.0f / out_scale;
  p.out_zp_f = static_cast<float>(out_zero_point);
  p.in_zp = in_zero_point;
  p.identity = in_scale == out_scale && in_zero_point == out_zero_point;
  const bool vec = in_row % 16 == 0 && out_row % 16 == 0 && out_col_offset % 16 == 0 && aligned(x, 16) &&
                   aligned(y, 16);
  const int64_t items = outer * (vec ? in_row / 16 : in_row);
  int64_t g = ceil_div(items, kEwThreads);
  g = g > (1 << 20) ? (1 << 20) : g;
  const dim3 grid(static_cast<unsigned>(g)), block(kEwThreads);
  hipStream_t s = as_stream(stream);
  const uint8_t* xb = static_cast<const uint8_t*>(x);
  uint8_t* yb = static_cast<uint8_t*>(y);
  if (vec) {
    if (q_signed)
      qcat_rows_kernel<true, 16><<<grid, block, 0, s>>>(xb, yb, outer, in_row, out_row, out_col_offset, p);
    else
      qcat_rows_kernel<false, 16><<<grid, block, 0, s>>>(xb, yb, outer, in_row, out_row, out_col_offset, p);
  } else {
    if (q_signed)
      qcat_rows_kernel<true, 1><<<grid, block, 0, s>>>(xb, yb, outer, in_row, out_row, out_col_offset, p);
    else
      qcat_rows_kernel<false, 1><<<grid, block, 0, s>>>(xb, yb, outer, in_row, out_row, out_col_offset, p);
  }
  return launch_status();
}

TMQ_EXPORT int tmq_qmaxpool2d(const void* x, void* y, int64_t B, int64_t H, int64_t W, int64_t C,
                              int32_t kh, int32_t kw, int32_t stride_h, int32_t stride_w, int32_t pad_h,
                              int32_t pad_w, int32_t dil_h, int32_t dil_w, int64_t OH, int64_t OW,
                              int q_signed, tmq_stream_t stream) {
  if (B < 0 || H <= 0 || W <= 0 || C < 0 || OH < 0 || OW < 0 || kh <= 0 || kw <= 0 || stride_h <= 0 ||
      stride_w <= 0 || pad_h < 0 || pad_w < 0 || dil_h <= 0 || dil_w <= 0)
    return TMQ_ERR_INVALID_ARGUMENT;
  // every window must touch the image, or its maximum is undefined
  if (OH > 0 && ((OH - 1) * stride_h - pad_h >= H || pad_h > (kh - 1) * dil_h)) return TMQ_ERR_INVALID_ARGUMENT;
  if (OW > 0 && ((OW - 1) * stride_w - pad_w >= W || pad_w > (kw - 1) * dil_w)) return TMQ_ERR_INVALID_ARGUMENT;
  const int64_t n = B * OH * OW * C;
  if (n == 0) return TMQ_OK;
  if (x == nullptr || y == nullptr) return TMQ_ERR_INVALID_ARGUMENT;
  PoolShape s{B, H, W, C, OH, OW, kh, kw, stride_h, stride_w, pad_h, pad_w, dil_h, dil_w};
  const bool vec = C % 16 == 0 && aligned(x, 16) && aligned(y, 16);
  int64_t g = ceil_div(vec ? n / 16 : n, kEwThreads);
  g = g > (1 << 20) ? (1 << 20) : g;
  const dim3 grid(static_cast<unsigned>(g)), block(kEwThreads);
  hipStream_t hs = as_stream(stream);
  const uint8_t* xb = static_cast<const uint8_t*>(x);
  uint8_t* yb = static_cast<uint8_t*>(y);
  if (vec && kh == 3 && kw == 3 && dil_h == 1 && dil_w == 1 && H * W * C < (int64_t{1} << 31) && OH <= 65535 &&
      B <= 65535 && OW * (C / 16) < (int64_t{1} << 30)) {
    const dim3 rgrid(static_cast<unsigned>(ceil_div(OW * (C / 16), kEwThreads)), static_cast<unsigned>(OH),
                     static_cast<unsigned>(B));
    const int h = static_cast<int>(H), w = static_cast<int>(W), c = static_cast<int>(C);
    const int oh = static_cast<int>(OH), ow = static_cast<int>(OW);
    if (q_signed)
      qmaxpool_k3_rows_kernel<true><<<rgrid, block, 0, hs>>>(xb, yb, h, w, c, oh, ow, stride_h, stride_w, pad_h, pad_w);
    else
      qmaxpool_k3_rows_kernel<false><<<rgrid, block, 0, hs>>>(xb, yb, h, w, c, oh, ow, stride_h, stride_w, pad_h, pad_w);
  } else if (vec && kh == 3 && kw == 3 && dil_h == 1 && dil_w == 1) {
    if (q_signed) qmaxpool_k3_kernel<true><<<grid, block, 0, hs>>>(xb, yb, s);
    else qmaxpool_k3_kernel<false><<<grid, block, 0, hs>>>(xb, yb, s);
  } else if (vec) {
    if (q_signed) qmaxpool_kernel<true, 16><<<grid, block, 0, hs>>>(xb, yb, s);
    else qmaxpool_kernel<false, 16><<<grid, block, 0, hs>>>(xb, yb, s);
  } else {
    if (q_signed) qmaxpool_kernel<true, 1><<<grid, block, 0, hs>>>(xb, yb, s);
    else qmaxpool_kernel<false, 1><<<grid, block, 0, hs>>>(xb, yb, s);
  }
  return launch_status();
}

TMQ_EXPORT int tmq_qadaptive_avgpool2d(const void* x, void* y, int64_t B, int64_t H, int64_t W, int64_t C,
                                       int64_t OH, int64_t OW, int32_t zero_point, int q_signed,
                                       tmq_stream_t stream) {
  if (B < 0 || H <= 0 || W <= 0 || C < 0 || OH < 0 || OW < 0) return TMQ_ERR_INVALID_ARGUMENT;
  if (!zp_ok(zero_point, q_signed)) return TMQ_ERR_INVALID_ARGUMENT;
  // int32 window sums: 255 * window must stay below 2**31
  if (H * W > (int64_t{1} << 23)) return TMQ_ERR_UNSUPPORTED;
  const int64_t n = B * OH * OW * C;
  if (n == 0) return TMQ_OK;
  if (x == nullptr || y == nullptr) return TMQ_ERR_INVALID_ARGUMENT;
  PoolShape s{B, H, W, C, OH, OW, 0, 0, 0, 0, 0, 0, 0, 0};
  const bool vec = C % 4 == 0 && aligned(x, 4) && aligned(y, 4);
  int64_t g = ceil_div(vec ? n / 4 : n, kEwThreads);
  g = g > (1 << 20) ? (1 << 20) : g;
  const dim3 grid(static_cast<unsigned>(g)), block(kEwThreads);
  hipStream_t hs = as_stream(stream);
  const uint8_t* xb = static_cast<const uint8_t*>(x);
  uint8_t* yb = static_cast<uint8_t*>(y);
  if (vec) {
    if (q_signed) qadaptive_avgpool_kernel<true, 4><<<grid, block, 0, hs>>>(xb, yb, s, zero_point);
    else qadaptive_avgpool_kernel<false, 4><<<grid, block, 0, hs>>>(xb, yb, s, zero_point);
  } else {
    if (q_signed) qadaptive_avgpool_kernel<true, 1><<<grid, block, 0, hs>>>(xb, yb, s, zero_point);
    else qadaptive_avgpool_kernel<false, 1><<<grid, block, 0, hs>>>(xb, yb, s, zero_point);
  }
  return launch_status();
}

TMQ_EXPORT int tmq_qunary(const void* x, void* y, int64_t n, int kind, float in_scale, int32_t in_zero_point,
                          float out_scale, int32_t out_zero_point, int q_signed, tmq_stream_t stream) {
  if (n < 0 || (n > 0 && (x == nullptr || y == nullptr))) return TMQ_ERR_INVALID_ARGUMENT;
  if (kind < 0 || kind > 2 || !(in_scale > 0.f) || !(out_scale > 0.f)) return TMQ_ERR_INVALID_ARGUMENT;
  if (!zp_ok(in_zero_point, q_signed) || !zp_ok(out_zero_point, q_signed)) return TMQ_ERR_INVALID_ARGUMENT;
  if (n == 0) return TMQ_OK;
  UnaryParams p;
  p.in_scale = static_cast<double>(in_scale);
  p.out_scale = static_cast<double>(out_scale);
  p.in_zp = in_zero_point;
  p.out_zp = out_zero_point;
  p.kind = kind;
  const bool vec = aligned(x, 16) && aligned(y, 16);
  const int64_t n16 = vec ? n / 16 : 0;
  int64_t g = ceil_div(vec ? (n16 > 0 ? n16 : 1) : n, static_cast<int64_t>(kEwThreads) * 4);
  g = g < 1 ? 1 : (g > kLutBlocksMax ? kLutBlocksMax : g);
  const dim3 grid(static_cast<unsigned>(g)), block(kEwThreads);
  hipStream_t s = as_stream(stream);
  const uint8_t* xb = static_cast<const uint8_t*>(x);
  uint8_t* yb = static_cast<uint8_t*>(y);
  const v4i* x16 = vec ? static_cast<const v4i*>(x) : nullptr;
  v4i* y16 = vec ? static_cast<v4i*>(y) : nullptr;
  if (q_signed) qunary_lut_kernel<true><<<grid, block, 0, s>>>(x16, y16, n16, xb, yb, n, p);
  else qunary_lut_kernel<false><<<grid, block, 0, s>>>(x16, y16, n16, xb, yb, n, p);
  return launch_status();
}
