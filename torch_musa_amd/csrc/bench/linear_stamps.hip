// Measurement only: the persistent int8 GEMM of quantized::linear in its
// instrumented instantiation (see gemm_i8_persistent.h), so that bench.py can
// say where a launch spends its time -- loop cycles, epilogue cycles, the
// hand-over between tiles and the shader clock the power limit leaves while
// all CUs multiply.  Not part of the operator library.
#include "../kernels/gemm_i8_persistent.h"
#include "tmq_bench.h"

namespace tmq {
namespace {
inline int64_t bench_packed_kchunks(int64_t K) { return (K + 127) / 128 * 8; }  // as linear_prepack lays it out
}  // namespace
}  // namespace tmq

TMQ_EXPORT int tmq_bench_linear_stamps(const tmq_linear_desc* d, uint64_t* stamps, int flags, tmq_stream_t stream) {
  using namespace tmq;
  if (d == nullptr || stamps == nullptr) return TMQ_ERR_INVALID_ARGUMENT;
  // what the product's dispatch checks before it launches this kernel: byte
  // outputs, aligned rows of 16-byte chunks, at least six 64-byte stages, 32-bit
  // offsets over 256 rows of either operand
  if (d->M <= 0 || d->N <= 0 || d->K < 6 * kBK || d->K % 16 != 0 || d->K > (int64_t{1} << 23)) return TMQ_ERR_UNSUPPORTED;
  if (d->out_signed || d->ldx < d->K || d->ldx % 16 != 0 || d->ldx > (int64_t{1} << 23) || d->ldy < d->N)
    return TMQ_ERR_UNSUPPORTED;
  if (d->x == nullptr || d->y == nullptr || d->w_packed == nullptr || d->w_colsum == nullptr || d->w_scales == nullptr)
    return TMQ_ERR_INVALID_ARGUMENT;
  if (!aligned(d->x, 16) || !aligned(d->w_packed, 16)) return TMQ_ERR_ALIGNMENT;
  if (!(d->x_scale > 0.f) || !(d->out_scale > 0.f) || d->out_zero_point < 0 || d->out_zero_point > 255)
    return TMQ_ERR_INVALID_ARGUMENT;
  const int64_t tiles = ceil_div(d->M, 256) * ceil_div(d->N, 256);
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 8)
    return TMQ_ERR_LAUNCH;
  if (tiles > 0x7fffffff) return TMQ_ERR_UNSUPPORTED;
  GemmArgs a{};
  XLinear xs{};
  a.M = d->M;
  a.N = d->N;
  a.K = d->K;
  a.w_packed = static_cast<const uint8_t*>(d->w_packed);
  a.w_kchunks = bench_packed_kchunks(d->K);
  a.colsum = d->w_colsum;
  a.x_xor = d->x_signed ? 0u : 0x80808080u;
  a.w_scales = d->w_scales;
  a.w_scale_stride = d->w_per_channel ? 1 : 0;
  a.bias = d->bias;
  a.acc_coef = (d->x_signed ? 0 : 128) - d->x_zero_point;
  a.x_scale = d->x_scale;
  a.out_scale = d->out_scale;
  a.zp_f = static_cast<float>(d->out_zero_point);
  a.lo_f = static_cast<float>(d->relu ? d->out_zero_point : 0);
  a.hi_f = 255.f;
  a.y = d->y;
  a.ldy = d->ldy;
  a.stamps = stamps;
  xs.x = static_cast<const uint8_t*>(d->x);
  xs.ldx = d->ldx;
  const int64_t grid = tiles <= cus ? tiles : cus / 8 * 8;  // as the product launches it
  const dim3 g(static_cast<unsigned>(grid)), b(kPersistThreads);
  hipStream_t s = as_stream(stream);
  a.late_ticks = static_cast<uint32_t>((flags >> 8) & 0xff) * 100u;  // microseconds of late start
  a.late_mode = static_cast<uint32_t>((flags >> 4) & 1);
  if ((flags & ~0xff13) != 0) return TMQ_ERR_INVALID_ARGUMENT;
  switch (flags & 3) {  // what to leave out is compiled in: the instrumented loop has the product's instructions
    case 0: gemm_i8_persistent_kernel<kOutU8, true, 0><<<g, b, 0, s>>>(a, xs); break;
    case 1: gemm_i8_persistent_kernel<kOutU8, true, 1><<<g, b, 0, s>>>(a, xs); break;
    case 2: gemm_i8_persistent_kernel<kOutU8, true, 2><<<g, b, 0, s>>>(a, xs); break;
    case 3: gemm_i8_persistent_kernel<kOutU8, true, 3><<<g, b, 0, s>>>(a, xs); break;
    default: return TMQ_ERR_INVALID_ARGUMENT;
  }
  return launch_status();
}
