// ATen front end of the tmq kernel library on PyTorch-ROCm.
//
// Mirrors, for the quantized-inference path only, what torch_musa registers in
// torch_musa/csrc/aten/quantized:
//   * the six affine-quantizer dispatch stubs (musa/AffineQuantizer.mu:340-357)
//     -> set on the GPU slot of the same stubs, so torch.quantize_per_tensor,
//        torch.quantize_per_channel and Tensor.dequantize run the tmq kernels;
//   * aten::quantize_per_tensor_dynamic (musa_functions.yaml:3515-3519) with the
//     two reductions fused into one pass;
//   * quantized::linear / linear_relu / linear_prepack (mudnn/Linear.cpp:134-158,
//     mudnn/LinearPrepack.cpp:39-57) and quantized::conv2d.new / conv2d_relu.new /
//     conv2d_prepack (mudnn/Conv.cpp:252-288, mudnn/ConvPrepack.cpp:109-225),
//     registered on the quantized GPU dispatch key with the upstream schemas;
//   * the fused variants quantized::conv2d_add / conv2d_add_relu / conv2d_add_silu
//     (mudnn/ConvAdd.cpp:63-99) and conv2d_silu.new (mudnn/Conv.cpp:285-287).
// This file only validates, allocates through the caching allocator and calls
// the C ABI of include/tmq.h on the current stream; it contains no kernels.
// Unlike the reference (muDNN: symmetric qint8 only, mudnn/Linear.cpp:80-85,
// aten/utils/Utils.cpp:142-153) activations may be quint8 with a zero point and
// weights may be per-channel, i.e. the semantics of PyTorch's CPU ops.
#include <ATen/ATen.h>
#include <ATen/native/quantized/AffineQuantizer.h>
#include <ATen/native/quantized/PackedParams.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPCachingAllocator.h>
#include <c10/hip/HIPStream.h>
#include <torch/library.h>

#include <array>
#include <cstdlib>
#include <list>
#include <memory>
#include <mutex>
#include <tuple>
#include <vector>

#include "tmq.h"

namespace {

tmq_stream_t current_stream(const at::Tensor& t) {
  return reinterpret_cast<tmq_stream_t>(c10::hip::getCurrentHIPStream(t.device().index()).stream());
}

// Typed views of a tensor's storage (the untyped accessors are the ones whose
// symbols every libtorch build exports).
template <typename T>
const T* cptr(const at::Tensor& t) { return static_cast<const T*>(t.const_data_ptr()); }
template <typename T>
T* mptr(const at::Tensor& t) { return static_cast<T*>(t.data_ptr()); }

void check_status(int status, const char* what) {
  TORCH_CHECK(status == TMQ_OK, what, " failed: ", tmq_status_string(status));
}

// Scratch memory for the split-K schedule of products with a few hundred rows:
// allocated through the caching allocator (stream-ordered reuse), attached to
// the descriptor, kept alive by the returned tensor until the call is queued.
at::Tensor attach_linear_workspace(tmq_linear_desc& d, const at::TensorOptions& like) {
  const int64_t bytes = tmq_linear_workspace_bytes(d.M, d.N, d.K);
  if (bytes <= 0) return at::Tensor();
  at::Tensor ws = at::empty({bytes}, like.dtype(at::kByte));
  d.workspace = ws.data_ptr();
  d.workspace_bytes = bytes;
  return ws;
}

bool is_signed_qtype(c10::ScalarType t, const char* what) {
  TORCH_CHECK(t == c10::kQInt8 || t == c10::kQUInt8, what, ": only QInt8 and QUInt8 are supported, got ",
              toString(t));
  return t == c10::kQInt8;
}

// ---------------------------------------------------------------------------
// affine quantizer stubs
// ---------------------------------------------------------------------------
void quantize_per_tensor_stub(const at::Tensor& r, at::Tensor& q, double scale, int64_t zp) {
  const bool sgn = is_signed_qtype(q.scalar_type(), "quantize_tensor_per_tensor_affine");
  TORCH_CHECK(r.scalar_type() == at::kFloat, "quantize_tensor_per_tensor_affine expects a Float tensor");
  const c10::OptionalDeviceGuard guard(at::device_of(q));
  check_status(tmq_quantize_per_tensor(cptr<float>(r), q.data_ptr(), q.numel(), scale, zp, sgn,
                                       current_stream(q)),
               "tmq_quantize_per_tensor");
}

void dequantize_per_tensor_stub(const at::Tensor& q, at::Tensor& r, double scale, int64_t zp) {
  const bool sgn = is_signed_qtype(q.scalar_type(), "dequantize_tensor_per_tensor_affine");
  TORCH_CHECK(r.scalar_type() == at::kFloat, "dequantize_tensor_per_tensor_affine writes a Float tensor");
  const c10::OptionalDeviceGuard guard(at::device_of(q));
  check_status(tmq_dequantize_per_tensor(q.data_ptr(), mptr<float>(r), q.numel(), scale, zp, sgn,
                                         current_stream(q)),
               "tmq_dequantize_per_tensor");
}

struct ChannelView {
  int64_t outer, channels, inner;
};

// [outer, C, inner] view of a dense tensor whose channel dimension is `axis`;
// a channels-last tensor with axis 1 has its channels innermost.
ChannelView channel_view(const at::Tensor& t, int64_t axis) {
  TORCH_CHECK(axis >= 0 && axis < t.dim(), "per-channel axis out of range");
  ChannelView v{1, t.size(axis), 1};
  if (t.is_contiguous()) {
    for (int64_t d = 0; d < axis; ++d) v.outer *= t.size(d);
    for (int64_t d = axis + 1; d < t.dim(); ++d) v.inner *= t.size(d);
    return v;
  }
  const bool cl = (t.dim() == 4 && t.is_contiguous(at::MemoryFormat::ChannelsLast)) ||
                  (t.dim() == 5 && t.is_contiguous(at::MemoryFormat::ChannelsLast3d));
  TORCH_CHECK(cl && axis == 1,
              "per-channel (de)quantize needs a contiguous tensor, or a channels-last one with axis 1");
  v.outer = t.numel() / std::max<int64_t>(v.channels, 1);
  return v;
}

struct ChannelParams {
  at::Tensor scales, zps;
};

ChannelParams channel_params(const at::Tensor& like, const at::Tensor& scales, const at::Tensor& zps,
                             int64_t channels, bool sgn) {
  TORCH_CHECK(scales.numel() == channels && zps.numel() == channels,
              "per-channel scales / zero points must have one entry per channel");
  ChannelParams p;
  p.scales = scales.to(like.device(), at::kDouble).contiguous();
  p.zps = zps.to(like.device(), at::kLong).contiguous();
  // same range check (and the same host synchronisation) as the reference's
  // check_zero_points_musa, AffineQuantizer.mu:23-33
  const int64_t qmin = sgn ? -128 : 0, qmax = sgn ? 127 : 255;
  if (channels > 0) {
    const bool bad = p.zps.lt(qmin).logical_or(p.zps.gt(qmax)).any().item<bool>();
    TORCH_CHECK(!bad, "per-channel zero point outside the range of the quantized dtype");
  }
  return p;
}

void quantize_per_channel_stub(const at::Tensor& r, at::Tensor& q, const at::Tensor& scales,
                               const at::Tensor& zps, int64_t axis) {
  const bool sgn = is_signed_qtype(q.scalar_type(), "quantize_tensor_per_channel_affine");
  TORCH_CHECK(r.scalar_type() == at::kFloat, "quantize_tensor_per_channel_affine expects a Float tensor");
  const c10::OptionalDeviceGuard guard(at::device_of(q));
  const ChannelView v = channel_view(q, axis);
  const ChannelParams p = channel_params(q, scales, zps, v.channels, sgn);
  check_status(tmq_quantize_per_channel(cptr<float>(r), q.data_ptr(), v.outer, v.channels, v.inner,
                                        cptr<double>(p.scales), cptr<int64_t>(p.zps),
                                        sgn, current_stream(q)),
               "tmq_quantize_per_channel");
}

void dequantize_per_channel_stub(const at::Tensor& q, at::Tensor& r, const at::Tensor& scales,
                                 const at::Tensor& zps, int64_t axis) {
  const bool sgn = is_signed_qtype(q.scalar_type(), "dequantize_tensor_per_channel_affine");
  TORCH_CHECK(r.scalar_type() == at::kFloat, "dequantize_tensor_per_channel_affine writes a Float tensor");
  const c10::OptionalDeviceGuard guard(at::device_of(q));
  const ChannelView v = channel_view(q, axis);
  const ChannelParams p = channel_params(q, scales, zps, v.channels, sgn);
  check_status(tmq_dequantize_per_channel(q.data_ptr(), mptr<float>(r), v.outer, v.channels, v.inner,
                                          cptr<double>(p.scales), cptr<int64_t>(p.zps),
                                          sgn, current_stream(q)),
               "tmq_dequantize_per_channel");
}

// Float scales and float zero points (qscheme per_channel_affine_float_qparams,
// AffineQuantizer.mu:259-336), with the reference's range check of the zero
// points (check_zero_points_musa, :23-33) and its host synchronisation.
struct FloatChannelParams {
  at::Tensor scales, zps;
};

FloatChannelParams float_channel_params(const at::Tensor& like, const at::Tensor& scales,
                                        const at::Tensor& zps, int64_t channels, bool sgn) {
  TORCH_CHECK(scales.numel() == channels && zps.numel() == channels,
              "per-channel scales / zero points must have one entry per channel");
  FloatChannelParams p;
  p.scales = scales.to(like.device(), at::kFloat).contiguous();
  p.zps = zps.to(like.device(), at::kFloat).contiguous();
  const int64_t qmin = sgn ? -128 : 0, qmax = sgn ? 127 : 255;
  if (channels > 0) {
    const bool bad = p.zps.lt(qmin).logical_or(p.zps.gt(qmax)).any().item<bool>();
    TORCH_CHECK(!bad, "per-channel zero point outside the range of the quantized dtype");
  }
  return p;
}

void quantize_per_channel_float_qparams_stub(const at::Tensor& r, at::Tensor& q, const at::Tensor& scales,
                                             const at::Tensor& zps, int64_t axis) {
  const bool sgn = is_signed_qtype(q.scalar_type(), "quantize_tensor_per_channel_float_qparams");
  TORCH_CHECK(r.scalar_type() == at::kFloat, "quantize_tensor_per_channel_float_qparams expects a Float tensor");
  const c10::OptionalDeviceGuard guard(at::device_of(q));
  const ChannelView v = channel_view(q, axis);
  const FloatChannelParams p = float_channel_params(q, scales, zps, v.channels, sgn);
  check_status(tmq_quantize_per_channel_float_qparams(cptr<float>(r), q.data_ptr(), v.outer, v.channels,
                                                      v.inner, cptr<float>(p.scales), cptr<float>(p.zps), sgn,
                                                      current_stream(q)),
               "tmq_quantize_per_channel_float_qparams");
}

void dequantize_per_channel_float_qparams_stub(const at::Tensor& q, at::Tensor& r, const at::Tensor& scales,
                                               const at::Tensor& zps, int64_t axis) {
  const bool sgn = is_signed_qtype(q.scalar_type(), "dequantize_tensor_per_channel_float_qparams");
  TORCH_CHECK(r.scalar_type() == at::kFloat, "dequantize_tensor_per_channel_float_qparams writes a Float tensor");
  const c10::OptionalDeviceGuard guard(at::device_of(q));
  const ChannelView v = channel_view(q, axis);
  const FloatChannelParams p = float_channel_params(q, scales, zps, v.channels, sgn);
  check_status(tmq_dequantize_per_channel_float_qparams(q.data_ptr(), mptr<float>(r), v.outer, v.channels,
                                                        v.inner, cptr<float>(p.scales), cptr<float>(p.zps), sgn,
                                                        current_stream(q)),
               "tmq_dequantize_per_channel_float_qparams");
}

// The stub objects live in libtorch; overriding their GPU slot at load time is
// the counterpart of REGISTER_PRIVATEUSE1_DISPATCH in the reference.
struct StubInstaller {
  StubInstaller() {
    at::native::quantize_tensor_per_tensor_affine_stub.set_cuda_dispatch_ptr(&quantize_per_tensor_stub);
    at::native::dequantize_tensor_per_tensor_affine_stub.set_cuda_dispatch_ptr(&dequantize_per_tensor_stub);
    at::native::quantize_tensor_per_channel_affine_stub.set_cuda_dispatch_ptr(&quantize_per_channel_stub);
    at::native::dequantize_tensor_per_channel_affine_stub.set_cuda_dispatch_ptr(&dequantize_per_channel_stub);
    at::native::quantize_tensor_per_channel_float_qparams_stub.set_cuda_dispatch_ptr(
        &quantize_per_channel_float_qparams_stub);
    at::native::dequantize_tensor_per_channel_float_qparams_stub.set_cuda_dispatch_ptr(
        &dequantize_per_channel_float_qparams_stub);
  }
} const g_stub_installer;

// ---------------------------------------------------------------------------
// aten::quantize_per_tensor_dynamic: one min/max pass, one small copy to the
// host (the quantizer object keeps the scale on the host), one quantize pass.
// ---------------------------------------------------------------------------
at::Tensor quantize_per_tensor_dynamic(const at::Tensor& self, at::ScalarType dtype, bool reduce_range) {
  TORCH_CHECK(dtype == at::kQInt8 || dtype == at::kQUInt8 || dtype == at::kHalf,
              "dtype ", dtype, " not supported");
  const c10::OptionalDeviceGuard guard(at::device_of(self));
  at::Tensor x = self.contiguous();
  if (dtype == at::kHalf) return x.to(at::kHalf);
  if (x.scalar_type() != at::kFloat) x = x.to(at::kFloat);
  if (reduce_range && at::globalContext().qEngine() == at::QEngine::QNNPACK) reduce_range = false;
  const bool sgn = dtype == at::kQInt8;
  float mm[2] = {0.f, 0.f};
  if (x.numel() > 0) {
    at::Tensor ws = at::empty({static_cast<int64_t>(tmq_minmax_workspace_bytes(x.numel()))},
                              x.options().dtype(at::kByte));
    at::Tensor out = at::empty({2}, x.options());
    check_status(tmq_minmax(cptr<float>(x), x.numel(), mptr<float>(out), ws.data_ptr(),
                            static_cast<size_t>(ws.numel()), current_stream(x)),
                 "tmq_minmax");
    const at::Tensor host = out.cpu();
    mm[0] = cptr<float>(host)[0];
    mm[1] = cptr<float>(host)[1];
  }
  TORCH_CHECK(mm[0] <= mm[1], "In ChooseQuantizationParams, min should be less than or equal to max");
  double scale = 0;
  int32_t zp = 0;
  check_status(tmq_choose_qparams_host(mm[0], mm[1], sgn, reduce_range, &scale, &zp),
               "tmq_choose_qparams_host");
  // quantize the original tensor, so that its memory format carries over
  return at::quantize_per_tensor(self.scalar_type() == at::kFloat ? self : self.to(at::kFloat), scale, zp, dtype);
}

// ---------------------------------------------------------------------------
// quantized::linear
// ---------------------------------------------------------------------------
struct WeightParams {
  at::Tensor scales_f32;   // [N] or [1], device
  at::Tensor scales_f64;   // as given (for unpack)
  at::Tensor zero_points;  // int64 (for unpack)
  c10::QScheme qscheme;
  int64_t axis = 0;
  double scale = 1.0;
  bool per_channel = false;
};

WeightParams weight_params(const at::Tensor& w, const char* what) {
  TORCH_CHECK(w.scalar_type() == c10::kQInt8, what, " requires weights in format QInt8, but got ",
              toString(w.scalar_type()));
  WeightParams p;
  p.qscheme = w.qscheme();
  if (p.qscheme == c10::kPerTensorAffine || p.qscheme == c10::kPerTensorSymmetric) {
    TORCH_CHECK(w.q_zero_point() == 0, what, " requires a symmetric weight (zero_point 0), got ",
                w.q_zero_point());
    p.scale = w.q_scale();
    p.scales_f32 = at::full({1}, static_cast<float>(p.scale), w.options().dtype(at::kFloat));
  } else if (p.qscheme == c10::kPerChannelAffine || p.qscheme == c10::kPerChannelSymmetric) {
    TORCH_CHECK(w.q_per_channel_axis() == 0, what, " requires per-channel weights quantized along dim 0");
    p.per_channel = true;
    p.axis = 0;
    p.scales_f64 = w.q_per_channel_scales().to(at::kDouble);
    p.zero_points = w.q_per_channel_zero_points().to(at::kLong);
    TORCH_CHECK(!p.zero_points.ne(0).any().item<bool>(), what,
                " requires symmetric per-channel weights (all zero points 0)");
    p.scales_f32 = p.scales_f64.to(w.device(), at::kFloat).contiguous();
  } else {
    TORCH_CHECK(false, "Unsupported qscheme: ", toString(p.qscheme));
  }
  return p;
}

std::optional<at::Tensor> prepare_bias(const std::optional<at::Tensor>& bias, int64_t channels,
                                       const at::Tensor& like) {
  if (!bias.has_value() || !bias->defined()) return std::nullopt;
  TORCH_CHECK(bias->dim() == 1, "bias should be a vector (1D Tensor)");
  TORCH_CHECK(bias->size(0) == channels, "bias should have K elements: " + std::to_string(channels));
  return bias->to(like.device(), at::kFloat).contiguous();
}

struct PackedLinearWeightTmq final : public LinearPackedParamsBase {
  PackedLinearWeightTmq(at::Tensor packed, at::Tensor colsum, WeightParams wp,
                        std::optional<at::Tensor> bias, int64_t N, int64_t K)
      : packed_(std::move(packed)), colsum_(std::move(colsum)), wp_(std::move(wp)),
        bias_(std::move(bias)), N_(N), K_(K) {}

  at::Tensor apply(at::Tensor input, double output_scale, int64_t output_zero_point) override {
    return apply_impl(input, output_scale, output_zero_point, false);
  }
  at::Tensor apply_relu(at::Tensor input, double output_scale, int64_t output_zero_point) override {
    return apply_impl(input, output_scale, output_zero_point, true);
  }
  // The reference declares these and throws (mudnn/Linear.h:35-46).  Here:
  // min/max -> qparams -> quint8 activations -> int8 product -> fp32 output on
  // the current stream (two launches for decode-sized inputs, four otherwise),
  // the parameters never visit the host.
  at::Tensor apply_dynamic(at::Tensor input, bool reduce_range) override {
    return apply_dynamic_impl(input, reduce_range, false);
  }
  at::Tensor apply_dynamic_relu(at::Tensor input, bool reduce_range) override {
    return apply_dynamic_impl(input, reduce_range, true);
  }

  // The packed buffer holds every weight byte, so the original tensor is
  // rebuilt from it instead of being kept alive next to it.
  std::tuple<at::Tensor, std::optional<at::Tensor>> unpack() override {
    const c10::OptionalDeviceGuard guard(at::device_of(packed_));
    at::Tensor w = at::empty({N_, K_}, packed_.options().dtype(at::kChar));
    check_status(tmq_linear_unpack(packed_.const_data_ptr(), N_, K_, mptr<int8_t>(w), K_,
                                   current_stream(packed_)),
                 "tmq_linear_unpack");
    at::Tensor q = wp_.per_channel
        ? at::_make_per_channel_quantized_tensor(w, wp_.scales_f64.to(w.device()),
                                                 wp_.zero_points.to(w.device()), wp_.axis)
        : at::_make_per_tensor_quantized_tensor(w, wp_.scale, 0);
    return {q, bias_};
  }
  std::optional<at::Tensor> bias() override { return bias_; }

  static c10::intrusive_ptr<LinearPackedParamsBase> prepack(at::Tensor weight,
                                                            std::optional<at::Tensor> bias) {
    TORCH_CHECK(weight.dim() == 2, "Quantized Linear weight must be 2D tensor");
    const c10::OptionalDeviceGuard guard(at::device_of(weight));
    WeightParams wp = weight_params(weight, "quantized::linear_prepack");
    const int64_t N = weight.size(0), K = weight.size(1);
    auto b = prepare_bias(bias, N, weight);
    const at::Tensor w8 = weight.int_repr().contiguous();
    at::Tensor packed = at::empty({std::max<int64_t>(tmq_linear_packed_bytes(N, K), 16)},
                                  weight.options().dtype(at::kByte));
    at::Tensor colsum = at::empty({std::max<int64_t>(N, 1)}, weight.options().dtype(at::kInt));
    check_status(tmq_linear_prepack(cptr<int8_t>(w8), N, K, K, packed.data_ptr(),
                                    mptr<int32_t>(colsum), current_stream(weight)),
                 "tmq_linear_prepack");
    return c10::make_intrusive<PackedLinearWeightTmq>(std::move(packed), std::move(colsum), std::move(wp),
                                                      std::move(b), N, K);
  }

 private:
  at::Tensor apply_dynamic_impl(const at::Tensor& input, bool reduce_range, bool relu) {
    TORCH_CHECK(input.scalar_type() == at::kFloat, "quantized::linear_dynamic: expected a float input");
    TORCH_CHECK(input.dim() >= 1, "quantized::linear_dynamic: input needs at least one dimension");
    TORCH_CHECK(input.size(-1) == K_, "quantized::linear_dynamic: input has ", input.size(-1),
                " features, the packed weight expects ", K_);
    TORCH_CHECK(input.device() == packed_.device(),
                "quantized::linear_dynamic: input and weight on different devices");
    const c10::OptionalDeviceGuard guard(at::device_of(input));
    const at::Tensor x = input.contiguous();
    std::vector<int64_t> out_shape = x.sizes().vec();
    out_shape.back() = N_;
    at::Tensor y = at::empty(out_shape, x.options());
    if (y.numel() == 0) return y;
    const int64_t M = y.numel() / N_;
    if (K_ == 0) {  // no input features: the product is empty, the bias remains (as the CPU op)
      if (bias_.has_value()) y.copy_(bias_->expand_as(y)); else y.zero_();
      return relu ? y.clamp_min_(0) : y;
    }
    const auto stream = current_stream(x);
    const auto bytes = x.options().dtype(at::kByte);
    if (tmq_linear_dynamic_small_takes(M, N_, K_) != 0 && reinterpret_cast<uintptr_t>(x.data_ptr()) % 16 == 0) {
      // a handful of rows: range, parameters, codes and product in one launch
      tmq_linear_desc d{};
      d.M = M;
      d.N = N_;
      d.K = K_;
      d.w_packed = packed_.const_data_ptr();
      d.w_colsum = cptr<int32_t>(colsum_);
      d.w_scales = cptr<float>(wp_.scales_f32);
      d.w_per_channel = wp_.per_channel;
      d.relu = relu;
      d.bias = bias_.has_value() ? cptr<float>(*bias_) : nullptr;
      check_status(tmq_linear_dynamic_small(&d, cptr<float>(x), K_, reduce_range, mptr<float>(y), N_, stream),
                   "tmq_linear_dynamic_small");
      return y;
    }
    at::Tensor ws = at::empty({static_cast<int64_t>(tmq_minmax_workspace_bytes(x.numel()))}, bytes);
    at::Tensor qp = at::empty({static_cast<int64_t>(sizeof(tmq_qparams))}, bytes);
    at::Tensor xq = at::empty({x.numel()}, bytes);
    auto* qpd = static_cast<tmq_qparams*>(qp.data_ptr());
    // the CPU op quantizes the activations while packing them, with product and
    // zero point rounded once
    check_status(tmq_quantize_per_tensor_dynamic_dev(cptr<float>(x), xq.data_ptr(), x.numel(), 0, reduce_range,
                                                     TMQ_ROUND_FUSED, qpd, ws.data_ptr(),
                                                     static_cast<size_t>(ws.numel()), stream),
                 "tmq_quantize_per_tensor_dynamic_dev");
    tmq_linear_desc d{};
    d.M = M;
    d.N = N_;
    d.K = K_;
    d.x = xq.data_ptr();
    d.ldx = K_;
    d.x_signed = 0;
    d.x_scale = 1.f;  // unused: read from qp on the device
    d.w_packed = packed_.const_data_ptr();
    d.w_colsum = cptr<int32_t>(colsum_);
    d.w_scales = cptr<float>(wp_.scales_f32);
    d.w_per_channel = wp_.per_channel;
    d.relu = relu;
    d.bias = bias_.has_value() ? cptr<float>(*bias_) : nullptr;
    const at::Tensor split_ws = attach_linear_workspace(d, bytes);
    check_status(tmq_linear_f32(&d, qpd, mptr<float>(y), N_, stream), "tmq_linear_f32");
    return y;
  }

  at::Tensor apply_impl(const at::Tensor& act, double output_scale, int64_t output_zero_point, bool relu) {
    TORCH_CHECK(act.qscheme() == c10::kPerTensorSymmetric || act.qscheme() == c10::kPerTensorAffine,
                "quantized::linear expects a per-tensor quantized activation");
    const bool x_signed = is_signed_qtype(act.scalar_type(), "quantized::linear");
    TORCH_CHECK(act.dim() >= 1, "quantized::linear: input needs at least one dimension");
    TORCH_CHECK(act.size(-1) == K_, "quantized::linear: input has ", act.size(-1),
                " features, the packed weight expects ", K_);
    TORCH_CHECK(act.device() == packed_.device(), "quantized::linear: input and weight on different devices");
    TORCH_CHECK(output_scale > 0, "quantized::linear: output scale must be positive");
    const c10::OptionalDeviceGuard guard(at::device_of(act));
    const at::Tensor x = act.contiguous();
    std::vector<int64_t> out_shape = x.sizes().vec();
    out_shape.back() = N_;
    // output dtype follows the activation dtype: quint8 as PyTorch's CPU op,
    // qint8 as the reference (mudnn/Linear.cpp:99-103)
    at::Tensor y = at::_empty_affine_quantized(out_shape, x.options(), output_scale, output_zero_point);
    if (y.numel() == 0) return y;
    // rows from the output: with K == 0 the input has no elements, and the
    // library then writes the requantised bias into every row
    const int64_t M = y.numel() / N_;
    tmq_linear_desc d{};
    d.M = M;
    d.N = N_;
    d.K = K_;
    d.x = x.data_ptr();
    d.ldx = K_;
    d.x_signed = x_signed;
    d.x_zero_point = static_cast<int32_t>(x.q_zero_point());
    d.x_scale = static_cast<float>(x.q_scale());
    d.w_packed = packed_.const_data_ptr();
    d.w_colsum = cptr<int32_t>(colsum_);
    d.w_scales = cptr<float>(wp_.scales_f32);
    d.w_per_channel = wp_.per_channel;
    d.relu = relu;
    d.bias = bias_.has_value() ? cptr<float>(*bias_) : nullptr;
    d.out_scale = static_cast<float>(output_scale);
    d.out_zero_point = static_cast<int32_t>(output_zero_point);
    d.out_signed = x_signed;
    d.y = y.data_ptr();
    d.ldy = N_;
    const at::Tensor split_ws = attach_linear_workspace(d, x.options());
    check_status(tmq_linear(&d, current_stream(x)), "tmq_linear");
    return y;
  }

  at::Tensor packed_, colsum_;
  WeightParams wp_;
  std::optional<at::Tensor> bias_;
  int64_t N_, K_;
};

at::Tensor qlinear_dynamic_run(at::Tensor x, const c10::intrusive_ptr<LinearPackedParamsBase>& w,
                               bool reduce_range) {
  return w->apply_dynamic(std::move(x), reduce_range);
}
at::Tensor qlinear_relu_dynamic_run(at::Tensor x, const c10::intrusive_ptr<LinearPackedParamsBase>& w,
                                    bool reduce_range) {
  return w->apply_dynamic_relu(std::move(x), reduce_range);
}

at::Tensor qlinear_run(at::Tensor act, const c10::intrusive_ptr<LinearPackedParamsBase>& w, double s, int64_t z) {
  return w->apply(std::move(act), s, z);
}
at::Tensor qlinear_relu_run(at::Tensor act, const c10::intrusive_ptr<LinearPackedParamsBase>& w, double s,
                            int64_t z) {
  return w->apply_relu(std::move(act), s, z);
}
c10::intrusive_ptr<LinearPackedParamsBase> qlinear_prepack_run(at::Tensor weight, std::optional<at::Tensor> bias) {
  return PackedLinearWeightTmq::prepack(std::move(weight), std::move(bias));
}

// ---------------------------------------------------------------------------
// quantized::conv2d
// ---------------------------------------------------------------------------
struct PackedConvWeightTmq final : public ConvPackedParamsBase<2> {
  PackedConvWeightTmq(at::Tensor orig_weight, at::Tensor packed, at::Tensor colsum, WeightParams wp,
                      std::optional<at::Tensor> bias, torch::List<int64_t> stride,
                      torch::List<int64_t> padding, torch::List<int64_t> dilation, int64_t groups)
      : orig_weight_(std::move(orig_weight)), packed_(std::move(packed)), colsum_(std::move(colsum)),
        wp_(std::move(wp)), bias_(std::move(bias)), stride_(std::move(stride)),
        padding_(std::move(padding)), dilation_(std::move(dilation)), groups_(groups) {}

  at::Tensor apply(const at::Tensor& input, double output_scale, int64_t output_zero_point) override {
    return apply_impl(input, std::nullopt, output_scale, output_zero_point, 0);
  }
  // Fused residual / activation variants (mudnn/ConvAdd.cpp:11-39, ActMode::SILU
  // of mudnn/Conv.cpp:38-133).  activation: 0 identity, 1 relu, 2 silu.
  at::Tensor apply_fused(const at::Tensor& input, const std::optional<at::Tensor>& accum,
                         double output_scale, int64_t output_zero_point, int activation) {
    return apply_impl(input, accum, output_scale, output_zero_point, activation);
  }
  at::Tensor apply_relu(const at::Tensor& input, double output_scale, int64_t output_zero_point) override {
    return apply_impl(input, std::nullopt, output_scale, output_zero_point, 1);
  }
  at::Tensor apply_dynamic(const at::Tensor&, bool) override {
    TORCH_CHECK(false, "apply_dynamic is not implemented for this packed parameter type");
  }
  std::tuple<at::Tensor, std::optional<at::Tensor>> unpack() override { return {orig_weight_, bias_}; }
  torch::List<int64_t> stride() const override { return stride_; }
  torch::List<int64_t> padding() const override { return padding_; }
  torch::List<int64_t> output_padding() const override { return torch::List<int64_t>({0, 0}); }
  torch::List<int64_t> dilation() const override { return dilation_; }
  int64_t groups() const override { return groups_; }
  bool transpose() const override { return false; }

  static c10::intrusive_ptr<ConvPackedParamsBase<2>> prepack(at::Tensor weight, std::optional<at::Tensor> bias,
                                                             torch::List<int64_t> stride,
                                                             torch::List<int64_t> padding,
                                                             torch::List<int64_t> dilation, int64_t groups) {
    TORCH_CHECK(weight.dim() == 4, "Weights are expected to have 4 dimensions");
    TORCH_CHECK(stride.size() == 2, "stride should contain 2 elements for 2D convolution.");
    TORCH_CHECK(padding.size() == 2, "quantized::conv2d_prepack: specify top/left padding only");
    TORCH_CHECK(dilation.size() == 2, "dilation should contain 2 elements for 2D convolution.");
    TORCH_CHECK(groups >= 1 && weight.size(0) % groups == 0,
                "quantized::conv2d_prepack: output channels must be divisible by groups");
    const c10::OptionalDeviceGuard guard(at::device_of(weight));
    WeightParams wp = weight_params(weight, "quantized::conv2d_prepack");
    const int64_t OC = weight.size(0);
    auto b = prepare_bias(bias, OC, weight);
    // OIHW -> OHWI, the one-time copy the reference makes at ConvPrepack.cpp:78
    const at::Tensor w8 = weight.int_repr().permute({0, 2, 3, 1}).contiguous();
    tmq_conv2d_geom g{};
    g.B = 1;
    g.IC = weight.size(1) * groups;
    g.OC = OC;
    g.KH = weight.size(2);
    g.KW = weight.size(3);
    // weights do not depend on the image: the smallest one the kernel window
    // fits (the library bounds H * W * IC, which a large stand-in would hit for
    // wide layers)
    g.H = g.KH;
    g.W = g.KW;
    g.stride_h = g.stride_w = 1;
    g.pad_h = g.pad_w = 0;
    g.dil_h = g.dil_w = 1;
    g.groups = groups;
    const int64_t bytes = tmq_conv2d_packed_bytes(&g);
    TORCH_CHECK(bytes > 0, "quantized::conv2d_prepack: unsupported weight geometry");
    at::Tensor packed = at::empty({bytes}, weight.options().dtype(at::kByte));
    at::Tensor colsum = at::empty({OC}, weight.options().dtype(at::kInt));
    check_status(tmq_conv2d_prepack(cptr<int8_t>(w8), &g, packed.data_ptr(),
                                    mptr<int32_t>(colsum), current_stream(weight)),
                 "tmq_conv2d_prepack");
    return c10::make_intrusive<PackedConvWeightTmq>(std::move(weight), std::move(packed), std::move(colsum),
                                                    std::move(wp), std::move(b), std::move(stride),
                                                    std::move(padding), std::move(dilation), groups);
  }

 private:
  at::Tensor apply_impl(const at::Tensor& act, const std::optional<at::Tensor>& accum, double output_scale,
                        int64_t output_zero_point, int activation) {
    TORCH_CHECK(act.qscheme() == c10::kPerTensorAffine || act.qscheme() == c10::kPerTensorSymmetric,
                "Conv2d only supports per-tensor quantized activation");
    const bool x_signed = is_signed_qtype(act.scalar_type(), "quantized::conv2d");
    TORCH_CHECK(act.dim() == 4, "quantized::conv2d expects a 4-D (N, C, H, W) input");
    TORCH_CHECK(act.device() == packed_.device(), "quantized::conv2d: input and weight on different devices");
    TORCH_CHECK(output_scale > 0, "quantized::conv2d: output scale must be positive");
    const c10::OptionalDeviceGuard guard(at::device_of(act));
    // NHWC in memory; a copy only if the input is not channels-last already
    // (reference: mudnn/Conv.cpp:192)
    const at::Tensor x = act.contiguous(c10::MemoryFormat::ChannelsLast);
    tmq_conv2d_desc d{};
    tmq_conv2d_geom& g = d.geom;
    g.B = x.size(0);
    g.IC = x.size(1);
    g.H = x.size(2);
    g.W = x.size(3);
    g.OC = orig_weight_.size(0);
    g.KH = orig_weight_.size(2);
    g.KW = orig_weight_.size(3);
    g.stride_h = stride_[0];
    g.stride_w = stride_[1];
    g.pad_h = padding_[0];
    g.pad_w = padding_[1];
    g.dil_h = dilation_[0];
    g.dil_w = dilation_[1];
    g.groups = groups_;
    TORCH_CHECK(g.IC == orig_weight_.size(1) * groups_, "quantized::conv2d: input has ", g.IC,
                " channels, the packed weight expects ", orig_weight_.size(1) * groups_);
    int64_t OH = 0, OW = 0;
    if (g.B > 0) {
      check_status(tmq_conv2d_out_hw(&g, &OH, &OW), "tmq_conv2d_out_hw");
    } else {  // same formula as mudnn/Conv.cpp:20-36
      OH = (g.H + 2 * g.pad_h - g.dil_h * (g.KH - 1) - 1) / g.stride_h + 1;
      OW = (g.W + 2 * g.pad_w - g.dil_w * (g.KW - 1) - 1) / g.stride_w + 1;
    }
    at::Tensor y = at::_empty_affine_quantized({g.B, g.OC, OH, OW}, x.options(), output_scale,
                                               output_zero_point, c10::MemoryFormat::ChannelsLast);
    if (y.numel() == 0) return y;
    d.x = x.data_ptr();
    d.x_signed = x_signed;
    d.x_zero_point = static_cast<int32_t>(x.q_zero_point());
    d.x_scale = static_cast<float>(x.q_scale());
    d.w_per_channel = wp_.per_channel;
    d.w_packed = packed_.const_data_ptr();
    d.w_colsum = cptr<int32_t>(colsum_);
    d.w_scales = cptr<float>(wp_.scales_f32);
    d.bias = bias_.has_value() ? cptr<float>(*bias_) : nullptr;
    d.out_scale = static_cast<float>(output_scale);
    d.out_zero_point = static_cast<int32_t>(output_zero_point);
    d.out_signed = x_signed;
    d.relu = activation == 1;
    d.y = y.data_ptr();
    // scratch for the layers that run on their patch rows or on a channel-padded copy of the
    // input (from the caching allocator: safe under stream capture, freed for reuse in stream order)
    at::Tensor workspace;
    const int64_t ws_bytes = tmq_conv2d_workspace_bytes(&g);
    if (ws_bytes > 0) {
      workspace = at::empty({ws_bytes}, x.options().dtype(at::kByte));
      d.workspace = workspace.data_ptr();
      d.workspace_bytes = ws_bytes;
    }
    if (!accum.has_value() && activation != 2) {
      check_status(tmq_conv2d(&d, current_stream(x)), "tmq_conv2d");
      return y;
    }
    tmq_conv2d_post post{};
    post.activation = activation;
    at::Tensor acc_nhwc;  // keeps a channels-last copy alive until the launch is enqueued
    if (accum.has_value()) {
      const at::Tensor& a = *accum;
      TORCH_CHECK(a.is_quantized(), "accum tensor in qconv must be a quantized Tensor");
      TORCH_CHECK(a.qscheme() == c10::kPerTensorAffine || a.qscheme() == c10::kPerTensorSymmetric,
                  "quantized::conv2d_add only supports a per-tensor quantized accum");
      TORCH_CHECK(a.sizes() == y.sizes(), "quantized::conv2d_add: accum has shape ", a.sizes(),
                  ", the convolution produces ", y.sizes());
      TORCH_CHECK(a.device() == x.device(), "quantized::conv2d_add: accum on a different device");
      acc_nhwc = a.contiguous(c10::MemoryFormat::ChannelsLast);
      post.accum = acc_nhwc.data_ptr();
      post.accum_signed = is_signed_qtype(a.scalar_type(), "quantized::conv2d_add");
      post.accum_zero_point = static_cast<int32_t>(a.q_zero_point());
      post.accum_scale = static_cast<float>(a.q_scale());
    }
    check_status(tmq_conv2d_fused(&d, &post, current_stream(x)), "tmq_conv2d_fused");
    return y;
  }

  at::Tensor orig_weight_, packed_, colsum_;
  WeightParams wp_;
  std::optional<at::Tensor> bias_;
  torch::List<int64_t> stride_, padding_, dilation_;
  int64_t groups_;
};

at::Tensor qconv2d_run(at::Tensor act, const c10::intrusive_ptr<ConvPackedParamsBase<2>>& w, double s, int64_t z) {
  return w->apply(act, s, z);
}
at::Tensor qconv2d_relu_run(at::Tensor act, const c10::intrusive_ptr<ConvPackedParamsBase<2>>& w, double s,
                            int64_t z) {
  return w->apply_relu(act, s, z);
}
PackedConvWeightTmq& tmq_conv(const c10::intrusive_ptr<ConvPackedParamsBase<2>>& w, const char* op) {
  auto* p = dynamic_cast<PackedConvWeightTmq*>(w.get());
  TORCH_CHECK(p != nullptr, op, ": the packed weight was not made by quantized::conv2d_prepack on this device");
  return *p;
}
at::Tensor qconv2d_add_run(at::Tensor act, at::Tensor accum, const c10::intrusive_ptr<ConvPackedParamsBase<2>>& w,
                           double s, int64_t z) {
  return tmq_conv(w, "quantized::conv2d_add").apply_fused(act, accum, s, z, 0);
}
at::Tensor qconv2d_add_relu_run(at::Tensor act, at::Tensor accum,
                                const c10::intrusive_ptr<ConvPackedParamsBase<2>>& w, double s, int64_t z) {
  return tmq_conv(w, "quantized::conv2d_add_relu").apply_fused(act, accum, s, z, 1);
}
at::Tensor qconv2d_silu_run(at::Tensor act, const c10::intrusive_ptr<ConvPackedParamsBase<2>>& w, double s,
                            int64_t z) {
  return tmq_conv(w, "quantized::conv2d_silu").apply_fused(act, std::nullopt, s, z, 2);
}
at::Tensor qconv2d_add_silu_run(at::Tensor act, at::Tensor accum,
                                const c10::intrusive_ptr<ConvPackedParamsBase<2>>& w, double s, int64_t z) {
  return tmq_conv(w, "quantized::conv2d_add_silu").apply_fused(act, accum, s, z, 2);
}
c10::intrusive_ptr<ConvPackedParamsBase<2>> qconv2d_prepack_run(at::Tensor weight, std::optional<at::Tensor> bias,
                                                                torch::List<int64_t> stride,
                                                                torch::List<int64_t> padding,
                                                                torch::List<int64_t> dilation, int64_t groups) {
  return PackedConvWeightTmq::prepack(std::move(weight), std::move(bias), std::move(stride),
                                      std::move(padding), std::move(dilation), groups);
}

// quantized::conv1d_prepack (mudnn/ConvPrepack.cpp:159-216): a 1-D convolution
// is the 2-D one over a height of 1 -- weight [OC, IC/g, L] -> [OC, IC/g, 1, L],
// stride / padding / dilation [v] -> [1 or 0, v] -- and shares its packed type.
torch::List<int64_t> conv1d_arg(const torch::List<int64_t>& arg, int64_t base, const char* what) {
  TORCH_CHECK(!arg.empty(), "quantized::conv1d_prepack: ", what, " must have elements");
  return torch::List<int64_t>({base, arg.size() == 1 ? arg.get(0) : arg.get(1)});
}
c10::intrusive_ptr<ConvPackedParamsBase<2>> qconv1d_prepack_run(at::Tensor weight, std::optional<at::Tensor> bias,
                                                                torch::List<int64_t> stride,
                                                                torch::List<int64_t> padding,
                                                                torch::List<int64_t> dilation, int64_t groups) {
  TORCH_CHECK(weight.dim() == 3 || weight.dim() == 4, "quantized::conv1d_prepack: weights are expected to have 3 dimensions");
  if (weight.dim() == 3) weight = weight.unsqueeze(-2);
  return PackedConvWeightTmq::prepack(std::move(weight), std::move(bias), conv1d_arg(stride, 1, "stride"),
                                      conv1d_arg(padding, 0, "padding"), conv1d_arg(dilation, 1, "dilation"),
                                      groups);
}
// quantized::conv1d / conv1d_relu as PyTorch's CPU ops run them: [N, C, L] ->
// [N, C, 1, L], the 2-D convolution, and back.
at::Tensor qconv1d_impl(const at::Tensor& act, const c10::intrusive_ptr<ConvPackedParamsBase<2>>& w, double s,
                        int64_t z, bool relu) {
  TORCH_CHECK(act.dim() == 3, "quantized::conv1d expects a 3-D (N, C, L) input");
  const at::Tensor x = act.unsqueeze(2);
  const at::Tensor y = relu ? w->apply_relu(x, s, z) : w->apply(x, s, z);
  return y.squeeze(2);
}
at::Tensor qconv1d_run(at::Tensor act, const c10::intrusive_ptr<ConvPackedParamsBase<2>>& w, double s, int64_t z) {
  return qconv1d_impl(act, w, s, z, false);
}
at::Tensor qconv1d_relu_run(at::Tensor act, const c10::intrusive_ptr<ConvPackedParamsBase<2>>& w, double s,
                            int64_t z) {
  return qconv1d_impl(act, w, s, z, true);
}

// ---------------------------------------------------------------------------
// quantized::add / add_relu (musa/BinaryOps.mu:154-207) and relu of a quantized
// tensor (musa/Activation.mu:165-186,215-220)
// ---------------------------------------------------------------------------
at::Tensor qadd_impl(const at::Tensor& qa, const at::Tensor& qb, double output_scale, int64_t output_zero_point,
                     bool relu) {
  TORCH_CHECK(qa.qscheme() == c10::kPerTensorAffine, "Only per tensor quantization is supported in Add.");
  TORCH_CHECK(qa.qscheme() == qb.qscheme(), "Both inputs to Add must have the same quantization scheme.");
  TORCH_CHECK(qa.scalar_type() == qb.scalar_type(), "Add operands should have same data type.");
  const bool sgn = is_signed_qtype(qa.scalar_type(), "quantized::add");
  TORCH_CHECK(qa.sizes() == qb.sizes(),
              "quantized::add currently expects both input tensors to be the same shape");
  TORCH_CHECK(qa.device() == qb.device(), "quantized::add: operands on different devices");
  TORCH_CHECK(output_scale > 0, "quantized::add: output scale must be positive");
  const c10::OptionalDeviceGuard guard(at::device_of(qa));
  const auto fmt = qa.suggest_memory_format();
  const at::Tensor a = qa.contiguous(fmt), b = qb.contiguous(fmt);
  at::Tensor y = at::_empty_affine_quantized(qa.sizes(), qa.options(), output_scale, output_zero_point, fmt);
  if (y.numel() == 0) return y;
  check_status(tmq_qadd(a.data_ptr(), b.data_ptr(), y.data_ptr(), y.numel(), static_cast<float>(a.q_scale()),
                        static_cast<int32_t>(a.q_zero_point()), static_cast<float>(b.q_scale()),
                        static_cast<int32_t>(b.q_zero_point()), static_cast<float>(output_scale),
                        static_cast<int32_t>(output_zero_point), sgn, relu, current_stream(a)),
               "tmq_qadd");
  return y;
}
at::Tensor qadd_run(at::Tensor qa, at::Tensor qb, double s, int64_t z) { return qadd_impl(qa, qb, s, z, false); }
at::Tensor qadd_relu_run(at::Tensor qa, at::Tensor qb, double s, int64_t z) { return qadd_impl(qa, qb, s, z, true); }

at::Tensor qrelu_run(const at::Tensor& self) {
  TORCH_CHECK(self.qscheme() == c10::kPerTensorAffine || self.qscheme() == c10::kPerTensorSymmetric,
              "we currently only support per-tensor quantized relu, but got ", toString(self.qscheme()));
  const bool sgn = is_signed_qtype(self.scalar_type(), "relu");
  const c10::OptionalDeviceGuard guard(at::device_of(self));
  const auto fmt = self.suggest_memory_format();
  const at::Tensor x = self.contiguous(fmt);
  at::Tensor y = at::_empty_affine_quantized(self.sizes(), self.options(), self.q_scale(), self.q_zero_point(), fmt);
  if (y.numel() == 0) return y;
  check_status(tmq_qrelu(x.data_ptr(), y.data_ptr(), y.numel(), static_cast<int32_t>(self.q_zero_point()), sgn,
                         current_stream(x)),
               "tmq_qrelu");
  return y;
}

// aten::gelu and aten::sigmoid of per-tensor quantized tensors (reference:
// ActQuantizedGeLU / ActQuantized<SIGMOID>, musa/Activation.mu:95-164,218-219).
// Output parameters as PyTorch's CPU ops choose them: gelu keeps the input's,
// sigmoid uses scale 1/256 with zero point 0 (quint8) or -128 (qint8).
at::Tensor qunary_impl(const at::Tensor& self, int kind, double out_scale, int64_t out_zp, const char* what) {
  TORCH_CHECK(self.qscheme() == c10::kPerTensorAffine || self.qscheme() == c10::kPerTensorSymmetric, what,
              ": only per-tensor quantized tensors are supported, got ", toString(self.qscheme()));
  const bool sgn = is_signed_qtype(self.scalar_type(), what);
  const c10::OptionalDeviceGuard guard(at::device_of(self));
  const auto fmt = self.suggest_memory_format();
  const at::Tensor x = self.contiguous(fmt);
  at::Tensor y = at::_empty_affine_quantized(self.sizes(), self.options(), out_scale, out_zp, fmt);
  if (y.numel() == 0) return y;
  check_status(tmq_qunary(x.data_ptr(), y.data_ptr(), y.numel(), kind, static_cast<float>(self.q_scale()),
                          static_cast<int32_t>(self.q_zero_point()), static_cast<float>(out_scale),
                          static_cast<int32_t>(out_zp), sgn, current_stream(x)),
               "tmq_qunary");
  return y;
}
at::Tensor qgelu_run(const at::Tensor& self, c10::string_view approximate) {
  const std::string a(approximate.data(), approximate.size());
  TORCH_CHECK(a == "none" || a == "tanh", "gelu: approximate must be 'none' or 'tanh', got ", a);
  // the CPU kernel carries the scale as a float and gives it to the output that way
  return qunary_impl(self, a == "tanh" ? 1 : 0, static_cast<double>(static_cast<float>(self.q_scale())),
                     self.q_zero_point(), "gelu");
}
at::Tensor qsigmoid_run(const at::Tensor& self) {
  const bool sgn = self.scalar_type() == c10::kQInt8;
  return qunary_impl(self, 2, 1.0 / 256.0, sgn ? -128 : 0, "sigmoid");
}

// ---------------------------------------------------------------------------
// quantized::cat (TensorShape.cpp:383-426 of the reference) and
// aten::quantized_max_pool2d (Pool.cpp:178-247)
// ---------------------------------------------------------------------------
// Checks the inputs of a concatenation against the first one and returns the
// output shape; `dim` comes back normalised.
std::vector<int64_t> qcat_shape(const c10::List<at::Tensor>& qxs, int64_t& dim, const char* op) {
  TORCH_CHECK(qxs.size() > 0, op, " expects at least one tensor");
  const at::Tensor qx0 = qxs[0];
  if (dim < 0) dim += qx0.dim();
  TORCH_CHECK(dim >= 0 && dim < qx0.dim(), "Wrong dim: ", dim);
  std::vector<int64_t> shape = qx0.sizes().vec();
  shape[dim] = 0;
  for (const at::Tensor& qx : qxs) {
    TORCH_CHECK(qx.scalar_type() == qx0.scalar_type() && qx.dim() == qx0.dim() && qx.device() == qx0.device(),
                op, ": all inputs need the dtype, rank and device of the first");
    TORCH_CHECK(qx.qscheme() == c10::kPerTensorAffine || qx.qscheme() == c10::kPerTensorSymmetric,
                "Quantized cat only supports quantize-per-tensor");
    for (int64_t d = 0; d < qx0.dim(); ++d)
      TORCH_CHECK(d == dim || qx.size(d) == qx0.size(d), op, ": sizes differ outside dim ", dim);
    shape[dim] += qx.size(dim);
  }
  return shape;
}

// Requantises every input to y's parameters and writes it at its offset along
// `dim`; y is contiguous and has the concatenated shape.
void qcat_into(const c10::List<at::Tensor>& qxs, int64_t dim, const at::Tensor& y) {
  if (y.numel() == 0) return;
  const bool sgn = is_signed_qtype(y.scalar_type(), "quantized::cat");
  int64_t outer = 1, inner = 1;
  for (int64_t d = 0; d < dim; ++d) outer *= y.size(d);
  for (int64_t d = dim + 1; d < y.dim(); ++d) inner *= y.size(d);
  int64_t off = 0;
  for (const at::Tensor& qx : qxs) {
    const at::Tensor x = qx.contiguous();
    const int64_t row = x.size(dim) * inner;
    check_status(tmq_qcat_rows(x.data_ptr(), y.data_ptr(), outer, row, y.size(dim) * inner, off,
                               static_cast<float>(x.q_scale()), static_cast<int32_t>(x.q_zero_point()),
                               static_cast<float>(y.q_scale()), static_cast<int32_t>(y.q_zero_point()), sgn,
                               current_stream(y)),
                 "tmq_qcat_rows");
    off += row;
  }
}

at::Tensor qcat_run(const c10::List<at::Tensor>& qxs, int64_t dim, std::optional<double> scale,
                    std::optional<int64_t> zero_point) {
  const std::vector<int64_t> shape = qcat_shape(qxs, dim, "quantized::cat");
  const at::Tensor qx0 = qxs[0];
  const double out_scale = scale.has_value() ? *scale : qx0.q_scale();
  const int64_t out_zp = zero_point.has_value() ? *zero_point : qx0.q_zero_point();
  TORCH_CHECK(out_scale > 0, "quantized::cat: output scale must be positive");
  const c10::OptionalDeviceGuard guard(at::device_of(qx0));
  at::Tensor y = at::_empty_affine_quantized(shape, qx0.options(), out_scale, out_zp, c10::MemoryFormat::Contiguous);
  qcat_into(qxs, dim, y);
  return y;
}

// quantized::cat_out and aten::cat.out (TensorShape.cpp:331-381 of the
// reference): the inputs are requantised to the parameters `out` already
// carries.  The reference accepts a qint8 `out` only; quint8 works here too.
// `out` must have the concatenated shape; one that is not contiguous is
// filled through a contiguous temporary.
at::Tensor& qcat_out_impl(const c10::List<at::Tensor>& qxs, int64_t dim, at::Tensor& out) {
  TORCH_CHECK(out.is_quantized() &&
                  (out.qscheme() == c10::kPerTensorAffine || out.qscheme() == c10::kPerTensorSymmetric),
              "Quantized cat only supports quantize-per-tensor");
  const std::vector<int64_t> shape = qcat_shape(qxs, dim, "quantized::cat_out");
  const at::Tensor qx0 = qxs[0];
  TORCH_CHECK(out.scalar_type() == qx0.scalar_type() && out.device() == qx0.device(),
              "quantized::cat_out: out needs the dtype and device of the inputs");
  TORCH_CHECK(out.sizes().vec() == shape, "quantized::cat_out: out has shape ", out.sizes(), ", the inputs give ",
              c10::IntArrayRef(shape));
  const c10::OptionalDeviceGuard guard(at::device_of(out));
  if (out.is_contiguous()) {
    qcat_into(qxs, dim, out);
  } else {
    at::Tensor y = at::_empty_affine_quantized(shape, out.options(), out.q_scale(), out.q_zero_point(),
                                               c10::MemoryFormat::Contiguous);
    qcat_into(qxs, dim, y);
    out.copy_(y);
  }
  return out;
}
at::Tensor qcat_out_run(const c10::List<at::Tensor>& qxs, int64_t dim, at::Tensor out) {
  return qcat_out_impl(qxs, dim, out);
}
at::Tensor& qcat_aten_out_run(const at::ITensorListRef& tensors, int64_t dim, at::Tensor& out) {
  c10::List<at::Tensor> list;
  for (const at::Tensor& t : tensors) list.push_back(t);
  return qcat_out_impl(list, dim, out);
}

// aten::add.Tensor with a quantized operand (mudnn/BinaryOps.cpp:11-31 of the
// reference): quantized graphs add a quantized tensor to a float one (or to
// another quantized one) and expect a float result; alpha must be 1.
at::Tensor qadd_tensor_run(const at::Tensor& a, const at::Tensor& b, const at::Scalar& alpha) {
  TORCH_CHECK(alpha.equal(1), "Quantized add don't support set alpha yet.");
  const at::Tensor fa = a.is_quantized() ? a.dequantize() : a;
  const at::Tensor fb = b.is_quantized() ? b.dequantize() : b;
  return at::add(fa, fb, alpha);
}

// aten::cat of quantized tensors (reference: TensorShape.cpp:383-426, the same
// function as quantized::cat): the result takes the first input's parameters.
at::Tensor qcat_aten_run(const at::ITensorListRef& tensors, int64_t dim) {
  c10::List<at::Tensor> list;
  for (const at::Tensor& t : tensors) list.push_back(t);
  return qcat_run(list, dim, std::nullopt, std::nullopt);
}

// aten::upsample_nearest2d of a per-tensor quantized tensor (reference:
// UpSampleNearest2d.cpp:15-52, a round trip through the integer
// representation): nearest-neighbour selection moves codes unchanged, so the
// integer tensor goes through PyTorch-ROCm's own byte kernel and is wrapped
// again with the input's parameters.
at::Tensor qupsample_nearest2d_run(const at::Tensor& input, c10::SymIntArrayRef output_size,
                                   std::optional<double> scales_h, std::optional<double> scales_w) {
  TORCH_CHECK(input.qscheme() == c10::kPerTensorAffine || input.qscheme() == c10::kPerTensorSymmetric,
              "upsample_nearest2d: only per-tensor quantized tensors are supported");
  is_signed_qtype(input.scalar_type(), "upsample_nearest2d");
  const c10::OptionalDeviceGuard guard(at::device_of(input));
  const at::Tensor codes = input.int_repr();
  const bool sgn = codes.scalar_type() == at::kChar;
  const at::Tensor bytes = sgn ? codes.view(at::kByte) : codes;
  at::Tensor up = at::upsample_nearest2d_symint(bytes, output_size, scales_h, scales_w);
  if (sgn) up = up.view(at::kChar);
  return at::_make_per_tensor_quantized_tensor(up, input.q_scale(), input.q_zero_point());
}

int64_t pool_out(int64_t n, int64_t k, int64_t s, int64_t p, int64_t d, bool ceil_mode) {
  int64_t out = (n + 2 * p - d * (k - 1) - 1 + (ceil_mode ? s - 1 : 0)) / s + 1;
  if (ceil_mode && (out - 1) * s >= n + p) --out;
  return out;
}

at::Tensor qmaxpool2d_run(const at::Tensor& input, at::IntArrayRef kernel_size, at::IntArrayRef stride,
                          at::IntArrayRef padding, at::IntArrayRef dilation, bool ceil_mode) {
  TORCH_CHECK(input.qscheme() == c10::kPerTensorAffine || input.qscheme() == c10::kPerTensorSymmetric,
              "MaxPool2dQuantized(): only supports per tensor quantized tensors");
  const bool sgn = is_signed_qtype(input.scalar_type(), "quantized_max_pool2d");
  TORCH_CHECK(input.dim() == 3 || input.dim() == 4, "Expecting the input tensor of rank 3 or 4.");
  TORCH_CHECK(kernel_size.size() == 1 || kernel_size.size() == 2, "quantized_max_pool2d: kernel_size must have 1 or 2 elements");
  TORCH_CHECK(stride.empty() || stride.size() == 1 || stride.size() == 2, "quantized_max_pool2d: stride must have 0, 1 or 2 elements");
  TORCH_CHECK(padding.size() == 1 || padding.size() == 2, "quantized_max_pool2d: padding must have 1 or 2 elements");
  TORCH_CHECK(dilation.size() == 1 || dilation.size() == 2, "quantized_max_pool2d: dilation must have 1 or 2 elements");
  const int64_t kh = kernel_size[0], kw = kernel_size.size() == 1 ? kh : kernel_size[1];
  const int64_t sh = stride.empty() ? kh : stride[0], sw = stride.empty() ? kw : (stride.size() == 1 ? sh : stride[1]);
  const int64_t ph = padding[0], pw = padding.size() == 1 ? ph : padding[1];
  const int64_t dh = dilation[0], dw = dilation.size() == 1 ? dh : dilation[1];
  TORCH_CHECK(kh > 0 && kw > 0 && sh > 0 && sw > 0 && dh > 0 && dw > 0 && ph >= 0 && pw >= 0,
              "quantized_max_pool2d: kernel, stride and dilation must be positive, padding non-negative");
  TORCH_CHECK(ph <= kh / 2 && pw <= kw / 2, "pad should be at most half of effective kernel size");
  const c10::OptionalDeviceGuard guard(at::device_of(input));
  const at::Tensor x4 = input.dim() == 3 ? input.unsqueeze(0) : input;
  const at::Tensor x = x4.contiguous(c10::MemoryFormat::ChannelsLast);
  const int64_t B = x.size(0), C = x.size(1), H = x.size(2), W = x.size(3);
  const int64_t OH = pool_out(H, kh, sh, ph, dh, ceil_mode), OW = pool_out(W, kw, sw, pw, dw, ceil_mode);
  TORCH_CHECK(OH > 0 && OW > 0, "quantized_max_pool2d: the output would be empty");
  at::Tensor y = at::_empty_affine_quantized({B, C, OH, OW}, x.options(), input.q_scale(), input.q_zero_point(),
                                             c10::MemoryFormat::ChannelsLast);
  if (y.numel() > 0)
    check_status(tmq_qmaxpool2d(x.data_ptr(), y.data_ptr(), B, H, W, C, static_cast<int32_t>(kh),
                                static_cast<int32_t>(kw), static_cast<int32_t>(sh), static_cast<int32_t>(sw),
                                static_cast<int32_t>(ph), static_cast<int32_t>(pw), static_cast<int32_t>(dh),
                                static_cast<int32_t>(dw), OH, OW, sgn, current_stream(x)),
                 "tmq_qmaxpool2d");
  return input.dim() == 3 ? y.squeeze(0) : y;
}

// aten::_adaptive_avg_pool2d on quantized GPU tensors (reference:
// AdaptiveAvgPool2dQuantized, torch_musa/csrc/aten/quantized/Pool.cpp:132-176).
// The result keeps the input's scale and zero point and comes back channels-last.
at::Tensor qadaptive_avgpool2d_run(const at::Tensor& input, c10::SymIntArrayRef output_size_sym) {
  TORCH_CHECK(input.qscheme() == c10::kPerTensorAffine || input.qscheme() == c10::kPerTensorSymmetric,
              "AdaptiveAvgPool2dQuantized only supports per tensor quantized tensors");
  TORCH_CHECK(output_size_sym.size() == 2, "AdaptiveAvgPool2d only supports output with 2-elements");
  const bool sgn = is_signed_qtype(input.scalar_type(), "adaptive_avg_pool2d");
  TORCH_CHECK(input.dim() == 3 || input.dim() == 4, "adaptive_avg_pool2d: expected a 3-D or 4-D input");
  const int64_t OH = output_size_sym[0].expect_int(), OW = output_size_sym[1].expect_int();
  TORCH_CHECK(OH >= 0 && OW >= 0, "adaptive_avg_pool2d: output sizes must be non-negative");
  const c10::OptionalDeviceGuard guard(at::device_of(input));
  const at::Tensor x4 = input.dim() == 3 ? input.unsqueeze(0) : input;
  TORCH_CHECK(x4.size(2) > 0 && x4.size(3) > 0, "adaptive_avg_pool2d: input spatial sizes must be positive");
  const at::Tensor x = x4.contiguous(c10::MemoryFormat::ChannelsLast);
  const int64_t B = x.size(0), C = x.size(1), H = x.size(2), W = x.size(3);
  at::Tensor y = at::_empty_affine_quantized({B, C, OH, OW}, x.options(), input.q_scale(), input.q_zero_point(),
                                             c10::MemoryFormat::ChannelsLast);
  if (y.numel() > 0)
    check_status(tmq_qadaptive_avgpool2d(x.data_ptr(), y.data_ptr(), B, H, W, C, OH, OW,
                                         static_cast<int32_t>(input.q_zero_point()), sgn, current_stream(x)),
                 "tmq_qadaptive_avgpool2d");
  return input.dim() == 3 ? y.squeeze(0) : y;
}

// ---------------------------------------------------------------------------
// quantized::linear_per_tensor, quantized::conv, quantized::conv_binary: the
// lowering targets of the reference's PT2E path (torch_musa/core/lowering.py:7-60),
// defined by its patch of ATen's quantized/library.cpp (lines 20-22) and
// implemented there as dequantize -> fp32 matmul / conv -> requantize fallbacks
// ("todo W8A8 kernel", mudnn/Qlinear.cpp:36-69, mudnn/Qconv.cpp:45-86,137-181).
// Activations and weights are plain uint8 / int8 tensors with their parameters
// passed beside them.  Here the products run on the int8 kernels; the weight
// is re-tiled on every call because the schema carries no packed object.
// ---------------------------------------------------------------------------
struct PlainOut {
  bool is_int = false, is_signed = false;
  c10::ScalarType dtype = c10::kFloat;
};
PlainOut plain_out(std::optional<c10::ScalarType> output_dtype, c10::ScalarType act_dtype, const char* what) {
  PlainOut o;
  o.dtype = output_dtype.value_or(act_dtype);
  if (o.dtype == c10::kByte || o.dtype == c10::kChar) {
    o.is_int = true;
    o.is_signed = o.dtype == c10::kChar;
  } else {
    TORCH_CHECK(o.dtype == c10::kFloat || o.dtype == c10::kBFloat16 || o.dtype == c10::kHalf, what,
                ": output dtype must be uint8, int8 or a floating type, got ", toString(o.dtype));
  }
  return o;
}
bool plain_signed(const at::Tensor& t, const char* what) {
  TORCH_CHECK(t.scalar_type() == c10::kByte || t.scalar_type() == c10::kChar, what,
              ": expected a uint8 or int8 tensor, got ", toString(t.scalar_type()));
  return t.scalar_type() == c10::kChar;
}
// per-output-channel weight scales as fp32 on the weight's device; zero points must be 0
at::Tensor plain_weight_scales(const at::Tensor& w_scale, const at::Tensor& w_zero_point, int64_t channels,
                               const at::Tensor& like, const char* what) {
  TORCH_CHECK(w_scale.numel() == channels || w_scale.numel() == 1, what, ": expected ", channels,
              " weight scales (or one), got ", w_scale.numel());
  TORCH_CHECK(!w_zero_point.defined() || w_zero_point.numel() == 0 || !w_zero_point.ne(0).any().item<bool>(), what,
              ": the int8 kernels take symmetric weights (zero point 0)");
  return w_scale.to(like.device(), at::kFloat).contiguous().reshape({-1});
}
// requantize a float result the way the reference's fallback does (round half to even)
at::Tensor plain_requant(const at::Tensor& r, double scale, int64_t zp, const PlainOut& o) {
  if (!o.is_int) return r.to(o.dtype);
  return at::clamp(at::round(r / scale + zp), o.is_signed ? -128 : 0, o.is_signed ? 127 : 255).to(o.dtype);
}

// ---------------------------------------------------------------------------
// Packed weights of the plain-tensor ops.  Their schemas carry the int8 weight as
// an ordinary tensor on every call, so the re-tiled copy, its column sums and the
// fp32 scales are kept from one call to the next: a most-recently-used
// list keyed on the identity of the weight, scale and zero-point tensors
// (storage, address, version counter, shape, strides) and on the geometry the
// packing depends on.  An in-place change of any of the three bumps its version
// counter and misses; a freed storage is recognised by its expired weak
// reference, so an address that is handed out again cannot hit.  Tensors without
// a version counter (inference mode) are never cached.  TMQ_PLAIN_WEIGHT_CACHE=0
// in the environment turns the cache off.
// ---------------------------------------------------------------------------
struct TensorIdentity {
  std::optional<c10::weak_intrusive_ptr<c10::StorageImpl>> storage;
  const void* data = nullptr;
  uint32_t version = 0;
  c10::ScalarType dtype = c10::ScalarType::Undefined;
  std::vector<int64_t> sizes, strides;
  bool defined = false;

  static bool cacheable(const at::Tensor& t) { return !t.defined() || !t.is_inference(); }
  explicit TensorIdentity(const at::Tensor& t) {
    if (!t.defined()) return;
    defined = true;
    storage = t.storage().getWeakStorageImpl();
    data = t.const_data_ptr();
    version = t._version();
    dtype = t.scalar_type();
    sizes = t.sizes().vec();
    strides = t.strides().vec();
  }
  bool matches(const at::Tensor& t) const {
    if (!t.defined()) return !defined;
    if (!defined || storage->expired()) return false;
    return t.const_data_ptr() == data && t._version() == version && t.scalar_type() == dtype &&
           t.storage().unsafeGetStorageImpl() == storage->_unsafe_get_target() && t.sizes() == c10::IntArrayRef(sizes) &&
           t.strides() == c10::IntArrayRef(strides);
  }
  bool alive() const { return !defined || !storage->expired(); }
};

// Streams.  The packing kernels of a miss run on the caller's current stream; the entry
// keeps an event recorded behind them.  A hit from the same stream is ordered by the
// stream; a hit from another stream (or another host thread's stream) makes that stream
// wait for the event and tells the caching allocator that the buffers are in use there.
// While the current stream is being captured into a graph nothing is inserted (the
// packing would only be recorded, not run) and only entries whose packing has already
// finished are handed out (waiting for an event of eager work cannot be recorded); a
// capture that misses is refused with an error -- the packing's zero-point check needs
// the host -- so a graph is warmed up with one eager call per weight first.
struct ReadyEvent {  // one HIP event without timing, destroyed with its last holder
  hipEvent_t ev = nullptr;
  ReadyEvent() { TORCH_CHECK(hipEventCreateWithFlags(&ev, hipEventDisableTiming) == hipSuccess, "hipEventCreate failed"); }
  ~ReadyEvent() {
    if (ev != nullptr) (void)hipEventDestroy(ev);
  }
  ReadyEvent(const ReadyEvent&) = delete;
  ReadyEvent& operator=(const ReadyEvent&) = delete;
  void record(hipStream_t s) { TORCH_CHECK(hipEventRecord(ev, s) == hipSuccess, "hipEventRecord failed"); }
  void block(hipStream_t s) { TORCH_CHECK(hipStreamWaitEvent(s, ev, 0) == hipSuccess, "hipStreamWaitEvent failed"); }
  bool query() {
    const hipError_t e = hipEventQuery(ev);
    if (e != hipSuccess) (void)hipGetLastError();  // hipErrorNotReady is an answer, not a failure
    return e == hipSuccess;
  }
};

struct PlainWeightEntry {
  TensorIdentity weight, scales, zero_points;
  std::array<int64_t, 8> geometry;  // what the packing depends on besides the weight (conv: taps, groups, ...)
  at::Tensor packed, colsum, scales_f32;
  std::shared_ptr<ReadyEvent> ready;  // behind the packing kernels on `stream`
  c10::hip::HIPStream stream;
  int64_t bytes = 0;
};

bool stream_is_capturing(const c10::hip::HIPStream& s) {
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(s.stream(), &st) != hipSuccess) {
    (void)hipGetLastError();
    return true;  // unknown: take the safe side
  }
  return st != hipStreamCaptureStatusNone;
}

class PlainWeightCache {
 public:
  static PlainWeightCache& get() {
    static PlainWeightCache c;
    return c;
  }
  bool enabled() const { return enabled_; }
  // `on`: the stream the caller is about to launch on.
  bool find(const at::Tensor& w, const at::Tensor& sc, const at::Tensor& zp, const std::array<int64_t, 8>& geom,
            const c10::hip::HIPStream& on, at::Tensor* packed, at::Tensor* colsum, at::Tensor* scales_f32) {
    const bool capturing = stream_is_capturing(on);
    std::lock_guard<std::mutex> lock(mu_);
    for (auto it = entries_.begin(); it != entries_.end(); ++it) {
      if (it->geometry == geom && it->weight.matches(w) && it->scales.matches(sc) && it->zero_points.matches(zp)) {
        if (capturing && !it->ready->query()) break;  // packing still in flight: not usable inside a capture
        if (!capturing && it->stream != on) {
          it->ready->block(on.stream());
          for (const at::Tensor* t : {&it->packed, &it->colsum, &it->scales_f32})
            c10::hip::HIPCachingAllocator::recordStream(t->storage().data_ptr(), on);
          ++cross_stream_hits_;
        }
        entries_.splice(entries_.begin(), entries_, it);  // most recently used first
        *packed = it->packed;
        *colsum = it->colsum;
        *scales_f32 = it->scales_f32;
        ++hits_;
        return true;
      }
    }
    ++misses_;
    return false;
  }
  // Call after the packing kernels were queued on `on`.
  void insert(const at::Tensor& w, const at::Tensor& sc, const at::Tensor& zp, const std::array<int64_t, 8>& geom,
              const c10::hip::HIPStream& on, const at::Tensor& packed, const at::Tensor& colsum,
              const at::Tensor& scales_f32) {
    if (stream_is_capturing(on)) return;
    auto ready = std::make_shared<ReadyEvent>();
    ready->record(on.stream());
    const int64_t bytes = static_cast<int64_t>(packed.nbytes() + colsum.nbytes() + scales_f32.nbytes());
    std::lock_guard<std::mutex> lock(mu_);
    entries_.remove_if([this](const PlainWeightEntry& e) {
      const bool dead = !(e.weight.alive() && e.scales.alive() && e.zero_points.alive());
      if (dead) bytes_ -= e.bytes;
      return dead;
    });
    if (bytes > max_bytes_) return;  // larger than the whole budget: never kept
    entries_.push_front(PlainWeightEntry{TensorIdentity(w), TensorIdentity(sc), TensorIdentity(zp), geom, packed,
                                         colsum, scales_f32, std::move(ready), on, bytes});
    bytes_ += bytes;
    while (bytes_ > max_bytes_ || entries_.size() > kMaxEntries) {
      bytes_ -= entries_.back().bytes;
      entries_.pop_back();
      ++evictions_;
    }
  }
  void clear() {
    std::lock_guard<std::mutex> lock(mu_);
    entries_.clear();
    bytes_ = 0;
  }
  void set_max_bytes(int64_t b) {
    std::lock_guard<std::mutex> lock(mu_);
    max_bytes_ = b < 0 ? 0 : b;
    while (bytes_ > max_bytes_ && !entries_.empty()) {
      bytes_ -= entries_.back().bytes;
      entries_.pop_back();
      ++evictions_;
    }
  }
  void counters(int64_t* out, int n) {
    std::lock_guard<std::mutex> lock(mu_);
    const int64_t v[7] = {hits_, misses_, static_cast<int64_t>(entries_.size()), bytes_, max_bytes_, evictions_,
                          cross_stream_hits_};
    for (int i = 0; i < n && i < 7; ++i) out[i] = v[i];
  }

 private:
  PlainWeightCache() {
    const char* e = std::getenv("TMQ_PLAIN_WEIGHT_CACHE");
    enabled_ = !(e != nullptr && e[0] == '0');
    if (const char* mb = std::getenv("TMQ_PLAIN_WEIGHT_CACHE_MB")) {
      char* end = nullptr;
      const long long v = std::strtoll(mb, &end, 10);
      if (end != mb && v >= 0) max_bytes_ = static_cast<int64_t>(v) << 20;
    }
  }
  // Bounded by bytes (packed copies are the size of the weights: a 7 B-parameter model's
  // linear layers are about 7 GB), with a cap on the entry count that keeps a lookup short.
  static constexpr size_t kMaxEntries = 4096;
  std::mutex mu_;
  std::list<PlainWeightEntry> entries_;
  int64_t bytes_ = 0, max_bytes_ = int64_t{16} << 30;
  int64_t hits_ = 0, misses_ = 0, evictions_ = 0, cross_stream_hits_ = 0;
  bool enabled_ = true;
};

constexpr const char* kPackBeforeCapture =
    ": this weight has not been packed yet (or its packing is still in flight) and the current stream is being "
    "captured into a graph; call the operator once on these weight tensors outside the capture first";

bool plain_cacheable(const at::Tensor& w, const at::Tensor& sc, const at::Tensor& zp) {
  return PlainWeightCache::get().enabled() && TensorIdentity::cacheable(w) && TensorIdentity::cacheable(sc) &&
         TensorIdentity::cacheable(zp);
}

at::Tensor qlinear_per_tensor_run(at::Tensor act, double act_scale, int64_t act_zero_point, at::Tensor weight,
                                  at::Tensor weight_scales, at::Tensor weight_zero_points,
                                  std::optional<at::Tensor> bias, double output_scale, int64_t output_zero_point,
                                  std::optional<c10::ScalarType> output_dtype, c10::string_view post_op_name,
                                  torch::List<std::optional<at::Scalar>> /*post_op_args*/,
                                  c10::string_view /*post_op_algorithm*/) {
  const char* what = "quantized::linear_per_tensor";
  TORCH_CHECK(act.dim() == 2, "qlinear: input dim should be 2, but got", act.dim());
  TORCH_CHECK(weight.dim() == 2 && weight.scalar_type() == c10::kChar, what, ": weight must be a 2-D int8 tensor");
  const bool x_signed = plain_signed(act, what);
  const std::string post(post_op_name.data(), post_op_name.size());
  TORCH_CHECK(post == "none" || post == "relu" || post == "tanh" || post == "gelu", what,
              ": unsupported post op ", post);
  const c10::OptionalDeviceGuard guard(at::device_of(act));
  const int64_t M = act.size(0), K = act.size(1), N = weight.size(1);
  TORCH_CHECK(weight.size(0) == K, what, ": weight is [", weight.size(0), ", ", N, "], the input has ", K, " features");
  TORCH_CHECK(act_scale > 0 && output_scale > 0, what, ": scales must be positive");
  const PlainOut o = plain_out(output_dtype, act.scalar_type(), what);
  std::optional<at::Tensor> b;
  if (bias.has_value() && bias->defined()) {
    TORCH_CHECK(bias->numel() == N, what, ": bias must have ", N, " elements");
    b = bias->to(act.device(), at::kFloat).contiguous();
  }
  const bool float_path = !o.is_int || post == "tanh" || post == "gelu";
  at::Tensor y = float_path ? at::empty({M, N}, act.options().dtype(at::kFloat))
                            : at::empty({M, N}, act.options().dtype(o.dtype));
  const auto stream = current_stream(act);
  const at::Tensor x = act.contiguous();
  if (y.numel() == 0) return float_path ? plain_requant(y, output_scale, output_zero_point, o) : y;
  // weight side: re-tiled copy, column sums and fp32 scales, made once per weight
  at::Tensor packed, colsum, ws;
  const std::array<int64_t, 8> geom{0, N, K, act.device().index(), 0, 0, 0, 0};
  const bool cacheable = plain_cacheable(weight, weight_scales, weight_zero_points);
  const auto hstream = c10::hip::getCurrentHIPStream(act.device().index());
  if (!cacheable ||
      !PlainWeightCache::get().find(weight, weight_scales, weight_zero_points, geom, hstream, &packed, &colsum, &ws)) {
    TORCH_CHECK(!stream_is_capturing(hstream), what, kPackBeforeCapture);
    ws = plain_weight_scales(weight_scales, weight_zero_points, N, act, what);
    packed = at::empty({std::max<int64_t>(tmq_linear_packed_bytes(N, K), 16)}, act.options().dtype(at::kByte));
    colsum = at::empty({N}, act.options().dtype(at::kInt));
    const at::Tensor w_nk = weight.t().contiguous();  // [N, K], the layout the prepack reads
    check_status(tmq_linear_prepack(cptr<int8_t>(w_nk), N, K, K, packed.data_ptr(), mptr<int32_t>(colsum), stream),
                 "tmq_linear_prepack");
    if (cacheable)
      PlainWeightCache::get().insert(weight, weight_scales, weight_zero_points, geom, hstream, packed, colsum, ws);
  }
  tmq_linear_desc d{};
  d.M = M;
  d.N = N;
  d.K = K;
  d.x = x.data_ptr();
  d.ldx = K;
  d.x_signed = x_signed;
  d.x_zero_point = static_cast<int32_t>(act_zero_point);
  d.x_scale = static_cast<float>(act_scale);
  d.w_packed = packed.const_data_ptr();
  d.w_colsum = cptr<int32_t>(colsum);
  d.w_scales = cptr<float>(ws);
  d.w_per_channel = ws.numel() > 1;
  d.relu = post == "relu";
  d.bias = b.has_value() ? cptr<float>(*b) : nullptr;
  const at::Tensor split_ws = attach_linear_workspace(d, act.options());
  if (float_path) {
    check_status(tmq_linear_f32(&d, nullptr, mptr<float>(y), N, stream), "tmq_linear_f32");
    if (post == "tanh") y = at::tanh(y);
    if (post == "gelu") y = at::gelu(y);
    return plain_requant(y, output_scale, output_zero_point, o);
  }
  d.out_scale = static_cast<float>(output_scale);
  d.out_zero_point = static_cast<int32_t>(output_zero_point);
  d.out_signed = o.is_signed;
  d.y = y.data_ptr();
  d.ldy = N;
  check_status(tmq_linear(&d, stream), "tmq_linear");
  return y;
}

// Shared body of quantized::conv and quantized::conv_binary.
at::Tensor qconv_plain(const at::Tensor& act, double act_scale, int64_t act_zero_point, const at::Tensor& weight,
                       const at::Tensor& weight_scales, const at::Tensor& weight_zero_points,
                       const std::optional<at::Tensor>& accum, double accum_scale, int64_t accum_zero_point,
                       double alpha, const std::optional<at::Tensor>& bias, const torch::List<int64_t>& stride,
                       const torch::List<int64_t>& padding, const torch::List<int64_t>& dilation, int64_t groups,
                       double output_scale, int64_t output_zero_point, std::optional<c10::ScalarType> output_dtype,
                       bool relu, const char* what) {
  TORCH_CHECK(act.dim() == 4 && weight.dim() == 4, what, ": expected 4-D input and weight");
  TORCH_CHECK(weight.scalar_type() == c10::kChar, what, ": weight must be int8");
  TORCH_CHECK(stride.size() == 2 && padding.size() == 2 && dilation.size() == 2, what,
              ": stride, padding and dilation need two elements each");
  const bool x_signed = plain_signed(act, what);
  TORCH_CHECK(act_scale > 0 && output_scale > 0, what, ": scales must be positive");
  const c10::OptionalDeviceGuard guard(at::device_of(act));
  const PlainOut o = plain_out(output_dtype, act.scalar_type(), what);
  tmq_conv2d_desc d{};
  tmq_conv2d_geom& g = d.geom;
  g.B = act.size(0);
  g.IC = act.size(1);
  g.H = act.size(2);
  g.W = act.size(3);
  g.OC = weight.size(0);
  g.KH = weight.size(2);
  g.KW = weight.size(3);
  g.stride_h = stride[0];
  g.stride_w = stride[1];
  g.pad_h = padding[0];
  g.pad_w = padding[1];
  g.dil_h = dilation[0];
  g.dil_w = dilation[1];
  g.groups = groups;
  TORCH_CHECK(groups > 0 && g.OC % groups == 0 && g.IC == weight.size(1) * groups, what, ": input has ", g.IC,
              " channels, weight expects ", weight.size(1) * groups, " in ", groups, " groups");
  std::optional<at::Tensor> b;
  if (bias.has_value() && bias->defined()) {
    TORCH_CHECK(bias->numel() == g.OC, what, ": bias must have ", g.OC, " elements");
    b = bias->to(act.device(), at::kFloat).contiguous();
  }
  int64_t OH = (g.H + 2 * g.pad_h - g.dil_h * (g.KH - 1) - 1) / g.stride_h + 1;
  int64_t OW = (g.W + 2 * g.pad_w - g.dil_w * (g.KW - 1) - 1) / g.stride_w + 1;
  TORCH_CHECK(OH > 0 && OW > 0, what, ": the kernel does not fit the padded input");
  const auto stream = current_stream(act);
  const at::Tensor x = act.contiguous(c10::MemoryFormat::ChannelsLast);
  // weight side: re-tiled copy, column sums and fp32 scales, made once per weight (the
  // packing depends on the weight's shape and the group count, not on the image)
  at::Tensor packed, colsum, ws;
  const std::array<int64_t, 8> geom{1, g.OC, g.IC, g.KH, g.KW, g.groups, act.device().index(), 0};
  const bool cacheable = g.B > 0 && plain_cacheable(weight, weight_scales, weight_zero_points);
  const auto hstream = c10::hip::getCurrentHIPStream(act.device().index());
  if (!cacheable ||
      !PlainWeightCache::get().find(weight, weight_scales, weight_zero_points, geom, hstream, &packed, &colsum, &ws)) {
    TORCH_CHECK(!stream_is_capturing(hstream), what, kPackBeforeCapture);
    ws = plain_weight_scales(weight_scales, weight_zero_points, g.OC, act, what);
    const at::Tensor w_ohwi = weight.permute({0, 2, 3, 1}).contiguous();
    packed = at::empty({std::max<int64_t>(tmq_conv2d_packed_bytes(&g), 16)}, act.options().dtype(at::kByte));
    colsum = at::empty({g.OC}, act.options().dtype(at::kInt));
    if (g.B > 0)
      check_status(tmq_conv2d_prepack(cptr<int8_t>(w_ohwi), &g, packed.data_ptr(), mptr<int32_t>(colsum), stream),
                   "tmq_conv2d_prepack");
    if (cacheable)
      PlainWeightCache::get().insert(weight, weight_scales, weight_zero_points, geom, hstream, packed, colsum, ws);
  }
  d.x = x.data_ptr();
  d.x_signed = x_signed;
  d.x_zero_point = static_cast<int32_t>(act_zero_point);
  d.x_scale = static_cast<float>(act_scale);
  d.w_per_channel = ws.numel() > 1;
  d.w_packed = packed.const_data_ptr();
  d.w_colsum = cptr<int32_t>(colsum);
  d.w_scales = cptr<float>(ws);
  d.bias = b.has_value() ? cptr<float>(*b) : nullptr;
  const std::vector<int64_t> out_shape{g.B, g.OC, OH, OW};
  if (accum.has_value())
    TORCH_CHECK(accum->sizes() == c10::IntArrayRef(out_shape) && accum->device() == act.device(), what,
                ": accum must have the output's shape ", c10::IntArrayRef(out_shape), " and device");
  at::Tensor workspace;  // (as in PackedConvWeightTmq::apply)
  const int64_t ws_bytes = tmq_conv2d_workspace_bytes(&g);
  if (ws_bytes > 0) {
    workspace = at::empty({ws_bytes}, act.options().dtype(at::kByte));
    d.workspace = workspace.data_ptr();
    d.workspace_bytes = ws_bytes;
  }
  if (!o.is_int) {
    // float output: exact int32 accumulators from the MFMA kernel, scaled here
    TORCH_CHECK(!accum.has_value() || accum_scale == 1.0, "fp32 or bf16 output, accum_scale must be 1.0.");
    at::Tensor acc = at::empty({g.B, OH, OW, g.OC}, act.options().dtype(at::kInt));
    if (acc.numel() > 0) check_status(tmq_conv2d_acc32(&d, mptr<int32_t>(acc), stream), "tmq_conv2d_acc32");
    at::Tensor r = acc.to(at::kFloat) * (ws * static_cast<float>(act_scale));
    if (b.has_value()) r = r + *b;
    r = r.permute({0, 3, 1, 2});  // NCHW-shaped, channels-last in memory
    if (accum.has_value()) r = r + (accum->to(at::kFloat) - accum_zero_point) * (accum_scale * alpha);
    if (relu) r = at::relu(r);
    return r.to(o.dtype);
  }
  at::Tensor y = at::empty(out_shape, act.options().dtype(o.dtype), c10::MemoryFormat::ChannelsLast);
  if (y.numel() == 0) return y;
  d.out_scale = static_cast<float>(output_scale);
  d.out_zero_point = static_cast<int32_t>(output_zero_point);
  d.out_signed = o.is_signed;
  d.relu = relu;
  d.y = y.data_ptr();
  if (!accum.has_value()) {
    check_status(tmq_conv2d(&d, stream), "tmq_conv2d");
    return y;
  }
  const bool a_signed = plain_signed(*accum, what);
  const at::Tensor a_nhwc = accum->contiguous(c10::MemoryFormat::ChannelsLast);
  tmq_conv2d_post post{};
  post.accum = a_nhwc.data_ptr();
  post.accum_signed = a_signed;
  post.accum_zero_point = static_cast<int32_t>(accum_zero_point);
  post.accum_scale = static_cast<float>(accum_scale * alpha);
  post.activation = relu ? 1 : 0;
  check_status(tmq_conv2d_fused(&d, &post, stream), "tmq_conv2d_fused");
  return y;
}

at::Tensor qconv_pointwise_run(at::Tensor act, double act_scale, int64_t act_zero_point, at::Tensor weight,
                               at::Tensor weight_scales, at::Tensor weight_zero_points,
                               std::optional<at::Tensor> bias, torch::List<int64_t> stride,
                               torch::List<int64_t> padding, torch::List<int64_t> dilation, int64_t groups,
                               double output_scale, int64_t output_zero_point,
                               std::optional<c10::ScalarType> output_dtype, c10::string_view attr,
                               torch::List<std::optional<at::Scalar>> /*scalars*/,
                               std::optional<c10::string_view> /*algorithm*/) {
  const std::string a(attr.data(), attr.size());
  // the reference also lets hardtanh / hardswish / swish through its check and then
  // ignores them (mudnn/Qconv.cpp:38-44,63-65); they are refused here instead
  TORCH_CHECK(a == "none" || a == "relu", "quantized::conv: unsupported post operation ", a);
  return qconv_plain(act, act_scale, act_zero_point, weight, weight_scales, weight_zero_points, std::nullopt, 1.0, 0,
                     1.0, bias, stride, padding, dilation, groups, output_scale, output_zero_point, output_dtype,
                     a == "relu", "quantized::conv");
}

at::Tensor qconv_binary_run(at::Tensor act, double act_scale, int64_t act_zero_point, at::Tensor weight,
                            at::Tensor weight_scales, at::Tensor weight_zero_points, at::Tensor accum,
                            std::optional<at::Tensor> bias, torch::List<int64_t> stride,
                            torch::List<int64_t> padding, torch::List<int64_t> dilation, int64_t groups,
                            double output_scale, int64_t output_zero_point,
                            std::optional<c10::ScalarType> output_dtype, double accum_scale,
                            int64_t accum_zero_point, c10::string_view binary_attr, std::optional<at::Scalar> alpha,
                            std::optional<c10::string_view> unary_attr,
                            torch::List<std::optional<at::Scalar>> /*unary_scalars*/,
                            std::optional<c10::string_view> /*unary_algorithm*/) {
  const std::string bin(binary_attr.data(), binary_attr.size());
  const std::string un = unary_attr.has_value() ? std::string(unary_attr->data(), unary_attr->size()) : "none";
  TORCH_CHECK(act.dim() == 4 && bin == "sum" && (un == "none" || un == "relu"),
              "post_op sum or post_op sum_relu is supported for quantized pointwise conv2d. Got binary_post_op: ",
              bin, " unary_post_op: ", un, ".");
  return qconv_plain(act, act_scale, act_zero_point, weight, weight_scales, weight_zero_points, accum, accum_scale,
                     accum_zero_point, alpha.has_value() ? alpha->to<double>() : 1.0, bias, stride, padding, dilation,
                     groups, output_scale, output_zero_point, output_dtype, un == "relu", "quantized::conv_binary");
}

}  // namespace

// The two SiLU schemas are not part of upstream PyTorch; the reference adds them
// by patching ATen's quantized/library.cpp
// (torch_patches/aten_src_ATen_native_quantized_library.cpp.patch:9,12).  Here
// they are defined from this library.
TORCH_LIBRARY_FRAGMENT(quantized, m) {
  m.def(TORCH_SELECTIVE_SCHEMA(
      "quantized::conv2d_silu.new(Tensor qx, __torch__.torch.classes.quantized.Conv2dPackedParamsBase "
      "packed_weight, float output_scale, int output_zero_point) -> Tensor"));
  m.def(TORCH_SELECTIVE_SCHEMA(
      "quantized::conv2d_add_silu(Tensor qx, Tensor qaccum, "
      "__torch__.torch.classes.quantized.Conv2dPackedParamsBase packed_weight, float output_scale, "
      "int output_zero_point) -> Tensor"));
  // torch_patches/aten_src_ATen_native_quantized_library.cpp.patch:20-22
  m.def(TORCH_SELECTIVE_SCHEMA(
      "quantized::linear_per_tensor(Tensor qx, float x_scale, int x_zero_point, Tensor qw, Tensor w_scale, "
      "Tensor w_zero_point,  Tensor? bias, float output_scale, int output_zero_point, ScalarType? output_dtype, "
      "str post_op_name, Scalar?[] post_op_args, str post_op_algorithm) -> Tensor"));
  m.def(TORCH_SELECTIVE_SCHEMA(
      "quantized::conv(Tensor qx, float x_scale, int x_zero_point, Tensor qw, Tensor w_scale, Tensor w_zero_point, "
      "Tensor? bias, int[] stride, int[] padding, int[] dilation, int groups, float output_scale, "
      "int output_zero_point, ScalarType? output_dtype, str attr, Scalar?[] scalars, str? algorithm) -> Tensor"));
  m.def(TORCH_SELECTIVE_SCHEMA(
      "quantized::conv_binary(Tensor qx, float x_scale, int x_zero_point, Tensor qw, Tensor w_scale, "
      "Tensor w_zero_point, Tensor qaccum, Tensor? bias, int[] stride, int[] padding, int[] dilation, int groups, "
      "float output_scale, int output_zero_point, ScalarType? output_dtype, float accum_scale, "
      "int accum_zero_point, str binary_attr, Scalar? alpha, str? unary_attr, Scalar?[] unary_scalars, "
      "str? unary_algorithm) -> Tensor"));
}

TORCH_LIBRARY_IMPL(quantized, QuantizedCUDA, m) {
  m.impl(TORCH_SELECTIVE_NAME("quantized::conv2d_add"), TORCH_FN(qconv2d_add_run));
  m.impl(TORCH_SELECTIVE_NAME("quantized::conv2d_add_relu"), TORCH_FN(qconv2d_add_relu_run));
  m.impl(TORCH_SELECTIVE_NAME("quantized::conv2d_silu.new"), TORCH_FN(qconv2d_silu_run));
  m.impl(TORCH_SELECTIVE_NAME("quantized::conv2d_add_silu"), TORCH_FN(qconv2d_add_silu_run));
  m.impl(TORCH_SELECTIVE_NAME("quantized::cat"), TORCH_FN(qcat_run));
  m.impl(TORCH_SELECTIVE_NAME("quantized::cat_out"), TORCH_FN(qcat_out_run));
  m.impl(TORCH_SELECTIVE_NAME("quantized::add"), TORCH_FN(qadd_run));
  m.impl(TORCH_SELECTIVE_NAME("quantized::add_relu"), TORCH_FN(qadd_relu_run));
  m.impl(TORCH_SELECTIVE_NAME("quantized::linear"), TORCH_FN(qlinear_run));
  m.impl(TORCH_SELECTIVE_NAME("quantized::linear_relu"), TORCH_FN(qlinear_relu_run));
  m.impl(TORCH_SELECTIVE_NAME("quantized::linear_prepack"), TORCH_FN(qlinear_prepack_run));
  m.impl(TORCH_SELECTIVE_NAME("quantized::conv2d.new"), TORCH_FN(qconv2d_run));
  m.impl(TORCH_SELECTIVE_NAME("quantized::conv2d_relu.new"), TORCH_FN(qconv2d_relu_run));
  m.impl(TORCH_SELECTIVE_NAME("quantized::conv2d_prepack"), TORCH_FN(qconv2d_prepack_run));
  m.impl(TORCH_SELECTIVE_NAME("quantized::conv1d_prepack"), TORCH_FN(qconv1d_prepack_run));
  m.impl(TORCH_SELECTIVE_NAME("quantized::conv1d"), TORCH_FN(qconv1d_run));
  m.impl(TORCH_SELECTIVE_NAME("quantized::conv1d_relu"), TORCH_FN(qconv1d_relu_run));
}

// float activations arrive under the plain CUDA key
TORCH_LIBRARY_IMPL(quantized, CUDA, m) {
  m.impl(TORCH_SELECTIVE_NAME("quantized::linear_dynamic"), TORCH_FN(qlinear_dynamic_run));
  m.impl(TORCH_SELECTIVE_NAME("quantized::linear_relu_dynamic"), TORCH_FN(qlinear_relu_dynamic_run));
  // plain uint8 / int8 tensors with their parameters beside them
  m.impl(TORCH_SELECTIVE_NAME("quantized::linear_per_tensor"), TORCH_FN(qlinear_per_tensor_run));
  m.impl(TORCH_SELECTIVE_NAME("quantized::conv"), TORCH_FN(qconv_pointwise_run));
  m.impl(TORCH_SELECTIVE_NAME("quantized::conv_binary"), TORCH_FN(qconv_binary_run));
}

// Replacing PyTorch's own GPU kernel of aten::quantize_per_tensor_dynamic is the
// point of the registration below; the dispatcher's "overriding a previously
// registered kernel" notice is muted for exactly that one registration
// (static objects of one translation unit are constructed in order).
namespace {
struct MuteWarnings final : c10::WarningHandler {
  void process(const c10::Warning&) override {}
} g_mute;
struct MuteOn {
  MuteOn() : previous(c10::WarningUtils::get_warning_handler()) {
    c10::WarningUtils::set_warning_handler(&g_mute);
  }
  c10::WarningHandler* previous;
} const g_mute_on;
}  // namespace

TORCH_LIBRARY_IMPL(aten, CUDA, m) {
  m.impl("quantize_per_tensor_dynamic", TORCH_FN(quantize_per_tensor_dynamic));
}
// one kernel instead of PyTorch-ROCm's int_repr / compare / where / re-wrap chain
TORCH_LIBRARY_IMPL(aten, QuantizedCUDA, m) {
  m.impl("relu", TORCH_FN(qrelu_run));
  m.impl("quantized_max_pool2d", TORCH_FN(qmaxpool2d_run));
  m.impl("_adaptive_avg_pool2d", TORCH_FN(qadaptive_avgpool2d_run));
  m.impl("gelu", TORCH_FN(qgelu_run));
  m.impl("sigmoid", TORCH_FN(qsigmoid_run));
  m.impl("cat", TORCH_FN(qcat_aten_run));
  m.impl("cat.out", TORCH_FN(qcat_aten_out_run));
  m.impl("add.Tensor", TORCH_FN(qadd_tensor_run));
  m.impl("upsample_nearest2d", TORCH_FN(qupsample_nearest2d_run));
}

namespace {
struct MuteOff {
  MuteOff() { c10::WarningUtils::set_warning_handler(g_mute_on.previous); }
} const g_mute_off;
}  // namespace

// Controls of the packed-weight cache of the plain-tensor ops (ctypes, for tests
// and for callers that want the memory back).
extern "C" __attribute__((visibility("default"))) void tmq_aten_plain_weight_cache_clear() {
  PlainWeightCache::get().clear();
}
extern "C" __attribute__((visibility("default"))) void tmq_aten_plain_weight_cache_counters(int64_t* hits,
                                                                                             int64_t* misses,
                                                                                             int64_t* entries) {
  int64_t v[3] = {0, 0, 0};
  PlainWeightCache::get().counters(v, 3);
  *hits = v[0];
  *misses = v[1];
  *entries = v[2];
}
// out[0..n): hits, misses, entries, bytes held, byte limit, evictions, hits from a stream
// other than the one that packed the entry.
extern "C" __attribute__((visibility("default"))) void tmq_aten_plain_weight_cache_stats(int64_t* out, int n) {
  PlainWeightCache::get().counters(out, n);
}
// The byte limit (default 16 GiB, or TMQ_PLAIN_WEIGHT_CACHE_MB in the environment);
// entries beyond it leave, least recently used first.
extern "C" __attribute__((visibility("default"))) void tmq_aten_plain_weight_cache_set_max_bytes(int64_t bytes) {
  PlainWeightCache::get().set_max_bytes(bytes);
}
