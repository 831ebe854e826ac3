// ChooseQuantizationParams for host and device code.
#pragma once

#include <cmath>
#include <cstdint>

#include <hip/hip_runtime.h>

namespace tmq {

// ChooseQuantizationParams, shared by host and device
// (ATen/native/quantized/cpu/QuantUtils.h:71-187).
__host__ __device__ inline void choose_qparams(float min, float max, int qmin, int qmax,
                                               bool reduce_range, double* out_scale,
                                               int32_t* out_zp) {
  if (reduce_range) {
    qmin = qmin / 2;
    qmax = qmax / 2;
  }
  min = fminf(min, 0.f);
  max = fmaxf(max, 0.f);
  double scale = (static_cast<double>(max) - min) / (qmax - qmin);
  const float scale_f = static_cast<float>(scale);
  if (scale_f == 0.0f || __builtin_isinf(1.0f / scale_f)) scale = 0.1;
  constexpr float kSmall = 6.1e-5f;
  if (scale < kSmall) {
    const float org_scale = static_cast<float>(scale);
    scale = kSmall;
    if (min == 0.0f) {
      max = kSmall * (qmax - qmin);
    } else if (max == 0.0f) {
      min = -kSmall * (qmax - qmin);
    } else {
      const float amplifier = kSmall / org_scale;
      min *= amplifier;
      max *= amplifier;
    }
  }
  const double zp_from_min = qmin - min / scale;
  const double zp_from_max = qmax - max / scale;
  const double err_min = (qmin < 0 ? -qmin : qmin) - fabs(min / scale);
  const double err_max = (qmax < 0 ? -qmax : qmax) - fabs(max / scale);
  const double initial = err_min < err_max ? zp_from_min : zp_from_max;
  int32_t nudged;
  if (initial < qmin) {
    nudged = qmin;
  } else if (initial > qmax) {
    nudged = qmax;
  } else {
    nudged = static_cast<int32_t>(rint(initial));
  }
  *out_scale = scale;
  *out_zp = nudged;
}


}  // namespace tmq
