/*
 * TEST INFRASTRUCTURE ONLY -- never linked, imported or called by the product.
 *
 * Scalar CPU restatement of the arithmetic that PyTorch's CPU quantized ops
 * (the numerics torch_musa's quantized operators are tested against,
 * reference torch_musa/testing/base_test_tool.py:814-825 "run on cpu, run on
 * device, compare") apply on the quantized-inference path:
 *
 *   quantize_per_tensor / quantize_per_channel / dequantize  (affine quantizer)
 *   quantize_per_tensor_dynamic's qparams selection
 *   quantized::linear  and  quantized::conv2d  (int32 accumulate + fp32 requant)
 *
 * The arithmetic itself lives in third-party code that is not under the
 * reference tree: PyTorch v2.7.1 ATen (reference build.sh:30 pins it) with its
 * bundled fbgemm.  Each function names the published header it restates
 * (paths relative to the torch wheel's include/ directory) and the reference
 * call site it stands behind.
 *
 * Pinning status (see tests/test_oracle_*.py):
 *   every function below is checked against golden vectors produced by the
 *   installed PyTorch CPU ops (tests/golden/make_golden.py, engine 'fbgemm')
 *   and against independent mathematical checks (exact int64 matmul, brute
 *   force over all 256 codes, ties-to-even cases, closed-form special cases).
 *   No function is "parity unpinned".
 *
 * Build: make -C oracle   (gcc -O2 -ffp-contract=off -fopenmp)
 * All fp32 steps are written so that no FMA contraction or excess precision can
 * change a result: every intermediate is stored to a float before the next op.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API __attribute__((visibility("default")))

static inline int64_t clamp_i64(int64_t v, int64_t lo, int64_t hi) {
  return v < lo ? lo : (v > hi ? hi : v);
}

ORC_API int orc_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* ------------------------------------------------------------------------- */
/* quantize, one element.  fbgemm/QuantUtils.h:67-101, non-LEGACY branch :95:
 *   inv = 1.0f / scale_f;  t = x * inv;  t = zp + nearbyint(t);  clamp.
 * Stands behind reference AffineQuantizer.mu:35-77 (device kernel) through the
 * op row musa_functions.yaml:3509-3513.  Domain of parity: finite x with
 * |x*inv| < 2^31 (outside it the CPU op's own result depends on its vector ISA).
 */
static inline int32_t quantize_one(float x, float inv, int64_t zp, int64_t qmin,
                                   int64_t qmax) {
  volatile float t = x * inv;          /* one fp32 rounding */
  float r = nearbyintf(t);             /* round-half-to-even (FE_TONEAREST) */
  if (!(r > -2147483648.0f)) return (int32_t)qmin; /* outside the parity domain */
  if (!(r < 2147483648.0f)) return (int32_t)qmax;
  return (int32_t)clamp_i64((int64_t)r + zp, qmin, qmax);
}

static inline void qrange(int is_signed, int64_t* qmin, int64_t* qmax) {
  *qmin = is_signed ? -128 : 0;
  *qmax = is_signed ? 127 : 255;
}

/* x[n] fp32 -> q[n] bytes (two's complement when is_signed). */
ORC_API void orc_quantize_per_tensor(const float* x, int64_t n, double scale,
                                     int64_t zp, int is_signed, uint8_t* q,
                                     int nthreads) {
  int64_t qmin, qmax;
  qrange(is_signed, &qmin, &qmax);
  const float scale_f = (float)scale;
  const float inv = 1.0f / scale_f;
  (void)nthreads;
#pragma omp parallel for num_threads(nthreads > 0 ? nthreads : 1) schedule(static)
  for (int64_t i = 0; i < n; ++i)
    q[i] = (uint8_t)quantize_one(x[i], inv, zp, qmin, qmax);
}

/* Activation quantization inside PyTorch's CPU quantized::linear_dynamic: the
 * activations are quantized while fbgemm packs them (PackAWithQuantRowOffset;
 * its source is not in this image, the form below is pinned by the op's outputs
 * on inputs chosen where the two forms differ, see tests/golden):
 *   t = fma(x, inv, zp)   (one fp32 rounding);  clip to [qmin, qmax];  round to
 *   nearest even
 * against quantize_one's rne(fl(x * inv)) + zp.  The reference declares
 * apply_dynamic and leaves it unimplemented (mudnn/Linear.h:35-46). */
ORC_API void orc_quantize_per_tensor_fused(const float* x, int64_t n, double scale,
                                           int64_t zp, int is_signed, uint8_t* q,
                                           int nthreads) {
  int64_t qmin, qmax;
  qrange(is_signed, &qmin, &qmax);
  const float scale_f = (float)scale;
  const float inv = 1.0f / scale_f;
  (void)nthreads;
#pragma omp parallel for num_threads(nthreads > 0 ? nthreads : 1) schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    float t = fmaf(x[i], inv, (float)zp);
    t = t < (float)qmin ? (float)qmin : (t > (float)qmax ? (float)qmax : t);
    q[i] = (uint8_t)(int32_t)nearbyintf(t);
  }
}

/* dequantize per tensor.  fbgemm/QuantUtils.h:155-158:
 *   r = scale_f * (float)(int32(q) - zp)
 * Stands behind reference AffineQuantizer.mu:79-97,145-179. */
ORC_API void orc_dequantize_per_tensor(const uint8_t* q, int64_t n, double scale,
                                       int64_t zp, int is_signed, float* r,
                                       int nthreads) {
  const float scale_f = (float)scale;
  (void)nthreads;
#pragma omp parallel for num_threads(nthreads > 0 ? nthreads : 1) schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    int32_t v = is_signed ? (int32_t)(int8_t)q[i] : (int32_t)q[i];
    float d = (float)(int32_t)(v - (int32_t)zp);
    r[i] = scale_f * d;
  }
}

/* per-channel quantize over a tensor viewed as [outer, C, inner] (axis = the C
 * dimension).  ATen quantize_val<T>(scale_c, zp_c, x) -> fbgemm Quantize with
 * scale cast to float, so the per-element formula is the per-tensor one with
 * inv_c = 1.0f / (float)scale_c.  scales are double and zero points int64, the
 * types the dispatch stub hands over (ATen/native/quantized/AffineQuantizer.h:
 * 51-56).  Stands behind reference AffineQuantizer.mu:181-224. */
ORC_API void orc_quantize_per_channel(const float* x, int64_t outer, int64_t C,
                                      int64_t inner, const double* scales,
                                      const int64_t* zps, int is_signed,
                                      uint8_t* q) {
  int64_t qmin, qmax;
  qrange(is_signed, &qmin, &qmax);
  for (int64_t o = 0; o < outer; ++o)
    for (int64_t c = 0; c < C; ++c) {
      const float inv = 1.0f / (float)scales[c];
      const int64_t base = (o * C + c) * inner;
      for (int64_t i = 0; i < inner; ++i)
        q[base + i] = (uint8_t)quantize_one(x[base + i], inv, zps[c], qmin, qmax);
    }
}

/* per-channel dequantize: r = (float)( (double)( (float)q - (float)zp_c ) * scale_c )
 * with scale_c kept in double (the CPU kernel multiplies a float difference by
 * the double scale and narrows once).  Stands behind reference
 * AffineQuantizer.mu:226-257. */
ORC_API void orc_dequantize_per_channel(const uint8_t* q, int64_t outer, int64_t C,
                                        int64_t inner, const double* scales,
                                        const int64_t* zps, int is_signed,
                                        float* r) {
  for (int64_t o = 0; o < outer; ++o)
    for (int64_t c = 0; c < C; ++c) {
      const int64_t base = (o * C + c) * inner;
      const float zf = (float)zps[c];
      for (int64_t i = 0; i < inner; ++i) {
        int32_t v = is_signed ? (int32_t)(int8_t)q[base + i] : (int32_t)q[base + i];
        volatile float d = (float)v - zf;
        r[base + i] = (float)((double)d * scales[c]);
      }
    }
}

/* per-channel quantize with float scales and float zero points (qscheme
 * per_channel_affine_float_qparams).  ATen quantize_val_float_qparams
 * (torch/include/ATen/native/quantized/AffineQuantizerBase.h:44):
 *   inv = scale == 0 ? 1.0f : 1.0f / scale;  q = clamp(lrintf(x * inv + zp)),
 * product and sum each rounded to fp32.  Stands behind reference
 * AffineQuantizer.mu:259-301, which states the same formula (:291-294). */
ORC_API void orc_quantize_per_channel_float(const float* x, int64_t outer, int64_t C,
                                            int64_t inner, const float* scales,
                                            const float* zps, int is_signed, uint8_t* q) {
  int64_t qmin, qmax;
  qrange(is_signed, &qmin, &qmax);
  for (int64_t o = 0; o < outer; ++o)
    for (int64_t c = 0; c < C; ++c) {
      const float inv = scales[c] == 0.0f ? 1.0f : 1.0f / scales[c];
      const int64_t base = (o * C + c) * inner;
      for (int64_t i = 0; i < inner; ++i) {
        volatile float t = x[base + i] * inv;
        volatile float u = t + zps[c];
        int64_t v = (int64_t)lrintf(u);
        if (v < qmin) v = qmin;
        if (v > qmax) v = qmax;
        q[base + i] = (uint8_t)v;
      }
    }
}

/* its inverse: r = (float(q) - zp_c) * scale_c in fp32 (reference
 * AffineQuantizer.mu:303-336, lambda at :331-333). */
ORC_API void orc_dequantize_per_channel_float(const uint8_t* q, int64_t outer, int64_t C,
                                              int64_t inner, const float* scales,
                                              const float* zps, int is_signed, float* r) {
  for (int64_t o = 0; o < outer; ++o)
    for (int64_t c = 0; c < C; ++c) {
      const int64_t base = (o * C + c) * inner;
      for (int64_t i = 0; i < inner; ++i) {
        int32_t v = is_signed ? (int32_t)(int8_t)q[base + i] : (int32_t)q[base + i];
        volatile float d = (float)v - zps[c];
        r[base + i] = d * scales[c];
      }
    }
}

/* global min / max of a float array (the two reductions that
 * quantize_per_tensor_dynamic performs before choosing qparams,
 * reference musa_functions.yaml:3515-3519). NaN-free input assumed. */
ORC_API void orc_minmax(const float* x, int64_t n, float* out_min, float* out_max,
                        int nthreads) {
  float mn = INFINITY, mx = -INFINITY;
  (void)nthreads;
#pragma omp parallel for num_threads(nthreads > 0 ? nthreads : 1) schedule(static) reduction(min : mn) reduction(max : mx)
  for (int64_t i = 0; i < n; ++i) {
    if (x[i] < mn) mn = x[i];
    if (x[i] > mx) mx = x[i];
  }
  *out_min = mn;
  *out_max = mx;
}

/* ChooseQuantizationParams, ATen/native/quantized/cpu/QuantUtils.h:71-187 with
 * preserve_sparsity = false and force_scale_power_of_two = false (the values
 * quantize_per_tensor_dynamic passes). Returns 0, or 1 when min > max. */
ORC_API int orc_choose_qparams(float min, float max, int32_t qmin, int32_t qmax,
                               int reduce_range, double* out_scale,
                               int32_t* out_zp) {
  if (!(min <= max)) return 1;
  if (reduce_range) {
    qmin = qmin / 2;
    qmax = qmax / 2;
  }
  min = fminf(min, 0.f);
  max = fmaxf(max, 0.f);
  double scale = ((double)max - min) / (qmax - qmin);
  if ((float)scale == 0.0f || isinf(1.0f / (float)scale)) scale = 0.1;
  const float kSmall = 6.1e-5f;
  if (scale < kSmall) {
    float org_scale = (float)scale;
    scale = kSmall;
    if (min == 0.0f) {
      max = kSmall * (qmax - qmin);
    } else if (max == 0.0f) {
      min = -kSmall * (qmax - qmin);
    } else {
      float amplifier = kSmall / org_scale;
      min *= amplifier;
      max *= amplifier;
    }
  }
  double zp_from_min = qmin - min / scale;
  double zp_from_max = qmax - max / scale;
  double err_min = abs(qmin) - fabs(min / scale);
  double err_max = abs(qmax) - fabs(max / scale);
  double initial = err_min < err_max ? zp_from_min : zp_from_max;
  int32_t nudged;
  if (initial < qmin)
    nudged = qmin;
  else if (initial > qmax)
    nudged = qmax;
  else
    nudged = (int32_t)nearbyint(initial);
  *out_scale = scale;
  *out_zp = nudged;
  return 0;
}

/* ------------------------------------------------------------------------- */
/* Raw int32 accumulators of quantized::linear:
 *   acc[m][n] = sum_k X[m][k] * W[n][k]      (X u8 or s8, W s8, exact int32)
 * i.e. what fbgemmPacked hands to its output stage before the column-offset
 * term.  GEMM shape [M,K] x [N,K]^T as in reference mudnn/Linear.cpp:48-58
 * (SetTranspose(false,true)). */
ORC_API void orc_linear_acc32(const uint8_t* x, int x_signed, const int8_t* w,
                              int64_t M, int64_t N, int64_t K, int32_t* acc,
                              int nthreads) {
  (void)nthreads;
#pragma omp parallel for num_threads(nthreads > 0 ? nthreads : 1) schedule(static)
  for (int64_t m = 0; m < M; ++m)
    for (int64_t n = 0; n < N; ++n) {
      int32_t s = 0;
      const uint8_t* xr = x + m * K;
      const int8_t* wr = w + n * K;
      if (x_signed)
        for (int64_t k = 0; k < K; ++k) s += (int32_t)(int8_t)xr[k] * (int32_t)wr[k];
      else
        for (int64_t k = 0; k < K; ++k) s += (int32_t)xr[k] * (int32_t)wr[k];
      acc[m * N + n] = s;
    }
}

/* colsum[n] = sum_k W[n][k]  (fbgemm "col_offsets" for a weight with zp 0). */
ORC_API void orc_weight_colsum(const int8_t* w, int64_t N, int64_t K, int32_t* colsum) {
  for (int64_t n = 0; n < N; ++n) {
    int32_t s = 0;
    for (int64_t k = 0; k < K; ++k) s += w[n * K + k];
    colsum[n] = s;
  }
}

/* One requantisation, fbgemm/OutputProcessing-inl.h:87-127 (scalar branch):
 *   raw   = acc - x_zp * colsum[n]                              (:90-92)
 *   raw_f = (float)raw (+ bias[n] / act_times_w_scale[n])       (:107-118)
 *           per-channel weight scales: the quotient is rounded, then added;
 *           one scale for the whole weight (per-tensor): the vector code of
 *           the CPU op multiplies by the reciprocal and fuses the addition,
 *           raw_f = fma(bias[n], fl(1 / act_times_w_scale), (float)raw);
 *           the two agree except on a few values in a million (pinned by the
 *           op's outputs on cases built where they differ, tests/golden)
 *   ab    = raw_f * C_multiplier[n]                             (:120)
 *   out   = clamp(lrintf(ab) + out_zp, relu ? out_zp : qmin, qmax)  (:121-125)
 * with act_times_w_scale[n] = x_scale_f * w_scale_f[n] and
 * C_multiplier[n] = act_times_w_scale[n] / out_scale_f, all fp32 (qlinear.cpp /
 * qconv.cpp set-up code). `raw` is passed in already corrected by the caller. */
static inline float add_bias(float raw_f, float bias, float atw, int per_tensor) {
  if (per_tensor) {
    volatile float rcp = 1.0f / atw;
    return fmaf(bias, rcp, raw_f);
  }
  volatile float b = bias / atw;
  volatile float sum = raw_f + b;
  return sum;
}

static inline int32_t requant_one(int32_t raw, int has_bias, float bias, float atw,
                                  int per_tensor, float mult, int64_t out_zp, int64_t lo,
                                  int64_t hi) {
  volatile float raw_f = (float)raw;
  if (has_bias) raw_f = add_bias(raw_f, bias, atw, per_tensor);
  volatile float ab = raw_f * mult;
  float r = nearbyintf(ab);
  if (!(r > -2147483648.0f)) return (int32_t)lo;
  if (!(r < 2147483648.0f)) return (int32_t)hi;
  return (int32_t)clamp_i64((int64_t)r + out_zp, lo, hi);
}

/* acc[M][N] (raw, as from orc_linear_acc32) -> y[M][N] bytes.
 * w_scales has N entries (per-channel) or 1 (per-tensor, n_scales == 1).
 * Output range: u8 [0,255] when !out_signed (the CPU op), s8 [-128,127] when
 * out_signed (the reference's device flavour, mudnn/Linear.cpp:99-103). */
ORC_API void orc_requantize(const int32_t* acc, int64_t M, int64_t N,
                            const int32_t* colsum, int64_t x_zp, double x_scale,
                            const double* w_scales, int64_t n_scales,
                            const float* bias, double out_scale, int64_t out_zp,
                            int out_signed, int relu, uint8_t* y) {
  int64_t qmin, qmax;
  qrange(out_signed, &qmin, &qmax);
  const int64_t lo = relu ? (out_zp > qmin ? out_zp : qmin) : qmin;
  const float xs = (float)x_scale;
  const float os = (float)out_scale;
  for (int64_t n = 0; n < N; ++n) {
    const float ws = (float)w_scales[n_scales == 1 ? 0 : n];
    volatile float atw = xs * ws;
    volatile float mult = atw / os;
    for (int64_t m = 0; m < M; ++m) {
      int32_t raw = acc[m * N + n] - (int32_t)x_zp * colsum[n];
      y[m * N + n] = (uint8_t)requant_one(raw, bias != NULL, bias ? bias[n] : 0.f,
                                          atw, n_scales == 1, mult, out_zp, lo, qmax);
    }
  }
}

/* quantized::linear end to end (reference mudnn/Linear.cpp:70-114 op semantics,
 * CPU numerics as above). */
ORC_API void orc_linear(const uint8_t* x, int x_signed, const int8_t* w, int64_t M,
                        int64_t N, int64_t K, int64_t x_zp, double x_scale,
                        const double* w_scales, int64_t n_scales, const float* bias,
                        double out_scale, int64_t out_zp, int out_signed, int relu,
                        uint8_t* y, int nthreads) {
  int32_t* acc = (int32_t*)malloc(sizeof(int32_t) * (size_t)M * (size_t)N);
  int32_t* colsum = (int32_t*)malloc(sizeof(int32_t) * (size_t)N);
  orc_linear_acc32(x, x_signed, w, M, N, K, acc, nthreads);
  orc_weight_colsum(w, N, K, colsum);
  orc_requantize(acc, M, N, colsum, x_zp, x_scale, w_scales, n_scales, bias,
                 out_scale, out_zp, out_signed, relu, y);
  free(acc);
  free(colsum);
}

/* Float output stage of a dynamically quantized linear (PyTorch's CPU
 * quantized::linear_dynamic, fbgemm ReQuantizeForFloat; the reference declares
 * apply_dynamic and leaves it unimplemented, mudnn/Linear.h:35-46):
 *   y[m][n] = fma((float)(acc - x_zp * colsum[n]), fl(x_scale_f * w_scale_f[n]), bias[n])
 * one fused multiply-add per value (what the vectorised CPU kernel executes:
 * separate multiply and add differ from it in the last bit on about a third of
 * the values), then max(y, 0) for the relu variant. */
ORC_API void orc_linear_f32(const uint8_t* x, int x_signed, const int8_t* w, int64_t M,
                            int64_t N, int64_t K, int64_t x_zp, double x_scale,
                            const double* w_scales, int64_t n_scales, const float* bias,
                            int relu, float* y, int nthreads) {
  int32_t* acc = (int32_t*)malloc(sizeof(int32_t) * (size_t)M * (size_t)N);
  int32_t* colsum = (int32_t*)malloc(sizeof(int32_t) * (size_t)N);
  orc_linear_acc32(x, x_signed, w, M, N, K, acc, nthreads);
  orc_weight_colsum(w, N, K, colsum);
  const float xs = (float)x_scale;
  for (int64_t n = 0; n < N; ++n) {
    const float ws = (float)w_scales[n_scales == 1 ? 0 : n];
    volatile float mult = xs * ws;
    const float b = bias ? bias[n] : 0.f;
    for (int64_t m = 0; m < M; ++m) {
      const int32_t raw = acc[m * N + n] - (int32_t)x_zp * colsum[n];
      float v = fmaf((float)raw, mult, b);
      if (relu && !(v > 0.f)) v = 0.f;
      y[m * N + n] = v;
    }
  }
  free(acc);
  free(colsum);
}

/* ------------------------------------------------------------------------- */
/* quantized::conv2d accumulators, NHWC activations x OHWI weights:
 *   acc[b][oh][ow][oc] = sum_{kh,kw,ic} (X[b][ih][iw][g*ICg+ic] - x_zp) * W[oc][kh][kw][ic]
 * over taps that fall inside the image (zero padding in the real domain adds
 * nothing), ih = oh*sh - ph + kh*dh, iw likewise; OH/OW from reference
 * mudnn/Conv.cpp:20-36; layouts from mudnn/Conv.cpp:58-72 (NHWC) and
 * mudnn/ConvPrepack.cpp:78 (OHWI). groups split IC and OC evenly. */
ORC_API void orc_conv2d_acc32(const uint8_t* x, int x_signed, const int8_t* w,
                              int64_t B, int64_t H, int64_t W, int64_t IC,
                              int64_t OC, int64_t KH, int64_t KW, int64_t sh,
                              int64_t sw, int64_t ph, int64_t pw, int64_t dh,
                              int64_t dw, int64_t groups, int64_t x_zp,
                              int32_t* acc, int nthreads) {
  const int64_t OH = (H + 2 * ph - dh * (KH - 1) - 1) / sh + 1;
  const int64_t OW = (W + 2 * pw - dw * (KW - 1) - 1) / sw + 1;
  const int64_t ICg = IC / groups, OCg = OC / groups;
  (void)nthreads;
#pragma omp parallel for num_threads(nthreads > 0 ? nthreads : 1) schedule(static) collapse(2)
  for (int64_t b = 0; b < B; ++b)
    for (int64_t oh = 0; oh < OH; ++oh)
      for (int64_t ow = 0; ow < OW; ++ow)
        for (int64_t oc = 0; oc < OC; ++oc) {
          const int64_t g = oc / OCg;
          int32_t s = 0;
          for (int64_t kh = 0; kh < KH; ++kh) {
            const int64_t ih = oh * sh - ph + kh * dh;
            if (ih < 0 || ih >= H) continue;
            for (int64_t kw = 0; kw < KW; ++kw) {
              const int64_t iw = ow * sw - pw + kw * dw;
              if (iw < 0 || iw >= W) continue;
              const uint8_t* xp = x + ((b * H + ih) * W + iw) * IC + g * ICg;
              const int8_t* wp = w + ((oc * KH + kh) * KW + kw) * ICg;
              for (int64_t ic = 0; ic < ICg; ++ic) {
                int32_t xv = x_signed ? (int32_t)(int8_t)xp[ic] : (int32_t)xp[ic];
                s += (xv - (int32_t)x_zp) * (int32_t)wp[ic];
              }
            }
          }
          acc[((b * OH + oh) * OW + ow) * OC + oc] = s;
        }
}

/* quantized::conv2d end to end; same output stage as linear with one output
 * channel per column (reference mudnn/Conv.cpp:158-204 op semantics). acc is
 * already zero-point corrected, so the column-offset term is zero here. */
ORC_API void orc_conv2d(const uint8_t* x, int x_signed, const int8_t* w, int64_t B,
                        int64_t H, int64_t W, int64_t IC, int64_t OC, int64_t KH,
                        int64_t KW, int64_t sh, int64_t sw, int64_t ph, int64_t pw,
                        int64_t dh, int64_t dw, int64_t groups, int64_t x_zp,
                        double x_scale, const double* w_scales, int64_t n_scales,
                        const float* bias, double out_scale, int64_t out_zp,
                        int out_signed, int relu, uint8_t* y, int nthreads) {
  const int64_t OH = (H + 2 * ph - dh * (KH - 1) - 1) / sh + 1;
  const int64_t OW = (W + 2 * pw - dw * (KW - 1) - 1) / sw + 1;
  const int64_t rows = B * OH * OW;
  int32_t* acc = (int32_t*)malloc(sizeof(int32_t) * (size_t)rows * (size_t)OC);
  int32_t* zero = (int32_t*)calloc((size_t)OC, sizeof(int32_t));
  orc_conv2d_acc32(x, x_signed, w, B, H, W, IC, OC, KH, KW, sh, sw, ph, pw, dh, dw,
                   groups, x_zp, acc, nthreads);
  orc_requantize(acc, rows, OC, zero, 0, x_scale, w_scales, n_scales, bias,
                 out_scale, out_zp, out_signed, relu, y);
  free(acc);
  free(zero);
}

/* ------------------------------------------------------------------------- */
/* Fused residual / activation variants of quantized::conv2d: conv2d_add,
 * conv2d_add_relu (reference mudnn/ConvAdd.cpp:11-39,63-99), conv2d_silu and
 * conv2d_add_silu (mudnn/Conv.cpp:278-288).  The reference hands the whole
 * expression to muDNN's Convolution::RunFusion (mudnn/Conv.cpp:86-130, closed
 * source); its tests define the result as
 *   quantize( act( conv(dq(x), dq(w)) + bias + dq(accum) ) )   within 1 LSB
 * (tests/unittest/quantized/test_quantized_conv.py:159-227, :236-360).
 * This restatement keeps the plain conv's requantisation and adds the residual
 * in output-scale units before the single rounding:
 *   t = (float(raw) + bias/atw) * mult                       (as requant_one)
 *   t = t + float(qa - za) * amult,  amult = fl(fl(accum_scale) / fl(out_scale))
 *   silu: r = t * out_scale;  t = (r / (1 + expf(-r))) / out_scale
 *   q = clamp(rne(t) + out_zp, relu ? out_zp : qmin, qmax)
 * every operation rounded to fp32.  With no accum and no silu this is exactly
 * orc_conv2d.  activation: 0 identity, 1 relu, 2 silu. */
ORC_API void orc_conv2d_fused(const uint8_t* x, int x_signed, const int8_t* w, int64_t B,
                              int64_t H, int64_t W, int64_t IC, int64_t OC, int64_t KH,
                              int64_t KW, int64_t sh, int64_t sw, int64_t ph, int64_t pw,
                              int64_t dh, int64_t dw, int64_t groups, int64_t x_zp,
                              double x_scale, const double* w_scales, int64_t n_scales,
                              const float* bias, const uint8_t* accum, int accum_signed,
                              int64_t accum_zp, double accum_scale, int activation,
                              double out_scale, int64_t out_zp, int out_signed, uint8_t* y,
                              int nthreads) {
  const int64_t OH = (H + 2 * ph - dh * (KH - 1) - 1) / sh + 1;
  const int64_t OW = (W + 2 * pw - dw * (KW - 1) - 1) / sw + 1;
  const int64_t rows = B * OH * OW;
  int32_t* acc = (int32_t*)malloc(sizeof(int32_t) * (size_t)rows * (size_t)OC);
  orc_conv2d_acc32(x, x_signed, w, B, H, W, IC, OC, KH, KW, sh, sw, ph, pw, dh, dw,
                   groups, x_zp, acc, nthreads);
  int64_t qmin, qmax;
  qrange(out_signed, &qmin, &qmax);
  const int64_t lo = activation == 1 ? (out_zp > qmin ? out_zp : qmin) : qmin;
  const float xs = (float)x_scale, os = (float)out_scale;
  volatile float amult = (float)accum_scale / os;
  for (int64_t n = 0; n < OC; ++n) {
    const float ws = (float)w_scales[n_scales == 1 ? 0 : n];
    volatile float atw = xs * ws;
    volatile float mult = atw / os;
    for (int64_t m = 0; m < rows; ++m) {
      volatile float raw_f = (float)acc[m * OC + n];
      if (bias != NULL) raw_f = add_bias(raw_f, bias[n], atw, n_scales == 1);
      volatile float t = raw_f * mult;
      if (accum != NULL) {
        const int32_t qa = accum_signed ? (int32_t)(int8_t)accum[m * OC + n]
                                        : (int32_t)accum[m * OC + n];
        volatile float a = (float)(qa - (int32_t)accum_zp) * amult;
        t = t + a;
      }
      if (activation == 2) {
        volatile float r = t * os;
        volatile float e = expf(-r);
        volatile float d = 1.0f + e;
        volatile float sl = r / d;
        t = sl / os;
      }
      float r = nearbyintf(t);
      int64_t q;
      if (!(r > -2147483648.0f)) q = lo;
      else if (!(r < 2147483648.0f)) q = qmax;
      else q = clamp_i64((int64_t)r + out_zp, lo, qmax);
      y[m * OC + n] = (uint8_t)q;
    }
  }
  free(acc);
}

/* ------------------------------------------------------------------------- */
/* quantized::add / add_relu on two per-tensor quantized tensors of one shape
 * (reference musa/BinaryOps.mu:154-207; the reference evaluates
 * (qa + qb*b_s/a_s)*a_s/out_s in double and clamps the relu variant at 0, not
 * at the zero point).  Restated from PyTorch's CPU kernel, vector body of
 * qadd_kernel (ATen/native/quantized/cpu/kernels/QuantizedOpKernels.cpp):
 *   a = fmaf((float)qa, a_scale, fl(-a_zp * a_scale))
 *   b = fmaf((float)qb, b_scale, fl(-b_zp * b_scale))
 *   c = a + b; relu: c = max(c, 0)
 *   q = clamp(rne(c * fl(1/out_scale)) + out_zp, qmin, qmax)
 * (the scalar tail of the CPU kernel dequantizes with (q - zp) * scale instead
 * of the fused form: about 1e-5 of values differ by one between the two). */
ORC_API void orc_qadd(const uint8_t* qa, const uint8_t* qb, int64_t n, double a_scale,
                      int64_t a_zp, double b_scale, int64_t b_zp, double out_scale,
                      int64_t out_zp, int is_signed, int relu, uint8_t* out) {
  int64_t qmin, qmax;
  qrange(is_signed, &qmin, &qmax);
  const float sa = (float)a_scale, sb = (float)b_scale;
  volatile float pa = -(float)a_zp * sa;
  volatile float pb = -(float)b_zp * sb;
  volatile float inv = 1.0f / (float)out_scale;
  for (int64_t i = 0; i < n; ++i) {
    const int32_t va = is_signed ? (int32_t)(int8_t)qa[i] : (int32_t)qa[i];
    const int32_t vb = is_signed ? (int32_t)(int8_t)qb[i] : (int32_t)qb[i];
    volatile float a = fmaf((float)va, sa, pa);
    volatile float b = fmaf((float)vb, sb, pb);
    volatile float c = a + b;
    if (relu && c < 0.0f) c = 0.0f;
    volatile float t = c * inv;
    int64_t q = (int64_t)nearbyintf(t) + out_zp;
    out[i] = (uint8_t)clamp_i64(q, qmin, qmax);
  }
}

/* relu of a per-tensor quantized tensor: y = max(x, zero_point) (reference
 * musa/Activation.mu:165-186; PyTorch CPU qrelu does the same clamp). */
ORC_API void orc_qrelu(const uint8_t* x, int64_t n, int64_t zp, int is_signed, uint8_t* y) {
  for (int64_t i = 0; i < n; ++i) {
    const int32_t v = is_signed ? (int32_t)(int8_t)x[i] : (int32_t)x[i];
    y[i] = (uint8_t)(v > zp ? v : (int32_t)zp);
  }
}

/* Max pooling over NHWC codes: the maximum of the window's in-image codes
 * (reference Pool.cpp:178-247 hands it to muDNN; PyTorch's CPU
 * quantized_max_pool2d takes the maximum of the underlying integers). */
ORC_API void orc_qmaxpool2d(const uint8_t* x, int64_t B, int64_t H, int64_t W, int64_t C,
                            int64_t kh, int64_t kw, int64_t sh, int64_t sw, int64_t ph, int64_t pw,
                            int64_t dh, int64_t dw, int64_t OH, int64_t OW, int is_signed, uint8_t* y) {
  for (int64_t b = 0; b < B; ++b)
    for (int64_t oh = 0; oh < OH; ++oh)
      for (int64_t ow = 0; ow < OW; ++ow)
        for (int64_t c = 0; c < C; ++c) {
          int32_t m = is_signed ? -128 : 0;
          for (int64_t i = 0; i < kh; ++i) {
            const int64_t ih = oh * sh - ph + i * dh;
            if (ih < 0 || ih >= H) continue;
            for (int64_t j = 0; j < kw; ++j) {
              const int64_t iw = ow * sw - pw + j * dw;
              if (iw < 0 || iw >= W) continue;
              const uint8_t byte = x[((b * H + ih) * W + iw) * C + c];
              const int32_t v = is_signed ? (int32_t)(int8_t)byte : (int32_t)byte;
              if (v > m) m = v;
            }
          }
          y[((b * OH + oh) * OW + ow) * C + c] = (uint8_t)m;
        }
}

/* Adaptive average pooling over NHWC codes (reference Pool.cpp:132-176 hands it
 * to muDNN; numerics of PyTorch's CPU op, qadaptive_avg_pool2d_nhwc_kernel in
 * aten/src/ATen/native/quantized/cpu/kernels/QuantizedOpKernels.cpp): window
 * rows floor(oh*H/OH) .. ceil((oh+1)*H/OH)-1, int32 sum minus zp * count, times
 * fl(1 / count) in fp32, round half to even, plus zp, clamp. */
ORC_API void orc_qadaptive_avgpool2d(const uint8_t* x, int64_t B, int64_t H, int64_t W, int64_t C,
                                     int64_t OH, int64_t OW, int64_t zp, int is_signed, uint8_t* y) {
  const int32_t lo = is_signed ? -128 : 0, hi = is_signed ? 127 : 255;
  for (int64_t b = 0; b < B; ++b)
    for (int64_t oh = 0; oh < OH; ++oh) {
      const int64_t h0 = (oh * H) / OH, h1 = ((oh + 1) * H + OH - 1) / OH;
      for (int64_t ow = 0; ow < OW; ++ow) {
        const int64_t w0 = (ow * W) / OW, w1 = ((ow + 1) * W + OW - 1) / OW;
        const int32_t count = (int32_t)((h1 - h0) * (w1 - w0));
        const float mult = 1.0f / (float)count;
        for (int64_t c = 0; c < C; ++c) {
          int32_t acc = -(int32_t)zp * count;
          for (int64_t ih = h0; ih < h1; ++ih)
            for (int64_t iw = w0; iw < w1; ++iw) {
              const uint8_t byte = x[((b * H + ih) * W + iw) * C + c];
              acc += is_signed ? (int32_t)(int8_t)byte : (int32_t)byte;
            }
          const float v = (float)acc * mult;
          int32_t q = (int32_t)nearbyintf(v) + (int32_t)zp;
          q = q < lo ? lo : (q > hi ? hi : q);
          y[((b * OH + oh) * OW + ow) * C + c] = (uint8_t)q;
        }
      }
    }
}
