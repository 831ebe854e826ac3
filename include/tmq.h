/*
 * tmq -- quantized-inference kernels for AMD MI355X (gfx950), C ABI.
 *
 * This is the whole device boundary of the library: raw device pointers, sizes,
 * scalars and a HIP stream go in, a status code comes out.  No operator entry point
 * allocates, frees, synchronises the device or touches global mutable state
 * (the library caches per-device constants -- the LDS limit, a kernel attribute
 * -- the first time a device is used, nothing else), so all of them are
 * asynchronous on `stream`, re-entrant, and callable from several host threads
 * on different streams.  Every buffer (inputs, outputs, packed weights,
 * workspaces) is owned by the caller.
 *
 * Each entry point names the interface of the reference (MooreThreads
 * torch_musa, paths relative to its tree) that it replaces.
 *
 * Numerics are those of PyTorch's CPU quantized ops (fbgemm):
 *   quantize      q = clamp(rne(fl(x * fl(1/fl(scale)))) + zp, qmin, qmax)
 *   dequantize    r = fl(fl(scale) * float(q - zp))
 *   linear/conv   exact int32 accumulation, then per output channel n
 *                   raw  = acc - x_zp * sum_k W[n][k]
 *                   v    = float(raw) (+ fl(bias[n] / atw[n]))
 *                   q    = clamp(rne(fl(v * mult[n])) + out_zp, lo, qmax)
 *                 atw[n] = fl(fl(x_scale) * fl(w_scale[n])), mult[n] = fl(atw[n] / fl(out_scale)),
 *                 lo = relu ? max(out_zp, qmin) : qmin.
 * rne = round half to even, fl = round to fp32.
 */
#ifndef TMQ_H_
#define TMQ_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TMQ_VERSION 100

/* A hipStream_t, passed as an opaque pointer so that this header needs no HIP
 * include. NULL is the default stream. */
typedef void* tmq_stream_t;

enum tmq_status {
  TMQ_OK = 0,
  TMQ_ERR_INVALID_ARGUMENT = 1, /* null pointer, negative size, bad enum value */
  TMQ_ERR_UNSUPPORTED = 2,      /* well-formed request outside what is built */
  TMQ_ERR_WORKSPACE = 3,        /* workspace missing or too small */
  TMQ_ERR_LAUNCH = 4,           /* the HIP runtime refused the launch */
  TMQ_ERR_ALIGNMENT = 5         /* pointer or leading dimension not aligned */
};

/* Static, human readable text for a status code. */
const char* tmq_status_string(int status);
int tmq_version(void);

/* ---------------------------------------------------------------------------
 * Affine quantizer, per tensor.
 * Replaces torch_musa/csrc/aten/quantized/musa/AffineQuantizer.mu:99-143
 * (quantize_tensor_per_tensor_affine_musa) and :145-179
 * (dequantize_tensor_per_tensor_affine_musa), the functions registered on
 * quantize_tensor_per_tensor_affine_stub / dequantize_..._stub (:340-357).
 * `x`/`r` are dense fp32, `q` is one byte per element in the same order
 * (uint8 when q_signed == 0, two's-complement int8 otherwise). n >= 0.
 * ------------------------------------------------------------------------- */
int tmq_quantize_per_tensor(const float* x, void* q, int64_t n, double scale,
                            int64_t zero_point, int q_signed, tmq_stream_t stream);
int tmq_dequantize_per_tensor(const void* q, float* r, int64_t n, double scale,
                              int64_t zero_point, int q_signed, tmq_stream_t stream);

/* ---------------------------------------------------------------------------
 * Range calibration for quantize_per_tensor_dynamic.
 * Replaces the two full reductions + host round trips behind
 * torch_musa/csrc/aten/ops/musa_functions.yaml:3515-3519
 * (aten::quantize_per_tensor_dynamic -> x.min().item(), x.max().item()).
 *
 * tmq_minmax writes {min, max} of x[0..n) to minmax[0..1] (device memory).
 * `workspace` must hold tmq_minmax_workspace_bytes(n) bytes of device memory.
 * n == 0 yields {+inf, -inf}.
 * ------------------------------------------------------------------------- */
size_t tmq_minmax_workspace_bytes(int64_t n);
int tmq_minmax(const float* x, int64_t n, float* minmax, void* workspace,
               size_t workspace_bytes, tmq_stream_t stream);

/* Quantization parameters as the device-side chain keeps them. */
typedef struct tmq_qparams {
  double scale;       /* as ChooseQuantizationParams returns it */
  int32_t zero_point;
  int32_t reserved;
} tmq_qparams;

/* Device-side ChooseQuantizationParams (ATen/native/quantized/cpu/QuantUtils.h:
 * 71-187 with preserve_sparsity = force_scale_power_of_two = false): reads
 * minmax[0..1] on the device, writes *qparams on the device, so that
 * tmq_quantize_per_tensor_dev can follow on the same stream without a host
 * round trip. */
int tmq_choose_qparams_dev(const float* minmax, int q_signed, int reduce_range,
                           tmq_qparams* qparams, tmq_stream_t stream);
/* Same as tmq_quantize_per_tensor with scale / zero point read from device
 * memory at kernel run time. */
int tmq_quantize_per_tensor_dev(const float* x, void* q, int64_t n,
                                const tmq_qparams* qparams, int q_signed,
                                tmq_stream_t stream);
/* The whole dynamic quantization on the device: min/max over x, the parameters
 * into *qparams (device memory), the codes into q.  Small inputs (at most
 * 32768 elements) take one launch, inputs of up to 2**25 elements two (the
 * quantizer's workgroups finish the range reduction themselves), larger or
 * unaligned ones three; `workspace` as for tmq_minmax (unused, and may be NULL,
 * for the small case).
 * rounding = TMQ_ROUND_PRODUCT: q = clamp(rne(fl(x * inv)) + zp), the same
 * results as tmq_minmax + tmq_choose_qparams_dev + tmq_quantize_per_tensor_dev
 * (aten::quantize_per_tensor_dynamic).
 * rounding = TMQ_ROUND_FUSED: q = clamp(rne(fl(x * inv + zp))), product and
 * zero point rounded once: the activation quantization inside PyTorch's CPU
 * quantized::linear_dynamic (fbgemm PackAWithQuantRowOffset), which differs
 * from the former for about one value in 10^5. */
#define TMQ_ROUND_PRODUCT 0
#define TMQ_ROUND_FUSED 1
int tmq_quantize_per_tensor_dynamic_dev(const float* x, void* q, int64_t n, int q_signed,
                                        int reduce_range, int rounding, tmq_qparams* qparams,
                                        void* workspace, size_t workspace_bytes, tmq_stream_t stream);
/* Host-side ChooseQuantizationParams, same arithmetic (pure CPU, no GPU call). */
int tmq_choose_qparams_host(float min, float max, int q_signed, int reduce_range,
                            double* scale, int32_t* zero_point);

/* ---------------------------------------------------------------------------
 * Affine quantizer, per channel.
 * Replaces AffineQuantizer.mu:181-224 (quantize_tensor_per_channel_affine_musa)
 * and :226-257 (dequantize_tensor_per_channel_affine_musa).
 * The tensor is viewed as [outer, channels, inner] with the quantization axis
 * in the middle; scales (double) and zero_points (int64) are device arrays of
 * `channels` entries, the types the dispatch stub hands over.
 * ------------------------------------------------------------------------- */
int tmq_quantize_per_channel(const float* x, void* q, int64_t outer,
                             int64_t channels, int64_t inner, const double* scales,
                             const int64_t* zero_points, int q_signed,
                             tmq_stream_t stream);
int tmq_dequantize_per_channel(const void* q, float* r, int64_t outer,
                               int64_t channels, int64_t inner, const double* scales,
                               const int64_t* zero_points, int q_signed,
                               tmq_stream_t stream);

/* Per channel with float scales and float zero points (qscheme
 * per_channel_affine_float_qparams): q = clamp(lrintf(x * (1/scale_c) + zp_c)),
 * r = (float(q) - zp_c) * scale_c, all in fp32; a zero scale quantizes with
 * inverse 1.  Replaces AffineQuantizer.mu:259-301
 * (quantize_tensor_per_channel_float_qparams_musa) and :303-336
 * (dequantize_tensor_per_channel_float_qparams_musa).  scales and zero_points
 * are device arrays of `channels` floats. */
int tmq_quantize_per_channel_float_qparams(const float* x, void* q, int64_t outer,
                                           int64_t channels, int64_t inner,
                                           const float* scales, const float* zero_points,
                                           int q_signed, tmq_stream_t stream);
int tmq_dequantize_per_channel_float_qparams(const void* q, float* r, int64_t outer,
                                             int64_t channels, int64_t inner,
                                             const float* scales, const float* zero_points,
                                             int q_signed, tmq_stream_t stream);

/* ---------------------------------------------------------------------------
 * quantized::linear weights.
 * Replaces PackedLinearWeightMudnn::prepack
 * (torch_musa/csrc/aten/quantized/mudnn/LinearPrepack.cpp:11-37), which keeps
 * the [N,K] int8 weight as is for muDNN.  Here the weight is re-tiled once into
 * the order the int8 MFMA kernels stream it in:
 *   packed[nb][kc][r][b] = W[16*nb + r][16*kc + b],  r,b in [0,16)
 * nb < ceil(N/16), kc < tmq_linear_packed_kchunks(K) (K rounded up to 128),
 * zero filled outside W.  colsum[n] = sum_k W[n][k] (int32) is produced in the
 * same pass; the epilogue needs it for the activation zero point.
 * ------------------------------------------------------------------------- */
int64_t tmq_linear_packed_kchunks(int64_t K);
int64_t tmq_linear_packed_bytes(int64_t N, int64_t K);
int tmq_linear_prepack(const int8_t* w, int64_t N, int64_t K, int64_t ldw,
                       void* packed, int32_t* colsum, tmq_stream_t stream);
/* Inverse re-tiling (packed -> [N,K] row major), for round-trip checks. */
int tmq_linear_unpack(const void* packed, int64_t N, int64_t K, int8_t* w,
                      int64_t ldw, tmq_stream_t stream);

/* ---------------------------------------------------------------------------
 * quantized::linear / quantized::linear_relu.
 * Replaces PackedLinearWeightMudnn::apply_impl_helper
 * (torch_musa/csrc/aten/quantized/mudnn/Linear.cpp:16-65: muDNN
 * MatMul::RunWithBiasAdd with SetTranspose(false,true), then a separate relu_).
 * Y[M,N] = requant(X[M,K] . W[N,K]^T + bias), everything fused in one kernel.
 * ------------------------------------------------------------------------- */
typedef struct tmq_linear_desc {
  int64_t M, N, K;
  const void* x;         /* [M,K] bytes, row pitch ldx (elements) */
  int64_t ldx;
  int32_t x_signed;      /* 0: quint8 activations, 1: qint8 */
  int32_t x_zero_point;
  float x_scale;
  const void* w_packed;  /* from tmq_linear_prepack */
  const int32_t* w_colsum; /* [N] */
  const float* w_scales;   /* [N] (per channel) or [1] (per tensor) */
  int32_t w_per_channel;   /* 0: w_scales[0] for every n */
  int32_t relu;            /* 1: lower clamp is the output zero point */
  const float* bias;       /* [N] fp32 or NULL */
  float out_scale;
  int32_t out_zero_point;
  int32_t out_signed;      /* 0: quint8 output, 1: qint8 */
  /* 0: the library chooses the kernel (what every caller wants).  k + 1 pins
   * kernel configuration k of the dispatch table in kernels/linear.hip, so
   * that tests can put every kernel in front of the oracle at any shape; a
   * configuration that cannot run the problem gives TMQ_ERR_UNSUPPORTED. */
  int32_t kernel;
  void* y;                 /* [M,N] bytes, row pitch ldy */
  int64_t ldy;
  /* Optional scratch device memory, owned by the caller like every other
   * buffer (16-byte aligned; contents undefined before and after the call).
   * With at least tmq_linear_workspace_bytes(M, N, K) bytes, products whose
   * tile grid is much smaller than the chip (some tens to a few hundred rows
   * against a long K) are computed
   * split along K: partial sums into the workspace, then one pass that adds
   * and requantises them.  NULL / too small: single-launch kernels, same
   * results. */
  void* workspace;
  int64_t workspace_bytes;
} tmq_linear_desc;

int tmq_linear(const tmq_linear_desc* desc, tmq_stream_t stream);

/* Bytes of workspace that tmq_linear / tmq_linear_f32 / tmq_linear_acc32 can
 * use for this problem size; 0 when the single-launch kernels are chosen
 * anyway.  No counterpart in the reference: muDNN allocates its own scratch
 * through the InternalMemAlloc callback (torch_musa/csrc/aten/utils/Utils.cpp:79-153). */
int64_t tmq_linear_workspace_bytes(int64_t M, int64_t N, int64_t K);
/* The split behind that figure: *splits runs of *stages k-stages (64 bytes of K
 * each), the last run taking everything that is left; *splits == 1: no split.
 * Pure host arithmetic, no GPU call. */
int tmq_linear_split_plan(int64_t M, int64_t N, int64_t K, int32_t* splits, int32_t* stages);

/* Which kernel tmq_linear / tmq_linear_f32 / tmq_linear_acc32 launch for a shape,
 * and on what grid.  Pure host arithmetic, no GPU call: the choice depends on
 * the sizes, the row pitch, the output kind and whether a workspace is attached,
 * never on the data.  No counterpart in the reference (muDNN chooses its kernels
 * out of sight, torch_musa/csrc/aten/quantized/mudnn/Linear.cpp:48-58); it is
 * here so that the choice and every kernel's preconditions can be swept on the
 * host over thousands of shapes. */
typedef struct tmq_linear_choice {
  int32_t kernel;        /* value that pins this kernel in tmq_linear_desc::kernel (configuration + 1);
                            0: no kernel takes the shape (TMQ_ERR_UNSUPPORTED from the call) */
  int32_t tile_rows;     /* activation rows per workgroup tile (0: plain kernel) */
  int32_t tile_channels; /* output channels per workgroup tile */
  int32_t waves;         /* wavefronts per workgroup */
  int32_t splits;        /* runs of k-stages (1: no split along K) */
  int32_t split_stages;  /* k-stages per run */
  int64_t tiles;         /* tiles of the product (x splits for split K) */
  int64_t blocks;        /* workgroups launched (the persistent kernel: fewer than tiles) */
  int64_t k_stages;      /* 64-byte stages of K */
} tmq_linear_choice;
enum tmq_linear_output_kind { TMQ_LINEAR_OUT_BYTES = 0, TMQ_LINEAR_OUT_F32 = 1, TMQ_LINEAR_OUT_ACC32 = 2 };
/* flags: bits 0-1 a tmq_linear_output_kind; bit 2: a workspace of
 * tmq_linear_workspace_bytes(M, N, K) is attached; bit 3: K, the row pitch or
 * the activation pointer is not a multiple of 16 (the plain kernel's case).
 * forced_kernel: tmq_linear_desc::kernel (0 = automatic).  compute_units: of
 * the device the product would run on (the persistent kernel's grid follows it). */
int tmq_linear_kernel_choice(int64_t M, int64_t N, int64_t K, int64_t ldx, int32_t flags, int32_t forced_kernel,
                             int32_t compute_units, tmq_linear_choice* out);

/* tmq_linear for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  No
 * counterpart in the reference.  Same arguments and the same bytes as
 * tmq_linear called with a workspace of tmq_linear_workspace_bytes(M, N, K);
 * desc->workspace / workspace_bytes are ignored: the split-K partial sums go to
 * a fixed array of TMQ_LINEAR_STATIC_WORKSPACE_BYTES in the library's own device
 * memory (one per GPU the library has run on, held until the process ends).
 * The call allocates and frees nothing.  A problem whose split needs more than
 * the array holds returns TMQ_ERR_WORKSPACE (the present split plan never asks
 * for more than 256 tiles of 128 x 128 int32 sums = the array's size).  Calls
 * on one GPU share that GPU's array: calls that may run at the same time
 * (different streams, different host threads) race on it and must be ordered
 * by the caller; calls queued on one stream are safe.  The partial sums are
 * written before they are read, so nothing has to be cleared between calls.
 * The first call on a device looks the array's address up (hipGetSymbolAddress):
 * make one call per device before capturing a graph.  The current device must
 * be the device that owns `stream` (each GPU holds its own array at its own
 * address): a stream of another GPU returns TMQ_ERR_INVALID_ARGUMENT. */
#define TMQ_LINEAR_STATIC_WORKSPACE_BYTES (16 * 1024 * 1024)
int tmq_linear_static_workspace(const tmq_linear_desc* desc, tmq_stream_t stream);

/* Raw accumulators acc[m][n] = sum_k X[m][k] * W[n][k] as int32 (row pitch
 * ldacc), from the same MFMA main loop, for bit-exactness checks.  Uses
 * M, N, K, x, ldx, x_signed, w_packed, w_colsum of `desc`. */
int tmq_linear_acc32(const tmq_linear_desc* desc, int32_t* acc, int64_t ldacc,
                     tmq_stream_t stream);

/* Float output of the same product, the second half of a dynamically quantized
 * linear (PackedLinearWeight::apply_dynamic, which the reference declares and
 * leaves unimplemented, torch_musa/csrc/aten/quantized/mudnn/Linear.h:35-46;
 * arithmetic of PyTorch's CPU op, fbgemm ReQuantizeForFloat):
 *   y[m][n] = fma(float(acc[m][n] - x_zp * colsum[n]), fl(x_scale * w_scale[n]), bias[n])
 * clamped below at 0 when desc->relu.  Uses M, N, K, x, ldx, x_signed, w_*,
 * relu, bias of `desc`; y is fp32 [M, ldy].  x_qparams_dev != NULL: the
 * activation scale and zero point are read from device memory when the kernel
 * runs (as written by tmq_choose_qparams_dev), desc->x_scale / x_zero_point are
 * ignored, and min/max -> qparams -> quantize -> linear runs without the host
 * seeing the parameters. */
int tmq_linear_f32(const tmq_linear_desc* desc, const tmq_qparams* x_qparams_dev, float* y,
                   int64_t ldy, tmq_stream_t stream);

/* The whole dynamically quantized linear for a handful of rows in one launch:
 * fp32 x [M, ldx] -> fp32 y [M, ldy] with M <= 16, K a multiple of 16, x 16-byte
 * aligned, ldx a multiple of 4, and either M * K <= 16384 (every block of the
 * weight-streaming kernel derives the activation range, parameters and codes
 * itself while its weights are on their way) or M * K <= 32768 with
 * 64 <= K <= 8192 (one block per CU does so once, keeps the codes in LDS and
 * streams the channel groups it owns; the library picks between the two where
 * both apply).  TMQ_ERR_UNSUPPORTED otherwise: use
 * tmq_quantize_per_tensor_dynamic_dev + tmq_linear_f32, which give the same
 * results; tmq_linear_dynamic_small_takes says beforehand (1 / 0, alignment
 * aside).  Uses M, N, K, w_*, relu, bias of `desc`; desc->kernel = 9 / 29 pins
 * the first / second kernel for tests.  Same reference note as tmq_linear_f32. */
int tmq_linear_dynamic_small_takes(int64_t M, int64_t N, int64_t K);
int tmq_linear_dynamic_small(const tmq_linear_desc* desc, const float* x, int64_t ldx, int reduce_range,
                             float* y, int64_t ldy, tmq_stream_t stream);

/* ---------------------------------------------------------------------------
 * quantized::conv2d weights.
 * Replaces PackedConvWeightMudnn<2>::prepack
 * (torch_musa/csrc/aten/quantized/mudnn/ConvPrepack.cpp:10-92), which permutes
 * OIHW to OHWI.  Input here is already OHWI ([OC, KH, KW, IC/groups] int8,
 * dense); per group g it is re-tiled like a linear weight with
 * N = OC/groups rows and K = KH*KW*ICg columns where every (kh,kw) tap is
 * padded to a multiple of 16 input channels:
 *   k = (kh*KW + kw) * roundup(ICg,16) + ic.
 * colsum[oc] = sum of all weights of output channel oc.
 * ------------------------------------------------------------------------- */
typedef struct tmq_conv2d_geom {
  int64_t B, H, W, IC; /* activations, NHWC */
  int64_t OC, KH, KW;  /* weights, OHWI with IC/groups innermost */
  int64_t stride_h, stride_w, pad_h, pad_w, dil_h, dil_w, groups;
} tmq_conv2d_geom;

int64_t tmq_conv2d_packed_bytes(const tmq_conv2d_geom* g);
int tmq_conv2d_prepack(const int8_t* w_ohwi, const tmq_conv2d_geom* g, void* packed,
                       int32_t* colsum, tmq_stream_t stream);
/* OH / OW as reference mudnn/Conv.cpp:20-36 computes them. */
int tmq_conv2d_out_hw(const tmq_conv2d_geom* g, int64_t* OH, int64_t* OW);

/* ---------------------------------------------------------------------------
 * quantized::conv2d / conv2d_relu, NHWC implicit GEMM.
 * Replaces PackedConvWeightMudnn<2>::apply_impl_helper
 * (torch_musa/csrc/aten/quantized/mudnn/Conv.cpp:38-133: muDNN
 * Convolution::RunFusion on NHWC tensors).
 * x is [B,H,W,IC] bytes dense, y is [B,OH,OW,OC] bytes dense.
 * ------------------------------------------------------------------------- */
typedef struct tmq_conv2d_desc {
  tmq_conv2d_geom geom;
  const void* x;
  int32_t x_signed;
  int32_t x_zero_point;
  float x_scale;
  int32_t w_per_channel;
  const void* w_packed;
  const int32_t* w_colsum; /* [OC] */
  const float* w_scales;   /* [OC] or [1] */
  const float* bias;       /* [OC] or NULL */
  float out_scale;
  int32_t out_zero_point;
  int32_t out_signed;
  int32_t relu;
  void* y;
  /* 0: the library chooses.  Otherwise, for tests of every kernel family at any
   * shape: 1 halo tiles, 2 implicit GEMM, 3 direct, 4 kernel rows as byte runs
   * (few input channels), 5 a pointwise layer as tmq_linear, 6 patch rows in the
   * workspace, then tmq_linear, 7 a depthwise layer four channels per lane on the
   * vector ALU, 8 the input copied into the workspace with its channels padded
   * to a multiple of 16, then whatever the library chooses for that, 9 a pointwise
   * layer over at most 256 input channels with its pixels straight from memory
   * (TMQ_ERR_UNSUPPORTED when the family cannot run the problem).  tile_rows / tile_cols > 0 pin the halo
   * kernel's patch height / bound its patch width. */
  int32_t kernel;
  int32_t tile_rows, tile_cols;
  int32_t reserved;
  /* Optional scratch device memory, owned by the caller like every other buffer
   * (16-byte aligned; contents undefined before and after the call).  With at
   * least tmq_conv2d_workspace_bytes(&geom) bytes, layers with few output pixels
   * against a long K (3 x 3 over hundreds of channels on a 14 x 14 or 7 x 7
   * image) and pointwise layers with a stride over 512 input channels and more
   * write their patch rows there and run as one quantized::linear over
   * them, and layers of one group whose channel count is no multiple of 16
   * under kernel rows of more than 256 bytes (3 x 3 over 40 channels) run the
   * matrix-core kernels on a copy of the input with padded channels instead of
   * the slow direct kernel.  NULL / too small: the single-launch kernels, same
   * results. */
  void* workspace;
  int64_t workspace_bytes;
} tmq_conv2d_desc;

int tmq_conv2d(const tmq_conv2d_desc* desc, tmq_stream_t stream);
/* Bytes of workspace that tmq_conv2d can use for this geometry (B, H, W included);
 * 0 when the single-launch kernels are chosen anyway.  No counterpart in the
 * reference: muDNN allocates its own scratch through the InternalMemAlloc
 * callback (torch_musa/csrc/aten/utils/Utils.cpp:79-153). */
int64_t tmq_conv2d_workspace_bytes(const tmq_conv2d_geom* g);
/* Zero-point-corrected accumulators, [B,OH,OW,OC] int32:
 * acc = sum over in-image taps of (x - x_zp) * w. */
int tmq_conv2d_acc32(const tmq_conv2d_desc* desc, int32_t* acc, tmq_stream_t stream);

/* ---------------------------------------------------------------------------
 * quantized::conv2d_add / conv2d_add_relu / conv2d_silu / conv2d_add_silu.
 * Replaces PackedConvWeightMudnn<2>::apply_add, apply_add_relu, apply_add_silu
 * (torch_musa/csrc/aten/quantized/mudnn/ConvAdd.cpp:11-39) and the SILU mode of
 * apply_impl_helper (mudnn/Conv.cpp:86-130: residual tensor `add` and
 * FusedActivationDesc handed to muDNN RunFusion).
 *   t = (float(acc) + bias/(x_scale*w_scale)) * (x_scale*w_scale/out_scale)
 *   t += float(accum_q - accum_zero_point) * (accum_scale/out_scale)   if accum
 *   t  = silu(t*out_scale)/out_scale                                    if activation == 2
 *   y  = clamp(rne(t) + out_zero_point), lower clamp out_zero_point if relu
 * accum is [B,OH,OW,OC] bytes dense (NHWC, the output's shape) or NULL.
 * activation: 0 identity, 1 relu, 2 silu; desc->relu also selects relu.
 * ------------------------------------------------------------------------- */
typedef struct tmq_conv2d_post {
  const void* accum;
  int32_t accum_signed;
  int32_t accum_zero_point;
  float accum_scale;
  int32_t activation;
} tmq_conv2d_post;

int tmq_conv2d_fused(const tmq_conv2d_desc* desc, const tmq_conv2d_post* post,
                     tmq_stream_t stream);

/* ---------------------------------------------------------------------------
 * Elementwise kernels on per-tensor quantized tensors (n codes, dense).
 * tmq_qadd replaces QAdd<kReluFused> / QuantizedAddKernel
 * (torch_musa/csrc/aten/quantized/musa/BinaryOps.mu:24-99,154-207) with the
 * arithmetic of PyTorch's CPU quantized::add / add_relu:
 *   a = fma(float(qa), a_scale, -a_zp*a_scale), b likewise, c = a + b,
 *   relu: c = max(c, 0), q = clamp(rne(c * (1/out_scale)) + out_zp).
 * tmq_qrelu replaces ActQuantized<ActMode::RELU>
 * (torch_musa/csrc/aten/quantized/musa/Activation.mu:165-186,215-220):
 *   y = max(x, zero_point), scale and zero point unchanged.
 * ------------------------------------------------------------------------- */
int tmq_qadd(const void* a, const void* b, void* out, int64_t n, float a_scale,
             int32_t a_zero_point, float b_scale, int32_t b_zero_point, float out_scale,
             int32_t out_zero_point, int q_signed, int relu, tmq_stream_t stream);
int tmq_qrelu(const void* x, void* y, int64_t n, int32_t zero_point, int q_signed,
              tmq_stream_t stream);

/* Building block of quantized::cat (replaces QuantizedCat / QuantizedCatOut,
 * torch_musa/csrc/aten/quantized/TensorShape.cpp:335-426, muDNN Concat): one
 * input viewed as [outer, in_row] codes is written into the output viewed as
 * [outer, out_row] at column out_col_offset, requantised from the input's to
 * the output's parameters (a plain copy when they agree):
 *   r = in_scale * float(q - in_zp);  q' = clamp(rne(r * (1/out_scale)) + out_zp)
 * i.e. the per-tensor dequantizer followed by the per-tensor quantizer.  For a
 * concatenation along dim d of contiguous tensors: outer = prod(sizes[:d]),
 * in_row = size_i[d] * prod(sizes[d+1:]), one call per input. */
int tmq_qcat_rows(const void* x, void* y, int64_t outer, int64_t in_row, int64_t out_row,
                  int64_t out_col_offset, float in_scale, int32_t in_zero_point, float out_scale,
                  int32_t out_zero_point, int q_signed, tmq_stream_t stream);

/* Max pooling over NHWC codes (replaces MaxPool2dQuantized /
 * QuantizedMaxPool2dImpl, torch_musa/csrc/aten/quantized/Pool.cpp:80-130,178-247,
 * muDNN Pooling): y[b,oh,ow,c] = max over the window's in-image positions of
 * x[b,ih,iw,c]; scale and zero point carry over.  OH / OW are the caller's
 * (floor or ceil mode); every window must overlap the image. */
int tmq_qmaxpool2d(const void* x, void* y, int64_t B, int64_t H, int64_t W, int64_t C, int32_t kh,
                   int32_t kw, int32_t stride_h, int32_t stride_w, int32_t pad_h, int32_t pad_w,
                   int32_t dil_h, int32_t dil_w, int64_t OH, int64_t OW, int q_signed,
                   tmq_stream_t stream);

/* Adaptive average pooling over NHWC codes (replaces AdaptiveAvgPool2dQuantized /
 * QuantizedAvgPool2dImpl, torch_musa/csrc/aten/quantized/Pool.cpp:93-127,132-176,
 * muDNN Pooling ADAPTIVE_AVGPOOL).  Output pixel (oh, ow) covers input rows
 * floor(oh*H/OH) .. ceil((oh+1)*H/OH)-1 and the like columns; scale and zero
 * point carry over:
 *   acc = sum(q) - zero_point * count;  q' = clamp(rne(float(acc) * (1.0f / count)) + zero_point) */
int tmq_qadaptive_avgpool2d(const void* x, void* y, int64_t B, int64_t H, int64_t W, int64_t C,
                            int64_t OH, int64_t OW, int32_t zero_point, int q_signed,
                            tmq_stream_t stream);

/* gelu / sigmoid of a per-tensor quantized tensor (replaces ActQuantizedGeLU and
 * ActQuantized<SIGMOID>, torch_musa/csrc/aten/quantized/musa/Activation.mu:95-164,
 * 218-219): y = f((q - in_zp) * in_scale), q' = clamp(rne(y / out_scale) + out_zp),
 * evaluated once per input code in double precision and applied as a table.
 * kind 0: gelu (erf), 1: gelu (tanh approximation), 2: sigmoid.  PyTorch's CPU ops
 * give gelu the input's parameters and sigmoid scale 1/256 with zero point 0
 * (quint8) or -128 (qint8); the caller passes them. */
int tmq_qunary(const void* x, void* y, int64_t n, int kind, float in_scale, int32_t in_zero_point,
               float out_scale, int32_t out_zero_point, int q_signed, tmq_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* TMQ_H_ */
