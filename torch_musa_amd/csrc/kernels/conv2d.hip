// quantized::conv2d for gfx950: NHWC implicit GEMM on the int8 MFMA core.
//
// GEMM view per group: rows m = (b, oh, ow) output pixels, columns n = output
// channels of the group, k = (kh, kw, ic) with every tap padded to a multiple
// of 16 input channels, so one 16-byte k-chunk is one run of 16 channels of one
// input pixel -- a single aligned load from the NHWC activation tensor.
// Taps outside the image are filled with the activation zero point (real value
// 0), which the accumulator start value then cancels exactly.
#include <atomic>
#include <type_traits>

#include "conv_runs.h"
#include "conv_depthwise.h"
#include "conv_tile.h"
#include "gemm_i8_core.h"

static_assert(sizeof(tmq_conv2d_geom) == 112, "tmq_conv2d_geom layout changed");
static_assert(sizeof(tmq_conv2d_desc) == 224, "tmq_conv2d_desc layout changed");
static_assert(sizeof(tmq_conv2d_post) == 24, "tmq_conv2d_post layout changed");

namespace tmq {
namespace {

constexpr int64_t kKPad = 128;
constexpr int64_t kTwoGroupTiles = 512;          // 64 x 64 tiles up to which the implicit GEMM splits K over two wave groups
constexpr int64_t kFourGroupTiles = 256;         // ... over four (K of 64 stages and more)
constexpr int64_t kPointwiseAsLinearRows = 8192;
constexpr int64_t kPatchRowsMax = 512;           // output pixels up to which a layer may run on its patch rows (workspace)
constexpr int64_t kPatchRowsMinK = 2048;         // and the K from which on  // pixels up to which a pointwise layer runs as a linear layer
inline int64_t packed_kchunks(int64_t K) { return (K + kKPad - 1) / kKPad * (kKPad / 16); }

struct ConvShape {
  int64_t B, H, W, IC, OC, KH, KW, OH, OW;
  int64_t sh, sw, ph, pw, dh, dw, groups;
  int64_t ICg, OCg, ICgp, Kp, KC, group_bytes;
  int64_t ICgo, OCgo;  // channels per group as the caller states them (see make_shape)
  // the second weight layout, behind the first, for the kernel of conv_runs.h: k-steps
  // (0: the shape is not that kernel's), run bytes, padded run bytes, offset and size in bytes
  int64_t runs_KS, runs_RL, runs_RP, runs_off, runs_bytes;
  // depthwise layers over a multiple of 4 channels: a [channel][kernel row][taps padded to a multiple
  // of 4] copy of the weight for the kernel of conv_depthwise.h in the same place (0: not such a layer)
  int64_t taps_bytes;
};

int make_shape(const tmq_conv2d_geom* g, ConvShape* s) {
  if (g == nullptr) return TMQ_ERR_INVALID_ARGUMENT;
  if (g->B < 0 || g->H <= 0 || g->W <= 0 || g->IC <= 0 || g->OC <= 0 || g->KH <= 0 || g->KW <= 0 ||
      g->stride_h <= 0 || g->stride_w <= 0 || g->pad_h < 0 || g->pad_w < 0 || g->dil_h <= 0 ||
      g->dil_w <= 0 || g->groups <= 0)
    return TMQ_ERR_INVALID_ARGUMENT;
  if (g->IC % g->groups != 0 || g->OC % g->groups != 0) return TMQ_ERR_INVALID_ARGUMENT;
  s->B = g->B; s->H = g->H; s->W = g->W; s->IC = g->IC; s->OC = g->OC; s->KH = g->KH; s->KW = g->KW;
  s->sh = g->stride_h; s->sw = g->stride_w; s->ph = g->pad_h; s->pw = g->pad_w;
  s->dh = g->dil_h; s->dw = g->dil_w; s->groups = g->groups;
  s->OH = (g->H + 2 * g->pad_h - g->dil_h * (g->KH - 1) - 1) / g->stride_h + 1;
  s->OW = (g->W + 2 * g->pad_w - g->dil_w * (g->KW - 1) - 1) / g->stride_w + 1;
  if (s->OH <= 0 || s->OW <= 0) return TMQ_ERR_INVALID_ARGUMENT;
  // Groups whose input channels are no multiple of 16 (depthwise and other narrow groups)
  // are merged: `merge` neighbouring groups become one group with a block-diagonal weight --
  // zeros where an output channel meets another group's input channels -- so that a 16-byte
  // k-chunk is again 16 channels of one pixel and the MFMA kernels take the problem.  The
  // matrix pipe multiplies the zeros at no cost that matters: these layers move bytes.
  // The merged group has as many channels as a tile of the kernels is wide (64) where the
  // group count allows.  groups / ICg / OCg below are the merged ones; the packed weight
  // is laid out for them.
  s->ICgo = g->IC / g->groups;
  s->OCgo = g->OC / g->groups;
  int64_t merge = 1;
  if (g->groups > 1 && s->ICgo % 16 != 0) {
    const int64_t low = s->ICgo & -s->ICgo;             // largest power of two in ICgo
    const int64_t v0 = 16 / (low < 16 ? low : 16);      // fewest groups that make a multiple of 16
    for (int64_t v = v0; v <= g->groups; v += v0) {
      if (v > v0 && (v * s->OCgo > 64 || v * s->ICgo > 64)) break;
      if (g->groups % v == 0) merge = v;
    }
    if ((merge * s->ICgo) % 16 != 0) merge = 1;         // (no such divisor of the group count)
  }
  s->groups = g->groups / merge;
  s->ICg = merge * s->ICgo;
  s->OCg = merge * s->OCgo;
  s->ICgp = round_up(s->ICg, 16);
  s->Kp = g->KH * g->KW * s->ICgp;
  s->KC = packed_kchunks(s->Kp);
  s->group_bytes = ceil_div(s->OCg, 16) * s->KC * 256;
  s->runs_KS = s->runs_RL = s->runs_RP = s->runs_bytes = 0;
  s->runs_off = s->groups * s->group_bytes;
  if (g->groups == 1 && g->dil_h == 1 && g->dil_w == 1) {
    const int64_t RL = g->KW * g->IC, RP = round_up(RL, 16);
    if (g->KH * RP <= 64 * kCrMaxKS) {
      s->runs_RL = RL;
      s->runs_RP = RP;
      s->runs_KS = ceil_div(g->KH * RP, 64);
      const int64_t tiles = conv_runs_tiles(g->OC);  // 16-channel tiles per block
      s->runs_bytes = ceil_div(g->OC, 16 * tiles) * tiles * s->runs_KS * kWave * 16;
    }
  }
  s->taps_bytes = 0;
  if (g->groups > 1 && g->groups == g->IC && g->IC == g->OC && g->IC % 4 == 0)
    s->taps_bytes = round_up(g->IC * g->KH * round_up(g->KW, 4), 16);
  // 32-bit index arithmetic inside the kernels
  if (g->H > (1 << 24) || g->W > (1 << 24) || g->IC > (1 << 24) || s->Kp > (1 << 30) ||
      g->B * s->OH * s->OW > 0x7fffffff || g->H * g->W * g->IC > 0x3fffffff)
    return TMQ_ERR_UNSUPPORTED;
  return TMQ_OK;
}

// One thread per 16-byte packed chunk (group, nb, kc, r).
__global__ __launch_bounds__(256) void conv_prepack_kernel(const int8_t* __restrict__ w,
                                                           ConvShape s, int64_t total,
                                                           uint8_t* __restrict__ packed) {
  const int64_t id = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (id >= total) return;
  const int64_t per_group = s.group_bytes / 16;
  const int64_t g = id / per_group, lid = id % per_group;
  const int r = static_cast<int>(lid & 15);
  const int64_t kc = (lid >> 4) % s.KC, nb = (lid >> 4) / s.KC;
  const int64_t n = nb * 16 + r;
  const int64_t k0 = kc * 16;
  const int64_t tap = k0 / s.ICgp, ic0 = k0 % s.ICgp;
  uint32_t words[4] = {0, 0, 0, 0};
  if (n < s.OCg && tap < s.KH * s.KW) {
    // the output channel's own group inside a merged one: its input channels lo .. lo + ICgo - 1
    const int64_t lo = n / s.OCgo * s.ICgo;
    const int8_t* src = w + ((g * s.OCg + n) * s.KH * s.KW + tap) * s.ICgo;
    for (int b = 0; b < 16; ++b)
      if (ic0 + b >= lo && ic0 + b < lo + s.ICgo)
        words[b >> 2] |= static_cast<uint32_t>(static_cast<uint8_t>(src[ic0 + b - lo])) << (8 * (b & 3));
  }
  *reinterpret_cast<v4i*>(packed + id * 16) =
      v4i{static_cast<int>(words[0]), static_cast<int>(words[1]), static_cast<int>(words[2]),
          static_cast<int>(words[3])};
}

// One thread per 16-byte slot of the per-lane layout of conv_runs.h.
__global__ __launch_bounds__(256) void conv_prepack_runs_kernel(const int8_t* __restrict__ w, ConvShape s,
                                                                int64_t total, uint8_t* __restrict__ dst) {
  const int64_t id = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (id >= total) return;
  *reinterpret_cast<v4i*>(dst + id * 16) =
      conv_runs_slot(w, id, static_cast<int>(s.OC), static_cast<int>(s.KH), static_cast<int>(s.runs_RL),
                     static_cast<int>(s.runs_RP), static_cast<int>(s.runs_KS));
}

// One thread per byte of the [channel][kernel row][padded taps] layout of conv_depthwise.h (the
// caller's weight is [channel][kernel row][tap]).
__global__ __launch_bounds__(256) void conv_prepack_taps_kernel(const int8_t* __restrict__ w, int64_t C, int64_t KH,
                                                                int64_t KW, int64_t total, uint8_t* __restrict__ dst) {
  const int64_t id = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (id >= total) return;
  const int64_t kwp = (KW + 3) / 4 * 4;
  const int64_t kw = id % kwp, kh = id / kwp % KH, c = id / (kwp * KH);
  dst[id] = c < C && kw < KW ? static_cast<uint8_t>(w[(c * KH + kh) * KW + kw]) : uint8_t{0};
}

__global__ __launch_bounds__(256) void conv_colsum_kernel(const int8_t* __restrict__ w, int64_t OC,
                                                          int64_t K, int32_t* __restrict__ colsum) {
  const int lane = threadIdx.x % kWave;
  const int64_t n = static_cast<int64_t>(blockIdx.x) * (256 / kWave) + threadIdx.x / kWave;
  if (n >= OC) return;
  int s = 0;
  for (int64_t i = lane; i < K; i += kWave) s += w[n * K + i];
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) s += __shfl_xor(s, off, kWave);
  if (lane == 0) colsum[n] = s;
}

// Patch rows (im2col) of a convolution over whole 16-channel blocks, one group: row m = output
// pixel (b, oh, ow), k = (kh, kw, ic) as in the packed weight; one thread per 16-byte chunk.
// Taps outside the image are the activation zero point.
__global__ __launch_bounds__(256) void conv_patch_rows_kernel(const uint8_t* __restrict__ x, ConvShape s, int64_t total,
                                                              uint32_t pad_word, uint8_t* __restrict__ rows) {
  const int64_t id = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (id >= total) return;
  const uint32_t kc = static_cast<uint32_t>(s.Kp / 16), icb = static_cast<uint32_t>(s.IC / 16);
  const uint32_t m = static_cast<uint32_t>(id / kc), c = static_cast<uint32_t>(id - static_cast<int64_t>(m) * kc);
  const uint32_t tap = c / icb, blk = c - tap * icb;
  const uint32_t kh = tap / static_cast<uint32_t>(s.KW), kw = tap - kh * static_cast<uint32_t>(s.KW);
  const uint32_t ow = m % static_cast<uint32_t>(s.OW), t = m / static_cast<uint32_t>(s.OW);
  const uint32_t oh = t % static_cast<uint32_t>(s.OH), b = t / static_cast<uint32_t>(s.OH);
  const int ih = static_cast<int>(oh * s.sh) - static_cast<int>(s.ph) + static_cast<int>(kh * s.dh);
  const int iw = static_cast<int>(ow * s.sw) - static_cast<int>(s.pw) + static_cast<int>(kw * s.dw);
  const int pw = static_cast<int>(pad_word);
  v4i v = {pw, pw, pw, pw};
  if (static_cast<unsigned>(ih) < static_cast<unsigned>(s.H) && static_cast<unsigned>(iw) < static_cast<unsigned>(s.W))
    v = ld16(x + ((static_cast<int64_t>(b) * s.H + ih) * s.W + iw) * s.IC + blk * 16);
  *reinterpret_cast<v4i*>(rows + id * 16) = v;
}

// Whether a layer may run on its patch rows, and the bytes they take: one group over whole
// 16-channel blocks, few output pixels, a long K, and no halo tiles for it.
int64_t patch_rows_bytes(const tmq_conv2d_geom& g, const ConvShape& s, bool pinned) {
  if (g.groups != 1 || s.IC % 16 != 0) return 0;
  const int64_t rows = s.B * s.OH * s.OW;
  if (rows == 0 || rows * (s.Kp / 16) > 0x7fffffff) return 0;
  if (!pinned) {
    const bool pointwise = s.KH == 1 && s.KW == 1 && s.ph == 0 && s.pw == 0;
    if (pointwise && s.sh == 1 && s.sw == 1) return 0;  // (already rows)
    if (pointwise) {
      // A pointwise layer with a stride: its patch rows are the pixels it reads, gathered.  From 512 input
      // channels on (batch 32: 512 -> 1024 on 28 x 28 19.5 -> 13.1 us, 1024 -> 2048 on 14 x 14 16.9 -> 12.8 us; batch 8,
      // 1024 -> 2048: 9.9 -> 8.8 us; 256 -> 512 on 56 x 56 level at batch 32 and behind at batch 8, 8.8 against 9.4 us).
      // (eight images, 512 -> 1024 on 28 x 28: 9.0 against 7.9 us on the implicit GEMM)
      if (s.IC < 512 || rows * s.IC * s.OC < (s.IC >= 1024 ? 500000000 : 2000000000)) return 0;
    } else if (rows > kPatchRowsMax || s.Kp < kPatchRowsMinK) {
      return 0;
    }
  }
  return rows * s.Kp;
}

// One group whose channel count is no multiple of 16 and whose kernel rows are too long for the
// byte-run kernel (3 x 3 over 40 channels, 11 x 11 over 3): with scratch memory the input is
// copied once with every pixel's channels padded to whole 16-channel blocks, and the MFMA kernels
// run on the copy -- the packed weight already holds zeros at the padded positions of K, so what
// the padding bytes are does not matter.  The bytes of that copy, 0 when the layer is not such a one.
int64_t padded_input_bytes(const tmq_conv2d_geom& g, const ConvShape& s, bool pinned) {
  if (g.groups != 1 || s.IC % 16 == 0) return 0;
  if (!pinned && s.runs_KS != 0) return 0;
  const int64_t pixels = s.B * s.H * s.W, blocks = ceil_div(s.IC, 16);
  if (pixels == 0 || pixels * blocks > 0x7fffffff) return 0;
  return pixels * blocks * 16;
}

// One thread per 16-byte block of the padded copy.
__global__ __launch_bounds__(256) void conv_pad_channels_kernel(const uint8_t* __restrict__ x, int IC, int blocks,
                                                                int64_t total, uint8_t* __restrict__ dst) {
  const int64_t id = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (id >= total) return;
  const int64_t pixel = id / blocks;
  const int c0 = static_cast<int>(id - pixel * blocks) * 16;
  const uint8_t* src = x + pixel * IC + c0;
  const int n = IC - c0 < 16 ? IC - c0 : 16;
  uint32_t words[4] = {0, 0, 0, 0};
#pragma unroll
  for (int b = 0; b < 16; ++b)
    if (b < n) words[b >> 2] |= static_cast<uint32_t>(src[b]) << (8 * (b & 3));
  *reinterpret_cast<v4i*>(dst + id * 16) = v4i{static_cast<int>(words[0]), static_cast<int>(words[1]),
                                               static_cast<int>(words[2]), static_cast<int>(words[3])};
}

struct PlainArgs {
  const uint8_t* x;
  const uint8_t* w_packed;
  const int32_t* colsum;
  const float* w_scales;
  const float* bias;
  int32_t w_scale_stride, x_signed, x_zp;
  float x_scale, out_scale, zp_f, lo_f, hi_f;
  void* y;
  PostOps post;
};

// Direct convolution, one thread per output value: any channel count, any
// grouping, any alignment.  Accumulates (x - x_zp) * w over in-image taps.
template <int MODE>
__global__ __launch_bounds__(256) void conv_plain_kernel(ConvShape s, PlainArgs a) {
  const int64_t id = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  const int64_t rows = s.B * s.OH * s.OW;
  if (id >= rows * s.OC) return;
  const int64_t oc = id % s.OC, m = id / s.OC;
  const int64_t g = oc / s.OCg, n = oc % s.OCg;
  const int64_t ow = m % s.OW, oh = (m / s.OW) % s.OH, b = m / (s.OW * s.OH);
  const uint8_t* wp = a.w_packed + g * s.group_bytes;
  const int64_t sub = n / s.OCgo * s.ICgo;  // first input channel of the channel's own group inside a merged one
  int acc = 0;
  for (int64_t kh = 0; kh < s.KH; ++kh) {
    const int64_t ih = oh * s.sh - s.ph + kh * s.dh;
    if (ih < 0 || ih >= s.H) continue;
    for (int64_t kw = 0; kw < s.KW; ++kw) {
      const int64_t iw = ow * s.sw - s.pw + kw * s.dw;
      if (iw < 0 || iw >= s.W) continue;
      const uint8_t* xp = a.x + ((b * s.H + ih) * s.W + iw) * s.IC + g * s.ICg + sub;
      const int64_t kbase = (kh * s.KW + kw) * s.ICgp + sub;
      for (int64_t ic = 0; ic < s.ICgo; ++ic) {
        const int xv = a.x_signed ? static_cast<int>(static_cast<int8_t>(xp[ic])) : static_cast<int>(xp[ic]);
        const int64_t k = kbase + ic;
        const int wv = static_cast<int8_t>(wp[(((n >> 4) * s.KC + (k >> 4)) * 16 + (n & 15)) * 16 + (k & 15)]);
        acc += (xv - a.x_zp) * wv;
      }
    }
  }
  if (MODE == kOutAcc32) {
    static_cast<int32_t*>(a.y)[id] = acc;
  } else {
    const float atw = a.x_scale * a.w_scales[oc * a.w_scale_stride];
    const float mult = atw / a.out_scale;
    float v = static_cast<float>(acc);
    if (a.bias != nullptr)
      v = __builtin_fmaf(bias_term(a.w_scale_stride == 0, a.bias[oc], atw), bias_mul(a.w_scale_stride == 0, atw), v);
    float ab = v * mult;
    if (a.post.accum != nullptr) {
      const uint8_t b8 = a.post.accum[id];
      const int qa = a.post.accum_signed ? static_cast<int>(static_cast<int8_t>(b8)) : static_cast<int>(b8);
      const float ad = static_cast<float>(qa - a.post.accum_zp) * a.post.amult;
      ab = ab + ad;
    }
    if (a.post.silu) ab = silu_in_output_units(ab, a.post.silu_c, a.post.silu_c_tail);
    float r = __builtin_rintf(ab) + a.zp_f;
    r = __builtin_amdgcn_fmed3f(r, a.lo_f, a.hi_f);
    static_cast<uint8_t*>(a.y)[id] = static_cast<uint8_t>(static_cast<int>(r));
  }
}

template <int BM, int BN, int WM, int WN, int MODE, int KW = 1>
int launch_conv_gemm(const GemmArgs& a, const XConv& xs, hipStream_t s) {
  const int64_t blocks = ceil_div(a.M, BM) * ceil_div(a.N, BN);
  if (blocks > 0x7fffffff) return TMQ_ERR_UNSUPPORTED;
  gemm_i8_kernel<BM, BN, WM, WN, MODE, XConv, 4, false, KW>
      <<<dim3(static_cast<unsigned>(blocks)), dim3(WM * WN * KW * kWave), 0, s>>>(a, xs);
  return launch_status();
}

// Patch shape and LDS layout of the halo-tiled kernel for one problem.
struct TilePlan {
  int TH, TW, HH, HW, pitch, KS;
  int row_slots;  // 16-byte LDS slots per halo row, padding included
  int lds_x, lds_t, lds_tab, lds_total;
};

constexpr int kMaxDevices = 64;

int current_device() {
  int dev = 0;
  return hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < kMaxDevices ? dev : -1;
}

// LDS bytes a block may use on the current device (cached per device; two
// threads that race on the first call store the same value).
int lds_limit() {
  static std::atomic<int> cache[kMaxDevices];
  const int dev = current_device();
  if (dev < 0) return 0;
  int v = cache[dev].load(std::memory_order_relaxed);
  if (v == 0) {
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess) return 0;
    cache[dev].store(v, std::memory_order_relaxed);
  }
  return v;
}

// Chooses the patch that minimises a time estimate fitted to per-phase cycle
// stamps and a sweep of patch shapes at [32,56,56,64] x [64,3,3,64].  Per block:
//   fixed      3000 cycles of set-up, barriers and first-load latency
//   mfma       the busiest SIMD's row tiles x k-steps x 64 cycles
//   copy       weight bytes / 16 + 290 cycles per pass of the block over the halo
//              (a pass moves floor(512 / slots per halo row) whole halo rows, so
//              narrow halos waste fewer lanes: 28x14 patches take 5 passes where
//              7x56 patches of the same 392 pixels take 9)
//   epilogue   8.4 cycles per output pixel
// Blocks that fit a CU's LDS together overlap: the first costs the whole chain,
// each further one the larger of its SIMD work (half the fixed cost + mfma +
// epilogue) and its copies; blocks that do not fit run one after the other.  Returns false when
// the weight slice or the smallest halo do not fit.
bool plan_tiles(const ConvShape& s, bool forced, int forced_rows, int forced_cols, TilePlan* best) {
  // A block loads every pixel of its halo, so a kernel smaller than its stride
  // (1x1 stride 2: three of four loaded pixels unused) runs 1.6-3.7x faster as an
  // implicit GEMM, which gathers only what it multiplies.  Everything else that
  // fits is faster here, measured over ResNet-50's layer shapes at batch 32:
  // 3x3 stride 1 and 7x7 stride 2 by 1.8x, 3x3 stride 2 by 1.2-1.7x, 1x1 stride 1
  // by 1.05-1.8x.  With few output pixels and one round of blocks the wasted pixels cost
  // less than the implicit GEMM's long k loop on a handful of tiles (one image, 1x1 stride 2:
  // 256 -> 512 on 56 x 56 4.6 against 5.7 us, 1024 -> 2048 on 14 x 14 5.8 against 9.4 us; eight
  // images, 1024 -> 2048: 512 blocks, 17.6 against 9.7 us).
  const bool wasteful = !forced && s.KH * s.KW < s.sh * s.sw;
  if (wasteful && s.B * s.OH * s.OW > 1024) return false;
  const int64_t icb = s.ICg / 16;
  const int64_t chunks = s.KH * s.KW * icb;
  const int64_t KS = round_up(ceil_div(chunks, 2), 2);  // <= packed k-chunks / 2 (padded to 8)
  const int64_t w_bytes = 2048 * KS;
  const int64_t budget = static_cast<int64_t>(lds_limit()) - 3 * kCtBN * 4 - 256;
  if (w_bytes > 96 * 1024 || icb > 64) return false;
  const int64_t pitch = (icb | 1) * 16;
  const int64_t n_tiles = ceil_div(s.OCg, kCtBN);
  constexpr int64_t kCuLds = 160 * 1024;
  // patch widths: the whole row or a power of two, and the row cut into 2..8 equal parts
  int64_t widths[14];
  int nw = 0;
  const auto add_width = [&](int64_t w) {
    if (w < 1) return;
    for (int i = 0; i < nw; ++i)
      if (widths[i] == w) return;
    widths[nw++] = w;
  };
  if (forced_cols > 0) {
    add_width(s.OW < forced_cols ? s.OW : forced_cols);
  } else {
    for (int64_t cap : {128, 64, 32, 16, 8, 4}) add_width(s.OW < cap ? s.OW : cap);
    for (int64_t parts = 2; parts <= 8; ++parts) add_width(ceil_div(s.OW, parts));
  }
  double best_cost = -1.0;
  for (int wi = 0; wi < nw; ++wi) {
    const int64_t TW = widths[wi];
    const int64_t HWd = (TW - 1) * s.sw + (s.KW - 1) * s.dw + 1;
    // Slots per halo row.  A lane's pixel in the k loop is (r, c) of its row tile,
    // r = m / TW, c = m % TW for 32 consecutive m; consecutive pixels of one row lie
    // P = pitch / 16 (odd) slots apart, which spreads 16 lanes over the 16 slot
    // groups of the LDS, but a row tile crosses a patch row every TW lanes.  The
    // halo rows are padded so that the first pixel of the next row continues the
    // sequence: sh * row_slots = TW * sw * P (mod 16).  (Measured at
    // [32,56,56,64] x [64,3,3,64], 28 x 14 patches: bank-conflict cycles 443 k -> 210 k
    // per launch, LDS-active cycles 1.56 M -> 1.34 M; the launch time does not change,
    // the kernel is not bound by LDS bandwidth.)
    int64_t row_slots = HWd * (pitch / 16);
    for (int64_t pad = 0; pad < 16; ++pad)
      if ((s.sh * (row_slots + pad) - TW * s.sw * (pitch / 16)) % 16 == 0) {
        row_slots += pad;
        break;
      }
    if (row_slots > kCtThreads) continue;  // one halo row is copied in one pass of the block
    const int64_t rows_per_pass = kCtThreads / row_slots;
    for (int64_t TH = 1; TH <= s.OH && TH * TW <= kCtMaxPixels; ++TH) {
      if (forced_rows > 0 && TH != forced_rows) continue;
      const int64_t HH = (TH - 1) * s.sh + (s.KH - 1) * s.dh + 1;
      const int64_t x_bytes = HH * row_slots * 16;
      const int64_t total = w_bytes + x_bytes + kCtWaves * kCtTBytes + round_up(8 * (KS + 4), 16);
      if (total > budget) break;
      const int64_t blocks = s.B * ceil_div(s.OH, TH) * ceil_div(s.OW, TW) * n_tiles * s.groups;
      const int64_t MT = ceil_div(TH * TW, 32);
      const double mfma = static_cast<double>(ceil_div(MT, 4) * KS * 64);
      const double copy = static_cast<double>(w_bytes) / 16.0 + 290.0 * static_cast<double>(ceil_div(HH, rows_per_pass));
      const double epilogue = 8.4 * static_cast<double>(TH * TW);
      const int64_t per_cu = ceil_div(blocks, 256);
      int64_t together = kCuLds / (total + 3 * kCtBN * 4);
      together = together < 1 ? 1 : (together > per_cu ? per_cu : together);
      // half of the fixed cost is instructions (set-up, address tables), which a
      // co-resident block cannot hide
      const double simd = 1500.0 + mfma + epilogue;
      const double overlapped = simd > copy ? simd : copy;
      const double group = 3000.0 + mfma + copy + epilogue + static_cast<double>(together - 1) * overlapped;
      const double cost = static_cast<double>(ceil_div(per_cu, together)) * group;
      if (wasteful && blocks > 256) continue;
      if (best_cost < 0 || cost < best_cost) {
        best_cost = cost;
        best->TH = static_cast<int>(TH); best->TW = static_cast<int>(TW);
        best->HH = static_cast<int>(HH); best->HW = static_cast<int>(HWd);
        best->pitch = static_cast<int>(pitch); best->KS = static_cast<int>(KS);
        best->row_slots = static_cast<int>(row_slots);
        best->lds_x = static_cast<int>(w_bytes);
        best->lds_t = static_cast<int>(w_bytes + x_bytes);
        best->lds_tab = best->lds_t + kCtWaves * kCtTBytes;
        best->lds_total = static_cast<int>(total);
      }
    }
  }
  return best_cost >= 0;
}

template <int MODE, int KIND, bool VEC>
int launch_conv_tiles_variant(const ConvShape& s, const TilePlan& p, const ConvTileArgs& a, hipStream_t stream) {
  // the kernel's LDS allowance is a per-device attribute: set once per device
  static std::atomic<uint64_t> done{0};
  const int dev = current_device();
  if (dev < 0) return TMQ_ERR_LAUNCH;
  if ((done.load(std::memory_order_acquire) >> dev & 1) == 0) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&conv_tile_kernel<MODE, KIND, VEC>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, lds_limit() - 3 * kCtBN * 4) != hipSuccess)
      return TMQ_ERR_LAUNCH;
    done.fetch_or(uint64_t{1} << dev, std::memory_order_release);
  }
  const int64_t bx = s.B * a.tiles_h * a.tiles_w, by = static_cast<int64_t>(a.n_tiles) * s.groups;
  if (bx > 0x7fffffff || by > 65535) return TMQ_ERR_UNSUPPORTED;
  conv_tile_kernel<MODE, KIND, VEC><<<dim3(static_cast<unsigned>(bx), static_cast<unsigned>(by)),
                                      dim3(kCtThreads), p.lds_total, stream>>>(a);
  return launch_status();
}

// Whether the packing conversion alone requantises this call's outputs (requant_plain_u8 of gemm_i8_core.h): zero
// point 0 and no bounds inside [0, 255] for unsigned bytes, the same 128 lower for signed ones.
template <int MODE>
bool plain_bytes(float zp_f, float lo_f, float hi_f) {
  const float shift = MODE == kOutS8 ? 128.f : 0.f;
  return requant_plain_u8(zp_f + shift, lo_f + shift, hi_f + shift);
}

// Which epilogue the launch needs (see conv_tile_kernel) is known on the host.
template <int MODE>
int launch_conv_tiles(const ConvShape& s, const TilePlan& p, const ConvTileArgs& a, hipStream_t stream) {
  const bool aligned16 = (reinterpret_cast<uintptr_t>(a.y) & 15) == 0;
  if constexpr (MODE == kOutAcc32) {
    const bool vec = (a.OC & 3) == 0 && (a.OCg & 3) == 0 && aligned16;
    return vec ? launch_conv_tiles_variant<MODE, 1, true>(s, p, a, stream)
               : launch_conv_tiles_variant<MODE, 1, false>(s, p, a, stream);
  } else {
    const bool vec = (a.OC & 15) == 0 && (a.OCg & 15) == 0 && aligned16;
    const int kind = a.post.silu ? 3
                     : a.post.accum != nullptr ? (plain_bytes<MODE>(a.zp_f, a.lo_f, a.hi_f) ? 5 : 0)
                     : plain_bytes<MODE>(a.zp_f, a.lo_f, a.hi_f) ? 4
                     : ((MODE == kOutU8 && a.lo_f <= 0.f && a.hi_f >= 255.f) ? 2 : 1);
    switch (kind * 2 + (vec ? 1 : 0)) {
      case 0: return launch_conv_tiles_variant<MODE, 0, false>(s, p, a, stream);
      case 1: return launch_conv_tiles_variant<MODE, 0, true>(s, p, a, stream);
      case 2: return launch_conv_tiles_variant<MODE, 1, false>(s, p, a, stream);
      case 3: return launch_conv_tiles_variant<MODE, 1, true>(s, p, a, stream);
      case 4: return launch_conv_tiles_variant<MODE, 2, false>(s, p, a, stream);
      case 5: return launch_conv_tiles_variant<MODE, 2, true>(s, p, a, stream);
      case 6: return launch_conv_tiles_variant<MODE, 3, false>(s, p, a, stream);
      case 7: return launch_conv_tiles_variant<MODE, 3, true>(s, p, a, stream);
      case 8: return launch_conv_tiles_variant<MODE, 4, false>(s, p, a, stream);
      case 9: return launch_conv_tiles_variant<MODE, 4, true>(s, p, a, stream);
      case 10: return launch_conv_tiles_variant<MODE, 5, false>(s, p, a, stream);
      default: return launch_conv_tiles_variant<MODE, 5, true>(s, p, a, stream);
    }
  }
}

// Tile shape and LDS use of the few-channel kernel (conv_runs.h) for one problem; false
// when the kernel does not take it: groups, dilation, kernel rows of more than 256 padded bytes.
struct RunPlan {
  int RL, RP, KS, TR, TW, mtw, rows_in, pitch, lds;
};
bool plan_runs(const ConvShape& s, int forced_rows, RunPlan* p) {
  if (s.runs_KS == 0) return false;
  const int64_t RL = s.runs_RL, RP = s.runs_RP, KS = s.runs_KS;
  // Tile = TR output rows x TW columns.  The staged image rows of a tile pass through
  // registers in units of 1 KB of a row, at most kCrUnits per wave; among the shapes that
  // fit, the one with the shortest schedule: rounds of tiles over the blocks the chip holds
  // (three per CU) times the turns its four waves need for the tile's 16-pixel pieces.
  constexpr int64_t kSlots = 3 * 256, kMaxUnits = int64_t{kCrUnits} * kCrWaves;
  int64_t best = -1;
  for (int64_t TW = s.OW < 128 ? s.OW : 128;; TW = round_up(TW / 2, 16)) {
    const int64_t mtw = ceil_div(TW, 16);
    const int64_t pitch = round_up((TW - 1) * s.sw * s.IC + RP + 20, 16);
    for (int64_t TR = 1; TR <= s.OH && TR <= 8; ++TR) {
      const int64_t rows_in = (TR - 1) * s.sh + s.KH;
      if (rows_in * ceil_div(pitch, 1024) > kMaxUnits) break;
      if (forced_rows > 0 && TR != forced_rows) continue;
      const int64_t tiles = s.B * ceil_div(s.OH, TR) * ceil_div(s.OW, TW);
      if (tiles > 0x7fffffff) continue;
      const int64_t cost = ceil_div(tiles, kSlots) * (ceil_div(TR * mtw, kCrWaves) * 10 + 5);
      if (best < 0 || cost < best) {
        best = cost;
        p->RL = static_cast<int>(RL); p->RP = static_cast<int>(RP); p->KS = static_cast<int>(KS);
        p->TR = static_cast<int>(TR); p->TW = static_cast<int>(TW); p->mtw = static_cast<int>(mtw);
        p->rows_in = static_cast<int>(rows_in); p->pitch = static_cast<int>(pitch);
        p->lds = static_cast<int>(rows_in * pitch);
      }
    }
    if (TW <= 16) break;
  }
  return best >= 0;
}

template <int MODE>
int launch_conv_runs(const tmq_conv2d_desc* d, const ConvShape& s, const RunPlan& p, const PostOps& po, float zp_f,
                     float lo_f, float hi_f, void* out, hipStream_t stream) {
  ConvRunArgs a{};
  a.x = static_cast<const uint8_t*>(d->x);
  a.w_runs = static_cast<const uint8_t*>(d->w_packed) + s.runs_off;
  a.colsum = d->w_colsum;
  a.w_scales = d->w_scales;
  a.bias = d->bias;
  a.y = out;
  a.B = static_cast<int>(s.B);
  a.H = static_cast<int>(s.H); a.W = static_cast<int>(s.W); a.IC = static_cast<int>(s.IC);
  a.OH = static_cast<int>(s.OH); a.OW = static_cast<int>(s.OW); a.OC = static_cast<int>(s.OC);
  a.KH = static_cast<int>(s.KH); a.KW = static_cast<int>(s.KW);
  a.sh = static_cast<int>(s.sh); a.sw = static_cast<int>(s.sw);
  a.ph = static_cast<int>(s.ph); a.pw = static_cast<int>(s.pw);
  a.RL = p.RL; a.RP = p.RP; a.KS = p.KS;
  a.TR = p.TR; a.TW = p.TW; a.mtw = p.mtw;
  a.rows_in = p.rows_in; a.pitch = p.pitch;
  a.tiles_h = static_cast<int>(ceil_div(s.OH, p.TR));
  a.tiles_w = static_cast<int>(ceil_div(s.OW, p.TW));
  a.tiles = static_cast<int32_t>(s.B * a.tiles_h * a.tiles_w);
  a.vec = aligned(out, 16) && s.OC % (MODE == kOutAcc32 ? 4 : 16) == 0 ? 1 : 0;
  a.w_scale_stride = d->w_per_channel ? 1 : 0;
  a.x_xor = d->x_signed ? 0u : 0x80808080u;
  a.pad_word = 0x01010101u * static_cast<uint32_t>(static_cast<uint8_t>(d->x_zero_point));
  a.acc_coef = (d->x_signed ? 0 : 128) - d->x_zero_point;
  a.x_scale = d->x_scale;
  a.out_scale = d->out_scale;
  a.zp_f = zp_f; a.lo_f = lo_f; a.hi_f = hi_f;
  a.post = po;
  const int nt = conv_runs_tiles(s.OC);
  const int64_t by = ceil_div(s.OC, 16 * nt);
  if (by > 65535) return TMQ_ERR_UNSUPPORTED;
  // three blocks per CU (their registers), each with its weights in registers for every tile it walks
  const int64_t bx = a.tiles < 768 ? a.tiles : 768;  // (plan_runs: kSlots)
  const dim3 grid(static_cast<unsigned>(bx), static_cast<unsigned>(by)), block(kCrThreads);
  const auto launch = [&](auto post_tag, auto nt_tag, auto plain_tag) {
    conv_runs_kernel<MODE, decltype(post_tag)::value, decltype(nt_tag)::value, decltype(plain_tag)::value>
        <<<grid, block, p.lds, stream>>>(a);
  };
  const auto launch_tiles = [&](auto nt_tag) {
    if constexpr (MODE != kOutAcc32) {
      if (po.any()) return launch(std::true_type{}, nt_tag, std::false_type{});
      if (plain_bytes<MODE>(zp_f, lo_f, hi_f)) return launch(std::false_type{}, nt_tag, std::true_type{});
    }
    launch(std::false_type{}, nt_tag, std::false_type{});
  };
  if (nt == 2)
    launch_tiles(std::integral_constant<int, 2>{});
  else
    launch_tiles(std::integral_constant<int, 4>{});
  return launch_status();
}

// Pointwise layers over at most 256 input channels with their pixels straight from memory
// (conv_runs_pointwise_kernel); false when the layer is not one of them.
bool pointwise_rows_ok(const tmq_conv2d_geom& g, const ConvShape& s) {
  return g.groups == 1 && s.KH == 1 && s.KW == 1 && s.sh == 1 && s.sw == 1 && s.ph == 0 && s.pw == 0 && s.runs_KS > 0 &&
         conv_runs_pointwise_lds(s.OC, s.runs_KS) <= kCrPointwiseLdsMax;
}

template <int MODE>
int launch_conv_pointwise_rows(const tmq_conv2d_desc* d, const ConvShape& s, const PostOps& po, float zp_f, float lo_f,
                               float hi_f, void* out, hipStream_t stream) {
  ConvRunArgs a{};
  a.x = static_cast<const uint8_t*>(d->x);
  a.w_runs = static_cast<const uint8_t*>(d->w_packed) + s.runs_off;
  a.colsum = d->w_colsum;
  a.w_scales = d->w_scales;
  a.bias = d->bias;
  a.y = out;
  a.B = static_cast<int>(s.B);
  a.H = static_cast<int>(s.H); a.W = static_cast<int>(s.W); a.IC = static_cast<int>(s.IC);
  a.OH = static_cast<int>(s.OH); a.OW = static_cast<int>(s.OW); a.OC = static_cast<int>(s.OC);
  a.KH = a.KW = 1;
  a.sh = a.sw = 1;
  a.RL = static_cast<int>(s.runs_RL); a.RP = static_cast<int>(s.runs_RP); a.KS = static_cast<int>(s.runs_KS);
  const int64_t pieces = ceil_div(s.B * s.H * s.W, 16);
  if (pieces > 0x7fffffff) return TMQ_ERR_UNSUPPORTED;
  a.tiles = static_cast<int32_t>(pieces);
  a.vec = aligned(out, 16) && s.OC % (MODE == kOutAcc32 ? 4 : 16) == 0 ? 1 : 0;
  a.w_scale_stride = d->w_per_channel ? 1 : 0;
  a.x_xor = d->x_signed ? 0u : 0x80808080u;
  a.acc_coef = (d->x_signed ? 0 : 128) - d->x_zero_point;
  a.x_scale = d->x_scale;
  a.out_scale = d->out_scale;
  a.zp_f = zp_f; a.lo_f = lo_f; a.hi_f = hi_f;
  a.post = po;
  const int nt = conv_runs_tiles(s.OC);
  const int64_t lds = conv_runs_pointwise_lds(s.OC, s.runs_KS);
  // as many blocks per CU as their registers and weights allow (three),
  // each walking the pieces its waves are dealt
  int64_t per_cu = (160 * 1024) / (lds + 512);
  const int64_t by_registers = 3;
  per_cu = per_cu < 1 ? 1 : per_cu > by_registers ? by_registers : per_cu;
  const int64_t want = ceil_div(pieces, kCrWaves), cap = 256 * per_cu;
  const dim3 grid(static_cast<unsigned>(want < cap ? want : cap)), block(kCrThreads);
  const auto launch = [&](auto post_tag, auto nt_tag, auto plain_tag) {
    auto* const kernel = conv_runs_pointwise_kernel<MODE, decltype(post_tag)::value, decltype(nt_tag)::value,
                                                    decltype(plain_tag)::value>;
    // the kernel's LDS allowance is a per-device attribute: set once per device (and kernel)
    static std::atomic<uint64_t> done{0};
    const int dev = current_device();
    if (dev < 0) return false;
    if ((done.load(std::memory_order_acquire) >> dev & 1) == 0) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                              kCrPointwiseLdsMax) != hipSuccess)
        return false;
      done.fetch_or(uint64_t{1} << dev, std::memory_order_release);
    }
    kernel<<<grid, block, static_cast<size_t>(lds), stream>>>(a);
    return true;
  };
  const auto launch_tiles = [&](auto nt_tag) {
    if constexpr (MODE != kOutAcc32) {
      if (po.any()) return launch(std::true_type{}, nt_tag, std::false_type{});
      if (plain_bytes<MODE>(zp_f, lo_f, hi_f)) return launch(std::false_type{}, nt_tag, std::true_type{});
    }
    return launch(std::false_type{}, nt_tag, std::false_type{});
  };
  const bool ok = nt == 2 ? launch_tiles(std::integral_constant<int, 2>{}) : launch_tiles(std::integral_constant<int, 4>{});
  return ok ? launch_status() : TMQ_ERR_LAUNCH;
}

// Depthwise layers on the vector ALU (conv_depthwise.h).
template <int MODE>
int launch_conv_depthwise(const tmq_conv2d_desc* d, const ConvShape& s, const PostOps& po, float zp_f, float lo_f,
                          float hi_f, void* out, hipStream_t stream) {
  DepthwiseArgs a{};
  a.x = static_cast<const uint8_t*>(d->x);
  a.w_taps = static_cast<const uint8_t*>(d->w_packed) + s.runs_off;
  a.colsum = d->w_colsum;
  a.w_scales = d->w_scales;
  a.bias = d->bias;
  a.y = out;
  a.B = static_cast<int>(s.B);
  a.H = static_cast<int>(s.H); a.W = static_cast<int>(s.W); a.C = static_cast<int>(s.IC);
  a.OH = static_cast<int>(s.OH); a.OW = static_cast<int>(s.OW);
  a.KH = static_cast<int>(s.KH); a.KW = static_cast<int>(s.KW);
  a.sh = static_cast<int>(s.sh); a.sw = static_cast<int>(s.sw);
  a.ph = static_cast<int>(s.ph); a.pw = static_cast<int>(s.pw);
  a.dh = static_cast<int>(s.dh); a.dw = static_cast<int>(s.dw);
  // Output rows per lane: long strips amortise the lane's weights and constants, short ones put
  // more waves in flight; the longest with a wave per SIMD (half a wave under a 7 x 7 kernel, whose
  // window of 49 taps is the larger part of a short strip's work).
  // Under 5 x 5 and 7 x 7 windows, whose first rows are the larger part of a short strip, up to 14 rows, and the
  // image in equal strips (7 x 7 over 96 channels on 56 x 56: 21.1 -> 18.9 us; 5 x 5 over 240 channels on 28 x 28:
  // 12.6 -> 10.8 us; 3 x 3 gains nothing beyond 8).
  const bool pinned_strip = d->kernel == 7 && d->tile_rows > 0;
  int64_t strip = pinned_strip ? d->tile_rows : kDwStripMax;
  // (images of 9 to 14 rows in two strips: 5 x 5 over 672 channels on 14 x 14 9.9 against 10.8 us in one)
  if (!pinned_strip && s.KH >= 5 && s.OH > 8) strip = ceil_div(s.OH, s.OH <= 14 ? 2 : ceil_div(s.OH, 14));
  const int64_t lanes_wanted = int64_t{1} << (s.KH == 7 && s.KW == 7 ? 15 : 16);
  if (!pinned_strip)
    while (strip > 1 && s.B * ceil_div(s.OH, strip) * s.OW * (s.IC / 4) < lanes_wanted) strip = ceil_div(strip, 2);
  if (strip > s.OH) strip = s.OH;
  a.strip = static_cast<int>(strip);
  const int64_t per_image = ceil_div(s.OH, strip) * s.OW * (s.IC / 4);
  const int64_t blocks_per_image = ceil_div(per_image, kDwThreads);
  a.per_image = static_cast<uint32_t>(per_image);
  a.blocks_per_image = static_cast<uint32_t>(blocks_per_image);
  a.w_scale_stride = d->w_per_channel ? 1 : 0;
  a.x_xor = d->x_signed ? 0u : 0x80808080u;
  a.pad_word = 0x01010101u * static_cast<uint32_t>(static_cast<uint8_t>(d->x_zero_point));
  a.acc_coef = (d->x_signed ? 0 : 128) - d->x_zero_point;
  a.x_scale = d->x_scale;
  a.out_scale = d->out_scale;
  a.zp_f = zp_f; a.lo_f = lo_f; a.hi_f = hi_f;
  a.post = po;
  const int64_t blocks = s.B * blocks_per_image;
  if (blocks > 0x7fffffff) return TMQ_ERR_UNSUPPORTED;
  const dim3 grid(static_cast<unsigned>(blocks)), block(kDwThreads);
  const auto launch = [&](auto post_tag) {
    constexpr bool kP = decltype(post_tag)::value;
    if (s.KH == 3 && s.KW == 3)
      conv_depthwise_kernel<MODE, kP, 3><<<grid, block, 0, stream>>>(a);
    else if (s.KH == 5 && s.KW == 5)
      conv_depthwise_kernel<MODE, kP, 5><<<grid, block, 0, stream>>>(a);
    else if (s.KH == 7 && s.KW == 7)
      conv_depthwise_kernel<MODE, kP, 7><<<grid, block, 0, stream>>>(a);
    else
      conv_depthwise_kernel<MODE, kP, 0><<<grid, block, 0, stream>>>(a);
  };
  if constexpr (MODE != kOutAcc32) {
    if (po.any()) {
      launch(std::true_type{});
      return launch_status();
    }
  }
  launch(std::false_type{});
  return launch_status();
}

// quantized::linear over `rows` rows of K bytes at `x` (the pixels of a pointwise layer, or patch
// rows) with the layer's packed weight, which for one group over whole 16-channel blocks is the
// linear layout: [OC, K] in 16-channel blocks, k = (kh, kw, ic).
int run_as_linear(const tmq_conv2d_desc* d, int64_t rows, int64_t OC, int64_t K, const void* x, bool relu, void* out,
                  hipStream_t stream) {
  tmq_linear_desc l{};
  l.M = rows; l.N = OC; l.K = K;
  l.x = x; l.ldx = K;
  l.x_signed = d->x_signed; l.x_zero_point = d->x_zero_point; l.x_scale = d->x_scale;
  l.w_packed = d->w_packed; l.w_colsum = d->w_colsum; l.w_scales = d->w_scales;
  l.w_per_channel = d->w_per_channel;
  l.relu = relu ? 1 : 0;
  l.bias = d->bias;
  l.out_scale = d->out_scale; l.out_zero_point = d->out_zero_point; l.out_signed = d->out_signed;
  l.y = out; l.ldy = OC;
  return tmq_linear(&l, reinterpret_cast<tmq_stream_t>(stream));
}

template <int MODE>
int run_conv(const tmq_conv2d_desc* d, const tmq_conv2d_post* post, void* out, hipStream_t stream) {
  ConvShape s;
  int rc = make_shape(&d->geom, &s);
  if (rc != TMQ_OK) return rc;
  const int64_t rows = s.B * s.OH * s.OW;
  if (rows == 0) return TMQ_OK;
  if (d->x == nullptr || d->w_packed == nullptr || d->w_colsum == nullptr || out == nullptr)
    return TMQ_ERR_INVALID_ARGUMENT;
  if (!aligned(d->w_packed, 16)) return TMQ_ERR_ALIGNMENT;
  const int qmin = d->out_signed ? -128 : 0, qmax = d->out_signed ? 127 : 255;
  const int xmin = d->x_signed ? -128 : 0, xmax = d->x_signed ? 127 : 255;
  if (d->x_zero_point < xmin || d->x_zero_point > xmax) return TMQ_ERR_INVALID_ARGUMENT;
  if (MODE != kOutAcc32) {
    if (d->w_scales == nullptr || !(d->x_scale > 0.f) || !(d->out_scale > 0.f))
      return TMQ_ERR_INVALID_ARGUMENT;
    if (d->out_zero_point < qmin || d->out_zero_point > qmax) return TMQ_ERR_INVALID_ARGUMENT;
  }
  PostOps po{};
  bool relu = d->relu != 0;
  if (post != nullptr) {
    if (MODE == kOutAcc32) return TMQ_ERR_INVALID_ARGUMENT;
    if (post->activation < 0 || post->activation > 2) return TMQ_ERR_INVALID_ARGUMENT;
    if (post->activation == 2 && relu) return TMQ_ERR_INVALID_ARGUMENT;
    relu = relu || post->activation == 1;
    po.silu = post->activation == 2;
    po.out_scale = d->out_scale;
    {
      const double exact = -static_cast<double>(d->out_scale) * 1.4426950408889634074;  // -s log2(e)
      po.silu_c = static_cast<float>(exact);
      po.silu_c_tail = static_cast<float>(exact - static_cast<double>(po.silu_c));
    }
    if (post->accum != nullptr) {
      const int amin = post->accum_signed ? -128 : 0, amax = post->accum_signed ? 127 : 255;
      if (!(post->accum_scale > 0.f) || post->accum_zero_point < amin || post->accum_zero_point > amax)
        return TMQ_ERR_INVALID_ARGUMENT;
      po.accum = static_cast<const uint8_t*>(post->accum);
      po.accum_signed = post->accum_signed;
      po.accum_zp = post->accum_zero_point;
      po.amult = post->accum_scale / d->out_scale;
    }
  }
  const float zp_f = static_cast<float>(d->out_zero_point);
  const float lo_f = static_cast<float>(relu ? d->out_zero_point : qmin);
  const float hi_f = static_cast<float>(qmax);

  const int forced = d->kernel > 0 ? d->kernel : -1;
  // A pointwise layer (1 x 1, stride 1, no padding, one group) is a linear layer over the
  // pixels: rows = pixels, K = input channels, and the packed weight is the linear one
  // (same 16-channel blocks, same k padding).  With few pixels -- the late stages of an
  // image network -- the linear kernels' choice for short M is ahead of the halo tiles
  // (1024 -> 256 channels on 14 x 14, batch 32: 12.8 -> 7.8 us; 512 -> 2048 on 7 x 7: 11.7 -> 7.1 us).
  if constexpr (MODE != kOutAcc32) {
    const bool pointwise = s.KH == 1 && s.KW == 1 && s.sh == 1 && s.sw == 1 && s.ph == 0 && s.pw == 0 &&
                           d->geom.groups == 1 && s.IC % 16 == 0 && aligned(d->x, 16) && !po.any();
    if (forced == 5 && !pointwise) return TMQ_ERR_UNSUPPORTED;
    // (and with 128 input and 256 output channels or more from about a billion products on: 256 -> 256 on
    // 56 x 56 at batch 32 35.9 -> 25.8 us, 512 -> 512 on 28 x 28 25.0 -> 16.1 us, 128 -> 512 13.7 -> 11.6 us; fewer
    // channels on either side stay with the tiles: 256 -> 64 on 56 x 56 11.7 against 19.9 us, 96 -> 576 on
    // 28 x 28 14.3 against 18.0 us)
    // (a detection head's 255 channels count as wide: 128 -> 255 on 80 x 80 at batch 8 18.0 -> 15.2 us)
    const bool wide = s.IC >= 128 && s.OC >= 224 && rows * s.IC * s.OC >= 1000000000;
    if (forced == 5 || (forced < 0 && pointwise && (rows <= kPointwiseAsLinearRows || wide))) {
      return run_as_linear(d, rows, s.OC, s.IC, d->x, relu, out, stream);
    }
  }
  // Few output pixels against a long K and a weight slice the halo tiles cannot hold: with a
  // workspace the patch rows are written out and the product runs on the linear kernels
  // (3 x 3, 256 -> 256 channels, one 14 x 14 image: 13.1 -> 10.1 us; 512 -> 512, one 7 x 7 image:
  // 19.8 -> 16.1 us, eight of them 19.7 -> 17.2 us; from about a thousand pixels on the implicit
  // GEMM with its wave groups is ahead: 1568 pixels, 256 -> 256: 13.6 against 15.4 us).
  if constexpr (MODE != kOutAcc32) {
    if (forced == 6 || forced < 0) {
      const int64_t need = po.any() || !aligned(d->x, 16) ? 0 : patch_rows_bytes(d->geom, s, forced == 6);
      TilePlan tp;
      const bool use = need > 0 && d->workspace != nullptr && d->workspace_bytes >= need && aligned(d->workspace, 16) &&
                       (forced == 6 || !plan_tiles(s, false, 0, 0, &tp));
      if (forced == 6 && !use) return TMQ_ERR_UNSUPPORTED;
      if (use) {
        const int64_t chunks = need / 16;
        conv_patch_rows_kernel<<<dim3(static_cast<unsigned>(ceil_div(chunks, 256))), dim3(256), 0, stream>>>(
            static_cast<const uint8_t*>(d->x), s, chunks,
            0x01010101u * static_cast<uint32_t>(static_cast<uint8_t>(d->x_zero_point)), static_cast<uint8_t*>(d->workspace));
        if (launch_status() != TMQ_OK) return TMQ_ERR_LAUNCH;
        return run_as_linear(d, rows, s.OC, s.Kp, d->workspace, relu, out, stream);
      }
    }
  }
  // Channel counts off the 16-channel grid under kernel rows too long for the byte runs: the MFMA kernels on a
  // padded copy of the input in the caller's scratch memory (3 x 3, 40 -> 40 channels on 56 x 56 at batch 32 and
  // the 11 x 11 stride 4 first layer of an early image network, 3 -> 64 on 224 x 224, otherwise on the direct kernel).
  if (forced == 8 || forced < 0) {
    const int64_t need = padded_input_bytes(d->geom, s, forced == 8);
    tmq_conv2d_geom padded_geom = d->geom;
    padded_geom.IC = round_up(s.IC, 16);
    ConvShape padded_shape;
    const bool use = need > 0 && d->workspace != nullptr && d->workspace_bytes >= need && aligned(d->workspace, 16) &&
                     make_shape(&padded_geom, &padded_shape) == TMQ_OK;
    if (forced == 8 && !use) return TMQ_ERR_UNSUPPORTED;
    if (use) {
      const int64_t chunks = need / 16;
      conv_pad_channels_kernel<<<dim3(static_cast<unsigned>(ceil_div(chunks, 256))), dim3(256), 0, stream>>>(
          static_cast<const uint8_t*>(d->x), static_cast<int>(s.IC), static_cast<int>(ceil_div(s.IC, 16)), chunks,
          static_cast<uint8_t*>(d->workspace));
      if (launch_status() != TMQ_OK) return TMQ_ERR_LAUNCH;
      tmq_conv2d_desc padded = *d;
      padded.x = d->workspace;
      padded.geom = padded_geom;
      padded.workspace = nullptr;
      padded.workspace_bytes = 0;
      padded.kernel = 0;
      padded.tile_rows = padded.tile_cols = 0;
      return run_conv<MODE>(&padded, post, out, stream);
    }
  }
  const bool mfma_ok = s.ICg % 16 == 0 && aligned(d->x, 16);
  if ((forced == 1 || forced == 2) && !mfma_ok) return TMQ_ERR_UNSUPPORTED;
  // pointwise layers over few input channels: pixels straight from memory against weights in LDS
  {
    const bool rows_ok = pointwise_rows_ok(d->geom, s) && (MODE != kOutAcc32 || aligned(out, 4));
    if (forced == 9 && !rows_ok) return TMQ_ERR_UNSUPPORTED;
    // Automatic where the image offers enough 16-pixel pieces for the chip's waves and few enough channel blocks
    // for a wave to run them all (batch 32, against the halo tiles or the byte-run kernel: 32 -> 16 channels on
    // 112 x 112 19.3 -> 10 us, 24 -> 144 on 56 x 56 21.5 -> 11.5 us, 16 -> 96 on 112 x 112 31 -> 25 us, 256 -> 128 on
    // 56 x 56 18.6 -> 15.6 us, 192 -> 32 on 28 x 28 4.7 -> 4.0 us; 128 -> 512 on 28 x 28 10.5 against 12.5 us and
    // 96 -> 576 on 14 x 14 5.8 against 11.4 us stay where they were).
    const int64_t pieces = ceil_div(s.B * s.H * s.W, 16), blocks = ceil_div(s.OC, 16 * conv_runs_tiles(s.OC));
    // (one channel block: from 128 pieces on -- one image, 32 -> 16 channels on 112 x 112 4.3 -> 3.7 us; and whenever the
    // channel count leaves only the byte-run kernel: one image, 24 -> 144 on 56 x 56 6.6 -> 5.0 us)
    const bool worth = (pieces >= 1024 && (blocks <= 3 || (pieces >= 4096 && blocks <= 4))) ||
                       (pieces >= 128 && blocks == 1) || !mfma_ok;
    if (forced == 9 || (forced < 0 && rows_ok && worth))
      return launch_conv_pointwise_rows<MODE>(d, s, po, zp_f, lo_f, hi_f, out, stream);
  }
  // depthwise layers: four channels per lane on the vector ALU
  {
    // (32-bit byte offsets into the input and the output, also for the rows a window reaches past the image)
    const bool lanes_ok = s.taps_bytes > 0 && s.B * s.H * s.W * s.IC < (int64_t{1} << 31) &&
                          (s.H + s.KH * s.dh + s.sh + 8) * s.W * s.IC < (int64_t{1} << 31) &&
                          s.B * s.OH * s.OW * s.OC < (int64_t{1} << (MODE == kOutAcc32 ? 29 : 31)) && aligned(d->x, 4) && aligned(out, MODE == kOutAcc32 ? 16 : 4) &&
                          (po.accum == nullptr || aligned(po.accum, 4));
    if (forced == 7 && !lanes_ok) return TMQ_ERR_UNSUPPORTED;
    // Also where the groups would merge into 16-channel blocks for the matrix pipe, for the kernel sizes with a
    // register window (batch 32, against the merged groups on the halo tiles or the implicit GEMM: 3 x 3, 32
    // channels on 112 x 112 12.6 against 16.7 us; 96 channels, 112 x 112 -> 56 x 56: 13.9 against 25.2 us; 5 x 5, 240
    // channels on 28 x 28: 13.0 against 17.1 us; 7 x 7, 96 channels on 56 x 56: 22 against 72 us, 768 on 7 x 7: 6.7
    // against 242 us); other kernel sizes stay with the matrix pipe where they can.
    const bool lanes_first = s.KH == s.KW && (s.KH == 3 || s.KH == 5 || s.KH == 7);
    if (forced == 7 || (forced < 0 && lanes_ok && (!mfma_ok || lanes_first)))
      return launch_conv_depthwise<MODE>(d, s, po, zp_f, lo_f, hi_f, out, stream);
  }
  // channel counts (or an address) the 16-byte chunks of the kernels below cannot take:
  // kernel rows as runs of bytes where they are short enough
  if (forced == 4 || (forced < 0 && !mfma_ok)) {
    RunPlan rp;
    if (plan_runs(s, forced == 4 ? d->tile_rows : 0, &rp)) return launch_conv_runs<MODE>(d, s, rp, po, zp_f, lo_f, hi_f, out, stream);
    if (forced == 4) return TMQ_ERR_UNSUPPORTED;
  }
  if (!mfma_ok || forced == 3) {
    PlainArgs p{};
    p.x = static_cast<const uint8_t*>(d->x);
    p.w_packed = static_cast<const uint8_t*>(d->w_packed);
    p.colsum = d->w_colsum;
    p.w_scales = d->w_scales;
    p.bias = d->bias;
    p.w_scale_stride = d->w_per_channel ? 1 : 0;
    p.x_signed = d->x_signed;
    p.x_zp = d->x_zero_point;
    p.x_scale = d->x_scale;
    p.out_scale = d->out_scale;
    p.zp_f = zp_f; p.lo_f = lo_f; p.hi_f = hi_f;
    p.y = out;
    p.post = po;
    const int64_t blocks = ceil_div(rows * s.OC, 256);
    if (blocks > 0x7fffffff) return TMQ_ERR_UNSUPPORTED;
    conv_plain_kernel<MODE><<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream>>>(s, p);
    return launch_status();
  }

  TilePlan plan;
  const bool tiles_ok = forced != 2 && plan_tiles(s, forced == 1, d->tile_rows, d->tile_cols, &plan);
  if (forced == 1 && !tiles_ok) return TMQ_ERR_UNSUPPORTED;
  if (tiles_ok) {
    ConvTileArgs t{};
    t.x = static_cast<const uint8_t*>(d->x);
    t.w_packed = static_cast<const uint8_t*>(d->w_packed);
    t.colsum = d->w_colsum;
    t.w_scales = d->w_scales;
    t.bias = d->bias;
    t.y = out;
    t.w_kchunks = s.KC;
    t.group_bytes = s.group_bytes;
    t.H = static_cast<int>(s.H); t.W = static_cast<int>(s.W); t.IC = static_cast<int>(s.IC);
    t.OH = static_cast<int>(s.OH); t.OW = static_cast<int>(s.OW); t.OC = static_cast<int>(s.OC);
    t.KW = static_cast<int>(s.KW); t.icb = static_cast<int>(s.ICg / 16);
    t.kchunks = static_cast<int>(s.KH * s.KW * (s.ICg / 16));
    t.KS = plan.KS;
    t.sh = static_cast<int>(s.sh); t.sw = static_cast<int>(s.sw);
    t.ph = static_cast<int>(s.ph); t.pw = static_cast<int>(s.pw);
    t.dh = static_cast<int>(s.dh); t.dw = static_cast<int>(s.dw);
    t.ICg = static_cast<int>(s.ICg); t.OCg = static_cast<int>(s.OCg);
    t.n_tiles = static_cast<int>(ceil_div(s.OCg, kCtBN));
    t.TH = plan.TH; t.TW = plan.TW; t.HH = plan.HH; t.HW = plan.HW; t.pitch = plan.pitch;
    t.tiles_h = static_cast<int>(ceil_div(s.OH, plan.TH));
    t.tiles_w = static_cast<int>(ceil_div(s.OW, plan.TW));
    t.lds_x = plan.lds_x; t.lds_t = plan.lds_t; t.lds_tab = plan.lds_tab;
    t.w_scale_stride = d->w_per_channel ? 1 : 0;
    t.x_xor = d->x_signed ? 0u : 0x80808080u;
    t.pad_word = 0x01010101u * static_cast<uint32_t>(static_cast<uint8_t>(d->x_zero_point));
    t.acc_coef = (d->x_signed ? 0 : 128) - d->x_zero_point;
    t.x_scale = d->x_scale;
    t.out_scale = d->out_scale;
    t.zp_f = zp_f; t.lo_f = lo_f; t.hi_f = hi_f;
    t.ri = plan.row_slots;
    t.rpp = kCtThreads / t.ri;
    t.cx = (plan.HH + t.rpp - 1) / t.rpp;
    t.xstep = static_cast<uint32_t>(t.rpp) * static_cast<uint32_t>(s.W) * static_cast<uint32_t>(s.IC);
    t.xdstep = t.rpp * t.ri * 16;
    t.post = po;
    t.rcp_tw = 1.0f / static_cast<float>(plan.TW);
    t.rcp_ri = 1.0f / static_cast<float>(t.ri);
    t.rcp_pslots = 16.0f / static_cast<float>(plan.pitch);
    t.rcp_icb = 1.0f / static_cast<float>(t.icb);
    t.rcp_kw = 1.0f / static_cast<float>(s.KW);
    return launch_conv_tiles<MODE>(s, plan, t, stream);
  }

  XConv xs{};
  xs.x = static_cast<const uint8_t*>(d->x);
  xs.H = static_cast<int>(s.H); xs.W = static_cast<int>(s.W); xs.IC = static_cast<int>(s.IC);
  xs.OH = static_cast<int>(s.OH); xs.OW = static_cast<int>(s.OW);
  xs.KW = static_cast<int>(s.KW); xs.icb = static_cast<int>(s.ICgp / 16);
  xs.stride_h = static_cast<int>(s.sh); xs.stride_w = static_cast<int>(s.sw);
  xs.pad_h = static_cast<int>(s.ph); xs.pad_w = static_cast<int>(s.pw);
  xs.dil_h = static_cast<int>(s.dh); xs.dil_w = static_cast<int>(s.dw);
  xs.pad_word = 0x01010101u * static_cast<uint32_t>(static_cast<uint8_t>(d->x_zero_point));
  xs.step_w = static_cast<int>(s.dw * s.IC - 16 * (s.ICgp / 16));
  xs.step_h = static_cast<int>(s.dh * s.W * s.IC - s.KW * s.dw * s.IC);

  GemmArgs a{};
  a.M = rows;
  a.N = s.OCg;
  a.K = s.Kp;
  a.w_kchunks = s.KC;
  a.colsum = d->w_colsum;
  a.w_scales = d->w_scales;
  a.bias = d->bias;
  a.w_scale_stride = d->w_per_channel ? 1 : 0;
  a.x_xor = d->x_signed ? 0u : 0x80808080u;
  a.acc_coef = (d->x_signed ? 0 : 128) - d->x_zero_point;
  a.x_scale = d->x_scale;
  a.out_scale = d->out_scale;
  a.zp_f = zp_f; a.lo_f = lo_f; a.hi_f = hi_f;
  a.y = out;
  a.ldy = s.OC;
  a.post = po;
  // Few 64 x 64 tiles against a long K (3 x 3 layers over hundreds of channels on small images):
  // two or four wave groups per block walk a half or a quarter of K each, as in quantized::linear.
  // (pinned for tests: tile_cols = 1, 2 or 4 groups)
  const int64_t stages = ceil_div(s.Kp, kBK);
  const int64_t tiles64 = ceil_div(rows, 64) * ceil_div(s.OCg, 64) * s.groups;
  const bool small_tiles = !(s.OCg > 64 && rows >= 128 * 128) && rows < 256 * 256;
  int wave_groups = 1;
  if (forced == 2 && d->tile_cols > 0) {
    wave_groups = d->tile_cols;
    if (wave_groups != 1 && ((wave_groups != 2 && wave_groups != 4) || !small_tiles || stages % wave_groups != 0))
      return TMQ_ERR_UNSUPPORTED;
  } else if (small_tiles && stages >= 32) {
    // (four groups from 64 stages on: K = 4608, 200 tiles: 20.9 against 21.9 us with two, 56 tiles: 19.7 against
    // 20.4 us; K = 2304: level at 100 tiles, 27 against 20.7 us at 392)
    if (stages % 4 == 0 && stages >= 64 && tiles64 <= kFourGroupTiles)
      wave_groups = 4;
    else if (stages % 2 == 0 && tiles64 <= kTwoGroupTiles)
      wave_groups = 2;
  }
  // More 64 x 64 tiles than CUs, at most two per CU: the second round would run half empty.  Tiles of 128 rows
  // make it one round (256 -> 256 channels, 3 x 3, 14 x 14 at batch 32, 392 tiles: 19.7 -> 17.0 us; 512 -> 512 on
  // 7 x 7 at batch 64: 29.7 -> 28.6 us).  (pinned for tests: tile_rows = 128)
  bool tall_tiles = small_tiles && forced == 2 && d->tile_rows == 128 && wave_groups <= 2;
  if (!(forced == 2 && (d->tile_cols > 0 || d->tile_rows > 0)) && small_tiles && stages >= 32 && stages % 2 == 0 &&
      tiles64 > 256 && tiles64 <= 512) {
    tall_tiles = true;
    wave_groups = 2;
  }
  for (int64_t g = 0; g < s.groups; ++g) {
    a.w_packed = static_cast<const uint8_t*>(d->w_packed) + g * s.group_bytes;
    a.n_off = static_cast<int32_t>(g * s.OCg);
    xs.ic_off = static_cast<int>(g * s.ICg);
    if (s.OCg > 64 && rows >= 128 * 128)
      rc = launch_conv_gemm<128, 128, 2, 2, MODE>(a, xs, stream);
    else if (rows >= 256 * 256)
      rc = launch_conv_gemm<256, 64, 4, 1, MODE>(a, xs, stream);
    else if (tall_tiles && wave_groups == 2)
      rc = launch_conv_gemm<128, 64, 2, 2, MODE, 2>(a, xs, stream);
    else if (tall_tiles)
      rc = launch_conv_gemm<128, 64, 2, 2, MODE>(a, xs, stream);
    else if (wave_groups == 4)
      rc = launch_conv_gemm<64, 64, 2, 2, MODE, 4>(a, xs, stream);
    else if (wave_groups == 2)
      rc = launch_conv_gemm<64, 64, 2, 2, MODE, 2>(a, xs, stream);
    else
      rc = launch_conv_gemm<64, 64, 2, 2, MODE>(a, xs, stream);
    if (rc != TMQ_OK) return rc;
  }
  return TMQ_OK;
}

}  // namespace
}  // namespace tmq

using namespace tmq;

TMQ_EXPORT int64_t tmq_conv2d_packed_bytes(const tmq_conv2d_geom* g) {
  ConvShape s;
  if (make_shape(g, &s) != TMQ_OK) return 0;
  return s.groups * s.group_bytes + s.runs_bytes + s.taps_bytes;
}

TMQ_EXPORT int64_t tmq_conv2d_workspace_bytes(const tmq_conv2d_geom* g) {
  ConvShape s;
  if (make_shape(g, &s) != TMQ_OK) return 0;
  TilePlan tp;
  const int64_t need = patch_rows_bytes(*g, s, false);
  if (need > 0 && !(s.ICg % 16 == 0 && plan_tiles(s, false, 0, 0, &tp))) return need;
  return padded_input_bytes(*g, s, false);
}

TMQ_EXPORT int tmq_conv2d_out_hw(const tmq_conv2d_geom* g, int64_t* OH, int64_t* OW) {
  ConvShape s;
  const int rc = make_shape(g, &s);
  if (rc != TMQ_OK) return rc;
  if (OH != nullptr) *OH = s.OH;
  if (OW != nullptr) *OW = s.OW;
  return TMQ_OK;
}

TMQ_EXPORT int tmq_conv2d_prepack(const int8_t* w_ohwi, const tmq_conv2d_geom* g, void* packed,
                                  int32_t* colsum, tmq_stream_t stream) {
  ConvShape s;
  const int rc = make_shape(g, &s);
  if (rc != TMQ_OK) return rc;
  if (w_ohwi == nullptr || packed == nullptr || colsum == nullptr) return TMQ_ERR_INVALID_ARGUMENT;
  if (!aligned(packed, 16)) return TMQ_ERR_ALIGNMENT;
  hipStream_t hs = as_stream(stream);
  const int64_t total = s.groups * s.group_bytes / 16;
  int64_t blocks = ceil_div(total, 256);
  if (blocks > 0x7fffffff) return TMQ_ERR_UNSUPPORTED;
  conv_prepack_kernel<<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, hs>>>(
      w_ohwi, s, total, static_cast<uint8_t*>(packed));
  if (launch_status() != TMQ_OK) return TMQ_ERR_LAUNCH;
  if (s.runs_bytes > 0) {
    const int64_t slots = s.runs_bytes / 16;
    conv_prepack_runs_kernel<<<dim3(static_cast<unsigned>(ceil_div(slots, 256))), dim3(256), 0, hs>>>(
        w_ohwi, s, slots, static_cast<uint8_t*>(packed) + s.runs_off);
    if (launch_status() != TMQ_OK) return TMQ_ERR_LAUNCH;
  }
  if (s.taps_bytes > 0) {
    conv_prepack_taps_kernel<<<dim3(static_cast<unsigned>(ceil_div(s.taps_bytes, 256))), dim3(256), 0, hs>>>(
        w_ohwi, s.IC, s.KH, s.KW, s.taps_bytes, static_cast<uint8_t*>(packed) + s.runs_off);
    if (launch_status() != TMQ_OK) return TMQ_ERR_LAUNCH;
  }
  blocks = ceil_div(s.OC, 256 / kWave);
  conv_colsum_kernel<<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, hs>>>(
      w_ohwi, s.OC, s.KH * s.KW * s.ICgo, colsum);
  return launch_status();
}

TMQ_EXPORT int tmq_conv2d(const tmq_conv2d_desc* d, tmq_stream_t stream) {
  if (d == nullptr) return TMQ_ERR_INVALID_ARGUMENT;
  return d->out_signed ? run_conv<kOutS8>(d, nullptr, d->y, as_stream(stream))
                       : run_conv<kOutU8>(d, nullptr, d->y, as_stream(stream));
}

TMQ_EXPORT int tmq_conv2d_fused(const tmq_conv2d_desc* d, const tmq_conv2d_post* post,
                                tmq_stream_t stream) {
  if (d == nullptr || post == nullptr) return TMQ_ERR_INVALID_ARGUMENT;
  return d->out_signed ? run_conv<kOutS8>(d, post, d->y, as_stream(stream))
                       : run_conv<kOutU8>(d, post, d->y, as_stream(stream));
}

TMQ_EXPORT int tmq_conv2d_acc32(const tmq_conv2d_desc* d, int32_t* acc, tmq_stream_t stream) {
  if (d == nullptr) return TMQ_ERR_INVALID_ARGUMENT;
  return run_conv<kOutAcc32>(d, nullptr, acc, as_stream(stream));
}
