// Depthwise quantized::conv2d (one input and one output channel per group) on the vector
// ALU (gfx950), for any channel count that is a multiple of 4.
//
// A depthwise layer has no sum over channels: per output value KH * KW products.  The matrix
// pipe can only take it as a block-diagonal product that is mostly zeros (conv2d.hip merges
// the groups for that, where the channel count allows); here a lane owns four consecutive
// channels of one output column and walks a strip of output rows.  For 3 x 3, 5 x 5 and 7 x 7
// kernels:
//   * per window row the lane loads one aligned dword per tap of the NHWC input (the same four
//     channels of the tap's pixel; neighbouring lanes read neighbouring channels, then
//     neighbouring pixels: whole cache lines per wave), puts the activation zero point where
//     the tap is outside the image, flips the sign of unsigned activations, and transposes
//     four pixels x four channels of bytes with eight v_perm_b32, so that a dword holds one
//     channel's bytes of four neighbouring taps;
//   * the weights come from a [channel][kernel row][taps padded to a multiple of 4] copy that
//     prepack appends to the packed weight, in the same shape, and stay in registers for the
//     strip: one v_dot4_i32_i8 then multiplies four taps of one channel -- a quarter of the
//     dot products that a dword of four channels against one tap would take;
//   * at stride 1 the window's rows stay in registers from one output row to the next (the
//     loop is unrolled over the kernel's height so that they never move), and the row that
//     enters is asked for before the current output row's arithmetic and looked at after it;
//   * requantisation of the four values as everywhere else, one dword store.
// Other kernel sizes take a plain loop over the taps.  What the kernel waits for besides the
// vector ALU is the latency of its loads: the strips are short where the problem is small
// (more waves in flight).  The x ^ 0x80 trick, the accumulator start value and the
// requantisation are those of gemm_i8_core.h.
#pragma once

#include "gemm_i8_core.h"

namespace tmq {

constexpr int kDwThreads = 256;
constexpr int kDwStripMax = 8;  // output rows per lane under 3 x 3 windows, at most (the host gives larger windows up to 14)

struct DepthwiseArgs {
  const uint8_t* x;        // NHWC, less than 2^31 bytes
  const uint8_t* w_taps;   // [C][KH][roundup(KW, 4)] bytes
  const int32_t* colsum;
  const float* w_scales;
  const float* bias;
  void* y;                 // less than 2^31 bytes
  uint32_t per_image;      // lanes with work per image: strips * OW * C / 4
  uint32_t blocks_per_image;
  int strip;               // output rows per lane
  int B, H, W, C, OH, OW, KH, KW;
  int sh, sw, ph, pw, dh, dw;
  int32_t w_scale_stride;
  uint32_t x_xor, pad_word;
  int32_t acc_coef;
  float x_scale, out_scale, zp_f, lo_f, hi_f;
  PostOps post;
};

// Four dwords of four bytes each, transposed: t[j] byte i = a[i] byte j.
__device__ __forceinline__ void transpose_4x4_bytes(uint32_t a0, uint32_t a1, uint32_t a2, uint32_t a3, uint32_t (&t)[4]) {
  // v_perm_b32 D, S0, S1, sel: byte i of D = byte sel[i] of {S0, S1} (S1 the low dword)
  const uint32_t lo01 = __builtin_amdgcn_perm(a1, a0, 0x05010400u);  // a0.0 a1.0 a0.1 a1.1
  const uint32_t hi01 = __builtin_amdgcn_perm(a1, a0, 0x07030602u);  // a0.2 a1.2 a0.3 a1.3
  const uint32_t lo23 = __builtin_amdgcn_perm(a3, a2, 0x05010400u);
  const uint32_t hi23 = __builtin_amdgcn_perm(a3, a2, 0x07030602u);
  t[0] = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);
  t[1] = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
  t[2] = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);
  t[3] = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u);
}

// KS = the side of a square 3 x 3 / 5 x 5 / 7 x 7 kernel, 0: any kernel size.
//
// Addresses are 32-bit offsets from the tensors' bases and advance by additions.  A tap outside
// the image still loads -- from row 0 / column 0 of the lane's image in its place, so that no
// load sits behind a branch -- and the zero point replaces what came back, chosen by bits (a
// select would let the compiler move the load behind a branch again).
template <int MODE, bool POST, int KS>
__global__ __launch_bounds__(kDwThreads, KS == 7 && !POST ? 3 : 1) void conv_depthwise_kernel(DepthwiseArgs a) {
  const uint32_t b = blockIdx.x / a.blocks_per_image;
  const uint32_t q0 = (blockIdx.x - b * a.blocks_per_image) * kDwThreads, q = q0 + threadIdx.x;
  const uint32_t C4 = static_cast<uint32_t>(a.C) >> 2;
  const uint32_t rest = q / C4, cg = q - rest * C4;
  const uint32_t strip = rest / static_cast<uint32_t>(a.OW), ow = rest - strip * static_cast<uint32_t>(a.OW);
  const uint32_t c = cg * 4;
  constexpr int kSide = KS > 0 ? KS : 1;
  constexpr int kGroups = (kSide + 3) / 4;  // dwords of four taps per kernel row

  // ---- the channels' constants: accumulator start value, requantisation multiplier, bias term.
  // (every load unconditional and independent of the others, so that they are in flight together:
  // without a bias the column sums stand in as something to read)
  const auto channel_constants = [&](uint32_t ch, int (&acc0)[4], v4f& mult, v4f& bdiv) {
    const bool has_bias = a.bias != nullptr;
    const float* const bias_src = has_bias ? a.bias : reinterpret_cast<const float*>(a.colsum);
    int cs[4];
    float wsc[4] = {0.f, 0.f, 0.f, 0.f}, bs[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      cs[j] = a.colsum[ch + j];
      if constexpr (MODE != kOutAcc32) {
        wsc[j] = a.w_scales[(ch + j) * a.w_scale_stride];
        bs[j] = bias_src[ch + j];
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      acc0[j] = a.acc_coef * cs[j];
      if constexpr (MODE != kOutAcc32) {
        const float atw = a.x_scale * wsc[j];
        mult[j] = atw / a.out_scale;
        bdiv[j] = has_bias ? bias_term(a.w_scale_stride == 0, bs[j], atw) : 0.f;
      }
    }
  };
  int acc0[4];
  v4f mult = {0.f, 0.f, 0.f, 0.f}, bdiv = {0.f, 0.f, 0.f, 0.f};
  // With at most a block's worth of channel groups, the lanes of a block share few of them: the
  // first C / 4 lanes work the constants out (a dozen divisions per group), the others read them.
  __shared__ int s_acc0[kDwThreads * 4];
  __shared__ float s_mult[kDwThreads * 4], s_bdiv[kDwThreads * 4];
  if (C4 <= kDwThreads) {
    if (threadIdx.x < C4) {
      const uint32_t g = (q0 + threadIdx.x) % C4;
      int a0[4];
      v4f m = {0.f, 0.f, 0.f, 0.f}, bd = {0.f, 0.f, 0.f, 0.f};
      channel_constants(g * 4, a0, m, bd);
      *reinterpret_cast<v4i*>(&s_acc0[g * 4]) = v4i{a0[0], a0[1], a0[2], a0[3]};
      *reinterpret_cast<v4f*>(&s_mult[g * 4]) = m;
      *reinterpret_cast<v4f*>(&s_bdiv[g * 4]) = bd;
    }
    __syncthreads();
    if (q >= a.per_image) return;
    const v4i a0 = *reinterpret_cast<const v4i*>(&s_acc0[cg * 4]);
    acc0[0] = a0[0]; acc0[1] = a0[1]; acc0[2] = a0[2]; acc0[3] = a0[3];
    mult = *reinterpret_cast<const v4f*>(&s_mult[cg * 4]);
    bdiv = *reinterpret_cast<const v4f*>(&s_bdiv[cg * 4]);
  } else {
    if (q >= a.per_image) return;
    channel_constants(c, acc0, mult, bdiv);
  }
  float bmul = 1.0f;
  if constexpr (MODE != kOutAcc32) bmul = bias_mul(a.w_scale_stride == 0, a.x_scale * a.w_scales[0]);

  // ---- this lane's four channels' weights
  uint32_t wreg[kSide][4][kGroups];
  if constexpr (KS > 0) {
    const uint32_t* const wl = reinterpret_cast<const uint32_t*>(a.w_taps) + c * (KS * kGroups);
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int kh = 0; kh < KS; ++kh)
#pragma unroll
        for (int g = 0; g < kGroups; ++g) wreg[kh][j][g] = wl[(j * KS + kh) * kGroups + g];
  }

  const uint32_t row_bytes = static_cast<uint32_t>(a.W * a.C);
  const uint32_t lane_base = b * static_cast<uint32_t>(a.H) * row_bytes + c;
  const int iw0 = static_cast<int>(ow) * a.sw - a.pw;
  const int oh_first = static_cast<int>(strip) * a.strip;
  const int oh_end = oh_first + a.strip < a.OH ? oh_first + a.strip : a.OH;
  uint32_t yoff = ((b * static_cast<uint32_t>(a.OH) + oh_first) * static_cast<uint32_t>(a.OW) + ow) * static_cast<uint32_t>(a.C) + c;
  const uint32_t ystep = static_cast<uint32_t>(a.OW * a.C);
  const auto finish = [&](const int (&acc)[4]) {
    if constexpr (MODE == kOutAcc32) {
      *reinterpret_cast<v4i*>(static_cast<int32_t*>(a.y) + yoff) = v4i{acc[0], acc[1], acc[2], acc[3]};
    } else {
      uint32_t packed;
      if constexpr (POST) {
        const uint32_t accw = a.post.accum != nullptr ? *reinterpret_cast<const uint32_t*>(a.post.accum + yoff) : 0u;
        packed = requant4_post<MODE>(acc, bdiv, bmul, mult, a.post, accw, a.zp_f, a.lo_f, a.hi_f);
      } else {
        packed = requant4<MODE, true, 2>(acc, bdiv, bmul, mult, a.zp_f, a.lo_f, a.hi_f);  // (tested here: 11.8 -> 10.8 us where it holds, level where not)
      }
      *reinterpret_cast<uint32_t*>(static_cast<uint8_t*>(a.y) + yoff) = packed;
    }
    yoff += ystep;
  };

  if constexpr (KS > 0) {
    // the window's columns: fixed for the lane (masks: all ones where the tap is inside the image)
    uint32_t col[KS], col_in[KS];
#pragma unroll
    for (int kw = 0; kw < KS; ++kw) {
      const int iw = iw0 + kw * a.dw;
      col_in[kw] = static_cast<unsigned>(iw) < static_cast<unsigned>(a.W) ? ~0u : 0u;
      col[kw] = lane_base + (static_cast<uint32_t>(iw * a.C) & col_in[kw]);
    }
    // loads of one window row (what comes back is not looked at here) ...
    const auto request_row = [&](int ih, int pos, uint32_t (&raw)[KS], uint32_t& row_in) {
      row_in = static_cast<unsigned>(ih) < static_cast<unsigned>(a.H) ? ~0u : 0u;
      const uint32_t rp = static_cast<uint32_t>(pos) & row_in;
#pragma unroll
      for (int kw = 0; kw < KS; ++kw) raw[kw] = *reinterpret_cast<const uint32_t*>(a.x + (rp + col[kw]));
    };
    // ... and the row they make: [channel][group of four taps]
    const auto settle_row = [&](const uint32_t (&raw)[KS], uint32_t row_in, uint32_t (&row)[4][kGroups]) {
      uint32_t v[4 * kGroups];
#pragma unroll
      for (int kw = 0; kw < 4 * kGroups; ++kw) {
        if (kw < KS) {
          const uint32_t in = row_in & col_in[kw];
          v[kw] = ((raw[kw] & in) | (a.pad_word & ~in)) ^ a.x_xor;
        } else {
          v[kw] = 0u;  // (against zero weights)
        }
      }
#pragma unroll
      for (int g = 0; g < kGroups; ++g) {
        uint32_t t[4];
        transpose_4x4_bytes(v[4 * g], v[4 * g + 1], v[4 * g + 2], v[4 * g + 3], t);
#pragma unroll
        for (int j = 0; j < 4; ++j) row[j][g] = t[j];
      }
    };
    uint32_t win[KS][4][kGroups];
    // window row kh of the current output row is win[(kh + ROT) % KS]
    const auto window_sums = [&](auto rot_tag, int (&acc)[4]) {
      constexpr int ROT = decltype(rot_tag)::value;
#pragma unroll
      for (int kh = 0; kh < KS; ++kh)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int g = 0; g < kGroups; ++g)
            acc[j] = __builtin_amdgcn_sdot4(static_cast<int>(win[(kh + ROT) % KS][j][g]), static_cast<int>(wreg[kh][j][g]), acc[j], false);
    };
    const int ih_first = oh_first * a.sh - a.ph;
    if (a.sh == 1 && a.dh == 1) {
      // Stride 1: the window moves down one image row per output row.  The fences keep the
      // compiler's scheduler from moving the entering row's loads down to their use.
      {
        uint32_t raw[KS][KS], row_in[KS];
#pragma unroll
        for (int kh = 0; kh < KS; ++kh) request_row(ih_first + kh, (ih_first + kh) * static_cast<int>(row_bytes), raw[kh], row_in[kh]);
#pragma unroll
        for (int kh = 0; kh < KS; ++kh) settle_row(raw[kh], row_in[kh], win[kh]);
      }
      int ih_next = ih_first + KS, pos_next = ih_next * static_cast<int>(row_bytes);
      int oh = oh_first;
      // one output row; the entering row (also asked for behind the strip's last row: rows outside the
      // image read row 0, and nothing uses them) takes the place of the window's row 0
      const auto step = [&](auto rot_tag) {
        constexpr int ROT = decltype(rot_tag)::value;
        uint32_t raw[KS], row_in;
        request_row(ih_next, pos_next, raw, row_in);
        ih_next += 1;
        pos_next += static_cast<int>(row_bytes);
        __builtin_amdgcn_sched_barrier(0);
        int acc[4] = {acc0[0], acc0[1], acc0[2], acc0[3]};
        window_sums(rot_tag, acc);
        finish(acc);
        __builtin_amdgcn_sched_barrier(0);
        settle_row(raw, row_in, win[ROT]);
        ++oh;
      };
      while (true) {
        if (oh >= oh_end) return;
        step(std::integral_constant<int, 0>{});
        if (oh >= oh_end) return;
        step(std::integral_constant<int, 1 % KS>{});
        if (oh >= oh_end) return;
        step(std::integral_constant<int, 2 % KS>{});
        if constexpr (KS >= 5) {
          if (oh >= oh_end) return;
          step(std::integral_constant<int, 3 % KS>{});
          if (oh >= oh_end) return;
          step(std::integral_constant<int, 4 % KS>{});
        }
        if constexpr (KS >= 7) {
          if (oh >= oh_end) return;
          step(std::integral_constant<int, 5 % KS>{});
          if (oh >= oh_end) return;
          step(std::integral_constant<int, 6 % KS>{});
        }
      }
    } else {
      // any stride and dilation: the whole window per output row
      for (int oh = oh_first; oh < oh_end; ++oh) {
        const int ih0 = oh * a.sh - a.ph;
        uint32_t raw[KS][KS], row_in[KS];
#pragma unroll
        for (int kh = 0; kh < KS; ++kh) request_row(ih0 + kh * a.dh, (ih0 + kh * a.dh) * static_cast<int>(row_bytes), raw[kh], row_in[kh]);
#pragma unroll
        for (int kh = 0; kh < KS; ++kh) settle_row(raw[kh], row_in[kh], win[kh]);
        int acc[4] = {acc0[0], acc0[1], acc0[2], acc0[3]};
        window_sums(std::integral_constant<int, 0>{}, acc);
        finish(acc);
      }
    }
  } else {
    const int kwp = (a.KW + 3) & ~3;
    for (int oh = oh_first; oh < oh_end; ++oh) {
      int acc[4] = {acc0[0], acc0[1], acc0[2], acc0[3]};
      const int ih0 = oh * a.sh - a.ph;
      for (int kh = 0; kh < a.KH; ++kh) {
        const int ihh = ih0 + kh * a.dh;
        const bool row_ok = static_cast<unsigned>(ihh) < static_cast<unsigned>(a.H);
        const uint32_t rp = lane_base + (row_ok ? static_cast<uint32_t>(ihh) * row_bytes : 0u);
        for (int kw = 0; kw < a.KW; ++kw) {
          const int iw = iw0 + kw * a.dw;
          const uint32_t in = row_ok && static_cast<unsigned>(iw) < static_cast<unsigned>(a.W) ? ~0u : 0u;
          const uint32_t got = *reinterpret_cast<const uint32_t*>(a.x + (rp + (static_cast<uint32_t>(iw * a.C) & in)));
          const uint32_t xs = ((got & in) | (a.pad_word & ~in)) ^ a.x_xor;
          const uint8_t* const wt = a.w_taps + static_cast<uint32_t>((static_cast<int>(c) * a.KH + kh) * kwp + kw);
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            // (one channel's byte of the activation dword against that channel's weight, both in byte j)
            const uint32_t wj = static_cast<uint32_t>(wt[static_cast<uint32_t>(j * a.KH * kwp)]) << (8 * j);
            acc[j] = __builtin_amdgcn_sdot4(static_cast<int>(xs & (0xffu << (8 * j))), static_cast<int>(wj), acc[j], false);
          }
        }
      }
      finish(acc);
    }
  }
}

}  // namespace tmq
