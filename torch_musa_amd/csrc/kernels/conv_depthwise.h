// Depthwise quantized::conv2d (one input and one output channel per group) on the vector
// ALU (gfx950), for any channel count that is a multiple of 4.
//
// A depthwise layer has no sum over channels: per output value KH * KW products.  The matrix
// pipe can only take it as a block-diagonal product that is mostly zeros (conv2d.hip merges
// the groups for that, where the channel count allows); here a lane owns four consecutive
// channels of one output column and walks a strip of output rows:
//   * the four channels' weights, one dword per tap from a [tap][channel] copy of the weight
//     that prepack appends to the packed one, stay in registers for the strip (3 x 3 and
//     5 x 5 kernels) -- for 3 x 3 already split into the four words (w & 0xff << 8 j) that
//     let v_dot4_i32_i8 deliver one channel's product each (the larger kernels split the
//     activation dword instead: one register per tap);
//   * per output value and tap one aligned dword of the NHWC input (the same four channels
//     of the tap's pixel; neighbouring lanes read neighbouring channels, then neighbouring
//     pixels: whole cache lines per wave), the activation zero point for taps outside the
//     image, the sign flip of unsigned activations, four dot products;
//   * requantisation of the four values as everywhere else, one dword store.
// The vector ALU is what the kernel runs on (some 100 instructions per 3 x 3 output dword, a
// third of them the dot products), then the latency of its loads: the strips are short where
// the problem is small (more waves in flight), at stride 1 the window keeps its rows in
// registers from one output row to the next, and the 3 x 3 and stride-1 loops ask for the next
// output row's taps before they work on the current one's.
// The x ^ 0x80 trick, the accumulator start value and the requantisation are those of
// gemm_i8_core.h.
#pragma once

#include "gemm_i8_core.h"

namespace tmq {

constexpr int kDwThreads = 256;
constexpr int kDwStripMax = 8;  // output rows per lane, at most

struct DepthwiseArgs {
  const uint8_t* x;        // NHWC, less than 2^31 bytes
  const uint8_t* w_taps;   // [KH * KW][C] bytes
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

// TAPS = KH * KW for the kernel sizes whose weights stay in registers (9: split, 25: whole
// dwords), 0: any kernel size, weights read at use.
//
// Addresses are 32-bit offsets from the tensors' bases and advance by additions.  A tap outside
// the image still loads -- from row 0 / column 0 of the lane's image in its place, so that no
// load sits behind a branch -- and the zero point replaces what came back.
template <int MODE, bool POST, int TAPS>
__global__ __launch_bounds__(kDwThreads) void conv_depthwise_kernel(DepthwiseArgs a) {
  const uint32_t b = blockIdx.x / a.blocks_per_image;
  const uint32_t q = (blockIdx.x - b * a.blocks_per_image) * kDwThreads + threadIdx.x;
  if (q >= a.per_image) return;
  const uint32_t C4 = static_cast<uint32_t>(a.C) >> 2;
  const uint32_t rest = q / C4, cg = q - rest * C4;
  const uint32_t strip = rest / static_cast<uint32_t>(a.OW), ow = rest - strip * static_cast<uint32_t>(a.OW);
  const uint32_t c = cg * 4;
  constexpr int kSide = TAPS == 9 ? 3 : TAPS == 25 ? 5 : 0;
  constexpr int kRegTaps = TAPS > 0 ? TAPS : 1;

  // ---- this lane's four channels: weights and constants
  uint32_t wsplit[TAPS == 9 ? 9 : 1][4];
  uint32_t wraw[TAPS == 25 ? 25 : 1];
  if constexpr (TAPS > 0) {
#pragma unroll
    for (int tp = 0; tp < TAPS; ++tp) {
      const uint32_t w4 = *reinterpret_cast<const uint32_t*>(a.w_taps + static_cast<uint32_t>(tp * a.C) + c);
      if constexpr (TAPS == 9) {
#pragma unroll
        for (int j = 0; j < 4; ++j) wsplit[tp][j] = w4 & (0xffu << (8 * j));
      } else {
        wraw[tp] = w4;
      }
    }
  }
  // (every load unconditional and independent of the others, so that they are in flight together:
  // without a bias the column sums stand in as something to read)
  int acc0[4];
  v4f mult = {0.f, 0.f, 0.f, 0.f}, bdiv = {0.f, 0.f, 0.f, 0.f};
  float bmul = 1.0f;
  {
    const bool has_bias = a.bias != nullptr;
    const float* const bias_src = has_bias ? a.bias : reinterpret_cast<const float*>(a.colsum);
    int cs[4];
    float wsc[4], bs[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      cs[j] = a.colsum[c + j];
      if constexpr (MODE != kOutAcc32) {
        wsc[j] = a.w_scales[(c + j) * a.w_scale_stride];
        bs[j] = bias_src[c + j];
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
    if constexpr (MODE != kOutAcc32) bmul = bias_mul(a.w_scale_stride == 0, a.x_scale * a.w_scales[0]);
  }

  const uint32_t row_bytes = static_cast<uint32_t>(a.W * a.C);
  const uint32_t lane_base = b * static_cast<uint32_t>(a.H) * row_bytes + c;
  const int iw0 = static_cast<int>(ow) * a.sw - a.pw;
  const int oh_first = static_cast<int>(strip) * a.strip;
  const int oh_end = oh_first + a.strip < a.OH ? oh_first + a.strip : a.OH;
  uint32_t yoff = ((b * static_cast<uint32_t>(a.OH) + oh_first) * static_cast<uint32_t>(a.OW) + ow) * static_cast<uint32_t>(a.C) + c;
  const uint32_t ystep = static_cast<uint32_t>(a.OW * a.C);
  const auto mac = [&](int (&acc)[4], uint32_t x4, const uint32_t (&ws)[4]) {
    const int xs = static_cast<int>(x4 ^ a.x_xor);
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[j] = __builtin_amdgcn_sdot4(xs, static_cast<int>(ws[j]), acc[j], false);
  };
  // (one weight dword against the activation's bytes one at a time: no per-tap weight words to keep)
  const auto mac_whole = [&](int (&acc)[4], uint32_t x4, uint32_t w4) {
    const uint32_t xs = x4 ^ a.x_xor;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      acc[j] = __builtin_amdgcn_sdot4(static_cast<int>(xs & (0xffu << (8 * j))), static_cast<int>(w4), acc[j], false);
  };
  const auto finish = [&](const int (&acc)[4]) {
    if constexpr (MODE == kOutAcc32) {
      *reinterpret_cast<v4i*>(static_cast<int32_t*>(a.y) + yoff) = v4i{acc[0], acc[1], acc[2], acc[3]};
    } else {
      uint32_t packed;
      if constexpr (POST) {
        const uint32_t accw = a.post.accum != nullptr ? *reinterpret_cast<const uint32_t*>(a.post.accum + yoff) : 0u;
        packed = requant4_post<MODE>(acc, bdiv, bmul, mult, a.post, accw, a.zp_f, a.lo_f, a.hi_f);
      } else {
        packed = requant4<MODE>(acc, bdiv, bmul, mult, a.zp_f, a.lo_f, a.hi_f);
      }
      *reinterpret_cast<uint32_t*>(static_cast<uint8_t*>(a.y) + yoff) = packed;
    }
    yoff += ystep;
  };

  if constexpr (TAPS > 0) {
    // the window's columns: fixed for the lane
    // (the masks, all ones where the tap is inside the image, choose by bits between what was
    // loaded and the zero point: a select would let the compiler move the load behind a branch)
    uint32_t col[kSide], col_in[kSide];
#pragma unroll
    for (int kw = 0; kw < kSide; ++kw) {
      const int iw = iw0 + kw * a.dw;
      col_in[kw] = static_cast<unsigned>(iw) < static_cast<unsigned>(a.W) ? ~0u : 0u;
      col[kw] = lane_base + (static_cast<uint32_t>(iw * a.C) & col_in[kw]);
    }
    // its rows: image row and byte position of that row, both advancing with the output row
    int ih[kSide], row_pos[kSide];
#pragma unroll
    for (int kh = 0; kh < kSide; ++kh) {
      ih[kh] = oh_first * a.sh - a.ph + kh * a.dh;
      row_pos[kh] = ih[kh] * static_cast<int>(row_bytes);
    }
    const int row_step = a.sh * static_cast<int>(row_bytes);
    // loads of one window (what comes back is not looked at here) ...
    uint32_t row_in[kSide];
    const auto request_window = [&](uint32_t (&raw)[kRegTaps]) {
#pragma unroll
      for (int kh = 0; kh < kSide; ++kh) {
        row_in[kh] = static_cast<unsigned>(ih[kh]) < static_cast<unsigned>(a.H) ? ~0u : 0u;
        const uint32_t rp = static_cast<uint32_t>(row_pos[kh]) & row_in[kh];
#pragma unroll
        for (int kw = 0; kw < kSide; ++kw) raw[kh * kSide + kw] = *reinterpret_cast<const uint32_t*>(a.x + (rp + col[kw]));
        ih[kh] += a.sh;
        row_pos[kh] += row_step;
      }
    };
    // ... and the window they make
    const auto settle_window = [&](const uint32_t (&raw)[kRegTaps], uint32_t (&xv)[kRegTaps]) {
#pragma unroll
      for (int kh = 0; kh < kSide; ++kh)
#pragma unroll
        for (int kw = 0; kw < kSide; ++kw) {
          const uint32_t in = row_in[kh] & col_in[kw];
          xv[kh * kSide + kw] = (raw[kh * kSide + kw] & in) | (a.pad_word & ~in);
        }
    };
    uint32_t xv[kRegTaps] = {}, raw[kRegTaps] = {};
    if (a.sh == 1 && a.dh == 1) {
      // Stride 1: the window moves down one image row per output row.  All but one of its rows
      // stay in registers (sign flip applied); the row that enters is asked for before the
      // current output row's arithmetic and looked at after it, also behind the strip's last row
      // (rows outside the image read row 0, and nothing uses them).  The fences keep the
      // compiler's scheduler from moving the loads down to their use.
      request_window(raw);
      settle_window(raw, xv);
#pragma unroll
      for (int tp = 0; tp < TAPS; ++tp) xv[tp] ^= a.x_xor;
      int ih_next = ih[kSide - 1], pos_next = row_pos[kSide - 1];  // (request_window advanced them by one row)
      uint32_t next[kSide] = {};
      for (int oh = oh_first; oh < oh_end; ++oh) {
        const uint32_t next_in = static_cast<unsigned>(ih_next) < static_cast<unsigned>(a.H) ? ~0u : 0u;
        const uint32_t rp = static_cast<uint32_t>(pos_next) & next_in;
#pragma unroll
        for (int kw = 0; kw < kSide; ++kw) next[kw] = *reinterpret_cast<const uint32_t*>(a.x + (rp + col[kw]));
        ih_next += 1;
        pos_next += static_cast<int>(row_bytes);
        __builtin_amdgcn_sched_barrier(0);
        int acc[4] = {acc0[0], acc0[1], acc0[2], acc0[3]};
#pragma unroll
        for (int tp = 0; tp < TAPS; ++tp)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            if constexpr (TAPS == 9)
              acc[j] = __builtin_amdgcn_sdot4(static_cast<int>(xv[tp]), static_cast<int>(wsplit[tp][j]), acc[j], false);
            else
              acc[j] = __builtin_amdgcn_sdot4(static_cast<int>(xv[tp] & (0xffu << (8 * j))), static_cast<int>(wraw[tp]), acc[j], false);
          }
        finish(acc);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int tp = 0; tp < TAPS - kSide; ++tp) xv[tp] = xv[tp + kSide];
#pragma unroll
        for (int kw = 0; kw < kSide; ++kw) {
          const uint32_t in = next_in & col_in[kw];
          xv[TAPS - kSide + kw] = ((next[kw] & in) | (a.pad_word & ~in)) ^ a.x_xor;
        }
      }
      return;
    }
    if constexpr (TAPS == 9) {
      request_window(raw);
      settle_window(raw, xv);
    }
    for (int oh = oh_first; oh < oh_end; ++oh) {
      int acc[4] = {acc0[0], acc0[1], acc0[2], acc0[3]};
      if constexpr (TAPS == 9) {
        // (the whole next window ahead, as above)
        request_window(raw);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int tp = 0; tp < 9; ++tp) mac(acc, xv[tp], wsplit[tp]);
        finish(acc);
        __builtin_amdgcn_sched_barrier(0);
        settle_window(raw, xv);
      } else {
        request_window(raw);
        settle_window(raw, xv);
#pragma unroll
        for (int tp = 0; tp < 25; ++tp) mac_whole(acc, xv[tp], wraw[tp]);
        finish(acc);
      }
    }
  } else {
    for (int oh = oh_first; oh < oh_end; ++oh) {
      int acc[4] = {acc0[0], acc0[1], acc0[2], acc0[3]};
      const int ih0 = oh * a.sh - a.ph;
      uint32_t wpos = c;
      for (int kh = 0; kh < a.KH; ++kh) {
        const int ihh = ih0 + kh * a.dh;
        const bool row_ok = static_cast<unsigned>(ihh) < static_cast<unsigned>(a.H);
        const uint32_t rp = lane_base + (row_ok ? static_cast<uint32_t>(ihh) * row_bytes : 0u);
        for (int kw = 0; kw < a.KW; ++kw, wpos += static_cast<uint32_t>(a.C)) {
          const int iw = iw0 + kw * a.dw;
          const uint32_t in = row_ok && static_cast<unsigned>(iw) < static_cast<unsigned>(a.W) ? ~0u : 0u;
          const uint32_t got = *reinterpret_cast<const uint32_t*>(a.x + (rp + (static_cast<uint32_t>(iw * a.C) & in)));
          const uint32_t w4 = *reinterpret_cast<const uint32_t*>(a.w_taps + wpos);
          mac_whole(acc, (got & in) | (a.pad_word & ~in), w4);
        }
      }
      finish(acc);
    }
  }
}

}  // namespace tmq
