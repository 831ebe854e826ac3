// quantized::conv2d for a few input channels (gfx950): the first layer of an image
// network (3 -> 64 channels, 7 x 7, stride 2), pointwise layers whose channel count is
// no multiple of 16, one group, no dilation.
//
// With so few channels a 16-byte k-chunk of the MFMA cannot be "16 channels of one
// pixel".  In NHWC the KW taps of one kernel row are KW * IC *contiguous* bytes of an
// image row, so k is ordered (kh, run) with run = the RL = KW * IC bytes of a kernel
// row, padded to RP = a multiple of 16 with zero weights: the bytes an operand picks
// up past the run's end are multiplied by zero.  K = KH * RP is at most 256 here, the
// weights of 64 output channels stay in registers (16 operands of
// v_mfma_i32_16x16x64_i8) for the whole launch.
//
// A block of four waves walks tiles of TR x TW output pixels of one image:
//   * it stages the (TR - 1) * stride + KH image rows the tile needs, as bytes, positions
//     outside the image as the activation zero point, sign flip of unsigned activations
//     applied.  The copy runs in aligned words of memory whatever the address of an image
//     row: each staged row starts 0 ... 3 bytes before the tile's first byte of its row;
//   * a wave takes 16 output pixels of one output row at a time: the operand of pixel
//     p, kernel row kh, 16-byte piece c of the run is the 16 bytes at
//       row (orow * stride + kh), byte p * stride * IC + 16 c
//     of the staged rows -- any byte alignment, so it is put together from five aligned
//     words with v_alignbyte_b32;
//   * operand roles: weights are the rows (i), pixels the columns (j) of the MFMA,
//     D[i][j]: lane l, register r -> i = 4 (l / 16) + r, j = l % 16.  Row i of channel
//     tile nt is channel 16 (i / 4) + 4 nt + i % 4, so that a lane ends up with 16
//     consecutive channels of one pixel: one 16-byte store.
// The x ^ 0x80 trick, the accumulator start value and the requantisation are those of
// gemm_i8_core.h.
#pragma once

#include "gemm_i8_core.h"

namespace tmq {

constexpr int kCrThreads = 256;
constexpr int kCrWaves = kCrThreads / kWave;
constexpr int kCrBN = 64;      // output channels per block (grid y)
constexpr int kCrMaxKS = 4;    // k-steps of 64 bytes
constexpr int kCrStage = 8;    // staged words per thread and tile: 8 KB of image rows

struct ConvRunArgs {
  const uint8_t* x;          // NHWC
  const uint8_t* w_packed;   // the packed layout of conv2d.hip: [16 channels][k-chunk][channel][16 B], taps of ICp bytes
  const int32_t* colsum;
  const float* w_scales;
  const float* bias;
  void* y;
  int64_t w_kchunks;
  int32_t tiles;             // B * tiles_h * tiles_w
  int B, H, W, IC, OH, OW, OC, KH, KW;
  int sh, sw, ph, pw;
  int ICp;                   // bytes of one tap in the packed weight (IC rounded up to 16)
  int RL, RP, KS;            // run bytes, padded run bytes, k-steps (KH * RP <= 64 KS)
  int TR, TW, mtw;           // output rows and columns per tile, 16-pixel pieces per tile row
  int rows_in, pitch;        // staged image rows, LDS bytes per staged row (multiple of 4)
  int tiles_h, tiles_w;
  int vec;                   // 16-byte (int32 mode: per 4 channels) stores are aligned
  int32_t w_scale_stride;
  uint32_t x_xor, pad_word;  // pad_word: the activation zero point in 4 bytes, before the xor
  int32_t acc_coef;
  float x_scale, out_scale, zp_f, lo_f, hi_f;
  float rcp_p4;              // 4 / pitch
  PostOps post;
};

template <int MODE, bool POST>
__global__ __launch_bounds__(kCrThreads, 3) void conv_runs_kernel(ConvRunArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  __shared__ __attribute__((aligned(16))) int s_acc0[kCrBN];
  __shared__ __attribute__((aligned(16))) float s_mult[kCrBN];
  __shared__ __attribute__((aligned(16))) float s_bdiv[kCrBN];

  const int t = threadIdx.x, lane = t % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(t / kWave);
  const int pj = lane & 15, pq = lane >> 4;
  const int n0 = static_cast<int>(blockIdx.y) * kCrBN;
  const int KS = a.KS;
  uint8_t* const sW = lds;                  // [channel tile nt][k-step][lane][16 B]
  uint8_t* const sX = lds + KS * 4096;      // staged image rows

  // ---- the weight operands of this block's 64 channels, once
  for (int item = t; item < kCrBN * 4 * KS; item += kCrThreads) {
    const int nl = item & 63, kc = item >> 6;      // channel of the tile, 16-byte piece of k
    const int n = n0 + nl;
    const int koff = kc * 16;
    const int kh = koff / a.RP, ro = koff - kh * a.RP;
    // sixteen byte loads without a condition (invalid positions read the row's first byte
    // and are masked): all of them are in flight together
    const bool row_ok = n < a.OC && kh < a.KH;
    const uint8_t* const wrow =
        a.w_packed + (row_ok ? static_cast<int64_t>(n >> 4) * a.w_kchunks * 256 + (n & 15) * 16 : 0);
    uint32_t bytes[16];
    {
      int kw = ro / a.IC, ic = ro - kw * a.IC;
#pragma unroll
      for (int bb = 0; bb < 16; ++bb) {
        const bool ok = row_ok && ro + bb < a.RL;
        const int kp = ok ? (kh * a.KW + kw) * a.ICp + ic : 0;
        const uint32_t v = wrow[(kp >> 4) * 256 + (kp & 15)];
        bytes[bb] = ok ? v : 0u;
        if (++ic == a.IC) {
          ic = 0;
          ++kw;
        }
      }
    }
    uint32_t words[4];
#pragma unroll
    for (int w4 = 0; w4 < 4; ++w4)
      words[w4] = bytes[4 * w4] | (bytes[4 * w4 + 1] << 8) | (bytes[4 * w4 + 2] << 16) | (bytes[4 * w4 + 3] << 24);
    const int i = 4 * (nl >> 4) + (nl & 3), nt = (nl & 15) >> 2;
    *reinterpret_cast<v4i*>(sW + (((nt * KS + (kc >> 2)) * kWave) + (kc & 3) * 16 + i) * 16) =
        v4i{static_cast<int>(words[0]), static_cast<int>(words[1]), static_cast<int>(words[2]),
            static_cast<int>(words[3])};
  }
  if (t < kCrBN) {
    const int n = n0 + t;
    int acc0 = 0;
    float mult = 0.f, bdiv = 0.f;
    if (n < a.OC) {
      acc0 = a.acc_coef * a.colsum[n];
      if constexpr (MODE != kOutAcc32) {
        const float atw = a.x_scale * a.w_scales[n * a.w_scale_stride];
        mult = atw / a.out_scale;
        bdiv = a.bias != nullptr ? bias_term(a.w_scale_stride == 0, a.bias[n], atw) : 0.f;
      }
    }
    s_acc0[t] = acc0;
    s_mult[t] = mult;
    s_bdiv[t] = bdiv;
  }
  __syncthreads();
  v4i wreg[4][kCrMaxKS];
#pragma unroll
  for (int nt = 0; nt < 4; ++nt)
#pragma unroll
    for (int ks = 0; ks < kCrMaxKS; ++ks)
      wreg[nt][ks] = ks < KS ? ld16(sW + ((nt * KS + ks) * kWave + lane) * 16) : v4i{0, 0, 0, 0};
  // this lane's piece of every k-step: staged row and byte inside the run
  int lk[kCrMaxKS];  // (a multiple of 4) | the row's share of the alignment shift, (kh * (row bytes % 4)) % 4
#pragma unroll
  for (int ks = 0; ks < kCrMaxKS; ++ks) {
    const int koff = ks * 64 + pq * 16;
    int kh = koff / a.RP, ro = koff - kh * a.RP;
    if (kh >= a.KH) {  // past the last kernel row: zero weights, any staged bytes
      kh = a.KH - 1;
      ro = 0;
    }
    lk[ks] = (kh * a.pitch + ro) | ((kh * (a.W * a.IC)) & 3);
  }
  float bmul = 1.0f;
  if constexpr (MODE != kOutAcc32) bmul = bias_mul(a.w_scale_stride == 0, a.x_scale * a.w_scales[0]);

  const int row_bytes = a.W * a.IC;
  const int P4 = a.pitch >> 2, stage_words = a.rows_in * P4;
  const int tile_mt = a.TR * a.mtw;
  // The staged rows of a tile pass through registers: kCrStage words per thread (the host
  // sizes the tiles for that), requested one tile ahead, so that they arrive while the
  // tile in hand is multiplied.  Word u of thread t is word t + 256 u of the staged rows:
  // its row and place in the row are the same for every tile.
  int spos[kCrStage];  // row << 16 | byte in the row; -1: no such word
#pragma unroll
  for (int u = 0; u < kCrStage; ++u) {
    const int idx = t + u * kCrThreads;
    int r = static_cast<int>(static_cast<float>(idx) * a.rcp_p4);
    int p4 = idx - r * P4;
    if (p4 < 0) {
      --r;
      p4 += P4;
    } else if (p4 >= P4) {
      ++r;
      p4 -= P4;
    }
    spos[u] = idx < stage_words ? (r << 16 | 4 * p4) : -1;
  }
  uint32_t pre[kCrStage];
  // Staged row r of a tile starts shift(r) = (c0 + r * (row bytes % 4)) % 4 bytes before the
  // tile's first byte of that image row, so that every staged word is an aligned word of
  // memory: LDS byte q of the row is image-row byte iwb0 - shift(r) + q.
  struct TilePos {
    int b, oh0, ow0, c0;
    int ih0, iwb0;        // image row and byte in the row of the tile's first staged byte (before the shift)
    int64_t first;        // the same as a byte offset into the tensor
    int edge;             // some staged word may reach outside the tensor
  };
  const int rb3 = row_bytes & 3;
  const int64_t x_bytes = static_cast<int64_t>(a.B) * a.H * row_bytes;
  auto tile_pos = [&](uint32_t tile) {
    TilePos tp;
    const uint32_t trb = tile / static_cast<uint32_t>(a.tiles_w);
    const int tcol = static_cast<int>(tile - trb * static_cast<uint32_t>(a.tiles_w));
    tp.b = static_cast<int>(trb / static_cast<uint32_t>(a.tiles_h));
    const int trow = static_cast<int>(trb) - tp.b * a.tiles_h;
    tp.oh0 = trow * a.TR;
    tp.ow0 = tcol * a.TW;
    tp.ih0 = tp.oh0 * a.sh - a.ph;
    tp.iwb0 = (tp.ow0 * a.sw - a.pw) * a.IC;
    tp.first = (static_cast<int64_t>(tp.b) * a.H + tp.ih0) * row_bytes + tp.iwb0;
    tp.c0 = static_cast<int>((reinterpret_cast<uintptr_t>(a.x) + static_cast<uintptr_t>(tp.first)) & 3);
    tp.edge = tp.first < 4 || tp.first + static_cast<int64_t>(a.rows_in) * row_bytes + a.pitch + 4 > x_bytes;
    return tp;
  };
  // The loads only: whole aligned words, also where a word hangs over the end of its image
  // row into the next one (store_tile masks those bytes); nothing here uses a loaded value,
  // so nothing waits.  Only in the first and the last tiles of the tensor can a word reach
  // outside it; those tiles check every byte.
  auto request = [&](const TilePos& tp) {
    const uint8_t* const base = a.x + (tp.first - 4);  // (an address to count from, not one to load from)
#pragma unroll
    for (int u = 0; u < kCrStage; ++u) {
      pre[u] = 0;
      if (u * kCrThreads >= stage_words) continue;  // (the same for the whole block)
      const int r = spos[u] >> 16, q = spos[u] & 0xffff;
      const int shift = (tp.c0 + r * rb3) & 3;
      const int colb = tp.iwb0 - shift + q;
      const bool ok = spos[u] >= 0 && static_cast<unsigned>(tp.ih0 + r) < static_cast<unsigned>(a.H) &&
                      static_cast<unsigned>(colb + 3) < static_cast<unsigned>(row_bytes + 3);
      const uint32_t off = static_cast<uint32_t>(r * row_bytes + q - shift + 4);
      if (ok) {
        if (!tp.edge) {
          pre[u] = *reinterpret_cast<const uint32_t*>(base + off);
        } else {
          const int64_t rel = tp.first - 4 + static_cast<int64_t>(off);
          uint32_t word = 0;
#pragma unroll
          for (int jj = 0; jj < 4; ++jj)
            if (rel + jj >= 0 && rel + jj < x_bytes) word |= static_cast<uint32_t>(a.x[rel + jj]) << (8 * jj);
          pre[u] = word;
        }
      }
    }
  };
  // Bytes outside the image (rows above and below, columns left and right of the row) become
  // the activation zero point; then the sign flip, and into LDS.
  auto store_tile = [&](const TilePos& tp) {
#pragma unroll
    for (int u = 0; u < kCrStage; ++u) {
      if (u * kCrThreads >= stage_words || spos[u] < 0) continue;
      const int r = spos[u] >> 16, q = spos[u] & 0xffff;
      const int colb = tp.iwb0 - ((tp.c0 + r * rb3) & 3) + q;
      uint32_t word = pre[u];
      const bool row_in = static_cast<unsigned>(tp.ih0 + r) < static_cast<unsigned>(a.H);
      if (!(row_in && colb >= 0 && colb + 3 < row_bytes)) {  // (the few words at the image's edges)
        uint32_t keep = 0;
        if (row_in) {
#pragma unroll
          for (int jj = 0; jj < 4; ++jj)
            if (static_cast<unsigned>(colb + jj) < static_cast<unsigned>(row_bytes)) keep |= 0xffu << (8 * jj);
        }
        word = (word & keep) | (a.pad_word & ~keep);
      }
      *reinterpret_cast<uint32_t*>(sX + r * a.pitch + q) = word ^ a.x_xor;
    }
  };
  TilePos cur{};
  if (static_cast<int>(blockIdx.x) < a.tiles) {
    cur = tile_pos(blockIdx.x);
    request(cur);
  }
  for (int tile = blockIdx.x; tile < a.tiles; tile += gridDim.x) {
    const int b = cur.b, oh0 = cur.oh0, ow0 = cur.ow0, c0 = cur.c0;
    // ---- the staged rows of this tile into LDS, the next tile's on their way
    store_tile(cur);
    __syncthreads();
    if (tile + static_cast<int>(gridDim.x) < a.tiles) {
      cur = tile_pos(static_cast<uint32_t>(tile) + gridDim.x);
      request(cur);
    }

    // ---- multiply: 16 pixels of one output row per wave and turn
    const int tw_valid = a.OW - ow0 < a.TW ? a.OW - ow0 : a.TW;
    const int th_valid = a.OH - oh0 < a.TR ? a.OH - oh0 : a.TR;
    int orow = 0, mcol = wave;  // this wave's piece: row of the tile, 16-pixel piece of the row
    for (int mt = wave; mt < tile_mt; mt += kCrWaves, mcol += kCrWaves) {
      while (mcol >= a.mtw) {
        mcol -= a.mtw;
        ++orow;
      }
      if (orow >= th_valid || mcol * 16 >= tw_valid) continue;  // (the same for the whole wave)
      const int pcol = mcol * 16 + pj;
      const int pc = pcol < tw_valid ? pcol : tw_valid - 1;
      const int base = orow * a.sh * a.pitch + pc * a.sw * a.IC;
      const int c0r = c0 + orow * a.sh * rb3;  // alignment shift of staged row orow * stride, before the % 4
      v4i acc[4];  // start: the zero point's share, acc_coef * colsum
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) acc[nt] = *reinterpret_cast<const v4i*>(&s_acc0[16 * pq + 4 * nt]);
#pragma unroll
      for (int ks = 0; ks < kCrMaxKS; ++ks) {
        if (ks < KS) {
          const int addr = base + (lk[ks] & ~3) + ((c0r + lk[ks]) & 3);
          const uint32_t* const src = reinterpret_cast<const uint32_t*>(sX + (addr & ~3));
          const uint32_t sb = static_cast<uint32_t>(addr & 3);
          const uint32_t d0 = src[0], d1 = src[1], d2 = src[2], d3 = src[3], d4 = src[4];
          const v4i xv = {static_cast<int>(__builtin_amdgcn_alignbyte(d1, d0, sb)),
                          static_cast<int>(__builtin_amdgcn_alignbyte(d2, d1, sb)),
                          static_cast<int>(__builtin_amdgcn_alignbyte(d3, d2, sb)),
                          static_cast<int>(__builtin_amdgcn_alignbyte(d4, d3, sb))};
#pragma unroll
          for (int nt = 0; nt < 4; ++nt)
            acc[nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wreg[nt][ks], xv, acc[nt], 0, 0, 0);
        }
      }
      // ---- requantise and store: this lane has channels n0 + 16 pq .. + 15 of pixel pj
      if (pcol >= tw_valid) continue;
      const int64_t opix = (static_cast<int64_t>(b) * a.OH + oh0 + orow) * a.OW + ow0 + pcol;
      const int cb = n0 + 16 * pq;
      if (cb >= a.OC) continue;
      const int64_t off = opix * a.OC + cb;
      uint32_t packed[4];
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) {
        const int cl = 16 * pq + 4 * nt;
        const int raw[4] = {acc[nt][0], acc[nt][1], acc[nt][2], acc[nt][3]};
        if constexpr (MODE == kOutAcc32) {
          int32_t* const dst = static_cast<int32_t*>(a.y) + off + 4 * nt;
          if (a.vec && cb + 4 * nt + 4 <= a.OC) {
            *reinterpret_cast<v4i*>(dst) = v4i{raw[0], raw[1], raw[2], raw[3]};
          } else {
#pragma unroll
            for (int r = 0; r < 4; ++r)
              if (cb + 4 * nt + r < a.OC) dst[r] = raw[r];
          }
        } else {
          const v4f mult = *reinterpret_cast<const v4f*>(&s_mult[cl]);
          const v4f bdiv = *reinterpret_cast<const v4f*>(&s_bdiv[cl]);
          if constexpr (POST) {
            const int left = a.OC - (cb + 4 * nt);
            const int nvalid = left < 0 ? 0 : (left < 4 ? left : 4);
            const uint32_t accw =
                a.post.accum != nullptr && nvalid > 0 ? load_accum4(a.post, off + 4 * nt, nvalid) : 0u;
            packed[nt] = requant4_post<MODE>(raw, bdiv, bmul, mult, a.post, accw, a.zp_f, a.lo_f, a.hi_f);
          } else {
            packed[nt] = requant4<MODE>(raw, bdiv, bmul, mult, a.zp_f, a.lo_f, a.hi_f);
          }
        }
      }
      if constexpr (MODE != kOutAcc32) {
        uint8_t* const dst = static_cast<uint8_t*>(a.y) + off;
        if (a.vec && cb + 16 <= a.OC) {
          *reinterpret_cast<v4i*>(dst) = v4i{static_cast<int>(packed[0]), static_cast<int>(packed[1]),
                                             static_cast<int>(packed[2]), static_cast<int>(packed[3])};
        } else {
#pragma unroll
          for (int c = 0; c < 16; ++c)
            if (cb + c < a.OC) dst[c] = static_cast<uint8_t>(packed[c >> 2] >> (8 * (c & 3)));
        }
      }
    }
    __syncthreads();  // the staged rows are overwritten by the next tile
  }
}

}  // namespace tmq
