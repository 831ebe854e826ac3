// quantized::conv2d for a few input channels (gfx950): the first layer of an image
// network (3 -> 64 channels, 7 x 7, stride 2), pointwise layers whose channel count is
// no multiple of 16, one group, no dilation.
//
// With so few channels a 16-byte k-chunk of the MFMA cannot be "16 channels of one
// pixel".  In NHWC the KW taps of one kernel row are KW * IC *contiguous* bytes of an
// image row, so k is ordered (kh, run) with run = the RL = KW * IC bytes of a kernel
// row, padded to RP = a multiple of 16 with zero weights: the bytes an operand picks
// up past the run's end are multiplied by zero.  K = KH * RP is at most 256 here, the
// weights of 64 (32) output channels stay in registers (16 operands of
// v_mfma_i32_16x16x64_i8) for the whole launch; prepack lays them out per lane
// (conv_runs_slot) behind the packed weight of the other kernels.
//
// A block of four waves walks tiles of TR x TW output pixels of one image:
//   * it stages the (TR - 1) * stride + KH image rows the tile needs, as bytes, positions
//     outside the image as the activation zero point, sign flip of unsigned activations
//     applied.  The copy runs in aligned 16-byte loads whatever the address of an image
//     row: each staged row starts 0 ... 15 bytes before the tile's first byte of its row;
//   * a wave takes 16 output pixels of one output row at a time: the operand of pixel
//     p, kernel row kh, 16-byte piece c of the run is the 16 bytes at
//       row (orow * stride + kh), byte p * stride * IC + 16 c
//     of the staged rows -- any byte alignment, so it is put together from five aligned
//     words with v_alignbyte_b32;
//   * operand roles: weights are the rows (i), pixels the columns (j) of the MFMA,
//     D[i][j]: lane l, register r -> i = 4 (l / 16) + r, j = l % 16.  Row i of channel
//     tile nt (of NT = 4, or 2 for at most 32 output channels) is channel
//     4 NT (i / 4) + 4 nt + i % 4, so that a lane ends up with 4 NT consecutive channels of
//     one pixel: one 16-byte (8-byte) store.
// The x ^ 0x80 trick, the accumulator start value and the requantisation are those of
// gemm_i8_core.h.
#pragma once

#include "gemm_i8_core.h"

namespace tmq {

constexpr int kCrThreads = 256;
constexpr int kCrWaves = kCrThreads / kWave;
constexpr int kCrMaxKS = 4;    // k-steps of 64 bytes
constexpr int kCrUnits = 4;    // 1 KB units of staged image rows per wave and tile: 16 KB per block

struct ConvRunArgs {
  const uint8_t* x;          // NHWC
  const uint8_t* w_runs;     // [channel block of 16 NT][channel tile nt][k-step][lane][16 B]: conv_runs_slot below
  const int32_t* colsum;
  const float* w_scales;
  const float* bias;
  void* y;
  int32_t tiles;             // B * tiles_h * tiles_w
  int B, H, W, IC, OH, OW, OC, KH, KW;
  int sh, sw, ph, pw;
  int RL, RP, KS;            // run bytes, padded run bytes, k-steps (KH * RP <= 64 KS)
  int TR, TW, mtw;           // output rows and columns per tile, 16-pixel pieces per tile row
  int rows_in, pitch;        // staged image rows, LDS bytes per staged row (multiple of 16)
  int tiles_h, tiles_w;
  int vec;                   // 16-byte (int32 mode: per 4 channels) stores are aligned
  int32_t w_scale_stride;
  uint32_t x_xor, pad_word;  // pad_word: the activation zero point in 4 bytes, before the xor
  int32_t acc_coef;
  float x_scale, out_scale, zp_f, lo_f, hi_f;
  PostOps post;
};

// One 16-byte slot of the per-lane weight layout: slot index ->
// (channel block cb of 16 NT channels, channel tile nt, k-step ks, lane).  NT = 4 tiles per block,
// 2 for layers of at most 32 output channels.  The lane's row i = lane % 16 of tile nt is channel
// 16 NT cb + 4 NT (i / 4) + 4 nt + i % 4 (a lane of the kernel then holds 4 NT consecutive
// channels); its bytes are k = 64 ks + 16 (lane / 16) ... + 15 in (kh, run) order: kernel row
// kh = k / RP, byte k % RP of the run, which in OHWI weights is byte (kw, ic) = k % RP of the
// contiguous row w[n][kh][.][.]; zeros past the run's RL bytes, past the last kernel row and for
// channels that do not exist.
__host__ __device__ inline int conv_runs_tiles(int64_t OC) { return OC <= 32 ? 2 : 4; }
__device__ __forceinline__ v4i conv_runs_slot(const int8_t* __restrict__ w, int64_t slot, int OC, int KH, int RL,
                                              int RP, int KS) {
  const int NT = conv_runs_tiles(OC);
  const int lane = static_cast<int>(slot & 63);
  const int64_t op = slot >> 6;
  const int ks = static_cast<int>(op % KS), nt = static_cast<int>((op / KS) % NT);
  const int64_t cb = op / (NT * KS);
  const int i = lane & 15;
  const int64_t n = cb * 16 * NT + 4 * NT * (i >> 2) + 4 * nt + (i & 3);
  const int k = 64 * ks + 16 * (lane >> 4);
  const int kh = k / RP, ro = k - kh * RP;
  uint32_t words[4] = {0, 0, 0, 0};
  if (n < OC && kh < KH) {
    const int8_t* const src = w + (n * KH + kh) * RL;
    for (int b = 0; b < 16; ++b)
      if (ro + b < RL) words[b >> 2] |= static_cast<uint32_t>(static_cast<uint8_t>(src[ro + b])) << (8 * (b & 3));
  }
  return v4i{static_cast<int>(words[0]), static_cast<int>(words[1]), static_cast<int>(words[2]),
             static_cast<int>(words[3])};
}

// Requantise (or pass on) the 4 NT consecutive channels cb ... of one pixel that a lane holds after the
// MFMAs of its NT channel tiles, and store them at element offset `off` of the output: one store of 4 NT
// bytes where all the channels exist.  mult / bdiv: the constants of channel cb onwards.  PLAIN: the host found
// requant_plain_u8 to hold (zero point 0 for unsigned bytes, -128 for signed ones, no bounds inside the range).
template <int MODE, bool POST, int NT, bool PLAIN = false>
__device__ __forceinline__ void runs_requant_store(const ConvRunArgs& a, const v4i (&acc)[NT], int64_t off, int cb,
                                                   const float* mult_cb, const float* bdiv_cb, float bmul) {
  constexpr int kLaneCh = 4 * NT;
  uint32_t packed[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
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
      const v4f mult = *reinterpret_cast<const v4f*>(mult_cb + 4 * nt);
      const v4f bdiv = *reinterpret_cast<const v4f*>(bdiv_cb + 4 * nt);
      if constexpr (POST) {
        const int left = a.OC - (cb + 4 * nt);
        const int nvalid = left < 0 ? 0 : (left < 4 ? left : 4);
        const uint32_t accw =
            a.post.accum != nullptr && nvalid > 0 ? load_accum4(a.post, off + 4 * nt, nvalid) : 0u;
        packed[nt] = requant4_post<MODE>(raw, bdiv, bmul, mult, a.post, accw, a.zp_f, a.lo_f, a.hi_f);
      } else {
        packed[nt] = requant4<MODE, true, PLAIN ? 1 : 0>(raw, bdiv, bmul, mult, a.zp_f, a.lo_f, a.hi_f);
      }
    }
  }
  if constexpr (MODE != kOutAcc32) {
    uint8_t* const dst = static_cast<uint8_t*>(a.y) + off;
    if (cb + kLaneCh <= a.OC) {  // one store of 4 NT bytes; any alignment unless the host found the rows aligned
      if constexpr (NT == 4) {
        const v4i all = {static_cast<int>(packed[0]), static_cast<int>(packed[1]), static_cast<int>(packed[2]),
                         static_cast<int>(packed[3])};
        if (a.vec)
          *reinterpret_cast<v4i*>(dst) = all;
        else
          st16_any(dst, all);
      } else {
        static_assert(NT == 2, "channel tiles per block: 2 or 4");
        const v2i all = {static_cast<int>(packed[0]), static_cast<int>(packed[1])};
        if (a.vec)
          *reinterpret_cast<v2i*>(dst) = all;
        else
          st8_any(dst, all);
      }
    } else {
#pragma unroll
      for (int c = 0; c < kLaneCh; ++c)
        if (cb + c < a.OC) dst[c] = static_cast<uint8_t>(packed[c >> 2] >> (8 * (c & 3)));
    }
  }
}

template <int MODE, bool POST, int NT, bool PLAIN = false>
__global__ __launch_bounds__(kCrThreads, 3) void conv_runs_kernel(ConvRunArgs a) {
  constexpr int kCrBN = 16 * NT;  // output channels per block (grid y)
  constexpr int kLaneCh = 4 * NT; // consecutive channels of one pixel in a lane
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  __shared__ __attribute__((aligned(16))) int s_acc0[kCrBN];
  __shared__ __attribute__((aligned(16))) float s_mult[kCrBN];
  __shared__ __attribute__((aligned(16))) float s_bdiv[kCrBN];

  const int t = threadIdx.x, lane = t % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(t / kWave);
  const int pj = lane & 15, pq = lane >> 4;
  const int n0 = static_cast<int>(blockIdx.y) * kCrBN;
  const int KS = a.KS;
  uint8_t* const sX = lds;                  // staged image rows

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
  // the weight operands of this block's 64 channels, laid out per lane at prepack
  v4i wreg[NT][kCrMaxKS];
  {
    const uint8_t* const wsrc = a.w_runs + (static_cast<int64_t>(blockIdx.y) * NT * KS * kWave + lane) * 16;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int ks = 0; ks < kCrMaxKS; ++ks)
        wreg[nt][ks] = ks < KS ? ld16(wsrc + (nt * KS + ks) * (kWave * 16)) : v4i{0, 0, 0, 0};
  }
  __syncthreads();
  // this lane's piece of every k-step: staged row and byte inside the run
  int lk[kCrMaxKS];  // (a multiple of 16) | the row's share of the alignment shift, (kh * (row bytes % 16)) % 16
#pragma unroll
  for (int ks = 0; ks < kCrMaxKS; ++ks) {
    const int koff = ks * 64 + pq * 16;
    int kh = koff / a.RP, ro = koff - kh * a.RP;
    if (kh >= a.KH) {  // past the last kernel row: zero weights, any staged bytes
      kh = a.KH - 1;
      ro = 0;
    }
    lk[ks] = (kh * a.pitch + ro) | ((kh * (a.W * a.IC)) & 15);
  }
  float bmul = 1.0f;
  if constexpr (MODE != kOutAcc32) bmul = bias_mul(a.w_scale_stride == 0, a.x_scale * a.w_scales[0]);

  const int row_bytes = a.W * a.IC;
  const int tile_mt = a.TR * a.mtw;
  // The staged rows of a tile pass through registers, requested one tile ahead, so that they
  // arrive while the tile in hand is multiplied.  The unit of the copy is 1 KB of one staged
  // row, one 16-byte load per lane; unit u belongs to wave u % 4 (the host sizes the tiles
  // for at most kCrUnits units per wave).  Staged row r starts
  //   shift(r) = (c0 + r * (row bytes % 16)) % 16
  // bytes before the tile's first byte of that image row, so that every load is an aligned
  // 16 bytes of memory: LDS byte q of the row is image-row byte iwb0 - shift(r) + q.
  const int segs = (a.pitch + 1023) >> 10, units = a.rows_in * segs;
  v4i pre[kCrUnits];
  struct TilePos {
    int b, oh0, ow0, c0;
    int ih0, iwb0;        // image row and byte in the row of the tile's first staged byte (before the shift)
    int64_t first;        // the same as a byte offset into the tensor
    int edge;             // some load may reach outside the tensor
  };
  const int rb15 = row_bytes & 15;
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
    tp.c0 = static_cast<int>((reinterpret_cast<uintptr_t>(a.x) + static_cast<uintptr_t>(tp.first)) & 15);
    tp.edge = tp.first < 16 || tp.first + static_cast<int64_t>(a.rows_in) * row_bytes + a.pitch + 16 > x_bytes;
    return tp;
  };
  // Unit `slot` of this wave: staged row, first LDS byte of the unit in that row (-1: none).
  auto unit_pos = [&](int slot, int* r, int* q0) {
    const int u = wave + kCrWaves * slot;
    *r = segs == 1 ? u : u / segs;
    *q0 = u < units ? (u - *r * segs) << 10 : -1;
  };
  // The loads only.  A load may hang over either end of its image row into the neighbouring
  // rows (store_tile overwrites those bytes); nothing here uses a loaded value, so nothing
  // waits.  Only in the first and the last tiles of the tensor can a load reach outside it;
  // those tiles check every byte.
  auto request = [&](const TilePos& tp) {
#pragma unroll
    for (int slot = 0; slot < kCrUnits; ++slot) {
      int r, q0;
      unit_pos(slot, &r, &q0);
      if (q0 < 0 || static_cast<unsigned>(tp.ih0 + r) >= static_cast<unsigned>(a.H)) continue;  // (wave-uniform)
      const int q = q0 + 16 * lane;
      const int64_t rel = tp.first + static_cast<int64_t>(r) * row_bytes - ((tp.c0 + r * rb15) & 15) + q0;
      if (q >= a.pitch) continue;
      if (!tp.edge) {
        pre[slot] = *reinterpret_cast<const v4i*>(a.x + rel + 16 * lane);
      } else {
        uint32_t w4[4] = {0, 0, 0, 0};
        for (int jj = 0; jj < 16; ++jj) {
          const int64_t o = rel + 16 * lane + jj;
          if (o >= 0 && o < x_bytes) w4[jj >> 2] |= static_cast<uint32_t>(a.x[o]) << (8 * (jj & 3));
        }
        pre[slot] = v4i{static_cast<int>(w4[0]), static_cast<int>(w4[1]), static_cast<int>(w4[2]), static_cast<int>(w4[3])};
      }
    }
  };
  // Into LDS with the sign flip; then the bytes outside the image -- whole rows above and
  // below it, the ends of a row left and right of it -- become the activation zero point.
  // A wave pads its own units, after its own stores to them.
  auto store_tile = [&](const TilePos& tp) {
    const int xw = static_cast<int>(a.x_xor), pw4 = static_cast<int>(a.pad_word ^ a.x_xor);
    const v4i xmask = {xw, xw, xw, xw}, padv = {pw4, pw4, pw4, pw4};
#pragma unroll
    for (int slot = 0; slot < kCrUnits; ++slot) {
      int r, q0;
      unit_pos(slot, &r, &q0);
      if (q0 < 0) continue;
      const bool row_in = static_cast<unsigned>(tp.ih0 + r) < static_cast<unsigned>(a.H);
      uint8_t* const row = sX + r * a.pitch;
      const int q = q0 + 16 * lane;
      if (q < a.pitch) *reinterpret_cast<v4i*>(row + q) = row_in ? (pre[slot] ^ xmask) : padv;
      if (!row_in) continue;
      const int shift = (tp.c0 + r * rb15) & 15;
      const int qend = q0 + 1024 < a.pitch ? q0 + 1024 : a.pitch;
      // left of the image row: LDS bytes [0, shift - iwb0); right of it: [shift + row bytes - iwb0, pitch)
      const int left = shift - tp.iwb0 < qend ? shift - tp.iwb0 : qend;
      for (int i = q0 + lane; i < left; i += kWave) row[i] = static_cast<uint8_t>(pw4);
      const int right = shift + row_bytes - tp.iwb0 > q0 ? shift + row_bytes - tp.iwb0 : q0;
      for (int i = right + lane; i < qend; i += kWave) row[i] = static_cast<uint8_t>(pw4);
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
      const int c0r = c0 + orow * a.sh * rb15;  // alignment shift of staged row orow * stride, before the % 16
      v4i acc[NT];  // start: the zero point's share, acc_coef * colsum
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) acc[nt] = *reinterpret_cast<const v4i*>(&s_acc0[kLaneCh * pq + 4 * nt]);
#pragma unroll
      for (int ks = 0; ks < kCrMaxKS; ++ks) {
        if (ks < KS) {
          const int addr = base + (lk[ks] & ~15) + ((c0r + lk[ks]) & 15);
          const uint32_t* const src = reinterpret_cast<const uint32_t*>(sX + (addr & ~3));
          const uint32_t sb = static_cast<uint32_t>(addr & 3);
          const uint32_t d0 = src[0], d1 = src[1], d2 = src[2], d3 = src[3], d4 = src[4];
          const v4i xv = {static_cast<int>(__builtin_amdgcn_alignbyte(d1, d0, sb)),
                          static_cast<int>(__builtin_amdgcn_alignbyte(d2, d1, sb)),
                          static_cast<int>(__builtin_amdgcn_alignbyte(d3, d2, sb)),
                          static_cast<int>(__builtin_amdgcn_alignbyte(d4, d3, sb))};
#pragma unroll
          for (int nt = 0; nt < NT; ++nt)
            acc[nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wreg[nt][ks], xv, acc[nt], 0, 0, 0);
        }
      }
      // ---- requantise and store: this lane has channels n0 + 4 NT pq .. + 4 NT - 1 of pixel pj
      if (pcol >= tw_valid) continue;
      const int64_t opix = (static_cast<int64_t>(b) * a.OH + oh0 + orow) * a.OW + ow0 + pcol;
      const int cb = n0 + kLaneCh * pq;
      if (cb >= a.OC) continue;
      const int64_t off = opix * a.OC + cb;
      runs_requant_store<MODE, POST, NT, PLAIN>(a, acc, off, cb, &s_mult[kLaneCh * pq], &s_bdiv[kLaneCh * pq], bmul);
    }
    __syncthreads();  // the staged rows are overwritten by the next tile
  }
}

// Pointwise layers (1 x 1, stride 1, no padding, one group) over at most 256 input channels,
// on the same per-lane weight layout: here a pixel's IC bytes *are* the run, a lane's MFMA
// operand for pixel p and k-step ks is the 16 bytes at p * IC + 64 ks + 16 (lane / 16) of the
// input -- straight from memory, any alignment, no staging -- and what it picks up past the
// pixel's last channel (the next pixel's bytes) meets zero weights.  The weights of all output
// channels sit in LDS as MFMA operands; a wave walks 16-pixel pieces of the image on its own
// (no barrier after set-up), asks for the next piece's bytes before it works on the current
// one's, and runs every 16 NT-channel block of the output over the piece in hand: the input is
// read once whatever OC is.  a.tiles: the number of 16-pixel pieces.
constexpr int kCrPointwiseLdsMax = 144 * 1024;
__host__ __device__ inline int64_t conv_runs_pointwise_lds(int64_t OC, int64_t KS) {
  const int64_t nt = conv_runs_tiles(OC), nblk = (OC + 16 * nt - 1) / (16 * nt);
  return nblk * nt * KS * 1024 + nblk * 16 * nt * 12;
}

template <int MODE, bool POST, int NT, bool PLAIN = false>
__global__ __launch_bounds__(kCrThreads, 3) void conv_runs_pointwise_kernel(ConvRunArgs a) {
  constexpr int kCrBN = 16 * NT;   // output channels per channel block
  constexpr int kLaneCh = 4 * NT;  // consecutive channels of one pixel in a lane
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  const int t = threadIdx.x, lane = t % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(t / kWave);
  const int pj = lane & 15, pq = lane >> 4;
  const int KS = a.KS;
  const int nblk = (a.OC + kCrBN - 1) / kCrBN;
  const int wslots = nblk * NT * KS * kWave;  // 16-byte operands
  int* const s_acc0 = reinterpret_cast<int*>(lds + wslots * 16);
  float* const s_mult = reinterpret_cast<float*>(s_acc0 + nblk * kCrBN);
  float* const s_bdiv = s_mult + nblk * kCrBN;
  const int64_t npix = static_cast<int64_t>(a.B) * a.H * a.W, x_bytes = npix * a.IC;
  // this lane's 16 bytes of every k-step for the pixel pj of a piece (zeros where the piece has no such pixel or the
  // k-step no such bytes; the tensor's last few bytes one by one)
  const auto fetch = [&](int64_t piece, v4i (&xv)[kCrMaxKS]) {
    const int64_t pix = piece * 16 + pj;
#pragma unroll
    for (int ks = 0; ks < kCrMaxKS; ++ks) {
      xv[ks] = v4i{0, 0, 0, 0};
      const int k0 = ks * 64 + pq * 16;
      if (ks < KS && pix < npix && k0 < a.RP) {
        const int64_t o = pix * a.IC + k0;
        if (o + 16 <= x_bytes) {
          xv[ks] = ld16_any(a.x + o);
        } else {
          uint32_t words[4] = {0, 0, 0, 0};
          for (int b = 0; b < 16; ++b)
            if (o + b < x_bytes) words[b >> 2] |= static_cast<uint32_t>(a.x[o + b]) << (8 * (b & 3));
          xv[ks] = v4i{static_cast<int>(words[0]), static_cast<int>(words[1]), static_cast<int>(words[2]), static_cast<int>(words[3])};
        }
      }
    }
  };
  // the first pieces' bytes are asked for before the weights and constants are set up: their latencies overlap
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kCrWaves;
  int64_t piece = static_cast<int64_t>(blockIdx.x) * kCrWaves + wave;
  // (KS == 1: pre[i] is the one k-step of the i-th piece ahead, four pieces in flight; otherwise the next piece's k-steps)
  static_assert(kCrMaxKS == 4, "the ring of four pieces shares the registers of one piece's four k-steps");
  v4i pre[kCrMaxKS] = {};
  if (KS == 1) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (piece + i * stride < a.tiles) {
        v4i tmp[kCrMaxKS];
        fetch(piece + i * stride, tmp);
        pre[i] = tmp[0];
      }
  } else if (piece < a.tiles) {
    fetch(piece, pre);
  }
  for (int i = t; i < wslots; i += kCrThreads) *reinterpret_cast<v4i*>(lds + i * 16) = ld16(a.w_runs + static_cast<int64_t>(i) * 16);
  for (int n = t; n < nblk * kCrBN; n += kCrThreads) {
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
    s_acc0[n] = acc0;
    s_mult[n] = mult;
    s_bdiv[n] = bdiv;
  }
  __syncthreads();
  float bmul = 1.0f;
  if constexpr (MODE != kOutAcc32) bmul = bias_mul(a.w_scale_stride == 0, a.x_scale * a.w_scales[0]);

  // every channel block over the piece in hand (xv: its bytes, sign flip applied)
  const auto multiply = [&](int64_t piece, const v4i (&xv)[kCrMaxKS]) {
    const int64_t pix = piece * 16 + pj;
    for (int cbi = 0; cbi < nblk; ++cbi) {
      const int cl = cbi * kCrBN + kLaneCh * pq;  // this lane's first channel of the block
      v4i acc[NT];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) acc[nt] = *reinterpret_cast<const v4i*>(&s_acc0[cl + 4 * nt]);
#pragma unroll
      for (int ks = 0; ks < kCrMaxKS; ++ks) {
        if (ks < KS) {
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) {
            const v4i w = *reinterpret_cast<const v4i*>(lds + ((((cbi * NT + nt) * KS + ks) * kWave + lane) << 4));
            acc[nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w, xv[ks], acc[nt], 0, 0, 0);
          }
        }
      }
      if (pix < npix && cl < a.OC)
        runs_requant_store<MODE, POST, NT, PLAIN>(a, acc, pix * a.OC + cl, cl, &s_mult[cl], &s_bdiv[cl], bmul);
    }
  };
  const int xo = static_cast<int>(a.x_xor);
  const v4i flip = {xo, xo, xo, xo};
  if (KS == 1) {
    // At most 64 input channels: one load per piece, four pieces' loads in flight per wave.
    while (piece < a.tiles) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (piece < a.tiles) {
          const v4i xv[kCrMaxKS] = {pre[i] ^ flip, v4i{0, 0, 0, 0}, v4i{0, 0, 0, 0}, v4i{0, 0, 0, 0}};
          if (piece + 4 * stride < a.tiles) {
            v4i tmp[kCrMaxKS];
            fetch(piece + 4 * stride, tmp);
            pre[i] = tmp[0];
          }
          multiply(piece, xv);
          piece += stride;
        }
      }
    }
    return;
  }
  for (; piece < a.tiles; piece += stride) {
    v4i xv[kCrMaxKS];
#pragma unroll
    for (int ks = 0; ks < kCrMaxKS; ++ks) xv[ks] = pre[ks] ^ flip;
    if (piece + stride < a.tiles) fetch(piece + stride, pre);
    multiply(piece, xv);
  }
}

}  // namespace tmq
