// Halo-tiled quantized::conv2d for gfx950.
//
// One block computes a TH x TW patch of output pixels of one image for 64
// output channels of one group.  It first copies into LDS
//   * the whole [64 x K] slice of the packed weight (K = KH*KW*ICg bytes), and
//   * the input halo the patch needs: HH x HW pixels x ICg channels, each input
//     byte read from memory exactly once per block; positions outside the image
//     are written as the activation zero point (real value 0),
// and after one barrier the eight waves run independently: every MFMA operand
// of every tap is a 16-byte LDS read at  pixel_base[lane] + tap_offset[k-chunk],
// so the k loop has no global loads, no barriers and no per-lane address
// arithmetic beyond one addition of a tabulated tap offset.
//
// LDS layout (byte offsets from the dynamic LDS base):
//   weights  [k-chunk][64 rows][16 B]          (the packed order, rows of this tile)
//   halo     [HH rows][ri slots of 16 B]: HW pixels of `pitch` bytes (ICg rounded up to an
//            odd number of slots: 16 consecutive pixels fall into distinct bank groups),
//            then padding slots chosen so that a row tile that crosses patch rows keeps
//            that property
//   staging  8 waves x [32 pixels][80 B] for the row-major output transpose
//   taps     int32[2*(KS+4)]: halo byte offset of every 16-byte k-chunk
//
// The operand roles, the x ^ 0x80 trick and the accumulator start value are
// those of gemm_i8_core.h.
#pragma once

#include "gemm_i8_core.h"

namespace tmq {

constexpr int kCtThreads = 512;
constexpr int kCtWaves = kCtThreads / kWave;
constexpr int kCtBN = 64;            // output channels per block
constexpr int kCtTPitch = 80;        // staging bytes per pixel (64 + 16: off one bank)
constexpr int kCtTBytes = 32 * kCtTPitch;
constexpr int kCtMaxPixels = 512;    // output pixels per block (16 MFMA row tiles)

struct ConvTileArgs {
  const uint8_t* x;          // NHWC
  const uint8_t* w_packed;   // all groups
  const int32_t* colsum;
  const float* w_scales;
  const float* bias;
  void* y;
  int64_t w_kchunks, group_bytes;
  int H, W, IC, OH, OW, OC;
  int KW, icb;               // icb = ICg / 16
  int kchunks;               // KH*KW*icb: k-chunks that carry weights
  int KS;                    // k-steps of 32 bytes, even (zero weights pad the last)
  int sh, sw, ph, pw, dh, dw;
  int ICg, OCg, n_tiles;     // n_tiles = 64-channel tiles per group
  int TH, TW, HH, HW, pitch;
  int ri, rpp;               // 16-byte LDS slots per halo row (<= 512; the last ones may be padding), halo rows per pass of the block
  int cx;                    // passes over the halo
  uint32_t xstep;            // image bytes between a thread's successive halo items
  int xdstep;                // and the LDS bytes between them
  int tiles_h, tiles_w;
  int lds_x, lds_t, lds_tab;
  int32_t w_scale_stride;
  uint32_t x_xor;            // 0x80808080 for quint8 activations
  uint32_t pad_word;         // activation zero point in 4 bytes (before the xor)
  int32_t acc_coef;
  float x_scale, out_scale, zp_f, lo_f, hi_f;
  float rcp_tw, rcp_ri, rcp_icb, rcp_kw, rcp_pslots;  // 1 / TW, 1 / ri, 1 / icb, 1 / KW, 16 / pitch
  PostOps post;
};

// n / d for n < 2**22 with rcp = 1.0f / d: the float estimate is off by at most
// one either way.
__device__ __forceinline__ uint32_t small_div(uint32_t n, uint32_t d, float rcp) {
  uint32_t q = static_cast<uint32_t>(static_cast<float>(n) * rcp);
  const int32_t r = static_cast<int32_t>(n - q * d);
  q = r < 0 ? q - 1 : (r >= static_cast<int32_t>(d) ? q + 1 : q);
  return q;
}

// KIND selects the requantisation compiled in: 0 a residual and no SiLU, 3 SiLU
// (with a residual if there is one), 1 plain with clamp, 2 plain for unsigned
// output without ReLU (the saturating pack conversion is the clamp), 4 plain for bytes with zero point 0 (-128 for
// signed ones) and no bounds inside the range (the pack conversion is rounding, zero point and clamp), 5 a residual
// and no SiLU into such bytes.  VEC: output rows take aligned 16-byte (int32 mode:
// 4-channel) stores.  One variant per launch keeps the straight-line code that
// every wave runs exactly once small: the kernel with all variants inside was
// five times longer and spent a quarter of its time fetching instructions.
template <int MODE, int KIND, bool VEC>
__global__ __launch_bounds__(kCtThreads) void conv_tile_kernel(ConvTileArgs a) {
  constexpr bool kPost = KIND == 0 || KIND == 3 || KIND == 5;  // the epilogue with post operations
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  __shared__ __attribute__((aligned(16))) int s_acc0[kCtBN];
  __shared__ __attribute__((aligned(16))) float s_mult[kCtBN];
  __shared__ __attribute__((aligned(16))) float s_bdiv[kCtBN];

  const int t = threadIdx.x;
  const int lane = t % kWave, wave = t / kWave;
  const int li = lane & 31, half = lane >> 5;

  // ---- which patch, which channels
  uint32_t sid = blockIdx.x;
  const uint32_t tcol = sid % static_cast<uint32_t>(a.tiles_w);
  sid /= static_cast<uint32_t>(a.tiles_w);
  const uint32_t trow = sid % static_cast<uint32_t>(a.tiles_h);
  const uint32_t b = sid / static_cast<uint32_t>(a.tiles_h);
  const int g = static_cast<int>(blockIdx.y) / a.n_tiles;
  const int nt = static_cast<int>(blockIdx.y) - g * a.n_tiles;
  const int oh0 = static_cast<int>(trow) * a.TH, ow0 = static_cast<int>(tcol) * a.TW;
  const int ih0 = oh0 * a.sh - a.ph, iw0 = ow0 * a.sw - a.pw;
  const int n0 = nt * kCtBN;           // first channel of the tile inside its group
  const int ch0 = g * a.OCg + n0;      // the same channel in the whole tensor

  // ---- per-channel constants: requested now, used after the copy below so
  // that their latency hides behind it
  const bool c_ok = t < kCtBN && n0 + t < a.OCg;
  int c_colsum = 0;
  float c_wscale = 1.f, c_bias = 0.f;
  if (c_ok) {
    const int np = ch0 + t;
    c_colsum = a.colsum[np];
    if (MODE != kOutAcc32) {
      c_wscale = a.w_scales[np * a.w_scale_stride];
      if (a.bias != nullptr) c_bias = a.bias[np];
    }
  }

  // ---- copy weights and halo into LDS with direct global-to-LDS loads: a wave
  // instruction moves 64 x 16 bytes from per-lane addresses to 64 consecutive
  // 16-byte LDS slots starting at a wave-uniform address, without passing
  // through registers, so the loads of the whole block are in flight at once.
  //   weights: wave w copies k-chunks w, w+8, ... (64 rows x 16 B = one slot run)
  //   halo:    slot s of a pass is thread s; a pass covers `rpp` whole halo rows
  //            of `ri` slots (pitch/16 per pixel, the padding slot left alone)
  // Out-of-image positions get the activation zero point from a plain LDS
  // store.  The sign-bit flip of unsigned activations (x ^ 0x80) is applied to
  // the fragments in the k loop.
  {
    const int nbv_all = (a.OCg + 15) / 16 - nt * 4;
    const int nbv = nbv_all < 4 ? nbv_all : 4;  // 16-row weight blocks that exist
    const uint8_t* const wsrc =
        a.w_packed + g * a.group_bytes + static_cast<int64_t>(nt) * 4 * a.w_kchunks * 256;
    const uint8_t* const img =
        a.x + static_cast<int64_t>(b) * (static_cast<int64_t>(a.H) * a.W * a.IC) + g * a.ICg;
    // copies as "uniform base + 32-bit lane offset" (lds_dma16): the host keeps a
    // 64-channel weight slice and one image below 4 GB
    const uint32_t lds0 = lds_address(lds);
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);

    const int nbl = (lane >> 4) & 3, nbc = nbl < nbv ? nbl : nbv - 1;
    uint32_t woff = static_cast<uint32_t>((static_cast<int64_t>(nbc) * a.w_kchunks + wave_u) * 256 + (lane & 15) * 16);
    for (int kc = wave_u; kc < 2 * a.KS; kc += kCtWaves) {
      lds_dma16(wsrc, woff, lds0 + kc * (kCtBN * 16));
      woff += kCtWaves * 256;
    }

    const int pslots = a.pitch >> 4;  // slots per pixel
    const int lr = static_cast<int>(small_div(t, a.ri, a.rcp_ri)), it = t - lr * a.ri;
    const int hc = static_cast<int>(small_div(it, pslots, a.rcp_pslots)), hb = it - hc * pslots;
    const bool active = lr < a.rpp && hb < a.icb && hc < a.HW;
    const bool col_ok = static_cast<unsigned>(iw0 + hc) < static_cast<unsigned>(a.W);
    // byte offset inside the image; wraps harmlessly where it is not used
    uint32_t xoff = (static_cast<uint32_t>(ih0 + lr) * static_cast<uint32_t>(a.W) +
                     static_cast<uint32_t>(iw0 + hc)) * static_cast<uint32_t>(a.IC) +
                    static_cast<uint32_t>(hb) * 16u;
    const int padx = static_cast<int>(a.pad_word);
    int wave_dst = a.lds_x + wave_u * (kWave * 16);  // first slot of this wave in the current pass
    int hr = lr;
    for (int i = 0; i < a.cx; ++i) {
      const bool live = active && hr < a.HH;
      const bool inside = live && col_ok && static_cast<unsigned>(ih0 + hr) < static_cast<unsigned>(a.H);
      if (inside)
        lds_dma16(img, xoff, lds0 + wave_dst);
      else if (live)
        *reinterpret_cast<v4i*>(lds + wave_dst + lane * 16) = v4i{padx, padx, padx, padx};
      hr += a.rpp;
      xoff += a.xstep;
      wave_dst += a.xdstep;
    }
    // Halo byte offset of the two 16-byte k-chunks of every k-step: chunk
    // c = tap * icb + blk lies at (kh*dil_h) * row bytes + (kw*dil_w) * pitch + blk*16.
    // Chunks past the last tap carry zero weights and read pixel 0; the k loop
    // reads three steps past the end.
    int* const s_tab = reinterpret_cast<int*>(lds + a.lds_tab);
    for (int c = t; c < 2 * (a.KS + 4); c += kCtThreads) {
      int off = 0;
      if (c < a.kchunks) {
        const int tap = static_cast<int>(small_div(c, a.icb, a.rcp_icb)), blk = c - tap * a.icb;
        const int kh = static_cast<int>(small_div(tap, a.KW, a.rcp_kw)), kw = tap - kh * a.KW;
        off = kh * a.dh * (a.ri * 16) + kw * a.dw * a.pitch + blk * 16;
      }
      s_tab[c] = off;
    }
    __builtin_amdgcn_s_waitcnt(0);  // the direct loads have landed in LDS
  }
  if (t < kCtBN) {
    int acc0 = 0;
    float mult = 0.f, bdiv = 0.f;
    if (c_ok) {
      acc0 = a.acc_coef * c_colsum;
      if (MODE != kOutAcc32) {
        const float atw = a.x_scale * c_wscale;
        mult = atw / a.out_scale;
        bdiv = a.bias != nullptr ? bias_term(a.w_scale_stride == 0, c_bias, atw) : 0.f;
      }
    }
    s_acc0[t] = acc0;
    s_mult[t] = mult;
    s_bdiv[t] = bdiv;
  }
  __syncthreads();

  // ---- compute.  Waves w and w+4 run on the same SIMD.  The row tiles (32
  // output pixels each) are dealt to the four SIMDs in contiguous, near-equal
  // runs; wave w takes the first half of a run, wave w+4 the rest, two row tiles
  // at a time.
  const int TP = a.TH * a.TW;
  const int MT = (TP + 31) / 32;
  int first, count;
  {
    const int pair = wave & 3, second = wave >> 2;
    const int per = MT / 4, extra = MT % 4;
    const int pfirst = pair * per + (pair < extra ? pair : extra);
    const int pcount = per + (pair < extra ? 1 : 0);
    const int mine = (pcount + 1) / 2;
    first = second ? pfirst + mine : pfirst;
    count = second ? pcount - mine : mine;
  }
  uint8_t* const sT = lds + a.lds_t + wave * kCtTBytes;
  const uint8_t* const sW = lds;
  const uint8_t* const sX = lds + a.lds_x;
  const int img_pix = static_cast<int>(b) * a.OH * a.OW;  // the host keeps pixel counts below 2**31
  constexpr bool vec_ok = VEC;  // the host checked channel counts and the output's alignment
  const v4i xmask = {static_cast<int>(a.x_xor), static_cast<int>(a.x_xor), static_cast<int>(a.x_xor),
                     static_cast<int>(a.x_xor)};
  const float bmul = MODE == kOutAcc32 ? 1.0f : bias_mul(a.w_scale_stride == 0, a.x_scale * a.w_scales[0]);

  auto run = [&](auto tm_tag, int mt0) {
    constexpr int TM = decltype(tm_tag)::value;
    int xb[TM];        // halo byte offset of this lane's pixel in each row tile
    int opix[TM];      // its output pixel index (b, oh, ow), -1 if outside
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      int m = (mt0 + tm) * 32 + li;
      const bool in_tile = m < TP;
      m = in_tile ? m : TP - 1;
      const int r = static_cast<int>(small_div(static_cast<uint32_t>(m), static_cast<uint32_t>(a.TW), a.rcp_tw));
      const int c = m - r * a.TW;
      xb[tm] = r * a.sh * (a.ri * 16) + c * a.sw * a.pitch;
      const int oh = oh0 + r, ow = ow0 + c;
      opix[tm] = (in_tile && oh < a.OH && ow < a.OW) ? img_pix + oh * a.OW + ow : -1;
    }
    v16i acc[2][TM];
#pragma unroll
    for (int tn = 0; tn < 2; ++tn) {
      v16i init;
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) {
        const v4i q = *reinterpret_cast<const v4i*>(&s_acc0[tn * 32 + 8 * gq + 4 * half]);
        init[4 * gq] = q.x;
        init[4 * gq + 1] = q.y;
        init[4 * gq + 2] = q.z;
        init[4 * gq + 3] = q.w;
      }
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) acc[tn][tm] = init;
    }

    // The residual bytes of the row tile are requested now and arrive while the
    // k loop runs.  Aligned case: whole pixels, 16 bytes per lane in the order of
    // the output stores (4 lanes per pixel, 16 pixels per pass: 16 cache lines per
    // instruction instead of the 32 that per-lane words of 32 pixels touch, 2
    // instructions instead of 8), turned into this lane's words (4 consecutive
    // channels each) through the staging rows before the requantisation.
    // Otherwise: the words themselves, byte by byte.
    uint32_t accw[TM][8];
    v4i accv[TM][2];
    const bool res_rows = kPost && VEC && a.post.accum != nullptr && n0 + kCtBN <= a.OCg &&
                          ((reinterpret_cast<uintptr_t>(a.post.accum) | static_cast<uintptr_t>(a.OC)) & 15) == 0;
    if (kPost && a.post.accum != nullptr) {
      if (res_rows) {
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
          for (int pass = 0; pass < 2; ++pass) {
            const int op = __shfl(opix[tm], pass * 16 + (lane >> 2), kWave);
            accv[tm][pass] = op >= 0 ? ld16(a.post.accum + static_cast<int64_t>(op) * a.OC + ch0 + (lane & 3) * 16)
                                     : v4i{0, 0, 0, 0};
          }
      } else {
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            const int nl = (u >> 2) * 32 + 8 * (u & 3) + 4 * half;
            const int left = a.OCg - (n0 + nl);
            const int nvalid = (opix[tm] >= 0 && left > 0) ? (left < 4 ? left : 4) : 0;
            accw[tm][u] = nvalid > 0 ? load_accum4(a.post, static_cast<int64_t>(opix[tm]) * a.OC + ch0 + nl, nvalid)
                                     : 0u;
          }
      }
    }

    // Fragments of successive k-steps; the two halves of the wave take the two
    // chunks of the step.  The tap offset of a step is fetched one step ahead.
    // Reading runs two steps past the end (results unused; the addresses stay
    // inside the block's LDS).
    int w_addr = (half * kCtBN + li) * 16;
    int tab_addr = a.lds_tab + half * 4;
    int toff = *reinterpret_cast<const int*>(lds + tab_addr);
    v4i wf0[2], xf0[TM], wf1[2], xf1[TM];
    auto read_step = [&](v4i(&wf)[2], v4i(&xf)[TM]) {
      const int cur = toff;
      tab_addr += 8;
      toff = *reinterpret_cast<const int*>(lds + tab_addr);
      wf[0] = ld16(sW + w_addr);
      wf[1] = ld16(sW + w_addr + 32 * 16);
      w_addr += 2 * kCtBN * 16;
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) xf[tm] = ld16(sX + xb[tm] + cur);
    };
    auto mul_step = [&](const v4i(&wf)[2], const v4i(&xf)[TM]) {
      v4i xs[TM];
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) xs[tm] = xf[tm] ^ xmask;
#pragma unroll
      for (int tn = 0; tn < 2; ++tn)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
          acc[tn][tm] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[tn], xs[tm], acc[tn][tm], 0, 0, 0);
    };
    // KS is even.  The fragments of a step are requested before the MFMAs of
    // the step before it are issued; the fences keep that order.
    read_step(wf0, xf0);
    for (int s = 0; s < a.KS; s += 2) {
      read_step(wf1, xf1);
      __builtin_amdgcn_sched_barrier(0);
      mul_step(wf0, xf0);
      __builtin_amdgcn_sched_barrier(0);
      read_step(wf0, xf0);
      __builtin_amdgcn_sched_barrier(0);
      mul_step(wf1, xf1);
      __builtin_amdgcn_sched_barrier(0);
    }

    // ---- epilogue: a lane holds channels 8g + 4*half + j of pixel li
    if constexpr (MODE == kOutAcc32) {
      int32_t* y = static_cast<int32_t*>(a.y);
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) {
        if (opix[tm] < 0) continue;
        int32_t* row = y + static_cast<int64_t>(opix[tm]) * a.OC + ch0;
#pragma unroll
        for (int tn = 0; tn < 2; ++tn)
#pragma unroll
          for (int gq = 0; gq < 4; ++gq) {
            const int nl = tn * 32 + 8 * gq + 4 * half;
            if (vec_ok && n0 + nl + 4 <= a.OCg) {
              *reinterpret_cast<v4i*>(row + nl) = v4i{acc[tn][tm][4 * gq], acc[tn][tm][4 * gq + 1],
                                                      acc[tn][tm][4 * gq + 2], acc[tn][tm][4 * gq + 3]};
            } else {
#pragma unroll
              for (int j = 0; j < 4; ++j)
                if (n0 + nl + j < a.OCg) row[nl + j] = acc[tn][tm][4 * gq + j];
            }
          }
      }
    } else {
      uint8_t* y = static_cast<uint8_t*>(a.y);
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) {
        if (kPost && res_rows) {  // residual pixels -> this lane's words, through the staging rows
#pragma unroll
          for (int pass = 0; pass < 2; ++pass)
            *reinterpret_cast<v4i*>(sT + (pass * 16 + (lane >> 2)) * kCtTPitch + (lane & 3) * 16) = accv[tm][pass];
          wave_sync_lds();
#pragma unroll
          for (int u = 0; u < 8; ++u)
            accw[tm][u] = *reinterpret_cast<const uint32_t*>(sT + li * kCtTPitch + (u >> 2) * 32 + 8 * (u & 3) + 4 * half);
          wave_sync_lds();  // the words are read before the results overwrite the rows
        }
        {
#pragma unroll
          for (int tn = 0; tn < 2; ++tn)
#pragma unroll
            for (int gq = 0; gq < 4; ++gq) {
              const int nl = tn * 32 + 8 * gq + 4 * half;
              const v4f mult = *reinterpret_cast<const v4f*>(&s_mult[nl]);
              const v4f bdiv = *reinterpret_cast<const v4f*>(&s_bdiv[nl]);
              int raw[4];
#pragma unroll
              for (int j = 0; j < 4; ++j) raw[j] = acc[tn][tm][4 * gq + j];
              uint32_t q4;
              if constexpr (kPost)
                q4 = requant4_post<MODE, KIND == 3 ? 2 : 1, KIND == 5>(raw, bdiv, bmul, mult, a.post, accw[tm][tn * 4 + gq],
                                                            a.zp_f, a.lo_f, a.hi_f);
              else
                q4 = requant4<MODE, KIND == 1, KIND == 4 ? 1 : 0>(raw, bdiv, bmul, mult, a.zp_f, a.lo_f, a.hi_f);
              *reinterpret_cast<uint32_t*>(sT + li * kCtTPitch + nl) = q4;
            }
        }
        wave_sync_lds();
        // whole pixels leave as 16 bytes per lane: 4 lanes per pixel, 16 pixels per pass
#pragma unroll
        for (int pass = 0; pass < 2; ++pass) {
          const int p = pass * 16 + (lane >> 2), cq = lane & 3;
          const v4i v = ld16(sT + p * kCtTPitch + cq * 16);
          const int op = __shfl(opix[tm], p, kWave);
          const int n = n0 + cq * 16;
          if (op >= 0 && n < a.OCg) {
            uint8_t* dst = y + static_cast<int64_t>(op) * a.OC + ch0 + cq * 16;
            if (vec_ok) {
              *reinterpret_cast<v4i*>(dst) = v;
            } else if (n + 16 <= a.OCg) {
              st16_any(dst, v);
            } else {
              const uint32_t w[4] = {static_cast<uint32_t>(v.x), static_cast<uint32_t>(v.y),
                                     static_cast<uint32_t>(v.z), static_cast<uint32_t>(v.w)};
              for (int bb = 0; bb < 16; ++bb)
                if (n + bb < a.OCg) dst[bb] = static_cast<uint8_t>(w[bb >> 2] >> (8 * (bb & 3)));
            }
          }
        }
        wave_sync_lds();  // the staging rows are rewritten by the next row tile
      }
    }
  };

  // Two row tiles at a time share the weight fragments (a third less LDS traffic).
  // With a residual the tiles go one at a time instead: the requantisation, the
  // residual rows and the stores of the first tile then run under the k loop of
  // the second, and the two waves of a SIMD drift out of phase (C5 with a residual
  // and ReLU: 14.3 -> 13.5 us per launch; without a residual it changes nothing).
  // (SiLU without a residual has nothing to overlap: two at a time as well)
  while ((!kPost || (KIND == 3 && a.post.accum == nullptr)) && count >= 2) {
    run(std::integral_constant<int, 2>{}, first);
    first += 2;
    count -= 2;
  }
  while (count >= 1) {
    run(std::integral_constant<int, 1>{}, first);
    first += 1;
    count -= 1;
  }
}

}  // namespace tmq
