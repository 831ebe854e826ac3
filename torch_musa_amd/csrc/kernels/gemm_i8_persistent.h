// Persistent int8 MFMA GEMM for quantized::linear products that fill the chip
// more than once (gfx950).
//
// One block per CU walks a sequence of 256 x 256 output tiles.  The arithmetic,
// the operand roles, the LDS layouts and the direct global->LDS copy pipeline
// are those of gemm_i8_kernel<256, 256, 2, 4, ..., WDMA, XWIDE> in
// gemm_i8_core.h; what changes is what happens between two tiles of a block:
//
//   * the operand copies of the next tile's first three stages and the next
//     tile's per-channel constants are requested BEFORE the epilogue of the
//     current tile, so that they land while the block requantises and stores
//     (a one-tile-per-block launch starts every tile with an empty pipeline);
//   * the epilogue is wave-private: a wave requantises its own 128 x 64 part
//     of the tile 32 rows at a time, transposes them through a 2.5 KB staging
//     area of its own and stores whole 64-byte row pieces, with no block
//     barrier -- the staging areas live in the one ring buffer that the next
//     tile's prologue does not touch (activation pair buffer 2);
//   * the per-channel constants are double-buffered (the next tile's are
//     written while the current tile's are still being read).
//
// LDS map (bytes): weights 3 x 16 KB | activation pairs 3 x 32 KB | constants
// 2 x 3 KB.  Activation pair buffer 2 doubles as 8 x 2560 B of staging (float
// output: 8 x 4608 B, which runs 4 KB past the ring into bytes appended for it).
#pragma once

#include <type_traits>

#include "gemm_i8_core.h"

namespace tmq {

constexpr int kPersistThreads = 512;

template <int MODE>
__global__ __launch_bounds__(kPersistThreads, 1) void gemm_i8_persistent_kernel(GemmArgs a, XLinear xsrc) {
  static_assert(MODE == kOutU8 || MODE == kOutS8 || MODE == kOutF32, "byte or float outputs");
  constexpr int BM = 256, BN = 256, WM = 2, WN = 4;
  constexpr int NWAVES = WM * WN;
  constexpr int WTM = BM / WM, WTN = BN / WN;      // 128 rows x 64 channels per wave
  constexpr int TM = WTM / 32, TN = WTN / 32;      // 4 x 2 MFMA tiles
  constexpr int Q = TN * TM, NF = TN + TM;
  constexpr int NDW = kChunks * (BN / 64) / NWAVES;  // weight copies per wave per stage
  constexpr int NDX = (BM / 16) / NWAVES;            // activation copies per wave per stage (half a pair)
  constexpr int ND = NDW + NDX;
  static_assert(NDW == 2 && NDX == 2 && (BM / 8) / NWAVES / 2 == NDX, "copy split");
  constexpr int kWStage = kChunks * BN * 16;       // 16 KB
  constexpr int kXStage = BM * 2 * kBK;            // 32 KB: two stages of every row
  constexpr int kRing = 3 * kWStage + 3 * kXStage;
  constexpr int kTPitch = 80;                      // staging bytes per row: 64 + 16, off one bank
  constexpr int kTBytes = 32 * kTPitch;
  constexpr int kStagingOff = 3 * kWStage + 2 * kXStage;  // activation pair buffer 2
  static_assert(NWAVES * kTBytes <= kXStage, "staging fits the idle pair buffer");
  // float output: a wave stages one 32 x 32 MFMA tile at a time, rows of 128 + 16 bytes;
  // eight such areas are 4 KB more than the idle pair buffer, appended to the ring
  constexpr int kFPitch = 32 * 4 + 16;
  constexpr int kFBytes = 32 * kFPitch;
  constexpr int kFExtra = MODE == kOutF32 ? NWAVES * kFBytes - kXStage : 0;
  static_assert(kFExtra >= 0 && kRing + kFExtra + 2 * 3 * BN * 4 <= 160 * 1024, "LDS budget");

  __shared__ __attribute__((aligned(16))) uint8_t smem[kRing + kFExtra];
  __shared__ __attribute__((aligned(16))) int s_acc0[2][BN];
  __shared__ __attribute__((aligned(16))) float s_mult[2][BN];
  __shared__ __attribute__((aligned(16))) float s_bdiv[2][BN];
  uint8_t* const sW = smem;
  uint8_t* const sX = smem + 3 * kWStage;

  const int t = threadIdx.x;
  const int lane = t % kWave, wave = t / kWave;
  const int li = lane & 31, half = lane >> 5;
  const int wm0 = (wave % WM) * WTM;
  const int wn0 = (wave / WM) * WTN;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const uint32_t lds0 = lds_address(smem);

  // (the host keeps the tile count below 2**31 and every per-lane operand offset
  // below 2**32: 32-bit index arithmetic throughout, 64-bit divisions would cost
  // a block two microseconds per tile)
  const uint32_t tiles_m = static_cast<uint32_t>(ceil_div(a.M, BM)), tiles_n = static_cast<uint32_t>(ceil_div(a.N, BN));
  const uint32_t nblocks = tiles_m * tiles_n;
  const int NB = static_cast<int>(ceil_div(a.N, 16));
  const int KT = static_cast<int>(ceil_div(a.K, kBK));
  const int pair_last = (KT - 1) >> 1;
  const int ktail = static_cast<int>(a.K) - 16 - pair_last * 2 * kBK;  // last chunk inside K of the last pair
  auto clampk = [&](int kt) { return kt < KT ? kt : KT - 1; };

  // ---- tile sequence: virtual block v = round * gridDim.x + blockIdx.x takes
  // the tile the one-tile-per-block kernel gives block v (every XCD owns one
  // contiguous run of the sequence, ordered in patches four channel tiles wide)
  auto tile_origin = [&](uint32_t v, int* m0, int* n0) {
    const uint32_t q = nblocks / 8, rem = nblocks % 8;
    const uint32_t xcd = v % 8, within = v / 8;
    const uint32_t tile = xcd * q + (xcd < rem ? xcd : rem) + within;
    constexpr uint32_t kGroupN = 4;
    const uint32_t group = tile / (tiles_m * kGroupN);
    const uint32_t gfirst = group * kGroupN;
    const uint32_t gwidth = tiles_n - gfirst < kGroupN ? tiles_n - gfirst : kGroupN;
    const uint32_t in_group = tile - group * (tiles_m * kGroupN);
    const uint32_t row = in_group / gwidth;
    *m0 = static_cast<int>(row * BM);
    *n0 = static_cast<int>((gfirst + in_group - row * gwidth) * BN);
  };
  // (a permutation of the tiles as long as the grid is a multiple of 8 or holds
  // every tile in one round, which the host guarantees)

  // ---- per-tile copy set-up: operand bases and per-lane offsets
  const uint8_t* wtile;
  const uint8_t* xtile;
  uint32_t wdma_off[NDW], xdma_off[2 * NDX], xdma_off_last[2 * NDX];
  const uint32_t wdma_lds = lds0 + ((wave_u & 3) * BN + (wave_u >> 2) * 64) * 16;
  const uint32_t xdma_lds = lds0 + 3 * kWStage + wave_u * 1024;
  const uint32_t kch = static_cast<uint32_t>(a.w_kchunks), ldx = static_cast<uint32_t>(xsrc.ldx);
  auto tile_setup = [&](int m0, int n0) {
    wtile = a.w_packed + static_cast<int64_t>(n0 / 16) * a.w_kchunks * 256;
    const int nb_last = NB - 1 - n0 / 16;  // rows past N: clamped, never stored
#pragma unroll
    for (int i = 0; i < NDW; ++i) {
      const int rg = (wave_u >> 2) + i * (NWAVES / 4);
      int rb = rg * 4 + (lane >> 4);
      rb = rb < nb_last ? rb : nb_last;
      wdma_off[i] = (static_cast<uint32_t>(rb) * kch + static_cast<uint32_t>(wave_u & 3)) * 256u + (lane & 15) * 16;
    }
    xtile = xsrc.x + static_cast<int64_t>(m0) * xsrc.ldx;
    const int m_last = static_cast<int>(a.M) - 1 - m0;
#pragma unroll
    for (int i = 0; i < 2 * NDX; ++i) {
      const int row = (wave_u + i * NWAVES) * 8 + (lane >> 3);
      const uint32_t r = static_cast<uint32_t>(row < m_last ? row : m_last);
      const int kc = ((lane & 7) ^ ((row >> 1) & 7)) * 16;
      xdma_off[i] = r * ldx + kc;
      // chunks past K: any valid bytes will do, the packed weight is zero there
      xdma_off_last[i] = r * ldx + (kc < ktail ? kc : ktail);
    }
  };
  auto dma_w = [&](int kt, int wb, int i) {
    lds_dma16(wtile + static_cast<int64_t>(kt) * (kChunks * 256), wdma_off[i],
              wdma_lds + wb * kWStage + i * (NWAVES / 4) * 64 * 16);
  };
  auto dma_x = [&](int u, int xb, int i) {
    const int uc = u < pair_last ? u : pair_last;
    lds_dma16(xtile + static_cast<int64_t>(uc) * (2 * kBK), uc == pair_last ? xdma_off_last[i] : xdma_off[i],
              xdma_lds + xb * kXStage + i * NWAVES * 1024);
  };
  // the first three stages of a tile: weights 0..2, activation pairs 0 and 1
  // (weight buffers 0..2, pair buffers 0 and 1; pair buffer 2 stays untouched)
  auto issue_prologue = [&]() {
#pragma unroll
    for (int i = 0; i < 2 * NDX; ++i) dma_x(0, 0, i);
#pragma unroll
    for (int i = 0; i < NDW; ++i) dma_w(0, 0, i);
#pragma unroll
    for (int i = 0; i < NDW; ++i) dma_w(clampk(1), 1, i);
#pragma unroll
    for (int i = 0; i < NDX; ++i) dma_x(1, 1, i);
#pragma unroll
    for (int i = 0; i < NDW; ++i) dma_w(clampk(2), 2, i);
#pragma unroll
    for (int i = 0; i < NDX; ++i) dma_x(1, 1, NDX + i);
  };
  auto wait_loads = [&](auto left_tag) {  // s_waitcnt vmcnt(left) only
    constexpr int kLeft = decltype(left_tag)::value;
    static_assert(kLeft < 64, "load counter range");
    __builtin_amdgcn_s_waitcnt((kLeft & 15) | ((kLeft >> 4) << 14) | (7 << 4) | (15 << 8));
  };

  // ---- per-channel constants of a tile's 256 channels: thread t < 256 requests
  // channel t's (load_consts) and writes them to buffer `par` later
  // (store_consts), so that the loads' latency hides behind whatever runs
  // between the two
  const XQuant xq = x_quant(a);
  struct Consts {
    int colsum;
    float wscale, bias;
    bool ok;
  };
  auto load_consts = [&](int n0) {
    Consts c{0, 1.f, 0.f, false};
    const int64_t n = n0 + t;
    if (t < BN && n < a.N) {
      c.ok = true;
      c.colsum = a.colsum[n];
      c.wscale = a.w_scales[n * a.w_scale_stride];
      if (a.bias != nullptr) c.bias = a.bias[n];
    }
    return c;
  };
  auto store_consts = [&](const Consts& c, int par) {
    if (t < BN) {
      int acc0 = 0;
      float mult = 0.f, bdiv = 0.f;
      if (c.ok) {
        acc0 = xq.coef * c.colsum;
        const float atw = xq.scale * c.wscale;
        if (MODE == kOutF32) {
          mult = atw;
          bdiv = c.bias;  // 0 without a bias
        } else {
          mult = atw / a.out_scale;
          bdiv = a.bias != nullptr ? bias_term(a.w_scale_stride == 0, c.bias, atw) : 0.f;
        }
      }
      s_acc0[par][t] = acc0;
      s_mult[par][t] = mult;
      s_bdiv[par][t] = bdiv;
    }
  };

  // ---- main-loop pieces (see the wide-copy pipeline in gemm_i8_core.h)
  v16i acc[TN][TM];
  const v4i xmask = {static_cast<int>(a.x_xor), static_cast<int>(a.x_xor), static_cast<int>(a.x_xor),
                     static_cast<int>(a.x_xor)};
  v4i wf0[TN], xf0[TM], wf1[TN], xf1[TM];
  auto mfma = [&](int q, const v4i(&wf)[TN], const v4i(&xf)[TM]) {
    static_assert(TN == 2, "the order below pairs the two channel tiles of a row tile");
    const int tm = q / 2, tn = (q % 2) ^ (tm & 1);  // consecutive products share one operand
    acc[tn][tm] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[tn], xf[tm], acc[tn][tm], 0, 0, 0);
  };
  auto flip = [&](v4i& f) { f ^= xmask; };
  const int xswz8 = (li >> 1) & 7;
  auto read_w = [&](int wb, int xb, int p, int s, int j, v4i(&wf)[TN], v4i(&xf)[TM]) {
    const int c = 2 * s + half;
    if (j < TN)
      wf[j] = ld16(&sW[wb * kWStage + (c * BN + wn0 + j * 32 + li) * 16]);
    else
      xf[j - TN] = ld16(&sX[xb * kXStage + (wm0 + (j - TN) * 32 + li) * (2 * kBK) + (((4 * p + c) ^ xswz8) << 4)]);
  };
  auto stage = [&](int kt, int ph) {
    const int wb = ph % 3, xb = (ph >> 1) % 3, p = ph & 1;
    const int phn = (ph + 1) % 6;
    const int wbn = phn % 3, xbn = (phn >> 1) % 3, pn = phn & 1;
#pragma unroll
    for (int q = 0; q < Q; ++q) {
      if (q < NF) read_w(wb, xb, p, 1, q, wf1, xf1);
      mfma(q, wf0, xf0);
      if (q + 1 < TM) flip(xf0[q + 1]);
      if (q == Q - 1) flip(xf1[0]);
      __builtin_amdgcn_sched_barrier(0);
    }
    // only the copies issued by the stage before this one may still be outstanding
    wait_loads(std::integral_constant<int, ND>{});
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    const int kload = clampk(kt + 3);
    const int uload = (kt + 4) >> 1;
    const int xbl = ((ph + 4) % 6 >> 1) % 3;
    const int ihalf = ((ph + 4) & 1) * NDX;
    constexpr int kFirstDma = (TM - 1 < Q - 1 - ND) ? TM - 1 : (Q - 1 - ND > 0 ? Q - 1 - ND : 0);
#pragma unroll
    for (int q = 0; q < Q; ++q) {
      if (q < NF) read_w(wbn, xbn, pn, 0, q, wf0, xf0);
      if (q >= kFirstDma && q - kFirstDma < ND) {
        const int i = q - kFirstDma;
        if (i < NDW) dma_w(kload, wb, i);
        else dma_x(uload, xbl, ihalf + i - NDW);
      }
      mfma(q, wf1, xf1);
      if (q + 1 < TM) flip(xf1[q + 1]);
      if (q == Q - 1) flip(xf0[0]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // ---- epilogue of the tile at (m0, n0), constants in buffer `par`: requantise in
  // registers, 32 rows at a time through this wave's staging rows, 16 bytes per
  // lane out (4 lanes per row, 16 rows per store instruction)
  uint8_t* const sT = smem + kStagingOff + wave * kTBytes;
  uint8_t* const ybase = static_cast<uint8_t*>(a.y);
  const bool vec_ok = ((a.ldy & 15) == 0) && ((reinterpret_cast<uintptr_t>(a.y) & 15) == 0);
  const float bmul = MODE == kOutF32 ? 1.0f : bias_mul(a.w_scale_stride == 0, xq.scale * a.w_scales[0]);
  const bool plain_u8 = MODE == kOutU8 && a.lo_f <= 0.f && a.hi_f >= 255.f;
  // float output: y = max(fma(float(acc), x_scale * w_scale[n], bias[n]), lo); a 32 x 32
  // MFMA tile at a time through this wave's staging rows, whole 128-byte row pieces out
  // (8 lanes per row, 8 rows per store instruction)
  auto epilogue_f32 = [&](int m0, int n0, int par) {
    uint8_t* const sF = smem + kStagingOff + wave * kFBytes;
    float* const yf = static_cast<float*>(a.y);
    const bool fvec_ok = ((a.ldy & 3) == 0) && ((reinterpret_cast<uintptr_t>(a.y) & 15) == 0);
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int cl = 8 * g + 4 * half;  // channel inside the MFMA tile
          const v4f mult = *reinterpret_cast<const v4f*>(&s_mult[par][wn0 + tn * 32 + cl]);
          const v4f bias = *reinterpret_cast<const v4f*>(&s_bdiv[par][wn0 + tn * 32 + cl]);
          v4f v;
#pragma unroll
          for (int j = 0; j < 4; ++j)
            v[j] = __builtin_fmaxf(__builtin_fmaf(static_cast<float>(acc[tn][tm][4 * g + j]), mult[j], bias[j]),
                                   a.lo_f);
          *reinterpret_cast<v4f*>(sF + li * kFPitch + cl * 4) = v;
        }
        wave_sync_lds();
        if (tm == 0 && tn == 0) wait_loads(std::integral_constant<int, 0>{});  // as in the byte epilogue
#pragma unroll
        for (int pass = 0; pass < 4; ++pass) {
          const int p = pass * 8 + (lane >> 3), cq = lane & 7;
          const v4f v = *reinterpret_cast<const v4f*>(sF + p * kFPitch + cq * 16);
          const int64_t m = m0 + wm0 + tm * 32 + p, n = n0 + wn0 + tn * 32 + cq * 4;
          if (m < a.M && n < a.N) {
            float* dst = yf + m * a.ldy + n;
            if (fvec_ok && n + 4 <= a.N) {
              // (four times the bytes of the operands and read by nobody in this launch: past
              // the caches, which hold the operands -- 210 -> 204 us for the dynamic linear at
              // M = K = 4096, N = 11008; the byte outputs measure the same either way)
              __builtin_nontemporal_store(v, reinterpret_cast<v4f*>(dst));
            } else {
              for (int j = 0; j < 4; ++j)
                if (n + j < a.N) dst[j] = v[j];
            }
          }
        }
        wave_sync_lds();  // the staging rows are rewritten by the next tile
      }
    }
  };
  auto epilogue = [&](int m0, int n0, int par, auto clamp_tag) {
    constexpr bool CL = decltype(clamp_tag)::value;
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int cl = tn * 32 + 8 * g + 4 * half;  // channel inside the wave's 64
          const v4f mult = *reinterpret_cast<const v4f*>(&s_mult[par][wn0 + cl]);
          const v4f bdiv = *reinterpret_cast<const v4f*>(&s_bdiv[par][wn0 + cl]);
          int raw[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) raw[j] = acc[tn][tm][4 * g + j];
          *reinterpret_cast<uint32_t*>(sT + li * kTPitch + cl) =
              requant4<MODE, CL>(raw, bdiv, bmul, mult, a.zp_f, a.lo_f, a.hi_f);
        }
      wave_sync_lds();
      // The next tile's first copies, requested before this epilogue, are waited
      // for here: after a quarter of the arithmetic and before the first store,
      // so that neither their latency nor the stores' sits at the top of the next
      // tile (a wait there would also wait for the last stores to be acknowledged).
      if (tm == 0) wait_loads(std::integral_constant<int, 0>{});
#pragma unroll
      for (int pass = 0; pass < 2; ++pass) {
        const int p = pass * 16 + (lane >> 2), cq = lane & 3;
        const v4i v = ld16(sT + p * kTPitch + cq * 16);
        const int64_t m = m0 + wm0 + tm * 32 + p, n = n0 + wn0 + cq * 16;
        if (m < a.M && n < a.N) {
          uint8_t* dst = ybase + m * a.ldy + n;
          if (vec_ok && n + 16 <= a.N) {
            *reinterpret_cast<v4i*>(dst) = v;
          } else if (n + 16 <= a.N) {
            st16_any(dst, v);  // (a row pitch or pointer off the 16-byte grid)
          } else {
            const uint32_t w[4] = {static_cast<uint32_t>(v.x), static_cast<uint32_t>(v.y),
                                   static_cast<uint32_t>(v.z), static_cast<uint32_t>(v.w)};
            for (int b = 0; b < 16; ++b)
              if (n + b < a.N) dst[b] = static_cast<uint8_t>(w[b >> 2] >> (8 * (b & 3)));
          }
        }
      }
      wave_sync_lds();  // the staging rows are rewritten by the next 32 rows
    }
  };

  // ---- the block's tiles
  uint32_t v = blockIdx.x;
  if (v >= nblocks) return;
  int m0, n0;
  tile_origin(v, &m0, &n0);
  tile_setup(m0, n0);
  {
    const Consts c = load_consts(n0);
    issue_prologue();
    store_consts(c, 0);
  }
  wait_loads(std::integral_constant<int, 0>{});
  int par = 0;
  while (true) {
    // this wave's first copies have landed (waited for above or inside the
    // previous epilogue); the barrier makes every wave's copies and the
    // constants visible and ends the previous epilogue's use of the staging rows
    __syncthreads();
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      v16i init;
#pragma unroll
      for (int r = 0; r < 16; ++r) init[r] = s_acc0[par][wn0 + tn * 32 + 8 * (r >> 2) + 4 * half + (r & 3)];
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) acc[tn][tm] = init;
    }
#pragma unroll
    for (int j = 0; j < NF; ++j) read_w(0, 0, 0, 0, j, wf0, xf0);
    flip(xf0[0]);
    // the host sends only K of at least six stages here
    int kt0 = 0;
    do {
#pragma unroll
      for (int j = 0; j < 6; ++j) stage(kt0 + j, j);
      kt0 += 6;
    } while (kt0 + 6 <= KT);
#pragma unroll
    for (int j = 0; j < 5; ++j)
      if (kt0 + j < KT) stage(kt0 + j, j);
    // the last copies (past the end of K, never read) must have landed, and every
    // wave must be done with the ring, before the next tile's copies reuse it
    wait_loads(std::integral_constant<int, 0>{});
    __syncthreads();

    const int em0 = m0, en0 = n0;
    v += gridDim.x;
    const bool more = v < nblocks;
    Consts next{0, 1.f, 0.f, false};
    if (more) {
      tile_origin(v, &m0, &n0);
      tile_setup(m0, n0);
      next = load_consts(n0);
      issue_prologue();
    }
    if constexpr (MODE == kOutF32) {
      epilogue_f32(em0, en0, par);
    } else {
      if (plain_u8)
        epilogue(em0, en0, par, std::false_type{});  // the saturating conversion is the clamp
      else
        epilogue(em0, en0, par, std::true_type{});
    }
    if (!more) break;
    store_consts(next, par ^ 1);
    par ^= 1;
  }
}

}  // namespace tmq
