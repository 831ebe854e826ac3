// int8 MFMA GEMM on 64 x 64 tiles whose operands reach LDS in phases of 256 bytes
// of K, four phases (128 KB) requested ahead.  For K <= 1024 that is all of K at
// once, which is what the kernel is for.
//
// The pipelined kernels of gemm_i8_core.h walk K one 64-byte stage after the
// other; a block that is alone on its CU spends 0.2 us per stage in the chain
// copy -> barrier -> LDS read -> MFMA whatever the prefetch depth, so a product
// like M = 128, K = N = 1024 (32 blocks, 16 stages) takes 6 us of which the
// multiplying is 0.5.  Here every wave requests its share of four phases of the
// tile at once with direct global -> LDS copies (128 KB in flight per block), the
// block meets at one barrier per phase as the copies land in the order issued,
// and between the barriers the waves multiply from LDS with no further
// synchronisation; behind the barrier that ends phase p the buffer it used takes
// phase p + 4.
//
// The automatic choice sends K <= 1024 here (grids of at most 256 tiles; up to 512
// tiles of 32 x 32 go to gemm_i8_ksplit_kernel at the end of this file).  Longer
// K runs (any K, for tests) but does not pay: with cold weights a phase then
// waits for memory, 96 KB in flight per CU against about 2 us of latency, and
// K = N = 4096 at M = 128 takes 15.0 us against 12.5 us for the 64 x 64 tiles
// with two wave groups.
//
// LDS layout (ring buffer b = phase % 4)
//   weights      [b][k-chunk (16 B of K)][64 rows][16 B]: the packed layout as it is
//   activations  [b][64 rows][256 B], the sixteen 16-byte slots of a row's 256
//                bytes XOR-ed with row % 16, so that the 16 rows a quarter wave
//                reads for one k-chunk fall on 16 different slots (every bank once)
// A copy instruction moves 1 KB: one weight k-chunk of the 64 rows, or the 256
// bytes of 4 activation rows (16 lanes per row: whole cache lines).
#pragma once

#include "gemm_i8_core.h"

namespace tmq {

constexpr int kOnePassMaxK = 1024;  // longest K the automatic choice sends here: four phases

// As lds_dma16 with 4 bytes per lane: lane l's dword lands at lds_dst + 4 l.
__device__ __forceinline__ void lds_dma4(const void* base, uint32_t off, uint32_t lds_dst) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1"
               :
               : "v"(off), "s"(base), "s"(lds_dst)
               : "memory", "m0");
}

template <int MODE>
__global__ __launch_bounds__(256) void gemm_i8_onepass_kernel(GemmArgs a, XLinear xs) {
  constexpr int BM = 64, BN = 64;
  constexpr int kPhaseChunks = 16;                 // k-chunks per barrier: 256 bytes of K
  constexpr int kRing = 4;                         // phases the LDS buffers hold
  constexpr int kCopiesPerPhase = 8;               // per wave: 4 weight chunks + 4 activation row groups
  __shared__ __attribute__((aligned(16))) uint8_t sW[kRing * kPhaseChunks * BN * 16];
  __shared__ __attribute__((aligned(16))) uint8_t sX[kRing * BM * 256];
  __shared__ __attribute__((aligned(16))) int s_raw[3][BN];  // colsum, weight scale, bias as fetched
  __shared__ __attribute__((aligned(16))) int s_acc0[BN];
  __shared__ __attribute__((aligned(16))) float s_mult[BN];
  __shared__ __attribute__((aligned(16))) float s_bdiv[BN];

  const int t = threadIdx.x, lane = t % kWave;
  const int wave_u = __builtin_amdgcn_readfirstlane(t / kWave);
  const int li = lane & 31, half = lane >> 5;
  const int wm0 = (wave_u & 1) * 32, wn0 = (wave_u >> 1) * 32;
  // grid (channel tiles, row tiles): no division to find the tile
  const int64_t m0 = static_cast<int64_t>(blockIdx.y) * BM;
  const int64_t n0 = static_cast<int64_t>(blockIdx.x) * BN;
  const int KC = static_cast<int>(a.K >> 4);       // k-chunks (K is a multiple of 16)
  const int S = (KC + 1) >> 1;                     // 32-byte k-steps
  const int NP = (KC + kPhaseChunks - 1) / kPhaseChunks;   // phases of 256 bytes of K

  // ---- requests, oldest first: the tile's per-channel constants (wave 0), then
  // phase by phase the weight chunks and activation row groups of this wave
  if (wave_u == 0) {
    const int64_t n = n0 + lane < a.N ? n0 + lane : a.N - 1;
    const uint32_t np = static_cast<uint32_t>(n + a.n_off);
    lds_dma4(a.colsum, np * 4u, lds_address(&s_raw[0][0]));
    if constexpr (MODE != kOutAcc32) {  // (raw accumulators: the caller passes no scales)
      lds_dma4(a.w_scales, np * static_cast<uint32_t>(a.w_scale_stride) * 4u, lds_address(&s_raw[1][0]));
      lds_dma4(a.bias != nullptr ? a.bias : a.w_scales, a.bias != nullptr ? np * 4u : 0u,
               lds_address(&s_raw[2][0]));
    }
  }
  const int64_t NB = ceil_div(a.N, 16);
  const int64_t nb_last = NB - 1 - n0 / 16;        // 16-row blocks past N: clamped, never stored
  const uint8_t* const wtile = a.w_packed + (n0 / 16) * a.w_kchunks * 256;
  const int64_t rb = (lane >> 4) < nb_last ? (lane >> 4) : nb_last;
  const uint32_t woff = static_cast<uint32_t>(rb * a.w_kchunks * 256 + (lane & 15) * 16);
  const int kc_last = static_cast<int>(a.w_kchunks) - 1;
  const uint8_t* const xtile = xs.x + m0 * xs.ldx;
  const int64_t m_last = a.M - 1 - m0;             // rows past M: clamped, never stored
  const uint32_t ldsW = lds_address(sW), ldsX = lds_address(sX);
  uint32_t xrow_off[4];                            // this lane's row of the wave's four activation copies
  int xslot[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = 4 * (4 * wave_u + i) + (lane >> 4);
    const int64_t rc = r < m_last ? r : m_last;
    xrow_off[i] = static_cast<uint32_t>(rc * xs.ldx);
    xslot[i] = (lane & 15) ^ (r & 15);
  }
  // the eight copies of this wave for phase p, into ring buffer p % kRing
  auto issue = [&](int p) {
    const int b = p & (kRing - 1);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int kc = p * kPhaseChunks + 4 * wave_u + i;
      const int kcc = kc < kc_last ? kc : kc_last;   // (chunks past the packed pitch are never multiplied)
      lds_dma16(wtile + static_cast<int64_t>(kcc) * 256, woff,
                ldsW + static_cast<uint32_t>(b * kPhaseChunks + 4 * wave_u + i) * 1024u);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int cc = p * kPhaseChunks + xslot[i];
      // chunks past K: any bytes of the row will do, they meet a zeroed operand or zero weights
      const int ccc = cc < KC ? cc : KC - 1;
      lds_dma16(xtile, xrow_off[i] + static_cast<uint32_t>(ccc) * 16u,
                ldsX + static_cast<uint32_t>(b * BM + 4 * (4 * wave_u + i)) * 256u);
    }
  };
  // waits until at most `phases` phases of this wave's copies (the youngest) are outstanding
  auto wait_phases = [&](int phases) {
    static_assert(kCopiesPerPhase == 8, "the wait counts below are multiples of the copies per phase");
    switch (phases) {
      case 0: __builtin_amdgcn_s_waitcnt((0 & 15) | ((0 >> 4) << 14) | (7 << 4) | (15 << 8)); break;
      case 1: __builtin_amdgcn_s_waitcnt((8 & 15) | ((8 >> 4) << 14) | (7 << 4) | (15 << 8)); break;
      case 2: __builtin_amdgcn_s_waitcnt((16 & 15) | ((16 >> 4) << 14) | (7 << 4) | (15 << 8)); break;
      default: __builtin_amdgcn_s_waitcnt((24 & 15) | ((24 >> 4) << 14) | (7 << 4) | (15 << 8)); break;
    }
  };

  const int first = NP < kRing ? NP : kRing;
  for (int p = 0; p < first; ++p) issue(p);

  const v4i xmask = {static_cast<int>(a.x_xor), static_cast<int>(a.x_xor), static_cast<int>(a.x_xor),
                     static_cast<int>(a.x_xor)};
  v16i acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0;
  const int xrow = wm0 + li;
  const uint8_t* const wrd = sW + (wn0 + li) * 16;
  const uint8_t* const xrd = sX + xrow * 256;

  wait_phases(first - 1);   // phase 0 (and, older than it, the constants) has landed
  __syncthreads();
  if (t < BN) {
    // turn the constants into the accumulator's start value and the requantisation factors
    const XQuant xq = x_quant(a);
    const bool live = n0 + t < a.N;
    float mult = 0.f, bdiv = 0.f;
    if constexpr (MODE != kOutAcc32) {
      const float ws = __int_as_float(s_raw[1][t]), bs = __int_as_float(s_raw[2][t]);
      const float atw = xq.scale * ws;
      if (MODE == kOutF32) {
        mult = atw;
        bdiv = a.bias != nullptr ? bs : 0.f;
      } else {
        mult = atw / a.out_scale;
        bdiv = a.bias != nullptr ? bias_term(a.w_scale_stride == 0, bs, atw) : 0.f;
      }
    }
    s_acc0[t] = live ? xq.coef * s_raw[0][t] : 0;
    s_mult[t] = live ? mult : 0.f;
    s_bdiv[t] = live ? bdiv : 0.f;
  }

  for (int p = 0; p < NP; ++p) {
    const int b = p & (kRing - 1);
    const int left = S - p * (kPhaseChunks / 2);
    const int nsteps = left < kPhaseChunks / 2 ? left : kPhaseChunks / 2;
    // (k-steps past the end of K in the last phase read whatever the buffers
    // hold and multiply it with a zeroed activation operand: no branches here)
    v4i wf[kPhaseChunks / 2], xf[kPhaseChunks / 2];
#pragma unroll
    for (int j = 0; j < kPhaseChunks / 2; ++j) {
      const int c = 2 * j + half;
      wf[j] = ld16(wrd + (b * kPhaseChunks + c) * (BN * 16));
      xf[j] = ld16(xrd + b * (BM * 256) + ((c ^ (xrow & 15)) << 4));
    }
#pragma unroll
    for (int j = 0; j < kPhaseChunks / 2; ++j) {
      const int keep = j < nsteps ? -1 : 0;
      const v4i xv = (xf[j] ^ xmask) & v4i{keep, keep, keep, keep};
      acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[j], xv, acc, 0, 0, 0);
    }
    if (p + 1 < NP) {
      // Phase p+1 must have landed; what this wave may still have on its way are
      // the phases after it that were already requested (up to p+3).  Behind the
      // barrier every wave is done with buffer p % kRing, which takes phase p+kRing.
      const int youngest = p + kRing - 1 < NP - 1 ? p + kRing - 1 : NP - 1;
      wait_phases(youngest - (p + 1));
      __syncthreads();
      if (p + kRing < NP) issue(p + kRing);
    }
  }

  // ---- epilogue.  A lane holds channels n = 8g + 4 half + j (g, j < 4) of
  // activation row li of its wave's 32 x 32 part; the tile goes through LDS (over
  // the weight chunks, which every wave has finished reading at the barrier) so
  // that whole rows leave with 16 bytes per lane.
  __syncthreads();
  if constexpr (MODE == kOutF32 || MODE == kOutAcc32) {
    constexpr int kPitch = BN * 4 + 16;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int nl = wn0 + 8 * g + 4 * half;
      const v4i add = *reinterpret_cast<const v4i*>(&s_acc0[nl]);
      const v4f mult = *reinterpret_cast<const v4f*>(&s_mult[nl]);
      const v4f bias = *reinterpret_cast<const v4f*>(&s_bdiv[nl]);
      v4f v;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int raw = acc[4 * g + j] + add[j];
        v[j] = MODE == kOutAcc32
                   ? __int_as_float(raw)
                   : __builtin_fmaxf(__builtin_fmaf(static_cast<float>(raw), mult[j], bias[j]), a.lo_f);
      }
      *reinterpret_cast<v4f*>(&sW[(wm0 + li) * kPitch + nl * 4]) = v;
    }
    __syncthreads();
    float* const yf = static_cast<float*>(a.y) + a.n_off;
    const bool vec_ok = ((a.ldy & 3) == 0) && ((reinterpret_cast<uintptr_t>(yf) & 15) == 0);
    constexpr int kRowChunks = BN / 4;
#pragma unroll
    for (int id = t; id < BM * kRowChunks; id += 256) {
      const int row = id / kRowChunks, cc = id % kRowChunks;
      const int64_t m = m0 + row, n = n0 + cc * 4;
      if (m >= a.M || n >= a.N) continue;
      const v4f v = *reinterpret_cast<const v4f*>(&sW[row * kPitch + cc * 16]);
      float* dst = yf + m * a.ldy + n;
      if (vec_ok && n + 4 <= a.N) {
        *reinterpret_cast<v4f*>(dst) = v;
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (n + j < a.N) dst[j] = v[j];
      }
    }
  } else {
    constexpr int kPitch = BN + 16;
    const float bmul = bias_mul(a.w_scale_stride == 0, x_quant(a).scale * __int_as_float(s_raw[1][0]));
    const bool plain_u8 = MODE == kOutU8 && a.lo_f <= 0.f && a.hi_f >= 255.f;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int nl = wn0 + 8 * g + 4 * half;
      const v4i add = *reinterpret_cast<const v4i*>(&s_acc0[nl]);
      const v4f mult = *reinterpret_cast<const v4f*>(&s_mult[nl]);
      const v4f bdiv = *reinterpret_cast<const v4f*>(&s_bdiv[nl]);
      int raw[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) raw[j] = acc[4 * g + j] + add[j];
      // unsigned output without ReLU: the saturating conversion is the clamp
      const uint32_t q4 = plain_u8 ? requant4<MODE, false>(raw, bdiv, bmul, mult, a.zp_f, a.lo_f, a.hi_f)
                                   : requant4<MODE, true>(raw, bdiv, bmul, mult, a.zp_f, a.lo_f, a.hi_f);
      *reinterpret_cast<uint32_t*>(&sW[(wm0 + li) * kPitch + nl]) = q4;
    }
    __syncthreads();
    uint8_t* const y = static_cast<uint8_t*>(a.y) + a.n_off;
    const bool vec_ok = ((a.ldy & 15) == 0) && ((reinterpret_cast<uintptr_t>(y) & 15) == 0);
    constexpr int kRowChunks = BN / 16;
    const int row = t / kRowChunks, cc = t % kRowChunks;   // 256 threads: one 16-byte piece each
    const int64_t m = m0 + row, n = n0 + cc * 16;
    if (m < a.M && n < a.N) {
      const v4i v = ld16(&sW[row * kPitch + cc * 16]);
      uint8_t* dst = y + m * a.ldy + n;
      if (vec_ok && n + 16 <= a.N) {
        *reinterpret_cast<v4i*>(dst) = v;
      } else if (n + 16 <= a.N) {
        st16_any(dst, v);  // (a row pitch or pointer off the 16-byte grid)
      } else {
        const uint32_t w[4] = {static_cast<uint32_t>(v.x), static_cast<uint32_t>(v.y), static_cast<uint32_t>(v.z),
                               static_cast<uint32_t>(v.w)};
        for (int b = 0; b < 16; ++b)
          if (n + b < a.N) dst[b] = static_cast<uint8_t>(w[b >> 2] >> (8 * (b & 3)));
      }
    }
  }
}

// (one thread's share of ksplit_finish: row idx / (BN / 4), channels 4 (idx % (BN / 4)) ... + 3)
template <int MODE, int BN, int WAVES>
__device__ __forceinline__ void ksplit_finish_four(const GemmArgs& a, const uint8_t* red, int red_stride,
                                                   const int (*s_raw)[kWave], int64_t m0, int64_t n0, int idx) {
  constexpr int kRedPitch = BN * 4 + 16;
  const int row = idx / (BN / 4), cl = (idx % (BN / 4)) * 4;
  const int64_t m = m0 + row, n = n0 + cl;
  if (m >= a.M || n >= a.N) return;
  v4i sum = *reinterpret_cast<const v4i*>(&red[row * kRedPitch + cl * 4]);
#pragma unroll
  for (int w = 1; w < WAVES; ++w) sum += *reinterpret_cast<const v4i*>(&red[w * red_stride + row * kRedPitch + cl * 4]);
  const XQuant xq = x_quant(a);
  int raw[4];
  v4f mult = {0.f, 0.f, 0.f, 0.f}, bdiv = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    raw[j] = sum[j] + xq.coef * s_raw[0][cl + j];
    if constexpr (MODE != kOutAcc32) {
      const float ws = __int_as_float(s_raw[1][cl + j]), bs = __int_as_float(s_raw[2][cl + j]);
      const float atw = xq.scale * ws;
      if (MODE == kOutF32) {
        mult[j] = atw;
        bdiv[j] = a.bias != nullptr ? bs : 0.f;
      } else {
        mult[j] = atw / a.out_scale;
        bdiv[j] = a.bias != nullptr ? bias_term(a.w_scale_stride == 0, bs, atw) : 0.f;
      }
    }
  }
  if constexpr (MODE == kOutF32 || MODE == kOutAcc32) {
    float* const dst = static_cast<float*>(a.y) + a.n_off + m * a.ldy + n;
    v4f v;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      v[j] = MODE == kOutAcc32 ? __int_as_float(raw[j])
                               : __builtin_fmaxf(__builtin_fmaf(static_cast<float>(raw[j]), mult[j], bdiv[j]), a.lo_f);
    if ((reinterpret_cast<uintptr_t>(dst) & 15) == 0 && n + 4 <= a.N) {
      *reinterpret_cast<v4f*>(dst) = v;
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (n + j < a.N) dst[j] = v[j];
    }
  } else {
    const float bmul = bias_mul(a.w_scale_stride == 0, xq.scale * __int_as_float(s_raw[1][0]));
    const bool plain_u8 = MODE == kOutU8 && a.lo_f <= 0.f && a.hi_f >= 255.f;
    // unsigned output without ReLU: the saturating conversion is the clamp
    const uint32_t q4 = plain_u8 ? requant4<MODE, false>(raw, bdiv, bmul, mult, a.zp_f, a.lo_f, a.hi_f)
                                 : requant4<MODE, true>(raw, bdiv, bmul, mult, a.zp_f, a.lo_f, a.hi_f);
    uint8_t* const dst = static_cast<uint8_t*>(a.y) + a.n_off + m * a.ldy + n;
    if ((reinterpret_cast<uintptr_t>(dst) & 3) == 0 && n + 4 <= a.N) {
      *reinterpret_cast<uint32_t*>(dst) = q4;
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (n + j < a.N) dst[j] = static_cast<uint8_t>(q4 >> (8 * j));
    }
  }
}

// The end of a tile of 32 rows x BN channels whose WAVES waves each hold a partial
// sum over their share of K: the partial tiles lie in LDS (wave w's at
// red + w * red_stride, rows of BN * 4 + 16 bytes, written before the barrier the
// caller has just passed); a thread adds them for four channels of one row,
// requantises and stores.  s_raw: colsum, weight scale and bias of the tile's
// channels as fetched.
constexpr int kSplitRedPitch = 32 * 4 + 16;
template <int MODE, int BN = 32, int WAVES = 4>
__device__ __forceinline__ void ksplit_finish(const GemmArgs& a, const uint8_t* red, int red_stride,
                                              const int (*s_raw)[kWave], int64_t m0, int64_t n0, int t) {
  static_assert(BN <= kWave && (32 * BN / 4) % (WAVES * kWave) == 0, "whole passes over the tile");
#pragma unroll
  for (int idx = t; idx < 32 * BN / 4; idx += WAVES * kWave) ksplit_finish_four<MODE, BN, WAVES>(a, red, red_stride, s_raw, m0, n0, idx);
}

// 32 x 32 tiles for K <= 1024 on grids of at most 256 such tiles: the four waves
// of a block split K between them.  A 64 x 64 tile of the kernel above pulls
// 128 KB into one CU's LDS, at 16 - 45 bytes per clock: 1.5 us of M = 128,
// K = N = 1024 on 32 of the chip's 256 CUs.  Here 128 blocks pull 64 KB each, and
// every wave copies only the quarter of K it multiplies itself (its own 16 KB of
// LDS), so it waits for nobody before its MFMAs; the four partial tiles meet in
// LDS behind the block's one barrier, where 256 threads add them, requantise
// four channels of one row each and store.
//
// LDS of wave w:  weights [k-step][k-chunk of the step][32 rows][16 B] (a copy
// instruction moves one k-step: two 16-row blocks of two k-chunks of the packed
// layout), activations [32 rows][256 B] with the slot swizzle of the kernel above.
template <int MODE>
__global__ __launch_bounds__(256) void gemm_i8_ksplit_kernel(GemmArgs a, XLinear xs) {
  constexpr int BM = 32, BN = 32;
  constexpr int kWaveSteps = 8;                    // 32-byte k-steps a wave can hold: 256 bytes of K
  constexpr int kRedPitch = kSplitRedPitch;        // a row of a wave's partial tile
  __shared__ __attribute__((aligned(16))) uint8_t sW[4][kWaveSteps * 1024];
  __shared__ __attribute__((aligned(16))) uint8_t sX[4][BM * 256];
  __shared__ __attribute__((aligned(16))) int s_raw[3][kWave];  // colsum, weight scale, bias as fetched
  static_assert(BM * kRedPitch <= kWaveSteps * 1024, "a wave's partial tile fits over its weights");

  const int t = threadIdx.x, lane = t % kWave;
  const int wave_u = __builtin_amdgcn_readfirstlane(t / kWave);
  const int li = lane & 31, half = lane >> 5;
  const int64_t m0 = static_cast<int64_t>(blockIdx.y) * BM;
  const int64_t n0 = static_cast<int64_t>(blockIdx.x) * BN;
  const int KC = static_cast<int>(a.K >> 4);       // k-chunks (K is a multiple of 16, at most 1024)
  const int S = (KC + 1) >> 1;                     // 32-byte k-steps, at most 32
  const int sp = (S + 3) >> 2;                     // k-steps per wave
  const int s0 = wave_u * sp;                      // this wave's first k-step
  const int mine = S - s0 < sp ? (S - s0 < 0 ? 0 : S - s0) : sp;

  // ---- requests: the tile's per-channel constants (wave 0), then this wave's operands
  if (wave_u == 0) {
    const int64_t n = n0 + lane < a.N ? n0 + lane : a.N - 1;
    const uint32_t np = static_cast<uint32_t>(n + a.n_off);
    lds_dma4(a.colsum, np * 4u, lds_address(&s_raw[0][0]));
    if constexpr (MODE != kOutAcc32) {  // (raw accumulators: the caller passes no scales)
      lds_dma4(a.w_scales, np * static_cast<uint32_t>(a.w_scale_stride) * 4u, lds_address(&s_raw[1][0]));
      lds_dma4(a.bias != nullptr ? a.bias : a.w_scales, a.bias != nullptr ? np * 4u : 0u,
               lds_address(&s_raw[2][0]));
    }
  }
  {
    const int64_t NB = ceil_div(a.N, 16);
    const int64_t nb_last = NB - 1 - n0 / 16;      // a 16-row block past N: clamped, never stored
    const uint8_t* const wtile = a.w_packed + (n0 / 16) * a.w_kchunks * 256;
    const int64_t rb = ((lane >> 4) & 1) < nb_last ? ((lane >> 4) & 1) : nb_last;
    const int kc_last = static_cast<int>(a.w_kchunks) - 1;
    const uint32_t ldsW = lds_address(&sW[wave_u][0]);
#pragma unroll
    for (int j = 0; j < kWaveSteps; ++j) {
      if (j < sp) {
        // (k-steps past the end of K fetch the last chunk again and are not multiplied;
        // an odd last chunk is followed by the zero padding of the packed layout)
        const int kc = 2 * (s0 + j) + half;
        const int kcc = kc < kc_last ? kc : kc_last;
        const uint32_t off = static_cast<uint32_t>((rb * a.w_kchunks + kcc) * 256 + (lane & 15) * 16);
        lds_dma16(wtile, off, ldsW + static_cast<uint32_t>(j) * 1024u);
      }
    }
    const uint8_t* const xtile = xs.x + m0 * xs.ldx;
    const int64_t m_last = a.M - 1 - m0;           // rows past M: clamped, never stored
    const uint32_t ldsX = lds_address(&sX[wave_u][0]);
#pragma unroll
    for (int i = 0; i < BM / 4; ++i) {
      const int r = 4 * i + (lane >> 4);
      const int64_t rc = r < m_last ? r : m_last;
      const int slot = (lane & 15) ^ (r & 15);
      // this wave's 256 bytes of the row; chunks past K: any bytes of the row will do
      const int cc = 2 * s0 + slot;
      const int ccc = cc < KC ? cc : KC - 1;
      if (slot < 2 * sp)
        lds_dma16(xtile, static_cast<uint32_t>(rc * xs.ldx) + static_cast<uint32_t>(ccc) * 16u,
                  ldsX + static_cast<uint32_t>(4 * i) * 256u);
    }
  }

  const v4i xmask = {static_cast<int>(a.x_xor), static_cast<int>(a.x_xor), static_cast<int>(a.x_xor),
                     static_cast<int>(a.x_xor)};
  v16i acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0;
  // this wave's own copies have landed: nobody else's are needed before the MFMAs
  __builtin_amdgcn_s_waitcnt((0 & 15) | ((0 >> 4) << 14) | (7 << 4) | (15 << 8));
  {
    const uint8_t* const wrd = &sW[wave_u][0] + half * 512 + (li >> 4) * 256 + (li & 15) * 16;
    const uint8_t* const xrd = &sX[wave_u][0] + li * 256;
    v4i wf[kWaveSteps], xf[kWaveSteps];
#pragma unroll
    for (int j = 0; j < kWaveSteps; ++j) {
      wf[j] = ld16(wrd + j * 1024);
      xf[j] = ld16(xrd + (((2 * j + half) ^ (li & 15)) << 4));
    }
#pragma unroll
    for (int j = 0; j < kWaveSteps; ++j) {
      const int keep = j < mine ? -1 : 0;
      const v4i xv = (xf[j] ^ xmask) & v4i{keep, keep, keep, keep};
      acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[j], xv, acc, 0, 0, 0);
    }
  }
  // ---- the partial tile of this wave, over its own weights: a lane holds channels
  // 8g + 4 half + j (g, j < 4) of activation row li
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const v4i part = {acc[4 * g], acc[4 * g + 1], acc[4 * g + 2], acc[4 * g + 3]};
    *reinterpret_cast<v4i*>(&sW[wave_u][li * kRedPitch + (8 * g + 4 * half) * 4]) = part;
  }
  __syncthreads();

  ksplit_finish<MODE>(a, &sW[0][0], kWaveSteps * 1024, s_raw, m0, n0, t);
}

// 32 x 32 tiles for K up to 32 * 4 * STEPS bytes (STEPS = 16: 2048, STEPS = 32: 4096)
// whose waves split K, the weights going through registers instead of LDS.
//
// What a CU can have on its way bounds what it pulls per microsecond: LDS holds
// at most 160 KB of copies in flight, which at the latency of cold memory is
// 16 - 45 bytes per clock, and that is what 64 x 64 tiles of a few dozen rows
// x several thousand channels run at (K = N = 4096, M = 64: 14.8 us for 17 MB of
// weights).  Here a wave copies its quarter of the activation rows' K into its own
// LDS (at K = 4096: 32 rows x 1024 bytes, 128 KB per block, L2 hits) and requests
// ALL of its weight fragments at once into registers (STEPS loads of 16 bytes per
// lane, one per MFMA: in the packed layout a fragment is four contiguous 256-byte
// runs), another 128 KB per block in flight, waits for nobody but its own
// requests and multiplies as they arrive.  Partial tiles and epilogue as in the
// kernel above.
// CT = 2 gives a wave two channel tiles (a block 32 rows x 64 channels, for grids
// that 32 x 32 tiles would overfill) and WAVES = 8 splits K eight ways, which keeps
// the weight fragments of two channel tiles within the register file at K up to
// 4096 (four waves with two channel tiles each measured 9.4 us where eight take 7.3).
template <int MODE, int STEPS, int CT = 1, int WAVES = 4>
__global__ __launch_bounds__(WAVES* kWave) void gemm_i8_wstream_kernel(GemmArgs a, XLinear xs) {
  constexpr int BM = 32, BN = 32 * CT;
  constexpr int SEGS = STEPS / 8;                  // 256-byte segments of K per wave
  constexpr int kRedPitch = BN * 4 + 16;
  static_assert(CT * STEPS == 16 || CT * STEPS == 32, "the wait below names the number of weight loads");
  __shared__ __attribute__((aligned(16))) uint8_t sX[WAVES][SEGS * BM * 256];
  __shared__ __attribute__((aligned(16))) int s_raw[3][kWave];  // colsum, weight scale, bias as fetched
  static_assert(BM * kRedPitch <= SEGS * BM * 256, "a wave's partial tile fits over its activations");

  const int t = threadIdx.x, lane = t % kWave;
  const int wave_u = __builtin_amdgcn_readfirstlane(t / kWave);
  const int li = lane & 31, half = lane >> 5;
  const int64_t m0 = static_cast<int64_t>(blockIdx.y) * BM;
  const int64_t n0 = static_cast<int64_t>(blockIdx.x) * BN;
  const int KC = static_cast<int>(a.K >> 4);       // k-chunks (K is a multiple of 16)
  const int S = (KC + 1) >> 1;                     // 32-byte k-steps, at most WAVES * STEPS
  const int sp = (S + WAVES - 1) / WAVES;          // k-steps per wave, at most STEPS
  const int s0 = wave_u * sp;                      // this wave's first k-step
  const int mine = S - s0 < sp ? (S - s0 < 0 ? 0 : S - s0) : sp;

  // ---- requests, oldest first: the tile's per-channel constants (wave 0), this
  // wave's activations (into LDS), this wave's weights (into registers)
  if (wave_u == 0) {
    const int64_t n = n0 + lane < a.N ? n0 + lane : a.N - 1;
    const uint32_t np = static_cast<uint32_t>(n + a.n_off);
    lds_dma4(a.colsum, np * 4u, lds_address(&s_raw[0][0]));
    if constexpr (MODE != kOutAcc32) {  // (raw accumulators: the caller passes no scales)
      lds_dma4(a.w_scales, np * static_cast<uint32_t>(a.w_scale_stride) * 4u, lds_address(&s_raw[1][0]));
      lds_dma4(a.bias != nullptr ? a.bias : a.w_scales, a.bias != nullptr ? np * 4u : 0u,
               lds_address(&s_raw[2][0]));
    }
  }
  {
    const uint8_t* const xtile = xs.x + m0 * xs.ldx;
    const int64_t m_last = a.M - 1 - m0;           // rows past M: clamped, never stored
    const uint32_t ldsX = lds_address(&sX[wave_u][0]);
#pragma unroll
    for (int seg = 0; seg < SEGS; ++seg) {
      if (seg * 8 < sp) {                          // (uniform: segments past this wave's share stay unwritten)
#pragma unroll
        for (int i = 0; i < BM / 4; ++i) {
          const int r = 4 * i + (lane >> 4);
          const int64_t rc = r < m_last ? r : m_last;
          const int slot = (lane & 15) ^ (r & 15);
          // chunks past K: any bytes of the row will do, they meet a zeroed operand or zero weights
          const int cc = 2 * s0 + 16 * seg + slot;
          const int ccc = cc < KC ? cc : KC - 1;
          lds_dma16(xtile, static_cast<uint32_t>(rc * xs.ldx) + static_cast<uint32_t>(ccc) * 16u,
                    ldsX + static_cast<uint32_t>(seg * BM + 4 * i) * 256u);
        }
      }
    }
  }
  v4i wf[CT][STEPS];
  {
    const int64_t NB = ceil_div(a.N, 16);
    const int64_t nb_last = NB - 1 - n0 / 16;      // 16-row blocks past N: clamped, never stored
    const int kc_last = static_cast<int>(a.w_kchunks) - 1;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      const int64_t rb0 = 2 * ct + ((lane >> 4) & 1);
      const int64_t rb = rb0 < nb_last ? rb0 : nb_last;
      const uint8_t* const wlane = a.w_packed + ((n0 / 16 + rb) * a.w_kchunks) * 256 + (lane & 15) * 16;
#pragma unroll
      for (int j = 0; j < STEPS; ++j) {
        // (k-steps past this wave's share fetch its last one again and are not multiplied;
        // an odd last chunk is followed by the zero padding of the packed layout)
        const int step = s0 + (j < sp ? j : sp - 1);
        const int kc = 2 * step + half;
        const int kcc = kc < kc_last ? kc : kc_last;
        wf[ct][j] = *reinterpret_cast<const v4i*>(wlane + static_cast<int64_t>(kcc) * 256);
      }
    }
  }

  const v4i xmask = {static_cast<int>(a.x_xor), static_cast<int>(a.x_xor), static_cast<int>(a.x_xor),
                     static_cast<int>(a.x_xor)};
  v16i acc[CT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[ct][r] = 0;
  // The copies into LDS are older than the weight loads and requests return in
  // order: at most as many requests outstanding as there are weight loads means the
  // activations have landed.  (An asm statement that clobbers memory: the compiler
  // may neither sink a weight load below it nor hoist an LDS read above it.)
  if constexpr (CT * STEPS == 16) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
  else asm volatile("s_waitcnt vmcnt(32)" ::: "memory");
  {
    const uint8_t* const xrd = &sX[wave_u][0] + li * 256;
#pragma unroll
    for (int j = 0; j < STEPS; ++j) {
      if (j / 8 * 8 < sp) {                        // (uniform, per segment)
        const v4i xf = ld16(xrd + (j / 8) * (BM * 256) + (((2 * (j % 8) + half) ^ (li & 15)) << 4));
        const int keep = j < mine ? -1 : 0;
        const v4i xv = (xf ^ xmask) & v4i{keep, keep, keep, keep};
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
          acc[ct] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[ct][j], xv, acc[ct], 0, 0, 0);
      }
    }
  }
  // ---- the partial tile of this wave, over its own activations: a lane holds
  // channels 32 ct + 8g + 4 half + j (g, j < 4) of activation row li
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const v4i part = {acc[ct][4 * g], acc[ct][4 * g + 1], acc[ct][4 * g + 2], acc[ct][4 * g + 3]};
      *reinterpret_cast<v4i*>(&sX[wave_u][li * kRedPitch + (32 * ct + 8 * g + 4 * half) * 4]) = part;
    }
  }
  __syncthreads();
  ksplit_finish<MODE, BN, WAVES>(a, &sX[0][0], SEGS * BM * 256, s_raw, m0, n0, t);
}

}  // namespace tmq
