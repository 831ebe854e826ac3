// int8 MFMA GEMM on 64 x 64 tiles for a few hundred rows against 2048 < K <= 4096
// (gfx950): eight waves split K, the weights go through registers, the activations
// through a ring in LDS that belongs to the wave.
//
// What bounds these shapes is what a CU can pull from the L2s (about 45 bytes per
// clock) and how much of it is on its way at once.  A 64 x 64 tile needs
// (64 + 64) x K bytes; the pipelined tiles of gemm_i8_core.h walk them one 64-byte
// stage after the other behind a barrier per stage and run at half that rate.
// Here a wave owns an eighth of K (at most 512 bytes, 16 k-steps of 32) and
// nobody waits for anybody before the partial tiles meet:
//   * all of the wave's weight fragments -- 2 channel tiles x 16 k-steps, one
//     16-byte load per lane and MFMA, 128 VGPRs -- are requested at the start
//     (32 KB per wave, 256 KB per block in flight);
//   * the wave's activation rows pass through a ring of four stages (a stage is
//     64 rows x 64 bytes of K, two k-steps) filled by direct global -> LDS copies:
//     stages 0..3 are requested before the weights, stage s + 4 into the slot of
//     stage s as soon as that has been read;
//   * requests return in the order issued, so every wait is a count of the younger
//     requests that may still be outstanding, and those counts are constants:
//     44 for an activation stage of the first round (12 - 4 s copies of stages
//     s + 1..3, 32 weight loads, 4 s copies of stages 4..s + 3), 30 and 28 for the
//     weight fragments of its two k-steps, 4 (7 - s) for a stage of the second
//     round (every weight load is older than it).
// Loads and copies are written as asm statements and every wait names the registers
// it releases, so that the compiler can neither move a use above its wait nor
// count the requests differently; the build checks that the kernel keeps every
// fragment in registers (no scratch).
// The eight partial tiles are written over the rings, added by all 512 threads,
// requantised and stored (ksplit_finish_four of gemm_i8_onepass.h).
#pragma once

#include "gemm_i8_onepass.h"

namespace tmq {

constexpr int kWringMaxK = 4096;
constexpr int kWringThreads = 512;

__device__ __forceinline__ v4i wring_load16(const uint8_t* base, uint32_t off) {
  v4i v;
  asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(v) : "v"(off), "s"(base) : "memory");
  return v;
}

// s_waitcnt vmcnt(N) that hands out the two fragments it releases.
template <int N>
__device__ __forceinline__ void wring_wait_pair(v4i& a, v4i& b) {
  static_assert(N >= 0 && N < 64, "load counter range");
  if constexpr (N == 30) asm volatile("s_waitcnt vmcnt(30)" : "+v"(a), "+v"(b)::"memory");
  else if constexpr (N == 28) asm volatile("s_waitcnt vmcnt(28)" : "+v"(a), "+v"(b)::"memory");
  else static_assert(N == 30 || N == 28, "the two counts of the first round");
}

template <int MODE>
__global__ __launch_bounds__(kWringThreads) void gemm_i8_wring_kernel(GemmArgs a, XLinear xs) {
  constexpr int BM = 64, BN = 64, WAVES = 8;
  constexpr int STEPS = 16;                        // k-steps of 32 bytes a wave can hold
  constexpr int STAGES = STEPS / 2, RING = 4;
  constexpr int kStageBytes = BM * 64;             // 4 KB: 64 rows x 64 bytes of K
  constexpr int kRedPitch = BN * 4 + 16;
  constexpr int kWaveLds = BM * kRedPitch;         // 17 408 B: the partial tile, over the ring
  static_assert(RING * kStageBytes <= kWaveLds, "the ring lies inside the wave's partial-tile area");
  __shared__ __attribute__((aligned(16))) uint8_t sX[WAVES][kWaveLds];
  __shared__ __attribute__((aligned(16))) int s_raw[3][kWave];  // colsum, weight scale, bias as fetched

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

  // ---- requests, oldest first: the tile's per-channel constants (wave 0) ...
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
  // ---- ... this wave's activation stages.  A copy moves 16 rows x 64 bytes: lane l
  // brings row l / 4 its 16-byte chunk (l % 4) ^ swz, swz = (row / 4) % 4 = (l / 16) % 4
  // for every group of 16 rows, into position l % 4 of the row (the slot swizzle of
  // gemm_i8_core.h: a column of 32 rows reads conflict-free).
  const uint8_t* const xtile = xs.x + m0 * xs.ldx;
  const uint32_t ldsX = lds_address(&sX[wave_u][0]);
  uint32_t xrow[BM / 16];
  {
    const int64_t m_last = a.M - 1 - m0;           // rows past M: clamped, never stored
#pragma unroll
    for (int i = 0; i < BM / 16; ++i) {
      const int r = 16 * i + (lane >> 2);
      xrow[i] = static_cast<uint32_t>((r < m_last ? r : m_last) * xs.ldx);
    }
  }
  const int xchunk = (lane & 3) ^ ((lane >> 4) & 3);
  auto copy_stage = [&](int s) {                   // stage s of this wave into ring slot s % RING
    // (chunks past K: any bytes of the row will do, they meet a zeroed operand or zero weights)
    const int cc = 2 * (s0 + 2 * s) + xchunk;
    const uint32_t koff = static_cast<uint32_t>(cc < KC ? cc : KC - 1) * 16u;
#pragma unroll
    for (int i = 0; i < BM / 16; ++i)
      lds_dma16(xtile, xrow[i] + koff, ldsX + static_cast<uint32_t>((s % RING) * kStageBytes + i * 1024));
  };
#pragma unroll
  for (int s = 0; s < RING; ++s) copy_stage(s);

  // ---- ... and all of its weight fragments: k-step j of channel tile ct is one
  // 16-byte load per lane (four contiguous 256-byte runs of the packed layout)
  v4i wf[2][STEPS];
  {
    const int64_t NB = ceil_div(a.N, 16);
    const int64_t nb_last = NB - 1 - n0 / 16;      // 16-row blocks past N: clamped, never stored
    const int kc_last = static_cast<int>(a.w_kchunks) - 1;
    const uint8_t* const wtile = a.w_packed + (n0 / 16) * a.w_kchunks * 256;
    uint32_t wlane[2];
#pragma unroll
    for (int ct = 0; ct < 2; ++ct) {
      const int64_t rb0 = 2 * ct + ((lane >> 4) & 1);
      const int64_t rb = rb0 < nb_last ? rb0 : nb_last;
      wlane[ct] = static_cast<uint32_t>(rb * a.w_kchunks * 256 + (lane & 15) * 16);
    }
#pragma unroll
    for (int j = 0; j < STEPS; ++j) {
      // (k-steps past this wave's share fetch its last one again and are not multiplied;
      // an odd last chunk is followed by the zero padding of the packed layout)
      const int step = s0 + (j < sp ? j : sp - 1);
      const int kc = 2 * step + half;
      const uint32_t koff = static_cast<uint32_t>(kc < kc_last ? kc : kc_last) * 256u;
      wf[0][j] = wring_load16(wtile, wlane[0] + koff);
      wf[1][j] = wring_load16(wtile, wlane[1] + koff);
    }
  }

  const v4i xmask = {static_cast<int>(a.x_xor), static_cast<int>(a.x_xor), static_cast<int>(a.x_xor),
                     static_cast<int>(a.x_xor)};
  v16i acc[2][2];  // [channel tile][row tile]
#pragma unroll
  for (int ct = 0; ct < 2; ++ct)
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[ct][rt][r] = 0;

  // a lane's fragment of row tile rt, k-step ks of a stage: row 32 rt + li, chunk 2 ks + half
  const uint8_t* const xrd = &sX[wave_u][0] + li * 64;
  const int xswz = (li >> 2) & 3;
  auto stage_fragments = [&](int s, v4i (&xf)[2][2]) {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
      for (int rt = 0; rt < 2; ++rt)
        xf[ks][rt] = ld16(xrd + (s % RING) * kStageBytes + rt * (32 * 64) + (((2 * ks + half) ^ xswz) << 4));
  };
  auto multiply = [&](int j, const v4i& w0, const v4i& w1, const v4i (&xf)[2]) {
    const int keep = j < mine ? -1 : 0;
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
      const v4i xv = (xf[rt] ^ xmask) & v4i{keep, keep, keep, keep};
      acc[0][rt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(w0, xv, acc[0][rt], 0, 0, 0);
      acc[1][rt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(w1, xv, acc[1][rt], 0, 0, 0);
    }
  };

  // ---- first round: stages 0..3 from the ring as filled above; each slot is refilled
  // with stage s + 4 when its fragments are in registers
#pragma unroll
  for (int s = 0; s < RING; ++s) {
    asm volatile("s_waitcnt vmcnt(44)" ::: "memory");   // stage s has landed (see the file header)
    v4i xf[2][2];
    stage_fragments(s, xf);
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(xf[0][0]), "+v"(xf[0][1]), "+v"(xf[1][0]), "+v"(xf[1][1])::"memory");
    wring_wait_pair<30>(wf[0][2 * s], wf[1][2 * s]);
    multiply(2 * s, wf[0][2 * s], wf[1][2 * s], xf[0]);
    wring_wait_pair<28>(wf[0][2 * s + 1], wf[1][2 * s + 1]);
    multiply(2 * s + 1, wf[0][2 * s + 1], wf[1][2 * s + 1], xf[1]);
    copy_stage(s + RING);
  }
  // ---- second round: every weight load is older than these stages
#pragma unroll
  for (int s = RING; s < STAGES; ++s) {
    if (s == 4) asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
    else if (s == 5) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    else if (s == 6) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    v4i xf[2][2];
    stage_fragments(s, xf);
    // (the weights of these stages landed before the stage did: name them, so that no
    // use of theirs can be scheduled above the wait)
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(xf[0][0]), "+v"(xf[0][1]), "+v"(xf[1][0]), "+v"(xf[1][1]), "+v"(wf[0][2 * s]),
                   "+v"(wf[1][2 * s]), "+v"(wf[0][2 * s + 1]), "+v"(wf[1][2 * s + 1])::"memory");
    multiply(2 * s, wf[0][2 * s], wf[1][2 * s], xf[0]);
    multiply(2 * s + 1, wf[0][2 * s + 1], wf[1][2 * s + 1], xf[1]);
  }

  // ---- the partial tile of this wave, over its own ring: a lane holds channels
  // 32 ct + 8 g + 4 half + j (g, j < 4) of row 32 rt + li
#pragma unroll
  for (int ct = 0; ct < 2; ++ct)
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const v4i part = {acc[ct][rt][4 * g], acc[ct][rt][4 * g + 1], acc[ct][rt][4 * g + 2], acc[ct][rt][4 * g + 3]};
        *reinterpret_cast<v4i*>(&sX[wave_u][(32 * rt + li) * kRedPitch + (32 * ct + 8 * g + 4 * half) * 4]) = part;
      }
  __syncthreads();
#pragma unroll
  for (int idx = t; idx < BM * BN / 4; idx += kWringThreads)
    ksplit_finish_four<MODE, BN, WAVES>(a, &sX[0][0], kWaveLds, s_raw, m0, n0, idx);
}

}  // namespace tmq
