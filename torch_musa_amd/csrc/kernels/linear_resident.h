// quantized::linear for up to 64 activation rows against many output channels (gfx950):
// one block per CU keeps the activations in LDS and streams the weights of one group
// of 16 channels after the other through its sixteen waves.
//
// The weight-streaming kernel of linear.hip gives every group of 16 channels a block of
// its own, and every block fetches all M x K activation bytes again from the L2s: at
// M = 16 those are as many bytes as the block's weights, and with more blocks than the
// chip holds at once each one starts its weight stream from nothing.  Here
//   * the block stages the activations once, already in MFMA operand order
//     ([k-block][16-byte piece][row][16 B], zeros past K: a wave's B operand of v_mfma_i32_16x16x64_i8
//     is four contiguous runs of 256 bytes) and with the sign flip of unsigned
//     activations applied, and the requantisation constants of every channel it owns
//     (accumulator start, multiplier, bias term) next to them;
//   * block b owns the channel groups b, b + G, b + 2 G, ...; the sixteen waves split
//     the 64-byte k-blocks of a group (wave w takes k-blocks w, w + 16, ...) and a wave's
//     loads run kDepth k-blocks ahead of its multiplications, across group boundaries,
//     so the stream never drains;
//   * the waves' partial sums of a group meet in LDS (atomic adds into one of two slots,
//     used in turn), one barrier per group, then one wave -- a different one each
//     group -- requantises and stores while the others go on multiplying.  The barrier
//     carries no memory fence: only the LDS counter is waited for, the weight loads in
//     flight stay in flight.
// D[i][j] of v_mfma_i32_16x16x64_i8: lane l, register r -> i = 4 (l / 16) + r (channel),
// j = l % 16 (activation row).
//
// HELD > 0: the dynamically quantized linear in one launch (float rows in, float out, up to
// 16 rows and HELD x 4096 values): the block reads the float rows instead of codes -- every
// thread holds HELD groups of four values in registers --, reduces their range, one thread
// derives the parameters (ChooseQuantizationParams), and the held values are quantized into
// the same LDS operand layout, product and zero point rounded once, as PyTorch's CPU
// quantized::linear_dynamic does while packing.  All of it runs under the latency of the
// first weight requests; the stream that follows is the same.
#pragma once

#include "gemm_i8_core.h"
#include "qparams.h"

namespace tmq {

constexpr int kResidentWaves = 16;
constexpr int kResidentThreads = kResidentWaves * kWave;
constexpr int kResidentDepth = 8;                 // k-blocks in flight per wave: 128 KB per block (12 and 16: no faster)
constexpr int kResidentMaxGroups = 64;            // channel groups a block of 16 waves can own (their constants sit in LDS)
constexpr int kResidentXBytes = 128 * 1024;       // 16 MG x K activation bytes

// LDS barrier of the block without a fence: every wave's LDS operations so far are
// complete before it arrives, global loads stay outstanding.
__device__ __forceinline__ void resident_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

template <int MODE, int MG, int W = kResidentWaves, int HELD = 0>
__global__ __launch_bounds__(W * kWave, 4) void linear_resident_kernel(GemmArgs a, XLinear xs, const float* __restrict__ xf,
                                                                       int64_t ldxf, int reduce_range) {
  static_assert(HELD == 0 || (MODE == kOutF32 && MG == 1 && W == kResidentWaves), "the dynamic form: float output, 16 rows");
  constexpr int D = kResidentDepth;
  constexpr int kXBytes = kResidentXBytes / kResidentWaves * W;  // (eight waves: two blocks share a CU)
  constexpr int kThreads = W * kWave;
  constexpr int kGroups = kThreads / 16;       // channel groups a block can own: a thread per channel stages the constants
  __shared__ __attribute__((aligned(16))) uint8_t s_x[kXBytes];
  __shared__ __attribute__((aligned(16))) int s_sum[2][MG][4][kWave];
  __shared__ __attribute__((aligned(16))) int s_acc0[kGroups * 16];
  __shared__ __attribute__((aligned(16))) float s_mult[kGroups * 16];
  __shared__ __attribute__((aligned(16))) float s_bdiv[kGroups * 16];
  __shared__ float s_bmul;
  __shared__ float s_mn[W], s_mx[W];
  __shared__ float s_scale, s_inv, s_zp;

  const int t = threadIdx.x, lane = t % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(t / kWave);
  const int lr = lane & 15, lc = lane >> 4;
  const int K = static_cast<int>(a.K), M = static_cast<int>(a.M), N = static_cast<int>(a.N);
  const int KB = (K + 63) >> 6;                    // 64-byte k-blocks
  const int KC = K >> 4;                           // 16-byte chunks (K is a multiple of 16)
  const int NG = (N + 15) >> 4;                    // channel groups
  const int G = static_cast<int>(gridDim.x), b = static_cast<int>(blockIdx.x);
  const int ngb = (NG - b + G - 1) / G;            // groups of this block (G <= NG: at least one)
  const int U = (KB + W - 1) / W;  // k-blocks of a group per wave
  const int KBP = U * W;              // k-blocks in LDS: those past K hold zeros
  const int Q = ngb * U;                           // this wave's stream of (group, k-block) units
  const int64_t slab = a.w_kchunks * 256;          // packed bytes of one channel group

  // ---- requests, oldest first: the activations (L2) ...
  // piece (mg, kb) = 16 rows x 64 bytes: lane -> row lane / 4, 16-byte chunk lane % 4
  // (four lanes ask for one cache line); pieces are dealt round-robin to the waves
  constexpr int kXPieces = HELD > 0 ? 1 : kXBytes / 1024 / W;  // per wave, at most
  v4i xr[kXPieces];
  constexpr int kHeldN = HELD > 0 ? HELD : 1;
  v4f held[kHeldN];
  const int sr = lane >> 2, sp = lane & 3;
  const int k4 = K >> 2, total4 = M * k4;          // (dynamic form) groups of four float values
  if constexpr (HELD > 0) {
#pragma unroll
    for (int u = 0; u < HELD; ++u) {
      const int e = t + u * kThreads;
      const int ec = e < total4 ? e : 0;           // unconditional loads keep the load counter exact
      const int row = ec / k4, c4 = ec - row * k4;
      held[u] = *reinterpret_cast<const v4f*>(xf + row * ldxf + c4 * 4);
    }
  } else {
#pragma unroll
    for (int j = 0; j < kXPieces; ++j) {
      const int p = wave + W * j;
      if (p < MG * KBP) {
        const int kb = p / MG, mg = p - kb * MG;
        const int row = mg * 16 + sr, c = kb * 4 + sp;
        const bool ok = row < M && c < KC;
        xr[j] = ld16(xs.x + (ok ? static_cast<int64_t>(row) * xs.ldx + c * 16 : 0));
      }
    }
  }
  // ... the constants of this block's channels (cold): thread -> group slot t / 16, channel t % 16
  const int cslot = t >> 4, cch = t & 15;
  int c_cs = 0;
  float c_ws = 1.f, c_b = 0.f;
  {
    const int n = (b + cslot * G) * 16 + cch;
    const int np = cslot < ngb && n < N ? n : 0;
    c_cs = a.colsum[np];
    if constexpr (MODE != kOutAcc32) {  // (raw accumulators: the caller passes no scales)
      c_ws = a.w_scales[np * a.w_scale_stride];
      const float* const bsrc = a.bias != nullptr ? a.bias : a.w_scales;  // a load that always has an address
      const float bv = bsrc[a.bias != nullptr ? np : 0];
      c_b = a.bias != nullptr ? bv : 0.f;
    }
  }
  // ... and the first kDepth k-blocks of the weight stream (memory).  The load cursor
  // (group li, k-block slot lu) runs kDepth units ahead of the multiply cursor.
  const uint8_t* const wlane = a.w_packed + lane * 16;
  int li = 0, lu = 0;
  auto next_weights = [&]() {
    const int kb = wave + W * lu;
    const int kbc = kb < KB ? kb : KB - 1;         // (slots past K: any k-block, it meets zeros)
    const v4i w = __builtin_nontemporal_load(
        reinterpret_cast<const v4i*>(wlane + static_cast<int64_t>(b + li * G) * slab + static_cast<int64_t>(kbc) * 1024));
    if (++lu == U) {
      lu = 0;
      ++li;
    }
    return w;
  };
  v4i wf[D];
#pragma unroll
  for (int j = 0; j < D; ++j)
    if (j < Q) wf[j] = next_weights();

  // ---- activations into LDS: piece (mg, kb), chunk c of row r -> ((4 kb + c) * 16 MG + 16 mg + r) * 16
  for (int i = t; i < 2 * MG * 4 * kWave; i += kThreads) (&s_sum[0][0][0][0])[i] = 0;
  XQuant xq;
  if constexpr (HELD > 0) {
    // rows past M and bytes past K stay zero: clear the area, then write the codes over it
    for (int i = t; i < KBP * 64; i += kThreads) *reinterpret_cast<v4i*>(&s_x[i * 16]) = v4i{0, 0, 0, 0};
    float mn = __builtin_inff(), mx = -__builtin_inff();
#pragma unroll
    for (int u = 0; u < HELD; ++u) {
      if (t + u * kThreads < total4) {
        const v4f v = held[u];
        mn = fminf(fminf(mn, v.x), fminf(v.y, fminf(v.z, v.w)));
        mx = fmaxf(fmaxf(mx, v.x), fmaxf(v.y, fmaxf(v.z, v.w)));
      }
    }
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
      mn = fminf(mn, __shfl_xor(mn, off, kWave));
      mx = fmaxf(mx, __shfl_xor(mx, off, kWave));
    }
    if (lane == 0) {
      s_mn[wave] = mn;
      s_mx[wave] = mx;
    }
    resident_barrier();
    if (t == 0) {
#pragma unroll
      for (int w = 1; w < W; ++w) {
        mn = fminf(mn, s_mn[w]);
        mx = fmaxf(mx, s_mx[w]);
      }
      double sc;
      int32_t zp;
      choose_qparams(mn, mx, 0, 255, reduce_range != 0, &sc, &zp);
      const float scf = static_cast<float>(sc);
      s_scale = scf;
      s_inv = 1.0f / scf;  // IEEE division, as the separate quantize kernels
      s_zp = static_cast<float>(zp);
    }
    resident_barrier();
    const float inv = s_inv, zp_f = s_zp;
#pragma unroll
    for (int u = 0; u < HELD; ++u) {
      const int e = t + u * kThreads;
      if (e < total4) {
        const int row = e / k4, c4 = e - row * k4;
        const v4f v = held[u];
        uint32_t q = 0;
        const float f[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          float r = __builtin_rintf(__builtin_fmaf(f[j], inv, zp_f));
          r = fminf(fmaxf(r, 0.f), 255.f);
          q |= static_cast<uint32_t>(static_cast<int>(r)) << (8 * j);
        }
        // bytes 4 c4 .. 4 c4 + 3 of the row: k-block c4 / 16, chunk (c4 / 4) % 4, byte 4 (c4 % 4) of the chunk
        *reinterpret_cast<uint32_t*>(&s_x[((c4 >> 2) * 16 + row) * 16 + (c4 & 3) * 4]) = q ^ 0x80808080u;
      }
    }
    xq = XQuant{s_scale, 128 - static_cast<int>(zp_f)};
  } else {
    const int xor_word = static_cast<int>(a.x_xor);
    const v4i xmask = {xor_word, xor_word, xor_word, xor_word};
#pragma unroll
    for (int j = 0; j < kXPieces; ++j) {
      const int p = wave + W * j;
      if (p < MG * KBP) {
        const int kb = p / MG, mg = p - kb * MG;
        const bool ok = mg * 16 + sr < M && kb * 4 + sp < KC;
        const v4i v = ok ? (xr[j] ^ xmask) : v4i{0, 0, 0, 0};
        *reinterpret_cast<v4i*>(&s_x[(((kb * 4 + sp) * MG + mg) * 16 + sr) * 16]) = v;
      }
    }
    xq = x_quant(a);
  }
  // ---- the channels' constants, ready for the epilogue
  {
    float mult = 0.f, bdiv = 0.f, bmul = 1.f;
    if constexpr (MODE == kOutF32) {
      mult = xq.scale * c_ws;
      bdiv = c_b;
    } else if constexpr (MODE != kOutAcc32) {
      const float atw = xq.scale * c_ws;
      mult = atw / a.out_scale;
      bdiv = a.bias != nullptr ? bias_term(a.w_scale_stride == 0, c_b, atw) : 0.f;
      bmul = bias_mul(a.w_scale_stride == 0, atw);  // (per tensor: the same for every channel)
    }
    s_acc0[t] = xq.coef * c_cs;
    s_mult[t] = mult;
    s_bdiv[t] = bdiv;
    if (t == 0) s_bmul = bmul;
  }
  resident_barrier();

  // ---- the stream
  v4i acc2[MG][2];  // two accumulators per row group, used in turn
#pragma unroll
  for (int mg = 0; mg < MG; ++mg) acc2[mg][0] = acc2[mg][1] = v4i{0, 0, 0, 0};
  const uint8_t* const xop = &s_x[(lc * MG * 16 + lr) * 16];   // + kb * MG * 1024 + mg * 256
  const int fm = lane >> 2, fg = lane & 3;         // finishing wave: lane -> row within a group, four channels

  auto finish_group = [&](int gi) {
    const int par = gi & 1;
#pragma unroll
    for (int mg = 0; mg < MG; ++mg) {
      const v4i acc = acc2[mg][0] + acc2[mg][1];
      acc2[mg][0] = acc2[mg][1] = v4i{0, 0, 0, 0};
#pragma unroll
      for (int r = 0; r < 4; ++r)
        __hip_atomic_fetch_add(&s_sum[par][mg][r][lane], acc[r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    resident_barrier();
    // One wave finishes the group and clears the slot.  The slot is next added to after
    // the following group's barrier, which this wave reaches only after its clears.
    if (wave != (gi & (W - 1))) return;
    const int64_t n = static_cast<int64_t>(b + gi * G) * 16 + 4 * fg;
    const v4i add = *reinterpret_cast<const v4i*>(&s_acc0[gi * 16 + 4 * fg]);
    const v4f mult = *reinterpret_cast<const v4f*>(&s_mult[gi * 16 + 4 * fg]);
    const v4f bdiv = *reinterpret_cast<const v4f*>(&s_bdiv[gi * 16 + 4 * fg]);
    const float bmul = s_bmul;
#pragma unroll
    for (int mg = 0; mg < MG; ++mg) {
      int raw[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {  // channel 4 fg + j of row fm: register j of lane 16 fg + fm
        raw[j] = s_sum[par][mg][j][16 * fg + fm] + add[j];
        s_sum[par][mg][j][16 * fg + fm] = 0;
      }
      const int64_t m = mg * 16 + fm;
      if (m >= a.M || n >= a.N) continue;
      if constexpr (MODE == kOutAcc32) {
        int32_t* dst = static_cast<int32_t*>(a.y) + m * a.ldy + n;
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (n + j < a.N) dst[j] = raw[j];
      } else if constexpr (MODE == kOutF32) {
        store_f32x4(a, m, n, raw, mult, bdiv);
      } else {
        const uint32_t packed = requant4<MODE>(raw, bdiv, bmul, mult, a.zp_f, a.lo_f, a.hi_f);
        uint8_t* dst = static_cast<uint8_t*>(a.y) + m * a.ldy + n;
        if (n + 3 < a.N && (a.ldy & 3) == 0 && (reinterpret_cast<uintptr_t>(a.y) & 3) == 0) {
          *reinterpret_cast<uint32_t*>(dst) = packed;
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (n + j < a.N) dst[j] = static_cast<uint8_t>(packed >> (8 * j));
        }
      }
    }
  };

  int ci = 0, cu = 0;  // multiply cursor: group, k-block slot
  // unit j of a run of kDepth: multiply with wf[j], refill it with the unit kDepth further on
  auto unit = [&](int j, bool refill) {
    const int kb = wave + W * cu;
#pragma unroll
    for (int mg = 0; mg < MG; ++mg) {
      const v4i xv = ld16(xop + kb * (MG * 1024) + mg * 256);
      acc2[mg][j & 1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[j], xv, acc2[mg][j & 1], 0, 0, 0);
    }
    if (refill) wf[j] = next_weights();
    if (++cu == U) {
      cu = 0;
      finish_group(ci);
      ++ci;
    }
  };
  // Runs whose every unit has a successor kDepth further on issue their loads without a
  // condition, so that the count of loads in flight the waits are derived from is exact;
  // the last two runs decide per unit.
  int q0 = 0;
  for (; q0 + 2 * D <= Q; q0 += D) {
#pragma unroll
    for (int j = 0; j < D; ++j) unit(j, true);
  }
  for (; q0 < Q; q0 += D) {
#pragma unroll
    for (int j = 0; j < D; ++j) {
      if (q0 + j >= Q) break;
      unit(j, q0 + j + D < Q);
    }
  }
}

}  // namespace tmq
