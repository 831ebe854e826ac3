// quantized::linear for gfx950: weight re-tiling, the MFMA GEMM dispatch, a
// weight-streaming kernel for decode-sized batches, and a plain kernel for
// shapes the vector paths do not take (K not a multiple of 16, unaligned rows).
#include <atomic>

#include "gemm_i8_core.h"
#include "gemm_i8_onepass.h"
#include "gemm_i8_persistent.h"
#include "gemm_i8_wring.h"
#include "linear_resident.h"
#include "qparams.h"

// Layout that non-C++ bindings rely on (natural alignment, x86-64).
static_assert(sizeof(tmq_linear_desc) == 144, "tmq_linear_desc layout changed");
static_assert(sizeof(tmq_qparams) == 16, "tmq_qparams layout changed");

namespace tmq {
namespace {

constexpr int64_t kKPad = 128;  // packed k extent is a multiple of this

__host__ __device__ inline int64_t packed_kchunks(int64_t K) { return (K + kKPad - 1) / kKPad * (kKPad / 16); }

// ---------------------------------------------------------------------------
// prepack: one thread per 16-byte packed chunk (nb, kc, r)
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void prepack_kernel(const int8_t* __restrict__ w, int64_t N,
                                                      int64_t K, int64_t ldw, int64_t KC,
                                                      int64_t total, bool vec,
                                                      uint8_t* __restrict__ packed) {
  const int64_t id = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (id >= total) return;
  const int r = static_cast<int>(id & 15);
  const int64_t kc = (id >> 4) % KC;
  const int64_t nb = (id >> 4) / KC;
  const int64_t n = nb * 16 + r, k0 = kc * 16;
  v4i out = {0, 0, 0, 0};
  if (n < N && k0 < K) {
    const int8_t* src = w + n * ldw + k0;
    if (vec && k0 + 16 <= K) {
      out = ld16(src);
    } else {
      uint32_t words[4] = {0, 0, 0, 0};
      for (int b = 0; b < 16 && k0 + b < K; ++b)
        words[b >> 2] |= static_cast<uint32_t>(static_cast<uint8_t>(src[b])) << (8 * (b & 3));
      out = v4i{static_cast<int>(words[0]), static_cast<int>(words[1]), static_cast<int>(words[2]),
                static_cast<int>(words[3])};
    }
  }
  *reinterpret_cast<v4i*>(packed + id * 16) = out;
}

__global__ __launch_bounds__(256) void unpack_kernel(const uint8_t* __restrict__ packed, int64_t N,
                                                     int64_t K, int64_t ldw, int64_t KC,
                                                     int8_t* __restrict__ w) {
  const int64_t id = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (id >= N * K) return;
  const int64_t n = id / K, k = id % K;
  w[n * ldw + k] = static_cast<int8_t>(packed[(((n >> 4) * KC + (k >> 4)) * 16 + (n & 15)) * 16 + (k & 15)]);
}

// colsum[n] = sum_k W[n][k]; one wavefront per weight row.
__global__ __launch_bounds__(256) void colsum_kernel(const int8_t* __restrict__ w, int64_t N,
                                                     int64_t K, int64_t ldw, bool vec,
                                                     int32_t* __restrict__ colsum) {
  const int lane = threadIdx.x % kWave;
  const int64_t n = static_cast<int64_t>(blockIdx.x) * (256 / kWave) + threadIdx.x / kWave;
  if (n >= N) return;
  const int8_t* row = w + n * ldw;
  int s = 0;
  int64_t k = 0;
  if (vec) {
    for (int64_t c = lane; c < K / 16; c += kWave) {
      const v4i v = ld16(row + c * 16);
      s = __builtin_amdgcn_sdot4(v.x, 0x01010101, s, false);
      s = __builtin_amdgcn_sdot4(v.y, 0x01010101, s, false);
      s = __builtin_amdgcn_sdot4(v.z, 0x01010101, s, false);
      s = __builtin_amdgcn_sdot4(v.w, 0x01010101, s, false);
    }
    k = K / 16 * 16;
  }
  for (int64_t i = k + lane; i < K; i += kWave) s += row[i];
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) s += __shfl_xor(s, off, kWave);
  if (lane == 0) colsum[n] = s;
}

// ---------------------------------------------------------------------------
// Decode-sized batches (M <= 16): the weight is read once, straight from HBM
// into MFMA operand registers (the packed layout is the 16x16x64 operand
// order), activations come from L2.  One block per 16 output channels, its
// eight waves split K and reduce through LDS.
//   D[i][j] of v_mfma_i32_16x16x64_i8: lane l, register r -> i = 4*(l/16)+r
//   (channel), j = l%16 (activation row).
// ---------------------------------------------------------------------------
constexpr int kDecodeWaves = 8;
constexpr int kDecodeMaxRows = 64;
constexpr int kDecodeRowsAuto = 16;  // up to here the automatic choice always streams the weights
// MG = groups of 16 activation rows (M <= 16 * MG): the weight operands are
// loaded once and multiplied with every group.
//
// The 14 dwords in front of GemmArgs are everything the kernel's loads need.  The
// library is compiled with kernel-argument preloading, which hands up to 14
// leading scalar dwords of a kernel to its waves in SGPRs at launch, so the
// requests leave without waiting for a read of the argument buffer; the rest of
// the arguments is fetched under the weight stream.  The finishing threads'
// per-channel constants are requested first (cold, and memory serves requests
// in the order issued), then each k-block's weights (HBM) and activations (L2).
// Measured at K = N = 4096 in a replayed graph of 40 cold weights: 5.25 us at
// M = 1, of which 1.9 us are what an empty kernel costs there, a kernel that
// only reads the 16.8 MB takes 4.1 us, and the one that also stores 4 KB of
// results 4.5 us (the store's acknowledgement ends the kernel); one or two
// accumulators and 4 / 8 / 16 waves all stay within 0.1 us.
// flags: bits 0-7 M, bit 8 per-channel weight scales, bit 9 unsigned activations.
template <int MODE, int MG>
__global__ __launch_bounds__(kDecodeWaves* kWave) void linear_decode_kernel(
    const uint8_t* __restrict__ w_packed, const uint8_t* __restrict__ x, const int32_t* __restrict__ colsum,
    const float* __restrict__ w_scales, const float* __restrict__ bias, int32_t K, int32_t ldx, int32_t N,
    uint32_t flags, GemmArgs a) {
  constexpr int kWaves = kDecodeWaves;
  constexpr int kBatch = 8;  // 64-byte k-blocks in flight per wave: 64 KB of weights per block
  // The eight waves' partial sums meet in one [4 registers][64 lanes] array per row group:
  // every wave adds its accumulators with LDS atomics as it finishes (a wave instruction covers
  // 64 consecutive words: no bank conflicts, and the early waves' additions are off the block's
  // critical path), and the 64 finishing threads read four words each instead of 32.
  __shared__ int s_sum[MG][4][kWave];
  const int t = threadIdx.x, lane = t % kWave, wave = t / kWave;
  const int lr = lane & 15, lc = lane >> 4;
  const int nb = blockIdx.x;
  const int M = static_cast<int>(flags & 0xffu);
  for (int i = t; i < MG * 4 * kWave; i += kWaves * kWave) (&s_sum[0][0][0])[i] = 0;
  // (before any global request is made: the barrier's wait for outstanding memory
  // operations is then a wait for this one LDS store)
  __syncthreads();
  const int KB = (K + 63) >> 6;
  // The 64 threads that finish a block: thread -> activation row within a
  // group, channel group of 4.
  const int fm = t >> 2, fg = t & 3;
  int c_cs[4] = {0, 0, 0, 0};
  float c_ws[4] = {1.f, 1.f, 1.f, 1.f}, c_b[4] = {0.f, 0.f, 0.f, 0.f};
  if (t < 64) {
    const int ws_stride = (flags >> 8) & 1;
    const float* const bsrc = bias != nullptr ? bias : w_scales;  // a load that always has an address
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = nb * 16 + 4 * fg + j;
      const int np = n < N ? n : 0;
      c_cs[j] = colsum[np];
      if (MODE != kOutAcc32) {
        c_ws[j] = w_scales[np * ws_stride];
        const float bv = bsrc[bias != nullptr ? np : 0];
        c_b[j] = bias != nullptr ? bv : 0.f;
      }
    }
  }
  const uint8_t* wp = w_packed + static_cast<int64_t>(nb) * (packed_kchunks(K) * 256) + lc * 256 + lr * 16;
  // Activations are loaded with four consecutive lanes on the 64 bytes one row
  // contributes to a k-block (lane -> row lane / 4, 16-byte piece lane % 4): a
  // quad of lanes then asks for one cache line instead of four.  The multiply
  // wants row lane % 16 and piece lane / 16, so every loaded register goes
  // through one cross-lane permutation (lane l takes from lane 4 (l % 16) + l / 16).
  const int sr = lane >> 2, sp = lane & 3;
  const int perm_addr = (4 * lr + lc) * 4;
  bool xrow[MG];
  const uint8_t* xp[MG];
#pragma unroll
  for (int mg = 0; mg < MG; ++mg) {
    xrow[mg] = mg * 16 + sr < M;
    xp[mg] = x + static_cast<int64_t>(xrow[mg] ? mg * 16 + sr : 0) * ldx;  // the row's first byte: always readable
  }
  const int xor_word = (flags >> 9) & 1 ? static_cast<int>(0x80808080u) : 0;
  const v4i xmask = {xor_word, xor_word, xor_word, xor_word};
  // Two accumulators per row group, used in turn: a multiply-accumulate does not
  // wait for the one before it.
  v4i acc2[MG][2];
#pragma unroll
  for (int mg = 0; mg < MG; ++mg) acc2[mg][0] = acc2[mg][1] = v4i{0, 0, 0, 0};
  // Every load of a batch is unconditional (addresses clamped into the operands,
  // the activation operand of a block that does not exist set to zero after the
  // load), so that the counts of outstanding loads are exact and the k-blocks are
  // multiplied one by one as they arrive; with a load under a condition the
  // compiler waits for all of them before the first product.
  auto batch = [&](int kb0) {
    v4i wf[kBatch], xf[MG][kBatch];
    bool xok[MG][kBatch];
    // Requests are counted back in the order issued.  With one group of rows the weights
    // (memory, the critical path) go first, each followed by its activations; with more
    // groups the activations (L2) all go first, so that their cross-lane permutations run
    // while the weights are still on their way (K = N = 4096: M = 1 5.25 against 5.46 us
    // the other way round, M = 32 7.5 against 7.8 us).
    if constexpr (MG >= 2) {
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        const int kb = kb0 + u * kWaves;
#pragma unroll
        for (int mg = 0; mg < MG; ++mg) {
          xok[mg][u] = kb < KB && xrow[mg] && (kb * 64 + sp * 16 < K);
          xf[mg][u] = ld16(xp[mg] + (xok[mg][u] ? kb * 64 + sp * 16 : 0));
        }
      }
    }
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int kb = kb0 + u * kWaves;
      const int kbc = kb < KB ? kb : KB - 1;
      wf[u] = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(wp + static_cast<int64_t>(kbc) * 1024));
      if constexpr (MG < 2) {
#pragma unroll
        for (int mg = 0; mg < MG; ++mg) {
          xok[mg][u] = kb < KB && xrow[mg] && (kb * 64 + sp * 16 < K);
          xf[mg][u] = ld16(xp[mg] + (xok[mg][u] ? kb * 64 + sp * 16 : 0));
        }
      }
    }
#pragma unroll
    for (int u = 0; u < kBatch; ++u)
#pragma unroll
      for (int mg = 0; mg < MG; ++mg) {
        const v4i xs = xok[mg][u] ? (xf[mg][u] ^ xmask) : v4i{0, 0, 0, 0};
        v4i xv;
#pragma unroll
        for (int c = 0; c < 4; ++c) xv[c] = __builtin_amdgcn_ds_bpermute(perm_addr, xs[c]);
        acc2[mg][u & 1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[u], xv, acc2[mg][u & 1], 0, 0, 0);
      }
  };
  for (int kb0 = wave; kb0 < KB; kb0 += kWaves * kBatch) batch(kb0);
  v4i acc[MG];
#pragma unroll
  for (int mg = 0; mg < MG; ++mg) acc[mg] = acc2[mg][0] + acc2[mg][1];
#pragma unroll
  for (int mg = 0; mg < MG; ++mg)
#pragma unroll
    for (int r = 0; r < 4; ++r)
      __hip_atomic_fetch_add(&s_sum[mg][r][lane], acc[mg][r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  // requantisation constants, before the barrier: off the block's critical path
  v4f bdiv = {0.f, 0.f, 0.f, 0.f}, mult = {0.f, 0.f, 0.f, 0.f};
  float bmul = 1.f;
  int acc0[4] = {0, 0, 0, 0};
  if (t < 64) {
    const XQuant xq = x_quant(a);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      acc0[j] = xq.coef * c_cs[j];
      if (MODE == kOutF32) {
        mult[j] = xq.scale * c_ws[j];
        bdiv[j] = c_b[j];
      } else if (MODE != kOutAcc32) {
        const float atw = xq.scale * c_ws[j];
        mult[j] = atw / a.out_scale;
        bdiv[j] = a.bias != nullptr ? bias_term(a.w_scale_stride == 0, c_b[j], atw) : 0.f;
        bmul = bias_mul(a.w_scale_stride == 0, atw);  // (per tensor: the same for every j)
      }
    }
  }
  __syncthreads();
  if (t < 64) {
    const int g = fg;
#pragma unroll
    for (int mg = 0; mg < MG; ++mg) {
      const int64_t m = mg * 16 + fm;
      if (m >= a.M) continue;
      int raw[4];
#pragma unroll
      for (int j = 0; j < 4; ++j)  // channel 4 g + j of row fm: register j of lane 16 g + fm
        raw[j] = s_sum[mg][j][16 * g + fm] + acc0[j];
      const int64_t n = nb * 16 + 4 * g;
      if (MODE == kOutAcc32) {
        int32_t* dst = static_cast<int32_t*>(a.y) + m * a.ldy + n;
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (n + j < a.N) dst[j] = raw[j];
      } else if (MODE == kOutF32) {
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
  }
}

// ---------------------------------------------------------------------------
// Dynamically quantized linear for a handful of rows (M <= 16, M * K <= 16384),
// float in, float out, one launch.  The weight-streaming kernel above with the
// activation quantization inside: every block requests its weights, then reads
// the whole float input (at most 64 KB, from L2), reduces min / max, derives the
// parameters (ChooseQuantizationParams, one thread), quantizes the values it
// holds into LDS -- product and zero point rounded once, as PyTorch's CPU
// quantized::linear_dynamic does while packing -- and multiplies from there.
// Every block repeats the same few microseconds of work on the input, under the
// latency of its own weight stream, instead of waiting for a launch that does
// it once.  Same arithmetic, same results as the two launches.
// ---------------------------------------------------------------------------
constexpr int64_t kDynSmallMaxValues = 16384;
// kHeld: float4 groups of the input per thread, M * K / 4 <= kHeld * 512 (a template
// parameter: the loads are unconditional so that the load counter stays exact).
template <int kHeld>
__global__ __launch_bounds__(kDecodeWaves* kWave) void linear_decode_dynamic_kernel(
    GemmArgs a, const float* __restrict__ x, int64_t ldxf, int reduce_range) {
  constexpr int kWaves = kDecodeWaves;
  constexpr int kBatch = 8;
  static_assert(kHeld * 4 * kWaves * kWave <= kDynSmallMaxValues, "held values");
  extern __shared__ __attribute__((aligned(16))) uint8_t sx[];  // [M][K + 16] activation codes
  __shared__ int s_sum[4][kWave];  // the waves' partial sums, added with LDS atomics (see linear_decode_kernel)
  __shared__ float s_mn[kWaves], s_mx[kWaves];
  __shared__ float s_scale, s_inv, s_zp;
  const int t = threadIdx.x, lane = t % kWave, wave = t / kWave;
  const int lr = lane & 15, lc = lane >> 4;
  const int64_t nb = blockIdx.x;
  const int64_t KB = ceil_div(a.K, 64);
  const int pitch = static_cast<int>(a.K) + 16;  // rows 16 bytes apart in the banks
  const uint8_t* wp = a.w_packed + nb * a.w_kchunks * 256 + lc * 256 + lr * 16;
  // per-channel constants of the 64 finishing threads, requested first
  const int fm = t >> 2, fg = t & 3;
  int c_cs[4] = {0, 0, 0, 0};
  float c_ws[4] = {1.f, 1.f, 1.f, 1.f}, c_b[4] = {0.f, 0.f, 0.f, 0.f};
  if (t < 64) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t n = nb * 16 + 4 * fg + j;
      const int64_t np = n < a.N ? n : 0;
      c_cs[j] = a.colsum[np];
      c_ws[j] = a.w_scales[np * a.w_scale_stride];
      if (a.bias != nullptr) c_b[j] = a.bias[np];
    }
  }
  // ---- the input: requested first (loads return in order: behind the weight
  // stream it would arrive only after it), held in registers between the range
  // pass and the quantization
  const int k4 = static_cast<int>(a.K / 4);
  const int total4 = static_cast<int>(a.M) * k4;
  v4f held[kHeld];
#pragma unroll
  for (int u = 0; u < kHeld; ++u) {
    const int e = t + u * (kWaves * kWave);
    const int ec = e < total4 ? e : 0;  // unconditional loads keep the load counter exact
    const int row = ec / k4, c4 = ec - row * k4;
    held[u] = *reinterpret_cast<const v4f*>(x + row * ldxf + c4 * 4);
  }
  // then the first batch of weights: on its way while the input is processed
  v4i wf[kBatch];
#pragma unroll
  for (int u = 0; u < kBatch; ++u) {
    const int64_t kb = wave + u * kWaves;
    const int64_t kbc = kb < KB ? kb : KB - 1;
    wf[u] = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(wp + kbc * 1024));
  }
  __builtin_amdgcn_sched_barrier(0);
  float mn = __builtin_inff(), mx = -__builtin_inff();
#pragma unroll
  for (int u = 0; u < kHeld; ++u) {
    const int e = t + u * (kWaves * kWave);
    if (e < total4) {
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
  if (t < 4 * kWave) (&s_sum[0][0])[t] = 0;  // (two barriers before the first addition)
  __syncthreads();
  if (t == 0) {
#pragma unroll
    for (int w = 1; w < kWaves; ++w) {
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
  __syncthreads();
  const float inv = s_inv, zp_f = s_zp;
#pragma unroll
  for (int u = 0; u < kHeld; ++u) {
    const int e = t + u * (kWaves * kWave);
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
      *reinterpret_cast<uint32_t*>(sx + row * pitch + c4 * 4) = q;
    }
  }
  __syncthreads();
  // ---- the product, activation operands from LDS (rows past M are zero)
  const v4i xmask = {static_cast<int>(0x80808080u), static_cast<int>(0x80808080u), static_cast<int>(0x80808080u),
                     static_cast<int>(0x80808080u)};
  const bool xrow = lr < a.M;
  const uint8_t* xp = sx + (xrow ? lr : 0) * pitch + lc * 16;
  v4i acc = {0, 0, 0, 0};
  for (int64_t kb0 = wave; kb0 < KB; kb0 += kWaves * kBatch) {
    if (kb0 != wave) {
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        const int64_t kb = kb0 + u * kWaves;
        wf[u] = kb < KB ? __builtin_nontemporal_load(reinterpret_cast<const v4i*>(wp + kb * 1024)) : v4i{0, 0, 0, 0};
      }
    }
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int64_t kb = kb0 + u * kWaves;
      const bool xok = kb < KB && xrow && (kb * 64 + lc * 16 < a.K);
      // (weights of a block past K were loaded from a clamped address: the zero
      // activation operand removes them from the sum, x ^ 0x80 alone would not)
      const v4i xf = xok ? ld16(xp + kb * 64) ^ xmask : v4i{0, 0, 0, 0};
      const v4i wv = kb < KB ? wf[u] : v4i{0, 0, 0, 0};
      acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(wv, xf, acc, 0, 0, 0);
    }
  }
#pragma unroll
  for (int r = 0; r < 4; ++r)
    __hip_atomic_fetch_add(&s_sum[r][lane], acc[r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  v4f mult = {0.f, 0.f, 0.f, 0.f}, bias = {0.f, 0.f, 0.f, 0.f};
  int acc0[4] = {0, 0, 0, 0};
  if (t < 64) {
    const int coef = 128 - static_cast<int>(zp_f);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      acc0[j] = coef * c_cs[j];
      mult[j] = s_scale * c_ws[j];
      bias[j] = c_b[j];
    }
  }
  __syncthreads();
  if (t < 64 && fm < a.M) {
    int raw[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) raw[j] = s_sum[j][16 * fg + fm] + acc0[j];
    store_f32x4(a, fm, nb * 16 + 4 * fg, raw, mult, bias);
  }
}

// ---------------------------------------------------------------------------
// Plain kernel: any K, any alignment.  One thread per (m, group of 4 channels).
// ---------------------------------------------------------------------------
template <int MODE>
__global__ __launch_bounds__(256) void linear_plain_kernel(GemmArgs a, XLinear xs, int x_signed) {
  const int64_t groups = ceil_div(a.N, 4);
  const int64_t id = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (id >= a.M * groups) return;
  const int64_t m = id / groups, n = (id % groups) * 4;
  const uint8_t* xr = xs.x + m * xs.ldx;
  int raw[4] = {0, 0, 0, 0};
  for (int64_t k = 0; k < a.K; ++k) {
    const int xv = x_signed ? static_cast<int>(static_cast<int8_t>(xr[k])) : static_cast<int>(xr[k]);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t nn = n + j;  // rows past N are zero in the packed buffer's last block
      const int wv = static_cast<int8_t>(
          a.w_packed[(((nn >> 4) * a.w_kchunks + (k >> 4)) * 16 + (nn & 15)) * 16 + (k & 15)]);
      raw[j] += xv * wv;
    }
  }
  v4f bdiv, mult;
  float bmul = 1.f;
  const XQuant xq = x_quant(a);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int64_t np = n + j < a.N ? n + j : 0;
    // plain accumulation used the true activation value, so only -x_zp*colsum is left
    raw[j] += xq.coef * a.colsum[np];
    if (MODE == kOutF32) {
      mult[j] = xq.scale * a.w_scales[np * a.w_scale_stride];
      bdiv[j] = a.bias != nullptr ? a.bias[np] : 0.f;
    } else if (MODE != kOutAcc32) {
      const float atw = xq.scale * a.w_scales[np * a.w_scale_stride];
      mult[j] = atw / a.out_scale;
      bdiv[j] = a.bias != nullptr ? bias_term(a.w_scale_stride == 0, a.bias[np], atw) : 0.f;
      bmul = bias_mul(a.w_scale_stride == 0, atw);
    }
  }
  if (MODE == kOutAcc32) {
    int32_t* dst = static_cast<int32_t*>(a.y) + m * a.ldy + n;
    for (int j = 0; j < 4; ++j)
      if (n + j < a.N) dst[j] = raw[j];
  } else if (MODE == kOutF32) {
    store_f32x4(a, m, n, raw, mult, bdiv);
  } else {
    const uint32_t packed = requant4<MODE>(raw, bdiv, bmul, mult, a.zp_f, a.lo_f, a.hi_f);
    uint8_t* dst = static_cast<uint8_t*>(a.y) + m * a.ldy + n;
    for (int j = 0; j < 4; ++j)
      if (n + j < a.N) dst[j] = static_cast<uint8_t>(packed >> (8 * j));
  }
}

template <int BM, int BN, int WM, int WN, int MODE, int PD = 4, bool WDMA = false, int KW = 1, bool XWIDE = false>
int launch_gemm(const GemmArgs& a, const XLinear& xs, hipStream_t s) {
  const int64_t blocks = ceil_div(a.M, BM) * ceil_div(a.N, BN);
  if (blocks > 0x7fffffff) return TMQ_ERR_UNSUPPORTED;
  if (KW > 1 && ceil_div(a.K, kBK) % KW != 0) return TMQ_ERR_UNSUPPORTED;  // equal runs of stages only
  gemm_i8_kernel<BM, BN, WM, WN, MODE, XLinear, PD, WDMA, KW, XWIDE>
      <<<dim3(static_cast<unsigned>(blocks)), dim3(WM * WN * KW * kWave), 0, s>>>(a, xs);
  return launch_status();
}

// 64 x 64 tiles with all of K in LDS (K <= 1024; the caller checked the address ranges).
template <int MODE>
int launch_gemm_onepass(const GemmArgs& a, const XLinear& xs, hipStream_t s) {
  const int64_t tiles_m = ceil_div(a.M, 64), tiles_n = ceil_div(a.N, 64);
  if (tiles_n > 0x7fffffff || tiles_m > 65535) return TMQ_ERR_UNSUPPORTED;
  gemm_i8_onepass_kernel<MODE>
      <<<dim3(static_cast<unsigned>(tiles_n), static_cast<unsigned>(tiles_m)), dim3(256), 0, s>>>(a, xs);
  return launch_status();
}

// 32 x 32 tiles whose four waves split K (K <= 1024; the caller checked the address ranges).
template <int MODE>
int launch_gemm_ksplit(const GemmArgs& a, const XLinear& xs, hipStream_t s) {
  const int64_t tiles_m = ceil_div(a.M, 32), tiles_n = ceil_div(a.N, 32);
  if (tiles_n > 0x7fffffff || tiles_m > 65535 || a.K > kOnePassMaxK) return TMQ_ERR_UNSUPPORTED;
  gemm_i8_ksplit_kernel<MODE>
      <<<dim3(static_cast<unsigned>(tiles_n), static_cast<unsigned>(tiles_m)), dim3(256), 0, s>>>(a, xs);
  return launch_status();
}

// Tiles of 32 rows whose waves split K, weights through registers (K <= 4096; the caller
// checked the address ranges).  wide: 64 channels per tile instead of 32.
template <int MODE>
int launch_gemm_wstream(const GemmArgs& a, const XLinear& xs, bool wide, hipStream_t s) {
  const int64_t tiles_m = ceil_div(a.M, 32), tiles_n = ceil_div(a.N, wide ? 64 : 32);
  if (tiles_n > 0x7fffffff || tiles_m > 65535 || a.K > 4096) return TMQ_ERR_UNSUPPORTED;
  const dim3 grid(static_cast<unsigned>(tiles_n), static_cast<unsigned>(tiles_m));
  if (!wide && a.K <= 2048)
    gemm_i8_wstream_kernel<MODE, 16><<<grid, dim3(256), 0, s>>>(a, xs);
  else if (!wide)
    gemm_i8_wstream_kernel<MODE, 32><<<grid, dim3(256), 0, s>>>(a, xs);
  else
    gemm_i8_wstream_kernel<MODE, 16, 2, 8><<<grid, dim3(512), 0, s>>>(a, xs);
  return launch_status();
}

// 64 x 64 tiles whose eight waves split K, weights through registers, activations through
// a ring per wave (K <= 4096; the caller checked the address ranges).
template <int MODE>
int launch_gemm_wring(const GemmArgs& a, const XLinear& xs, hipStream_t s) {
  const int64_t tiles_m = ceil_div(a.M, 64), tiles_n = ceil_div(a.N, 64);
  if (tiles_n > 0x7fffffff || tiles_m > 65535 || a.K > kWringMaxK || a.K % 16 != 0) return TMQ_ERR_UNSUPPORTED;
  gemm_i8_wring_kernel<MODE><<<dim3(static_cast<unsigned>(tiles_n), static_cast<unsigned>(tiles_m)),
                               dim3(kWringThreads), 0, s>>>(a, xs);
  return launch_status();
}

constexpr int kMaxDevices = 64;

// Compute units of the current device (cached per device; two threads that race
// on a device's first call store the same value).
int cu_count() {
  static std::atomic<int> cache[kMaxDevices];
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 0;
  int v = cache[dev].load(std::memory_order_relaxed);
  if (v == 0) {
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    cache[dev].store(v, std::memory_order_relaxed);
  }
  return v;
}

// One block per CU walks the 256 x 256 tiles (byte or float outputs, direct copies two
// stages wide: the caller checked their address and K ranges).
template <int MODE>
int launch_gemm_persistent(const GemmArgs& a, const XLinear& xs, hipStream_t s) {
  if constexpr (MODE == kOutU8 || MODE == kOutS8 || MODE == kOutF32) {
    const int64_t tiles = ceil_div(a.M, 256) * ceil_div(a.N, 256);
    const int cus = cu_count();
    if (cus < 8 || tiles > 0x7fffffff) return TMQ_ERR_UNSUPPORTED;
    // several rounds: a multiple of 8 blocks, so that the tile sequence deals
    // every XCD its own run of tiles
    const int64_t grid = tiles <= cus ? tiles : cus / 8 * 8;
    gemm_i8_persistent_kernel<MODE><<<dim3(static_cast<unsigned>(grid)), dim3(kPersistThreads), 0, s>>>(a, xs);
    return launch_status();
  } else {
    return TMQ_ERR_UNSUPPORTED;
  }
}

// Weight streaming for up to 64 rows: one block per 16 channels.
template <int MODE>
int launch_linear_decode(const GemmArgs& a, const XLinear& xs, hipStream_t s) {
  // (the kernel derives the packed pitch from K, as prepack does)
  if (a.w_kchunks != packed_kchunks(a.K)) return TMQ_ERR_UNSUPPORTED;
  const dim3 grid(static_cast<unsigned>(ceil_div(a.N, 16))), block(kDecodeWaves * kWave);
  const int32_t k32 = static_cast<int32_t>(a.K), ldx32 = static_cast<int32_t>(xs.ldx);
  const int32_t n32 = static_cast<int32_t>(a.N);
  const uint32_t flags = static_cast<uint32_t>(a.M) | (a.w_scale_stride != 0 ? 0x100u : 0u) |
                         (a.x_xor != 0 ? 0x200u : 0u);
  switch ((a.M + 15) / 16) {
    case 1: linear_decode_kernel<MODE, 1><<<grid, block, 0, s>>>(a.w_packed, xs.x, a.colsum, a.w_scales, a.bias, k32, ldx32, n32, flags, a); break;
    case 2: linear_decode_kernel<MODE, 2><<<grid, block, 0, s>>>(a.w_packed, xs.x, a.colsum, a.w_scales, a.bias, k32, ldx32, n32, flags, a); break;
    case 3: linear_decode_kernel<MODE, 3><<<grid, block, 0, s>>>(a.w_packed, xs.x, a.colsum, a.w_scales, a.bias, k32, ldx32, n32, flags, a); break;
    default: linear_decode_kernel<MODE, 4><<<grid, block, 0, s>>>(a.w_packed, xs.x, a.colsum, a.w_scales, a.bias, k32, ldx32, n32, flags, a); break;
  }
  return launch_status();
}

// Up to 64 rows whose activations (16 MG x K bytes, MG = groups of 16 rows) fit the
// kernel's LDS area: one block per CU streams the channel groups it owns.
bool resident_limits_ok(int64_t M, int64_t N, int64_t K, int64_t ldx, int cus) {
  if (M < 1 || M > 64 || K < 64 || K % 16 != 0 || cus < 1) return false;
  const int64_t mg = ceil_div(M, 16), groups = ceil_div(N, 16);
  return 16 * mg * ceil_div(K, 64 * kResidentWaves) * (64 * kResidentWaves) <= kResidentXBytes && groups <= static_cast<int64_t>(kResidentMaxGroups) * cus &&
         N <= 0x7ffffff0 && ldx <= (int64_t{1} << 40);
}

// Two blocks of eight waves per CU where the rows fit half the LDS area (one group of rows,
// K <= 4096) and a block still owns at most 32 channel groups: the two blocks' bursts of
// requests interleave (M = 8, K = 4096, N = 32000: 25.2 -> 24.0 us; N = 16384, K = 1024: 6.7 -> 6.0 us;
// N = 8192, K = 2048: 6.2 -> 5.8 us).  Not below two groups per block at K > 2048: the rows are then
// staged twice per CU for nothing (N = 5120, K = 4096, M = 16: 7.7 -> 8.8 us; N = 11008: 10.6 -> 11.0 us).
bool resident_pair(int64_t M, int64_t N, int64_t K, int cus) {
  const int64_t groups = ceil_div(N, 16);
  return M <= 16 && 16 * ceil_div(K, 64 * 8) * (64 * 8) <= kResidentXBytes / 2 && groups <= int64_t{32} * 2 * cus &&
         groups >= (K <= 2048 ? 2 : 4) * static_cast<int64_t>(cus);
}

template <int MODE>
int launch_linear_resident(const GemmArgs& a, const XLinear& xs, hipStream_t s) {
  const int cus = cu_count();
  if (!resident_limits_ok(a.M, a.N, a.K, xs.ldx, cus)) return TMQ_ERR_UNSUPPORTED;
  const int64_t groups = ceil_div(a.N, 16);
  if (resident_pair(a.M, a.N, a.K, cus)) {
    const dim3 grid(static_cast<unsigned>(groups < 2 * cus ? groups : 2 * cus)), block(8 * kWave);
    linear_resident_kernel<MODE, 1, 8><<<grid, block, 0, s>>>(a, xs, nullptr, 0, 0);
    return launch_status();
  }
  const dim3 grid(static_cast<unsigned>(groups < cus ? groups : cus)), block(kResidentThreads);
  switch ((a.M + 15) / 16) {
    case 1: linear_resident_kernel<MODE, 1><<<grid, block, 0, s>>>(a, xs, nullptr, 0, 0); break;
    case 2: linear_resident_kernel<MODE, 2><<<grid, block, 0, s>>>(a, xs, nullptr, 0, 0); break;
    case 3: linear_resident_kernel<MODE, 3><<<grid, block, 0, s>>>(a, xs, nullptr, 0, 0); break;
    default: linear_resident_kernel<MODE, 4><<<grid, block, 0, s>>>(a, xs, nullptr, 0, 0); break;
  }
  return launch_status();
}

// ---- split K for a few hundred rows against a long K.  The tile grid of such a
// product is far smaller than the chip (M = 128, N = 4096: 32 tiles of
// 128 x 128) and every block walks all of K alone at the latency of one stage
// after the other, so K is cut into `splits` runs of whole stages: splits x
// tiles blocks write raw int32 partial sums [split][M][ldp] into a caller-owned
// workspace and a second kernel adds them up and requantises.  Writing and
// re-reading the partial sums costs about 10 us at these sizes, which the
// shorter k loops repay from K = 8192 on (measured: M = 128, N = 4096,
// K = 11008: 38.5 -> 25 us; K = 4096: 14.6 -> 20 us, hence no split there).
struct SplitPlan {
  int splits = 1;   // 1: single launch
  int stages = 0;   // k stages (64 bytes of K) per split
  int64_t ldp = 0;  // row pitch of a partial-sum slice, int32 elements
};

constexpr int64_t kSplitBlocks = 256;    // blocks wanted: one per CU
constexpr int64_t kSplitMinKT = 128;     // shortest k loop (stages) worth cutting
constexpr int64_t kSplitMinStages = 16;  // shortest run of stages per split

// ---- 17 ... 64 rows: several kernels can run such a product, and which is fastest
// depends on the shape.  Estimated microseconds per launch, fitted to sweeps with
// cold weights (more weight sets in rotation than the last-level cache holds):
//  * the weight-streaming kernel: a block of 16 channels streams its K x 16 weight
//    bytes once and re-reads the activations of every group of 16 rows, so one round
//    of blocks (N <= 4096) costs a base that grows with the weight bytes plus a share
//    per row group that grows with K (K = N = 4096: 6.4 / 7.5 / 11.3 us at M = 17 / 32 / 64;
//    N = 4096, K = 8192: 10.2 / 12.2 / 18.8 us), and further rounds cost about three
//    quarters of the first (N = K = 8192, two rounds: 19.2 / 20.9 / 34.8 us; N = 11008,
//    K = 4096, three rounds: 15.1 / 16.3 / 28.1 us);
//  * 64 x 64 tiles walk K at the latency of one stage after the other, almost
//    whatever M is (K = N = 4096 with two wave groups: 12.6 / 14.3 us at
//    M = 32 / 64; N = 11008: 14.6 / 16.9 us), and K <= 1024 fits LDS whole
//    (gemm_i8_onepass.h: K = 1024 on 32 x 32 tiles: 3.8 / 4.1 / 4.9 us at N = 1024 / 4096 / 8192);
//  * split K moves the weights at about 4.5 TB/s plus 10 us for the partial sums
//    (N = 4096, K = 11008: 21.7 us at M = 64 against 27.0 us streaming; K = 8192, M = 48:
//    18.0 against 15.5 us streaming).
enum class SmallRows { kStream, kTiles, kSplit };

bool two_wave_groups_fit(int64_t M, int64_t N, int64_t K) {
  const int64_t stages = ceil_div(K, kBK);
  return ceil_div(M, 64) * ceil_div(N, 64) <= 256 && stages >= 32 && stages % 2 == 0;
}

SplitPlan plan_split_tiles(int64_t M, int64_t N, int64_t K);

// Shapes for the tiles of 32 rows whose waves split K and stream their weights through
// registers: K beyond what the kernels with all operands in LDS take, one round of
// blocks (two blocks share a CU while a block's activations, 32 rows x K, are at
// most 64 KB).  With more blocks than that it loses to the larger tiles (K = 4096:
// N = 4096, M = 96: 13.7 against 12.8 us; K = 2048, N = 4096, M = 256: 10.7 against 9.7 us).
// Returns the channels per tile: 32; 64 (eight waves, K > 2048 only: at K <= 2048 it
// never beat the 32 x 32 tiles where they fit nor the larger tiles where they do not)
// when only those fit one round (K = N = 4096: M = 96 12.8 -> 9.9 us, M = 128 14.1 -> 10.0 us;
// N = 8192, M = 64: 15.7 -> 11.5 us; N = 2048, M = 256: 13.6 -> 9.5 us; where both fit, 32
// channels are 1.5 us ahead); 0: neither.
int wstream_tile(int64_t M, int64_t N, int64_t K) {
  if (K <= kOnePassMaxK || K > 4096) return 0;
  if (ceil_div(M, 32) * ceil_div(N, 32) <= (K <= 2048 ? 512 : 256)) return 32;
  if (K > 2048 && ceil_div(M, 32) * ceil_div(N, 64) <= 256) return 64;
  return 0;
}

// One round of 64 x 64 tiles against K > 4096 whose last row tile is at least three
// quarters full, up to 128 rows: the kernel that copies K through LDS in phases takes the
// same time whatever the rows (N = K = 5120: 17.1 ... 17.9 us from 40 to 128 rows; N = K = 8192:
// 26.5 us at 64 rows), while two wave groups slow down as the tiles fill (20.9 us and 29.3 us
// at 64 rows; N = 4096, K = 11008, M = 64: 32.2 against 37.3 us).  With a tile half empty, or
// from 192 rows on, the wave groups are ahead (N = 4096, K = 14336, M = 256: 42.4 against 45.6 us).
// (K = 4096 against N >= 10240, where the tiles of 32 rows no longer fit one round: M = 64, N = 11008: 16.2 against
// 17.5 us; N = 14336: 17.3 against 18.1 us; at 128 rows the wave groups are ahead, N = 8192: 15.7 against 16.2 us)
bool phased_ring_preferred(int64_t M, int64_t N, int64_t K) {
  if (K % 16 != 0 || ceil_div(M, 64) * ceil_div(N, 64) > 256 || (M - 1) % 64 < 47) return false;
  return K > 4096 ? M <= 128 : (K == 4096 && M <= 64 && N >= 10240);
}

SmallRows small_rows_path(int64_t M, int64_t N, int64_t K, bool workspace) {
  // Where the 32 x 32 tiles with the weights through registers fit, they are measured
  // directly against the weight-streaming kernel (us at M = 17 / 32 / 40 / 64, tiles | streaming):
  //   K = 2048, N = 4096:  5.2 / 5.4 / 5.5 / 5.5 | 5.7 / 5.9 / 7.2 / 9.3    K = 4096, N = 1024:  6.7 / 6.7 / 6.7 / 6.7 | 5.3 / 5.5 / 6.9 / 8.6
  //   K = 4096, N = 4096:  8.4 / 8.5 / 8.6 / 8.7 | 6.4 / 7.5 / 8.6 / 11.3   K = 3072, N = 3072:  7.2 / 7.2 / 7.2 / 7.4 | 5.5 / 6.1 / 7.2 / 10.0
  //   K = 3072, N = 4096:  7.4 / 7.4 / 7.5 / 7.7 | 5.9 / 6.5 / 7.7 / 10.9   K = 4096, N = 8192: 10.8 / 10.9 / -   / -   | 11.1 / 12.2 / 14.5 / 20.6
  // streaming keeps K > 2048 up to 32 rows (two row groups) while its blocks fit one round.
  if (wstream_tile(M, N, K) != 0)
    return K > 2048 && M <= 32 && N <= 4096 ? SmallRows::kStream : SmallRows::kTiles;
  const double mib = static_cast<double>(N) * static_cast<double>(K) / 1048576.0;
  const double stages = static_cast<double>(ceil_div(K, kBK));
  const double rows = static_cast<double>(M);
  const double kk = static_cast<double>(K) / 1024.0;
  const double stream_rounds = static_cast<double>(ceil_div(ceil_div(N, 16), 256));
  const double round_mib = static_cast<double>(std::min<int64_t>(N, 4096)) * static_cast<double>(K) / 1048576.0;
  const double one_round = 1.9 + 0.09 * round_mib + static_cast<double>(ceil_div(M, 16)) * std::max(1.6, 0.42 * kk);
  const double stream = stream_rounds <= 1.0 ? one_round : one_round * (0.3 + 0.75 * stream_rounds);
  const double nblk = static_cast<double>(ceil_div(M, 64) * ceil_div(N, 64));
  double tiles;
  if (K <= kOnePassMaxK && K > 256 && ceil_div(M, 32) * ceil_div(N, 32) <= 512)
    // all of K in LDS, 32 x 32 tiles (K = 1024: 3.8 / 3.8 / 4.1 / 4.9 us at N = 1024 / 2048 / 4096 / 8192;
    // more than 256 tiles, N = 8192, M = 40: 5.4 us)
    tiles = 3.6 + 0.13 * mib + (ceil_div(M, 32) * ceil_div(N, 32) > 256 ? 0.5 : 0.0);
  else if (K <= kOnePassMaxK && nblk <= 256.0)  // 64 x 64 tiles (K = N = 1024: 5.6 us, N = 1024, K = 256: 3.1 us)
    tiles = 2.0 + 3.8 * kk + 0.012 * std::max(0.0, nblk - 64.0);
  else if (phased_ring_preferred(M, N, K))
    // (N = 4096: 25.3 / 32.2 / 40.9 us at K = 8192 / 11008 / 14336; N = K = 5120: 17.4 us; N = K = 8192: 26.5 us)
    tiles = 3.3 + 2.65 * kk + 0.2 * std::max(0.0, static_cast<double>(N) - 4096.0) / 1024.0;
  else if (two_wave_groups_fit(M, N, K))
    tiles = (4.4 + 0.123 * stages + 0.013 * std::max(0.0, nblk - 64.0)) *
            (1.0 + 0.35 * (rows / 64.0) * (rows / 64.0) * std::min(1.0, stages / 172.0));
  else
    tiles = (3.0 + 0.2 * stages) * (1.0 + nblk / 1024.0);
  const double best = std::min(stream, tiles);
  if (workspace && plan_split_tiles(M, N, K).splits > 1) {
    // (N = 4096: 18.0 / 21.3 / 23.5 us at K = 8192 / 11008 / 14336, 48 rows)
    const double split = 10.0 + 0.23 * mib + 0.025 * rows;
    if (split < best) return SmallRows::kSplit;
  }
  return stream <= tiles ? SmallRows::kStream : SmallRows::kTiles;
}

SplitPlan plan_split_tiles(int64_t M, int64_t N, int64_t K) {
  SplitPlan p;
  if (M <= kDecodeRowsAuto || K % 16 != 0) return p;
  const int64_t KT = ceil_div(K, kBK);
  const int64_t tiles = ceil_div(M, 128) * ceil_div(N, 128);
  if (KT < kSplitMinKT || tiles > kSplitBlocks / 2) return p;
  int64_t splits = kSplitBlocks / tiles;
  if (splits > KT / kSplitMinStages) splits = KT / kSplitMinStages;
  if (splits < 2) return p;
  const int64_t stages = ceil_div(KT, splits);
  splits = ceil_div(KT, stages);
  // a last run of fewer than six stages (one turn of the direct-copy ring) is
  // merged into the split before it: the kernel's last split multiplies
  // everything from (splits - 1) * stages to the end of K
  if (KT - (splits - 1) * stages < 6) --splits;
  if (splits < 2) return p;
  p.splits = static_cast<int>(splits);
  p.stages = static_cast<int>(stages);
  p.ldp = (N + 3) / 4 * 4;
  return p;
}

// The plan the automatic choice follows: none for the rows that stream the
// weights, and for 17 ... 64 rows only where the estimate above prefers it.
SplitPlan plan_split(int64_t M, int64_t N, int64_t K) {
  if (M > kDecodeRowsAuto && M <= kDecodeMaxRows && small_rows_path(M, N, K, true) != SmallRows::kSplit)
    return SplitPlan{};
  return plan_split_tiles(M, N, K);
}

int64_t split_workspace_bytes(const SplitPlan& p, int64_t M) {
  return p.splits > 1 ? p.splits * M * p.ldp * static_cast<int64_t>(sizeof(int32_t)) : 0;
}

// Second kernel of a split-K product: a block owns 256 consecutive channels and
// `rows` rows.  Its threads first compute the 256 channels' constants, one
// channel each, into LDS (the two divisions per channel would otherwise be
// repeated by every row); then a thread adds the `splits` partial sums of four
// consecutive channels of one row at a time and runs the epilogue of the
// single-launch kernels (same helper, same operation order).
template <int MODE>
__global__ __launch_bounds__(256) void splitk_finish_kernel(GemmArgs a, const int32_t* parts, int splits,
                                                            int64_t ldp, int64_t slice, int rows) {
  __shared__ __attribute__((aligned(16))) int s_add[256];
  __shared__ __attribute__((aligned(16))) float s_mult[256];
  __shared__ __attribute__((aligned(16))) float s_bdiv[256];
  const int t = threadIdx.x;
  const int64_t n0 = static_cast<int64_t>(blockIdx.x) * 256;
  {
    const XQuant xq = x_quant(a);
    const int64_t nj = n0 + t < a.N ? n0 + t : a.N - 1;
    float mult = 0.f, bdiv = 0.f;
    if (MODE != kOutAcc32) {
      const float atw = xq.scale * a.w_scales[nj * a.w_scale_stride];
      if (MODE == kOutF32) {
        mult = atw;
        bdiv = a.bias != nullptr ? a.bias[nj] : 0.f;
      } else {
        mult = atw / a.out_scale;
        bdiv = a.bias != nullptr ? bias_term(a.w_scale_stride == 0, a.bias[nj], atw) : 0.f;
      }
    }
    s_add[t] = xq.coef * a.colsum[nj];
    s_mult[t] = mult;
    s_bdiv[t] = bdiv;
  }
  __syncthreads();
  const int q = t & 63;
  const int64_t n = n0 + q * 4;
  if (n >= a.N) return;
  const v4i add = *reinterpret_cast<const v4i*>(&s_add[q * 4]);
  const v4f mult = *reinterpret_cast<const v4f*>(&s_mult[q * 4]);
  const v4f bdiv = *reinterpret_cast<const v4f*>(&s_bdiv[q * 4]);
  const bool plain_u8 = MODE == kOutU8 && a.lo_f <= 0.f && a.hi_f >= 255.f;
  const float bmul = (MODE == kOutU8 || MODE == kOutS8)
                         ? bias_mul(a.w_scale_stride == 0, x_quant(a).scale * a.w_scales[0]) : 1.0f;
  const int64_t mbeg = static_cast<int64_t>(blockIdx.y) * rows;
  const int64_t mend = mbeg + rows < a.M ? mbeg + rows : a.M;
  for (int64_t m = mbeg + (t >> 6); m < mend; m += 4) {
    const int32_t* src = parts + m * ldp + n;
    v4i sum = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(src));
    for (int sp = 1; sp < splits; ++sp)
      sum += __builtin_nontemporal_load(reinterpret_cast<const v4i*>(src + sp * slice));
    sum += add;
    const int raw[4] = {sum.x, sum.y, sum.z, sum.w};
    if constexpr (MODE == kOutAcc32) {
      int32_t* dst = static_cast<int32_t*>(a.y) + m * a.ldy + n;
      for (int j = 0; j < 4; ++j)
        if (n + j < a.N) dst[j] = raw[j];
    } else if constexpr (MODE == kOutF32) {
      store_f32x4(a, m, n, raw, mult, bdiv);
    } else {
      const uint32_t q4 = plain_u8 ? requant4<MODE, false>(raw, bdiv, bmul, mult, a.zp_f, a.lo_f, a.hi_f)
                                   : requant4<MODE, true>(raw, bdiv, bmul, mult, a.zp_f, a.lo_f, a.hi_f);
      uint8_t* dst = static_cast<uint8_t*>(a.y) + m * a.ldy + n;
      if (n + 3 < a.N && (reinterpret_cast<uintptr_t>(dst) & 3) == 0) {
        *reinterpret_cast<uint32_t*>(dst) = q4;
      } else {
        for (int j = 0; j < 4; ++j)
          if (n + j < a.N) dst[j] = static_cast<uint8_t>(q4 >> (8 * j));
      }
    }
  }
}

template <int BM, int BN, int WM, int WN, int PD = 4, bool WDMA = false, bool XWIDE = false>
int launch_gemm_split(const GemmArgs& a, const XLinear& xs, const SplitPlan& p, hipStream_t s) {
  const int64_t blocks = ceil_div(a.M, BM) * ceil_div(a.N, BN);
  if (blocks > 0x7fffffff) return TMQ_ERR_UNSUPPORTED;
  gemm_i8_kernel<BM, BN, WM, WN, kOutAcc32, XLinear, PD, WDMA, 1, XWIDE>
      <<<dim3(static_cast<unsigned>(blocks), static_cast<unsigned>(p.splits)), dim3(WM * WN * kWave), 0, s>>>(a, xs);
  return launch_status();
}

template <int MODE>
int run_split(const GemmArgs& a, const XLinear& xs, const SplitPlan& p, void* workspace, bool dma_ok,
              hipStream_t s) {
  GemmArgs part = a;  // first kernel: pure sums of (x ^ flip) * w, no zero-point term
  part.acc_coef = 0;
  part.acc_base = 0;
  part.x_qp_dev = nullptr;
  part.y = workspace;
  part.ldy = p.ldp;
  part.splits = p.splits;
  part.split_stages = p.stages;
  part.split_stride = a.M * p.ldp;
  const int rc = dma_ok ? launch_gemm_split<128, 128, 2, 2, 3, true, true>(part, xs, p, s)
                        : launch_gemm_split<128, 128, 2, 2>(part, xs, p, s);
  if (rc != TMQ_OK) return rc;
  // rows per block: enough blocks to hide the loads' latency, then longer runs
  const int rows = a.M <= 256 ? 4 : 16;
  const int64_t bx = ceil_div(a.N, 256), by = ceil_div(a.M, rows);
  if (bx > 0x7fffffff || by > 65535) return TMQ_ERR_UNSUPPORTED;  // a split product has a few hundred rows
  splitk_finish_kernel<MODE><<<dim3(static_cast<unsigned>(bx), static_cast<unsigned>(by)), dim3(256), 0, s>>>(
      a, static_cast<const int32_t*>(workspace), p.splits, p.ldp, a.M * p.ldp, rows);
  return launch_status();
}

// ---- which kernel runs a product: a host-side function of the shape alone, so that
// it can be queried (tmq_linear_kernel_choice) and swept without a device.
struct LinearQuery {
  int64_t M, N, K, ldx;
  int64_t n_off = 0;
  int mode = kOutU8;             // EpilogueMode
  bool vec_ok = true;            // K, the row pitch and the activation pointer are multiples of 16
  bool workspace_attached = false;
  int64_t workspace_bytes = 0;   // usable (16-byte aligned) split-K scratch
};
// cfg: tmq_linear_desc::kernel - 1.  0-7, 14, 17, 19, 22, 23: tiles of gemm_i8_kernel; 8: weight
// streaming; 9: plain kernel; 13: split K (plan in `split`); 20: persistent 256 x 256 tiles;
// 21 / 24: all of K in LDS (64 x 64 / 32 x 32 tiles); 25 / 26: weights through registers
// (32 x 32 / 32 x 64 tiles); 27: the same with 64 x 64 tiles and the activations in a ring
// per wave; 28: activations resident in LDS, one block per CU streams its channel groups;
// kNoKernel: the forced kernel does not take this shape.
constexpr int kNoKernel = -2;
struct LinearChoice {
  int cfg = kNoKernel;
  SplitPlan split;
};

// Limits of the kernels' own index arithmetic, shared by the choice and the launches.
// Direct-copy kernels: 256 rows of either operand addressed with 32-bit offsets, and
// their three-stage ring runs at least once around.
bool dma_limits_ok(int64_t K, int64_t ldx) { return ldx <= (int64_t{1} << 23) && K <= (int64_t{1} << 23) && K > 2 * kBK; }
// The copies two stages wide walk K in runs of six stages.
bool wide_limits_ok(int64_t K, int64_t ldx) { return dma_limits_ok(K, ldx) && K > 5 * kBK; }
// All of K in LDS / weights through registers: 32-bit offsets over 64 rows of either
// operand, N * 4 as a 32-bit offset.
bool onepass_limits_ok(const LinearQuery& q) {
  return q.K % 16 == 0 && q.K <= (int64_t{1} << 23) && q.ldx <= (int64_t{1} << 23) && q.N + q.n_off < (int64_t{1} << 29);
}
// The weight-streaming kernel takes K, the row pitch and N as 32-bit arguments.
bool stream_limits_ok(const LinearQuery& q) {
  return q.M <= kDecodeMaxRows && ceil_div(q.N, 16) <= 0x7fffffff && q.K <= 0x7fffff00 && q.ldx <= 0x7fffffff &&
         q.N <= 0x7ffffff0;
}

// Where the kernel that keeps the activations in LDS is ahead of a block per 16 channels
// (cold weights, us, resident | streaming; neither depends on N beyond what is shown):
//   K <= 2048, from N = 2048 on, any M <= 16:  K = N = 2048: 4.0 ... 4.2 | 4.2 ... 4.7;  N = 4096, K = 1024: 3.9 | 4.2 ... 4.5;  N = 8192, K = 1024:
//     4.8 ... 5.0 | 5.8 ... 6.3;  N = 4096, K = 2048: 4.5 | 4.7 ... 5.0;  N = 65536, K = 2048: 24.5 | 35 ... 42
//   longer K, 14 rows and more (the streaming blocks re-read the rows from the L2s), from N = 5120 on:
//     K = 4096, M = 16: N = 5120 7.7 | 8.6, N = 11008 10.6 | 12.3, N = 32000 25.4 | 32.2, N = 128256 97 | 122;
//     N = K = 8192, M = 16: 14.7 | 16.1  (M = 12: N = 5120 7.6 | 7.8, N = 8192 9.1 | 8.6: one full round of
//     streaming blocks, two per CU, is that kernel's best case)
//   5 ... 13 rows at K = 4096 beyond that round, N >= 10240: M = 8: N = 11008 10.8 | 11.3 ... 12.2, N = 32000
//     24.0 | 25.6, N = 128256 91.7 | 95.7;  M = 12: N = 49152 38.2 | 39.6, N = 65536 50.3 | 54.4
//   (fewer rows: level up to N = 32000, then the independent blocks stream faster: N = 128256, M = 1: 89 | 85;
//   N = 4096 at K >= 4096: level or behind, 6.1 | 5.9 at M = 16)
//   a K that leaves the streaming blocks a short last pass (K = N = 5120: 8.4 ... 8.7 | 9.2 ... 11.3 at M = 1 ... 12)
//   17 ... 32 rows: a narrow band between the tiles of 32 rows, which no longer fit one round, and the 64 x 128
//   tiles (K = 4096, M = 24 / 32: N = 11008 11.9 / 12.2 against 12.5 / 12.7 us, N = 16384 15.5 / 15.7 against
//   16.4 / 16.7 us; N = 8192: level with 32 x 32 tiles; N = 32000: 26.6 against 24.5 us for 64 x 128 tiles).
bool resident_preferred(const LinearQuery& q) {
  if (!q.vec_ok || q.K < 1024 || q.M > 32 || !resident_limits_ok(q.M, q.N, q.K, q.ldx, 256)) return false;
  if (q.M > 16) return q.K > 2048 && q.N >= 10240 && q.N <= 20480;
  if (q.K <= 2048) return q.N >= 2048;
  if (q.K > 4096 && q.K % 4096 != 0 && q.K % 4096 <= 2048 && q.N >= 5120) return true;
  return (q.M >= 14 && q.N >= 5120) || (q.M >= 5 && q.N >= 10240);
}

// Five rows and more against the very largest N at K > 2048: the pipelined 64 x 128 tiles, mostly padding
// in their rows, stream such a weight faster than either kernel above -- two and more long-running blocks
// per CU, each with its own ring of stages (cold weights, K = 4096, us, tiles | rows resident | a block per 16
// channels: N = 128256: M = 16 85.0 | 93.5 | 118, M = 8 87.3 | 93.5 | 97.2, M = 1 87.4 | 88 | 85.0;
// N = 65536: M = 16 47.6 | 51.4 | 63.8, M = 8 47.6 | 48.9 | 51.2; below, the resident rows are ahead:
// N = 49152, M = 16: 40.1 | 38.7; N = 32000: 26.8 | 25.8; at K = 2048 the two are level up to N = 128256).
bool huge_n_tiles_preferred(const LinearQuery& q) {
  return q.vec_ok && q.M >= 5 && q.M <= 16 && q.K > 2048 && q.N >= 65536;
}

// The one-launch dynamic linear: which of its two kernels, where both take the shape.  The block per CU
// that quantizes the rows once is ahead almost everywhere (cold weights, us, it | a block per 16 channels
// each quantizing the rows: K = N = 4096, M = 4: 7.7 | 8.1; N = 11008, M = 4: 12.3 | 15.2; N = 32000, M = 4:
// 26.3 | 35.2; N = 4096, K = 1024, M = 16: 6.1 | 7.0; N = 16384, K = 1024, M = 1: 6.7 | 10.3; N = 4096,
// K = 8192, M = 1: 9.8 | 10.1), except one or two rows against a single round of blocks at K = 4096
// (K = N = 4096, M = 1: 6.6 | 6.1).
bool dynamic_resident_preferred(int64_t M, int64_t N, int64_t K) {
  return !(M <= 2 && N <= 4096 && K > 2048 && K <= 4096);
}

// forced: tmq_linear_desc::kernel - 1 (-1 = automatic choice).
LinearChoice choose_linear(const LinearQuery& q, int forced) {
  LinearChoice c;
  if (!q.vec_ok || forced == 9) {
    c.cfg = 9;
    return c;
  }
  if (forced < 0 && huge_n_tiles_preferred(q)) {
    c.cfg = 23;
    return c;
  }
  if (forced < 0 && resident_preferred(q)) {
    c.cfg = 28;
    return c;
  }
  const bool stream_auto =
      forced < 0 && (q.M <= kDecodeRowsAuto ||
                     (q.M <= kDecodeMaxRows &&
                      small_rows_path(q.M, q.N, q.K, q.workspace_attached && q.K % 16 == 0) == SmallRows::kStream));
  if (stream_auto || forced == 8) {
    c.cfg = stream_limits_ok(q) ? 8 : kNoKernel;
    return c;
  }
  const bool dma_ok = dma_limits_ok(q.K, q.ldx);
  if (forced < 0 || forced == 13) {
    const SplitPlan p = forced == 13 ? plan_split_tiles(q.M, q.N, q.K) : plan_split(q.M, q.N, q.K);
    if (p.splits > 1 && q.workspace_bytes >= split_workspace_bytes(p, q.M)) {
      c.cfg = 13;
      c.split = p;
      return c;
    }
    if (forced == 13) return c;
  }
  const bool onepass_ok = onepass_limits_ok(q);
  const int64_t M = q.M, N = q.N, K = q.K;
  int cfg = forced;
  if (cfg < 0 && onepass_ok && K <= kOnePassMaxK && ceil_div(M, 64) * ceil_div(N, 64) <= 256) {
    // short K on a grid no larger than the chip: one latency instead of one per stage
    // (M = 128, K = N = 1024: 6.0 -> 5.6 us with cold weights); up to 512 tiles of 32 x 32
    // whose waves split K spread the copies over more CUs (3.8 us; M = 512: 5.7 -> 4.4 us;
    // N = 4096, K = 512, M = 128: 4.4 -> 4.3 us; 640 tiles and more, or K <= 256: slower)
    cfg = K > 256 && ceil_div(M, 32) * ceil_div(N, 32) <= 512 ? 24 : 21;
  } else if (cfg < 0 && onepass_ok && wstream_tile(M, N, K) != 0) {
    // K up to 4096 on a grid of 32 x 32 tiles that the chip holds at once: the waves split
    // K and take their weights through registers (cold weights, K = N = 4096, M = 64:
    // 12.2 -> 8.6 us; K = 2048, N = 4096: M = 64 9.4 -> 5.5 us, M = 128 9.4 -> 7.0 us;
    // K = N = 2048: M = 128 7.8 -> 5.0 us, M = 256 8.0 -> 6.3 us)
    cfg = wstream_tile(M, N, K) == 32 ? 25 : 26;
  } else if (cfg < 0) {
    // Thresholds from timing sweeps over M, N, K on the chip (256 CUs, cold weights): the
    // 256x256 tile (one block per CU) wins from 129 tiles on, the 128x256 tile while
    // it fits one round, the 128x128 tile (two blocks per CU) down to 128 tiles.
    const auto nblk = [&](int bm, int bn) { return ceil_div(M, bm) * ceil_div(N, bn); };
    // (and only when the rows fill at least 55 % of the row tiles: a tile's time
    // does not shrink with its padding; M = 100 and 150 against N = 49152 sit on
    // either side)
    const auto rows_used = [&](int bm) { return M * 20 >= ceil_div(M, bm) * bm * 11; };
    // One block of either large tile runs per CU.  The 128x256 tile (128 activation rows,
    // 256 channels; 8 waves of 64x64) keeps a single round to itself (M = 2048, N = 4096,
    // 256 tiles: 34.4 us against 40.1 us for 128 tiles of 256x256); once it needs a second
    // round the 256x256 tiles take over (M = 768, N = 11008, 129 tiles: 43.4 against 49.4 us;
    // M = 3072, K = N = 3072, 144 tiles: 34.3 against 39.1 us), except just past a full round
    // of them, where the second round of 256x256 tiles is nearly empty and three rounds of
    // 128x256 are shorter (258 tiles, M = 1536, N = 11008: 84.9 against 91.8 us; 344 tiles:
    // 90.6 against 91.6 us; at 375 ... 384 tiles the two are within 4 % of each other, either
    // way round from box to box; 430 tiles: 102.4 against 115.8 us; at 516 tiles, just past
    // two rounds, the two are level: 146.8 against 146.3 us).  Its
    // mirror image, 256 rows x 128 channels, is 17 % slower than 256x256 at C3: activation
    // rows arrive as 64-byte pieces of far-apart rows, weight rows as 256-byte pieces of
    // the packed layout.
    const int64_t t256 = nblk(256, 256), t128x256 = nblk(128, 256);
    // (the 128x256 tile's activation copies two stages wide pay within one round of tiles only:
    // M = 512, N = 11008: 36.3 -> 32.7 us, but M = 1024, N = 11008: 53.0 -> 57.7 us)
    const int cfg128x256 = t128x256 <= 256 ? 19 : 17;
    // equal tile counts: the 64 x 128 tile; more row tiles than its mirror image has fewer
    // blocks and idle CUs (M = 192: N = 6144, K = 3072: 17.1 against 15.3 us with 128 x 64;
    // N = 4096, K = 11008: 46.8 against 43.4 us); up to 96 rows fill three of the 128 x 64 tile's
    // four row strips and it is ahead at equal counts too (M = 96, N = 13824, K = 5120: 28.4
    // against 31.0 us; N = 11008, K = 4096: 20.2 against 21.2 us)
    const int cfg_half =
        nblk(128, 64) <= 256 && (nblk(128, 64) > nblk(64, 128) || (M <= 96 && nblk(128, 64) == nblk(64, 128))) ? 22 : 23;
    // Many rows against a short K are bound by the epilogue, and 256-channel tiles requantise the padding behind
    // N as well: 128 x 128 tiles where those pad a quarter less (M = 100352 pixels of a 56 x 56 feature map at batch
    // 32: N = 384, K = 96: 35.1 -> 27 us; N = 96, K = 384: 20.9 -> 15.7 us; N = 512, K = 128 has nothing to gain and
    // stays: 10.4 against 12.5 us).
    const bool padding_bound = K <= 512 && round_up(N, 256) * 4 >= round_up(N, 128) * 5;
    if (t128x256 > 256 && rows_used(256) && padding_bound)
      cfg = 7;
    else if (t128x256 > 256 && rows_used(256))
      cfg = t256 > 256 && t256 <= 400 ? 17 : 6;  // 6: 8 waves of 128x64, operands copied straight into LDS
    else if (t128x256 >= 160 && rows_used(128))
      // (barely more than half a round of them, against a long K: 128x128 tiles, at most 320,
      // all resident at once: M = 640, N = K = 8192: 53.9 against 59.7 us; N = 8192, K = 4096:
      // 30.2 against 31.6 us; at K = 2048 the 128x256 tiles stay ahead)
      cfg = K >= 4096 && nblk(128, 128) <= 320 ? 7 : cfg128x256;
    else if (N >= 2048 && (N >= 4096 || K >= 4096) && nblk(64, 64) > 256 && (nblk(64, 128) <= 256 || M <= 64))
      // a few hundred rows whose 128 x 128 tiles would leave half the chip idle and whose
      // 64 x 64 tiles need a second round: 64 rows x 128 channels, one round (K = N = 4096,
      // cold weights: M = 448: 24.6 -> 19.1 us, M = 512: 24.8 -> 19.3 us; K = 2048: 14.7 -> 11.7 us;
      // N = 8192, M = 192: 25.9 -> 19.9 us; against N = 1024 the 128 x 128 tiles stay ahead:
      // M = 1536, K = 4096: 17.4 against 20.2 us, and at K = N = 2048, M = 1024: 11.5 against 12.2 us);
      // up to 64 rows also over several rounds, ahead of 128 x 128 tiles that are three quarters padding
      // (M = 32, K = 4096: N = 65536 48.2 against 53.4 us, N = 128256 87.7 against 95 us; K = 2048, N = 65536:
      // 26.5 against 30.8 us; N = 49152: level)
      cfg = cfg_half;
    else if (N >= 2048 && (N >= 4096 || K >= 4096) && nblk(64, 64) > 256 && nblk(128, 64) <= 256)
      cfg = 22;
    else if (nblk(128, 128) >= 128 && M > 64)  // (64 tiles: 64x64 wins, 15.2 against 17.9 us at M = 256, K = N = 4096;
                                               // up to 64 rows half of every tile is padding: M = 64, N = 16384, K = 4096:
                                               // 27.5 us against 17.5 us for the 64 x 64 tiles that walk K in phases)
      cfg = 7;
    else if (onepass_ok && K >= 3072 && K <= kWringMaxK && nblk(64, 64) <= 256 && N * K <= (int64_t{3} << 23))
      // one round of 64 x 64 tiles against a long K: eight waves split K, weights through
      // registers, activations through a ring per wave, no barrier before the partial tiles
      // meet (cold weights, K = N = 4096: M = 130 12.1 -> 11.8 us, M = 192 14.0 -> 12.8 us,
      // M = 256 14.3 -> 13.6 us; N = 2048: M = 512 14.0 -> 13.0 us; K = 3072: M = 192
      // 13.0 -> 12.1 us; behind the two wave groups at K = 2560 (12.3 against 11.7 us) and
      // against 32 MB of weights, N = 8192: 15.3 against 14.6 us; 24 MB, N = 6144, K = 4096,
      // M = 128: 13.7 against 15.0 us)
      cfg = 27;
    else if (onepass_ok && phased_ring_preferred(M, N, K))
      cfg = 21;
    else if (nblk(64, 64) <= 256 && ceil_div(K, kBK) >= 32 && ceil_div(K, kBK) % 2 == 0)
      cfg = 14;  // at most one block per CU and a long k loop: two wave groups halve it (14.7 -> 11.7 us
                 // at M = 128, K = N = 4096; four groups run into the L2's bandwidth: 12.3 us)
    else
      cfg = 2;
  }
  const bool wide_ok = wide_limits_ok(K, q.ldx);
  if (cfg == 19 && !wide_ok) cfg = 17;
  // 256 x 256 tiles with byte or float outputs: the persistent kernel, which hides each
  // tile's pipeline fill behind the tile before it and whose epilogue needs no block
  // barrier (also ahead on a single round: M = N = K = 4096, 256 tiles: 61.9 -> 59.7 us;
  // 2560 x 4096: 46.4 -> 45.8 us; never behind in a sweep of one to three rounds)
  if (forced < 0 && cfg == 6 && wide_ok && q.mode != kOutAcc32) cfg = 20;
  if (cfg == 20 && q.mode == kOutAcc32) cfg = 6;  // raw outputs: one tile per block
  if (cfg == 20 && !wide_ok) cfg = 3;
  if (cfg == 6 && !wide_ok) cfg = 3;
  if (cfg == 17 && !dma_ok) cfg = 3;
  if (cfg == 7 && !wide_ok) cfg = 1;
  switch (cfg) {
    case 0: case 1: case 2: case 3: case 4: case 5: case 6: case 7: case 17: case 19: case 20: case 22: case 23:
      break;
    case 14:  // two wave groups: equal runs of stages only
      if (ceil_div(K, kBK) % 2 != 0) cfg = kNoKernel;
      break;
    case 21:
      if (!onepass_ok) cfg = kNoKernel;
      break;
    case 24:
      if (!onepass_ok || K > kOnePassMaxK) cfg = kNoKernel;
      break;
    case 25: case 26:
      if (!onepass_ok || K > 4096) cfg = kNoKernel;
      break;
    case 27:
      if (!onepass_ok || K > kWringMaxK) cfg = kNoKernel;
      break;
    case 28:
      if (!resident_limits_ok(M, N, K, q.ldx, 256)) cfg = kNoKernel;
      break;
    default:
      cfg = kNoKernel;
  }
  c.cfg = cfg;
  return c;
}

template <int MODE>
int dispatch_linear(const GemmArgs& a, const XLinear& xs, int x_signed, bool vec_ok, int forced,
                    hipStream_t s, void* workspace = nullptr, int64_t workspace_bytes = 0) {
  LinearQuery q;
  q.M = a.M;
  q.N = a.N;
  q.K = a.K;
  q.ldx = xs.ldx;
  q.n_off = a.n_off;
  q.mode = MODE;
  q.vec_ok = vec_ok;
  q.workspace_attached = workspace != nullptr;
  q.workspace_bytes = workspace != nullptr && aligned(workspace, 16) ? workspace_bytes : 0;
  if (a.splits != 1) return TMQ_ERR_INVALID_ARGUMENT;  // the split is this function's to plan
  const LinearChoice c = choose_linear(q, forced);
  switch (c.cfg) {
    case 9: {
      // plain kernel accumulates true activation values: undo the +128 share
      GemmArgs b = a;
      if (!x_signed) {
        b.acc_coef -= 128;
        b.acc_base -= 128;
      }
      const int64_t work = a.M * ceil_div(a.N, 4);
      const int64_t blocks = ceil_div(work, 256);
      if (blocks > 0x7fffffff) return TMQ_ERR_UNSUPPORTED;
      linear_plain_kernel<MODE><<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s>>>(b, xs, x_signed);
      return launch_status();
    }
    case 8: return launch_linear_decode<MODE>(a, xs, s);
    case 28: {
      const int rc = launch_linear_resident<MODE>(a, xs, s);
      // (a device with too few CUs for this many channel groups: the automatic choice streams instead)
      return rc == TMQ_ERR_UNSUPPORTED && forced < 0 && stream_limits_ok(q) ? launch_linear_decode<MODE>(a, xs, s) : rc;
    }
    case 13: return run_split<MODE>(a, xs, c.split, workspace, dma_limits_ok(a.K, xs.ldx), s);
    case 0: return launch_gemm<256, 256, 2, 2, MODE>(a, xs, s);
    case 1: return launch_gemm<128, 128, 2, 2, MODE>(a, xs, s);
    case 2: return launch_gemm<64, 64, 2, 2, MODE>(a, xs, s);
    case 3: return launch_gemm<256, 256, 2, 4, MODE, 3>(a, xs, s);
    case 4: return launch_gemm<128, 256, 2, 2, MODE>(a, xs, s);
    case 5: return launch_gemm<256, 128, 2, 2, MODE>(a, xs, s);
    case 6: return launch_gemm<256, 256, 2, 4, MODE, 3, true, 1, true>(a, xs, s);
    case 7: return launch_gemm<128, 128, 2, 2, MODE, 3, true, 1, true>(a, xs, s);
    case 14: return launch_gemm<64, 64, 2, 2, MODE, 4, false, 2>(a, xs, s);
    case 17: return launch_gemm<128, 256, 2, 4, MODE, 3, true>(a, xs, s);
    case 19: return launch_gemm<128, 256, 2, 4, MODE, 3, true, 1, true>(a, xs, s);
    case 20: return launch_gemm_persistent<MODE>(a, xs, s);
    case 22: return launch_gemm<128, 64, 2, 2, MODE>(a, xs, s);
    case 23: return launch_gemm<64, 128, 2, 2, MODE>(a, xs, s);
    case 21: return launch_gemm_onepass<MODE>(a, xs, s);
    case 24: return launch_gemm_ksplit<MODE>(a, xs, s);
    case 25: return launch_gemm_wstream<MODE>(a, xs, false, s);
    case 26: return launch_gemm_wstream<MODE>(a, xs, true, s);
    case 27: return launch_gemm_wring<MODE>(a, xs, s);
    default: return TMQ_ERR_UNSUPPORTED;
  }
}

int fill_args(const tmq_linear_desc* d, GemmArgs* a, XLinear* xs, bool* vec_ok) {
  if (d == nullptr) return TMQ_ERR_INVALID_ARGUMENT;
  if (d->M < 0 || d->N < 0 || d->K < 0) return TMQ_ERR_INVALID_ARGUMENT;
  if (d->M == 0 || d->N == 0) return TMQ_OK;
  if (d->x == nullptr && d->K > 0) return TMQ_ERR_INVALID_ARGUMENT;
  if (d->w_packed == nullptr || d->w_colsum == nullptr) return TMQ_ERR_INVALID_ARGUMENT;
  if (d->ldx < d->K) return TMQ_ERR_INVALID_ARGUMENT;
  if (!aligned(d->w_packed, 16)) return TMQ_ERR_ALIGNMENT;
  a->M = d->M;
  a->N = d->N;
  a->K = d->K;
  a->w_packed = static_cast<const uint8_t*>(d->w_packed);
  a->w_kchunks = packed_kchunks(d->K);
  a->colsum = d->w_colsum;
  a->x_xor = d->x_signed ? 0u : 0x80808080u;
  a->n_off = 0;
  xs->x = static_cast<const uint8_t*>(d->x);
  xs->ldx = d->ldx;
  *vec_ok = d->K >= 16 && d->K % 16 == 0 && d->ldx % 16 == 0 && aligned(d->x, 16);
  return TMQ_OK;
}

}  // namespace
}  // namespace tmq

using namespace tmq;

TMQ_EXPORT int64_t tmq_linear_packed_kchunks(int64_t K) { return K < 0 ? 0 : packed_kchunks(K); }

TMQ_EXPORT int64_t tmq_linear_packed_bytes(int64_t N, int64_t K) {
  if (N < 0 || K < 0) return 0;
  return ceil_div(N, 16) * packed_kchunks(K) * 256;
}

TMQ_EXPORT int tmq_linear_prepack(const int8_t* w, int64_t N, int64_t K, int64_t ldw, void* packed,
                                  int32_t* colsum, tmq_stream_t stream) {
  if (N < 0 || K < 0 || ldw < K) return TMQ_ERR_INVALID_ARGUMENT;
  if (N == 0) return TMQ_OK;
  if (packed == nullptr || colsum == nullptr || (w == nullptr && K > 0))
    return TMQ_ERR_INVALID_ARGUMENT;
  if (!aligned(packed, 16)) return TMQ_ERR_ALIGNMENT;
  hipStream_t s = as_stream(stream);
  const int64_t KC = packed_kchunks(K);
  const int64_t total = ceil_div(N, 16) * KC * 16;
  const bool vec = aligned(w, 16) && ldw % 16 == 0;
  if (total > 0) {
    const int64_t blocks = ceil_div(total, 256);
    if (blocks > 0x7fffffff) return TMQ_ERR_UNSUPPORTED;
    prepack_kernel<<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s>>>(
        w, N, K, ldw, KC, total, vec, static_cast<uint8_t*>(packed));
    if (launch_status() != TMQ_OK) return TMQ_ERR_LAUNCH;
  }
  const int64_t blocks = ceil_div(N, 256 / kWave);
  if (blocks > 0x7fffffff) return TMQ_ERR_UNSUPPORTED;
  colsum_kernel<<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s>>>(w, N, K, ldw, vec, colsum);
  return launch_status();
}

TMQ_EXPORT int tmq_linear_unpack(const void* packed, int64_t N, int64_t K, int8_t* w, int64_t ldw,
                                 tmq_stream_t stream) {
  if (N < 0 || K < 0 || ldw < K) return TMQ_ERR_INVALID_ARGUMENT;
  if (N == 0 || K == 0) return TMQ_OK;
  if (packed == nullptr || w == nullptr) return TMQ_ERR_INVALID_ARGUMENT;
  const int64_t blocks = ceil_div(N * K, 256);
  if (blocks > 0x7fffffff) return TMQ_ERR_UNSUPPORTED;
  unpack_kernel<<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, as_stream(stream)>>>(
      static_cast<const uint8_t*>(packed), N, K, ldw, packed_kchunks(K), w);
  return launch_status();
}

TMQ_EXPORT int64_t tmq_linear_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  return split_workspace_bytes(plan_split(M, N, K), M);
}

TMQ_EXPORT int tmq_linear_split_plan(int64_t M, int64_t N, int64_t K, int32_t* splits, int32_t* stages) {
  if (M < 0 || N < 0 || K < 0 || splits == nullptr || stages == nullptr) return TMQ_ERR_INVALID_ARGUMENT;
  const SplitPlan p = (M > 0 && N > 0 && K > 0) ? plan_split(M, N, K) : SplitPlan{};
  *splits = p.splits;
  *stages = p.stages;
  return TMQ_OK;
}

static_assert(sizeof(tmq_linear_choice) == 48, "tmq_linear_choice layout changed");

TMQ_EXPORT int tmq_linear_kernel_choice(int64_t M, int64_t N, int64_t K, int64_t ldx, int32_t flags,
                                        int32_t forced_kernel, int32_t compute_units, tmq_linear_choice* out) {
  if (out == nullptr || M < 0 || N < 0 || K < 0 || ldx < K || (flags & 3) == 3 || compute_units < 0)
    return TMQ_ERR_INVALID_ARGUMENT;
  *out = tmq_linear_choice{};
  out->splits = 1;
  out->k_stages = ceil_div(K, kBK);
  if (M == 0 || N == 0) return TMQ_OK;  // nothing is launched
  LinearQuery q;
  q.M = M;
  q.N = N;
  q.K = K;
  q.ldx = ldx;
  q.mode = (flags & 3) == TMQ_LINEAR_OUT_F32 ? kOutF32 : (flags & 3) == TMQ_LINEAR_OUT_ACC32 ? kOutAcc32 : kOutU8;
  q.vec_ok = (flags & 8) == 0 && K >= 16 && K % 16 == 0 && ldx % 16 == 0;
  q.workspace_attached = (flags & 4) != 0;
  q.workspace_bytes = q.workspace_attached && K > 0 ? split_workspace_bytes(plan_split(M, N, K), M) : 0;
  const LinearChoice c = choose_linear(q, forced_kernel - 1);
  if (c.cfg == kNoKernel) return TMQ_OK;
  int bm = 0, bn = 0, waves = 4;
  switch (c.cfg) {
    case 0: bm = 256, bn = 256; break;
    case 3: case 6: case 20: bm = 256, bn = 256, waves = 8; break;
    case 1: case 7: case 13: bm = 128, bn = 128; break;
    case 2: case 21: bm = 64, bn = 64; break;
    case 14: bm = 64, bn = 64, waves = 8; break;
    case 4: bm = 128, bn = 256; break;
    case 17: case 19: bm = 128, bn = 256, waves = 8; break;
    case 5: bm = 256, bn = 128; break;
    case 22: bm = 128, bn = 64; break;
    case 23: bm = 64, bn = 128; break;
    case 24: case 25: bm = 32, bn = 32; break;
    case 26: bm = 32, bn = 64, waves = 8; break;
    case 27: bm = 64, bn = 64, waves = 8; break;
    case 8: bm = 16 * static_cast<int>(ceil_div(M, 16)), bn = 16, waves = kDecodeWaves; break;
    case 28: bm = 16 * static_cast<int>(ceil_div(M, 16)), bn = 16, waves = resident_pair(M, N, K, compute_units) ? 8 : kResidentWaves; break;
    default: break;  // 9: one thread per four outputs
  }
  out->kernel = c.cfg + 1;
  out->tile_rows = bm;
  out->tile_channels = bn;
  out->waves = waves;
  out->splits = c.split.splits;
  out->split_stages = c.split.stages;
  if (c.cfg == 9) {
    out->tiles = out->blocks = ceil_div(M * ceil_div(N, 4), 256);
  } else {
    out->tiles = ceil_div(M, bm) * ceil_div(N, bn) * c.split.splits;
    out->blocks = out->tiles;
    if (c.cfg == 20 && out->tiles > compute_units) out->blocks = compute_units / 8 * 8;
    if (c.cfg == 28) out->blocks = std::min<int64_t>(out->tiles, (waves == 8 ? 2 : 1) * static_cast<int64_t>(compute_units));
  }
  return TMQ_OK;
}

namespace tmq {
namespace {

// quantized::linear with the split-K scratch passed beside the descriptor.
int linear_u8s8(const tmq_linear_desc* d, void* workspace, int64_t workspace_bytes, tmq_stream_t stream) {
  GemmArgs a{};
  XLinear xs{};
  bool vec_ok = false;
  const int rc = fill_args(d, &a, &xs, &vec_ok);
  if (rc != TMQ_OK || d->M == 0 || d->N == 0) return rc;
  if (d->y == nullptr || d->w_scales == nullptr || d->ldy < d->N) return TMQ_ERR_INVALID_ARGUMENT;
  if (!(d->x_scale > 0.f) || !(d->out_scale > 0.f)) return TMQ_ERR_INVALID_ARGUMENT;
  const int qmin = d->out_signed ? -128 : 0, qmax = d->out_signed ? 127 : 255;
  if (d->out_zero_point < qmin || d->out_zero_point > qmax) return TMQ_ERR_INVALID_ARGUMENT;
  a.w_scales = d->w_scales;
  a.w_scale_stride = d->w_per_channel ? 1 : 0;
  a.bias = d->bias;
  a.acc_coef = (d->x_signed ? 0 : 128) - d->x_zero_point;
  a.x_scale = d->x_scale;
  a.out_scale = d->out_scale;
  a.zp_f = static_cast<float>(d->out_zero_point);
  a.lo_f = static_cast<float>(d->relu ? d->out_zero_point : qmin);
  a.hi_f = static_cast<float>(qmax);
  a.y = d->y;
  a.ldy = d->ldy;
  hipStream_t s = as_stream(stream);
  return d->out_signed
             ? dispatch_linear<kOutS8>(a, xs, d->x_signed, vec_ok, d->kernel - 1, s, workspace, workspace_bytes)
             : dispatch_linear<kOutU8>(a, xs, d->x_signed, vec_ok, d->kernel - 1, s, workspace, workspace_bytes);
}

}  // namespace
}  // namespace tmq

TMQ_EXPORT int tmq_linear(const tmq_linear_desc* d, tmq_stream_t stream) {
  if (d == nullptr) return TMQ_ERR_INVALID_ARGUMENT;
  return linear_u8s8(d, d->workspace, d->workspace_bytes, stream);
}

// ---------------------------------------------------------------------------
// quantized::linear for callers that cannot allocate: the split-K partial sums
// go to a fixed array in the library's own device memory.
// ---------------------------------------------------------------------------
namespace tmq {
namespace {

// Every split plan fits: splits x tiles <= 256 blocks of 128 x 128 int32 sums.
constexpr int64_t kStaticWorkspaceBytes = int64_t{16} << 20;
static_assert(kStaticWorkspaceBytes == TMQ_LINEAR_STATIC_WORKSPACE_BYTES, "header and library disagree");
static __device__ __align__(256) uint8_t scratch[kStaticWorkspaceBytes];

// Device address of `scratch` on every device used so far.  The array's name
// is a host-side handle in host code; each device holds its own copy of the
// array at its own address, which hipGetSymbolAddress reports for the current
// device.  Two threads that race on a device's first call store the same value.
std::atomic<void*> g_scratch_addr[kMaxDevices];

// The array of the device that owns `s` -- which must be the current device: the
// symbol's address can only be asked for on the current device.
int static_workspace(hipStream_t s, void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return TMQ_ERR_LAUNCH;
  if (s != nullptr) {
    int sdev = -1;
    if (hipStreamGetDevice(s, &sdev) != hipSuccess) {
      (void)hipGetLastError();
      return TMQ_ERR_INVALID_ARGUMENT;
    }
    if (sdev != dev) return TMQ_ERR_INVALID_ARGUMENT;  // another GPU's stream: that GPU has its own array
  }
  void* p = g_scratch_addr[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr) return TMQ_ERR_LAUNCH;
    g_scratch_addr[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return TMQ_OK;
}

}  // namespace
}  // namespace tmq

TMQ_EXPORT int tmq_linear_static_workspace(const tmq_linear_desc* d, tmq_stream_t stream) {
  if (d == nullptr) return TMQ_ERR_INVALID_ARGUMENT;
  if (d->M < 0 || d->N < 0 || d->K < 0) return TMQ_ERR_INVALID_ARGUMENT;
  const int64_t need = (d->M > 0 && d->N > 0 && d->K > 0) ? split_workspace_bytes(plan_split(d->M, d->N, d->K), d->M) : 0;
  if (need > kStaticWorkspaceBytes) return TMQ_ERR_WORKSPACE;  // the caller's own workspace and tmq_linear then
  void* ws = nullptr;
  if (need > 0) {
    const int rc = static_workspace(as_stream(stream), &ws);
    if (rc != TMQ_OK) return rc;
  }
  return linear_u8s8(d, ws, need, stream);
}

TMQ_EXPORT int tmq_linear_acc32(const tmq_linear_desc* d, int32_t* acc, int64_t ldacc,
                                tmq_stream_t stream) {
  GemmArgs a{};
  XLinear xs{};
  bool vec_ok = false;
  const int rc = fill_args(d, &a, &xs, &vec_ok);
  if (rc != TMQ_OK || d->M == 0 || d->N == 0) return rc;
  if (acc == nullptr || ldacc < d->N) return TMQ_ERR_INVALID_ARGUMENT;
  a.acc_coef = d->x_signed ? 0 : 128;  // undo the x ^ 0x80 shift only
  a.y = acc;
  a.ldy = ldacc;
  return dispatch_linear<kOutAcc32>(a, xs, d->x_signed, vec_ok, d->kernel - 1, as_stream(stream), d->workspace,
                                    d->workspace_bytes);
}

TMQ_EXPORT int tmq_linear_f32(const tmq_linear_desc* d, const tmq_qparams* x_qparams_dev, float* y,
                              int64_t ldy, tmq_stream_t stream) {
  GemmArgs a{};
  XLinear xs{};
  bool vec_ok = false;
  const int rc = fill_args(d, &a, &xs, &vec_ok);
  if (rc != TMQ_OK || d->M == 0 || d->N == 0) return rc;
  if (y == nullptr || d->w_scales == nullptr || ldy < d->N) return TMQ_ERR_INVALID_ARGUMENT;
  if (x_qparams_dev == nullptr && !(d->x_scale > 0.f)) return TMQ_ERR_INVALID_ARGUMENT;
  if (!aligned(y, 4)) return TMQ_ERR_ALIGNMENT;
  a.w_scales = d->w_scales;
  a.w_scale_stride = d->w_per_channel ? 1 : 0;
  a.bias = d->bias;
  a.acc_base = d->x_signed ? 0 : 128;
  a.acc_coef = a.acc_base - d->x_zero_point;
  a.x_scale = d->x_scale;
  a.x_qp_dev = x_qparams_dev;
  a.out_scale = 1.f;
  a.lo_f = d->relu ? 0.f : -__builtin_inff();
  a.y = y;
  a.ldy = ldy;
  return dispatch_linear<kOutF32>(a, xs, d->x_signed, vec_ok, d->kernel - 1, as_stream(stream), d->workspace,
                                  d->workspace_bytes);
}

// The float rows of the one-launch dynamic linear as the resident kernel holds them: 16 waves x 64
// lanes x up to 8 groups of four values (16 groups -- M = 16 at K = 4096 -- spill registers and every
// CU then reads 256 KB of rows: 14.2 us against 11.0 us for the two launches at N = 4096).
constexpr int64_t kDynResidentMaxValues = 32768;

TMQ_EXPORT int tmq_linear_dynamic_small_takes(int64_t M, int64_t N, int64_t K) {
  if (M < 1 || M > 16 || N < 1 || K < 16 || K % 16 != 0 || ceil_div(N, 16) > 0x7fffffff) return 0;
  if (M * K <= kDynSmallMaxValues) return 1;
  const int cus = cu_count();
  return M * K <= kDynResidentMaxValues && resident_limits_ok(M, N, K, K, cus > 0 ? cus : 256) ? 1 : 0;
}

TMQ_EXPORT int tmq_linear_dynamic_small(const tmq_linear_desc* d, const float* x, int64_t ldx, int reduce_range,
                                        float* y, int64_t ldy, tmq_stream_t stream) {
  if (d == nullptr) return TMQ_ERR_INVALID_ARGUMENT;
  if (d->M < 0 || d->N < 0 || d->K < 0) return TMQ_ERR_INVALID_ARGUMENT;
  if (d->M == 0 || d->N == 0) return TMQ_OK;
  if (d->M > 16 || d->K < 16 || d->K % 16 != 0) return TMQ_ERR_UNSUPPORTED;
  if (x == nullptr || y == nullptr || d->w_packed == nullptr || d->w_colsum == nullptr || d->w_scales == nullptr)
    return TMQ_ERR_INVALID_ARGUMENT;
  if (ldx < d->K || ldy < d->N) return TMQ_ERR_INVALID_ARGUMENT;
  if (!aligned(x, 16) || ldx % 4 != 0 || !aligned(d->w_packed, 16) || !aligned(y, 4)) return TMQ_ERR_UNSUPPORTED;
  const int64_t blocks = ceil_div(d->N, 16);
  if (blocks > 0x7fffffff) return TMQ_ERR_UNSUPPORTED;
  GemmArgs a{};
  a.M = d->M;
  a.N = d->N;
  a.K = d->K;
  a.w_packed = static_cast<const uint8_t*>(d->w_packed);
  a.w_kchunks = packed_kchunks(d->K);
  a.colsum = d->w_colsum;
  a.w_scales = d->w_scales;
  a.w_scale_stride = d->w_per_channel ? 1 : 0;
  a.bias = d->bias;
  a.lo_f = d->relu ? 0.f : -__builtin_inff();
  a.y = y;
  a.ldy = ldy;
  hipStream_t s = as_stream(stream);
  // Two kernels: a block per 16 channels that repeats the work on the input (up to 16384 values), and
  // one block per CU that does it once for all its channel groups (up to 32768 values, K <= 8192).
  // desc->kernel pins one for tests: 9 the first, 29 the second.
  const int cus = cu_count();
  const bool resident_ok = d->M * d->K <= kDynResidentMaxValues && resident_limits_ok(d->M, d->N, d->K, d->K, cus);
  const bool small_ok = d->M * d->K <= kDynSmallMaxValues;
  if ((d->kernel == 9 && !small_ok) || (d->kernel == 29 && !resident_ok) || (!small_ok && !resident_ok))
    return TMQ_ERR_UNSUPPORTED;
  const bool resident =
      resident_ok && (d->kernel == 29 || (d->kernel != 9 && (!small_ok || dynamic_resident_preferred(d->M, d->N, d->K))));
  if (resident) {
    const XLinear none{nullptr, 0};
    const dim3 grid(static_cast<unsigned>(blocks < cus ? blocks : cus)), block(kResidentThreads);
    const int64_t held = ceil_div(d->M * d->K / 4, kResidentThreads);  // float4 per thread
    if (held <= 2)
      linear_resident_kernel<kOutF32, 1, kResidentWaves, 2><<<grid, block, 0, s>>>(a, none, x, ldx, reduce_range);
    else if (held <= 4)
      linear_resident_kernel<kOutF32, 1, kResidentWaves, 4><<<grid, block, 0, s>>>(a, none, x, ldx, reduce_range);
    else
      linear_resident_kernel<kOutF32, 1, kResidentWaves, 8><<<grid, block, 0, s>>>(a, none, x, ldx, reduce_range);
    return launch_status();
  }
  const size_t lds = static_cast<size_t>(d->M) * static_cast<size_t>(d->K + 16);
  const dim3 grid(static_cast<unsigned>(blocks)), block(kDecodeWaves * kWave);
  const int64_t groups = ceil_div(d->M * d->K / 4, kDecodeWaves * kWave);  // float4 per thread
  if (groups <= 1)
    linear_decode_dynamic_kernel<1><<<grid, block, lds, s>>>(a, x, ldx, reduce_range);
  else if (groups <= 2)
    linear_decode_dynamic_kernel<2><<<grid, block, lds, s>>>(a, x, ldx, reduce_range);
  else if (groups <= 4)
    linear_decode_dynamic_kernel<4><<<grid, block, lds, s>>>(a, x, ldx, reduce_range);
  else
    linear_decode_dynamic_kernel<8><<<grid, block, lds, s>>>(a, x, ldx, reduce_range);
  return launch_status();
}
