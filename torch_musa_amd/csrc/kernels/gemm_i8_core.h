// int8 MFMA GEMM core for gfx950, shared by quantized::linear and the NHWC
// implicit-GEMM quantized::conv2d.
//
//   acc[n][m] = sum_k W[n][k] * X[m][k]          (int32, exact)
//
// The weight is the MFMA "A" operand and the activations the "B" operand, so a
// lane ends up holding four consecutive output channels of one output row and
// can pack them into one 32-bit store of the row-major [M,N] result.
//
// Operands: v_mfma_i32_32x32x32_i8 takes 16 consecutive k-bytes of one row per
// lane (lanes 0-31: rows 0-31 of k-chunk 2s, lanes 32-63: the same rows of
// k-chunk 2s+1).  The instruction multiplies signed bytes; quint8 activations
// are fed as x ^ 0x80 (= x - 128) and the exact difference 128 * colsum[n] is
// folded, with the activation zero point, into the accumulator's start value:
//   acc_0[n] = (128 - x_zp) * colsum[n]   (quint8)      -x_zp * colsum[n] (qint8)
// so the main loop ends with raw = sum_k (x - x_zp) * w, all in int32.
//
// LDS staging (64 k-bytes per stage, two stages):
//   weights     [k-chunk][row][16 B]      straight copy of the packed layout,
//                                         lanes read consecutive 16-byte slots
//   activations [row][64 B], the 16-byte slot index XOR-ed with
//               ((row >> 1) ^ (row >> 3)) & 3, so that both the row-major fill
//               and the column-wise operand reads of any 8 or 16 consecutive
//               lanes fall into distinct 16-byte bank groups
// Pipeline per stage: registers -> LDS for stage t+1, global -> registers for
// stage t+2, MFMAs on stage t, one barrier.
#pragma once

#include "common.h"

namespace tmq {

constexpr int kBK = 64;       // k-bytes per LDS stage
constexpr int kChunks = 4;    // 16-byte k-chunks per stage

enum EpilogueMode { kOutU8 = 0, kOutS8 = 1, kOutAcc32 = 2 };

// Where a tile's activation rows come from.
struct XLinear {
  const uint8_t* x;
  int64_t ldx;
};

struct XConv {
  const uint8_t* x;  // NHWC
  int H, W, IC;      // IC = all input channels (row pitch of a pixel)
  int OH, OW;
  int KW, icb;       // icb = 16-byte blocks per tap (ICg / 16)
  int stride_h, stride_w, pad_h, pad_w, dil_h, dil_w;
  int ic_off;        // first input channel of this group
  uint32_t pad_word; // activation zero point replicated in 4 bytes
};

struct GemmArgs {
  int64_t M, N;          // logical problem (N = rows of this weight matrix)
  int64_t K;             // k extent in bytes, multiple of 16
  const uint8_t* w_packed;
  int64_t w_kchunks;     // packed k-chunks per 16-row block
  const int32_t* colsum; // [N]
  const float* w_scales; // [N] or [1]
  const float* bias;     // [N] or null
  int32_t w_scale_stride;  // 1: per channel, 0: per tensor
  uint32_t x_xor;        // 0x80808080 for quint8 activations, 0 for qint8
  int32_t acc_coef;      // multiplies colsum[n] into the accumulator start
  float x_scale, out_scale;
  float zp_f, lo_f, hi_f;  // output zero point and clamp bounds
  void* y;               // bytes [M, ldy] or int32 [M, ldy]
  int64_t ldy;
  int32_t n_off;         // conv groups: channel offset of this group in y/params
};

__device__ __forceinline__ v4i ld16(const void* p) { return *reinterpret_cast<const v4i*>(p); }

template <class XSRC>
struct XLoader;

// One loader per 16-byte chunk slot a thread stages: fixed activation row,
// k-chunk index `kc` supplied per stage.
template <>
struct XLoader<XLinear> {
  const uint8_t* p;
  bool row_ok;
  __device__ __forceinline__ void init(const XLinear& s, int64_t m, int64_t M) {
    row_ok = m < M;
    p = s.x + (row_ok ? m : 0) * s.ldx;
  }
  __device__ __forceinline__ v4i load(const XLinear&, int kc, int64_t K) const {
    const int64_t k = static_cast<int64_t>(kc) * 16;
    if (row_ok && k < K) return ld16(p + k);
    return v4i{0, 0, 0, 0};
  }
};

template <>
struct XLoader<XConv> {
  const uint8_t* img;  // first byte of this row's image (+ group channel offset)
  int ih0, iw0;        // top-left input coordinate of the receptive field
  bool row_ok;
  __device__ __forceinline__ void init(const XConv& s, int64_t m, int64_t M) {
    row_ok = m < M;
    const int64_t mm = row_ok ? m : 0;
    const int ow = static_cast<int>(mm % s.OW);
    const int64_t t = mm / s.OW;
    const int oh = static_cast<int>(t % s.OH);
    const int64_t b = t / s.OH;
    img = s.x + b * (static_cast<int64_t>(s.H) * s.W * s.IC) + s.ic_off;
    ih0 = oh * s.stride_h - s.pad_h;
    iw0 = ow * s.stride_w - s.pad_w;
  }
  // Out-of-image taps read as the activation zero point, i.e. real value 0.
  __device__ __forceinline__ v4i load(const XConv& s, int kc, int64_t K) const {
    const int pw = static_cast<int>(s.pad_word);
    const v4i pad = {pw, pw, pw, pw};
    if (!row_ok || static_cast<int64_t>(kc) * 16 >= K) return pad;
    const int tap = kc / s.icb;
    const int blk = kc - tap * s.icb;
    const int kh = tap / s.KW;
    const int kw = tap - kh * s.KW;
    const int ih = ih0 + kh * s.dil_h;
    const int iw = iw0 + kw * s.dil_w;
    if (ih < 0 || ih >= s.H || iw < 0 || iw >= s.W) return pad;
    return ld16(img + (static_cast<int64_t>(ih) * s.W + iw) * s.IC + blk * 16);
  }
};

// Slot swizzle of the activation stage: see the file header.
__device__ __forceinline__ int x_swizzle(int row) { return ((row >> 1) ^ (row >> 3)) & 3; }

// One requantised byte group: four consecutive channels of one output row.
template <int MODE>
__device__ __forceinline__ uint32_t requant4(const int (&raw)[4], v4f bdiv, v4f mult, float zp_f,
                                             float lo_f, float hi_f) {
  uint32_t packed = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    float v = static_cast<float>(raw[j]);  // int -> fp32, round to nearest even
    v = v + bdiv[j];
    const float ab = v * mult[j];
    float r = __builtin_rintf(ab) + zp_f;
    r = __builtin_amdgcn_fmed3f(r, lo_f, hi_f);
    if constexpr (MODE == kOutU8) {
      packed = __builtin_amdgcn_cvt_pk_u8_f32(r, j, packed);
    } else {
      packed |= (static_cast<uint32_t>(static_cast<int>(r)) & 0xffu) << (8 * j);
    }
  }
  return packed;
}

// BM x BN output tile per block (BM activation rows, BN weight rows),
// WM x WN waves, each wave (BM/WM) x (BN/WN).
template <int BM, int BN, int WM, int WN, int MODE, class XSRC>
__global__ __launch_bounds__(WM* WN* kWave) void gemm_i8_kernel(GemmArgs a, XSRC xsrc) {
  constexpr int NT = WM * WN * kWave;
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int NW = BN * kChunks / NT;  // 16-byte weight chunks per thread per stage
  constexpr int NX = BM * kChunks / NT;
  static_assert(TM >= 1 && TN >= 1 && NW >= 1 && NX >= 1, "tile too small for the wave grid");
  static_assert(BN * kChunks % NT == 0 && BM * kChunks % NT == 0, "uneven staging");

  __shared__ __attribute__((aligned(16))) uint8_t sW[2][kChunks * BN * 16];
  __shared__ __attribute__((aligned(16))) uint8_t sX[2][BM * kBK];
  __shared__ __attribute__((aligned(16))) int s_acc0[BN];
  __shared__ __attribute__((aligned(16))) float s_mult[BN];
  __shared__ __attribute__((aligned(16))) float s_bdiv[BN];

  const int t = threadIdx.x;
  const int lane = t % kWave, wave = t / kWave;
  const int li = lane & 31, half = lane >> 5;
  const int wm0 = (wave % WM) * WTM;
  const int wn0 = (wave / WM) * WTN;

  // ---- tile assignment: blocks are dealt round-robin to the 8 XCDs; give each
  // XCD one contiguous run of tiles (row tiles fastest) so its L2 sees reuse.
  const int64_t tiles_m = ceil_div(a.M, BM), tiles_n = ceil_div(a.N, BN);
  const int64_t nblocks = tiles_m * tiles_n;
  int64_t tile;
  {
    const int64_t bid = blockIdx.x;
    const int64_t q = nblocks / 8, rem = nblocks % 8;
    const int64_t xcd = bid % 8, within = bid / 8;
    tile = xcd * q + (xcd < rem ? xcd : rem) + within;
  }
  const int64_t m0 = (tile % tiles_m) * BM;
  const int64_t n0 = (tile / tiles_m) * BN;
  const int64_t NB = ceil_div(a.N, 16);

  // ---- per-channel constants of this tile's BN output channels
  for (int i = t; i < BN; i += NT) {
    const int64_t n = n0 + i;
    int acc0 = 0;
    float mult = 0.f, bdiv = 0.f;
    if (n < a.N) {
      const int64_t np = n + a.n_off;
      acc0 = a.acc_coef * a.colsum[np];
      if (MODE != kOutAcc32) {
        const float atw = a.x_scale * a.w_scales[np * a.w_scale_stride];
        mult = atw / a.out_scale;
        bdiv = a.bias != nullptr ? a.bias[np] / atw : 0.f;
      }
    }
    s_acc0[i] = acc0;
    s_mult[i] = mult;
    s_bdiv[i] = bdiv;
  }

  // ---- staging assignments
  const uint8_t* wsrc[NW];
  bool wok[NW];
  int wdst[NW];
#pragma unroll
  for (int i = 0; i < NW; ++i) {
    const int id = t + i * NT;
    const int nbl = id >> 6, kcl = (id >> 4) & 3, r = id & 15;
    const int64_t nb = n0 / 16 + nbl;
    wok[i] = nb < NB;
    wsrc[i] = a.w_packed + ((wok[i] ? nb : 0) * a.w_kchunks + kcl) * 256 + r * 16;
    wdst[i] = (kcl * BN + nbl * 16 + r) * 16;
  }
  XLoader<XSRC> xl[NX];
  int xdst[NX];
#pragma unroll
  for (int i = 0; i < NX; ++i) {
    const int id = t + i * NT;
    const int row = id >> 2, c = id & 3;
    xl[i].init(xsrc, m0 + row, a.M);
    xdst[i] = row * kBK + ((c ^ x_swizzle(row)) << 4);
  }
  const v4i xmask = {static_cast<int>(a.x_xor), static_cast<int>(a.x_xor),
                     static_cast<int>(a.x_xor), static_cast<int>(a.x_xor)};

  v4i wreg[NW], xreg[NX];
  auto load_global = [&](int kt) {
#pragma unroll
    for (int i = 0; i < NW; ++i)
      wreg[i] = wok[i] ? ld16(wsrc[i] + static_cast<int64_t>(kt) * (kChunks * 256)) : v4i{0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < NX; ++i) xreg[i] = xl[i].load(xsrc, kt * kChunks + (t & 3), a.K);
  };
  auto store_lds = [&](int buf) {
#pragma unroll
    for (int i = 0; i < NW; ++i) *reinterpret_cast<v4i*>(&sW[buf][wdst[i]]) = wreg[i];
#pragma unroll
    for (int i = 0; i < NX; ++i) *reinterpret_cast<v4i*>(&sX[buf][xdst[i]]) = xreg[i] ^ xmask;
  };

  const int KT = static_cast<int>(ceil_div(a.K, kBK));
  load_global(0);
  store_lds(0);
  if (KT > 1) load_global(1);
  __syncthreads();

  // ---- accumulators start at the per-channel offset (see file header)
  v16i acc[TN][TM];
#pragma unroll
  for (int tn = 0; tn < TN; ++tn) {
    v16i init;
#pragma unroll
    for (int r = 0; r < 16; ++r)
      init[r] = s_acc0[wn0 + tn * 32 + 8 * (r >> 2) + 4 * half + (r & 3)];
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) acc[tn][tm] = init;
  }

  const int xswz = x_swizzle(li);
  for (int kt = 0; kt < KT; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < KT) store_lds(buf ^ 1);
    if (kt + 2 < KT) load_global(kt + 2);
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const int c = 2 * s + half;
      v4i wf[TN], xf[TM];
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
        wf[tn] = ld16(&sW[buf][(c * BN + wn0 + tn * 32 + li) * 16]);
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
        xf[tm] = ld16(&sX[buf][(wm0 + tm * 32 + li) * kBK + ((c ^ xswz) << 4)]);
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
          acc[tn][tm] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[tn], xf[tm], acc[tn][tm], 0, 0, 0);
    }
    __syncthreads();
  }

  // ---- epilogue: lane holds, per 32x32 tile, rows n = 8g + 4*half + j (g,j <4)
  // of column m = li.
#pragma unroll
  for (int tn = 0; tn < TN; ++tn) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int nl = wn0 + tn * 32 + 8 * g + 4 * half;
      const int64_t n = n0 + nl;
      if (n >= a.N) continue;
      if constexpr (MODE == kOutAcc32) {
        int32_t* y = static_cast<int32_t*>(a.y);
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
          const int64_t m = m0 + wm0 + tm * 32 + li;
          if (m >= a.M) continue;
          int32_t* dst = y + m * a.ldy + a.n_off + n;
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (n + j < a.N) dst[j] = acc[tn][tm][4 * g + j];
        }
      } else {
        const v4f mult = *reinterpret_cast<const v4f*>(&s_mult[nl]);
        const v4f bdiv = *reinterpret_cast<const v4f*>(&s_bdiv[nl]);
        uint8_t* y = static_cast<uint8_t*>(a.y);
        const bool full = (n + 3 < a.N) && ((a.ldy & 3) == 0) && ((a.n_off & 3) == 0) &&
                          ((reinterpret_cast<uintptr_t>(y) & 3) == 0);
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
          const int64_t m = m0 + wm0 + tm * 32 + li;
          if (m >= a.M) continue;
          int raw[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) raw[j] = acc[tn][tm][4 * g + j];
          const uint32_t packed = requant4<MODE>(raw, bdiv, mult, a.zp_f, a.lo_f, a.hi_f);
          uint8_t* dst = y + m * a.ldy + a.n_off + n;
          if (full) {
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
}

}  // namespace tmq
