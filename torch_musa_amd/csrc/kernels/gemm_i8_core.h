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
//   activations [row][64 B], the 16-byte slot index XOR-ed with (row >> 2) & 3:
//               rows r, r+4, r+8, r+12 start on the same bank and the XOR moves
//               them to four different 16-byte bank groups.  Measured on the
//               chip: column-wise ds_read_b128 of 32 rows runs at 224 B/clk per
//               CU with this swizzle (as fast as consecutive addresses), at
//               128 B/clk with XORs built from (row >> 1) or (row >> 3), and at
//               64 B/clk with none
// Pipeline: see the comment at the software pipeline inside gemm_i8_kernel.
#pragma once

#include <type_traits>

#include "common.h"

namespace tmq {

constexpr int kBK = 64;       // k-bytes per LDS stage
constexpr int kChunks = 4;    // 16-byte k-chunks per stage

// kOutF32: y = fma(float(raw), x_scale * w_scale[n], bias[n]), optionally
// clamped below at 0 -- the float output of a dynamically quantized linear
// (fbgemm's ReQuantizeForFloat as PyTorch's CPU op runs it, one fused
// multiply-add per value).
enum EpilogueMode { kOutU8 = 0, kOutS8 = 1, kOutAcc32 = 2, kOutF32 = 3 };

// Where a tile's activation rows come from.
struct XLinear {
  static constexpr bool kPostOps = false;
  const uint8_t* x;
  int64_t ldx;
};

struct XConv {
  static constexpr bool kPostOps = true;
  const uint8_t* x;  // NHWC
  int H, W, IC;      // IC = all input channels (row pitch of a pixel)
  int OH, OW;
  int KW, icb;       // icb = 16-byte blocks per tap (ICg / 16)
  int stride_h, stride_w, pad_h, pad_w, dil_h, dil_w;
  int ic_off;        // first input channel of this group
  uint32_t pad_word; // activation zero point replicated in 4 bytes
  int kc0;           // first 16-byte k-chunk of this wave group's share of K (k-split groups), else 0
  // byte offset gained, beyond a block's 16 bytes, when the k order wraps from a tap's last 16-channel block into the
  // next tap (dil_w * IC - 16 icb), and on top of that from a kernel row's last tap into the next row
  // (dil_h * W * IC - KW * dil_w * IC)
  int step_w, step_h;
};

// Optional work between the requantisation's multiply and its rounding:
//   t += float(accum_q - accum_zp) * amult     (quantized residual, output-scale units)
//   t  = silu(t * out_scale) / out_scale
struct PostOps {
  const uint8_t* accum;  // bytes laid out like the output, or null
  int32_t accum_signed, accum_zp;
  float amult;           // accum_scale / out_scale
  int32_t silu;
  float out_scale;
  float silu_c, silu_c_tail;  // -out_scale * log2(e) as a float and what that float leaves of it (silu_in_output_units)
  __host__ __device__ bool any() const { return accum != nullptr || silu != 0; }
};

// silu(t * s) / s for a value t in output-scale units (s = out_scale): t / (1 + e^(-t s)) with the
// hardware's exp2 and reciprocal (1 ulp each) in place of expf and two IEEE divisions -- ten vector
// instructions for some fifty.  e^(-t s) = 2^(hi + lo) with hi = fl(t c), c = fl(-s log2 e), and lo
// the rounding error of that product plus t times what c leaves of -s log2 e (c_tail, from the
// host in double precision), so that the argument's rounding (|hi| 2^-24 in the exponent: 40 ulp of
// the result at |t s| = 80) does not reach the result; 2^lo = 1 + lo ln 2 to well below an ulp.  hi is
// capped at 126: the sum 1 + 2^hi and its reciprocal stay finite, and the result is the 0 that
// r e^r rounds to anyway.  The result is within a few ulp of the CPU op's float sequence
// r = t s, (r / (1 + expf(-r))) / s; a requantised byte differs from it (by one) where the exact value
// lies within about 1e-5 of a rounding boundary: 2 of 4.2 million outputs measured.
__device__ __forceinline__ float silu_in_output_units(float t, float c, float c_tail) {
  constexpr float kLn2 = 0.693147182464599609375f;
  const float p = t * c;
  const float lo = __builtin_fmaf(t, c_tail, __builtin_fmaf(t, c, -p));
  const float hi = __builtin_fminf(p, 126.0f);
  const float e0 = __builtin_amdgcn_exp2f(hi);
  const float e = __builtin_fmaf(e0, lo * kLn2, e0);
  return t * __builtin_amdgcn_rcpf(1.0f + e);
}

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
  PostOps post;          // all zero for quantized::linear
  // Activation scale and zero point read from device memory at run time (the
  // tail of a min/max -> qparams -> quantize chain with no host round trip);
  // null: x_scale and acc_coef above hold.  acc_base is acc_coef + zero point.
  const tmq_qparams* x_qp_dev = nullptr;
  int32_t acc_base = 0;
  // Split K (raw int32 output of plain activation rows only): block row
  // blockIdx.y multiplies stages [y * split_stages, (y + 1) * split_stages) of
  // the k loop -- the last one everything from y * split_stages on -- and
  // writes its partial sums to y + blockIdx.y * split_stride.
  int32_t splits = 1;
  int32_t split_stages = 0;
  int64_t split_stride = 0;
};

struct XQuant {
  float scale;
  int32_t coef;  // multiplies colsum[n] into the accumulator start
};
__device__ __forceinline__ XQuant x_quant(const GemmArgs& a) {
  if (a.x_qp_dev != nullptr)
    return XQuant{static_cast<float>(a.x_qp_dev->scale), a.acc_base - a.x_qp_dev->zero_point};
  return XQuant{a.x_scale, a.acc_coef};
}

// Four float results of one output row (kOutF32), channels n .. n+3.
__device__ __forceinline__ void store_f32x4(const GemmArgs& a, int64_t m, int64_t n, const int (&raw)[4],
                                            v4f mult, v4f bias) {
  float* dst = static_cast<float*>(a.y) + m * a.ldy + a.n_off + n;
  v4f v;
#pragma unroll
  for (int j = 0; j < 4; ++j)
    v[j] = __builtin_fmaxf(__builtin_fmaf(static_cast<float>(raw[j]), mult[j], bias[j]), a.lo_f);
  if (n + 3 < a.N && (reinterpret_cast<uintptr_t>(dst) & 15) == 0) {
    *reinterpret_cast<v4f*>(dst) = v;
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (n + j < a.N) dst[j] = v[j];
  }
}

__device__ __forceinline__ v4i ld16(const void* p) { return *reinterpret_cast<const v4i*>(p); }
// 16 bytes to an address of any alignment (output rows whose channel count is no multiple of 16):
// still one store instruction, where byte stores would be sixteen.
struct __attribute__((packed, aligned(1))) V4iAnyAlignment {
  v4i v;
};
__device__ __forceinline__ void st16_any(void* p, v4i v) { reinterpret_cast<V4iAnyAlignment*>(p)->v = v; }
__device__ __forceinline__ v4i ld16_any(const void* p) { return reinterpret_cast<const V4iAnyAlignment*>(p)->v; }
typedef int v2i __attribute__((ext_vector_type(2)));
struct __attribute__((packed, aligned(1))) V2iAnyAlignment {
  v2i v;
};
__device__ __forceinline__ void st8_any(void* p, v2i v) { reinterpret_cast<V2iAnyAlignment*>(p)->v = v; }
// Streaming load: data that this CU reads exactly once (packed weight tiles)
// should not push reusable lines out of the vector L1.
__device__ __forceinline__ v4i ld16_stream(const void* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const v4i*>(p));
}

// One direct global->LDS copy: every active lane moves the 16 bytes at
// base + off (uniform 64-bit base, per-lane 32-bit offset) to LDS byte
// lds_dst + 16 * lane (wave-uniform destination, passed in M0).
// Issued through inline assembly on purpose: for the compiler's own builtin
// every later LDS access may alias the copy, and it drains all outstanding
// loads (vmcnt(0)) before it, which serialises a pipeline of copies.  The
// caller waits (s_waitcnt vmcnt) before the data is read.
__device__ __forceinline__ void lds_dma16(const uint8_t* base, uint32_t off, uint32_t lds_dst) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :
               : "v"(off), "s"(base), "s"(lds_dst)
               : "memory", "m0");
}
// LDS byte address of a pointer into shared memory, as a wave-uniform value.
__device__ __forceinline__ uint32_t lds_address(const void* p) {
  typedef __attribute__((address_space(3))) void* lptr_t;
  return __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lptr_t)p)));
}

__device__ __forceinline__ void wave_sync_lds() {
  // orders this wave's LDS writes before its later LDS reads of other lanes'
  // data (the LDS executes one wave's instructions in order)
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <class XSRC>
struct XLoader;

// One loader per 16-byte chunk slot a thread stages: fixed activation row,
// k-chunk index `kc` supplied per stage.  Loads are never predicated: rows past
// M are clamped to the last row (their results are never stored) and k-chunks
// past K to the last chunk (the packed weight is zero there), so that every
// stage issues the same number of loads and the wait counters stay exact.
template <>
struct XLoader<XLinear> {
  const uint8_t* p;
  __device__ __forceinline__ void init(const XLinear& s, int64_t m, int64_t M) {
    p = s.x + (m < M ? m : M - 1) * s.ldx;
  }
};

template <>
struct XLoader<XConv> {
  const uint8_t* img;  // first byte of this row's image (+ group channel offset)
  int ih0, iw0;        // top-left input coordinate of the receptive field
  int off0;            // byte offset of (ih0, iw0) inside the image (may be negative)
  __device__ __forceinline__ void init(const XConv& s, int64_t m, int64_t M) {
    // the host guarantees fewer than 2**31 output pixels and image bytes:
    // 32-bit divisions and offsets
    const uint32_t mm = static_cast<uint32_t>(m < M ? m : M - 1);
    const uint32_t t = mm / static_cast<uint32_t>(s.OW);
    const int ow = static_cast<int>(mm - t * static_cast<uint32_t>(s.OW));
    const uint32_t b = t / static_cast<uint32_t>(s.OH);
    const int oh = static_cast<int>(t - b * static_cast<uint32_t>(s.OH));
    img = s.x + static_cast<int64_t>(b) * (static_cast<int64_t>(s.H) * s.W * s.IC) + s.ic_off;
    ih0 = oh * s.stride_h - s.pad_h;
    iw0 = ow * s.stride_w - s.pad_w;
    off0 = (ih0 * s.W + iw0) * s.IC;
  }
};

// Position of a thread's k-chunk (chunk c of stage kt) in the k dimension.
// Stages are visited in increasing order, so the position advances
// incrementally instead of being decoded with divisions every stage.
template <class XSRC>
struct KCursor;

template <>
struct KCursor<XLinear> {
  int kc;
  int c;
  __device__ __forceinline__ void init(const XLinear&, int c_) { c = c_; kc = c_; }
  __device__ __forceinline__ void seek(const XLinear&, int kt) { kc = kt * kChunks + c; }
  __device__ __forceinline__ v4i load(const XLinear&, const XLoader<XLinear>& row, int64_t K) const {
    int64_t k = static_cast<int64_t>(kc) * 16;
    k = k < K ? k : K - 16;
    return ld16(row.p + k);
  }
};

template <>
struct KCursor<XConv> {
  int kt_cur, c;
  int kw, blk;          // tap column and 16-channel block of the current chunk
  int dh, dw, tapoff;   // the tap's input displacement and the chunk's byte offset from the window's corner
  __device__ __forceinline__ void init(const XConv& s, int c_) {
    c = c_;
    kt_cur = 0;
    const int tap = (c_ + s.kc0) / s.icb;
    blk = c_ + s.kc0 - tap * s.icb;
    const int kh = tap / s.KW;
    kw = tap - kh * s.KW;
    dh = kh * s.dil_h;
    dw = kw * s.dil_w;
    tapoff = (dh * s.W + dw) * s.IC + blk * 16;
  }
  // `n` blocks on (fewer than a tap holds: one wrap into the next tap at most), by additions only:
  // s.step_w / s.step_h are what the offset gains at the wrap into the next tap / next kernel row
  // beyond the blocks' own 16 bytes each.
  __device__ __forceinline__ void advance(const XConv& s, int n) {
    int b = blk + n, off = tapoff + 16 * n;
    const bool wrap = b >= s.icb;
    b -= wrap ? s.icb : 0;
    off += wrap ? s.step_w : 0;
    const int w = kw + (wrap ? 1 : 0), x = dw + (wrap ? s.dil_w : 0);
    const bool row = w == s.KW;
    kw = row ? 0 : w;
    dw = row ? 0 : x;
    dh += row ? s.dil_h : 0;
    tapoff = off + (row ? s.step_h : 0);
    blk = b;
  }
  // Advances by at most one stage per call (stages are requested in order, the
  // last one repeatedly).  Written with selects only where lanes differ: a divergent branch
  // between the global loads would make the compiler drain all outstanding loads.  (The
  // branch on the layer's channel count is the same for every lane and holds no load.)
  __device__ __forceinline__ void seek(const XConv& s, int kt) {
    const bool adv = kt > kt_cur;
    kt_cur = adv ? kt_cur + 1 : kt_cur;
    if (s.icb >= kChunks) {
      advance(s, adv ? kChunks : 0);
    } else {
#pragma unroll
      for (int i = 0; i < kChunks; ++i) advance(s, adv ? 1 : 0);
    }
  }
  // Out-of-image taps read as the activation zero point, i.e. real value 0;
  // chunks past K land on taps past the kernel window: any in-bounds address
  // will do there because the packed weight is zero.
  __device__ __forceinline__ v4i load(const XConv& s, const XLoader<XConv>& row, int64_t K) const {
    const int pw = static_cast<int>(s.pad_word);
    const bool in_k = static_cast<int64_t>(kt_cur * kChunks + c) * 16 < K;
    const bool inside = in_k && static_cast<unsigned>(row.ih0 + dh) < static_cast<unsigned>(s.H) &&
                        static_cast<unsigned>(row.iw0 + dw) < static_cast<unsigned>(s.W);
    const int off = inside ? row.off0 + tapoff : 0;
    const v4i v = ld16(row.img + off);
    return v4i{inside ? v.x : pw, inside ? v.y : pw, inside ? v.z : pw, inside ? v.w : pw};
  }
};

// Slot swizzle of the activation stage: see the file header.
__device__ __forceinline__ int x_swizzle(int row) { return (row >> 2) & 3; }

// The bias enters the requantisation as v = fma(bterm, bmul, float(raw)), which
// covers both forms of PyTorch's CPU ops (fbgemm's output stage):
//   per-channel weight scales   v = float(raw) + fl(bias / atw)      bterm = fl(bias / atw), bmul = 1
//   one scale for the weight    v = fma(bias, fl(1 / atw), float(raw))   bterm = bias, bmul = fl(1 / atw)
// (atw = fl(x_scale * w_scale); a product with 1 is exact, so the first line is
// a plain addition.)  The two differ on a few outputs in a million.
__host__ __device__ __forceinline__ float bias_term(bool per_tensor, float bias, float atw) {
  return per_tensor ? bias : bias / atw;
}
__host__ __device__ __forceinline__ float bias_mul(bool per_tensor, float atw) {
  return per_tensor ? 1.0f / atw : 1.0f;
}

// One requantised byte group: four consecutive channels of one output row.
// CLAMP = false (unsigned output, bounds 0 and 255 only): the packing
// conversion v_cvt_pk_u8_f32 already saturates to [0, 255], no separate clamp.
//
// Unsigned output with zero point 0 (what a layer with a fused ReLU has, whose observed minimum is 0)
// and no bounds inside [0, 255]: v_cvt_pk_u8_f32 itself rounds to nearest even and saturates, so it
// stands for rint, + zero point, clamp and pack at once -- the same byte for every input (checked on
// the device against nearbyintf + clamp over a million values between -2 and 258 and the special
// ones), four vector instructions per value for seven.  PLAIN says who decides: 0 never (the kernels
// bound by the matrix pipe or by latencies, where a second epilogue in the code only costs), 1 the
// host has checked requant_plain_u8 and launched the variant, 2 the kernel tests it per call (a branch
// on kernel arguments; their bit patterns are compared as integers, which the scalar unit can do).
__host__ __device__ __forceinline__ bool requant_plain_u8(float zp_f, float lo_f, float hi_f) {
  return __builtin_bit_cast(int, zp_f) == 0 && __builtin_bit_cast(int, lo_f) <= 0 &&
         __builtin_bit_cast(int, hi_f) >= 0x437f0000;
}

template <int MODE, bool CLAMP = true, int PLAIN = 0>
__device__ __forceinline__ uint32_t requant4(const int (&raw)[4], v4f bdiv, float bmul, v4f mult, float zp_f,
                                             float lo_f, float hi_f) {
  // Signed bytes are the unsigned ones of the same sequence with zero point and bounds 128 higher, sign bits flipped
  // at the end (clamp(r + zp, lo, hi) = clamp(r + zp + 128, lo + 128, hi + 128) - 128, every term a small integer in
  // fp32): the packing conversion serves them too, where a signed byte took a float-to-int conversion, a mask, a shift
  // and an or.
  if constexpr (MODE == kOutS8)
    return requant4<kOutU8, CLAMP, PLAIN>(raw, bdiv, bmul, mult, zp_f + 128.f, lo_f + 128.f, hi_f + 128.f) ^ 0x80808080u;
  uint32_t packed = 0;
  if constexpr (MODE == kOutU8 && PLAIN != 0) {
    if (PLAIN == 1 || requant_plain_u8(zp_f, lo_f, hi_f)) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float v = __builtin_fmaf(bdiv[j], bmul, static_cast<float>(raw[j]));
        packed = __builtin_amdgcn_cvt_pk_u8_f32(v * mult[j], j, packed);
      }
      return packed;
    }
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    float v = static_cast<float>(raw[j]);  // int -> fp32, round to nearest even
    v = __builtin_fmaf(bdiv[j], bmul, v);
    const float ab = v * mult[j];
    float r = __builtin_rintf(ab) + zp_f;
    if constexpr (CLAMP || MODE != kOutU8) r = __builtin_amdgcn_fmed3f(r, lo_f, hi_f);
    if constexpr (MODE == kOutU8) {
      packed = __builtin_amdgcn_cvt_pk_u8_f32(r, j, packed);
    } else {
      packed |= (static_cast<uint32_t>(static_cast<int>(r)) & 0xffu) << (8 * j);
    }
  }
  return packed;
}

// Up to four residual bytes of one output row, starting at byte offset `off`
// of the residual tensor; `nvalid` of them exist.
__device__ __forceinline__ uint32_t load_accum4(const PostOps& p, int64_t off, int nvalid) {
  const uint8_t* src = p.accum + off;
  if (nvalid >= 4 && (reinterpret_cast<uintptr_t>(src) & 3) == 0)
    return *reinterpret_cast<const uint32_t*>(src);
  uint32_t w = 0;
  for (int j = 0; j < 4; ++j)
    if (j < nvalid) w |= static_cast<uint32_t>(src[j]) << (8 * j);
  return w;
}

// requant4 with the post operations (see PostOps) before the rounding.  POST says
// what the caller knows at compile time: 0 nothing (both operations are looked up
// in `p`), 1 a residual and no SiLU, 2 SiLU (a residual if `p` has one).  PLAIN: as in requant4.
template <int MODE, int POST = 0, bool PLAIN = false>
__device__ __forceinline__ uint32_t requant4_post(const int (&raw)[4], v4f bdiv, float bmul, v4f mult,
                                                  const PostOps& p, uint32_t accw, float zp_f,
                                                  float lo_f, float hi_f) {
  if constexpr (MODE == kOutS8)  // (see requant4)
    return requant4_post<kOutU8, POST, PLAIN>(raw, bdiv, bmul, mult, p, accw, zp_f + 128.f, lo_f + 128.f,
                                              hi_f + 128.f) ^
           0x80808080u;
  uint32_t packed = 0;
  // The residual bytes are taken as unsigned values (one conversion instruction
  // per byte): a signed byte s equals (s ^ 0x80) - 128, so the word is flipped
  // once and 128 joins the zero point.  Both terms of the difference are small
  // integers, exact in fp32, so it equals float(q - zero_point).
  const uint32_t accu = p.accum_signed ? accw ^ 0x80808080u : accw;
  const float acc_zp_f = static_cast<float>(p.accum_zp + (p.accum_signed ? 128 : 0));
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    float v = static_cast<float>(raw[j]);
    v = __builtin_fmaf(bdiv[j], bmul, v);
    float t = v * mult[j];
    if (POST == 1 || p.accum != nullptr) {
      const float qf = static_cast<float>((accu >> (8 * j)) & 0xffu);
      const float a = (qf - acc_zp_f) * p.amult;
      t = t + a;
    }
    if (POST == 2 || (POST == 0 && p.silu)) t = silu_in_output_units(t, p.silu_c, p.silu_c_tail);
    if constexpr (PLAIN && MODE == kOutU8) {  // (the host has checked requant_plain_u8: see requant4)
      packed = __builtin_amdgcn_cvt_pk_u8_f32(t, j, packed);
      continue;
    }
    float r = __builtin_rintf(t) + zp_f;
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
// WM x WN waves, each wave (BM/WM) x (BN/WN).  PD = prefetch distance in
// stages: the global loads of stage t+PD are issued while stage t is being
// multiplied, so PD-1 stages of 16-byte loads are in flight per thread.
//
// WDMA = true (quantized::linear only): no operand passes through registers on
// its way to LDS.  Each wave copies 1 KB per instruction straight from global
// memory into LDS (global_load_lds_dwordx4: lane L's 16 bytes land in slot L
// of the 1 KB destination), kDmaBufs stages ahead, into a ring of kDmaBufs
// buffers; the sign-bit flip of unsigned activations is applied to the
// fragments after they are read from LDS.  Register staging costs the matrix
// pipe about a quarter of its time on this chip: the ds_write_b128 traffic of
// eight waves, mixed with their fragment reads, backs up the LDS queue and the
// fragment reads behind it.
//
// KW > 1 (register staging only): KW groups of WM x WN
// waves share one output tile and split its k loop into KW equal runs of
// stages, each group with its own LDS stages and registers; after the loop the
// groups' accumulators are added through LDS and group 0 runs the epilogue.
// For grids far smaller than the chip: a lone block per CU spends most of a
// stage waiting on its own chain LDS store -> barrier -> LDS read -> MFMA, and
// the other groups' waves fill those gaps.  The host sends only k loops whose
// stage count KW divides.
template <int BM, int BN, int WM, int WN, int MODE, class XSRC, int PD = 4, bool WDMA = false, int KW = 1,
          bool XWIDE = false>
__global__ __launch_bounds__(WM* WN* KW* kWave, (WDMA && WM * WN == 4 && (BM / WM) * (BN / WN) <= 128 * 64) ? 2 : 1)
void gemm_i8_kernel(GemmArgs a, XSRC xsrc) {
  constexpr int NT = WM * WN * kWave;   // threads of one group
  constexpr int NTB = NT * KW;          // threads of the block
  static_assert(KW >= 1 && (KW == 1 || !WDMA), "k-split groups: register staging only");
  const int kg = KW == 1 ? 0 : static_cast<int>(threadIdx.x) / NT;  // this thread's group
  if constexpr (KW > 1) {  // this group's share of K: move the operands, shorten K
    const int64_t per = ceil_div(a.K, kBK) / KW;
    const int64_t k0 = kg * per * kBK;
    const int64_t left = a.K - k0;
    a.K = left < per * kBK ? left : per * kBK;
    a.w_packed += kg * per * (kChunks * 256);
    if constexpr (std::is_same<XSRC, XLinear>::value)
      xsrc.x += k0;
    else
      xsrc.kc0 += static_cast<int>(k0 / 16);
  }
  constexpr bool kHasPost = XSRC::kPostOps;  // residual / activation epilogue compiled in
  if constexpr (MODE == kOutAcc32 && std::is_same<XSRC, XLinear>::value) {
    if (a.splits > 1) {  // this block's share of K: move the operands, shorten K
      const int64_t sp = blockIdx.y;
      const int64_t k0 = sp * a.split_stages * kBK;
      // the last split takes everything that is left (the host may have merged a
      // short tail into it)
      const int64_t left = a.K - k0, mine = static_cast<int64_t>(a.split_stages) * kBK;
      a.K = (sp == a.splits - 1 || left < mine) ? left : mine;
      a.w_packed += sp * a.split_stages * (kChunks * 256);
      xsrc.x += k0;
      a.y = static_cast<int32_t*>(a.y) + sp * a.split_stride;
    }
  }
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int NW = BN * kChunks / NT;  // 16-byte weight chunks per thread per stage
  constexpr int NX = BM * kChunks / NT;
  constexpr int NWAVES = WM * WN;
  constexpr int NSET = PD - 1;           // register sets holding stages in flight
  static_assert(TM >= 1 && TN >= 1 && NW >= 1 && NX >= 1, "tile too small for the wave grid");
  static_assert(BN * kChunks % NT == 0 && BM * kChunks % NT == 0, "uneven staging");
  static_assert(PD >= 3, "prefetch distance");
  // direct copies: 1 KB (64 weight rows of one k-chunk, or 16 activation rows) each
  constexpr int kDmaBufs = PD;
  constexpr int NDW = kChunks * (BN / 64) / NWAVES;  // weight copies per wave per stage
  constexpr int NDX = (BM / 16) / NWAVES;            // activation copies per wave per stage
  constexpr int ND = NDW + NDX;
  static_assert(!WDMA || std::is_same<XSRC, XLinear>::value, "direct copies need plain activation rows");
  static_assert(!WDMA || (BN % 64 == 0 && kChunks * (BN / 64) % NWAVES == 0 && BM % 16 == 0 &&
                          (BM / 16) % NWAVES == 0),
                "direct copies do not divide among the waves");
  static_assert(!WDMA || (TN + TM <= TN * TM && ND <= TN * TM), "one LDS read and one copy per MFMA at most");
  constexpr int kWBufs = WDMA ? kDmaBufs : 2, kXBufs = WDMA ? kDmaBufs : 2;
  static_assert(!XWIDE || (WDMA && PD == 3 && KW == 1 && (BM / 8) % (2 * NWAVES) == 0),
                "wide activation copies: three-stage direct-copy ring only");

  // LDS: two stages of {weights, activations}; the same bytes are reused after
  // the main loop to transpose the output tile into row-major order.
  // (XWIDE: an activation buffer holds two stages, 128 k-bytes of every row)
  constexpr int kWStage = kChunks * BN * 16, kXStage = XWIDE ? BM * 2 * kBK : BM * kBK;
  constexpr int kOutPitch = BN + 16;  // bytes; keeps rows 16-byte aligned and off one bank
  constexpr int kMainBytes = kWBufs * kWStage + kXBufs * kXStage;
  constexpr int kF32Pitch = BN * 4 + 16;  // float rows of the tile, same idea
  constexpr int kOutBytes =
      (MODE == kOutAcc32 || MODE == kOutF32) ? WM * 32 * kF32Pitch : BM * kOutPitch;
  constexpr int kSumBytes = (KW - 1) * NT * TN * TM * 64;  // the other groups' accumulators
  constexpr int kLoopBytes = KW * kMainBytes > kSumBytes ? KW * kMainBytes : kSumBytes;
  constexpr int kTileBytes = kLoopBytes > kOutBytes ? kLoopBytes : kOutBytes;
  __shared__ __attribute__((aligned(16))) uint8_t smem[kTileBytes];
  __shared__ __attribute__((aligned(16))) int s_acc0[BN];
  __shared__ __attribute__((aligned(16))) float s_mult[BN];
  __shared__ __attribute__((aligned(16))) float s_bdiv[BN];
  uint8_t* const gmem = smem + kg * kMainBytes;  // this group's stages
  uint8_t* const sW = gmem;                      // [kWBufs][kWStage]
  uint8_t* const sX = gmem + kWBufs * kWStage;   // [kXBufs][kXStage]

  const int tb = threadIdx.x;
  const int t = KW == 1 ? tb : tb - kg * NT;
  const int lane = t % kWave, wave = t / kWave;
  const int li = lane & 31, half = lane >> 5;
  const int wm0 = (wave % WM) * WTM;
  const int wn0 = (wave / WM) * WTN;

  // ---- tile assignment.  Blocks are dealt round-robin to the 8 XCDs, each with
  // its own L2: give every XCD one contiguous run of the tile sequence, and order
  // the sequence so that the ~32 tiles an XCD runs at once form a compact patch
  // (kGroupN channel tiles wide, row tiles next) that shares operand tiles.
  // (32-bit arithmetic: the host launches fewer than 2**31 blocks, and a 64-bit
  // division costs a block that is alone on its CU a hundred instructions before
  // its first load)
  const uint32_t tiles_m = static_cast<uint32_t>(ceil_div(a.M, BM)), tiles_n = static_cast<uint32_t>(ceil_div(a.N, BN));
  const uint32_t nblocks = tiles_m * tiles_n;
  uint32_t tile;
  {
    const uint32_t bid = blockIdx.x;
    const uint32_t q = nblocks / 8, rem = nblocks % 8;
    const uint32_t xcd = bid % 8, within = bid / 8;
    tile = xcd * q + (xcd < rem ? xcd : rem) + within;
  }
  constexpr uint32_t kGroupN = 4;
  const uint32_t group = tile / (tiles_m * kGroupN);
  const uint32_t gfirst = group * kGroupN;
  const uint32_t gwidth = tiles_n - gfirst < kGroupN ? tiles_n - gfirst : kGroupN;
  const uint32_t in_group = tile - group * (tiles_m * kGroupN);
  const uint32_t tile_row = in_group / gwidth;
  const int64_t m0 = static_cast<int64_t>(tile_row) * BM;
  const int64_t n0 = static_cast<int64_t>(gfirst + in_group - tile_row * gwidth) * BN;
  const int64_t NB = ceil_div(a.N, 16);

  // ---- per-channel constants of this tile's BN output channels, then the
  // accumulators' start value (see file header).  Called once per tile, after
  // the first operand copies are on their way.
  v16i acc[TN][TM];
  auto init_tile = [&]() {
    const XQuant xq = x_quant(a);
    for (int i = t; i < BN; i += NT) {
      const int64_t n = n0 + i;
      int acc0 = 0;
      float mult = 0.f, bdiv = 0.f;
      if (n < a.N) {
        const int64_t np = n + a.n_off;
        acc0 = xq.coef * a.colsum[np];
        if (MODE == kOutF32) {
          mult = xq.scale * a.w_scales[np * a.w_scale_stride];
          bdiv = a.bias != nullptr ? a.bias[np] : 0.f;
        } else if (MODE != kOutAcc32) {
          const float atw = xq.scale * a.w_scales[np * a.w_scale_stride];
          mult = atw / a.out_scale;
          bdiv = a.bias != nullptr ? bias_term(a.w_scale_stride == 0, a.bias[np], atw) : 0.f;
        }
      }
      s_acc0[i] = acc0;
      s_mult[i] = mult;
      s_bdiv[i] = bdiv;
    }
    __syncthreads();  // s_acc0 / s_mult / s_bdiv are written
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      v16i init;
#pragma unroll
      for (int r = 0; r < 16; ++r)
        init[r] = s_acc0[wn0 + tn * 32 + 8 * (r >> 2) + 4 * half + (r & 3)];
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) acc[tn][tm] = init;
    }
    if (KW > 1 && kg > 0) {  // the start value is added once, by group 0
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[tn][tm][r] = 0;
    }
  };

  const int KT = static_cast<int>(ceil_div(a.K, kBK));
  auto clampk = [&](int kt) { return kt < KT ? kt : KT - 1; };
  const int xswz = x_swizzle(li);
  const v4i xmask = {static_cast<int>(a.x_xor), static_cast<int>(a.x_xor),
                     static_cast<int>(a.x_xor), static_cast<int>(a.x_xor)};
  v4i wf0[TN], xf0[TM], wf1[TN], xf1[TM];
  // j-th fragment read of k-step s (weights first, then activations)
  auto read_one = [&](int wbuf, int xbuf, int s, int j, v4i(&wf)[TN], v4i(&xf)[TM]) {
    const int c = 2 * s + half;
    if (j < TN)
      wf[j] = ld16(&sW[wbuf * kWStage + (c * BN + wn0 + j * 32 + li) * 16]);
    else
      xf[j - TN] = ld16(&sX[xbuf * kXStage + (wm0 + (j - TN) * 32 + li) * kBK + ((c ^ xswz) << 4)]);
  };
  constexpr int Q = TN * TM;    // MFMAs per k-step
  constexpr int NF = TN + TM;   // fragment reads per k-step
  auto mfma = [&](int q, const v4i(&wf)[TN], const v4i(&xf)[TM]) {
    acc[q / TM][q % TM] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[q / TM], xf[q % TM],
                                                               acc[q / TM][q % TM], 0, 0, 0);
  };

  if constexpr (WDMA && XWIDE) {
    // ---- direct-copy pipeline with activation copies two stages wide.  As the
    // pipeline below, except that an activation copy moves 8 rows x 128 bytes
    // (whole 128-byte lines of the row-major activations; the narrow copies
    // take 16 rows x 64 bytes and touch every line twice, in two successive
    // stages), into a ring of three buffers of two stages each:
    //   pair u = stages 2u and 2u+1, buffer u % 3, row pitch 128 bytes, 16-byte
    //   slot XOR-ed with (row >> 1) & 7 (16 consecutive rows then cover all
    //   sixteen 16-byte slots of the 256-byte bank window once)
    // Stage t's second half issues the weight copies of stage t+3 and one half
    // of the activation copies of pair (t+4)/2: the first half when t is even,
    // the second when t is odd (the pair then starts at stage t+3).  Everything
    // a stage reads was issued at least two stages earlier, so the wait of the
    // narrow pipeline holds unchanged: all but the copies of the last stage.
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const uint32_t lds0 = lds_address(smem);
    static_assert(NWAVES % 4 == 0, "weight copies: one k-chunk per wave");
    constexpr int NDXH = (BM / 8) / NWAVES / 2;  // activation copies per wave per stage (half a pair)
    static_assert(NDXH == NDX, "as many copies per stage as the narrow pipeline");
    const uint8_t* const wtile = a.w_packed + (n0 / 16) * a.w_kchunks * 256;
    const int64_t nb_last = NB - 1 - n0 / 16;  // rows past N: clamped, never stored
    uint32_t wdma_off[NDW];
#pragma unroll
    for (int i = 0; i < NDW; ++i) {
      const int rg = (wave_u >> 2) + i * (NWAVES / 4);
      int64_t rb = rg * 4 + (lane >> 4);
      rb = rb < nb_last ? rb : nb_last;
      wdma_off[i] = static_cast<uint32_t>((rb * a.w_kchunks + (wave_u & 3)) * 256 + (lane & 15) * 16);
    }
    const uint32_t wdma_lds = lds0 + ((wave_u & 3) * BN + (wave_u >> 2) * 64) * 16;
    // activation copy i (of 2 NDX per pair) of wave w: rows 8 (w + i NWAVES) .. + 7,
    // eight lanes per row; the lane of slot sl fetches the k-chunk the swizzle puts there
    const uint8_t* const xtile = xsrc.x + m0 * xsrc.ldx;
    const int64_t m_last = a.M - 1 - m0;
    const int pair_last = (KT - 1) >> 1;
    const int ktail = static_cast<int>(a.K) - 16 - pair_last * 2 * kBK;  // last chunk inside K of the last pair
    uint32_t xdma_off[2 * NDX], xdma_off_last[2 * NDX];
#pragma unroll
    for (int i = 0; i < 2 * NDX; ++i) {
      const int row = (wave_u + i * NWAVES) * 8 + (lane >> 3);
      const int64_t r = row < m_last ? row : m_last;
      const int kc = ((lane & 7) ^ ((row >> 1) & 7)) * 16;
      xdma_off[i] = static_cast<uint32_t>(r * xsrc.ldx + kc);
      // chunks past K: any valid bytes will do, the packed weight is zero there
      xdma_off_last[i] = static_cast<uint32_t>(r * xsrc.ldx + (kc < ktail ? kc : ktail));
    }
    const uint32_t xdma_lds = lds0 + kWBufs * kWStage + wave_u * 1024;
    // weight copies of stage kt into weight buffer wb
    auto dma_w = [&](int kt, int wb, int i) {
      lds_dma16(wtile + static_cast<int64_t>(kt) * (kChunks * 256), wdma_off[i],
                wdma_lds + wb * kWStage + i * (NWAVES / 4) * 64 * 16);
    };
    // copy i (0 .. 2 NDX - 1) of activation pair u into activation buffer xb
    auto dma_x = [&](int u, int xb, int i) {
      const int uc = u < pair_last ? u : pair_last;
      lds_dma16(xtile + static_cast<int64_t>(uc) * (2 * kBK), uc == pair_last ? xdma_off_last[i] : xdma_off[i],
                xdma_lds + xb * kXStage + i * NWAVES * 1024);
    };
    auto wait_loads = [&](auto left_tag) {  // s_waitcnt vmcnt(left) only
      constexpr int kLeft = decltype(left_tag)::value;
      static_assert(kLeft < 64, "load counter range");
      __builtin_amdgcn_s_waitcnt((kLeft & 15) | ((kLeft >> 4) << 14) | (7 << 4) | (15 << 8));
    };
    auto flip = [&](v4i& f) { f ^= xmask; };
    const int xswz8 = (li >> 1) & 7;
    // j-th fragment read of k-step s of a stage in weight buffer wb, activation
    // buffer xb, half p of its pair
    auto read_w = [&](int wb, int xb, int p, int s, int j, v4i(&wf)[TN], v4i(&xf)[TM]) {
      const int c = 2 * s + half;
      if (j < TN)
        wf[j] = ld16(&sW[wb * kWStage + (c * BN + wn0 + j * 32 + li) * 16]);
      else
        xf[j - TN] = ld16(&sX[xb * kXStage + (wm0 + (j - TN) * 32 + li) * (2 * kBK) + (((4 * p + c) ^ xswz8) << 4)]);
    };
    // ph = kt % 6 as a compile-time constant
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
      const int uload = (kt + 4) >> 1;                 // pair whose copies this stage issues ...
      const int xbl = ((ph + 4) % 6 >> 1) % 3;         // ... into this buffer,
      const int ihalf = ((ph + 4) & 1) * NDX;          // this half of them
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
    // prologue: pair 0 and weights 0 first (they alone are waited for), then
    // weights 1, the first half of pair 1, and last what stage "-1" would have
    // issued: weights 2 and the second half of pair 1
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
    init_tile();
    wait_loads(std::integral_constant<int, 2 * NDW + 2 * NDX>{});
    __syncthreads();
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
    wait_loads(std::integral_constant<int, 0>{});
  } else if constexpr (WDMA) {
    // ---- direct-copy pipeline.  Stage s lives in buffer s % kDmaBufs.  The
    // schedule of stage t, one LDS or copy operation per MFMA:
    //   first half   MFMAs of k-step 0 + LDS reads of the k-step 1 fragments
    //   wait + barrier: stage t+1 has landed for every wave; buffer t % kDmaBufs
    //                is dead (its last reads were waited for before the barrier)
    //   second half  MFMAs of k-step 1 + LDS reads of the k-step 0 fragments of
    //                stage t+1 + this wave's copies of stage t+kDmaBufs into the
    //                dead buffer
    // Activation fragments get their sign-bit flip one MFMA ahead of their
    // first use, so that the flip never sits between a barrier and an MFMA.
    // Every copy is "uniform 64-bit base + per-lane 32-bit offset" on the global
    // side and a wave-uniform LDS address in M0 on the other: per stage only the
    // scalar bases move, no vector instruction is spent on addresses.  The host
    // keeps 256 rows of either operand within 32 bits of the tile's base.
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const uint32_t lds0 = lds_address(smem);
    // weight copy i of wave w: k-chunk w & 3, 64-row group (w >> 2) + i * NWAVES / 4
    static_assert(NWAVES % 4 == 0, "weight copies: one k-chunk per wave");
    const uint8_t* const wtile = a.w_packed + (n0 / 16) * a.w_kchunks * 256;
    const int64_t nb_last = NB - 1 - n0 / 16;  // rows past N: clamped, never stored
    uint32_t wdma_off[NDW];
#pragma unroll
    for (int i = 0; i < NDW; ++i) {
      const int rg = (wave_u >> 2) + i * (NWAVES / 4);
      int64_t rb = rg * 4 + (lane >> 4);
      rb = rb < nb_last ? rb : nb_last;
      wdma_off[i] = static_cast<uint32_t>((rb * a.w_kchunks + (wave_u & 3)) * 256 + (lane & 15) * 16);
    }
    const uint32_t wdma_lds = lds0 + ((wave_u & 3) * BN + (wave_u >> 2) * 64) * 16;
    // activation copy i of wave w: rows 16 (w + i NWAVES) .. + 15, four lanes per
    // row; the lane of slot sl fetches the k-chunk that the swizzle puts there
    const uint8_t* const xtile = xsrc.x + m0 * xsrc.ldx;
    const int64_t m_last = a.M - 1 - m0;
    const int ktail = static_cast<int>(a.K) - 16 - (KT - 1) * kBK;  // last chunk inside K of the last stage
    uint32_t xdma_off[NDX], xdma_off_last[NDX];
#pragma unroll
    for (int i = 0; i < NDX; ++i) {
      const int row = (wave_u + i * NWAVES) * 16 + (lane >> 2);
      const int64_t r = row < m_last ? row : m_last;
      const int kc = ((lane & 3) ^ x_swizzle(row)) * 16;
      xdma_off[i] = static_cast<uint32_t>(r * xsrc.ldx + kc);
      // chunks past K: any valid bytes will do, the packed weight is zero there
      xdma_off_last[i] = static_cast<uint32_t>(r * xsrc.ldx + (kc < ktail ? kc : ktail));
    }
    const uint32_t xdma_lds = lds0 + kWBufs * kWStage + wave_u * 1024;
    auto dma = [&](const uint8_t* base, uint32_t off, uint32_t lds_dst) { lds_dma16(base, off, lds_dst); };
    // i-th copy of stage kt into buffer b
    auto dma_one = [&](int kt, int b, int i) {
      if (i < NDW) {
        dma(wtile + static_cast<int64_t>(kt) * (kChunks * 256), wdma_off[i],
            wdma_lds + b * kWStage + i * (NWAVES / 4) * 64 * 16);
      } else {
        const int j = i - NDW;
        dma(xtile + static_cast<int64_t>(kt) * kBK, kt == KT - 1 ? xdma_off_last[j] : xdma_off[j],
            xdma_lds + b * kXStage + j * NWAVES * 1024);
      }
    };
    auto wait_loads = [&](auto left_tag) {  // s_waitcnt vmcnt(left) only
      constexpr int kLeft = decltype(left_tag)::value;
      static_assert(kLeft < 64, "load counter range");
      __builtin_amdgcn_s_waitcnt((kLeft & 15) | ((kLeft >> 4) << 14) | (7 << 4) | (15 << 8));
    };
    auto flip = [&](v4i& f) { f ^= xmask; };
    // b = kt % kDmaBufs as a compile-time constant
    auto stage = [&](int kt, int b) {
      const int bn = (b + 1) % kDmaBufs;
#pragma unroll
      for (int q = 0; q < Q; ++q) {
        if (q < NF) read_one(b, b, 1, q, wf1, xf1);
        mfma(q, wf0, xf0);
        if (q + 1 < TM) flip(xf0[q + 1]);
        if (q == Q - 1) flip(xf1[0]);
        __builtin_amdgcn_sched_barrier(0);
      }
      // only the copies of stages t+2 .. t+kDmaBufs-1 may still be outstanding
      wait_loads(std::integral_constant<int, (kDmaBufs - 2) * ND>{});
      __syncthreads();
      __builtin_amdgcn_sched_barrier(0);
      const int kload = clampk(kt + kDmaBufs);
      // copies go to the MFMA slots that carry no sign flip
      constexpr int kFirstDma = (TM - 1 < Q - 1 - ND) ? TM - 1 : (Q - 1 - ND > 0 ? Q - 1 - ND : 0);
#pragma unroll
      for (int q = 0; q < Q; ++q) {
        if (q < NF) read_one(bn, bn, 0, q, wf0, xf0);
        if (q >= kFirstDma && q - kFirstDma < ND) dma_one(kload, b, q - kFirstDma);
        mfma(q, wf1, xf1);
        if (q + 1 < TM) flip(xf1[q + 1]);
        if (q == Q - 1) flip(xf0[0]);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    // prologue: all buffers in flight, stage 0 landed and visible
#pragma unroll
    for (int st = 0; st < kDmaBufs; ++st)
#pragma unroll
      for (int i = 0; i < ND; ++i) dma_one(clampk(st), st, i);
    init_tile();
    wait_loads(std::integral_constant<int, (kDmaBufs - 1) * ND>{});
    __syncthreads();
#pragma unroll
    for (int j = 0; j < NF; ++j) read_one(0, 0, 0, j, wf0, xf0);
    flip(xf0[0]);
    // the host sends only K >= kDmaBufs stages here: a loop that always runs
    // keeps the prologue's fragments out of the way of the register allocator
    int kt0 = 0;
    do {
#pragma unroll
      for (int j = 0; j < kDmaBufs; ++j) stage(kt0 + j, j);
      kt0 += kDmaBufs;
    } while (kt0 + kDmaBufs <= KT);
#pragma unroll
    for (int j = 0; j < kDmaBufs - 1; ++j)
      if (kt0 + j < KT) stage(kt0 + j, j);
    // the last copies (past the end of K, never read) must have landed before
    // the LDS is reused below or handed to another block
    wait_loads(std::integral_constant<int, 0>{});
  } else {
  init_tile();
  // ---- staging assignments (weight rows past N are clamped: never stored)
  const uint8_t* wsrc[NW];
  int wdst[NW];
#pragma unroll
  for (int i = 0; i < NW; ++i) {
    const int id = t + i * NT;
    const int nbl = id >> 6, kcl = (id >> 4) & 3, r = id & 15;
    int64_t nb = n0 / 16 + nbl;
    nb = nb < NB ? nb : NB - 1;
    wsrc[i] = a.w_packed + (nb * a.w_kchunks + kcl) * 256 + r * 16;
    wdst[i] = (kcl * BN + nbl * 16 + r) * 16;
  }
  XLoader<XSRC> xl[NX];
  int xdst[NX];
#pragma unroll
  for (int i = 0; i < NX; ++i) {
    const int id = t + i * NT;
    const int row = id >> 2, c = id & 3;
    xl[i].init(xsrc, m0 + row, a.M);
    xdst[i] = kWBufs * kWStage + row * kBK + ((c ^ x_swizzle(row)) << 4);
  }
  KCursor<XSRC> kcur;
  kcur.init(xsrc, t & 3);

  v4i wreg[NSET][NW], xreg[NSET][NX];
  // k-th global load of a stage (weights first, then activations)
  auto load_one = [&](int set, int kt, int k) {
    if (k < NW)
      wreg[set][k] = ld16_stream(wsrc[k] + static_cast<int64_t>(kt) * (kChunks * 256));
    else {
      if (k == NW) kcur.seek(xsrc, kt);
      xreg[set][k - NW] = kcur.load(xsrc, xl[k - NW], a.K);
    }
  };
  // k-th LDS store of a stage
  auto store_one = [&](int set, int buf, int k) {
    if (k < NW)
      *reinterpret_cast<v4i*>(&gmem[buf * kWStage + wdst[k]]) = wreg[set][k];
    else
      *reinterpret_cast<v4i*>(&gmem[buf * kXStage + xdst[k - NW]]) = xreg[set][k - NW] ^ xmask;
  };

  // ---- software pipeline.
  // Stage t of the k loop = 64 k-bytes = two MFMA k-steps.  The schedule of one
  // stage, written out in issue order with one memory operation per MFMA so
  // that the matrix pipe never waits for the other pipes:
  //   first half   MFMAs of k-step 0 (fragments already in registers)
  //                + LDS reads of the k-step 1 fragments of stage t
  //                + global loads of stage t+PD into a free register set
  //   barrier      (stage t+1 is now visible in LDS; buffer t&1 is dead)
  //   second half  MFMAs of k-step 1
  //                + LDS reads of the k-step 0 fragments of stage t+1
  //                + LDS stores of stage t+2 (loaded PD-2 stages ago) into buffer t&1
  // Stage s lives in register set s % NSET and in LDS buffer s & 1.  Every
  // operation is unconditional: past the last stage it touches valid memory
  // and its result is never consumed, so the compiler's count of outstanding
  // loads stays exact (a predicated load would force it to drain them all).
  // The scheduling fences keep this order; without them the compiler sinks the
  // global loads to the end of the stage and loses the prefetch distance.
  constexpr int NG = NW + NX;   // global loads (and LDS stores) per stage
  auto stage = [&](int kt, int load_set, int store_set) {
    const int buf = kt & 1;
    const int kload = clampk(kt + PD);
#pragma unroll
    for (int q = 0; q < Q; ++q) {
#pragma unroll
      for (int o = q * (NF + NG) / Q; o < (q + 1) * (NF + NG) / Q; ++o) {
        if (o < NF) read_one(buf, buf, 1, o, wf1, xf1);
        else load_one(load_set, kload, o - NF);
      }
      mfma(q, wf0, xf0);
      __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int q = 0; q < Q; ++q) {
#pragma unroll
      for (int o = q * (NF + NG) / Q; o < (q + 1) * (NF + NG) / Q; ++o) {
        if (o < NF) read_one(buf ^ 1, buf ^ 1, 0, o, wf0, xf0);
        else store_one(store_set, buf, o - NF);
      }
      mfma(q, wf1, xf1);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // prologue: stages 0 and 1 into LDS, stages 2 .. PD-1 in flight
#pragma unroll
  for (int k = 0; k < NG; ++k) load_one(0, 0, k);
#pragma unroll
  for (int k = 0; k < NG; ++k) load_one(1 % NSET, clampk(1), k);
#pragma unroll
  for (int k = 0; k < NG; ++k) store_one(0, 0, k);
#pragma unroll
  for (int s = 2; s < PD; ++s)
#pragma unroll
    for (int k = 0; k < NG; ++k) load_one(s % NSET, clampk(s), k);
  // (with NSET == 2 the loads of stage 2 reuse set 0, already stored above)
#pragma unroll
  for (int k = 0; k < NG; ++k) store_one(1 % NSET, 1, k);
  __syncthreads();
#pragma unroll
  for (int j = 0; j < NF; ++j) read_one(0, 0, 0, j, wf0, xf0);

  int kt0 = 0;
  for (; kt0 + NSET <= KT; kt0 += NSET) {
#pragma unroll
    for (int j = 0; j < NSET; ++j) stage(kt0 + j, (j + 1) % NSET, (j + 2) % NSET);
  }
#pragma unroll
  for (int j = 0; j < NSET - 1; ++j)
    if (kt0 + j < KT) stage(kt0 + j, (j + 1) % NSET, (j + 2) % NSET);
  }

  if constexpr (KW > 1) {
    // add the groups' partial sums: groups 1 .. KW-1 park theirs in LDS (16 B per
    // lane, consecutive lanes on consecutive addresses), group 0 adds them up
    __syncthreads();  // every group is done with its stages
    v4i* const park = reinterpret_cast<v4i*>(smem);
    if (kg > 0) {
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const v4i v = {acc[tn][tm][4 * g], acc[tn][tm][4 * g + 1], acc[tn][tm][4 * g + 2],
                           acc[tn][tm][4 * g + 3]};
            park[(((kg - 1) * TN * TM + tn * TM + tm) * 4 + g) * NT + t] = v;
          }
    }
    __syncthreads();
    if (kg == 0) {
#pragma unroll
      for (int og = 0; og < KW - 1; ++og)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
#pragma unroll
          for (int tm = 0; tm < TM; ++tm)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
              const v4i v = park[((og * TN * TM + tn * TM + tm) * 4 + g) * NT + t];
              acc[tn][tm][4 * g] += v.x;
              acc[tn][tm][4 * g + 1] += v.y;
              acc[tn][tm][4 * g + 2] += v.z;
              acc[tn][tm][4 * g + 3] += v.w;
            }
    }
  }

  // ---- epilogue.  A lane holds, per 32x32 MFMA tile, channels
  // n = 8g + 4*half + j (g, j < 4) of activation row m = li.
  // (KW > 1: only group 0 holds sums; all threads of the block copy rows out.)
  if constexpr (MODE == kOutF32 || MODE == kOutAcc32) {
    // Float results (or the raw accumulators, moved as 32-bit patterns through
    // the same path), one 32-row MFMA tile of every wave at a time: the waves
    // write their rows into LDS, then all threads copy whole rows out, 16 B per
    // lane on consecutive addresses (a lane's own four floats of 32 different
    // rows would make 32 partial lines per store instruction).
    float* const yf = static_cast<float*>(a.y) + a.n_off;
    const bool vec_ok = ((a.ldy & 3) == 0) && ((reinterpret_cast<uintptr_t>(yf) & 15) == 0);
    constexpr int kRowChunks = BN / 4;
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      __syncthreads();  // the operand stages, or the previous pass, are read out
      if (KW == 1 || kg == 0) {
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int nl = wn0 + tn * 32 + 8 * g + 4 * half;
          const v4f mult = *reinterpret_cast<const v4f*>(&s_mult[nl]);
          const v4f bias = *reinterpret_cast<const v4f*>(&s_bdiv[nl]);
          v4f v;
#pragma unroll
          for (int j = 0; j < 4; ++j)
            v[j] = MODE == kOutAcc32
                       ? __int_as_float(acc[tn][tm][4 * g + j])
                       : __builtin_fmaxf(
                             __builtin_fmaf(static_cast<float>(acc[tn][tm][4 * g + j]), mult[j], bias[j]),
                             a.lo_f);
          *reinterpret_cast<v4f*>(&smem[((wave % WM) * 32 + li) * kF32Pitch + nl * 4]) = v;
        }
      }
      __syncthreads();
#pragma unroll 4
      for (int id = tb; id < WM * 32 * kRowChunks; id += NTB) {
        const int lr = id / kRowChunks, cc = id % kRowChunks;
        const int64_t m = m0 + (lr / 32) * WTM + tm * 32 + (lr % 32), n = n0 + cc * 4;
        if (m >= a.M || n >= a.N) continue;
        const v4f v = *reinterpret_cast<const v4f*>(&smem[lr * kF32Pitch + cc * 16]);
        float* dst = yf + m * a.ldy + n;
        if (vec_ok && n + 4 <= a.N) {
          *reinterpret_cast<v4f*>(dst) = v;
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (n + j < a.N) dst[j] = v[j];
        }
      }
    }
  } else {
    // Requantise in registers, transpose through LDS, then write whole rows:
    // 16 bytes per lane, consecutive lanes on consecutive addresses.
    __syncthreads();  // every wave is done with the operand stages
    const float bmul = bias_mul(a.w_scale_stride == 0, x_quant(a).scale * a.w_scales[0]);
    auto requant_tile = [&](auto clamp_tag) {
      constexpr bool CL = decltype(clamp_tag)::value;
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int nl = wn0 + tn * 32 + 8 * g + 4 * half;
        const v4f mult = *reinterpret_cast<const v4f*>(&s_mult[nl]);
        const v4f bdiv = *reinterpret_cast<const v4f*>(&s_bdiv[nl]);
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
          int raw[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) raw[j] = acc[tn][tm][4 * g + j];
          uint32_t q4;
          if (kHasPost && a.post.any()) {
            const int64_t m = m0 + wm0 + tm * 32 + li, n = n0 + nl;
            const int64_t left = a.N - n;
            const int nvalid = (m < a.M && left > 0) ? (left < 4 ? static_cast<int>(left) : 4) : 0;
            const uint32_t accw =
                (a.post.accum != nullptr && nvalid > 0) ? load_accum4(a.post, m * a.ldy + a.n_off + n, nvalid) : 0u;
            q4 = requant4_post<MODE>(raw, bdiv, bmul, mult, a.post, accw, a.zp_f, a.lo_f, a.hi_f);
          } else {
            q4 = requant4<MODE, CL>(raw, bdiv, bmul, mult, a.zp_f, a.lo_f, a.hi_f);
          }
          *reinterpret_cast<uint32_t*>(&smem[(wm0 + tm * 32 + li) * kOutPitch + nl]) = q4;
        }
      }
    };
    // unsigned output without ReLU: the saturating conversion is the clamp
    if (KW > 1 && kg > 0) {
      // nothing to requantise in this group
    } else if (MODE == kOutU8 && a.lo_f <= 0.f && a.hi_f >= 255.f) {
      requant_tile(std::false_type{});
    } else {
      requant_tile(std::true_type{});
    }
    __syncthreads();
    uint8_t* y = static_cast<uint8_t*>(a.y) + a.n_off;
    const bool vec_ok = ((a.ldy & 15) == 0) && ((reinterpret_cast<uintptr_t>(y) & 15) == 0);
    constexpr int kRowChunks = BN / 16;
#pragma unroll 4
    for (int id = tb; id < BM * kRowChunks; id += NTB) {
      const int row = id / kRowChunks, cc = id % kRowChunks;
      const int64_t m = m0 + row, n = n0 + cc * 16;
      if (m >= a.M || n >= a.N) continue;
      const v4i v = ld16(&smem[row * kOutPitch + cc * 16]);
      uint8_t* dst = y + m * a.ldy + n;
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
}

}  // namespace tmq
