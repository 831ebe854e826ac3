"""Seeded test cases shared by the golden-vector generator and the tests.

Every input is rebuilt from a numpy seed, so fixtures only have to hold the
expected outputs (plus a CRC of each rebuilt input, so a change in numpy's
random stream is reported as such and not as a parity failure).

Shapes, scales and zero points replay the reference's own quantized tests:
  tests/unittest/quantized/test_quantized_ops.py:25-99   (quantize cases)
  tests/unittest/quantized/test_quantized_linear.py:14-49 (linear shapes)
  tests/unittest/quantized/test_quantized_conv.py:14-80   (conv configs)
plus the C1 parity configuration (x [128,1024], W [1024,1024] per channel,
bias, output scale 0.05 / zero point 128) and adversarial cases the reference
leaves out (exact ties, tail lengths, extreme zero points, clamping).
"""
from __future__ import annotations

import zlib

import functools

import numpy as np


def crc(a: np.ndarray) -> int:
    return zlib.crc32(np.ascontiguousarray(a).tobytes()) & 0xFFFFFFFF


def randn(seed: int, shape, std: float = 1.0) -> np.ndarray:
    rng = np.random.default_rng(seed)
    return (rng.standard_normal(shape, dtype=np.float32) * np.float32(std)).astype(np.float32)


def absmax_scale(x: np.ndarray, div: float = 128.0) -> float:
    # float(x.abs().max() / 2**7) as in the reference tests: an fp32 division
    return float(np.float32(np.abs(x).max()) / np.float32(div))


# --------------------------------------------------------------------------
# per-tensor quantize / dequantize
# --------------------------------------------------------------------------
def quantize_per_tensor_cases():
    """-> list of dict(name, x, scale, zp, signed)."""
    out = []
    for i, shape in enumerate([(2, 3, 4), (2, 3, 4, 5), (2, 16, 32, 32)]):
        x = randn(100 + i, shape)
        for signed in (False, True):
            out.append(dict(name=f"ref_shape{i}_{'s8' if signed else 'u8'}", x=x,
                            scale=absmax_scale(x), zp=0 if signed else 128,
                            signed=signed))
    # exact ties: x = (k + 0.5) * scale with a power-of-two scale
    k = np.arange(-300, 300, dtype=np.float32)
    for signed in (False, True):
        out.append(dict(name=f"ties_{'s8' if signed else 'u8'}",
                        x=((k + np.float32(0.5)) * np.float32(0.25)).astype(np.float32),
                        scale=0.25, zp=-3 if signed else 7, signed=signed))
    # the fbgemm comment's example where x*inv and x/scale differ
    out.append(dict(name="inv_vs_div", x=np.array([0.273939937], dtype=np.float32),
                    scale=float(np.float32(0.00214854861)), zp=0, signed=False))
    # tail lengths around vector widths
    for n in list(range(1, 20)) + [63, 64, 65, 255, 256, 257, 1023, 1025, 4095,
                                   4096, 4097, 4098, 4099]:
        x = randn(1000 + n, (n,), std=3.0)
        out.append(dict(name=f"tail_{n}", x=x, scale=0.05, zp=100, signed=False))
    # clamping at both ends and extreme zero points
    x = randn(77, (4099,), std=40.0)
    out.append(dict(name="clamp_u8_zp0", x=x, scale=0.1, zp=0, signed=False))
    out.append(dict(name="clamp_u8_zp255", x=x, scale=0.1, zp=255, signed=False))
    out.append(dict(name="clamp_s8_zpm128", x=x, scale=0.1, zp=-128, signed=True))
    out.append(dict(name="clamp_s8_zp127", x=x, scale=0.1, zp=127, signed=True))
    # scale that is not exactly representable + large magnitudes
    x = randn(78, (3001,), std=1000.0)
    out.append(dict(name="big_values", x=x, scale=7.3, zp=13, signed=False))
    return out


def dynamic_qparams_cases():
    """(min, max) pairs for ChooseQuantizationParams, each x reduce_range."""
    pairs = [(-1.0, 1.0), (0.0, 6.0), (-5.0, 0.0), (0.5, 3.0), (-3.0, -0.5),
             (0.0, 0.0), (-1e-9, 1e-9), (-1e-4, 3e-4), (0.0, 1e-3), (-2e-3, 0.0),
             (-50.0, 50.0), (-49.71, 50.33), (-3.4e37, 3.4e37), (-0.1, 25.4),
             (-12.7, 12.8), (-1.0, 254.0), (-1e-7, 2.0)]
    for i in range(12):
        x = randn(300 + i, (64,), std=10.0 ** (i % 4 - 1))
        pairs.append((float(x.min()), float(x.max())))
    return [(np.float32(a), np.float32(b)) for a, b in pairs]


def dynamic_tensor_cases():
    out = []
    for i, shape in enumerate([(2, 3, 4), (2, 3, 4, 5), (2, 16, 32, 32)]):
        out.append(dict(name=f"dyn_shape{i}", x=randn(200 + i, shape)))
    x = randn(210, (70001,), std=3.0)
    x[::101] = 50.0
    x[7::103] = -50.0
    out.append(dict(name="dyn_outliers", x=x))
    out.append(dict(name="dyn_positive", x=np.abs(randn(211, (1000,))) + np.float32(0.5)))
    return out


# --------------------------------------------------------------------------
# per-channel quantize / dequantize
# --------------------------------------------------------------------------
def quantize_per_channel_cases():
    out = []
    out.append(dict(name="ref_2x3_axis0", x=randn(400, (2, 3)),
                    scales=np.array([0.1, 0.01]), zps=np.array([10, 1]), axis=0,
                    signed=False))
    out.append(dict(name="ref_5d_axis3", x=randn(401, (2, 3, 4, 5, 6)),
                    scales=np.array([0.1] * 5), zps=np.array([1] * 5), axis=3,
                    signed=False))
    x = randn(402, (37, 19), std=0.02)
    s = (np.abs(x).max(axis=1) / 127.0).astype(np.float64)
    out.append(dict(name="weight_axis0_s8", x=x, scales=s, zps=np.zeros(37, np.int64),
                    axis=0, signed=True))
    x = randn(403, (4, 6, 5, 3))
    out.append(dict(name="axis1_u8", x=x,
                    scales=np.array([0.013, 0.1, 0.5, 0.02, 0.3, 0.07]),
                    zps=np.array([0, 255, 128, 3, 77, 200]), axis=1, signed=False))
    out.append(dict(name="last_axis_s8", x=x, scales=np.array([0.011, 0.2, 0.05]),
                    zps=np.array([-128, 127, 0]), axis=3, signed=True))
    # float64 scales that are not fp32-representable (pins the double multiply
    # in per-channel dequantize)
    x = randn(404, (8, 301))
    out.append(dict(name="double_scales", x=x,
                    scales=np.array([0.1, 1 / 3, 0.0123456789, 2 / 7, 0.7, 0.05,
                                     1e-2 / 3, 0.9]),
                    zps=np.array([1, 2, 3, 4, 5, 6, 7, 8]), axis=0, signed=False))
    return out


def quantize_per_channel_float_cases():
    """float scales / float zero points (qscheme per_channel_affine_float_qparams):
    embedding-style rows along axis 0, an inner axis, fractional zero points,
    ties (x * inv + zp exactly halfway) and a zero scale."""
    out = []
    x = randn(410, (6, 50))
    mn, mx = x.min(axis=1), x.max(axis=1)
    s = ((mx - mn) / 255.0).astype(np.float32)
    z = (-mn / s).astype(np.float32)
    out.append(dict(name="rows_minmax_u8", x=x, scales=s, zps=z, axis=0, signed=False))
    x = randn(411, (3, 5, 8))
    out.append(dict(name="axis1_u8", x=x, scales=np.array([0.02, 0.5, 0.013, 0.1, 0.25], np.float32),
                    zps=np.array([0.0, 10.5, 127.25, 3.75, 200.0], np.float32), axis=1, signed=False))
    out.append(dict(name="last_axis_s8", x=x, scales=np.full(8, 0.05, np.float32),
                    zps=np.array([-3.5, 0, 1.25, -100, 100, 0.5, -0.5, 7], np.float32), axis=2,
                    signed=True))
    # exact ties: scale 0.25 (a power of two) and zp .0 / .5 make x*inv+zp land on k + 0.5
    k = np.arange(-20, 21, dtype=np.float32)
    x = np.stack([(k + 0.5) * 0.25, k * 0.25]).astype(np.float32)
    out.append(dict(name="ties_u8", x=x, scales=np.array([0.25, 0.25], np.float32),
                    zps=np.array([30.0, 30.5], np.float32), axis=0, signed=False))
    x = randn(412, (2, 7))
    out.append(dict(name="zero_scale_u8", x=x * 40, scales=np.array([0.0, 0.5], np.float32),
                    zps=np.array([100.0, 1.0], np.float32), axis=0, signed=False))
    return out


# --------------------------------------------------------------------------
# quantized::linear
# --------------------------------------------------------------------------
def _int_inputs(seed, m, n, k, x_signed):
    rng = np.random.default_rng(seed)
    if x_signed:
        xq = rng.integers(-128, 128, size=(m, k), dtype=np.int8)
    else:
        xq = rng.integers(0, 256, size=(m, k), dtype=np.uint8)
    wq = rng.integers(-127, 128, size=(n, k), dtype=np.int8)
    bias = (rng.standard_normal(n, dtype=np.float32)).astype(np.float32)
    return xq, wq, bias


def linear_cases():
    """Integer-domain cases: list of dict(name, xq, wq, bias, x_scale, x_zp,
    w_scales, out_scale, out_zp, relu). Weight zero points are 0."""
    out = []
    spec = [
        # name, M, N, K, per_channel, bias, relu, x_zp
        ("ref_8x128_512", 8, 512, 128, False, False, False, 128),
        ("ref_8x128_512_relu", 8, 512, 128, False, False, True, 128),
        ("ref_80x128_512", 80, 512, 128, False, False, False, 120),
        ("pc_bias", 33, 70, 96, True, True, False, 131),
        ("pc_bias_relu", 33, 70, 96, True, True, True, 0),
        ("pt_bias", 17, 40, 64, False, True, False, 255),
        ("odd_k", 5, 9, 37, True, True, False, 17),
        ("one_row", 1, 256, 512, True, True, False, 127),
        ("wide", 3, 1031, 48, True, False, False, 64),
    ]
    for i, (name, m, n, k, pc, has_bias, relu, x_zp) in enumerate(spec):
        xq, wq, bias = _int_inputs(500 + i, m, n, k, False)
        rng = np.random.default_rng(900 + i)
        x_scale = float(np.float32(0.02 + 0.01 * i))
        if pc:
            w_scales = (0.001 + 0.002 * rng.random(n)).astype(np.float32).astype(np.float64)
        else:
            w_scales = np.array([float(np.float32(0.0031))])
        # output scale so that roughly +-3 sigma of the result spans the range
        sigma = np.sqrt(k) * 74.0 * 74.0 * x_scale * float(np.mean(w_scales))
        out_scale = float(np.float32(3.0 * sigma / 128.0))
        out.append(dict(name=name, xq=xq, wq=wq, bias=bias * np.float32(sigma) if has_bias else None,
                        x_scale=x_scale, x_zp=x_zp, w_scales=w_scales,
                        out_scale=out_scale, out_zp=128 if not relu else 10,
                        relu=relu))
    return out


def c1_case():
    """benchmark configuration 1: x fp32 [128,1024] ~N(0,1) -> dynamic quint8;
    W fp32 [1024,1024] ~N(0,0.02) -> per-channel symmetric qint8
    (scale_c = absmax_c / 127); bias fp32 [1024]; out scale 0.05, zp 128."""
    x = randn(41, (128, 1024))
    w = randn(42, (1024, 1024), std=0.02)
    bias = randn(43, (1024,))
    w_scales = (np.abs(w).max(axis=1).astype(np.float32) / np.float32(127.0)).astype(np.float64)
    return dict(x=x, w=w, bias=bias, w_scales=w_scales, out_scale=0.05, out_zp=128)


# --------------------------------------------------------------------------
# quantized::conv2d  (logical NCHW shapes; tensors are built NHWC / OHWI)
# --------------------------------------------------------------------------
def conv_cases():
    spec = [
        # name, B, IC, H, W, OC, k, stride, pad, dil, groups, bias, relu, per_channel
        ("ref_32to64_k3", 2, 32, 16, 16, 64, 3, 1, 1, 1, 1, False, False, False),
        ("ref_32to64_k3_relu", 2, 32, 16, 16, 64, 3, 1, 1, 1, 1, False, True, False),
        ("ref_3to32_k3s2_bias_relu", 2, 3, 16, 16, 32, 3, 2, 1, 1, 1, True, True, False),
        ("ref_64to32_g32_relu", 2, 64, 16, 16, 32, 3, 2, 1, 1, 32, False, True, False),
        ("ref_3to32_k7s2p3_bias", 8, 3, 32, 32, 32, 7, 2, 3, 1, 1, True, False, False),
        ("pc_64to64_k3_bias", 2, 64, 14, 14, 64, 3, 1, 1, 1, 1, True, False, True),
        ("pc_16to48_k1", 3, 16, 9, 11, 48, 1, 1, 0, 1, 1, True, False, True),
        ("pc_32to32_k3_dil2", 1, 32, 13, 13, 32, 3, 1, 2, 2, 1, True, True, True),
        ("pc_groups2", 2, 32, 10, 10, 64, 3, 1, 1, 1, 2, True, False, True),
    ]
    out = []
    for i, (name, b, ic, h, w, oc, k, s, p, d, g, has_bias, relu, pc) in enumerate(spec):
        rng = np.random.default_rng(700 + i)
        x_zp = int(rng.integers(0, 200))
        xq = rng.integers(0, 256, size=(b, h, w, ic), dtype=np.uint8)
        wq = rng.integers(-127, 128, size=(oc, k, k, ic // g), dtype=np.int8)
        bias = rng.standard_normal(oc, dtype=np.float32)
        x_scale = float(np.float32(0.03))
        if pc:
            w_scales = (0.001 + 0.002 * rng.random(oc)).astype(np.float32).astype(np.float64)
        else:
            w_scales = np.array([float(np.float32(0.0027))])
        kk = k * k * (ic // g)
        sigma = np.sqrt(kk) * 74.0 * 74.0 * x_scale * float(np.mean(w_scales))
        out_scale = float(np.float32(3.0 * sigma / 128.0))
        out.append(dict(name=name, xq=xq, wq=wq,
                        bias=bias * np.float32(sigma) if has_bias else None,
                        x_scale=x_scale, x_zp=x_zp, w_scales=w_scales,
                        stride=(s, s), padding=(p, p), dilation=(d, d), groups=g,
                        out_scale=out_scale, out_zp=128 if not relu else 5,
                        relu=relu))
    return out


# --------------------------------------------------------------------------
# fused residual / activation variants of quantized::conv2d
# --------------------------------------------------------------------------
def conv_fused_cases():
    """conv2d_add, conv2d_add_relu, conv2d_silu, conv2d_add_silu on float-born
    data, the way the reference's tests build them (a quantized input, a
    quantized residual of the output's shape, weights quantized per tensor or
    per channel)."""
    spec = [
        # name, B, IC, H, W, OC, k, stride, pad, groups, bias, per_channel, activation, accum, signed
        ("add_16to32_k3", 2, 16, 12, 12, 32, 3, 1, 1, 1, True, False, "none", True, False),
        ("add_relu_32to64_k3s2", 2, 32, 15, 15, 64, 3, 2, 1, 1, True, True, "relu", True, False),
        ("silu_16to16_k3", 1, 16, 10, 10, 16, 3, 1, 1, 1, False, False, "silu", False, False),
        ("add_silu_32to48_k1", 2, 32, 9, 7, 48, 1, 1, 0, 1, True, True, "silu", True, False),
        ("add_groups2_64to64", 2, 64, 8, 8, 64, 3, 1, 1, 2, True, True, "none", True, False),
        ("add_relu_3to8_k3_direct", 2, 3, 11, 11, 8, 3, 1, 1, 1, True, False, "relu", True, False),
        ("add_s8_16to24_k3", 2, 16, 10, 10, 24, 3, 1, 1, 1, True, False, "none", True, True),
        ("add_silu_s8_16to32_k3", 1, 16, 9, 9, 32, 3, 1, 1, 1, False, False, "silu", True, True),
    ]
    out = []
    for i, (name, b, ic, h, w, oc, k, s, p, g, has_bias, pc, act, has_acc, signed) in enumerate(spec):
        rng = np.random.default_rng(1200 + i)
        x = rng.standard_normal((b, h, w, ic), dtype=np.float32)
        wt = rng.standard_normal((oc, k, k, ic // g), dtype=np.float32) * np.float32(0.1)
        bias = rng.standard_normal(oc, dtype=np.float32) if has_bias else None
        x_scale = float(np.float32(np.abs(x).max() / 128.0))
        x_zp = 0 if signed else 128
        lo, hi = (-128, 127) if signed else (0, 255)
        xq = np.clip(np.rint(x / np.float32(x_scale)) + x_zp, lo, hi).astype(np.int8 if signed else np.uint8)
        if pc:
            w_scales = (np.abs(wt).reshape(oc, -1).max(axis=1) / np.float32(127.0)).astype(np.float64)
            wq = np.clip(np.rint(wt / w_scales.astype(np.float32)[:, None, None, None]), -127, 127).astype(np.int8)
        else:
            w_scales = np.array([float(np.float32(np.abs(wt).max() / 128.0))])
            wq = np.clip(np.rint(wt / np.float32(w_scales[0])), -127, 127).astype(np.int8)
        oh = (h + 2 * p - (k - 1) - 1) // s + 1
        ow = (w + 2 * p - (k - 1) - 1) // s + 1
        acc = accq = None
        acc_scale, acc_zp = 1.0, 0
        if has_acc:
            acc = rng.standard_normal((b, oh, ow, oc), dtype=np.float32) * np.float32(2.0)
            acc_scale = float(np.float32(np.abs(acc).max() / 128.0))
            acc_zp = 0 if signed else 128
            accq = np.clip(np.rint(acc / np.float32(acc_scale)) + acc_zp, lo, hi).astype(xq.dtype)
        # spread of conv + residual, for an output scale that uses the range
        sigma = float(np.sqrt(k * k * (ic // g)) * 0.1 + (2.0 if has_acc else 0.0))
        out_scale = float(np.float32(3.0 * sigma / 128.0))
        out.append(dict(name=name, xq=xq, x_scale=x_scale, x_zp=x_zp, wq=wq, w_scales=w_scales, bias=bias,
                        stride=(s, s), padding=(p, p), dilation=(1, 1), groups=g, accq=accq,
                        acc_scale=acc_scale, acc_zp=acc_zp, activation=act, out_scale=out_scale,
                        out_zp=0 if signed else 128, signed=signed))
    return out


# --------------------------------------------------------------------------
# quantized::add / add_relu and relu of a quantized tensor
# --------------------------------------------------------------------------
def qadd_cases():
    spec = [
        # name, shape, signed, relu, (a_scale, a_zp), (b_scale, b_zp), (out_scale, out_zp)
        ("ref_u8", (2, 16, 8, 8), False, False, (0.05, 128), (0.031, 120), (0.07, 128)),
        ("ref_u8_relu", (2, 16, 8, 8), False, True, (0.05, 128), (0.031, 120), (0.07, 128)),
        ("s8", (3, 5, 7), True, False, (0.02, 0), (0.045, -3), (0.05, 4)),
        ("s8_relu", (3, 5, 7), True, True, (0.02, 0), (0.045, -3), (0.05, -20)),
        ("saturating_u8", (4099,), False, False, (0.1, 10), (0.2, 250), (0.05, 100)),
        ("odd_sizes_u8_relu", (1, 3, 5, 11), False, True, (0.013, 77), (0.4, 3), (0.11, 9)),
        ("big_u8", (64, 1031), False, False, (1 / 3, 128), (0.0123456789, 127), (0.21, 101)),
    ]
    out = []
    for i, (name, shape, signed, relu, (sa, za), (sb, zb), (so, zo)) in enumerate(spec):
        rng = np.random.default_rng(1300 + i)
        lo, hi = (-128, 128) if signed else (0, 256)
        dt = np.int8 if signed else np.uint8
        out.append(dict(name=name, qa=rng.integers(lo, hi, shape).astype(dt),
                        qb=rng.integers(lo, hi, shape).astype(dt), a_scale=sa, a_zp=za, b_scale=sb,
                        b_zp=zb, out_scale=so, out_zp=zo, signed=signed, relu=relu))
    return out


# --------------------------------------------------------------------------
# quantized::cat and quantized max pooling
# --------------------------------------------------------------------------
def qcat_cases():
    spec = [
        # name, shapes (differ along axis only), axis, signed, per-input (scale, zp), out (scale, zp)
        ("same_params_axis1", [(2, 3, 4), (2, 5, 4)], 1, False, [(0.1, 10), (0.1, 10)], (0.1, 10)),
        ("requant_axis1", [(2, 3, 4), (2, 5, 4), (2, 1, 4)], 1, False, [(0.1, 10), (0.2, 20), (0.05, 0)], (0.15, 30)),
        ("requant_axis0_s8", [(3, 7), (2, 7)], 0, True, [(0.02, -3), (0.045, 5)], (0.03, 1)),
        ("last_axis", [(4, 6, 16), (4, 6, 32)], -1, False, [(0.3, 128), (0.11, 100)], (0.2, 120)),
        ("channels_16aligned", [(2, 16, 5, 5), (2, 32, 5, 5)], 1, False, [(0.07, 77), (0.09, 99)], (0.08, 88)),
    ]
    out = []
    for i, (name, shapes, axis, signed, params, (so, zo)) in enumerate(spec):
        rng = np.random.default_rng(1400 + i)
        lo, hi = (-128, 128) if signed else (0, 256)
        dt = np.int8 if signed else np.uint8
        out.append(dict(name=name, qs=[rng.integers(lo, hi, sh).astype(dt) for sh in shapes], axis=axis,
                        scales=[p[0] for p in params], zps=[p[1] for p in params], out_scale=so, out_zp=zo,
                        signed=signed))
    return out


def qmaxpool_cases():
    spec = [
        # name, (B, H, W, C), kernel, stride, padding, dilation, ceil_mode, signed
        ("k3s2p1_c16", (2, 13, 13, 16), (3, 3), (2, 2), (1, 1), (1, 1), False, False),
        ("k3s2p1_ceil_c16", (2, 14, 14, 16), (3, 3), (2, 2), (1, 1), (1, 1), True, False),
        ("k2s2_c5_s8", (3, 8, 10, 5), (2, 2), (2, 2), (0, 0), (1, 1), False, True),
        ("k3s1p1_dil2_c32", (1, 9, 9, 32), (3, 3), (1, 1), (1, 1), (2, 2), False, False),
        ("k5x3_s2x1_c7", (2, 11, 6, 7), (5, 3), (2, 1), (2, 1), (1, 1), True, True),
    ]
    out = []
    for i, (name, shape, k, s, p, d, ceil_mode, signed) in enumerate(spec):
        rng = np.random.default_rng(1500 + i)
        lo, hi = (-128, 128) if signed else (0, 256)
        out.append(dict(name=name, x=rng.integers(lo, hi, shape).astype(np.int8 if signed else np.uint8),
                        kernel=k, stride=s, padding=p, dilation=d, ceil_mode=ceil_mode, signed=signed))
    return out


def qavgpool_cases():
    spec = [
        # name, (B, H, W, C), (OH, OW), zero point, signed
        ("global_7x7_c64", (2, 7, 7, 64), (1, 1), 120, False),
        ("ties_4x4_to_2x2_c8", (2, 4, 4, 8), (2, 2), 3, False),
        ("ragged_13x9_to_5x3_c48", (2, 13, 9, 48), (5, 3), 77, False),
        ("c7_10x11_to_3x4_s8", (1, 10, 11, 7), (3, 4), -9, True),
        ("upsample_3x3_to_5x5_c4", (1, 3, 3, 4), (5, 5), 0, False),
        ("global_14x14_c130_s8", (1, 14, 14, 130), (1, 1), 5, True),
    ]
    out = []
    for i, (name, shape, ohw, zp, signed) in enumerate(spec):
        rng = np.random.default_rng(1600 + i)
        lo, hi = (-128, 128) if signed else (0, 256)
        out.append(dict(name=name, x=rng.integers(lo, hi, shape).astype(np.int8 if signed else np.uint8),
                        out_hw=ohw, zp=zp, signed=signed))
    return out


@functools.lru_cache(maxsize=None)
def _rounding_probe_rows():
    """[8, 64] float activations with minimum -8 and maximum 9 (scale 17/255,
    zero point 120) whose other values are picked where rne(fl(x * inv)) + zp
    and rne(fl(x * inv + zp)) disagree -- about six values in a million do -- so
    that a dynamic linear that quantizes its activations in the wrong one of the
    two forms cannot pass."""
    rng = np.random.default_rng(1799)
    cand = (rng.standard_normal(6_000_000) * 2.5).astype(np.float32)
    cand = cand[(cand > -7.9) & (cand < 8.9)]
    inv = np.float32(1.0) / np.float32(17.0 / 255.0)
    two_step = np.rint(cand * inv) + np.float32(120)
    fused = np.rint((cand.astype(np.float64) * np.float64(inv) + 120.0).astype(np.float32))
    picked = cand[two_step != fused]
    assert picked.size >= 16, picked.size
    x = (rng.standard_normal(512) * 2.0).astype(np.float32)
    x[: picked.size][:400] = picked[:400]
    x[510], x[511] = np.float32(-8.0), np.float32(9.0)
    return rng.permutation(x).reshape(8, 64).copy()


def linear_dynamic_cases():
    """Float activations for quantized::linear_dynamic: dict(name, x, wq, w_scales,
    bias, relu, reduce_range). Weight zero points are 0."""
    spec = [
        # name, x shape, N, per_channel, bias, relu, reduce_range
        ("pc_bias_8x64_48", (8, 64), 48, True, True, False, False),
        ("pt_bias_33x100_70", (33, 100), 70, False, True, False, False),
        ("pc_relu_16x256_33", (16, 256), 33, True, True, True, False),
        ("pt_relu_rr_16x256_33", (16, 256), 33, False, True, True, True),
        ("pc_nobias_rr_5x37_9", (5, 37), 9, True, False, False, True),
        ("batched_3x7x128_130", (3, 7, 128), 130, True, True, False, True),
        ("one_row_1x512_256", (1, 512), 256, True, True, False, False),
        ("tall_300x192_72", (300, 192), 72, True, True, False, False),
    ]
    out = []
    for i, (name, xshape, n, pc, has_bias, relu, rr) in enumerate(spec):
        rng = np.random.default_rng(1700 + i)
        k = xshape[-1]
        x = (rng.standard_normal(xshape) * 1.7 + 0.3).astype(np.float32)
        wq = rng.integers(-127, 128, (n, k), dtype=np.int8)
        if pc:
            w_scales = (0.0005 + 0.001 * rng.random(n)).astype(np.float32).astype(np.float64)
        else:
            w_scales = np.array([float(np.float32(0.00093))])
        bias = rng.standard_normal(n).astype(np.float32) if has_bias else None
        out.append(dict(name=name, x=x, wq=wq, w_scales=w_scales, bias=bias, relu=relu, reduce_range=rr))
    rng = np.random.default_rng(1798)
    out.append(dict(name="rounding_forms_8x64_40", x=_rounding_probe_rows(),
                    wq=rng.integers(-127, 128, (40, 64), dtype=np.int8),
                    w_scales=(0.0005 + 0.001 * rng.random(40)).astype(np.float32).astype(np.float64),
                    bias=rng.standard_normal(40).astype(np.float32), relu=False, reduce_range=False))
    return out


def plain_linear_cases():
    """quantized::linear_per_tensor: plain uint8 / int8 activations [M,K], int8 weight
    [K,N] (the layout the schema takes), parameters beside them.  The first three
    are the reference's (test_quantized_ops.py:745-795: small non-negative
    integers, unit activation and output scale), where every arithmetic order
    gives the same integers."""
    out = []
    for i, (s1, s2) in enumerate([((1, 10), (10, 5)), ((2, 3), (3, 4)), ((10, 7), (7, 10))]):
        rng = np.random.default_rng(1800 + i)
        for dt in ("uint8", "float32"):
            out.append(dict(name=f"ref{i}_{dt}", x=rng.integers(0, 10, s1).astype(np.int8),
                            w=rng.integers(0, 10, s2).astype(np.int8), x_scale=1.0, x_zp=0,
                            w_scale=rng.integers(1, 10, s2[1]).astype(np.float32), bias=np.ones(s2[1], np.float32),
                            out_scale=1.0, out_zp=0, out_dtype=dt, post="none"))
    spec = [
        # name, M, K, N, act dtype, x_zp, out dtype, post, bias
        ("u8_relu_33x96_70", 33, 96, 70, np.uint8, 121, "uint8", "relu", True),
        ("s8_s8_17x64_40", 17, 64, 40, np.int8, -5, "int8", "none", True),
        ("u8_f32_5x37_9", 5, 37, 9, np.uint8, 17, "float32", "none", False),
        ("u8_f32_relu_64x256_130", 64, 256, 130, np.uint8, 128, "float32", "relu", True),
        ("u8_tall_300x192_72", 300, 192, 72, np.uint8, 100, "uint8", "none", True),
    ]
    for i, (name, m, k, n, adt, zp, odt, post, has_bias) in enumerate(spec):
        rng = np.random.default_rng(1850 + i)
        lo, hi = (-128, 128) if adt == np.int8 else (0, 256)
        x_scale = float(np.float32(0.02))
        w_scale = (0.001 + 0.002 * rng.random(n)).astype(np.float32)
        sigma = np.sqrt(k) * 74.0 * 74.0 * x_scale * float(w_scale.mean())
        out_int = odt != "float32"
        out.append(dict(name=name, x=rng.integers(lo, hi, (m, k)).astype(adt),
                        w=rng.integers(-127, 128, (k, n)).astype(np.int8), x_scale=x_scale, x_zp=zp,
                        w_scale=w_scale, bias=(rng.standard_normal(n) * sigma).astype(np.float32) if has_bias else None,
                        out_scale=float(np.float32(3 * sigma / 128)) if out_int else 1.0,
                        out_zp=(-3 if odt == "int8" else 128) if out_int else 0, out_dtype=odt, post=post))
    return out


def plain_conv_cases():
    """quantized::conv / quantized::conv_binary: plain NCHW uint8 activations, OIHW int8
    weights.  The first three shapes are the reference's (test_quantized_ops.py:798-951)."""
    out = []
    spec = [
        # name, x shape, w shape, stride, pad, groups, small ints?, out dtype, relu, accum ("none" | "uint8" | "float32")
        ("ref0_f32", (1, 1, 5, 5), (1, 1, 3, 3), 1, 0, 1, True, "float32", False, "none"),
        ("ref1_f32_relu", (1, 3, 10, 10), (4, 3, 2, 2), 1, 0, 1, True, "float32", True, "none"),
        ("ref2_f32", (10, 5, 6, 6), (8, 5, 2, 2), 1, 0, 1, True, "float32", False, "none"),
        ("ref2_sum_f32", (10, 5, 6, 6), (8, 5, 2, 2), 1, 0, 1, True, "float32", False, "float32"),
        ("u8_relu_2x32x12x12_k3", (2, 32, 12, 12), (48, 32, 3, 3), 1, 1, 1, False, "uint8", True, "none"),
        ("u8_s2_groups2", (2, 32, 13, 13), (64, 16, 3, 3), 2, 1, 2, False, "uint8", False, "none"),
        ("f32_1x1_64", (3, 64, 7, 7), (32, 64, 1, 1), 1, 0, 1, False, "float32", True, "none"),
        ("u8_sum_relu", (2, 16, 8, 8), (32, 16, 3, 3), 1, 1, 1, False, "uint8", True, "uint8"),
        ("u8_sum", (2, 16, 8, 8), (32, 16, 3, 3), 1, 1, 1, False, "uint8", False, "uint8"),
        ("f32_sum_relu", (2, 16, 8, 8), (32, 16, 3, 3), 1, 1, 1, False, "float32", True, "float32"),
    ]
    for i, (name, xs, wshape, st, pd, groups, small, odt, relu, accum) in enumerate(spec):
        rng = np.random.default_rng(1900 + i)
        oc = wshape[0]
        kh, kw = wshape[2], wshape[3]
        oh = (xs[2] + 2 * pd - kh) // st + 1
        ow = (xs[3] + 2 * pd - kw) // st + 1
        if small:
            x = rng.integers(0, 10, xs).astype(np.uint8)
            w = rng.integers(0, 10, wshape).astype(np.int8)
            x_scale, x_zp = 1.0, 0
            w_scale = (np.abs(rng.standard_normal(oc)) + 0.1).astype(np.float32)
            bias = None
            out_scale, out_zp = 1.0, 0
        else:
            x = rng.integers(0, 256, xs).astype(np.uint8)
            w = rng.integers(-127, 128, wshape).astype(np.int8)
            x_scale, x_zp = float(np.float32(0.03)), 120
            w_scale = (0.002 + 0.01 * rng.random(oc)).astype(np.float32)
            bias = rng.standard_normal(oc).astype(np.float32)
            k = wshape[1] * kh * kw
            sigma = np.sqrt(k) * 74.0 * 74.0 * x_scale * float(w_scale.mean())
            out_scale, out_zp = (float(np.float32(3 * sigma / 128)), 10 if relu else 128) if odt == "uint8" else (1.0, 0)
        c = dict(name=name, x=x, w=w, x_scale=x_scale, x_zp=x_zp, w_scale=w_scale, bias=bias, stride=st, pad=pd,
                 groups=groups, out_scale=out_scale, out_zp=out_zp, out_dtype=odt, relu=relu, accum=None,
                 accum_scale=1.0, accum_zp=0)
        if accum == "uint8":
            c["accum"] = rng.integers(0, 256, (xs[0], oc, oh, ow)).astype(np.uint8)
            c["accum_scale"], c["accum_zp"] = float(np.float32(out_scale * 0.7)), 100
        elif accum == "float32":
            c["accum"] = (rng.standard_normal((xs[0], oc, oh, ow)) * (1.0 if small else 3.0)).astype(np.float32)
        out.append(c)
    return out


def qunary_cases():
    spec = [
        # name, shape, scale, zero point, signed
        ("u8_zp128_4x3000", (4, 3000), 0.0679, 128, False),
        ("s8_zp0_2x16x9x9", (2, 16, 9, 9), 0.0431, 0, True),
        ("u8_zp37_777", (777,), 0.0213, 37, False),
        ("s8_zpm20_33x65", (33, 65), 0.11, -20, True),
    ]
    out = []
    for i, (name, shape, scale, zp, signed) in enumerate(spec):
        rng = np.random.default_rng(2000 + i)
        lo, hi = (-128, 128) if signed else (0, 256)
        out.append(dict(name=name, x=rng.integers(lo, hi, shape).astype(np.int8 if signed else np.uint8),
                        scale=float(np.float32(scale)), zp=zp, signed=signed))
    return out
