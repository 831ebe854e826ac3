"""The CPU oracle against what the mathematics fixes, independently of any
fixture: exact rational rounding, brute force over all codes, exact int64
matmul, closed-form special cases of the output stage, conv == GEMM on im2col."""
from fractions import Fraction

import numpy as np
import pytest

import oracle


def _rne(fr: Fraction) -> int:
    fl = fr.numerator // fr.denominator
    rem = fr - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1):
        return fl + 1
    return fl


@pytest.mark.parametrize("signed", [False, True])
def test_quantize_matches_exact_rational_rounding(signed):
    # power-of-two scale: x*inv is exact in fp32, so the result is RNE of the
    # exact quotient, shifted and clamped.
    rng = np.random.default_rng(1)
    x = (rng.integers(-4000, 4000, size=5000).astype(np.float32) / np.float32(8.0))
    scale, zp = 0.5, (-5 if signed else 9)
    q = oracle.quantize_per_tensor(x, scale, zp, signed)
    lo, hi = (-128, 127) if signed else (0, 255)
    want = [min(hi, max(lo, _rne(Fraction(float(v)) / Fraction(scale)) + zp)) for v in x]
    np.testing.assert_array_equal(q.astype(np.int64), np.array(want))


def test_ties_round_to_even_not_away():
    x = np.array([0.5, 1.5, 2.5, 3.5, -0.5, -1.5, -2.5], dtype=np.float32)
    q = oracle.quantize_per_tensor(x, 1.0, 10, False)
    np.testing.assert_array_equal(q, np.array([10, 12, 12, 14, 10, 8, 8], dtype=np.uint8))


def test_multiply_by_reciprocal_not_divide():
    # fbgemm's documented example: x*inv gives 127.5 -> 128, x/scale gives 127
    q = oracle.quantize_per_tensor(np.array([0.273939937], np.float32),
                                   float(np.float32(0.00214854861)), 0, False)
    assert int(q[0]) == 128


@pytest.mark.parametrize("signed", [False, True])
def test_dequantize_all_codes_and_roundtrip(signed):
    codes = np.arange(-128, 128, dtype=np.int8) if signed else np.arange(256, dtype=np.uint8)
    for scale, zp in [(0.1, 3), (0.0143444, 127 if not signed else -7), (1 / 3, 0)]:
        r = oracle.dequantize_per_tensor(codes, scale, zp)
        want = (np.float32(scale) * (codes.astype(np.int32) - zp).astype(np.float32)).astype(np.float32)
        np.testing.assert_array_equal(r, want)
        # every code is a fixed point of dequantize -> quantize
        back = oracle.quantize_per_tensor(r, scale, zp, signed)
        np.testing.assert_array_equal(back, codes)


def test_per_channel_reduces_to_per_tensor():
    rng = np.random.default_rng(2)
    x = rng.standard_normal((5, 7, 3), dtype=np.float32)
    scales = np.array([0.02, 0.3, 0.011, 0.07, 0.5, 0.09, 0.013])
    zps = np.array([0, 255, 7, 128, 64, 1, 200])
    q = oracle.quantize_per_channel(x, scales, zps, 1, False)
    for c in range(7):
        np.testing.assert_array_equal(
            q[:, c, :], oracle.quantize_per_tensor(x[:, c, :], scales[c], zps[c], False))
    dq = oracle.dequantize_per_channel(q, scales, zps, 1)
    want = ((q.astype(np.float32) - zps.astype(np.float32)[None, :, None]).astype(np.float64)
            * scales[None, :, None]).astype(np.float32)
    np.testing.assert_array_equal(dq, want)


def test_choose_qparams_invariants():
    rng = np.random.default_rng(3)
    for _ in range(300):
        a, b = np.sort(rng.standard_normal(2).astype(np.float32) * np.float32(10.0 ** rng.integers(-3, 3)))
        for rr in (False, True):
            s, z = oracle.choose_qparams(a, b, False, rr)
            qmax = 127 if rr else 255
            assert s > 0 and 0 <= z <= qmax
            # zero is exactly representable
            assert oracle.dequantize_per_tensor(np.array([z], np.uint8), s, z)[0] == 0.0
            # closed form of the scale when no cut-off applies
            lo, hi = min(float(a), 0.0), max(float(b), 0.0)
            if (hi - lo) / qmax >= 6.1e-5:
                assert s == (hi - lo) / qmax
    assert oracle.choose_qparams(0.0, 0.0)[0] == 0.1  # degenerate range fallback
    with pytest.raises(ValueError):
        oracle.choose_qparams(1.0, -1.0)


@pytest.mark.parametrize("x_signed", [False, True])
def test_linear_acc32_is_exact_integer_matmul(x_signed):
    rng = np.random.default_rng(4)
    m, n, k = 13, 29, 257
    x = rng.integers(-128, 128, (m, k), dtype=np.int8) if x_signed else rng.integers(0, 256, (m, k), dtype=np.uint8)
    w = rng.integers(-128, 128, (n, k), dtype=np.int8)
    acc = oracle.linear_acc32(x, w)
    np.testing.assert_array_equal(acc.astype(np.int64), x.astype(np.int64) @ w.astype(np.int64).T)
    np.testing.assert_array_equal(oracle.weight_colsum(w), w.astype(np.int64).sum(axis=1))
    # worst-case magnitudes stay inside int32 for K this small
    xmax = np.full((1, k), -128 if x_signed else 255, dtype=x.dtype)
    wmin = np.full((1, k), -128, dtype=np.int8)
    assert int(oracle.linear_acc32(xmax, wmin)[0, 0]) == int(xmax[0, 0]) * -128 * k


def test_requantize_special_cases():
    rng = np.random.default_rng(5)
    acc = rng.integers(-400, 400, (6, 9)).astype(np.int32)
    colsum = rng.integers(-50, 50, 9).astype(np.int32)
    # multiplier exactly 1 (x_scale*w_scale == out_scale), no bias:
    #   y = clamp(acc - x_zp*colsum + out_zp)
    y = oracle.requantize(acc, colsum, 3, 0.5, [0.25], None, 0.125, 100)
    want = np.clip(acc.astype(np.int64) - 3 * colsum + 100, 0, 255)
    np.testing.assert_array_equal(y.astype(np.int64), want)
    # relu raises the lower clamp to the zero point
    y = oracle.requantize(acc, colsum, 3, 0.5, [0.25], None, 0.125, 100, relu=True)
    np.testing.assert_array_equal(y.astype(np.int64), np.clip(want, 100, 255))
    # signed output range
    y = oracle.requantize(acc, colsum, 0, 0.5, [0.25], None, 0.125, -3, out_signed=True)
    np.testing.assert_array_equal(y.astype(np.int64),
                                  np.clip(acc.astype(np.int64) - 3, -128, 127))
    # power-of-two multiplier 1/4 with exact halves -> ties to even
    acc2 = np.array([[2, 6, 10, -2, -6, 1, 3]], dtype=np.int32)
    y = oracle.requantize(acc2, np.zeros(7, np.int32), 0, 0.5, [0.5], None, 1.0, 100)
    np.testing.assert_array_equal(y[0], np.array([100, 102, 102, 100, 98, 100, 101], np.uint8))
    # bias enters as bias / (x_scale*w_scale) BEFORE the multiply:
    #   bias = 3*atw exactly  ->  same as adding 3 to the accumulator
    atw = 0.5 * 0.25
    y_b = oracle.requantize(acc, colsum, 3, 0.5, [0.25], np.full(9, 3 * atw, np.float32), 0.125, 100)
    np.testing.assert_array_equal(y_b.astype(np.int64),
                                  np.clip(acc.astype(np.int64) - 3 * colsum + 103, 0, 255))
    # per-channel scales pick the column's own multiplier
    ws = np.array([0.25 * 2.0 ** (j % 3) for j in range(9)])
    y_pc = oracle.requantize(acc, np.zeros(9, np.int32), 0, 0.5, ws, None, 0.125, 0)
    want_pc = np.clip(acc.astype(np.int64) * (2 ** (np.arange(9) % 3))[None, :], 0, 255)
    np.testing.assert_array_equal(y_pc.astype(np.int64), want_pc)


def _im2col(x, kh, kw, stride, padding, dilation, x_zp):
    b, h, w, c = x.shape
    oh, ow = oracle.conv_out_hw(h, w, kh, kw, stride, padding, dilation)
    cols = np.zeros((b, oh, ow, kh, kw, c), dtype=np.int64)
    for i in range(oh):
        for j in range(ow):
            for a in range(kh):
                for e in range(kw):
                    ih = i * stride[0] - padding[0] + a * dilation[0]
                    iw = j * stride[1] - padding[1] + e * dilation[1]
                    if 0 <= ih < h and 0 <= iw < w:
                        cols[:, i, j, a, e, :] = x[:, ih, iw, :].astype(np.int64) - x_zp
    return cols.reshape(b * oh * ow, kh * kw * c), (b, oh, ow)


@pytest.mark.parametrize("stride,padding,dilation", [((1, 1), (1, 1), (1, 1)),
                                                     ((2, 1), (0, 2), (1, 2)),
                                                     ((3, 2), (2, 0), (2, 1))])
def test_conv_acc32_equals_gemm_on_im2col(stride, padding, dilation):
    rng = np.random.default_rng(6)
    x = rng.integers(0, 256, (2, 9, 8, 5), dtype=np.uint8)
    w = rng.integers(-128, 128, (7, 3, 3, 5), dtype=np.int8)
    acc = oracle.conv2d_acc32(x, w, stride, padding, dilation, 1, 77)
    cols, (b, oh, ow) = _im2col(x, 3, 3, stride, padding, dilation, 77)
    want = cols @ w.reshape(7, -1).astype(np.int64).T
    np.testing.assert_array_equal(acc.reshape(-1, 7).astype(np.int64), want)


def test_conv_groups_are_independent_convs():
    rng = np.random.default_rng(7)
    x = rng.integers(0, 256, (1, 6, 6, 8), dtype=np.uint8)
    w = rng.integers(-128, 128, (6, 3, 3, 4), dtype=np.int8)   # groups=2: 2x(4 -> 3)
    acc = oracle.conv2d_acc32(x, w, (1, 1), (1, 1), (1, 1), 2, 9)
    for g in range(2):
        part = oracle.conv2d_acc32(np.ascontiguousarray(x[..., 4 * g:4 * g + 4]),
                                   np.ascontiguousarray(w[3 * g:3 * g + 3]),
                                   (1, 1), (1, 1), (1, 1), 1, 9)
        np.testing.assert_array_equal(acc[..., 3 * g:3 * g + 3], part)


def test_conv_1x1_is_linear():
    rng = np.random.default_rng(8)
    x = rng.integers(0, 256, (2, 5, 4, 16), dtype=np.uint8)
    w = rng.integers(-127, 128, (12, 1, 1, 16), dtype=np.int8)
    ws = 0.001 + 0.002 * rng.random(12)
    bias = rng.standard_normal(12).astype(np.float32)
    yc = oracle.conv2d(x, 0.03, 50, w, ws, bias, (1, 1), (0, 0), (1, 1), 1, 0.08, 120)
    yl = oracle.linear(x.reshape(-1, 16), 0.03, 50, w.reshape(12, 16), ws, bias, 0.08, 120)
    np.testing.assert_array_equal(yc.reshape(-1, 12), yl)


# ---------------------------------------------------------------------------
# fused conv variants: special cases that fix each term of the closed form
# ---------------------------------------------------------------------------
def _fused_inputs(seed=5):
    rng = np.random.default_rng(seed)
    x = rng.integers(0, 256, (2, 7, 6, 16), dtype=np.uint8)
    w = rng.integers(-127, 128, (8, 3, 3, 16), dtype=np.int8)
    ws = (0.001 + 0.002 * rng.random(8)).astype(np.float32).astype(np.float64)
    bias = rng.standard_normal(8).astype(np.float32)
    return rng, x, w, ws, bias


def test_fused_without_post_ops_is_plain_conv():
    _, x, w, ws, bias = _fused_inputs()
    for relu in (False, True):
        a = oracle.conv2d(x, 0.03, 90, w, ws, bias, (1, 1), (1, 1), (1, 1), 1, 0.4, 100, relu=relu)
        b = oracle.conv2d_fused(x, 0.03, 90, w, ws, bias, (1, 1), (1, 1), (1, 1), 1, 0.4, 100,
                                activation="relu" if relu else "none")
        np.testing.assert_array_equal(a, b)


def test_fused_residual_at_its_zero_point_adds_nothing():
    _, x, w, ws, bias = _fused_inputs()
    acc = np.full((2, 7, 6, 8), 77, np.uint8)
    a = oracle.conv2d(x, 0.03, 90, w, ws, bias, (1, 1), (1, 1), (1, 1), 1, 0.4, 100)
    b = oracle.conv2d_fused(x, 0.03, 90, w, ws, bias, (1, 1), (1, 1), (1, 1), 1, 0.4, 100, accum=acc,
                            accum_scale=0.123, accum_zp=77)
    np.testing.assert_array_equal(a, b)


def test_fused_zero_weights_pass_the_residual_through():
    """conv == 0 and accum_scale == out_scale: y = qa - za + zp, clamped; with a
    scale ratio of 2 the residual's distance from its zero point doubles."""
    rng, x, w, ws, _ = _fused_inputs()
    acc = rng.integers(0, 256, (2, 7, 6, 8), dtype=np.uint8)
    y = oracle.conv2d_fused(x, 0.03, 90, np.zeros_like(w), ws, None, (1, 1), (1, 1), (1, 1), 1, 0.25,
                            100, accum=acc, accum_scale=0.25, accum_zp=120)
    np.testing.assert_array_equal(y, np.clip(acc.astype(int) - 120 + 100, 0, 255))
    y2 = oracle.conv2d_fused(x, 0.03, 90, np.zeros_like(w), ws, None, (1, 1), (1, 1), (1, 1), 1, 0.25,
                             100, accum=acc, accum_scale=0.5, accum_zp=120, activation="relu")
    np.testing.assert_array_equal(y2, np.clip(2 * (acc.astype(int) - 120) + 100, 100, 255))


def test_fused_silu_of_a_known_value():
    """One output value at a time: conv == 0, residual r, silu(r) = r / (1 + e^-r)."""
    _, x, w, ws, _ = _fused_inputs()
    acc = np.arange(2 * 7 * 6 * 8, dtype=np.int64).reshape(2, 7, 6, 8) % 256
    acc = acc.astype(np.uint8)
    s = 0.05
    y = oracle.conv2d_fused(x, 0.03, 90, np.zeros_like(w), ws, None, (1, 1), (1, 1), (1, 1), 1, s, 30,
                            accum=acc, accum_scale=s, accum_zp=128, activation="silu")
    r = (acc.astype(np.float64) - 128) * s
    want = np.clip(np.rint(r / (1 + np.exp(-r)) / s) + 30, 0, 255)
    d = np.abs(y.astype(int) - want.astype(int))
    assert d.max() <= 1 and np.count_nonzero(d) <= 2  # float32 vs float64 at exact ties only


# ---------------------------------------------------------------------------
# quantized::add: cases with an exact answer
# ---------------------------------------------------------------------------
def test_qadd_equal_power_of_two_scales_is_integer_addition():
    rng = np.random.default_rng(8)
    qa = rng.integers(0, 256, 5000, dtype=np.uint8)
    qb = rng.integers(0, 256, 5000, dtype=np.uint8)
    y = oracle.qadd(qa, 0.25, 100, qb, 0.25, 90, 0.25, 60)
    np.testing.assert_array_equal(y, np.clip(qa.astype(int) - 100 + qb.astype(int) - 90 + 60, 0, 255))
    yr = oracle.qadd(qa, 0.25, 100, qb, 0.25, 90, 0.25, 60, relu=True)
    np.testing.assert_array_equal(yr, np.clip(np.maximum(qa.astype(int) - 100 + qb.astype(int) - 90, 0) + 60, 0, 255))
    # output scale twice as coarse: halves, ties to even
    y2 = oracle.qadd(qa, 0.25, 100, qb, 0.25, 90, 0.5, 60)
    np.testing.assert_array_equal(y2, np.clip(np.rint((qa.astype(int) - 100 + qb.astype(int) - 90) / 2.0) + 60, 0, 255))


def test_qadd_close_to_real_arithmetic():
    rng = np.random.default_rng(9)
    qa = rng.integers(-128, 128, 20000).astype(np.int8)
    qb = rng.integers(-128, 128, 20000).astype(np.int8)
    y = oracle.qadd(qa, 0.037, -5, qb, 0.11, 17, 0.09, 3)
    real = (qa.astype(np.float64) + 5) * np.float64(np.float32(0.037)) + (qb.astype(np.float64) - 17) * np.float64(np.float32(0.11))
    want = np.clip(np.rint(real / np.float64(np.float32(0.09))) + 3, -128, 127)
    d = np.abs(y.astype(int) - want.astype(int))
    assert d.max() <= 1 and np.count_nonzero(d) < 100  # fp32 steps: only values next to a rounding boundary move


def test_qrelu_is_a_clamp_at_the_zero_point():
    q = np.arange(256, dtype=np.uint8)
    np.testing.assert_array_equal(oracle.qrelu(q, 77), np.maximum(q, 77))
    s = np.arange(-128, 128).astype(np.int8)
    np.testing.assert_array_equal(oracle.qrelu(s, -5), np.maximum(s, -5))


def test_qmaxpool_brute_force_and_global_window():
    rng = np.random.default_rng(12)
    x = rng.integers(0, 256, (2, 6, 7, 3), dtype=np.uint8)
    # a window that covers the whole image is the per-channel maximum
    y = oracle.qmaxpool2d(x, (6, 7), (6, 7), (0, 0))
    np.testing.assert_array_equal(y[:, 0, 0, :], x.max(axis=(1, 2)))
    # 1x1 window, stride 1: identity
    np.testing.assert_array_equal(oracle.qmaxpool2d(x, (1, 1), (1, 1), (0, 0)), x)
    # 2x2 / 2 against a reshape-based maximum
    x2 = x[:, :6, :6, :]
    want = x2.reshape(2, 3, 2, 3, 2, 3).max(axis=(2, 4))
    np.testing.assert_array_equal(oracle.qmaxpool2d(x2, (2, 2), (2, 2), (0, 0)), want)


def test_qcat_with_equal_parameters_is_concatenation():
    rng = np.random.default_rng(13)
    a = rng.integers(0, 256, (2, 3, 4), dtype=np.uint8)
    b = rng.integers(0, 256, (2, 5, 4), dtype=np.uint8)
    np.testing.assert_array_equal(oracle.qcat([a, b], [0.1, 0.1], [7, 7], 1, 0.1, 7), np.concatenate([a, b], 1))
    # scale ratio 2 with zero points 0: codes halve (ties to even)
    y = oracle.qcat([a], [0.25], [0], 0, 0.5, 0)
    np.testing.assert_array_equal(y, np.rint(a / 2.0).astype(np.uint8))


def test_qadaptive_avgpool_identity_constant_and_exact_means():
    rng = np.random.default_rng(77)
    x = rng.integers(0, 256, (2, 6, 5, 9)).astype(np.uint8)
    # output grid = input grid: every window is one pixel
    np.testing.assert_array_equal(oracle.qadaptive_avgpool2d(x, (6, 5), 17), x)
    # a constant image stays constant whatever the windows and the zero point
    k = np.full((1, 7, 9, 3), 201, np.uint8)
    np.testing.assert_array_equal(oracle.qadaptive_avgpool2d(k, (3, 4), 250), np.full((1, 3, 4, 3), 201, np.uint8))
    # 2x2 windows: sums of four codes; exact quarters, ties to even (brute force in integers)
    x2 = rng.integers(-128, 128, (1, 4, 6, 2)).astype(np.int8)
    zp = -3
    s = x2.astype(np.int64).reshape(1, 2, 2, 3, 2, 2).sum(axis=(2, 4)) - 4 * zp
    q, r = np.divmod(s, 4)
    want = q + (r > 2) + ((r == 2) & (q % 2 == 1)) + zp       # round half to even of s / 4
    np.testing.assert_array_equal(oracle.qadaptive_avgpool2d(x2, (2, 3), zp), np.clip(want, -128, 127).astype(np.int8))
    # window bounds: 10 rows -> 3 outputs use rows [0,4) [3,7) [6,10)
    ramp = np.arange(10, dtype=np.uint8).reshape(1, 10, 1, 1) * 10
    np.testing.assert_array_equal(oracle.qadaptive_avgpool2d(ramp, (3, 1), 0).ravel(), [15, 45, 75])


def test_linear_f32_exact_cases():
    rng = np.random.default_rng(31)
    xq = rng.integers(0, 256, (6, 40), dtype=np.uint8)
    wq = rng.integers(-127, 128, (11, 40), dtype=np.int8)
    acc = (xq.astype(np.int64) - 99) @ wq.astype(np.int64).T
    # power-of-two scales, no bias: the result is the integer product, scaled exactly
    y = oracle.linear_f32(xq, 0.5, 99, wq, np.full(11, 0.25), None)
    np.testing.assert_array_equal(y, (acc * 0.125).astype(np.float32))
    # bias and relu: still exact while everything stays representable
    b = (np.arange(11, dtype=np.float32) - 5) * 4096
    y = oracle.linear_f32(xq, 0.5, 99, wq, [0.25], b, relu=True)
    np.testing.assert_array_equal(y, np.maximum(acc * 0.125 + b[None, :].astype(np.float64), 0).astype(np.float32))
    # one rounding, not two: over many accumulators the fused form and
    # multiply-then-add differ somewhere, and the oracle is the fused one
    x1 = rng.integers(0, 256, (200, 64), dtype=np.uint8)
    w1 = rng.integers(-127, 128, (1, 64), dtype=np.int8)
    acc1 = (x1.astype(np.int64) @ w1.astype(np.int64).T).astype(np.float32)
    m = np.float32(np.float32(0.1) * np.float32(0.3))
    b1 = np.float32(0.7431)
    want = (acc1.astype(np.float64) * np.float64(m) + np.float64(b1)).astype(np.float32)
    two_step = ((acc1 * m).astype(np.float32) + b1).astype(np.float32)
    y = oracle.linear_f32(x1, 0.1, 0, w1, [0.3], np.array([b1], np.float32))
    np.testing.assert_array_equal(y, want)
    assert (want != two_step).any()   # the data does tell the two apart


def test_linear_dynamic_matches_float_linear_within_quantization_error():
    rng = np.random.default_rng(32)
    x = rng.standard_normal((20, 64)).astype(np.float32)
    wq = rng.integers(-127, 128, (12, 64), dtype=np.int8)
    ws = np.full(12, 0.01)
    y = oracle.linear_dynamic(x, wq, ws, None)
    ref = x.astype(np.float64) @ (wq.astype(np.float64) * 0.01).T
    step = (x.max() - min(x.min(), 0)) / 255
    # each activation is off by at most half a step
    bound = 0.5 * step * np.abs(wq.astype(np.float64) * 0.01).sum(axis=1)
    assert np.all(np.abs(y - ref) <= bound[None, :] * 1.001 + 1e-4)


def test_qunary_known_values():
    codes = np.arange(256, dtype=np.uint8)
    # sigmoid: the zero point maps to 0.5 = code 128; far negative -> 0, far positive saturates at 255
    y = oracle.qunary(codes, "sigmoid", 0.1, 128, 1 / 256, 0)
    assert y[128] == 128 and y[0] == 0 and y[255] == 255 and np.all(np.diff(y.astype(int)) >= 0)
    # sigmoid(-x) = 1 - sigmoid(x): codes mirror around the zero point (up to the rounding of .5)
    assert np.all(np.abs((y[128 + np.arange(1, 100)].astype(int) + y[128 - np.arange(1, 100)].astype(int)) - 256) <= 1)
    # gelu: 0 at the zero point, identity for large positive, 0 for large negative values
    g = oracle.qunary(codes, "gelu", 0.1, 100, 0.1, 100)
    assert g[100] == 100 and g[255] == 255 and g[0] == 100 and g[160] == 160
    # minimum of gelu is about -0.17 at x = -0.75: one or two steps below the zero point at this scale
    assert g.min() == 98
    # the tanh approximation stays within one step of the erf form
    t = oracle.qunary(codes, "gelu_tanh", 0.1, 100, 0.1, 100)
    assert np.abs(t.astype(int) - g.astype(int)).max() <= 1
