"""The CPU oracle against golden vectors written by PyTorch's CPU quantized ops
(tests/golden/make_golden.py).  Bit-exact for quantize, dequantize, qparams and
accumulators; the requantised uint8 of linear/conv must also be exact here
because the oracle restates fbgemm's scalar output stage and the fixtures were
produced by its vector one -- a difference would show an order-of-operations
mistake (the two agree on every element of these cases)."""
import numpy as np
import pytest

import cases
import oracle


def _check_crc(golden, key, arr):
    assert int(golden[key]) == cases.crc(arr), (
        f"{key}: rebuilt input differs from the one the fixture was made from "
        "(numpy random stream changed?)")


@pytest.mark.parametrize("c", cases.quantize_per_tensor_cases(), ids=lambda c: c["name"])
def test_quantize_dequantize_per_tensor(golden, c):
    k = "qpt/" + c["name"]
    _check_crc(golden, k + "/x_crc", c["x"])
    q = oracle.quantize_per_tensor(c["x"], c["scale"], c["zp"], c["signed"])
    np.testing.assert_array_equal(q, golden[k + "/q"])
    dq = oracle.dequantize_per_tensor(q, c["scale"], c["zp"])
    assert cases.crc(dq) == int(golden[k + "/dq_crc"])
    if k + "/dq" in golden:
        np.testing.assert_array_equal(dq, golden[k + "/dq"])


def test_choose_qparams_pairs(golden):
    rows = golden["dynq/pairs"]
    assert len(rows) == 2 * len(cases.dynamic_qparams_cases())
    for mn, mx, rr, s, z in rows:
        so, zo = oracle.choose_qparams(np.float32(mn), np.float32(mx), False, bool(rr))
        assert so == s and zo == int(z), (mn, mx, rr, so, s, zo, z)


@pytest.mark.parametrize("c", cases.dynamic_tensor_cases(), ids=lambda c: c["name"])
@pytest.mark.parametrize("rr", [False, True])
def test_quantize_per_tensor_dynamic(golden, c, rr):
    k = f"dyn/{c['name']}/rr{int(rr)}"
    _check_crc(golden, k + "/x_crc", c["x"])
    mn, mx = oracle.minmax(c["x"])
    assert mn == float(c["x"].min()) and mx == float(c["x"].max())
    s, z = oracle.choose_qparams(mn, mx, False, rr)
    assert s == float(golden[k + "/scale"]) and z == int(golden[k + "/zp"])
    q = oracle.quantize_per_tensor(c["x"], s, z, False)
    np.testing.assert_array_equal(q, golden[k + "/q"])


@pytest.mark.parametrize("c", cases.quantize_per_channel_cases(), ids=lambda c: c["name"])
def test_quantize_dequantize_per_channel(golden, c):
    k = "qpc/" + c["name"]
    _check_crc(golden, k + "/x_crc", c["x"])
    q = oracle.quantize_per_channel(c["x"], c["scales"], c["zps"], c["axis"], c["signed"])
    np.testing.assert_array_equal(q, golden[k + "/q"])
    dq = oracle.dequantize_per_channel(q, c["scales"], c["zps"], c["axis"])
    assert cases.crc(dq) == int(golden[k + "/dq_crc"])
    if k + "/dq" in golden:
        np.testing.assert_array_equal(dq, golden[k + "/dq"])


@pytest.mark.parametrize("c", cases.quantize_per_channel_float_cases(), ids=lambda c: c["name"])
def test_quantize_dequantize_per_channel_float_qparams(golden, c):
    k = "qpcf/" + c["name"]
    _check_crc(golden, k + "/x_crc", c["x"])
    q = oracle.quantize_per_channel_float(c["x"], c["scales"], c["zps"], c["axis"], c["signed"])
    np.testing.assert_array_equal(q, golden[k + "/q"])
    dq = oracle.dequantize_per_channel_float(q, c["scales"], c["zps"], c["axis"])
    assert cases.crc(dq) == int(golden[k + "/dq_crc"])
    if k + "/dq" in golden:
        np.testing.assert_array_equal(dq, golden[k + "/dq"])


@pytest.mark.parametrize("c", cases.linear_cases(), ids=lambda c: c["name"])
def test_linear(golden, c):
    k = "lin/" + c["name"]
    _check_crc(golden, k + "/xq_crc", c["xq"])
    _check_crc(golden, k + "/wq_crc", c["wq"])
    assert float(golden[k + "/out_scale"]) == c["out_scale"]
    y = oracle.linear(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"],
                      c["bias"], c["out_scale"], c["out_zp"], relu=c["relu"])
    want = golden[k + "/y"]
    assert 0 < np.count_nonzero((want > 0) & (want < 255)), "degenerate case"
    np.testing.assert_array_equal(y, want)


def test_c1(golden):
    c1 = cases.c1_case()
    _check_crc(golden, "c1/x_crc", c1["x"])
    _check_crc(golden, "c1/w_crc", c1["w"])
    mn, mx = oracle.minmax(c1["x"])
    s, z = oracle.choose_qparams(mn, mx, False, False)
    assert s == float(golden["c1/x_scale"]) and z == int(golden["c1/x_zp"])
    xq = oracle.quantize_per_tensor(c1["x"], s, z, False)
    assert cases.crc(xq) == int(golden["c1/xq_crc"])
    wq = oracle.quantize_per_channel(c1["w"], c1["w_scales"], np.zeros(1024, np.int64), 0, True)
    assert cases.crc(wq) == int(golden["c1/wq_crc"])
    y = oracle.linear(xq, s, z, wq, c1["w_scales"], c1["bias"], c1["out_scale"], c1["out_zp"])
    np.testing.assert_array_equal(y, golden["c1/y"])
    dq = oracle.dequantize_per_tensor(y, c1["out_scale"], c1["out_zp"])
    assert cases.crc(dq) == int(golden["c1/y_dq_crc"])


@pytest.mark.parametrize("c", cases.conv_cases(), ids=lambda c: c["name"])
def test_conv2d(golden, c):
    k = "conv/" + c["name"]
    _check_crc(golden, k + "/xq_crc", c["xq"])
    _check_crc(golden, k + "/wq_crc", c["wq"])
    y = oracle.conv2d(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                      c["stride"], c["padding"], c["dilation"], c["groups"],
                      c["out_scale"], c["out_zp"], relu=c["relu"])
    want = golden[k + "/y"]
    assert y.shape == want.shape
    np.testing.assert_array_equal(y, want)


@pytest.mark.parametrize("c", cases.conv_fused_cases(), ids=lambda c: c["name"])
def test_conv2d_fused_vs_float_pipeline(golden, c):
    """The fused variants are defined by the reference's tests as the float
    pipeline quantize(act(conv(dq x, dq w) + bias + dq accum)) within 1 LSB;
    the golden file holds that pipeline evaluated in float64."""
    k = "convf/" + c["name"]
    _check_crc(golden, k + "/xq_crc", c["xq"])
    _check_crc(golden, k + "/wq_crc", c["wq"])
    y = oracle.conv2d_fused(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                            c["stride"], c["padding"], c["dilation"], c["groups"], c["out_scale"],
                            c["out_zp"], accum=c["accq"], accum_scale=c["acc_scale"],
                            accum_zp=c["acc_zp"], activation=c["activation"], out_signed=c["signed"])
    want = golden[k + "/y"]
    lo, hi = (-128, 127) if c["signed"] else (0, 255)
    assert 0.5 < np.mean((want > lo) & (want < hi)), "degenerate case"
    d = np.abs(y.astype(np.int32) - want.astype(np.int32))
    assert d.max() <= 1
    assert np.count_nonzero(d) <= 0.002 * d.size, f"{np.count_nonzero(d)} of {d.size} differ"


@pytest.mark.parametrize("c", cases.qadd_cases(), ids=lambda c: c["name"])
def test_qadd_and_qrelu(golden, c):
    k = "qadd/" + c["name"]
    _check_crc(golden, k + "/qa_crc", c["qa"])
    _check_crc(golden, k + "/qb_crc", c["qb"])
    y = oracle.qadd(c["qa"], c["a_scale"], c["a_zp"], c["qb"], c["b_scale"], c["b_zp"], c["out_scale"],
                    c["out_zp"], relu=c["relu"])
    # the CPU kernel's scalar tail dequantizes without the fused multiply-add:
    # a handful of values per 100 000 may differ by one
    d = np.abs(y.astype(np.int32) - golden[k + "/y"].astype(np.int32))
    assert d.max() <= 1 and np.count_nonzero(d) <= max(1, d.size // 20000), np.count_nonzero(d)
    np.testing.assert_array_equal(oracle.qrelu(c["qa"], c["a_zp"]), golden[k + "/relu_a"])


@pytest.mark.parametrize("c", cases.qcat_cases(), ids=lambda c: c["name"])
def test_qcat(golden, c):
    k = "qcat/" + c["name"]
    _check_crc(golden, k + "/q0_crc", c["qs"][0])
    y = oracle.qcat(c["qs"], c["scales"], c["zps"], c["axis"], c["out_scale"], c["out_zp"])
    np.testing.assert_array_equal(y, golden[k + "/y"])


@pytest.mark.parametrize("c", cases.qmaxpool_cases(), ids=lambda c: c["name"])
def test_qmaxpool2d(golden, c):
    k = "qmaxpool/" + c["name"]
    _check_crc(golden, k + "/x_crc", c["x"])
    y = oracle.qmaxpool2d(c["x"], c["kernel"], c["stride"], c["padding"], c["dilation"], c["ceil_mode"])
    np.testing.assert_array_equal(y, golden[k + "/y"])


@pytest.mark.parametrize("c", cases.qavgpool_cases(), ids=lambda c: c["name"])
def test_qadaptive_avgpool2d(golden, c):
    k = "qavgpool/" + c["name"]
    assert int(golden[k + "/x_crc"]) == cases.crc(c["x"])
    y = oracle.qadaptive_avgpool2d(c["x"], c["out_hw"], c["zp"])
    np.testing.assert_array_equal(y, golden[k + "/y"])


@pytest.mark.parametrize("c", cases.linear_dynamic_cases(), ids=lambda c: c["name"])
def test_linear_dynamic(golden, c):
    # float results, compared bit for bit: the oracle's single fused multiply-add
    # per value is what the CPU op executes
    k = "lindyn/" + c["name"]
    assert int(golden[k + "/x_crc"]) == cases.crc(c["x"]) and int(golden[k + "/wq_crc"]) == cases.crc(c["wq"])
    y = oracle.linear_dynamic(c["x"], c["wq"], c["w_scales"], c["bias"], c["relu"], c["reduce_range"])
    assert y.dtype == np.float32 and y.shape == golden[k + "/y"].shape
    np.testing.assert_array_equal(y, golden[k + "/y"])


def test_per_tensor_weight_bias_form(golden):
    """Rows picked where float(raw) + fl(bias / atw) and fma(bias, fl(1 / atw), float(raw))
    requantise differently: the CPU op takes the second for a per-tensor weight (the
    oracle follows), the first for per-channel scales."""
    xq, wq, bias = golden["ptbias/xq"], golden["ptbias/wq"], golden["ptbias/bias"]
    x_scale, x_zp, w_scale, out_scale, out_zp = golden["ptbias/params"]
    want = golden["ptbias/y"]
    y = oracle.linear(xq, x_scale, int(x_zp), wq, np.array([w_scale]), bias, out_scale, int(out_zp))
    np.testing.assert_array_equal(y, want)
    # the same weight declared per channel (equal scales) takes the division form: it differs here
    y_pc = oracle.linear(xq, x_scale, int(x_zp), wq, np.full(wq.shape[0], w_scale), bias, out_scale, int(out_zp))
    assert np.count_nonzero(y_pc != want) >= 6


def test_linear_dynamic_pins_the_activation_rounding(golden):
    """On the case built from values where the two forms disagree, only the fused
    form (one rounding of x * inv + zp) reproduces the CPU op; the form of
    quantize_per_tensor does not."""
    c = [c for c in cases.linear_dynamic_cases() if c["name"].startswith("rounding_forms")][0]
    want = golden["lindyn/" + c["name"] + "/y"]
    mn, mx = oracle.minmax(c["x"])
    scale, zp = oracle.choose_qparams(mn, mx, False, False)
    assert (scale, zp) == (17.0 / 255.0, 120)
    fused = oracle.quantize_per_tensor_fused(c["x"], scale, zp)
    plain = oracle.quantize_per_tensor(c["x"], scale, zp)
    assert np.count_nonzero(fused != plain) >= 16
    y_fused = oracle.linear_f32(fused, scale, zp, c["wq"], c["w_scales"], c["bias"])
    y_plain = oracle.linear_f32(plain, scale, zp, c["wq"], c["w_scales"], c["bias"])
    np.testing.assert_array_equal(y_fused, want)
    assert np.count_nonzero(y_plain != want) > 0


def _close_to(y, want, out_dtype, what):
    assert y.shape == want.shape and y.dtype == want.dtype, what
    if out_dtype == "float32":
        np.testing.assert_allclose(y, want, rtol=1e-5, atol=1e-5 * max(1.0, float(np.abs(want).max())), err_msg=what)
    else:
        d = np.abs(y.astype(np.int32) - want.astype(np.int32))
        assert d.max() <= 1, f"{what}: max diff {d.max()}"
        assert np.count_nonzero(d) <= 0.002 * d.size + 1, f"{what}: {np.count_nonzero(d)} of {d.size} differ"


@pytest.mark.parametrize("c", cases.plain_linear_cases(), ids=lambda c: c["name"])
def test_plain_linear(golden, c):
    # golden = PyTorch's oneDNN CPU op, which the reference's tests compare with
    k = "plainlin/" + c["name"]
    assert int(golden[k + "/x_crc"]) == cases.crc(c["x"]) and int(golden[k + "/w_crc"]) == cases.crc(c["w"])
    y = oracle.plain_linear(c["x"], c["x_scale"], c["x_zp"], c["w"], c["w_scale"], c["bias"], c["out_scale"],
                            c["out_zp"], c["out_dtype"], c["post"])
    _close_to(y, golden[k + "/y"], c["out_dtype"], c["name"])
    if c["name"].startswith("ref"):   # small integers, unit scales: exact in any order
        np.testing.assert_array_equal(y, golden[k + "/y"])


@pytest.mark.parametrize("c", cases.plain_conv_cases(), ids=lambda c: c["name"])
def test_plain_conv(golden, c):
    k = "plainconv/" + c["name"]
    assert int(golden[k + "/x_crc"]) == cases.crc(c["x"]) and int(golden[k + "/w_crc"]) == cases.crc(c["w"])
    y = oracle.plain_conv(c["x"], c["x_scale"], c["x_zp"], c["w"], c["w_scale"], c["bias"], c["stride"], c["pad"],
                          c["groups"], c["out_scale"], c["out_zp"], c["out_dtype"], c["relu"], c["accum"],
                          c["accum_scale"], c["accum_zp"])
    _close_to(y, golden[k + "/y"], c["out_dtype"], c["name"])


@pytest.mark.parametrize("kind", ["gelu", "gelu_tanh", "sigmoid"])
@pytest.mark.parametrize("c", cases.qunary_cases(), ids=lambda c: c["name"])
def test_qunary(golden, c, kind):
    # golden = PyTorch's CPU op (float32 vector math); the oracle evaluates the same
    # definition in float64: equal except, at most, where a value sits on a rounding boundary
    k = "qunary/" + c["name"]
    assert int(golden[k + "/x_crc"]) == cases.crc(c["x"])
    out_scale, out_zp = golden[k + "/" + kind + "/qparams"]
    if kind == "sigmoid":
        assert out_scale == 1.0 / 256 and out_zp == (-128 if c["signed"] else 0)
    else:
        assert out_scale == c["scale"] and out_zp == c["zp"]
    y = oracle.qunary(c["x"], kind, c["scale"], c["zp"], out_scale, int(out_zp))
    want = golden[k + "/" + kind + "/y"]
    d = np.abs(y.astype(np.int32) - want.astype(np.int32))
    assert d.max() <= 1 and np.count_nonzero(d) <= 0.001 * d.size + 1
