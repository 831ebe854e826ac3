"""GPU parity of the affine quantizer kernels, through the C ABI, against the
CPU oracle and the golden vectors.  Everything here is bit-exact."""
import numpy as np
import pytest
import torch

import cases
import oracle
from gpu_util import dev, host, say

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def cabi():
    from torch_musa_amd import cabi as m
    assert torch.cuda.is_available()
    m.lib()
    return m


@pytest.mark.parametrize("c", cases.quantize_per_tensor_cases(), ids=lambda c: c["name"])
def test_quantize_dequantize_per_tensor(cabi, golden, c):
    say("qpt", c["name"])
    x = dev(c["x"].reshape(-1))
    q = cabi.quantize_per_tensor(x, c["scale"], c["zp"], c["signed"])
    want = oracle.quantize_per_tensor(c["x"], c["scale"], c["zp"], c["signed"]).reshape(-1)
    np.testing.assert_array_equal(host(q), want)
    np.testing.assert_array_equal(host(q).view(np.uint8), golden["qpt/" + c["name"] + "/q"].reshape(-1).view(np.uint8))
    r = cabi.dequantize_per_tensor(q, c["scale"], c["zp"])
    np.testing.assert_array_equal(host(r), oracle.dequantize_per_tensor(want, c["scale"], c["zp"]))
    assert cases.crc(host(r)) == int(golden["qpt/" + c["name"] + "/dq_crc"])


@pytest.mark.parametrize("offset", [1, 2, 3])
@pytest.mark.parametrize("n", [1, 5, 17, 1000, 4099])
def test_unaligned_pointers(cabi, offset, n):
    say("unaligned", offset, n)
    x_full = cases.randn(5000 + n, (n + offset,), std=3.0)
    xd = dev(x_full)[offset:]              # x is 4-byte but not 16-byte aligned
    qbuf = torch.zeros(n + offset + 8, dtype=torch.uint8, device="cuda")
    qv = qbuf[offset:offset + n]           # q is not 4-byte aligned
    cabi.quantize_per_tensor_into(xd, qv, 0.05, 100, False)
    want = oracle.quantize_per_tensor(x_full[offset:], 0.05, 100, False)
    np.testing.assert_array_equal(host(qv), want)
    assert int(qbuf[:offset].sum()) == 0 and int(qbuf[offset + n:].sum()) == 0  # no stray writes
    rbuf = torch.zeros(n + offset + 8, dtype=torch.float32, device="cuda")
    rv = rbuf[offset:offset + n]
    cabi.dequantize_per_tensor_into(qv, rv, 0.05, 100)
    np.testing.assert_array_equal(host(rv), oracle.dequantize_per_tensor(want, 0.05, 100))
    assert float(rbuf[:offset].abs().sum()) == 0 and float(rbuf[offset + n:].abs().sum()) == 0


def test_empty_and_bad_arguments(cabi):
    x = torch.empty(0, dtype=torch.float32, device="cuda")
    assert cabi.quantize_per_tensor(x, 0.1, 0, False).numel() == 0
    x = torch.zeros(4, dtype=torch.float32, device="cuda")
    with pytest.raises(cabi.TmqError):
        cabi.quantize_per_tensor(x, 0.1, 256, False)     # zero point outside quint8
    with pytest.raises(cabi.TmqError):
        cabi.quantize_per_tensor(x, 0.1, -129, True)


@pytest.mark.parametrize("n", [0, 1, 3, 4, 5, 63, 1024, 2049, 8191, 70001, 2 ** 22 + 3])
@pytest.mark.parametrize("offset", [0, 1])
def test_minmax(cabi, n, offset):
    say("minmax", n, offset)
    x = cases.randn(600 + n % 97, (n + offset,), std=2.0)
    got = host(cabi.minmax(dev(x)[offset:]))
    if n == 0:
        assert got[0] == np.inf and got[1] == -np.inf
    else:
        assert got[0] == x[offset:].min() and got[1] == x[offset:].max()


@pytest.mark.parametrize("c", cases.dynamic_tensor_cases(), ids=lambda c: c["name"])
@pytest.mark.parametrize("rr", [False, True])
def test_dynamic_chain_on_device(cabi, golden, c, rr):
    """min/max -> qparams -> quantize without leaving the device."""
    say("dyn", c["name"], rr)
    k = f"dyn/{c['name']}/rr{int(rr)}"
    x = dev(c["x"].reshape(-1))
    mm = cabi.minmax(x)
    qp = cabi.choose_qparams_dev(mm, False, rr)
    q = cabi.quantize_per_tensor_dev(x, qp, False)
    s, z = cabi.read_qparams(qp)
    assert s == float(golden[k + "/scale"]) and z == int(golden[k + "/zp"])
    np.testing.assert_array_equal(host(q), golden[k + "/q"].reshape(-1))


def test_choose_qparams_dev_matches_oracle(cabi):
    for mn, mx in cases.dynamic_qparams_cases():
        for rr in (False, True):
            for signed in (False, True):
                mm = dev(np.array([mn, mx], dtype=np.float32))
                got = cabi.read_qparams(cabi.choose_qparams_dev(mm, signed, rr))
                assert got == oracle.choose_qparams(mn, mx, signed, rr), (mn, mx, rr, signed)


@pytest.mark.parametrize("c", cases.quantize_per_channel_cases(), ids=lambda c: c["name"])
def test_quantize_dequantize_per_channel(cabi, golden, c):
    say("qpc", c["name"])
    k = "qpc/" + c["name"]
    x = dev(c["x"])
    scales = dev(c["scales"].astype(np.float64))
    zps = dev(c["zps"].astype(np.int64))
    q = cabi.quantize_per_channel(x, scales, zps, c["axis"], c["signed"])
    np.testing.assert_array_equal(host(q), golden[k + "/q"])
    r = cabi.dequantize_per_channel(q, scales, zps, c["axis"])
    want = oracle.dequantize_per_channel(golden[k + "/q"], c["scales"], c["zps"], c["axis"])
    np.testing.assert_array_equal(host(r), want)
    assert cases.crc(host(r)) == int(golden[k + "/dq_crc"])


@pytest.mark.parametrize("c", cases.quantize_per_channel_float_cases(), ids=lambda c: c["name"])
def test_quantize_dequantize_per_channel_float_qparams(cabi, golden, c):
    say("qpcf", c["name"])
    k = "qpcf/" + c["name"]
    scales, zps = dev(c["scales"]), dev(c["zps"])
    q = cabi.quantize_per_channel_float_qparams(dev(c["x"]), scales, zps, c["axis"], c["signed"])
    np.testing.assert_array_equal(host(q), golden[k + "/q"])
    np.testing.assert_array_equal(
        host(q), oracle.quantize_per_channel_float(c["x"], c["scales"], c["zps"], c["axis"], c["signed"]))
    r = cabi.dequantize_per_channel_float_qparams(q, scales, zps, c["axis"])
    want = oracle.dequantize_per_channel_float(golden[k + "/q"], c["scales"], c["zps"], c["axis"])
    np.testing.assert_array_equal(host(r), want)
    assert cases.crc(host(r)) == int(golden[k + "/dq_crc"])


def test_per_channel_float_qparams_embedding_sized(cabi):
    """[rows, dim] table quantized row-wise, unaligned inner size (scalar path)
    and an aligned one (vector path)."""
    for rows, dim in ((1000, 130), (257, 64)):
        say("qpcf table", rows, dim)
        w = cases.randn(33 + dim, (rows, dim))
        mn, mx = w.min(axis=1), w.max(axis=1)
        s = ((mx - mn) / 255.0).astype(np.float32)
        z = (-mn / s).astype(np.float32)
        q = cabi.quantize_per_channel_float_qparams(dev(w), dev(s), dev(z), 0, False)
        want = oracle.quantize_per_channel_float(w, s, z, 0, False)
        np.testing.assert_array_equal(host(q), want)
        r = cabi.dequantize_per_channel_float_qparams(q, dev(s), dev(z), 0)
        np.testing.assert_array_equal(host(r), oracle.dequantize_per_channel_float(want, s, z, 0))


def test_per_channel_weight_sized(cabi):
    """[N,K] weight, axis 0, the shape quantized::linear weights come in."""
    say("qpc weight 1000x4096")
    w = cases.randn(31, (1000, 4096), std=0.02)
    s = (np.abs(w).max(axis=1) / 127.0).astype(np.float64)
    z = np.zeros(1000, np.int64)
    q = cabi.quantize_per_channel(dev(w), dev(s), dev(z), 0, True)
    np.testing.assert_array_equal(host(q), oracle.quantize_per_channel(w, s, z, 0, True))


@pytest.mark.parametrize("shape,axis", [
    ((3, 5, 64), 1),        # shortest rows of the row kernel, channel index wraps inside a block
    ((2, 3, 1024), 1),      # one run per row, 8 rows per block, 6 rows in all
    ((7, 4096), 0),         # four accesses per row, two rows per block, odd row count
    ((3, 2, 9000), 1),      # two segments per row, ragged end
    ((5, 301), 0),          # rows that are not a multiple of 4: scalar accesses
    ((2, 2, 1500, 2), 1),   # inner = 3000 from two trailing axes
    ((1, 70000), 0),        # nine segments of 8192
], ids=str)
def test_per_channel_row_kernel_shapes(cabi, shape, axis):
    """Rows of 64 elements and more take the kernel that derives the channel from
    the block index: every decomposition (runs per row, rows per block, segments,
    ragged ends, scalar accesses), both parameter kinds, both directions."""
    say("qpc rows", shape, axis)
    rng = np.random.default_rng(sum(shape) + axis)
    C = shape[axis]
    x = cases.randn(500 + sum(shape), shape)
    for signed in (False, True):
        s = rng.uniform(0.005, 0.05, C).astype(np.float64)
        z = rng.integers(-128 if signed else 0, 128 if signed else 256, C).astype(np.int64)
        q = cabi.quantize_per_channel(dev(x), dev(s), dev(z), axis, signed)
        want = oracle.quantize_per_channel(x, s, z, axis, signed)
        np.testing.assert_array_equal(host(q), want)
        r = cabi.dequantize_per_channel(q, dev(s), dev(z), axis)
        np.testing.assert_array_equal(host(r), oracle.dequantize_per_channel(want, s, z, axis))
        sf = s.astype(np.float32)
        zf = (z + rng.uniform(-0.4, 0.4, C)).astype(np.float32)
        q = cabi.quantize_per_channel_float_qparams(dev(x), dev(sf), dev(zf), axis, signed)
        want = oracle.quantize_per_channel_float(x, sf, zf, axis, signed)
        np.testing.assert_array_equal(host(q), want)
        r = cabi.dequantize_per_channel_float_qparams(q, dev(sf), dev(zf), axis)
        np.testing.assert_array_equal(host(r), oracle.dequantize_per_channel_float(want, sf, zf, axis))


def test_full_size_properties(cabi):
    """benchmark configuration 2 at full size (2**28 fp32): properties that need no
    full-size oracle run, plus oracle parity on sampled windows."""
    n = 2 ** 28
    say("C2 full size", n)
    g = torch.Generator(device="cuda").manual_seed(7)
    x = torch.randn(n, device="cuda", generator=g) * 3.0
    x[::100] = 50.0
    x[37::100] = -50.0
    mm = host(cabi.minmax(x))
    assert mm[0] == -50.0 and mm[1] == 50.0
    s, z = oracle.choose_qparams(mm[0], mm[1], False, False)
    q = cabi.quantize_per_tensor(x, s, z, False)
    r = cabi.dequantize_per_tensor(q, s, z)
    # round trip error is at most half a step (everything is inside the range)
    err = (r - x).abs().max().item()
    assert err <= 0.5 * np.float32(s) * (1 + 1e-5), err
    # idempotence: dequantized values are fixed points
    q2 = cabi.quantize_per_tensor(r, s, z, False)
    assert torch.equal(q, q2)
    # device-side chain gives the same bytes
    qp = cabi.choose_qparams_dev(cabi.minmax(x), False, False)
    assert cabi.read_qparams(qp) == (s, z)
    assert torch.equal(cabi.quantize_per_tensor_dev(x, qp, False), q)
    # oracle parity on windows, including the very end of the buffer
    for start in (0, 123_456_789 // 4 * 4 + 1, n - 2 ** 20):
        xs = host(x[start:start + 2 ** 20])
        np.testing.assert_array_equal(host(q[start:start + 2 ** 20]),
                                      oracle.quantize_per_tensor(xs, s, z, False))
        np.testing.assert_array_equal(host(r[start:start + 2 ** 20]),
                                      oracle.dequantize_per_tensor(host(q[start:start + 2 ** 20]), s, z))


# ---------------------------------------------------------------------------
# quantized::add / add_relu, relu
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("c", cases.qadd_cases(), ids=lambda c: c["name"])
def test_qadd_qrelu(cabi, golden, c):
    say("qadd", c["name"])
    k = "qadd/" + c["name"]
    qa, qb = dev(c["qa"]), dev(c["qb"])
    y = host(cabi.qadd(qa, c["a_scale"], c["a_zp"], qb, c["b_scale"], c["b_zp"], c["out_scale"],
                       c["out_zp"], relu=c["relu"]))
    want = oracle.qadd(c["qa"], c["a_scale"], c["a_zp"], c["qb"], c["b_scale"], c["b_zp"], c["out_scale"],
                       c["out_zp"], relu=c["relu"])
    np.testing.assert_array_equal(y, want)
    d = np.abs(y.astype(np.int32) - golden[k + "/y"].astype(np.int32))
    assert d.max() <= 1 and np.count_nonzero(d) <= max(1, d.size // 20000)
    np.testing.assert_array_equal(host(cabi.qrelu(qa, c["a_zp"])), golden[k + "/relu_a"])


def test_qadd_unaligned_and_large(cabi):
    """Scalar path (operands off a 16-byte boundary) and a 64 Mi element add."""
    say("qadd unaligned")
    rng = np.random.default_rng(77)
    a = rng.integers(0, 256, 100003, dtype=np.uint8)
    b = rng.integers(0, 256, 100003, dtype=np.uint8)
    da, db = dev(a), dev(b)
    y = torch.empty(100003, dtype=torch.uint8, device="cuda")
    got = host(cabi.qadd(da[1:], 0.05, 128, db[1:], 0.03, 100, 0.06, 120, relu=True, out=y[1:]))
    np.testing.assert_array_equal(got, oracle.qadd(a[1:], 0.05, 128, b[1:], 0.03, 100, 0.06, 120, relu=True))
    say("qadd 2**26")
    n = 2 ** 26
    g = torch.Generator(device="cuda").manual_seed(3)
    ta = torch.randint(0, 256, (n,), dtype=torch.uint8, device="cuda", generator=g)
    tb = torch.randint(0, 256, (n,), dtype=torch.uint8, device="cuda", generator=g)
    ty = cabi.qadd(ta, 0.05, 128, tb, 0.03, 100, 0.06, 120)
    for lo in (0, n // 2 - 5000, n - 10000):
        sl = slice(lo, lo + 10000)
        np.testing.assert_array_equal(host(ty[sl]), oracle.qadd(host(ta[sl]), 0.05, 128, host(tb[sl]), 0.03, 100, 0.06, 120))
    # commutes when the operands' quantization parameters are swapped too
    tz = cabi.qadd(tb, 0.03, 100, ta, 0.05, 128, 0.06, 120)
    assert torch.equal(ty, tz)


# ---------------------------------------------------------------------------
# quantized::cat, quantized max pooling
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("c", cases.qcat_cases(), ids=lambda c: c["name"])
def test_qcat(cabi, golden, c):
    say("qcat", c["name"])
    y = host(cabi.qcat([dev(q) for q in c["qs"]], c["scales"], c["zps"], c["axis"], c["out_scale"], c["out_zp"]))
    np.testing.assert_array_equal(y, golden["qcat/" + c["name"] + "/y"])
    np.testing.assert_array_equal(y, oracle.qcat(c["qs"], c["scales"], c["zps"], c["axis"], c["out_scale"], c["out_zp"]))


@pytest.mark.parametrize("c", cases.qmaxpool_cases(), ids=lambda c: c["name"])
def test_qmaxpool2d(cabi, golden, c):
    say("qmaxpool", c["name"])
    want = golden["qmaxpool/" + c["name"] + "/y"]
    y = host(cabi.qmaxpool2d(dev(c["x"]), c["kernel"], c["stride"], c["padding"], c["dilation"], want.shape[1:3]))
    np.testing.assert_array_equal(y, want)


@pytest.mark.parametrize("signed", [False, True])
@pytest.mark.parametrize("geom", [((3, 17, 19, 32), (2, 2), (1, 1)), ((2, 9, 30, 16), (1, 1), (1, 1)),
                                  ((1, 12, 12, 48), (2, 1), (0, 1)), ((2, 8, 8, 16), (3, 3), (1, 0)),
                                  ((1, 3, 3, 16), (1, 1), (1, 1))])
def test_qmaxpool_3x3_sixteen_channel_kernels(cabi, signed, geom):
    """The 3 x 3 kernels that take 16 channels per thread compare bytes as 16-bit lanes:
    extreme codes, runs of equal codes and both code types against the oracle."""
    shape, stride, padding = geom
    say("qmaxpool 3x3 x16", shape, stride, padding, signed)
    rng = np.random.default_rng(hash((shape, stride, padding, signed)) % (1 << 31))
    lo, hi = (-128, 128) if signed else (0, 256)
    x = rng.integers(lo, hi, shape).astype(np.int8 if signed else np.uint8)
    x[rng.random(shape) < 0.2] = lo                       # many taps at the lowest code
    x[rng.random(shape) < 0.1] = hi - 1
    x[0, : shape[1] // 2] = np.where(rng.random((shape[1] // 2,) + shape[2:]) < 0.5, -1 if signed else 127, 0 if signed else 128)
    want = oracle.qmaxpool2d(x, (3, 3), stride, padding)
    y = host(cabi.qmaxpool2d(dev(x), (3, 3), stride, padding, (1, 1), want.shape[1:3]))
    np.testing.assert_array_equal(y, want)


def test_qmaxpool_resnet_stem_sized(cabi):
    """[32,112,112,64] -> 3x3 / 2, pad 1: the pooling after a ResNet stem."""
    say("qmaxpool stem")
    rng = np.random.default_rng(91)
    x = rng.integers(0, 256, (32, 112, 112, 64), dtype=np.uint8)
    y = host(cabi.qmaxpool2d(dev(x), (3, 3), (2, 2), (1, 1), (1, 1), (56, 56)))
    # separable maximum in numpy: rows then columns over the padded image
    xp = np.pad(x, ((0, 0), (1, 1), (1, 1), (0, 0)))
    r = np.maximum(np.maximum(xp[:, 0:-2:2], xp[:, 1:-1:2]), xp[:, 2::2])
    want = np.maximum(np.maximum(r[:, :, 0:-2:2], r[:, :, 1:-1:2]), r[:, :, 2::2])
    np.testing.assert_array_equal(y, want[:, :56, :56])


@pytest.mark.parametrize("c", cases.qavgpool_cases(), ids=lambda c: c["name"])
def test_qadaptive_avgpool2d(cabi, golden, c):
    say("qavgpool", c["name"])
    want = golden["qavgpool/" + c["name"] + "/y"]
    y = host(cabi.qadaptive_avgpool2d(dev(c["x"]), c["out_hw"], c["zp"]))
    np.testing.assert_array_equal(y, want)
    np.testing.assert_array_equal(y, oracle.qadaptive_avgpool2d(c["x"], c["out_hw"], c["zp"]))


def test_qadaptive_avgpool_resnet_head_sized(cabi):
    # [64, 7, 7, 2048] -> [64, 1, 1, 2048]: bit-exact against the oracle
    say("qavgpool head")
    x = np.random.default_rng(5).integers(0, 256, (64, 7, 7, 2048)).astype(np.uint8)
    y = host(cabi.qadaptive_avgpool2d(dev(x), (1, 1), 128))
    np.testing.assert_array_equal(y, oracle.qadaptive_avgpool2d(x, (1, 1), 128))


@pytest.mark.parametrize("n,offset", [(1, 0), (7, 0), (4096, 0), (4099, 1), (32768, 0), (32769, 0), (32772, 0), (65541, 3),
                                      (1 << 20, 0), ((1 << 20) + 3, 1), ((1 << 23) + 1029, 0), ((1 << 25) + 4, 0)])
@pytest.mark.parametrize("signed,reduce_range", [(False, False), (False, True), (True, False)])
def test_quantize_dynamic_on_device(cabi, n, offset, signed, reduce_range):
    # one call: range, parameters (left in device memory) and codes; small inputs take the
    # single-block kernel, aligned ones of up to 2**25 elements two launches (the quantizer's
    # blocks finish the reduction; 2**23 + 1029 walks its grid-stride loop more than once and
    # ends inside a chunk), larger or unaligned ones the three-launch chain -- same results
    say("dynamic dev", n, offset, signed, reduce_range)
    rng = np.random.default_rng(n + offset)
    x = (rng.standard_normal(n + offset) * 2.5 + 0.4).astype(np.float32)
    xd = dev(x)[offset:]
    q, qp = cabi.quantize_per_tensor_dynamic_dev(xd.contiguous() if offset == 0 else xd, signed, reduce_range)
    mn, mx = oracle.minmax(x[offset:], nthreads=8)
    scale, zp = oracle.choose_qparams(mn, mx, signed, reduce_range)
    assert cabi.read_qparams(qp) == (scale, zp)
    np.testing.assert_array_equal(host(q), oracle.quantize_per_tensor(x[offset:], scale, zp, signed, nthreads=8))


@pytest.mark.parametrize("n,offset", [(4099, 1), (32768, 0), (32772, 0), ((1 << 22) + 3, 0), ((1 << 23) + 1029, 0)])
@pytest.mark.parametrize("signed", [False, True])
def test_quantize_dynamic_fused_rounding(cabi, n, offset, signed):
    # the activation quantization of the CPU quantized::linear_dynamic: x * inv + zp
    # rounded once; at 4 Mi elements a few dozen codes differ from the two-step form
    say("dynamic dev fused", n, offset, signed)
    rng = np.random.default_rng(77 + n)
    x = (rng.standard_normal(n + offset) * 2.5 + 0.4).astype(np.float32)
    xd = dev(x)[offset:]
    q, qp = cabi.quantize_per_tensor_dynamic_dev(xd.contiguous() if offset == 0 else xd, signed, False, fused=True)
    mn, mx = oracle.minmax(x[offset:])
    scale, zp = oracle.choose_qparams(mn, mx, signed, False)
    assert cabi.read_qparams(qp) == (scale, zp)
    want = oracle.quantize_per_tensor_fused(x[offset:], scale, zp, signed, nthreads=8)
    np.testing.assert_array_equal(host(q), want)
    if n > (1 << 22) and not signed:   # (with a zero point near 0 the two forms rarely part)
        assert np.count_nonzero(want != oracle.quantize_per_tensor(x[offset:], scale, zp, signed, nthreads=8)) > 0


@pytest.mark.parametrize("kind", ["gelu", "gelu_tanh", "sigmoid"])
@pytest.mark.parametrize("c", cases.qunary_cases(), ids=lambda c: c["name"])
def test_qunary(cabi, golden, c, kind):
    say("qunary", kind, c["name"])
    out_scale, out_zp = golden["qunary/" + c["name"] + "/" + kind + "/qparams"]
    y = host(cabi.qunary(dev(c["x"]), kind, c["scale"], c["zp"], float(out_scale), int(out_zp)))
    # the table is computed in double precision on the device: equal to the float64 oracle
    np.testing.assert_array_equal(y, oracle.qunary(c["x"], kind, c["scale"], c["zp"], out_scale, int(out_zp)))
    d = np.abs(y.astype(np.int32) - golden["qunary/" + c["name"] + "/" + kind + "/y"].astype(np.int32))
    assert d.max() <= 1 and np.count_nonzero(d) <= 0.001 * d.size + 1


def test_qunary_unaligned_and_large(cabi):
    say("qunary unaligned / large")
    x = np.random.default_rng(9).integers(0, 256, (1 << 22) + 5).astype(np.uint8)
    xd = dev(x)
    y = host(cabi.qunary(xd[3:], "gelu", 0.05, 120, 0.05, 120))     # misaligned view
    np.testing.assert_array_equal(y, oracle.qunary(x[3:], "gelu", 0.05, 120, 0.05, 120))
    y = host(cabi.qunary(xd, "sigmoid", 0.05, 120, 1 / 256, 0))
    np.testing.assert_array_equal(y, oracle.qunary(x, "sigmoid", 0.05, 120, 1 / 256, 0))


def test_qunary_several_sweeps_of_the_grid(cabi):
    # more 16-byte groups than the largest grid has threads (4096 blocks), a partial last sweep
    # and a few stray bytes: every thread walks the array several times.  The output is a
    # function of the code alone, so the oracle's 256 answers check all of it.
    say("qunary several sweeps of the grid")
    import torch
    n = 2048 * 16384 * 2 + 16 * 700 + 7
    g = torch.Generator(device="cuda").manual_seed(5)
    xd = torch.randint(0, 256, (n,), dtype=torch.uint8, device="cuda", generator=g)
    codes = np.arange(256, dtype=np.uint8)
    for kind, (os_, oz) in (("gelu", (0.05, 120)), ("sigmoid", (1 / 256, 0))):
        table = torch.from_numpy(oracle.qunary(codes, kind, 0.05, 120, os_, oz)).cuda()
        y = cabi.qunary(xd, kind, 0.05, 120, os_, oz)
        assert torch.equal(y, table[xd.long()])
        xs = xd.view(torch.int8)
        table_s = torch.from_numpy(oracle.qunary(codes.view(np.int8), kind, 0.05, -8, os_, oz - 128)).cuda()
        ys = cabi.qunary(xs, kind, 0.05, -8, os_, oz - 128)
        assert torch.equal(ys.view(torch.uint8), table_s.view(torch.uint8)[xd.long()])
