"""The oracle against the installed PyTorch CPU ops on millions of values.

The golden vectors pin the oracle on small cases; a rounding form that parts
from the CPU op on a few values in a million (as the activation quantization of
quantized::linear_dynamic did) only shows at this size.  CPU only, a few
seconds; the ops run with the fbgemm engine, as the golden vectors were made.
"""
import numpy as np
import pytest
import torch

import oracle


@pytest.fixture(scope="module", autouse=True)
def _engine():
    if "fbgemm" not in torch.backends.quantized.supported_engines:
        pytest.skip("this PyTorch build has no fbgemm engine")
    old = torch.backends.quantized.engine
    torch.backends.quantized.engine = "fbgemm"
    yield
    torch.backends.quantized.engine = old


def _same(a, b, what):
    a, b = np.asarray(a), np.asarray(b)
    assert a.shape == b.shape and a.dtype == b.dtype, what
    n = np.count_nonzero(a != b)
    assert n == 0, f"{what}: {n} of {a.size} values differ"


def _nhwc(q):
    return q.int_repr().permute(0, 2, 3, 1).contiguous().numpy()


@pytest.mark.parametrize("dtype,signed,scale,zp", [(torch.quint8, False, 100 / 255, 128),
                                                   (torch.qint8, True, 0.0472, -3)])
def test_quantize_dequantize_4mi(dtype, signed, scale, zp):
    x = (np.random.default_rng(1).standard_normal(1 << 22) * 3).astype(np.float32)
    q = torch.quantize_per_tensor(torch.from_numpy(x), scale, zp, dtype)
    _same(q.int_repr().numpy(), oracle.quantize_per_tensor(x, scale, zp, signed, nthreads=8), "quantize")
    _same(q.dequantize().numpy().view(np.uint32),
          oracle.dequantize_per_tensor(q.int_repr().numpy(), scale, zp, nthreads=8).view(np.uint32), "dequantize")


@pytest.mark.parametrize("reduce_range", [False, True])
def test_dynamic_quantize_4mi(reduce_range):
    x = (np.random.default_rng(2).standard_normal(1 << 22) * 2.5 + 0.4).astype(np.float32)
    q = torch.quantize_per_tensor_dynamic(torch.from_numpy(x), torch.quint8, reduce_range)
    mn, mx = oracle.minmax(x, nthreads=8)
    scale, zp = oracle.choose_qparams(mn, mx, False, reduce_range)
    assert (q.q_scale(), q.q_zero_point()) == (scale, zp)
    _same(q.int_repr().numpy(), oracle.quantize_per_tensor(x, scale, zp, False, nthreads=8), "dynamic quantize")


def test_per_channel_2mi():
    rng = np.random.default_rng(3)
    x = (rng.standard_normal((16, 512, 256)) * 2).astype(np.float32)
    sc, zc = 0.01 + rng.random(512) * 0.05, rng.integers(-20, 20, 512)
    q = torch.quantize_per_channel(torch.from_numpy(x), torch.from_numpy(sc), torch.from_numpy(zc), 1, torch.qint8)
    _same(q.int_repr().numpy(), oracle.quantize_per_channel(x, sc, zc, 1, True), "quantize_per_channel")
    _same(q.dequantize().numpy().view(np.uint32),
          oracle.dequantize_per_channel(q.int_repr().numpy(), sc, zc, 1).view(np.uint32), "dequantize_per_channel")


def test_linear_and_linear_dynamic_512x4096():
    torch.manual_seed(4)
    M, K, N = 512, 4096, 256
    xf, w, b = torch.randn(M, K), torch.randn(N, K) * 0.02, torch.randn(N)
    xq = torch.quantize_per_tensor_dynamic(xf, torch.quint8, False)
    ws = (w.abs().amax(dim=1) / 127).double()
    wq = torch.quantize_per_channel(w, ws, torch.zeros(N, dtype=torch.int64), 0, torch.qint8)
    packed = torch.ops.quantized.linear_prepack(wq, b)
    wn = wq.int_repr().numpy()
    for relu in (False, True):
        op = torch.ops.quantized.linear_relu if relu else torch.ops.quantized.linear
        y = op(xq, packed, 0.02, 128).int_repr().numpy()
        _same(y, oracle.linear(xq.int_repr().numpy(), xq.q_scale(), xq.q_zero_point(), wn, ws.numpy(), b.numpy(),
                               0.02, 128, relu=relu, nthreads=8), f"linear relu={relu}")
    # 2 Mi activations: a few of them sit where the two rounding forms part
    for rr in (False, True):
        y = torch.ops.quantized.linear_dynamic(xf, packed, rr).numpy()
        _same(y.view(np.uint32), oracle.linear_dynamic(xf.numpy(), wn, ws.numpy(), b.numpy(),
                                                       reduce_range=rr).view(np.uint32), f"linear_dynamic rr={rr}")


def test_per_tensor_weight_with_bias_2mi():
    # 2.8 Mi outputs: a handful of them requantise differently under the per-channel form
    torch.manual_seed(10)
    M, K, N = 700, 448, 4096
    x, w, b = torch.randn(M, K) * 2, torch.randn(N, K) * 0.05, torch.randn(N) * 3
    xq = torch.quantize_per_tensor_dynamic(x, torch.quint8, False)
    wq = torch.quantize_per_tensor(w, float(w.abs().max() / 127), 0, torch.qint8)
    out_scale = float((x @ w.t()).std()) / 40
    y = torch.ops.quantized.linear(xq, torch.ops.quantized.linear_prepack(wq, b), out_scale, 100).int_repr().numpy()
    args = (xq.int_repr().numpy(), xq.q_scale(), xq.q_zero_point(), wq.int_repr().numpy())
    _same(y, oracle.linear(*args, np.array([wq.q_scale()]), b.numpy(), out_scale, 100, nthreads=8), "per-tensor + bias")
    as_pc = oracle.linear(*args, np.full(N, wq.q_scale()), b.numpy(), out_scale, 100, nthreads=8)
    assert np.count_nonzero(as_pc != y) > 0


def test_conv2d_per_tensor_weight_with_bias():
    torch.manual_seed(202)
    x, w, b = torch.relu(torch.randn(16, 64, 28, 28)), torch.randn(96, 64, 3, 3) * 0.05, torch.randn(96) * 3
    xq = torch.quantize_per_tensor_dynamic(x, torch.quint8, False).contiguous(memory_format=torch.channels_last)
    wq = torch.quantize_per_tensor(w, float(w.abs().max() / 127), 0, torch.qint8)
    packed = torch.ops.quantized.conv2d_prepack(wq, b, [1, 1], [1, 1], [1, 1], 1)
    y = torch.ops.quantized.conv2d(xq, packed, 0.05, 100)
    want = oracle.conv2d(_nhwc(xq), xq.q_scale(), xq.q_zero_point(),
                         wq.int_repr().permute(0, 2, 3, 1).contiguous().numpy(), np.array([wq.q_scale()]), b.numpy(),
                         (1, 1), (1, 1), (1, 1), 1, 0.05, 100, nthreads=8)
    _same(_nhwc(y), want, "conv2d per-tensor + bias")


@pytest.mark.parametrize("geom", [(8, 64, 28, 64, 3, 1, 1, 1), (4, 32, 32, 64, 3, 2, 1, 4), (2, 3, 96, 32, 7, 2, 3, 1)])
def test_conv2d(geom):
    B, C, H, OC, k, s, p, g = geom
    torch.manual_seed(5)
    x, w, b = torch.relu(torch.randn(B, C, H, H)), torch.randn(OC, C // g, k, k) * 0.05, torch.randn(OC)
    xq = torch.quantize_per_tensor_dynamic(x, torch.quint8, False).contiguous(memory_format=torch.channels_last)
    ws = (w.abs().amax(dim=(1, 2, 3)) / 127).double()
    wq = torch.quantize_per_channel(w, ws, torch.zeros(OC, dtype=torch.int64), 0, torch.qint8)
    packed = torch.ops.quantized.conv2d_prepack(wq, b, [s, s], [p, p], [1, 1], g)
    for relu in (False, True):
        op = torch.ops.quantized.conv2d_relu if relu else torch.ops.quantized.conv2d
        y = op(xq, packed, 0.05, 3 if relu else 100)
        want = oracle.conv2d(_nhwc(xq), xq.q_scale(), xq.q_zero_point(),
                             wq.int_repr().permute(0, 2, 3, 1).contiguous().numpy(), ws.numpy(), b.numpy(),
                             (s, s), (p, p), (1, 1), g, 0.05, 3 if relu else 100, relu=relu, nthreads=8)
        _same(_nhwc(y), want, f"conv2d relu={relu}")


def test_elementwise_1mi():
    torch.manual_seed(6)
    a = torch.quantize_per_tensor(torch.randn(1 << 20) * 2, 0.03, 120, torch.quint8)
    b = torch.quantize_per_tensor(torch.randn(1 << 20) * 3, 0.05, 100, torch.quint8)
    an, bn = a.int_repr().numpy(), b.int_repr().numpy()
    for relu in (False, True):
        op = torch.ops.quantized.add_relu if relu else torch.ops.quantized.add
        _same(op(a, b, 0.06, 110).int_repr().numpy(), oracle.qadd(an, 0.03, 120, bn, 0.05, 100, 0.06, 110, relu=relu),
              f"add relu={relu}")
    for kind, fn in (("gelu", torch.nn.functional.gelu),
                     ("gelu_tanh", lambda t: torch.nn.functional.gelu(t, approximate="tanh")),
                     ("sigmoid", torch.sigmoid)):
        y = fn(a)
        _same(y.int_repr().numpy(), oracle.qunary(an, kind, 0.03, 120, y.q_scale(), y.q_zero_point()), kind)
    x4 = torch.quantize_per_tensor(torch.randn(4, 64, 56, 56), 0.03, 120, torch.quint8).contiguous(
        memory_format=torch.channels_last)
    for out in ((7, 7), (1, 1), (5, 3)):
        y = torch.nn.functional.adaptive_avg_pool2d(x4, out)
        _same(_nhwc(y), oracle.qadaptive_avgpool2d(_nhwc(x4), out, 120), f"adaptive_avg_pool2d {out}")
    _same(_nhwc(torch.nn.functional.max_pool2d(x4, 3, 2, 1)), oracle.qmaxpool2d(_nhwc(x4), (3, 3), (2, 2), (1, 1)),
          "max_pool2d")
