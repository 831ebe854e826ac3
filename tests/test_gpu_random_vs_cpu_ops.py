"""Randomized shapes and options through the operators on the GPU against the
same operators of the installed PyTorch on the CPU (fbgemm engine), bit for bit.

The fixed cases and golden vectors pin chosen shapes; this sweep is what found
the two rounding forms that only show on a few values in a million (the
activation quantization of linear_dynamic, the bias of a per-tensor weight).
Seeds are fixed: the same cases on every run."""
import numpy as np
import pytest
import torch

from gpu_util import say

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _ops():
    import torch_musa_amd  # noqa: F401  (registers the operators)
    if "fbgemm" not in torch.backends.quantized.supported_engines:
        pytest.skip("this PyTorch build has no fbgemm engine")
    old = torch.backends.quantized.engine
    torch.backends.quantized.engine = "fbgemm"
    yield
    torch.backends.quantized.engine = old


def _same_q(got, ref, what):
    assert got.is_cuda and got.shape == ref.shape and got.dtype == ref.dtype, what
    assert got.q_scale() == ref.q_scale() and got.q_zero_point() == ref.q_zero_point(), what
    n = int((got.int_repr().cpu() != ref.int_repr()).sum())
    assert n == 0, f"{what}: {n} of {ref.numel()} codes differ"


def _close_q(got, ref, inp, what):
    """As _same_q, for the two activations of a quantized tensor `inp` that the CPU evaluates in
    float32 vector arithmetic and the GPU once per input code in double precision: the output of
    an input code whose exact value lies next to a rounding boundary may differ by 1 -- for every
    element that holds that code, so the bound is on input codes, not on elements."""
    assert got.is_cuda and got.shape == ref.shape and got.dtype == ref.dtype, what
    assert got.q_scale() == ref.q_scale() and got.q_zero_point() == ref.q_zero_point(), what
    d = (got.int_repr().cpu().int() - ref.int_repr().int()).abs()
    assert int(d.max()) <= 1, f"{what}: a code differs by {int(d.max())}"
    codes = torch.unique(inp.int_repr().cpu()[d != 0])
    assert codes.numel() <= 4, f"{what}: the outputs of {codes.numel()} input codes differ"


@pytest.mark.parametrize("seed", list(range(1, 13)))
def test_linear_ops(seed):
    rng = np.random.default_rng(seed)
    done = 0
    for it in range(40):
        M = int(rng.choice([1, 3, 17, 24, 32, 48, 64, 65, 100, 128, 200, 256, 300, 384, 448, 512, 700, 1024, 1500, 2048]))
        K = int(rng.choice([16, 64, 100, 128, 320, 384, 448, 1024, 1536, 2048, 3072, 4096, 8192, 11008]))
        N = int(rng.choice([1, 16, 33, 64, 100, 256, 300, 512, 1000, 2048, 4096]))
        pc, relu, bias = (bool(rng.integers(2)) for _ in range(3))
        xs = float(rng.uniform(0.5, 3))
        if M * K * N > 2e10:
            continue
        say("random linear", seed, it, (M, K, N), pc, relu, bias)
        torch.manual_seed(1000 * seed + it)
        x, w = torch.randn(M, K) * xs, torch.randn(N, K) * 0.05
        b = torch.randn(N) * 2 if bias else None
        xq = torch.quantize_per_tensor_dynamic(x, torch.quint8, False)
        if pc:
            s = (w.abs().amax(dim=1) / 127).clamp_min(1e-4).double()
            wq = torch.quantize_per_channel(w, s, torch.zeros(N, dtype=torch.int64), 0, torch.qint8)
        else:
            wq = torch.quantize_per_tensor(w, float(w.abs().max() / 127), 0, torch.qint8)
        cpu_packed = torch.ops.quantized.linear_prepack(wq, b)
        gpu_packed = torch.ops.quantized.linear_prepack(wq.cuda(), None if b is None else b.cuda())
        out_scale = max(float((x @ w.t()).std()) / 40, 1e-3) if M * N > 1 else 0.05
        op = torch.ops.quantized.linear_relu if relu else torch.ops.quantized.linear
        _same_q(op(xq.cuda(), gpu_packed, out_scale, 100), op(xq, cpu_packed, out_scale, 100),
                f"linear {(M, K, N)} pc={pc} relu={relu} bias={bias}")
        dyn = torch.ops.quantized.linear_relu_dynamic if relu else torch.ops.quantized.linear_dynamic
        assert torch.equal(dyn(x.cuda(), gpu_packed, False).cpu(), dyn(x, cpu_packed, False)), \
            f"linear_dynamic {(M, K, N)} pc={pc} relu={relu} bias={bias}"
        done += 1
    assert done >= 25


@pytest.mark.parametrize("seed", list(range(1, 7)))
def test_linear_ops_few_rows_many_channels(seed):
    """Decode-sized batches against wide layers: the kernels that stream the weights (a block per 16
    channels, rows resident in LDS as one or two blocks per CU, their float-input forms, tiles over several
    rounds) against PyTorch's CPU ops, static and dynamic."""
    rng = np.random.default_rng(900 + seed)
    for it in range(14):
        M = int(rng.choice([1, 2, 4, 5, 8, 12, 14, 16, 17, 32]))
        K = int(rng.choice([1024, 1040, 2048, 3072, 4096, 8192]))
        N = int(rng.choice([4096, 5120, 8200, 11008, 16400, 33000, 66000]))
        pc, relu, bias = (bool(rng.integers(2)) for _ in range(3))
        if K * N > 1.4e8:
            continue
        say("random decode-sized linear", seed, it, (M, K, N), pc, relu, bias)
        torch.manual_seed(7000 * seed + it)
        x, w = torch.randn(M, K) * float(rng.uniform(0.5, 3)), torch.randn(N, K) * 0.05
        b = torch.randn(N) * 2 if bias else None
        xq = torch.quantize_per_tensor_dynamic(x, torch.quint8, False)
        if pc:
            s = (w.abs().amax(dim=1) / 127).clamp_min(1e-4).double()
            wq = torch.quantize_per_channel(w, s, torch.zeros(N, dtype=torch.int64), 0, torch.qint8)
        else:
            wq = torch.quantize_per_tensor(w, float(w.abs().max() / 127), 0, torch.qint8)
        cpu_packed = torch.ops.quantized.linear_prepack(wq, b)
        gpu_packed = torch.ops.quantized.linear_prepack(wq.cuda(), None if b is None else b.cuda())
        out_scale = max(float((x @ w.t()).std()) / 40, 1e-3)
        op = torch.ops.quantized.linear_relu if relu else torch.ops.quantized.linear
        _same_q(op(xq.cuda(), gpu_packed, out_scale, 100), op(xq, cpu_packed, out_scale, 100),
                f"linear {(M, K, N)} pc={pc} relu={relu} bias={bias}")
        dyn = torch.ops.quantized.linear_relu_dynamic if relu else torch.ops.quantized.linear_dynamic
        assert torch.equal(dyn(x.cuda(), gpu_packed, False).cpu(), dyn(x, cpu_packed, False)), \
            f"linear_dynamic {(M, K, N)} pc={pc} relu={relu} bias={bias}"


@pytest.mark.parametrize("seed", list(range(1, 13)))
def test_conv_and_glue_ops(seed):
    rng = np.random.default_rng(100 + seed)
    done = 0
    for it in range(30):
        B = int(rng.choice([1, 2, 8, 16]))
        H, W = int(rng.choice([7, 14, 19, 28, 56])), int(rng.choice([7, 14, 28, 33, 56]))
        g = int(rng.choice([1, 1, 1, 2, 4]))
        IC, OC = g * int(rng.choice([16, 32, 64, 128])), g * int(rng.choice([8, 16, 64, 96]))
        k, s = int(rng.choice([1, 3, 3, 5])), int(rng.choice([1, 1, 2]))
        p = int(rng.choice([0, k // 2]))
        d = int(rng.choice([1, 1, 1, 2]))
        pc, relu, bias = (bool(rng.integers(2)) for _ in range(3))
        if H + 2 * p < d * (k - 1) + 1 or W + 2 * p < d * (k - 1) + 1:
            continue
        say("random conv", seed, it, (B, H, W, IC, OC, k, s, p, d, g), pc, relu, bias)
        torch.manual_seed(5000 * seed + it)
        x, w = torch.relu(torch.randn(B, IC, H, W)) * 1.5, torch.randn(OC, IC // g, k, k) * 0.05
        b = torch.randn(OC) * 2 if bias else None
        xq = torch.quantize_per_tensor_dynamic(x, torch.quint8, False).contiguous(memory_format=torch.channels_last)
        if pc:
            sc = (w.abs().amax(dim=(1, 2, 3)) / 127).clamp_min(1e-4).double()
            wq = torch.quantize_per_channel(w, sc, torch.zeros(OC, dtype=torch.int64), 0, torch.qint8)
        else:
            wq = torch.quantize_per_tensor(w, float(w.abs().max() / 127), 0, torch.qint8)
        geom = ([s, s], [p, p], [d, d], g)
        cpu_packed = torch.ops.quantized.conv2d_prepack(wq, b, *geom)
        gpu_packed = torch.ops.quantized.conv2d_prepack(wq.cuda(), None if b is None else b.cuda(), *geom)
        out_scale = max(float(torch.nn.functional.conv2d(x, w, b, s, p, d, g).std()) / 40, 1e-3)
        op = torch.ops.quantized.conv2d_relu if relu else torch.ops.quantized.conv2d
        zp = 0 if relu else 110
        ref, got = op(xq, cpu_packed, out_scale, zp), op(xq.cuda(), gpu_packed, out_scale, zp)
        what = f"conv {(B, H, W, IC, OC, k, s, p, d, g)} pc={pc} relu={relu} bias={bias}"
        _same_q(got, ref, what)
        ref2 = torch.ops.quantized.add(ref, ref, out_scale * 1.7, 100)
        got2 = torch.ops.quantized.add(got, got, out_scale * 1.7, 100)
        _same_q(got2, ref2, what + " add")
        if ref.shape[2] >= 3 and ref.shape[3] >= 3:
            _same_q(torch.nn.functional.max_pool2d(got, 3, 2, 1), torch.nn.functional.max_pool2d(ref, 3, 2, 1),
                    what + " max_pool2d")
        _same_q(torch.nn.functional.adaptive_avg_pool2d(got, (1, 1)),
                torch.nn.functional.adaptive_avg_pool2d(ref, (1, 1)), what + " adaptive_avg_pool2d")
        _close_q(torch.nn.functional.gelu(got), torch.nn.functional.gelu(ref), ref, what + " gelu")
        _close_q(torch.sigmoid(got), torch.sigmoid(ref), ref, what + " sigmoid")
        _same_q(torch.ops.quantized.cat([got, got2], 1, out_scale * 1.5, 90),
                torch.ops.quantized.cat([ref, ref2], 1, out_scale * 1.5, 90), what + " cat")
        done += 1
    assert done >= 20
