"""The operator-level drop-in: torch.quantize_per_*, Tensor.dequantize and
torch.ops.quantized.{linear,conv2d}* on GPU tensors, written the way the
reference's own tests are (tests/unittest/quantized/test_quantized_ops.py:25-99,
test_quantized_linear.py:52-111, test_quantized_conv.py:83-150: run on CPU, run
on the device, compare int_repr / dequantize / qparams), plus the CPU-op
semantics the reference's device path does not have (quint8 activations with a
zero point, per-channel weights)."""
import numpy as np
import pytest
import torch
import torch.ao.nn.intrinsic.quantized as nniq
import torch.ao.nn.quantized as nnq

import cases
import oracle
from gpu_util import say

pytestmark = pytest.mark.gpu

LSB_TOL = 1


@pytest.fixture(scope="module", autouse=True)
def tmq():
    import torch_musa_amd
    assert torch.cuda.is_available() and torch_musa_amd.is_loaded()
    torch.backends.quantized.engine = "fbgemm"
    return torch_musa_amd


def assert_q_equal(q_gpu, q_cpu, abs_diff=0):
    """QuantizedComparator of the reference (base_test_tool.py:233-289)."""
    assert q_gpu.is_cuda and q_gpu.dtype == q_cpu.dtype and q_gpu.shape == q_cpu.shape
    assert q_gpu.qscheme() == q_cpu.qscheme()
    if q_cpu.qscheme() in (torch.per_tensor_affine, torch.per_tensor_symmetric):
        assert q_gpu.q_scale() == q_cpu.q_scale() and q_gpu.q_zero_point() == q_cpu.q_zero_point()
    else:
        assert torch.equal(q_gpu.q_per_channel_scales().cpu(), q_cpu.q_per_channel_scales())
        assert torch.equal(q_gpu.q_per_channel_zero_points().cpu(), q_cpu.q_per_channel_zero_points())
        assert q_gpu.q_per_channel_axis() == q_cpu.q_per_channel_axis()
    d = (q_gpu.int_repr().cpu().to(torch.int32) - q_cpu.int_repr().to(torch.int32)).abs().max().item() \
        if q_cpu.numel() else 0
    assert d <= abs_diff, f"int_repr differs by {d}"
    if abs_diff == 0:
        assert torch.equal(q_gpu.dequantize().cpu(), q_cpu.dequantize())


@pytest.mark.parametrize("shape", [(2, 3, 4), (2, 3, 4, 5), (2, 16, 32, 32), (0, 4), (7,)])
@pytest.mark.parametrize("dtype", [torch.quint8, torch.qint8])
def test_quantize_per_tensor(shape, dtype):
    say("aten qpt", shape, dtype)
    torch.manual_seed(41)
    x = torch.randn(shape)
    scale = float(x.abs().max() / 2 ** 7) if x.numel() else 0.1
    zp = 0 if dtype == torch.qint8 else 128
    assert_q_equal(torch.quantize_per_tensor(x.cuda(), scale, zp, dtype),
                   torch.quantize_per_tensor(x, scale, zp, dtype))


@pytest.mark.parametrize("shape", [(2, 3, 4), (2, 3, 4, 5), (2, 16, 32, 32)])
@pytest.mark.parametrize("reduce_range", [True, False])
@pytest.mark.parametrize("dtype", [torch.quint8, torch.qint8])
def test_quantize_per_tensor_dynamic(shape, reduce_range, dtype):
    say("aten dyn", shape, reduce_range, dtype)
    torch.manual_seed(42)
    x = torch.randn(shape) * 3
    assert_q_equal(torch.quantize_per_tensor_dynamic(x.cuda(), dtype, reduce_range),
                   torch.quantize_per_tensor_dynamic(x, dtype, reduce_range))


def test_memory_format_is_preserved():
    x = torch.randn(2, 8, 5, 7).contiguous(memory_format=torch.channels_last)
    q = torch.quantize_per_tensor(x.cuda(), 0.05, 10, torch.quint8)
    assert q.is_contiguous(memory_format=torch.channels_last)
    assert_q_equal(q, torch.quantize_per_tensor(x, 0.05, 10, torch.quint8))
    assert q.dequantize().is_contiguous(memory_format=torch.channels_last)
    qd = torch.quantize_per_tensor_dynamic(x.cuda(), torch.quint8, False)
    assert qd.is_contiguous(memory_format=torch.channels_last)
    assert_q_equal(qd, torch.quantize_per_tensor_dynamic(x, torch.quint8, False))


@pytest.mark.parametrize("c", cases.quantize_per_channel_cases(), ids=lambda c: c["name"])
def test_quantize_per_channel(c):
    say("aten qpc", c["name"])
    x = torch.from_numpy(c["x"])
    s = torch.from_numpy(c["scales"].astype(np.float64))
    z = torch.from_numpy(c["zps"].astype(np.int64))
    dt = torch.qint8 if c["signed"] else torch.quint8
    assert_q_equal(torch.quantize_per_channel(x.cuda(), s.cuda(), z.cuda(), c["axis"], dt),
                   torch.quantize_per_channel(x, s, z, c["axis"], dt))


@pytest.mark.parametrize("c", cases.quantize_per_channel_float_cases(), ids=lambda c: c["name"])
def test_quantize_per_channel_float_qparams(c):
    say("aten qpcf", c["name"])
    x = torch.from_numpy(c["x"])
    s, z = torch.from_numpy(c["scales"]), torch.from_numpy(c["zps"])
    dt = torch.qint8 if c["signed"] else torch.quint8
    q_gpu = torch.quantize_per_channel(x.cuda(), s.cuda(), z.cuda(), c["axis"], dt)
    q_cpu = torch.quantize_per_channel(x, s, z, c["axis"], dt)
    assert q_gpu.qscheme() == torch.per_channel_affine_float_qparams
    assert torch.equal(q_gpu.int_repr().cpu(), q_cpu.int_repr())
    assert torch.equal(q_gpu.dequantize().cpu(), q_cpu.dequantize())


def test_quantize_per_channel_rejects_bad_zero_point():
    x = torch.randn(2, 3).cuda()
    with pytest.raises(RuntimeError):
        torch.quantize_per_channel(x, torch.tensor([0.1, 0.1]).cuda(), torch.tensor([0, 256]).cuda(), 0,
                                   torch.quint8)


# ---------------------------------------------------------------------------
# linear
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("shape", [(8, 128), (8, 10, 128)])
@pytest.mark.parametrize("relu", [False, True])
def test_qlinear_reference_flavour(shape, relu):
    """qint8 activations, per-tensor symmetric qint8 weight, qint8 output, no
    bias: the configuration of the reference's test_qlinear, same assertion."""
    say("aten qlinear ref", shape, relu)
    torch.manual_seed(41)
    data = torch.randn(shape)
    module = torch.nn.Linear(128, 512, False)
    fweight = module.weight.detach()
    qweight = torch.quantize_per_tensor(fweight, float(fweight.abs().max() / 2 ** 7), 0, torch.qint8)
    module.weight = torch.nn.Parameter(qweight.dequantize())
    qmodule = (nniq.LinearReLU if relu else nnq.Linear)(128, 512, False, torch.qint8)
    qmodule.set_weight_bias(qweight.cuda(), None)
    qdata = torch.quantize_per_tensor(data, float(data.abs().max() / 2 ** 7), 0, torch.qint8)
    foutput = module(qdata.dequantize()).detach()
    out_scale = float(foutput.abs().max() / 2 ** 7)
    qmodule.scale, qmodule.zero_point = out_scale, 0
    qoutput = qmodule(qdata.cuda())
    assert qoutput.dtype == torch.qint8 and tuple(qoutput.shape) == shape[:-1] + (512,)
    if relu:
        foutput = torch.relu(foutput)
    assert (qoutput.dequantize().cpu() - foutput).mean().abs() < 1e-3
    fq = torch.quantize_per_tensor(foutput, out_scale, 0, torch.qint8)
    d = (qoutput.int_repr().cpu().to(torch.int32) - fq.int_repr().to(torch.int32)).abs().max()
    assert d <= LSB_TOL


@pytest.mark.parametrize("per_channel", [False, True])
@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("bias", [False, True])
def test_qlinear_matches_cpu_op(per_channel, relu, bias):
    """quint8 activations / per-channel weights: the CPU op is the oracle."""
    say("aten qlinear cpu", per_channel, relu, bias)
    torch.manual_seed(7)
    x = torch.randn(3, 17, 256)
    w = torch.randn(300, 256) * 0.05
    b = torch.randn(300) if bias else None
    xq = torch.quantize_per_tensor_dynamic(x, torch.quint8, False)
    if per_channel:
        s = (w.abs().amax(dim=1) / 127).to(torch.float64)
        wq = torch.quantize_per_channel(w, s, torch.zeros(300, dtype=torch.int64), 0, torch.qint8)
    else:
        wq = torch.quantize_per_tensor(w, float(w.abs().max() / 127), 0, torch.qint8)
    op = torch.ops.quantized.linear_relu if relu else torch.ops.quantized.linear
    ref = op(xq, torch.ops.quantized.linear_prepack(wq, b), 0.1, 100)
    packed = torch.ops.quantized.linear_prepack(wq.cuda(), None if b is None else b.cuda())
    got = op(xq.cuda(), packed, 0.1, 100)
    assert_q_equal(got, ref, abs_diff=LSB_TOL)
    n_off = (got.int_repr().cpu() != ref.int_repr()).sum().item()
    assert n_off == 0, f"{n_off} outputs off by one LSB"
    # unpack returns what was packed (reference: mudnn/LinearUnpackImpl.cpp:9-12)
    w2, b2 = torch.ops.quantized.linear_unpack(packed)
    assert_q_equal(w2, wq)
    assert (b2 is None) == (b is None) and (b is None or torch.equal(b2.cpu(), b))


def test_qlinear_long_k_through_the_operators():
    """150 rows against K = 8192: the operators hand the C ABI a workspace and the
    product runs split along K; quantized::linear and quantized::linear_dynamic
    against the CPU ops, bit for bit."""
    say("aten qlinear split K")
    torch.manual_seed(11)
    x = torch.randn(150, 8192)
    w = torch.randn(200, 8192) * 0.05
    b = torch.randn(200)
    xq = torch.quantize_per_tensor_dynamic(x, torch.quint8, False)
    s = (w.abs().amax(dim=1) / 127).to(torch.float64)
    wq = torch.quantize_per_channel(w, s, torch.zeros(200, dtype=torch.int64), 0, torch.qint8)
    cpu_packed = torch.ops.quantized.linear_prepack(wq, b)
    packed = torch.ops.quantized.linear_prepack(wq.cuda(), b.cuda())
    ref = torch.ops.quantized.linear(xq, cpu_packed, 0.25, 120)
    got = torch.ops.quantized.linear(xq.cuda(), packed, 0.25, 120)
    assert 0.2 < ((ref.int_repr() > 0) & (ref.int_repr() < 255)).float().mean()
    assert_q_equal(got, ref, abs_diff=0)
    refd = torch.ops.quantized.linear_dynamic(x, cpu_packed, False)
    gotd = torch.ops.quantized.linear_dynamic(x.cuda(), packed, False)
    assert torch.equal(gotd.cpu(), refd)


def test_qlinear_errors():
    w = torch.quantize_per_tensor(torch.randn(8, 16), 0.1, 3, torch.qint8).cuda()
    with pytest.raises(RuntimeError):
        torch.ops.quantized.linear_prepack(w, None)                # weight zero point != 0
    wu = torch.quantize_per_tensor(torch.randn(8, 16), 0.1, 0, torch.quint8).cuda()
    with pytest.raises(RuntimeError):
        torch.ops.quantized.linear_prepack(wu, None)               # weight dtype
    w = torch.quantize_per_tensor(torch.randn(8, 16), 0.1, 0, torch.qint8).cuda()
    with pytest.raises(RuntimeError):
        torch.ops.quantized.linear_prepack(w, torch.zeros(9).cuda())  # bias length
    packed = torch.ops.quantized.linear_prepack(w, None)
    x = torch.quantize_per_tensor(torch.randn(4, 15), 0.1, 0, torch.quint8).cuda()
    with pytest.raises(RuntimeError):
        torch.ops.quantized.linear(x, packed, 0.1, 0)              # feature mismatch
    x = torch.quantize_per_tensor(torch.randn(4, 16), 0.1, 0, torch.quint8).cuda()
    y = torch.ops.quantized.linear_dynamic(x.dequantize(), packed)  # implemented here, unlike the reference
    assert y.dtype == torch.float32 and tuple(y.shape) == (4, 8)
    empty = torch.quantize_per_tensor(torch.randn(0, 16), 0.1, 0, torch.quint8).cuda()
    assert tuple(torch.ops.quantized.linear(empty, packed, 0.1, 0).shape) == (0, 8)


def test_c1_through_the_operators(golden):
    """benchmark configuration 1 with nothing but torch calls on GPU tensors."""
    say("aten C1")
    c1 = cases.c1_case()
    xq = torch.quantize_per_tensor_dynamic(torch.from_numpy(c1["x"]).cuda(), torch.quint8, False)
    assert xq.q_scale() == float(golden["c1/x_scale"]) and xq.q_zero_point() == int(golden["c1/x_zp"])
    wq = torch.quantize_per_channel(torch.from_numpy(c1["w"]).cuda(), torch.from_numpy(c1["w_scales"]).cuda(),
                                    torch.zeros(1024, dtype=torch.int64).cuda(), 0, torch.qint8)
    packed = torch.ops.quantized.linear_prepack(wq, torch.from_numpy(c1["bias"]).cuda())
    y = torch.ops.quantized.linear(xq, packed, c1["out_scale"], c1["out_zp"])
    assert y.dtype == torch.quint8
    d = np.abs(y.int_repr().cpu().numpy().astype(np.int32) - golden["c1/y"].astype(np.int32))
    assert d.max() <= LSB_TOL and d.max() == 0
    assert cases.crc(y.dequantize().cpu().numpy()) == int(golden["c1/y_dq_crc"])


# ---------------------------------------------------------------------------
# conv2d
# ---------------------------------------------------------------------------
CONV_CONFIGS = [
    dict(shape=(2, 32, 16, 16), oc=64, k=3, s=1, p=1, d=1, g=1, bias=False, relu=False),
    dict(shape=(2, 32, 16, 16), oc=64, k=3, s=1, p=1, d=1, g=1, bias=False, relu=True),
    dict(shape=(2, 3, 16, 16), oc=32, k=3, s=2, p=1, d=1, g=1, bias=True, relu=True),
    dict(shape=(2, 64, 16, 16), oc=32, k=3, s=2, p=1, d=1, g=32, bias=False, relu=True),
    dict(shape=(8, 3, 32, 32), oc=32, k=7, s=2, p=3, d=1, g=1, bias=True, relu=False),
    dict(shape=(4, 64, 28, 28), oc=64, k=3, s=1, p=1, d=1, g=1, bias=True, relu=False),
    # the layers of a mobile network: depthwise (four channels per lane; 5 x 5 at stride 2 on 144 channels: merged
    # groups on the matrix pipe), pointwise off the 16-channel grid (byte runs), pointwise over few pixels (as a
    # linear layer); and a long K on one small image (patch rows in a workspace)
    dict(shape=(2, 32, 20, 20), oc=32, k=3, s=1, p=1, d=1, g=32, bias=True, relu=True),
    dict(shape=(1, 144, 14, 14), oc=144, k=3, s=2, p=1, d=1, g=144, bias=False, relu=False),
    dict(shape=(2, 72, 15, 15), oc=72, k=5, s=1, p=2, d=1, g=72, bias=True, relu=True),
    dict(shape=(1, 144, 14, 14), oc=144, k=5, s=2, p=2, d=1, g=144, bias=True, relu=False),
    dict(shape=(2, 24, 14, 14), oc=144, k=1, s=1, p=0, d=1, g=1, bias=True, relu=False),
    dict(shape=(2, 256, 6, 6), oc=48, k=1, s=1, p=0, d=1, g=1, bias=True, relu=True),
    dict(shape=(1, 256, 7, 7), oc=64, k=3, s=1, p=1, d=1, g=1, bias=True, relu=False),
    # 40 channels under a 3 x 3 kernel: the MFMA kernels on a channel-padded copy in a workspace
    dict(shape=(2, 40, 14, 14), oc=24, k=3, s=1, p=1, d=1, g=1, bias=True, relu=True),
]


@pytest.mark.parametrize("cfg", CONV_CONFIGS, ids=lambda c: f"{c['shape']}-{c['oc']}-k{c['k']}g{c['g']}")
@pytest.mark.parametrize("per_channel", [False, True])
@pytest.mark.parametrize("channels_last_input,out_zp", [(False, 90), (True, 90), (True, 0)])
def test_qconv2d_matches_cpu_op(cfg, per_channel, channels_last_input, out_zp):
    """Configurations of the reference's test_qconv2d, through nnq.Conv2d with
    weights set from outside (test_quantized_conv.py:83-150), against the CPU op."""
    say("aten qconv", cfg, per_channel, channels_last_input, out_zp)
    torch.manual_seed(41)
    ic = cfg["shape"][1]
    x = torch.randn(cfg["shape"])
    if channels_last_input:
        x = x.contiguous(memory_format=torch.channels_last)
    w = torch.randn(cfg["oc"], ic // cfg["g"], cfg["k"], cfg["k"]) * 0.1
    b = torch.randn(cfg["oc"]) if cfg["bias"] else None
    xq = torch.quantize_per_tensor_dynamic(x, torch.quint8, False)
    if per_channel:
        s = (w.abs().amax(dim=(1, 2, 3)) / 127).to(torch.float64)
        wq = torch.quantize_per_channel(w, s, torch.zeros(cfg["oc"], dtype=torch.int64), 0, torch.qint8)
    else:
        wq = torch.quantize_per_tensor(w, float(w.abs().max() / 127), 0, torch.qint8)
    cls = nniq.ConvReLU2d if cfg["relu"] else nnq.Conv2d
    mods = []
    for dev in ("cpu", "cuda"):
        m = cls(ic, cfg["oc"], cfg["k"], cfg["s"], cfg["p"], cfg["d"], cfg["g"], cfg["bias"])
        m.set_weight_bias(wq.to(dev), None if b is None else b.to(dev))
        m.scale, m.zero_point = 0.25, out_zp
        mods.append(m)
    ref = mods[0](xq)
    got = mods[1](xq.cuda())
    assert got.is_contiguous(memory_format=torch.channels_last) or got.numel() == 0
    if cfg["g"] == ic and per_channel:
        # PyTorch's CPU depthwise kernels are not exact integer arithmetic with per-channel weights (every channel
        # then has weights of +-127): the 144-channel case differs from the exact sums by up to 3 LSB on 59 of its
        # 7056 outputs on a CPU-only machine.  The float pipeline judges instead, as in the reference's own tests
        # (test_quantized_conv.py:83-150): quantize(conv(dequantized operands)) within one LSB.
        rf = torch.nn.functional.conv2d(xq.dequantize(), wq.dequantize(), b, cfg["s"], cfg["p"], cfg["d"], cfg["g"])
        ref = torch.quantize_per_tensor(torch.relu(rf) if cfg["relu"] else rf, 0.25, out_zp, torch.quint8)
    assert_q_equal(got, ref, abs_diff=LSB_TOL)
    n_off = (got.int_repr().cpu() != ref.int_repr()).sum().item()
    if cfg["g"] == ic and per_channel:
        assert n_off <= 0.02 * ref.numel(), f"{n_off} outputs off by one LSB"
    elif cfg["g"] > 1 and cfg["bias"]:
        # PyTorch's x86 engine hands grouped convolutions to oneDNN on CPUs with VNNI and to fbgemm on the others;
        # with a bias the two differ from one another by one LSB on a few outputs in ten thousand.  The kernels
        # follow fbgemm's output stage bit for bit (tests/test_gpu_conv.py against the oracle).
        assert n_off <= 0.005 * ref.numel(), f"{n_off} outputs off by one LSB"
    else:
        assert n_off == 0, f"{n_off} outputs off by one LSB"
    w2, b2 = mods[1]._weight_bias()
    assert_q_equal(w2, wq)
    assert (b2 is None) == (b is None) and (b is None or torch.equal(b2.cpu(), b))


def test_qconv2d_errors():
    w = torch.quantize_per_tensor(torch.randn(8, 4, 3, 3), 0.1, 5, torch.qint8).cuda()
    with pytest.raises(RuntimeError):
        torch.ops.quantized.conv2d_prepack(w, None, [1, 1], [0, 0], [1, 1], 1)   # zero point != 0
    w = torch.quantize_per_tensor(torch.randn(8, 4, 3, 3), 0.1, 0, torch.qint8).cuda()
    packed = torch.ops.quantized.conv2d_prepack(w, None, [1, 1], [1, 1], [1, 1], 1)
    x = torch.quantize_per_tensor(torch.randn(1, 5, 8, 8), 0.1, 0, torch.quint8).cuda()
    with pytest.raises(RuntimeError):
        torch.ops.quantized.conv2d(x, packed, 0.1, 0)                             # channel mismatch


# ---------------------------------------------------------------------------
# fused conv ops (quantized::conv2d_add, conv2d_add_relu, conv2d_silu, conv2d_add_silu)
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("c", cases.conv_fused_cases(), ids=lambda c: c["name"])
def test_conv2d_fused_ops(golden, c):
    say("aten conv fused", c["name"])
    qd = torch.qint8 if c["signed"] else torch.quint8
    xq = torch._make_per_tensor_quantized_tensor(
        torch.from_numpy(c["xq"]).cuda().permute(0, 3, 1, 2), c["x_scale"], c["x_zp"])
    wt = torch.from_numpy(c["wq"]).permute(0, 3, 1, 2).contiguous().cuda()
    if len(c["w_scales"]) == 1:
        w = torch._make_per_tensor_quantized_tensor(wt, float(c["w_scales"][0]), 0)
    else:
        w = torch._make_per_channel_quantized_tensor(
            wt, torch.from_numpy(c["w_scales"]).cuda(), torch.zeros(wt.shape[0], dtype=torch.int64).cuda(), 0)
    b = None if c["bias"] is None else torch.from_numpy(c["bias"]).cuda()
    packed = torch.ops.quantized.conv2d_prepack(w, b, list(c["stride"]), list(c["padding"]),
                                                list(c["dilation"]), c["groups"])
    ops = torch.ops.quantized
    if c["accq"] is not None:
        aq = torch._make_per_tensor_quantized_tensor(
            torch.from_numpy(c["accq"]).cuda().permute(0, 3, 1, 2), c["acc_scale"], c["acc_zp"])
        op = {"none": ops.conv2d_add, "relu": ops.conv2d_add_relu, "silu": ops.conv2d_add_silu}[c["activation"]]
        y = op(xq, aq, packed, c["out_scale"], c["out_zp"])
    else:
        assert c["activation"] == "silu"
        y = ops.conv2d_silu(xq, packed, c["out_scale"], c["out_zp"])
    assert y.dtype == qd and y.q_scale() == c["out_scale"] and y.q_zero_point() == c["out_zp"]
    assert y.is_contiguous(memory_format=torch.channels_last)
    got = y.int_repr().permute(0, 2, 3, 1).contiguous().cpu().numpy()
    d = np.abs(got.astype(np.int32) - golden["convf/" + c["name"] + "/y"].astype(np.int32))
    assert d.max() <= 1 and np.count_nonzero(d) <= 0.003 * d.size


def test_conv2d_add_rejects_wrong_accum():
    w = torch._make_per_tensor_quantized_tensor(torch.zeros(8, 16, 3, 3, dtype=torch.int8).cuda(), 0.1, 0)
    packed = torch.ops.quantized.conv2d_prepack(w, None, [1, 1], [1, 1], [1, 1], 1)
    x = torch._make_per_tensor_quantized_tensor(torch.zeros(1, 16, 5, 5, dtype=torch.uint8).cuda(), 0.1, 0)
    bad = torch._make_per_tensor_quantized_tensor(torch.zeros(1, 8, 4, 4, dtype=torch.uint8).cuda(), 0.1, 0)
    with pytest.raises(RuntimeError):
        torch.ops.quantized.conv2d_add(x, bad, packed, 0.1, 0)
    with pytest.raises(RuntimeError):
        torch.ops.quantized.conv2d_add(x, torch.zeros(1, 8, 5, 5).cuda(), packed, 0.1, 0)


# ---------------------------------------------------------------------------
# quantized::add / add_relu, relu
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("c", cases.qadd_cases(), ids=lambda c: c["name"])
def test_quantized_add_ops(golden, c):
    say("aten qadd", c["name"])
    qa = torch._make_per_tensor_quantized_tensor(torch.from_numpy(c["qa"]).cuda(), c["a_scale"], c["a_zp"])
    qb = torch._make_per_tensor_quantized_tensor(torch.from_numpy(c["qb"]).cuda(), c["b_scale"], c["b_zp"])
    op = torch.ops.quantized.add_relu if c["relu"] else torch.ops.quantized.add
    y = op(qa, qb, c["out_scale"], c["out_zp"])
    assert y.q_scale() == c["out_scale"] and y.q_zero_point() == c["out_zp"] and y.dtype == qa.dtype
    d = np.abs(y.int_repr().cpu().numpy().astype(np.int32) - golden["qadd/" + c["name"] + "/y"].astype(np.int32))
    assert d.max() <= 1 and np.count_nonzero(d) <= max(1, d.size // 20000)
    r = torch.relu(qa)
    assert r.q_scale() == qa.q_scale() and r.q_zero_point() == qa.q_zero_point()
    np.testing.assert_array_equal(r.int_repr().cpu().numpy(), golden["qadd/" + c["name"] + "/relu_a"])


def test_quantized_add_keeps_channels_last_and_checks_shapes():
    x = torch.randn(2, 8, 5, 5).contiguous(memory_format=torch.channels_last)
    qa = torch.quantize_per_tensor(x.cuda(), 0.05, 128, torch.quint8)
    qb = torch.quantize_per_tensor((x * 0.5).cuda(), 0.04, 120, torch.quint8)
    y = torch.ops.quantized.add(qa, qb, 0.08, 128)
    assert y.is_contiguous(memory_format=torch.channels_last)
    want = torch.ops.quantized.add(qa.cpu(), qb.cpu(), 0.08, 128)
    assert (y.int_repr().cpu().int() - want.int_repr().int()).abs().max() <= 1
    with pytest.raises(RuntimeError):
        torch.ops.quantized.add(qa, qb[:, :4], 0.08, 128)


@pytest.mark.parametrize("dtype,zp", [(torch.quint8, 128), (torch.qint8, 0)])
@pytest.mark.parametrize("shape", [(128, 512), (256, 256), (2, 32, 32, 16)])
def test_qfunctional(shape, dtype, zp):
    # the reference's test_qfunctional (test_quantized_binary_ops.py:36-80): nnq.QFunctional's
    # add / add_relu (and cat) on device tensors against the same calls on the CPU, within 1 LSB
    say("nnq.QFunctional", shape, dtype)
    torch.manual_seed(41)
    a, b = torch.randn(shape), torch.randn(shape)
    scale = float(a.abs().max() / 2 ** 7)
    qa, qb = (torch.quantize_per_tensor(t, scale, zp, dtype) for t in (a, b))
    if len(shape) == 4:
        qa, qb = qa.permute(0, 3, 1, 2), qb.permute(0, 3, 1, 2)
    f = nnq.QFunctional()
    f.scale, f.zero_point = 0.05, zp
    for call in (f.add, f.add_relu):
        assert_q_equal(call(qa.cuda(), qb.cuda()), call(qa, qb), abs_diff=1)
    assert_q_equal(f.cat([qa.cuda(), qb.cuda()], 1), f.cat([qa, qb], 1), abs_diff=1)


@pytest.mark.parametrize("c", cases.qcat_cases(), ids=lambda c: c["name"])
def test_quantized_cat_op(golden, c):
    say("aten qcat", c["name"])
    qs = [torch._make_per_tensor_quantized_tensor(torch.from_numpy(q).cuda(), s_, z_)
          for q, s_, z_ in zip(c["qs"], c["scales"], c["zps"])]
    y = torch.ops.quantized.cat(qs, c["axis"], c["out_scale"], c["out_zp"])
    assert y.q_scale() == c["out_scale"] and y.q_zero_point() == c["out_zp"]
    np.testing.assert_array_equal(y.int_repr().cpu().numpy(), golden["qcat/" + c["name"] + "/y"])
    # scale / zero point default to the first input's
    y0 = torch.ops.quantized.cat(qs, c["axis"], None, None)
    assert y0.q_scale() == qs[0].q_scale() and y0.q_zero_point() == qs[0].q_zero_point()


@pytest.mark.parametrize("c", cases.qmaxpool_cases(), ids=lambda c: c["name"])
def test_quantized_max_pool2d_op(golden, c):
    say("aten qmaxpool", c["name"])
    zp = -7 if c["signed"] else 33
    xq = torch._make_per_tensor_quantized_tensor(torch.from_numpy(c["x"]).cuda().permute(0, 3, 1, 2), 0.1, zp)
    y = torch.nn.functional.max_pool2d(xq, c["kernel"], c["stride"], c["padding"], c["dilation"], c["ceil_mode"])
    assert y.q_scale() == 0.1 and y.q_zero_point() == zp
    np.testing.assert_array_equal(y.int_repr().permute(0, 2, 3, 1).contiguous().cpu().numpy(),
                                  golden["qmaxpool/" + c["name"] + "/y"])


# ---------------------------------------------------------------------------
# torch.ao modules on the GPU (the reference's tests drive its ops through
# nnq.Linear / nnq.Conv2d with set_weight_bias, test_quantized_linear.py:58-60)
# ---------------------------------------------------------------------------
def test_ao_modules_run_on_gpu_and_round_trip_state():
    import torch.ao.nn.intrinsic.quantized as nniq
    import torch.ao.nn.quantized as nnq
    say("ao modules")
    torch.manual_seed(3)
    x = torch.randn(4, 64)
    w = torch.randn(32, 64) * 0.1
    b = torch.randn(32)
    wq = torch.quantize_per_tensor(w, float(w.abs().max()) / 128, 0, torch.qint8)
    xq = torch.quantize_per_tensor(x, float(x.abs().max()) / 128, 128, torch.quint8)
    m, mc = nnq.Linear(64, 32), nnq.Linear(64, 32)
    m.set_weight_bias(wq.cuda(), b.cuda())
    mc.set_weight_bias(wq, b)
    for mod in (m, mc):
        mod.scale, mod.zero_point = 0.1, 128
    assert torch.equal(m(xq.cuda()).int_repr().cpu(), mc(xq).int_repr())
    assert torch.equal(m.weight().int_repr().cpu(), wq.int_repr()) and m.bias().is_cuda
    m2 = nnq.Linear(64, 32)
    m2.load_state_dict(m.state_dict())
    assert torch.equal(m2(xq.cuda()).int_repr().cpu(), mc(xq).int_repr())

    xc = torch.randn(2, 16, 9, 9)
    wc = torch.randn(8, 16, 3, 3) * 0.1
    bc = torch.randn(8)
    wcq = torch.quantize_per_tensor(wc, float(wc.abs().max()) / 128, 0, torch.qint8)
    xcq = torch.quantize_per_tensor(xc, float(xc.abs().max()) / 128, 128, torch.quint8)
    for cls in (nnq.Conv2d, nniq.ConvReLU2d):
        g, c = cls(16, 8, 3, padding=1), cls(16, 8, 3, padding=1)
        g.set_weight_bias(wcq.cuda(), bc.cuda())
        c.set_weight_bias(wcq, bc)
        for mod in (g, c):
            mod.scale, mod.zero_point = 0.05, 128
        assert torch.equal(g(xcq.cuda()).int_repr().cpu(), c(xcq).int_repr()), cls.__name__
        wt, bt = g._weight_bias()
        assert torch.equal(wt.int_repr().cpu(), wcq.int_repr()) and torch.equal(bt.cpu(), bc)


def test_residual_block_end_to_end():
    """conv_relu -> conv_add_relu -> max_pool -> cat with the block's input pooled,
    all on quantized GPU tensors, against the float pipeline on dequantized values."""
    import torch.nn.functional as F
    say("residual block")
    torch.manual_seed(5)
    ops = torch.ops.quantized
    x = torch.relu(torch.randn(2, 32, 16, 16)).contiguous(memory_format=torch.channels_last)
    xq = torch.quantize_per_tensor(x, float(x.max()) / 255, 0, torch.quint8)
    ws, ps = [], []
    for _ in range(2):
        w = torch.randn(32, 32, 3, 3) * 0.05
        s = (w.abs().amax(dim=(1, 2, 3)) / 127).double()
        wq = torch.quantize_per_channel(w, s, torch.zeros(32, dtype=torch.int64), 0, torch.qint8)
        b = torch.randn(32) * 0.1
        ws.append((wq, b))
        ps.append(ops.conv2d_prepack(wq.cuda(), b.cuda(), [1, 1], [1, 1], [1, 1], 1))
    # float pipeline with a quantize -> dequantize after every op, as the quantized graph does
    def qdq(t, s, z=0):
        return torch.quantize_per_tensor(t, s, z, torch.quint8)
    f1 = torch.relu(F.conv2d(xq.dequantize(), ws[0][0].dequantize(), ws[0][1], 1, 1))
    s1 = float(f1.max()) / 255
    q1 = qdq(f1, s1)
    f2 = torch.relu(F.conv2d(q1.dequantize(), ws[1][0].dequantize(), ws[1][1], 1, 1) + xq.dequantize())
    s2 = float(f2.max()) / 255
    q2 = qdq(f2, s2)
    want = torch.cat([F.max_pool2d(q2.dequantize(), 2), F.max_pool2d(xq.dequantize(), 2)], 1)
    want_q = qdq(want, s2)

    g = xq.cuda()
    y1 = ops.conv2d_relu(g, ps[0], s1, 0)
    y2 = ops.conv2d_add_relu(y1, g, ps[1], s2, 0)
    y = ops.cat([F.max_pool2d(y2, 2), F.max_pool2d(g, 2)], 1, s2, 0)
    assert y.shape == want_q.shape
    d = (y.int_repr().cpu().int() - want_q.int_repr().int()).abs()
    # one LSB per requantisation boundary crossed; a second-layer value may move
    # by one more when its input moved
    assert d.max() <= 2 and (d > 1).float().mean() < 1e-3 and (d > 0).float().mean() < 0.02, (d.max(), (d > 0).float().mean())


@pytest.mark.parametrize("c", cases.qavgpool_cases(), ids=lambda c: c["name"])
def test_adaptive_avg_pool2d_op(golden, c):
    say("aten adaptive_avg_pool2d", c["name"])
    x_nchw = torch.from_numpy(c["x"]).permute(0, 3, 1, 2)
    xq = torch._make_per_tensor_quantized_tensor(x_nchw.contiguous().cuda(), 0.05, c["zp"])
    for inp in (xq, xq.contiguous(memory_format=torch.channels_last)):
        y = torch.nn.functional.adaptive_avg_pool2d(inp, c["out_hw"])
        assert y.is_quantized and y.q_scale() == 0.05 and y.q_zero_point() == c["zp"]
        np.testing.assert_array_equal(y.int_repr().permute(0, 2, 3, 1).contiguous().cpu().numpy(),
                                      golden["qavgpool/" + c["name"] + "/y"])
    m = torch.nn.AdaptiveAvgPool2d(c["out_hw"])
    np.testing.assert_array_equal(m(xq).int_repr().cpu().numpy(), y.int_repr().cpu().numpy())


def _wq_from_case(c):
    n = c["wq"].shape[0]
    w = torch.from_numpy(c["wq"])
    if len(c["w_scales"]) == 1:
        return torch._make_per_tensor_quantized_tensor(w, float(c["w_scales"][0]), 0)
    return torch._make_per_channel_quantized_tensor(w, torch.from_numpy(c["w_scales"]),
                                                    torch.zeros(n, dtype=torch.int64), 0)


@pytest.mark.parametrize("c", cases.linear_dynamic_cases(), ids=lambda c: c["name"])
def test_linear_dynamic_op(golden, c):
    # float in, float out; live CPU op and golden vector, bit for bit
    say("aten linear_dynamic", c["name"])
    wq = _wq_from_case(c)
    b = None if c["bias"] is None else torch.from_numpy(c["bias"])
    name = "linear_relu_dynamic" if c["relu"] else "linear_dynamic"
    op = getattr(torch.ops.quantized, name)
    x = torch.from_numpy(c["x"])
    ref = op(x, torch.ops.quantized.linear_prepack(wq, b), c["reduce_range"])
    packed = torch.ops.quantized.linear_prepack(wq.cuda(), None if b is None else b.cuda())
    y = op(x.cuda(), packed, c["reduce_range"])
    assert y.is_cuda and y.dtype == torch.float32 and y.shape == ref.shape
    assert torch.equal(y.cpu(), ref)
    np.testing.assert_array_equal(y.cpu().numpy(), golden["lindyn/" + c["name"] + "/y"])


def test_dynamic_linear_module():
    # torch.ao.nn.quantized.dynamic.Linear with GPU packed parameters (set_weight_bias, as
    # the reference's tests populate quantized modules, test_quantized_linear.py:58-60)
    say("nnqd.Linear")
    import torch.ao.nn.quantized.dynamic as nnqd
    torch.manual_seed(5)
    w = torch.randn(96, 160) * 0.05
    b = torch.randn(96)
    wq = torch.quantize_per_tensor(w, float(w.abs().max() / 127), 0, torch.qint8)
    x = torch.randn(4, 9, 160)
    m_cpu = nnqd.Linear(160, 96)
    m_cpu.set_weight_bias(wq, b)
    m_gpu = nnqd.Linear(160, 96)
    m_gpu.set_weight_bias(wq.cuda(), b.cuda())
    y = m_gpu(x.cuda())
    assert y.is_cuda and torch.equal(y.cpu(), m_cpu(x))
    wq2, b2 = m_gpu._packed_params._packed_params.unpack()
    assert torch.equal(wq2.int_repr().cpu(), wq.int_repr()) and torch.equal(b2.cpu(), b)


def test_linear_dynamic_errors():
    say("aten linear_dynamic errors")
    w = torch.quantize_per_tensor(torch.randn(8, 16), 0.1, 0, torch.qint8).cuda()
    packed = torch.ops.quantized.linear_prepack(w, None)
    with pytest.raises(RuntimeError):
        torch.ops.quantized.linear_dynamic(torch.randn(3, 15).cuda(), packed, False)     # feature count
    with pytest.raises(RuntimeError):
        torch.ops.quantized.linear_dynamic(torch.randn(3, 16).cuda().half(), packed, False)  # dtype
    y = torch.ops.quantized.linear_dynamic(torch.zeros(0, 16).cuda(), packed, False)
    assert y.shape == (0, 8)


# ---- plain-tensor int8 ops (the reference's PT2E lowering targets) ----------------------
_TD = {"uint8": torch.uint8, "int8": torch.int8, "float32": torch.float32}


def _close_to(y, want, out_dtype, what, exact=False):
    assert y.shape == want.shape and y.dtype == want.dtype, what
    if exact:
        np.testing.assert_array_equal(y, want, err_msg=what)
    elif out_dtype == "float32":
        np.testing.assert_allclose(y, want, rtol=1e-5, atol=1e-5 * max(1.0, float(np.abs(want).max())), err_msg=what)
    else:
        d = np.abs(y.astype(np.int32) - want.astype(np.int32))
        assert d.max() <= 1, f"{what}: max diff {d.max()}"
        assert np.count_nonzero(d) <= 0.002 * d.size + 1, f"{what}: {np.count_nonzero(d)} of {d.size} differ"


@pytest.mark.parametrize("c", cases.plain_linear_cases(), ids=lambda c: c["name"])
def test_linear_per_tensor_op(golden, c):
    say("aten linear_per_tensor", c["name"])
    n = c["w"].shape[1]
    b = None if c["bias"] is None else torch.from_numpy(c["bias"]).cuda()
    y = torch.ops.quantized.linear_per_tensor(
        torch.from_numpy(c["x"]).cuda(), c["x_scale"], c["x_zp"], torch.from_numpy(c["w"]).cuda(),
        torch.from_numpy(c["w_scale"]).cuda(), torch.zeros(n, dtype=torch.int).cuda(), b, c["out_scale"], c["out_zp"],
        _TD[c["out_dtype"]], c["post"], [], "")
    assert y.is_cuda and y.dtype == _TD[c["out_dtype"]]
    y = y.cpu().numpy()
    exact = c["name"].startswith("ref")
    _close_to(y, golden["plainlin/" + c["name"] + "/y"], c["out_dtype"], "vs oneDNN CPU op", exact)
    want = oracle.plain_linear(c["x"], c["x_scale"], c["x_zp"], c["w"], c["w_scale"], c["bias"], c["out_scale"],
                               c["out_zp"], c["out_dtype"], c["post"])
    _close_to(y, want, c["out_dtype"], "vs closed form", exact)


@pytest.mark.parametrize("c", cases.plain_conv_cases(), ids=lambda c: c["name"])
def test_plain_conv_ops(golden, c):
    say("aten conv / conv_binary", c["name"])
    oc = c["w"].shape[0]
    b = None if c["bias"] is None else torch.from_numpy(c["bias"]).cuda()
    args = [torch.from_numpy(c["x"]).cuda(), c["x_scale"], c["x_zp"], torch.from_numpy(c["w"]).cuda(),
            torch.from_numpy(c["w_scale"]).cuda(), torch.zeros(oc, dtype=torch.int).cuda()]
    geom = [[c["stride"]] * 2, [c["pad"]] * 2, [1, 1], c["groups"], c["out_scale"], c["out_zp"], _TD[c["out_dtype"]]]
    if c["accum"] is None:
        y = torch.ops.quantized.conv(*args, b, *geom, "relu" if c["relu"] else "none", [], None)
    else:
        acc = torch.from_numpy(c["accum"]).cuda()
        y = torch.ops.quantized.conv_binary(*args, acc, b, *geom, c["accum_scale"], c["accum_zp"], "sum", 1.0,
                                            "relu" if c["relu"] else "none", [], None)
        assert torch.equal(acc.cpu(), torch.from_numpy(c["accum"]))   # the input is left alone
    assert y.is_cuda and y.dtype == _TD[c["out_dtype"]]
    y = y.contiguous().cpu().numpy()
    _close_to(y, golden["plainconv/" + c["name"] + "/y"], c["out_dtype"], "vs oneDNN CPU op")
    want = oracle.plain_conv(c["x"], c["x_scale"], c["x_zp"], c["w"], c["w_scale"], c["bias"], c["stride"], c["pad"],
                             c["groups"], c["out_scale"], c["out_zp"], c["out_dtype"], c["relu"], c["accum"],
                             c["accum_scale"], c["accum_zp"])
    _close_to(y, want, c["out_dtype"], "vs closed form")


def test_plain_ops_errors():
    say("aten plain ops errors")
    x = torch.randint(0, 255, (4, 16), dtype=torch.uint8).cuda()
    w = torch.randint(-127, 127, (16, 8), dtype=torch.int8).cuda()
    ws, wz = torch.full((8,), 0.01).cuda(), torch.zeros(8, dtype=torch.int).cuda()
    call = lambda *a: torch.ops.quantized.linear_per_tensor(*a)
    with pytest.raises(RuntimeError):
        call(x[None], 0.1, 0, w, ws, wz, None, 1.0, 0, torch.uint8, "none", [], "")       # 3-D input
    with pytest.raises(RuntimeError):
        call(x, 0.1, 0, w, ws, wz + 1, None, 1.0, 0, torch.uint8, "none", [], "")         # weight zero point
    with pytest.raises(RuntimeError):
        call(x, 0.1, 0, w, ws, wz, None, 1.0, 0, torch.uint8, "hardswish", [], "")        # post op
    with pytest.raises(RuntimeError):
        call(x, 0.1, 0, w[:8], ws, wz, None, 1.0, 0, torch.uint8, "none", [], "")         # K mismatch
    # tanh goes through the float result, like the reference's fallback
    y = call(x, 0.02, 128, w, ws, wz, None, 1 / 128, 128, torch.uint8, "tanh", [], "").cpu()
    r = torch.tanh(((x.cpu().float() - 128) * 0.02) @ (w.cpu().float() * 0.01))
    assert (y.int() - torch.clamp(torch.round(r * 128 + 128), 0, 255).int()).abs().max() <= 1


def test_plain_ops_keep_their_packed_weight():
    """The plain-tensor ops re-tile a weight once: a second call with the same weight, scale and
    zero-point tensors hits the cache and gives the same bytes; an in-place change of the weight,
    other scales, or a new tensor at a recycled address miss and give the new result."""
    import torch_musa_amd as tm
    say("aten plain-op weight cache")
    tm.plain_weight_cache_clear()
    g = torch.Generator().manual_seed(5)
    x = torch.randint(0, 255, (33, 64), dtype=torch.uint8, generator=g).cuda()
    w = torch.randint(-127, 127, (64, 48), dtype=torch.int8, generator=g).cuda()
    ws, wz = (torch.rand(48, generator=g) * 0.01 + 0.001).cuda(), torch.zeros(48, dtype=torch.int).cuda()
    call = lambda w_, ws_: torch.ops.quantized.linear_per_tensor(x, 0.02, 120, w_, ws_, wz, None, 0.3, 100,
                                                                  torch.uint8, "none", [], "")

    def same(y, w_, ws_, what):
        want = oracle.plain_linear(x.cpu().numpy(), 0.02, 120, w_.cpu().numpy(), ws_.cpu().numpy(), None, 0.3, 100,
                                   "uint8", "none")
        _close_to(y.cpu().numpy(), want, "uint8", what)

    h0, m0, _ = tm.plain_weight_cache_counters()
    y1 = call(w, ws)
    y2 = call(w, ws)
    h1, m1, e1 = tm.plain_weight_cache_counters()
    assert (h1 - h0, m1 - m0) == (1, 1) and e1 >= 1
    assert torch.equal(y1, y2)
    same(y1, w, ws, "first call")
    w[0, :] = 5                      # in place: the version counter moves, the entry no longer matches
    y3 = call(w, ws)
    assert tm.plain_weight_cache_counters()[1] - m1 == 1
    same(y3, w, ws, "after an in-place change of the weight")
    assert not torch.equal(y3, y1)
    ws2 = ws * 2                     # other scales with the same weight
    same(call(w, ws2), w, ws2, "other scales")
    # a weight freed and another allocated (very likely at the same address): must not hit
    for seed in range(3):
        wn = torch.randint(-127, 127, (64, 48), dtype=torch.int8, generator=g).cuda()
        same(call(wn, ws), wn, ws, f"fresh weight {seed}")
        del wn
    # conv: the same packed weight serves two image sizes
    wc = torch.randint(-127, 127, (16, 16, 3, 3), dtype=torch.int8, generator=g).cuda()
    wcs, wcz = torch.full((16,), 0.004).cuda(), torch.zeros(16, dtype=torch.int).cuda()
    hc0 = tm.plain_weight_cache_counters()[0]
    for hw in (9, 14, 9):
        xc = torch.randint(0, 255, (2, 16, hw, hw), dtype=torch.uint8, generator=g).cuda()
        yc = torch.ops.quantized.conv(xc, 0.03, 3, wc, wcs, wcz, None, [1, 1], [1, 1], [1, 1], 1, 0.5, 10,
                                      torch.uint8, "none", [], None)
        want = oracle.plain_conv(xc.cpu().numpy(), 0.03, 3, wc.cpu().numpy(), wcs.cpu().numpy(), None, 1, 1, 1, 0.5, 10,
                                 "uint8", False, None, 1.0, 0)
        _close_to(yc.contiguous().cpu().numpy(), want, "uint8", f"conv {hw}x{hw}")
    assert tm.plain_weight_cache_counters()[0] - hc0 == 2
    tm.plain_weight_cache_clear()
    assert tm.plain_weight_cache_counters()[2] == 0


def test_plain_weight_cache_across_streams_and_graph_capture():
    """A miss packs on the caller's stream; a hit from another stream must wait for that packing.
    A capture takes an entry whose packing has finished and records no wait for it."""
    import torch_musa_amd as tm
    say("aten plain-op weight cache: streams and capture")
    tm.plain_weight_cache_clear()
    g = torch.Generator().manual_seed(11)
    M, K, N = 64, 4096, 4096            # a packing long enough to be in flight when the hit arrives
    x = torch.randint(0, 255, (M, K), dtype=torch.uint8, generator=g).cuda()
    wz = torch.zeros(N, dtype=torch.int).cuda()
    ws = (torch.rand(N, generator=g) * 0.002 + 0.001).cuda()
    call = lambda w_: torch.ops.quantized.linear_per_tensor(x, 0.02, 120, w_, ws, wz, None, 0.6, 100, torch.uint8,
                                                             "none", [], "")

    def want(w_):
        return oracle.plain_linear(x.cpu().numpy(), 0.02, 120, w_.cpu().numpy(), ws.cpu().numpy(), None, 0.6, 100,
                                   "uint8", "none")

    side = torch.cuda.Stream()
    for rep in range(3):
        w = torch.randint(-127, 127, (K, N), dtype=torch.int8, generator=g).cuda()
        torch.cuda.synchronize()
        before = tm.plain_weight_cache_stats()
        with torch.cuda.stream(side):
            # a long queue in front of the packing, so that the default stream's hit arrives first
            filler = torch.empty(1 << 26, device="cuda")
            for _ in range(4):
                filler.normal_()
            y_side = call(w)            # miss: packs on `side`
        y_main = call(w)                # hit from the default stream, packing possibly still queued
        torch.cuda.synchronize()
        after = tm.plain_weight_cache_stats()
        assert after["misses"] - before["misses"] == 1 and after["hits"] - before["hits"] == 1
        assert after["cross_stream_hits"] - before["cross_stream_hits"] == 1
        ref = want(w)
        _close_to(y_main.cpu().numpy(), ref, "uint8", f"hit on the default stream, round {rep}")
        _close_to(y_side.cpu().numpy(), ref, "uint8", f"miss on the side stream, round {rep}")
        assert torch.equal(y_main, y_side)
        del filler
    # capture: a weight packed by an eager call beforehand (a miss inside a capture is refused
    # with an error: the zero-point check alone needs the host)
    w2 = torch.randint(-127, 127, (K, N), dtype=torch.int8, generator=g).cuda()
    ref2 = want(w2)
    y_eager = call(w2)
    torch.cuda.synchronize()
    _close_to(y_eager.cpu().numpy(), ref2, "uint8", "eager call before the capture")
    # a capture that finds a finished entry uses it (no packing kernels in the graph)
    graph2 = torch.cuda.CUDAGraph()
    h0 = tm.plain_weight_cache_stats()["hits"]
    with torch.cuda.stream(side):
        side.synchronize()
        with torch.cuda.graph(graph2, stream=side):
            y_cap2 = call(w2)
    torch.cuda.synchronize()
    assert tm.plain_weight_cache_stats()["hits"] == h0 + 1
    assert tm.plain_weight_cache_stats()["cross_stream_hits"] == after["cross_stream_hits"]   # no wait recorded
    for _ in range(2):
        y_cap2.zero_()
        torch.cuda.synchronize()
        graph2.replay()
        torch.cuda.synchronize()
        _close_to(y_cap2.cpu().numpy(), ref2, "uint8", "graph that hit the cache")
    tm.plain_weight_cache_clear()


def test_plain_weight_cache_holds_more_than_64_weights_and_respects_its_byte_limit():
    import torch_musa_amd as tm
    say("aten plain-op weight cache: 65 weights in rotation, byte limit")
    tm.plain_weight_cache_clear()
    g = torch.Generator().manual_seed(12)
    x = torch.randint(0, 255, (8, 64), dtype=torch.uint8, generator=g).cuda()
    wz, ws = torch.zeros(32, dtype=torch.int).cuda(), torch.full((32,), 0.01).cuda()
    weights = [torch.randint(-127, 127, (64, 32), dtype=torch.int8, generator=g).cuda() for _ in range(65)]
    call = lambda w_: torch.ops.quantized.linear_per_tensor(x, 0.02, 120, w_, ws, wz, None, 0.3, 100, torch.uint8,
                                                             "none", [], "")
    first = [call(w_) for w_ in weights]
    s1 = tm.plain_weight_cache_stats()
    second = [call(w_) for w_ in weights]          # a model's second pass: every layer hits
    s2 = tm.plain_weight_cache_stats()
    assert s2["hits"] - s1["hits"] == 65 and s2["misses"] == s1["misses"] and s2["entries"] >= 65
    assert all(torch.equal(a, b) for a, b in zip(first, second))
    per_entry = s2["bytes"] // s2["entries"]
    default_limit = s2["max_bytes"]
    try:
        tm.plain_weight_cache_set_max_bytes(10 * per_entry)      # room for ten: the rest leaves, oldest first
        s3 = tm.plain_weight_cache_stats()
        assert s3["entries"] == 10 and s3["bytes"] <= 10 * per_entry and s3["evictions"] - s2["evictions"] == 55
        third = [call(w_) for w_ in weights]       # rotation over more than the limit holds: misses, same bytes
        s4 = tm.plain_weight_cache_stats()
        assert s4["entries"] == 10 and s4["misses"] - s3["misses"] == 65
        assert all(torch.equal(a, b) for a, b in zip(first, third))
    finally:
        tm.plain_weight_cache_set_max_bytes(default_limit)
        tm.plain_weight_cache_clear()


def test_quantized_modules_to_device():
    # a populated CPU model (conv -> relu -> pool -> flatten -> linear, dynamic linear beside
    # it) moved to the GPU with its packed parameters; same bytes out as on the CPU
    say("quantized_modules_to")
    import torch.ao.nn.quantized.dynamic as nnqd
    import torch_musa_amd
    torch.manual_seed(11)

    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.conv = nniq.ConvReLU2d(16, 32, 3, padding=1)
            self.pool = torch.nn.AdaptiveAvgPool2d((2, 2))
            self.fc = nnq.Linear(128, 24)
            self.dyn = nnqd.Linear(24, 10)

        def forward(self, xq):
            y = self.fc(torch.flatten(self.pool(self.conv(xq)), 1))
            return y, self.dyn(y.dequantize())

    net = Net()
    wc = torch.randn(32, 16, 3, 3) * 0.1
    net.conv.set_weight_bias(torch.quantize_per_channel(wc, wc.abs().amax(dim=(1, 2, 3)).double() / 127,
                                                        torch.zeros(32, dtype=torch.int64), 0, torch.qint8),
                             torch.randn(32))
    net.conv.scale, net.conv.zero_point = 0.05, 0
    wl = torch.randn(24, 128) * 0.1
    net.fc.set_weight_bias(torch.quantize_per_tensor(wl, float(wl.abs().max() / 127), 0, torch.qint8), torch.randn(24))
    net.fc.scale, net.fc.zero_point = 0.1, 128
    wd = torch.randn(10, 24) * 0.2
    net.dyn.set_weight_bias(torch.quantize_per_tensor(wd, float(wd.abs().max() / 127), 0, torch.qint8), torch.randn(10))
    xq = torch.quantize_per_tensor(torch.randn(3, 16, 8, 8), 0.03, 128, torch.quint8)
    q_cpu, f_cpu = net(xq)
    torch_musa_amd.quantized_modules_to(net, "cuda")
    q_gpu, f_gpu = net(xq.cuda())
    assert q_gpu.is_cuda and f_gpu.is_cuda
    d = (q_gpu.int_repr().cpu().int() - q_cpu.int_repr().int()).abs().max().item()
    assert d <= 1, f"quantized head differs by {d}"
    if d == 0:
        assert torch.equal(f_gpu.cpu(), f_cpu)
    # and back
    torch_musa_amd.quantized_modules_to(net, "cpu")
    q2, f2 = net(xq)
    assert torch.equal(q2.int_repr(), q_cpu.int_repr()) and torch.equal(f2, f_cpu)


@pytest.mark.parametrize("c", cases.qunary_cases(), ids=lambda c: c["name"])
def test_gelu_sigmoid_ops(golden, c):
    say("aten gelu / sigmoid", c["name"])
    xq = torch._make_per_tensor_quantized_tensor(torch.from_numpy(c["x"]).cuda(), c["scale"], c["zp"])
    for kind, fn in (("gelu", lambda t: torch.nn.functional.gelu(t)),
                     ("gelu_tanh", lambda t: torch.nn.functional.gelu(t, approximate="tanh")),
                     ("sigmoid", torch.sigmoid)):
        y = fn(xq)
        out_scale, out_zp = golden["qunary/" + c["name"] + "/" + kind + "/qparams"]
        assert y.is_cuda and y.is_quantized and y.q_scale() == out_scale and y.q_zero_point() == out_zp
        d = (y.int_repr().cpu().numpy().astype(np.int32)
             - golden["qunary/" + c["name"] + "/" + kind + "/y"].astype(np.int32))
        assert np.abs(d).max() <= 1 and np.count_nonzero(d) <= 0.001 * d.size + 1


@pytest.mark.parametrize("dtype,zp", [(torch.quint8, 128), (torch.qint8, -3)])
def test_aten_cat_and_upsample_nearest(dtype, zp):
    # the reference's test_concat and test_upsample_nearest2d (test_quantized_ops.py:394-462):
    # torch.cat and nearest-neighbour interpolation of quantized tensors against the CPU ops
    say("aten cat / upsample_nearest2d", dtype)
    torch.manual_seed(3)
    a = torch.quantize_per_tensor(torch.randn(2, 6, 5, 7), 0.05, zp, dtype)
    b = torch.quantize_per_tensor(torch.randn(2, 3, 5, 7), 0.05, zp, dtype)
    for dim in (1, 0, -1):
        x2 = a if dim != 1 else b
        assert_q_equal(torch.cat([a.cuda(), x2.cuda()], dim), torch.cat([a, x2], dim))
    for kw in (dict(scale_factor=2), dict(size=(7, 9)), dict(scale_factor=(1.5, 2.5))):
        for t in (a, a.contiguous(memory_format=torch.channels_last)):
            got = torch.nn.functional.interpolate(t.cuda(), mode="nearest", **kw)
            assert_q_equal(got, torch.nn.functional.interpolate(t, mode="nearest", **kw))
    m = torch.nn.Upsample(scale_factor=2, mode="nearest")
    assert_q_equal(m(b.cuda()), m(b))


@pytest.mark.parametrize("dtype,zp", [(torch.quint8, 128), (torch.qint8, -3)])
def test_cat_out_and_add_tensor(dtype, zp):
    # quantized::cat_out / aten::cat.out requantise into the parameters `out` carries
    # (reference: TensorShape.cpp:331-381); aten::add.Tensor with a quantized operand
    # gives the float sum (reference: mudnn/BinaryOps.cpp:11-31)
    say("aten cat_out / add.Tensor", dtype)
    torch.manual_seed(5)
    a = torch.quantize_per_tensor(torch.randn(2, 6, 5, 7), 0.05, zp, dtype)
    b = torch.quantize_per_tensor(torch.randn(2, 3, 5, 7), 0.03, zp + 2, dtype)

    def out_like(shape, device):
        return torch._empty_affine_quantized(shape, scale=0.07, zero_point=zp + 1, dtype=dtype, device=device)

    for dim, second in ((1, b), (0, a), (-1, a)):
        shape = list(torch.cat([a, second], dim).shape)
        want = torch.ops.quantized.cat_out([a, second], dim, out_like(shape, "cpu"))
        o = out_like(shape, "cuda")
        got = torch.ops.quantized.cat_out([a.cuda(), second.cuda()], dim, o)
        assert got.data_ptr() == o.data_ptr()
        assert_q_equal(got, want)
        o2 = out_like(shape, "cuda")
        assert torch.cat([a.cuda(), second.cuda()], dim, out=o2).data_ptr() == o2.data_ptr()
        assert_q_equal(o2, want)
    # an `out` that is not contiguous is filled in place as well
    base = out_like((2, 7, 5, 9), "cuda")
    view = base.permute(0, 3, 2, 1)[:, :, :, :]          # shape (2, 9, 5, 7), strided
    want = torch.ops.quantized.cat_out([a, b], 1, out_like((2, 9, 5, 7), "cpu"))
    torch.ops.quantized.cat_out([a.cuda(), b.cuda()], 1, view)
    assert_q_equal(view, want)
    with pytest.raises(RuntimeError):
        torch.ops.quantized.cat_out([a.cuda(), b.cuda()], 1, out_like((2, 8, 5, 7), "cuda"))
    with pytest.raises(RuntimeError):
        torch.ops.quantized.cat_out([a.cuda(), b.cuda()], 1,
                                    torch._empty_affine_quantized((2, 9, 5, 7), scale=0.1, zero_point=0,
                                                                  dtype=torch.qint8 if dtype == torch.quint8
                                                                  else torch.quint8, device="cuda"))

    f = torch.randn(2, 6, 5, 7)
    a2 = torch.quantize_per_tensor(torch.randn(2, 6, 5, 7), 0.02, zp, dtype)
    for x, y, want in ((a.cuda(), f.cuda(), a.dequantize() + f),
                       (f.cuda(), a.cuda(), f + a.dequantize()),
                       (a.cuda(), a2.cuda(), a.dequantize() + a2.dequantize())):
        got = torch.add(x, y)
        assert not got.is_quantized and got.dtype == torch.float32
        assert torch.equal(got.cpu(), want)
    assert torch.equal((a.cuda() + f.cuda()).cpu(), a.dequantize() + f)
    with pytest.raises(RuntimeError):
        torch.add(a.cuda(), f.cuda(), alpha=2)


def test_tensor_utilities_on_quantized_gpu_tensors():
    """The view, fill, select and reduction helpers the reference registers for its
    quantized device key (musa_functions.yaml: squeeze / unsqueeze / view / unfold /
    as_strided / fill_ / masked_fill_ / index_select / flip / max.dim / min.dim / clone /
    int_repr / empty_like / set_ and the q_* accessors) come from PyTorch-ROCm's own
    QuantizedCUDA kernels here: each must give what the CPU op gives."""
    say("aten tensor utilities on quantized tensors")
    torch.manual_seed(0)
    x = torch.randn(2, 3, 8, 8)
    q = torch.quantize_per_tensor(x, 0.05, 128, torch.quint8)

    def per_channel(t, d):
        return torch._make_per_channel_quantized_tensor(
            t.int_repr(), torch.tensor([0.1, 0.2, 0.3], dtype=torch.float64, device=d),
            torch.tensor([1, 2, 3], device=d), 1)

    def empty_q(shape, d):
        return torch._empty_affine_quantized(shape, scale=0.05, zero_point=128, dtype=torch.quint8, device=d)

    utilities = {
        "make_per_tensor": lambda t, d: torch._make_per_tensor_quantized_tensor(t.int_repr(), 0.1, 3),
        "make_per_channel": per_channel,
        "squeeze": lambda t, d: t[:1].squeeze(0),
        "unsqueeze": lambda t, d: t.unsqueeze(0),
        "fill_": lambda t, d: t.clone().fill_(0.5),
        "masked_fill_": lambda t, d: t.clone().masked_fill_(torch.arange(8, device=d) % 2 == 0, 1.0),
        "index_select": lambda t, d: torch.index_select(t, 1, torch.tensor([2, 0], device=d)),
        "index_select_out": lambda t, d: torch.index_select(t, 1, torch.tensor([2, 0], device=d),
                                                            out=empty_q((2, 2, 8, 8), d)),
        "as_strided": lambda t, d: torch.as_strided(t, (2, 3, 4, 4), (192, 64, 16, 2)),
        "relu_": lambda t, d: torch.relu_(t.clone()),
        "unfold": lambda t, d: t.unfold(2, 2, 2),
        "max.dim": lambda t, d: t.max(dim=1)[0],
        "min.dim": lambda t, d: t.min(dim=1, keepdim=True)[0],
        "flip": lambda t, d: t.flip(3),
        "clone": lambda t, d: t.clone(),
        "channels_last": lambda t, d: t.contiguous(memory_format=torch.channels_last),
        "permute": lambda t, d: t.permute(0, 2, 3, 1),
        "reshape": lambda t, d: t.reshape(6, 64),
        "view": lambda t, d: t.view(2, 3, 64),
        "slice": lambda t, d: t[:, 1:, ::2],
        "flatten": lambda t, d: torch.flatten(t, 1),
        "transpose": lambda t, d: t.transpose(1, 3),
        "copy_": lambda t, d: empty_q(t.shape, d).copy_(t),
        "empty_like": lambda t, d: torch.empty_like(t).copy_(t),
        "set_": lambda t, d: empty_q((0,), d).set_(t.untyped_storage(), 0, (2, 192), (192, 1)),
        "int_repr": lambda t, d: t.int_repr(),
        "dequantize per channel": lambda t, d: per_channel(t, d).dequantize(),
        "q_per_channel_zero_points": lambda t, d: per_channel(t, d).q_per_channel_zero_points(),
        "q_per_channel_axis": lambda t, d: per_channel(t, d).q_per_channel_axis(),
        "qscheme": lambda t, d: t.qscheme(),
        "to cpu": lambda t, d: t.cpu(),
    }
    g = q.cuda()
    for name, f in utilities.items():
        want, got = f(q, "cpu"), f(g, "cuda")
        if isinstance(want, torch.Tensor) and want.is_quantized:
            assert got.is_quantized, name
            if name != "to cpu":
                assert got.is_cuda, name
            assert got.shape == want.shape and got.qscheme() == want.qscheme(), name
            assert torch.equal(got.int_repr().cpu(), want.int_repr()), name
            assert torch.equal(got.dequantize().cpu(), want.dequantize()), name
        elif isinstance(want, torch.Tensor):
            assert torch.equal(got.cpu(), want), name
        else:
            assert got == want, name


@pytest.mark.parametrize("dtype", [torch.quint8, torch.qint8])
@pytest.mark.parametrize("cfg", [
    dict(in_channels=16, out_channels=32, kernel_size=3, stride=1, padding=1, dilation=1, groups=1, bias=True),
    dict(in_channels=32, out_channels=64, kernel_size=3, stride=2, padding=1, dilation=1, groups=1, bias=False),
    dict(in_channels=64, out_channels=64, kernel_size=1, stride=1, padding=0, dilation=1, groups=1, bias=True),
    dict(in_channels=32, out_channels=32, kernel_size=3, stride=1, padding=2, dilation=2, groups=2, bias=True),
], ids=lambda c: "{in_channels}to{out_channels}k{kernel_size}s{stride}g{groups}".format(**c))
def test_silu_conv_modules(cfg, dtype):
    """nniq.ConvSiLU2d / nniq.ConvAddSiLU2d the way the reference tests them
    (test_quantized_conv.py:236-375): weights through set_weight_bias, output parameters
    set on the module, result against quantize(silu(float conv of the dequantized
    operands [+ dequantized residual])) within 1 LSB."""
    import torch.ao.nn.intrinsic.quantized as nniq
    say("nniq SiLU conv modules", cfg, dtype)
    torch.manual_seed(41)
    zp = 128 if dtype == torch.quint8 else 0
    data = torch.randn(2, cfg["in_channels"], 14, 14)
    module = torch.nn.Conv2d(**cfg)
    fweight, fbias = module.weight.detach(), None if module.bias is None else module.bias.detach()
    qweight = torch.quantize_per_tensor(fweight, float(fweight.abs().max() / 2 ** 7), 0, torch.qint8)
    qdata = torch.quantize_per_tensor(data, float(data.abs().max()) / 2 ** 7, zp, dtype)
    with torch.no_grad():
        conv_out = torch.nn.functional.conv2d(qdata.dequantize(), qweight.dequantize(), fbias, cfg["stride"],
                                              cfg["padding"], cfg["dilation"], cfg["groups"])
    accum = torch.randn_like(conv_out)
    qaccum = torch.quantize_per_tensor(accum, float(accum.abs().max()) / 2 ** 7, zp, dtype)

    for cls, extra, want_f in (
            (nniq.ConvSiLU2d, (), torch.nn.functional.silu(conv_out)),
            (nniq.ConvAddSiLU2d, (qaccum.cuda(),), torch.nn.functional.silu(conv_out + qaccum.dequantize()))):
        qmodule = cls(**cfg)
        qmodule.set_weight_bias(qweight.cuda(), None if fbias is None else fbias.cuda())
        out_scale = float(want_f.abs().max() / 2 ** 7)
        qmodule.scale, qmodule.zero_point = out_scale, zp
        got = qmodule(qdata.cuda(), *extra)
        want = torch.quantize_per_tensor(want_f, out_scale, zp, dtype)
        assert got.is_cuda and got.dtype == dtype and got.shape == want.shape
        assert got.q_scale() == out_scale and got.q_zero_point() == zp
        d = (got.int_repr().cpu().int() - want.int_repr().int()).abs()
        assert d.max() <= 1, f"{cls.__name__}: differs by {d.max()}"
        w_back, b_back = qmodule._weight_bias()
        assert torch.equal(w_back.int_repr().cpu(), qweight.int_repr())
        assert (b_back is None) == (fbias is None)
        with pytest.raises(ValueError):
            qmodule(qdata.cuda()[0], *extra)


def test_silu_conv_eager_workflow_to_gpu():
    """Float model with the fused containers -> prepare -> calibrate -> convert with the
    package's mapping (all on the CPU) -> quantized_modules_to("cuda") -> forward; the
    quantized model stays close to the float one and equals the ops called by hand."""
    import torch.ao.quantization as tq
    from torch_musa_amd import ao, quantized_modules_to
    say("eager quantization workflow with SiLU convolutions")
    torch.manual_seed(11)

    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.quant = tq.QuantStub()
            self.stem = ao.fused.ConvSiLU2d(torch.nn.Conv2d(3, 16, 3, padding=1), torch.nn.SiLU())
            self.body = ao.fused.ConvAddSiLU2d(torch.nn.Conv2d(16, 16, 3, padding=1), torch.add, torch.nn.SiLU())
            self.dequant = tq.DeQuantStub()

        def forward(self, x):
            h = self.stem(self.quant(x))
            return self.dequant(self.body(h, h))

    net = Net().eval()
    x = torch.randn(4, 3, 24, 24)
    with torch.no_grad():
        want = net(x)
    import warnings
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        net.qconfig = tq.get_default_qconfig("fbgemm")
        prepared = tq.prepare(net)
        prepared(x)
        mapping = dict(tq.get_default_static_quant_module_mappings())
        mapping.update(ao.STATIC_QUANT_MODULE_MAPPINGS)
        qnet = tq.convert(prepared, mapping=mapping)
    assert type(qnet.stem) is ao.quantized.ConvSiLU2d and type(qnet.body) is ao.quantized.ConvAddSiLU2d
    quantized_modules_to(qnet, "cuda")
    got = qnet(x.cuda())
    assert got.is_cuda and not got.is_quantized and got.shape == want.shape
    err = (got.cpu() - want).abs().max().item()
    assert err < 0.06 * want.abs().max().item(), err
    # the same three steps by hand
    xq = torch.quantize_per_tensor(x.cuda(), float(qnet.quant.scale), int(qnet.quant.zero_point), torch.quint8)
    h = torch.ops.quantized.conv2d_silu(xq, qnet.stem._packed_params, qnet.stem.scale, qnet.stem.zero_point)
    y = torch.ops.quantized.conv2d_add_silu(h, h, qnet.body._packed_params, qnet.body.scale, qnet.body.zero_point)
    assert torch.equal(y.dequantize(), got)


def test_silu_conv_qat_on_gpu_then_int8():
    """Quantization-aware training of the fused SiLU convolution on the GPU (PyTorch-ROCm's
    fake-quantize kernels), then `from_float` on the device: weights are quantized and packed
    there, and the int8 module reproduces the QAT module's own fake-quantized forward pass
    to within one output step."""
    import copy
    import warnings
    import torch.ao.quantization as tq
    from torch_musa_amd import ao
    say("QAT ConvBnSiLU2d on the GPU -> quantized ConvSiLU2d")
    torch.manual_seed(17)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        qconfig = tq.get_default_qat_qconfig("fbgemm")
        float_mod = ao.fused.ConvBnSiLU2d(torch.nn.Conv2d(8, 16, 3, padding=1), torch.nn.BatchNorm2d(16),
                                          torch.nn.SiLU()).train()
        float_mod.qconfig = qconfig
        tq.propagate_qconfig_(float_mod)
        qat = ao.qat.ConvBnSiLU2d.from_float(float_mod).cuda()
        qat.activation_post_process = qconfig.activation().cuda()
        in_obs = qconfig.activation().cuda()
    opt = torch.optim.SGD(qat.parameters(), lr=0.01)
    x = torch.randn(8, 8, 12, 12, device="cuda")
    for _ in range(4):
        opt.zero_grad()
        y = qat.activation_post_process(qat(in_obs(x)))
        y.square().mean().backward()
        opt.step()
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in qat.parameters())
    qat.eval()
    in_obs.disable_observer()
    qat.apply(tq.disable_observer)
    with torch.no_grad():
        want = qat.activation_post_process(qat(in_obs(x)))       # fake-quantized end to end
    on_cpu = copy.deepcopy(qat).cpu()
    q = ao.quantized.ConvSiLU2d.from_float(qat)
    assert type(q) is ao.quantized.ConvSiLU2d
    w, b = q._weight_bias()
    assert w.is_cuda and b.is_cuda
    q_cpu = ao.quantized.ConvSiLU2d.from_float(on_cpu)           # same conversion on the CPU
    assert (w.int_repr().cpu().int() - q_cpu.weight().int_repr().int()).abs().max() <= 1
    assert torch.allclose(b.cpu(), q_cpu.bias(), rtol=1e-5, atol=1e-6)
    assert q.scale == pytest.approx(q_cpu.scale, rel=1e-6) and q.zero_point == q_cpu.zero_point
    s_in, z_in = in_obs.calculate_qparams()
    xq = torch.quantize_per_tensor(x, float(s_in), int(z_in), torch.quint8)
    got = q(xq)
    assert got.is_cuda and got.q_scale() == q.scale
    steps = ((got.dequantize() - want).abs().max() / q.scale).item()
    assert steps <= 1.01, steps


def test_fake_quantize_ops_on_gpu_tensors():
    """The fake-quantize operators quantization-aware training runs on (the reference tests
    its own device kernels for them, test_quantized_ops.py:465-700) are PyTorch-ROCm's own
    GPU kernels here; each gives the CPU op's values to 1e-6 (relative for the summed gradients), masks included."""
    say("fake-quantize ops against the CPU ops")
    torch.manual_seed(9)
    aten = torch.ops.aten

    def close(got, want):
        got = got if isinstance(got, (tuple, list)) else (got,)
        want = want if isinstance(want, (tuple, list)) else (want,)
        for g_, w_ in zip(got, want):
            assert g_.is_cuda and g_.dtype == w_.dtype and g_.shape == w_.shape
            if w_.dtype == torch.bool:
                assert torch.equal(g_.cpu(), w_)
            else:
                # (summed gradients: the order of the sum differs, so relative to their size)
                assert (g_.cpu().double() - w_.double()).abs().max().item() <= 1e-6 * max(1.0, w_.abs().max().item())

    for shape, qmin, qmax, axis in (((2, 2), 0, 255, 1), ((2, 3, 16), 0, 255, 1), ((1, 4, 8, 8), 0, 127, 1),
                                    ((2, 2, 32), 0, 240, 1)):
        x = torch.randn(shape) * 4
        scale = torch.rand(shape[axis]) * 0.1 + 0.01
        zp = torch.randint(0, 10, (shape[axis],)).float()
        close(aten.fake_quantize_per_channel_affine_cachemask(x.cuda(), scale.cuda(), zp.cuda(), axis, qmin, qmax),
              aten.fake_quantize_per_channel_affine_cachemask(x, scale, zp, axis, qmin, qmax))
        outs = []
        for dev_ in ("cpu", "cuda"):
            xi, si, zi = (t.clone().to(dev_).requires_grad_(True) for t in (x, scale, zp))
            y = aten._fake_quantize_learnable_per_channel_affine(xi, si, zi, axis, qmin, qmax, 1.0)
            y.sum().backward()
            outs.append((y.detach(), xi.grad, si.grad, zi.grad))
        close(outs[1], outs[0])
    for shape, qmin, qmax, scale, zp in (((2, 2), 0, 255, 0.1, 4), ((2, 3, 16), 0, 255, 0.2, 254),
                                         ((1, 4, 8, 8), 0, 127, 10.0, 1), ((2, 2, 32), 10, 240, 1.0, 100)):
        x = torch.randn(shape) * 40
        s_t, z_t = torch.tensor(scale), torch.tensor(zp, dtype=torch.int)
        close(aten.fake_quantize_per_tensor_affine_cachemask(x.cuda(), scale, zp, qmin, qmax),
              aten.fake_quantize_per_tensor_affine_cachemask(x, scale, zp, qmin, qmax))
        on = torch.tensor(1, dtype=torch.long)
        close(aten._fake_quantize_per_tensor_affine_cachemask_tensor_qparams(x.cuda(), s_t.cuda(), z_t.cuda(),
                                                                             on.cuda(), qmin, qmax),
              aten._fake_quantize_per_tensor_affine_cachemask_tensor_qparams(x, s_t, z_t, on, qmin, qmax))
        outs = []
        for dev_ in (("cpu", "cuda") if qmin == 0 else ()):   # (the learnable form wants 0 inside the range)
            xi = x.clone().to(dev_).requires_grad_(True)
            si = torch.tensor([scale], device=dev_, requires_grad=True)
            zi = torch.tensor([float(zp)], device=dev_, requires_grad=True)
            y = aten._fake_quantize_learnable_per_tensor_affine(xi, si, zi, qmin, qmax, 1.0)
            y.sum().backward()
            outs.append((y.detach(), xi.grad, si.grad, zi.grad))
        if outs:
            close(outs[1], outs[0])
    # the fused observer + fake-quantize step of torch.ao's FusedMovingAvgObsFakeQuantize
    x = torch.randn(4, 8, 6, 6)
    outs = []
    for dev_ in ("cpu", "cuda"):
        st = dict(obs=torch.tensor(1, dtype=torch.int, device=dev_), fq=torch.tensor(1, dtype=torch.int, device=dev_),
                  mn=torch.tensor([float("inf")], device=dev_), mx=torch.tensor([float("-inf")], device=dev_),
                  sc=torch.ones(1, device=dev_), zp=torch.zeros(1, dtype=torch.int, device=dev_))
        y = None
        for k in range(3):
            y = torch.fused_moving_avg_obs_fake_quant(x.to(dev_) * (k + 1), st["obs"], st["fq"], st["mn"], st["mx"],
                                                      st["sc"], st["zp"], 0.01, 0, 255, 0, False, False)
        outs.append((y, st["mn"], st["mx"], st["sc"], st["zp"]))
    close(outs[1], outs[0])


def test_ops_replay_from_a_hip_graph():
    """The operators inside a captured HIP graph (allocations from the graph's pool, no
    host round trip in the captured region): quantized::linear on a split-K shape and on a
    large-tile shape, quantized::linear_dynamic, quantized::conv2d_relu and quantized::add.
    Every replay, with new input contents and eager work in between, equals the eager
    result."""
    say("graph replay")
    torch.manual_seed(21)
    dev = "cuda"
    w1 = torch.randn(192, 8192) * 0.05
    wq1 = torch.quantize_per_tensor(w1, float(w1.abs().max() / 127), 0, torch.qint8).cuda()
    p1 = torch.ops.quantized.linear_prepack(wq1, torch.randn(192).cuda())
    w2 = torch.randn(64, 32, 3, 3) * 0.05
    s2 = (w2.abs().amax(dim=(1, 2, 3)) / 127).double()
    wq2 = torch.quantize_per_channel(w2, s2, torch.zeros(64, dtype=torch.int64), 0, torch.qint8).cuda()
    p2 = torch.ops.quantized.conv2d_prepack(wq2, torch.randn(64).cuda(), [1, 1], [1, 1], [1, 1], 1)
    xf = torch.randn(130, 8192, device=dev)                         # float activations (dynamic linear)
    xq = torch.quantize_per_tensor(torch.randn(130, 8192, device=dev), 0.04, 120, torch.quint8)
    xc = torch.quantize_per_tensor(torch.randn(2, 32, 20, 20, device=dev).relu(), 0.03, 0, torch.quint8).contiguous(
        memory_format=torch.channels_last)

    x1 = torch.randn(2, 8192, device=dev)                           # two rows: the one-launch dynamic linear

    def work():
        y1 = torch.ops.quantized.linear(xq, p1, 0.3, 128)
        y2 = torch.ops.quantized.linear_dynamic(xf, p1, False)
        y5 = torch.ops.quantized.linear_dynamic(x1, p1, False)
        y3 = torch.ops.quantized.conv2d_relu(xc, p2, 0.05, 0)
        y4 = torch.ops.quantized.add(y3, y3, 0.1, 0)
        return y1, y2, y3, y4, y5

    work()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        work()
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            outs = work()
    torch.cuda.synchronize()
    for it in range(3):
        # new contents in the captured input buffers
        xf.copy_(torch.randn(130, 8192, device=dev) * (1.0 + it))
        x1.copy_(torch.randn(2, 8192, device=dev) * (2.0 + it))
        xq_new = torch.quantize_per_tensor(torch.randn(130, 8192, device=dev) * (1.0 + 0.3 * it), 0.04, 120, torch.quint8)
        xq.copy_(xq_new)
        xc.copy_(torch.quantize_per_tensor(torch.randn(2, 32, 20, 20, device=dev).relu() * (1.0 + it), 0.03, 0,
                                           torch.quint8).contiguous(memory_format=torch.channels_last))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        eager = work()
        torch.cuda.synchronize()
        for got, want in zip(outs, eager):
            if got.is_quantized:
                assert torch.equal(got.int_repr(), want.int_repr()), f"replay {it}"
            else:
                assert torch.equal(got, want), f"replay {it}"


# ---- interface leftovers ------------------------------------------------------------------
def test_quantize_per_tensor_with_tensor_qparams():
    # aten::quantize_per_tensor.tensor_qparams (musa_functions.yaml:3527-3531): scale and
    # zero point arrive as one-element tensors
    say("aten qpt tensor_qparams")
    torch.manual_seed(41)
    x = torch.randn(5, 33, 7)
    for dtype, zp in ((torch.quint8, 121), (torch.qint8, -4)):
        scale = torch.tensor(float(x.abs().max()) / 120)
        zpt = torch.tensor(zp, dtype=torch.int64)
        want = torch.quantize_per_tensor(x, scale, zpt, dtype)
        got = torch.quantize_per_tensor(x.cuda(), scale.cuda(), zpt.cuda(), dtype)
        assert_q_equal(got, want)


@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("groups,stride,padding,dilation", [(1, 1, 1, 1), (2, 2, 3, 2)])
def test_qconv1d_matches_cpu_op(relu, groups, stride, padding, dilation):
    # quantized::conv1d_prepack (mudnn/ConvPrepack.cpp:159-221) and quantized::conv1d{,_relu}
    say("conv1d", relu, groups, stride, padding, dilation)
    torch.manual_seed(41)
    x = torch.randn(3, 32, 50)
    w = torch.randn(48, 32 // groups, 5) * 0.1
    b = torch.randn(48)
    xq = torch.quantize_per_tensor(x, float(x.abs().max()) / 127, 128, torch.quint8)
    wq = torch.quantize_per_channel(w, w.abs().amax(dim=(1, 2)).double() / 127,
                                    torch.zeros(48, dtype=torch.int64), 0, torch.qint8)
    op = torch.ops.quantized.conv1d_relu if relu else torch.ops.quantized.conv1d
    pc = torch.ops.quantized.conv1d_prepack(wq, b, [stride], [padding], [dilation], groups)
    want = op(xq, pc, 0.08, 100)
    pg = torch.ops.quantized.conv1d_prepack(wq.cuda(), b.cuda(), [stride], [padding], [dilation], groups)
    got = op(xq.cuda(), pg, 0.08, 100)
    assert got.dim() == 3
    assert_q_equal(got, want, abs_diff=LSB_TOL)
    wu, bu = torch.ops.quantized.conv1d_unpack(pg)
    assert wu.is_cuda and wu.dim() == 3 and torch.equal(wu.int_repr().cpu(), wq.int_repr())
    assert torch.equal(bu.cpu(), b)


def test_qconv2d_prepack_wide_input():
    # 1x1 weights with 2048 input channels (ResNet-50 layer4): the packed size must not
    # depend on an image size
    say("conv prepack 2048 -> 512")
    torch.manual_seed(2)
    x = torch.randn(2, 2048, 7, 7)
    w = torch.randn(512, 2048, 1, 1) * 0.02
    xq = torch.quantize_per_tensor(x, float(x.abs().max()) / 255, 128, torch.quint8)
    wq = torch.quantize_per_tensor(w, float(w.abs().max()) / 127, 0, torch.qint8)
    pc = torch.ops.quantized.conv2d_prepack(wq, None, [1, 1], [0, 0], [1, 1], 1)
    pg = torch.ops.quantized.conv2d_prepack(wq.cuda(), None, [1, 1], [0, 0], [1, 1], 1)
    want = torch.ops.quantized.conv2d(xq, pc, 0.05, 128)
    got = torch.ops.quantized.conv2d(xq.cuda(), pg, 0.05, 128)
    assert_q_equal(got, want, abs_diff=LSB_TOL)


def test_qlinear_without_input_features():
    # K == 0: the product is empty and every row is the requantised bias
    say("linear K = 0")
    b = torch.tensor([0.0, 1.0, -2.0, 300.0])
    wq = torch.quantize_per_tensor(torch.zeros(4, 0), 0.1, 0, torch.qint8)
    xq = torch.quantize_per_tensor(torch.zeros(3, 0), 0.1, 128, torch.quint8)
    pg = torch.ops.quantized.linear_prepack(wq.cuda(), b.cuda())
    y = torch.ops.quantized.linear(xq.cuda(), pg, 0.5, 10)
    want = torch.quantize_per_tensor(b, 0.5, 10, torch.quint8).int_repr()
    assert y.shape == (3, 4) and torch.equal(y.int_repr().cpu(), want.expand(3, 4))
    yd = torch.ops.quantized.linear_dynamic(torch.zeros(3, 0).cuda(), pg)
    assert torch.equal(yd.cpu(), b.expand(3, 4))
    yr = torch.ops.quantized.linear_relu_dynamic(torch.zeros(3, 0).cuda(), pg)
    assert torch.equal(yr.cpu(), b.clamp_min(0).expand(3, 4))


def test_saved_modules_with_gpu_packed_params(tmp_path):
    """torch.save / torch.load / deepcopy of modules whose packed parameters live on the GPU
    (the limitation the reference notes at test_quantized_linear.py:56-60,87-89).  The
    pickled state of a packed-parameter object is its unpacked weight, and PyTorch's
    unpickling re-packs it with the CPU engine whatever device the weight is on; so the
    supported routes are: load onto the CPU (map_location) or move to the CPU first, then
    quantized_modules_to(..., "cuda"); or carry the state dict."""
    import copy
    import torch_musa_amd
    say("save / load of packed modules")
    torch.manual_seed(9)
    lin = nnq.Linear(64, 32)
    w = torch.randn(32, 64) * 0.1
    lin.set_weight_bias(torch.quantize_per_channel(w, w.abs().amax(dim=1).double() / 127,
                                                   torch.zeros(32, dtype=torch.int64), 0, torch.qint8),
                        torch.randn(32))
    lin.scale, lin.zero_point = 0.1, 128
    conv = nniq.ConvReLU2d(16, 8, 3, padding=1)
    wc = torch.randn(8, 16, 3, 3) * 0.1
    conv.set_weight_bias(torch.quantize_per_tensor(wc, float(wc.abs().max()) / 127, 0, torch.qint8), torch.randn(8))
    conv.scale, conv.zero_point = 0.05, 0
    net = torch.nn.ModuleDict({"lin": lin, "conv": conv})
    xl = torch.quantize_per_tensor(torch.randn(5, 64), 0.03, 128, torch.quint8)
    xc = torch.quantize_per_tensor(torch.randn(2, 16, 9, 9), 0.03, 128, torch.quint8)
    want_l, want_c = net["lin"](xl).int_repr(), net["conv"](xc).int_repr()

    def check_gpu(m, what):
        assert m["lin"]._weight_bias()[0].is_cuda and m["conv"]._weight_bias()[0].is_cuda, what
        assert torch.equal(m["lin"](xl.cuda()).int_repr().cpu(), want_l), what
        assert torch.equal(m["conv"](xc.cuda()).int_repr().cpu(), want_c), what

    def check_cpu(m, what):
        assert not m["lin"]._weight_bias()[0].is_cuda, what
        assert torch.equal(m["lin"](xl).int_repr(), want_l) and torch.equal(m["conv"](xc).int_repr(), want_c), what

    torch_musa_amd.quantized_modules_to(net, "cuda")
    check_gpu(net, "moved")
    path = str(tmp_path / "net.pt")
    # whole-module pickles: the linear module only (PyTorch's quantized conv modules do not
    # survive pickle.load on any device: their __setstate__ skips Module.__init__)
    torch.save(net["lin"], path)               # GPU packed parameters pickle as their unpacked GPU weights
    lin_cpu = torch.load(path, weights_only=False, map_location="cpu")   # a file this test wrote
    assert not lin_cpu._weight_bias()[0].is_cuda and torch.equal(lin_cpu(xl).int_repr(), want_l)
    torch_musa_amd.quantized_modules_to(lin_cpu, "cuda")
    assert lin_cpu._weight_bias()[0].is_cuda and torch.equal(lin_cpu(xl.cuda()).int_repr().cpu(), want_l)
    # deepcopy: through the CPU
    torch_musa_amd.quantized_modules_to(net, "cpu")
    twin = copy.deepcopy(net)
    check_cpu(twin, "deepcopy on the CPU")
    check_gpu(torch_musa_amd.quantized_modules_to(twin, "cuda"), "deepcopy, then moved")
    check_gpu(torch_musa_amd.quantized_modules_to(net, "cuda"), "moved back")
    # the state dict alone (GPU tensors inside), into a fresh CPU model, then moved
    fresh = torch.nn.ModuleDict({"lin": nnq.Linear(64, 32), "conv": nniq.ConvReLU2d(16, 8, 3, padding=1)})
    torch.save(net.state_dict(), path)
    fresh.load_state_dict(torch.load(path, map_location="cpu", weights_only=False))
    check_cpu(fresh, "state dict")
    check_gpu(torch_musa_amd.quantized_modules_to(fresh, "cuda"), "state dict, then moved")
