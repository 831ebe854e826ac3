"""Host-side logic of the fused SiLU convolution modules (torch_musa_amd.ao): the
names they are published under, the QAT forms against PyTorch's own float
arithmetic, and the conversion to the quantized modules (weights, bias, output
parameters) against what PyTorch's ConvReLU2d conversion gives for the same
convolution.  No GPU: the quantized forward pass is tested in
test_gpu_aten_ops.py."""
import copy

import pytest
import torch
import torch.ao.nn.intrinsic as nni
import torch.ao.nn.intrinsic.qat as nniqat
import torch.ao.nn.intrinsic.quantized as nniq
import torch.ao.quantization as tq
import torch.nn.functional as F

import torch_musa_amd
from torch_musa_amd import ao

pytestmark = [pytest.mark.filterwarnings("ignore::DeprecationWarning"),
              pytest.mark.filterwarnings("ignore::UserWarning")]


@pytest.fixture(autouse=True)
def _engine():
    torch.backends.quantized.engine = "fbgemm"


def test_published_names():
    # reference: torch_musa/core/ao/register_helper.py:12-20
    assert torch_musa_amd.is_loaded()
    assert nni.ConvSiLU2d is ao.fused.ConvSiLU2d and nni.ConvBnSiLU2d is ao.fused.ConvBnSiLU2d
    assert nni.ConvAddSiLU2d is ao.fused.ConvAddSiLU2d
    assert nniq.ConvSiLU2d is ao.quantized.ConvSiLU2d and nniq.ConvAddSiLU2d is ao.quantized.ConvAddSiLU2d
    assert nniqat.ConvSiLU2d is ao.qat.ConvSiLU2d and nniqat.ConvBnSiLU2d is ao.qat.ConvBnSiLU2d
    assert repr(nniq.ConvSiLU2d(4, 8, 3)).startswith("QuantizedConvSiLU2d(4, 8")
    assert repr(nniq.ConvAddSiLU2d(4, 8, 3)).startswith("QuantizedConvAddSiLU2d(4, 8")


def test_float_containers():
    torch.manual_seed(1)
    conv, bn, silu = torch.nn.Conv2d(4, 6, 3, padding=1), torch.nn.BatchNorm2d(6), torch.nn.SiLU()
    x, r = torch.randn(2, 4, 5, 5), torch.randn(2, 6, 5, 5)
    assert torch.equal(ao.fused.ConvSiLU2d(conv, silu)(x), F.silu(conv(x)))
    bn.eval()
    assert torch.equal(ao.fused.ConvBnSiLU2d(conv, bn, silu)(x), F.silu(bn(conv(x))))
    m = ao.fused.ConvAddSiLU2d(conv, torch.add, silu)
    assert torch.equal(m(x, r), F.silu(conv(x) + r)) and m[0] is conv
    with pytest.raises(AssertionError):
        ao.fused.ConvSiLU2d(conv, torch.nn.ReLU())
    with pytest.raises(AssertionError):
        ao.fused.ConvBnSiLU2d(conv, torch.nn.BatchNorm1d(6), silu)


def test_qat_modules_match_float_arithmetic():
    torch.manual_seed(2)
    qconfig = tq.get_default_qat_qconfig("fbgemm")
    x = torch.randn(3, 4, 7, 7)

    conv = torch.nn.Conv2d(4, 6, 3, padding=1)
    float_mod = ao.fused.ConvSiLU2d(copy.deepcopy(conv), torch.nn.SiLU())
    float_mod.qconfig = qconfig
    tq.propagate_qconfig_(float_mod)
    qat = ao.qat.ConvSiLU2d.from_float(float_mod)
    assert type(qat) is ao.qat.ConvSiLU2d
    relu_twin = nni.ConvReLU2d(copy.deepcopy(conv), torch.nn.ReLU())
    relu_twin.qconfig = qconfig
    tq.propagate_qconfig_(relu_twin)
    twin = nniqat.ConvReLU2d.from_float(relu_twin)
    torch.manual_seed(3)
    got = qat(x)
    # same convolution of the same fake-quantized weight; only the activation differs
    want = F.silu(twin._conv_forward(x, twin.weight_fake_quant(twin.weight), twin.bias))
    assert torch.equal(got, want)
    back = qat.to_float()
    assert type(back) is ao.fused.ConvSiLU2d and type(back[1]) is torch.nn.SiLU
    with pytest.raises(AssertionError):
        ao.qat.ConvSiLU2d(4, 6, 3)

    bn = torch.nn.BatchNorm2d(6)
    float_bn = ao.fused.ConvBnSiLU2d(copy.deepcopy(conv), bn, torch.nn.SiLU())
    float_bn.qconfig = qconfig
    tq.propagate_qconfig_(float_bn)
    float_bn.train()
    qat_bn = ao.qat.ConvBnSiLU2d.from_float(float_bn)
    assert type(qat_bn) is ao.qat.ConvBnSiLU2d
    relu_bn = nni.ConvBnReLU2d(copy.deepcopy(conv), copy.deepcopy(bn), torch.nn.ReLU())
    relu_bn.qconfig = qconfig
    tq.propagate_qconfig_(relu_bn)
    relu_bn.train()
    twin_bn = nniqat.ConvBnReLU2d.from_float(relu_bn)
    assert torch.equal(qat_bn(x), F.silu(twin_bn._forward(x)))
    qat_bn.eval()
    back = qat_bn.to_float()
    assert type(back) is ao.fused.ConvSiLU2d and type(back[1]) is torch.nn.SiLU


def _observed(float_mod, x, *more):
    # `prepare` gives a fused container one output observer when it meets it as a child
    class Holder(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.child = float_mod

        def forward(self, *args):
            return self.child(*args)

    holder = Holder()
    holder.qconfig = tq.get_default_qconfig("fbgemm")
    prepared = tq.prepare(holder, inplace=False)
    prepared(x, *more)
    return prepared.child


def test_quantized_modules_from_float():
    torch.manual_seed(4)
    x = torch.randn(2, 8, 9, 9)
    conv = torch.nn.Conv2d(8, 12, 3, stride=2, padding=1)

    prepared = _observed(ao.fused.ConvSiLU2d(copy.deepcopy(conv), torch.nn.SiLU()), x)
    q = nniq.ConvSiLU2d.from_float(prepared)
    twin = nniq.ConvReLU2d.from_float(_observed(nni.ConvReLU2d(copy.deepcopy(conv), torch.nn.ReLU()), x))
    assert type(q) is ao.quantized.ConvSiLU2d
    assert q.stride == (2, 2) and q.padding == (1, 1) and q.in_channels == 8 and q.out_channels == 12
    assert torch.equal(q.weight().int_repr(), twin.weight().int_repr())
    assert torch.equal(q.weight().q_per_channel_scales(), twin.weight().q_per_channel_scales())
    assert torch.equal(q.bias(), twin.bias())
    # the output observer saw silu(conv(x)), not relu(conv(x))
    y = F.silu(conv(x))
    obs = tq.get_default_qconfig("fbgemm").activation()
    obs(y)
    s, z = obs.calculate_qparams()
    assert q.scale == float(s) and q.zero_point == int(z)

    r = torch.randn(2, 12, 5, 5)
    prepared = _observed(ao.fused.ConvAddSiLU2d(copy.deepcopy(conv), torch.add, torch.nn.SiLU()), x, r)
    qa = nniq.ConvAddSiLU2d.from_float(prepared)
    assert type(qa) is ao.quantized.ConvAddSiLU2d
    assert torch.equal(qa.weight().int_repr(), twin.weight().int_repr())
    assert torch.equal(qa.bias(), twin.bias())

    with pytest.raises(AssertionError):
        nniq.ConvSiLU2d.from_float(_observed(torch.nn.Sequential(copy.deepcopy(conv)), x))


def test_quantized_module_from_qat_folds_the_batch_norm():
    torch.manual_seed(5)
    qconfig = tq.get_default_qat_qconfig("fbgemm")
    x = torch.randn(4, 4, 6, 6)
    conv, bn = torch.nn.Conv2d(4, 6, 3, padding=1), torch.nn.BatchNorm2d(6)
    with torch.no_grad():
        bn.weight.uniform_(0.5, 1.5)
        bn.bias.normal_()

    def trained(container, qat_cls):
        container.qconfig = qconfig
        tq.propagate_qconfig_(container)
        container.train()
        m = qat_cls.from_float(container)
        m.activation_post_process = qconfig.activation()
        torch.manual_seed(6)
        for _ in range(3):
            m.activation_post_process(m(x))
        m.eval()
        return m

    silu = trained(ao.fused.ConvBnSiLU2d(copy.deepcopy(conv), copy.deepcopy(bn), torch.nn.SiLU()),
                   ao.qat.ConvBnSiLU2d)
    relu = trained(nni.ConvBnReLU2d(copy.deepcopy(conv), copy.deepcopy(bn), torch.nn.ReLU()),
                   nniqat.ConvBnReLU2d)
    q = nniq.ConvSiLU2d.from_float(silu)
    twin = nniq.ConvReLU2d.from_float(relu)
    assert type(q) is ao.quantized.ConvSiLU2d
    assert torch.equal(q.weight().int_repr(), twin.weight().int_repr())
    assert torch.allclose(q.bias(), twin.bias())
    assert not torch.equal(q.weight().dequantize(), conv.weight)   # batch norm folded in


def test_convert_with_the_mapping():
    torch.manual_seed(7)

    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.quant = tq.QuantStub()
            self.block = ao.fused.ConvSiLU2d(torch.nn.Conv2d(3, 8, 3, padding=1), torch.nn.SiLU())
            self.dequant = tq.DeQuantStub()

        def forward(self, x):
            return self.dequant(self.block(self.quant(x)))

    net = Net().eval()
    net.qconfig = tq.get_default_qconfig("fbgemm")
    prepared = tq.prepare(net)
    prepared(torch.randn(2, 3, 8, 8))
    mapping = dict(tq.get_default_static_quant_module_mappings())
    mapping.update(ao.STATIC_QUANT_MODULE_MAPPINGS)
    converted = tq.convert(prepared, mapping=mapping)
    assert type(converted.block) is ao.quantized.ConvSiLU2d
    state = converted.state_dict()
    assert "block.scale" in state and "block.zero_point" in state
    clone = ao.quantized.ConvSiLU2d(3, 8, 3, padding=1)
    clone.load_state_dict({k[len("block."):]: v for k, v in state.items() if k.startswith("block.")})
    assert torch.equal(clone.weight().int_repr(), converted.block.weight().int_repr())
    assert clone.scale == converted.block.scale and clone.zero_point == converted.block.zero_point
