"""Quantization-aware-training forms of the SiLU-fused convolutions: the weight goes
through a FakeQuantize module, the activation is SiLU (reference:
torch_musa/core/ao/nn/intrinsic/qat/modules/conv_fused.py:19-144).  They train on
PyTorch's own float kernels; `torch_musa_amd.ao.quantized.ConvSiLU2d.from_float`
turns either into the int8 module."""
import torch
import torch.ao.nn.intrinsic as nni
import torch.ao.nn.qat as nnqat
import torch.nn.functional as F

from . import fused

__all__ = ["ConvBnSiLU2d", "ConvSiLU2d"]


class ConvBnSiLU2d(nni.qat.ConvBn2d):
    """Conv2d + BatchNorm2d + SiLU with a fake-quantized, batch-norm-folded weight."""

    _FLOAT_MODULE = fused.ConvBnSiLU2d
    _FLOAT_CONV_MODULE = torch.nn.Conv2d
    _FLOAT_BN_MODULE = torch.nn.BatchNorm2d
    _FLOAT_RELU_MODULE = torch.nn.SiLU      # the slot `to_float` puts after the convolution
    _FUSED_FLOAT_MODULE = fused.ConvSiLU2d  # what remains once the batch norm is folded

    def forward(self, input):  # pylint: disable=redefined-builtin
        return F.silu(self._forward(input))


class ConvSiLU2d(nnqat.Conv2d, nni._FusedModule):
    """Conv2d + SiLU with a fake-quantized weight."""

    _FLOAT_MODULE = fused.ConvSiLU2d
    _FLOAT_CONV_MODULE = torch.nn.Conv2d
    _FLOAT_BN_MODULE = None
    _FLOAT_RELU_MODULE = torch.nn.SiLU

    def __init__(self, *args, qconfig=None, **kwargs):
        assert qconfig, "qconfig must be provided for QAT module"
        super().__init__(*args, qconfig=qconfig, **kwargs)

    def forward(self, input):  # pylint: disable=redefined-builtin
        return F.silu(self._conv_forward(input, self.weight_fake_quant(self.weight), self.bias))
