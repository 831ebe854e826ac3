"""Quantized modules over `quantized::conv2d_silu` and `quantized::conv2d_add_silu`
(reference: torch_musa/core/ao/nn/intrinsic/quantized/modules/conv_silu.py:21-98,
conv_add.py:15-78; used by tests/unittest/quantized/test_quantized_conv.py:236-375).
Same constructor, `set_weight_bias`, `scale` / `zero_point` and state dict as
`torch.ao.nn.quantized.Conv2d`; the two ops exist for GPU tensors only, so a module
built on the CPU (`from_float`) is moved with `torch_musa_amd.quantized_modules_to`."""
import torch
import torch.ao.nn.quantized as nnq
import torch.nn.functional as F

from . import fused, qat

__all__ = ["ConvSiLU2d", "ConvAddSiLU2d"]


class _SiLUConv2d(nnq.Conv2d):
    def _prepared_input(self, x):
        if len(x.shape) != 4:
            raise ValueError("Input shape must be `(N, C, H, W)`!")
        if self.padding_mode != "zeros":
            pad = nnq.modules.conv._reverse_repeat_padding(self.padding)
            x = F.pad(x, pad, mode=self.padding_mode)
        return x

    @classmethod
    def from_reference(cls, ref_qconv, output_scale, output_zero_point):
        # the reference-quantized pattern is a fused container whose first child is the convolution
        return super().from_reference(ref_qconv[0], output_scale, output_zero_point)


class ConvSiLU2d(_SiLUConv2d):
    """`silu(conv2d(x))` in one kernel, output requantised to `scale` / `zero_point`."""

    _FLOAT_MODULE = fused.ConvSiLU2d
    _NNIQAT_CONV_BN_MODULE = qat.ConvBnSiLU2d    # from_float folds its batch norm into the weight
    _NNI_CONV_RELU_MODULE = fused.ConvSiLU2d     # from_float takes the convolution out of this container

    def forward(self, input):  # pylint: disable=redefined-builtin
        return torch.ops.quantized.conv2d_silu(self._prepared_input(input), self._packed_params,
                                               self.scale, self.zero_point)

    def _get_name(self):
        return "QuantizedConvSiLU2d"


class ConvAddSiLU2d(_SiLUConv2d):
    """`silu(conv2d(x) + extra)` in one kernel; `extra` is a quantized tensor of the
    output's shape and memory format."""

    _FLOAT_MODULE = fused.ConvAddSiLU2d
    _NNI_CONV_ADD_MODULE = fused.ConvAddSiLU2d   # from_float takes the convolution out of this container

    def forward(self, input, extra_input):  # pylint: disable=redefined-builtin,arguments-differ
        return torch.ops.quantized.conv2d_add_silu(self._prepared_input(input), extra_input,
                                                   self._packed_params, self.scale, self.zero_point)

    def _get_name(self):
        return "QuantizedConvAddSiLU2d"
