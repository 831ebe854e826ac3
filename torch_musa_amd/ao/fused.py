"""Float containers that mark a Conv2d (+ BatchNorm2d) (+ residual add) + SiLU group
as one unit for the quantization passes (reference:
torch_musa/core/ao/nn/intrinsic/modules/fused.py:11-48).  They compute exactly what
their parts compute; `convert` swaps them for the fused quantized modules of
`torch_musa_amd.ao.quantized`."""
import torch
from torch.ao.nn.intrinsic import _FusedModule
from torch.nn.utils.parametrize import type_before_parametrizations as _plain_type

__all__ = ["ConvSiLU2d", "ConvBnSiLU2d", "ConvAddSiLU2d"]


def _expect(parts, kinds):
    got = tuple(_plain_type(p) for p in parts)
    if got != kinds:
        raise AssertionError(f"expected modules of types {[k.__name__ for k in kinds]}, "
                             f"got {[g.__name__ for g in got]}")


class ConvSiLU2d(_FusedModule):
    """`silu(conv(x))`."""

    def __init__(self, conv, silu):
        _expect((conv, silu), (torch.nn.Conv2d, torch.nn.SiLU))
        super().__init__(conv, silu)


class ConvBnSiLU2d(_FusedModule):
    """`silu(bn(conv(x)))`."""

    def __init__(self, conv, bn, silu):
        _expect((conv, bn, silu), (torch.nn.Conv2d, torch.nn.BatchNorm2d, torch.nn.SiLU))
        super().__init__(conv, bn, silu)


class ConvAddSiLU2d(_FusedModule):
    """`silu(add(conv(x1), x2))`: the convolution is child 0 of the container, `add`
    and `silu` are attributes (any callables of two tensors and of one)."""

    def __init__(self, conv, add, silu):
        super().__init__(conv)
        self.add = add
        self.silu = silu

    def forward(self, x1, x2):  # pylint: disable=arguments-differ
        return self.silu(self.add(self[0](x1), x2))
