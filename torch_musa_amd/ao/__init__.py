"""Module-level callers of the fused SiLU convolutions: float containers (`fused`),
their quantization-aware-training forms (`qat`) and the quantized modules
(`quantized`).  `register()` publishes them under the `torch.ao.nn.intrinsic*`
names the reference gives them (torch_musa/core/ao/register_helper.py:12-20), which
is where its users and tests look them up (`nniq.ConvSiLU2d`)."""
import torch
import torch.ao.nn.intrinsic
import torch.ao.nn.intrinsic.qat
import torch.ao.nn.intrinsic.quantized

from . import fused, qat, quantized

__all__ = ["fused", "qat", "quantized", "register", "STATIC_QUANT_MODULE_MAPPINGS"]

# float or QAT class -> quantized class, for `torch.ao.quantization.convert(..., mapping=...)`
STATIC_QUANT_MODULE_MAPPINGS = {
    fused.ConvSiLU2d: quantized.ConvSiLU2d,
    fused.ConvAddSiLU2d: quantized.ConvAddSiLU2d,
    qat.ConvSiLU2d: quantized.ConvSiLU2d,
    qat.ConvBnSiLU2d: quantized.ConvSiLU2d,
}


def register() -> None:
    """Idempotent."""
    for namespace, source in ((torch.ao.nn.intrinsic, fused), (torch.ao.nn.intrinsic.qat, qat),
                              (torch.ao.nn.intrinsic.quantized, quantized)):
        for name in source.__all__:
            setattr(namespace, name, getattr(source, name))
