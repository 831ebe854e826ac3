"""MI355X-native quantized-inference operators behind PyTorch's own op names.

Importing this package loads two in-tree native libraries:

  libtmq.so        hand-written HIP kernels for gfx950 behind the C ABI of
                   ``include/tmq.h`` (quantize / dequantize / min-max, int8 MFMA
                   linear, NHWC implicit-GEMM conv2d)
  libtmq_aten.so   registrations that put those kernels behind
                   ``torch.quantize_per_tensor``, ``torch.quantize_per_channel``,
                   ``torch.quantize_per_tensor_dynamic``, ``Tensor.dequantize`` and
                   ``torch.ops.quantized.{linear,linear_relu,linear_prepack,
                   conv2d,conv2d_relu,conv2d_prepack}`` for tensors on the GPU

so that a model written against ``torch.ops.quantized.*`` runs unchanged (the
counterpart of ``import torch_musa`` for this operator path; reference:
torch_musa/csrc/aten/quantized).  There is no CPU or eager fallback: if a
library is missing the import fails.
"""
from __future__ import annotations

import os
import warnings

import torch

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_KERNELS = os.path.join(_PKG, "libtmq.so")
LIB_ATEN = os.path.join(_PKG, "libtmq_aten.so")

__all__ = ["LIB_KERNELS", "LIB_ATEN", "is_loaded", "load", "quantized_device", "quantized_modules_to",
           "plain_weight_cache_clear", "plain_weight_cache_counters", "plain_weight_cache_stats",
           "plain_weight_cache_set_max_bytes"]

_loaded = False


def load() -> None:
    """Load the native libraries and register the operators (idempotent)."""
    global _loaded
    if _loaded:
        return
    for lib in (LIB_KERNELS, LIB_ATEN):
        if not os.path.exists(lib):
            raise ImportError(
                f"{lib} is missing: build the native libraries with "
                "`python torch_musa_amd/build.py` (there is no fallback path)")
    with warnings.catch_warnings():
        # replacing PyTorch's own GPU kernel of aten::quantize_per_tensor_dynamic
        # is intended; the dispatcher warns about it once
        warnings.filterwarnings("ignore", message=".*Overriding a previously registered kernel.*")
        torch.ops.load_library(LIB_ATEN)
    from . import ao  # the fused SiLU convolution modules, under the reference's torch.ao names
    ao.register()
    _loaded = True


def is_loaded() -> bool:
    return _loaded


def _aten_lib():
    import ctypes

    load()
    lib = ctypes.CDLL(LIB_ATEN)  # already loaded by torch.ops.load_library: the same handle
    lib.tmq_aten_plain_weight_cache_counters.argtypes = [ctypes.POINTER(ctypes.c_int64)] * 3
    lib.tmq_aten_plain_weight_cache_stats.argtypes = [ctypes.POINTER(ctypes.c_int64), ctypes.c_int]
    lib.tmq_aten_plain_weight_cache_set_max_bytes.argtypes = [ctypes.c_int64]
    return lib


def plain_weight_cache_clear() -> None:
    """Drop the packed weights kept for ``quantized::linear_per_tensor`` / ``conv`` / ``conv_binary``
    (their schemas pass the int8 weight as a plain tensor on every call; the re-tiled copy is kept
    per weight tensor, least recently used entries leaving once the byte limit is exceeded)."""
    _aten_lib().tmq_aten_plain_weight_cache_clear()


def plain_weight_cache_counters():
    """-> (hits, misses, entries) of that cache."""
    import ctypes

    h, m, e = ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int64()
    _aten_lib().tmq_aten_plain_weight_cache_counters(ctypes.byref(h), ctypes.byref(m), ctypes.byref(e))
    return h.value, m.value, e.value


def plain_weight_cache_stats() -> dict:
    """Counters of that cache: hits, misses, entries, bytes held, byte limit, evictions, and hits
    from a stream other than the one that packed the entry (those wait for the packing's event)."""
    import ctypes

    v = (ctypes.c_int64 * 7)()
    _aten_lib().tmq_aten_plain_weight_cache_stats(v, 7)
    names = ("hits", "misses", "entries", "bytes", "max_bytes", "evictions", "cross_stream_hits")
    return dict(zip(names, (int(x) for x in v)))


def plain_weight_cache_set_max_bytes(nbytes: int) -> None:
    """Byte limit of that cache (default 16 GiB, or ``TMQ_PLAIN_WEIGHT_CACHE_MB`` in the environment).
    A model whose plain-tensor weights exceed it re-packs the evicted ones on every pass."""
    _aten_lib().tmq_aten_plain_weight_cache_set_max_bytes(int(nbytes))


def quantized_device() -> torch.device:
    """The device the operators run on (PyTorch-ROCm names the GPU "cuda")."""
    if not torch.cuda.is_available():
        raise RuntimeError("no MI355X visible: the tmq operators have no CPU path")
    return torch.device("cuda", torch.cuda.current_device())


def _qtensor_to(t, device):
    """A dense copy of a (possibly per-channel, possibly strided) quantized tensor on ``device``."""
    if t is None or not t.is_quantized:
        return None if t is None else t.to(device)
    codes = t.int_repr().contiguous().to(device)
    if t.qscheme() in (torch.per_tensor_affine, torch.per_tensor_symmetric):
        return torch._make_per_tensor_quantized_tensor(codes, t.q_scale(), t.q_zero_point())
    return torch._make_per_channel_quantized_tensor(codes, t.q_per_channel_scales().to(device),
                                                    t.q_per_channel_zero_points().to(device),
                                                    t.q_per_channel_axis())


def quantized_modules_to(module: torch.nn.Module, device) -> torch.nn.Module:
    """Move a populated quantized model to ``device``, packed parameters included.

    ``nn.Module.to`` moves parameters and buffers but not the packed-parameter
    objects that ``torch.ao.nn.quantized`` (and ``.dynamic``, ``.intrinsic``)
    modules hold, and unpickling such an object re-creates it with the CPU
    engine.  The reference leaves this to the caller, who re-populates each
    module with ``set_weight_bias`` on device tensors
    (tests/unittest/quantized/test_quantized_linear.py:58-60,87-89); this does
    the same for every submodule that has the ``_weight_bias`` /
    ``set_weight_bias`` pair, in place, and returns ``module``.
    """
    device = torch.device(device)
    repack = []
    for m in module.modules():
        if callable(getattr(m, "_weight_bias", None)) and callable(getattr(m, "set_weight_bias", None)):
            w, b = m._weight_bias()
            repack.append((m, w, b))
    module.to(device)
    for m, w, b in repack:
        m.set_weight_bias(_qtensor_to(w, device), _qtensor_to(b, device))
    return module


load()
