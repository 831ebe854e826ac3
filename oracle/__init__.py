"""CPU oracle for the quantized-inference path -- TEST INFRASTRUCTURE ONLY.

ctypes front end of ``oracle/liboracle.so`` (built from ``quant_oracle.c`` by
``make -C oracle``).  Only tests, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import this module; the product
(``torch_musa_amd``) never does.

All arrays are numpy, C-contiguous.  Quantized values travel as ``uint8``
(``is_signed=False``) or ``int8`` (``is_signed=True``) arrays.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile liboracle.so with gcc (a no-op when it is already there)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE] + (["-B"] if force else []),
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.orc_max_threads.restype = C.c_int
        _lib.orc_choose_qparams.restype = C.c_int
    return _lib


def _p(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def _qdtype(is_signed: bool):
    return np.int8 if is_signed else np.uint8


def _as_bytes(q: np.ndarray) -> np.ndarray:
    q = np.ascontiguousarray(q)
    assert q.dtype in (np.uint8, np.int8), q.dtype
    return q


def max_threads() -> int:
    return int(lib().orc_max_threads())


def quantize_per_tensor(x, scale, zp, is_signed=False, nthreads=1):
    x = np.ascontiguousarray(x, dtype=np.float32)
    q = np.empty(x.shape, dtype=_qdtype(is_signed))
    lib().orc_quantize_per_tensor(_p(x), C.c_int64(x.size), C.c_double(scale),
                                  C.c_int64(zp), C.c_int(is_signed), _p(q),
                                  C.c_int(nthreads))
    return q


def quantize_per_tensor_fused(x, scale, zp, is_signed=False, nthreads=1):
    """clamp(rne(fma(x, 1/scale, zp))): the activation quantization of the CPU
    quantized::linear_dynamic."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    q = np.empty(x.shape, dtype=_qdtype(is_signed))
    lib().orc_quantize_per_tensor_fused(_p(x), C.c_int64(x.size), C.c_double(scale),
                                        C.c_int64(zp), C.c_int(is_signed), _p(q),
                                        C.c_int(nthreads))
    return q


def dequantize_per_tensor(q, scale, zp, nthreads=1):
    q = _as_bytes(q)
    r = np.empty(q.shape, dtype=np.float32)
    lib().orc_dequantize_per_tensor(_p(q), C.c_int64(q.size), C.c_double(scale),
                                    C.c_int64(zp), C.c_int(q.dtype == np.int8),
                                    _p(r), C.c_int(nthreads))
    return r


def _outer_c_inner(shape, axis):
    axis = axis % len(shape)
    outer = int(np.prod(shape[:axis], dtype=np.int64))
    inner = int(np.prod(shape[axis + 1:], dtype=np.int64))
    return outer, int(shape[axis]), inner


def quantize_per_channel(x, scales, zps, axis, is_signed=False):
    x = np.ascontiguousarray(x, dtype=np.float32)
    scales = np.ascontiguousarray(scales, dtype=np.float64)
    zps = np.ascontiguousarray(zps, dtype=np.int64)
    outer, c, inner = _outer_c_inner(x.shape, axis)
    assert scales.size == c and zps.size == c
    q = np.empty(x.shape, dtype=_qdtype(is_signed))
    lib().orc_quantize_per_channel(_p(x), C.c_int64(outer), C.c_int64(c),
                                   C.c_int64(inner), _p(scales), _p(zps),
                                   C.c_int(is_signed), _p(q))
    return q


def dequantize_per_channel(q, scales, zps, axis):
    q = _as_bytes(q)
    scales = np.ascontiguousarray(scales, dtype=np.float64)
    zps = np.ascontiguousarray(zps, dtype=np.int64)
    outer, c, inner = _outer_c_inner(q.shape, axis)
    r = np.empty(q.shape, dtype=np.float32)
    lib().orc_dequantize_per_channel(_p(q), C.c_int64(outer), C.c_int64(c),
                                     C.c_int64(inner), _p(scales), _p(zps),
                                     C.c_int(q.dtype == np.int8), _p(r))
    return r


def quantize_per_channel_float(x, scales, zps, axis, is_signed=False):
    """float scales / float zero points (per_channel_affine_float_qparams)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    scales = np.ascontiguousarray(scales, dtype=np.float32)
    zps = np.ascontiguousarray(zps, dtype=np.float32)
    outer, c, inner = _outer_c_inner(x.shape, axis)
    assert scales.size == c and zps.size == c
    q = np.empty(x.shape, dtype=_qdtype(is_signed))
    lib().orc_quantize_per_channel_float(_p(x), C.c_int64(outer), C.c_int64(c), C.c_int64(inner),
                                         _p(scales), _p(zps), C.c_int(is_signed), _p(q))
    return q


def dequantize_per_channel_float(q, scales, zps, axis):
    q = _as_bytes(q)
    scales = np.ascontiguousarray(scales, dtype=np.float32)
    zps = np.ascontiguousarray(zps, dtype=np.float32)
    outer, c, inner = _outer_c_inner(q.shape, axis)
    r = np.empty(q.shape, dtype=np.float32)
    lib().orc_dequantize_per_channel_float(_p(q), C.c_int64(outer), C.c_int64(c), C.c_int64(inner),
                                           _p(scales), _p(zps), C.c_int(q.dtype == np.int8), _p(r))
    return r


def minmax(x, nthreads=1):
    x = np.ascontiguousarray(x, dtype=np.float32)
    mn, mx = C.c_float(), C.c_float()
    lib().orc_minmax(_p(x), C.c_int64(x.size), C.byref(mn), C.byref(mx),
                     C.c_int(nthreads))
    return float(mn.value), float(mx.value)


def choose_qparams(mn, mx, is_signed=False, reduce_range=False):
    """-> (scale: float (double precision), zero_point: int)."""
    qmin, qmax = (-128, 127) if is_signed else (0, 255)
    s, z = C.c_double(), C.c_int32()
    rc = lib().orc_choose_qparams(C.c_float(mn), C.c_float(mx), C.c_int32(qmin),
                                  C.c_int32(qmax), C.c_int(reduce_range),
                                  C.byref(s), C.byref(z))
    if rc != 0:
        raise ValueError("min must be <= max")
    return float(s.value), int(z.value)


def linear_acc32(xq, wq, nthreads=1):
    xq = _as_bytes(xq)
    wq = np.ascontiguousarray(wq, dtype=np.int8)
    m, k = xq.shape
    n, k2 = wq.shape
    assert k == k2
    acc = np.empty((m, n), dtype=np.int32)
    lib().orc_linear_acc32(_p(xq), C.c_int(xq.dtype == np.int8), _p(wq),
                           C.c_int64(m), C.c_int64(n), C.c_int64(k), _p(acc),
                           C.c_int(nthreads))
    return acc


def weight_colsum(wq):
    wq = np.ascontiguousarray(wq, dtype=np.int8)
    n = wq.shape[0]
    k = wq.size // n
    out = np.empty(n, dtype=np.int32)
    lib().orc_weight_colsum(_p(wq), C.c_int64(n), C.c_int64(k), _p(out))
    return out


def requantize(acc, colsum, x_zp, x_scale, w_scales, bias, out_scale, out_zp,
               out_signed=False, relu=False):
    acc = np.ascontiguousarray(acc, dtype=np.int32)
    m, n = acc.shape
    colsum = np.ascontiguousarray(colsum, dtype=np.int32)
    w_scales = np.ascontiguousarray(np.atleast_1d(w_scales), dtype=np.float64)
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    y = np.empty((m, n), dtype=_qdtype(out_signed))
    lib().orc_requantize(_p(acc), C.c_int64(m), C.c_int64(n), _p(colsum),
                         C.c_int64(x_zp), C.c_double(x_scale), _p(w_scales),
                         C.c_int64(w_scales.size), _p(b) if b is not None else None,
                         C.c_double(out_scale), C.c_int64(out_zp),
                         C.c_int(out_signed), C.c_int(relu), _p(y))
    return y


def linear(xq, x_scale, x_zp, wq, w_scales, bias, out_scale, out_zp,
           out_signed=None, relu=False, nthreads=1):
    """quantized::linear on 2-D ``xq`` [M,K] and ``wq`` [N,K] (zero point 0)."""
    xq = _as_bytes(xq)
    wq = np.ascontiguousarray(wq, dtype=np.int8)
    if out_signed is None:
        out_signed = xq.dtype == np.int8
    m, k = xq.shape
    n = wq.shape[0]
    w_scales = np.ascontiguousarray(np.atleast_1d(w_scales), dtype=np.float64)
    assert w_scales.size in (1, n)
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    y = np.empty((m, n), dtype=_qdtype(out_signed))
    lib().orc_linear(_p(xq), C.c_int(xq.dtype == np.int8), _p(wq), C.c_int64(m),
                     C.c_int64(n), C.c_int64(k), C.c_int64(x_zp),
                     C.c_double(x_scale), _p(w_scales), C.c_int64(w_scales.size),
                     _p(b) if b is not None else None, C.c_double(out_scale),
                     C.c_int64(out_zp), C.c_int(out_signed), C.c_int(relu), _p(y),
                     C.c_int(nthreads))
    return y


def linear_f32(xq, x_scale, x_zp, wq, w_scales, bias, relu=False, nthreads=1):
    """Float output of quantized activations times a quantized weight (zero point 0)."""
    xq = _as_bytes(xq)
    wq = np.ascontiguousarray(wq, dtype=np.int8)
    m, k = xq.shape
    n = wq.shape[0]
    w_scales = np.ascontiguousarray(np.atleast_1d(w_scales), dtype=np.float64)
    assert w_scales.size in (1, n)
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    y = np.empty((m, n), dtype=np.float32)
    lib().orc_linear_f32(_p(xq), C.c_int(xq.dtype == np.int8), _p(wq), C.c_int64(m), C.c_int64(n),
                         C.c_int64(k), C.c_int64(x_zp), C.c_double(x_scale), _p(w_scales),
                         C.c_int64(w_scales.size), _p(b) if b is not None else None, C.c_int(relu),
                         _p(y), C.c_int(nthreads))
    return y


def linear_dynamic(x, wq, w_scales, bias, relu=False, reduce_range=False):
    """quantized::linear_dynamic: per-tensor dynamic quint8 quantization of the
    float activations, integer product, float output."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    mn, mx = minmax(x)
    scale, zp = choose_qparams(mn, mx, False, reduce_range)
    xq = quantize_per_tensor_fused(x.reshape(-1, x.shape[-1]), scale, zp, False)
    y = linear_f32(xq, scale, zp, wq, w_scales, bias, relu)
    return y.reshape(x.shape[:-1] + (y.shape[-1],))


def conv_out_hw(h, w, kh, kw, stride, padding, dilation):
    oh = (h + 2 * padding[0] - dilation[0] * (kh - 1) - 1) // stride[0] + 1
    ow = (w + 2 * padding[1] - dilation[1] * (kw - 1) - 1) // stride[1] + 1
    return oh, ow


def conv2d_acc32(x_nhwc, w_ohwi, stride, padding, dilation, groups, x_zp,
                 nthreads=1):
    x = _as_bytes(x_nhwc)
    w = np.ascontiguousarray(w_ohwi, dtype=np.int8)
    b, h, wd, ic = x.shape
    oc, kh, kw, icg = w.shape
    assert icg * groups == ic and oc % groups == 0
    oh, ow = conv_out_hw(h, wd, kh, kw, stride, padding, dilation)
    acc = np.empty((b, oh, ow, oc), dtype=np.int32)
    lib().orc_conv2d_acc32(_p(x), C.c_int(x.dtype == np.int8), _p(w),
                           *[C.c_int64(v) for v in (b, h, wd, ic, oc, kh, kw,
                                                    stride[0], stride[1],
                                                    padding[0], padding[1],
                                                    dilation[0], dilation[1],
                                                    groups, x_zp)],
                           _p(acc), C.c_int(nthreads))
    return acc


def conv2d(x_nhwc, x_scale, x_zp, w_ohwi, w_scales, bias, stride, padding,
           dilation, groups, out_scale, out_zp, out_signed=None, relu=False,
           nthreads=1):
    """quantized::conv2d on NHWC ``x`` and OHWI ``w``; returns NHWC bytes."""
    x = _as_bytes(x_nhwc)
    w = np.ascontiguousarray(w_ohwi, dtype=np.int8)
    if out_signed is None:
        out_signed = x.dtype == np.int8
    b, h, wd, ic = x.shape
    oc, kh, kw, icg = w.shape
    assert icg * groups == ic and oc % groups == 0
    oh, ow = conv_out_hw(h, wd, kh, kw, stride, padding, dilation)
    w_scales = np.ascontiguousarray(np.atleast_1d(w_scales), dtype=np.float64)
    assert w_scales.size in (1, oc)
    bb = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    y = np.empty((b, oh, ow, oc), dtype=_qdtype(out_signed))
    lib().orc_conv2d(_p(x), C.c_int(x.dtype == np.int8), _p(w),
                     *[C.c_int64(v) for v in (b, h, wd, ic, oc, kh, kw,
                                              stride[0], stride[1], padding[0],
                                              padding[1], dilation[0],
                                              dilation[1], groups, x_zp)],
                     C.c_double(x_scale), _p(w_scales), C.c_int64(w_scales.size),
                     _p(bb) if bb is not None else None, C.c_double(out_scale),
                     C.c_int64(out_zp), C.c_int(out_signed), C.c_int(relu), _p(y),
                     C.c_int(nthreads))
    return y


_ACT = {"none": 0, "relu": 1, "silu": 2}


def conv2d_fused(x_nhwc, x_scale, x_zp, w_ohwi, w_scales, bias, stride, padding, dilation,
                 groups, out_scale, out_zp, accum=None, accum_scale=1.0, accum_zp=0,
                 activation="none", out_signed=None, nthreads=1):
    """conv2d with an optional quantized residual (NHWC bytes, the output's
    shape) and an activation ("none", "relu", "silu"); returns NHWC bytes."""
    x = _as_bytes(x_nhwc)
    w = np.ascontiguousarray(w_ohwi, dtype=np.int8)
    if out_signed is None:
        out_signed = x.dtype == np.int8
    b, h, wd, ic = x.shape
    oc, kh, kw, icg = w.shape
    assert icg * groups == ic and oc % groups == 0
    oh, ow = conv_out_hw(h, wd, kh, kw, stride, padding, dilation)
    w_scales = np.ascontiguousarray(np.atleast_1d(w_scales), dtype=np.float64)
    assert w_scales.size in (1, oc)
    bb = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    aa = None
    if accum is not None:
        aa = _as_bytes(accum)
        assert aa.shape == (b, oh, ow, oc)
    y = np.empty((b, oh, ow, oc), dtype=_qdtype(out_signed))
    lib().orc_conv2d_fused(_p(x), C.c_int(x.dtype == np.int8), _p(w),
                           *[C.c_int64(v) for v in (b, h, wd, ic, oc, kh, kw, stride[0], stride[1],
                                                    padding[0], padding[1], dilation[0], dilation[1],
                                                    groups, x_zp)],
                           C.c_double(x_scale), _p(w_scales), C.c_int64(w_scales.size),
                           _p(bb) if bb is not None else None,
                           _p(aa) if aa is not None else None,
                           C.c_int(aa is not None and aa.dtype == np.int8), C.c_int64(accum_zp),
                           C.c_double(accum_scale), C.c_int(_ACT[activation]),
                           C.c_double(out_scale), C.c_int64(out_zp), C.c_int(out_signed), _p(y),
                           C.c_int(nthreads))
    return y


def qadd(qa, a_scale, a_zp, qb, b_scale, b_zp, out_scale, out_zp, relu=False):
    """quantized::add / add_relu of two per-tensor quantized tensors (bytes)."""
    qa, qb = _as_bytes(qa), _as_bytes(qb)
    assert qa.shape == qb.shape and qa.dtype == qb.dtype
    out = np.empty(qa.shape, dtype=qa.dtype)
    lib().orc_qadd(_p(qa), _p(qb), C.c_int64(qa.size), C.c_double(a_scale), C.c_int64(a_zp),
                   C.c_double(b_scale), C.c_int64(b_zp), C.c_double(out_scale), C.c_int64(out_zp),
                   C.c_int(qa.dtype == np.int8), C.c_int(relu), _p(out))
    return out


def qrelu(q, zp):
    q = _as_bytes(q)
    y = np.empty(q.shape, dtype=q.dtype)
    lib().orc_qrelu(_p(q), C.c_int64(q.size), C.c_int64(zp), C.c_int(q.dtype == np.int8), _p(y))
    return y


def pool_out_size(n, k, s, p, d, ceil_mode):
    """Output extent of a pooling window sweep (PyTorch's pooling_output_shape)."""
    out = (n + 2 * p - d * (k - 1) - 1 + (s - 1 if ceil_mode else 0)) // s + 1
    if ceil_mode and (out - 1) * s >= n + p:
        out -= 1
    return out


def qmaxpool2d(x_nhwc, kernel, stride, padding, dilation=(1, 1), ceil_mode=False):
    x = _as_bytes(x_nhwc)
    b, h, w, c = x.shape
    oh = pool_out_size(h, kernel[0], stride[0], padding[0], dilation[0], ceil_mode)
    ow = pool_out_size(w, kernel[1], stride[1], padding[1], dilation[1], ceil_mode)
    y = np.empty((b, oh, ow, c), dtype=x.dtype)
    lib().orc_qmaxpool2d(_p(x), *[C.c_int64(v) for v in (b, h, w, c, kernel[0], kernel[1], stride[0],
                                                        stride[1], padding[0], padding[1], dilation[0],
                                                        dilation[1], oh, ow)],
                         C.c_int(x.dtype == np.int8), _p(y))
    return y


def qadaptive_avgpool2d(x_nhwc, out_hw, zero_point):
    """adaptive_avg_pool2d of per-tensor quantized NHWC codes; qparams carry over."""
    x = _as_bytes(x_nhwc)
    b, h, w, c = x.shape
    y = np.empty((b, out_hw[0], out_hw[1], c), dtype=x.dtype)
    lib().orc_qadaptive_avgpool2d(_p(x), *[C.c_int64(v) for v in (b, h, w, c, out_hw[0], out_hw[1], zero_point)],
                                  C.c_int(x.dtype == np.int8), _p(y))
    return y


def qunary(q, kind, in_scale, in_zp, out_scale, out_zp):
    """gelu / gelu_tanh / sigmoid of per-tensor quantized codes, the way PyTorch's CPU
    ops define them (dequantize, activation, quantize), evaluated in float64:
    y = f((q - in_zp) * fl(in_scale)); q' = clamp(rne(y / fl(out_scale)) + out_zp)."""
    from math import erf, tanh, exp, sqrt, pi
    q = _as_bytes(q)
    signed = q.dtype == np.int8
    lo, hi = (-128, 127) if signed else (0, 255)
    s_in, s_out = float(np.float32(in_scale)), float(np.float32(out_scale))
    table = {}
    for code in range(lo, hi + 1):
        r = (code - in_zp) * s_in
        if kind == "gelu":
            f = 0.5 * r * (1.0 + erf(r / sqrt(2.0)))
        elif kind == "gelu_tanh":
            f = 0.5 * r * (1.0 + tanh(sqrt(2.0 / pi) * (r + 0.044715 * r ** 3)))
        elif kind == "sigmoid":
            f = 1.0 / (1.0 + exp(-r))
        else:
            raise ValueError(kind)
        table[code] = int(min(max(np.rint(f / s_out) + out_zp, lo), hi))
    lut = np.array([table[c] for c in range(lo, hi + 1)], dtype=q.dtype)
    return lut[q.astype(np.int64) - lo]


def qcat(qs, scales, zps, axis, out_scale, out_zp):
    """quantized::cat: every input dequantized and requantized to the output's
    parameters (the composition PyTorch's CPU op performs), then concatenated."""
    signed = _as_bytes(qs[0]).dtype == np.int8
    parts = [quantize_per_tensor(dequantize_per_tensor(q, s, z), out_scale, out_zp, signed)
             for q, s, z in zip(qs, scales, zps)]
    return np.concatenate(parts, axis=axis)


# ---------------------------------------------------------------------------
# Plain-tensor int8 ops (quantized::linear_per_tensor, quantized::conv,
# quantized::conv_binary).  The reference implements them as dequantize ->
# fp32 matmul / conv -> (+ accum) -> relu -> round(r / out_scale + zp) -> clamp
# (mudnn/Qlinear.cpp:36-69, mudnn/Qconv.cpp:45-86,137-181).  Restated here with
# the product in exact integers and everything after it in float64, i.e. that
# formula without its fp32 summation error; int8 kernels are held to 1 LSB of
# it, float outputs to a relative 1e-5.
# ---------------------------------------------------------------------------
def _plain_finish(r, out_scale, out_zp, out_dtype, relu):
    if relu:
        r = np.maximum(r, 0.0)
    if out_dtype == "float32":
        return r.astype(np.float32)
    lo, hi = (-128, 127) if out_dtype == "int8" else (0, 255)
    return np.clip(np.rint(r / out_scale + out_zp), lo, hi).astype(np.int8 if out_dtype == "int8" else np.uint8)


def plain_linear(x, x_scale, x_zp, w_kn, w_scale, bias, out_scale, out_zp, out_dtype, post="none"):
    acc = (np.asarray(x, dtype=np.int64) - x_zp) @ np.asarray(w_kn, dtype=np.int64)
    r = acc.astype(np.float64) * (np.float64(np.float32(x_scale)) * np.asarray(w_scale, dtype=np.float64))[None, :]
    if bias is not None:
        r = r + np.asarray(bias, dtype=np.float64)[None, :]
    assert post in ("none", "relu")
    return _plain_finish(r, out_scale, out_zp, out_dtype, post == "relu")


def plain_conv(x_nchw, x_scale, x_zp, w_oihw, w_scale, bias, stride, pad, groups, out_scale, out_zp, out_dtype,
               relu=False, accum=None, accum_scale=1.0, accum_zp=0):
    x = np.ascontiguousarray(np.transpose(np.asarray(x_nchw), (0, 2, 3, 1)))
    w = np.ascontiguousarray(np.transpose(np.asarray(w_oihw, dtype=np.int8), (0, 2, 3, 1)))
    acc = conv2d_acc32(x, w, (stride, stride), (pad, pad), (1, 1), groups, x_zp)      # [B,OH,OW,OC], exact
    r = acc.astype(np.float64) * (np.float64(np.float32(x_scale)) * np.asarray(w_scale, dtype=np.float64))
    if bias is not None:
        r = r + np.asarray(bias, dtype=np.float64)
    r = np.transpose(r, (0, 3, 1, 2))
    if accum is not None:
        r = r + (np.asarray(accum, dtype=np.float64) - accum_zp) * np.float64(np.float32(accum_scale))
    return _plain_finish(r, out_scale, out_zp, out_dtype, relu)
