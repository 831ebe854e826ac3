"""ctypes binding of the C ABI in ``include/tmq.h`` (``libtmq.so``).

Thin by design: device pointers come from ``torch.Tensor.data_ptr()``, the
stream from ``torch.cuda.current_stream()``; torch is only the allocator here.
Every wrapper raises ``TmqError`` on a non-zero status.  There is no CPU
fallback: if ``libtmq.so`` is missing the import of this module's library
fails loudly.
"""
from __future__ import annotations

import ctypes as C
import os

import torch  # first: libtmq.so must bind to the HIP runtime torch has loaded

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libtmq.so")

DECLARED_SYMBOLS = [
    "tmq_status_string", "tmq_version",
    "tmq_quantize_per_tensor", "tmq_dequantize_per_tensor",
    "tmq_minmax_workspace_bytes", "tmq_minmax", "tmq_choose_qparams_dev",
    "tmq_quantize_per_tensor_dev", "tmq_choose_qparams_host",
    "tmq_quantize_per_channel", "tmq_dequantize_per_channel",
    "tmq_quantize_per_channel_float_qparams", "tmq_dequantize_per_channel_float_qparams",
    "tmq_linear_packed_kchunks", "tmq_linear_packed_bytes", "tmq_linear_prepack",
    "tmq_linear_unpack", "tmq_linear", "tmq_linear_workspace_bytes", "tmq_linear_split_plan", "tmq_linear_kernel_choice", "tmq_linear_static_workspace", "tmq_linear_acc32", "tmq_linear_f32", "tmq_linear_dynamic_small", "tmq_linear_dynamic_small_takes", "tmq_quantize_per_tensor_dynamic_dev",
    "tmq_conv2d_packed_bytes", "tmq_conv2d_prepack", "tmq_conv2d_out_hw", "tmq_conv2d_workspace_bytes",
    "tmq_conv2d", "tmq_conv2d_acc32", "tmq_conv2d_fused",
    "tmq_qadd", "tmq_qrelu", "tmq_qcat_rows", "tmq_qmaxpool2d", "tmq_qadaptive_avgpool2d", "tmq_qunary",
]


class TmqError(RuntimeError):
    pass


class QParams(C.Structure):
    _fields_ = [("scale", C.c_double), ("zero_point", C.c_int32), ("reserved", C.c_int32)]


class LinearDesc(C.Structure):
    _fields_ = [
        ("M", C.c_int64), ("N", C.c_int64), ("K", C.c_int64),
        ("x", C.c_void_p), ("ldx", C.c_int64),
        ("x_signed", C.c_int32), ("x_zero_point", C.c_int32), ("x_scale", C.c_float),
        ("w_packed", C.c_void_p), ("w_colsum", C.c_void_p), ("w_scales", C.c_void_p),
        ("w_per_channel", C.c_int32), ("relu", C.c_int32),
        ("bias", C.c_void_p),
        ("out_scale", C.c_float), ("out_zero_point", C.c_int32),
        ("out_signed", C.c_int32), ("kernel", C.c_int32),
        ("y", C.c_void_p), ("ldy", C.c_int64),
        ("workspace", C.c_void_p), ("workspace_bytes", C.c_int64),
    ]


class LinearChoice(C.Structure):
    _fields_ = [("kernel", C.c_int32), ("tile_rows", C.c_int32), ("tile_channels", C.c_int32), ("waves", C.c_int32),
                ("splits", C.c_int32), ("split_stages", C.c_int32), ("tiles", C.c_int64), ("blocks", C.c_int64),
                ("k_stages", C.c_int64)]


class Conv2dGeom(C.Structure):
    _fields_ = [(n, C.c_int64) for n in (
        "B", "H", "W", "IC", "OC", "KH", "KW", "stride_h", "stride_w", "pad_h", "pad_w",
        "dil_h", "dil_w", "groups")]


class Conv2dDesc(C.Structure):
    _fields_ = [
        ("geom", Conv2dGeom),
        ("x", C.c_void_p),
        ("x_signed", C.c_int32), ("x_zero_point", C.c_int32), ("x_scale", C.c_float),
        ("w_per_channel", C.c_int32),
        ("w_packed", C.c_void_p), ("w_colsum", C.c_void_p), ("w_scales", C.c_void_p),
        ("bias", C.c_void_p),
        ("out_scale", C.c_float), ("out_zero_point", C.c_int32),
        ("out_signed", C.c_int32), ("relu", C.c_int32),
        ("y", C.c_void_p),
        ("kernel", C.c_int32), ("tile_rows", C.c_int32), ("tile_cols", C.c_int32), ("reserved", C.c_int32),
        ("workspace", C.c_void_p), ("workspace_bytes", C.c_int64),
    ]


class Conv2dPost(C.Structure):
    _fields_ = [
        ("accum", C.c_void_p),
        ("accum_signed", C.c_int32), ("accum_zero_point", C.c_int32), ("accum_scale", C.c_float),
        ("activation", C.c_int32),
    ]


ACTIVATIONS = {"none": 0, "relu": 1, "silu": 2}

_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise TmqError(f"{LIB_PATH} is missing: build it with `python torch_musa_amd/build.py`")
        l = C.CDLL(LIB_PATH)
        l.tmq_status_string.restype = C.c_char_p
        l.tmq_minmax_workspace_bytes.restype = C.c_size_t
        l.tmq_minmax_workspace_bytes.argtypes = [C.c_int64]
        for name in ("tmq_linear_packed_kchunks", "tmq_linear_packed_bytes"):
            getattr(l, name).restype = C.c_int64
        l.tmq_linear_packed_kchunks.argtypes = [C.c_int64]
        l.tmq_linear_packed_bytes.argtypes = [C.c_int64, C.c_int64]
        l.tmq_linear_workspace_bytes.restype = C.c_int64
        l.tmq_linear_workspace_bytes.argtypes = [C.c_int64, C.c_int64, C.c_int64]
        l.tmq_linear_split_plan.argtypes = [C.c_int64, C.c_int64, C.c_int64, C.POINTER(C.c_int32),
                                            C.POINTER(C.c_int32)]
        l.tmq_linear_kernel_choice.argtypes = [C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_int32, C.c_int32,
                                               C.c_int32, C.POINTER(LinearChoice)]
        l.tmq_conv2d_packed_bytes.restype = C.c_int64
        l.tmq_conv2d_packed_bytes.argtypes = [C.POINTER(Conv2dGeom)]
        l.tmq_conv2d_workspace_bytes.restype = C.c_int64
        l.tmq_conv2d_workspace_bytes.argtypes = [C.POINTER(Conv2dGeom)]
        v = C.c_void_p
        l.tmq_quantize_per_tensor.argtypes = [v, v, C.c_int64, C.c_double, C.c_int64, C.c_int, v]
        l.tmq_dequantize_per_tensor.argtypes = [v, v, C.c_int64, C.c_double, C.c_int64, C.c_int, v]
        l.tmq_minmax.argtypes = [v, C.c_int64, v, v, C.c_size_t, v]
        l.tmq_choose_qparams_dev.argtypes = [v, C.c_int, C.c_int, v, v]
        l.tmq_quantize_per_tensor_dev.argtypes = [v, v, C.c_int64, v, C.c_int, v]
        l.tmq_choose_qparams_host.argtypes = [C.c_float, C.c_float, C.c_int, C.c_int,
                                              C.POINTER(C.c_double), C.POINTER(C.c_int32)]
        l.tmq_quantize_per_channel.argtypes = [v, v, C.c_int64, C.c_int64, C.c_int64, v, v, C.c_int, v]
        l.tmq_dequantize_per_channel.argtypes = [v, v, C.c_int64, C.c_int64, C.c_int64, v, v, C.c_int, v]
        l.tmq_quantize_per_channel_float_qparams.argtypes = [v, v, C.c_int64, C.c_int64, C.c_int64, v, v, C.c_int, v]
        l.tmq_dequantize_per_channel_float_qparams.argtypes = [v, v, C.c_int64, C.c_int64, C.c_int64, v, v, C.c_int, v]
        l.tmq_linear_prepack.argtypes = [v, C.c_int64, C.c_int64, C.c_int64, v, v, v]
        l.tmq_linear_unpack.argtypes = [v, C.c_int64, C.c_int64, v, C.c_int64, v]
        l.tmq_linear.argtypes = [C.POINTER(LinearDesc), v]
        l.tmq_linear_static_workspace.argtypes = [C.POINTER(LinearDesc), v]
        l.tmq_linear_acc32.argtypes = [C.POINTER(LinearDesc), v, C.c_int64, v]
        l.tmq_linear_f32.argtypes = [C.POINTER(LinearDesc), v, v, C.c_int64, v]
        l.tmq_linear_dynamic_small.argtypes = [C.POINTER(LinearDesc), v, C.c_int64, C.c_int, v, C.c_int64, v]
        l.tmq_linear_dynamic_small_takes.argtypes = [C.c_int64, C.c_int64, C.c_int64]
        l.tmq_quantize_per_tensor_dynamic_dev.argtypes = [v, v, C.c_int64, C.c_int, C.c_int, C.c_int, v, v, C.c_size_t, v]
        l.tmq_conv2d_prepack.argtypes = [v, C.POINTER(Conv2dGeom), v, v, v]
        l.tmq_conv2d_out_hw.argtypes = [C.POINTER(Conv2dGeom), C.POINTER(C.c_int64), C.POINTER(C.c_int64)]
        l.tmq_conv2d.argtypes = [C.POINTER(Conv2dDesc), v]
        l.tmq_conv2d_acc32.argtypes = [C.POINTER(Conv2dDesc), v, v]
        l.tmq_conv2d_fused.argtypes = [C.POINTER(Conv2dDesc), C.POINTER(Conv2dPost), v]
        l.tmq_qadd.argtypes = [v, v, v, C.c_int64, C.c_float, C.c_int32, C.c_float, C.c_int32, C.c_float,
                               C.c_int32, C.c_int, C.c_int, v]
        l.tmq_qrelu.argtypes = [v, v, C.c_int64, C.c_int32, C.c_int, v]
        l.tmq_qcat_rows.argtypes = [v, v, C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_float, C.c_int32,
                                    C.c_float, C.c_int32, C.c_int, v]
        l.tmq_qmaxpool2d.argtypes = [v, v] + [C.c_int64] * 4 + [C.c_int32] * 8 + [C.c_int64] * 2 + [C.c_int, v]
        l.tmq_qadaptive_avgpool2d.argtypes = [v, v] + [C.c_int64] * 6 + [C.c_int32, C.c_int, v]
        l.tmq_qunary.argtypes = [v, v, C.c_int64, C.c_int, C.c_float, C.c_int32, C.c_float, C.c_int32, C.c_int, v]
        _lib = l
    return _lib


def check(status: int, what: str) -> None:
    if status != 0:
        raise TmqError(f"{what}: {lib().tmq_status_string(status).decode()} (status {status})")


def stream_ptr() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t):
    return None if t is None else t.data_ptr()


# ---------------------------------------------------------------------------
# quantizer
# ---------------------------------------------------------------------------
def quantize_per_tensor(x: torch.Tensor, scale: float, zp: int, signed: bool) -> torch.Tensor:
    assert x.dtype == torch.float32 and x.is_contiguous()
    q = torch.empty(x.shape, dtype=torch.int8 if signed else torch.uint8, device=x.device)
    check(lib().tmq_quantize_per_tensor(x.data_ptr(), q.data_ptr(), x.numel(), scale, zp,
                                        int(signed), stream_ptr()), "tmq_quantize_per_tensor")
    return q


def quantize_per_tensor_into(x, q, scale, zp, signed):
    check(lib().tmq_quantize_per_tensor(x.data_ptr(), q.data_ptr(), x.numel(), scale, zp,
                                        int(signed), stream_ptr()), "tmq_quantize_per_tensor")


def dequantize_per_tensor(q: torch.Tensor, scale: float, zp: int) -> torch.Tensor:
    assert q.dtype in (torch.int8, torch.uint8) and q.is_contiguous()
    r = torch.empty(q.shape, dtype=torch.float32, device=q.device)
    check(lib().tmq_dequantize_per_tensor(q.data_ptr(), r.data_ptr(), q.numel(), scale, zp,
                                          int(q.dtype == torch.int8), stream_ptr()),
          "tmq_dequantize_per_tensor")
    return r


def dequantize_per_tensor_into(q, r, scale, zp):
    check(lib().tmq_dequantize_per_tensor(q.data_ptr(), r.data_ptr(), q.numel(), scale, zp,
                                          int(q.dtype == torch.int8), stream_ptr()),
          "tmq_dequantize_per_tensor")


def minmax_workspace(device) -> torch.Tensor:
    return torch.empty(lib().tmq_minmax_workspace_bytes(0), dtype=torch.uint8, device=device)


def minmax(x: torch.Tensor, out: torch.Tensor = None, ws: torch.Tensor = None) -> torch.Tensor:
    assert x.dtype == torch.float32 and x.is_contiguous()
    if out is None:
        out = torch.empty(2, dtype=torch.float32, device=x.device)
    if ws is None:
        ws = minmax_workspace(x.device)
    check(lib().tmq_minmax(x.data_ptr(), x.numel(), out.data_ptr(), ws.data_ptr(), ws.numel(),
                           stream_ptr()), "tmq_minmax")
    return out


def choose_qparams_dev(mm: torch.Tensor, signed: bool, reduce_range: bool) -> torch.Tensor:
    qp = torch.empty(16, dtype=torch.uint8, device=mm.device)
    check(lib().tmq_choose_qparams_dev(mm.data_ptr(), int(signed), int(reduce_range),
                                       qp.data_ptr(), stream_ptr()), "tmq_choose_qparams_dev")
    return qp


def read_qparams(qp: torch.Tensor):
    raw = bytes(qp.cpu().numpy().tobytes())
    s = QParams.from_buffer_copy(raw)
    return float(s.scale), int(s.zero_point)


def quantize_per_tensor_dev(x: torch.Tensor, qp: torch.Tensor, signed: bool) -> torch.Tensor:
    q = torch.empty(x.shape, dtype=torch.int8 if signed else torch.uint8, device=x.device)
    check(lib().tmq_quantize_per_tensor_dev(x.data_ptr(), q.data_ptr(), x.numel(), qp.data_ptr(),
                                            int(signed), stream_ptr()),
          "tmq_quantize_per_tensor_dev")
    return q


def quantize_per_tensor_dynamic_dev(x: torch.Tensor, signed: bool, reduce_range: bool, fused: bool = False):
    """-> (codes, 16 device bytes of qparams); one launch for small inputs, two or three otherwise.
    fused: round x * inv + zp once (the CPU linear_dynamic's activation quantization)
    instead of rne(x * inv) + zp (quantize_per_tensor)."""
    assert x.dtype == torch.float32 and x.is_contiguous()
    q = torch.empty(x.shape, dtype=torch.int8 if signed else torch.uint8, device=x.device)
    qp = torch.empty(16, dtype=torch.uint8, device=x.device)
    ws = minmax_workspace(x.device)
    check(lib().tmq_quantize_per_tensor_dynamic_dev(x.data_ptr(), q.data_ptr(), x.numel(), int(signed),
                                                    int(reduce_range), int(fused), qp.data_ptr(), ws.data_ptr(),
                                                    ws.numel(), stream_ptr()), "tmq_quantize_per_tensor_dynamic_dev")
    return q, qp


def choose_qparams_host(mn: float, mx: float, signed: bool, reduce_range: bool):
    s, z = C.c_double(), C.c_int32()
    check(lib().tmq_choose_qparams_host(mn, mx, int(signed), int(reduce_range), C.byref(s),
                                        C.byref(z)), "tmq_choose_qparams_host")
    return float(s.value), int(z.value)


def _outer_c_inner(shape, axis):
    axis = axis % len(shape)
    outer = 1
    for d in shape[:axis]:
        outer *= d
    inner = 1
    for d in shape[axis + 1:]:
        inner *= d
    return outer, shape[axis], inner


def quantize_per_channel(x, scales, zps, axis, signed):
    assert x.dtype == torch.float32 and x.is_contiguous()
    assert scales.dtype == torch.float64 and zps.dtype == torch.int64
    outer, c, inner = _outer_c_inner(tuple(x.shape), axis)
    q = torch.empty(x.shape, dtype=torch.int8 if signed else torch.uint8, device=x.device)
    check(lib().tmq_quantize_per_channel(x.data_ptr(), q.data_ptr(), outer, c, inner,
                                         scales.data_ptr(), zps.data_ptr(), int(signed),
                                         stream_ptr()), "tmq_quantize_per_channel")
    return q


def dequantize_per_channel(q, scales, zps, axis):
    assert q.is_contiguous()
    outer, c, inner = _outer_c_inner(tuple(q.shape), axis)
    r = torch.empty(q.shape, dtype=torch.float32, device=q.device)
    check(lib().tmq_dequantize_per_channel(q.data_ptr(), r.data_ptr(), outer, c, inner,
                                           scales.data_ptr(), zps.data_ptr(),
                                           int(q.dtype == torch.int8), stream_ptr()),
          "tmq_dequantize_per_channel")
    return r


# ---------------------------------------------------------------------------
# linear
# ---------------------------------------------------------------------------
class PackedLinear:
    """Device buffers produced by tmq_linear_prepack for one [N,K] int8 weight."""

    def __init__(self, w: torch.Tensor):
        assert w.dtype == torch.int8 and w.dim() == 2 and w.stride(1) == 1
        self.N, self.K = w.shape
        nbytes = lib().tmq_linear_packed_bytes(self.N, self.K)
        self.packed = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=w.device)
        self.colsum = torch.empty(max(self.N, 1), dtype=torch.int32, device=w.device)
        check(lib().tmq_linear_prepack(w.data_ptr(), self.N, self.K, w.stride(0),
                                       self.packed.data_ptr(), self.colsum.data_ptr(),
                                       stream_ptr()), "tmq_linear_prepack")

    def unpack(self) -> torch.Tensor:
        w = torch.empty((self.N, self.K), dtype=torch.int8, device=self.packed.device)
        check(lib().tmq_linear_unpack(self.packed.data_ptr(), self.N, self.K, w.data_ptr(),
                                      self.K, stream_ptr()), "tmq_linear_unpack")
        return w


# False: never hand a workspace to the linear entry points (single-launch kernels only)
use_linear_workspace = True
# False: linear_dynamic always takes the two-launch path (quantize, then multiply)
fused_small_dynamic = True
dynamic_small_kernel = 0     # tmq_linear_dynamic_small: 0 the library's choice, 9 / 29 pin one of its two kernels
# a preallocated uint8 tensor that every call on its device shares instead (calls
# on one stream run in order, so one buffer serves them all); None: per call
linear_workspace = None


def _linear_desc(x, pw, x_scale, x_zp, w_scales, bias, out_scale, out_zp, out_signed, relu, y):
    d = LinearDesc()
    d.M, d.K = x.shape
    d.N = pw.N
    assert d.K == pw.K
    d.x, d.ldx = x.data_ptr(), x.stride(0)
    d.x_signed = int(x.dtype == torch.int8)
    d.x_zero_point, d.x_scale = x_zp, x_scale
    d.w_packed, d.w_colsum = pw.packed.data_ptr(), pw.colsum.data_ptr()
    if w_scales is not None:
        assert w_scales.dtype == torch.float32
        d.w_scales = w_scales.data_ptr()
        d.w_per_channel = int(w_scales.numel() > 1)
    d.relu = int(relu)
    d.bias = _ptr(bias)
    d.out_scale, d.out_zero_point, d.out_signed = out_scale, out_zp, int(out_signed)
    d.kernel = _linear_config + 1
    if y is not None:
        d.y, d.ldy = y.data_ptr(), y.stride(0)
    nbytes = lib().tmq_linear_workspace_bytes(d.M, d.N, d.K) if use_linear_workspace else 0
    if nbytes > 0:
        # split-K scratch, from the caching allocator; the descriptor keeps it
        # alive until the call is queued on the current stream
        shared = linear_workspace
        if shared is not None and shared.device == x.device and shared.numel() >= nbytes:
            d._workspace = shared
        else:
            d._workspace = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
        d.workspace, d.workspace_bytes = d._workspace.data_ptr(), nbytes
    return d


def linear(x, pw: PackedLinear, x_scale, x_zp, w_scales, bias, out_scale, out_zp,
           out_signed=None, relu=False, out=None):
    """x: [M,K] uint8/int8 (row stride free), w_scales: fp32 [N] or [1]."""
    assert x.dim() == 2 and x.stride(1) == 1
    if out_signed is None:
        out_signed = x.dtype == torch.int8
    y = out if out is not None else torch.empty(
        (x.shape[0], pw.N), dtype=torch.int8 if out_signed else torch.uint8, device=x.device)
    d = _linear_desc(x, pw, x_scale, x_zp, w_scales, bias, out_scale, out_zp, out_signed, relu, y)
    check(lib().tmq_linear(C.byref(d), stream_ptr()), "tmq_linear")
    return y


def linear_static_workspace(x, pw: PackedLinear, x_scale, x_zp, w_scales, bias, out_scale, out_zp,
                            out_signed=None, relu=False, out=None):
    """tmq_linear_static_workspace: as linear(), the split-K scratch inside the library.
    `out` given: the call allocates nothing at all."""
    assert x.dim() == 2 and x.stride(1) == 1
    if out_signed is None:
        out_signed = x.dtype == torch.int8
    y = out if out is not None else torch.empty(
        (x.shape[0], pw.N), dtype=torch.int8 if out_signed else torch.uint8, device=x.device)
    global use_linear_workspace
    keep, use_linear_workspace = use_linear_workspace, False   # no workspace tensor in the descriptor
    try:
        d = _linear_desc(x, pw, x_scale, x_zp, w_scales, bias, out_scale, out_zp, out_signed, relu, y)
    finally:
        use_linear_workspace = keep
    check(lib().tmq_linear_static_workspace(C.byref(d), stream_ptr()), "tmq_linear_static_workspace")
    return y


def linear_acc32(x, pw: PackedLinear):
    acc = torch.empty((x.shape[0], pw.N), dtype=torch.int32, device=x.device)
    d = _linear_desc(x, pw, 1.0, 0, None, None, 1.0, 0, False, False, None)
    check(lib().tmq_linear_acc32(C.byref(d), acc.data_ptr(), acc.stride(0), stream_ptr()),
          "tmq_linear_acc32")
    return acc


def linear_f32(x, pw: PackedLinear, x_scale, x_zp, w_scales, bias, relu=False, qparams_dev=None):
    """fp32 [M,N] = dequantized product; qparams_dev (16 device bytes from
    choose_qparams_dev) replaces x_scale / x_zp when given."""
    assert x.dim() == 2 and x.stride(1) == 1
    y = torch.empty((x.shape[0], pw.N), dtype=torch.float32, device=x.device)
    d = _linear_desc(x, pw, x_scale, x_zp, w_scales, bias, 1.0, 0, False, relu, None)
    check(lib().tmq_linear_f32(C.byref(d), qparams_dev.data_ptr() if qparams_dev is not None else None,
                               y.data_ptr(), y.stride(0), stream_ptr()), "tmq_linear_f32")
    return y


def linear_dynamic(x, pw: PackedLinear, w_scales, bias, relu=False, reduce_range=False):
    """min/max -> qparams -> quantize -> product, all on the device, no host round trip."""
    assert x.dtype == torch.float32 and x.is_contiguous()
    x2 = x.reshape(-1, x.shape[-1])
    m, k = x2.shape
    takes = 0 < m <= 16 and k % 16 == 0 and lib().tmq_linear_dynamic_small_takes(m, pw.N, k) != 0
    if dynamic_small_kernel == 9:                               # a block per 16 channels quantizes the rows itself
        takes = takes and m * k <= 16384
    elif dynamic_small_kernel == 29:                            # one block per CU does, once
        takes = takes and 64 <= k <= 8192 and m * k <= 32768
    if fused_small_dynamic and takes and x2.data_ptr() % 16 == 0:
        # a handful of rows: range, parameters, codes and product in one launch
        y = torch.empty((m, pw.N), dtype=torch.float32, device=x.device)
        assert k == pw.K and w_scales.dtype == torch.float32
        d = LinearDesc()
        d.M, d.K, d.N = m, k, pw.N
        d.w_packed, d.w_colsum, d.w_scales = pw.packed.data_ptr(), pw.colsum.data_ptr(), w_scales.data_ptr()
        d.w_per_channel, d.relu, d.bias = int(w_scales.numel() > 1), int(relu), _ptr(bias)
        d.kernel = dynamic_small_kernel
        check(lib().tmq_linear_dynamic_small(C.byref(d), x2.data_ptr(), x2.stride(0), int(reduce_range),
                                             y.data_ptr(), y.stride(0), stream_ptr()), "tmq_linear_dynamic_small")
        return y.reshape(tuple(x.shape[:-1]) + (pw.N,))
    xq, qp = quantize_per_tensor_dynamic_dev(x2, False, reduce_range, fused=True)
    y = linear_f32(xq, pw, 1.0, 0, w_scales, bias, relu, qparams_dev=qp)
    return y.reshape(tuple(x.shape[:-1]) + (pw.N,))


def quantize_per_channel_float_qparams(x, scales, zps, axis, signed):
    assert x.dtype == torch.float32 and x.is_contiguous()
    assert scales.dtype == torch.float32 and zps.dtype == torch.float32
    outer, c, inner = _outer_c_inner(tuple(x.shape), axis)
    q = torch.empty(x.shape, dtype=torch.int8 if signed else torch.uint8, device=x.device)
    check(lib().tmq_quantize_per_channel_float_qparams(x.data_ptr(), q.data_ptr(), outer, c, inner,
                                                       scales.data_ptr(), zps.data_ptr(), int(signed),
                                                       stream_ptr()),
          "tmq_quantize_per_channel_float_qparams")
    return q


def dequantize_per_channel_float_qparams(q, scales, zps, axis):
    assert q.is_contiguous()
    assert scales.dtype == torch.float32 and zps.dtype == torch.float32
    outer, c, inner = _outer_c_inner(tuple(q.shape), axis)
    r = torch.empty(q.shape, dtype=torch.float32, device=q.device)
    check(lib().tmq_dequantize_per_channel_float_qparams(q.data_ptr(), r.data_ptr(), outer, c, inner,
                                                         scales.data_ptr(), zps.data_ptr(),
                                                         int(q.dtype == torch.int8), stream_ptr()),
          "tmq_dequantize_per_channel_float_qparams")
    return r


# Kernel pins of this binding (tests and benchmarks): they travel in the
# descriptors' `kernel` fields, call by call; the library keeps no such state.
_linear_config = -1
_conv_path = -1
_conv_tile = (0, 0)


def force_linear_config(cfg: int) -> None:
    """Pin the GEMM tile configuration of later calls through this binding (-1 = automatic)."""
    global _linear_config
    _linear_config = int(cfg)


def force_conv_path(path: int) -> None:
    """Pin the conv2d kernel family of later calls through this binding
    (-1 automatic, 1 halo tiles, 2 implicit GEMM, 3 direct, 4 byte runs, 5 pointwise as linear,
    6 patch rows in a workspace + linear, 7 depthwise on the vector ALU, 8 channels padded to 16 in a
    workspace, then the automatic choice for that, 9 pointwise with the pixels straight from memory)."""
    global _conv_path
    _conv_path = int(path)


_conv_workspace = True


def use_conv_workspace(on: bool) -> None:
    """Whether later conv2d calls through this binding pass the scratch memory the library asks for."""
    global _conv_workspace
    _conv_workspace = bool(on)


def force_conv_tile(rows: int, cols: int) -> None:
    """Pin the halo kernel's patch height / bound its patch width (0 = automatic)."""
    global _conv_tile
    _conv_tile = (int(rows), int(cols))


def linear_split_plan(m: int, n: int, k: int):
    """-> (splits, stages per split) of the split-K schedule for this shape."""
    sp, st = C.c_int32(), C.c_int32()
    check(lib().tmq_linear_split_plan(m, n, k, C.byref(sp), C.byref(st)), "tmq_linear_split_plan")
    return sp.value, st.value


LINEAR_OUT_KINDS = {"bytes": 0, "f32": 1, "acc32": 2}


def linear_kernel_choice(m: int, n: int, k: int, ldx: int = None, out: str = "bytes", workspace: bool = False,
                         misaligned: bool = False, forced: int = 0, compute_units: int = 256) -> dict:
    """Which kernel the library launches for this shape (host arithmetic only): a dict of
    include/tmq.h's tmq_linear_choice fields; kernel == 0 says that no kernel takes it."""
    c = LinearChoice()
    flags = LINEAR_OUT_KINDS[out] | (4 if workspace else 0) | (8 if misaligned else 0)
    check(lib().tmq_linear_kernel_choice(m, n, k, k if ldx is None else ldx, flags, forced, compute_units,
                                         C.byref(c)), "tmq_linear_kernel_choice")
    return {f: getattr(c, f) for f, _ in LinearChoice._fields_}


# ---------------------------------------------------------------------------
# conv2d
# ---------------------------------------------------------------------------
def conv_geom(x_shape_nhwc, w_shape_ohwi, stride, padding, dilation, groups) -> Conv2dGeom:
    g = Conv2dGeom()
    g.B, g.H, g.W, g.IC = x_shape_nhwc
    g.OC, g.KH, g.KW = w_shape_ohwi[:3]
    g.stride_h, g.stride_w = stride
    g.pad_h, g.pad_w = padding
    g.dil_h, g.dil_w = dilation
    g.groups = groups
    return g


def conv_out_hw(g: Conv2dGeom):
    oh, ow = C.c_int64(), C.c_int64()
    check(lib().tmq_conv2d_out_hw(C.byref(g), C.byref(oh), C.byref(ow)), "tmq_conv2d_out_hw")
    return oh.value, ow.value


class PackedConv2d:
    def __init__(self, w_ohwi: torch.Tensor, g: Conv2dGeom):
        assert w_ohwi.dtype == torch.int8 and w_ohwi.is_contiguous()
        nbytes = lib().tmq_conv2d_packed_bytes(C.byref(g))
        if nbytes <= 0:
            raise TmqError("invalid convolution geometry")
        self.packed = torch.empty(nbytes, dtype=torch.uint8, device=w_ohwi.device)
        self.colsum = torch.empty(g.OC, dtype=torch.int32, device=w_ohwi.device)
        check(lib().tmq_conv2d_prepack(w_ohwi.data_ptr(), C.byref(g), self.packed.data_ptr(),
                                       self.colsum.data_ptr(), stream_ptr()),
              "tmq_conv2d_prepack")


def _conv_desc(x, pw, g, x_scale, x_zp, w_scales, bias, out_scale, out_zp, out_signed, relu, y):
    d = Conv2dDesc()
    d.geom = g
    d.x = x.data_ptr()
    d.x_signed = int(x.dtype == torch.int8)
    d.x_zero_point, d.x_scale = x_zp, x_scale
    d.w_packed, d.w_colsum = pw.packed.data_ptr(), pw.colsum.data_ptr()
    if w_scales is not None:
        d.w_scales = w_scales.data_ptr()
        d.w_per_channel = int(w_scales.numel() > 1)
    d.bias = _ptr(bias)
    d.out_scale, d.out_zero_point, d.out_signed, d.relu = out_scale, out_zp, int(out_signed), int(relu)
    d.y = _ptr(y)
    d.kernel = _conv_path if _conv_path > 0 else 0
    d.tile_rows, d.tile_cols = _conv_tile
    # scratch for the layers that run on their patch rows or on a channel-padded copy of the input
    # (pinned for tests: whatever the size)
    need = lib().tmq_conv2d_workspace_bytes(C.byref(g))
    if _conv_path == 6 and g.groups == 1 and g.IC % 16 == 0:
        oh, ow = conv_out_hw(g)
        need = g.B * oh * ow * g.KH * g.KW * g.IC
    if _conv_path == 8 and g.groups == 1 and g.IC % 16 != 0:
        need = g.B * g.H * g.W * ((g.IC + 15) // 16 * 16)
    if need > 0 and _conv_workspace:
        d._ws = torch.empty(need, dtype=torch.uint8, device=x.device)   # (kept alive by the descriptor)
        d.workspace, d.workspace_bytes = d._ws.data_ptr(), need
    return d


def conv2d(x_nhwc, pw: PackedConv2d, g: Conv2dGeom, x_scale, x_zp, w_scales, bias, out_scale,
           out_zp, out_signed=None, relu=False, out=None):
    assert x_nhwc.is_contiguous() and tuple(x_nhwc.shape) == (g.B, g.H, g.W, g.IC)
    if out_signed is None:
        out_signed = x_nhwc.dtype == torch.int8
    oh, ow = conv_out_hw(g)
    y = out if out is not None else torch.empty(
        (g.B, oh, ow, g.OC), dtype=torch.int8 if out_signed else torch.uint8, device=x_nhwc.device)
    d = _conv_desc(x_nhwc, pw, g, x_scale, x_zp, w_scales, bias, out_scale, out_zp, out_signed,
                   relu, y)
    check(lib().tmq_conv2d(C.byref(d), stream_ptr()), "tmq_conv2d")
    return y


def conv2d_fused(x_nhwc, pw: PackedConv2d, g: Conv2dGeom, x_scale, x_zp, w_scales, bias, out_scale,
                 out_zp, accum=None, accum_scale=1.0, accum_zp=0, activation="none", out_signed=None,
                 out=None):
    """conv2d + optional quantized residual (NHWC bytes, the output's shape) + activation."""
    assert x_nhwc.is_contiguous() and tuple(x_nhwc.shape) == (g.B, g.H, g.W, g.IC)
    if out_signed is None:
        out_signed = x_nhwc.dtype == torch.int8
    oh, ow = conv_out_hw(g)
    y = out if out is not None else torch.empty(
        (g.B, oh, ow, g.OC), dtype=torch.int8 if out_signed else torch.uint8, device=x_nhwc.device)
    d = _conv_desc(x_nhwc, pw, g, x_scale, x_zp, w_scales, bias, out_scale, out_zp, out_signed,
                   False, y)
    post = Conv2dPost()
    if accum is not None:
        assert accum.is_contiguous() and tuple(accum.shape) == (g.B, oh, ow, g.OC)
        post.accum = accum.data_ptr()
        post.accum_signed = int(accum.dtype == torch.int8)
    post.accum_zero_point = int(accum_zp)
    post.accum_scale = float(accum_scale)
    post.activation = ACTIVATIONS[activation]
    check(lib().tmq_conv2d_fused(C.byref(d), C.byref(post), stream_ptr()), "tmq_conv2d_fused")
    return y


def conv2d_acc32(x_nhwc, pw: PackedConv2d, g: Conv2dGeom, x_zp):
    oh, ow = conv_out_hw(g)
    acc = torch.empty((g.B, oh, ow, g.OC), dtype=torch.int32, device=x_nhwc.device)
    d = _conv_desc(x_nhwc, pw, g, 1.0, x_zp, None, None, 1.0, 0, False, False, None)
    check(lib().tmq_conv2d_acc32(C.byref(d), acc.data_ptr(), stream_ptr()), "tmq_conv2d_acc32")
    return acc


# ---------------------------------------------------------------------------
# elementwise
# ---------------------------------------------------------------------------
def qadd(qa, a_scale, a_zp, qb, b_scale, b_zp, out_scale, out_zp, relu=False, out=None):
    assert qa.shape == qb.shape and qa.dtype == qb.dtype and qa.is_contiguous() and qb.is_contiguous()
    y = out if out is not None else torch.empty_like(qa)
    check(lib().tmq_qadd(qa.data_ptr(), qb.data_ptr(), y.data_ptr(), qa.numel(), a_scale, a_zp, b_scale,
                         b_zp, out_scale, out_zp, int(qa.dtype == torch.int8), int(relu), stream_ptr()),
          "tmq_qadd")
    return y


def qrelu(q, zp, out=None):
    assert q.is_contiguous()
    y = out if out is not None else torch.empty_like(q)
    check(lib().tmq_qrelu(q.data_ptr(), y.data_ptr(), q.numel(), zp, int(q.dtype == torch.int8),
                          stream_ptr()), "tmq_qrelu")
    return y


QUNARY_KINDS = {"gelu": 0, "gelu_tanh": 1, "sigmoid": 2}


def qunary(q, kind, in_scale, in_zp, out_scale, out_zp):
    y = torch.empty_like(q)
    check(lib().tmq_qunary(q.data_ptr(), y.data_ptr(), q.numel(), QUNARY_KINDS[kind], in_scale, in_zp, out_scale,
                           out_zp, int(q.dtype == torch.int8), stream_ptr()), "tmq_qunary")
    return y


def qcat(qs, scales, zps, axis, out_scale, out_zp):
    """quantized::cat of contiguous tensors along ``axis``."""
    shape = list(qs[0].shape)
    axis = axis % len(shape)
    shape[axis] = sum(q.shape[axis] for q in qs)
    y = torch.empty(shape, dtype=qs[0].dtype, device=qs[0].device)
    outer = 1
    for d in shape[:axis]:
        outer *= d
    inner = 1
    for d in shape[axis + 1:]:
        inner *= d
    off = 0
    for q, s, z in zip(qs, scales, zps):
        assert q.is_contiguous() and q.dtype == y.dtype
        row = q.shape[axis] * inner
        check(lib().tmq_qcat_rows(q.data_ptr(), y.data_ptr(), outer, row, shape[axis] * inner, off, s, z,
                                  out_scale, out_zp, int(q.dtype == torch.int8), stream_ptr()),
              "tmq_qcat_rows")
        off += row
    return y


def qmaxpool2d(x_nhwc, kernel, stride, padding, dilation, out_hw):
    assert x_nhwc.is_contiguous()
    b, h, w, c = x_nhwc.shape
    y = torch.empty((b, out_hw[0], out_hw[1], c), dtype=x_nhwc.dtype, device=x_nhwc.device)
    check(lib().tmq_qmaxpool2d(x_nhwc.data_ptr(), y.data_ptr(), b, h, w, c, kernel[0], kernel[1], stride[0],
                               stride[1], padding[0], padding[1], dilation[0], dilation[1], out_hw[0],
                               out_hw[1], int(x_nhwc.dtype == torch.int8), stream_ptr()), "tmq_qmaxpool2d")
    return y


def qadaptive_avgpool2d(x_nhwc, out_hw, zero_point):
    assert x_nhwc.is_contiguous()
    b, h, w, c = x_nhwc.shape
    y = torch.empty((b, out_hw[0], out_hw[1], c), dtype=x_nhwc.dtype, device=x_nhwc.device)
    check(lib().tmq_qadaptive_avgpool2d(x_nhwc.data_ptr(), y.data_ptr(), b, h, w, c, out_hw[0], out_hw[1],
                                        zero_point, int(x_nhwc.dtype == torch.int8), stream_ptr()),
          "tmq_qadaptive_avgpool2d")
    return y


# ---------------------------------------------------------------------------
# measurement probe (include/tmq_bench.h, libtmq_bench.so: not part of libtmq.so)
# ---------------------------------------------------------------------------
BENCH_LIB_PATH = os.path.join(_PKG, "libtmq_bench.so")
_bench_lib = None


def bench_lib() -> C.CDLL:
    global _bench_lib
    if _bench_lib is None:
        if not os.path.exists(BENCH_LIB_PATH):
            raise TmqError(f"{BENCH_LIB_PATH} is missing: build it with `python torch_musa_amd/build.py`")
        l = C.CDLL(BENCH_LIB_PATH)
        l.tmq_probe_mfma_i8.argtypes = [C.c_int, C.c_int, C.c_int, C.c_void_p, C.POINTER(C.c_double),
                                        C.POINTER(C.c_double)]
        l.tmq_bench_stream_read.argtypes = [C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p]
        l.tmq_bench_empty_kernel.argtypes = [C.c_int, C.c_void_p, C.c_void_p]
        _bench_lib = l
    return _bench_lib


def bench_stream_read(src: torch.Tensor, sink: torch.Tensor) -> None:
    """A kernel that only reads `src` (bytes a multiple of 64 KiB), shaped like the decode kernel."""
    check(bench_lib().tmq_bench_stream_read(src.data_ptr(), src.numel() * src.element_size(), sink.data_ptr(),
                                            stream_ptr()), "tmq_bench_stream_read")


def bench_empty_kernel(blocks: int, sink: torch.Tensor) -> None:
    check(bench_lib().tmq_bench_empty_kernel(blocks, sink.data_ptr(), stream_ptr()), "tmq_bench_empty_kernel")


def probe_mfma_i8(data_mode: int, blocks: int = 256, iters: int = 20000):
    """-> (TOP/s, shader GHz) of a register-only int8 MFMA loop; synchronises."""
    scratch = torch.zeros(2048, dtype=torch.uint8, device="cuda")
    tops, ghz = C.c_double(), C.c_double()
    torch.cuda.synchronize()
    check(bench_lib().tmq_probe_mfma_i8(data_mode, blocks, iters, scratch.data_ptr(), C.byref(tops),
                                        C.byref(ghz)), "tmq_probe_mfma_i8")
    return float(tops.value), float(ghz.value)
