"""GPU parity of quantized::conv2d (NHWC implicit GEMM) through the C ABI."""
import numpy as np
import pytest
import torch

import cases
import oracle
from gpu_util import dev, host, say

pytestmark = pytest.mark.gpu

LSB_TOL = 1


@pytest.fixture(scope="module")
def cabi():
    from torch_musa_amd import cabi as m
    assert torch.cuda.is_available()
    m.lib()
    return m


def _check(y, want, what):
    d = np.abs(y.astype(np.int32) - want.astype(np.int32))
    assert d.max() <= LSB_TOL, f"{what}: max diff {d.max()}"
    assert d.max() == 0, f"{what}: {np.count_nonzero(d)} of {d.size} bytes differ by 1 LSB"


def _run(cabi, c):
    g = cabi.conv_geom(c["xq"].shape, c["wq"].shape, c["stride"], c["padding"], c["dilation"],
                       c["groups"])
    pw = cabi.PackedConv2d(dev(c["wq"]), g)
    ws = dev(c["w_scales"].astype(np.float32))
    b = None if c["bias"] is None else dev(c["bias"])
    x = dev(c["xq"])
    y = cabi.conv2d(x, pw, g, c["x_scale"], c["x_zp"], ws, b, c["out_scale"], c["out_zp"],
                    relu=c["relu"])
    acc = cabi.conv2d_acc32(x, pw, g, c["x_zp"])
    return host(y), host(acc), pw


@pytest.mark.parametrize("c", cases.conv_cases(), ids=lambda c: c["name"])
def test_conv_cases(cabi, golden, c):
    say("conv", c["name"])
    y, acc, pw = _run(cabi, c)
    np.testing.assert_array_equal(
        acc, oracle.conv2d_acc32(c["xq"], c["wq"], c["stride"], c["padding"], c["dilation"],
                                 c["groups"], c["x_zp"]))
    np.testing.assert_array_equal(host(pw.colsum),
                                  c["wq"].reshape(c["wq"].shape[0], -1).astype(np.int64).sum(1))
    want = oracle.conv2d(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                         c["stride"], c["padding"], c["dilation"], c["groups"], c["out_scale"],
                         c["out_zp"], relu=c["relu"])
    _check(y, want, "vs oracle")
    _check(y, golden["conv/" + c["name"] + "/y"], "vs golden")


def _conv_case(b, h, w, ic, oc, k, s, p, d, g, seed, x_signed=False, relu=False):
    rng = np.random.default_rng(seed)
    xq = (rng.integers(-128, 128, (b, h, w, ic), dtype=np.int8) if x_signed
          else rng.integers(0, 256, (b, h, w, ic), dtype=np.uint8))
    wq = rng.integers(-127, 128, (oc, k, k, ic // g), dtype=np.int8)
    ws = (0.001 + 0.002 * rng.random(oc)).astype(np.float32).astype(np.float64)
    kk = k * k * (ic // g)
    sigma = np.sqrt(kk) * 74.0 * 74.0 * 0.03 * float(ws.mean())
    return dict(xq=xq, wq=wq, bias=rng.standard_normal(oc).astype(np.float32) * np.float32(sigma),
                x_scale=0.03, x_zp=-9 if x_signed else 60, w_scales=ws, stride=(s, s),
                padding=(p, p), dilation=(d, d), groups=g,
                out_scale=float(np.float32(3 * sigma / 128)), out_zp=4 if x_signed else 128,
                relu=relu)


@pytest.mark.parametrize("spec", [
    (2, 20, 20, 64, 64, 3, 1, 1, 1, 1),      # C5's channel geometry, small image
    (1, 30, 30, 128, 160, 3, 2, 1, 1, 1),    # OC > 64 -> 128x128 tiles when large
    (4, 64, 64, 16, 256, 3, 1, 1, 1, 1),     # many rows, 128x128 tiles
    (5, 120, 120, 16, 32, 3, 1, 0, 1, 1),    # > 65536 rows -> 256x64 tiles
    (2, 17, 13, 48, 24, 5, 2, 2, 1, 1),      # ragged everything
    (2, 16, 16, 64, 96, 3, 1, 1, 1, 2),      # two groups on the MFMA path
    (2, 15, 15, 32, 40, 3, 1, 2, 2, 1),      # dilation
])
@pytest.mark.parametrize("x_signed", [False, True])
@pytest.mark.parametrize("path", [1, 2], ids=["tiles", "gemm"])
def test_conv_mfma_shapes(cabi, spec, x_signed, path):
    say("conv mfma", spec, x_signed, path)
    c = _conv_case(*spec, seed=sum(spec), x_signed=x_signed, relu=x_signed)
    cabi.force_conv_path(path)
    try:
        y, acc, _ = _run(cabi, c)
    finally:
        cabi.force_conv_path(-1)
    np.testing.assert_array_equal(
        acc, oracle.conv2d_acc32(c["xq"], c["wq"], c["stride"], c["padding"], c["dilation"],
                                 c["groups"], c["x_zp"], nthreads=8))
    want = oracle.conv2d(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                         c["stride"], c["padding"], c["dilation"], c["groups"], c["out_scale"],
                         c["out_zp"], relu=c["relu"], nthreads=8)
    _check(y, want, "mfma conv")


@pytest.mark.parametrize("spec", [
    (1, 9, 300, 16, 16, 3, 1, 1, 1, 1),      # wide rows: patches split the width
    (2, 33, 21, 32, 72, 3, 2, 1, 2, 1),      # stride 2 with dilation 2, OC over two 64-channel tiles
    (1, 12, 12, 96, 48, 3, 1, 1, 1, 4),      # four groups of 24 in, 12 out: merged in pairs
    (3, 10, 10, 64, 48, 3, 1, 1, 1, 2),      # groups whose 24 channels break 16-byte stores
    (1, 14, 14, 128, 64, 3, 1, 1, 1, 1),     # 72 KB weight slice in LDS
    (1, 14, 14, 256, 64, 3, 1, 1, 1, 1),     # weight slice too large for LDS: implicit GEMM
    (2, 28, 28, 64, 128, 1, 1, 0, 1, 1),     # 1x1
    (1, 40, 40, 16, 64, 7, 2, 3, 1, 1),      # 7x7 stride 2
    (1, 1, 1, 16, 1, 1, 1, 0, 1, 1),         # a single output value
    (8, 56, 56, 64, 64, 3, 1, 1, 1, 1),      # 56-wide rows: patches a quarter of a row wide, tall
    (3, 57, 57, 32, 64, 3, 1, 1, 1, 1),      # a width no patch width divides
    (9, 28, 28, 512, 128, 1, 1, 0, 1, 1),    # 1x1 over many input channels: halo tiles (32 KB slice)
    (4, 56, 56, 256, 96, 1, 2, 0, 1, 1),     # 1x1 stride 2: kernel smaller than the stride, implicit GEMM
    (4, 56, 56, 64, 128, 3, 2, 1, 1, 1),     # 3x3 stride 2: halo tiles
    (2, 38, 19, 16, 64, 2, 2, 0, 1, 1),      # 2x2 stride 2: every pixel used once
    (1, 128, 128, 128, 512, 1, 1, 0, 1, 1),  # pointwise, 16384 pixels, a billion products: as a linear layer
    (1, 128, 128, 128, 192, 1, 1, 0, 1, 1),  # fewer output channels: halo tiles
])
def test_conv_auto_path_shapes(cabi, spec):
    say("conv auto", spec)
    c = _conv_case(*spec, seed=sum(spec) + 1)
    y, acc, _ = _run(cabi, c)
    np.testing.assert_array_equal(
        acc, oracle.conv2d_acc32(c["xq"], c["wq"], c["stride"], c["padding"], c["dilation"],
                                 c["groups"], c["x_zp"], nthreads=8))
    want = oracle.conv2d(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                         c["stride"], c["padding"], c["dilation"], c["groups"], c["out_scale"],
                         c["out_zp"], relu=c["relu"], nthreads=8)
    _check(y, want, "auto conv")


@pytest.mark.parametrize("spec", [
    (2, 64, 64, 3, 64, 7, 2, 3, 1, 1),       # an image network's first layer: 7 x 7 stride 2, 3 -> 64
    (2, 33, 33, 3, 32, 3, 2, 1, 1, 1),       # 3 x 3 stride 2, 3 -> 32; image rows of 99 bytes: byte copies
    (1, 36, 36, 3, 48, 6, 2, 2, 1, 1),       # 6 x 6 stride 2
    (3, 28, 28, 24, 144, 1, 1, 0, 1, 1),     # pointwise, 24 channels in, three 64-channel blocks out
    (2, 14, 14, 40, 100, 1, 1, 0, 1, 1),     # pointwise, nothing a multiple of 16
    (2, 30, 30, 1, 16, 5, 1, 2, 1, 1),       # one input channel
    (1, 20, 20, 4, 20, 3, 1, 1, 1, 1),       # four input channels, 20 out: byte stores
    (1, 8, 600, 3, 16, 3, 2, 1, 1, 1),       # 300 output columns: three tile columns
    (1, 300, 9, 3, 8, 3, 1, 1, 1, 1),        # narrow and tall
    (2, 19, 23, 8, 64, 3, 1, 0, 1, 1),       # eight channels, 3 x 3: runs of 24 bytes
    (1, 9, 9, 5, 7, 4, 3, 0, 1, 1),          # 4 x 4 stride 3, 5 -> 7 channels
    (2, 12, 12, 48, 32, 1, 2, 0, 1, 1),      # a multiple of 16 (pinned only): one run of 48 bytes
])
@pytest.mark.parametrize("x_signed", [False, True])
def test_conv_few_channels_as_byte_runs(cabi, spec, x_signed):
    say("conv byte runs", spec, x_signed)
    c = _conv_case(*spec, seed=sum(spec) + 7, x_signed=x_signed, relu=not x_signed)
    want_acc = oracle.conv2d_acc32(c["xq"], c["wq"], c["stride"], c["padding"], c["dilation"],
                                   c["groups"], c["x_zp"], nthreads=8)
    want = oracle.conv2d(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                         c["stride"], c["padding"], c["dilation"], c["groups"], c["out_scale"],
                         c["out_zp"], relu=c["relu"], nthreads=8)
    for path in (4, -1):
        cabi.force_conv_path(path)
        try:
            y, acc, _ = _run(cabi, c)
        finally:
            cabi.force_conv_path(-1)
        np.testing.assert_array_equal(acc, want_acc)
        _check(y, want, f"path {path}")


@pytest.mark.parametrize("spec", [
    (2, 20, 20, 32, 32, 3, 1, 1, 1, 32),     # depthwise, 32 channels: one merged group
    (1, 29, 29, 144, 144, 3, 2, 1, 1, 144),  # depthwise stride 2, 144 channels: three merged groups of 48
    (1, 15, 15, 96, 96, 5, 1, 2, 1, 96),     # depthwise 5 x 5
    (1, 14, 14, 384, 384, 3, 1, 1, 1, 384),  # depthwise, six merged groups of 64
    (2, 16, 16, 128, 128, 3, 1, 1, 1, 32),   # 32 groups of 4 -> 4: two merged groups of 64
    (1, 12, 12, 32, 64, 3, 1, 1, 1, 4),      # groups of 8 in, 16 out: two of them make 16 / 32
    (1, 10, 10, 16, 32, 3, 1, 1, 1, 16),     # depthwise with two output channels per input channel
    (1, 12, 12, 96, 48, 3, 1, 1, 1, 4),      # groups of 24 in, 12 out: pairs
    (1, 9, 9, 40, 40, 3, 1, 1, 1, 40),       # depthwise, 40 channels: no multiple of 16 divides it, direct kernel
    (1, 9, 9, 48, 48, 3, 1, 1, 2, 48),       # depthwise with dilation
])
@pytest.mark.parametrize("x_signed", [False, True])
def test_conv_narrow_groups_merged(cabi, spec, x_signed):
    say("conv narrow groups", spec, x_signed)
    c = _conv_case(*spec, seed=sum(spec) + 11, x_signed=x_signed, relu=x_signed)
    want_acc = oracle.conv2d_acc32(c["xq"], c["wq"], c["stride"], c["padding"], c["dilation"],
                                   c["groups"], c["x_zp"], nthreads=8)
    want = oracle.conv2d(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                         c["stride"], c["padding"], c["dilation"], c["groups"], c["out_scale"],
                         c["out_zp"], relu=c["relu"], nthreads=8)
    merged = spec[3] != 40
    for path in (-1, 1, 2, 3):
        cabi.force_conv_path(path)
        try:
            if path in (1, 2) and not merged:
                with pytest.raises(cabi.TmqError):
                    _run(cabi, c)
                continue
            y, acc, pw = _run(cabi, c)
        finally:
            cabi.force_conv_path(-1)
        np.testing.assert_array_equal(acc, want_acc)
        np.testing.assert_array_equal(host(pw.colsum), c["wq"].reshape(c["wq"].shape[0], -1).astype(np.int64).sum(1))
        _check(y, want, f"path {path}")


@pytest.mark.parametrize("spec", [
    (2, 19, 23, 72, 72, 3, 1, 1, 1, 72),     # 72 channels: no whole 16-channel blocks to merge into
    (1, 9, 9, 40, 40, 3, 2, 1, 1, 40),       # stride 2
    (3, 17, 13, 24, 24, 5, 1, 2, 1, 24),     # 5 x 5: whole weight dwords in registers
    (2, 21, 21, 120, 120, 5, 2, 2, 1, 120),
    (1, 15, 15, 12, 12, 7, 1, 3, 1, 12),     # 7 x 7: two dwords of taps per kernel row
    (2, 20, 9, 96, 96, 7, 2, 3, 1, 96),      # ... at stride 2: the whole window per output row
    (1, 13, 13, 8, 8, 9, 1, 4, 1, 8),        # any other kernel size: a plain loop over the taps
    (2, 11, 14, 20, 20, 3, 1, 2, 2, 20),     # dilation
    (1, 6, 6, 4, 4, 3, 1, 0, 1, 4),          # one lane per pixel, no padding
    (2, 3, 40, 36, 36, 3, 1, 1, 1, 36),      # fewer output rows than a strip
    (2, 30, 30, 96, 96, 3, 2, 1, 1, 96),     # channels that would also merge
    (1, 12, 12, 8, 8, (1, 3), 1, 0, 1, 8),   # a kernel that is not square
])
@pytest.mark.parametrize("x_signed", [False, True])
def test_conv_depthwise_on_the_vector_alu(cabi, spec, x_signed):
    """Depthwise layers, four channels per lane: every strip length against the oracle, with
    the integer sums, plain and fused requantisation."""
    say("conv depthwise lanes", spec, x_signed)
    b, h, w, ic, oc, k, st, p, dl, g = spec
    kh, kw = (k, k) if isinstance(k, int) else k
    c = _conv_case(b, h, w, ic, oc, kh, st, p, dl, g, seed=sum(spec[:5]) + 17, x_signed=x_signed, relu=x_signed)
    if kh != kw:
        rng = np.random.default_rng(5)
        c["wq"] = rng.integers(-127, 128, (oc, kh, kw, 1), dtype=np.int8)
    want_acc = oracle.conv2d_acc32(c["xq"], c["wq"], c["stride"], c["padding"], c["dilation"],
                                   c["groups"], c["x_zp"], nthreads=8)
    want = oracle.conv2d(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                         c["stride"], c["padding"], c["dilation"], c["groups"], c["out_scale"],
                         c["out_zp"], relu=c["relu"], nthreads=8)
    for strip in (0, 1, 3, 8):
        cabi.force_conv_path(7)
        cabi.force_conv_tile(strip, 0)
        try:
            y, acc, pw = _run(cabi, c)
        finally:
            cabi.force_conv_path(-1)
            cabi.force_conv_tile(0, 0)
        np.testing.assert_array_equal(acc, want_acc)
        _check(y, want, f"strip {strip}")
    y, acc, _ = _run(cabi, c)
    np.testing.assert_array_equal(acc, want_acc)
    _check(y, want, "automatic")
    # fused: residual + ReLU into a signed output, and SiLU
    rng = np.random.default_rng(sum(spec[:5]))
    for activation, signed in (("relu", True), ("silu", False)):
        f = dict(c, accq=(rng.integers(-128, 128, want.shape, dtype=np.int8) if activation == "relu" else None),
                 acc_scale=0.35, acc_zp=-7, activation=activation, signed=signed, relu=False,
                 out_zp=-20 if signed else 30)
        want_f = oracle.conv2d_fused(f["xq"], f["x_scale"], f["x_zp"], f["wq"], f["w_scales"], f["bias"],
                                     f["stride"], f["padding"], f["dilation"], f["groups"], f["out_scale"],
                                     f["out_zp"], accum=f["accq"], accum_scale=f["acc_scale"],
                                     accum_zp=f["acc_zp"], activation=activation, out_signed=signed, nthreads=8)
        cabi.force_conv_path(7)
        try:
            yf = _run_fused(cabi, f)
        finally:
            cabi.force_conv_path(-1)
        d = np.abs(yf.astype(np.int32) - want_f.astype(np.int32))
        if activation == "silu":
            assert d.max() <= LSB_TOL and np.count_nonzero(d) <= max(2, 0.001 * d.size), (d.max(), np.count_nonzero(d))
        else:
            assert d.max() == 0, f"{np.count_nonzero(d)} of {d.size} bytes differ (max {d.max()})"


@pytest.mark.parametrize("spec", [
    (2, 14, 14, 40, 40, 3, 1, 1, 1, 1),      # 3 x 3 over 40 channels: kernel rows of 128 padded bytes, 384 in all
    (1, 35, 35, 3, 16, 11, 4, 2, 1, 1),      # the 11 x 11 stride 4 first layer of an early image network
    (2, 9, 9, 72, 24, 3, 2, 1, 1, 1),
    (1, 10, 10, 300, 32, 1, 1, 0, 1, 1),     # a pointwise layer over 300 channels: then a linear layer over 304
    (2, 12, 12, 24, 32, 5, 1, 2, 2, 1),      # dilation keeps the byte-run kernel away
    (2, 12, 12, 3, 20, 3, 1, 1, 1, 1),       # a byte-run shape, pinned here
])
@pytest.mark.parametrize("x_signed", [False, True])
def test_conv_on_channel_padded_copy(cabi, spec, x_signed):
    """One group off the 16-channel grid: the MFMA kernels on a copy of the input with padded
    channels in the workspace, against the oracle and against the run without a workspace."""
    say("conv padded channels", spec, x_signed)
    c = _conv_case(*spec, seed=sum(spec) + 23, x_signed=x_signed, relu=not x_signed)
    want_acc = oracle.conv2d_acc32(c["xq"], c["wq"], c["stride"], c["padding"], c["dilation"],
                                   c["groups"], c["x_zp"], nthreads=8)
    want = oracle.conv2d(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                         c["stride"], c["padding"], c["dilation"], c["groups"], c["out_scale"],
                         c["out_zp"], relu=c["relu"], nthreads=8)
    g = cabi.conv_geom(c["xq"].shape, c["wq"].shape, c["stride"], c["padding"], c["dilation"], c["groups"])
    automatic = not (spec[3] == 3 and spec[5] == 3)   # (3 x 3 over 3 channels: the byte-run kernel's)
    assert (cabi.lib().tmq_conv2d_workspace_bytes(g) > 0) == automatic
    for path, workspace in ((8, True), (-1, True), (-1, False)):
        cabi.force_conv_path(path)
        cabi.use_conv_workspace(workspace)
        try:
            y, acc, _ = _run(cabi, c)
        finally:
            cabi.force_conv_path(-1)
            cabi.use_conv_workspace(True)
        np.testing.assert_array_equal(acc, want_acc)
        _check(y, want, f"path {path}, workspace {workspace}")
    cabi.force_conv_path(8)
    cabi.use_conv_workspace(False)
    try:
        with pytest.raises(cabi.TmqError):
            _run(cabi, c)
    finally:
        cabi.force_conv_path(-1)
        cabi.use_conv_workspace(True)
    # fused: residual + ReLU
    rng = np.random.default_rng(sum(spec))
    f = dict(c, accq=rng.integers(0, 256, want.shape, dtype=np.uint8), acc_scale=0.35, acc_zp=110,
             activation="relu", signed=False, relu=False, out_zp=20)
    want_f = oracle.conv2d_fused(f["xq"], f["x_scale"], f["x_zp"], f["wq"], f["w_scales"], f["bias"],
                                 f["stride"], f["padding"], f["dilation"], f["groups"], f["out_scale"],
                                 f["out_zp"], accum=f["accq"], accum_scale=f["acc_scale"],
                                 accum_zp=f["acc_zp"], activation="relu", out_signed=False, nthreads=8)
    cabi.force_conv_path(8)
    try:
        yf = _run_fused(cabi, f)
    finally:
        cabi.force_conv_path(-1)
    np.testing.assert_array_equal(yf, want_f)
    # groups, or channels already on the grid: not this path's
    for bad in [(1, 8, 8, 32, 16, 3, 1, 1, 1, 1), (1, 8, 8, 24, 24, 3, 1, 1, 1, 2)]:
        cb = _conv_case(*bad, seed=1)
        cabi.force_conv_path(8)
        try:
            with pytest.raises(cabi.TmqError):
                _run(cabi, cb)
        finally:
            cabi.force_conv_path(-1)


@pytest.mark.parametrize("spec", [
    (2, 14, 14, 24, 144, 1, 1, 0, 1, 1),     # 24 channels in: pixels at 8-byte addresses
    (1, 9, 9, 3, 5, 1, 1, 0, 1, 1),          # 3 in, 5 out: any address, two channel tiles, byte stores
    (2, 7, 7, 64, 256, 1, 1, 0, 1, 1),       # one whole k-step, four channel blocks
    (1, 5, 5, 256, 64, 1, 1, 0, 1, 1),       # four k-steps
    (3, 10, 10, 100, 40, 1, 1, 0, 1, 1),     # 100 in: the second k-step's last operand reaches into the next pixel
    (1, 20, 20, 16, 16, 1, 1, 0, 1, 1),
    (1, 3, 3, 32, 300, 1, 1, 0, 1, 1),       # fewer pixels than a piece, five channel blocks, the last one ragged
    (1, 33, 31, 32, 16, 1, 1, 0, 1, 1),      # more pieces than one round of the waves
])
@pytest.mark.parametrize("x_signed", [False, True])
def test_conv_pointwise_rows_from_memory(cabi, spec, x_signed):
    """Pointwise layers over at most 256 input channels: MFMA operands straight from the NHWC input."""
    say("conv pointwise rows", spec, x_signed)
    c = _conv_case(*spec, seed=sum(spec) + 29, x_signed=x_signed, relu=x_signed)
    want_acc = oracle.conv2d_acc32(c["xq"], c["wq"], c["stride"], c["padding"], c["dilation"],
                                   c["groups"], c["x_zp"], nthreads=8)
    want = oracle.conv2d(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                         c["stride"], c["padding"], c["dilation"], c["groups"], c["out_scale"],
                         c["out_zp"], relu=c["relu"], nthreads=8)
    cabi.force_conv_path(9)
    try:
        y, acc, _ = _run(cabi, c)
    finally:
        cabi.force_conv_path(-1)
    np.testing.assert_array_equal(acc, want_acc)
    _check(y, want, "pinned")
    y, acc, _ = _run(cabi, c)
    np.testing.assert_array_equal(acc, want_acc)
    _check(y, want, "automatic")
    rng = np.random.default_rng(sum(spec))
    for activation, signed in (("relu", True), ("silu", False)):
        f = dict(c, accq=(rng.integers(-128, 128, want.shape, dtype=np.int8) if activation == "relu" else None),
                 acc_scale=0.35, acc_zp=-7, activation=activation, signed=signed, relu=False,
                 out_zp=-20 if signed else 30)
        want_f = oracle.conv2d_fused(f["xq"], f["x_scale"], f["x_zp"], f["wq"], f["w_scales"], f["bias"],
                                     f["stride"], f["padding"], f["dilation"], f["groups"], f["out_scale"],
                                     f["out_zp"], accum=f["accq"], accum_scale=f["acc_scale"],
                                     accum_zp=f["acc_zp"], activation=activation, out_signed=signed, nthreads=8)
        cabi.force_conv_path(9)
        try:
            yf = _run_fused(cabi, f)
        finally:
            cabi.force_conv_path(-1)
        d = np.abs(yf.astype(np.int32) - want_f.astype(np.int32))
        if activation == "silu":
            assert d.max() <= LSB_TOL and np.count_nonzero(d) <= max(2, 0.001 * d.size), (d.max(), np.count_nonzero(d))
        else:
            assert d.max() == 0, f"{np.count_nonzero(d)} of {d.size} bytes differ (max {d.max()})"


@pytest.mark.parametrize("spec", [
    (8, 56, 56, 24, 144, 1, 1, 0, 1, 1),     # 1568 pieces, three channel blocks: the automatic choice at size
    (4, 112, 112, 32, 16, 1, 1, 0, 1, 1),    # 3136 pieces, two channel tiles
    (6, 56, 56, 256, 128, 1, 1, 0, 1, 1),    # four k-steps
    (4, 56, 56, 96, 96, 7, 1, 3, 1, 96),     # depthwise 7 x 7, whole strips and several blocks per image
    (3, 112, 112, 32, 32, 3, 1, 1, 1, 32),   # depthwise 3 x 3
    (2, 112, 112, 96, 96, 3, 2, 1, 1, 96),   # ... at stride 2
    (2, 56, 56, 40, 40, 3, 1, 1, 1, 1),      # channel-padded copy, then halo tiles
])
def test_conv_layers_of_mobile_networks_at_size(cabi, spec):
    """The kernels for pointwise, depthwise and off-grid layers as the library picks them at sizes where
    every lane, strip and block of theirs has work, against the oracle."""
    say("conv mobile layers at size", spec)
    c = _conv_case(*spec, seed=sum(spec) + 31, x_signed=False, relu=True)
    y, acc, _ = _run(cabi, c)
    np.testing.assert_array_equal(
        acc, oracle.conv2d_acc32(c["xq"], c["wq"], c["stride"], c["padding"], c["dilation"], c["groups"], c["x_zp"],
                                 nthreads=8))
    want = oracle.conv2d(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"], c["stride"],
                         c["padding"], c["dilation"], c["groups"], c["out_scale"], c["out_zp"], relu=c["relu"],
                         nthreads=8)
    _check(y, want, "at size")


@pytest.mark.parametrize("spec,path", [
    ((2, 20, 20, 64, 64, 3, 1, 1, 1, 1), 1), ((2, 20, 20, 64, 64, 3, 1, 1, 1, 1), 2), ((1, 14, 14, 256, 64, 3, 1, 1, 1, 1), 2),
    ((2, 19, 19, 3, 40, 7, 2, 3, 1, 1), 4), ((2, 14, 14, 24, 144, 1, 1, 0, 1, 1), 9), ((2, 14, 14, 256, 64, 1, 1, 0, 1, 1), 5),
    ((2, 19, 23, 72, 72, 3, 1, 1, 1, 72), 7), ((2, 15, 15, 96, 96, 7, 1, 3, 1, 96), 7), ((1, 9, 9, 40, 40, 3, 2, 1, 1, 40), 3),
    ((2, 14, 14, 40, 40, 3, 1, 1, 1, 1), 8), ((1, 7, 7, 512, 72, 3, 1, 1, 1, 1), 6), ((2, 12, 12, 96, 48, 3, 1, 1, 1, 4), -1),
])
@pytest.mark.parametrize("relu", [False, True])
def test_conv_unsigned_output_with_zero_point_0(cabi, spec, path, relu):
    """quint8 output with zero point 0 (what follows a ReLU) through every kernel family, plain and fused: the
    packing conversion alone rounds and saturates there."""
    say("conv zero point 0", spec, path, relu)
    c = _conv_case(*spec, seed=sum(spec) + 37, x_signed=False, relu=relu)
    c["out_zp"] = 0
    c["out_scale"] /= 3     # (255 at two standard deviations of the sums: the upper bound is met too)
    want = oracle.conv2d(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"], c["stride"],
                         c["padding"], c["dilation"], c["groups"], c["out_scale"], 0, relu=relu, nthreads=8)
    assert 0.25 < np.mean(want == 0) < 0.75 and np.any(want == 255)
    cabi.force_conv_path(path)
    try:
        y, _, _ = _run(cabi, c)
        _check(y, want, f"path {path}")
        if path not in (5, 6):   # (the linear kernels take no residual)
            rng = np.random.default_rng(3)
            for activation in ("relu", "silu"):
                f = dict(c, accq=rng.integers(0, 256, want.shape, dtype=np.uint8), acc_scale=0.35, acc_zp=110,
                         activation=activation, signed=False, relu=False)
                want_f = oracle.conv2d_fused(f["xq"], f["x_scale"], f["x_zp"], f["wq"], f["w_scales"], f["bias"],
                                             f["stride"], f["padding"], f["dilation"], f["groups"], f["out_scale"], 0,
                                             accum=f["accq"], accum_scale=0.35, accum_zp=110, activation=activation,
                                             out_signed=False, nthreads=8)
                yf = _run_fused(cabi, f)
                d = np.abs(yf.astype(np.int32) - want_f.astype(np.int32))
                if activation == "silu":
                    assert d.max() <= LSB_TOL and np.count_nonzero(d) <= max(2, 0.001 * d.size), (d.max(), np.count_nonzero(d))
                else:
                    assert d.max() == 0, f"{np.count_nonzero(d)} of {d.size} bytes differ (max {d.max()})"
    finally:
        cabi.force_conv_path(-1)


def test_conv_pointwise_rows_limits(cabi):
    """Not that kernel's: a 3 x 3 kernel, a stride, padding, groups, more than 256 input channels."""
    say("conv pointwise rows limits")
    for spec in [(1, 8, 8, 16, 16, 3, 1, 1, 1, 1), (1, 8, 8, 16, 16, 1, 2, 0, 1, 1), (1, 8, 8, 16, 16, 1, 1, 1, 1, 1),
                 (1, 8, 8, 32, 32, 1, 1, 0, 1, 2), (1, 4, 4, 272, 16, 1, 1, 0, 1, 1)]:
        c = _conv_case(*spec, seed=5)
        cabi.force_conv_path(9)
        try:
            with pytest.raises(cabi.TmqError):
                _run(cabi, c)
        finally:
            cabi.force_conv_path(-1)


def test_conv_depthwise_lanes_limits(cabi):
    """What the four-channels-per-lane kernel refuses: groups that are not single channels, channel
    counts off the dword grid, more output channels than input channels."""
    say("conv depthwise lanes limits")
    for spec in [(1, 8, 8, 32, 32, 3, 1, 1, 1, 1), (1, 8, 8, 32, 32, 3, 1, 1, 1, 16), (1, 8, 8, 10, 10, 3, 1, 1, 1, 10),
                 (1, 8, 8, 8, 16, 3, 1, 1, 1, 8)]:
        c = _conv_case(*spec, seed=3)
        cabi.force_conv_path(7)
        try:
            with pytest.raises(cabi.TmqError):
                _run(cabi, c)
        finally:
            cabi.force_conv_path(-1)
        y, _, _ = _run(cabi, c)   # ... and the automatic choice still serves
        want = oracle.conv2d(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                             c["stride"], c["padding"], c["dilation"], c["groups"], c["out_scale"],
                             c["out_zp"], relu=c["relu"], nthreads=8)
        _check(y, want, "automatic")


@pytest.mark.parametrize("spec", [
    (2, 14, 14, 256, 64, 1, 1, 0, 1, 1),
    (32, 7, 7, 512, 200, 1, 1, 0, 1, 1),     # 1568 pixels, channels off the 16 grid on the output side
    (1, 5, 5, 16, 24, 1, 1, 0, 1, 1),
    (3, 56, 56, 64, 48, 1, 1, 0, 1, 1),      # more pixels than the automatic choice sends this way
])
@pytest.mark.parametrize("x_signed", [False, True])
def test_conv_pointwise_as_linear(cabi, spec, x_signed):
    say("conv pointwise as linear", spec, x_signed)
    c = _conv_case(*spec, seed=sum(spec) + 13, x_signed=x_signed, relu=not x_signed)
    want = oracle.conv2d(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                         c["stride"], c["padding"], c["dilation"], c["groups"], c["out_scale"],
                         c["out_zp"], relu=c["relu"], nthreads=8)
    for path in (5, 1, -1):
        cabi.force_conv_path(path)
        try:
            y, _, _ = _run(cabi, c)
        finally:
            cabi.force_conv_path(-1)
        _check(y, want, f"path {path}")
    # not a pointwise layer: stride, padding, kernel size, groups
    for bad in [(1, 8, 8, 16, 16, 1, 2, 0, 1, 1), (1, 8, 8, 16, 16, 1, 1, 1, 1, 1), (1, 8, 8, 16, 16, 3, 1, 1, 1, 1),
                (1, 8, 8, 32, 32, 1, 1, 0, 1, 2)]:
        cb = _conv_case(*bad, seed=5)
        cabi.force_conv_path(5)
        try:
            with pytest.raises(cabi.TmqError):
                _run(cabi, cb)
        finally:
            cabi.force_conv_path(-1)


@pytest.mark.parametrize("spec", [
    (1, 14, 14, 256, 64, 3, 1, 1, 1, 1),     # 36 stages of 64 bytes: 18 per wave group
    (2, 7, 7, 512, 96, 3, 1, 1, 1, 1),       # 72 stages, channels over two tiles
    (1, 9, 9, 128, 64, 3, 2, 1, 1, 1),       # 18 stages (pinned only), stride 2
    (2, 10, 10, 256, 64, 3, 1, 1, 1, 2),     # two groups of 128 -> 32
    (1, 6, 6, 48, 40, 5, 1, 2, 1, 1),        # 1200 bytes of K: 19 stages, odd: refused
    (1, 8, 8, 128, 64, 3, 1, 1, 1, 1),       # 18 stages: two groups, not four
    (17, 14, 14, 256, 200, 3, 1, 1, 1, 1),   # 53 x 4 tiles of 64 x 64: tiles of 128 rows by themselves
])
@pytest.mark.parametrize("x_signed", [False, True])
@pytest.mark.parametrize("wave_groups,tile_rows", [(2, 0), (4, 0), (2, 128), (1, 128)],
                         ids=["two", "four", "two-128-rows", "one-128-rows"])
def test_conv_gemm_wave_groups(cabi, spec, x_signed, wave_groups, tile_rows):
    say("conv gemm wave groups", spec, x_signed, wave_groups, tile_rows)
    c = _conv_case(*spec, seed=sum(spec) + 17, x_signed=x_signed, relu=x_signed)
    kbytes = spec[5] * spec[5] * spec[3] // spec[9]
    even = (-(-kbytes // 64)) % wave_groups == 0
    cabi.force_conv_path(2)
    cabi.force_conv_tile(tile_rows, wave_groups)
    try:
        if not even:
            with pytest.raises(cabi.TmqError):
                _run(cabi, c)
            return
        y, acc, _ = _run(cabi, c)
    finally:
        cabi.force_conv_path(-1)
        cabi.force_conv_tile(0, 0)
    np.testing.assert_array_equal(
        acc, oracle.conv2d_acc32(c["xq"], c["wq"], c["stride"], c["padding"], c["dilation"], c["groups"], c["x_zp"],
                                 nthreads=8))
    want = oracle.conv2d(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"], c["stride"],
                         c["padding"], c["dilation"], c["groups"], c["out_scale"], c["out_zp"], relu=c["relu"],
                         nthreads=8)
    _check(y, want, "wave groups")
    y2, _, _ = _run(cabi, c)   # the automatic choice
    _check(y2, want, "auto")


@pytest.mark.parametrize("activation", ["relu", "silu"])
@pytest.mark.parametrize("wave_groups", [2, 4])
def test_conv_gemm_wave_groups_fused(cabi, activation, wave_groups):
    """residual and activation behind the wave groups' sum (256 -> 64 channels, 3 x 3, 14 x 14)."""
    say("conv gemm wave groups fused", activation, wave_groups)
    rng = np.random.default_rng(58)
    xq = rng.integers(0, 256, (2, 14, 14, 256), dtype=np.uint8)
    wq = rng.integers(-127, 128, (64, 3, 3, 256), dtype=np.int8)
    accq = rng.integers(0, 256, (2, 14, 14, 64), dtype=np.uint8)
    ws = (0.001 + 0.002 * rng.random(64)).astype(np.float32).astype(np.float64)
    bias = rng.standard_normal(64).astype(np.float32)
    c = dict(xq=xq, wq=wq, accq=accq, w_scales=ws, bias=bias, x_scale=0.02, x_zp=3, stride=(1, 1),
             padding=(1, 1), dilation=(1, 1), groups=1, out_scale=1.8, out_zp=20, acc_scale=0.35,
             acc_zp=110, activation=activation, signed=False)
    cabi.force_conv_path(2)
    cabi.force_conv_tile(0, wave_groups)
    try:
        y = _run_fused(cabi, c)
    finally:
        cabi.force_conv_path(-1)
        cabi.force_conv_tile(0, 0)
    want = oracle.conv2d_fused(xq, 0.02, 3, wq, ws, bias, (1, 1), (1, 1), (1, 1), 1, 1.8, 20, accum=accq,
                               accum_scale=0.35, accum_zp=110, activation=activation, nthreads=8)
    d = np.abs(y.astype(np.int32) - want.astype(np.int32))
    if activation == "silu":
        assert d.max() <= LSB_TOL and np.count_nonzero(d) <= 0.001 * d.size, (d.max(), np.count_nonzero(d))
    else:
        assert d.max() == 0, f"{np.count_nonzero(d)} of {d.size} bytes differ (max {d.max()})"


@pytest.mark.parametrize("spec", [
    (1, 7, 7, 512, 72, 3, 1, 1, 1, 1),       # one 7 x 7 image, K = 4608: the library asks for the workspace itself
    (2, 14, 14, 256, 96, 3, 1, 1, 1, 1),     # 392 pixels, K = 2304
    (3, 14, 14, 256, 64, 3, 2, 1, 1, 1),     # stride 2
    (2, 9, 9, 32, 24, 3, 2, 1, 1, 1),        # small K: pinned only
    (1, 10, 10, 16, 16, 3, 1, 2, 2, 1),      # dilation (pinned only)
    (1, 5, 5, 48, 20, 1, 1, 0, 1, 1),        # pointwise (pinned only): the patch rows are the pixels
    (8, 14, 14, 1024, 1280, 1, 2, 0, 1, 1),  # pointwise at stride 2 over many channels: its pixels gathered, by itself
    (1, 14, 14, 1024, 64, 1, 2, 0, 1, 1),    # ... over few pixels: halo tiles by themselves
])
@pytest.mark.parametrize("x_signed", [False, True])
def test_conv_on_patch_rows(cabi, spec, x_signed):
    say("conv on patch rows", spec, x_signed)
    c = _conv_case(*spec, seed=sum(spec) + 19, x_signed=x_signed, relu=not x_signed)
    want = oracle.conv2d(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"], c["stride"],
                         c["padding"], c["dilation"], c["groups"], c["out_scale"], c["out_zp"], relu=c["relu"],
                         nthreads=8)
    g = cabi.conv_geom(c["xq"].shape, c["wq"].shape, c["stride"], c["padding"], c["dilation"], c["groups"])
    oh, ow = cabi.conv_out_hw(g)
    kbytes = spec[5] * spec[5] * spec[3]
    asked = cabi.lib().tmq_conv2d_workspace_bytes(g)
    if spec[5] == 1 and spec[6] == 2:
        assert asked == (spec[0] * oh * ow * kbytes if spec[0] == 8 else 0)
    else:
        assert asked == (spec[0] * oh * ow * kbytes if kbytes >= 2048 else 0)
    for path, ws in ((6, True), (-1, True), (-1, False)):
        cabi.force_conv_path(path)
        cabi.use_conv_workspace(ws)
        try:
            y, _, _ = _run(cabi, c)
        finally:
            cabi.force_conv_path(-1)
            cabi.use_conv_workspace(True)
        _check(y, want, f"path {path} workspace {ws}")
    # pinned without a workspace, or for a shape that has no patch rows of whole 16-channel blocks
    cabi.force_conv_path(6)
    cabi.use_conv_workspace(False)
    try:
        with pytest.raises(cabi.TmqError):
            _run(cabi, c)
    finally:
        cabi.force_conv_path(-1)
        cabi.use_conv_workspace(True)
    for bad in [(1, 8, 8, 32, 32, 3, 1, 1, 1, 2), (1, 8, 8, 24, 16, 3, 1, 1, 1, 1)]:
        cb = _conv_case(*bad, seed=5)
        cabi.force_conv_path(6)
        try:
            with pytest.raises(cabi.TmqError):
                _run(cabi, cb)
        finally:
            cabi.force_conv_path(-1)


def _random_geometry(rng):
    """A small convolution drawn so that every kernel family comes up: few channels, narrow groups
    that merge (or cannot), whole 16-channel blocks, pointwise layers, long K."""
    kind = rng.integers(0, 6)
    k = int(rng.choice([1, 2, 3, 3, 5, 7]))
    s = int(rng.choice([1, 1, 2, 3]))
    p = int(rng.integers(0, k // 2 + 2))
    d = int(rng.choice([1, 1, 1, 2]))
    b = int(rng.integers(1, 4))
    h, w = int(rng.integers(5, 34)), int(rng.integers(5, 34))
    groups = 1
    if kind == 0:      # few input channels
        ic, oc = int(rng.choice([1, 2, 3, 4, 5, 8, 12, 24, 40, 72, 100])), int(rng.integers(1, 80))
    elif kind == 1:    # depthwise, with or without a channel multiplier
        ic = int(rng.choice([8, 16, 20, 32, 40, 48, 72, 96, 120, 144]))
        groups, oc = ic, ic * int(rng.choice([1, 1, 2]))
    elif kind == 2:    # narrow groups
        icg, ocg, groups = int(rng.choice([2, 4, 8, 24])), int(rng.choice([2, 4, 6, 16])), int(rng.choice([2, 4, 8, 16]))
        ic, oc = icg * groups, ocg * groups
    elif kind == 3:    # whole 16-channel blocks
        ic, oc = 16 * int(rng.integers(1, 9)), int(rng.integers(1, 150))
        groups = int(rng.choice([1, 1, 2])) if ic % 32 == 0 and oc % 2 == 0 else 1
    elif kind == 4:    # pointwise
        k, s, p, d = 1, int(rng.choice([1, 1, 2])), 0, 1
        ic, oc = int(rng.choice([16, 24, 64, 200, 256])), int(rng.integers(1, 300))
    else:              # long K on a small image
        k, d = 3, 1
        ic, oc, h, w = int(rng.choice([256, 512])), int(rng.choice([48, 64, 130])), int(rng.integers(5, 15)), int(rng.integers(5, 15))
    if (h + 2 * p - d * (k - 1) - 1) // s + 1 <= 0 or (w + 2 * p - d * (k - 1) - 1) // s + 1 <= 0:
        p = d * (k - 1)
    return (b, h, w, ic, oc, k, s, p, d, groups)


@pytest.mark.parametrize("seed", range(48))
def test_conv_random_geometries(cabi, seed):
    rng = np.random.default_rng(7000 + seed)
    spec = _random_geometry(rng)
    say("conv random geometry", seed, spec)
    c = _conv_case(*spec, seed=seed, x_signed=bool(seed & 1), relu=bool(seed & 2))
    y, acc, pw = _run(cabi, c)
    np.testing.assert_array_equal(
        acc, oracle.conv2d_acc32(c["xq"], c["wq"], c["stride"], c["padding"], c["dilation"], c["groups"], c["x_zp"],
                                 nthreads=8))
    np.testing.assert_array_equal(host(pw.colsum), c["wq"].reshape(c["wq"].shape[0], -1).astype(np.int64).sum(1))
    want = oracle.conv2d(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"], c["stride"],
                         c["padding"], c["dilation"], c["groups"], c["out_scale"], c["out_zp"], relu=c["relu"],
                         nthreads=8)
    _check(y, want, f"seed {seed} {spec}")


def test_conv_byte_runs_limits(cabi):
    """groups, dilation and kernel rows beyond 256 padded bytes are not this kernel's."""
    say("conv byte runs limits")
    for spec in [(1, 12, 12, 6, 6, 3, 1, 1, 1, 2), (1, 12, 12, 3, 8, 3, 1, 2, 2, 1), (1, 24, 24, 3, 8, 11, 1, 0, 1, 1)]:
        c = _conv_case(*spec, seed=3)
        cabi.force_conv_path(4)
        try:
            with pytest.raises(cabi.TmqError):
                _run(cabi, c)
        finally:
            cabi.force_conv_path(-1)
        y, acc, _ = _run(cabi, c)   # the direct kernel takes them
        np.testing.assert_array_equal(
            acc, oracle.conv2d_acc32(c["xq"], c["wq"], c["stride"], c["padding"], c["dilation"], c["groups"], c["x_zp"]))


def test_conv_first_layer_full_size(cabi):
    """[32, 224, 224, 3] (x) [64, 7, 7, 3], stride 2, pad 3, with ReLU: the first layer of a ResNet at batch 32."""
    say("conv first layer full size")
    c = _conv_case(32, 224, 224, 3, 64, 7, 2, 3, 1, 1, seed=77, relu=True)
    y, acc, _ = _run(cabi, c)
    np.testing.assert_array_equal(
        acc, oracle.conv2d_acc32(c["xq"], c["wq"], c["stride"], c["padding"], c["dilation"], c["groups"], c["x_zp"],
                                 nthreads=8))
    want = oracle.conv2d(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"], c["stride"],
                         c["padding"], c["dilation"], c["groups"], c["out_scale"], c["out_zp"], relu=True, nthreads=8)
    _check(y, want, "first layer")


def test_c5_full_size(cabi):
    """benchmark configuration 5: [32,56,56,64] (x) [64,3,3,64], stride 1, pad 1."""
    say("C5 full size")
    rng = np.random.default_rng(55)
    xf = np.maximum(rng.standard_normal((32, 56, 56, 64), dtype=np.float32), 0)
    wf = rng.standard_normal((64, 3, 3, 64), dtype=np.float32) * np.float32(0.05)
    xs, xz = oracle.choose_qparams(float(xf.min()), float(xf.max()))
    assert xz == 0
    xq = oracle.quantize_per_tensor(xf, xs, xz, False, nthreads=8)
    ws = (np.abs(wf).reshape(64, -1).max(axis=1) / np.float32(127.0)).astype(np.float64)
    wq = oracle.quantize_per_channel(wf, ws, np.zeros(64, np.int64), 0, True)
    c = dict(xq=xq, wq=wq, bias=rng.standard_normal(64).astype(np.float32), x_scale=xs, x_zp=xz,
             w_scales=ws, stride=(1, 1), padding=(1, 1), dilation=(1, 1), groups=1,
             out_scale=0.02, out_zp=128, relu=False)
    y, acc, _ = _run(cabi, c)
    np.testing.assert_array_equal(
        acc, oracle.conv2d_acc32(xq, wq, (1, 1), (1, 1), (1, 1), 1, xz, nthreads=8))
    want = oracle.conv2d(xq, xs, xz, wq, ws, c["bias"], (1, 1), (1, 1), (1, 1), 1, 0.02, 128,
                         nthreads=8)
    assert 0.2 < np.mean((want > 0) & (want < 255))
    _check(y, want, "C5")


# ---------------------------------------------------------------------------
# fused residual / activation variants
# ---------------------------------------------------------------------------
def _run_fused(cabi, c):
    g = cabi.conv_geom(c["xq"].shape, c["wq"].shape, c["stride"], c["padding"], c["dilation"],
                       c["groups"])
    pw = cabi.PackedConv2d(dev(c["wq"]), g)
    ws = dev(c["w_scales"].astype(np.float32))
    b = None if c["bias"] is None else dev(c["bias"])
    acc = None if c["accq"] is None else dev(c["accq"])
    y = cabi.conv2d_fused(dev(c["xq"]), pw, g, c["x_scale"], c["x_zp"], ws, b, c["out_scale"],
                          c["out_zp"], accum=acc, accum_scale=c["acc_scale"], accum_zp=c["acc_zp"],
                          activation=c["activation"], out_signed=c["signed"])
    return host(y)


@pytest.mark.parametrize("path", [-1, 2, 3, 4], ids=["auto", "gemm", "direct", "runs"])
@pytest.mark.parametrize("c", cases.conv_fused_cases(), ids=lambda c: c["name"])
def test_conv_fused(cabi, golden, c, path):
    say("conv fused", c["name"], path)
    if path == 2 and (c["xq"].shape[3] // c["groups"]) % 16 != 0:
        pytest.skip("the MFMA kernels need 16-channel blocks")
    if path == 4:
        oc_, kh_, kw_, ic_ = c["wq"].shape
        if c["groups"] != 1 or kh_ * (-(-kw_ * ic_ // 16) * 16) > 256:
            pytest.skip("the byte-run kernel takes one group and kernel rows of at most 256 padded bytes in all")
    cabi.force_conv_path(path)
    try:
        y = _run_fused(cabi, c)
    finally:
        cabi.force_conv_path(-1)
    want = oracle.conv2d_fused(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                               c["stride"], c["padding"], c["dilation"], c["groups"], c["out_scale"],
                               c["out_zp"], accum=c["accq"], accum_scale=c["acc_scale"],
                               accum_zp=c["acc_zp"], activation=c["activation"], out_signed=c["signed"],
                               nthreads=8)
    d = np.abs(y.astype(np.int32) - want.astype(np.int32))
    if c["activation"] == "silu":
        # expf on the device and on the host may differ in the last bit
        assert d.max() <= LSB_TOL and np.count_nonzero(d) <= 0.001 * d.size, (d.max(), np.count_nonzero(d))
    else:
        assert d.max() == 0, f"{np.count_nonzero(d)} of {d.size} bytes differ (max {d.max()})"
    dg = np.abs(y.astype(np.int32) - golden["convf/" + c["name"] + "/y"].astype(np.int32))
    assert dg.max() <= LSB_TOL and np.count_nonzero(dg) <= 0.003 * dg.size


def test_conv_fused_c5_sized(cabi):
    """conv2d_add_relu at benchmark configuration 5's size (the residual block of a ResNet stage)."""
    say("conv fused C5 size")
    rng = np.random.default_rng(56)
    xq = rng.integers(0, 256, (32, 56, 56, 64), dtype=np.uint8)
    wq = rng.integers(-127, 128, (64, 3, 3, 64), dtype=np.int8)
    accq = rng.integers(0, 256, (32, 56, 56, 64), dtype=np.uint8)
    ws = (0.001 + 0.002 * rng.random(64)).astype(np.float32).astype(np.float64)
    bias = rng.standard_normal(64).astype(np.float32)
    c = dict(xq=xq, wq=wq, accq=accq, w_scales=ws, bias=bias, x_scale=0.02, x_zp=3, stride=(1, 1),
             padding=(1, 1), dilation=(1, 1), groups=1, out_scale=0.9, out_zp=20, acc_scale=0.35,
             acc_zp=110, activation="relu", signed=False)
    y = _run_fused(cabi, c)
    want = oracle.conv2d_fused(xq, 0.02, 3, wq, ws, bias, (1, 1), (1, 1), (1, 1), 1, 0.9, 20, accum=accq,
                               accum_scale=0.35, accum_zp=110, activation="relu", nthreads=8)
    assert 0.2 < np.mean((want > 20) & (want < 255))
    np.testing.assert_array_equal(y, want)
