"""tmq_linear_static_workspace: quantized::linear whose split-K partial sums live in a
fixed array inside the library, for callers that cannot allocate.  Its bytes must equal
those of tmq_linear with a caller-owned workspace (and the oracle's) on calls in a row
that share the array, the second smaller than the first."""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle
from gpu_util import dev, host, say
from test_gpu_linear import _tile_case

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def cabi():
    from torch_musa_amd import cabi as m
    assert torch.cuda.is_available()
    m.force_linear_config(-1)
    return m


def _both(cabi, c, allocations_allowed=True):
    pw = cabi.PackedLinear(dev(c["wq"]))
    xq, ws = dev(c["xq"]), dev(c["w_scales"].astype(np.float32))
    b = None if c["bias"] is None else dev(c["bias"])
    signed = c["xq"].dtype == np.int8
    args = (xq, pw, c["x_scale"], c["x_zp"], ws, b, c["out_scale"], c["out_zp"])
    want = cabi.linear(*args, out_signed=signed, relu=c["relu"])
    out = torch.empty_like(want)
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    free_before, _ = torch.cuda.mem_get_info()       # the driver's own count: sees a hipMalloc inside the library too
    got = cabi.linear_static_workspace(*args, out_signed=signed, relu=c["relu"], out=out)
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == before, "the call allocated through torch"
    assert torch.cuda.mem_get_info()[0] == free_before, "the call changed the device's free memory"
    return host(got), host(want)


def test_static_workspace_matches_caller_workspace(cabi):
    shapes = [((130, 4096, 11008), False, True, True, True),     # 4 splits, 8.5 MB of partial sums
              ((100, 520, 8208), False, False, True, True),      # smaller: 8 splits, 1.7 MB, ragged
              ((128, 128, 13328), True, False, True, False),     # the merged tail, qint8
              ((96, 512, 1024), False, True, True, True)]        # no split at all: the array is not touched
    for i, (shape, x_signed, relu, bias, pc) in enumerate(shapes):
        say("static workspace", shape)
        M, N, K = shape
        assert (cabi.lib().tmq_linear_workspace_bytes(M, N, K) > 0) == (i < 3)
        c = _tile_case(M, N, K, seed=900 + i, x_signed=x_signed, relu=relu, bias=bias, per_channel=pc)
        got, want = _both(cabi, c)
        np.testing.assert_array_equal(got, want)
        ref = oracle.linear(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                            c["out_scale"], c["out_zp"], relu=c["relu"], nthreads=8)
        np.testing.assert_array_equal(got, ref)


def test_static_workspace_argument_checks(cabi):
    assert cabi.lib().tmq_linear_static_workspace(None, None) == 1          # invalid argument
    d = cabi.LinearDesc()
    d.M, d.N, d.K = -1, 4, 4
    assert cabi.lib().tmq_linear_static_workspace(C.byref(d), None) == 1
    d.M = 0
    assert cabi.lib().tmq_linear_static_workspace(C.byref(d), None) == 0    # empty batch: nothing to do
    # every split plan fits the array
    worst = max(cabi.lib().tmq_linear_workspace_bytes(m, n, k)
                for m in (65, 128, 129, 256, 511, 1024) for n in (16, 128, 4096, 16384, 49152)
                for k in (8192, 11008, 16384, 65536))
    assert 0 < worst <= 16 * 1024 * 1024
