"""CPU-side checks of the C-ABI library: it loads, exports every symbol that
include/tmq.h declares, and its host-only entry points agree with the oracle.
No kernel is launched here."""
import os
import re

import numpy as np
import pytest

import cases
import oracle
from torch_musa_amd import cabi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_in_header():
    text = open(os.path.join(ROOT, "include", "tmq.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tmq_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_list_agree():
    assert _declared_in_header() == sorted(cabi.DECLARED_SYMBOLS)


def test_library_exports_every_declared_symbol():
    lib = cabi.lib()
    for name in _declared_in_header():
        assert hasattr(lib, name), f"{name} is declared in include/tmq.h but not exported"
    assert lib.tmq_version() == 100
    assert lib.tmq_status_string(0) == b"ok"
    assert lib.tmq_status_string(3) != lib.tmq_status_string(4)


def test_measurement_probe_lives_in_its_own_library():
    # include/tmq_bench.h is bench.py's, not the operator boundary: its symbols are
    # exported by libtmq_bench.so and absent from libtmq.so
    text = open(os.path.join(ROOT, "include", "tmq_bench.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = sorted(set(re.findall(r"\b(tmq_[a-z0-9_]+)\s*\(", text)))
    assert names == ["tmq_bench_empty_kernel", "tmq_bench_stream_read", "tmq_probe_mfma_i8"]
    for name in names:
        assert hasattr(cabi.bench_lib(), name)
        assert not hasattr(cabi.lib(), name)
        assert name not in cabi.DECLARED_SYMBOLS


def test_struct_sizes_match_the_header():
    # natural alignment on x86-64: see include/tmq.h
    import ctypes as C
    assert C.sizeof(cabi.QParams) == 16
    assert C.sizeof(cabi.LinearDesc) == 144
    assert C.sizeof(cabi.Conv2dGeom) == 14 * 8
    assert C.sizeof(cabi.Conv2dDesc) == 14 * 8 + 8 + 16 + 32 + 16 + 8 + 16
    assert C.sizeof(cabi.Conv2dPost) == 24


def test_packed_size_arithmetic():
    lib = cabi.lib()
    assert lib.tmq_linear_packed_kchunks(1) == 8
    assert lib.tmq_linear_packed_kchunks(128) == 8
    assert lib.tmq_linear_packed_kchunks(129) == 16
    assert lib.tmq_linear_packed_bytes(11008, 4096) == 11008 * 4096
    assert lib.tmq_linear_packed_bytes(17, 130) == 2 * 16 * 256
    g = cabi.conv_geom((32, 56, 56, 64), (64, 3, 3), (1, 1), (1, 1), (1, 1), 1)
    assert cabi.conv_out_hw(g) == (56, 56)
    assert lib.tmq_conv2d_packed_bytes(g) == 4 * 40 * 256  # K = 576 -> 640 padded
    g2 = cabi.conv_geom((8, 32, 32, 3), (32, 7, 7), (2, 2), (3, 3), (1, 1), 1)
    assert cabi.conv_out_hw(g2) == (16, 16)


def test_split_k_workspace_arithmetic():
    # host-only: which problem sizes ask for a split-K workspace, and how much
    wsb = cabi.lib().tmq_linear_workspace_bytes
    assert wsb(16, 4096, 11008) == 0 and wsb(32, 4096, 11008) == 0     # weight-streaming rows
    assert wsb(64, 4096, 11008) == 8 * 64 * 4096 * 4                   # 33 ... 64 rows against a long K: split
    assert wsb(64, 4096, 4096) == 0 and wsb(48, 11008, 4096) == 0      # (K too short for it)
    assert wsb(128, 4096, 4096) == 0                                   # K too short to repay the partial sums
    assert wsb(4096, 11008, 4096) == 0 and wsb(2048, 4096, 16384) == 0  # grids that fill the chip
    assert wsb(128, 4096, 11008) == 8 * 128 * 4096 * 4                 # 32 tiles of 128 x 128 -> 8 splits
    assert wsb(512, 4096, 11008) == 2 * 512 * 4096 * 4                 # 128 tiles -> 2 splits
    assert wsb(100, 30, 8192) == 8 * 100 * 32 * 4                      # rows of partial sums padded to 16 bytes
    assert wsb(128, 4096, 8200) == 0                                   # K not a multiple of 16: plain kernel
    assert wsb(0, 8, 8192) == 0 and wsb(-3, 8, 8192) == 0


def test_split_k_plan_covers_k():
    # The plan is `splits` runs of `stages` k-stages with the last run taking
    # whatever is left: every run must start inside K, the last one must hold at
    # least six stages (one turn of the direct-copy ring), and the workspace
    # figure must follow from the plan.  Shapes include those where a short tail
    # is merged into the split before it (K = 16640, 13328).
    wsb = cabi.lib().tmq_linear_workspace_bytes
    merged = 0
    shapes = [(128, 1024, 16640), (128, 128, 13328), (100, 520, 8208), (130, 4096, 11008)]
    rng = np.random.default_rng(7)
    for _ in range(4000):
        shapes.append((int(rng.integers(65, 1100)), int(rng.integers(16, 5000)),
                       16 * int(rng.integers(8192 // 16, 40000 // 16))))
    for m, n, k in shapes:
        splits, stages = cabi.linear_split_plan(m, n, k)
        kt = -(-k // 64)
        if splits == 1:
            assert wsb(m, n, k) == 0
            continue
        assert splits >= 2 and stages >= 16
        assert (splits - 1) * stages < kt, (m, n, k, splits, stages)
        last = kt - (splits - 1) * stages
        assert last >= 6, (m, n, k, splits, stages)
        merged += last > stages
        assert wsb(m, n, k) == splits * m * (-(-n // 4) * 4) * 4
    assert merged > 0, "no shape exercised the merged tail"
    assert cabi.linear_split_plan(128, 1024, 16640) == (15, 17)    # 260 stages: 14 x 17 + 22
    assert cabi.linear_split_plan(128, 128, 13328) == (12, 17)     # 209 stages: 11 x 17 + 22


def test_host_choose_qparams_matches_oracle(golden):
    for mn, mx in cases.dynamic_qparams_cases():
        for rr in (False, True):
            for signed in (False, True):
                assert cabi.choose_qparams_host(float(mn), float(mx), signed, rr) == \
                    oracle.choose_qparams(mn, mx, signed, rr)
    for mn, mx, rr, s, z in golden["dynq/pairs"]:
        assert cabi.choose_qparams_host(mn, mx, False, bool(rr)) == (s, int(z))
    with pytest.raises(cabi.TmqError):
        cabi.choose_qparams_host(1.0, -1.0, False, False)
