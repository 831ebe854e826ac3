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
    assert C.sizeof(cabi.LinearChoice) == 48
    assert C.sizeof(cabi.Conv2dGeom) == 14 * 8
    assert C.sizeof(cabi.Conv2dDesc) == 14 * 8 + 8 + 16 + 32 + 16 + 8 + 16 + 16
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
    # few input channels: 49 taps of 16 padded bytes (784 -> 896) for two blocks of 16 channels, then the
    # per-lane layout of the byte-run kernel: one 32-channel block x 2 channel tiles x 4 k-steps x 1 KB
    assert lib.tmq_conv2d_packed_bytes(g2) == 2 * 56 * 256 + 2 * 4 * 1024
    # (64 output channels: one block of four tiles)
    g2b = cabi.conv_geom((8, 32, 32, 3), (64, 7, 7), (2, 2), (3, 3), (1, 1), 1)
    assert lib.tmq_conv2d_packed_bytes(g2b) == 4 * 56 * 256 + 4 * 4 * 1024
    # kernel rows beyond 256 padded bytes in all (11 rows of 48): no second layout
    g3 = cabi.conv_geom((1, 64, 64, 3), (16, 11, 11), (4, 4), (0, 0), (1, 1), 1)
    assert lib.tmq_conv2d_packed_bytes(g3) == 1 * (121 * 16 + 127) // 128 * 8 * 256
    # depthwise, 32 channels: the 32 groups are packed as one block-diagonal group, K = 9 taps x 32 channels;
    # behind it, for channel counts on the dword grid, the weight once more as [channel][3 rows][4 bytes]
    g4 = cabi.conv_geom((1, 20, 20, 32), (32, 3, 3), (1, 1), (1, 1), (1, 1), 32)
    assert lib.tmq_conv2d_packed_bytes(g4) == 2 * 24 * 256 + 12 * 32
    # 144 channels: three merged groups of 48; 40 channels: no multiple of 16 divides them, 40 groups of one
    g5 = cabi.conv_geom((1, 20, 20, 144), (144, 3, 3), (1, 1), (1, 1), (1, 1), 144)
    assert lib.tmq_conv2d_packed_bytes(g5) == 3 * 3 * 32 * 256 + 12 * 144
    g6 = cabi.conv_geom((1, 20, 20, 40), (40, 3, 3), (1, 1), (1, 1), (1, 1), 40)
    assert lib.tmq_conv2d_packed_bytes(g6) == 40 * 1 * 16 * 256 + 12 * 40
    g7 = cabi.conv_geom((1, 20, 20, 10), (10, 3, 3), (1, 1), (1, 1), (1, 1), 10)                  # off the dword grid: no copy
    assert lib.tmq_conv2d_packed_bytes(g7) == 10 * 1 * 16 * 256
    # scratch for layers that run on their patch rows: few pixels against a long K that the halo tiles do not hold
    wsb = lib.tmq_conv2d_workspace_bytes
    assert wsb(cabi.conv_geom((1, 7, 7, 512), (512, 3, 3), (1, 1), (1, 1), (1, 1), 1)) == 49 * 4608
    assert wsb(cabi.conv_geom((2, 14, 14, 256), (256, 3, 3), (1, 1), (1, 1), (1, 1), 1)) == 392 * 2304
    assert wsb(cabi.conv_geom((8, 14, 14, 256), (256, 3, 3), (1, 1), (1, 1), (1, 1), 1)) == 0    # 1568 pixels
    assert wsb(g) == 0 and wsb(g2) == 0 and wsb(g4) == 0                                       # C5, few channels, depthwise
    assert wsb(cabi.conv_geom((1, 14, 14, 2048), (512, 1, 1), (1, 1), (0, 0), (1, 1), 1)) == 0    # pointwise: rows already
    # ... and for one group off the 16-channel grid under kernel rows too long for the byte-run kernel:
    # the input once more with 48 channels per pixel
    assert wsb(cabi.conv_geom((2, 20, 20, 40), (40, 3, 3), (1, 1), (1, 1), (1, 1), 1)) == 2 * 400 * 48
    assert wsb(cabi.conv_geom((2, 20, 20, 24), (40, 3, 3), (1, 1), (1, 1), (1, 1), 1)) == 0      # 3 rows of 80 bytes: byte runs
    assert wsb(cabi.conv_geom((2, 20, 20, 40), (40, 3, 3), (1, 1), (1, 1), (1, 1), 2)) == 0      # groups


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


# ---- the automatic kernel choice of quantized::linear, swept on the host.  Each kernel's
# preconditions are restated here from the kernels' own index arithmetic and LDS / register
# budgets (not from the dispatcher's code): a choice outside them is a wrong result or a fault.
def _ceil(a, b):
    return -(-a // b)


def _check_choice(c, m, n, k, ldx, out, workspace, misaligned, forced=0, cus=256):
    what = (m, n, k, ldx, out, workspace, misaligned, forced, c)
    cfg = c["kernel"] - 1
    kt = _ceil(k, 64)
    assert c["k_stages"] == kt, what
    vec_ok = (not misaligned) and k >= 16 and k % 16 == 0 and ldx % 16 == 0
    if cfg == 9 - 0 and not vec_ok:
        assert c["tile_rows"] == 0 and c["blocks"] == _ceil(m * _ceil(n, 4), 256), what
        return
    # every other kernel loads 16 aligned bytes per lane
    assert vec_ok or cfg == 9, what
    if cfg == 9:
        return
    bm, bn = c["tile_rows"], c["tile_channels"]
    tiles = _ceil(m, bm) * _ceil(n, bn)
    assert c["tiles"] == tiles * c["splits"] and 0 < c["blocks"] <= c["tiles"] < 2 ** 31, what
    if cfg != 13:
        assert c["splits"] == 1, what
    if cfg == 8:                                    # weight streaming: up to four groups of 16 rows
        assert m <= 64 and bm == 16 * _ceil(m, 16) and bn == 16 and k <= 0x7fffff00 and ldx < 2 ** 31, what
    elif cfg == 13:                                 # split K: runs of whole stages into a workspace
        sp, st = c["splits"], c["split_stages"]
        assert workspace and (bm, bn) == (128, 128) and sp >= 2 and tiles * sp <= 256, what
        assert (sp - 1) * st < kt and kt - (sp - 1) * st >= 6 and st >= 6, what
        assert cabi.lib().tmq_linear_workspace_bytes(m, n, k) == sp * m * _ceil(n, 4) * 4 * 4, what
    elif cfg in (6, 7, 19, 20):                     # direct copies two stages wide: K walked in runs of six stages,
        assert kt >= 6 and 256 * ldx <= 2 ** 31 and 15 * 16 * _ceil(k, 128) * 128 < 2 ** 32, what   # 32-bit offsets
        if cfg == 20:                               # persistent: byte / float outputs, several rounds, whole XCD runs
            assert out != "acc32" and (bm, bn) == (256, 256), what
            # (the tile sequence is a permutation only on a multiple of 8 blocks or with every tile in one round)
            assert c["blocks"] == (cus // 8 * 8 if tiles > cus else tiles), what
        else:
            assert c["blocks"] == tiles, what
    elif cfg == 17:                                 # direct copies one stage wide: a ring of three stages
        assert kt >= 3 and 256 * ldx <= 2 ** 31, what
    elif cfg == 14:                                 # two wave groups halve the k loop
        assert kt % 2 == 0 and (bm, bn) == (64, 64), what
        if forced == 0:
            assert tiles <= 256 and kt >= 32, what
    elif cfg == 21:                                 # 64 x 64, four phases of 256 bytes of K in LDS: all of K <= 1024,
        assert (bm, bn) == (64, 64) and 64 * ldx <= 2 ** 29, what      # a longer K as a ring of phases
        if forced == 0:                             # one round; the ring only beyond the kernels with weights in registers
            assert tiles <= 256 and (k <= 1024 or (k >= 4096 and m <= 128)), what
    elif cfg == 24:                                 # all of K in LDS, 32 x 32, a quarter of K per wave
        assert k <= 1024 and (bm, bn) == (32, 32) and 64 * ldx <= 2 ** 29, what
        if forced == 0:
            assert tiles <= 512 and k > 256, what
    elif cfg == 25:                                 # weights through registers: 32 fragments per wave at most
        assert k <= 4096 and (bm, bn) == (32, 32) and 64 * ldx <= 2 ** 29, what
        if forced == 0:                             # one round: two blocks per CU while 32 x K <= 64 KB
            assert k > 1024 and tiles <= (512 if k <= 2048 else 256), what
    elif cfg == 26:
        assert k <= 4096 and (bm, bn) == (32, 64) and c["waves"] == 8 and 64 * ldx <= 2 ** 29, what
        if forced == 0:
            assert k > 2048 and tiles <= 256, what
    elif cfg == 27:                                 # 64 x 64, an eighth of K per wave: 16 k-steps of weights in registers
        assert k <= 4096 and (bm, bn) == (64, 64) and c["waves"] == 8 and 64 * ldx <= 2 ** 29, what
        if forced == 0:                             # one round, and a K long enough to fill the waves' shares
            assert k >= 3072 and tiles <= 256, what
    elif cfg == 28:                                 # activations resident in LDS: 16 MG x K bytes, K padded to 16 k-blocks,
        mg = _ceil(m, 16)                           # in 128 KB; the constants of at most 64 channel groups per block
        assert m <= 64 and (bm, bn) == (16 * mg, 16) and c["waves"] in (8, 16), what
        if c["waves"] == 16:                        # one block per CU
            assert 16 * mg * _ceil(k, 1024) * 1024 <= 128 * 1024 and _ceil(n, 16) <= 64 * cus, what
            assert c["blocks"] == min(tiles, cus), what
        else:                                       # two blocks of eight waves per CU: half the LDS area, 32 groups each
            assert mg == 1 and 16 * _ceil(k, 512) * 512 <= 64 * 1024 and 2 * cus <= _ceil(n, 16) <= 64 * cus, what
            assert c["blocks"] == min(tiles, 2 * cus), what
        if forced == 0:                             # rows that share the streamed weights, or a short K
            assert k >= 1024 and m <= 32 and (m <= 16 or 10240 <= n <= 20480), what
        return
    else:                                           # register-staged tiles take any aligned shape
        assert cfg in (0, 1, 2, 3, 4, 5, 22, 23), what
    if forced == 0 and cfg in (22, 23):             # a few hundred rows: one round of oblong tiles; up to 64 rows: any number
        assert tiles <= 256 or (cfg == 23 and m <= 64), what


def _random_linear_shapes(rng, count):
    for _ in range(count):
        m = int(2 ** rng.uniform(0, 13.2))
        n = int(2 ** rng.uniform(0, 15.7))
        k = 16 * int(2 ** rng.uniform(0, 11.2))
        if rng.random() < 0.1:
            k += int(rng.integers(1, 16))           # not a multiple of 16: the plain kernel's
        if rng.random() < 0.25:                     # the sizes the thresholds were fitted at
            m = int(rng.choice([1, 16, 17, 24, 25, 32, 64, 65, 96, 128, 200, 256, 448, 512, 1024, 2048, 4096]))
            n = int(rng.choice([1024, 2048, 4096, 8192, 11008, 12288, 32000]))
            k = int(rng.choice([256, 272, 512, 1024, 1040, 2048, 2064, 3072, 4096, 4112, 8192, 11008]))
        ldx = k + (16 * int(rng.integers(0, 9)) if rng.random() < 0.2 else 0)
        if rng.random() < 0.02:
            ldx = k + int(rng.integers(1, 16))      # a pitch that breaks the alignment
        yield m, n, k, ldx


def test_automatic_kernel_choice_keeps_every_kernels_preconditions():
    rng = np.random.default_rng(20)
    seen = set()
    for m, n, k, ldx in _random_linear_shapes(rng, 6000):
        for out in ("bytes", "f32", "acc32"):
            for workspace in (False, True):
                c = cabi.linear_kernel_choice(m, n, k, ldx, out, workspace)
                assert c["kernel"] != 0, (m, n, k, ldx, out, workspace)      # the automatic choice always runs
                _check_choice(c, m, n, k, ldx, out, workspace, False)
                seen.add(c["kernel"] - 1)
    # huge pitches and K: the 32-bit offset limits of the direct-copy kernels
    for m, n, k, ldx in ((4096, 11008, 4096, 2 ** 23 + 16), (4096, 11008, 2 ** 23 + 64, 2 ** 23 + 64),
                         (512, 4096, 4096, 2 ** 24), (128, 1024, 1024, 2 ** 23 + 16), (64, 4096, 4096, 2 ** 23 + 16)):
        for out in ("bytes", "acc32"):
            c = cabi.linear_kernel_choice(m, n, k, ldx, out)
            assert c["kernel"] != 0
            _check_choice(c, m, n, k, ldx, out, False, False)
            seen.add(c["kernel"] - 1)
    c = cabi.linear_kernel_choice(300, 500, 4096, misaligned=True)
    assert c["kernel"] == 10
    assert seen >= {2, 3, 7, 8, 9, 13, 14, 17, 19, 20, 21, 22, 23, 24, 25, 26, 27, 28}, sorted(seen)
    # the benchmark configurations
    assert cabi.linear_kernel_choice(4096, 11008, 4096)["kernel"] - 1 == 20
    assert cabi.linear_kernel_choice(4096, 11008, 4096)["blocks"] == 256
    assert cabi.linear_kernel_choice(4096, 11008, 4096, compute_units=252)["blocks"] == 248
    assert cabi.linear_kernel_choice(128, 1024, 1024)["kernel"] - 1 == 24
    for m in (1, 4, 16):
        assert cabi.linear_kernel_choice(m, 4096, 4096)["kernel"] - 1 == 8
    assert cabi.linear_kernel_choice(0, 4096, 4096) == dict(kernel=0, tile_rows=0, tile_channels=0, waves=0, splits=1,
                                                           split_stages=0, tiles=0, blocks=0, k_stages=64)


def test_forced_kernels_run_inside_their_preconditions_or_not_at_all():
    rng = np.random.default_rng(21)
    refused = 0
    for m, n, k, ldx in _random_linear_shapes(rng, 1500):
        for cfg in (0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 13, 14, 17, 19, 20, 21, 22, 23, 24, 25, 26, 27, 28):
            for out in ("bytes", "acc32"):
                c = cabi.linear_kernel_choice(m, n, k, ldx, out, workspace=True, forced=cfg + 1)
                if c["kernel"] == 0:
                    refused += 1
                    continue
                _check_choice(c, m, n, k, ldx, out, True, False, forced=cfg + 1)
    assert refused > 0
    with pytest.raises(cabi.TmqError):
        cabi.linear_kernel_choice(8, 8, 64, ldx=32)


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
