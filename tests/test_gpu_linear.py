"""GPU parity of quantized::linear through the C ABI.

int32 accumulators: bit-exact against the oracle (exact integer matmul).
Requantised bytes: the stated bar is 1 LSB; the epilogue restates the oracle's
operation order, so the tests also report (and require) exact equality against
the oracle, and stay within 1 LSB of the golden vectors of PyTorch's CPU op."""
import ctypes as C
import numpy as np
import pytest
import torch

import cases
import oracle
from gpu_util import dev, host, say

pytestmark = pytest.mark.gpu

LSB_TOL = 1  # north-star tolerance for requantised int8/uint8 outputs


@pytest.fixture(scope="module")
def cabi():
    from torch_musa_amd import cabi as m
    assert torch.cuda.is_available()
    m.lib()
    yield m
    m.force_linear_config(-1)


def _run(cabi, c, cfg=-1, x=None):
    xq = c["xq"] if x is None else x
    pw = cabi.PackedLinear(dev(c["wq"]))
    ws = dev(c["w_scales"].astype(np.float32))
    b = None if c["bias"] is None else dev(c["bias"])
    cabi.force_linear_config(cfg)
    try:
        y = cabi.linear(dev(xq), pw, c["x_scale"], c["x_zp"], ws, b, c["out_scale"], c["out_zp"],
                        relu=c["relu"])
        acc = cabi.linear_acc32(dev(xq), pw)
    finally:
        cabi.force_linear_config(-1)
    return host(y), host(acc), pw


def _check(y, want, what):
    d = np.abs(y.astype(np.int32) - want.astype(np.int32))
    assert d.max() <= LSB_TOL, f"{what}: max diff {d.max()}"
    assert d.max() == 0, f"{what}: {np.count_nonzero(d)} of {d.size} bytes differ by 1 LSB"


@pytest.mark.parametrize("c", cases.linear_cases(), ids=lambda c: c["name"])
def test_linear_cases(cabi, golden, c):
    say("lin", c["name"], c["xq"].shape, c["wq"].shape)
    y, acc, pw = _run(cabi, c)
    np.testing.assert_array_equal(acc, oracle.linear_acc32(c["xq"], c["wq"]))
    np.testing.assert_array_equal(host(pw.colsum), oracle.weight_colsum(c["wq"]))
    np.testing.assert_array_equal(host(pw.unpack()), c["wq"])
    want = oracle.linear(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                         c["out_scale"], c["out_zp"], relu=c["relu"])
    _check(y, want, "vs oracle")
    _check(y, golden["lin/" + c["name"] + "/y"], "vs golden")


def _tile_case(m, n, k, seed, x_signed=False, relu=False, bias=True, per_channel=True):
    rng = np.random.default_rng(seed)
    xq = (rng.integers(-128, 128, (m, k), dtype=np.int8) if x_signed
          else rng.integers(0, 256, (m, k), dtype=np.uint8))
    wq = rng.integers(-127, 128, (n, k), dtype=np.int8)
    ws = (0.001 + 0.002 * rng.random(n if per_channel else 1)).astype(np.float32).astype(np.float64)
    x_scale = 0.02
    sigma = np.sqrt(k) * 74.0 * 74.0 * x_scale * float(ws.mean())
    return dict(xq=xq, wq=wq, bias=(rng.standard_normal(n).astype(np.float32) * np.float32(sigma)) if bias else None,
                x_scale=x_scale, x_zp=-5 if x_signed else 121, w_scales=ws,
                out_scale=float(np.float32(3 * sigma / 128)), out_zp=-3 if x_signed else 128,
                relu=relu)


@pytest.mark.parametrize("cfg", [-1, 2, 9])
def test_per_tensor_weight_bias_form(cabi, golden, cfg):
    # rows picked where the two ways of adding the bias requantise differently: the
    # kernels take fma(bias, 1 / atw, raw) for a per-tensor weight, as the CPU op does
    say("per-tensor bias form", cfg)
    x_scale, x_zp, w_scale, out_scale, out_zp = golden["ptbias/params"]
    c = dict(xq=golden["ptbias/xq"], wq=golden["ptbias/wq"], bias=golden["ptbias/bias"], x_scale=float(x_scale),
             x_zp=int(x_zp), w_scales=np.array([float(w_scale)]), out_scale=float(out_scale), out_zp=int(out_zp),
             relu=False)
    y, _, _ = _run(cabi, c, cfg)
    np.testing.assert_array_equal(y, golden["ptbias/y"])


# every tile configuration of the MFMA kernel, with ragged M / N / K-stage tails
@pytest.mark.parametrize("cfg", [0, 1, 2, 3, 4, 5, 6, 7, 9, 17, 19, 20, 21, 22, 23, 24, 25, 26, 27])
@pytest.mark.parametrize("shape", [(300, 520, 448), (257, 33, 64), (64, 1040, 1168), (130, 260, 144), (256, 256, 192),
                                   (270, 300, 400), (40, 70, 784)])
def test_tile_configs(cabi, cfg, shape):
    say("tile cfg", cfg, shape)
    if cfg == 24 and shape[2] > 1024:
        pytest.skip("the 32 x 32 tiles whose waves split K take K <= 1024")
    c = _tile_case(*shape, seed=cfg * 10 + shape[0])
    y, acc, _ = _run(cabi, c, cfg)
    np.testing.assert_array_equal(acc, oracle.linear_acc32(c["xq"], c["wq"]))
    want = oracle.linear(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                         c["out_scale"], c["out_zp"], relu=c["relu"])
    _check(y, want, f"cfg {cfg}")


@pytest.mark.parametrize("shape, kw", [
    ((1300, 4300, 704), dict(x_signed=False, relu=False, bias=True, per_channel=True)),    # 102 tiles, one per block
    ((4389, 4120, 448), dict(x_signed=False, relu=True, bias=False, per_channel=False)),   # 306 tiles: 50 blocks take two
])
def test_persistent_kernel_one_and_several_tiles_per_block(cabi, shape, kw):
    """The persistent GEMM on a grid smaller than the chip and on one where some blocks walk a
    second tile (ragged rows and channels in both): accumulators and bytes equal the oracle's."""
    say("persistent kernel", shape)
    c = _tile_case(*shape, seed=77 + shape[0] % 7, **kw)
    y, acc, _ = _run(cabi, c, 20)
    np.testing.assert_array_equal(acc, oracle.linear_acc32(c["xq"], c["wq"], nthreads=8))
    want = oracle.linear(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                         c["out_scale"], c["out_zp"], relu=c["relu"], nthreads=8)
    _check(y, want, "cfg 20")


# all of K in LDS (K <= 1024): every number of 256-byte phases, K that ends inside a phase and on
# an odd 16-byte chunk, one row, ragged rows and channels, both activation types, every epilogue
@pytest.mark.parametrize("shape", [(128, 1024, 1024), (1, 16, 16), (64, 64, 32), (65, 70, 48), (100, 130, 1008),
                                   (33, 200, 272), (257, 129, 528), (1000, 1000, 1024), (90, 33, 784)])
@pytest.mark.parametrize("x_signed", [False, True])
# 64 x 64 tiles; 32 x 32 tiles whose waves split K, weights through LDS / through registers
@pytest.mark.parametrize("cfg", [21, 24, 25])
def test_whole_k_in_lds_kernel(cabi, shape, x_signed, cfg):
    say("K in LDS", shape, x_signed, cfg)
    M, N, K = shape
    c = _tile_case(M, N, K, seed=2100 + M, x_signed=x_signed, relu=N % 2 == 1, bias=M % 3 != 0,
                   per_channel=(M + N) % 2 == 0)
    y, acc, pw = _run(cabi, c, cfg)
    np.testing.assert_array_equal(acc, oracle.linear_acc32(c["xq"], c["wq"], nthreads=8))
    want = oracle.linear(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                         c["out_scale"], c["out_zp"], relu=c["relu"], nthreads=8)
    _check(y, want, "K in LDS")
    ws = dev(c["w_scales"].astype(np.float32))
    b = None if c["bias"] is None else dev(c["bias"])
    cabi.force_linear_config(cfg)
    try:
        yf = host(cabi.linear_f32(dev(c["xq"]), pw, c["x_scale"], c["x_zp"], ws, b, relu=c["relu"]))
    finally:
        cabi.force_linear_config(-1)
    np.testing.assert_array_equal(
        yf, oracle.linear_f32(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"], relu=c["relu"],
                              nthreads=8))
    if M * N <= 64 * 64 * 256:      # the automatic choice for grids no larger than the chip
        y1, acc1, _ = _run(cabi, c)
        np.testing.assert_array_equal(y1, y)
        np.testing.assert_array_equal(acc1, acc)


# 32 x 32 tiles whose waves split K with the weights through registers: K up to 4096 (both
# instantiations: 16 and 32 k-steps per wave), K that leaves waves without work, odd chunks
@pytest.mark.parametrize("shape", [(64, 160, 4096), (33, 200, 2064), (100, 130, 4080), (17, 70, 3088),
                                   (128, 64, 2048), (40, 33, 1040), (5, 32, 2304), (200, 300, 3600), (256, 192, 16)])
@pytest.mark.parametrize("x_signed", [False, True])
@pytest.mark.parametrize("cfg", [25, 26, 27])   # 32 x 32, 32 x 64, and 64 x 64 tiles with an activation ring
def test_weights_through_registers_kernel(cabi, shape, x_signed, cfg):
    say("weights through registers", shape, x_signed, cfg)
    M, N, K = shape
    c = _tile_case(M, N, K, seed=2500 + K, x_signed=x_signed, relu=N % 2 == 1, bias=M % 3 != 0,
                   per_channel=(M + N) % 2 == 0)
    y, acc, pw = _run(cabi, c, cfg)
    np.testing.assert_array_equal(acc, oracle.linear_acc32(c["xq"], c["wq"], nthreads=8))
    want = oracle.linear(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                         c["out_scale"], c["out_zp"], relu=c["relu"], nthreads=8)
    _check(y, want, "weights through registers")
    y1, acc1, _ = _run(cabi, c)          # the automatic choice, whichever kernel it is
    np.testing.assert_array_equal(y1, y)
    np.testing.assert_array_equal(acc1, acc)


# K beyond 4096 on one round of 64 x 64 tiles whose last row tile is nearly full: the automatic
# choice is the kernel that walks K through LDS as a ring of 256-byte phases (K that ends inside
# a phase and on an odd 16-byte chunk, ragged channels, both activation types)
@pytest.mark.parametrize("shape, x_signed", [((64, 4500, 8208), False), ((128, 1000, 5136), True),
                                             ((48, 4200, 4112), False), ((113, 130, 4112), True),
                                             ((64, 10300, 4096), False)])
def test_long_k_as_a_ring_of_phases(cabi, shape, x_signed):
    say("ring of phases", shape, x_signed)
    M, N, K = shape
    assert cabi.linear_kernel_choice(M, N, K)["kernel"] - 1 == 21
    c = _tile_case(M, N, K, seed=3300 + M, x_signed=x_signed, relu=N % 2 == 1, bias=M % 3 != 0,
                   per_channel=(M + N) % 2 == 0)
    y, acc, _ = _run(cabi, c)
    np.testing.assert_array_equal(acc, oracle.linear_acc32(c["xq"], c["wq"], nthreads=8))
    want = oracle.linear(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                         c["out_scale"], c["out_zp"], relu=c["relu"], nthreads=8)
    _check(y, want, "ring of phases")
    y2, acc2, _ = _run(cabi, c, 2)
    np.testing.assert_array_equal(y2, y)
    np.testing.assert_array_equal(acc2, acc)


# up to 64 rows against the very largest N: the automatic choice is the pipelined 64 x 128 tile over
# several rounds (rows mostly padding, ragged channels, K that ends inside a stage)
@pytest.mark.parametrize("shape, x_signed", [((9, 65600, 2064), False), ((40, 66000, 1040), True)])
def test_few_rows_against_the_largest_n(cabi, shape, x_signed):
    say("largest N", shape, x_signed)
    M, N, K = shape
    assert cabi.linear_kernel_choice(M, N, K)["kernel"] - 1 == 23
    c = _tile_case(M, N, K, seed=6500 + M, x_signed=x_signed, relu=M % 2 == 1, bias=True, per_channel=M % 2 == 0)
    y, acc, _ = _run(cabi, c)
    np.testing.assert_array_equal(acc, oracle.linear_acc32(c["xq"], c["wq"], nthreads=8))
    want = oracle.linear(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                         c["out_scale"], c["out_zp"], relu=c["relu"], nthreads=8)
    _check(y, want, "64 x 128 tiles over several rounds")


# up to 64 rows with the activations resident in LDS, one block per CU walking its channel groups:
# one group and several per block (ragged last round), K that ends inside a k-block / inside the
# padding to 16 k-blocks, every number of row groups, a single row, both activation types; the last
# two (and the third) as two blocks of eight waves per CU
@pytest.mark.parametrize("shape, x_signed", [((16, 4113, 1024), False), ((1, 100, 1040), True), ((13, 12300, 1024), False),
                                             ((32, 1000, 2048), True), ((64, 300, 1040), False), ((9, 5000, 8192), True),
                                             ((40, 530, 2048), False), ((12, 8200, 4112), True),
                                             ((7, 16400, 4096), True), ((16, 8200, 2048), False)])
def test_activations_resident_in_lds(cabi, shape, x_signed):
    say("resident activations", shape, x_signed)
    M, N, K = shape
    assert cabi.linear_kernel_choice(M, N, K, forced=29)["kernel"] == 29
    c = _tile_case(M, N, K, seed=2800 + M, x_signed=x_signed, relu=N % 2 == 1, bias=M % 3 != 0,
                   per_channel=(M + N) % 2 == 0)
    y, acc, pw = _run(cabi, c, 28)
    np.testing.assert_array_equal(acc, oracle.linear_acc32(c["xq"], c["wq"], nthreads=8))
    want = oracle.linear(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                         c["out_scale"], c["out_zp"], relu=c["relu"], nthreads=8)
    _check(y, want, "resident activations")
    # the float output against the streaming kernel's, and the automatic choice, whichever kernel it is
    ws = dev(c["w_scales"].astype(np.float32))
    b = None if c["bias"] is None else dev(c["bias"])
    f = {}
    for cfg in (28, 8):
        cabi.force_linear_config(cfg)
        try:
            f[cfg] = cabi.linear_f32(dev(c["xq"]), pw, c["x_scale"], c["x_zp"], ws, b, relu=c["relu"])
        finally:
            cabi.force_linear_config(-1)
    assert torch.equal(f[28], f[8])
    y1, acc1, _ = _run(cabi, c)
    np.testing.assert_array_equal(y1, y)
    np.testing.assert_array_equal(acc1, acc)


def test_small_batch_kernels_on_random_shapes(cabi):
    """The kernels that hold or stream all of K (64 x 64 and 32 x 32 tiles in LDS, 32-row tiles
    with weights through registers) against the pipelined 64 x 64 tiles on seeded random shapes
    around their tile and K boundaries: bytes, accumulators and float outputs equal, and the
    automatic choice with them."""
    import random
    rnd = random.Random(7)
    torch.manual_seed(7)
    for it in range(48):
        M = rnd.choice([1, 2, 17, 31, 32, 33, 63, 64, 65, 100, 129, 255, 300]) if it % 3 else rnd.randint(1, 300)
        N = rnd.choice([1, 15, 16, 17, 31, 32, 33, 63, 64, 65, 100, 257, 600]) if it % 2 else rnd.randint(1, 600)
        K = 16 * rnd.randint(1, 256)
        signed, pc, relu, bias = (bool(rnd.getrandbits(1)) for _ in range(4))
        say("random small-batch shape", it, (M, N, K), signed, pc, relu, bias)
        xq = (torch.randint(-128, 128, (M, K), device="cuda", dtype=torch.int8) if signed
              else torch.randint(0, 256, (M, K), device="cuda", dtype=torch.uint8))
        pw = cabi.PackedLinear(torch.randint(-127, 128, (N, K), device="cuda", dtype=torch.int8))
        ws = torch.rand(N if pc else 1, device="cuda") * 0.002 + 0.0005
        b = torch.randn(N, device="cuda") if bias else None
        zp = rnd.randint(-20, 20) if signed else rnd.randint(0, 255)
        ozp = rnd.randint(-128, 127) if signed else rnd.randint(0, 255)

        def run(cfg):
            cabi.force_linear_config(cfg)
            try:
                return (cabi.linear(xq, pw, 0.03, zp, ws, b, 0.7, ozp, relu=relu), cabi.linear_acc32(xq, pw),
                        cabi.linear_f32(xq, pw, 0.03, zp, ws, b, relu=relu))
            finally:
                cabi.force_linear_config(-1)

        want = run(2)
        fits28 = cabi.linear_kernel_choice(M, N, K, forced=29)["kernel"] == 29
        for cfg in [c for c in (21, 24, 25, 26, 27, 28, -1) if not (c == 24 and K > 1024) and not (c == 28 and not fits28)]:
            for got, ref, what in zip(run(cfg), want, ("bytes", "accumulators", "float output")):
                assert torch.equal(got, ref), f"cfg {cfg} {what} at {(M, N, K)}"


# the persistent kernel over more tiles than the chip has CUs: every block walks two tiles
# (ragged last row and column tiles, K that ends inside a stage and inside a pair of stages)
@pytest.mark.parametrize("shape,x_signed,relu,pc", [((4389, 4120, 448), False, False, True),
                                                     ((4100, 4352, 400), True, True, False),
                                                     ((8200, 2100, 656), False, True, True)])
def test_persistent_rounds(cabi, shape, x_signed, relu, pc):
    say("persistent rounds", shape, x_signed, relu, pc)
    M, N, K = shape
    assert -(-M // 256) * -(-N // 256) > 256
    c = _tile_case(M, N, K, seed=77 + K, x_signed=x_signed, relu=relu, per_channel=pc)
    pw = cabi.PackedLinear(dev(c["wq"]))
    ws, b = dev(c["w_scales"].astype(np.float32)), dev(c["bias"])
    want = oracle.linear(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                         c["out_scale"], c["out_zp"], relu=relu, nthreads=8)
    for cfg in (20, -1, 6):   # pinned, the automatic choice (the same kernel), and one tile per block
        cabi.force_linear_config(cfg)
        try:
            y = host(cabi.linear(dev(c["xq"]), pw, c["x_scale"], c["x_zp"], ws, b, c["out_scale"], c["out_zp"],
                                 out_signed=x_signed, relu=relu))
        finally:
            cabi.force_linear_config(-1)
        _check(y, want, f"cfg {cfg}")
    # the same tiles with float output (the product inside a dynamically quantized linear)
    wantf = oracle.linear_f32(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"], relu=relu,
                              nthreads=8)
    for cfg in (20, -1):
        cabi.force_linear_config(cfg)
        try:
            yf = host(cabi.linear_f32(dev(c["xq"]), pw, c["x_scale"], c["x_zp"], ws, b, relu=relu))
        finally:
            cabi.force_linear_config(-1)
        np.testing.assert_array_equal(yf, wantf, err_msg=f"float output, cfg {cfg}")


# wave groups that split the k loop inside a block (stage counts the group count divides)
@pytest.mark.parametrize("cfg", [14])
@pytest.mark.parametrize("shape", [(300, 520, 512), (257, 33, 256), (64, 1040, 1024), (130, 260, 1008), (100, 70, 4096), (65, 48, 128)])
def test_k_split_wave_groups(cabi, cfg, shape):
    say("k-split groups cfg", cfg, shape)
    c = _tile_case(*shape, seed=cfg * 7 + shape[0], relu=bool(shape[0] & 1))
    y, acc, pw = _run(cabi, c, cfg)
    np.testing.assert_array_equal(acc, oracle.linear_acc32(c["xq"], c["wq"], nthreads=8))
    want = oracle.linear(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                         c["out_scale"], c["out_zp"], relu=c["relu"], nthreads=8)
    _check(y, want, f"cfg {cfg}")
    cabi.force_linear_config(cfg)
    try:
        yf = host(cabi.linear_f32(dev(c["xq"]), pw, c["x_scale"], c["x_zp"], dev(c["w_scales"].astype(np.float32)),
                                  dev(c["bias"]), relu=c["relu"]))
    finally:
        cabi.force_linear_config(-1)
    np.testing.assert_array_equal(
        yf, oracle.linear_f32(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"], relu=c["relu"],
                              nthreads=8))


@pytest.mark.parametrize("x_signed,relu,bias,pc", [(True, False, True, True), (True, True, False, False),
                                                   (False, True, True, False), (False, False, False, True)])
def test_dtype_and_epilogue_variants(cabi, x_signed, relu, bias, pc):
    say("variants", x_signed, relu, bias, pc)
    c = _tile_case(150, 200, 256, seed=99, x_signed=x_signed, relu=relu, bias=bias, per_channel=pc)
    y, acc, _ = _run(cabi, c)
    np.testing.assert_array_equal(acc, oracle.linear_acc32(c["xq"], c["wq"]))
    want = oracle.linear(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                         c["out_scale"], c["out_zp"], relu=c["relu"])
    assert want.dtype == (np.int8 if x_signed else np.uint8) and y.dtype == want.dtype
    _check(y, want, "variant")


@pytest.mark.parametrize("m", [1, 4, 16])
def test_decode_shapes(cabi, m):
    """benchmark configuration 4: M in {1,4,16}, K = N = 4096."""
    say("decode", m)
    c = _tile_case(m, 4096, 4096, seed=40 + m)
    y, acc, _ = _run(cabi, c)
    np.testing.assert_array_equal(acc, oracle.linear_acc32(c["xq"], c["wq"], nthreads=8))
    want = oracle.linear(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                         c["out_scale"], c["out_zp"], nthreads=8)
    _check(y, want, "decode")


@pytest.mark.parametrize("m,n,k", [(3, 50, 100), (16, 16, 64), (9, 130, 4096 + 64), (16, 17, 16),
                                   (17, 48, 256), (32, 4096, 4096), (33, 130, 1024 + 16), (48, 64, 512),
                                   (64, 1000, 2048)])
def test_decode_ragged(cabi, m, n, k):
    say("decode ragged", m, n, k)
    c = _tile_case(m, n, k, seed=m * n)
    y, acc, _ = _run(cabi, c)
    np.testing.assert_array_equal(acc, oracle.linear_acc32(c["xq"], c["wq"]))
    want = oracle.linear(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                         c["out_scale"], c["out_zp"])
    _check(y, want, "decode ragged")


def test_row_strided_and_unaligned_activations(cabi):
    say("strided x")
    c = _tile_case(70, 90, 128, seed=5)
    big = np.zeros((70, 160), dtype=np.uint8)
    big[:, :128] = c["xq"]
    pw = cabi.PackedLinear(dev(c["wq"]))
    ws, b = dev(c["w_scales"].astype(np.float32)), dev(c["bias"])
    want = oracle.linear(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                         c["out_scale"], c["out_zp"])
    xb = dev(big)
    y = cabi.linear(xb[:, :128], pw, c["x_scale"], c["x_zp"], ws, b, c["out_scale"], c["out_zp"])
    _check(host(y), want, "ldx=160")
    big2 = np.zeros((70, 131), dtype=np.uint8)      # rows not 16-byte aligned -> plain kernel
    big2[:, 3:] = c["xq"]
    y = cabi.linear(dev(big2)[:, 3:], pw, c["x_scale"], c["x_zp"], ws, b, c["out_scale"], c["out_zp"])
    _check(host(y), want, "unaligned rows")


def test_decode_row_pitch_and_exact_buffers(cabi):
    """The weight-streaming kernel with a row pitch larger than K, and with activation
    buffers that end exactly at the last row's last byte (its clamped loads must stay
    inside: every load of a missing k-block reads the row's first bytes)."""
    say("decode strided x")
    for m, n, k, pitch in ((5, 48, 128, 160), (1, 16, 16, 16), (16, 130, 4096 + 64, 4096 + 64), (3, 33, 80, 96)):
        c = _tile_case(m, n, k, seed=900 + m + k)
        pw = cabi.PackedLinear(dev(c["wq"]))
        ws, b = dev(c["w_scales"].astype(np.float32)), dev(c["bias"])
        want = oracle.linear(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                             c["out_scale"], c["out_zp"])
        flat = np.zeros(m * pitch - (pitch - k), dtype=np.uint8)   # ends with the last row's last byte
        for r in range(m):
            flat[r * pitch:r * pitch + k] = c["xq"][r]
        xb = torch.as_strided(dev(flat), (m, k), (pitch, 1))
        y = cabi.linear(xb, pw, c["x_scale"], c["x_zp"], ws, b, c["out_scale"], c["out_zp"])
        _check(host(y), want, f"decode m={m} k={k} pitch={pitch}")


def test_empty_batch(cabi):
    c = _tile_case(4, 32, 64, seed=1)
    pw = cabi.PackedLinear(dev(c["wq"]))
    x = torch.empty((0, 64), dtype=torch.uint8, device="cuda")
    y = cabi.linear(x, pw, 0.1, 0, dev(c["w_scales"].astype(np.float32)), None, 0.1, 0)
    assert tuple(y.shape) == (0, 32)


def test_c1_golden(cabi, golden):
    """benchmark configuration 1 end to end on the device: dynamic quantize of x,
    per-channel quantize of W, prepack, linear."""
    say("C1")
    c1 = cases.c1_case()
    x = dev(c1["x"].reshape(-1))
    qp = cabi.choose_qparams_dev(cabi.minmax(x), False, False)
    s, z = cabi.read_qparams(qp)
    assert s == float(golden["c1/x_scale"]) and z == int(golden["c1/x_zp"])
    xq = cabi.quantize_per_tensor_dev(x, qp, False).reshape(128, 1024)
    assert cases.crc(host(xq)) == int(golden["c1/xq_crc"])
    wq = cabi.quantize_per_channel(dev(c1["w"]), dev(c1["w_scales"]),
                                   torch.zeros(1024, dtype=torch.int64, device="cuda"), 0, True)
    assert cases.crc(host(wq)) == int(golden["c1/wq_crc"])
    pw = cabi.PackedLinear(wq)
    y = cabi.linear(xq, pw, s, z, dev(c1["w_scales"].astype(np.float32)), dev(c1["bias"]),
                    c1["out_scale"], c1["out_zp"])
    acc = cabi.linear_acc32(xq, pw)
    np.testing.assert_array_equal(host(acc), oracle.linear_acc32(host(xq), host(wq), nthreads=8))
    _check(host(y), golden["c1/y"], "C1 vs golden")
    dq = cabi.dequantize_per_tensor(y, c1["out_scale"], c1["out_zp"])
    assert cases.crc(host(dq)) == int(golden["c1/y_dq_crc"])


def test_c3_full_size(cabi):
    """benchmark configuration 3 (M=4096, K=4096, N=11008): oracle parity on sampled
    rows, integer identities on the whole output, and every output byte against the live CPU operator."""
    M, K, N = 4096, 4096, 11008
    say("C3 full size")
    rng = np.random.default_rng(3)
    x = rng.standard_normal((M, K), dtype=np.float32)
    w = rng.standard_normal((N, K), dtype=np.float32) * np.float32(0.02)
    mn, mx = oracle.minmax(x, nthreads=8)
    s, z = oracle.choose_qparams(mn, mx)
    xq = cabi.quantize_per_tensor(dev(x.reshape(-1)), s, z, False).reshape(M, K)
    ws = (np.abs(w).max(axis=1) / np.float32(127.0)).astype(np.float64)
    wq = cabi.quantize_per_channel(dev(w), dev(ws), torch.zeros(N, dtype=torch.int64, device="cuda"), 0, True)
    bias = rng.standard_normal(N, dtype=np.float32)
    pw = cabi.PackedLinear(wq)
    out_scale, out_zp = 0.02, 128
    y = cabi.linear(xq, pw, s, z, dev(ws.astype(np.float32)), dev(bias), out_scale, out_zp)
    acc = cabi.linear_acc32(xq, pw)
    rows = np.array([0, 1, 255, 256, 1023, 2048, 4000, 4095])
    xq_h, wq_h = host(xq[torch.from_numpy(rows).cuda()]), host(wq)
    np.testing.assert_array_equal(host(acc[torch.from_numpy(rows).cuda()]),
                                  oracle.linear_acc32(xq_h, wq_h, nthreads=8))
    want = oracle.linear(xq_h, s, z, wq_h, ws, bias, out_scale, out_zp, nthreads=8)
    got = host(y[torch.from_numpy(rows).cuda()])
    assert 0.2 < np.mean((got > 0) & (got < 255)), "output saturated: test would prove nothing"
    _check(got, want, "C3 rows")
    # every tile of the output: activations of all ones reproduce the column sums
    ones = torch.ones((M, K), dtype=torch.uint8, device="cuda")
    acc1 = cabi.linear_acc32(ones, pw)
    assert torch.equal(acc1, pw.colsum[None, :].expand(M, N))
    # the GEMM is linear in x: acc(x) + acc(255 - x) = 255 * colsum
    acc2 = cabi.linear_acc32(255 - xq, pw)
    assert torch.equal(acc + acc2, 255 * pw.colsum[None, :].expand(M, N))
    del acc, acc1, acc2, ones
    # all 45 M requantised bytes against the live CPU operator on the same codes (the way the
    # reference's harness compares device and CPU results, torch_musa/testing/base_test_tool.py:814-825)
    torch.backends.quantized.engine = "fbgemm"
    x_cpu = torch._make_per_tensor_quantized_tensor(xq.cpu(), s, z)
    w_cpu = torch._make_per_channel_quantized_tensor(wq.cpu(), torch.from_numpy(ws), torch.zeros(N, dtype=torch.int64), 0)
    p_cpu = torch.ops.quantized.linear_prepack(w_cpu, torch.from_numpy(bias))
    y_cpu = torch.ops.quantized.linear(x_cpu, p_cpu, out_scale, out_zp).int_repr()
    y_gpu = y.cpu()
    differ = int((y_cpu != y_gpu).sum())
    assert differ == 0, f"{differ} of {M * N} bytes differ from the CPU operator's (max " \
                        f"{int((y_cpu.int() - y_gpu.int()).abs().max())} LSB)"


# ---- split K (a few hundred rows, long K: partial sums in a caller-owned workspace) --------
@pytest.mark.parametrize("shape,x_signed,relu,bias,pc", [
    ((100, 520, 8208), False, False, True, True),     # 8 splits, K ends inside a stage, ragged M and N
    ((300, 300, 8192), True, True, False, False),     # qint8 activations, per-tensor weight scale
    ((130, 4096, 11008), False, True, True, True),    # 64 tiles, 4 splits of 43 stages
    ((128, 1024, 16640), False, False, True, True),   # 260 stages as 14 x 17 + 22: the tail joins the last split
    ((128, 128, 13328), True, False, True, False),    # 209 stages as 11 x 17 + 22, K ends inside a stage
])
def test_split_k(cabi, shape, x_signed, relu, bias, pc):
    say("split K", shape, x_signed, relu, bias, pc)
    M, N, K = shape
    assert cabi.lib().tmq_linear_workspace_bytes(M, N, K) > 0, "this shape is meant to take the split schedule"
    c = _tile_case(M, N, K, seed=4242 + M, x_signed=x_signed, relu=relu, bias=bias, per_channel=pc)
    y, acc, pw = _run(cabi, c, 13)      # 13: split schedule or an error
    np.testing.assert_array_equal(acc, oracle.linear_acc32(c["xq"], c["wq"], nthreads=8))
    want = oracle.linear(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                         c["out_scale"], c["out_zp"], relu=c["relu"], nthreads=8)
    _check(y, want, "split K")
    ws = dev(c["w_scales"].astype(np.float32))
    b = None if c["bias"] is None else dev(c["bias"])
    yf = host(cabi.linear_f32(dev(c["xq"]), pw, c["x_scale"], c["x_zp"], ws, b, relu=relu))
    np.testing.assert_array_equal(
        yf, oracle.linear_f32(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"], relu=relu,
                              nthreads=8))
    # without a workspace the single-launch kernels give the same bytes
    cabi.use_linear_workspace = False
    try:
        y1, acc1, _ = _run(cabi, c)
        yf1 = host(cabi.linear_f32(dev(c["xq"]), pw, c["x_scale"], c["x_zp"], ws, b, relu=relu))
    finally:
        cabi.use_linear_workspace = True
    np.testing.assert_array_equal(y1, y)
    np.testing.assert_array_equal(acc1, acc)
    np.testing.assert_array_equal(yf1, yf)


@pytest.mark.parametrize("shape,path", [((24, 4096, 4096), "stream"), ((40, 11008, 4096), "tiles"),
                                        ((48, 1024, 1024), "tiles"), ((64, 4096, 11008), "split"),
                                        ((33, 2048, 8192), "stream"), ((17, 520, 80), "tiles")])
def test_rows_17_to_64_automatic_choice(cabi, shape, path):
    """Between 17 and 64 rows the library picks the weight-streaming kernel, 64 x 64 tiles
    or split K from a time estimate; every choice gives the oracle's bytes, and forcing
    the streaming kernel gives them too.  (Which kernel ran is visible through the
    workspace the shape asks for: only the split schedule wants one.)"""
    say("17-64 rows", shape, path)
    M, N, K = shape
    assert (cabi.lib().tmq_linear_workspace_bytes(M, N, K) > 0) == (path == "split")
    c = _tile_case(M, N, K, seed=99 + M, x_signed=M % 2 == 0, relu=M % 3 == 0, bias=True, per_channel=True)
    want = oracle.linear(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                         c["out_scale"], c["out_zp"], relu=c["relu"], nthreads=8)
    want_acc = oracle.linear_acc32(c["xq"], c["wq"], nthreads=8)
    for cfg in (-1, 8):
        y, acc, _ = _run(cabi, c, cfg)
        _check(y, want, f"cfg {cfg}")
        np.testing.assert_array_equal(acc, want_acc)
    cabi.use_linear_workspace = False
    try:
        y, acc, _ = _run(cabi, c)
    finally:
        cabi.use_linear_workspace = True
    _check(y, want, "no workspace")
    np.testing.assert_array_equal(acc, want_acc)


def test_split_k_workspace_rules(cabi):
    """No workspace for the weight-streaming rows and for grids that fill the chip; a
    workspace that is too small is ignored, not overrun."""
    wsb = cabi.lib().tmq_linear_workspace_bytes
    assert wsb(16, 4096, 4096) == 0 and wsb(64, 4096, 4096) == 0
    assert wsb(4096, 11008, 4096) == 0 and wsb(2048, 4096, 4096) == 0
    assert wsb(128, 4096, 4096) == 0                     # K too short for the cut to pay
    assert wsb(128, 4096, 11008) == 8 * 128 * 4096 * 4   # 32 tiles of 128 x 128, 8 splits
    assert wsb(512, 4096, 11008) == 2 * 512 * 4096 * 4   # 128 tiles, 2 splits
    assert wsb(128, 4098, 8192) == 7 * 128 * 4100 * 4    # 33 tiles, 7 splits; partial rows padded to 16 bytes
    assert wsb(0, 10, 10) == 0 and wsb(-1, 10, 10) == 0
    c = _tile_case(100, 520, 8208, seed=5)
    pw = cabi.PackedLinear(dev(c["wq"]))
    xq, ws, b = dev(c["xq"]), dev(c["w_scales"].astype(np.float32)), dev(c["bias"])
    y = torch.empty((100, 520), dtype=torch.uint8, device="cuda")
    d = cabi._linear_desc(xq, pw, c["x_scale"], c["x_zp"], ws, b, c["out_scale"], c["out_zp"], False, False, y)
    assert d.workspace_bytes > 1024
    guard = torch.full((4096,), 0x5A, dtype=torch.uint8, device="cuda")
    d.workspace, d.workspace_bytes = guard.data_ptr(), 1024    # far too small
    cabi.check(cabi.lib().tmq_linear(C.byref(d), cabi.stream_ptr()), "tmq_linear")
    want = oracle.linear(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                         c["out_scale"], c["out_zp"])
    _check(host(y), want, "small workspace")
    assert bool((guard == 0x5A).all())


# ---- float output (the second half of a dynamically quantized linear) --------------
# Float results are compared bit for bit: the kernel's epilogue is the oracle's
# single fused multiply-add, and the dynamic quantization in front of it is
# bit-exact by the quantizer tests.
@pytest.mark.parametrize("cfg", [0, 1, 2, 3, 6, 7, 8, 9, 17, 19, 20, 21, 22, 23, 24, 25, 26])
@pytest.mark.parametrize("shape,relu,bias,pc,x_signed", [((60, 264, 448), False, True, True, False),
                                                         ((257, 33, 144), True, True, False, False),
                                                         ((16, 1040, 1168), False, False, True, True)])
def test_linear_f32_configs(cabi, cfg, shape, relu, bias, pc, x_signed):
    say("linear_f32 cfg", cfg, shape, relu, bias, pc, x_signed)
    c = _tile_case(*shape, seed=300 + cfg, x_signed=x_signed, relu=relu, bias=bias, per_channel=pc)
    if cfg == 8 and shape[0] > 64:
        pytest.skip("the weight-streaming kernel takes at most 64 rows")
    if cfg == 24 and shape[2] > 1024:
        pytest.skip("the 32 x 32 tiles whose waves split K take K <= 1024")
    pw = cabi.PackedLinear(dev(c["wq"]))
    ws = dev(c["w_scales"].astype(np.float32))
    b = None if c["bias"] is None else dev(c["bias"])
    cabi.force_linear_config(cfg)
    try:
        y = host(cabi.linear_f32(dev(c["xq"]), pw, c["x_scale"], c["x_zp"], ws, b, relu=relu))
    finally:
        cabi.force_linear_config(-1)
    want = oracle.linear_f32(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"], relu=relu)
    np.testing.assert_array_equal(y, want)


@pytest.mark.parametrize("c", cases.linear_dynamic_cases(), ids=lambda c: c["name"])
def test_linear_dynamic_cases(cabi, golden, c):
    say("linear_dynamic", c["name"])
    pw = cabi.PackedLinear(dev(c["wq"]))
    ws = dev(c["w_scales"].astype(np.float32))
    b = None if c["bias"] is None else dev(c["bias"])
    y = host(cabi.linear_dynamic(dev(c["x"]), pw, ws, b, relu=c["relu"], reduce_range=c["reduce_range"]))
    np.testing.assert_array_equal(y, golden["lindyn/" + c["name"] + "/y"])
    np.testing.assert_array_equal(y, oracle.linear_dynamic(c["x"], c["wq"], c["w_scales"], c["bias"], c["relu"],
                                                           c["reduce_range"]))


@pytest.mark.parametrize("shape,relu,bias,pc,rr", [((1, 4096, 4096), False, True, True, False),
                                                   ((4, 4096, 1000), True, True, False, False),
                                                   ((16, 1024, 300), False, False, True, True),
                                                   ((3, 48, 17), False, True, True, False),
                                                   ((1, 16384, 64), True, True, True, False),
                                                   ((5, 1040, 130), False, True, False, True),
                                                   ((8, 4096, 1000), False, True, True, False),
                                                   ((4, 8192, 130), True, False, False, True),
                                                   ((11, 2064, 9000), False, True, True, False)])
def test_linear_dynamic_one_launch(cabi, shape, relu, bias, pc, rr):
    # a handful of rows: range, parameters, codes and product inside the weight-streaming
    # kernel or the kernel that keeps the rows in LDS (each pinned where it takes the shape,
    # and the library's choice); bit for bit the oracle and the two-launch path
    say("linear_dynamic one launch", shape, relu, bias, pc, rr)
    M, K, N = shape
    rng = np.random.default_rng(M * 7 + K)
    x = (rng.standard_normal((M, K)) * 1.7 + 0.3).astype(np.float32)
    wq = rng.integers(-127, 128, (N, K), dtype=np.int8)
    wsc = ((0.0005 + 0.001 * rng.random(N)) if pc else np.array([0.00093])).astype(np.float32).astype(np.float64)
    b = rng.standard_normal(N).astype(np.float32) if bias else None
    pw = cabi.PackedLinear(dev(wq))
    args = (dev(x), pw, dev(wsc.astype(np.float32)), None if b is None else dev(b))
    assert cabi.fused_small_dynamic
    y = host(cabi.linear_dynamic(*args, relu=relu, reduce_range=rr))
    np.testing.assert_array_equal(y, oracle.linear_dynamic(x, wq, wsc, b, relu=relu, reduce_range=rr))
    for pin in ([9] if M * K <= 16384 else []) + ([29] if 64 <= K <= 8192 and M * K <= 32768 else []):
        cabi.dynamic_small_kernel = pin
        try:
            yp = host(cabi.linear_dynamic(*args, relu=relu, reduce_range=rr))
        finally:
            cabi.dynamic_small_kernel = 0
        np.testing.assert_array_equal(yp, y)
    cabi.fused_small_dynamic = False
    try:
        y2 = host(cabi.linear_dynamic(*args, relu=relu, reduce_range=rr))
    finally:
        cabi.fused_small_dynamic = True
    np.testing.assert_array_equal(y2, y)


def test_linear_dynamic_prefill_sized(cabi):
    # [2048, 1024] x [4096, 1024]^T through the large-tile kernel, against the oracle
    say("linear_dynamic prefill")
    rng = np.random.default_rng(8)
    x = rng.standard_normal((2048, 1024)).astype(np.float32)
    wq = rng.integers(-127, 128, (4096, 1024), dtype=np.int8)
    wsc = (0.0005 + 0.001 * rng.random(4096)).astype(np.float32).astype(np.float64)
    bias = rng.standard_normal(4096).astype(np.float32)
    pw = cabi.PackedLinear(dev(wq))
    y = host(cabi.linear_dynamic(dev(x), pw, dev(wsc.astype(np.float32)), dev(bias)))
    mn, mx = oracle.minmax(x)
    scale, zp = oracle.choose_qparams(mn, mx, False, False)
    xq = oracle.quantize_per_tensor_fused(x, scale, zp, False, nthreads=8)
    want = oracle.linear_f32(xq, scale, zp, wq, wsc, bias, nthreads=8)
    np.testing.assert_array_equal(y, want)


@pytest.mark.parametrize("cfg,shape", [(-1, (130, 260, 448)), (0, (130, 260, 448)), (2, (300, 520, 448)), (7, (300, 520, 448)),
                                       (9, (40, 70, 784)), (17, (270, 300, 400)), (20, (1300, 1100, 704)), (21, (64, 1040, 1168)),
                                       (24, (40, 70, 784)), (25, (64, 1040, 1168)), (26, (64, 1040, 1168)), (27, (130, 260, 1168)),
                                       (8, (3, 300, 448)), (28, (16, 300, 448)), (-1, (1, 4096, 256)), (-1, (256, 300, 4608))])
@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("per_channel", [False, True])
def test_unsigned_output_with_zero_point_0(cabi, cfg, shape, relu, per_channel):
    """quint8 output with zero point 0 (what follows a ReLU): the packing conversion alone rounds and
    saturates in the kernels; half of the sums are negative and must come out as 0, ties go to even."""
    say("zero point 0", cfg, shape, relu, per_channel)
    c = _tile_case(*shape, seed=cfg * 7 + shape[1], relu=relu, per_channel=per_channel)
    c["out_zp"] = 0
    c["out_scale"] /= 3     # (255 at two standard deviations of the sums: the upper bound is met too)
    y, _, _ = _run(cabi, c, cfg)
    want = oracle.linear(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                         c["out_scale"], 0, relu=relu)
    assert 0.3 < np.mean(want == 0) < 0.7 and np.any(want == 255)
    _check(y, want, f"cfg {cfg}")


def _random_shapes(seed, count):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        m = int(rng.choice([1, 3, 17, 64, 65, 130, 255, 256, 257, 300, 513, 700]))
        n = int(rng.choice([1, 5, 16, 31, 48, 100, 255, 256, 257, 300, 520, 777]))
        k = int(rng.choice([16, 48, 64, 128, 144, 192, 208, 256, 320, 448, 1040]))
        out.append((m, n, k))
    return out


@pytest.mark.parametrize("cfg", [-1, 6, 7, 17, 19])
def test_random_shapes_against_oracle(cabi, cfg):
    # ragged everything: rows, channels and k tails in all combinations, for the automatic
    # choice and for the two direct-copy tiles (which fall back below three k stages)
    for i, (m, n, k) in enumerate(_random_shapes(1234 + cfg, 24)):
        say("random shape", cfg, m, n, k)
        c = _tile_case(m, n, k, seed=7000 + 31 * i + cfg, x_signed=bool(i & 1), relu=bool(i & 2), bias=bool(i & 4),
                       per_channel=not (i & 8))
        y, acc, _ = _run(cabi, c, cfg)
        np.testing.assert_array_equal(acc, oracle.linear_acc32(c["xq"], c["wq"]), err_msg=f"{(m, n, k)}")
        want = oracle.linear(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                             c["out_scale"], c["out_zp"], relu=c["relu"])
        _check(y, want, f"cfg {cfg} shape {(m, n, k)}")


def test_row_pitch_and_output_pitch(cabi):
    # activations and outputs that are column slices of wider buffers (ldx > K, ldy > N)
    say("pitches")
    c = _tile_case(300, 264, 448, seed=77)   # seven k stages: the direct-copy kernels take it
    pw = cabi.PackedLinear(dev(c["wq"]))
    xbig = torch.zeros((300, 448 + 64), dtype=torch.uint8, device="cuda")
    xbig[:, 16:464] = dev(c["xq"])
    ybig = torch.full((300, 264 + 40), 7, dtype=torch.uint8, device="cuda")
    want = oracle.linear(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                         c["out_scale"], c["out_zp"])
    # (output slices that start on a 4-byte boundary and off it: word and byte stores)
    for cfg, y0 in [(f, 8) for f in (-1, 6, 7, 3, 17, 19, 21, 24, 25, 26)] + [(f, 6) for f in (-1, 2, 21, 24, 25, 26)]:
        cabi.force_linear_config(cfg)
        try:
            cabi.linear(xbig[:, 16:464], pw, c["x_scale"], c["x_zp"], dev(c["w_scales"].astype(np.float32)),
                        dev(c["bias"]), c["out_scale"], c["out_zp"], out=ybig[:, y0:y0 + 264])
        finally:
            cabi.force_linear_config(-1)
        got = host(ybig)
        _check(got[:, y0:y0 + 264], want, f"cfg {cfg} at column {y0}")
        assert (got[:, :y0] == 7).all() and (got[:, y0 + 264:] == 7).all()   # nothing written outside the slice
        ybig.fill_(7)


def test_row_pitch_beyond_the_direct_copy_range(cabi):
    # activation rows 8 MiB + 64 B apart: past the 32-bit lane offsets of the direct-copy
    # kernels, the register-staged kernels take over; same bytes
    say("huge pitch")
    c = _tile_case(300, 264, 448, seed=78)
    pitch = (1 << 23) + 64
    pw = cabi.PackedLinear(dev(c["wq"]))
    xbig = torch.zeros(300 * pitch, dtype=torch.uint8, device="cuda")
    xv = xbig.as_strided((300, 448), (pitch, 1))
    xv.copy_(dev(c["xq"]))
    want = oracle.linear(c["xq"], c["x_scale"], c["x_zp"], c["wq"], c["w_scales"], c["bias"],
                         c["out_scale"], c["out_zp"])
    for cfg in (-1, 6, 7, 17):
        cabi.force_linear_config(cfg)
        try:
            y = cabi.linear(xv, pw, c["x_scale"], c["x_zp"], dev(c["w_scales"].astype(np.float32)), dev(c["bias"]),
                            c["out_scale"], c["out_zp"])
        finally:
            cabi.force_linear_config(-1)
        _check(host(y), want, f"cfg {cfg}")
    del xbig
