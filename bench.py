"""Benchmark of the quantized-inference operator path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one quantized::linear at benchmark configuration 3 (x quint8 [4096,4096] from
N(0,1), W qint8 per-channel [11008,4096] from N(0,0.02), fp32 bias, quint8
output), issued through torch.ops.quantized.linear on tensors that are already
resident in HBM.  The last line of stdout is one JSON object:

  value / unit     whole-job int8 throughput of those K steps (TOP/s)
  roofline         the GEMM kernel against the dense int8 MFMA peak, its average
                   launch duration measured with HIP events on the launch stream
  cpu_baseline     PyTorch's quantized CPU op (fbgemm) on this host's cores at
                   the same configuration, with a one-thread figure, the CPU
                   model, the scalar C oracle port and the other configurations
  secondary        the other benchmark configurations: quantize / dequantize / min-max
                   over 2**28 fp32 (HBM bound), decode-shaped linear (weight
                   read bound), conv2d NHWC

Everything here is synthetic data of the benchmark shapes and distributions
("N(0,s)" read as standard deviation s).
"""
from __future__ import annotations

import argparse
import collections
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# Published MI355X peaks used for roofline.frac
PEAK_INT8_TOPS = 5000.0   # dense int8 MFMA, 5.0 POP/s
PEAK_HBM_GBS = 8000.0     # HBM3E, 8 TB/s

# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE (KiB per
# dispatch, one run each: `rocprofv3 --pmc FETCH_SIZE -- python3 bench.py --only linear --steps 6`).
# Calibration against a plain 1 GiB device copy (`--only copy`): FETCH_SIZE reads 524 300 for
# 1 048 576 KiB actually read (factor 2.0), WRITE_SIZE reads 1 048 576 (factor 1.0).
# Summaries: profiles/hbm_traffic_pmc.md.
def _traffic(fetch_kib, write_kib):
    return int((fetch_kib * 2.0 + write_kib) * 1024)


MEASURED_TRAFFIC = {
    "linear_c3": _traffic(161_134, 44_033),       # 375 MB: operands re-fetched 5.3x by the 8 L2s
    "quantize_c2": _traffic(524_304, 262_144),    # 1.342 GB = algorithmic
    "dequantize_c2": _traffic(131_084, 1_048_819),
    "minmax_c2": _traffic(524_316, 64),
    "quantize_pc": _traffic(89_478, 44_032),
    "dequantize_pc": _traffic(23_423, 176_136),
    "decode_m1": _traffic(8_300, 8),              # 17.0 MB for 16.8 MB algorithmic
    "rows64": _traffic(9_347, 256),               # 19.4 MB for 17.4 MB (two row tiles fetch each weight)
    "c1": _traffic(1_076, 128),
    "conv_c5": _traffic(3_940, 6_272),            # 14.5 MB for 12.9 MB algorithmic (halo overlap)
    "conv_add_relu_c5": _traffic(7_066, 6_272),
}


PROBE_MODES = ((0, "zero_operands"), (1, "uniform_random_int8"), (2, "gaussian_int8"),
               (3, "gaussian_int8_fresh_from_lds"), (4, "gaussian_int8_one_operand_non_negative"),
               (5, "gaussian_int8_16x16x64"))

# Socket power and shader clock while a load runs: a child process, started before this
# process touches the GPU and never touching the GPU runtime itself, waits on its stdin for
# "S <seconds>", then reads the amdgpu hwmon files of card 0 every ~2 ms for that long, asks
# amd-smi for the per-XCD shader clocks once in the middle, and answers with one JSON line.
# Everything is optional: a box that hides the files gives {"available": false, ...}.
_SAMPLER = r"""
import glob, json, subprocess, sys, time
def rd(p):
    with open(p) as f:
        return int(f.read().strip())
def sample(seconds):
    out = {"available": False}
    try:
        hw = sorted(glob.glob("/sys/class/drm/card[0-9]*/device/hwmon/hwmon*"))
        hw = [h for h in hw if glob.glob(h + "/power1_input") or glob.glob(h + "/power1_average")]
        h = hw[0]
        pfile = (glob.glob(h + "/power1_input") + glob.glob(h + "/power1_average"))[0]
        try:
            out["power_cap_w"] = rd(h + "/power1_cap") / 1e6
        except Exception:
            out["power_cap_w"] = None
        watts, clocks, t0, asked = [], [], time.time(), False
        while time.time() - t0 < seconds:
            watts.append(rd(pfile) / 1e6)
            if not asked and time.time() - t0 > seconds * 0.4:
                asked = True
                try:
                    r = subprocess.run(["amd-smi", "metric", "--clock", "--json"], stdout=subprocess.PIPE,
                                       stderr=subprocess.DEVNULL, text=True, timeout=10)
                    g = json.loads(r.stdout)
                    g = g["gpu_data"][0] if isinstance(g, dict) else g[0]
                    clocks = [v["clk"]["value"] for k, v in g["clock"].items()
                              if k.startswith("gfx_") and isinstance(v.get("clk"), dict)
                              and isinstance(v["clk"].get("value"), (int, float))]
                except Exception as e:
                    out["clock_error"] = str(e)[:120]
            time.sleep(0.002)
        watts.sort()
        out.update(available=True, samples=len(watts), socket_power_w_avg=round(sum(watts) / len(watts), 1),
                   socket_power_w_median=watts[len(watts) // 2], socket_power_w_max=watts[-1],
                   source=pfile, xcd_shader_clocks_mhz=clocks,
                   shader_clock_mhz_avg=round(sum(clocks) / len(clocks), 1) if clocks else None)
    except Exception as e:
        out["error"] = (type(e).__name__ + ": " + str(e))[:200]
    return out
for line in sys.stdin:
    parts = line.split()
    if not parts or parts[0] != "S":
        break
    print(json.dumps(sample(float(parts[1]))), flush=True)
"""
_sampler_proc = None


def start_power_sampler():
    """Call before the first GPU call of this process."""
    global _sampler_proc
    import subprocess
    try:
        _sampler_proc = subprocess.Popen([sys.executable, "-c", _SAMPLER], stdin=subprocess.PIPE,
                                         stdout=subprocess.PIPE, stderr=subprocess.DEVNULL, text=True)
    except OSError:
        _sampler_proc = None


def stop_power_sampler():
    global _sampler_proc
    if _sampler_proc is not None:
        try:
            _sampler_proc.stdin.close()
            _sampler_proc.wait(timeout=5)
        except Exception:  # noqa: BLE001
            _sampler_proc.kill()
        _sampler_proc = None


def sample_power_while(load, seconds=0.6):
    """Runs load() again and again for `seconds` while the sampler reads the socket power."""
    if _sampler_proc is None or _sampler_proc.poll() is not None:
        return {"available": False, "error": "sampler process not running"}
    try:
        _sampler_proc.stdin.write(f"S {seconds}\n")
        _sampler_proc.stdin.flush()
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < seconds + 0.02:
            load()
        return json.loads(_sampler_proc.stdout.readline())
    except Exception as e:  # noqa: BLE001
        return {"available": False, "error": (type(e).__name__ + ": " + str(e))[:200]}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--skip-secondary", action="store_true")
    ap.add_argument("--skip-cpu", action="store_true")
    ap.add_argument("--no-power", action="store_true",
                    help="do not start the child process that samples the socket power (for runs under a profiler, "
                         "whose library has initialised the GPU before this program starts)")
    ap.add_argument("--only", choices=["linear", "quantize", "dequantize", "minmax", "copy", "quantize_pc",
                                       "dequantize_pc", "decode", "rows64", "rows256", "c1", "decode16_proj", "conv", "conv_add_relu", "conv_first_layer", "conv_depthwise", "conv_depthwise7",
                                       "probe", "choice"],
                    help="run just this kernel --steps times (for rocprofv3 --kernel-trace / --pmc runs, so that "
                         "every launch of the kernel in the trace has the benchmark size); 'copy' is a plain "
                         "1 GiB device copy used to calibrate the FETCH_SIZE / WRITE_SIZE counters")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: the quantized operator path is single-device "
              "(no collectives); run it with --gpus 1", file=sys.stderr)
        sys.exit(2)

    if args.only is None and not args.skip_secondary and not args.no_power:
        start_power_sampler()

    import numpy as np
    import torch

    import torch_musa_amd
    from torch_musa_amd import cabi

    assert torch.cuda.is_available(), "bench.py needs the GPU"
    assert torch_musa_amd.is_loaded()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    torch.manual_seed(41)

    def events_ms(fn, n):
        """n launches, one HIP event pair each, on the current (launch) stream."""
        evs = []
        for _ in range(n):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            fn()
            b.record()
            evs.append((a, b))
        torch.cuda.synchronize()
        return [a.elapsed_time(b) for a, b in evs]

    if args.only in ("quantize", "dequantize", "minmax", "copy"):
        n = 2 ** 28
        xf = torch.randn(n, device=dev) * 3.0
        if args.only == "copy":
            yf = torch.empty_like(xf)
            fn = lambda: yf.copy_(xf)
        elif args.only == "quantize":
            # (the last three outputs stay alive: a different output buffer every launch)
            keep_ = collections.deque(maxlen=3)
            fn = lambda: keep_.append(torch.quantize_per_tensor(xf, 0.39, 128, torch.quint8))
        elif args.only == "dequantize":
            # two code tensors in turn: one alone (256 MiB) is the size of the last-level cache
            qs_ = [torch.quantize_per_tensor(xf, 0.39, 128, torch.quint8),
                   torch.quantize_per_tensor(xf * 0.5, 0.39, 128, torch.quint8)]
            cnt_ = [0]

            def fn():
                cnt_[0] += 1
                return qs_[cnt_[0] % 2].dequantize()
        else:
            ws_, mm_ = cabi.minmax_workspace(dev), torch.empty(2, device=dev)
            fn = lambda: cabi.minmax(xf, mm_, ws_)
        for _ in range(args.steps):
            fn()
        torch.cuda.synchronize()
        print(json.dumps({"only": args.only, "launches": args.steps, "elements": n}))
        return

    if args.only == "probe":
        # the int8 MFMA ceiling probes alone (for counter runs: matrix-pipe busy cycles and
        # shader clock of a loop that does nothing but multiply)
        res = {}
        for mode, name in PROBE_MODES:
            tops_p, ghz_p = cabi.probe_mfma_i8(mode)
            res[name] = {"tops": round(tops_p, 1), "shader_ghz": round(ghz_p, 3)}
        print(json.dumps({"only": "probe", "modes": res}))
        return

    if args.only == "choice":
        # The automatic kernel choice of quantized::linear against every kernel that can run the
        # shape, at shapes on either side of the dispatcher's thresholds: cold weights (as many
        # weight sets in rotation as exceed the 256 MB last-level cache, at most 40) replayed
        # in one HIP graph per candidate.  A ratio well above 1 says a threshold has gone stale.
        shapes = [(17, 4096, 4096), (24, 4096, 4096), (32, 4096, 4096), (64, 4096, 4096), (96, 4096, 4096),
                  (128, 4096, 4096), (256, 4096, 4096), (448, 4096, 4096), (512, 4096, 4096), (1024, 4096, 4096),
                  (2048, 4096, 4096), (64, 11008, 4096), (256, 11008, 4096), (2048, 11008, 4096),
                  (64, 4096, 11008), (256, 4096, 11008), (128, 1024, 1024), (512, 1024, 1024), (640, 1024, 1024),
                  (128, 2048, 2048), (256, 4096, 2048), (4096, 4096, 4096),
                  (8, 11008, 4096), (16, 11008, 4096), (16, 32000, 4096), (16, 4096, 4096), (4, 8192, 1024),
                  (32, 8192, 8192), (64, 5120, 5120), (768, 11008, 4096), (1536, 11008, 4096), (192, 6144, 3072),
                  (640, 8192, 8192)]
        candidates = (2, 3, 6, 7, 8, 13, 14, 17, 19, 20, 21, 22, 23, 24, 25, 26, 27, 28)
        rows = []
        for (Ms, Ns, Ks) in shapes:
            sets = max(2, min(40, (600 << 20) // (Ns * Ks)))
            pws = [cabi.PackedLinear(torch.randint(-127, 128, (Ns, Ks), dtype=torch.int8, device=dev))
                   for _ in range(sets)]
            wsd, bd = torch.rand(Ns, device=dev) * 0.002 + 0.001, torch.randn(Ns, device=dev)
            xd = torch.randint(0, 256, (Ms, Ks), dtype=torch.uint8, device=dev)
            yd = torch.empty((Ms, Ns), dtype=torch.uint8, device=dev)
            wbytes = cabi.lib().tmq_linear_workspace_bytes(Ms, Ns, Ks)
            cabi.linear_workspace = torch.empty(max(wbytes, 16), dtype=torch.uint8, device=dev)

            def timed(cfg):
                cabi.force_linear_config(cfg)
                try:
                    def run_sets():
                        for p_ in pws:
                            cabi.linear(xd, p_, 0.02, 128, wsd, bd, 0.05, 128, out=yd)
                    run_sets()
                    torch.cuda.synchronize()
                    side_, graph_ = torch.cuda.Stream(), torch.cuda.CUDAGraph()
                    with torch.cuda.stream(side_):
                        side_.synchronize()
                        with torch.cuda.graph(graph_, stream=side_):
                            run_sets()
                    torch.cuda.synchronize()
                    graph_.replay()
                    ts_ = sorted(events_ms(graph_.replay, 5))
                    return ts_[len(ts_) // 2] / sets * 1e3
                finally:
                    cabi.force_linear_config(-1)

            auto = cabi.linear_kernel_choice(Ms, Ns, Ks, workspace=wbytes > 0)
            t_auto = timed(-1)
            others = {}
            for cfg in candidates:
                c_ = cabi.linear_kernel_choice(Ms, Ns, Ks, workspace=wbytes > 0, forced=cfg + 1)
                if c_["kernel"] - 1 != cfg or cfg == auto["kernel"] - 1:
                    continue          # refused, or replaced by another kernel
                if c_["blocks"] > 8192 or (cfg in (2, 14, 21, 24, 25, 26, 27) and Ms * Ns > 1 << 22):
                    continue          # small tiles on a large product: not a candidate
                others[cfg] = round(timed(cfg), 2)
            best = min(others, key=others.get) if others else None
            rows.append({"M": Ms, "N": Ns, "K": Ks, "auto_kernel": auto["kernel"] - 1, "auto_us": round(t_auto, 2),
                         "best_other_kernel": best, "best_other_us": others.get(best),
                         "auto_over_best": round(t_auto / min([t_auto] + list(others.values())), 3),
                         "others_us": others})
            log(f"[bench] choice M={Ms} N={Ns} K={Ks}: auto cfg {auto['kernel'] - 1} {t_auto:.2f} us; "
                f"best other cfg {best} {others.get(best)} us")
            cabi.linear_workspace = None
            del pws
        print(json.dumps({"only": "choice", "worst_auto_over_best": max(r["auto_over_best"] for r in rows),
                          "rows": rows}))
        return

    def per_channel_sets(nsets):
        """[11008, 4096] fp32 weights (config 3's weight shape) with per-row scales."""
        out = []
        for _ in range(nsets):
            w_ = torch.randn(11008, 4096, device=dev) * 0.02
            sc_ = (w_.abs().amax(dim=1) / 127.0).to(torch.float64)
            out.append((w_, sc_, torch.zeros(11008, dtype=torch.int64, device=dev)))
        return out

    if args.only in ("quantize_pc", "dequantize_pc"):
        # inputs and outputs in rotation over more bytes than the last-level cache holds:
        # three fp32 tensors (540 MB), eight tensors of codes (360 MB)
        sets_ = per_channel_sets(3)
        keep_ = collections.deque(maxlen=8 if args.only == "quantize_pc" else 3)
        qs_ = [torch.quantize_per_channel(*sets_[i % 3], 0, torch.qint8) for i in range(8)] \
            if args.only == "dequantize_pc" else None
        for i in range(args.steps):
            if args.only == "quantize_pc":
                w_, sc_, zp_ = sets_[i % 3]
                keep_.append(torch.quantize_per_channel(w_, sc_, zp_, 0, torch.qint8))
            else:
                keep_.append(qs_[i % 8].dequantize())
        torch.cuda.synchronize()
        print(json.dumps({"only": args.only, "launches": args.steps, "shape": [11008, 4096], "axis": 0}))
        return

    if args.only in ("decode", "rows64", "rows256", "c1", "decode16_proj"):
        # config 4 at M = 1, or 64 / 256 rows against the same weights: 40 packed weights in turn
        # (cold); config 1 (M = 128, K = N = 1024) likewise; 16 rows against an output projection
        # (K = 4096, N = 32000, nine weights in turn); plain launches
        Mo, No, Ko, nsets = {"decode": (1, 4096, 4096, 40), "rows64": (64, 4096, 4096, 40), "rows256": (256, 4096, 4096, 40),
                             "c1": (128, 1024, 1024, 40), "decode16_proj": (16, 32000, 4096, 9)}[args.only]
        pws = [cabi.PackedLinear(torch.randint(-127, 128, (No, Ko), dtype=torch.int8, device=dev))
               for _ in range(nsets)]
        wsd = torch.rand(No, device=dev) * 0.002 + 0.001
        bd = torch.randn(No, device=dev)
        xd = torch.randint(0, 256, (Mo, Ko), dtype=torch.uint8, device=dev)
        yd = torch.empty((Mo, No), dtype=torch.uint8, device=dev)
        for i in range(args.steps):
            cabi.linear(xd, pws[i % nsets], 0.02, 128, wsd, bd, 0.05, 128, out=yd)
        torch.cuda.synchronize()
        print(json.dumps({"only": args.only, "launches": args.steps, "M": Mo, "K": Ko, "N": No}))
        return

    if args.only in ("conv", "conv_add_relu"):
        # config 5: 48 inputs in turn (308 MB, more than the last-level cache)
        csets = 48
        xcqs = [torch._make_per_tensor_quantized_tensor(
            torch.randint(0, 120, (32, 56, 56, 64), dtype=torch.uint8, device=dev).permute(0, 3, 1, 2), 0.03, 0)
            for _ in range(csets)]
        accs = [torch._make_per_tensor_quantized_tensor(
            torch.randint(0, 256, (32, 56, 56, 64), dtype=torch.uint8, device=dev).permute(0, 3, 1, 2), 0.03, 128)
            for _ in range(csets)] if args.only == "conv_add_relu" else None
        wc = torch.randn(64, 64, 3, 3, device=dev) * 0.05
        wcs = (wc.abs().amax(dim=(1, 2, 3)) / 127.0).to(torch.float64)
        wcq = torch.quantize_per_channel(wc, wcs, torch.zeros(64, dtype=torch.int64, device=dev), 0, torch.qint8)
        pc = torch.ops.quantized.conv2d_prepack(wcq, torch.randn(64, device=dev), [1, 1], [1, 1], [1, 1], 1)
        for i in range(args.steps):
            if accs is None:
                torch.ops.quantized.conv2d(xcqs[i % csets], pc, 0.05, 0)
            else:
                torch.ops.quantized.conv2d_add_relu(xcqs[i % csets], accs[i % csets], pc, 0.05, 0)
        torch.cuda.synchronize()
        print(json.dumps({"only": args.only, "launches": args.steps, "x": [32, 56, 56, 64], "w": [64, 3, 3, 64]}))
        return

    if args.only in ("conv_first_layer", "conv_depthwise", "conv_depthwise7"):
        # the convolution lines off the 16-channel grid: 7 x 7 stride 2, 3 -> 64 on [32,3,224,224];
        # depthwise 3 x 3 over 32 channels on [32,32,112,112] and 7 x 7 over 96 channels on [32,96,56,56];
        # twelve inputs in turn
        ic, oc, k, st, pad, groups, hw = {"conv_first_layer": (3, 64, 7, 2, 3, 1, 224), "conv_depthwise": (32, 32, 3, 1, 1, 32, 112),
                                          "conv_depthwise7": (96, 96, 7, 1, 3, 96, 56)}[args.only]
        xs_ = [torch._make_per_tensor_quantized_tensor(
            torch.randint(0, 120, (32, hw, hw, ic), dtype=torch.uint8, device=dev).permute(0, 3, 1, 2), 0.03, 0)
            for _ in range(12)]
        wf_ = torch.randn(oc, ic // groups, k, k, device=dev) * 0.05
        wq_ = torch.quantize_per_channel(wf_, (wf_.abs().amax(dim=(1, 2, 3)) / 127.0).to(torch.float64),
                                         torch.zeros(oc, dtype=torch.int64, device=dev), 0, torch.qint8)
        pk_ = torch.ops.quantized.conv2d_prepack(wq_, torch.randn(oc, device=dev), [st, st], [pad, pad], [1, 1], groups)
        for i in range(args.steps):
            torch.ops.quantized.conv2d_relu(xs_[i % 12], pk_, 0.05, 0)
        torch.cuda.synchronize()
        print(json.dumps({"only": args.only, "launches": args.steps, "x": [32, hw, hw, ic], "w": [oc, k, k, ic // groups]}))
        return

    # ------------------------------------------------------------------ C3
    M, K, N = 4096, 4096, 11008
    log(f"[bench] building config 3: M={M} K={K} N={N}")
    # Operands rotate over 4 sets (4 x 107 MB of inputs and outputs, more than the
    # 256 MB last-level cache) so that no step finds its operands cached by the
    # step before.
    NSETS = 4
    xqs, packs = [], []
    for i in range(NSETS):
        x = torch.randn(M, K, device=dev)
        w = torch.randn(N, K, device=dev) * 0.02
        bias = torch.randn(N, device=dev)
        xq = torch.quantize_per_tensor_dynamic(x, torch.quint8, False)
        w_scales = (w.abs().amax(dim=1) / 127.0).to(torch.float64)
        wq = torch.quantize_per_channel(w, w_scales, torch.zeros(N, dtype=torch.int64, device=dev), 0, torch.qint8)
        xqs.append(xq)
        packs.append(torch.ops.quantized.linear_prepack(wq, bias))
        if i == 0:
            # output scale from a calibration pass of the fp32 result, fixed thereafter
            y_f = torch.nn.functional.linear(xq.dequantize()[:256], wq.dequantize(), bias)
            out_scale = float((y_f.max() - y_f.min()) / 255.0)
            out_zp = int(round(float(-y_f.min()) / out_scale))
            out_zp = max(0, min(255, out_zp))
            xq0, wq0, w_scales0, bias0 = xq, wq, w_scales, bias
            del y_f
        del x, w
    xq, wq, w_scales, bias = xq0, wq0, w_scales0, bias0
    packed = packs[0]
    counter = [0]

    def step():
        i = counter[0] % NSETS
        counter[0] += 1
        return torch.ops.quantized.linear(xqs[i], packs[i], out_scale, out_zp)

    def settle():
        """The clock governor needs ~40 ms of this load before the launch time settles (206 us
        for the first launches, 170 us from about the 200th on): 0.2 s of untimed steps."""
        t_, n_ = time.perf_counter(), 0
        while time.perf_counter() - t_ < 0.2:
            for _ in range(20):
                step()
            torch.cuda.synchronize()
            n_ += 20
        return n_

    if args.only == "linear":
        # the timed region of the full run and nothing else: the same settle phase, then
        # --steps launches between one pair of events (a kernel trace of this command holds
        # settle + steps launches of the one kernel; its last --steps rows are the timed ones)
        settle_steps = settle()
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record()
        for _ in range(args.steps):
            step()
        ev1.record()
        torch.cuda.synchronize()
        us = ev0.elapsed_time(ev1) / args.steps * 1e3
        print(json.dumps({"only": "linear", "launches": args.steps, "untimed_settle_steps": settle_steps,
                          "avg_launch_us": round(us, 2), "tops": round(2.0 * M * N * K / us / 1e6, 1),
                          "frac_of_int8_peak": round(2.0 * M * N * K / us / 1e6 / PEAK_INT8_TOPS, 4),
                          "M": M, "K": K, "N": N}))
        return

    settle_steps = settle()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    for _ in range(args.steps):
        step()
    ev1.record()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps
    ops = 2.0 * M * N * K
    value = ops / (ms_per_step * 1e-3) / 1e12
    # one GEMM kernel per step and no gaps between them on the stream: the HIP
    # events around the timed region give the average launch duration
    kern_ms = ev0.elapsed_time(ev1) / args.steps
    achieved = ops / (kern_ms * 1e-3) / 1e12
    # the same launches one by one, an event record between them (the short idle
    # gaps let the clock recover: the part is power-limited under this load)
    iso = events_ms(step, args.steps)
    iso_ms = sum(iso) / len(iso)
    log(f"[bench] linear C3: {ms_per_step*1e3:.1f} us/step wall, {kern_ms*1e3:.1f} us/launch (events over the "
        f"timed region), {achieved:.0f} TOP/s; {iso_ms*1e3:.1f} us/launch when launches are timed one by one")
    roofline = {"bound": "mfma", "achieved": round(achieved, 1), "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
                "frac": round(achieved / PEAK_INT8_TOPS, 4), "traffic": MEASURED_TRAFFIC["linear_c3"],
                "kernel": "tmq::gemm_i8_persistent_kernel", "ops_per_launch": ops,
                "avg_launch_us": round(kern_ms * 1e3, 2),
                "isolated_launch_us": round(iso_ms * 1e3, 2),
                "algorithmic_bytes_per_launch": M * K + N * K + M * N + 12 * N,
                "operand_sets_rotated": NSETS, "untimed_settle_steps_before_warmup": settle_steps}

    secondary = {}
    if not args.skip_secondary:
        # ---------------------------------------------- matrix-pipe ceiling probe
        log("[bench] int8 MFMA ceiling probe (register-only loop, 256 workgroups)")
        probe = {}
        for mode, name in PROBE_MODES:
            tops_p, ghz_p = cabi.probe_mfma_i8(mode)
            probe[name] = {"tops": round(tops_p, 1), "shader_ghz": round(ghz_p, 3)}
            log(f"[bench]   {name}: {tops_p:.0f} TOP/s at {ghz_p:.2f} GHz")
        secondary["mfma_i8_ceiling_probe"] = probe

        # ---------------------------------------------- power under the timed load, and a control
        # The product kernel (torch.ops.quantized.linear, config 3's shape, same settle phase and
        # timing as the headline) on operands that barely toggle the multipliers: every
        # activation byte 128 (the kernel feeds x ^ 0x80 = 0) and weights 0..3.  Same
        # instruction stream, same bytes moved; what differs is the energy of a multiply.  The
        # socket power is sampled by a child process while each load runs.
        log("[bench] socket power under config 3, and the same kernel on low-toggle operands")

        def load20():
            for _ in range(20):
                step()
            torch.cuda.synchronize()

        power_c3 = sample_power_while(load20)
        lt_x, lt_p = [], []
        for i in range(NSETS):
            lt_x.append(torch._make_per_tensor_quantized_tensor(
                torch.full((M, K), 128, dtype=torch.uint8, device=dev), xq.q_scale(), 128))
            wlt = torch._make_per_channel_quantized_tensor(
                torch.randint(0, 4, (N, K), dtype=torch.int8, device=dev), w_scales,
                torch.zeros(N, dtype=torch.int64, device=dev), 0)
            lt_p.append(torch.ops.quantized.linear_prepack(wlt, bias))
            del wlt
        lt_count = [0]

        def lt_step():
            i = lt_count[0] % NSETS
            lt_count[0] += 1
            return torch.ops.quantized.linear(lt_x[i], lt_p[i], out_scale, out_zp)

        def lt_load20():
            for _ in range(20):
                lt_step()
            torch.cuda.synchronize()

        t_ = time.perf_counter()
        while time.perf_counter() - t_ < 0.2:
            lt_load20()
        ea, eb = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ea.record()
        for _ in range(args.steps):
            lt_step()
        eb.record()
        torch.cuda.synchronize()
        lt_us = ea.elapsed_time(eb) / args.steps * 1e3
        power_lt = sample_power_while(lt_load20)
        # back to the benchmark operands for a second reading of the headline in the same state
        settle()
        ea.record()
        for _ in range(args.steps):
            step()
        eb.record()
        torch.cuda.synchronize()
        again_us = ea.elapsed_time(eb) / args.steps * 1e3
        lt_tops = ops / lt_us / 1e6
        log(f"[bench]   low-toggle operands: {lt_us:.1f} us/launch = {lt_tops:.0f} TOP/s ({lt_tops / PEAK_INT8_TOPS:.3f} of "
            f"peak), benchmark operands again {again_us:.1f} us; socket power {power_c3.get('socket_power_w_avg')} W "
            f"(benchmark) / {power_lt.get('socket_power_w_avg')} W (low toggle), cap {power_c3.get('power_cap_w')} W")
        secondary["linear_c3_low_toggle"] = {
            "avg_launch_us": round(lt_us, 2), "value": round(lt_tops, 1), "unit": "TOP/s",
            "frac_of_int8_peak": round(lt_tops / PEAK_INT8_TOPS, 4),
            "benchmark_operands_same_state_us": round(again_us, 2),
            "speedup_over_benchmark_operands": round(again_us / lt_us, 4),
            "power": power_lt,
            "method": "torch.ops.quantized.linear at config 3's shape, x = 128 everywhere (fed to the matrix "
                      "pipe as 0), weights uniform in 0..3, 4 operand sets rotated; 0.2 s settle, then --steps "
                      "launches between one pair of events, as the headline"}
        roofline["socket_power"] = power_c3
        del lt_x, lt_p
        roofline["power_limited_ceiling_tops"] = probe["gaussian_int8"]["tops"]
        roofline["frac_of_power_limited_ceiling"] = round(achieved / probe["gaussian_int8"]["tops"], 4)
        # the same with operands that change every instruction, as a GEMM's do
        roofline["fresh_operand_ceiling_tops"] = probe["gaussian_int8_fresh_from_lds"]["tops"]
        roofline["frac_of_fresh_operand_ceiling"] = round(
            achieved / probe["gaussian_int8_fresh_from_lds"]["tops"], 4)

        # -------------------------------------------------------------- C2
        n = 2 ** 28
        log("[bench] config 2: quantize / dequantize / min-max over 2**28 fp32")
        xf = torch.randn(n, device=dev) * 3.0
        idx = torch.randint(0, n, (n // 100,), device=dev)
        xf[idx] = torch.where(torch.rand(idx.numel(), device=dev) < 0.5, 50.0, -50.0)
        del idx
        mm = cabi.minmax(xf).cpu()
        scale, zp = cabi.choose_qparams_host(float(mm[0]), float(mm[1]), False, False)
        q = torch.quantize_per_tensor(xf, scale, zp, torch.quint8)
        ws = cabi.minmax_workspace(dev)
        mm_out = torch.empty(2, device=dev)

        def hbm(name, fn, bytes_per_launch, key, back_to_back=10):
            # The last three results stay alive, so that an operator's output goes to a
            # different buffer every launch: written again and again, one 256 MiB buffer of codes
            # stays in the last-level cache (256 MB) and its writes never reach memory
            # (quantize_per_tensor then takes 193 instead of 213 us).  One event pair around
            # a run of launches (a pair per launch adds 1.5 - 2 us to each, 5 % of the
            # per-channel kernels), three runs.
            keep = collections.deque(maxlen=3)

            def run():
                for _ in range(back_to_back):
                    keep.append(fn())

            run()
            ts = [t_ / back_to_back for t_ in events_ms(run, 3)]
            keep.clear()
            avg = sum(ts) / len(ts)
            gbs = bytes_per_launch / (avg * 1e-3) / 1e9
            log(f"[bench] {name}: {avg*1e3:.1f} us/launch, {gbs:.0f} GB/s")
            secondary[name] = {"avg_launch_us": round(avg * 1e3, 2), "value": round(gbs, 1), "unit": "GB/s",
                               "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS,
                                            "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4),
                                            "traffic": MEASURED_TRAFFIC.get(key)},
                               "algorithmic_bytes_per_launch": bytes_per_launch}

        hbm("quantize_per_tensor_c2", lambda: torch.quantize_per_tensor(xf, scale, zp, torch.quint8), 5 * n,
            "quantize_c2")
        for _ in range(3):
            torch.quantize_per_tensor(xf, scale, zp, torch.quint8)
        ts_same = events_ms(lambda: torch.quantize_per_tensor(xf, scale, zp, torch.quint8), 10)
        secondary["quantize_per_tensor_c2"]["reusing_one_output_buffer_us"] = round(sum(ts_same) / len(ts_same) * 1e3, 2)
        # two code tensors in turn: one alone (256 MiB) is the size of the last-level cache
        q_alt = torch.quantize_per_tensor(xf * 0.5, scale, zp, torch.quint8)
        dq_count = [0]

        def dequantize_rotating():
            dq_count[0] += 1
            return (q if dq_count[0] % 2 else q_alt).dequantize()

        hbm("dequantize_c2", dequantize_rotating, 5 * n, "dequantize_c2")
        del q_alt
        hbm("minmax_c2", lambda: cabi.minmax(xf, mm_out, ws), 4 * n, "minmax_c2")
        hbm("quantize_per_tensor_dynamic_c2", lambda: torch.quantize_per_tensor_dynamic(xf, torch.quint8, False),
            9 * n, None)
        # elementwise glue on quantized tensors of the same element count
        q2 = torch.quantize_per_tensor(xf * 0.5, scale, zp, torch.quint8)
        hbm("quantized_add_2p28", lambda: torch.ops.quantized.add(q, q2, scale * 1.5, zp), 3 * n, None)
        hbm("quantized_relu_2p28", lambda: torch.relu(q), 2 * n, None)
        hbm("quantized_gelu_2p28", lambda: torch.nn.functional.gelu(q), 2 * n, None)
        del xf, q, q2

        # per-channel quantize / dequantize at config 3's weight shape, axis 0: 45 M elements,
        # three tensors in turn (3 x 225 MB of input and output, more than the last-level cache)
        log("[bench] per-channel quantize / dequantize, fp32 [11008, 4096], axis 0")
        pcs = per_channel_sets(3)
        pc_count = [0]
        # (eight buffers of codes, 360 MB: three would fit the last-level cache together)
        pc_out = [torch.empty((11008, 4096), dtype=torch.int8, device=dev) for _ in range(8)]
        lib = cabi.lib()

        def quantize_pc_kernel():
            # the kernel through the C ABI (the operator adds a host-side check of the zero
            # points' range in front of it, as the reference does: timed below)
            pc_count[0] += 1
            i = pc_count[0] % 8
            w_, sc_, zp_ = pcs[pc_count[0] % 3]
            cabi.check(lib.tmq_quantize_per_channel(w_.data_ptr(), pc_out[i].data_ptr(), 1, 11008, 4096,
                                                    sc_.data_ptr(), zp_.data_ptr(), 1, cabi.stream_ptr()),
                       "tmq_quantize_per_channel")

        npc = 11008 * 4096
        hbm("quantize_per_channel_11008x4096", quantize_pc_kernel, 5 * npc + 16 * 11008, "quantize_pc", back_to_back=30)

        def quantize_pc_op():
            pc_count[0] += 1
            w_, sc_, zp_ = pcs[pc_count[0] % 3]
            return torch.quantize_per_channel(w_, sc_, zp_, 0, torch.qint8)

        for _ in range(3):
            quantize_pc_op()
        ts = events_ms(quantize_pc_op, 20)
        secondary["quantize_per_channel_11008x4096"]["operator_call_us"] = round(sum(ts) / len(ts) * 1e3, 1)
        pc_r = [torch.empty((11008, 4096), dtype=torch.float32, device=dev) for _ in range(3)]

        def dequantize_pc_kernel():
            pc_count[0] += 1
            i = pc_count[0] % 8
            _, sc_, zp_ = pcs[pc_count[0] % 3]
            cabi.check(lib.tmq_dequantize_per_channel(pc_out[i].data_ptr(), pc_r[pc_count[0] % 3].data_ptr(), 1, 11008, 4096,
                                                      sc_.data_ptr(), zp_.data_ptr(), 1, cabi.stream_ptr()),
                       "tmq_dequantize_per_channel")

        hbm("dequantize_per_channel_11008x4096", dequantize_pc_kernel, 5 * npc + 16 * 11008, "dequantize_pc",
            back_to_back=30)
        del pcs, pc_out, pc_r

        # -------------------------------------------------------------- C1
        # x [128,1024] quint8 x W [1024,1024] per-channel qint8: 268 MOP and 1.2 MB, a
        # latency measurement (50 launches replayed from one HIP graph)
        log("[bench] config 1: linear M=128, K=N=1024")
        x1 = torch.quantize_per_tensor_dynamic(torch.randn(128, 1024, device=dev), torch.quint8, False)
        w1 = torch.randn(1024, 1024, device=dev) * 0.02
        w1q = torch.quantize_per_channel(w1, (w1.abs().amax(dim=1) / 127.0).to(torch.float64),
                                         torch.zeros(1024, dtype=torch.int64, device=dev), 0, torch.qint8)
        p1 = torch.ops.quantized.linear_prepack(w1q, torch.randn(1024, device=dev))

        def lin1():
            return torch.ops.quantized.linear(x1, p1, 0.05, 128)

        for _ in range(5):
            lin1()
        side = torch.cuda.Stream()
        g1 = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            lin1()
            side.synchronize()
            with torch.cuda.graph(g1, stream=side):
                for _ in range(50):
                    lin1()
        torch.cuda.synchronize()
        for _ in range(3):
            g1.replay()
        ts = events_ms(g1.replay, 10)
        per1 = sum(ts) / len(ts) / 50
        ops1 = 2.0 * 128 * 1024 * 1024
        log(f"[bench] linear C1: {per1*1e3:.2f} us/launch in a replayed graph, {ops1 / (per1 * 1e-3) / 1e12:.1f} TOP/s")
        secondary["linear_c1"] = {
            "avg_launch_us": round(per1 * 1e3, 3), "value": round(ops1 / (per1 * 1e-3) / 1e12, 2), "unit": "TOP/s",
            "roofline": {"bound": "mfma", "achieved": round(ops1 / (per1 * 1e-3) / 1e12, 2), "peak": PEAK_INT8_TOPS,
                         "unit": "TOP/s", "frac": round(ops1 / (per1 * 1e-3) / 1e12 / PEAK_INT8_TOPS, 5),
                         "traffic": None},
            "traffic_with_cold_weights": MEASURED_TRAFFIC["c1"],
            "method": "50 launches replayed in one HIP graph; launch-latency-bound at this size",
            "ops_per_launch": ops1, "algorithmic_bytes_per_launch": 128 * 1024 + 1024 * 1024 + 128 * 1024 + 12 * 1024}
        del x1, w1, w1q, p1, g1

        # -------------------------------------------------------------- C4
        log("[bench] config 4: decode-shaped linear, K=N=4096, cold weights (40 weight sets, HIP graph)")
        Kd = Nd = 4096
        sets = 40  # 40 x 16.8 MB > 2 x the 256 MB last-level cache
        pws = [cabi.PackedLinear(torch.randint(-127, 128, (Nd, Kd), dtype=torch.int8, device=dev))
               for _ in range(sets)]
        wsd = torch.rand(Nd, device=dev) * 0.002 + 0.001
        bd = torch.randn(Nd, device=dev)
        def graph_us(run_once, calls):
            run_once()
            torch.cuda.synchronize()
            side_ = torch.cuda.Stream()
            graph_ = torch.cuda.CUDAGraph()
            with torch.cuda.stream(side_):
                run_once()
                side_.synchronize()
                with torch.cuda.graph(graph_, stream=side_):
                    run_once()
            torch.cuda.synchronize()
            for _ in range(3):
                graph_.replay()
            ts_ = events_ms(graph_.replay, 10)
            return sum(ts_) / len(ts_) / calls * 1e3

        # floors, measured the same way: an empty kernel of the decode kernel's grid, and a kernel
        # of its shape that only reads the 16.8 MB of packed weights (nothing computed, nothing stored)
        sink = torch.zeros(4096, dtype=torch.uint8, device=dev)
        empty_us = graph_us(lambda: [cabi.bench_empty_kernel(Nd // 16, sink) for _ in range(sets)], sets)
        read_us = graph_us(lambda: [cabi.bench_stream_read(p.packed, sink) for p in pws], sets)
        log(f"[bench] decode floors in a replayed graph: empty kernel {empty_us:.2f} us, read-only kernel "
            f"{read_us:.2f} us per launch")
        secondary["linear_decode_floors"] = {
            "empty_kernel_us": round(empty_us, 3), "read_only_kernel_us": round(read_us, 3),
            "read_only_gbs": round(Nd * Kd / read_us / 1e3, 1),
            "method": f"{sets} launches replayed in one HIP graph, as for the operator: an empty kernel on "
                      f"{Nd // 16} workgroups of eight waves; a kernel of the decode kernel's shape that only "
                      "reads the packed weight of each of the 40 sets"}
        for Md in (1, 4, 16):
            xd = torch.randint(0, 256, (Md, Kd), dtype=torch.uint8, device=dev)
            yd = torch.empty((Md, Nd), dtype=torch.uint8, device=dev)

            def run_sets():
                for p in pws:
                    cabi.linear(xd, p, 0.02, 128, wsd, bd, 0.05, 128, out=yd)

            per = graph_us(run_sets, sets) * 1e-3
            nbytes = Nd * Kd + Md * Kd + Md * Nd + 12 * Nd
            gbs = nbytes / (per * 1e-3) / 1e9
            log(f"[bench] decode M={Md}: {per*1e3:.2f} us/launch in a replayed graph, {gbs:.0f} GB/s")
            secondary[f"linear_decode_m{Md}"] = {
                "avg_launch_us": round(per * 1e3, 3), "value": round(gbs, 1), "unit": "GB/s",
                "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                             "frac": round(gbs / PEAK_HBM_GBS, 4),
                             "traffic": MEASURED_TRAFFIC["decode_m1"] if Md == 1 else None},
                "frac_of_read_only_kernel": round(read_us / (per * 1e3), 4),
                "method": f"{sets} distinct packed weights replayed back to back in one HIP graph",
                "algorithmic_bytes_per_launch": nbytes}

        # ----------------------------- decode rows against an output projection: K = 4096, N = 32000
        # (131 MB of weights per launch, nine sets in rotation; from 12 rows on the kernel that keeps
        # the rows in LDS, below it a block per 16 channels), torch._int_mm beside it
        Np = 32000
        sets_p = 9
        pwp = [cabi.PackedLinear(torch.randint(-127, 128, (Np, Kd), dtype=torch.int8, device=dev))
               for _ in range(sets_p)]
        wsp = torch.rand(Np, device=dev) * 0.002 + 0.001
        bp = torch.randn(Np, device=dev)
        wts_p = None
        for Md in (1, 16):
            xd = torch.randint(0, 256, (Md, Kd), dtype=torch.uint8, device=dev)
            yd = torch.empty((Md, Np), dtype=torch.uint8, device=dev)

            def run_proj():
                for p in pwp:
                    cabi.linear(xd, p, 0.02, 128, wsp, bp, 0.05, 128, out=yd)

            per = graph_us(run_proj, sets_p)
            vendor = None
            try:
                if wts_p is None:
                    wts_p = [torch.randint(-127, 128, (Np, Kd), dtype=torch.int8, device=dev).t() for _ in range(sets_p)]
                xs8 = torch.randint(-128, 128, (max(Md, 32), Kd), dtype=torch.int8, device=dev)  # (the op wants > 16 rows)
                vendor = graph_us(lambda: [torch._int_mm(xs8, wt) for wt in wts_p], sets_p)
            except Exception as ex:
                log(f"[bench] torch._int_mm not timed: {ex}")
            nbytes = Np * Kd + Md * Kd + Md * Np + 12 * Np
            gbs = nbytes / per / 1e3
            kern = cabi.linear_kernel_choice(Md, Np, Kd)["kernel"] - 1
            log(f"[bench] decode M={Md} against N={Np}: {per:.2f} us/launch (kernel {kern}), {gbs:.0f} GB/s"
                + (f" (torch._int_mm on {max(Md, 32)} rows: {vendor:.2f} us)" if vendor else ""))
            secondary[f"linear_decode_m{Md}_n{Np}"] = {
                "avg_launch_us": round(per, 3), "value": round(gbs, 1), "unit": "GB/s", "kernel": kern,
                "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                             "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": None},
                "torch_int_mm_us": None if vendor is None else round(vendor, 3),
                "method": f"{sets_p} distinct packed weights replayed back to back in one HIP graph",
                "algorithmic_bytes_per_launch": nbytes}
        del pwp, wts_p

        # ----------------------------- the same cold weights against a few dozen to a few hundred rows
        # (32 x 32 / 32 x 64 / 64 x 64 tiles whose waves split K and take their weights through
        # registers; 64 x 128 pipelined tiles at 512 rows), with the vendor's int8 GEMM
        # (torch._int_mm: int32 output, no requantisation) beside it
        wts_mm = None
        for Md in (64, 128, 256, 512):
            xd = torch.randint(0, 256, (Md, Kd), dtype=torch.uint8, device=dev)
            yd = torch.empty((Md, Nd), dtype=torch.uint8, device=dev)

            def run_sets():
                for p in pws:
                    cabi.linear(xd, p, 0.02, 128, wsd, bd, 0.05, 128, out=yd)

            per = graph_us(run_sets, sets)
            vendor = None
            try:
                if wts_mm is None:
                    wts_mm = [torch.randint(-127, 128, (Nd, Kd), dtype=torch.int8, device=dev).t() for _ in range(sets)]
                xs8 = torch.randint(-128, 128, (Md, Kd), dtype=torch.int8, device=dev)
                vendor = graph_us(lambda: [torch._int_mm(xs8, wt) for wt in wts_mm], sets)
            except Exception as ex:  # the comparison is optional: a torch build without the op
                log(f"[bench] torch._int_mm not timed: {ex}")
            nbytes = Nd * Kd + Md * Kd + Md * Nd + 12 * Nd
            log(f"[bench] M={Md} against config 4's cold weights: {per:.2f} us/launch in a replayed graph"
                + (f" (torch._int_mm: {vendor:.2f} us)" if vendor else ""))
            secondary[f"linear_m{Md}_k4096_n4096"] = {
                "avg_launch_us": round(per, 3), "value": round(2.0 * Md * Kd * Nd / per / 1e6, 1), "unit": "TOP/s",
                "weights_gbs": round(Nd * Kd / per / 1e3, 1),
                "torch_int_mm_us": None if vendor is None else round(vendor, 3),
                "traffic": MEASURED_TRAFFIC["rows64"] if Md == 64 else None,
                "method": f"{sets} distinct packed weights replayed back to back in one HIP graph; the vendor GEMM "
                          "the same way on as many int8 matrices of the shape",
                "algorithmic_bytes_per_launch": nbytes}
        del wts_mm

        # ----------------------------- dynamically quantized linear, decode-sized
        # fp32 [M, 4096] -> fp32 [M, 4096]: up to 16384 input values one launch (every block
        # of the weight-streaming kernel quantizes the input itself), else one launch for
        # range + parameters + codes and one for the product; 40 cold weights replayed in
        # one HIP graph as above
        for Md in (1, 16):
            xdf = torch.randn(Md, Kd, device=dev)

            def run_dyn():
                for p in pws:
                    cabi.linear_dynamic(xdf, p, wsd, bd)

            run_dyn()
            torch.cuda.synchronize()
            side = torch.cuda.Stream()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.stream(side):
                run_dyn()
                side.synchronize()
                with torch.cuda.graph(graph, stream=side):
                    run_dyn()
            torch.cuda.synchronize()
            for _ in range(3):
                graph.replay()
            ts = events_ms(graph.replay, 10)
            per = sum(ts) / len(ts) / sets
            nbytes = Nd * Kd + 2 * 4 * Md * Kd + 2 * Md * Kd + 4 * Md * Nd + 12 * Nd
            gbs = nbytes / (per * 1e-3) / 1e9
            nl = 1 if Md * Kd <= 16384 else 2
            log(f"[bench] dynamic decode M={Md}: {per*1e3:.2f} us per call ({nl} launch{'es' if nl > 1 else ''}) "
                "in a replayed graph")
            secondary[f"linear_dynamic_decode_m{Md}"] = {
                "avg_call_us": round(per * 1e3, 3), "value": round(gbs, 1), "unit": "GB/s",
                "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                             "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": None},
                "method": f"{sets} distinct packed weights replayed back to back in one HIP graph",
                "algorithmic_bytes_per_call": nbytes}
        del pws

        # ----------------------------- a few hundred rows against a long K (split K)
        # M = 256, K = 11008, N = 4096 (the down projection of config 3's layer at a
        # batch of 256 rows): 64 tiles of 128 x 128, cut four ways along K into a
        # caller-owned workspace, then one pass that adds and requantises
        log("[bench] linear M=256, K=11008, N=4096: split K against the single-launch kernel (8 weight sets, HIP graph)")
        Ms, Ks, Ns = 256, 11008, 4096
        pws = [cabi.PackedLinear(torch.randint(-127, 128, (Ns, Ks), dtype=torch.int8, device=dev)) for _ in range(8)]
        cabi.linear_workspace = torch.empty(cabi.lib().tmq_linear_workspace_bytes(Ms, Ns, Ks), dtype=torch.uint8,
                                            device=dev)
        wts_mm = None
        for Ms in (256, 64):
            xs_ = torch.randint(0, 256, (Ms, Ks), dtype=torch.uint8, device=dev)
            ys_ = torch.empty((Ms, Ns), dtype=torch.uint8, device=dev)
            split_us = {}
            for use in (False, True):
                cabi.use_linear_workspace = use

                def run_split_sets():
                    for p in pws:
                        cabi.linear(xs_, p, 0.02, 128, wsd, bd, 0.05, 128, out=ys_)

                split_us[use] = graph_us(run_split_sets, len(pws))
            cabi.use_linear_workspace = True
            vendor = None
            try:
                if wts_mm is None:
                    wts_mm = [torch.randint(-127, 128, (Ns, Ks), dtype=torch.int8, device=dev).t() for _ in range(8)]
                xs8 = torch.randint(-128, 128, (Ms, Ks), dtype=torch.int8, device=dev)
                vendor = graph_us(lambda: [torch._int_mm(xs8, wt) for wt in wts_mm], len(wts_mm))
            except Exception as ex:  # the comparison is optional
                log(f"[bench] torch._int_mm not timed: {ex}")
            ops_s = 2.0 * Ms * Ns * Ks
            plan = cabi.linear_split_plan(Ms, Ns, Ks)
            log(f"[bench] M={Ms}, K=11008, N=4096: {split_us[True]:.1f} us per call (split K, 2 launches), single "
                f"launch {split_us[False]:.1f} us" + (f", torch._int_mm {vendor:.1f} us" if vendor else ""))
            key = "linear_split_k_m256_k11008_n4096" if Ms == 256 else f"linear_m{Ms}_k11008_n4096"
            secondary[key] = {
                "avg_call_us": round(split_us[True], 2), "single_launch_us": round(split_us[False], 2),
                "torch_int_mm_us": None if vendor is None else round(vendor, 2),
                "value": round(ops_s / (split_us[True] * 1e-6) / 1e12, 1), "unit": "TOP/s",
                "method": f"8 distinct packed weights replayed back to back in one HIP graph; {plan[0]} splits of "
                          f"{plan[1]} stages, int32 partial sums in a shared workspace; the vendor GEMM the same way "
                          "(int32 output, no requantisation)"}
        cabi.linear_workspace = None
        del pws, xs_, ys_, wts_mm

        # ------------------------------------------- dynamically quantized linear
        # quantized::linear_dynamic at config 3's shape: fp32 in, min/max + qparams +
        # quantize + int8 product + fp32 out: three launches (range, codes, product), no host round trip
        log("[bench] linear_dynamic at config 3's shape (fp32 in, fp32 out)")
        xds = [torch.randn(M, K, device=dev) for _ in range(2)]
        dcount = [0]

        def dyn():
            dcount[0] += 1
            return torch.ops.quantized.linear_dynamic(xds[dcount[0] % 2], packs[dcount[0] % NSETS], False)

        for _ in range(30):
            dyn()
        torch.cuda.synchronize()
        a_, b_ = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a_.record()
        for _ in range(50):
            dyn()
        b_.record()
        torch.cuda.synchronize()
        dms = a_.elapsed_time(b_) / 50
        dbytes = 2 * 4 * M * K + 2 * M * K + N * K + 4 * M * N + 12 * N
        log(f"[bench] linear_dynamic: {dms*1e3:.1f} us per call, {ops / (dms * 1e-3) / 1e12:.0f} TOP/s")
        secondary["linear_dynamic_c3_shape"] = {
            "avg_call_us": round(dms * 1e3, 1), "value": round(ops / (dms * 1e-3) / 1e12, 1), "unit": "TOP/s",
            "roofline": {"bound": "mfma", "achieved": round(ops / (dms * 1e-3) / 1e12, 1), "peak": PEAK_INT8_TOPS,
                         "unit": "TOP/s", "frac": round(ops / (dms * 1e-3) / 1e12 / PEAK_INT8_TOPS, 4),
                         "traffic": None},
            "method": "50 calls back to back between two events, 2 inputs x 4 weights rotated",
            "algorithmic_bytes_per_call": dbytes, "ops_per_call": ops}
        del xds

        # --------------------- the plain-tensor op at config 3's shape, steady state
        # quantized::linear_per_tensor takes the int8 weight as an ordinary [K, N] tensor on
        # every call; its re-tiled copy is kept per weight tensor, so calls after the first
        # launch the GEMM only
        log("[bench] quantized::linear_per_tensor at config 3's shape (plain uint8 / int8 tensors)")
        w_kn = wq.int_repr().t().contiguous()
        x_u8 = xq.int_repr()
        ws32 = w_scales.to(torch.float32)
        wz32 = torch.zeros(N, dtype=torch.int32, device=dev)

        def lin_plain():
            return torch.ops.quantized.linear_per_tensor(x_u8, xq.q_scale(), xq.q_zero_point(), w_kn, ws32, wz32, bias,
                                                         out_scale, out_zp, torch.uint8, "none", [], "")

        ev_a, ev_b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev_a.record()
        y_first = lin_plain()
        ev_b.record()
        torch.cuda.synchronize()
        first_us = ev_a.elapsed_time(ev_b) * 1e3
        assert torch.equal(y_first, torch.ops.quantized.linear(xq, packed, out_scale, out_zp).int_repr())
        for _ in range(20):
            lin_plain()
        ts = events_ms(lin_plain, 50)
        steady_us = sum(ts) / len(ts) * 1e3
        ts = events_ms(lambda: torch.ops.quantized.linear(xq, packed, out_scale, out_zp), 50)
        packed_us = sum(ts) / len(ts) * 1e3
        log(f"[bench] linear_per_tensor: first call {first_us:.0f} us (re-tiles the weight), then {steady_us:.1f} us "
            f"per call; quantized::linear with the packed weight {packed_us:.1f} us")
        secondary["linear_per_tensor_c3_shape"] = {
            "first_call_us": round(first_us, 1), "steady_call_us": round(steady_us, 1),
            "quantized_linear_same_operands_us": round(packed_us, 1),
            "value": round(ops / (steady_us * 1e-6) / 1e12, 1), "unit": "TOP/s",
            "method": "one operand set, 50 calls timed one by one with HIP events after 20 warm-up calls; "
                      "output bytes equal quantized::linear's"}
        del w_kn, x_u8

        # -------------------------------------------------------------- C5
        log("[bench] config 5: conv2d NHWC [32,56,56,64] x [64,3,3,64]")
        xc = torch.relu(torch.randn(32, 64, 56, 56, device=dev)).contiguous(memory_format=torch.channels_last)
        xcq = torch.quantize_per_tensor_dynamic(xc, torch.quint8, False)
        wc = torch.randn(64, 64, 3, 3, device=dev) * 0.05
        wcs = (wc.abs().amax(dim=(1, 2, 3)) / 127.0).to(torch.float64)
        wcq = torch.quantize_per_channel(wc, wcs, torch.zeros(64, dtype=torch.int64, device=dev), 0, torch.qint8)
        pc = torch.ops.quantized.conv2d_prepack(wcq, torch.randn(64, device=dev), [1, 1], [1, 1], [1, 1], 1)
        # 48 input tensors: 308 MB, more than the last-level cache, so a launch does not
        # find its input cached
        csets = 48
        xcqs = [xcq]
        for _ in range(csets - 1):
            xf_ = torch.relu(torch.randn(32, 64, 56, 56, device=dev)).contiguous(memory_format=torch.channels_last)
            xcqs.append(torch.quantize_per_tensor(xf_, xcq.q_scale(), xcq.q_zero_point(), torch.quint8))
            del xf_
        assert all(t_.is_contiguous(memory_format=torch.channels_last) for t_ in xcqs)
        ccount = [0]

        def conv():
            ccount[0] += 1
            return torch.ops.quantized.conv2d(xcqs[ccount[0] % csets], pc, 0.05, 0)

        for _ in range(5):
            conv()
        ts = events_ms(conv, 30)
        single = sum(ts) / len(ts)
        # a ~10 us kernel: one launch between two events mostly times the launch
        # path, so the figure of merit is 50 launches replayed from a HIP graph
        reps = 2 * csets
        side = torch.cuda.Stream()
        cgraph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            conv()
            side.synchronize()
            with torch.cuda.graph(cgraph, stream=side):
                for _ in range(reps):
                    conv()
        torch.cuda.synchronize()
        for _ in range(3):
            cgraph.replay()
        ts = events_ms(cgraph.replay, 10)
        avg = sum(ts) / len(ts) / reps
        cops = 2.0 * 32 * 56 * 56 * 64 * 576
        cbytes = 2 * 32 * 56 * 56 * 64 + 64 * 576 + 768
        log(f"[bench] conv2d C5: {avg*1e3:.1f} us/launch in a replayed graph ({single*1e3:.1f} us as a single "
            f"launch between events), {cops/(avg*1e-3)/1e12:.0f} TOP/s, {cbytes/(avg*1e-3)/1e9:.0f} GB/s")
        secondary["conv2d_c5"] = {
            "avg_launch_us": round(avg * 1e3, 2), "single_launch_us": round(single * 1e3, 2),
            "value": round(cops / (avg * 1e-3) / 1e12, 1), "unit": "TOP/s",
            "roofline": {"bound": "mfma", "achieved": round(cops / (avg * 1e-3) / 1e12, 1),
                         "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
                         "frac": round(cops / (avg * 1e-3) / 1e12 / PEAK_INT8_TOPS, 4),
                         "traffic": MEASURED_TRAFFIC["conv_c5"]},
            "hbm_frac": round(cbytes / (avg * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
            "method": f"{reps} launches over {csets} rotating inputs replayed back to back in one HIP graph",
            "algorithmic_bytes_per_launch": cbytes, "ops_per_launch": cops}

        # ---------------------------------------- C5 with a fused residual + ReLU
        log("[bench] config 5 + residual: conv2d_add_relu, same shapes, quantized residual of the output's shape")
        accs = []
        for _ in range(csets):
            af_ = torch.randn(32, 64, 56, 56, device=dev).contiguous(memory_format=torch.channels_last)
            accs.append(torch.quantize_per_tensor(af_, 0.03, 128, torch.quint8))
            del af_
        fcount = [0]

        def conv_add_relu():
            fcount[0] += 1
            i = fcount[0] % csets
            return torch.ops.quantized.conv2d_add_relu(xcqs[i], accs[i], pc, 0.05, 0)

        for _ in range(5):
            conv_add_relu()
        fgraph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            conv_add_relu()
            side.synchronize()
            with torch.cuda.graph(fgraph, stream=side):
                for _ in range(reps):
                    conv_add_relu()
        torch.cuda.synchronize()
        for _ in range(3):
            fgraph.replay()
        ts = events_ms(fgraph.replay, 10)
        favg = sum(ts) / len(ts) / reps
        fbytes = cbytes + 32 * 56 * 56 * 64
        log(f"[bench] conv2d_add_relu C5: {favg*1e3:.1f} us/launch in a replayed graph, "
            f"{cops/(favg*1e-3)/1e12:.0f} TOP/s, {fbytes/(favg*1e-3)/1e9:.0f} GB/s")
        secondary["conv2d_add_relu_c5"] = {
            "avg_launch_us": round(favg * 1e3, 2), "value": round(cops / (favg * 1e-3) / 1e12, 1), "unit": "TOP/s",
            "roofline": {"bound": "mfma", "achieved": round(cops / (favg * 1e-3) / 1e12, 1),
                         "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
                         "frac": round(cops / (favg * 1e-3) / 1e12 / PEAK_INT8_TOPS, 4),
                         "traffic": MEASURED_TRAFFIC["conv_add_relu_c5"]},
            "hbm_frac": round(fbytes / (favg * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
            "method": f"{reps} launches over {csets} rotating inputs and residuals replayed in one HIP graph",
            "algorithmic_bytes_per_launch": fbytes, "ops_per_launch": cops}
        del accs, xcqs

        # ------------------------- quantized max pooling, the ResNet stem's shape
        log("[bench] quantized max_pool2d 3x3/2 on [32,64,112,112] channels-last")
        psets = 12  # 12 x 25.7 MB of input, more than the last-level cache
        pxs = []
        for _ in range(psets):
            pf_ = torch.randn(32, 64, 112, 112, device=dev).contiguous(memory_format=torch.channels_last)
            pxs.append(torch.quantize_per_tensor(pf_, 0.03, 128, torch.quint8))
            del pf_
        pcount = [0]

        def pool():
            pcount[0] += 1
            return torch.nn.functional.max_pool2d(pxs[pcount[0] % psets], 3, 2, 1)

        for _ in range(3):
            pool()
        pgraph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            pool()
            side.synchronize()
            with torch.cuda.graph(pgraph, stream=side):
                for _ in range(2 * psets):
                    pool()
        torch.cuda.synchronize()
        for _ in range(3):
            pgraph.replay()
        ts = events_ms(pgraph.replay, 10)
        pavg = sum(ts) / len(ts) / (2 * psets)
        pbytes = 32 * 64 * (112 * 112 + 56 * 56)
        log(f"[bench] quantized max_pool2d: {pavg*1e3:.1f} us/launch in a replayed graph, {pbytes/(pavg*1e-3)/1e9:.0f} GB/s")
        secondary["quantized_max_pool2d_stem"] = {
            "avg_launch_us": round(pavg * 1e3, 2), "value": round(pbytes / (pavg * 1e-3) / 1e9, 1), "unit": "GB/s",
            "roofline": {"bound": "hbm", "achieved": round(pbytes / (pavg * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBS,
                         "unit": "GB/s", "frac": round(pbytes / (pavg * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                         "traffic": None},
            "method": f"{2 * psets} launches over {psets} rotating inputs replayed in one HIP graph",
            "algorithmic_bytes_per_launch": pbytes}
        del pxs

        # ------------------------- convolutions off the 16-channel grid: an image network's first
        # layer (3 -> 64 channels, 7 x 7, stride 2, 224 x 224) and a depthwise layer (32 channels,
        # 3 x 3, 112 x 112), batch 32, through torch.ops.quantized.conv2d_relu
        def conv_line(name, ic, oc, k, stride, pad, groups, hw, what, op="conv2d_relu", batch=32):
            wf_ = torch.randn(oc, ic // groups, k, k) * 0.05
            wq_ = torch.quantize_per_channel(wf_, wf_.abs().amax(dim=(1, 2, 3)) / 127, torch.zeros(oc, dtype=torch.long),
                                             0, torch.qint8).to(dev)
            packed_ = torch.ops.quantized.conv2d_prepack(wq_, torch.randn(oc, device=dev), [stride, stride], [pad, pad],
                                                         [1, 1], groups)
            nsets = 6
            xqs_ = []
            for _ in range(nsets):
                xf_ = torch.relu(torch.randn(batch, ic, hw, hw, device=dev)).contiguous(memory_format=torch.channels_last)
                xqs_.append(torch.quantize_per_tensor(xf_, 0.03, 0, torch.quint8))
                del xf_
            cnt = [0]

            def one():
                cnt[0] += 1
                return getattr(torch.ops.quantized, op)(xqs_[cnt[0] % nsets], packed_, 0.05, 0)

            for _ in range(3):
                y_ = one()
            oh_ = y_.shape[2]
            g_ = torch.cuda.CUDAGraph()
            with torch.cuda.stream(side):
                one()
                side.synchronize()
                with torch.cuda.graph(g_, stream=side):
                    for _ in range(2 * nsets):
                        one()
            torch.cuda.synchronize()
            for _ in range(3):
                g_.replay()
            ts_ = events_ms(g_.replay, 10)
            avg_ = sum(ts_) / len(ts_) / (2 * nsets)
            nbytes_ = batch * hw * hw * ic + batch * oh_ * oh_ * oc + oc * (ic // groups) * k * k
            ops_ = 2 * batch * oh_ * oh_ * oc * (ic // groups) * k * k
            log(f"[bench] {what}: {avg_*1e3:.1f} us/launch in a replayed graph, {nbytes_/(avg_*1e-3)/1e9:.0f} GB/s, "
                f"{ops_/(avg_*1e-3)/1e12:.1f} TOP/s")
            secondary[name] = {
                "avg_launch_us": round(avg_ * 1e3, 2), "value": round(nbytes_ / (avg_ * 1e-3) / 1e9, 1), "unit": "GB/s",
                "roofline": {"bound": "hbm", "achieved": round(nbytes_ / (avg_ * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBS,
                             "unit": "GB/s", "frac": round(nbytes_ / (avg_ * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                             "traffic": None},
                "tops": round(ops_ / (avg_ * 1e-3) / 1e12, 2),
                "method": f"{what}; {2 * nsets} launches over {nsets} rotating inputs replayed in one HIP graph",
                "algorithmic_bytes_per_launch": nbytes_, "ops_per_launch": ops_}

        # ------------------------- every convolution of a ResNet-50 (53 layers, 23 distinct shapes), per
        # shape through the C ABI in a replayed graph over rotating inputs, summed with the shape's count:
        # what the layers of the operator cost next to one another at batch 32 and on a single image
        def conv_stack(shapes, batch):
            total_us, rows_, layers = 0.0, [], 0
            for ic, oc, k, st, hw, count, groups in shapes:
                g_ = cabi.conv_geom((batch, hw, hw, ic), (oc, k, k), (st, st), (k // 2, k // 2), (1, 1), groups)
                oh_, ow_ = cabi.conv_out_hw(g_)
                nbytes_ = batch * hw * hw * ic + batch * oh_ * ow_ * oc
                nsets = max(2, min(6, (600 << 20) // nbytes_))
                xs_ = [torch.randint(0, 256, (batch, hw, hw, ic), dtype=torch.uint8, device=dev) for _ in range(nsets)]
                pw_ = cabi.PackedConv2d(torch.randint(-127, 128, (oc, k, k, ic // groups), dtype=torch.int8, device=dev), g_)
                ws_, b_ = torch.rand(oc, device=dev) * 0.002 + 0.001, torch.randn(oc, device=dev)
                ys_ = [torch.empty((batch, oh_, ow_, oc), dtype=torch.uint8, device=dev) for _ in range(nsets)]

                def run_():
                    for x_, y_ in zip(xs_, ys_):
                        cabi.conv2d(x_, pw_, g_, 0.02, 0, ws_, b_, 0.05, 0, relu=True, out=y_)

                us_ = graph_us(run_, nsets)
                total_us += count * us_
                layers += count
                rows_.append({"ic": ic, "oc": oc, "k": k, "stride": st, "hw": hw, "groups": groups, "count": count,
                              "us": round(us_, 2)})
                del xs_, ys_, pw_
            return total_us, layers, rows_

        # (input channels, output channels, kernel, stride, image side, count, groups)
        resnet50 = [(3, 64, 7, 2, 224, 1), (64, 64, 1, 1, 56, 1), (64, 64, 3, 1, 56, 3), (64, 256, 1, 1, 56, 4),
                    (256, 64, 1, 1, 56, 2), (256, 128, 1, 1, 56, 1), (128, 128, 3, 2, 56, 1), (128, 512, 1, 1, 28, 4),
                    (256, 512, 1, 2, 56, 1), (512, 128, 1, 1, 28, 3), (128, 128, 3, 1, 28, 3), (512, 256, 1, 1, 28, 1),
                    (256, 256, 3, 2, 28, 1), (256, 1024, 1, 1, 14, 6), (512, 1024, 1, 2, 28, 1), (1024, 256, 1, 1, 14, 5),
                    (256, 256, 3, 1, 14, 5), (1024, 512, 1, 1, 14, 1), (512, 512, 3, 2, 14, 1), (512, 2048, 1, 1, 7, 3),
                    (1024, 2048, 1, 2, 14, 1), (2048, 512, 1, 1, 7, 2), (512, 512, 3, 1, 7, 2)]
        for batch_ in (32, 1):
            tot_, layers_, rows_ = conv_stack([sh + (1,) for sh in resnet50], batch_)
            log(f"[bench] ResNet-50 convolutions, batch {batch_}: {layers_} layers, {tot_:.0f} us in all "
                f"({tot_/layers_:.1f} us per layer)")
            secondary[f"conv2d_relu_resnet50_stack_b{batch_}"] = {
                "layers": layers_, "total_us": round(tot_, 1), "per_layer_us": round(tot_ / layers_, 2),
                "images_per_s_convs_only": round(batch_ / (tot_ * 1e-6), 1), "shapes": rows_,
                "method": "each distinct shape timed alone through tmq_conv2d (with ReLU; input and output zero point 0, "
                          "as tensors behind a ReLU have it) in a replayed HIP graph over rotating inputs, times its "
                          "count; 224 x 224 images, NHWC"}

        # ... and of a MobileNetV2 (52 layers, 30 distinct shapes: a 3-channel first layer, depthwise 3 x 3 layers
        # at both strides, pointwise layers whose channel counts -- 24, 144, 160, 320 -- are mostly off the 64 grid)
        dwl = lambda c, st, hw, count: (c, c, 3, st, hw, count, c)
        pwl = lambda ic, oc, hw, count: (ic, oc, 1, 1, hw, count, 1)
        mobilenet_v2 = [(3, 32, 3, 2, 224, 1, 1), dwl(32, 1, 112, 1), pwl(32, 16, 112, 1), pwl(16, 96, 112, 1),
                        dwl(96, 2, 112, 1), pwl(96, 24, 56, 1), pwl(24, 144, 56, 2), dwl(144, 1, 56, 1), pwl(144, 24, 56, 1),
                        dwl(144, 2, 56, 1), pwl(144, 32, 28, 1), pwl(32, 192, 28, 3), dwl(192, 1, 28, 2), pwl(192, 32, 28, 2),
                        dwl(192, 2, 28, 1), pwl(192, 64, 14, 1), pwl(64, 384, 14, 4), dwl(384, 1, 14, 4), pwl(384, 64, 14, 3),
                        pwl(384, 96, 14, 1), pwl(96, 576, 14, 3), dwl(576, 1, 14, 2), pwl(576, 96, 14, 2), dwl(576, 2, 14, 1),
                        pwl(576, 160, 7, 1), pwl(160, 960, 7, 3), dwl(960, 1, 7, 3), pwl(960, 160, 7, 2), pwl(960, 320, 7, 1),
                        pwl(320, 1280, 7, 1)]
        for batch_ in (32, 1):
            tot_, layers_, rows_ = conv_stack(mobilenet_v2, batch_)
            log(f"[bench] MobileNetV2 convolutions, batch {batch_}: {layers_} layers, {tot_:.0f} us in all "
                f"({tot_/layers_:.1f} us per layer)")
            secondary[f"conv2d_relu_mobilenet_v2_stack_b{batch_}"] = {
                "layers": layers_, "total_us": round(tot_, 1), "per_layer_us": round(tot_ / layers_, 2),
                "images_per_s_convs_only": round(batch_ / (tot_ * 1e-6), 1), "shapes": rows_,
                "method": "as the ResNet-50 stack"}

        conv_line("conv2d_relu_first_layer_7x7_s2_3to64", 3, 64, 7, 2, 3, 1, 224,
                  "conv2d_relu 7x7 stride 2, 3 -> 64 channels, [32,3,224,224]")
        conv_line("conv2d_relu_depthwise_3x3_32ch", 32, 32, 3, 1, 1, 32, 112,
                  "conv2d_relu depthwise 3x3, 32 channels, [32,32,112,112]")
        # the depthwise 7 x 7 of a ConvNeXt stage: 96 channels on 56 x 56
        conv_line("conv2d_depthwise_7x7_96ch", 96, 96, 7, 1, 3, 96, 56,
                  "conv2d depthwise 7x7, 96 channels, [32,96,56,56]", op="conv2d")
        # the fused SiLU form the reference adds for detectors: 32 -> 64 channels, 3 x 3 stride 2 on 320 x 320, batch 8
        conv_line("conv2d_silu_3x3_s2_32to64_320", 32, 64, 3, 2, 1, 1, 320,
                  "conv2d_silu 3x3 stride 2, 32 -> 64 channels, [8,32,320,320]", op="conv2d_silu", batch=8)

    # ------------------------------------------------------------ CPU baseline
    # The reference CPU path = PyTorch's own quantized CPU ops (fbgemm engine), timed on
    # this host's cores on bounded samples of the same workloads; the scalar C port of the
    # same arithmetic (the parity oracle) is reported next to it as `oracle_port`.
    cpu_baseline = None
    if not args.skip_cpu:
        import oracle

        cores = min(os.cpu_count() or 1, 16)
        cpu_model = "unknown"
        try:
            with open("/proc/cpuinfo") as f:
                for line in f:
                    if line.startswith("model name"):
                        cpu_model = line.split(":", 1)[1].strip()
                        break
        except OSError:
            pass
        torch.backends.quantized.engine = "fbgemm"

        def cpu_time(fn, min_s=0.5, max_reps=50):
            fn()
            reps, t0 = 0, time.perf_counter()
            while True:
                fn()
                reps += 1
                dt = time.perf_counter() - t0
                if dt >= min_s or reps >= max_reps:
                    return dt / reps

        xs_all = xq.int_repr().cpu()
        wq_cpu, bias_cpu = wq.cpu(), bias.cpu()
        p_cpu = torch.ops.quantized.linear_prepack(wq_cpu, bias_cpu)

        def cpu_linear_tops(rows, threads):
            torch.set_num_threads(threads)
            xs_q = torch._make_per_tensor_quantized_tensor(xs_all[:rows].contiguous(), xq.q_scale(),
                                                           xq.q_zero_point())
            dt_ = cpu_time(lambda: torch.ops.quantized.linear(xs_q, p_cpu, out_scale, out_zp), min_s=2.0)
            return 2.0 * rows * N * K / dt_ / 1e12, dt_

        log(f"[bench] CPU baseline on {cpu_model}, {cores} threads: torch.ops.quantized.linear (fbgemm), config 3")
        all_tops, all_dt = cpu_linear_tops(M, cores)
        one_rows = 256
        one_tops, one_dt = cpu_linear_tops(one_rows, 1)
        log(f"[bench]   {cores} threads: {all_tops:.3f} TOP/s ({all_dt*1e3:.0f} ms per call); "
            f"1 thread: {one_tops:.4f} TOP/s on {one_rows} rows")
        cpu_baseline = {"value": round(all_tops, 4), "unit": "TOP/s", "cores": cores, "kind": "reference",
                        "what": "torch.ops.quantized.linear on CPU tensors, engine fbgemm (the CPU ops the "
                                "north star names as the reference; the reference's own device code cannot be "
                                "built without the MUSA SDK)",
                        "cpu_model": cpu_model,
                        "sample": f"config 3 at full size (all {M} rows), {all_dt*1e3:.0f} ms per call, repeated "
                                  "for about 2 s",
                        "one_thread": {"value": round(one_tops, 5), "unit": "TOP/s", "cores": 1,
                                       "sample": f"first {one_rows} of {M} rows, {one_dt*1e3:.0f} ms per call"}}

        # the oracle (scalar C, OpenMP over rows) on a bounded sample, and the GPU against it
        rows = 512
        xs = xs_all[:rows].numpy()
        t0 = time.perf_counter()
        y_ref = oracle.linear(xs, xq.q_scale(), xq.q_zero_point(), wq.int_repr().cpu().numpy(), w_scales.cpu().numpy(),
                              bias_cpu.numpy(), out_scale, out_zp, nthreads=cores)
        dt = time.perf_counter() - t0
        got = torch.ops.quantized.linear(xq, packed, out_scale, out_zp).int_repr()[:rows].cpu().numpy()
        max_diff = int(np.abs(got.astype(np.int32) - y_ref.astype(np.int32)).max())
        y_cpu = torch.ops.quantized.linear(
            torch._make_per_tensor_quantized_tensor(xs_all[:rows].contiguous(), xq.q_scale(), xq.q_zero_point()),
            p_cpu, out_scale, out_zp).int_repr().numpy()
        max_diff_cpu_op = int(np.abs(got.astype(np.int32) - y_cpu.astype(np.int32)).max())
        log(f"[bench]   oracle port: {2.0 * rows * N * K / dt / 1e12 * 1e3:.1f} GOP/s; GPU vs oracle max diff "
            f"{max_diff} LSB, GPU vs the CPU op {max_diff_cpu_op} LSB on {rows} rows")
        cpu_baseline["oracle_port"] = {"value": round(2.0 * rows * N * K / dt / 1e12, 5), "unit": "TOP/s",
                                       "cores": cores, "kind": "port",
                                       "sample": f"first {rows} of {M} rows, {dt:.1f} s of CPU work"}
        cpu_baseline["gpu_vs_oracle_max_lsb"] = max_diff
        cpu_baseline["gpu_vs_cpu_op_max_lsb"] = max_diff_cpu_op
        del xs_all, p_cpu, wq_cpu

        # the other configurations on the CPU ops, all threads (extra information: a failure here
        # must not cost the benchmark line)
        try:
            torch.set_num_threads(cores)
            others = {}
            nc2 = 2 ** 26
            xc2 = torch.randn(nc2) * 3.0
            dtq = cpu_time(lambda: torch.quantize_per_tensor(xc2, 0.39, 128, torch.quint8))
            qc2 = torch.quantize_per_tensor(xc2, 0.39, 128, torch.quint8)
            dtd = cpu_time(lambda: qc2.dequantize())
            dtm = cpu_time(lambda: torch.aminmax(xc2))
            others["config2"] = {"sample": "2**26 of the 2**28 fp32 elements", "unit": "GB/s",
                                 "quantize_per_tensor": round(5 * nc2 / dtq / 1e9, 1),
                                 "dequantize": round(5 * nc2 / dtd / 1e9, 1),
                                 "aminmax": round(4 * nc2 / dtm / 1e9, 1)}
            del xc2, qc2
            wd = torch.randint(-127, 128, (4096, 4096), dtype=torch.int8)
            wdq = torch._make_per_channel_quantized_tensor(wd, torch.rand(4096, dtype=torch.float64) * 0.002 + 0.001,
                                                           torch.zeros(4096, dtype=torch.int64), 0)
            pd_cpu = torch.ops.quantized.linear_prepack(wdq, torch.randn(4096))
            dec = {}
            for Md in (1, 4, 16):
                xd_ = torch._make_per_tensor_quantized_tensor(torch.randint(0, 256, (Md, 4096), dtype=torch.uint8),
                                                              0.02, 128)
                dt_ = cpu_time(lambda: torch.ops.quantized.linear(xd_, pd_cpu, 0.05, 128), min_s=0.3, max_reps=2000)
                dec[f"m{Md}_us_per_call"] = round(dt_ * 1e6, 1)
            others["config4"] = dict(dec, sample="K = N = 4096, one weight (cache-warm on the CPU)")
            xc_ = torch._make_per_tensor_quantized_tensor(
                torch.randint(0, 120, (32, 56, 56, 64), dtype=torch.uint8).permute(0, 3, 1, 2), 0.03, 0)
            wc_ = torch._make_per_channel_quantized_tensor(
                torch.randint(-127, 128, (64, 3, 3, 64), dtype=torch.int8).permute(0, 3, 1, 2),
                torch.rand(64, dtype=torch.float64) * 0.002 + 0.001, torch.zeros(64, dtype=torch.int64), 0)
            pc_cpu = torch.ops.quantized.conv2d_prepack(wc_, torch.randn(64), [1, 1], [1, 1], [1, 1], 1)
            dtc = cpu_time(lambda: torch.ops.quantized.conv2d(xc_, pc_cpu, 0.05, 0))
            others["config5"] = {"sample": "full size, [32,56,56,64] x [64,3,3,64]", "us_per_call": round(dtc * 1e6, 1),
                                 "value": round(2.0 * 32 * 56 * 56 * 64 * 576 / dtc / 1e12, 4), "unit": "TOP/s"}
            log(f"[bench]   config 2 {others['config2']}; config 4 {dec}; config 5 {others['config5']['us_per_call']} us")
            cpu_baseline["other_configs"] = others
        except Exception as e:  # noqa: BLE001
            cpu_baseline["other_configs"] = {"error": str(e)[:200]}

    out = {
        "metric": "int8 quantized::linear TOPS (% MFMA peak) + quantize GB/s (% HBM), 1 GPU",
        "value": round(value, 2), "unit": "TOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "int8", "data": "synthetic",
        "config": {"workload": "quantized::linear prefill, BASELINE config 3: x quint8 [4096,4096] from N(0,1), "
                               "W qint8 per-channel [11008,4096] from N(0,0.02), fp32 bias, int32 accumulate, "
                               "quint8 output", "M": M, "K": K, "N": N,
                   "api": "torch.ops.quantized.linear on GPU tensors"},
        "roofline": roofline, "cpu_baseline": cpu_baseline, "secondary": secondary,
        "device": torch.cuda.get_device_name(0),
    }
    stop_power_sampler()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
