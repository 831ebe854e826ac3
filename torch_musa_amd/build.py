"""Builds the native libraries in-tree with hipcc (cross-compiles without a GPU).

  libtmq.so       torch-free HIP kernel library behind include/tmq.h
  libtmq_bench.so measurement probe behind include/tmq_bench.h (bench.py only)
  libtmq_aten.so  ATen registrations (TORCH_LIBRARY_IMPL + dispatch stubs)
                  that call libtmq.so

    python torch_musa_amd/build.py [--kernels-only] [--verbose]

Run it as a script (not with -m): importing the package loads the libraries
this script is about to produce.
"""
from __future__ import annotations

import argparse
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
OBJ = os.path.join(PKG, "build")
LIB_KERNELS = os.path.join(PKG, "libtmq.so")
LIB_ATEN = os.path.join(PKG, "libtmq_aten.so")
LIB_BENCH = os.path.join(PKG, "libtmq_bench.so")
ARCH = "gfx950"

KERNEL_SOURCES = ["kernels/quantize.hip", "kernels/linear.hip", "kernels/conv2d.hip",
                  "kernels/elementwise.hip"]
BENCH_SOURCES = ["bench/bench_kernels.hip"]
ATEN_SOURCES = ["aten/register.cpp"]

# -ffp-contract=off: the requantisation epilogue and the quantizer must round
# after every fp32 operation, as the CPU ops they mirror do.
# packed-fp32-ops disabled: never emit v_pk_{add,mul,fma}_f32.
# amdgpu-kernarg-preload-count: the leading scalar arguments of a kernel (up to
# 14 dwords) reach its waves in SGPRs at launch instead of through a read of the
# argument buffer; the latency-bound kernels put what their first loads need there.
DEVICE_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-ffp-contract=off", "-fPIC",
    "-fvisibility=hidden", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-mllvm", "-amdgpu-kernarg-preload-count=14",
    "-Wno-unused-command-line-argument",
]


# Kernels whose loads are asm statements with hand-counted waits: a fragment that the
# compiler moved to scratch memory would be copied before its load has landed, so the
# build fails if any of them uses scratch (the compiler reports each kernel's resources).
NO_SCRATCH_KERNELS = ("gemm_i8_wring_kernel",)
RESOURCE_REMARKS = ["-Rpass-analysis=kernel-resource-usage", "-save-temps=obj"]
# The same kernels, on the assembly of the same compilation: besides the request itself and the
# matrix instruction that consumes a fragment, nothing in the generated code may touch a fragment's
# registers once the request for them is out (a copy the register allocator placed between a
# request and its wait would move stale data).
IN_FLIGHT_KERNELS = ("gemm_i8_wring_kernel",)
# Kernels that wait for their copies into LDS with a literal count of the weight loads issued after them.
COUNTED_LOAD_KERNELS = ("gemm_i8_wstream_kernel",)


def _needs_register_check(obj):
    return os.path.basename(obj) == "linear.hip.o"


def _check_no_scratch(remarks, kernels):
    name, seen = None, set()
    for line in remarks.splitlines():
        if "Function Name:" in line:
            name = line.split("Function Name:", 1)[1].split()[0]
        elif "ScratchSize [bytes/lane]:" in line and name is not None:
            for k in kernels:
                if k in name:
                    seen.add(k)
                    size = int(line.split("ScratchSize [bytes/lane]:", 1)[1].split()[0])
                    if size != 0:
                        raise RuntimeError(f"{name} uses {size} bytes of scratch per lane: its asm loads "
                                           "must stay in registers")
    missing = set(kernels) - seen
    if missing:
        raise RuntimeError(f"no resource report for {sorted(missing)}: the register check did not run")


def _vgprs(operand_text):
    """VGPR numbers named in an operand list: v7, v[8:11]."""
    import re
    regs = set()
    for m in re.finditer(r"\bv\[(\d+):(\d+)\]|\bv(\d+)\b", operand_text):
        if m.group(3) is not None:
            regs.add(int(m.group(3)))
        else:
            regs.update(range(int(m.group(1)), int(m.group(2)) + 1))
    return regs


def _check_in_flight_registers(asm_path, kernels):
    import re
    request = re.compile(r"^\s*global_load_dwordx4\s+(v\[\d+:\d+\]),\s*v\d+,\s*s\[\d+:\d+\]")
    text = open(asm_path).read().split("\n")
    seen = set()
    name, body = None, []
    def check(name, body):
        pending = {}                                # register -> line of the request that is on its way
        requests = 0
        for i, line in enumerate(body):
            code = line.split(";")[0].strip()
            if not code or code.endswith(":") or code.startswith("."):
                continue
            m = request.match(line)
            if m:
                requests += 1
                for r in _vgprs(m.group(1)):
                    pending[r] = i
                continue
            touched = _vgprs(code) & pending.keys()
            if not touched:
                continue
            if code.startswith("v_mfma_"):
                ops = code.split(None, 1)[1].split(",")
                # a fragment is consumed as the first source operand, behind a wait for the requests;
                # its registers are free again from there on
                if touched - _vgprs(ops[1]):
                    raise RuntimeError(f"{name}: a v_mfma touches a fragment on its way other than as its first "
                                       f"source (registers {sorted(touched - _vgprs(ops[1]))}): {code}")
                if not any("s_waitcnt vmcnt" in b for b in body[max(pending[r] for r in touched):i]):
                    raise RuntimeError(f"{name}: no wait between a fragment's request and {code}")
                for r in touched:
                    del pending[r]
                continue
            raise RuntimeError(f"{name}: an instruction other than the request and the consuming v_mfma touches a "
                               f"fragment on its way (registers {sorted(touched)}, requested at line "
                               f"{min(pending[r] for r in touched)} of the kernel): {code}")
        if requests == 0:
            raise RuntimeError(f"{name}: no fragment requests found: the in-flight register check did not run")
    for line in text:
        m = re.match(r"^(_Z\w+):", line)
        if m:
            name, body = m.group(1), []
            continue
        if name is not None:
            body.append(line)
            if "s_endpgm" in line:
                for k in kernels:
                    if k in name:
                        check(name, body)
                        seen.add(k)
                name = None
    missing = set(kernels) - seen
    if missing:
        raise RuntimeError(f"no assembly for {sorted(missing)}: the in-flight register check did not run")


def _check_counted_loads(asm_path, kernels):
    """Kernels whose copies into LDS are waited for with a literal `s_waitcnt vmcnt(N)` that counts on N
    younger weight loads: the compiler must have emitted at least N loads between the last copy and the wait."""
    import re
    text = open(asm_path).read().split("\n")
    seen = set()
    name, body = None, []
    for line in text:
        m = re.match(r"^(_Z\w+):", line)
        if m:
            name, body = m.group(1), []
            continue
        if name is None:
            continue
        body.append(line)
        if "s_endpgm" not in line:
            continue
        for k in kernels:
            if k not in name:
                continue
            copies = [i for i, b in enumerate(body) if "global_load_lds_dwordx4" in b]
            waits = [(i, int(re.search(r"vmcnt\((\d+)\)", b).group(1))) for i, b in enumerate(body)
                     if i > 0 and "#ASMSTART" in body[i - 1] and re.search(r"s_waitcnt vmcnt\(\d+\)", b)]
            if not copies or not waits:
                raise RuntimeError(f"{name}: copies or their wait not found: the load count check did not run")
            wait_line, counted = next(((i, n) for i, n in waits if i > copies[-1]), (None, None))
            if wait_line is None:
                raise RuntimeError(f"{name}: no wait behind the last copy into LDS")
            loads = sum(1 for b in body[copies[-1]:wait_line]
                        if re.match(r"^\s*global_load_dwordx4\s", b) and "lds" not in b)
            if loads < counted:
                raise RuntimeError(f"{name}: vmcnt({counted}) behind the copies counts on {counted} younger loads, "
                                   f"the compiler emitted {loads}")
            seen.add(k)
        name = None
    missing = set(kernels) - seen
    if missing:
        raise RuntimeError(f"no assembly for {sorted(missing)}: the load count check did not run")


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in p.stdout.splitlines()
                    if "is not a recognized feature for this target" not in l)
    if p.returncode != 0:
        raise RuntimeError(f"command failed ({p.returncode}): {' '.join(cmd)}\n{out}")
    if verbose and out.strip():
        print(out, flush=True)
    return out


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def build_kernels(verbose=False):
    return _build_hip_library(KERNEL_SOURCES, LIB_KERNELS, verbose)


def build_bench(verbose=False):
    return _build_hip_library(BENCH_SOURCES, LIB_BENCH, verbose)


def _build_hip_library(sources, lib_path, verbose):
    os.makedirs(OBJ, exist_ok=True)
    hipcc = _hipcc()
    inc = ["-I", os.path.join(ROOT, "include"), "-I", os.path.join(CSRC, "kernels")]
    jobs = []
    for src in sources:
        path = os.path.join(CSRC, src)
        if not os.path.exists(path):
            continue
        obj = os.path.join(OBJ, os.path.basename(src) + ".o")
        jobs.append((obj, [hipcc] + DEVICE_FLAGS + inc + ["-c", path, "-o", obj]))
    with ThreadPoolExecutor(max_workers=min(8, len(jobs))) as ex:
        outs = list(ex.map(lambda j: _run(j[1] + (RESOURCE_REMARKS if _needs_register_check(j[0]) else []),
                                          verbose and not _needs_register_check(j[0])), jobs))
    for (obj, _), out in zip(jobs, outs):
        if _needs_register_check(obj):
            _check_no_scratch(out, NO_SCRATCH_KERNELS)
            stem = os.path.basename(obj).split(".")[0]
            temps = [f for f in os.listdir(OBJ) if f.startswith(stem + "-") or f.startswith(stem + ".hip-")]
            asm = [f for f in temps if f.endswith(f"{ARCH}.s")]
            if len(asm) != 1:
                raise RuntimeError(f"expected one device assembly file for {stem}, found {asm}")
            try:
                _check_in_flight_registers(os.path.join(OBJ, asm[0]), IN_FLIGHT_KERNELS)
                _check_counted_loads(os.path.join(OBJ, asm[0]), COUNTED_LOAD_KERNELS)
            finally:
                for f in temps:                      # tens of MB of intermediates: not part of the build's output
                    os.remove(os.path.join(OBJ, f))
    _run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", lib_path]
         + [j[0] for j in jobs], verbose)
    return lib_path


def build_aten(verbose=False):
    import torch
    from torch.utils import cpp_extension as ce

    os.makedirs(OBJ, exist_ok=True)
    hipcc = _hipcc()
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    inc = []
    for d in ce.include_paths("cuda") if hasattr(ce, "include_paths") else []:
        inc += ["-isystem", d]
    inc += ["-I", os.path.join(ROOT, "include")]
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    objs = []
    for src in ATEN_SOURCES:
        path = os.path.join(CSRC, src)
        obj = os.path.join(OBJ, os.path.basename(src) + ".o")
        _run([hipcc, "-x", "hip", f"--offload-arch={ARCH}", "-O2", "-std=c++17", "-fPIC",
              "-fvisibility=hidden", f"-D_GLIBCXX_USE_CXX11_ABI={abi}", "-DUSE_ROCM",
              "-D__HIP_PLATFORM_AMD__=1", "-Wno-unused-command-line-argument",
              "-Wno-deprecated-declarations"] + inc + ["-c", path, "-o", obj], verbose)
        objs.append(obj)
    _run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", LIB_ATEN] + objs
         + ["-L", PKG, "-ltmq", "-L", tlib, "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-lc10",
            "-lc10_hip", "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{tlib}"], verbose)
    return LIB_ATEN


def build_all(verbose=False, kernels_only=False):
    out = [build_kernels(verbose), build_bench(verbose)]
    if not kernels_only and all(os.path.exists(os.path.join(CSRC, s)) for s in ATEN_SOURCES):
        out.append(build_aten(verbose))
    return out


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--kernels-only", action="store_true")
    ap.add_argument("--verbose", action="store_true")
    a = ap.parse_args()
    for lib in build_all(a.verbose, a.kernels_only):
        print("built", lib, os.path.getsize(lib), "bytes")
    sys.exit(0)
