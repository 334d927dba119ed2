"""Builds libwallx_mi355.so (the C-ABI library) for gfx950 with hipcc.

    python wall-x_amd/csrc/build.py [--force] [--no-probe]

Sources are compiled one by one (objects under csrc/build/) and linked into
wall-x_amd/wallx_mi355/libwallx_mi355.so, next to the Python package that loads it.  The benchmark's MFMA rate
probe (probe.hip) goes into a library of its own, libwallx_probe.so, beside it.
"""

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
REPO = os.path.dirname(os.path.dirname(HERE))
INCLUDE = os.path.join(REPO, "include")
OUT_DIR = os.path.join(os.path.dirname(HERE), "wallx_mi355")
LIB = os.path.join(OUT_DIR, "libwallx_mi355.so")
OBJ_DIR = os.path.join(HERE, "build")

SOURCES = ["common.hip", "partition.hip", "dual_gemm.hip", "mrope.hip", "rope_index.hip", "vision_index.hip",
           "fused_movers.hip", "swiglu_bwd.hip"]
HEADERS = ["common.h", "grid_prefix.h", "tiled_layout.h", os.path.join(INCLUDE, "wallx_mi355.h")]
# benchmark-only MFMA rate probe: its own library, not part of the product library or its ABI
PROBE_SOURCE = "probe.hip"
PROBE_LIB = os.path.join(OUT_DIR, "libwallx_probe.so")

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    # packed fp32 math is kept off for every kernel in this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # no implicit fused multiply-add: the elementwise kernels reproduce eager mul-then-add rounding exactly
    "-ffp-contract=off",
    "-Wno-unused-command-line-argument",
    f"-I{INCLUDE}", f"-I{HERE}",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libwallx_mi355.so cannot be built")
    return exe


def _newer(target: str, deps) -> bool:
    if not os.path.exists(target):
        return False
    t = os.path.getmtime(target)
    return all(os.path.getmtime(d) <= t for d in deps)


# The large-tile GEMM kernels use every register a wave can have; a small source change can push values of the K
# loop into scratch memory, which costs a factor of three and shows in no test.  Their compile prints the
# resource-usage remarks and this limit on "ScratchSize [bytes/lane]" turns a spill into a loud warning.
# (Values that are only live outside the K loop do spill: up to 52 bytes in the tiled kernels and 88 in the
# large-tile variants with K-major operands, all measured at full speed.)
RESOURCE_CHECKED = {"dual_gemm.hip": ("dual_gemm_kernel", 96)}


def _check_resources(src, stderr):
    name_part, limit = RESOURCE_CHECKED[src]
    current = None
    for line in stderr.splitlines():
        if "Function Name:" in line:
            current = line.split("Function Name:")[1].split()[0]
        elif "ScratchSize [bytes/lane]:" in line and current and name_part in current:
            size = int(line.split("ScratchSize [bytes/lane]:")[1].split()[0])
            if size > limit:
                sys.stderr.write(f"[wallx_mi355] WARNING: {current} spills {size} bytes per lane to scratch "
                                 f"(limit {limit}): check that no spill sits inside the K loop\n")


def _run(cmd):
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = ("is not a recognized feature for this target", "-Rpass-analysis=kernel-resource-usage")
    src = os.path.basename(cmd[-3]) if len(cmd) > 3 else ""
    if proc.returncode == 0 and src in RESOURCE_CHECKED:
        _check_resources(src, proc.stderr)
    err = "\n".join(line for line in proc.stderr.splitlines() if not any(n in line for n in noise))
    if proc.returncode != 0:
        raise RuntimeError(f"command failed: {' '.join(cmd)}\n{proc.stdout}\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")


def build_probe(force: bool = False, verbose: bool = True) -> str:
    hipcc = _hipcc()
    path = os.path.join(HERE, PROBE_SOURCE)
    if force or not _newer(PROBE_LIB, [path]):
        _run([hipcc] + FLAGS + ["-shared", path, "-o", PROBE_LIB])
        if verbose:
            print(f"[wallx_mi355] built {PROBE_LIB}", flush=True)
    return PROBE_LIB


def build(force: bool = False, verbose: bool = True, probe: bool = True) -> str:
    hipcc = _hipcc()
    os.makedirs(OBJ_DIR, exist_ok=True)
    headers = [h if os.path.isabs(h) else os.path.join(HERE, h) for h in HEADERS]
    objs, jobs = [], []
    for src in SOURCES:
        path = os.path.join(HERE, src)
        obj = os.path.join(OBJ_DIR, src.replace(".hip", ".o"))
        objs.append(obj)
        if force or not _newer(obj, [path] + headers):
            extra = ["-Rpass-analysis=kernel-resource-usage", "-fno-caret-diagnostics"] if src in RESOURCE_CHECKED else []
            jobs.append([hipcc] + FLAGS + extra + ["-c", path, "-o", obj])
    if jobs:
        if verbose:
            print(f"[wallx_mi355] compiling {len(jobs)} source(s) for gfx950", flush=True)
        with ThreadPoolExecutor(max_workers=min(len(jobs), 6)) as pool:
            list(pool.map(_run, jobs))
    if jobs or force or not _newer(LIB, objs):
        _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs)
        if verbose:
            print(f"[wallx_mi355] linked {LIB}", flush=True)
    if probe:
        build_probe(force, verbose)
    return LIB


if __name__ == "__main__":
    build(force="--force" in sys.argv, probe="--no-probe" not in sys.argv)
