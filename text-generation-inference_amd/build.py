"""Build recipe for libq4linear.so (hipcc, gfx950 only) and for the benchmark's two side libraries.

libq4linear.so           the product: every kernel and the C ABI of include/q4_linear.h
libq4probe.so            read-only / LDS probe kernels of bench.py (csrc/bench/q4_probe.hip)
libq4linear_stamps.so    the product's sources with -DQ4_PHASE_STAMPS: the decode kernels also leave
                         clock readings per wave and phase (bench.py --phase-breakdown)
All three are built in-tree next to this file so that they travel with the source tree.
Run as a script (`python build.py`) or call build_all().
"""

from __future__ import annotations

import os
import subprocess
import sys
from pathlib import Path

HERE = Path(__file__).resolve().parent
ROOT = HERE.parent
CSRC = HERE / "csrc"
LIB_NAME = "libq4linear.so"
LIB_PATH = HERE / LIB_NAME

SOURCES = ["q4_api.hip", "q4_dequant.hip", "q4_generic.hip", "q4_gemv.hip", "q4_gemv_lean.hip", "q4_gemv_direct.hip", "q4_gemv_awq.hip", "q4_gemv_gate_up.hip", "q4_gemm.hip", "q4_gemm_awq.hip", "q4_gemm_awq_direct.hip", "q4_act_mul.hip", "q4_moe.hip", "q4_sequential.hip", "q4_gptq_solve.hip"]
# translation units that see the decode kernels' parameter block (recompiled for the stamps build)
STAMP_SOURCES = ["q4_gemv.hip", "q4_gemv_lean.hip", "q4_gemv_direct.hip", "q4_gemv_direct.hip", "q4_gemv_awq.hip", "q4_gemv_gate_up.hip", "q4_moe.hip"]
PROBE_LIB_PATH = HERE / "libq4probe.so"
STAMPS_LIB_PATH = HERE / "libq4linear_stamps.so"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wall",
    "-Wno-unused-function",
    # never let the compiler form packed-fp32 VALU ops from float code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    f"-I{ROOT / 'include'}",
    f"-I{CSRC}",
]


def build_library(verbose: bool = False, extra_flags: list[str] | None = None,
                  only: list[str] | None = None) -> Path:
    """Compile every kernel translation unit and link the shared library.

    `only` (development aid) recompiles just the named sources and links them with the
    objects a previous full build left in build/."""
    objs = []
    procs = []
    build_dir = HERE / "build"
    build_dir.mkdir(exist_ok=True)
    flags = FLAGS + (extra_flags or [])
    for src in SOURCES:
        obj = build_dir / (Path(src).stem + ".o")
        objs.append(str(obj))
        if only and src not in only and obj.exists():
            continue
        cmd = [HIPCC, *flags, "-c", str(CSRC / src), "-o", str(obj)]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    failed = False
    for src, proc in procs:
        out, _ = proc.communicate()
        lines = [l for l in out.splitlines() if "is not a recognized feature for this target" not in l]
        if proc.returncode != 0:
            failed = True
            print(f"[build] {src} FAILED\n" + "\n".join(lines), file=sys.stderr)
        elif lines and verbose:
            print("\n".join(lines))
    if failed:
        raise RuntimeError("hipcc failed")
    tmp = LIB_PATH.with_suffix(".so.tmp")
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", str(tmp)]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


def _compile(jobs, verbose):
    """jobs: (label, command) pairs run side by side; raises when one fails."""
    procs = [(label, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)) for label, cmd in jobs]
    failed = False
    for label, proc in procs:
        out, _ = proc.communicate()
        lines = [l for l in out.splitlines() if "is not a recognized feature for this target" not in l]
        if proc.returncode != 0:
            failed = True
            print(f"[build] {label} FAILED\n" + "\n".join(lines), file=sys.stderr)
        elif lines and verbose:
            print("\n".join(lines))
    if failed:
        raise RuntimeError("hipcc failed")


def _link(objs, path, verbose):
    tmp = path.with_suffix(".so.tmp")
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", str(tmp)]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    os.replace(tmp, path)
    return path


def build_bench_libraries(verbose: bool = False) -> list[Path]:
    """The benchmark's side libraries: the probe kernels, and the product's objects with the decode
    translation units recompiled under -DQ4_PHASE_STAMPS (needs the objects of build_library())."""
    build_dir = HERE / "build"
    stamps_dir = build_dir / "stamps"
    stamps_dir.mkdir(parents=True, exist_ok=True)
    probe_obj = build_dir / "q4_probe.o"
    jobs = [("bench/q4_probe.hip", [HIPCC, *FLAGS, "-c", str(CSRC / "bench" / "q4_probe.hip"), "-o", str(probe_obj)])]
    objs = []
    for src in SOURCES:
        if src in STAMP_SOURCES:
            obj = stamps_dir / (Path(src).stem + ".o")
            jobs.append((src + " (stamps)", [HIPCC, *FLAGS, "-DQ4_PHASE_STAMPS", "-c", str(CSRC / src), "-o", str(obj)]))
        else:
            obj = build_dir / (Path(src).stem + ".o")
        objs.append(str(obj))
    _compile(jobs, verbose)
    return [_link([str(probe_obj)], PROBE_LIB_PATH, verbose), _link(objs, STAMPS_LIB_PATH, verbose)]


def build_all(verbose: bool = False) -> list[Path]:
    return [build_library(verbose=verbose)] + build_bench_libraries(verbose=verbose)


if __name__ == "__main__":
    if sys.argv[1:]:
        print(build_library(verbose=True, only=sys.argv[1:]))
    else:
        print(build_all(verbose=True))
