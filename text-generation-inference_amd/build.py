"""Build recipe for libq4linear.so (hipcc, gfx950 only).

The library is built in-tree next to this file so that it travels with the source tree.
Run as a script (`python build.py`) or call build_library().
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

SOURCES = ["q4_api.hip", "q4_dequant.hip", "q4_generic.hip", "q4_gemv.hip", "q4_gemv_lean.hip", "q4_gemv_awq.hip", "q4_gemv_gate_up.hip", "q4_gemm.hip", "q4_gemm_awq.hip", "q4_gemm_awq_direct.hip", "q4_act_mul.hip", "q4_moe.hip", "q4_sequential.hip", "q4_gptq_solve.hip", "q4_probe.hip"]

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


if __name__ == "__main__":
    print(build_library(verbose=True, only=sys.argv[1:] or None))
