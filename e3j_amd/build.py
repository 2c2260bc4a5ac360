"""Build `libe3j_amd.so` for gfx950 with hipcc, in-tree.

`python -m e3j_amd.build` regenerates the compile-time-unrolled kernel sources
(`e3j_amd/codegen/gen_conv.py`) and compiles every `.hip` under `e3j_amd/csrc/`
(one object per source, in parallel) into `e3j_amd/lib/libe3j_amd.so`.
hipcc cross-compiles, so no GPU is needed.  Takes the place of the reference's
CMake/nvcc build of `e3j_ops` (`lib/e3j_ops/CMakeLists.txt:10-50`).
"""

from __future__ import annotations

import concurrent.futures
import glob
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
GENERATED = os.path.join(CSRC, "generated")
OBJ_DIR = os.path.join(HERE, "lib", "obj")
LIB_PATH = os.path.join(HERE, "lib", "libe3j_amd.so")

HIPCC = os.environ.get("HIPCC", shutil.which("hipcc") or "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
# Packed-FP32 VALU forms are switched off for every translation unit.
COMMON_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-munsafe-fp-atomics",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
]


def _compile_one(src: str, extra: list[str]) -> str:
    rel = os.path.relpath(src, CSRC).replace(os.sep, "_")
    obj = os.path.join(OBJ_DIR, os.path.splitext(rel)[0] + ".o")
    cmd = [HIPCC, *COMMON_FLAGS, *extra, "-c", src, "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{' '.join(cmd)}\n{proc.stdout}\n{proc.stderr}")
    return obj


def sources() -> list[str]:
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")) + glob.glob(os.path.join(GENERATED, "*.hip")))


def build(regenerate: bool = True, jobs: int | None = None, verbose: bool = True,
          save_temps: bool = False) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(GENERATED, exist_ok=True)
    if regenerate:
        from .codegen import gen_conv, gen_tp
        gen_conv.write_all(GENERATED)
        gen_tp.write_all(GENERATED)
    srcs = sources()
    extra = ["-save-temps=obj"] if save_temps else []
    jobs = jobs or min(8, os.cpu_count() or 1)
    if verbose:
        print(f"[e3j_amd.build] compiling {len(srcs)} sources for {ARCH} with {jobs} jobs", flush=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(lambda s: _compile_one(s, extra), srcs))
    cmd = [HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", LIB_PATH + ".tmp", *objs]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stdout}\n{proc.stderr}")
    os.replace(LIB_PATH + ".tmp", LIB_PATH)
    if verbose:
        print(f"[e3j_amd.build] wrote {LIB_PATH}", flush=True)
    return LIB_PATH


if __name__ == "__main__":
    build(regenerate="--no-codegen" not in sys.argv, save_temps="--save-temps" in sys.argv)
