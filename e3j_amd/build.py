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


# Sources whose kernels hold DPP instructions written as inline assembly.  The compiler's hazard
# pass does not look inside inline assembly, so the build reads the assembly it wrote for them.
DPP_ASM_SOURCES = ("conv_planned.hip", "conv_planned_f16.hip")
# The planned kernels' loop over blocks of 16 output coordinates is past the compiler's size limit
# for `#pragma unroll` in the largest instantiations; unrolled, the per-block numbers of the plan
# become compile-time lane indices (120k edges, K=128, l<=3: backward 4.12 -> 3.98 ms).
EXTRA_FLAGS = {name: ["-mllvm", "-pragma-unroll-threshold=100000"] for name in DPP_ASM_SOURCES}


def dpp_read_hazards(assembly: str) -> list[str]:
    """The inline `v_fmac_f32_dpp` instructions of an assembly listing whose DPP operand (the first
    source) was written by a vector instruction fewer than two wait states before: on gfx9 the
    hardware does not wait for that, and the kernels are written so that the operand always
    comes from an LDS read.  Returns one line of text per violation (none expected)."""
    import re

    def vgprs(token: str) -> set[int]:
        m = re.match(r"v\[(\d+):(\d+)\]", token)
        if m:
            return set(range(int(m.group(1)), int(m.group(2)) + 1))
        m = re.match(r"v(\d+)$", token)
        return {int(m.group(1))} if m else set()

    lines = [line.strip() for line in assembly.splitlines()]
    lines = [line for line in lines if line and not line.startswith((";", ".", "//")) and not line.endswith(":")]
    found = []
    for i, line in enumerate(lines):
        if not line.startswith("v_fmac_f32_dpp"):
            continue
        operands = [o.strip() for o in line.split(None, 1)[1].split(",")]
        source = vgprs(operands[1].split()[0])
        states = 0
        for before in reversed(lines[max(i - 3, 0):i]):
            if states >= 2:
                break
            if before.startswith("s_nop"):
                states += int(before.split()[1]) + 1
                continue
            if before.startswith("v_") and not before.startswith(("v_readlane", "v_readfirstlane", "v_cmp")):
                written = vgprs(before.split(None, 1)[1].split(",")[0].strip())
                if written & source:
                    found.append(f"{before}  ->  {line}")
            states += 1
    return found


def _compile_one(src: str, extra: list[str]) -> str:
    rel = os.path.relpath(src, CSRC).replace(os.sep, "_")
    obj = os.path.join(OBJ_DIR, os.path.splitext(rel)[0] + ".o")
    check_dpp = os.path.basename(src) in DPP_ASM_SOURCES
    keep_temps = "-save-temps=obj" in extra
    extra = [*extra, *EXTRA_FLAGS.get(os.path.basename(src), [])]
    if check_dpp and not keep_temps:
        extra = [*extra, "-save-temps=obj"]
    cmd = [HIPCC, *COMMON_FLAGS, *extra, "-c", src, "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{' '.join(cmd)}\n{proc.stdout}\n{proc.stderr}")
    if check_dpp:
        listing = os.path.join(OBJ_DIR, f"{os.path.splitext(rel)[0]}-hip-amdgcn-amd-amdhsa-{ARCH}.s")
        with open(listing) as f:
            hazards = dpp_read_hazards(f.read())
        if not keep_temps:  # (the listing came with the compiler's other intermediate files)
            stem = os.path.join(OBJ_DIR, os.path.splitext(rel)[0])
            for path in glob.glob(stem + "-h*") + glob.glob(stem + ".hip-*"):
                os.remove(path)
        if hazards:
            raise RuntimeError(f"{src}: a DPP operand is read too soon after a vector write:\n" + "\n".join(hazards[:10]))
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
