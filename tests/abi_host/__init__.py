"""A host program in plain C over the C ABI (`conv_host.c`) and the recipe that compiles it."""

import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
LIB_DIR = os.path.join(ROOT, "e3j_amd", "lib")
BINARY = os.path.join(LIB_DIR, "conv_host")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")


def build() -> str:
    """gcc -std=c99: the program needs no C++ and no hipcc, only the HIP runtime's C API."""
    cmd = ["gcc", "-std=c99", "-O2", "-Wall", "-Wextra", "-Werror", "-D__HIP_PLATFORM_AMD__",
           f"-I{ROCM}/include", f"-I{os.path.join(ROOT, 'include')}", os.path.join(HERE, "conv_host.c"),
           "-o", BINARY, f"-L{LIB_DIR}", "-le3j_amd", f"-L{ROCM}/lib", "-lamdhip64",
           "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{ROCM}/lib"]
    subprocess.run(cmd, check=True)
    return BINARY


def binary() -> str:
    """The built program; compiled again when the header or the source is newer than it (a
    program built against an older layout of the parameter structs would pass garbage)."""
    sources = (os.path.join(ROOT, "include", "e3j_amd.h"), os.path.join(HERE, "conv_host.c"))
    if not os.path.exists(BINARY) or any(os.path.getmtime(s) > os.path.getmtime(BINARY) for s in sources):
        return build()
    return BINARY
