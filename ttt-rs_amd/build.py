"""Build the gfx950 shared library (libttt_mi355x.so) in-tree with hipcc.

Usage: python ttt-rs_amd/build.py   (or build_library() from Python)
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libttt_mi355x.so")
SOURCES = [os.path.join(HERE, "csrc", "ttt_api.hip")]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # keep the compiler from forming packed-f32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # let MFMA results live in ordinary VGPRs: the kernels consume them with VALU code right away,
    # and the default AGPR placement costs a v_accvgpr move per register and use
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",
]


def build_library(verbose: bool = False, extra_flags=()) -> str:
    """Compiles the library, then scans the gfx950 assembly the compiler produced on the way (isa_check.py: a
    matrix-instruction hazard the compiler does not guard and the hardware does not interlock).  The library is
    installed only if the scan is clean."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    os.makedirs(LIB_DIR, exist_ok=True)
    tmp = os.path.join(HERE, "build", "lib")   # intermediate files of the compilation land beside the output
    shutil.rmtree(tmp, ignore_errors=True)
    os.makedirs(tmp)
    out = os.path.join(tmp, os.path.basename(LIB_PATH))
    cmd = [hipcc, *HIPCC_FLAGS, *extra_flags, "-save-temps=obj", "-o", out, *SOURCES]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        sys.stderr.write(res.stdout + res.stderr)
        raise RuntimeError("hipcc failed building " + LIB_PATH)
    sys.path.insert(0, HERE)
    try:
        import isa_check
    finally:
        sys.path.pop(0)
    asm = [os.path.join(tmp, f) for f in os.listdir(tmp) if f.endswith("gfx950.s")]
    if not asm:
        raise RuntimeError("no gfx950 assembly found beside " + out + ": the hazard scan cannot run")
    for path in asm:
        bad = isa_check.check_file(path)
        if bad:
            for func, no, a, b, ws in bad[:20]:
                sys.stderr.write(f"{os.path.basename(path)}:{no}: in {func}: {ws} wait state(s) between\n    {a}\n    {b}\n")
            raise RuntimeError(f"{len(bad)} in-place accumulations onto a matrix instruction of another shape sit closer "
                               "than the hardware needs (see isa_check.py); library not installed")
        sel = isa_check.check_scc_select_file(path)
        if sel:
            for func, no, a, b in sel[:20]:
                sys.stderr.write(f"{os.path.basename(path)}:{no}: in {func}: scalar select on a vector comparison\n    {a}\n    {b}\n")
            raise RuntimeError(f"{len(sel)} s_cselect instruction(s) read a condition code that the comparison in front "
                               "of them does not set (see isa_check.py); library not installed")
    shutil.copyfile(out, LIB_PATH)
    shutil.copymode(out, LIB_PATH)
    shutil.rmtree(os.path.join(HERE, "build"), ignore_errors=True)
    if verbose:
        # the host pass does not know the gfx950 feature flag and says so; drop that noise
        for line in (res.stdout + res.stderr).splitlines():
            if "packed-fp32-ops" not in line:
                print(line)
    return LIB_PATH


DRIVER_PATH = os.path.join(LIB_DIR, "libttt_host_driver.so")


def build_host_driver() -> str:
    """The C++ host classes (host/*.hpp) behind C entry points, for the GPU test that drives them;
    plain host code (g++), linked against the library."""
    cmd = ["g++", "-std=c++17", "-O2", "-Wall", "-Wextra", "-Werror", "-fPIC", "-shared",
           os.path.join(HERE, "host", "host_driver.cpp"), "-o", DRIVER_PATH,
           "-L", LIB_DIR, "-lttt_mi355x", "-Wl,-rpath,$ORIGIN"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        sys.stderr.write(res.stdout + res.stderr)
        raise RuntimeError("g++ failed building " + DRIVER_PATH)
    return DRIVER_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
    print(build_host_driver())
