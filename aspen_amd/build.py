"""Builds the C-ABI shared library ``aspen_amd/libaspen_amd.so`` in tree.

Host side: C (gcc) -- aspen_amd/csrc/host/*.c, the library behind include/aspen.h.
Device side: HIP for gfx950 (hipcc) -- aspen_amd/csrc/hip/engine.hip, behind include/aspen_hip.h.
"""
from __future__ import annotations

import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
LIB = os.path.join(HERE, "libaspen_amd.so")
OBJ = os.path.join(HERE, "csrc", "_obj")

HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-Wno-unused-command-line-argument"]
C_FLAGS = ["-O2", "-fPIC", "-std=gnu11", "-Wall", "-Wextra", "-Wno-unused-parameter"]


def _run(cmd):
    print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def build(verbose: bool = True, extra_hip_flags=(), lib_path: str = LIB, obj_dir: str = OBJ) -> str:
    """Compiles the host C files and the HIP file and links them; extra_hip_flags / lib_path / obj_dir
    let an experiment build a differently configured copy next to the product library."""
    OBJ, LIB = obj_dir, lib_path
    os.makedirs(OBJ, exist_ok=True)
    inc = ["-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(HERE, "csrc", "hip"),
           "-I" + os.path.join(HERE, "csrc", "host")]
    objs = []
    for src in sorted(glob.glob(os.path.join(HERE, "csrc", "host", "*.c"))):
        o = os.path.join(OBJ, os.path.basename(src)[:-2] + ".o")
        _run(["gcc"] + C_FLAGS + inc + ["-c", src, "-o", o])
        objs.append(o)
    for src in sorted(glob.glob(os.path.join(HERE, "csrc", "hip", "*.hip"))):
        o = os.path.join(OBJ, os.path.basename(src)[:-4] + ".o")
        _run(["hipcc"] + HIP_FLAGS + list(extra_hip_flags) + inc + ["-c", src, "-o", o])
        objs.append(o)
    _run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
         + ["-Wl,-rpath,/opt/rocm/lib", "-lm"])
    return LIB


if __name__ == "__main__":
    build()
    sys.exit(0)
