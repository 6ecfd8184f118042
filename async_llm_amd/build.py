"""Compile libviewattn.so (gfx950) in-tree with hipcc.

    python async_llm_amd/build.py
"""

from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(HERE, "libviewattn.so")
SOURCES = ["viewattn.hip", "va_mfma.hip", "va_mfma_wide.hip", "va_mfma_stream.hip", "va_block_copy.hip", "va_plan.cpp"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-fvisibility=hidden",
    "-Wall",
    "-Wno-unused-function",
    # packed fp32 forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def build(verbose: bool = True, out: str = LIB_PATH, extra_flags=()) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, *HIPCC_FLAGS, "-DVA_BUILDING=1", *extra_flags]
    for src in SOURCES:
        path = os.path.join(CSRC, src)
        if src.endswith(".cpp"):
            cmd += ["-x", "hip", path]
        else:
            cmd.append(path)
    cmd += ["-o", out]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True, cwd=CSRC)
    return out


if __name__ == "__main__":
    # usage: build.py [output.so [extra hipcc flags...]]
    target = os.path.abspath(sys.argv[1]) if len(sys.argv) > 1 else LIB_PATH
    print(build(out=target, extra_flags=sys.argv[2:]))
    sys.exit(0)
