"""Compile libviewattn.so (gfx950) in-tree with hipcc.

    python async_llm_amd/build.py [--incremental] [output.so [extra hipcc flags...]]

Every HIP source is compiled in two passes: the device pass (``--cuda-device-only``)
carries the target feature that keeps packed fp32 forms out of the generated code,
the host pass (``--cuda-host-only``) embeds the device binary the first pass wrote.
The feature is an AMDGPU one: given to a single hipcc invocation it would also reach
the x86 pass, which ignores it with a warning.  Sources compile in parallel.
"""

from __future__ import annotations

import hashlib
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build")
LIB_PATH = os.path.join(HERE, "libviewattn.so")
HIP_SOURCES = ["viewattn.hip", "va_mfma.hip", "va_mfma_wide.hip", "va_mfma_stream.hip", "va_block_copy.hip"]
HOST_SOURCES = ["va_plan.cpp"]

COMMON_FLAGS = ["-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-Wall", "-Wno-unused-function", "-DVA_BUILDING=1"]
DEVICE_FLAGS = ["--offload-arch=gfx950", "--cuda-device-only",
                # packed fp32 forms are kept out of the generated code
                "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
HOST_FLAGS = ["--offload-arch=gfx950", "--cuda-host-only"]
# Device flags of single sources.  The wide kernel may use all 512 registers of a lane, for which the
# compiler gives every matrix product it selects an accumulator in the accumulation registers; its
# score products are read by the vector ALU at once and want ordinary registers (the long-lived
# output accumulators are pinned in accumulation registers by hand).
SOURCE_DEVICE_FLAGS = {"va_mfma_wide.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True, cwd=CSRC)


def _newest_header() -> float:
    roots = [CSRC, os.path.join(HERE, "..", "include")]
    return max(os.path.getmtime(os.path.join(r, f)) for r in roots for f in os.listdir(r) if f.endswith(".h"))


def _compile_one(hipcc, src, obj, extra, verbose):
    path = os.path.join(CSRC, src)
    if src.endswith(".hip"):
        fatbin = obj[:-2] + ".hipfb"
        _run([hipcc, *COMMON_FLAGS, *DEVICE_FLAGS, *SOURCE_DEVICE_FLAGS.get(src, []), *extra, "-c", path, "-o", fatbin],
             verbose)
        _run([hipcc, *COMMON_FLAGS, *HOST_FLAGS, *extra, "-Xclang", "-fcuda-include-gpubinary", "-Xclang", fatbin,
              "-c", path, "-o", obj], verbose)
    else:  # host code only (hipcc would take a .cpp for HIP and run a device pass over it)
        _run([os.environ.get("CXX", "g++"), *COMMON_FLAGS, *extra, "-c", path, "-o", obj], verbose)


def build(verbose: bool = True, out: str = LIB_PATH, extra_flags=(), incremental: bool = False) -> str:
    """Compile every source and link ``out``.  ``incremental`` keeps objects that are newer than
    their source and every header (same flags assumed); the default recompiles everything."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    os.makedirs(OBJ_DIR, exist_ok=True)
    # objects are named after everything that shapes them besides the source text: the output they
    # are linked into and every flag (a digest that is the same in every process, unlike hash())
    flags = repr((out, tuple(extra_flags), COMMON_FLAGS, DEVICE_FLAGS, HOST_FLAGS, sorted(SOURCE_DEVICE_FLAGS.items())))
    default = out == LIB_PATH and not extra_flags
    tag = "" if default else "." + hashlib.sha1(flags.encode()).hexdigest()[:10]
    stamp = os.path.join(OBJ_DIR, "flags" + tag + ".txt")
    if incremental and not (os.path.exists(stamp) and open(stamp).read() == flags):
        incremental = False  # the flags changed since these objects were made
    jobs, objects = [], []
    headers = _newest_header() if incremental else 0.0
    for src in HIP_SOURCES + HOST_SOURCES:
        obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + tag + ".o")
        objects.append(obj)
        fresh = incremental and os.path.exists(obj) and os.path.getmtime(obj) > max(
            headers, os.path.getmtime(os.path.join(CSRC, src)))
        if not fresh:
            jobs.append((src, obj))
    with ThreadPoolExecutor(max_workers=min(8, max(1, len(jobs)))) as pool:
        for f in [pool.submit(_compile_one, hipcc, s, o, list(extra_flags), verbose) for s, o in jobs]:
            f.result()
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objects, "-o", out], verbose)
    with open(stamp, "w") as f:
        f.write(flags)
    return out


if __name__ == "__main__":
    argv = sys.argv[1:]
    inc = "--incremental" in argv
    argv = [a for a in argv if a != "--incremental"]
    target = os.path.abspath(argv[0]) if argv else LIB_PATH
    print(build(out=target, extra_flags=argv[1:], incremental=inc))
    sys.exit(0)
