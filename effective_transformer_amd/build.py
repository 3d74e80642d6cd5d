"""Builds effective_transformer_amd/lib/libet_hip.so for gfx950 with hipcc.

    python -m effective_transformer_amd.build            # rebuild everything
    python -m effective_transformer_amd.build --if-missing

The objects and the library stay in-tree (git-ignored) so that a GPU box that receives a
copy of the tree can load the library without a compiler run.
"""
from __future__ import annotations

import argparse
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(LIBDIR, "obj")
LIB = os.path.join(LIBDIR, "libet_hip.so")
EXAMPLE = os.path.join(LIBDIR, "et_encoder_example")      # C++ host sample (csrc/encoder_example.cpp)

SOURCES = ["input_output.hip", "row_kernels.hip", "attention.hip", "gemm.hip", "generic.hip", "calibrate.hip", "et_api.cpp"]

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    # packed-FP32 instructions are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes",
]


# per source: the attention kernels keep their MFMA accumulators in VGPRs (with the accumulator registers as
# destination every score and output value costs a v_accvgpr_read before the VALU can touch it: 24 of the 193 VALU
# instructions per head and query tile of the short fp16 kernel)
EXTRA_FLAGS = {"attention.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"]}


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the library cannot be built")
    return exe


def _compile(src: str) -> str:
    obj = os.path.join(OBJDIR, os.path.splitext(src)[0] + ".o")
    cmd = [hipcc(), *FLAGS, *EXTRA_FLAGS.get(src, []), "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, r.stdout, r.stderr))
    warn = [l for l in r.stderr.splitlines() if "warning" in l and "packed-fp32-ops" not in l]
    if warn:
        sys.stderr.write("\n".join(warn) + "\n")
    return obj


def build(force: bool = True, jobs: int = 4) -> str:
    if not force and os.path.exists(LIB):
        return LIB
    os.makedirs(OBJDIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(_compile, SOURCES))
    tmp = LIB + ".tmp"
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", *objs, "-o", tmp]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n%s\n%s" % (r.stdout, r.stderr))
    os.replace(tmp, LIB)
    # the C++ host sample links against the library it sits beside
    cmd = [hipcc(), "--offload-arch=gfx950", "-O2", "-std=c++17", os.path.join(CSRC, "encoder_example.cpp"), "-o", EXAMPLE,
           "-L" + LIBDIR, "-let_hip", "-Wl,-rpath,$ORIGIN"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("building the C++ sample failed:\n%s\n%s" % (r.stdout, r.stderr))
    return LIB


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--if-missing", action="store_true")
    a = ap.parse_args()
    print(build(force=not a.if_missing))
