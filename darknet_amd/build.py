"""Build recipe of the native library: ``python -m darknet_amd.build``.

hipcc cross-compiles the HIP sources for gfx950 (no GPU needed to build), gcc compiles the host
C files, and one link step produces ``darknet_amd/libdarknet_hip.so`` in-tree.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
OBJDIR = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libdarknet_hip.so")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")

HIP_SOURCES = ["pointwise.hip", "pool.hip", "conv_direct.hip", "conv_mfma.hip", "conv_first.hip", "conv_group.hip", "xnor.hip", "detect.hip", "image.hip", "local.hip"]
C_SOURCES = ["hip.c", "cfg_reader.c", "cfg_parser.c", "layers.c", "network.c", "weights_io.c", "boxes.c", "images.c", "pipeline.c"]

# -packed-fp32-ops: keep the compiler from forming packed fp32 instructions.
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-ffp-contract=off", "-Wno-comment",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-I" + CSRC, "-I" + INCLUDE]
C_FLAGS = ["-O2", "-fPIC", "-fopenmp", "-Wall", "-Wno-comment", "-D__HIP_PLATFORM_AMD__=1",
           "-I" + CSRC, "-I" + INCLUDE, "-I" + os.path.join(ROCM, "include")]


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    noise = ("packed-fp32-ops' is not a recognized feature", "warning generated")
    out = "\n".join(l for l in r.stdout.splitlines() if not any(n in l for n in noise))
    if r.returncode != 0:
        raise RuntimeError("build step failed: " + " ".join(cmd) + "\n" + out)
    return out


def build(verbose: bool = False, jobs: int = 6) -> str:
    hipcc = shutil.which("hipcc") or os.path.join(ROCM, "bin", "hipcc")
    os.makedirs(OBJDIR, exist_ok=True)
    steps = []
    objs = []
    for s in HIP_SOURCES:
        o = os.path.join(OBJDIR, s + ".o")
        objs.append(o)
        steps.append([hipcc] + HIP_FLAGS + ["-c", os.path.join(CSRC, s), "-o", o])
    for s in C_SOURCES:
        o = os.path.join(OBJDIR, s + ".o")
        objs.append(o)
        steps.append(["gcc"] + C_FLAGS + ["-c", os.path.join(CSRC, s), "-o", o])
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        for out in ex.map(_run, steps):
            if verbose and out.strip():
                print(out)
    out = _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-Wl,-Bsymbolic", "-o", LIB] + objs +
               ["-L" + os.path.join(ROCM, "lib"), "-lamdhip64", "-lm", "-lgomp"])
    if verbose and out.strip():
        print(out)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
    sys.exit(0)
