"""Builds libdz_amd.so (HIP kernels + C ABI) in-tree for gfx950 with hipcc.

Run as `python -m deltazip_amd.build`.  The library is written next to this file so that it
travels with the source tree; nothing is installed into site-packages.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libdz_amd.so")

SOURCES = ["dz_repack.cpp", "dz_kernels.hip", "dz_mdl32.hip", "dz_gemm.hip", "dz_gemm24.hip", "dz_obs.hip", "dz_probe.hip"]

# packed fp32 VALU instructions are switched off for every device compilation in this project
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def build_library(verbose: bool = False, extra_flags=()) -> str:
    """Compiles every source (one hipcc process each, side by side) and links libdz_amd.so."""
    from concurrent.futures import ThreadPoolExecutor
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]

    def run(cmd):
        if verbose:
            print(" ".join(cmd), flush=True)
        res = subprocess.run(cmd, capture_output=True, text=True)
        # hipcc's host pass reports that it does not know the packed-fp32 feature; that is expected
        err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
        if res.returncode != 0:
            raise RuntimeError("hipcc failed:\n" + err)
        return err

    def compile_one(src):
        obj = os.path.join(objdir, os.path.splitext(src)[0] + ".o")
        err = run([hipcc, *[f for f in HIPCC_FLAGS if f != "-shared"], *extra_flags,
                   "-Rpass-analysis=kernel-resource-usage", "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj])
        # The kernels are written to fit the register file: a variant that starts to use scratch
        # memory (register spills) has lost the performance it was tuned for.  Say so at build time.
        name, rest = None, []
        for line in err.splitlines():
            if "remark:" not in line:
                rest.append(line)
            elif "Function Name:" in line:
                name = line.split("Function Name:")[1].split("[")[0].strip()
            elif "ScratchSize [bytes/lane]:" in line and int(line.split("ScratchSize [bytes/lane]:")[1].split("[")[0]) > 0:
                print(f"warning: {src}: kernel {name} uses scratch memory", file=sys.stderr)
        if verbose and "\n".join(rest).strip():
            print("\n".join(rest), file=sys.stderr)
        return obj

    with ThreadPoolExecutor(max_workers=min(len(srcs), os.cpu_count() or 4)) as pool:
        objs = list(pool.map(compile_one, srcs))
    run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB])
    return LIB


if __name__ == "__main__":
    print(build_library(verbose=True))
