"""Builds libsqattn_hip.so in-tree with plain hipcc for gfx950 (no torch extension, no pybind)."""
from __future__ import annotations

import os
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
INCLUDE = os.path.join(os.path.dirname(PKG_DIR), "include")
LIB_PATH = os.path.join(PKG_DIR, "libsqattn_hip.so")
SOURCES = ["capi.hip", "decode_gfx950.hip", "prefill_gfx950.hip", "kmeans_gfx950.hip", "prepass_gfx950.hip", "kvcache_gfx950.hip", "layer_gfx950.hip", "linear_gfx950.hip", "calib_gfx950.hip", "probe_gfx950.hip"]

HIPCC_FLAGS = [
    "-O3", "-std=c++17", "--offload-arch=gfx950", "-fPIC", "-shared",
    # keep the compiler from forming packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


# Per-source flags.  The k-means assign kernel reads its MFMA results with the vector ALU right away (arg-max): the MFMAs
# are kept in their VGPR form there, otherwise every score passes through a v_accvgpr_read first.
SOURCE_FLAGS = {"kmeans_gfx950.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}


def build(verbose: bool = True, extra_flags=()) -> str:
    """Compile every HIP source (in parallel, one object each) and link them into one shared library; returns its
    path.  Always recompiles."""
    import tempfile

    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    compile_flags = [f for f in HIPCC_FLAGS if f != "-shared"]
    with tempfile.TemporaryDirectory(prefix="sqattn_build_") as tmp:
        jobs = []
        for s in srcs:
            obj = os.path.join(tmp, s.replace(".hip", ".o"))
            cmd = [hipcc, *compile_flags, *SOURCE_FLAGS.get(s, []), *extra_flags, "-I", INCLUDE, "-I", CSRC, "-c", os.path.join(CSRC, s), "-o", obj]
            if verbose:
                print(" ".join(cmd), flush=True)
            jobs.append((cmd, obj, subprocess.Popen(cmd)))
        objs = []
        for cmd, obj, proc in jobs:
            if proc.wait() != 0:
                raise subprocess.CalledProcessError(proc.returncode, cmd)
            objs.append(obj)
        link = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB_PATH]
        if verbose:
            print(" ".join(link), flush=True)
        subprocess.run(link, check=True)
    return LIB_PATH


if __name__ == "__main__":
    build(extra_flags=sys.argv[1:])
