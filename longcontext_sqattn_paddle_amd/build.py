"""Builds libsqattn_hip.so (the product: everything include/sqattn.h declares) and libsqattn_probe.so (a measurement
aid the benchmark loads) in-tree with plain hipcc for gfx950 (no torch extension, no pybind)."""
from __future__ import annotations

import os
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
INCLUDE = os.path.join(os.path.dirname(PKG_DIR), "include")
LIB_PATH = os.path.join(PKG_DIR, "libsqattn_hip.so")
PROBE_LIB_PATH = os.path.join(PKG_DIR, "libsqattn_probe.so")
SOURCES = ["capi.hip", "decode_gfx950.hip", "prefill_gfx950.hip", "kmeans_gfx950.hip", "prepass_gfx950.hip", "kvcache_gfx950.hip", "layer_gfx950.hip", "linear_gfx950.hip", "calib_gfx950.hip"]
PROBE_SOURCES = ["capi.hip", "probe_gfx950.hip"]   # its own copy of the error string and the tensor checks

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
    """Compile every HIP source (in parallel, one object each) and link the two shared libraries; returns the path of
    the product library.  Always recompiles; a listed source that is missing is an error."""
    import tempfile

    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    srcs = list(dict.fromkeys(SOURCES + PROBE_SOURCES))
    missing = [s for s in srcs if not os.path.exists(os.path.join(CSRC, s))]
    if missing:
        raise FileNotFoundError(f"HIP sources missing from {CSRC}: {', '.join(missing)}")
    compile_flags = [f for f in HIPCC_FLAGS if f != "-shared"]
    with tempfile.TemporaryDirectory(prefix="sqattn_build_") as tmp:
        jobs = []
        for s in srcs:
            obj = os.path.join(tmp, s.replace(".hip", ".o"))
            cmd = [hipcc, *compile_flags, *SOURCE_FLAGS.get(s, []), *extra_flags, "-I", INCLUDE, "-I", CSRC, "-c", os.path.join(CSRC, s), "-o", obj]
            if verbose:
                print(" ".join(cmd), flush=True)
            jobs.append((cmd, obj, subprocess.Popen(cmd)))
        for cmd, obj, proc in jobs:
            if proc.wait() != 0:
                raise subprocess.CalledProcessError(proc.returncode, cmd)
        for names, path in ((SOURCES, LIB_PATH), (PROBE_SOURCES, PROBE_LIB_PATH)):
            objs = [os.path.join(tmp, s.replace(".hip", ".o")) for s in names]
            link = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", path]
            if verbose:
                print(" ".join(link), flush=True)
            subprocess.run(link, check=True)
    return LIB_PATH


if __name__ == "__main__":
    build(extra_flags=sys.argv[1:])
