"""Builds the backend's shared library for gfx950 with hipcc, in-tree.

    python -m cudabackend_amd.build            # compile what changed, link cudabackend_amd/libavocado_hip.so
    python -m cudabackend_amd.build --force    # recompile everything

hipcc cross-compiles without a GPU.  Every translation unit is compiled with packed-fp32 code generation disabled.
"""
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "_obj")
LIB = os.path.join(HERE, "libavocado_hip.so")
ARCH = "gfx950"

SOURCES = [
    "backend.cpp",
    "winograd_transforms.hip",
    "gemm.hip",
    "conv_implicit_gemm.hip",
    "conv_tile.hip",
    "conv_small.hip",
    "conv_stem.hip",
    "conv_thin.hip",
    "conv_pointwise.hip",
    "conv_winograd_fused.hip",
    "conv_winograd_rows.hip",
    "conv_strided.hip",
    "conv_pointwise_block.hip",
    "elementwise.hip",
]
HEADERS = ["common.hpp", "mfma_core.hpp", "conv_epilogue.hpp", "conv_tile.hpp", "conv_small.hpp", "conv_stem.hpp", "conv_thin.hpp", "conv_pointwise.hpp", "persistent_gemm.hpp", "resident_gemm.hpp", "../../include/avocado_hip_kernels.h", "../../include/avocado_hip_backend.h",
           "../../include/avocado_backend_defs.h"]

FLAGS = ["-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden", "--offload-arch=" + ARCH, "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument"]


def _stale(src, obj):
    if not os.path.exists(obj):
        return True
    t = os.path.getmtime(obj)
    deps = [os.path.join(CSRC, src)] + [os.path.join(CSRC, h) for h in HEADERS]
    return any(os.path.getmtime(d) > t for d in deps)


def _compile(src, force):
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
    if not force and not _stale(src, obj):
        return obj, ""
    cmd = ["hipcc"] + FLAGS + ["-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    log = "\n".join(l for l in r.stdout.splitlines() if "is not a recognized feature for this target" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s" % (src, log))
    return obj, log


def build(force=False, verbose=False):
    os.makedirs(OBJ, exist_ok=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(6, os.cpu_count() or 1)) as pool:
        results = list(pool.map(lambda s: _compile(s, force), SOURCES))
    objs = [o for o, _ in results]
    if verbose:
        for _, log in results:
            if log.strip():
                print(log)
    if force or not os.path.exists(LIB) or any(os.path.getmtime(o) > os.path.getmtime(LIB) for o in objs):
        cmd = ["hipcc", "-shared", "-fPIC", "--offload-arch=" + ARCH, "-o", LIB] + objs
        r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n" + r.stdout)
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv, verbose=True))
