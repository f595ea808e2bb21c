"""Builds libhgcalml_amd.so (HIP kernels + C ABI) for gfx950 with hipcc.

Run as ``python -m hgcalml_amd.build``. hipcc cross-compiles, so no GPU is
needed. The library is written next to the sources (in-tree) so that it travels
with the repository snapshot to the GPU box.
"""
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
LIB_PATH = os.path.join(HERE, "libhgcalml_amd.so")

SOURCES = ["binning.hip", "knn.hip", "accumulate.hip", "accumulate_grad_fused.hip", "accumulate_grad_records.hip", "split_sort.hip", "sample_sort.hip", "inverse_index.hip", "neighbour_ops.hip", "condensates.hip", "pipelines.hip"]

# -ffp-contract=off: distances and accumulations must be separate fp32
#   multiplies and adds in source order to reproduce the reference bit for bit.
# -packed-fp32-ops disabled: hipcc must not form v_pk_*_f32 on this hardware pool.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result", "-Wno-unknown-warning-option",
    "-I", INCLUDE, "-I", CSRC,
]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; ROCm is required to build hgcalml_amd")
    return exe


def _compile(src):
    obj = os.path.join(CSRC, os.path.splitext(src)[0] + ".o")
    cmd = [hipcc(), *HIPCC_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, res.stdout, res.stderr))
    return obj


def build(verbose=True, sources=None):
    """Compile `sources` (default: all) and link every object into the library."""
    sources = sources or SOURCES
    with ThreadPoolExecutor(max_workers=min(6, len(sources))) as pool:
        list(pool.map(_compile, sources))
    objs = [os.path.join(CSRC, os.path.splitext(src)[0] + ".o") for src in SOURCES]
    missing = [o for o in objs if not os.path.exists(o)]
    if missing:
        with ThreadPoolExecutor(max_workers=4) as pool:
            list(pool.map(_compile, [os.path.basename(o)[:-2] + ".hip" for o in missing]))
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n%s\n%s" % (res.stdout, res.stderr))
    if verbose:
        print("built", LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    build(sources=sys.argv[1:] or None)
