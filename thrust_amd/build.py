"""Builds libthrust_amd.so (the gfx950 kernels and their C ABI) in-tree with hipcc.

Usage: python -m thrust_amd.build [--force]
"""
import concurrent.futures
import os
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
OBJ_DIR = os.path.join(PKG_DIR, "build")
LIB_PATH = os.path.join(PKG_DIR, "libthrust_amd.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option",
]


# Sources that take longest to compile (many template instances) go first, so that the
# worker pool does not end on one of them.
SLOWEST_FIRST = ["transform_scan.hip", "transform_scan_exclusive.hip", "merge_sort.hip", "scan.hip",
                 "reduce_by_key.hip", "radix_sort.hip", "select_stencil_in_place.hip", "scan_by_key.hip", "transform_reduce.hip"]


def sources():
    found = sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))
    return [f for f in SLOWEST_FIRST if f in found] + [f for f in found if f not in SLOWEST_FIRST]


def _compile(src):
    obj = os.path.join(OBJ_DIR, src[:-4] + ".o")
    cmd = [HIPCC, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose=True):
    """Compiles every csrc/*.hip for gfx950 and links libthrust_amd.so.  Always recompiles."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = sources()
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(_compile, srcs))
    cmd = [HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    if verbose:
        print(f"built {LIB_PATH} from {len(srcs)} sources")
    return LIB_PATH


if __name__ == "__main__":
    build()
