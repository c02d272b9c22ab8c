"""Builds libcrit_pkv.so (the C-ABI library of gfx950 kernels) with hipcc, in-tree, one object per source in parallel.

    python -m crit_amd.build            # compile everything, link crit_amd/lib/libcrit_pkv.so

hipcc cross-compiles for gfx950 without a GPU. No fast-math; FP contraction is off so that every fused multiply-add in
the kernels is one the source spells out (a column's bits must not depend on which template instance computed it).
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIB_DIR, "libcrit_pkv.so")
OBJ_DIR = os.path.join(LIB_DIR, "obj")

# (--offload-compress: the device code is stored compressed and unpacked by the HIP runtime when a source file's kernels
# are first used: the library is 8 MB instead of 26)
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fno-fast-math", "--offload-compress",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile(src):
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
    cmd = ["hipcc", *FLAGS, *os.environ.get("CRIT_PKV_EXTRA_FLAGS", "").split(), "-c", src, "-o", obj]
    done = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(line for line in done.stderr.splitlines() if noise not in line)
    if done.returncode:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    return obj, err


def build(verbose=True, jobs=None):
    """Compile every .hip under csrc/ for gfx950 and link the shared library; returns its path."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1)
    with ThreadPoolExecutor(jobs) as pool:
        found = list(pool.map(_compile, sources()))
    for _, err in found:
        if err.strip() and verbose:
            print(err, file=sys.stderr)
    out = os.environ.get("CRIT_PKV_OUT", LIB)
    link = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out, *[obj for obj, _ in found]]
    done = subprocess.run(link, capture_output=True, text=True)
    if done.returncode:
        raise RuntimeError(f"link failed:\n{done.stderr}")
    if verbose:
        print(f"built {out}")
    return out


if __name__ == "__main__":
    build()
