"""Builds libmi355x_kmeans.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

Usage:  python sklearn-numba-dpex_amd/_build.py [-j N]
The library is written next to this file; tests, the smoke check and the benchmark load it
from there and never build it themselves.
"""

import argparse
import concurrent.futures
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_NAME = "libmi355x_kmeans.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)

# -packed-fp32-ops: packed fp32 VALU instructions stay off (they have produced silently
# wrong results on these machines); the host pass prints a harmless "not a recognized
# feature" warning for it.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-munsafe-fp-atomics",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA results go to architectural VGPRs: the argmax reads them without accvgpr moves
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",
    "-Wno-unused-command-line-argument",
]


# Per source file.  lloyd_mfma_screen.hip: atomics stay as written - the rewrite of an atomic on a
# uniform address into a wave-wide reduction reads the returned value at once, and the kernel
# wants the answer of its chunk counter a tile later, not on the spot.
EXTRA_FLAGS = {
    "lloyd_mfma_screen.hip": ["-mllvm", "-amdgpu-atomic-optimizer-strategy=None"],
}


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile(src, obj):
    cmd = ["hipcc", *HIPCC_FLAGS, *EXTRA_FLAGS.get(src, []), "-c", os.path.join(CSRC, src), "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    return src, proc.returncode, err


def build(jobs=None, verbose=True):
    if shutil.which("hipcc") is None:
        raise RuntimeError("hipcc not found on PATH; cannot build " + LIB_NAME)
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    srcs = sources()
    objs = [os.path.join(objdir, s[:-4] + ".o") for s in srcs]
    jobs = jobs or min(len(srcs), os.cpu_count() or 4, 16)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        results = list(pool.map(_compile, srcs, objs))
    failed = False
    for src, code, err in results:
        if verbose and err.strip():
            print(f"[{src}]\n{err}", file=sys.stderr)
        if code != 0:
            failed = True
    if failed:
        raise RuntimeError("hipcc failed; see messages above")
    link = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
    proc = subprocess.run(link, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("link failed:\n" + proc.stderr)
    if verbose:
        print(f"built {LIB_PATH} from {len(srcs)} sources")
    return LIB_PATH


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("-j", type=int, default=None)
    args = ap.parse_args()
    build(jobs=args.j)
