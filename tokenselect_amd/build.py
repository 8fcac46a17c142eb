"""Build ``libtokenselect_hip.so`` for gfx950 with hipcc, in-tree.

``python -m tokenselect_amd.build`` compiles every ``csrc/*.hip`` translation
unit (in parallel) and links them into ``tokenselect_amd/libtokenselect_hip.so``.
hipcc cross-compiles without a GPU, so this runs on a CPU-only host.
"""

import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
BUILD_DIR = os.path.join(PKG_DIR, "csrc", "build")
LIB_PATH = os.path.join(PKG_DIR, "libtokenselect_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
# Packed-FP32 instruction selection is switched off for all device code.
CXXFLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def _compile(src: str, extra) -> str:
    obj = os.path.join(BUILD_DIR, os.path.basename(src)[:-4] + ".o")
    cmd = [HIPCC, *CXXFLAGS, *extra, "-c", src, "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{res.stdout}\n{res.stderr}")
    noise = "'-packed-fp32-ops' is not a recognized feature"
    warn = "\n".join(line for line in res.stderr.splitlines() if line and noise not in line)
    if warn.strip():
        sys.stderr.write(warn + "\n")
    return obj


def build(extra_flags=(), jobs: int = 8, verbose: bool = True) -> str:
    os.makedirs(BUILD_DIR, exist_ok=True)
    srcs = sources()
    if not srcs:
        raise RuntimeError(f"no .hip sources under {CSRC}")
    with ThreadPoolExecutor(max_workers=min(jobs, len(srcs))) as pool:
        objs = list(pool.map(lambda s: _compile(s, list(extra_flags)), srcs))
    tmp = LIB_PATH + ".tmp"
    cmd = [HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", *objs, "-o", tmp]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH} from {len(srcs)} translation units")
    return LIB_PATH


if __name__ == "__main__":
    build(extra_flags=sys.argv[1:])
