"""Builds the gfx950 operator library (blackforge_amd/lib/libbf_hip.so) with hipcc.

hipcc cross-compiles for gfx950 without a GPU, so this runs anywhere ROCm is installed.  Every
csrc/*.hip file is compiled to an object (in parallel) and linked into one shared library whose only
exported interface is the C ABI declared in include/bf_hip.h.
"""
from __future__ import annotations

import concurrent.futures
import glob
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libbf_hip.so")

ARCH = "gfx950"
# -packed-fp32-ops off: keep the compiler from forming v_pk_*_f32 from ordinary float code.
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-ffp-contract=off",
    "-Wno-unused-value", "-Wno-unknown-warning-option",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
]


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found: the gfx950 library cannot be built")


def _compile(src: str, force: bool) -> str:
    obj = os.path.join(OBJ_DIR, os.path.basename(src).rsplit(".", 1)[0] + ".o")
    deps = [src] + glob.glob(os.path.join(CSRC, "*.hpp")) + glob.glob(os.path.join(ROOT, "include", "*.h"))
    if not force and os.path.exists(obj) and all(os.path.getmtime(obj) >= os.path.getmtime(d) for d in deps):
        return obj
    # BF_HIPCC_EXTRA: extra compiler flags for experiments (e.g. "-DSOME_SWITCH"); empty in normal builds
    cmd = [hipcc()] + HIPCC_FLAGS + os.environ.get("BF_HIPCC_EXTRA", "").split() + ["-c", src, "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass warns that it does not know the packed-fp32 feature: harmless, filtered out
    err = "\n".join(l for l in proc.stderr.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(force: bool = True, jobs: int = 8, verbose: bool = True) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    sources = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    if not sources:
        raise RuntimeError("no HIP sources found")
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        objects = list(pool.map(lambda s: _compile(s, force), sources))
    cmd = [hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", LIB_PATH] + objects + ["-Wl,-rpath,/opt/rocm/lib"]
    subprocess.run(cmd, check=True, capture_output=True, text=True)
    if verbose:
        print(f"built {LIB_PATH} from {len(sources)} sources")
    return LIB_PATH


if __name__ == "__main__":
    build(force="--incremental" not in sys.argv)
