"""Builds libsmlm_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

Usage: python -m loquetier_amd.build
"""
from __future__ import annotations

import os
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_DIR = os.path.dirname(PKG_DIR)
CSRC_DIR = os.path.join(PKG_DIR, "csrc")
LIB_DIR = os.path.join(PKG_DIR, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libsmlm_hip.so")
PROBE_PATH = os.path.join(LIB_DIR, "libsmlm_probe.so")
# library -> its translation units (headers are found through -I csrc)
LIBRARIES = {
    LIB_PATH: ["smlm_api.hip"],        # the operator library (include/smlm.h)
    PROBE_PATH: ["stream_probe.hip"],  # plain streaming kernels bench.py calibrates against
}

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
    # keep the compiler from forming packed-fp32 VALU ops out of scalar float code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _compile(out: str, sources, verbose: bool) -> None:
    cmd = [hipcc_path(), *HIPCC_FLAGS, "-I", os.path.join(REPO_DIR, "include"), "-I", CSRC_DIR,
           *[os.path.join(CSRC_DIR, s) for s in sources], "-o", out + ".tmp"]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass warns that it does not know the packed-fp32 feature: harmless
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{err}")
    if err.strip() and verbose:
        print(err, file=sys.stderr)
    os.replace(out + ".tmp", out)


def build_library(verbose: bool = False) -> str:
    """Compile every HIP source into loquetier_amd/lib/ (always recompiles); returns the path of
    the operator library."""
    os.makedirs(LIB_DIR, exist_ok=True)
    for out, sources in LIBRARIES.items():
        _compile(out, sources, verbose)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
