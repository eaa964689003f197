"""Build libvrl_hip.so (gfx950 code object + host launchers) in-tree with hipcc.

Run as ``python -m verl_amd.build``. The library is what ``verl_amd._lib`` loads;
nothing in the package compiles at import time.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_DIR = os.path.dirname(PKG_DIR)
CSRC_DIR = os.path.join(PKG_DIR, "csrc")
INCLUDE_DIR = os.path.join(REPO_DIR, "include")
LIB_PATH = os.path.join(PKG_DIR, "libvrl_hip.so")

SOURCES = ["vrl_abi.hip"]

# -ffp-contract=off: a*b+c is fused only where the source says fma().
# -packed-fp32-ops is switched off so the compiler emits no v_pk_*_f32.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-ffp-contract=off",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc)")


def build(verbose: bool = True) -> str:
    """Compile every HIP source into ``verl_amd/libvrl_hip.so`` and return its path."""
    cmd = [hipcc_path(), *HIPCC_FLAGS, f"-I{INCLUDE_DIR}", f"-I{CSRC_DIR}"]
    cmd += [os.path.join(CSRC_DIR, s) for s in SOURCES]
    tmp = LIB_PATH + ".tmp"
    cmd += ["-o", tmp]
    if verbose:
        print("[verl_amd.build]", " ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # hipcc's host pass warns that it does not know the packed-fp32 feature; drop that line only.
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{out}")
    if verbose and out.strip():
        print(out, flush=True)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    build()
    sys.exit(0)
