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


# Host pass only (the argument checks and launchers of the C ABI) under AddressSanitizer and UBSan; the device
# code is compiled as usual. Each -fsanitize= sits directly behind -Xarch_host.
HOST_SANITIZE_FLAGS = [
    "-Xarch_host", "-fsanitize=address",
    "-Xarch_host", "-fsanitize=undefined",
    "-Xarch_host", "-fno-omit-frame-pointer",
    "-g",
]


def asan_runtime() -> str:
    """The shared AddressSanitizer runtime of hipcc's clang: a sanitised shared library needs it preloaded into the
    process that loads it (``LD_PRELOAD``)."""
    clang = os.path.join(os.path.dirname(os.path.realpath(hipcc_path())), "..", "lib", "llvm", "bin", "clang")
    if not os.path.exists(clang):
        clang = "/opt/rocm/lib/llvm/bin/clang"
    out = subprocess.run([clang, "--print-file-name=libclang_rt.asan-x86_64.so"], stdout=subprocess.PIPE, text=True)
    path = out.stdout.strip()
    if out.returncode != 0 or not os.path.isabs(path) or not os.path.exists(path):
        raise RuntimeError("AddressSanitizer runtime of hipcc's clang not found")
    return path


def build(verbose: bool = True, sanitize_host: bool = False, out_path: str | None = None) -> str:
    """Compile every HIP source into ``verl_amd/libvrl_hip.so`` (or ``out_path``) and return its path. With
    ``sanitize_host`` the host side is instrumented with ASan + UBSan (for tests of the ABI's argument handling;
    load it through ``VERL_AMD_LIB`` with ``asan_runtime()`` preloaded)."""
    lib_path = out_path or LIB_PATH
    flags = list(HIPCC_FLAGS)
    if sanitize_host:
        flags = [("-O1" if f == "-O3" else f) for f in flags] + HOST_SANITIZE_FLAGS
    cmd = [hipcc_path(), *flags, f"-I{INCLUDE_DIR}", f"-I{CSRC_DIR}"]
    cmd += [os.path.join(CSRC_DIR, s) for s in SOURCES]
    tmp = lib_path + ".tmp"
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
    os.replace(tmp, lib_path)
    return lib_path


if __name__ == "__main__":
    build()
    sys.exit(0)
