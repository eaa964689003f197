"""Measurement aids of bench.py (``--ceilings``, ``--lm-head``): a second, bench-side library, ``libvrl_probe.so``, with
the memory-system and matrix-core probes the kernels of ``verl_amd`` are measured against. Nothing in ``verl_amd``
imports this; the scoring library does not contain it."""

from __future__ import annotations

import ctypes
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
REPO = os.path.dirname(HERE)
LIB_PATH = os.path.join(HERE, "libvrl_probe.so")

_P, _I64, _INT = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
SIGNATURES = {
    "vrl_stream_probe": (_INT, [_P, _P, _I64, _I64, _INT, _P, _P]),
    "vrl_mfma_probe": (_INT, [_I64, _I64, _INT, _INT, _P, _P, _P, _P]),
}
MAX_ITERS = 4000000

_lib = None


def build(verbose: bool = True) -> str:
    """Compile libvrl_probe.so for gfx950 with the flags of the scoring library."""
    from verl_amd import build as hip_build

    cmd = [hip_build.hipcc_path(), *hip_build.HIPCC_FLAGS, f"-I{hip_build.INCLUDE_DIR}", f"-I{hip_build.CSRC_DIR}",
           f"-I{HERE}", os.path.join(HERE, "vrl_probe.hip"), "-o", LIB_PATH + ".tmp"]
    if verbose:
        print("[bench_probes.build]", " ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{out}")
    os.replace(LIB_PATH + ".tmp", LIB_PATH)
    return LIB_PATH


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} does not exist; build it with `python -c 'import bench_probes; bench_probes.build()'`")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = restype, argtypes
        _lib = lib
    return _lib
