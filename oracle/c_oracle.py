"""TEST INFRASTRUCTURE — ctypes binding of oracle/vrl_oracle.c (built by oracle/Makefile).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this.
"""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libvrl_oracle.so")

_lib = None


def build() -> str:
    """(Re)compile libvrl_oracle.so with gcc through the Makefile."""
    subprocess.run(["make", "-C", HERE, "-B", "libvrl_oracle.so"], check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    return LIB_PATH


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        lib = ctypes.CDLL(LIB_PATH)
        P, I64, F32, INT = ctypes.c_void_p, ctypes.c_int64, ctypes.c_float, ctypes.c_int
        lib.vrl_oracle_rowscore.restype = INT
        lib.vrl_oracle_rowscore.argtypes = [P, INT, I64, I64, I64, P, P, P, P]
        lib.vrl_oracle_spec_verify.restype = INT
        lib.vrl_oracle_spec_verify.argtypes = [P, P, P, P, P, I64, I64, F32, F32, P, P, P, P, P, I64, P, P]
        _lib = lib
    return _lib


def _np_ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def rowscore(logits: torch.Tensor, labels=None, temperature=None):
    """fp64 (log-probs, entropy) of a 2-D fp32 or bf16 CPU tensor; log-probs is None without labels."""
    assert logits.dim() == 2 and not logits.is_cuda
    x = logits.contiguous()
    if x.dtype == torch.float32:
        buf, dt = x.numpy(), 0
    elif x.dtype == torch.bfloat16:
        buf, dt = x.view(torch.int16).numpy(), 1
    elif x.dtype == torch.float16:
        buf, dt = x.float().numpy(), 0  # every half is an exact float
    else:
        raise TypeError(x.dtype)
    n, V = x.shape
    lab = None if labels is None else np.ascontiguousarray(torch.as_tensor(labels).cpu().numpy().astype(np.int64).reshape(n))
    temp = None if temperature is None else np.ascontiguousarray(torch.as_tensor(temperature).cpu().float().numpy().reshape(n))
    lp = np.empty(n, dtype=np.float64) if lab is not None else None
    h = np.empty(n, dtype=np.float64)
    st = load().vrl_oracle_rowscore(_np_ptr(buf), dt, n, V, V, _np_ptr(lab), _np_ptr(temp), _np_ptr(lp), _np_ptr(h))
    assert st == 0, st
    return lp, h


def spec_verify(logp_new, logp_old, log_u, mask, thresh_offset, near_eps=1e-6, cu_seqlens=None, draft_ids=None, pad_id=0):
    """Same return dict as oracle.verify.verify_loops, computed by the C loops."""
    ln = np.ascontiguousarray(torch.as_tensor(logp_new).cpu().float().numpy())
    lo = np.ascontiguousarray(torch.as_tensor(logp_old).cpu().float().numpy())
    lu = np.ascontiguousarray(torch.as_tensor(log_u).cpu().float().numpy())
    shape = ln.shape
    mk = None if mask is None else np.ascontiguousarray((torch.as_tensor(mask).cpu().numpy() != 0).astype(np.uint8))
    if cu_seqlens is None:
        B, T = shape
        cu = None
    else:
        cu = np.ascontiguousarray(torch.as_tensor(cu_seqlens).cpu().numpy().astype(np.int64))
        B, T = len(cu) - 1, 0
    ids = None if draft_ids is None else np.ascontiguousarray(torch.as_tensor(draft_ids).cpu().numpy().astype(np.int64))
    accept = np.zeros(shape, dtype=np.uint8)
    first = np.zeros(B, dtype=np.int32)
    prefix = np.zeros(B, dtype=np.int32)
    near = np.zeros(B, dtype=np.int32)
    out_ids = None if ids is None else np.zeros(shape, dtype=np.int64)
    out_mask = None if ids is None else np.zeros(shape, dtype=np.uint8)
    st = load().vrl_oracle_spec_verify(
        _np_ptr(ln), _np_ptr(lo), _np_ptr(lu), _np_ptr(mk), _np_ptr(cu), B, T, float(np.float32(thresh_offset)),
        float(np.float32(near_eps)), _np_ptr(accept), _np_ptr(first), _np_ptr(prefix), _np_ptr(near), _np_ptr(ids),
        int(pad_id), _np_ptr(out_ids), _np_ptr(out_mask),
    )
    assert st == 0, st
    res = {"accept": accept, "first_reject": first, "prefix_len": prefix, "near_count": near}
    if ids is not None:
        res["out_ids"] = out_ids
        res["out_mask"] = out_mask
    return res
