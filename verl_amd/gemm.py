"""``out = y @ x.T`` on the matrix cores with this package's own kernel (``vrl_gemm_nt``): the two products of the LM-head
backward (``d hidden = G @ W``, ``d W += G.T @ H``) once their operands are contiguous along the contraction axis.

The reference forms them with ``torch.matmul`` (verl/utils/kernel/kernels.py:1710-1720); ``fused_linear_for_ppo`` uses this
module instead when ``kernels="mfma"``.
"""

from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import _lib

_DTYPE_CODES = {torch.bfloat16: _lib.VRL_BF16, torch.float16: _lib.VRL_F16}

# vrl_gemm_nt launches from this module since import (what a caller can count to see which products were its own)
counters = {"gemm_nt": 0}


def gemm_nt_takes(x: torch.Tensor, y: torch.Tensor) -> bool:
    """Whether ``gemm_nt`` accepts these operands (16-bit, >= 256 rows each, contraction a multiple of 64, >= 128)."""
    return (x.dtype in _DTYPE_CODES and y.dtype == x.dtype and x.dim() == 2 and y.dim() == 2 and x.shape[1] == y.shape[1]
            and x.shape[0] >= 256 and y.shape[0] >= 256 and x.shape[0] % 4 == 0 and x.shape[1] % 64 == 0
            and x.shape[1] >= 128)


def gemm_nt(x: torch.Tensor, y: torch.Tensor, out: Optional[torch.Tensor] = None, accumulate: bool = False,
            k_parts: Optional[int] = None) -> torch.Tensor:
    """``out[j, i] (+)= sum_k y[j, k] * x[i, k]``: ``x`` is ``(NX, K)``, ``y`` is ``(NY, K)``, ``out`` is ``(NY, NX)``, all
    bf16 or all fp16, fp32 accumulation with one rounding. ``accumulate`` adds to what ``out`` holds.

    ``k_parts`` cuts the contraction into ranges that are summed in a fixed order through a temporary fp32 buffer
    (``k_parts * NX * NY`` floats): how a product with few 256 x 256 output tiles still fills the CUs. None lets the
    library choose.
    """
    if not (x.is_cuda and y.is_cuda):
        raise RuntimeError("gemm_nt: tensors must be on the GPU; verl_amd has no CPU implementation")
    if not gemm_nt_takes(x, y):
        raise ValueError(f"gemm_nt: unsupported operands {tuple(x.shape)} {x.dtype} / {tuple(y.shape)} {y.dtype}")
    if x.stride(1) != 1 or y.stride(1) != 1:
        raise ValueError("gemm_nt: operands must be contiguous along the contraction axis")
    NX, K = x.shape
    NY = y.shape[0]
    dev = x.device
    if out is None:
        if accumulate:
            raise ValueError("gemm_nt: accumulate needs an out tensor")
        out = torch.empty((NY, NX), dtype=x.dtype, device=dev)
    if tuple(out.shape) != (NY, NX) or out.dtype != x.dtype or out.stride(1) != 1 or out.device != dev:
        raise ValueError(f"gemm_nt: out must be ({NY}, {NX}) {x.dtype} on {dev}, contiguous along its last axis")
    lib = _lib.load()
    code = _DTYPE_CODES[x.dtype]
    need = ctypes.c_int64(0)
    planned = lib.vrl_gemm_nt_plan(code, NX, NY, K, ctypes.addressof(need))
    if planned < 0:
        _lib.check("vrl_gemm_nt_plan", planned)
    parts = planned if k_parts is None else int(k_parts)
    work = torch.empty(parts * NX * NY, dtype=torch.float32, device=dev) if parts > 1 else None
    with torch.cuda.device(dev):
        st = lib.vrl_gemm_nt(x.data_ptr(), y.data_ptr(), code, NX, NY, K, x.stride(0), y.stride(0), out.data_ptr(),
                             out.stride(0), 1 if accumulate else 0, parts, None if work is None else work.data_ptr(),
                             _lib.stream_ptr(dev))
    _lib.check("vrl_gemm_nt", st)
    counters["gemm_nt"] += 1
    return out
