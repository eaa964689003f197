"""``out = y @ x.T`` on the matrix cores with this package's own kernel (``vrl_gemm``): the two products of the LM-head
backward, ``d hidden = G @ W`` and ``d W += G.T @ H``, straight from the tensors the backward holds. Each operand is
either row-major, ``(rows, K)`` contiguous along the contraction, or contraction-major, ``(K, rows)`` contiguous along
its rows (``x_t`` / ``y_t``), so neither product needs a transposed copy.

The reference forms them with ``torch.matmul`` (verl/utils/kernel/kernels.py:1710-1720); ``fused_linear_for_ppo`` uses this
module instead unless ``kernels="library"``.
"""

from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import _lib

_DTYPE_CODES = {torch.bfloat16: _lib.VRL_BF16, torch.float16: _lib.VRL_F16}

# vrl_gemm launches from this module since import (what a caller can count to see which products were its own)
counters = {"gemm": 0}


def _dims(x: torch.Tensor, y: torch.Tensor, x_t: bool, y_t: bool):
    NX, KX = (x.shape[1], x.shape[0]) if x_t else (x.shape[0], x.shape[1])
    NY, KY = (y.shape[1], y.shape[0]) if y_t else (y.shape[0], y.shape[1])
    return NX, NY, KX, KY


def gemm_takes(x: torch.Tensor, y: torch.Tensor, x_t: bool = False, y_t: bool = False) -> bool:
    """Whether ``gemm`` accepts these operands, i.e. everything ``vrl_gemm`` checks about them: 16-bit, >= 256 rows each,
    contraction a multiple of 64 and >= 128, last axis contiguous, row strides multiples of 8, 16-byte aligned storage;
    ``NX`` a multiple of 4, a contraction-major operand's rows a multiple of 8."""
    if not (x.dtype in _DTYPE_CODES and y.dtype == x.dtype and x.dim() == 2 and y.dim() == 2):
        return False
    NX, NY, KX, KY = _dims(x, y, x_t, y_t)
    return (KX == KY and NX >= 256 and NY >= 256 and NX % 4 == 0 and KX % 64 == 0 and KX >= 128
            and x.stride(1) == 1 and y.stride(1) == 1 and x.stride(0) % 8 == 0 and y.stride(0) % 8 == 0
            and x.stride(0) >= x.shape[1] and y.stride(0) >= y.shape[1]
            and x.data_ptr() % 16 == 0 and y.data_ptr() % 16 == 0
            and (not x_t or NX % 8 == 0) and (not y_t or NY % 8 == 0))


def gemm_nt_takes(x: torch.Tensor, y: torch.Tensor) -> bool:
    """``gemm_takes`` for two row-major operands."""
    return gemm_takes(x, y, False, False)


def gemm(x: torch.Tensor, y: torch.Tensor, x_t: bool = False, y_t: bool = False, out: Optional[torch.Tensor] = None,
         accumulate: bool = False, k_parts: Optional[int] = None) -> torch.Tensor:
    """``out[j, i] (+)= sum_k Y[j, k] * X[i, k]`` with ``X = x`` of shape ``(NX, K)`` (``x.T`` when ``x_t``: ``x`` is then
    ``(K, NX)``) and ``Y = y`` of shape ``(NY, K)`` (``y.T`` when ``y_t``); ``out`` is ``(NY, NX)``. All bf16 or all fp16,
    fp32 accumulation with one rounding. ``accumulate`` adds to what ``out`` holds.

    ``k_parts`` cuts the contraction into ranges that are summed in a fixed order through a temporary fp32 buffer
    (``k_parts * NX * NY`` floats): how a product with few 256 x 256 output tiles still fills the CUs. None lets the
    library choose.
    """
    if not (x.is_cuda and y.is_cuda):
        raise RuntimeError("gemm: tensors must be on the GPU; verl_amd has no CPU implementation")
    if not gemm_takes(x, y, x_t, y_t):
        raise ValueError(f"gemm: unsupported operands {tuple(x.shape)} {x.dtype} (x_t={x_t}) / {tuple(y.shape)} {y.dtype} "
                         f"(y_t={y_t}), strides {x.stride()} / {y.stride()}")
    NX, NY, K, _ = _dims(x, y, x_t, y_t)
    dev = x.device
    if out is None:
        if accumulate:
            raise ValueError("gemm: accumulate needs an out tensor")
        out = torch.empty((NY, NX), dtype=x.dtype, device=dev)
    if tuple(out.shape) != (NY, NX) or out.dtype != x.dtype or out.stride(1) != 1 or out.device != dev:
        raise ValueError(f"gemm: out must be ({NY}, {NX}) {x.dtype} on {dev}, contiguous along its last axis")
    lib = _lib.load()
    code = _DTYPE_CODES[x.dtype]
    need = ctypes.c_int64(0)
    planned = lib.vrl_gemm_nt_plan(code, NX, NY, K, ctypes.addressof(need))
    if planned < 0:
        _lib.check("vrl_gemm_nt_plan", planned)
    parts = planned if k_parts is None else int(k_parts)
    work = torch.empty(parts * NX * NY, dtype=torch.float32, device=dev) if parts > 1 else None
    with torch.cuda.device(dev):
        st = lib.vrl_gemm(x.data_ptr(), y.data_ptr(), code, NX, NY, K, x.stride(0), y.stride(0), 1 if x_t else 0,
                          1 if y_t else 0, out.data_ptr(), out.stride(0), 1 if accumulate else 0, parts,
                          None if work is None else work.data_ptr(), _lib.stream_ptr(dev))
    _lib.check("vrl_gemm", st)
    counters["gemm"] += 1
    return out


def gemm_nt(x: torch.Tensor, y: torch.Tensor, out: Optional[torch.Tensor] = None, accumulate: bool = False,
            k_parts: Optional[int] = None) -> torch.Tensor:
    """``gemm`` for two row-major operands: ``out[j, i] (+)= sum_k y[j, k] * x[i, k]``."""
    return gemm(x, y, False, False, out=out, accumulate=accumulate, k_parts=k_parts)
