"""Layout steps either side of the scoring path, on the GPU.

``roll_labels`` restates the one-line label construction of the reference's engine
(verl/workers/engine/fsdp/transformer_impl.py:1177); ``expand_per_sequence`` builds the per-token temperature from the
per-sample one (verl/utils/torch_functional.py:989-1011); ``response_slice`` replaces the
per-sequence Python loop of verl/workers/utils/padding.py:97-141 with one kernel launch;
``transpose_2d`` is the bit-exact transposed copy the LM-head backward uses to give the library GEMM
operands that are contiguous along the contraction axis.
"""

from __future__ import annotations

from typing import Optional

import torch

from . import _lib
from . import errors as _errors

__all__ = ["roll_labels", "expand_per_sequence", "response_slice", "response_from_packed", "transpose_2d"]


def roll_labels(input_ids_rmpad: torch.Tensor) -> torch.Tensor:
    """Labels of the packed token axis: every position is scored against the NEXT token id.

    The roll is over the whole packed axis, so the last token of a sequence gets the first id of the next
    one; that position is never part of a response slice. Under sequence parallelism it must happen before
    the per-rank split (tests/models/test_fused_kernels_ulysses_sp_on_cpu.py:69-90 in the reference).
    """
    return torch.roll(input_ids_rmpad, shifts=-1, dims=-1)


def _slice_messages(what: str, n_tokens: int) -> dict:
    return {
        _lib.VRL_FLAG_SEQ_RANGE: (ValueError, f"{what}: cu_seqlens is not a partition of the {n_tokens} values "
                                  "(it must start at 0, never decrease and end at the number of values)"),
        _lib.VRL_FLAG_SLICE_RANGE: (ValueError, f"{what}: a sequence has no prompt token, or a response length "
                                    "outside its bounds"),
    }


def _rows(values: torch.Tensor, what: str):
    """-> (contiguous values, bytes per row of the leading axis, trailing shape)."""
    if not values.is_cuda:
        raise RuntimeError(f"values is on {values.device}; verl_amd only runs on the GPU, it has no CPU implementation")
    if values.dim() < 1:
        raise ValueError(f"{what}: values must be (total_nnz, *), got a scalar")
    if values.is_nested or values.is_sparse:
        raise TypeError(f"{what}: values must be a dense tensor (pass a nested tensor's .values())")
    trailing = tuple(values.shape[1:])
    inner = 1
    for d in trailing:
        inner *= int(d)
    if inner == 0:
        raise ValueError(f"{what}: values has an empty trailing dimension, shape {tuple(values.shape)}")
    return values.contiguous(), inner * values.element_size(), trailing


def response_slice(values: torch.Tensor, cu_seqlens: torch.Tensor, response_lens: torch.Tensor,
                   max_response_len: Optional[int] = None, check=None) -> torch.Tensor:
    """Packed per-token ``values`` (total_nnz, *) -> ``(B, max_response_len, *)`` block of response positions, in
    ``values``' dtype (any: the rows are copied bit for bit) with trailing dimensions kept as they are, like the
    reference's ``no_padding_2_padding`` (verl/workers/utils/padding.py:100-101, :133-138).

    Row b holds ``values[end_b - r_b - 1 : end_b - 1]`` (model output is shifted left by one token) padded
    with zeros, where ``end_b = cu_seqlens[b+1]`` and ``r_b = response_lens[b]``. Like the reference it
    requires every sequence to have a prompt token and ``cu_seqlens`` to partition ``values``
    (verl/workers/utils/padding.py:129-130); a violation writes a zero row and raises ValueError, when and how is
    ``check``'s business (verl_amd.errors: None = the mode in force, True = now, False = never, "deferred").
    With ``max_response_len`` given the call does not synchronise with the device; without it the longest response is
    read back first, as the reference does (``response_lens.max().item()``, padding.py:117).
    """
    _errors.poll()
    v, row_bytes, trailing = _rows(values, "response_slice")
    dev = v.device
    cu = cu_seqlens.to(device=dev, dtype=torch.int64).contiguous()
    rl = response_lens.to(device=dev, dtype=torch.int64).contiguous()
    B = rl.numel()
    if cu.numel() != B + 1:
        raise ValueError(f"cu_seqlens must have B+1 = {B + 1} entries, got {cu.numel()}")
    if max_response_len is None or max_response_len < 0:
        max_response_len = int(rl.max().item()) if B > 0 else 0
    T = int(max_response_len)
    out = torch.empty((B, T) + trailing, dtype=v.dtype, device=dev)
    flag = torch.zeros(1, dtype=torch.int32, device=dev)
    lib = _lib.load()
    with torch.cuda.device(dev):
        st = lib.vrl_response_slice(v.data_ptr() if v.numel() else None, row_bytes, cu.data_ptr(), rl.data_ptr(), B,
                                    v.shape[0], T, out.data_ptr(), flag.data_ptr(), _lib.stream_ptr(dev))
    _lib.check("vrl_response_slice", st)
    if B > 0 and T > 0:
        _errors.report(flag, _slice_messages("response_slice", v.shape[0]), check)
    return out


def response_from_packed(values: torch.Tensor, cu_seqlens: torch.Tensor, response_lens: torch.Tensor,
                         check=None, total_response_tokens: Optional[int] = None):
    """Packed per-token ``values`` (total_nnz, *) -> (packed response values ``(sum(response_lens), *)`` in the same
    dtype, their ``cu_seqlens`` ``(B+1,)`` int64): sequence b contributes ``values[end_b - r_b - 1 : end_b - 1]``. The
    packed counterpart of ``response_slice``; the reference does it with a Python loop and ``as_nested_tensor``
    (verl/workers/utils/padding.py:194-210), to whose ``(values, offsets)`` pair the two results correspond.
    ``total_response_tokens`` (= ``sum(response_lens)``, which sizes the result) spares the call its one read-back from
    the device when the caller knows it; a value that is not the sum is reported like any other inconsistent offsets."""
    v, row_bytes, trailing = _rows(values, "response_from_packed")
    dev = v.device
    cu = cu_seqlens.to(device=dev, dtype=torch.int64).contiguous()
    rl = response_lens.to(device=dev, dtype=torch.int64).contiguous()
    B = rl.numel()
    if cu.numel() != B + 1:
        raise ValueError(f"cu_seqlens must have B+1 = {B + 1} entries, got {cu.numel()}")
    out_cu = torch.zeros(B + 1, dtype=torch.int64, device=dev)
    if B > 0:
        out_cu[1:] = torch.cumsum(rl.clamp(min=0), 0)
    if total_response_tokens is not None:
        total = int(total_response_tokens)
        if total < 0:
            raise ValueError(f"total_response_tokens must not be negative, got {total}")
    else:
        total = int(out_cu[-1].item()) if B > 0 else 0
    out = torch.empty((total,) + trailing, dtype=v.dtype, device=dev)
    flag = torch.zeros(1, dtype=torch.int32, device=dev)
    lib = _lib.load()
    with torch.cuda.device(dev):
        st = lib.vrl_response_pack(v.data_ptr() if v.numel() else None, row_bytes, cu.data_ptr(), rl.data_ptr(),
                                   out_cu.data_ptr(), B, v.shape[0], total, out.data_ptr() if total > 0 else None,
                                   flag.data_ptr(), _lib.stream_ptr(dev))
    _lib.check("vrl_response_pack", st)
    if B > 0:
        _errors.report(flag, _slice_messages("response_from_packed", v.shape[0]), check)
    return out, out_cu


def transpose_2d(x: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Contiguous ``(cols, rows)`` copy of the 2-D tensor ``x`` (``rows, cols``; bf16, fp16 or fp32; any row
    stride, unit column stride), bit for bit equal to ``x.t().contiguous()``. ``out`` may supply the result
    buffer (same dtype, shape ``(cols, rows)``, unit column stride)."""
    if not x.is_cuda:
        raise RuntimeError(f"x is on {x.device}; verl_amd only runs on the GPU, it has no CPU implementation")
    if x.dim() != 2:
        raise ValueError(f"transpose_2d needs a 2-D tensor, got shape {tuple(x.shape)}")
    if x.element_size() not in (2, 4) or x.is_complex():
        raise TypeError(f"transpose_2d handles 2- and 4-byte element types, got {x.dtype}")
    rows, cols = x.shape
    if cols > 1 and x.stride(1) != 1 or (rows > 1 and x.stride(0) < cols):
        x = x.contiguous()
    if out is None:
        out = torch.empty((cols, rows), dtype=x.dtype, device=x.device)
    elif (out.dtype != x.dtype or tuple(out.shape) != (cols, rows) or out.device != x.device
          or (rows > 1 and out.stride(1) != 1) or (cols > 1 and out.stride(0) < rows)):
        raise ValueError("transpose_2d: out must be a (cols, rows) tensor of x's dtype and device with unit column stride")
    lib = _lib.load()
    with torch.cuda.device(x.device):
        st = lib.vrl_transpose(x.data_ptr(), x.element_size(), rows, cols, x.stride(0) if rows > 1 else cols,
                               out.data_ptr(), out.stride(0) if cols > 1 else rows,
                               _lib.stream_ptr(x.device))
    _lib.check("vrl_transpose", st)
    return out


def expand_per_sequence(values: torch.Tensor, cu_seqlens: torch.Tensor, total_nnz: Optional[int] = None,
                        check=None) -> torch.Tensor:
    """One value per sequence ``(B,)`` -> one per token of the packed batch ``(total_nnz,)`` fp32: token t gets
    ``values[b]`` for ``cu_seqlens[b] <= t < cu_seqlens[b+1]``. The values of the reference's
    ``expand_as_nested(temperature, input_ids)`` (verl/utils/torch_functional.py:989-1011,
    ``repeat_interleave`` by the sequence lengths), which is how the engine builds the per-token temperature
    (verl/workers/engine/fsdp/transformer_impl.py:1158-1162).

    ``total_nnz`` (= ``cu_seqlens[-1]``, which sizes the result) spares the call its read-back from the device when
    the caller knows it; offsets that are not a partition of ``[0, total_nnz]`` raise ValueError as ``check`` says
    (verl_amd.errors)."""
    _errors.poll()
    if values.dim() != 1:
        raise ValueError(f"expand_per_sequence: values must have one entry per sequence, got shape {tuple(values.shape)}")
    if not values.is_cuda:
        raise RuntimeError(f"values is on {values.device}; verl_amd only runs on the GPU, it has no CPU implementation")
    dev = values.device
    v = values.to(dtype=torch.float32).contiguous()
    cu = cu_seqlens.to(device=dev, dtype=torch.int64).contiguous()
    B = v.numel()
    if cu.dim() != 1 or cu.numel() != B + 1:
        raise ValueError(f"expand_per_sequence: cu_seqlens must have B+1 = {B + 1} entries, got {tuple(cu.shape)}")
    n = int(cu[-1].item()) if total_nnz is None else int(total_nnz)
    if n < 0:
        raise ValueError("expand_per_sequence: total_nnz must not be negative")
    out = torch.empty(n, dtype=torch.float32, device=dev)
    flag = torch.zeros(1, dtype=torch.int32, device=dev)
    lib = _lib.load()
    with torch.cuda.device(dev):
        st = lib.vrl_expand_per_sequence(v.data_ptr() if B else None, cu.data_ptr(), B, n,
                                         out.data_ptr() if n else None, flag.data_ptr(), _lib.stream_ptr(dev))
    _lib.check("vrl_expand_per_sequence", st)
    if B > 0:
        _errors.report(flag, {_lib.VRL_FLAG_SEQ_RANGE: (ValueError, f"expand_per_sequence: cu_seqlens is not a "
                              f"partition of the {n} tokens (it must start at 0, never decrease and end there)")}, check)
    return out
