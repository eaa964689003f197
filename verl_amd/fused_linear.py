"""LM head + scoring without ever holding the full ``(tokens, vocab)`` logits.

Same call as the reference's ``FusedLinearForPPO`` (verl/utils/experimental/torch_functional.py:211-231):
``(hidden_states, vocab_weights, input_ids, temperature) -> (log_probs fp32, entropy)``, chunked over
tokens. Per chunk the projection ``hidden @ W^T`` is one library GEMM (torch.matmul, i.e. hipBLASLt)
into a reusable ``(chunk, vocab)`` buffer, and everything after it is the HIP row kernel: forward
``vrl_rowscore`` (one pass over the chunk's logits), backward ``vrl_rowscore_backward`` writing the
gradient over the recomputed logits in place, followed by the two GEMMs for ``d hidden`` and ``d W``.
The reference does the post-GEMM part with ~10 torch ops per chunk (softmax, logsumexp, log_softmax,
gather, scatter, ...; :27-79); peak extra memory here is one ``(chunk, vocab)`` buffer.
"""

from __future__ import annotations

import os
from typing import Optional

import torch

from . import _lib
from . import errors as _errors
from . import gemm as _gemm
from .layout import transpose_2d
from .torch_functional import _DTYPE_CODES, _ptr

__all__ = ["FusedLinearForPPO", "fused_linear_for_ppo", "linear_cross_entropy", "lm_head_score_mfma",
           "DEFAULT_CHUNK_TOKENS"]

# The reference's default is 512 tokens per chunk. On a 288 GB part a (4096, 152064) bf16 buffer is 1.2 GB, the
# projection reaches 1.4 PFLOP/s instead of 0.86 at 512, and the weight gradient is accumulated 8x less often.
DEFAULT_CHUNK_TOKENS = 4096

# Which matrix products are this package's own kernels.
#   "library": every product is torch.matmul (hipBLASLt); the row kernels run over the chunk buffer.
#   "mfma":    every step that has a hand-written matrix-core kernel uses it: the forward without gradients is one
#              kernel that never writes logits (vrl_lmhead_score), the backward forms the logits again and writes their
#              gradient from registers (vrl_lmhead_dlogits) and forms d hidden with vrl_gemm_nt; d W stays a library
#              product (the hand-written one needs a transposed copy of the gradient buffer).
#   "auto":    each step by what is measured fastest on MI355X at 8192 x 3584 -> 152064 bf16, as long as the forward is the
#              same arithmetic with and without gradients: library GEMM + row kernel for the forward; in the backward
#              vrl_lmhead_dlogits (3.46 ms per 4096 tokens against 3.53 ms for the library GEMM + row backward) and
#              vrl_gemm_nt for d hidden (3.36 against 3.73 ms), library for d W. The single forward kernel is
#              as fast as the library GEMM + row kernel (6.52 against 6.53 ms) and needs no buffer, but it keeps the
#              logits in fp32 where the GEMM rounds them to the operand type: old log-probs from it (no gradients)
#              and new ones from the GEMM (gradients) would differ by that rounding, a policy ratio other than 1 before
#              any update. "mfma" accepts that; "auto" does not.
# The environment variable and the ``kernels`` argument select; shapes a hand-written kernel does not take go to the library.
DEFAULT_KERNELS = os.environ.get("VERL_AMD_LMHEAD_KERNELS", "auto")


def _mfma_takes(hidden: torch.Tensor, weight: torch.Tensor, n_tokens: int) -> bool:
    """Shape rules of vrl_lmhead_score / vrl_lmhead_dlogits (include/vrl.h)."""
    V, K = weight.shape
    return (hidden.dtype in (torch.bfloat16, torch.float16) and n_tokens >= 256 and V >= 256 and V % 8 == 0
            and K % 64 == 0 and hidden.stride(-1) == 1 and weight.stride(-1) == 1
            and hidden.stride(0) % 8 == 0 and weight.stride(0) % 8 == 0
            and V * weight.stride(0) * 2 < (1 << 32) and n_tokens * hidden.stride(0) * 2 < (1 << 32)
            and hidden.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0)


# From this many tokens on, one transposed copy of the weight per backward (0.44 ms for 152064 x 3584 bf16) is
# repaid by the faster `d hidden` product.
_WEIGHT_TRANSPOSE_MIN_TOKENS = 2048


def _score_chunk(lib, logits, labels, temp, lp, h, lse, flag, stream):
    n, V = logits.shape
    st = lib.vrl_rowscore(logits.data_ptr(), _DTYPE_CODES[logits.dtype], n, V, logits.stride(0) if n > 1 else V,
                          labels.data_ptr(), _ptr(temp), lp.data_ptr(), h.data_ptr(), None, lse.data_ptr(),
                          flag.data_ptr(), stream)
    _lib.check("vrl_rowscore", st)


def _d_hidden(grad_logits, weight, weight_t, out, own_kernel):
    """out = grad_logits @ weight: this package's matrix-core kernel (``vrl_gemm_nt``) when asked for and the shapes
    allow, the library otherwise (with the transposed copy of the weight when there is one: both operands contiguous
    along the vocabulary)."""
    if own_kernel and weight_t is not None and _gemm.gemm_nt_takes(weight_t, grad_logits) and out.stride(0) % 4 == 0:
        _gemm.gemm_nt(weight_t, grad_logits, out=out)
    else:
        torch.matmul(grad_logits, weight if weight_t is None else weight_t.t(), out=out)


class _FusedLinearForPPOFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, hidden, weight, input_ids, temperature, chunk_size, keep_logits, kernels):
        ctx.set_materialize_grads(False)
        ctx.kernels = kernels
        T, D = hidden.shape
        V = weight.shape[0]
        dev = hidden.device
        f32 = dict(dtype=torch.float32, device=dev)
        lp = torch.empty(T, **f32)
        h = torch.empty(T, **f32)
        lse = torch.empty(T, **f32)
        flag = torch.zeros(1, dtype=torch.int32, device=dev)
        temp = None if temperature == 1.0 else torch.full((min(chunk_size, max(T, 1)),), float(temperature), **f32)
        lib = _lib.load()
        keep = bool(keep_logits) and T > 0 and (ctx.needs_input_grad[0] or ctx.needs_input_grad[1])
        rows = T if keep else min(chunk_size, max(T, 1))
        buf = torch.empty((rows, V), dtype=hidden.dtype, device=dev)
        with torch.cuda.device(dev):
            stream = _lib.stream_ptr(dev)
            for lo in range(0, T, chunk_size):
                hi = min(lo + chunk_size, T)
                logits = buf[lo:hi] if keep else buf[: hi - lo]
                torch.matmul(hidden[lo:hi], weight.t(), out=logits)
                _score_chunk(lib, logits, input_ids[lo:hi], None if temp is None else temp[: hi - lo],
                             lp[lo:hi], h[lo:hi], lse[lo:hi], flag, stream)
        if T > 0:
            _errors.report(flag, {_lib.VRL_FLAG_LABEL_OOB: (IndexError, f"fused_linear_for_ppo: an input id is outside [0, {V})")})
        ctx.save_for_backward(hidden, weight, input_ids, lse, h)
        ctx.temperature = float(temperature)
        ctx.chunk_size = int(chunk_size)
        ctx.kept_logits = buf if keep else None
        return lp, h.clone()

    @staticmethod
    def backward(ctx, g_lp: Optional[torch.Tensor], g_h: Optional[torch.Tensor]):
        hidden, weight, input_ids, lse, h = ctx.saved_tensors
        if g_lp is None and g_h is None:
            return None, None, None, None, None, None, None
        kept = ctx.kept_logits
        if kept is not None:
            ctx.kept_logits = None        # the gradient is written over them: they serve one backward
        elif getattr(ctx, "kept_consumed", False):
            raise RuntimeError("fused_linear_for_ppo(keep_logits=True): the kept logits were overwritten by the first "
                               "backward; run the forward again, or use keep_logits=False")
        ctx.kept_consumed = kept is not None
        T, D = hidden.shape
        V = weight.shape[0]
        dev = hidden.device
        chunk = ctx.chunk_size
        f32 = dict(dtype=torch.float32, device=dev)
        gl = None if g_lp is None else g_lp.to(torch.float32).contiguous()
        gh = None if g_h is None else g_h.to(torch.float32).contiguous()
        temp = None if ctx.temperature == 1.0 else torch.full((min(chunk, max(T, 1)),), ctx.temperature, **f32)
        need_dh, need_dw = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        d_hidden = torch.empty_like(hidden) if need_dh else None
        d_weight = (torch.empty_like(weight) if kept is not None else torch.zeros_like(weight)) if need_dw else None
        lib = _lib.load()
        buf = kept if kept is not None else torch.empty((min(chunk, max(T, 1)), V), dtype=hidden.dtype, device=dev)
        dt = _DTYPE_CODES[hidden.dtype]
        # For 16-bit operands the library GEMM is 25-35 % faster when both operands are contiguous along the
        # contraction axis (vocab for `d hidden`, tokens for `d W`); fp32 runs at the fp32 matrix peak either way.
        half = hidden.element_size() == 2
        weight_t = transpose_2d(weight) if (half and need_dh and T >= _WEIGHT_TRANSPOSE_MIN_TOKENS) else None
        with torch.cuda.device(dev):
            stream = _lib.stream_ptr(dev)
            for lo in range(0, T, chunk):
                hi = min(lo + chunk, T)
                n = hi - lo
                if kept is None and ctx.kernels != "library" and _mfma_takes(hidden[lo:hi], weight, n) and V % 8 == 0:
                    # logits formed again on the matrix cores, their gradient written straight into the buffer
                    logits = buf[:n]
                    st = lib.vrl_lmhead_dlogits(
                        hidden[lo:hi].data_ptr(), weight.data_ptr(), dt, n, V, D, hidden.stride(0), weight.stride(0),
                        input_ids[lo:hi].data_ptr(), None if temp is None else temp.data_ptr(), lse[lo:hi].data_ptr(),
                        h[lo:hi].data_ptr(), None if gl is None else gl[lo:hi].data_ptr(),
                        None if gh is None else gh[lo:hi].data_ptr(), lib.vrl_lmhead_plan(n, V), logits.data_ptr(),
                        logits.stride(0), stream)
                    _lib.check("vrl_lmhead_dlogits", st)
                    if need_dh:
                        _d_hidden(logits, weight, weight_t, d_hidden[lo:hi], True)
                    if need_dw:
                        d_weight.addmm_(logits.t(), transpose_2d(hidden[lo:hi]).t() if half else hidden[lo:hi])
                    continue
                if kept is not None:
                    logits = buf[lo:hi]
                else:
                    logits = buf[:n]
                    torch.matmul(hidden[lo:hi], weight.t(), out=logits)
                st = lib.vrl_rowscore_backward(
                    logits.data_ptr(), dt, n, V, logits.stride(0) if n > 1 else V, input_ids[lo:hi].data_ptr(),
                    None if temp is None else temp.data_ptr(), lse[lo:hi].data_ptr(), h[lo:hi].data_ptr(),
                    None if gl is None else gl[lo:hi].data_ptr(), None if gh is None else gh[lo:hi].data_ptr(),
                    logits.data_ptr(), logits.stride(0) if n > 1 else V, stream)   # gradient over the logits, in place
                _lib.check("vrl_rowscore_backward", st)
                if kept is not None:
                    continue
                if need_dh:
                    _d_hidden(logits, weight, weight_t, d_hidden[lo:hi], ctx.kernels != "library")
                if need_dw:
                    d_weight.addmm_(logits.t(), transpose_2d(hidden[lo:hi]).t() if half else hidden[lo:hi])
            if kept is not None:
                # the gradient over all tokens' logits is in `kept`: one product each, nothing to accumulate
                if need_dh:
                    _d_hidden(kept, weight, weight_t, d_hidden, ctx.kernels != "library")
                if need_dw:
                    torch.matmul(kept.t(), transpose_2d(hidden).t() if half else hidden, out=d_weight)
        return d_hidden, d_weight, None, None, None, None, None


def fused_linear_for_ppo(hidden_states: torch.Tensor, vocab_weights: torch.Tensor, input_ids: torch.Tensor,
                         temperature: float = 1.0, chunk_size: int = DEFAULT_CHUNK_TOKENS, keep_logits: bool = False,
                         kernels: Optional[str] = None):
    """(log_probs fp32, entropy fp32) of ``softmax((hidden_states @ vocab_weights.T) / temperature)`` at ``input_ids``.

    ``hidden_states`` is ``(tokens, hidden)`` or ``(batch, seq, hidden)`` with ``input_ids`` of the matching leading
    shape; ``vocab_weights`` is ``(vocab, hidden)``; both bf16, fp16 or fp32 on the GPU. Differentiable with respect
    to both. ``chunk_size`` tokens are projected at a time (one reusable ``(chunk_size, vocab)`` buffer); the result
    depends on it only through the order in which the library sums a product of that height; the default is sized for
    this GPU rather than the reference's 512.

    ``keep_logits=True`` trades memory for time when gradients are needed: the forward keeps all
    ``tokens x vocab`` logits (2.5 GB for 8192 x 152064 bf16), the backward writes their gradient over them instead of
    projecting again and forms ``d hidden`` and ``d W`` with one product each. Such a graph can be differentiated once.

    ``kernels`` chooses which matrix products are this package's own kernels: ``"library"`` (none: torch.matmul
    throughout), ``"mfma"`` (all that exist: no buffer at all when no gradient is recorded, a backward that forms the
    logits again and writes their gradient straight from registers, ``d hidden`` from ``vrl_gemm_nt``; ``d W`` stays a
    library product) or ``"auto"`` (each step by what measures fastest on MI355X while log-probs computed with and
    without gradients stay bit-identical: a library product for the forward's logits, this package's kernels for the
    backward's gradient of the logits and ``d hidden``); None takes ``DEFAULT_KERNELS`` ("auto" unless ``VERL_AMD_LMHEAD_KERNELS`` says
    otherwise).
    """
    kernels = DEFAULT_KERNELS if kernels is None else kernels
    if kernels not in ("auto", "library", "mfma"):
        raise ValueError(f"kernels must be 'auto', 'library' or 'mfma', got {kernels!r}")
    if not hidden_states.is_cuda or not vocab_weights.is_cuda:
        raise RuntimeError("fused_linear_for_ppo: tensors must be on the GPU; verl_amd has no CPU implementation")
    if hidden_states.dtype != vocab_weights.dtype or hidden_states.dtype not in _DTYPE_CODES:
        raise TypeError(f"fused_linear_for_ppo: hidden {hidden_states.dtype} / weights {vocab_weights.dtype} must share "
                        "one of float32, bfloat16, float16")
    if hidden_states.dim() not in (2, 3):
        raise ValueError(f"fused_linear_for_ppo: hidden_states must be 2-D or 3-D, got shape {tuple(hidden_states.shape)}")
    if tuple(input_ids.shape) != tuple(hidden_states.shape[:-1]):
        raise ValueError(f"fused_linear_for_ppo: input_ids shape {tuple(input_ids.shape)} does not match "
                         f"hidden_states {tuple(hidden_states.shape)}")
    if vocab_weights.dim() != 2 or vocab_weights.shape[1] != hidden_states.shape[-1]:
        raise ValueError("fused_linear_for_ppo: vocab_weights must be (vocab, hidden)")
    if int(chunk_size) <= 0:
        raise ValueError(f"chunk_size must be positive, got {chunk_size}")
    if input_ids.dtype.is_floating_point or input_ids.dtype == torch.bool:
        raise TypeError(f"fused_linear_for_ppo: input_ids must be an integer tensor, got {input_ids.dtype}")
    _errors.poll()
    lead = hidden_states.shape[:-1]
    h2 = hidden_states.reshape(-1, hidden_states.shape[-1]).contiguous()
    # the kernels read the ids through a raw device pointer: they must live next to the hidden states
    ids = input_ids.reshape(-1).to(device=h2.device, dtype=torch.int64).contiguous()
    w2 = vocab_weights.contiguous()
    needs_grad = torch.is_grad_enabled() and (h2.requires_grad or w2.requires_grad)
    if kernels == "mfma" and not needs_grad and _mfma_takes(h2, w2, h2.shape[0]):
        lp, ent = lm_head_score_mfma(h2, w2, ids, float(temperature))
        return lp.reshape(lead), ent.reshape(lead)
    lp, ent = _FusedLinearForPPOFunction.apply(h2, w2, ids, float(temperature), int(chunk_size), bool(keep_logits),
                                               kernels)
    return lp.reshape(lead), ent.reshape(lead)


def lm_head_score_mfma(hidden_states: torch.Tensor, vocab_weights: torch.Tensor, input_ids: torch.Tensor,
                       temperature=1.0, n_splits: Optional[int] = None):
    """Forward-only (log_probs, entropy), fp32, from one hand-written matrix-core kernel that never writes logits
    (``vrl_lmhead_score``): the counterpart of the reference's Triton ``efficient_entropy_forward``
    (verl/utils/kernel/kernels.py:531-756). bf16 or fp16 operands, at least 256 tokens and 256 vocabulary entries,
    hidden size a multiple of 64. ``temperature`` is a float or one value per token. The logits are kept in fp32
    (a GEMM that writes them rounds them to the operand type first), so results are slightly closer to the
    all-fp32 value than a path that writes them. On MI355X it takes as long as the library GEMM + row kernel (6.5 ms at
    8192 x 3584 -> 152064) and needs no logits buffer at all; ``fused_linear_for_ppo(kernels="mfma")`` uses it when no
    gradient is recorded.
    """
    if not hidden_states.is_cuda or not vocab_weights.is_cuda:
        raise RuntimeError("lm_head_score_mfma: tensors must be on the GPU; verl_amd has no CPU implementation")
    if hidden_states.dtype != vocab_weights.dtype or hidden_states.dtype not in (torch.bfloat16, torch.float16):
        raise TypeError(f"lm_head_score_mfma: hidden {hidden_states.dtype} / weights {vocab_weights.dtype} must both be "
                        "bfloat16 or both float16")
    if torch.is_grad_enabled() and (hidden_states.requires_grad or vocab_weights.requires_grad):
        raise NotImplementedError("lm_head_score_mfma is forward-only; use fused_linear_for_ppo when gradients are needed")
    if hidden_states.dim() not in (2, 3) or vocab_weights.dim() != 2 or vocab_weights.shape[1] != hidden_states.shape[-1]:
        raise ValueError("lm_head_score_mfma: hidden_states must be (tokens, hidden) or (batch, seq, hidden) and "
                         "vocab_weights (vocab, hidden)")
    if tuple(input_ids.shape) != tuple(hidden_states.shape[:-1]):
        raise ValueError(f"lm_head_score_mfma: input_ids shape {tuple(input_ids.shape)} does not match hidden_states "
                         f"{tuple(hidden_states.shape)}")
    lead = hidden_states.shape[:-1]
    h = hidden_states.detach().reshape(-1, hidden_states.shape[-1]).contiguous()
    w = vocab_weights.detach().contiguous()
    T, K = h.shape
    V = w.shape[0]
    if T < 256 or V < 256 or K % 64 != 0:
        raise ValueError(f"lm_head_score_mfma needs >= 256 tokens, >= 256 vocabulary entries and a hidden size that is "
                         f"a multiple of 64; got {T}, {V}, {K}")
    dev = h.device
    ids = input_ids.reshape(-1).to(device=dev, dtype=torch.int64).contiguous()
    temp = None
    if isinstance(temperature, torch.Tensor):
        temp = temperature.to(device=dev, dtype=torch.float32).reshape(-1)
        temp = temp.expand(T).contiguous() if temp.numel() == 1 else temp.contiguous()
        if temp.numel() != T:
            raise ValueError(f"temperature has {temp.numel()} entries, expected one per token ({T})")
    elif float(temperature) != 1.0:
        temp = torch.full((T,), float(temperature), dtype=torch.float32, device=dev)
    lib = _lib.load()
    splits = lib.vrl_lmhead_plan(T, V) if n_splits is None else int(n_splits)
    f32 = dict(dtype=torch.float32, device=dev)
    partials = torch.empty(T * splits * 4, **f32)
    lp = torch.empty(T, **f32)
    ent = torch.empty(T, **f32)
    flag = torch.zeros(1, dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        st = lib.vrl_lmhead_score(h.data_ptr(), w.data_ptr(), _DTYPE_CODES[h.dtype], T, V, K, h.stride(0), w.stride(0),
                                  ids.data_ptr(), _ptr(temp), splits, partials.data_ptr(), lp.data_ptr(), ent.data_ptr(),
                                  None, flag.data_ptr(), _lib.stream_ptr(dev))
    _lib.check("vrl_lmhead_score", st)
    _errors.report(flag, {_lib.VRL_FLAG_LABEL_OOB: (IndexError, f"lm_head_score_mfma: an input id is outside [0, {V})")})
    return lp.reshape(lead), ent.reshape(lead)


def linear_cross_entropy(hidden: torch.Tensor, weight: torch.Tensor, labels: torch.Tensor, temperature: float = 1.0,
                         reduction: str = "none", dist_process_group=None):
    """Same call as the reference's Triton-backed ``linear_cross_entropy``
    (verl/utils/kernel/linear_cross_entropy.py:38-119): ``hidden`` ``(..., hidden_size)``, ``weight``
    ``(vocab, hidden_size)``, ``labels`` ``(...)`` -> ``(logprobs, entropy)``, both fp32 over the flattened tokens.
    ``reduction`` ("none", "sum", "mean") applies to the log-probs only, as there (verl/utils/kernel/kernels.py:431-438);
    the entropy stays per token. Served by ``fused_linear_for_ppo``. A vocabulary sharded over a process group is not
    part of this one-GPU build and raises."""
    if dist_process_group is not None:
        raise NotImplementedError("linear_cross_entropy: a vocabulary sharded over a process group is not supported")
    if not isinstance(temperature, float):
        raise TypeError(f"temperature must be a float, but got {type(temperature)}")
    red = str(reduction).lower()
    if red not in ("none", "sum", "mean"):
        raise ValueError(f"Invalid reduction: {reduction}")
    h2 = hidden.reshape(-1, hidden.shape[-1])
    lp, ent = fused_linear_for_ppo(h2, weight, labels.reshape(-1), temperature)
    if red == "sum":
        lp = lp.sum()
    elif red == "mean":
        lp = lp.mean()
    return lp, ent


class FusedLinearForPPO(torch.nn.Module):
    """Module form, constructed and called like verl's (verl/utils/experimental/torch_functional.py:211-231)."""

    def __init__(self, chunk_size: int = DEFAULT_CHUNK_TOKENS, keep_logits: bool = False, kernels: Optional[str] = None):
        super().__init__()
        self.chunk_size = chunk_size
        self.keep_logits = keep_logits
        self.kernels = kernels

    def forward(self, hidden_states, vocab_weights, input_ids, temperature: float = 1.0):
        return fused_linear_for_ppo(hidden_states, vocab_weights, input_ids, temperature, self.chunk_size,
                                    self.keep_logits, self.kernels)
