"""LM head + scoring without ever holding the full ``(tokens, vocab)`` logits.

Same call as the reference's ``FusedLinearForPPO`` (verl/utils/experimental/torch_functional.py:211-231):
``(hidden_states, vocab_weights, input_ids, temperature) -> (log_probs fp32, entropy)``.

Default path (bf16 / fp16 models): the forward is one hand-written matrix-core kernel that folds the logits into the
softmax state as it forms them and never writes them (``vrl_lmhead_score``); the backward walks the tokens in chunks, forms
each chunk's logits again on the matrix cores and writes their gradient into a reusable ``(chunk, vocab)`` buffer
(``vrl_lmhead_dlogits``), then forms ``d hidden`` and ``d W`` with ``vrl_gemm``, which reads the weight, the hidden states
and the gradient buffer as they lie (no transposed copies). No library GEMM runs. Peak extra memory is that one buffer, in
the backward only. With ``keep_logits=True`` the same forward kernel also writes the logits from its registers, and the
backward turns them into their gradient in place (``vrl_rowscore_backward``) and forms each of the two products once with
``vrl_gemm``: a quarter fewer matrix-core flops for ``tokens x vocab`` elements of memory, still without a library GEMM.

Library path (``kernels="library"``, fp32 models, models the kernels' shape rules do not take): per chunk the projection
``hidden @ W^T`` is one library GEMM (torch.matmul, i.e. hipBLASLt) into the buffer, and everything after it is the HIP row
kernel: forward ``vrl_rowscore`` (one pass over the chunk's logits), backward ``vrl_rowscore_backward`` writing the gradient
over the recomputed logits in place, followed by the two GEMMs. The reference does the post-GEMM part with ~10 torch ops per
chunk (softmax, logsumexp, log_softmax, gather, scatter, ...; :27-79). fp32 models are served by the library on purpose:
the fp32 matrix rate of the part (157 TFLOP/s) is what the library already delivers, and no model in verl's recipes runs
its LM head in fp32.
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
#   "auto" (default) and "mfma" (the same today): every step runs this package's own matrix-core kernel.
#              The forward is one kernel (vrl_lmhead_score: 6.0-6.25 ms at 8192 x 3584 -> 152064 bf16 against 6.5 ms for the
#              library GEMM + row kernel, logits kept in fp32), with and without gradients and whatever the number of
#              tokens, and a token's results are the same bits whatever else the call holds, so that old (no-grad) and new
#              (grad) log-probs of the same weights are bit-identical for any micro-batch sizes. It never writes the
#              logits unless keep_logits=True asks for them (they then leave the kernel's registers rounded once).
#              Without kept logits the backward forms them again and writes their gradient from registers
#              (vrl_lmhead_dlogits, 3.2-3.3 ms per 4096 tokens against 3.5 ms for the library GEMM + row backward); with
#              kept logits vrl_rowscore_backward turns them into their gradient in place. d hidden and d W come from
#              vrl_gemm, which reads W, the hidden states and the gradient buffer in place: the contraction of either
#              product runs over rows of its operands, and the kernel takes such operands through transposing LDS reads.
#              Per 4096-token chunk d hidden takes 3.1 ms against 3.75 ms for the library (which also wants a transposed
#              copy of W); d W 3.4 / 3.7 ms stored / accumulated against 3.3 / 3.5 ms for the library on transposed copies
#              (which also needs the copies and a zero fill of d W).
# The environment variable and the ``kernels`` argument select; models the kernels do not take (fp32, a hidden size that is
# not a multiple of 64, fewer than 256 or not a multiple of 8 vocabulary entries) go to the library.
DEFAULT_KERNELS = os.environ.get("VERL_AMD_LMHEAD_KERNELS", "auto")

# Into how many shares per 256-token block the forward kernel's work is dealt. None lets the library plan per call (the
# number that finishes soonest on this part's CUs). Results do not depend on it: the kernel hands a token's softmax state
# over at fixed places of the vocabulary, and the states are merged in a fixed order. `forward_splits` / the environment
# variable VERL_AMD_LMHEAD_SPLITS (1..64) are for measurements.
_env_splits = os.environ.get("VERL_AMD_LMHEAD_SPLITS", "")
DEFAULT_FORWARD_SPLITS = int(_env_splits) if _env_splits.strip() else None


def _mfma_takes_model(hidden: torch.Tensor, weight: torch.Tensor) -> bool:
    """Whether the matrix-core LM-head kernels take this model (element type, hidden size, vocabulary): everything
    about their shape rules (include/vrl.h) that does not depend on how many tokens a call brings."""
    V, K = weight.shape
    return (hidden.dtype in (torch.bfloat16, torch.float16) and V >= 256 and V % 8 == 0 and K % 64 == 0
            and hidden.stride(-1) == 1 and weight.stride(-1) == 1
            and hidden.stride(0) % 8 == 0 and weight.stride(0) % 8 == 0
            and hidden.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0)


def _own_forward_in_use(kernels: str, hidden: torch.Tensor, weight: torch.Tensor) -> bool:
    """Whether the forward is vrl_lmhead_score. Decided by the ``kernels`` option and by the model only, never by the
    number of tokens, by ``keep_logits`` or by whether gradients are recorded: a trainer's old (no-grad) and new (grad)
    log-probs of the same weights then come from the same kernel, and from the same summation order, whatever the
    micro-batch sizes are."""
    return kernels != "library" and _mfma_takes_model(hidden, weight)


# keep_logits=None (the default) keeps for the backward as many logits as fit this many bytes: on a 288 GB part the
# 2.5 GB of an 8192 x 152064 bf16 micro-batch are under 1 % of the memory and save a quarter of the matrix-core flops
# (21 ms forward + backward instead of 26.5 ms). Of a call whose logits are larger the leading tokens' are kept, as many
# as fit and leave whole chunks, and the rest is formed again chunk by chunk as the reference does (the library path keeps
# all or nothing). The environment variable VERL_AMD_LMHEAD_KEEP_BYTES sets the limit (0: never keep unless asked).
DEFAULT_KEEP_LOGITS_BYTES = int(os.environ.get("VERL_AMD_LMHEAD_KEEP_BYTES", str(4 << 30)))

# From this many tokens on, one transposed copy of the weight per backward (0.44 ms for 152064 x 3584 bf16) is
# repaid by the faster `d hidden` product.
_WEIGHT_TRANSPOSE_MIN_TOKENS = 2048


def _score_chunk(lib, logits, labels, temp, lp, h, lse, flag, stream):
    n, V = logits.shape
    st = lib.vrl_rowscore(logits.data_ptr(), _DTYPE_CODES[logits.dtype], n, V, logits.stride(0) if n > 1 else V,
                          labels.data_ptr(), _ptr(temp), lp.data_ptr(), h.data_ptr(), None, lse.data_ptr(),
                          flag.data_ptr(), stream)
    _lib.check("vrl_rowscore", st)


def _padded(x: torch.Tensor, rows: int) -> torch.Tensor:
    """``x`` with zero rows appended up to ``rows``."""
    out = torch.zeros((rows,) + tuple(x.shape[1:]), dtype=x.dtype, device=x.device)
    out[: x.shape[0]] = x
    return out


def _d_hidden(grad_logits, weight, weight_t, out, own_kernel):
    """out = grad_logits @ weight: this package's matrix-core kernel (``vrl_gemm``, the weight read as it lies) when
    asked for and the shapes allow, the library otherwise (with the transposed copy of the weight when there is one:
    both operands contiguous along the vocabulary). The kernel contracts in steps of 64: of a vocabulary that is not a
    multiple of 64 it takes the whole steps and the library adds the last, partial one (fewer than 64 columns)."""
    V = weight.shape[0]
    main = V // 64 * 64
    if own_kernel and main >= 128 and _own_d_hidden_takes(grad_logits[:, :main], weight[:main], out):
        _gemm.gemm(weight[:main], grad_logits[:, :main], x_t=True, out=out)
        if main != V:
            out.addmm_(grad_logits[:, main:], weight[main:])
    else:
        torch.matmul(grad_logits, weight if weight_t is None else weight_t.t(), out=out)


def _own_d_hidden_takes(grad_logits, weight, out) -> bool:
    """Everything vrl_gemm checks about the operands of d hidden, so that what it would refuse goes to the library."""
    return (_gemm.gemm_takes(weight, grad_logits, True, False) and out.stride(0) % 4 == 0 and out.stride(1) == 1
            and out.data_ptr() % 8 == 0 and out.stride(0) >= weight.shape[1])


class _FusedLinearForPPOFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, hidden, weight, input_ids, temperature, chunk_size, keep_rows, kernels, forward_splits=None):
        # keep_rows: the logits of this many leading tokens are kept for the backward (all of them when it reaches the
        # token count; a part only on the package's own path, in whole 256-token blocks)
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
        wants_grad = T > 0 and (ctx.needs_input_grad[0] or ctx.needs_input_grad[1])
        keep = wants_grad and int(keep_rows) >= T
        ctx.own_kept = False
        if _own_forward_in_use(kernels, hidden, weight):
            temp_all = None if temperature == 1.0 else torch.full((T,), float(temperature), **f32)
            rows = T if keep else (int(keep_rows) // 256 * 256 if wants_grad else 0)
            lp, h, lse, kept = _own_forward(hidden, weight, input_ids, temp_all, forward_splits, "fused_linear_for_ppo",
                                            keep_rows=rows)
            ctx.save_for_backward(hidden, weight, input_ids, lse, h)
            ctx.temperature = float(temperature)
            ctx.chunk_size = int(chunk_size)
            ctx.kept_logits = kept
            ctx.own_kept = kept is not None
            return lp.clone(), h.clone()
        temp = None if temperature == 1.0 else torch.full((min(chunk_size, max(T, 1)),), float(temperature), **f32)
        lib = _lib.load()
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
            return None, None, None, None, None, None, None, None
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
        d_weight = torch.empty_like(weight) if need_dw else None
        dw_started = False     # whether d_weight holds a partial sum yet
        lib = _lib.load()
        base = 0               # tokens before this one are done
        if kept is not None and ctx.own_kept:
            # The forward kernel left the logits of the first tokens, or of all of them (then in rows padded to a multiple
            # of 64 with zero hidden states, whose logits and hence gradients are zero): their gradient is written over
            # them, and each product runs once over those tokens with this package's kernel. What follows them, if
            # anything, is formed again chunk by chunk below and added.
            m = kept.shape[0]
            n_k = min(m, T)
            temp_rows = None if ctx.temperature == 1.0 else torch.full((n_k,), ctx.temperature, **f32)
            with torch.cuda.device(dev):
                st = lib.vrl_rowscore_backward(
                    kept.data_ptr(), _DTYPE_CODES[hidden.dtype], n_k, V, kept.stride(0), input_ids.data_ptr(),
                    _ptr(temp_rows), lse.data_ptr(), h.data_ptr(), _ptr(gl), _ptr(gh), kept.data_ptr(), kept.stride(0),
                    _lib.stream_ptr(dev))
            _lib.check("vrl_rowscore_backward", st)
            if need_dh:
                out = d_hidden[:m] if m <= T else torch.empty((m, D), dtype=hidden.dtype, device=dev)
                _d_hidden(kept, weight, None, out, True)
                if m > T:
                    d_hidden.copy_(out[:T])
            if need_dw:
                c_h = hidden[:m] if m <= T else _padded(hidden, m)
                if _gemm.gemm_takes(c_h, kept, True, True):
                    _gemm.gemm(c_h, kept, x_t=True, y_t=True, out=d_weight)
                else:
                    torch.matmul(kept[:n_k].t(), hidden[:n_k], out=d_weight)
                dw_started = True
            if m >= T:
                return d_hidden, d_weight, None, None, None, None, None, None
            base, kept = m, None
        # With this package's own kernels every chunk is at least one block of 256 tokens: a smaller chunk size is raised
        # to 256, a short tail joins the chunk before it, and a call with fewer than 256 tokens is padded to one block
        # (zero hidden states and zero incoming gradients give zero rows), so the backward never falls back to logits
        # that a library GEMM rounded differently from the forward's. A chunk is also padded to a multiple of 64 tokens,
        # the step of the contraction of d W.
        own = kept is None and ctx.kernels != "library" and V % 8 == 0 and _mfma_takes_model(hidden, weight)
        step = max(chunk, 256) if own else chunk
        starts = list(range(base, T, step))
        if own and len(starts) > 1 and T - starts[-1] < 256:
            starts.pop()
        bounds = [(lo, starts[i + 1] if i + 1 < len(starts) else T) for i, lo in enumerate(starts)]
        rows = max([hi - lo for lo, hi in bounds] + [1])
        if own:
            rows = max((rows + 63) // 64 * 64, 256)
        if temp is not None and temp.numel() < rows:
            temp = torch.full((rows,), ctx.temperature, **f32)
        buf = kept if kept is not None else torch.empty((rows, V), dtype=hidden.dtype, device=dev)
        dt = _DTYPE_CODES[hidden.dtype]
        # For 16-bit operands the library GEMM is 25-35 % faster when both operands are contiguous along the
        # contraction axis (vocab for `d hidden`, tokens for `d W`); fp32 runs at the fp32 matrix peak either way.
        half = hidden.element_size() == 2
        # (only a library `d hidden` wants the transposed weight; the package's own product reads W as it lies)
        own_dh = ctx.kernels != "library" and need_dh and _own_d_hidden_takes(buf[:256], weight, d_hidden)
        weight_t = (transpose_2d(weight)
                    if (half and need_dh and not own_dh and T >= _WEIGHT_TRANSPOSE_MIN_TOKENS) else None)
        with torch.cuda.device(dev):
            stream = _lib.stream_ptr(dev)
            for lo, hi in bounds:
                n = hi - lo
                if own:
                    # logits formed again on the matrix cores, their gradient written straight into the buffer
                    logits = buf[:n]
                    c_h, c_ids, c_lse, c_ent = hidden[lo:hi], input_ids[lo:hi], lse[lo:hi], h[lo:hi]
                    c_gl = None if gl is None else gl[lo:hi]
                    c_gh = None if gh is None else gh[lo:hi]
                    m = max((n + 63) // 64 * 64, 256)
                    if m != n:
                        c_h = _padded(c_h, m)
                        c_ids, c_lse, c_ent = _padded(c_ids, m), _padded(c_lse, m), _padded(c_ent, m)
                        c_gl = None if c_gl is None else _padded(c_gl, m)
                        c_gh = None if c_gh is None else _padded(c_gh, m)
                    st = lib.vrl_lmhead_dlogits(
                        c_h.data_ptr(), weight.data_ptr(), dt, m, V, D, c_h.stride(0), weight.stride(0),
                        c_ids.data_ptr(), None if temp is None else temp.data_ptr(), c_lse.data_ptr(),
                        c_ent.data_ptr(), None if c_gl is None else c_gl.data_ptr(),
                        None if c_gh is None else c_gh.data_ptr(), lib.vrl_lmhead_plan(m, V), buf.data_ptr(),
                        buf.stride(0), stream)
                    _lib.check("vrl_lmhead_dlogits", st)
                    if need_dh:
                        _d_hidden(logits, weight, weight_t, d_hidden[lo:hi], True)
                    if need_dw:
                        # d W (+)= G^T . H over the padded chunk (its extra rows are zero in both), read in place
                        if _gemm.gemm_takes(c_h, buf[:m], True, True):
                            _gemm.gemm(c_h, buf[:m], x_t=True, y_t=True, out=d_weight, accumulate=dw_started)
                        else:
                            if not dw_started:
                                d_weight.zero_()
                            d_weight.addmm_(logits.t(), transpose_2d(hidden[lo:hi]).t())
                        dw_started = True
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
                    if not dw_started:
                        d_weight.zero_()
                        dw_started = True
                    d_weight.addmm_(logits.t(), transpose_2d(hidden[lo:hi]).t() if half else hidden[lo:hi])
            if kept is not None:
                # the gradient over all tokens' logits is in `kept`: one product each, nothing to accumulate
                if need_dh:
                    _d_hidden(kept, weight, weight_t, d_hidden, ctx.kernels != "library")
                if need_dw:
                    # one product over all tokens: here the library is the faster one (6.7 against 7.2 ms at 8192 tokens)
                    torch.matmul(kept.t(), transpose_2d(hidden).t() if half else hidden, out=d_weight)
                    dw_started = True
            if need_dw and not dw_started:
                d_weight.zero_()          # no tokens
        return d_hidden, d_weight, None, None, None, None, None, None


def fused_linear_for_ppo(hidden_states: torch.Tensor, vocab_weights: torch.Tensor, input_ids: torch.Tensor,
                         temperature: float = 1.0, chunk_size: int = DEFAULT_CHUNK_TOKENS,
                         keep_logits: Optional[bool] = None, kernels: Optional[str] = None,
                         forward_splits: Optional[int] = None):
    """(log_probs fp32, entropy fp32) of ``softmax((hidden_states @ vocab_weights.T) / temperature)`` at ``input_ids``.

    ``hidden_states`` is ``(tokens, hidden)`` or ``(batch, seq, hidden)`` with ``input_ids`` of the matching leading
    shape; ``vocab_weights`` is ``(vocab, hidden)``; both bf16, fp16 or fp32 on the GPU. Differentiable with respect
    to both. ``chunk_size`` tokens are projected at a time (one reusable ``(chunk_size, vocab)`` buffer); the result
    depends on it only through the order in which the library sums a product of that height; the default is sized for
    this GPU rather than the reference's 512.

    ``keep_logits=True`` trades memory for time when gradients are needed: the forward keeps all
    ``tokens x vocab`` logits (2.5 GB for 8192 x 152064 bf16; written by the same forward kernel from its registers), the
    backward writes their gradient over them instead of projecting again and forms ``d hidden`` and ``d W`` with one
    product each. Such a graph can be differentiated once. The scores do not depend on it. ``None`` (the default) keeps
    what fits ``DEFAULT_KEEP_LOGITS_BYTES`` (4 GiB unless ``VERL_AMD_LMHEAD_KEEP_BYTES`` says otherwise): all of them, or the
    logits of the leading tokens, so many that the rest is whole chunks (the same forward kernel writes just those; the
    backward forms the others again chunk by chunk and adds their share of ``d W``); ``False`` never holds more than one
    chunk of logits, like the reference.

    ``kernels`` chooses which matrix products are this package's own kernels: ``"library"`` (none: torch.matmul
    throughout) or ``"auto"`` / ``"mfma"`` (all of them: a forward that is one kernel and never
    writes logits, a backward that forms the logits again, writes their gradient straight from registers and forms
    ``d hidden`` and ``d W`` with ``vrl_gemm``: no library GEMM is called). Which forward runs depends on this option, on
    ``keep_logits`` and on the model, never on the number of tokens or on whether gradients are recorded, so log-probs
    computed with and without gradients are bit-identical. None takes ``DEFAULT_KERNELS`` ("auto" unless
    ``VERL_AMD_LMHEAD_KERNELS`` says otherwise).

    ``forward_splits`` sets into how many shares per 256-token block that forward's work is dealt (1..64; None: planned
    per call; ``DEFAULT_FORWARD_SPLITS`` / ``VERL_AMD_LMHEAD_SPLITS`` override). It changes the time only: a token gets the
    same bits for any value and in calls of any size, so a trainer's old and new log-probs of unchanged weights are
    bit-identical whatever its micro-batches.
    """
    kernels = DEFAULT_KERNELS if kernels is None else kernels
    if kernels not in ("auto", "library", "mfma"):
        raise ValueError(f"kernels must be 'auto', 'library' or 'mfma', got {kernels!r}")
    forward_splits = DEFAULT_FORWARD_SPLITS if forward_splits is None else forward_splits
    if forward_splits is not None and not 1 <= int(forward_splits) <= 64:
        raise ValueError(f"forward_splits must be in 1..64, got {forward_splits}")
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
    T = h2.shape[0]
    if keep_logits is None:
        # what fits the budget: everything, or (the package's own kernels) the leading whole 256-token blocks
        keep_rows = min(T, DEFAULT_KEEP_LOGITS_BYTES // max(w2.shape[0] * h2.element_size(), 1)) if needs_grad else 0
        if keep_rows < T:
            # a part: so many that what is formed again is whole chunks (a short last chunk costs nearly a full one:
            # 16384 tokens under 4 GiB, 12288 kept + one chunk of 4096: 45.0 ms; 14080 kept + 2304: 48.3; none kept: 52.2)
            again = -(-(T - keep_rows) // int(chunk_size)) * int(chunk_size)
            keep_rows = max(T - again, 0) // 256 * 256 if _own_forward_in_use(kernels, h2, w2) else 0
    else:
        keep_rows = T if keep_logits else 0
    if not needs_grad and _own_forward_in_use(kernels, h2, w2):
        temp = None if float(temperature) == 1.0 else torch.full((h2.shape[0],), float(temperature), dtype=torch.float32,
                                                                  device=h2.device)
        with torch.no_grad():
            lp, ent, _, _ = _own_forward(h2, w2, ids, temp, forward_splits, "fused_linear_for_ppo")
        return lp.reshape(lead), ent.reshape(lead)
    lp, ent = _FusedLinearForPPOFunction.apply(h2, w2, ids, float(temperature), int(chunk_size), int(keep_rows),
                                               kernels, None if forward_splits is None else int(forward_splits))
    return lp.reshape(lead), ent.reshape(lead)


def _own_forward(h, w, ids, temp, n_splits, what, keep_rows=0):
    """(log-prob, entropy, logsumexp, kept logits), the first three fp32 per row of ``h``, from vrl_lmhead_score. ``temp``
    is None or one value per token. The kernels work on blocks of 256 tokens: a shorter input is copied into a zero-padded
    block first. With ``keep_rows`` the kernel also writes the logits of that many leading tokens. All of them
    (``keep_rows`` = the token count) go into a buffer whose rows are padded to a multiple of 64, the step of the
    contraction of d W: rows past the input hold the logits of zero hidden states, zeros. A part of them (a multiple of
    256 below the token count) goes into a buffer of exactly that many rows."""
    T, K = h.shape
    V = w.shape[0]
    dev = h.device
    f32 = dict(dtype=torch.float32, device=dev)
    if T == 0:
        return torch.empty(0, **f32), torch.empty(0, **f32), torch.empty(0, **f32), None
    keep_rows = min(int(keep_rows), T)
    keep_all = keep_rows == T
    if not keep_all and keep_rows % 256 != 0:
        raise ValueError(f"{what}: a part of the logits is kept in whole 256-token blocks, got {keep_rows} of {T} tokens")
    n = max((T + 63) // 64 * 64, 256) if keep_all else max(T, 256)
    if n != T:
        hp = torch.zeros((n, K), dtype=h.dtype, device=dev)
        hp[:T] = h
        ip = torch.zeros(n, dtype=torch.int64, device=dev)
        ip[:T] = ids
        tp = None
        if temp is not None:
            tp = torch.ones(n, **f32)
            tp[:T] = temp
        h, ids, temp = hp, ip, tp
    lib = _lib.load()
    splits = lib.vrl_lmhead_plan(n, V) if n_splits is None else min(int(n_splits), (V + 255) // 256)
    partials = torch.empty(int(lib.vrl_lmhead_partials(n, V)), **f32)
    lp = torch.empty(n, **f32)
    ent = torch.empty(n, **f32)
    lse = torch.empty(n, **f32)
    rows = n if keep_all else keep_rows
    kept = torch.empty((rows, V), dtype=h.dtype, device=dev) if rows > 0 else None
    flag = torch.zeros(1, dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        st = lib.vrl_lmhead_score(h.data_ptr(), w.data_ptr(), _DTYPE_CODES[h.dtype], n, V, K, h.stride(0), w.stride(0),
                                  ids.data_ptr(), _ptr(temp), splits, partials.data_ptr(), lp.data_ptr(), ent.data_ptr(),
                                  lse.data_ptr(), flag.data_ptr(), _ptr(kept), V if rows > 0 else 0, rows,
                                  _lib.stream_ptr(dev))
    _lib.check("vrl_lmhead_score", st)
    _errors.report(flag, {_lib.VRL_FLAG_LABEL_OOB: (IndexError, f"{what}: an input id is outside [0, {V})")})
    return lp[:T], ent[:T], lse[:T], kept


def lm_head_score_mfma(hidden_states: torch.Tensor, vocab_weights: torch.Tensor, input_ids: torch.Tensor,
                       temperature=1.0, n_splits: Optional[int] = None):
    """Forward-only (log_probs, entropy), fp32, from one hand-written matrix-core kernel that never writes logits
    (``vrl_lmhead_score``): the counterpart of the reference's Triton ``efficient_entropy_forward``
    (verl/utils/kernel/kernels.py:531-756). bf16 or fp16 operands, at least 256 vocabulary entries, hidden size a
    multiple of 64 (fewer than 256 tokens are padded to 256 rows for the call). ``temperature`` is a float or one value per token. The logits are kept in fp32
    (a GEMM that writes them rounds them to the operand type first), so results are slightly closer to the
    all-fp32 value than a path that writes them. On MI355X it takes as long as the library GEMM + row kernel (6.5 ms at
    8192 x 3584 -> 152064) and needs no logits buffer at all; it is ``fused_linear_for_ppo``'s default forward.
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
    if V < 256 or K % 64 != 0:
        raise ValueError(f"lm_head_score_mfma needs >= 256 vocabulary entries and a hidden size that is a multiple of "
                         f"64; got {V}, {K}")
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
    lp, ent, _, _ = _own_forward(h, w, ids, temp, n_splits, "lm_head_score_mfma")
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

    def __init__(self, chunk_size: int = DEFAULT_CHUNK_TOKENS, keep_logits: Optional[bool] = None,
                 kernels: Optional[str] = None, forward_splits: Optional[int] = None):
        super().__init__()
        self.chunk_size = chunk_size
        self.keep_logits = keep_logits
        self.kernels = kernels
        self.forward_splits = forward_splits

    def forward(self, hidden_states, vocab_weights, input_ids, temperature: float = 1.0):
        return fused_linear_for_ppo(hidden_states, vocab_weights, input_ids, temperature, self.chunk_size,
                                    self.keep_logits, self.kernels, self.forward_splits)
