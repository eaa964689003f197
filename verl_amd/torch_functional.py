"""Per-token scoring on MI355X behind the names of verl.utils.torch_functional.

Same names, argument meaning and leading-shape handling as the reference
functions (verl/utils/torch_functional.py:73-107, 155-207, 231-270); the work
is done by the HIP row kernel through the C ABI (include/vrl.h). Inputs must
live on the GPU: there is no CPU or eager-torch path in this module, and a
missing libvrl_hip.so raises.

Differences from the reference that a caller can observe:
  * results are fp32 for bf16 inputs too (the reference's non-fp32 branch
    returns the input dtype, :199-206; its flash-attn branch returns fp32);
  * a label outside [0, vocab) raises IndexError after the kernel ran
    (torch.gather device-asserts);
  * the sum of squared probabilities is not differentiable here (the reference
    computes it under no_grad for the optimal-baseline estimator only).
Log-probs and entropy are differentiable with respect to the logits through one
HIP backward kernel (vrl_rowscore_backward).
"""

from __future__ import annotations

from typing import Optional, Union

import torch

from . import _lib
from . import errors as _errors

__all__ = [
    "logprobs_from_logits",
    "logprobs_from_logits_v2",
    "logprobs_from_logits_naive",
    "entropy_from_logits",
    "entropy_from_logits_with_chunking",
    "calculate_sum_pi_squared_from_logits",
    "fused_logprob_entropy",
    "score_responses",
]

# A label outside [0, vocab) makes that row's log-prob NaN and sets a bit in the kernel's error flag. How the flag
# turns into an IndexError is verl_amd.errors' business: "sync" reads it back at once (one host synchronisation per
# call, the default for direct calls), "deferred" looks at it later without ever waiting for the GPU (what the
# installed shims use), "off" never looks. ``check_labels`` arguments take None (the mode in force), True ("sync"),
# False ("off") or a mode name.

_DTYPE_CODES = {torch.float32: _lib.VRL_F32, torch.bfloat16: _lib.VRL_BF16, torch.float16: _lib.VRL_F16}


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _check_logits(logits: torch.Tensor, what: str) -> None:
    if not isinstance(logits, torch.Tensor):
        raise TypeError(f"{what}: logits must be a torch.Tensor, got {type(logits).__name__}")
    if not logits.is_cuda:
        raise RuntimeError(
            f"{what}: logits are on {logits.device}; verl_amd only runs on the GPU (HIP kernels), "
            "it has no CPU implementation"
        )
    if logits.dtype not in _DTYPE_CODES:
        raise TypeError(f"{what}: logits dtype {logits.dtype} is not supported (float32, bfloat16 and float16 are)")
    if logits.dim() < 1 or logits.shape[-1] == 0:
        raise ValueError(f"{what}: logits need a non-empty last (vocab) dimension, got shape {tuple(logits.shape)}")


def _is_view_safe(logits: torch.Tensor) -> bool:
    """True when _rows_2d returns a view of ``logits`` (so writing a gradient over it is what the caller asked
    for) and the tensor is not a leaf that autograd will want to read again."""
    return logits.is_contiguous() and not logits.is_leaf


_MAX_ROW_SLICE_BATCH = 256


def _is_batch_of_row_slices(logits: torch.Tensor) -> bool:
    """A 3-D (B, R, V) tensor with unit vocab stride and rows V or more apart whose batch stride does not let it be
    viewed as (B*R, V): a slice along the sequence axis of a longer tensor."""
    if logits.dim() != 3 or logits.shape[0] < 2 or logits.shape[0] > _MAX_ROW_SLICE_BATCH or logits.shape[1] == 0:
        return False
    B, Rr, V = logits.shape
    sb, sr, sv = logits.stride()
    return sv == 1 and sr >= V and sb != Rr * sr


def _rows_2d(logits: torch.Tensor) -> torch.Tensor:
    """(..., V) -> (N, V) with unit stride along V; a view whenever torch allows one."""
    V = logits.shape[-1]
    if logits.dim() == 2:
        x = logits
    else:
        x = logits.reshape(-1, V)
    if x.stride(-1) != 1 or (x.shape[0] > 1 and x.stride(0) < V):
        x = x.contiguous()
    return x


def _temperature_rows(temperature, lead_shape, n_rows, device) -> Optional[torch.Tensor]:
    if temperature is None:
        return None
    if isinstance(temperature, (int, float)):
        return torch.full((n_rows,), float(temperature), dtype=torch.float32, device=device)
    t = temperature.to(device=device, dtype=torch.float32)
    if t.numel() == 1:
        return t.reshape(1).expand(n_rows).contiguous()
    if t.numel() != n_rows:
        raise ValueError(
            f"temperature has {t.numel()} entries, expected one per token ({n_rows}) for logits leading shape {tuple(lead_shape)}"
        )
    return t.reshape(n_rows).contiguous()


def _label_messages(what: str, vocab: int) -> dict:
    return {_lib.VRL_FLAG_LABEL_OOB: (IndexError, f"{what}: a label is outside [0, {vocab})")}


def _forward_2d(x, lab, temp, want_logprob, want_entropy, want_sum_pi_sq, want_lse, n_splits, flag=None):
    """Launch the forward kernels on (N, V) rows; returns (logprob, entropy, sum_pi_sq, lse, flag), None where not
    asked. ``flag`` may bring the int32 error flag to OR into (several launches then share one)."""
    n, V = x.shape
    dev = x.device
    f32 = dict(dtype=torch.float32, device=dev)
    out_lp = torch.empty(n, **f32) if want_logprob else None
    out_h = torch.empty(n, **f32) if want_entropy else None
    out_q = torch.empty(n, **f32) if want_sum_pi_sq else None
    out_lse = torch.empty(n, **f32) if want_lse else None
    if flag is None and want_logprob:
        flag = torch.zeros(1, dtype=torch.int32, device=dev)
    if n == 0:
        return out_lp, out_h, out_q, out_lse, flag
    lib = _lib.load()
    dt = _DTYPE_CODES[x.dtype]
    stride = x.stride(0) if n > 1 else V
    splits = lib.vrl_rowscore_split_plan(dt, n, V) if n_splits is None else int(n_splits)
    with torch.cuda.device(dev):
        stream = _lib.stream_ptr(dev)
        if splits > 1:
            partials = torch.empty(n * splits * 4, **f32)
            st = lib.vrl_rowscore_split(
                x.data_ptr(), dt, n, V, stride, _ptr(lab), _ptr(temp), _ptr(out_lp), _ptr(out_h), _ptr(out_q),
                _ptr(out_lse), _ptr(flag), splits, partials.data_ptr(), stream,
            )
            _lib.check("vrl_rowscore_split", st)
        else:
            st = lib.vrl_rowscore(
                x.data_ptr(), dt, n, V, stride, _ptr(lab), _ptr(temp), _ptr(out_lp), _ptr(out_h), _ptr(out_q),
                _ptr(out_lse), _ptr(flag), stream,
            )
            _lib.check("vrl_rowscore", st)
    counters["forward_passes"] += 1
    return out_lp, out_h, out_q, out_lse, flag


# Kernel passes over (N, V) logits launched from this module since import (what a caller can count to see how many
# times its logits were streamed): forward row kernels, backward row kernels, per-row label gathers.
counters = {"forward_passes": 0, "backward_passes": 0, "label_gathers": 0}


def _backward_2d(x, lab, temp, lse, h, g_lp, g_h, inplace):
    """dlogits of (N, V) rows from vrl_rowscore_backward, one pass; over x's own storage when ``inplace``."""
    n, V = x.shape
    dev = x.device
    # In place: the gradient replaces the logits in their own storage, like the reference's
    # flash-attn path does with inplace_backward=True (verl/utils/torch_functional.py:110-131).
    dx = x if inplace else torch.empty((n, V), dtype=x.dtype, device=dev)
    if n > 0:
        gl = None if g_lp is None else g_lp.to(torch.float32).contiguous()
        gh = None if g_h is None else g_h.to(torch.float32).contiguous()
        lib = _lib.load()
        with torch.cuda.device(dev):
            st = lib.vrl_rowscore_backward(
                x.data_ptr(), _DTYPE_CODES[x.dtype], n, V, x.stride(0) if n > 1 else V, _ptr(lab), _ptr(temp),
                lse.data_ptr(), h.data_ptr(), _ptr(gl), _ptr(gh), dx.data_ptr(), dx.stride(0) if n > 1 else V,
                _lib.stream_ptr(dev),
            )
        _lib.check("vrl_rowscore_backward", st)
        counters["backward_passes"] += 1
    return dx


def _label_logprob(x, lab, temp, lse, flag=None):
    """(logprob, flag) of (N, V) rows from a logsumexp an earlier pass left behind (vrl_label_logprob)."""
    n, V = x.shape
    dev = x.device
    out = torch.empty(n, dtype=torch.float32, device=dev)
    if flag is None:
        flag = torch.zeros(1, dtype=torch.int32, device=dev)
    if n > 0:
        lib = _lib.load()
        with torch.cuda.device(dev):
            st = lib.vrl_label_logprob(x.data_ptr(), _DTYPE_CODES[x.dtype], n, V, x.stride(0) if n > 1 else V,
                                       lab.data_ptr(), _ptr(temp), lse.data_ptr(), out.data_ptr(), flag.data_ptr(),
                                       _lib.stream_ptr(dev))
        _lib.check("vrl_label_logprob", st)
        counters["label_gathers"] += 1
    return out, flag


class _EntropyLseFunction(torch.autograd.Function):
    """(entropy, logsumexp) of the rows of ``x`` from one pass, for a caller that asks for the entropy first and for the
    label log-probs of the same logits afterwards (the order of verl/workers/engine/fsdp/transformer_impl.py:1364-1399).
    The log-probs then come from ``_LabelLogprobFunction``, which consumes this node's logsumexp; autograd therefore
    runs that node's backward first, it leaves the log-probs' incoming gradient and the labels in ``pair``, and this
    node's backward makes ONE pass over the logits with both gradients instead of two passes and an accumulation."""

    @staticmethod
    def forward(ctx, x, temp, n_splits, pair):
        ctx.set_materialize_grads(False)
        _, h, _, lse, _ = _forward_2d(x, None, temp, False, True, False, True, n_splits)
        ctx.save_for_backward(x, temp, lse, h)
        ctx.pair = pair
        return h, lse

    @staticmethod
    def backward(ctx, g_h, g_lse):
        x, temp, lse, h = ctx.saved_tensors
        g_lp, lab = ctx.pair.get("g_lp"), ctx.pair.get("labels")
        if g_lse is not None and g_lp is None:
            raise RuntimeError("verl_amd: the shared logsumexp received a gradient that did not come from the label "
                               "log-probs; it is an internal tensor and must not be used elsewhere")
        if g_lp is None and g_h is None:
            return None, None, None, None
        inplace = bool(ctx.pair.get("inplace", False))
        ctx.pair.pop("g_lp", None)
        return _backward_2d(x, lab, temp, lse, h, g_lp, g_h, inplace), None, None, None


class _LabelLogprobFunction(torch.autograd.Function):
    """logprob = z[label] - lse with ``lse`` from ``_EntropyLseFunction``. Its backward hands the incoming gradient to
    that node (through ``pair`` and, so that the node runs at all, as the gradient of lse) and returns no dense
    gradient for the logits itself."""

    @staticmethod
    def forward(ctx, x, lab, temp, lse, pair, inplace, flag):
        ctx.set_materialize_grads(False)
        lp, flag = _label_logprob(x, lab, temp, lse, flag)
        ctx.save_for_backward(lab)
        ctx.pair = pair
        ctx.inplace = bool(inplace)
        ctx.mark_non_differentiable(flag)
        return lp, flag

    @staticmethod
    def backward(ctx, g_lp, _g_flag):
        if g_lp is None:
            return None, None, None, None, None, None, None
        (lab,) = ctx.saved_tensors
        ctx.pair["g_lp"] = g_lp
        ctx.pair["labels"] = lab
        ctx.pair["inplace"] = ctx.inplace
        return None, None, None, -g_lp, None, None, None


class _RowScoreFunction(torch.autograd.Function):
    """Differentiable (log-prob, entropy) of the rows of ``x``; the gradient comes from vrl_rowscore_backward."""

    @staticmethod
    def forward(ctx, x, lab, temp, want_logprob, want_entropy, n_splits, inplace_backward, flag):
        ctx.set_materialize_grads(False)
        lp, h, _, lse, flag = _forward_2d(x, lab, temp, want_logprob, True, False, True, n_splits, flag)
        ctx.save_for_backward(x, lab, temp, lse, h)
        ctx.inplace = bool(inplace_backward)
        if flag is not None:
            ctx.mark_non_differentiable(flag)
        return lp, (h if want_entropy else None), flag

    @staticmethod
    def backward(ctx, g_lp, g_h, _g_flag):
        x, lab, temp, lse, h = ctx.saved_tensors
        if g_lp is None and g_h is None:
            return None, None, None, None, None, None, None, None
        dx = _backward_2d(x, lab if g_lp is not None else None, temp, lse, h, g_lp, g_h, ctx.inplace)
        return dx, None, None, None, None, None, None, None


def rowscore(
    logits: torch.Tensor,
    labels: Optional[torch.Tensor],
    temperature: Union[None, float, torch.Tensor] = None,
    *,
    want_logprob: bool = True,
    want_entropy: bool = True,
    want_sum_pi_sq: bool = False,
    check_labels=None,
    n_splits: Optional[int] = None,
    inplace_backward: bool = False,
    what: str = "rowscore",
    _flag: Optional[torch.Tensor] = None,
):
    """Launch the row kernel; returns (logprob | None, entropy | None) and, with ``want_sum_pi_sq``,
    a third entry, each fp32 of shape logits.shape[:-1].

    With few rows the work of one row is spread over ``n_splits`` workgroups (vrl_rowscore_split);
    ``n_splits=None`` lets the library choose, 1 forces one workgroup per row. When grad is enabled
    and the logits require it, log-prob and entropy are differentiable with respect to the logits
    (vrl_rowscore_backward); the sum of squared probabilities is not. ``check_labels`` says how a label outside
    the vocabulary becomes an IndexError (verl_amd.errors: None = the mode in force, True = read the flag back now,
    False = never, "deferred" = later and without waiting for the GPU). ``_flag`` (internal) brings a shared error
    flag; whoever passes it reports it.
    """
    _check_logits(logits, what)
    if _flag is None:
        _errors.poll()
    if not (want_logprob or want_entropy or want_sum_pi_sq):
        raise ValueError(f"{what}: nothing to compute")
    if _is_batch_of_row_slices(logits):
        # (B, R, V) cut out of a longer (B, S, V) tensor, e.g. logits[:, -R-1:-1] in
        # verl/utils/torch_functional.py:615: flattening would copy B*R*V elements; each logits[b] is a 2-D block
        # the kernel reads in place (its rows are V apart), so it is scored per b instead.
        if want_logprob and (labels is None or tuple(labels.shape) != tuple(logits.shape[:-1])):
            raise ValueError(f"{what}: labels shape {None if labels is None else tuple(labels.shape)} does not match "
                             f"logits leading shape {tuple(logits.shape[:-1])}")
        per_b_temperature = isinstance(temperature, torch.Tensor) and temperature.numel() != 1
        if per_b_temperature and temperature.numel() != logits.shape[0] * logits.shape[1]:
            raise ValueError(f"temperature has {temperature.numel()} entries, expected one per token "
                             f"({logits.shape[0] * logits.shape[1]}) for logits leading shape {tuple(logits.shape[:-1])}")
        t3 = temperature.reshape(logits.shape[:-1]) if per_b_temperature else None
        # one error flag for the whole loop, looked at once
        shared = _flag
        if shared is None and want_logprob:
            shared = torch.zeros(1, dtype=torch.int32, device=logits.device)
        parts = [rowscore(logits[b], None if labels is None else labels[b], t3[b] if per_b_temperature else temperature,
                          want_logprob=want_logprob, want_entropy=want_entropy, want_sum_pi_sq=want_sum_pi_sq,
                          n_splits=n_splits, inplace_backward=False, what=what, _flag=shared)
                 for b in range(logits.shape[0])]
        if want_logprob and _flag is None:
            _errors.report(shared, _label_messages(what, logits.shape[-1]), check_labels)
        return tuple(None if parts[0][k] is None else torch.stack([p[k] for p in parts]) for k in range(len(parts[0])))
    lead = logits.shape[:-1]
    V = logits.shape[-1]
    x = _rows_2d(logits)
    n = x.shape[0]
    dev = x.device

    lab = None
    if want_logprob:
        if labels is None:
            raise ValueError(f"{what}: labels are required for log-probs")
        if tuple(labels.shape) != tuple(lead):
            raise ValueError(f"{what}: labels shape {tuple(labels.shape)} does not match logits leading shape {tuple(lead)}")
        if labels.dtype.is_floating_point or labels.dtype == torch.bool:
            raise TypeError(f"{what}: labels must be an integer tensor, got {labels.dtype}")
        lab = labels.to(device=dev, dtype=torch.int64).reshape(n).contiguous()
    temp = _temperature_rows(temperature, lead, n, dev)

    needs_grad = torch.is_grad_enabled() and logits.requires_grad
    out_q = None
    if needs_grad and (want_logprob or want_entropy):
        lp, h, flag = _RowScoreFunction.apply(x, lab, temp, want_logprob, want_entropy, n_splits, inplace_backward,
                                              _flag)
        if want_sum_pi_sq:
            with torch.no_grad():
                out_q = _forward_2d(x, None, temp, False, False, True, False, n_splits)[2]
    else:
        with torch.no_grad():
            lp, h, out_q, _, flag = _forward_2d(x, lab, temp, want_logprob, want_entropy, want_sum_pi_sq, False,
                                                n_splits, _flag)
    if want_logprob and n > 0 and _flag is None:
        _errors.report(flag, _label_messages(what, V), check_labels)

    lp = lp.reshape(lead) if want_logprob else None
    h = h.reshape(lead) if want_entropy else None
    if want_sum_pi_sq:
        return lp, h, out_q.reshape(lead)
    return lp, h


def logprobs_from_logits(logits: torch.Tensor, labels: torch.Tensor, inplace_backward: bool = True) -> torch.Tensor:
    """log softmax(logits)[labels], shape logits.shape[:-1], fp32.

    Mirrors verl/utils/torch_functional.py:73-107. Differentiable with respect to the logits. With
    ``inplace_backward`` (the reference's default, honoured by its flash-attn branch, :110-131) the
    backward pass writes the gradient over the logits' own storage instead of allocating
    another (N, V) tensor; as there, the logits must not be used again after backward.
    """
    return rowscore(logits, labels, want_entropy=False, inplace_backward=inplace_backward and _is_view_safe(logits),
                    what="logprobs_from_logits")[0]


def logprobs_from_logits_v2(logits: torch.Tensor, labels: torch.Tensor) -> torch.Tensor:
    """Same result as logprobs_from_logits (verl/utils/torch_functional.py:173-207)."""
    return rowscore(logits, labels, want_entropy=False, what="logprobs_from_logits_v2")[0]


def logprobs_from_logits_naive(logits: torch.Tensor, labels: torch.Tensor) -> torch.Tensor:
    """Same result as logprobs_from_logits (verl/utils/torch_functional.py:155-170)."""
    return rowscore(logits, labels, want_entropy=False, what="logprobs_from_logits_naive")[0]


def entropy_from_logits(logits: torch.Tensor) -> torch.Tensor:
    """logsumexp(logits) - sum(softmax(logits) * logits) over the last dim, fp32.

    Mirrors verl/utils/torch_functional.py:231-245.
    """
    return rowscore(logits, None, want_logprob=False, what="entropy_from_logits")[1]


def entropy_from_logits_with_chunking(logits: torch.Tensor, chunk_size: int = 2048) -> torch.Tensor:
    """Same value as entropy_from_logits (verl/utils/torch_functional.py:248-270).

    The reference chunks rows to bound the size of its softmax temporaries; the
    row kernel has no temporaries, so ``chunk_size`` is validated and unused.
    """
    if int(chunk_size) <= 0:
        raise ValueError(f"chunk_size must be positive, got {chunk_size}")
    return rowscore(logits, None, want_logprob=False, what="entropy_from_logits_with_chunking")[1]


def calculate_sum_pi_squared_from_logits(logits: torch.Tensor) -> torch.Tensor:
    """sum(softmax(logits)^2) over the last dim, fp32.

    Mirrors verl/utils/torch_functional.py:690-704 (exp(logsumexp(2x) - 2 logsumexp(x))).
    """
    return rowscore(logits, None, want_logprob=False, want_entropy=False, want_sum_pi_sq=True,
                    what="calculate_sum_pi_squared_from_logits")[2]


def fused_logprob_entropy(
    logits: torch.Tensor,
    labels: torch.Tensor,
    temperature: Union[None, float, torch.Tensor] = None,
    *,
    check_labels=None,
    want_sum_pi_sq: bool = False,
    n_splits: Optional[int] = None,
):
    """(log-probs, entropy) of softmax(logits / temperature) in one pass over the logits.

    Replaces the three steps of the reference's engine
    (verl/workers/engine/fsdp/transformer_impl.py:1357 divide, :1364-1376 entropy,
    :1395-1399 log-probs). ``temperature`` is a float, or a tensor with one entry
    per token (same leading shape as ``labels``), clamped below at 1e-8 like the
    reference. For fp32 logits the quotient is rounded per element exactly like
    ``logits / temperature``; for bf16 logits it is formed in fp32 from the bf16
    values (the reference rounds the quotient back to bf16). With ``want_sum_pi_sq`` a third
    tensor, sum(softmax^2), comes out of the same pass
    (verl/workers/engine/fsdp/transformer_impl.py:1361-1362).
    """
    return rowscore(logits, labels, temperature, check_labels=check_labels, want_sum_pi_sq=want_sum_pi_sq,
                    n_splits=n_splits, what="fused_logprob_entropy")


def _score_responses_launch(x, lab, rolled, temp, cu, rl, T, want_logprob, want_entropy, per_token, want_lse, flag):
    """One vrl_score_responses launch; returns (resp_logprob, resp_entropy, logprob, entropy, resp_lse)."""
    n, V = x.shape
    dev = x.device
    B = rl.numel()
    f32 = dict(dtype=torch.float32, device=dev)
    r_lp = torch.empty((B, T), **f32) if want_logprob else None
    r_h = torch.empty((B, T), **f32) if want_entropy else None
    r_lse = torch.empty((B, T), **f32) if want_lse else None
    t_lp = torch.empty(n, **f32) if (per_token and want_logprob) else None
    t_h = torch.empty(n, **f32) if (per_token and want_entropy) else None
    if B > 0:
        lib = _lib.load()
        with torch.cuda.device(dev):
            st = lib.vrl_score_responses(
                x.data_ptr() if n else None, _DTYPE_CODES[x.dtype], n, V, x.stride(0) if n > 1 else V,
                _ptr(lab) if not rolled else None, _ptr(lab) if rolled else None, _ptr(temp),
                cu.data_ptr(), rl.data_ptr(), B, T, _ptr(t_lp), _ptr(t_h), _ptr(r_lp), _ptr(r_h), _ptr(r_lse),
                flag.data_ptr(), _lib.stream_ptr(dev))
        _lib.check("vrl_score_responses", st)
        counters["forward_passes"] += 1
    return r_lp, r_h, t_lp, t_h, r_lse


class _ScoreResponsesFunction(torch.autograd.Function):
    """Differentiable padded response blocks of packed logits: vrl_score_responses forward (which also leaves the
    logsumexp block), vrl_score_responses_backward for the logits' gradient — one pass each; rows outside every
    response window get a zero gradient without their logits being read."""

    @staticmethod
    def forward(ctx, x, lab, rolled, temp, cu, rl, T, want_logprob, want_entropy, per_token, inplace, flag):
        ctx.set_materialize_grads(False)
        r_lp, r_h, t_lp, t_h, r_lse = _score_responses_launch(x, lab, rolled, temp, cu, rl, T, want_logprob, True,
                                                              per_token, True, flag)
        ctx.save_for_backward(x, lab, temp, cu, rl, r_lse, r_h)
        ctx.rolled, ctx.T, ctx.inplace = bool(rolled), int(T), bool(inplace)
        if not want_entropy:
            r_h_out = None
        else:
            r_h_out = r_h
        for t in (t_lp, t_h):
            if t is not None:
                ctx.mark_non_differentiable(t)
        return r_lp, r_h_out, t_lp, (t_h if want_entropy else None)

    @staticmethod
    def backward(ctx, g_lp, g_h, _g_tlp, _g_th):
        none = (None,) * 12
        if g_lp is None and g_h is None:
            return none
        x, lab, temp, cu, rl, r_lse, r_h = ctx.saved_tensors
        n, V = x.shape
        dev = x.device
        B = rl.numel()
        dx = x if ctx.inplace else torch.empty((n, V), dtype=x.dtype, device=dev)
        if n > 0:
            gl = None if g_lp is None else g_lp.to(torch.float32).contiguous()
            gh = None if g_h is None else g_h.to(torch.float32).contiguous()
            use_lab = lab if gl is not None else None
            lib = _lib.load()
            with torch.cuda.device(dev):
                st = lib.vrl_score_responses_backward(
                    x.data_ptr(), _DTYPE_CODES[x.dtype], n, V, x.stride(0) if n > 1 else V,
                    _ptr(use_lab) if not ctx.rolled else None, _ptr(use_lab) if ctx.rolled else None, _ptr(temp),
                    cu.data_ptr(), rl.data_ptr(), B, ctx.T, r_lse.data_ptr(), r_h.data_ptr(), _ptr(gl), _ptr(gh),
                    dx.data_ptr(), dx.stride(0) if n > 1 else V, _lib.stream_ptr(dev))
            _lib.check("vrl_score_responses_backward", st)
            counters["backward_passes"] += 1
        return (dx,) + none[1:]


def score_responses(
    logits: torch.Tensor,
    cu_seqlens: torch.Tensor,
    response_lens: torch.Tensor,
    max_response_len: int,
    *,
    labels: Optional[torch.Tensor] = None,
    input_ids: Optional[torch.Tensor] = None,
    temperature: Union[None, float, torch.Tensor] = None,
    want_logprob: bool = True,
    want_entropy: bool = True,
    per_token: bool = False,
    inplace_backward: bool = False,
    check=None,
):
    """Packed ``logits`` ``(total_nnz, V)`` -> padded ``(B, max_response_len)`` response log-probs and entropies in ONE
    kernel launch (``vrl_score_responses``).

    The engine's sequence on a packed micro-batch — ``labels = roll(input_ids, -1)``
    (verl/workers/engine/fsdp/transformer_impl.py:1177), divide by the temperature (:1357), entropy and log-probs
    (:1364-1399), then ``no_padding_2_padding`` (verl/workers/utils/padding.py:97-141: per sequence take
    ``values[end - r - 1 : end - 1]`` and right-pad with zeros) — done by the row kernel itself: give ``input_ids``
    (the packed ids, rolled inside the kernel) or ready ``labels``; ``temperature`` is a float, one value per token or one per
    sequence (expanded over its tokens like ``expand_as_nested``, verl/utils/torch_functional.py:989-1011).

    Returns ``(resp_logprob | None, resp_entropy | None)``; with ``per_token`` also the ``(total_nnz,)`` vectors, as
    ``(resp_logprob, resp_entropy, logprob, entropy)``. Without ``per_token`` the logits of tokens outside every
    response window (the prompts) are never read. When grad is enabled and the logits require it, the two blocks are
    differentiable with respect to the logits (``vrl_score_responses_backward``: one pass, zero rows for the prompts,
    over the logits' own storage with ``inplace_backward``); the per-token vectors are not. Device-side findings (a
    label outside the vocabulary: IndexError; a sequence without a prompt token, a response longer than
    ``max_response_len``, offsets that do not partition the rows: ValueError) follow ``check`` as in verl_amd.errors.
    """
    what = "score_responses"
    _check_logits(logits, what)
    _errors.poll()
    if logits.dim() != 2:
        raise ValueError(f"{what}: logits must be packed (total_nnz, vocab), got shape {tuple(logits.shape)}")
    if not (want_logprob or want_entropy):
        raise ValueError(f"{what}: nothing to compute")
    if want_logprob and (labels is None) == (input_ids is None):
        raise ValueError(f"{what}: give exactly one of labels and input_ids for the log-probs")
    x = _rows_2d(logits)
    n, V = x.shape
    dev = x.device
    rolled = labels is None
    src = labels if labels is not None else input_ids
    lab = None
    if want_logprob:
        if tuple(src.shape) != (n,):
            raise ValueError(f"{what}: labels / input_ids must have shape ({n},), got {tuple(src.shape)}")
        if src.dtype.is_floating_point or src.dtype == torch.bool:
            raise TypeError(f"{what}: labels / input_ids must be an integer tensor, got {src.dtype}")
        lab = src.to(device=dev, dtype=torch.int64).contiguous()
    cu = cu_seqlens.to(device=dev, dtype=torch.int64).contiguous()
    rl = response_lens.to(device=dev, dtype=torch.int64).contiguous()
    B = rl.numel()
    if cu.dim() != 1 or cu.numel() != B + 1:
        raise ValueError(f"{what}: cu_seqlens must have B+1 = {B + 1} entries, got {tuple(cu.shape)}")
    if isinstance(temperature, torch.Tensor) and temperature.dim() == 1 and temperature.numel() == B and B != n and B > 1:
        # one value per sample, as the engine holds it (fsdp/transformer_impl.py:1149-1162)
        from .layout import expand_per_sequence
        temperature = expand_per_sequence(temperature.to(dev), cu, n, check)
    temp = _temperature_rows(temperature, (n,), n, dev)
    T = int(max_response_len)
    if T < 0:
        raise ValueError(f"{what}: max_response_len must not be negative")
    if B == 0 and n > 0:
        raise ValueError(f"{what}: {n} rows but no sequence")
    flag = torch.zeros(1, dtype=torch.int32, device=dev)
    if torch.is_grad_enabled() and logits.requires_grad:
        r_lp, r_h, t_lp, t_h = _ScoreResponsesFunction.apply(
            x, lab, rolled, temp, cu, rl, T, want_logprob, want_entropy, per_token,
            inplace_backward and _is_view_safe(logits), flag)
    else:
        with torch.no_grad():
            r_lp, r_h, t_lp, t_h, _ = _score_responses_launch(x, lab, rolled, temp, cu, rl, T, want_logprob,
                                                              want_entropy, per_token, False, flag)
    if B > 0:
        _errors.report(flag, {
            _lib.VRL_FLAG_LABEL_OOB: (IndexError, f"{what}: a label is outside [0, {V})"),
            _lib.VRL_FLAG_SEQ_RANGE: (ValueError, f"{what}: cu_seqlens is not a partition of the {n} rows "
                                      "(it must start at 0, never decrease and end at the number of rows)"),
            _lib.VRL_FLAG_SLICE_RANGE: (ValueError, f"{what}: a sequence has no prompt token, or a response length "
                                        f"outside [0, {T}]"),
        }, check)
    if per_token:
        return r_lp, r_h, t_lp, t_h
    return r_lp, r_h


# ``LABEL_CHECK`` was this module's switch for the label check before verl_amd.errors took it over; code that still sets
# ``verl_amd.torch_functional.LABEL_CHECK = False`` keeps its meaning (no read-back of the error flag, no host
# synchronisation per direct call) instead of silently losing it.
import sys as _sys
import types as _types
import warnings as _warnings


class _ModuleWithLabelCheck(_types.ModuleType):
    @property
    def LABEL_CHECK(self) -> bool:
        return _errors.DEFAULT_MODE != "off"

    @LABEL_CHECK.setter
    def LABEL_CHECK(self, value) -> None:
        _warnings.warn("verl_amd.torch_functional.LABEL_CHECK is deprecated: set verl_amd.errors.DEFAULT_MODE "
                       "('sync', 'deferred' or 'off'), the VERL_AMD_CHECK environment variable or pass check_labels",
                       DeprecationWarning, stacklevel=2)
        _errors.DEFAULT_MODE = "sync" if value else "off"


_sys.modules[__name__].__class__ = _ModuleWithLabelCheck
