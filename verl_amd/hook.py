"""Put the HIP scoring path behind verl's own function names.

What gets replaced (verl/utils/torch_functional.py):
    logprobs_from_logits :73, logprobs_from_logits_v2 :173, logprobs_from_logits_naive :155,
    entropy_from_logits :231, entropy_from_logits_with_chunking :248,
    calculate_sum_pi_squared_from_logits :690
and every copy of those names that an already imported ``verl.*`` module bound
with ``from verl.utils.torch_functional import ...`` (the engines do so at
verl/workers/engine/fsdp/transformer_impl.py:66 and siblings; the reference's
own tests patch exactly that bound name,
tests/workers/test_distillation_topk_symmetry_on_cpu.py:143-146).

Also replaced, when the modules import (they are opt-in paths of the reference, use_fused_kernels):
    verl.utils.experimental.torch_functional.FusedLinearForPPO :211-231
    verl.utils.kernel.linear_cross_entropy.linear_cross_entropy :119
which the model forwards look up at call time (verl/models/transformers/dense_common.py:89,157).

A replaced function sends GPU tensors of a supported dtype to the HIP kernels
(forward, and backward when the logits need a gradient). Anything else (CPU
tensors on the driver, fp64) is handed to the function it replaced, i.e. verl's own
code, and counted in ``stats()``: this package adds no second implementation.
"""

from __future__ import annotations

import functools
import importlib
import os
import sys
import threading
import weakref
from typing import Callable, Dict, List, Optional, Tuple

import torch

from . import _lib
from . import errors as _errors
from . import fused_linear as _fl
from . import torch_functional as _amd

# Device-side errors (a label outside the vocabulary) of the installed functions are looked at without ever waiting for
# the GPU, like the asynchronous device assert of the torch.gather they replace (verl/utils/torch_functional.py:69):
# at a later shim call once the kernel has finished, or in check_errors(). VERL_AMD_CHECK=sync|off overrides.
SHIM_CHECK_MODE = _errors.ENV_MODE or "deferred"
check_errors = _errors.check_errors

TARGET_MODULE = "verl.utils.torch_functional"
PATCHED_NAMES = (
    "logprobs_from_logits",
    "logprobs_from_logits_v2",
    "logprobs_from_logits_naive",
    "entropy_from_logits",
    "entropy_from_logits_with_chunking",
    "calculate_sum_pi_squared_from_logits",
)

# One pass serves two calls. verl's engines ask for the entropy and for the label log-probs of the SAME logits tensor
# in two separate calls (verl/workers/engine/fsdp/transformer_impl.py:1364-1376 and :1395-1399). The first of the two
# runs the row kernel once and leaves what the other needs: after an entropy call the per-row logsumexp (the log-prob
# call is then one element load per row, vrl_label_logprob), after a log-prob call the per-row entropy. With
# gradients the pair also shares ONE backward pass over the logits (see _EntropyLseFunction in torch_functional).
#
# What is left behind is tied to the tensor OBJECT (weak reference), its version counter (any in-place write through
# torch bumps it, also through views), its address, shape, strides, dtype, the stream and whether gradients are being
# recorded. It is single-use and short-lived: only the NEXT shim call can take it, only a call of the other kind
# (log-prob after entropy, entropy after log-prob), and it is dropped whatever that next call is. A write that torch's
# version counter does not see (``logits.data`` ops, a raw-pointer kernel such as the in-place backward, replay of a
# captured graph into a static buffer) between the two calls of a pair is NOT detected. Nothing is shared while the
# stream is being captured. VERL_AMD_MEMO=0 switches the sharing off.
MEMO = os.environ.get("VERL_AMD_MEMO", "1") not in ("0", "false", "False")


class _RowMemo:
    """What one pass over a logits tensor left for the other call of the pair."""

    __slots__ = ("ref", "version", "ptr", "shape", "stride", "dtype", "stream", "needs_grad", "kind", "entropy", "lse",
                 "pair", "_watch")

    def __init__(self, logits, stream, needs_grad, kind, entropy=None, lse=None, pair=None):
        self.ref = weakref.ref(logits)
        self.version = logits._version
        self.ptr = logits.data_ptr()
        self.shape = tuple(logits.shape)
        self.stride = tuple(logits.stride())
        self.dtype = logits.dtype
        self.stream = stream
        self.needs_grad = needs_grad
        self.kind = kind          # "entropy": left by an entropy call (holds lse); "logprob": by a log-prob call (holds entropy)
        self.entropy = entropy
        self.lse = lse
        self.pair = pair          # grad mode, kind "entropy": the dict the two autograd nodes share
        self._watch = None

    def release_with(self, result) -> None:
        """With gradients what is held carries the first call's autograd graph, and through it the logits. Let it go
        when ``result``, the tensor that call returned, dies: a caller that never makes the second call of the pair then
        keeps nothing alive beyond its own reference to the result."""
        self._watch = weakref.finalize(result, self.drop)
        self._watch.atexit = False

    def drop(self) -> None:
        self.entropy = self.lse = self.pair = None
        if self._watch is not None:
            self._watch.detach()     # (the finalizer holds this record; without it the record dies with its last user)
            self._watch = None

    def matches(self, logits, stream, needs_grad) -> bool:
        return (self.ref() is logits and self.version == logits._version and self.ptr == logits.data_ptr()
                and self.shape == tuple(logits.shape) and self.stride == tuple(logits.stride())
                and self.dtype == logits.dtype and self.stream == stream and self.needs_grad == needs_grad)


_memo_local = threading.local()   # per thread: a pair of calls is made by one thread


def _memo_take() -> Optional[_RowMemo]:
    """The record the thread's last shim call left, which is gone from the thread afterwards; its tensors stay with the
    returned object until the caller lets go of it."""
    memo = getattr(_memo_local, "memo", None)
    _memo_local.memo = None
    if memo is not None and memo._watch is not None:
        memo._watch.detach()
        memo._watch = None
    return memo


def _memo_store(memo: _RowMemo, result=None) -> None:
    _memo_clear()
    if memo.needs_grad and result is not None:
        memo.release_with(result)
    _memo_local.memo = memo


def _memo_clear() -> None:
    memo = getattr(_memo_local, "memo", None)
    _memo_local.memo = None
    if memo is not None:
        memo.drop()


def clear_memo() -> None:
    """Drop what the calling thread's last shim call left for the other call of its pair. With gradients that record
    holds a per-row vector with the first call's autograd graph, and through it the logits; it goes by itself at the
    thread's next shim call or when the tensor that first call returned dies, whichever comes first."""
    _memo_clear()


_LOGPROB_NAMES = ("logprobs_from_logits", "logprobs_from_logits_v2", "logprobs_from_logits_naive")
_ENTROPY_NAMES = ("entropy_from_logits", "entropy_from_logits_with_chunking")


def _plain_rows(logits):
    """(N, V) view of ``logits`` when it is one plain row-major block, else None."""
    if _amd._is_batch_of_row_slices(logits):
        return None
    x = _amd._rows_2d(logits)
    if x.data_ptr() != logits.data_ptr() or x.shape[0] == 0:
        return None
    return x


def _memo_serve(name, logits, args, kwargs):
    """The result of ``name(logits, ...)`` from a pass shared with the other call of the pair, or None when the
    ordinary route must be taken. Whatever happens, a record left by the call before is gone afterwards."""
    memo = _memo_take()
    if not MEMO or logits.is_inference() or torch.cuda.is_current_stream_capturing():
        return None   # (inference-mode tensors have no version counter to check against)
    if name not in _ENTROPY_NAMES and name not in _LOGPROB_NAMES:
        return None
    x = _plain_rows(logits)
    if x is None:
        return None
    lead = logits.shape[:-1]
    needs_grad = torch.is_grad_enabled() and logits.requires_grad
    stream = _lib.stream_ptr(logits.device)
    hit = memo is not None and memo.matches(logits, stream, needs_grad)

    if name in _ENTROPY_NAMES:
        if name == "entropy_from_logits_with_chunking":
            chunk = args[0] if args else kwargs.get("chunk_size", 2048)
            if int(chunk) <= 0:
                return None   # the ordinary route raises
        if hit and memo.kind == "logprob":
            _stats["memo_hits"] += 1
            return memo.entropy
        if needs_grad:
            pair = {}
            h, lse = _amd._EntropyLseFunction.apply(x, None, None, pair)
            out = h.reshape(lead)
            _memo_store(_RowMemo(logits, stream, True, "entropy", lse=lse, pair=pair), out)
            return out
        with torch.no_grad():
            _, h, _, lse, _ = _amd._forward_2d(x, None, None, False, True, False, True, None)
        _memo_store(_RowMemo(logits, stream, False, "entropy", lse=lse))
        return h.reshape(lead)

    labels = args[0] if args else kwargs.get("labels")
    if (not isinstance(labels, torch.Tensor) or tuple(labels.shape) != tuple(lead) or labels.dtype.is_floating_point
            or labels.dtype == torch.bool):
        return None
    lab = labels.to(device=x.device, dtype=torch.int64).reshape(-1).contiguous()
    inplace = False
    if name == "logprobs_from_logits":
        inplace = bool(args[1] if len(args) > 1 else kwargs.get("inplace_backward", True)) and _amd._is_view_safe(logits)
    messages = _amd._label_messages(name, logits.shape[-1])
    if hit and memo.kind == "entropy":
        _stats["memo_hits"] += 1
        if needs_grad:
            lp, flag = _amd._LabelLogprobFunction.apply(x, lab, None, memo.lse, memo.pair, inplace, None)
        else:
            with torch.no_grad():
                lp, flag = _amd._label_logprob(x, lab, None, memo.lse)
        _errors.report(flag, messages)
        return lp.reshape(lead)
    if needs_grad:
        lp, h, flag = _amd._RowScoreFunction.apply(x, lab, None, True, True, None, inplace, None)
    else:
        with torch.no_grad():
            lp, h, _, _, flag = _amd._forward_2d(x, lab, None, True, True, False, False, None)
    out = lp.reshape(lead)
    _memo_store(_RowMemo(logits, stream, needs_grad, "logprob", entropy=h.reshape(lead)), out)
    _errors.report(flag, messages)
    return out


_originals: Dict[str, Callable] = {}
_rebound: List[Tuple[object, str, Callable]] = []
_stats = {"hip_calls": 0, "passed_to_verl": 0, "memo_hits": 0}


def _eligible(logits) -> bool:
    # plain tensors only: a DTensor, a nested or a fake tensor has no single device buffer to hand to a kernel
    return (
        type(logits) in (torch.Tensor, torch.nn.Parameter)
        and not logits.is_nested
        and logits.is_cuda
        and logits.dtype in (torch.float32, torch.bfloat16, torch.float16)
        and logits.dim() >= 1
        and logits.shape[-1] > 0
    )


def _make_shim(name: str, original: Callable) -> Callable:
    ours = getattr(_amd, name)

    def serve(logits, *args, **kwargs):
        if _eligible(logits):
            _stats["hip_calls"] += 1
            with _errors.using(SHIM_CHECK_MODE):
                _errors.poll()
                served = _memo_serve(name, logits, args, kwargs)
                if served is not None:
                    return served
                return ours(logits, *args, **kwargs)
        _memo_clear()
        _stats["passed_to_verl"] += 1
        return original(logits, *args, **kwargs)

    # The engines wrap entropy_from_logits in torch.compile when use_torch_compile is set
    # (verl/workers/engine/fsdp/transformer_impl.py:164-168). There is nothing to trace in a ctypes call into a
    # finished kernel. torch.compile unwraps a function that is itself marked torch.compiler.disable and traces
    # it anyway, so the mark goes on an inner function and the patched name is a plain wrapper around it: the
    # tracer sees one call it must not enter and runs it as it is.
    serve_untraced = torch.compiler.disable(serve)

    @functools.wraps(original)
    def shim(logits, *args, **kwargs):
        return serve_untraced(logits, *args, **kwargs)

    shim.__verl_amd_original__ = original
    return shim


def _eligible_pair(hidden, weight) -> bool:
    return (_eligible(hidden) and isinstance(weight, torch.Tensor) and weight.is_cuda and weight.dtype == hidden.dtype
            and weight.dim() == 2)


def _make_fused_linear_class(original_cls):
    class FusedLinearForPPO(_fl.FusedLinearForPPO):
        """verl_amd's module with the reference's class as the fallback for inputs the kernels do not take."""

        def __init__(self, chunk_size=None):
            super().__init__(_fl.DEFAULT_CHUNK_TOKENS if chunk_size is None else chunk_size)
            self._verl_module = original_cls() if chunk_size is None else original_cls(chunk_size)

        def forward(self, hidden_states, vocab_weights, input_ids, temperature=1.0):
            if _eligible_pair(hidden_states, vocab_weights):
                _stats["hip_calls"] += 1
                with _errors.using(SHIM_CHECK_MODE):
                    return super().forward(hidden_states, vocab_weights, input_ids, temperature)
            _stats["passed_to_verl"] += 1
            return self._verl_module.forward(hidden_states, vocab_weights, input_ids, temperature)

    FusedLinearForPPO.__verl_amd_original__ = original_cls
    return FusedLinearForPPO


def _make_linear_cross_entropy(original):
    def serve(hidden, weight, labels, temperature=1.0, reduction="none", dist_process_group=None):
        if dist_process_group is None and _eligible_pair(hidden, weight):
            _stats["hip_calls"] += 1
            with _errors.using(SHIM_CHECK_MODE):
                return _fl.linear_cross_entropy(hidden, weight, labels, temperature, reduction)
        _stats["passed_to_verl"] += 1
        return original(hidden, weight, labels, temperature, reduction, dist_process_group)

    serve_untraced = torch.compiler.disable(serve)   # see _make_shim

    @functools.wraps(original)
    def linear_cross_entropy(hidden, weight, labels, temperature=1.0, reduction="none", dist_process_group=None):
        return serve_untraced(hidden, weight, labels, temperature, reduction, dist_process_group)

    linear_cross_entropy.__verl_amd_original__ = original
    return linear_cross_entropy


# (module below the package root, attribute, shim factory)
_OPTIONAL_TARGETS = (
    ("utils.experimental.torch_functional", "FusedLinearForPPO", _make_fused_linear_class),
    ("utils.kernel.linear_cross_entropy", "linear_cross_entropy", _make_linear_cross_entropy),
)
_optional_patched: List[Tuple[object, str, object]] = []


def stats() -> dict:
    """Calls served by the HIP kernels vs handed back to verl since install(), second calls of a pair served from the
    first one's pass, and the passes over logits launched so far (forward, backward, label gathers)."""
    return {**_stats, **_amd.counters}


def install(target_module: str = TARGET_MODULE) -> List[str]:
    """Patch ``target_module`` and re-bind the names in already imported ``verl.*`` modules.

    Returns the fully qualified names that were replaced. Calling it twice is a no-op.
    """
    if _originals:
        return []
    mod = importlib.import_module(target_module)
    replaced = []
    shims = {}
    for name in PATCHED_NAMES:
        original = getattr(mod, name, None)
        if original is None:
            continue
        shim = _make_shim(name, original)
        _originals[name] = original
        shims[name] = shim
        setattr(mod, name, shim)
        replaced.append(f"{target_module}.{name}")
    root = target_module.split(".")[0] + "."
    for mod_name, other in list(sys.modules.items()):
        if other is None or other is mod or not mod_name.startswith(root):
            continue
        for name, shim in shims.items():
            if getattr(other, name, None) is _originals[name]:
                setattr(other, name, shim)
                _rebound.append((other, name, _originals[name]))
                replaced.append(f"{mod_name}.{name}")
    _installed_in.append(mod)
    for sub, name, factory in _OPTIONAL_TARGETS:
        try:
            other = importlib.import_module(root + sub)
        except ImportError:
            continue
        original = getattr(other, name, None)
        if original is None:
            continue
        setattr(other, name, factory(original))
        _optional_patched.append((other, name, original))
        replaced.append(f"{root}{sub}.{name}")
    return replaced


_installed_in: List[object] = []


def uninstall() -> None:
    """Undo install()."""
    for other, name, original in _rebound:
        setattr(other, name, original)
    _rebound.clear()
    for mod in _installed_in:
        for name, original in _originals.items():
            setattr(mod, name, original)
    _installed_in.clear()
    _originals.clear()
    for other, name, original in _optional_patched:
        setattr(other, name, original)
    _optional_patched.clear()
    _stats["hip_calls"] = 0
    _stats["passed_to_verl"] = 0
    _stats["memo_hits"] = 0
    _memo_clear()
