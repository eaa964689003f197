"""Device-side errors without a host synchronisation.

Kernels report what only the device can see (a label outside the vocabulary, packed offsets that do not fit the
arrays, a response window outside its sequence) by OR-ing bits into a caller-owned int32 flag (include/vrl.h,
VRL_FLAG_*). Reading that flag with ``.item()`` drains the whole launch queue, which the reference never does on
this path: its ``torch.gather`` asserts on the device and the error surfaces later
(verl/utils/torch_functional.py:69). This module gives the wrappers the same choice:

``"sync"``      read the flag right after the launch and raise (one host synchronisation per call);
``"deferred"``  copy the flag to pinned host memory behind the kernel (asynchronous, on the same stream), mark it
                with an event, and look at it when the event has completed: at the next verl_amd call on this
                thread or in ``check_errors()``. Nothing ever waits for the GPU except ``check_errors()``, which
                waits on the events only;
``"off"``       never look (the affected results are NaN / zero / unwritten, as documented per entry point).

The default for direct calls is "sync"; ``verl_amd.hook.install()`` runs the installed shims "deferred".
``VERL_AMD_CHECK`` (sync | deferred | off) overrides both; the older ``VERL_AMD_LABEL_CHECK=0`` still means off.
While the current stream is being captured into a HIP graph nothing is read or recorded in any mode.
"""

from __future__ import annotations

import collections
import contextlib
import os
import threading
from typing import Dict, Optional, Tuple, Type

import torch

__all__ = ["check_errors", "pending", "mode", "using", "report", "poll", "discard"]

_MODES = ("sync", "deferred", "off")


def _mode_from_env() -> Optional[str]:
    v = os.environ.get("VERL_AMD_CHECK")
    if v is not None:
        v = v.strip().lower()
        if v not in _MODES:
            raise ValueError(f"VERL_AMD_CHECK must be one of {_MODES}, got {v!r}")
        return v
    legacy = os.environ.get("VERL_AMD_LABEL_CHECK")
    if legacy is not None:
        return "off" if legacy in ("0", "false", "False") else "sync"
    return None


ENV_MODE = _mode_from_env()
DEFAULT_MODE = ENV_MODE or "sync"

_local = threading.local()


def mode() -> str:
    """The mode in force on this thread: the innermost ``using(...)`` block, else the process default."""
    stack = getattr(_local, "stack", None)
    return stack[-1] if stack else DEFAULT_MODE


@contextlib.contextmanager
def using(m: str):
    """Run a block under another mode (thread-local)."""
    if m not in _MODES:
        raise ValueError(f"mode must be one of {_MODES}, got {m!r}")
    stack = getattr(_local, "stack", None)
    if stack is None:
        stack = _local.stack = []
    stack.append(m)
    try:
        yield
    finally:
        stack.pop()


def resolve(check) -> str:
    """A wrapper's ``check_*`` argument -> mode: None = the mode in force, True = "sync", False = "off", or a mode."""
    if check is None:
        return mode()
    if check is True:
        return "sync"
    if check is False:
        return "off"
    if check in _MODES:
        return check
    raise ValueError(f"check must be None, a bool or one of {_MODES}, got {check!r}")


# bit -> (exception type, message)
Messages = Dict[int, Tuple[Type[Exception], str]]


class _Pending:
    __slots__ = ("event", "host", "messages")

    def __init__(self, event, host, messages):
        self.event = event
        self.host = host
        self.messages = messages


_lock = threading.Lock()
_queue: "collections.deque[_Pending]" = collections.deque()
_free_hosts: list = []


def _raise_for(value: int, messages: Messages) -> None:
    for bit, (exc, text) in messages.items():
        if value & bit:
            raise exc(text)


def _take_host() -> torch.Tensor:
    with _lock:
        if _free_hosts:
            return _free_hosts.pop()
    return torch.zeros(1, dtype=torch.int32, pin_memory=True)


def report(flag: torch.Tensor, messages: Messages, check=None) -> None:
    """Handle the device flag of a launch that was just enqueued on the current stream, according to the mode."""
    m = resolve(check)
    if m == "off" or torch.cuda.is_current_stream_capturing():
        return
    if m == "sync":
        _raise_for(int(flag.item()), messages)
        return
    host = _take_host()
    with torch.cuda.device(flag.device):   # copy and event go behind the kernel, on its device's current stream
        host.copy_(flag, non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
    with _lock:
        _queue.append(_Pending(ev, host, messages))


def _pop_completed(block: bool):
    """Entries whose event has completed (all of them, after waiting, when ``block``), oldest first."""
    done = []
    while True:
        with _lock:
            if not _queue:
                break
            head = _queue[0]
        if block:
            head.event.synchronize()
        elif not head.event.query():
            break
        with _lock:
            if _queue and _queue[0] is head:
                _queue.popleft()
            else:
                continue
        done.append(head)
    return done


def _settle(done) -> None:
    first = None
    for p in done:
        view = p.host.numpy()       # pinned host memory: a plain read, no device involved
        value = int(view[0])
        view[0] = 0
        with _lock:
            _free_hosts.append(p.host)
        if first is None and value:
            first = (value, p.messages)
    if first is not None:
        _raise_for(*first)


def poll() -> None:
    """Raise the oldest error among the deferred checks that have completed; never waits for the GPU."""
    if not _queue or torch.cuda.is_current_stream_capturing():
        return
    _settle(_pop_completed(block=False))


def check_errors() -> None:
    """Wait for every deferred check (on its event only, not on the device) and raise the oldest error found."""
    if not _queue:
        return
    _settle(_pop_completed(block=True))


def pending() -> int:
    """Deferred checks not looked at yet."""
    return len(_queue)


def discard() -> None:
    """Forget every deferred check without looking (their kernels may still be running; the buffers are dropped)."""
    with _lock:
        _queue.clear()
