"""ctypes binding of libvrl_hip.so (the C ABI declared in include/vrl.h).

There is no other implementation behind these functions: if the library is
missing or was not built, every call raises, it never computes elsewhere.
"""

from __future__ import annotations

import ctypes
import os
import threading

LIB_NAME = "libvrl_hip.so"
# VERL_AMD_LIB names another build of the same library (the host-sanitised one the ABI tests run against).
LIB_PATH = os.environ.get("VERL_AMD_LIB") or os.path.join(os.path.dirname(os.path.abspath(__file__)), LIB_NAME)

VRL_OK = 0
VRL_ERR_NULL = -1
VRL_ERR_DTYPE = -2
VRL_ERR_SHAPE = -3
VRL_ERR_ALIGN = -4
VRL_ERR_HIP = -5
VRL_ERR_ARG = -6
VRL_ERR_SCRATCH = -7
STATIC_PARTIALS_MAX = 8192

VRL_F32 = 0
VRL_BF16 = 1
VRL_F16 = 2

VRL_FLAG_LABEL_OOB = 1
VRL_FLAG_SLICE_RANGE = 2
VRL_FLAG_SEQ_RANGE = 4

ABI_VERSION = 4

_c = ctypes
_P = _c.c_void_p
_I64 = _c.c_int64
_INT = _c.c_int
_F32 = _c.c_float

# name -> (restype, argtypes); mirrors include/vrl.h one to one.
SIGNATURES = {
    "vrl_rowscore": (_INT, [_P, _INT, _I64, _I64, _I64, _P, _P, _P, _P, _P, _P, _P, _P]),
    "vrl_label_logprob": (_INT, [_P, _INT, _I64, _I64, _I64, _P, _P, _P, _P, _P, _P]),
    "vrl_rowscore_split": (_INT, [_P, _INT, _I64, _I64, _I64, _P, _P, _P, _P, _P, _P, _P, _INT, _P, _P]),
    "vrl_rowscore_split_static": (_INT, [_P, _INT, _I64, _I64, _I64, _P, _P, _P, _P, _P, _P, _P, _INT, _P]),
    "vrl_rowscore_backward": (_INT, [_P, _INT, _I64, _I64, _I64, _P, _P, _P, _P, _P, _P, _P, _I64, _P]),
    "vrl_rowscore_split_plan": (_INT, [_INT, _I64, _I64]),
    "vrl_score_responses": (_INT, [_P, _INT, _I64, _I64, _I64, _P, _P, _P, _P, _P, _I64, _I64, _P, _P, _P, _P, _P, _P, _P]),
    "vrl_score_responses_backward": (
        _INT, [_P, _INT, _I64, _I64, _I64, _P, _P, _P, _P, _P, _I64, _I64, _P, _P, _P, _P, _P, _I64, _P]),
    "vrl_response_slice": (_INT, [_P, _I64, _P, _P, _I64, _I64, _I64, _P, _P, _P]),
    "vrl_response_pack": (_INT, [_P, _I64, _P, _P, _P, _I64, _I64, _I64, _P, _P, _P]),
    "vrl_expand_per_sequence": (_INT, [_P, _P, _I64, _I64, _P, _P, _P]),
    "vrl_lmhead_score": (_INT, [_P, _P, _INT, _I64, _I64, _I64, _I64, _I64, _P, _P, _INT, _P, _P, _P, _P, _P, _P, _I64, _I64,
                                _P]),
    "vrl_lmhead_dlogits": (_INT, [_P, _P, _INT, _I64, _I64, _I64, _I64, _I64, _P, _P, _P, _P, _P, _P, _INT, _P, _I64, _P]),
    "vrl_gemm_nt_plan": (_INT, [_INT, _I64, _I64, _I64, _P]),
    "vrl_gemm_nt": (_INT, [_P, _P, _INT, _I64, _I64, _I64, _I64, _I64, _P, _I64, _INT, _INT, _P, _P]),
    "vrl_gemm": (_INT, [_P, _P, _INT, _I64, _I64, _I64, _I64, _I64, _INT, _INT, _P, _I64, _INT, _INT, _P, _P]),
    "vrl_lmhead_plan": (_INT, [_I64, _I64]),
    "vrl_lmhead_partials": (_I64, [_I64, _I64]),
    "vrl_transpose": (_INT, [_P, _INT, _I64, _I64, _I64, _P, _I64, _P]),
    "vrl_rollout_corr": (
        _INT,
        [_P, _P, _P, _I64, _I64, _INT, _INT, _F32, _F32, _F32, _c.c_uint32, _P, _P, _P, _P, _P, _P, _P],
    ),
    "vrl_rollout_corr_num_stats": (_INT, []),
    "vrl_spec_verify": (
        _INT,
        [_P, _P, _P, _P, _P, _I64, _I64, _I64, _F32, _F32, _P, _P, _P, _P, _P, _I64, _P, _P, _P, _P, _I64, _P],
    ),
    "vrl_spec_verify_workspace": (_I64, [_I64]),
    "vrl_spec_verify_plan": (_INT, [_INT, _I64, _I64, _I64]),
    "vrl_truncate_draft": (_INT, [_P, _P, _P, _I64, _I64, _I64, _P, _I64, _P, _P, _P, _P]),
    "vrl_fused_score_verify": (
        _INT,
        [_P, _INT, _I64, _I64, _I64, _P, _P, _P, _P, _P, _P, _P]
        + [_P, _P, _P, _P, _I64, _I64, _F32, _F32, _P, _P, _P, _P, _P, _I64, _P, _P, _P],
    ),
    "vrl_strerror": (_c.c_char_p, [_INT]),
    "vrl_last_hip_error": (_c.c_char_p, []),
    "vrl_abi_version": (_INT, []),
}


class VrlLibraryError(RuntimeError):
    """The HIP library is absent, unloadable, or of another ABI version."""


class VrlCallError(RuntimeError):
    """An entry point returned a negative status."""

    def __init__(self, func: str, status: int, text: str):
        super().__init__(f"{func} failed with status {status}: {text}")
        self.func = func
        self.status = status


_lock = threading.Lock()
_lib = None


def load(path: str | None = None):
    """Load the library once and return the ctypes handle; raise VrlLibraryError if impossible."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    with _lock:
        if _lib is not None and path is None:
            return _lib
        p = path or LIB_PATH
        if not os.path.exists(p):
            raise VrlLibraryError(
                f"{p} does not exist. Build it with `python -m verl_amd.build` (needs hipcc); "
                "verl_amd has no other implementation to fall back to."
            )
        try:
            lib = ctypes.CDLL(p)
        except OSError as exc:  # missing libamdhip64 etc.
            raise VrlLibraryError(f"cannot load {p}: {exc}") from exc
        for name, (restype, argtypes) in SIGNATURES.items():
            try:
                fn = getattr(lib, name)
            except AttributeError as exc:
                raise VrlLibraryError(f"{p} does not export {name}") from exc
            fn.restype = restype
            fn.argtypes = argtypes
        got = lib.vrl_abi_version()
        if got != ABI_VERSION:
            raise VrlLibraryError(f"{p} has ABI version {got}, this package needs {ABI_VERSION}")
        if path is None:
            _lib = lib
        return lib


def strerror(status: int) -> str:
    return load().vrl_strerror(status).decode()


def stream_ptr(device) -> int:
    """The raw ``hipStream_t`` of torch's current stream on ``device``, as the integer the ``void* stream`` arguments
    take. Read from the runtime directly: the ``torch.cuda.Stream`` wrapper is replaced by a generic object without a
    handle inside functions that torch.compile was told not to trace."""
    import torch

    index = device.index if getattr(device, "index", None) is not None else torch.cuda.current_device()
    return int(torch._C._cuda_getCurrentRawStream(index))


def check(func: str, status: int) -> None:
    """Raise VrlCallError for a negative status."""
    if status == VRL_OK:
        return
    lib = load()
    text = lib.vrl_strerror(status).decode()
    if status == VRL_ERR_HIP:
        text += f" ({lib.vrl_last_hip_error().decode()})"
    raise VrlCallError(func, status, text)
