"""ctypes binding of libcce_hip.so (the C ABI declared in include/cce_hip.h).

The library is built in-tree by ``csrc/Makefile`` into ``cut_cross_entropy/_lib``.
There is no fallback: every cce entry point raises if the library is missing or
reports a non-zero status.
"""

import ctypes
import os
import threading
from typing import Optional

import torch

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "_lib", "libcce_hip.so")
_lib: Optional[ctypes.CDLL] = None
_lock = threading.Lock()

ABI_VERSION = 8
DTYPE_CODES = {torch.bfloat16: 0, torch.float16: 1}
STAT_ROWS = 32
STAT_COLS = 32
NUM_COUNTERS = 4
STATIC_SCRATCH_BYTES = 8 * 1024 * 1024

_i64, _i32, _f32, _ptr = ctypes.c_int64, ctypes.c_int, ctypes.c_float, ctypes.c_void_p

_SIGNATURES = {
    "cce_version": (ctypes.c_int, []),
    "cce_error_string": (ctypes.c_char_p, [_i32]),
    "cce_source_hash": (ctypes.c_char_p, []),
    "cce_tile_stat_elems": (_i64, [_i64, _i64]),
    "cce_lse_forward_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "cce_backward_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "cce_lse_forward": (
        _i32,
        [_ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _i64]
        + [_i64] * 4 + [_i64] * 3 + [_f32, _i32, _ptr],
    ),
    "cce_lse_forward_static": (
        _i32,
        [_ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr]
        + [_i64] * 4 + [_i64] * 3 + [_f32, _i32, _ptr],
    ),
    "cce_lse_forward_static_init": (_i32, []),
    "cce_indexed_neg_dot": (
        _i32,
        [_ptr] * 6 + [_i64] * 4 + [_i64] * 3 + [_i64, _i64, _f32, _i32, _ptr],
    ),
    "cce_backward": (
        _i32,
        [_ptr, _ptr, _ptr, _ptr, _ptr, _i32, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _ptr]
        + [_i64] * 4 + [_i64] * 3 + [_f32, _f32, _i32, _i32, _i32, _i32, _i64, _i64, _f32, _i32, _ptr],
    ),
    "cce_count_flagged_cells": (_i32, [_ptr, _ptr, _i64, _i64, _f32, _ptr, _ptr]),
    "cce_backward_dense_workspace_bytes": (_i64, [_i64, _i64, _i64, _i32, _i64]),
    "cce_backward_dense_fixed_bytes": (_i64, [_i64, _i64, _i64, _i32]),
    "cce_backward_dense_dz_bytes": (_i64, [_i64, _i64, _i64, _i32, _i64]),
    "cce_backward_dense": (
        _i32,
        [_ptr, _ptr, _ptr, _ptr, _ptr, _i32, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _i64]
        + [_i64] * 4 + [_i64] * 3 + [_f32, _i32, _i32, _i64, _i64, _f32, _i32, _ptr],
    ),
    "cce_backward_products": (
        _i32,
        [_ptr, _i64, _ptr, _i64, _ptr, _i64, _ptr, _ptr, _i64, _ptr, _i64, _i32, _i64, _i64, _i64, _i32, _ptr],
    ),
    "cce_backward_dz": (
        _i32,
        [_ptr, _ptr, _ptr, _ptr, _ptr, _i32, _ptr, _ptr, _ptr, _ptr, _i64, _i32]
        + [_i64] * 4 + [_i64] * 3 + [_f32, _i64, _i64, _f32, _i32, _ptr],
    ),
}


def lib_path() -> str:
    return _LIB_PATH


_CSRC = os.path.normpath(os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "csrc"))


def _hash_of_sources() -> Optional[str]:
    """The hash csrc/Makefile builds into the library, recomputed from the files in the tree (None when the
    sources are not there, e.g. an installed copy of the package)."""
    import hashlib
    import re

    try:
        text = open(os.path.join(_CSRC, "Makefile")).read()
        names = []
        for var in ("SRCS", "HDRS"):
            names += re.search(rf"^{var} := (.*)$", text, flags=re.M).group(1).split()
        digest = hashlib.sha256()
        for name in names:
            with open(os.path.join(_CSRC, name), "rb") as f:
                digest.update(f.read())
        return digest.hexdigest()[:16]
    except (OSError, AttributeError):
        return None


def load() -> ctypes.CDLL:
    """Load the HIP library once; raise RuntimeError with build instructions if absent."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(
                f"Cut Cross-Entropy HIP library not found at {_LIB_PATH}. "
                "Build it with `make -C ml-cross-entropy_amd/csrc` (needs hipcc, targets gfx950). "
                "There is no non-HIP fallback for the cce implementations."
            )
        lib = ctypes.CDLL(_LIB_PATH)
        for name, (restype, argtypes) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        if lib.cce_version() != ABI_VERSION:
            raise RuntimeError(
                f"libcce_hip.so ABI version {lib.cce_version()} does not match the Python binding ({ABI_VERSION}); rebuild it"
            )
        built_from, sources = lib.cce_source_hash().decode(), _hash_of_sources()
        if sources is not None and built_from != sources:
            raise RuntimeError(
                f"libcce_hip.so was built from other sources (hash {built_from}) than those in {_CSRC} (hash {sources}): "
                "rebuild it with `make -C ml-cross-entropy_amd/csrc`"
            )
        _lib = lib
    return _lib


def check(status: int, what: str) -> None:
    if status != 0:
        msg = load().cce_error_string(status)
        raise RuntimeError(f"{what} failed with status {status}: {msg.decode() if msg else '?'}")


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def dtype_code(dtype: torch.dtype) -> int:
    if dtype not in DTYPE_CODES:
        raise NotImplementedError(
            f"the gfx950 CCE kernels take bfloat16 or float16 inputs, got {dtype}"
        )
    return DTYPE_CODES[dtype]


def require_gpu_tensor(name: str, t: torch.Tensor) -> None:
    if not t.is_cuda:
        raise RuntimeError(
            f"{name} is on {t.device}; the cce implementations run on an AMD GPU only "
            "(use impl='torch_compile' for other devices)"
        )


def current_stream_ptr(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


# Device timings for a benchmark: while a dict is set here, every launcher brackets its library calls with a
# pair of events on the stream it launches on and appends the pair under its name.
_timers: Optional[dict] = None


def set_timers(timers: Optional[dict]) -> None:
    global _timers
    _timers = timers


class timed:
    """``with timed("name", device): lib.call(...)``: free when no benchmark is collecting."""

    def __init__(self, name: str, device: torch.device):
        self.name, self.device = name, device
        self.start = None

    def __enter__(self):
        if _timers is not None:
            self.start = torch.cuda.Event(enable_timing=True)
            self.start.record(torch.cuda.current_stream(self.device))
        return self

    def __exit__(self, *exc):
        if self.start is not None and _timers is not None:
            end = torch.cuda.Event(enable_timing=True)
            end.record(torch.cuda.current_stream(self.device))
            _timers.setdefault(self.name, []).append((self.start, end))
        return False
