"""Python face of the host library (csrc/host/xrt_host.cpp): the runtime's bookkeeping in native code.

Pools of slots and blocks, the block tables of the cache's groups, the packing of a step and the
generation loop's decisions run in C++, as the reference keeps them in native code
(crates/xrt-runtime/src/kv_cache.rs, session.rs). The library has no part on the GPU and is built with
the host compiler the first time it is needed; if it cannot be built or loaded, loading fails with the
reason: there is no second implementation in Python to fall back on.
"""
from __future__ import annotations

import ctypes
from typing import Optional

from .ops import build as _build

OK, FULL, ERROR = 0, 1, 2
GOES_ON, FINISH_STOP, FINISH_CONTEXT, FINISH_LENGTH = 0, 1, 2, 3
FINISH_REASONS = {GOES_ON: None, FINISH_STOP: "stop", FINISH_CONTEXT: "context", FINISH_LENGTH: "length"}


class HostError(RuntimeError):
    """The host library is missing and cannot be built, or cannot be loaded."""


class StepFacts(ctypes.Structure):
    _fields_ = [("n_tokens", ctypes.c_int), ("n_rows", ctypes.c_int), ("max_count", ctypes.c_int),
                ("max_context", ctypes.c_int), ("is_decode", ctypes.c_int)]


_LIBRARY: Optional[ctypes.CDLL] = None


def load_host() -> ctypes.CDLL:
    global _LIBRARY
    if _LIBRARY is not None:
        return _LIBRARY
    path = _build.find_host_library()
    if path is None:
        try:
            path = _build.build_host(verbose=True)
        except _build.BuildError as error:
            raise HostError(f"the host library is missing and cannot be built: {error}") from None
    try:
        lib = ctypes.CDLL(path)
    except OSError as error:
        raise HostError(f"cannot load {path}: {error}") from None
    P, I, L = ctypes.c_void_p, ctypes.c_int, ctypes.c_long
    IP = ctypes.POINTER(ctypes.c_int)
    signatures = {
        "xrt_host_last_error": (ctypes.c_char_p, []),
        "xrt_pool_new": (P, [I, ctypes.c_char_p]), "xrt_pool_delete": (None, [P]),
        "xrt_pool_acquire": (I, [P, IP]), "xrt_pool_release": (I, [P, I]), "xrt_pool_size": (I, [P]),
        "xrt_pool_n_free": (I, [P]), "xrt_pool_is_held": (I, [P, I]), "xrt_pool_check": (I, [P]),
        "xrt_tables_new": (P, [I, I, I, I, I, P]), "xrt_tables_delete": (None, [P]), "xrt_tables_pool": (P, [P]),
        "xrt_tables_grow": (I, [P, I, I, P, IP]), "xrt_tables_drop": (I, [P, I, P, I]),
        "xrt_tables_shrink_to": (I, [P, I, I]), "xrt_tables_release_all": (I, [P, I]),
        "xrt_tables_first_needed_block": (I, [P, I]), "xrt_tables_floor": (I, [P, I]),
        "xrt_tables_take_changed": (None, [P, IP, IP]), "xrt_tables_check": (I, [P, P]),
        "xrt_step_room": (L, [I, L, L, I]),
        "xrt_step_check": (I, [I, P, P, P, P, P, P, I, I]),
        "xrt_step_pack": (I, [I, P, P, P, P, P, P, I, P, L, ctypes.POINTER(StepFacts)]),
        "xrt_loop_decide": (I, [I, P, I, I, I, I, I, IP]),
        "xrt_loop_goes_on_whatever_it_draws": (I, [I, I, I, I]),
        "xrt_loop_plan_batches": (I, [I, P, P, I, I, L, I, P]),
    }
    for name, (result, arguments) in signatures.items():
        function = getattr(lib, name)
        function.restype, function.argtypes = result, arguments
    lib.path = path
    _LIBRARY = lib
    return lib


def last_error() -> str:
    return load_host().xrt_host_last_error().decode()
