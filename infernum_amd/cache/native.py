"""ctypes face of the host library (``csrc/host_core.cpp``): page pools, block
tables, state slots and the packing of a step, kept natively.  The library is
plain C++ and needs no GPU; it is compiled at its first use like the kernel
libraries."""
from __future__ import annotations

import ctypes
from ctypes import POINTER, c_char_p, c_float, c_int, c_int32, c_int64, c_size_t, c_void_p
from typing import Optional

from ..csrc import build as _build

HOST_ERROR = -2
_lib: Optional[ctypes.CDLL] = None

_SIGNATURES = {
    "ia_pool_create": (c_void_p, [c_int]),
    "ia_pool_destroy": (None, [c_void_p]),
    "ia_pool_error": (c_char_p, [c_void_p]),
    "ia_pool_num_pages": (c_int, [c_void_p]),
    "ia_pool_num_free": (c_int, [c_void_p]),
    "ia_pool_allocate": (c_int, [c_void_p]),
    "ia_pool_allocate_many": (c_int, [c_void_p, c_int, POINTER(c_int)]),
    "ia_pool_free": (c_int, [c_void_p, c_int]),
    "ia_pool_is_used": (c_int, [c_void_p, c_int]),
    "ia_cache_create": (c_void_p, [c_int, POINTER(c_int), POINTER(c_int), c_int, c_int, c_int]),
    "ia_cache_destroy": (None, [c_void_p]),
    "ia_cache_error": (c_char_p, [c_void_p]),
    "ia_cache_group_pool": (c_void_p, [c_void_p, c_int]),
    "ia_cache_num_free_slots": (c_int, [c_void_p]),
    "ia_cache_num_requests": (c_int, [c_void_p]),
    "ia_cache_has": (c_int, [c_void_p, c_int64]),
    "ia_cache_acquire_slot": (c_int, [c_void_p]),
    "ia_cache_release_slot": (c_int, [c_void_p, c_int]),
    "ia_cache_admit": (c_int, [c_void_p, c_int64]),
    "ia_cache_state_slot": (c_int, [c_void_p, c_int64]),
    "ia_cache_num_tokens": (c_int64, [c_void_p, c_int64]),
    "ia_cache_pages_needed": (c_int, [c_void_p, c_int, c_int64, c_int64, POINTER(c_int)]),
    "ia_cache_tokens_that_fit": (c_int64, [c_void_p, c_int, c_int64, POINTER(c_int)]),
    "ia_cache_can_reserve": (c_int, [c_void_p, c_int64, c_int64]),
    "ia_cache_reserve": (c_int, [c_void_p, c_int64, c_int64]),
    "ia_cache_commit": (c_int, [c_void_p, c_int64, c_int64]),
    "ia_cache_release": (c_int, [c_void_p, c_int64]),
    "ia_cache_last_freed": (c_int, [c_void_p, POINTER(c_int), c_int]),
    "ia_cache_table": (c_int, [c_void_p, c_int, c_int64, POINTER(c_int), c_int, POINTER(c_int64), POINTER(c_int)]),
    "ia_cache_step_fits": (c_int, [c_void_p, c_int, POINTER(c_int64), POINTER(c_int), POINTER(c_int)]),
    "ia_cache_reserve_step": (c_int, [c_void_p, c_int, POINTER(c_int64), POINTER(c_int)]),
    "ia_cache_commit_step": (c_int, [c_void_p, c_int, POINTER(c_int64), POINTER(c_int)]),
    "ia_cache_unreserve_step": (c_int, [c_void_p, c_int, POINTER(c_int64)]),
    "ia_cache_check": (c_int, [c_void_p]),
    # the interpreter of a step's program (csrc/step_program.cpp)
    "ia_program_create": (c_void_p, []),
    "ia_program_destroy": (None, [c_void_p]),
    "ia_program_error": (c_char_p, [c_void_p]),
    "ia_program_num_ops": (c_int, [c_void_p]),
    "ia_program_last_launches": (ctypes.c_longlong, [c_void_p]),
    "ia_program_add_op": (c_int, [c_void_p, c_void_p, c_char_p, POINTER(c_int64), c_int, POINTER(c_int64), c_int, c_int]),
    "ia_program_finish": (c_int, [c_void_p, c_int, c_int]),
    "ia_program_run": (c_int, [c_void_p, POINTER(c_int64), c_int, POINTER(c_void_p), c_int, c_void_p]),
    "ia_cache_token_slots": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int, POINTER(c_int32)]),
    "ia_cache_pack_step": (c_int, [c_void_p, c_int, POINTER(c_int64), POINTER(c_int), POINTER(c_int32), POINTER(c_int),
                                   POINTER(c_int32), c_int, c_int, POINTER(c_int32), c_int]),
    "ia_cache_packed": (POINTER(c_int32), [c_void_p]),
    "ia_sched_step": (c_int, [c_void_p, c_int, POINTER(c_int64), POINTER(c_int), POINTER(c_int64), c_int,
                              POINTER(c_int64), c_int, c_int, c_int, c_int, POINTER(c_int), c_int]),
}


class HostLibraryError(RuntimeError):
    """The host library could not be built or loaded."""


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        try:
            loaded = ctypes.CDLL(_build.ensure("host"))
        except (OSError, _build.BuildError) as e:
            raise HostLibraryError(f"the host library could not be built or loaded: {e}") from e
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(loaded, name)
            fn.restype, fn.argtypes = res, args
        _lib = loaded
    return _lib
