"""The host-side runtime core (C++, `arle_amd/csrc/host/runtime.cpp`) through ctypes.

Built with the host compiler the first time it is asked for, like the kernel libraries.  There is no
Python implementation behind it: if the library cannot be built or loaded, the call raises.
"""
from __future__ import annotations

import ctypes
import threading

from ..kernels import build

_p, _i, _ll = ctypes.c_void_p, ctypes.c_int, ctypes.c_longlong
_ip, _cp = ctypes.POINTER(ctypes.c_int), ctypes.c_char_p

_SIGNATURES = {
    "arle_group_create": (_p, [_i, _i, _i]),
    "arle_group_destroy": (None, [_p]),
    "arle_group_num_pages": (_i, [_p]),
    "arle_group_free_count": (_i, [_p]),
    "arle_group_held_count": (_i, [_p]),
    "arle_group_take": (_i, [_p, _i, _ip]),
    "arle_group_give_back": (_i, [_p, _ip, _i]),
    "arle_group_open": (_i, [_p, _ll]),
    "arle_group_pages_needed": (_i, [_p, _ll, _i]),
    "arle_group_free_tokens": (_ll, [_p]),
    "arle_group_append": (_i, [_p, _ll, _i, _ip, _ip, _i]),
    "arle_group_truncate": (_i, [_p, _ll, _i, _ip, _ip, _i]),
    "arle_group_trim": (_i, [_p, _ll, _ip, _i]),
    "arle_group_close": (_i, [_p, _ll]),
    "arle_group_table": (_i, [_p, _ll, _ip, _i, _ip, _ip]),
    "arle_group_check": (_i, [_p, ctypes.c_char_p, _i]),
    "arle_pack_step": (_i, [_i, _p, _p, _p, _p, _p, _p, _i, _p, _ll, _ip, _ip]),
    "arle_retract_victim": (_i, [_i, _ip, _ip]),
    "arle_plan_prefill": (_i, [_i, _p, _i, _p, _ip, _i, _p, _ip, _ip, _i, _i, _i, _i, _i, _i, _i, _ip, _ip]),
    "arle_aligned_portion": (_i, [_i, _i, _i, _i]),
    "arle_admit": (_i, [_i, _ip, _ip, _i, _i, _ip, _ip, _i, _ip, _ip]),
}

UNKNOWN_KEY, OUT_OF_PAGES, BUFFER_TOO_SMALL, OUT_OF_RANGE, NOT_HELD, KEY_EXISTS = -1, -2, -3, -4, -5, -6

_lib = None
_lock = threading.Lock()


def lib() -> ctypes.CDLL:
    global _lib
    with _lock:
        if _lib is None:
            path = build.ensure("host")
            try:
                loaded = ctypes.CDLL(path)
            except OSError as exc:
                raise RuntimeError(f"cannot load the host runtime library {path}: {exc}") from exc
            for name, (restype, argtypes) in _SIGNATURES.items():
                fn = getattr(loaded, name)
                fn.restype, fn.argtypes = restype, argtypes
            _lib = loaded
        return _lib


def int_array(n: int):
    return (ctypes.c_int * max(n, 1))()
