"""Loading of the built kernel libraries through ctypes, one library at a time.

A library is compiled the first time one of its functions is asked for (see
`build.ensure`), so a program compiles only what it uses.  There is no other
implementation behind these functions: if a library cannot be built or loaded,
the call raises.
"""
from __future__ import annotations

import ctypes
import threading

from . import build

_p = ctypes.c_void_p
_i = ctypes.c_int
_ll = ctypes.c_longlong
_f = ctypes.c_float

# function name -> (library, argument types); every function returns a hipError_t as int
SIGNATURES = {
    "arle_embed_gather": ("elementwise", [_p, _i, _p, _p, _i, _i, _p]),
    "arle_silu_mul": ("elementwise", [_p, _p, _ll, _p, _i, _i, _i, _i, _p]),
    "arle_rmsnorm": ("norm", [_p, _i, _ll, _p, _i, _p, _i, _p, _i, _i, _f, _p]),
    "arle_add_rmsnorm": ("norm", [_p, _p, _i, _ll, _i, _p, _i, _p, _i, _p, _i, _i, _f, _p]),
    "arle_sum_partials": ("elementwise", [_p, _i, _ll, _p, _i, _ll, _p]),
    "arle_gemm_rows_rounds": ("gemm_rows", [_p, _ll, _p, _ll, _i, _p, _ll, _i, _i, _i, _i, _i, _p]),
    "arle_gemm_rows": ("gemm_rows", [_p, _ll, _p, _ll, _i, _p, _ll, _ll, _i, _i, _i, _i, _i, _i, _i, _i, _p]),
    "arle_gemm_rows_geometry": ("gemm_rows", [_i]),
    "arle_gemm_stream_geometry": ("gemm_rows", [_i]),
    "arle_gemm_stream_lds": ("gemm_rows", [_i, _i, _i]),
    "arle_gemm_stream": ("gemm_rows", [_p, _ll, _p, _ll, _i, _p, _ll, _ll, _i, _i, _i, _i, _i, _i, _i, _i, _p]),
    "arle_gemm_rows_lds": ("gemm_rows", [_i, _i, _i]),
    "arle_gemm_tiles": ("gemm_tiles", [_p, _ll, _p, _p, _ll, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _ll, _p]),
    "arle_gemm_tiles_patch": ("gemm_tiles", [_i, _i]),
    "arle_gemm_rows_lds_max": ("gemm_rows", []),
    "arle_gemm_f32": ("gemm_f32", [_p, _ll, _p, _ll, _p, _ll, _i, _i, _i, _p]),
    "arle_qk_prep": ("rope_kv", [_p, _ll, _p, _ll, _p, _ll, _i, _p, _p, _i, _p, _p, _i, _p, _p, _p,
                                 _i, _p, _p, _i, _i, _i, _i, _i, _f, _p, _i, _ll, _ll, _p]),
    "arle_attn_paged_simt": ("attention_simt", [_p, _ll, _p, _ll, _p, _p, _i, _p, _i, _p, _p, _p, _i,
                                                _i, _i, _i, _i, _f, _i, _p]),
    "arle_attn_decode_prep": ("attention_mfma", [_p, _i, _i, _ll, _ll, _p, _p, _i, _p, _p, _i, _f, _p, _ll, _p, _p, _p, _i, _p,
                                                 _p, _p, _i, _i, _i, _i, _i, _f, _i, _i, _p, _p, _p]),
    "arle_attn_decode_inwg": ("attention_mfma", [_i]),
    "arle_attn_prefill_variant": ("attention_mfma", [_i]),
    "arle_attn_prefill_pair_up": ("attention_mfma", [_i]),
    "arle_attn_prefill_fixed_rounds": ("attention_mfma", [_i]),
    "arle_attn_prefill_groups": ("attention_mfma", [_i]),
    "arle_attn_side_branch": ("attention_mfma", [_i]),
    "arle_attn_paged_mfma": ("attention_mfma", [_p, _ll, _p, _ll, _p, _p, _p, _i, _p, _p, _p, _i, _i, _i, _i, _i, _i,
                                                _i, _i, _i, _f, _i, _i, _p, _p, _i, _p, _p, _ll, _p]),
    "arle_argmax_chunks": ("sampling", [_i, _i]),
    "arle_argmax_rows": ("sampling", [_p, _i, _i, _p, _p, _p]),
    "arle_sample_scratch_bytes": ("sampling", [_i, _i]),
    "arle_sample_rows": ("sampling", [_p, _i, _i, _p, _p, _p, _p, _p, _p, _p, _p, _i, _i, _p]),
    "arle_apply_penalties": ("sampling", [_p, _i, _i, _p, _p, _p, _p, _p, _p, _p]),
    "arle_token_logprobs": ("sampling", [_p, _i, _i, _p, _p, _p]),
    "arle_attn_decode_static": ("attention_mfma", [_p, _ll, _p, _ll, _p, _p, _p, _i, _p, _p, _p, _i, _i, _i, _i, _i,
                                                   _i, _f, _i, _i, _p]),
    "arle_ceiling_read": ("ceilings", [_p, _ll, _i, _p, _p, _p]),
    "arle_ceiling_mfma": ("ceilings", [_i, _i, _i, _i, _p, _p]),
}

_libs: dict = {}
_funcs: dict = {}
_lock = threading.Lock()


class KernelError(RuntimeError):
    pass


def register_signature(name: str, library: str, argtypes: list) -> None:
    SIGNATURES[name] = (library, argtypes)


def library(name: str) -> ctypes.CDLL:
    with _lock:
        lib = _libs.get(name)
        if lib is None:
            path = build.ensure(name)
            try:
                lib = ctypes.CDLL(path)
            except OSError as exc:
                raise KernelError(f"cannot load kernel library {path}: {exc}") from exc
            _libs[name] = lib
        return lib


def loaded_libraries() -> dict:
    """name -> path of the libraries this process has loaded so far."""
    return {n: lib._name for n, lib in _libs.items()}


def function(name: str):
    fn = _funcs.get(name)
    if fn is None:
        lib_name, argtypes = SIGNATURES[name]
        fn = getattr(library(lib_name), name)
        fn.argtypes = argtypes
        fn.restype = ctypes.c_int
        _funcs[name] = fn
    return fn


def function_raw(name: str, restype, library_name: str = "attention_mfma", argtypes=()):
    """A function outside the `int f(...)` convention (one that returns text, say)."""
    fn = getattr(library(library_name), name)
    fn.argtypes = list(argtypes)
    fn.restype = restype
    return fn


def call(name: str, *args) -> None:
    status = function(name)(*args)
    if status != 0:
        raise KernelError(f"{name} failed with HIP error {status}")
