"""ctypes binding of the HIP kernel library. There is no fallback: a missing GPU or library is an error."""
from __future__ import annotations

import ctypes
from ctypes import c_int, c_long, c_float, c_void_p, c_uint64

from . import build as _build

_lib = None

P, I, L, F = c_void_p, c_int, c_long, c_float

_SIGNATURES = {
    "tw_error_string": (ctypes.c_char_p, [I]),
    "tw_abi_version": (I, []),
    "tw_graph_begin": (I, [P]),
    "tw_graph_end": (I, [P, ctypes.POINTER(c_void_p)]),
    "tw_graph_launch": (I, [P, P]),
    "tw_graph_destroy": (I, [P]),
    "tw_probe_read": (I, [P, L, P, I, ctypes.POINTER(c_long), P]),
    "tw_upload_words": (I, [P, P, I, ctypes.POINTER(c_int), ctypes.POINTER(c_int), P]),
    "tw_embed_gather": (I, [I, P, P, P, I, I, I, P, I, P]),
    "tw_rmsnorm": (I, [I, P, P, P, P, I, I, F, P, I, L, P, P]),
    "tw_rope_table": (I, [P, P, P, P, I, I, P]),
    "tw_rope_kv_write": (I, [I, P, L, P, P, P, P, P, I, I, I, I, I, I, I, P, I, P, I, P]),
    "tw_silu_mul": (I, [I, P, P, I, I, P]),
    "tw_linear_workspace_bytes": (L, [I, I, I, I]),
    "tw_linear_partial_splits": (I, [I, I, I]),
    "tw_linear_partial_splits_rows": (I, [I, I, I, I, I, L]),
    "tw_linear_partials": (I, [I, P, L, P, L, I, P, L, I, I, I, P]),
    "tw_linear_glu": (I, [I, P, L, P, L, I, P, P, L, I, I, I, I, P]),
    "tw_linear": (I, [I, I, P, L, P, L, I, P, P, L, P, L, P, L, I, I, I, I, P]),
    "tw_attn_decode_splits": (I, [I, I, I, I]),
    "tw_attn_decode_workspace_floats": (L, [I, I, I, I]),
    "tw_attn_decode": (I, [I, P, L, P, P, P, I, P, P, I, I, P, L, P, L, I, I, I, I, I, F, F, I, I, P]),
    "tw_attn_prefill_split": (I, [I, I, I, I, I, I, ctypes.POINTER(c_int), ctypes.POINTER(c_int)]),
    "tw_attn_prefill_workspace_floats": (L, [I, I, I, I]),
    "tw_attn_prefill": (I, [I, P, L, P, P, P, I, P, P, I, I, I, P, L, P, L, I, I, I, I, I, I, I, I, I, F, F, I, P]),
    "tw_sampling_uniform": (F, [c_uint64, c_uint64]),
    "tw_sample_workspace_bytes": (L, [I]),
    "tw_sample_rows": (I, [P, L, I, I, P, P, P, P, P, L, P]),
    "tw_sample_rows_static": (I, [P, L, I, I, P, P, P, P, P]),
}


class KernelError(RuntimeError):
    pass


def library():
    """The loaded kernel library; built on first use if it does not exist yet."""
    global _lib
    if _lib is None:
        path = _build.ensure_built()
        lib = ctypes.CDLL(str(path))
        for name, (restype, argtypes) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        if lib.tw_abi_version() != 1:
            raise KernelError(f"{path} has an unexpected ABI version")
        _lib = lib
    return _lib


def loaded_library_path():
    return None if _lib is None else _lib._name


def check(code, what):
    if code != 0:
        text = library().tw_error_string(int(code))
        raise KernelError(f"{what} failed: {text.decode() if text else code} (code {code})")
