"""ctypes binding of libkascade_hip.so (the C ABI declared in include/kascade_hip.h; the
benchmark's two measurement helpers in include/kascade_hip_diag.h).

Loading fails loudly: there is no fallback implementation.  ``load()`` returns
the library with argument types set; ``check(rc)`` turns a -1 return code into
a ``KascadeError`` carrying ``kascade_get_last_error()``.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libkascade_hip.so"


class KascadeError(RuntimeError):
    pass


class Strides(C.Structure):
    """kascade_strides: element strides (b, l, h) of a [B,L,H,D] view."""
    _fields_ = [("b", C.c_int64), ("l", C.c_int64), ("h", C.c_int64)]


_P = C.c_void_p
_I = C.c_int
_F = C.c_float
_L = C.c_int64
_SP = C.POINTER(Strides)   # optional kascade_strides*

# name -> (restype, argtypes); must list every symbol of include/kascade_hip.h and include/kascade_hip_diag.h
SIGNATURES = {
    "kascade_init": (_I, []),
    "kascade_get_last_error": (C.c_char_p, []),
    "kascade_abi_version": (_I, []),
    "kascade_device_cu_count": (_I, []),
    "kascade_decode_reuse_call": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P, _P]),
    "kascade_decode_reuse_paged_call": (_I, [_P, _P, _P, _P, _P, _P, _F, _P, _P, _P, _I, _I, _I, _I,
                                             _P, _I, _I, _SP, _P, _P, _P, _P, _P]),
    "kascade_decode_reuse_rows_call": (_I, [_P, _P, _P, _P, _P, _P, _F, _P, _P, _P, _I, _I, _I, _P, _I, _I, _I,
                                            _P, _P, _P, _P, _P]),
    "kascade_decode_reuse_paged_noalloc_call": (_I, [_P, _P, _P, _P, _P, _P, _F, _P, _I, _I, _I, _I,
                                                     _P, _I, _I, _SP, _P, _P, _P]),
    "kascade_decode_dense_paged_call": (_I, [_P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _P, _I, _I, _SP,
                                             _P, _P, _P, _P]),
    "kascade_decode_recompute_paged_call": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I,
                                                 _I, _I, _P, _I, _I, _SP, _P, _P, _P, _P]),
    "kascade_topk_workspace_bytes": (_L, [_I, _L]),
    "kascade_topk_call": (_I, [_P, _P, _I, _L, _I, _P, _P, _I, _I, _I, _P, _P]),
    "kascade_topk_sorted_workspace_bytes": (_L, [_I, _L, _I]),
    "kascade_topk_sorted_call": (_I, [_P, _P, _I, _L, _I, _P, _I, _I, _P, _P]),
    "kascade_topk_rows_call": (_I, [_P, _P, _I, _L, _I, _P, _P, _I, _I, _I, _P, _P, _P, _I, _I, _I, _P]),
    "kascade_prefill_dense_call": (_I, [_P, _P, _P, _P, _P, _I, _I, Strides, Strides, _I, _P]),
    "kascade_prefill_aggregate_call": (_I, [_P, _P, _P, _P, _I, _I, Strides, Strides, _I, _P]),
    "kascade_prefill_aggregate_range_call": (_I, [_P, _P, _P, _P, _I, _I, _I, Strides, Strides, _I, _P]),
    "kascade_prefill_reuse_call": (_I, [_P, _P, _P, _P, _P, _F, _P, _I, _I, _I, _I, Strides, Strides,
                                        _P, _P]),
    "kascade_paged_kv_append_call": (_I, [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, Strides, _P, _P]),
    "kascade_rope_append_paged_call": (_I, [_P, _SP, _P, _P, _SP, _P, _I, _P, _P, _F, _P, _I, _P, _P, _P,
                                            _P, _I, _I, _I, _I, _P]),
    "kascade_decode_budgets_call": (_I, [_P, _I, _F, _I, _P, _P, _P]),
    "kascade_prefill_chunk_dense_call": (_I, [_P, _P, _P, _P, _P, _I, _I, _I, Strides, _P, _I, _I, _I,
                                              _I, _P, _P, _P]),
    "kascade_prefill_chunk_aggregate_call": (_I, [_P, _P, _P, _P, _I, _I, _I, Strides, _P, _I, _I, _I,
                                                  _I, _P, _P, _P]),
    "kascade_prefill_chunk_reuse_call": (_I, [_P, _P, _P, _P, _P, _F, _P, _I, _I, _I, _I, _I, Strides,
                                              _P, _I, _I, _I, _P, _P, _P, _P]),
    "kascade_translate_indices_call": (_I, [_P, _P, _P, _I, C.c_int64, _I, _I, _I, _P]),
    "kascade_ref_decode_reuse_call": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _P]),
    "kascade_ref_decode_reuse_kvcache_call": (_I, [_P, _P, _P, _P, _P, _P, _F, _P, _P, _P, _I, _I, _I, _P]),
    "kascade_ref_prefill_aggregate_call": (_I, [_P, _P, _P, _P, _I, _I, _P]),
    "kascade_ref_prefill_reuse_rolling_call": (_I, [_P, _P, _P, _P, _P, _F, _P, _I, _I, _I, _P]),
    "kascade_ref_prefill_reuse_call": (_I, [_P, _P, _P, _P, _P, _F, _P, _I, _I, _I, _P]),
    "kascade_diag_stream_read_call": (_I, [_P, _L, _P, _P]),
    "kascade_diag_gather_rows_call": (_I, [_P, _P, _P, _L, _L, _P, _P]),
}

class Shape(C.Structure):
    """kascade_shape: KV heads, head dimension, element type (0 fp16, 1 bf16), query heads per KV
    head (0 = 4)."""
    _fields_ = [("kv_heads", C.c_int32), ("head_dim", C.c_int32), ("dtype", C.c_int32), ("group_size", C.c_int32)]


# every *_shaped_call takes a kascade_shape* followed by the arguments of the plain entry
for _name in ("decode_reuse_paged", "decode_reuse_rows", "decode_dense_paged", "decode_recompute_paged",
              "prefill_dense", "prefill_aggregate", "prefill_aggregate_range", "prefill_reuse", "paged_kv_append",
              "rope_append_paged", "decode_budgets", "prefill_chunk_dense", "prefill_chunk_aggregate",
              "prefill_chunk_reuse"):
    _res, _args = SIGNATURES[f"kascade_{_name}_call"]
    SIGNATURES[f"kascade_{_name}_shaped_call"] = (_res, [C.POINTER(Shape)] + list(_args))

_lib = None
_initialised = False


def load() -> C.CDLL:
    """dlopen the in-tree library and bind every declared symbol."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise KascadeError(
            f"{LIB_PATH} is missing: build it with `python -m kascade_amd.build` "
            "(there is no fallback path)")
    lib = C.CDLL(str(LIB_PATH))
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)   # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def last_error() -> str:
    return load().kascade_get_last_error().decode("utf-8", "replace")


def check(rc: int) -> None:
    if rc != 0:
        raise KascadeError(last_error())


def init() -> C.CDLL:
    """Load the library and run kascade_init() once on the current device."""
    global _initialised
    lib = load()
    if not _initialised:
        check(lib.kascade_init())
        _initialised = True
    return lib
