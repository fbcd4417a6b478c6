"""Loading the HIP kernel library and declaring its entry points.

There is no fallback: when the library cannot be loaded, every op raises.
"""
from __future__ import annotations

import ctypes
import struct
import threading
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p
from typing import Optional

_lock = threading.Lock()
_lib: Optional[ctypes.CDLL] = None
_lib_path: Optional[str] = None

P, I, L, F = c_void_p, c_int, c_int64, c_float

_PROTOTYPES = {
    "zi_abi_version": [],
    "zi_embedding": [P, I, P, I, P, I, I, I, P],
    "zi_gather_rows": [P, P, I, P, I, I, I, P],
    "zi_add": [P, I, P, I, P, I, L, P],
    "zi_swiglu": [P, I, P, P, I, I, I, L, L, I, I, L, P],
    "zi_swiglu_t": [P, P, I, I, I, L, P],
    "zi_rmsnorm": [P, I, P, I, P, I, I, I, L, L, F, I, P],
    "zi_add_rmsnorm": [P, I, P, P, I, I, L, P, I, I, I, F, I, P],
    "zi_rope_kv_store": [P, P, P, I, I, L, L, L, P, P, P, P, L, I, I, I, I, I, I, P],
    "zi_rope": [P, P, I, I, L, L, P, P, I, I, I, P],
    "zi_attention_generic": [P, P, I, I, L, L, P, P, P, P, P, P, I, I, I, I, I, I, I, F, P],
    "zi_attention_decode": [P, P, I, I, L, L, P, P, P, P, P, P, I, I, I, I, I, I, I, F, I, P, L, P],
    "zi_attention_decode_supported": [I, I, I, I, I],
    "zi_attention_decode_fused": [P, I, I, L, P, I, L, L, P, I, P, I, P, L, I, P, P, P, P, P, P, I, I, I, I, I, I, I, F,
                                  I, P, L, P],
    "zi_attention_decode_fused_supported": [I, I, I, I, I, I, I, L, L],
    "zi_attention_decode_project": [P, P, L, I, P, I, I, P, I, L, I, I, I, P],
    "zi_attention_decode_project_supported": [I, I, I, I, L],
    "zi_attention_decode_project_heads": [I],
    "zi_rope_table": [P, P, P, I, I, P],
    "zi_decode_layer": [P, I, I, I, P, P, I, F, F, I, P, L, P, I, P, L, P, L, P, L, I, P, I, P, L, P, P, P, P, I, I, I, I,
                        I, I, I, F, I, P, L, P, P, I, P],
    "zi_decode_layer_supported": [I, I, I, I, I, I, I, I, I, I, I],
    "zi_decode_layer_sync_words": [],
    "zi_decode_layer_stamps": [],
    "zi_attention_decode_chunks": [I],
    "zi_attention_prefill": [P, P, I, I, L, L, P, P, P, P, P, P, P, P, I, I, I, I, I, I, I, F, I, I, P, L, I, I, I, P],
    "zi_attention_prefill_chunk_keys_for": [I, I],
    "zi_attention_prefill_cuts": [I, I, I, P],
    "zi_attention_prefill_tile_min": [],
    "zi_compute_units": [],
    "zi_gemm_skinny_pays": [I, I, I],
    "zi_attention_prefill_chunks": [I],
    "zi_attention_prefill_variant": [I],
    "zi_attention_prefill_supported": [I, I, I, I, I],
    "zi_attention_prefill_tile": [I, I],
    "zi_attention_prefill_chunk_keys": [],
    "zi_gemm_generic": [P, I, P, I, P, I, P, I, I, I, I, L, L, L, P],
    "zi_gemm_skinny": [P, I, I, P, P, P, I, I, I, L, L, L, P, L, P],
    "zi_gemm_skinny_splits": [I, I, I],
    "zi_gemm_lt": [P, I, P, P, P, I, L, L, L, L, L, L, P, L, P],
    "zi_gemm_lt_tune": [P, I, P, P, P, I, L, L, L, L, L, L, P, L, I, I, P, P, P, P],
    "zi_gemm_lt_choose": [I, I, I, L, L, L, L, L, L, L, I],
    "zi_reduce_splits": [P, I, P, P, I, I, L, I, P],
    "zi_rope_kv_store_split": [P, I, L, P, I, L, L, P, I, I, P, P, P, P, L, I, I, I, I, I, I, P],
    "zi_gemm_skinny_supported": [I, I, I, L, L],
    "zi_argmax": [P, P, P, I, I, I, L, P, L, P],
    "zi_sample": [P, P, L, P, I, I, P, P, P, P, P, P, P, I, P],
    "zi_tape_record": [P, c_char_p, P, I],
    "zi_tape_record_many": [P, c_char_p, P, P, I],
    "zi_tape_run": [P, P],
    "zi_tape_length": [P],
}


class KernelLibraryError(RuntimeError):
    pass


def library_path() -> Optional[str]:
    return _lib_path


def load() -> ctypes.CDLL:
    """The loaded library; builds it first when nothing built matches the sources."""
    global _lib, _lib_path
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        import torch  # noqa: F401  (loads the HIP runtime the library links against)
        from ..csrc.build import ensure_library
        try:
            path = ensure_library()
            lib = ctypes.CDLL(path)
        except (OSError, RuntimeError) as e:
            raise KernelLibraryError(f"cannot load the HIP kernel library: {e}") from e
        lib.zi_last_error.restype = c_char_p
        lib.zi_last_error.argtypes = []
        for name, args in _PROTOTYPES.items():
            try:
                fn = getattr(lib, name)
            except AttributeError as e:
                raise KernelLibraryError(f"{path} lacks entry point {name}; rebuild it") from e
            fn.argtypes = args
            fn.restype = c_int
        lib.zi_gemm_skinny_workspace.argtypes = [I, I, I]
        lib.zi_gemm_skinny_workspace.restype = c_int64
        lib.zi_attention_decode_workspace.argtypes = [I, I, I]
        lib.zi_attention_decode_workspace.restype = c_int64
        lib.zi_attention_prefill_workspace.argtypes = [I, I, I, I]
        lib.zi_attention_prefill_workspace.restype = c_int64
        lib.zi_decode_layer_workspace.argtypes = [I, I, I, I, I, I, I, I]
        lib.zi_decode_layer_workspace.restype = c_int64
        lib.zi_argmax_workspace.argtypes = [I, I]
        lib.zi_argmax_workspace.restype = c_int64
        lib.zi_tape_new.argtypes = []
        lib.zi_tape_new.restype = c_void_p
        lib.zi_tape_free.argtypes = [P]
        lib.zi_tape_free.restype = None
        _lib, _lib_path = lib, path
        return lib


# The calls made while a tape records (``ops.tape.Recording``): a list of (name, arguments), or None.
_recorded: Optional[list] = None


def call(name: str, *args) -> None:
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise KernelLibraryError(lib.zi_last_error().decode("utf-8", "replace"))
    if _recorded is not None:
        _recorded.append((name, args))


def argument_words(name: str, args) -> list:
    """The arguments of a call as the 64-bit words a tape holds: integers and pointers by value, floats as
    the bits of a double."""
    kinds = _PROTOTYPES[name]
    if len(kinds) != len(args):
        raise KernelLibraryError(f"{name} takes {len(kinds)} arguments, {len(args)} were given")
    words = []
    for kind, a in zip(kinds, args):
        if kind is F:
            words.append(struct.unpack("<q", struct.pack("<d", float(a.value if isinstance(a, c_float) else a)))[0])
        elif kind is P:
            v = a.value if isinstance(a, c_void_p) else a
            if v is not None and not isinstance(v, int):
                raise KernelLibraryError(f"{name}: an argument of a kind a tape cannot hold ({type(a).__name__})")
            words.append(int(v or 0))
        else:
            words.append(int(a.value if hasattr(a, "value") else a))
    return words
