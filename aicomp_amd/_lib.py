"""ctypes binding of libaicomp_kv.so (the C ABI declared in include/aicomp_kv.h).

There is no CPU fallback: if the HIP library is missing, loading raises.
"""
from __future__ import annotations

import ctypes as C
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libaicomp_kv.so")

# every symbol include/aicomp_kv.h declares
SYMBOLS = (
    "aicomp_kv_version",
    "aicomp_kv_last_error",
    "aicomp_kv_set_small_decode_tokens",
    "aicomp_kv_append",
    "aicomp_paged_decode_attn",
    "aicomp_paged_decode_attn_append",
    "aicomp_paged_decode_attn_append_static",
    "aicomp_paged_decode_workspace_bytes",
    "aicomp_paged_decode_partition_size",
    "aicomp_paged_prefill_attn",
    "aicomp_paged_prefill_attn_items",
    "aicomp_paged_prefill_tile_positions",
    "aicomp_rope_kv_append",
    "aicomp_sample_tokens",
)

F32, BF16, FP8_E4M3, F16 = 0, 1, 2, 3
MIN_VERSION = 200            # 0.2.0: the entry points of SYMBOLS above

_lock = threading.RLock()       # torch_ops() loads the HIP library while holding it
_lib = None


class LibraryMissing(RuntimeError):
    pass


def _declare(lib: C.CDLL) -> None:
    vp, i64, i32, f32, sz = C.c_void_p, C.c_int64, C.c_int, C.c_float, C.c_size_t
    lib.aicomp_kv_version.restype = i32
    lib.aicomp_kv_version.argtypes = []
    lib.aicomp_kv_last_error.restype = C.c_char_p
    lib.aicomp_kv_last_error.argtypes = []
    lib.aicomp_kv_set_small_decode_tokens.restype = C.c_longlong
    lib.aicomp_kv_set_small_decode_tokens.argtypes = [C.c_longlong]
    lib.aicomp_kv_append.restype = i32
    lib.aicomp_kv_append.argtypes = [vp, vp, i64, i64, vp, vp, vp, i64, i32, i32, i32, i64,
                                     i32, i32, vp, vp, vp]
    lib.aicomp_paged_decode_attn.restype = i32
    lib.aicomp_paged_decode_attn.argtypes = [vp, vp, vp, vp, vp, i64, vp, i32, i32, i32, i32,
                                             i32, i32, i64, f32, i32, i32, vp, vp, i32, vp, sz, vp]
    lib.aicomp_paged_decode_attn_append.restype = i32
    lib.aicomp_paged_decode_attn_append.argtypes = [vp, vp, vp, vp, i64, i64, vp, vp, vp, i64, vp, i32, i32,
                                                    i32, i32, i32, i32, i64, f32, i32, i32, vp, vp, i32,
                                                    vp, sz, vp]
    lib.aicomp_paged_decode_attn_append_static.restype = i32
    lib.aicomp_paged_decode_attn_append_static.argtypes = [vp, vp, vp, vp, i64, i64, vp, vp, vp, i64, vp, i32,
                                                           i32, i32, i32, i32, i32, i64, f32, i32, i32, vp,
                                                           vp, i32, vp]
    lib.aicomp_paged_decode_workspace_bytes.restype = sz
    lib.aicomp_paged_decode_workspace_bytes.argtypes = [i32] * 9
    lib.aicomp_paged_decode_partition_size.restype = i32
    lib.aicomp_paged_decode_partition_size.argtypes = [i32] * 8
    lib.aicomp_paged_prefill_attn.restype = i32
    lib.aicomp_paged_prefill_attn.argtypes = [vp, vp, vp, vp, vp, i64, vp, vp, i32, i64, i32,
                                              i32, i32, i32, i32, i32, i64, f32, i32, i32,
                                              vp, vp, vp]
    lib.aicomp_paged_prefill_attn_items.restype = i32
    lib.aicomp_paged_prefill_attn_items.argtypes = [vp, vp, vp, vp, vp, i64, vp, vp, i32, i64, i32,
                                                    i32, i32, i32, i32, i32, i64, f32, i32, i32,
                                                    vp, vp, vp, i32, vp]
    lib.aicomp_paged_prefill_tile_positions.restype = i32
    lib.aicomp_paged_prefill_tile_positions.argtypes = [i32] * 7
    lib.aicomp_rope_kv_append.restype = i32
    lib.aicomp_rope_kv_append.argtypes = [vp, vp, i64, i64, i64, i64, vp, vp, i64, i64, vp, vp, i64, i64, vp,
                                          vp, vp, vp, i64, i32, i32, i32, i32, i64, i32, i32, vp, vp, vp]
    lib.aicomp_sample_tokens.restype = i32
    lib.aicomp_sample_tokens.argtypes = [vp, vp, i64, vp, vp, i32, i32, f32, i32, f32, i32, i32, vp]


def load() -> C.CDLL:
    """Load the HIP library built by ``python -m aicomp_amd.build``."""
    global _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(LIB_PATH):
                raise LibraryMissing(
                    f"{LIB_PATH} is missing: build it with `python -m aicomp_amd.build` "
                    "(hipcc, gfx950). There is no CPU fallback for this path.")
            lib = C.CDLL(LIB_PATH)
            for s in SYMBOLS:
                if not hasattr(lib, s):
                    raise LibraryMissing(f"{LIB_PATH} does not export {s}")
            _declare(lib)
            if lib.aicomp_kv_version() < MIN_VERSION:
                raise LibraryMissing(f"{LIB_PATH} is version {lib.aicomp_kv_version()}, this package needs "
                                     f">= {MIN_VERSION}: rebuild it with `python -m aicomp_amd.build`")
            _lib = lib
        return _lib


TORCH_LIB_PATH = os.path.join(_HERE, "libaicomp_kv_torch.so")
_torch_ns = None


def torch_ops():
    """The ``torch.ops.mi355_kv`` namespace (``kv_append``, ``paged_decode_attn``,
    ``paged_decode_attn_append``, ``paged_prefill_attn``, ``decode_step``): the C ABI registered as
    PyTorch operators by csrc/torch_ops.cpp, built by ``python -m aicomp_amd.build``.  Loads the
    registration library on first use; raises ``LibraryMissing`` if it was not built."""
    global _torch_ns
    if _torch_ns is None:
        with _lock:
            if _torch_ns is None:
                if not os.path.exists(TORCH_LIB_PATH):
                    raise LibraryMissing(f"{TORCH_LIB_PATH} is missing: build it with `python -m aicomp_amd.build`")
                import torch
                load()                              # the HIP library it links against, checked first
                torch.ops.load_library(TORCH_LIB_PATH)
                _torch_ns = torch.ops.mi355_kv
    return _torch_ns


def check(rc: int, lib: C.CDLL) -> None:
    if rc != 0:
        msg = lib.aicomp_kv_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"aicomp_kv error {rc}: {msg}")
