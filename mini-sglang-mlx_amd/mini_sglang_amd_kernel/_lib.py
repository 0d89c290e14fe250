"""ctypes binding of ``libmsgl_paged_attention.so`` (the C ABI in ``include/msgl_paged_attention.h``,
``include/msgl_radix_cache.h`` and ``include/msgl_state_pool.h``).

The library is built in-tree by ``mini-sglang-mlx_amd/build.py``; nothing here compiles at
import time and nothing falls back to another implementation: a missing library is an
``ImportError``-class failure at first use.
"""
from __future__ import annotations

import ctypes
import os

_PKG_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_PATH = os.path.join(_PKG_ROOT, "lib", "libmsgl_paged_attention.so")

_i64 = ctypes.c_int64
_i32 = ctypes.c_int32
_f32 = ctypes.c_float
_vp = ctypes.c_void_p
_sz = ctypes.c_size_t

# name -> (restype, argtypes); one entry per MSGL_API declaration of the headers
SIGNATURES = {
    "msgl_version": (ctypes.c_int, []),
    "msgl_strerror": (ctypes.c_char_p, [ctypes.c_int]),
    "msgl_set_tuning": (ctypes.c_int, [_i32, _i64]),
    "msgl_get_tuning": (ctypes.c_int, [_i32, ctypes.POINTER(ctypes.c_int64)]),
    "msgl_store_kv_cache": (
        ctypes.c_int,
        [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i32, _vp]),
    "msgl_paged_decode_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64, _i64]),
    "msgl_paged_decode_attention": (
        ctypes.c_int,
        [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _i64, _i64, _i64, _i64, _i64, _i64,
         _i64, _i64, _f32, _i32, _i32, _vp]),
    "msgl_paged_decode_attention_noalloc": (
        ctypes.c_int,
        [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64,
         _i64, _i64, _f32, _i32, _i32, _vp]),
    "msgl_paged_prefill_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64, _i64, _i64, _i64]),
    "msgl_paged_prefill_attention": (
        ctypes.c_int,
        [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _i64, _i64, _i64, _i64, _i64, _i64,
         _i64, _i64, _i64, _f32, _i32, _i32, _i32, _i32, _vp]),
    "msgl_build_attention_metadata": (
        ctypes.c_int,
        [_vp, _i64, _i64, _i64, _vp, _vp, _vp, _i64, _vp, _vp, _i64, _vp, _vp, _vp, _i64, _vp,
         _i32, _vp]),
    "msgl_qk_norm_rope_store": (
        ctypes.c_int,
        [_vp, _vp, _vp, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64,
         _i64, _i64, _i64, _i64, _f32, _f32, _i32, _vp]),
    "msgl_gdn_state_inplace": (
        ctypes.c_int,
        [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64,
         _i64, _i64, _i64, _i64, _i32, _vp]),
    # include/msgl_state_pool.h (recurrent-state pool)
    "msgl_copy_state_slots": (ctypes.c_int, [_vp, _i64, _i64, _i64, _i64, _i64, _vp, _vp, _i64, _vp]),
    # include/msgl_radix_cache.h (host-side prefix cache)
    "msgl_fast_compare_key": (_sz, [_vp, _sz, _vp, _sz, _i32, _vp]),
    "msgl_radix_create": (_vp, []),
    "msgl_radix_destroy": (None, [_vp]),
    "msgl_radix_walk": (_i64, [_vp, _vp, _i64, _i64, _vp]),
    "msgl_radix_path_values": (_i64, [_vp, _i64, _vp, _i64]),
    "msgl_radix_insert": (_i64, [_vp, _vp, _vp, _i64, _i32, _i64, _vp]),
    "msgl_radix_lock": (_i32, [_vp, _i64, _i32]),
    "msgl_radix_evict": (_i64, [_vp, _i64, _i64, _vp]),
    "msgl_radix_evicted": (_i32, [_vp, _vp, _i64, _vp, _i64]),
    "msgl_radix_sizes": (_i32, [_vp, _vp, _vp]),
    "msgl_radix_node_info": (_i32, [_vp, _i64, _vp, _vp, _vp, _vp, _vp, _vp]),
    "msgl_radix_node_set": (_i32, [_vp, _i64, _i32, _i64]),
    "msgl_radix_node_child": (_i64, [_vp, _i64, _i32]),
    "msgl_radix_node_children": (_i64, [_vp, _i64, _vp, _vp, _i64]),
    "msgl_radix_node_key_value": (_i64, [_vp, _i64, _vp, _vp, _i64]),
    "msgl_radix_find_mamba_ancestor": (_i64, [_vp, _i64, _i64, _vp]),
    "msgl_radix_collect_mamba_slots": (_i64, [_vp, _vp, _i64]),
    "msgl_radix_coldest_snapshot": (_i64, [_vp, _i64]),
    "msgl_radix_node_count": (_i64, [_vp]),
}

MSGL_DTYPE_BF16 = 0
MSGL_DTYPE_F16 = 1
TUNE_SEGMENTS = 0
TUNE_MIN_SEGMENT = 1
TUNE_SMALLQ_MAXCOLS = 2
TUNE_PREFILL_VARIANT = 3
TUNE_SPLITKV_WAVES = 4
TUNE_GDN_ROWS = 5
TUNE_PREFILL_KEY_SPLITS = 6
TUNE_SPLITKV_BOUNDARY = 7
TUNE_PREFILL_GANGS = 8
TUNE_CLOCK_PROBE = 9

_lib = None


class KernelLibraryMissing(ImportError):
    pass


def load() -> ctypes.CDLL:
    """Load the shared library once; raise loudly if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise KernelLibraryMissing(
            f"{LIB_PATH} not found: build it with `python mini-sglang-mlx_amd/build.py` "
            "(or __graft_entry__.build()); there is no fallback implementation")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def strerror(code: int) -> str:
    return load().msgl_strerror(int(code)).decode()


def set_tuning(knob: int, value: int) -> None:
    rc = load().msgl_set_tuning(int(knob), int(value))
    if rc != 0:
        raise ValueError(f"msgl_set_tuning({knob}, {value}): {strerror(rc)}")


def get_tuning(knob: int) -> int:
    """What the calling thread last set for `knob` (knobs are per host thread)."""
    out = ctypes.c_int64(0)
    rc = load().msgl_get_tuning(int(knob), ctypes.byref(out))
    if rc != 0:
        raise ValueError(f"msgl_get_tuning({knob}): {strerror(rc)}")
    return out.value
