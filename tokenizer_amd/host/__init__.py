"""The host core: page allocator, cache manager bookkeeping, batch packing and the host sampler, written
in C++ (`csrc/host/`) and bound here through ctypes.  It has no GPU code; it is compiled with the C++
compiler at first use if no built library is found (a few seconds).
"""
from __future__ import annotations

import ctypes
import threading

from ..kernels import build as _build

_i32p = ctypes.POINTER(ctypes.c_int32)
_i64p = ctypes.POINTER(ctypes.c_int64)
_f32p = ctypes.POINTER(ctypes.c_float)
_vp, _int, _i64, _u64, _f32 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_uint64, ctypes.c_float

_SIGNATURES = {
    "ta_host_message": (ctypes.c_char_p, []),
    "ta_alloc_new": (_vp, [_int, _int]),
    "ta_alloc_delete": (None, [_vp]),
    "ta_alloc_get": (_int, [_vp, _int, _int]),
    "ta_alloc_rewind_peaks": (None, [_vp, _int, _int]),
    "ta_alloc_alloc": (_int, [_vp]),
    "ta_alloc_alloc_n": (_int, [_vp, _int, _i32p]),
    "ta_alloc_free": (_int, [_vp, _int, _i32p]),
    "ta_alloc_incref": (_int, [_vp, _int]),
    "ta_prefix_page_hash": (_u64, [_u64, _i32p, _int]),
    "ta_alloc_publish_full_page": (_int, [_vp, _u64, _i32p, _int, _int]),
    "ta_alloc_find_full_page": (_int, [_vp, _u64, _int, _i32p, _int]),
    "ta_alloc_publish_at": (_int, [_vp, _u64, _u64, _int, _i32p, _int, _int]),
    "ta_alloc_find_at": (_int, [_vp, _u64, _u64, _int, _i32p, _int]),
    "ta_alloc_take_shared_prefix": (_int, [_vp, _i32p, _int, _i32p]),
    "ta_alloc_publish_prompt_pages": (None, [_vp, _i32p, _int, _i32p, _int]),
    "ta_alloc_reclaim_cached": (None, [_vp]),
    "ta_alloc_check": (_int, [_vp]),
    "ta_cache_new": (_vp, [_int, _i32p, _int, _int, _int, _int, _int]),
    "ta_cache_delete": (None, [_vp]),
    "ta_cache_allocator": (_vp, [_vp, _int]),
    "ta_cache_prefix_enabled": (_int, [_vp]),
    "ta_cache_n_requests": (_int, [_vp]),
    "ta_cache_free_slots": (_int, [_vp]),
    "ta_cache_add_request": (_int, [_vp, _i64]),
    "ta_cache_has_request": (_int, [_vp, _i64]),
    "ta_cache_seq_len": (_int, [_vp, _i64]),
    "ta_cache_slot": (_int, [_vp, _i64]),
    "ta_cache_table_len": (_int, [_vp, _i64, _int]),
    "ta_cache_table": (_int, [_vp, _i64, _int, _i32p]),
    "ta_cache_first_needed_position": (_int, [_vp, _int, _int]),
    "ta_cache_pages_missing": (_int, [_vp, _i64, _int, _i32p]),
    "ta_cache_can_reserve": (_int, [_vp, _i64, _int]),
    "ta_cache_reserve": (_int, [_vp, _i64, _int]),
    "ta_cache_advance": (_int, [_vp, _i64, _int]),
    "ta_cache_release": (_int, [_vp, _i64]),
    "ta_cache_detach": (_int, [_vp, _i64]),
    "ta_cache_attach_shared_prefix": (_int, [_vp, _i64, _i32p, _int]),
    "ta_cache_publish": (_int, [_vp, _i64, _i32p, _int]),
    "ta_cache_check": (_int, [_vp]),
    "ta_cache_pack_batch": (_i64, [_vp, _int, _i64p, _i32p, _i32p, _i32p, _i32p, _int, _i64p, _i32p, _i64, _i64p,
                                   _i32p, _i32p]),
    "ta_cache_request_ids": (_int, [_vp, _i64p]),
    "ta_sched_new": (_vp, [_vp, _int, _int, _int, _int, _int]),
    "ta_sched_delete": (None, [_vp]),
    "ta_sched_enqueue": (_int, [_vp, _i64, _i32p, _int]),
    "ta_sched_append_token": (_int, [_vp, _i64, ctypes.c_int32]),
    "ta_sched_get": (_i64, [_vp, _int, _i64]),
    "ta_sched_plan_step": (_int, [_vp, _int, _i64p, _i32p, _i64p, _i32p, _i64p, _i32p]),
    "ta_sched_list": (_int, [_vp, _int, _i64p]),
    "ta_sched_tokens": (_int, [_vp, _i64, _int, _int, _i32p]),
    "ta_sched_commit": (_int, [_vp, _i64, _int]),
    "ta_sched_finish": (_int, [_vp, _i64]),
    "ta_bpe_new": (_vp, []),
    "ta_bpe_delete": (None, [_vp]),
    "ta_bpe_add_token": (_int, [_vp, ctypes.c_int32, ctypes.c_char_p, _int, _int]),
    "ta_bpe_add_merge": (_int, [_vp, ctypes.c_char_p, _int, _int]),
    "ta_bpe_vocab_size": (_int, [_vp]),
    "ta_bpe_encode_piece": (_int, [_vp, ctypes.c_char_p, _int, _i32p, _int]),
    "ta_bpe_decode": (_i64, [_vp, _i32p, _int, ctypes.c_char_p, _i64, _i32p]),
    "ta_uniform_f32": (_f32, [_u64, _u64]),
    "ta_greedy_token": (_int, [_f32p, _i64]),
    "ta_sample_with_uniform": (_int, [_f32p, _i64, _f32, _f32, _f32]),
}

_lib = None
_lock = threading.Lock()


def lib() -> ctypes.CDLL:
    """The loaded host library; builds it first if there is none (or its sources are newer)."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                path = _build.find_host_library() or _build.build_host_library()
                loaded = ctypes.CDLL(path)
                for name, (restype, argtypes) in _SIGNATURES.items():
                    fn = getattr(loaded, name)
                    fn.restype, fn.argtypes = restype, argtypes
                _lib = loaded
    return _lib


def message() -> str:
    return lib().ta_host_message().decode()


def int_array(values):
    """A C array of int32 from a sequence of ints (numpy int32 arrays pass through without a copy).
    Returns (the array, which the caller keeps alive during the call; its pointer)."""
    import numpy as np
    array = np.ascontiguousarray(values, dtype=np.int32)
    return array, array.ctypes.data_as(_i32p)


def token_array(tokens):
    """Token ids as int32 bit patterns of their low 32 bits."""
    import numpy as np
    array = (np.asarray(tokens, dtype=np.int64) & 0xFFFFFFFF).astype(np.uint32).view(np.int32) if len(tokens) \
        else np.zeros(0, dtype=np.int32)
    array = np.ascontiguousarray(array)
    return array, array.ctypes.data_as(_i32p)
