"""ctypes signatures of the host library (csrc/host.cpp): page pools, the book of
live requests and the layout of a step's batch."""
from __future__ import annotations

import ctypes
from ctypes import POINTER, c_char_p, c_int, c_int32, c_int64, c_long, c_void_p

from ..kernels import build

_lib = None

IP = POINTER(c_int)


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        l = build.load("host")
        sig = {
            "li_pool_create": ([c_int, IP], c_void_p), "li_pool_destroy": ([c_void_p], None),
            "li_pool_error": ([c_void_p], c_char_p), "li_pool_capacity": ([c_void_p], c_int),
            "li_pool_free": ([c_void_p], c_int), "li_pool_total_allocations": ([c_void_p], c_long),
            "li_pool_peak_used": ([c_void_p], c_int),
            "li_pool_alloc": ([c_void_p], c_int), "li_pool_release": ([c_void_p, c_int], c_int),
            "li_pool_is_held": ([c_void_p, c_int], c_int),
            "li_book_create": ([c_int, c_int, c_int, IP, IP, IP], c_void_p),
            "li_book_destroy": ([c_void_p], None), "li_book_error": ([c_void_p], c_char_p),
            "li_book_pool": ([c_void_p, c_int], c_void_p), "li_book_has": ([c_void_p, c_int64], c_int),
            "li_book_num_live": ([c_void_p], c_int), "li_book_free_slots": ([c_void_p], c_int),
            "li_book_free_pages": ([c_void_p, IP], None), "li_book_admit": ([c_void_p, c_int64], c_int),
            "li_book_slot": ([c_void_p, c_int64], c_int), "li_book_cached": ([c_void_p, c_int64], c_int),
            "li_book_table_len": ([c_void_p, c_int64, c_int], c_int),
            "li_book_table": ([c_void_p, c_int64, c_int, IP, c_int], c_int),
            "li_book_pages_needed": ([c_void_p, c_int64, c_int, c_int, IP], c_int),
            "li_book_reserve": ([c_void_p, c_int64, c_int], c_int),
            "li_book_commit": ([c_void_p, c_int64, c_int], c_int),
            "li_book_rewind": ([c_void_p, c_int64, c_int], c_int),
            "li_book_pages_needed_many": ([c_void_p, c_int, c_void_p, c_void_p, c_void_p], c_int),
            "li_book_reserve_many": ([c_void_p, c_int, c_void_p, c_void_p], c_int),
            "li_book_max_table_len": ([c_void_p, c_int, c_void_p, c_void_p], c_int),
            "li_book_cached_many": ([c_void_p, c_int, c_void_p, c_void_p], c_int),
            "li_book_commit_many": ([c_void_p, c_int, c_void_p, c_void_p], c_int),
            "li_book_release": ([c_void_p, c_int64], c_int), "li_book_check": ([c_void_p], c_int),
            "li_book_build_batch": ([c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                     c_void_p, c_int, c_int, c_void_p, c_long, c_void_p, c_void_p], c_long),
        }
        for name, (args, res) in sig.items():
            f = getattr(l, name)
            f.argtypes, f.restype = args, res
        _lib = l
    return _lib


ERR_FULL, ERR_UNKNOWN, ERR_POOL, ERR_ARG, ERR_LIVE, ERR_INVARIANT = -1, -2, -3, -4, -5, -6


def int_array(values):
    return (c_int * len(values))(*values) if len(values) else None
