"""ctypes binding of the host runtime library (cache manager, scheduler)."""
from __future__ import annotations

from ctypes import c_int, c_longlong, c_ulonglong, c_void_p, c_char_p, POINTER

from . import build

_lib = None
PI = POINTER(c_int)
PLL = POINTER(c_longlong)
PULL = POINTER(c_ulonglong)


def lib():
    global _lib
    if _lib is None:
        l = build.load("host")
        l.spite_host_last_error.restype = c_char_p
        P, I, LL, ULL = c_void_p, c_int, c_longlong, c_ulonglong
        sigs = {
            "spc_create": (P, [I, I, I, PI, PI, PI]),
            "spc_destroy": (None, [P]),
            "spc_admit": (I, [P]),
            "spc_take_fresh": (I, [P, PI, I]),
            "spc_fill_step": (I, [P, I, c_void_p, c_void_p, c_void_p, I, I, c_void_p, c_void_p]),
            "spc_live": (I, [P, I]),
            "spc_cached": (LL, [P, I]),
            "spc_can_reserve": (I, [P, I, LL]),
            "spc_can_reserve_new": (I, [P, LL]),
            "spc_reserve": (I, [P, I, LL]),
            "spc_reserve_all": (I, [P, I, PI, PLL]),
            "spc_commit": (I, [P, I, LL]),
            "spc_release": (I, [P, I]),
            "spc_free_pages": (I, [P, I]),
            "spc_total_pages": (I, [P, I]),
            "spc_free_slots": (I, [P]),
            "spc_peak_pages": (LL, [P, LL, LL, I]),
            "spc_table": (I, [P, I, I, PI, I]),
            "spc_table_len": (I, [P, I, I]),
            "spc_slot_mapping": (I, [P, I, I, LL, LL, c_void_p]),
            "spc_check": (I, [P]),
            "sps_create": (P, [P, I, LL, PI, I]),
            "sps_destroy": (None, [P]),
            "sps_submit": (ULL, [P, PI, I, I, PI, I]),
            "sps_schedule": (I, [P, I, I, PULL, PI, PLL, PI, PI, PI, PI]),
            "sps_update": (I, [P, PI, I, I, PULL, PI, PI, PI]),
            "sps_cancel": (I, [P, ULL]),
            "sps_n_waiting": (I, [P]),
            "sps_n_running": (I, [P]),
            "sps_n_preemptions": (ULL, [P]),
            "sps_request_info": (I, [P, ULL, PLL]),
        }
        for name, (res, args) in sigs.items():
            fn = getattr(l, name)
            fn.restype = res
            fn.argtypes = args
        _lib = l
    return _lib


def last_error() -> str:
    return lib().spite_host_last_error().decode()


def int_array(values):
    values = list(values)
    return (c_int * max(len(values), 1))(*values)
