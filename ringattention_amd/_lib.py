"""ctypes binding of the C ABI in include/ringattn.h.

This is the stub a maintainer of the reference harness would write to call the
engine from Python; it mirrors the header one to one and adds nothing.
The library must have been built (ringattention_amd._build.build_library or
__graft_entry__.build); there is no fallback implementation.
"""
import ctypes
import os

from ._build import LIB_PATH

_lib = None

c_int_p = ctypes.POINTER(ctypes.c_int)
c_float_p = ctypes.POINTER(ctypes.c_float)


class RingattnParams(ctypes.Structure):
    """struct ringattn_params (replaces Ring_fwd_params, csrc/ring.h:5-19)."""
    _fields_ = [
        ("npes", ctypes.c_int),
        ("h_seqlen", c_int_p),
        ("dim", ctypes.c_int),
        ("softmax_scale", ctypes.c_float),
        ("batch", ctypes.c_int),
        ("heads", ctypes.c_int),
        ("dtype", ctypes.c_int),
        ("causal", ctypes.c_int),
        ("flags", ctypes.c_int),
        ("kv_heads", ctypes.c_int),
        ("layout", ctypes.c_int),
    ]


class RingattnWorkItem(ctypes.Structure):
    """struct ringattn_work_item."""
    _fields_ = [(n, ctypes.c_int) for n in ("q_start", "q_len", "kv_start", "kv_len", "diag_off", "slot")]


SYMBOLS = {
    "ringattn_workspace_bytes": (ctypes.c_size_t, [ctypes.POINTER(RingattnParams)]),
    "ringattn_plan_create": (ctypes.c_int, [ctypes.POINTER(RingattnParams), ctypes.c_void_p, ctypes.c_size_t,
                                            ctypes.POINTER(ctypes.c_void_p)]),
    "ringattn_plan_destroy": (ctypes.c_int, [ctypes.c_void_p]),
    "ringattn_fwd": (ctypes.c_int, [ctypes.c_void_p] * 7),
    "ringattn_block_fwd": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int] + [ctypes.c_void_p] * 6),
    "ringattn_merge": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_int,
                                      ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]),
    "ringattn_merge_ring": (ctypes.c_int, [ctypes.c_void_p] * 6),
    "ringattn_rank_step_fwd": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int, ctypes.c_int] + [ctypes.c_void_p] * 6),
    "ringattn_rank_merge": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int] + [ctypes.c_void_p] * 5),
    "ringattn_plan_work_items": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int, ctypes.POINTER(RingattnWorkItem),
                                                ctypes.c_int, c_int_p]),
    "ringattn_plan_launch_times": (ctypes.c_int, [ctypes.c_void_p, c_float_p, ctypes.c_int, c_int_p]),
    "ringattn_plan_forward_kernel": (ctypes.c_char_p, [ctypes.c_void_p]),
    "ringattn_plan_merge_regions": (ctypes.c_int, [ctypes.c_void_p, c_int_p, c_int_p,
                                                   ctypes.POINTER(ctypes.c_uint64), ctypes.c_int, c_int_p]),
    "ringattn_ring_attention": (ctypes.c_int, [ctypes.c_void_p] * 5 + [ctypes.c_int, ctypes.c_int, c_int_p,
                                                                       ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                                       ctypes.c_int, ctypes.c_float]),
    "ringattn_ring_attention_noalloc": (ctypes.c_int, [ctypes.c_void_p] * 5 + [ctypes.c_int, ctypes.c_int, c_int_p,
                                                                               ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                                               ctypes.c_int, ctypes.c_float, ctypes.c_void_p]),
    "ringattn_noalloc_scratch_bytes": (ctypes.c_size_t, []),
    "ringattn_fill_normal": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_uint64,
                                            ctypes.c_int64, ctypes.c_double]),
    "ringattn_fill_reference_pattern": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "ringattn_strerror": (ctypes.c_char_p, [ctypes.c_int]),
    "ringattn_last_hip_error": (ctypes.c_int, []),
}


def load():
    """Load libringattn.so; raise if it has not been built (no fallback path exists)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: the HIP extension has not been built. "
            "Run `python -c 'import __graft_entry__ as g; g.build()'` at the repository root.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SYMBOLS.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


class RingattnError(RuntimeError):
    def __init__(self, code, where):
        self.code = code
        lib = load()
        msg = lib.ringattn_strerror(code).decode()
        hip = lib.ringattn_last_hip_error()
        super().__init__(f"{where}: ringattn error {code} ({msg})" + (f", hipError {hip}" if code == 10 else ""))


def check(code, where):
    if code != 0:
        raise RingattnError(code, where)
