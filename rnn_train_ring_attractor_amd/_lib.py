"""ctypes binding of libringattr.so (the C ABI declared in include/ringattr.h).

The library is looked up next to this file (prebuilt, in-tree); if it is absent it is built once
with hipcc (same prebuilt-then-build order as the reference's cpp/ring_rnn_cuda.py:6-16).  There is
no CPU fallback: a missing or unloadable library raises.
"""
from __future__ import annotations

import ctypes
import os
import threading

import torch  # noqa: F401  (loads torch's libamdhip64 first so the library binds to the same HIP runtime)

from . import build as _build

_lock = threading.Lock()
_lib = None

c_void_p, c_int, c_float, c_size_t, c_char_p = (ctypes.c_void_p, ctypes.c_int, ctypes.c_float,
                                                ctypes.c_size_t, ctypes.c_char_p)

# name -> (restype, argtypes): one entry per prototype in include/ringattr.h
PROTOTYPES = {
    "ringattr_version": (c_int, []),
    "ringattr_last_error": (c_char_p, []),
    "ringattr_saved_bytes": (c_size_t, [c_int] * 4),
    "ringattr_fwd_workspace_bytes": (c_size_t, [c_int] * 4),
    "ringattr_bwd_workspace_bytes": (c_size_t, [c_int] * 5),
    "ringattr_fwd": (c_int, [c_void_p, c_void_p, c_float, c_float, c_void_p, c_void_p, c_void_p, c_float,
                             c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_size_t, c_void_p]),
    "ringattr_fwd_loss": (c_int, [c_void_p, c_void_p, c_float, c_float, c_void_p, c_void_p, c_void_p, c_float,
                                  c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_size_t,
                                  c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_size_t, c_void_p]),
    "ringattr_fwd_noalloc": (c_int, [c_void_p, c_void_p, c_float, c_float, c_void_p, c_void_p, c_void_p, c_float,
                                     c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p]),
    "ringattr_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_float, c_float, c_void_p, c_void_p, c_void_p,
                             c_void_p, c_void_p, c_float, c_int, c_int, c_int, c_int, c_int, c_int,
                             c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "ringattr_loss_workspace_bytes": (c_size_t, [c_int] * 3),
    "ringattr_loss_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_int, c_int, c_int,
                                  c_void_p, c_size_t, c_void_p]),
    "ringattr_loss_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_int, c_int, c_int,
                                  c_void_p, c_size_t, c_void_p]),
    "ringattr_bwd_loss_available": (c_int, [c_int] * 4),
    "ringattr_bwd_loss": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_float, c_void_p, c_void_p, c_void_p,
                                  c_void_p, c_void_p, c_float, c_int, c_int, c_int, c_int, c_int, c_int,
                                  c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "ringattr_gain_workspace_bytes": (c_size_t, [c_int] * 4),
    "ringattr_gain_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    "ringattr_gain_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                  c_void_p, c_size_t, c_void_p]),
    "ringattr_generator_initial_zeros": (c_int, [c_int, ctypes.c_double]),
    "ringattr_generate_inputs": (c_int, [ctypes.c_ulonglong, c_int, c_int, c_int, c_int, ctypes.c_double,
                                         ctypes.POINTER(c_float), c_int, c_float, c_int, c_int, c_float,
                                         c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "ringattr_clip_adam_workspace_bytes": (c_size_t, [c_int, ctypes.POINTER(c_size_t)]),
    "ringattr_clip_adam": (c_int, [c_int, ctypes.POINTER(c_void_p), ctypes.POINTER(c_void_p), ctypes.POINTER(c_void_p),
                                   ctypes.POINTER(c_void_p), ctypes.POINTER(c_size_t), c_float, c_float, c_float,
                                   c_float, c_float, c_int, c_void_p, c_size_t, c_void_p]),
    "ringattr_clip_adam_counted": (c_int, [c_int, ctypes.POINTER(c_void_p), ctypes.POINTER(c_void_p),
                                           ctypes.POINTER(c_void_p), ctypes.POINTER(c_void_p), ctypes.POINTER(c_size_t),
                                           c_float, c_float, c_float, c_float, c_float, c_void_p, c_void_p, c_size_t,
                                           c_void_p]),
    "ringattr_profile_enable": (c_int, [c_int]),
    "ringattr_profile_read": (c_int, [ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_longlong)]),
    "ringattr_last_kernel_name": (c_int, [c_int, ctypes.c_char_p, ctypes.c_size_t]),
    "ringattr_dw_segments": (c_int, [c_int] * 4),
    "fwd_cuda": (None, [c_void_p, c_void_p, c_float, c_float, c_void_p, c_void_p, c_void_p, c_float,
                        c_int, c_int, c_int, c_int, c_int]),
    "bwd_cuda": (None, [c_void_p, c_void_p, c_void_p, c_float, c_float, c_void_p, c_void_p, c_void_p, c_void_p,
                        c_void_p, c_void_p, c_float, c_int, c_int, c_int, c_int, c_int,
                        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
}


def library_path() -> str:
    """In-tree library, or the file named by RINGATTR_LIB (to try an experimental build)."""
    return os.environ.get("RINGATTR_LIB") or _build.LIB_PATH


def load():
    """Return the loaded library, building it first if no prebuilt file exists."""
    global _lib
    with _lock:
        if _lib is not None:
            return _lib
        path = library_path()
        if not os.path.exists(path):
            _build.build_library()
        lib = ctypes.CDLL(path)
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(lib, name)          # AttributeError if the library lacks a declared symbol
            fn.restype = res
            fn.argtypes = args
        _lib = lib
        return lib


def last_error() -> str:
    return load().ringattr_last_error().decode("utf-8", "replace")


def check(rc: int) -> None:
    """Turn a status code into a Python exception (the reference exits the process instead,
    cpp/cuda_common.cuh:30-39)."""
    if rc == 0:
        return
    msg = last_error()
    if rc == 1:
        raise ValueError(msg)
    raise RuntimeError(msg)


KERNEL_NAMES = ("pack_weights", "fwd", "rebuild_saved", "bptt", "dw", "dw_reduce")


def profile_enable(on) -> None:
    """False / 0: off.  True / 1: bracket every kernel launch with HIP events; n > 1: every n-th launch of each kernel
    (the two event records cost the stream 4-5 us per bracketed launch)."""
    check(load().ringattr_profile_enable(int(on)))


def last_kernel_names():
    """{kernel slot name: name of the kernel launched last in it} for the slots that have launched."""
    out = {}
    buf = ctypes.create_string_buffer(256)
    for i, key in enumerate(KERNEL_NAMES):
        check(load().ringattr_last_kernel_name(i, buf, len(buf)))
        if buf.value:
            out[key] = buf.value.decode()
    return out


def profile_read():
    """Returns {kernel name: (total ms, launches)} of the launches recorded since the last read."""
    n = len(KERNEL_NAMES)
    ms = (ctypes.c_double * n)()
    cnt = (ctypes.c_longlong * n)()
    check(load().ringattr_profile_read(ms, cnt))
    return {KERNEL_NAMES[i]: (ms[i], cnt[i]) for i in range(n)}
