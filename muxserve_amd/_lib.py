"""ctypes loaders for the package's two shared libraries.

Both loaders fail loudly: there is no Python or CPU fallback for anything the
libraries provide.  Build them first with ``python -m muxserve_amd.build``.
"""
import ctypes
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
HOST_LIB_PATH = os.path.join(_PKG, "libmuxhost.so")
ATTN_LIB_PATH = os.path.join(_PKG, "libmuxattn.so")

_host = None
_attn = None

c_i32 = ctypes.c_int32
c_i64 = ctypes.c_int64
c_vp = ctypes.c_void_p
p_i32 = ctypes.POINTER(ctypes.c_int32)
p_i64 = ctypes.POINTER(ctypes.c_int64)


class MuxLibraryMissing(RuntimeError):
    pass


def _open(path):
    if not os.path.exists(path):
        raise MuxLibraryMissing(
            f"{path} is not built; run `python -m muxserve_amd.build` (there is no fallback path)")
    return ctypes.CDLL(path)


def host():
    """libmuxhost.so with argument/return types declared (include/muxserve_host.h)."""
    global _host
    if _host is not None:
        return _host
    lib = _open(HOST_LIB_PATH)
    sig = {
        "mux_kvstorage_create": (c_vp, [c_i32]),
        "mux_kvstorage_destroy": (None, [c_vp]),
        "mux_kvstorage_allocate": (c_i32, [c_vp, c_i32, c_vp]),
        "mux_kvstorage_allocate_batch_bound": (c_i64, [c_vp, c_i32, c_i32, c_i32]),
        "mux_kvstorage_allocate_batch": (c_i64, [c_vp, c_vp, c_i32, c_i32, c_i32, c_vp, c_i64]),
        "mux_kvstorage_free_batch": (c_i64, [c_vp, c_vp, c_i32]),
        "mux_kvstorage_new_blocks_allocated": (c_i32, [c_vp]),
        "mux_kvstorage_num_free": (c_i64, [c_vp]),
        "mux_kvstorage_num_held": (c_i64, [c_vp, c_i32]),
        "mux_sched_create": (c_vp, [c_i32, c_i32, c_i32, c_i32]),
        "mux_sched_destroy": (None, [c_vp]),
        "mux_sched_add_request": (c_i32, [c_vp, c_vp, c_i32, c_i32, c_i32]),
        "mux_sched_try_batch": (c_i32, [c_vp, c_vp, c_i32, c_vp, c_i32, c_vp]),
        "mux_sched_get_batch_info": (c_i32, [c_vp, c_vp, c_i32, c_vp, c_i64, c_vp, c_i32]),
        "mux_sched_get_batch": (c_i64, [c_vp, c_vp, c_i32, c_vp, c_i64, c_vp, c_vp, c_i64,
                                        c_vp, c_i64, c_vp, c_i64, c_vp, c_i64]),
        "mux_sched_get_batch_permuted": (c_i64, [c_vp, c_vp, c_i32, c_vp, c_i64, c_vp, c_vp, c_i64,
                                                 c_vp, c_i64, c_vp, c_i64, c_i32, c_vp, c_i64]),
        "mux_sched_release_requests": (c_i32, [c_vp, c_vp, c_i32]),
        "mux_sched_get_preempt_requests": (c_i32, [c_vp, c_vp, c_i32]),
        "mux_sched_get_prompt_info": (c_i32, [c_vp, c_vp, c_i32]),
        "mux_sched_get_batch_reqs": (c_i32, [c_vp, c_vp, c_i32]),
        "mux_sched_request_state": (c_i32, [c_vp, c_i32, c_vp]),
        "mux_sched_num_requests": (c_i32, [c_vp]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _host = lib
    return lib


HOST_ERRORS = {-1: "invalid argument", -2: "buffer too small / pool exhausted",
               -3: "unknown request id", -4: "call sequence violates the step protocol"}


def check_host(rc, what):
    if rc < 0:
        msg = f"{what}: {HOST_ERRORS.get(int(rc), 'error')} (code {int(rc)})"
        if rc == -3:
            raise KeyError(msg)
        if rc == -2:
            raise MemoryError(msg)
        raise ValueError(msg)
    return rc
