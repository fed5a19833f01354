"""ctypes loaders for the package's two shared libraries.

Both loaders fail loudly: there is no Python or CPU fallback for anything the
libraries provide.  Build them first with ``python -m muxserve_amd.build``.
"""
import ctypes
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
# The in-tree builds; the environment variables let a developer point at an
# alternative build of the same ABI (e.g. one compiled with other flags).
HOST_LIB_PATH = os.environ.get("MUXSERVE_HOST_LIB", os.path.join(_PKG, "libmuxhost.so"))
ATTN_LIB_PATH = os.environ.get("MUXSERVE_ATTN_LIB", os.path.join(_PKG, "libmuxattn.so"))
PROBE_LIB_PATH = os.environ.get("MUXSERVE_PROBE_LIB", os.path.join(_PKG, "libmuxprobe.so"))

_host = None
_attn = None
_probe = None

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
        "mux_sched_enable_device_rows": (c_i32, [c_vp, c_i32]),
        "mux_sched_get_batch_compact": (c_i64, [c_vp, c_vp, c_i32, c_vp, c_i64, c_vp, c_vp, c_i64,
                                                c_vp, c_i64, c_vp, c_i64]),
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


# ---------------------------------------------------------------------------
# libmuxattn.so (include/muxserve_attn.h)
# ---------------------------------------------------------------------------
c_f32 = ctypes.c_float
c_sz = ctypes.c_size_t

MUXA_MAX_DECODE_ITEMS = 8
DTYPE_F16, DTYPE_BF16 = 0, 1


class MuxDecodeItem(ctypes.Structure):
    _fields_ = [
        ("out", c_vp), ("q", c_vp),
        ("out_row_stride", c_i64), ("q_row_stride", c_i64),
        ("block_tables", c_vp), ("context_lens", c_vp),
        ("total_context_len", c_i64),
        ("layer", c_i32), ("num_layers", c_i32), ("num_seqs", c_i32),
        ("num_q_heads", c_i32), ("num_kv_heads", c_i32),
        ("max_blocks", c_i32), ("max_context_len", c_i32),
        ("scale", c_f32),
        ("context_lens_host", c_vp),
    ]


class MuxPrefillItem(ctypes.Structure):
    _fields_ = [
        ("out", c_vp), ("out_row_stride", c_i64), ("q", c_vp), ("q_row_stride", c_i64),
        ("k", c_vp), ("v", c_vp), ("kv_row_stride", c_i64),
        ("cu_seqlens", c_vp), ("prompt_lens_host", c_vp),
        ("num_prompts", c_i32), ("max_prompt_len", c_i32), ("num_q_heads", c_i32), ("num_kv_heads", c_i32),
        ("scale", c_f32),
    ]


class MuxCacheWriteItem(ctypes.Structure):
    _fields_ = [
        ("positions", c_vp), ("q", c_vp), ("q_row_stride", c_i64),
        ("k", c_vp), ("v", c_vp), ("kv_row_stride", c_i64),
        ("cos_sin", c_vp), ("slot_mapping", c_vp),
        ("max_position", c_i32), ("rotary_dim", c_i32), ("layer", c_i32), ("num_layers", c_i32),
        ("num_tokens", c_i32), ("num_q_heads", c_i32), ("num_kv_heads", c_i32),
    ]


ATTN_SIGNATURES = {
    "mux_attn_version": (c_i32, []),
    "mux_last_hip_error": (c_i32, []),
    "mux_reshape_and_cache": (c_i32, [c_vp, c_vp, c_i64, c_vp, c_vp, c_i64, c_vp, c_i32, c_i32,
                                      c_i32, c_i32, c_i32, c_i32, c_i32, c_vp]),
    "mux_multi_prefill_causal": (c_i32, [c_vp, c_i32, c_i32, c_i32, c_vp]),
    "mux_multi_rope_reshape_and_cache": (c_i32, [c_vp, c_i32, c_vp, c_vp, c_i64, c_i32, c_i32, c_i32, c_vp]),
    "mux_paged_decode_workspace_bytes": (c_sz, [c_vp, c_i32, c_i32]),
    "mux_paged_decode_host_pairs": (c_i32, [c_vp, c_i32, c_i32]),
    "mux_paged_decode_workspace_init": (c_i32, [c_vp, c_sz, c_vp]),
    "mux_multi_decode": (c_i32, [c_vp, c_i32, c_vp, c_vp, c_i64, c_i32, c_i32, c_i32, c_i32,
                                 c_vp, c_sz, c_vp]),
    "mux_multi_decode_noalloc_max_bytes": (c_sz, []),
    "mux_multi_decode_noalloc": (c_i32, [c_vp, c_i32, c_vp, c_vp, c_i64, c_i32, c_i32, c_i32, c_i32, c_vp]),
    "mux_paged_decode": (c_i32, [c_vp, c_i64, c_vp, c_i64, c_vp, c_vp, c_i64, c_vp, c_vp,
                                 c_i32, c_i32, c_i32, c_i32, c_i32, c_i32, c_i32, c_i32, c_i32,
                                 c_f32, c_i32, c_i32, c_vp, c_sz, c_vp]),
    "mux_prefill_causal": (c_i32, [c_vp, c_i64, c_vp, c_i64, c_vp, c_vp, c_i64, c_vp, c_vp, c_vp, c_i32, c_i32,
                                   c_i32, c_i32, c_i32, c_f32, c_i32, c_vp]),
    "mux_rotary_neox": (c_i32, [c_vp, c_vp, c_i64, c_vp, c_i64, c_vp, c_i32, c_i32, c_i32, c_i32, c_i32, c_i32,
                                c_i32, c_vp]),
    "mux_rope_reshape_and_cache": (c_i32, [c_vp, c_vp, c_i64, c_vp, c_vp, c_i64, c_vp, c_i32, c_i32, c_vp, c_vp, c_i64,
                                           c_vp, c_i32, c_i32, c_i32, c_i32, c_i32, c_i32, c_i32, c_i32, c_vp]),
    "mux_rms_norm": (c_i32, [c_vp, c_i64, c_vp, c_i64, c_vp, c_f32, c_i32, c_i32, c_i32, c_vp]),
    "mux_silu_and_mul": (c_i32, [c_vp, c_i64, c_vp, c_i64, c_i32, c_i32, c_i32, c_vp]),
    "mux_greedy_sample_workspace_bytes": (c_sz, [c_i32]),
    "mux_greedy_sample_workspace_init": (c_i32, [c_vp, c_sz, c_vp]),
    "mux_greedy_sample": (c_i32, [c_vp, c_vp, c_i64, c_i32, c_vp, c_i32, c_vp, c_i64, c_i32, c_i32, c_i32, c_i32,
                                  c_vp, c_sz, c_vp]),
    "mux_build_step_inputs": (c_i32, [c_vp, c_i32, c_i32, c_i32, c_i32, c_i32, c_vp, c_i32, c_vp, c_i64, c_i32,
                                      c_i32, c_vp, c_vp, c_i32, c_vp]),
    "mux_cu_parts_mask": (c_i32, [ctypes.c_uint32, c_i32, c_vp, c_i32]),
    "mux_stream_create_cu_parts": (c_i32, [c_vp, ctypes.c_uint32, c_vp]),
    "mux_stream_create_cu_range": (c_i32, [c_vp, c_i32, c_i32, c_vp]),
    "mux_stream_destroy": (c_i32, [c_vp]),
    "mux_device_cu_info": (c_i32, [c_vp]),
}


def attn():
    """libmuxattn.so with argument/return types declared."""
    global _attn
    if _attn is not None:
        return _attn
    lib = _open(ATTN_LIB_PATH)
    for name, (res, args) in ATTN_SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _attn = lib
    return lib


def probe():
    """libmuxprobe.so (muxserve_amd/csrc/probe/mux_probe.h): the bare gather-read
    kernel bench.py times next to the attention kernel.  Not part of the product."""
    global _probe
    if _probe is None:
        lib = _open(PROBE_LIB_PATH)
        lib.mux_probe_gather_read.restype = c_i32
        lib.mux_probe_gather_read.argtypes = [c_vp, c_vp, c_i64, c_vp, c_i64, c_i32, c_vp, c_vp]
        lib.mux_probe_copy.restype = c_i32
        lib.mux_probe_copy.argtypes = [c_vp, c_vp, c_i64, c_vp]
        lib.mux_probe_where.restype = c_i32
        lib.mux_probe_where.argtypes = [c_vp, c_i32, c_i32, c_vp]
        lib.mux_probe_scatter_copy.restype = c_i32
        lib.mux_probe_scatter_copy.argtypes = [c_vp, c_vp, c_i64, c_vp, c_vp, c_vp, c_i64, c_vp]
        lib.mux_probe_mfma.restype = c_i32
        lib.mux_probe_mfma.argtypes = [c_i32] * 6 + [c_vp, c_vp, c_vp]
        _probe = lib
    return _probe


ATTN_ERRORS = {-1: "invalid argument", -2: "unsupported shape or dtype",
               -3: "workspace missing or too small", -4: "HIP runtime error",
               -5: "the call needs more scratch than the library's fixed static array holds"}


def check_attn(rc, what):
    if rc != 0:
        extra = ""
        if rc == -4:
            extra = f", hipError {attn().mux_last_hip_error()}"
        raise RuntimeError(f"{what}: {ATTN_ERRORS.get(int(rc), 'error')} (code {int(rc)}{extra})")
