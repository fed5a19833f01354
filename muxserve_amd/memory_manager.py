"""KVStorage - the head-granular KV block allocator, same Python surface as
the reference's pybind11 module ``muxserve.memory_manager``
(csrc/memory_manager.cpp:159-166): KVStorage(num_blocks), allocate,
allocate_batch, free_batch, get_new_blocks_allocated.  The work is done by
libmuxhost.so; this file only marshals numpy arrays across the C ABI.

Error behaviour differs from the reference where the reference has none: an
allocate() larger than the free list raises MemoryError (reference: pops an
empty vector), a malformed request vector raises ValueError (reference:
assert/abort).
"""
import numpy as np

from . import _lib


def _i32(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.int32).reshape(-1))


class KVStorage:
    def __init__(self, num_blocks: int):
        self._lib = _lib.host()
        self._h = self._lib.mux_kvstorage_create(int(num_blocks))
        if not self._h:
            raise ValueError(f"KVStorage: bad num_blocks {num_blocks}")
        self.num_blocks = int(num_blocks)

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.mux_kvstorage_destroy(h)

    def allocate(self, size: int) -> np.ndarray:
        out = np.empty(int(size), dtype=np.int32)
        _lib.check_host(self._lib.mux_kvstorage_allocate(self._h, int(size), out.ctypes.data),
                        "KVStorage.allocate")
        return out

    def allocate_batch(self, batch_alloc_info, num_layers: int, num_heads: int) -> np.ndarray:
        info = _i32(batch_alloc_info)
        cap = _lib.check_host(
            self._lib.mux_kvstorage_allocate_batch_bound(info.ctypes.data, info.size,
                                                         int(num_layers), int(num_heads)),
            "KVStorage.allocate_batch")
        out = np.empty(cap, dtype=np.int32)
        n = _lib.check_host(
            self._lib.mux_kvstorage_allocate_batch(self._h, info.ctypes.data, info.size,
                                                   int(num_layers), int(num_heads),
                                                   out.ctypes.data, cap),
            "KVStorage.allocate_batch")
        return out[:n].copy() if n != cap else out

    def free_batch(self, request_ids) -> int:
        ids = _i32(list(request_ids))
        return int(_lib.check_host(self._lib.mux_kvstorage_free_batch(self._h, ids.ctypes.data, ids.size),
                                   "KVStorage.free_batch"))

    def get_new_blocks_allocated(self) -> int:
        return int(self._lib.mux_kvstorage_new_blocks_allocated(self._h))

    # -- not in the reference's Python surface (its C++ members are private to
    #    pybind): used by the invariants tests and the pool accounting --------
    def num_free(self) -> int:
        return int(self._lib.mux_kvstorage_num_free(self._h))

    def num_held(self, request_id: int) -> int:
        return int(self._lib.mux_kvstorage_num_held(self._h, int(request_id)))
