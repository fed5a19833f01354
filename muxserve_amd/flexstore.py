"""The request side of FlexStore: what the memory manager process answers to
the runtimes' requests about the shared KV pool.

In the reference every model runtime is a process of its own and talks to the
FlexStoreManager process over a ZMQ REQ/REP socket; the manager's loop
(FlexStoreManager.deploy, muxserve/flexstore/manager.py:709-838) parses a
``(request type, arguments)`` tuple, acts on the one shared KVStorage and sends
the reply back.  This module is that loop's body as a function of the request
- no socket, no process: ``CacheRequestHandler.handle(request) -> reply`` - so
it serves an in-process call (prepare_inputs' ``cache_alloc`` callable), a pipe
or any transport a deployment brings.

Answered exactly as the reference frames them:
  ("cache_alloc", [model_name, batch_block_request])  manager.py:807-811
      -> KVStorage.allocate_batch(batch_block_request, num_layers, num_heads)
  ("free_cache", [model_name, finished_request_ids])  manager.py:814-819
      -> None; the freed head-blocks leave the model's occupancy count
  ("get_num_blocks", None)                             manager.py:768-769
  the start-up bookkeeping: "get_rank", "init_finished",
  "query_num_ready_processes", "start_warmup", "warmup_ready"  manager.py:762-783
  "log_stats" -> None, "exit" -> None and the handler is closed  manager.py:820-827
  ("cache_init", [rank, model_name])                   manager.py:789-793
      -> (metadata of the K pool, metadata of the V pool) as get_tensor_metadata
         makes it (manager.py:893-911): the IPC handle of the pool's storage
         plus sizes, strides, dtype - what the runtime side hands to
         torch.multiprocessing.reductions.rebuild_cuda_tensor, as the reference's
         model_loader.py:46 does with the weights.  Answered only when the handler
         was given the pool tensors and each stays under MAX_IPC_BYTES: a shared
         allocation of 2 GiB or more cannot be opened by another process on the
         hosts this build runs on, so a pool of that size raises
         IpcExportExcluded instead.
Requests for the other GPU memory handles - "weight", "lock_init"
(manager.py:784-806) - raise IpcExportExcluded: model weights and the lock
tensor are not part of this build.  A request type outside the reference's list is answered with the
string "Incorrect format" (manager.py:756-759); one that is in the list but has
no branch in the loop ("blocktable_load", "blocktable_store") raises
RuntimeError("Unknown request type") as the reference does (manager.py:828-830).
"""
from typing import Any, Dict, Optional, Sequence, Tuple

import numpy as np

REQUEST_TYPES = (
    "get_rank", "init_finished", "query_num_ready_processes", "get_num_blocks", "weight", "cache_init",
    "cache_alloc", "start_warmup", "warmup_ready", "blocktable_load", "blocktable_store", "free_cache",
    "lock_init", "log_stats", "exit",
)
INCORRECT_FORMAT = "Incorrect format"


class IpcExportExcluded(NotImplementedError):
    """The request asks for a GPU memory handle this build does not export."""


# Shared device allocations of 2 GiB and more do not open in a second process here.
MAX_IPC_BYTES = (2 << 30) - 1


def tensor_metadata(tensor) -> Dict[str, Any]:
    """What another process needs to map `tensor`'s memory: the fields of
    get_tensor_metadata (muxserve/flexstore/manager.py:893-911), which are the
    keyword arguments of torch.multiprocessing.reductions.rebuild_cuda_tensor.
    The tensor's storage must stay alive in this process while others use it."""
    storage = tensor.untyped_storage()
    t = storage._share_cuda_()
    return {
        "tensor_size": tensor.size(),
        "tensor_stride": tensor.stride(),
        "tensor_offset": tensor.storage_offset(),
        "storage_cls": type(storage),
        "dtype": tensor.dtype,
        "storage_device": t[0],
        "storage_handle": t[1],
        "storage_size_bytes": t[2],
        "storage_offset_bytes": t[3],
        "requires_grad": tensor.requires_grad,
        "ref_counter_handle": t[4],
        "ref_counter_offset": t[5],
        "event_handle": t[6],
        "event_sync_required": t[7],
    }


def rebuild_tensor(metadata: Dict[str, Any]):
    """The runtime side of tensor_metadata: a tensor over the other process's
    memory (muxserve/flexserver/model_loader.py:46)."""
    import torch
    from torch.multiprocessing.reductions import rebuild_cuda_tensor
    return rebuild_cuda_tensor(torch.Tensor, **metadata)


class CacheRequestHandler:
    """State of the manager's loop next to the allocator: per-model (layers,
    heads) and occupancy, the start-up counters."""

    def __init__(self, storage, model_cache_info: Dict[str, Tuple[int, int]], num_gpu_blocks: int,
                 num_runtime_processes: int = 1, rank: int = 0, local_world_size: int = 1, gpu_cache=None):
        """gpu_cache: optional (k_pool, v_pool) device tensors this process owns;
        with them "cache_init" is answered (pools under MAX_IPC_BYTES each)."""
        self.gpu_cache = gpu_cache
        self._gpu_cache_metadata = None
        self.block_manager = storage
        self.model_cache_info = {k: (int(v[0]), int(v[1])) for k, v in model_cache_info.items()}
        self.model_occupy_info = {k: 0 for k in self.model_cache_info}
        self.num_gpu_blocks = int(num_gpu_blocks)
        self.num_runtime_processes = int(num_runtime_processes)
        self.rank, self.local_world_size = int(rank), int(local_world_size)
        self.ready_processes = 0
        self.process_in_warmup = False
        self.closed = False

    @staticmethod
    def parse_request(req: Sequence) -> Optional[Tuple[str, Any]]:
        req_type, req_args = req[0], req[1]
        if req_type not in REQUEST_TYPES:
            return None
        return req_type, req_args

    def handle(self, req: Sequence):
        """One request, one reply (what the loop would send back)."""
        if self.closed:
            raise RuntimeError("the handler has answered an exit request")
        parsed = self.parse_request(req)
        if parsed is None:
            return INCORRECT_FORMAT
        kind, args = parsed
        if kind == "cache_alloc":
            model_name, batch_info = args
            num_layers, num_heads = self.model_cache_info[model_name]
            return self.block_manager.allocate_batch(np.ascontiguousarray(batch_info, dtype=np.int32), num_layers,
                                                     num_heads)
        if kind == "free_cache":
            model_name, finished_request_ids = args
            freed = self.block_manager.free_batch(list(finished_request_ids))
            self.model_occupy_info[model_name] -= int(freed)
            return None
        if kind == "get_num_blocks":
            return self.num_gpu_blocks
        if kind == "get_rank":
            return self.rank * self.local_world_size + int(args)
        if kind == "init_finished":
            return self.ready_processes == self.num_runtime_processes
        if kind == "query_num_ready_processes":
            return self.ready_processes
        if kind == "start_warmup":
            if self.process_in_warmup:
                return False
            self.process_in_warmup = True
            return True
        if kind == "warmup_ready":
            self.process_in_warmup = False
            self.ready_processes += 1
            return self.ready_processes == self.num_runtime_processes
        if kind == "log_stats":
            return None
        if kind == "exit":
            self.closed = True
            return None
        if kind == "cache_init":
            if self.gpu_cache is None:
                raise IpcExportExcluded("cache_init: this handler was not given the pool tensors")
            if self._gpu_cache_metadata is None:          # once, as at manager.py:390-393
                for t in self.gpu_cache:
                    if t.untyped_storage().nbytes() > MAX_IPC_BYTES:
                        raise IpcExportExcluded(
                            f"cache_init: a pool tensor of {t.untyped_storage().nbytes()} bytes cannot be opened by "
                            f"another process here (shared allocations stay under {MAX_IPC_BYTES + 1} bytes)")
                self._gpu_cache_metadata = tuple(tensor_metadata(t) for t in self.gpu_cache)
            return self._gpu_cache_metadata
        if kind in ("weight", "lock_init"):
            raise IpcExportExcluded(f"{kind}: not exported by this build (no model weights, no lock tensor)")
        raise RuntimeError("Unknown request type")

    def cache_alloc_for(self, model_name: str):
        """The ``cache_alloc`` callable prepare_inputs takes, bound to a model:
        the runtime's request at llm_runtime.py:284-286 without the socket."""
        return lambda batch_block_request: self.handle(("cache_alloc", [model_name, batch_block_request]))
