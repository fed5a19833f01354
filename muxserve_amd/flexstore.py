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
Requests whose answer is a GPU memory handle to open in another process -
"weight", "cache_init", "lock_init" (manager.py:784-806) - raise
IpcExportExcluded: exporting the pool across processes is not part of this
build.  A request type outside the reference's list is answered with the
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
    """The request asks for a GPU memory handle for another process."""


class CacheRequestHandler:
    """State of the manager's loop next to the allocator: per-model (layers,
    heads) and occupancy, the start-up counters."""

    def __init__(self, storage, model_cache_info: Dict[str, Tuple[int, int]], num_gpu_blocks: int,
                 num_runtime_processes: int = 1, rank: int = 0, local_world_size: int = 1):
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
        if kind in ("weight", "cache_init", "lock_init"):
            raise IpcExportExcluded(f"{kind}: GPU memory handles for other processes are not exported by this build")
        raise RuntimeError("Unknown request type")

    def cache_alloc_for(self, model_name: str):
        """The ``cache_alloc`` callable prepare_inputs takes, bound to a model:
        the runtime's request at llm_runtime.py:284-286 without the socket."""
        return lambda batch_block_request: self.handle(("cache_alloc", [model_name, batch_block_request]))
