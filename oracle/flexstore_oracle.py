"""TEST INFRASTRUCTURE ONLY - a CPU restatement of two small pieces of the
reference's control side that touch the shared KV pool, for the parity tests of
muxserve_amd.flexstore and muxserve_amd.cu_resource.  Nothing outside tests/
may import this module.

  * deploy_step(): the body of FlexStoreManager.deploy's request loop
    (muxserve/flexstore/manager.py:747-831) for the requests that need no GPU
    memory handle, over any KVStorage with the reference's method names (the
    compiled reference, the oracle's, the product's).
  * SMPart / SMResource: muxserve/muxsched/resource.py:15-81.

Pinned by: the allocator underneath is the compiled reference where oracle/_ref
is built (tests/test_flexstore_parity.py drives it through these same tuples);
the dispatch itself is checked against hand-written expectations of the
reference's documented request formats (manager.py:710-741) and closed forms
of the part bookkeeping (counts conserved, hand-out order of a fresh pool).
"""
import random

_TYPES = ["get_rank", "init_finished", "query_num_ready_processes", "get_num_blocks", "weight", "cache_init",
          "cache_alloc", "start_warmup", "warmup_ready", "blocktable_load", "blocktable_store", "free_cache",
          "lock_init", "log_stats", "exit"]


def new_state(block_manager, model_cache_info, num_gpu_blocks, num_runtime_processes=1, rank=0, local_world_size=1):
    return {"block_manager": block_manager, "model_cache_info": dict(model_cache_info),
            "model_occupy_info": {k: 0 for k in model_cache_info}, "num_gpu_blocks": num_gpu_blocks,
            "num_runtime_processes": num_runtime_processes, "rank": rank, "local_world_size": local_world_size,
            "ready_processes": 0, "process_in_warmup": False, "exited": False}


def deploy_step(st, req):
    """One iteration of the loop at manager.py:747-831; returns what
    tcp_server.send_pyobj would be given."""
    req_type, req_args = req[0], req[1]                     # parse_request, manager.py:684-707
    if req_type not in _TYPES:
        return "Incorrect format"                           # manager.py:756-759
    if req_type == "get_rank":
        ret = st["rank"] * st["local_world_size"] + req_args
    elif req_type == "init_finished":
        ret = st["ready_processes"] == st["num_runtime_processes"]
    elif req_type == "query_num_ready_processes":
        ret = st["ready_processes"]
    elif req_type == "get_num_blocks":
        ret = st["num_gpu_blocks"]
    elif req_type == "start_warmup":
        if st["process_in_warmup"]:
            ret = False
        else:
            st["process_in_warmup"] = True
            ret = True
    elif req_type == "warmup_ready":
        st["process_in_warmup"] = False
        st["ready_processes"] += 1
        ret = st["ready_processes"] == st["num_runtime_processes"]
    elif req_type == "cache_alloc":                         # manager.py:807-811
        model_name, batch_info = req_args
        num_layers, num_heads = st["model_cache_info"][model_name]
        ret = st["block_manager"].allocate_batch(batch_info, num_layers, num_heads)
    elif req_type == "free_cache":                          # manager.py:814-819
        model_name, finished_request_ids = req_args
        num_freed_blocks = st["block_manager"].free_batch(finished_request_ids)
        st["model_occupy_info"][model_name] -= num_freed_blocks
        ret = None
    elif req_type == "log_stats":
        ret = None
    elif req_type == "exit":
        st["exited"] = True
        ret = None
    elif req_type in ("weight", "cache_init", "lock_init"):
        raise NotImplementedError(req_type)                 # needs CUDA IPC handles (manager.py:784-806)
    else:
        raise RuntimeError("Unknown request type")          # manager.py:828-830
    return ret


class SMPart:                                               # resource.py:15-32
    def __init__(self, id):
        self.id = id
        self.ref_count = 0

    def acquire(self):
        self.ref_count += 1

    def release(self):
        self.ref_count -= 1

    def is_idle(self):
        return self.ref_count == 0

    def is_overloaded(self):
        return self.ref_count > 1


class SMResource:                                           # resource.py:35-81
    def __init__(self, overload_threshold=4):
        self.overload_threshold = overload_threshold
        self._sm_parts = {}
        self.free_sms = []
        self.unoverloaded_sms = []
        for i in range(10):
            self._sm_parts[i] = SMPart(i)
            self.free_sms.append(self._sm_parts[i])
            self.unoverloaded_sms.append(i)

    def can_allocate(self, num_sms, overload=False):
        extra = min(self.overload_threshold, len(self.unoverloaded_sms)) if overload else 0
        return len(self.free_sms) + extra >= num_sms

    def allocate(self, num_sms, overload=False):
        ret = []
        for _ in range(num_sms):
            if len(self.free_sms) > 0:
                sm = self.free_sms.pop()
            else:
                sm_id = random.choice(self.unoverloaded_sms)
                sm = self._sm_parts[sm_id]
                self.unoverloaded_sms.remove(sm_id)
            sm.acquire()
            ret.append(sm)
        return ret

    def free(self, sms):
        for sm in sms:
            sm.release()
            if sm.is_idle():
                self.free_sms.append(sm)
            if not sm.is_overloaded() and sm.id not in self.unoverloaded_sms:
                self.unoverloaded_sms.append(sm.id)

    @property
    def num_free_sms(self):
        return len(self.free_sms)

    @property
    def num_overloaded_sms(self):
        return len(self._sm_parts) - len(self.unoverloaded_sms)
