"""CPU restatement of the reference's host-side block allocator and batch builder.

TEST INFRASTRUCTURE ONLY: this module is the checker for
muxserve_amd.memory_manager / muxserve_amd.batch_scheduler.  Nothing in the
product package may import it.

Each function follows the reference lines cited in its docstring (paths are
relative to the reference checkout).  Pinning: tests/test_host_oracle.py drives
this restatement and the compiled reference (oracle/_ref, built from the
reference's own csrc/*.cpp) through identical scripted scenarios and compares
every return value; the committed fixtures under tests/golden/ hold the
compiled reference's outputs so the comparison also runs where the reference
checkout is absent.

Deliberate differences from the reference, both on memory the reference leaves
uninitialised: Request.allocated_blocks starts at -1 (reference: uninitialised
py::array_t, csrc/batch_scheduler.cpp:16-17) and get_batch() leaves block-table
entries past a request's physical blocks untouched (reference copies its own
uninitialised scratch there, csrc/batch_scheduler.cpp:156-168,190-191).
"""
from __future__ import annotations

import numpy as np


class KVStorage:
    """csrc/memory_manager.h:8-28, csrc/memory_manager.cpp:4-157."""

    def __init__(self, num_blocks: int):
        # memory_manager.cpp:4-10 - free list is 0..N-1 in ascending order.
        self.num_blocks = int(num_blocks)
        self.free_blocks = list(range(self.num_blocks))
        self.allocated = {}          # request id -> list of head-block ids
        self.num_blocks_allocated = 0
        self.new_blocks_allocated = 0

    def allocate(self, size: int) -> np.ndarray:
        # memory_manager.cpp:12-23 - pop from the back, one id at a time.
        out = np.empty(size, dtype=np.int32)
        for i in range(size):
            out[i] = self.free_blocks.pop()
        return out

    def allocate_batch(self, batch_alloc_info, num_layers: int, num_heads: int) -> np.ndarray:
        # memory_manager.cpp:25-142
        info = np.asarray(batch_alloc_info, dtype=np.int32).reshape(-1)
        num_requests = info.size // 3
        num_free = len(self.free_blocks)
        per_token_block = num_layers * num_heads

        total_new = 0
        to_allocate = []                 # numBlocksToAllocate
        total_request = [0] * (num_requests + 1)
        new_needed_prefix = []           # newBlocksNeededList (running sum)
        old_allocated = []               # oldBlocksAllocatedList
        for i in range(num_requests):    # :34-55
            rid = int(info[3 * i])
            n_req = int(info[3 * i + 1]) * per_token_block
            prompt_allocated = int(info[3 * i + 2])
            n_new = n_req
            if not prompt_allocated:
                if rid in self.allocated:
                    n_new -= len(self.allocated[rid])
                    old_allocated.append(len(self.allocated[rid]))
                else:
                    old_allocated.append(0)
            else:
                # std::map::operator[] default-constructs an empty entry (:50)
                old_allocated.append(len(self.allocated.setdefault(rid, [])))
            total_new += n_new
            new_needed_prefix.append(total_new)
            to_allocate.append(n_new)
            total_request[i + 1] = total_request[i] + n_req

        suffix = [0] * (num_requests + 1)      # :57-62
        for i in range(num_requests - 1, -1, -1):
            suffix[i] = suffix[i + 1] + old_allocated[i]

        preempt_idx = num_requests             # :64-72
        while preempt_idx >= 0:
            expected = num_free + suffix[preempt_idx]
            if preempt_idx == 0 or new_needed_prefix[preempt_idx - 1] <= expected:
                break
            preempt_idx -= 1

        freed = 0                               # :74-86
        for i in range(preempt_idx, num_requests):
            rid = int(info[3 * i])
            if old_allocated[i] > 0:
                freed += old_allocated[i]
                self.free_blocks.extend(self.allocated[rid])
                del self.allocated[rid]
        self.num_blocks_allocated -= freed
        self.new_blocks_allocated = -freed

        if preempt_idx <= 0:                    # :88-94
            return np.array([preempt_idx], dtype=np.int32)

        out = np.empty(total_request[preempt_idx] + 1, dtype=np.int32)   # :96-102
        out[0] = preempt_idx
        take = new_needed_prefix[preempt_idx - 1]
        assert len(self.free_blocks) >= take
        tail = self.free_blocks[len(self.free_blocks) - take:]           # :106

        offset = 0
        batch_offset = 1
        for i in range(preempt_idx):            # :107-136
            n_new = to_allocate[i]
            rid = int(info[3 * i])
            n_req = int(info[3 * i + 1]) * per_token_block
            if n_new > 0:
                self.allocated.setdefault(rid, []).extend(tail[offset:offset + n_new])
                offset += n_new
            if n_req > 0:
                held = self.allocated.setdefault(rid, [])
                assert len(held) >= n_req
                out[batch_offset:batch_offset + n_req] = held[len(held) - n_req:]
                batch_offset += n_req
        self.new_blocks_allocated += take       # :137-140
        self.num_blocks_allocated += self.new_blocks_allocated
        if take > 0:
            del self.free_blocks[len(self.free_blocks) - take:]
        return out

    def free_batch(self, request_ids) -> int:
        # memory_manager.cpp:144-157
        freed = 0
        for rid in request_ids:
            rid = int(rid)
            if rid in self.allocated:
                freed += len(self.allocated[rid])
                self.free_blocks.extend(self.allocated[rid])
                del self.allocated[rid]
        self.num_blocks_allocated -= freed
        return freed

    def get_new_blocks_allocated(self) -> int:
        # memory_manager.h:17
        return self.new_blocks_allocated


class _Request:
    """csrc/batch_scheduler.h:9-68."""

    def __init__(self, req_id, max_tokens, prompts, block_size):
        # batch_scheduler.h:22-29
        self.idx = int(req_id)
        self.max_tokens = int(max_tokens)
        self.block_size = int(block_size)
        self.num_physical_blocks = 0
        self.prompts = np.array(prompts, dtype=np.int32).reshape(-1)
        self.outputs = []
        p = int(self.prompts.size)
        # C++ integer division/modulo truncate toward zero (matters only for
        # p == 0, which the reference never submits).
        self.logical_block_idx = (p + block_size - 1) // block_size - 1
        self.logical_block_offset = int(np.fmod(p - 1, block_size))
        self.context_len = p
        self.allocated_blocks = None

    def append_logical_token(self, token_id):
        # batch_scheduler.h:31-40
        self.outputs.append(int(token_id))
        self.context_len += 1
        self.logical_block_offset += 1
        if self.logical_block_offset == self.block_size:
            self.logical_block_idx += 1
            self.logical_block_offset = 0
        return self.logical_block_idx + 1 - self.num_physical_blocks

    def prompt_slots(self, num_layers, num_heads, out):
        # batch_scheduler.h:42-56
        per = num_layers * num_heads
        flat = self.allocated_blocks.reshape(-1)
        for i in range(self.prompts.size):
            tb, off = divmod(i, self.block_size)
            for j in range(per):
                out.append(int(flat[tb * per + j]) * self.block_size + off)

    def last_empty_slot(self, num_layers, num_heads, out):
        # batch_scheduler.h:58-67
        per = num_layers * num_heads
        flat = self.allocated_blocks.reshape(-1)
        base = (self.num_physical_blocks - 1) * per
        for i in range(per):
            out.append(int(flat[base + i]) * self.block_size + self.logical_block_offset)


def _flat_view(t):
    """Flat writable numpy view of a caller-allocated CPU tensor / array."""
    if isinstance(t, np.ndarray):
        return t.reshape(-1)
    return t.view(-1).numpy()   # torch CPU tensor, shares memory


class BatchScheduler:
    """csrc/batch_scheduler.h:70-106, csrc/batch_scheduler.cpp:4-199."""

    def __init__(self, num_layers, num_heads, max_seq_len, block_size):
        # batch_scheduler.cpp:4-10
        self.num_layers = int(num_layers)
        self.num_heads = int(num_heads)
        self.max_seq_len = int(max_seq_len)
        self.block_size = int(block_size)
        self.max_blocks_per_seq = (self.max_seq_len + self.block_size - 1) // self.block_size
        self.requests = {}
        self.preempt_requests = []
        self.prompt_info = []
        self.batch_reqs = []

    def add_request(self, prompt, req_id, max_tokens):
        # batch_scheduler.cpp:12-19
        r = _Request(req_id, max_tokens, prompt, self.block_size)
        r.allocated_blocks = np.full(
            (self.max_blocks_per_seq, self.num_layers, self.num_heads), -1, dtype=np.int32)
        self.requests[int(req_id)] = r

    def try_batch(self, request_ids, last_output_tokens) -> np.ndarray:
        # batch_scheduler.cpp:21-48
        decoding = len(last_output_tokens) > 0
        n = len(request_ids)
        info = np.empty(3 * n + 1, dtype=np.int32)
        total = 0
        for i, rid in enumerate(request_ids):
            r = self.requests[int(rid)]
            need = r.logical_block_idx + 1
            if decoding:
                need = r.append_logical_token(last_output_tokens[i])
            info[3 * i] = r.idx
            info[3 * i + 1] = need
            info[3 * i + 2] = min(r.num_physical_blocks, 1)
            total += need
        info[3 * n] = total
        return info

    def get_batch_info(self, batch_block_request, block_info):
        # batch_scheduler.cpp:50-97
        req = np.asarray(batch_block_request, dtype=np.int32).reshape(-1)
        blk = np.asarray(block_info, dtype=np.int32).reshape(-1)
        per = self.num_layers * self.num_heads
        num_tokens = num_contexts = max_ctx = max_blocks = 0
        prompt_info = []
        preempt_idx = int(blk[0])
        off = 1
        for i in range(preempt_idx):
            rid = int(req[3 * i])
            need = int(req[3 * i + 1]) * per
            r = self.requests[rid]
            if need > 0:
                flat = r.allocated_blocks.reshape(-1)
                dst = r.num_physical_blocks * per
                flat[dst:dst + need] = blk[off:off + need]
                off += need
                r.num_physical_blocks += int(req[3 * i + 1])
            if len(r.outputs) > 0:
                max_blocks = max(max_blocks, r.num_physical_blocks)
                max_ctx = max(max_ctx, r.context_len)
                num_contexts += 1
                num_tokens += 1
            else:
                prompt_info.append(int(r.prompts.size))
                num_tokens += int(r.prompts.size)
        return [num_tokens, num_contexts, max_ctx, max_blocks,
                self.num_layers, self.num_heads] + prompt_info

    def get_batch(self, batch_info, block_info, token_t, pos_t, ctxlen_t, blocktable_t, slot_t):
        # batch_scheduler.cpp:99-193
        req = np.asarray(batch_info, dtype=np.int32).reshape(-1)
        blk = np.asarray(block_info, dtype=np.int32).reshape(-1)
        per = self.num_layers * self.num_heads
        tokens, positions, ctx_lens, slots = [], [], [], []
        self.preempt_requests = []
        self.prompt_info = []
        self.batch_reqs = []
        num_tokens = max_ctx = max_blocks = 0
        n = req.size // 3
        preempt_idx = int(blk[0])
        for i in range(n):
            rid = int(req[3 * i])
            if i >= preempt_idx:                      # :123-129
                self.preempt_requests.append(rid)
                self.requests.pop(rid, None)
                continue
            r = self.requests[rid]
            if len(r.outputs) > 0:                    # :132-140
                max_blocks = max(max_blocks, r.num_physical_blocks)
                tokens.append(r.outputs[-1])
                positions.append(r.context_len - 1)
                ctx_lens.append(r.context_len)
                max_ctx = max(max_ctx, r.context_len)
                r.last_empty_slot(self.num_layers, self.num_heads, slots)
                num_tokens += 1
            else:                                     # :141-151
                tokens.extend(int(x) for x in r.prompts)
                positions.extend(range(int(r.prompts.size)))
                self.prompt_info.append(int(r.prompts.size))
                r.prompt_slots(self.num_layers, self.num_heads, slots)
                num_tokens += int(r.prompts.size)
            self.batch_reqs.append([rid, r.max_tokens])
        self.prompt_info.append(max_ctx)              # :154

        tok = _flat_view(token_t)
        pos = _flat_view(pos_t)
        ctx = _flat_view(ctxlen_t)
        slot = _flat_view(slot_t)
        tok[:len(tokens)] = tokens                    # :171-186
        pos[:len(positions)] = positions
        tok[len(tokens):] = 0
        pos[len(positions):] = 0
        ctx[:len(ctx_lens)] = ctx_lens
        slot[:len(slots)] = slots
        if max_blocks > 0:                            # :156-169
            bt = _flat_view(blocktable_t)
            for i in range(preempt_idx):
                r = self.requests[int(req[3 * i])]
                cnt = r.num_physical_blocks * per
                dst = i * max_blocks * per
                bt[dst:dst + cnt] = r.allocated_blocks.reshape(-1)[:cnt]

    def release_requests(self, request_ids):
        # batch_scheduler.cpp:195-199
        for rid in request_ids:
            self.requests.pop(int(rid), None)

    def get_preempt_requests(self):
        return list(self.preempt_requests)

    def get_prompt_info(self):
        return list(self.prompt_info)

    def get_batch_reqs(self):
        return [list(x) for x in self.batch_reqs]


def prepare_inputs(sched, storage, num_layers, num_heads, request_ids, output_tokens, *, fill=0):
    """Restatement of LLMRuntime.prepare_inputs with the FlexStore round trip
    replaced by a direct call (muxserve/flexserver/llm_runtime.py:277-339,
    muxserve/flexstore/manager.py:807-811).  Works with any (sched, storage)
    pair exposing the reference method names (this module's classes, the
    compiled reference, or the product's).  Tensors are CPU torch tensors as in
    the reference; memory the reference leaves to torch.empty is pre-filled
    with `fill` so results are comparable.

    Returns a dict with the reference's names: input_tensor/input_positions
    (int64, padded to a multiple of 8), slot_mapping int64 [T, L, H],
    context_lens int32 [num_contexts], block_tables int32 [L, B, H, maxBlk]
    (after the permute(2,0,3,1) at llm_runtime.py:327), plus prompt_lens,
    max_context_len, batch_reqs, preempted_reqs and the raw allocator reply.
    """
    import torch

    info = np.asarray(sched.try_batch(list(request_ids), list(output_tokens)), dtype=np.int32)
    total_needed = int(info[-1])
    req = np.ascontiguousarray(info[:-1])
    if total_needed > 0:
        block_info = np.asarray(storage.allocate_batch(req, num_layers, num_heads), dtype=np.int32)
    else:
        block_info = np.array([len(request_ids)], dtype=np.int32)
    bi = list(sched.get_batch_info(req, block_info))
    num_tokens, num_contexts, max_ctx, max_blk, L, H = bi[:6]
    prompt_lens = list(bi[6:])
    padded = (num_tokens + 7) // 8 * 8
    slot_mapping = torch.full((num_tokens, L, H), fill, dtype=torch.int64)
    if max_ctx > 0:
        block_tables = torch.full((num_tokens, max_blk, L, H), fill, dtype=torch.int32)
    else:
        block_tables = torch.full((0, max_blk, 0, 0), fill, dtype=torch.int32)
    input_tensor = torch.full((padded,), fill, dtype=torch.int32)
    input_positions = torch.full((padded,), fill, dtype=torch.int32)
    context_lens = torch.full((num_contexts,), fill, dtype=torch.int32)
    sched.get_batch(req, block_info, input_tensor, input_positions, context_lens,
                    block_tables, slot_mapping)
    return {
        "input_tensor": input_tensor.long(),
        "input_positions": input_positions.long(),
        "slot_mapping": slot_mapping,
        "context_lens": context_lens,
        "block_tables_raw": block_tables,
        "block_tables": block_tables.permute(2, 0, 3, 1).contiguous(),
        "prompt_lens": prompt_lens,
        "max_context_len": max_ctx,
        "batch_reqs": sched.get_batch_reqs(),
        "preempted_reqs": sched.get_preempt_requests(),
        "block_info": block_info,
        "batch_block_request": req,
    }
