"""Per-step input construction, as LLMRuntime.prepare_inputs does it
(muxserve/flexserver/llm_runtime.py:277-339): BatchScheduler.try_batch ->
block allocation -> get_batch_info -> get_batch -> device tensors ->
InputMetadata.

The FlexStore round trip (a ZMQ "cache_alloc" request served by
FlexStoreManager.deploy, muxserve/flexstore/manager.py:807-811) is a callable
here: ``cache_alloc(batch_block_request) -> block_info``; with one process and
one pool it is simply ``lambda r: storage.allocate_batch(r, L, H)``.
"""
from typing import Callable, List, Sequence, Tuple

import numpy as np
import torch

from .attention import InputMetadata
from .batch_scheduler import BatchScheduler


def prepare_inputs(batch_scheduler: BatchScheduler, cache_alloc: Callable[[np.ndarray], np.ndarray],
                   batch_request_ids: Sequence[int], batch_output_tokens: Sequence[int], device="cuda:0",
                   permuted_tables: bool = False, device_tables=None
                   ) -> Tuple[torch.Tensor, torch.Tensor, InputMetadata, List[List[int]], List[int]]:
    """Returns (input_tensor int64 [T_pad], input_positions int64 [T_pad],
    input_metadata, batch_reqs, preempted_reqs) - the reference's return tuple.

    permuted_tables=False follows the reference literally: the block table is
    written as [T, max_blocks, L, H] on the host, then
    permute(2, 0, 3, 1).contiguous() on the device (llm_runtime.py:327); True
    lets the builder emit [L, B, H, max_blocks] on the host (no device permute,
    but the host-side transpose costs more than it saves: 0.5 against 0.25 ms
    per decode step of a 7B model).  Both give identical tensors on the valid
    entries.

    device_tables (a muxserve_amd.device_tables.DeviceBlockTables bound to this
    scheduler): the block table and the slot mapping are not built on the host
    at all; the step uploads one small buffer and the device derives both from
    its mirror of the requests' block ids - same tensors again.
    """
    info = batch_scheduler.try_batch(list(batch_request_ids), list(batch_output_tokens))
    total_blocks_needed = int(info[-1])
    batch_block_request = np.ascontiguousarray(info[:-1])
    if total_blocks_needed > 0:
        block_info = np.asarray(cache_alloc(batch_block_request), dtype=np.int32)
    else:
        block_info = np.array([len(batch_request_ids)], dtype=np.int32)        # llm_runtime.py:287-288

    batch_info = batch_scheduler.get_batch_info(batch_block_request, block_info)
    num_tokens, num_contexts, max_context_len, max_num_blocks_per_seq, num_layers, num_heads = batch_info[:6]
    prompt_lens = batch_info[6:]

    padded_len = (num_tokens + 7) // 8 * 8                                      # llm_runtime.py:300
    if device_tables is not None:
        return _prepare_on_device(batch_scheduler, device_tables, batch_block_request, block_info, num_tokens,
                                  num_contexts, max_context_len, max_num_blocks_per_seq, prompt_lens, padded_len)
    pin = torch.cuda.is_available()
    slot_mapping = torch.empty((num_tokens, num_layers, num_heads), dtype=torch.int64, pin_memory=pin)
    input_tensor = torch.empty((padded_len,), dtype=torch.int32, pin_memory=pin)
    input_positions = torch.empty((padded_len,), dtype=torch.int32, pin_memory=pin)
    context_lens = torch.empty((num_contexts,), dtype=torch.int32, pin_memory=pin)
    decoding = max_context_len > 0
    if decoding and permuted_tables:
        # Entries past a sequence's blocks are never read; zero keeps them defined.
        block_tables = torch.zeros((num_layers, num_contexts, num_heads, max_num_blocks_per_seq),
                                   dtype=torch.int32, pin_memory=pin)
        batch_scheduler.get_batch_permuted(batch_block_request, block_info, input_tensor, input_positions,
                                           context_lens, block_tables, slot_mapping)
    else:
        if decoding:
            block_tables = torch.zeros((num_tokens, max_num_blocks_per_seq, num_layers, num_heads),
                                       dtype=torch.int32, pin_memory=pin)
        else:
            block_tables = torch.empty((0, max_num_blocks_per_seq, 0, 0), dtype=torch.int32)   # llm_runtime.py:307-309
        batch_scheduler.get_batch(batch_block_request, block_info, input_tensor, input_positions,
                                  context_lens, block_tables, slot_mapping)

    preempted_reqs = batch_scheduler.get_preempt_requests()
    batch_reqs = batch_scheduler.get_batch_reqs()
    total_context_len = int(context_lens.sum()) if num_contexts else 0

    context_lens_host = context_lens if num_contexts else None      # stays as written; the copy below only reads it
    slot_mapping = slot_mapping.to(device, non_blocking=True)
    block_tables = block_tables.to(device, non_blocking=True)
    input_tensor = input_tensor.to(device, non_blocking=True).long()            # llm_runtime.py:324-325
    input_positions = input_positions.to(device, non_blocking=True).long()
    context_lens = context_lens.to(device, non_blocking=True)
    if not (decoding and permuted_tables):
        block_tables = block_tables.permute(2, 0, 3, 1).contiguous()            # llm_runtime.py:327

    input_metadata = InputMetadata(prompt_lens=prompt_lens, slot_mapping=slot_mapping, context_lens=context_lens,
                                   max_context_len=max_context_len, block_tables=block_tables,
                                   total_context_len=total_context_len, context_lens_host=context_lens_host)
    return input_tensor, input_positions, input_metadata, batch_reqs, preempted_reqs


def _prepare_on_device(sched, dt, batch_block_request, block_info, num_tokens, num_contexts, max_context_len,
                       max_num_blocks_per_seq, prompt_lens, padded_len):
    """The device_tables path of prepare_inputs: everything the step uploads is
    packed into one pinned int32 buffer
        [tokens | positions | context_lens | descriptors | allocator reply]
    and copied once."""
    n_entries = max(int(block_info[0]), 0)
    D = sched.STEP_DESC_INTS
    n_info = int(block_info.size)
    o_tok, o_pos = 0, padded_len
    o_ctx = 2 * padded_len
    o_desc = o_ctx + (num_contexts + 3) // 4 * 4
    o_info = o_desc + n_entries * D
    total = o_info + n_info
    host = dt.staging(total)
    sched.get_batch_compact(batch_block_request, block_info, host[o_tok:o_pos], host[o_pos:o_ctx],
                            host[o_ctx:o_ctx + num_contexts], host[o_desc:o_info])
    host[o_info:total] = torch.from_numpy(block_info)
    desc_host = host[o_desc:o_info].view(n_entries, D)
    max_new = int(desc_host[:, 3].max()) if n_entries else 0
    total_context_len = int(host[o_ctx:o_ctx + num_contexts].sum()) if num_contexts else 0
    # (the staging buffer is reused by the next step: the host copy is its own tensor)
    context_lens_host = host[o_ctx:o_ctx + num_contexts].clone() if num_contexts else None
    preempted_reqs = sched.get_preempt_requests()
    batch_reqs = sched.get_batch_reqs()

    dev = dt.upload(total)
    input_tensor = dev[o_tok:o_pos].long()                                       # llm_runtime.py:324-325
    input_positions = dev[o_pos:o_ctx].long()
    context_lens = dev[o_ctx:o_ctx + num_contexts]
    decoding = max_context_len > 0
    slot_mapping, block_tables = dt.build(dev[o_desc:o_info], dev[o_info:total], n_entries, max_new, num_tokens,
                                          max_num_blocks_per_seq if decoding else 0)
    input_metadata = InputMetadata(prompt_lens=prompt_lens, slot_mapping=slot_mapping, context_lens=context_lens,
                                   max_context_len=max_context_len, block_tables=block_tables,
                                   total_context_len=total_context_len, context_lens_host=context_lens_host)
    return input_tensor, input_positions, input_metadata, batch_reqs, preempted_reqs
