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
                   permuted_tables: bool = True
                   ) -> Tuple[torch.Tensor, torch.Tensor, InputMetadata, List[List[int]], List[int]]:
    """Returns (input_tensor int64 [T_pad], input_positions int64 [T_pad],
    input_metadata, batch_reqs, preempted_reqs) - the reference's return tuple.

    permuted_tables=True lets the builder emit the block table directly as
    [L, B, H, max_blocks] on the host (one copy to the device); False follows
    the reference literally: [T, max_blocks, L, H] on the host, then
    permute(2, 0, 3, 1).contiguous() on the device (llm_runtime.py:327).
    Both give identical tensors on the valid entries.
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

    slot_mapping = slot_mapping.to(device, non_blocking=True)
    block_tables = block_tables.to(device, non_blocking=True)
    input_tensor = input_tensor.to(device, non_blocking=True).long()            # llm_runtime.py:324-325
    input_positions = input_positions.to(device, non_blocking=True).long()
    context_lens = context_lens.to(device, non_blocking=True)
    if not (decoding and permuted_tables):
        block_tables = block_tables.permute(2, 0, 3, 1).contiguous()            # llm_runtime.py:327

    input_metadata = InputMetadata(prompt_lens=prompt_lens, slot_mapping=slot_mapping, context_lens=context_lens,
                                   max_context_len=max_context_len, block_tables=block_tables,
                                   total_context_len=total_context_len)
    return input_tensor, input_positions, input_metadata, batch_reqs, preempted_reqs
