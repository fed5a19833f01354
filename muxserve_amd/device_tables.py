"""Device-resident mirror of the requests' block-id runs and the step-input
builder on top of it.

The reference rebuilds the whole block table and one slot per (token, layer,
head) on the host every step and uploads them
(csrc/batch_scheduler.cpp:131-169, muxserve/flexserver/llm_runtime.py:301-327).
With a DeviceBlockTables attached to a BatchScheduler a step uploads only the
token ids, positions, context lengths, the allocator's reply and 8 ints per
sequence - in one copy - and `mux_build_step_inputs` derives slot_mapping and
the step's block table on the device, bit-identical to the reference path's.
"""
from typing import Tuple

import torch

from . import _lib
from .batch_scheduler import BatchScheduler


class DeviceBlockTables:
    def __init__(self, scheduler: BatchScheduler, max_rows: int, device="cuda:0"):
        self.scheduler = scheduler
        self.device = torch.device(device)
        self.max_rows = int(max_rows)
        self.L, self.H = scheduler.num_layers, scheduler.num_heads
        self.block_size = scheduler.block_size
        self.max_blocks_per_seq = scheduler.max_blocks_per_seq
        # int32 [row][token block][layer][head]; written only by build().
        self.mirror = torch.zeros((self.max_rows, self.max_blocks_per_seq, self.L, self.H), dtype=torch.int32,
                                  device=self.device)
        self._staging = None
        self._uploaded = None
        scheduler.enable_device_rows(self.max_rows)

    def staging(self, n_ints: int) -> torch.Tensor:
        """Grow-only pinned int32 buffer the step's upload is packed into.  The
        previous step's copy out of it must have run before it is overwritten."""
        if self._uploaded is not None:
            self._uploaded.synchronize()
        if self._staging is None or self._staging.numel() < n_ints:
            self._staging = torch.empty((max(n_ints, 1 << 16),), dtype=torch.int32,
                                        pin_memory=torch.cuda.is_available())
        return self._staging

    def upload(self, n_ints: int) -> torch.Tensor:
        """One asynchronous copy of the first n_ints of the staging buffer."""
        dev = self._staging[:n_ints].to(self.device, non_blocking=True)
        if self._uploaded is None:
            self._uploaded = torch.cuda.Event()
        self._uploaded.record(torch.cuda.current_stream(self.device))
        return dev

    def build(self, desc: torch.Tensor, block_info: torch.Tensor, num_seqs: int, max_new_blocks: int,
              num_tokens: int, max_blocks_out: int, stream=None) -> Tuple[torch.Tensor, torch.Tensor]:
        """desc int32 [num_seqs, 8] and block_info int32 [n] on the device ->
        (slot_mapping int64 [num_tokens, L, H], block_tables int32
        [L, num_seqs, H, max_blocks_out] or the reference's empty prefill table)."""
        slot_mapping = torch.empty((num_tokens, self.L, self.H), dtype=torch.int64, device=self.device)
        if max_blocks_out > 0:
            block_tables = torch.empty((self.L, num_seqs, self.H, max_blocks_out), dtype=torch.int32,
                                       device=self.device)
            bt_ptr = block_tables.data_ptr()
        else:
            block_tables = torch.empty((0, 0, 0, self.max_blocks_per_seq), dtype=torch.int32, device=self.device)
            bt_ptr = None
        st = torch.cuda.current_stream(self.device).cuda_stream if stream is None else stream
        rc = _lib.attn().mux_build_step_inputs(
            self.mirror.data_ptr(), self.max_rows, self.max_blocks_per_seq, self.L, self.H, self.block_size,
            desc.data_ptr(), int(num_seqs), block_info.data_ptr(), block_info.numel(), int(max_new_blocks),
            int(num_tokens), slot_mapping.data_ptr() if num_tokens else None, bt_ptr, int(max_blocks_out), st)
        _lib.check_attn(rc, "mux_build_step_inputs")
        return slot_mapping, block_tables
