"""BatchScheduler - per-step block-table / slot-mapping builder, same Python
surface as the reference's pybind11 module ``muxserve.batch_scheduler``
(csrc/batch_scheduler.cpp:201-212): add_request, try_batch, get_batch_info,
get_batch, release_requests, get_preempt_requests, get_prompt_info,
get_batch_reqs.  The work is done by libmuxhost.so.

get_batch() takes the caller-allocated CPU torch tensors of
muxserve/flexserver/llm_runtime.py:300-320 (int32 tokens, int32 positions,
int32 context lens, int32 block table, int64 slot mapping).  Unlike the
reference it checks dtypes, contiguity and sizes and raises instead of writing
out of bounds.
"""
import numpy as np

from . import _lib


def _i32(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.int32).reshape(-1))


def _buf(t, np_dtype, what):
    """(address, numel) of a contiguous CPU torch tensor or numpy array."""
    if isinstance(t, np.ndarray):
        if t.dtype != np_dtype or not t.flags["C_CONTIGUOUS"]:
            raise TypeError(f"{what}: expected contiguous {np.dtype(np_dtype).name} array")
        return t.ctypes.data, t.size
    import torch
    want = {np.int32: torch.int32, np.int64: torch.int64}[np_dtype]
    if t.dtype != want:
        raise TypeError(f"{what}: expected {want}, got {t.dtype}")
    if t.device.type != "cpu" or not t.is_contiguous():
        raise TypeError(f"{what}: expected a contiguous CPU tensor")
    return t.data_ptr(), t.numel()


class BatchScheduler:
    def __init__(self, num_layers: int, num_heads: int, max_seq_len: int, block_size: int):
        self._lib = _lib.host()
        self._h = self._lib.mux_sched_create(int(num_layers), int(num_heads),
                                             int(max_seq_len), int(block_size))
        if not self._h:
            raise ValueError("BatchScheduler: all four arguments must be positive")
        self.num_layers, self.num_heads = int(num_layers), int(num_heads)
        self.max_seq_len, self.block_size = int(max_seq_len), int(block_size)
        self.max_blocks_per_seq = (self.max_seq_len + self.block_size - 1) // self.block_size

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.mux_sched_destroy(h)

    def add_request(self, prompt, req_id: int, max_tokens: int) -> None:
        p = _i32(prompt)
        _lib.check_host(self._lib.mux_sched_add_request(self._h, p.ctypes.data, p.size,
                                                        int(req_id), int(max_tokens)),
                        "BatchScheduler.add_request")

    def try_batch(self, batch_request_ids, batch_last_output_tokens) -> np.ndarray:
        ids = _i32(list(batch_request_ids))
        last = _i32(list(batch_last_output_tokens))
        out = np.empty(3 * ids.size + 1, dtype=np.int32)
        _lib.check_host(self._lib.mux_sched_try_batch(self._h, ids.ctypes.data, ids.size,
                                                      last.ctypes.data, last.size, out.ctypes.data),
                        "BatchScheduler.try_batch")
        return out

    def get_batch_info(self, batch_block_request, block_info):
        req, blk = _i32(batch_block_request), _i32(block_info)
        out = np.empty(6 + req.size // 3, dtype=np.int32)
        n = _lib.check_host(self._lib.mux_sched_get_batch_info(self._h, req.ctypes.data, req.size,
                                                               blk.ctypes.data, blk.size,
                                                               out.ctypes.data, out.size),
                            "BatchScheduler.get_batch_info")
        return [int(x) for x in out[:n]]

    def get_batch(self, batch_info, block_info, token_tensor, token_position_tensor,
                  context_len_tensor, block_table_tensor, slot_mapping_tensor) -> None:
        req, blk = _i32(batch_info), _i32(block_info)
        tok, n_tok = _buf(token_tensor, np.int32, "token_tensor")
        pos, n_pos = _buf(token_position_tensor, np.int32, "token_position_tensor")
        ctx, n_ctx = _buf(context_len_tensor, np.int32, "context_len_tensor")
        bt, n_bt = _buf(block_table_tensor, np.int32, "block_table_tensor")
        slot, n_slot = _buf(slot_mapping_tensor, np.int64, "slot_mapping_tensor")
        if n_pos != n_tok:
            raise ValueError("token and position tensors must have the same length")
        _lib.check_host(self._lib.mux_sched_get_batch(self._h, req.ctypes.data, req.size,
                                                      blk.ctypes.data, blk.size,
                                                      tok, pos, n_tok, ctx, n_ctx, bt, n_bt,
                                                      slot, n_slot),
                        "BatchScheduler.get_batch")

    def get_batch_permuted(self, batch_info, block_info, token_tensor, token_position_tensor,
                           context_len_tensor, block_table_lbhm, slot_mapping_tensor) -> None:
        """Not in the reference: same as get_batch but the block table comes out
        as int32 [L, num_contexts, H, max_blocks] (max_blocks = last dim of the
        tensor passed in), i.e. already in the layout that
        block_tables.permute(2,0,3,1).contiguous() produces at
        muxserve/flexserver/llm_runtime.py:327."""
        req, blk = _i32(batch_info), _i32(block_info)
        tok, n_tok = _buf(token_tensor, np.int32, "token_tensor")
        pos, n_pos = _buf(token_position_tensor, np.int32, "token_position_tensor")
        ctx, n_ctx = _buf(context_len_tensor, np.int32, "context_len_tensor")
        bt, n_bt = _buf(block_table_lbhm, np.int32, "block_table_lbhm")
        slot, n_slot = _buf(slot_mapping_tensor, np.int64, "slot_mapping_tensor")
        if n_pos != n_tok:
            raise ValueError("token and position tensors must have the same length")
        max_blocks = int(block_table_lbhm.shape[-1]) if n_bt else 0
        _lib.check_host(self._lib.mux_sched_get_batch_permuted(self._h, req.ctypes.data, req.size,
                                                               blk.ctypes.data, blk.size,
                                                               tok, pos, n_tok, ctx, n_ctx, bt, n_bt,
                                                               max_blocks, slot, n_slot),
                        "BatchScheduler.get_batch_permuted")

    STEP_DESC_INTS = 8

    def enable_device_rows(self, max_rows: int) -> None:
        """Not in the reference: switch on the bookkeeping for a device-resident
        mirror of the requests' block-id runs (see get_batch_compact)."""
        _lib.check_host(self._lib.mux_sched_enable_device_rows(self._h, int(max_rows)),
                        "BatchScheduler.enable_device_rows")

    def get_batch_compact(self, batch_info, block_info, token_tensor, token_position_tensor,
                          context_len_tensor, desc_tensor) -> None:
        """Not in the reference: get_batch without the block table and the slot
        mapping; instead one row of STEP_DESC_INTS int32 per batch entry goes to
        desc_tensor, from which the device builds both."""
        req, blk = _i32(batch_info), _i32(block_info)
        tok, n_tok = _buf(token_tensor, np.int32, "token_tensor")
        pos, n_pos = _buf(token_position_tensor, np.int32, "token_position_tensor")
        ctx, n_ctx = _buf(context_len_tensor, np.int32, "context_len_tensor")
        desc, n_desc = _buf(desc_tensor, np.int32, "desc_tensor")
        if n_pos != n_tok:
            raise ValueError("token and position tensors must have the same length")
        _lib.check_host(self._lib.mux_sched_get_batch_compact(self._h, req.ctypes.data, req.size,
                                                              blk.ctypes.data, blk.size,
                                                              tok, pos, n_tok, ctx, n_ctx, desc, n_desc),
                        "BatchScheduler.get_batch_compact")

    def release_requests(self, request_ids) -> None:
        ids = _i32(list(request_ids))
        _lib.check_host(self._lib.mux_sched_release_requests(self._h, ids.ctypes.data, ids.size),
                        "BatchScheduler.release_requests")

    def _vec(self, fn):
        n = fn(self._h, None, 0)
        out = np.empty(max(n, 1), dtype=np.int32)
        fn(self._h, out.ctypes.data, n)
        return [int(x) for x in out[:n]]

    def get_preempt_requests(self):
        return self._vec(self._lib.mux_sched_get_preempt_requests)

    def get_prompt_info(self):
        return self._vec(self._lib.mux_sched_get_prompt_info)

    def get_batch_reqs(self):
        flat = self._vec(self._lib.mux_sched_get_batch_reqs)
        return [[flat[i], flat[i + 1]] for i in range(0, len(flat), 2)]

    # -- introspection for tests (no reference counterpart) -------------------
    def request_state(self, req_id: int) -> dict:
        out = np.empty(6, dtype=np.int32)
        _lib.check_host(self._lib.mux_sched_request_state(self._h, int(req_id), out.ctypes.data),
                        "BatchScheduler.request_state")
        keys = ("context_len", "num_physical_blocks", "logical_block_idx",
                "logical_block_offset", "prompt_len", "num_outputs")
        return dict(zip(keys, (int(x) for x in out)))

    def num_requests(self) -> int:
        return int(self._lib.mux_sched_num_requests(self._h))
