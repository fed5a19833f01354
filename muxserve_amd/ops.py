"""Tensor-level wrappers over the C ABI of libmuxattn.so.

torch is used here for device memory and streams only: every function takes
CUDA(HIP) tensors, checks what the C ABI cannot (device, dtype, contiguity of
the innermost dimension), and passes raw pointers plus the current stream.
There is no fallback: without the library, or with CPU tensors, these raise.
"""
import ctypes
from dataclasses import dataclass
from typing import List, Optional

import torch

from . import _lib

HEAD_SIZE = 128   # muxserve/flexstore/manager.py:337


def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.float16:
        return _lib.DTYPE_F16
    if t.dtype == torch.bfloat16:
        return _lib.DTYPE_BF16
    raise TypeError(f"expected float16 or bfloat16, got {t.dtype}")


def _need_cuda(*tensors):
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError("muxserve_amd.ops: tensors must live on the GPU (no CPU path)")


def _stream_ptr(stream=None) -> int:
    if stream is None:
        return torch.cuda.current_stream().cuda_stream
    if isinstance(stream, int):
        return stream
    return stream.cuda_stream


def _rows(t: torch.Tensor, what: str) -> int:
    """Row stride (elements) of a 2-D [rows, width] tensor with unit inner stride."""
    if t.dim() != 2 or t.stride(1) != 1:
        raise ValueError(f"{what}: expected [rows, width] with contiguous rows")
    return t.stride(0)


def pool_block_size(k_pool: torch.Tensor) -> int:
    """K pool is [N, D/8, block_size, 8] (muxserve/flexstore/manager.py:456-462)."""
    if k_pool.dim() != 4 or k_pool.shape[1] * k_pool.shape[3] != HEAD_SIZE or k_pool.shape[3] != 8:
        raise ValueError(f"k_pool: expected [N, 16, block_size, 8], got {tuple(k_pool.shape)}")
    return int(k_pool.shape[2])


def _check_pools(k_pool, v_pool):
    bs = pool_block_size(k_pool)
    if tuple(v_pool.shape) != (k_pool.shape[0], HEAD_SIZE, bs):
        raise ValueError(f"v_pool: expected {(k_pool.shape[0], HEAD_SIZE, bs)}, got {tuple(v_pool.shape)}")
    if not (k_pool.is_contiguous() and v_pool.is_contiguous()):
        raise ValueError("pools must be contiguous")
    if k_pool.dtype != v_pool.dtype:
        raise TypeError("k_pool and v_pool dtypes differ")
    return bs


def reshape_and_cache(k: torch.Tensor, v: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                      slot_mapping: torch.Tensor, layer: int = 0, num_tokens: Optional[int] = None,
                      stream=None) -> None:
    """Scatter k, v [T_pad, Hkv*128] into the pool through slot_mapping
    int64 [T, L, Hkv] (slice `layer`).  Rows >= T of k/v are padding
    (muxserve/flexserver/llm_runtime.py:300) and are not read."""
    _need_cuda(k, v, k_pool, v_pool, slot_mapping)
    bs = _check_pools(k_pool, v_pool)
    if slot_mapping.dtype != torch.int64 or slot_mapping.dim() != 3 or not slot_mapping.is_contiguous():
        raise ValueError("slot_mapping: expected contiguous int64 [T, L, Hkv]")
    T, L, H = slot_mapping.shape
    if num_tokens is not None:
        T = min(T, int(num_tokens))
    stride = _rows(k, "k")
    if _rows(v, "v") != stride or k.shape != v.shape or k.dtype != v.dtype or k.dtype != k_pool.dtype:
        raise ValueError("k and v must have the same shape, strides and dtype as each other and the pool's dtype")
    if k.shape[0] < T or k.shape[1] != H * HEAD_SIZE:
        raise ValueError(f"k: expected [>={T}, {H * HEAD_SIZE}], got {tuple(k.shape)}")
    rc = _lib.attn().mux_reshape_and_cache(
        k.data_ptr(), v.data_ptr(), stride, k_pool.data_ptr(), v_pool.data_ptr(), k_pool.shape[0],
        slot_mapping.data_ptr(), int(layer), L, T, H, HEAD_SIZE, bs, _dtype_code(k), _stream_ptr(stream))
    _lib.check_attn(rc, "mux_reshape_and_cache")


@dataclass
class DecodeCall:
    """One model's decode step for one layer (an element of a fused launch)."""
    out: torch.Tensor             # [>=B, Hq*128]
    q: torch.Tensor               # [>=B, Hq*128] (may be a column slice of qkv)
    block_tables: torch.Tensor    # int32 [L, B, Hkv, max_blocks]
    context_lens: torch.Tensor    # int32 [B]
    max_context_len: int
    scale: float
    layer: int = 0
    total_context_len: int = 0    # host-side bound on sum(context_lens); 0 = unknown
    # Optional host copy of context_lens (CPU int32 tensor [B], equal to the device
    # tensor): small batches are then enumerated on the host and the launch does
    # not read the device tensor.  Leave None under HIP graph capture.
    context_lens_host: Optional[torch.Tensor] = None

    def to_item(self) -> _lib.MuxDecodeItem:
        bt, cl = self.block_tables, self.context_lens
        _need_cuda(self.out, self.q, bt, cl)
        if bt.dtype != torch.int32 or bt.dim() != 4 or not bt.is_contiguous():
            raise ValueError("block_tables: expected contiguous int32 [L, B, Hkv, max_blocks]")
        if cl.dtype != torch.int32 or cl.dim() != 1 or not cl.is_contiguous():
            raise ValueError("context_lens: expected contiguous int32 [B]")
        L, B, Hkv, max_blocks = bt.shape
        if cl.shape[0] != B:
            raise ValueError("context_lens and block_tables disagree on the number of sequences")
        if self.q.shape[1] % HEAD_SIZE or self.q.shape[0] < B or self.out.shape != self.q.shape:
            raise ValueError("q/out: expected [>=B, Hq*128] of equal shape")
        if self.q.dtype != self.out.dtype:
            raise TypeError("q and out dtypes differ")
        it = _lib.MuxDecodeItem()
        it.out, it.q = self.out.data_ptr(), self.q.data_ptr()
        it.out_row_stride, it.q_row_stride = _rows(self.out, "out"), _rows(self.q, "q")
        it.block_tables, it.context_lens = bt.data_ptr(), cl.data_ptr()
        it.layer, it.num_layers, it.num_seqs = int(self.layer), L, B
        it.num_q_heads, it.num_kv_heads = self.q.shape[1] // HEAD_SIZE, Hkv
        it.max_blocks, it.max_context_len = max_blocks, int(self.max_context_len)
        it.scale = float(self.scale)
        it.total_context_len = int(self.total_context_len)
        ch = self.context_lens_host
        if ch is not None:
            if ch.is_cuda or ch.dtype != torch.int32 or ch.dim() != 1 or ch.shape[0] != B or not ch.is_contiguous():
                raise ValueError("context_lens_host: expected a contiguous CPU int32 [B] tensor")
            it.context_lens_host = ch.data_ptr()      # self keeps the tensor alive over the call
        return it


_workspaces = {}


def _scratch(cache: dict, nbytes: int, device, stream_ptr: int, floor: int) -> Optional[torch.Tensor]:
    """Grow-only zero-filled scratch, one per (device, stream the launches that
    use it go to).  Lifetime rules, because that stream need not be torch's
    current one (a CU-masked stream passed as ``stream=``):
      * a new buffer is allocated and zero-filled under the device's DEFAULT
        stream - its memory then belongs to the allocator's pool of a stream
        that is never destroyed - and waited for once before its first use;
      * a buffer that has become too small is only dropped after the stream it
        is keyed to has been synchronised: launches there may still be writing
        partial results into it, and torch would hand the block out again."""
    if nbytes == 0:
        return None
    key = (device, stream_ptr)
    ws = cache.get(key)
    if ws is None or ws.numel() < nbytes:
        if ws is not None:
            (torch.cuda.ExternalStream(stream_ptr, device=device) if stream_ptr
             else torch.cuda.default_stream(device)).synchronize()
        default = torch.cuda.default_stream(device)
        with torch.cuda.stream(default):
            ws = torch.zeros(max(nbytes, floor), dtype=torch.uint8, device=device)
        default.synchronize()
        cache[key] = ws
    return ws


def _workspace(nbytes: int, device, stream_ptr: int) -> Optional[torch.Tensor]:
    """Scratch for split partials.  Born zeroed: it starts with arrival counters
    that every launch leaves at zero."""
    return _scratch(_workspaces, nbytes, device, stream_ptr, 1 << 20)


def multi_decode(calls: List[DecodeCall], k_pool: torch.Tensor, v_pool: torch.Tensor,
                 partition_size: int = 0, workspace: Optional[torch.Tensor] = None, stream=None) -> None:
    """Paged decode attention for several colocated models in one launch."""
    if not 1 <= len(calls) <= _lib.MUXA_MAX_DECODE_ITEMS:
        raise ValueError(f"1..{_lib.MUXA_MAX_DECODE_ITEMS} models per launch")
    _need_cuda(k_pool, v_pool)
    bs = _check_pools(k_pool, v_pool)
    items = (_lib.MuxDecodeItem * len(calls))(*[c.to_item() for c in calls])
    for c in calls:
        if c.q.dtype != k_pool.dtype:
            raise TypeError("q dtype must equal the pool dtype")
    lib = _lib.attn()
    need = lib.mux_paged_decode_workspace_bytes(ctypes.addressof(items), len(calls), int(partition_size))
    sp = _stream_ptr(stream)
    ws = workspace if workspace is not None else _workspace(need, k_pool.device, sp)
    ws_ptr, ws_bytes = (ws.data_ptr(), ws.numel() * ws.element_size()) if ws is not None else (None, 0)
    rc = lib.mux_multi_decode(ctypes.addressof(items), len(calls), k_pool.data_ptr(), v_pool.data_ptr(),
                              k_pool.shape[0], HEAD_SIZE, bs, _dtype_code(k_pool), int(partition_size),
                              ws_ptr, ws_bytes, sp)
    _lib.check_attn(rc, "mux_multi_decode")


class DecodeLaunch:
    """A fused decode launch prepared once and issued many times.

    The serving loop runs the same step shape for every layer of a model, and a
    benchmark loop repeats the same batch: the tensor checks, the descriptor
    array and the workspace are made here, once, and ``launch()`` is a single
    call into the C ABI.  The tensors of `calls` (and the host copies of the
    context lengths) must stay alive and unchanged in shape while the object is
    used; their contents may change between launches."""

    def __init__(self, calls: List[DecodeCall], k_pool: torch.Tensor, v_pool: torch.Tensor,
                 partition_size: int = 0, workspace: Optional[torch.Tensor] = None, stream=None):
        if not 1 <= len(calls) <= _lib.MUXA_MAX_DECODE_ITEMS:
            raise ValueError(f"1..{_lib.MUXA_MAX_DECODE_ITEMS} models per launch")
        _need_cuda(k_pool, v_pool)
        bs = _check_pools(k_pool, v_pool)
        for c in calls:
            if c.q.dtype != k_pool.dtype:
                raise TypeError("q dtype must equal the pool dtype")
        self.calls = list(calls)                  # keeps the tensors alive
        self.pools = (k_pool, v_pool)
        self.items = (_lib.MuxDecodeItem * len(calls))(*[c.to_item() for c in calls])
        lib = _lib.attn()
        need = lib.mux_paged_decode_workspace_bytes(ctypes.addressof(self.items), len(calls), int(partition_size))
        self.stream_ptr = _stream_ptr(stream)
        self.workspace = workspace if workspace is not None else _workspace(need, k_pool.device, self.stream_ptr)
        ws = self.workspace
        ws_ptr, ws_bytes = (ws.data_ptr(), ws.numel() * ws.element_size()) if ws is not None else (None, 0)
        # (sequence, unit) pairs enumerated on the host; 0: the units are enumerated on the device
        self.host_pairs = int(lib.mux_paged_decode_host_pairs(ctypes.addressof(self.items), len(calls),
                                                              int(partition_size)))
        self._fn = lib.mux_multi_decode
        self._args = (ctypes.addressof(self.items), len(calls), k_pool.data_ptr(), v_pool.data_ptr(),
                      k_pool.shape[0], HEAD_SIZE, bs, _dtype_code(k_pool), int(partition_size), ws_ptr, ws_bytes,
                      self.stream_ptr)

    def launch(self) -> None:
        rc = self._fn(*self._args)
        if rc != 0:
            _lib.check_attn(rc, "mux_multi_decode")

    __call__ = launch


def multi_decode_noalloc(calls: List[DecodeCall], k_pool: torch.Tensor, v_pool: torch.Tensor,
                         partition_size: int = 0, stream=None) -> None:
    """multi_decode through the entry point that allocates nothing: scratch is
    the library's static per-GPU array (a fixed 32 MiB; larger needs raise).
    Calls that overlap in time on one GPU race on that array."""
    if not 1 <= len(calls) <= _lib.MUXA_MAX_DECODE_ITEMS:
        raise ValueError(f"1..{_lib.MUXA_MAX_DECODE_ITEMS} models per launch")
    _need_cuda(k_pool, v_pool)
    bs = _check_pools(k_pool, v_pool)
    items = (_lib.MuxDecodeItem * len(calls))(*[c.to_item() for c in calls])
    for c in calls:
        if c.q.dtype != k_pool.dtype:
            raise TypeError("q dtype must equal the pool dtype")
    rc = _lib.attn().mux_multi_decode_noalloc(ctypes.addressof(items), len(calls), k_pool.data_ptr(),
                                              v_pool.data_ptr(), k_pool.shape[0], HEAD_SIZE, bs,
                                              _dtype_code(k_pool), int(partition_size), _stream_ptr(stream))
    _lib.check_attn(rc, "mux_multi_decode_noalloc")


def paged_decode(out, q, k_pool, v_pool, block_tables, context_lens, max_context_len, scale,
                 layer: int = 0, partition_size: int = 0, workspace=None, stream=None,
                 total_context_len: int = 0, context_lens_host: Optional[torch.Tensor] = None) -> None:
    multi_decode([DecodeCall(out, q, block_tables, context_lens, max_context_len, scale, layer,
                             total_context_len, context_lens_host)],
                 k_pool, v_pool, partition_size, workspace, stream)


def prefill_causal(out, q, k, v, cu_seqlens: torch.Tensor, max_prompt_len: int, scale: float,
                   num_kv_heads: int, stream=None, prompt_order: Optional[torch.Tensor] = None,
                   prompt_lens=None) -> None:
    """Causal attention over packed prompts; cu_seqlens int32 [P+1] on the device.
    prompt_lens: optional host-side lengths (a sequence of P ints): the launch
    then holds only the query tiles that exist, heaviest first.  prompt_order:
    optional int32 [P] on the device, the prompts longest first, used when the
    lengths are not given.  Scheduling only; results are the same."""
    _need_cuda(out, q, k, v, cu_seqlens)
    order_ptr = None
    if prompt_order is not None:
        _need_cuda(prompt_order)
        if prompt_order.dtype != torch.int32 or prompt_order.dim() != 1 or not prompt_order.is_contiguous() \
                or prompt_order.shape[0] != cu_seqlens.shape[0] - 1:
            raise ValueError("prompt_order: expected contiguous int32 [P]")
        order_ptr = prompt_order.data_ptr()
    if cu_seqlens.dtype != torch.int32 or cu_seqlens.dim() != 1 or not cu_seqlens.is_contiguous():
        raise ValueError("cu_seqlens: expected contiguous int32 [P+1]")
    if q.shape[1] % HEAD_SIZE or k.shape[1] != num_kv_heads * HEAD_SIZE or k.shape != v.shape:
        raise ValueError("q [T, Hq*128], k/v [T, Hkv*128] expected")
    if not (q.dtype == k.dtype == v.dtype == out.dtype):
        raise TypeError("q, k, v, out dtypes differ")
    kv_stride = _rows(k, "k")
    if _rows(v, "v") != kv_stride:
        raise ValueError("k and v row strides differ")
    lens_arg = None
    if prompt_lens is not None:
        if len(prompt_lens) != cu_seqlens.shape[0] - 1:
            raise ValueError("prompt_lens: expected one length per prompt")
        lens_arg = prompt_lens if isinstance(prompt_lens, ctypes.Array) else \
            (ctypes.c_int32 * len(prompt_lens))(*[int(x) for x in prompt_lens])
    rc = _lib.attn().mux_prefill_causal(
        out.data_ptr(), _rows(out, "out"), q.data_ptr(), _rows(q, "q"), k.data_ptr(), v.data_ptr(), kv_stride,
        cu_seqlens.data_ptr(), order_ptr, lens_arg, cu_seqlens.shape[0] - 1, int(max_prompt_len), q.shape[1] // HEAD_SIZE,
        int(num_kv_heads), HEAD_SIZE, float(scale), _dtype_code(q), _stream_ptr(stream))
    _lib.check_attn(rc, "mux_prefill_causal")


@dataclass
class PrefillCall:
    """One model's prompts of a prefill step (an element of a fused launch)."""
    out: torch.Tensor             # [>=T, Hq*128]
    q: torch.Tensor               # [>=T, Hq*128]
    k: torch.Tensor               # [>=T, Hkv*128]
    v: torch.Tensor
    cu_seqlens: torch.Tensor      # int32 [P+1], device
    prompt_lens: List[int]        # host-side lengths
    scale: float
    num_kv_heads: int

    def to_item(self) -> _lib.MuxPrefillItem:
        out, q, k, v, cu = self.out, self.q, self.k, self.v, self.cu_seqlens
        _need_cuda(out, q, k, v, cu)
        if cu.dtype != torch.int32 or cu.dim() != 1 or not cu.is_contiguous() or cu.shape[0] != len(self.prompt_lens) + 1:
            raise ValueError("cu_seqlens: expected contiguous int32 [P+1] for P host-side prompt lengths")
        if q.shape[1] % HEAD_SIZE or k.shape[1] != self.num_kv_heads * HEAD_SIZE or k.shape != v.shape:
            raise ValueError("q [T, Hq*128], k/v [T, Hkv*128] expected")
        if not (q.dtype == k.dtype == v.dtype == out.dtype):
            raise TypeError("q, k, v, out dtypes differ")
        kv_stride = _rows(k, "k")
        if _rows(v, "v") != kv_stride:
            raise ValueError("k and v row strides differ")
        self._lens = (ctypes.c_int32 * len(self.prompt_lens))(*[int(x) for x in self.prompt_lens])   # kept alive by self
        it = _lib.MuxPrefillItem()
        it.out, it.out_row_stride, it.q, it.q_row_stride = out.data_ptr(), _rows(out, "out"), q.data_ptr(), _rows(q, "q")
        it.k, it.v, it.kv_row_stride = k.data_ptr(), v.data_ptr(), kv_stride
        it.cu_seqlens, it.prompt_lens_host = cu.data_ptr(), ctypes.addressof(self._lens)
        it.num_prompts, it.max_prompt_len = len(self.prompt_lens), max([int(x) for x in self.prompt_lens], default=0)
        it.num_q_heads, it.num_kv_heads, it.scale = q.shape[1] // HEAD_SIZE, int(self.num_kv_heads), float(self.scale)
        return it


def multi_prefill_causal(calls: List[PrefillCall], stream=None) -> None:
    """Causal prefill attention of several colocated models' prompts in one launch
    (the heaviest query tiles of all models first); bit-identical to one
    prefill_causal call per model."""
    if not 1 <= len(calls) <= _lib.MUXA_MAX_DECODE_ITEMS:
        raise ValueError(f"1..{_lib.MUXA_MAX_DECODE_ITEMS} models per launch")
    if len({c.q.dtype for c in calls}) != 1:
        raise TypeError("the models of a fused launch must share a dtype")
    items = (_lib.MuxPrefillItem * len(calls))(*[c.to_item() for c in calls])
    rc = _lib.attn().mux_multi_prefill_causal(ctypes.addressof(items), len(calls), HEAD_SIZE, _dtype_code(calls[0].q),
                                              _stream_ptr(stream))
    _lib.check_attn(rc, "mux_multi_prefill_causal")


def rotary_neox(positions: torch.Tensor, q: torch.Tensor, k: torch.Tensor, cos_sin: torch.Tensor,
                num_tokens: Optional[int] = None, stream=None) -> None:
    """NeoX rotary embedding in place on q [T_pad, Hq*128] and k [T_pad, Hkv*128];
    positions int64 [T_pad]; cos_sin fp32 [max_position, rotary_dim] on the device."""
    _need_cuda(positions, q, k, cos_sin)
    if positions.dtype != torch.int64 or positions.dim() != 1 or not positions.is_contiguous():
        raise ValueError("positions: expected contiguous int64 [T]")
    if cos_sin.dtype != torch.float32 or cos_sin.dim() != 2 or not cos_sin.is_contiguous():
        raise ValueError("cos_sin: expected contiguous float32 [max_position, rotary_dim]")
    if q.dtype != k.dtype or q.shape[1] % HEAD_SIZE or k.shape[1] % HEAD_SIZE:
        raise ValueError("q [T, Hq*128], k [T, Hkv*128] of one dtype expected")
    T = positions.shape[0] if num_tokens is None else int(num_tokens)
    if min(q.shape[0], k.shape[0], positions.shape[0]) < T:
        raise ValueError("fewer rows than tokens")
    rc = _lib.attn().mux_rotary_neox(positions.data_ptr(), q.data_ptr(), _rows(q, "q"), k.data_ptr(), _rows(k, "k"),
                                     cos_sin.data_ptr(), cos_sin.shape[0], cos_sin.shape[1], T,
                                     q.shape[1] // HEAD_SIZE, k.shape[1] // HEAD_SIZE, HEAD_SIZE, _dtype_code(q),
                                     _stream_ptr(stream))
    _lib.check_attn(rc, "mux_rotary_neox")


def rope_reshape_and_cache(positions: torch.Tensor, q: Optional[torch.Tensor], k: torch.Tensor, v: torch.Tensor,
                           cos_sin: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                           slot_mapping: torch.Tensor, layer: int = 0, num_tokens: Optional[int] = None,
                           stream=None) -> None:
    """rotary_neox (rotary_dim = 128) on q and k in place, then reshape_and_cache
    of the rotated k and v, in one launch.  Same results as the two calls."""
    _need_cuda(positions, k, v, cos_sin, k_pool, v_pool, slot_mapping)
    bs = _check_pools(k_pool, v_pool)
    if positions.dtype != torch.int64 or positions.dim() != 1 or not positions.is_contiguous():
        raise ValueError("positions: expected contiguous int64 [T]")
    if cos_sin.dtype != torch.float32 or cos_sin.dim() != 2 or not cos_sin.is_contiguous():
        raise ValueError("cos_sin: expected contiguous float32 [max_position, rotary_dim]")
    if slot_mapping.dtype != torch.int64 or slot_mapping.dim() != 3 or not slot_mapping.is_contiguous():
        raise ValueError("slot_mapping: expected contiguous int64 [T, L, Hkv]")
    T, L, H = slot_mapping.shape
    if num_tokens is not None:
        T = min(T, int(num_tokens))
    stride = _rows(k, "k")
    if _rows(v, "v") != stride or k.shape != v.shape or k.dtype != v.dtype or k.dtype != k_pool.dtype:
        raise ValueError("k and v must have the same shape, strides and dtype as each other and the pool's dtype")
    if k.shape[0] < T or positions.shape[0] < T or k.shape[1] != H * HEAD_SIZE:
        raise ValueError(f"k: expected [>={T}, {H * HEAD_SIZE}], got {tuple(k.shape)}")
    q_ptr, q_stride, hq = None, 0, 0
    if q is not None:
        _need_cuda(q)
        if q.dtype != k.dtype or q.shape[1] % HEAD_SIZE or q.shape[0] < T:
            raise ValueError("q [>=T, Hq*128] of the dtype of k expected")
        q_ptr, q_stride, hq = q.data_ptr(), _rows(q, "q"), q.shape[1] // HEAD_SIZE
    rc = _lib.attn().mux_rope_reshape_and_cache(
        positions.data_ptr(), q_ptr, q_stride, k.data_ptr(), v.data_ptr(), stride, cos_sin.data_ptr(),
        cos_sin.shape[0], cos_sin.shape[1], k_pool.data_ptr(), v_pool.data_ptr(), k_pool.shape[0],
        slot_mapping.data_ptr(), int(layer), L, T, hq, H, HEAD_SIZE, bs, _dtype_code(k), _stream_ptr(stream))
    _lib.check_attn(rc, "mux_rope_reshape_and_cache")


@dataclass
class CacheWriteCall:
    """One model's cache write of a step (an element of a fused launch).  With
    positions and cos_sin the write rotates q and k in place first (rotary_dim
    = 128); without, it is the plain scatter."""
    k: torch.Tensor                       # [>=T, Hkv*128]
    v: torch.Tensor
    slot_mapping: torch.Tensor            # int64 [T, L, Hkv]
    layer: int = 0
    positions: Optional[torch.Tensor] = None     # int64 [>=T]
    cos_sin: Optional[torch.Tensor] = None       # float32 [max_position, 128]
    q: Optional[torch.Tensor] = None             # [>=T, Hq*128]
    num_tokens: Optional[int] = None

    def to_item(self, pool_dtype) -> _lib.MuxCacheWriteItem:
        k, v, sm = self.k, self.v, self.slot_mapping
        _need_cuda(k, v, sm)
        if sm.dtype != torch.int64 or sm.dim() != 3 or not sm.is_contiguous():
            raise ValueError("slot_mapping: expected contiguous int64 [T, L, Hkv]")
        T, L, H = sm.shape
        if self.num_tokens is not None:
            T = min(T, int(self.num_tokens))
        stride = _rows(k, "k")
        if _rows(v, "v") != stride or k.shape != v.shape or k.dtype != v.dtype or k.dtype != pool_dtype:
            raise ValueError("k and v must have the same shape, strides and dtype as each other and the pool's dtype")
        if k.shape[0] < T or k.shape[1] != H * HEAD_SIZE:
            raise ValueError(f"k: expected [>={T}, {H * HEAD_SIZE}], got {tuple(k.shape)}")
        it = _lib.MuxCacheWriteItem()
        it.k, it.v, it.kv_row_stride = k.data_ptr(), v.data_ptr(), stride
        it.slot_mapping, it.layer, it.num_layers, it.num_tokens, it.num_kv_heads = sm.data_ptr(), int(self.layer), L, T, H
        if self.positions is not None:
            pos, cs = self.positions, self.cos_sin
            if cs is None:
                raise ValueError("positions without cos_sin")
            _need_cuda(pos, cs)
            if pos.dtype != torch.int64 or pos.dim() != 1 or not pos.is_contiguous() or pos.shape[0] < T:
                raise ValueError("positions: expected contiguous int64 [>=T]")
            if cs.dtype != torch.float32 or cs.dim() != 2 or not cs.is_contiguous():
                raise ValueError("cos_sin: expected contiguous float32 [max_position, rotary_dim]")
            it.positions, it.cos_sin = pos.data_ptr(), cs.data_ptr()
            it.max_position, it.rotary_dim = cs.shape[0], cs.shape[1]
            if self.q is not None:
                q = self.q
                _need_cuda(q)
                if q.dtype != k.dtype or q.shape[1] % HEAD_SIZE or q.shape[0] < T:
                    raise ValueError("q [>=T, Hq*128] of the dtype of k expected")
                it.q, it.q_row_stride, it.num_q_heads = q.data_ptr(), _rows(q, "q"), q.shape[1] // HEAD_SIZE
        return it


def cache_write_items(calls: List[CacheWriteCall], pool_dtype):
    """The checked descriptor array of a fused cache write.  A loop that issues
    the same write again and again (same tensors) may build it once and pass it
    to multi_reshape_and_cache in place of the calls; the tensors must stay alive."""
    return (_lib.MuxCacheWriteItem * len(calls))(*[c.to_item(pool_dtype) for c in calls])


def multi_reshape_and_cache(calls, k_pool: torch.Tensor, v_pool: torch.Tensor, stream=None) -> None:
    """The cache writes (fused with the rotary embedding when the calls carry
    positions) of several colocated models' step in one launch; bit-identical
    to one reshape_and_cache / rope_reshape_and_cache call per model.  `calls`:
    a list of CacheWriteCall or the array cache_write_items made from one."""
    if not 1 <= len(calls) <= _lib.MUXA_MAX_DECODE_ITEMS:
        raise ValueError(f"1..{_lib.MUXA_MAX_DECODE_ITEMS} models per launch")
    _need_cuda(k_pool, v_pool)
    bs = _check_pools(k_pool, v_pool)
    items = calls if isinstance(calls, ctypes.Array) else cache_write_items(calls, k_pool.dtype)
    rc = _lib.attn().mux_multi_rope_reshape_and_cache(ctypes.addressof(items), len(calls), k_pool.data_ptr(),
                                                      v_pool.data_ptr(), k_pool.shape[0], HEAD_SIZE, bs,
                                                      _dtype_code(k_pool), _stream_ptr(stream))
    _lib.check_attn(rc, "mux_multi_rope_reshape_and_cache")


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: Optional[torch.Tensor] = None,
             num_tokens: Optional[int] = None, stream=None) -> torch.Tensor:
    """out[t] = T(x[t] * rsqrt(mean(x[t]^2) + eps)) * weight for x [T, hidden]."""
    _need_cuda(x, weight)
    if out is None:
        out = torch.empty_like(x)
    _need_cuda(out)
    if weight.dim() != 1 or weight.shape[0] != x.shape[1] or weight.dtype != x.dtype or not weight.is_contiguous():
        raise ValueError("weight: expected contiguous [hidden] of the dtype of x")
    if out.shape != x.shape or out.dtype != x.dtype:
        raise ValueError("out: expected the shape and dtype of x")
    T = x.shape[0] if num_tokens is None else min(int(num_tokens), x.shape[0])
    rc = _lib.attn().mux_rms_norm(out.data_ptr(), _rows(out, "out"), x.data_ptr(), _rows(x, "x"), weight.data_ptr(),
                                  float(eps), T, x.shape[1], _dtype_code(x), _stream_ptr(stream))
    _lib.check_attn(rc, "mux_rms_norm")
    return out


def silu_and_mul(x: torch.Tensor, out: Optional[torch.Tensor] = None, num_tokens: Optional[int] = None,
                 stream=None) -> torch.Tensor:
    """x [T, 2 d] = [gate | up] -> out [T, d] = silu(gate) * up."""
    _need_cuda(x)
    if x.dim() != 2 or x.shape[1] % 2:
        raise ValueError("x: expected [T, 2 d]")
    d = x.shape[1] // 2
    if out is None:
        out = torch.empty((x.shape[0], d), dtype=x.dtype, device=x.device)
    _need_cuda(out)
    if tuple(out.shape) != (x.shape[0], d) or out.dtype != x.dtype:
        raise ValueError("out: expected [T, d] of the dtype of x")
    T = x.shape[0] if num_tokens is None else min(int(num_tokens), x.shape[0])
    rc = _lib.attn().mux_silu_and_mul(out.data_ptr(), _rows(out, "out"), x.data_ptr(), _rows(x, "x"), T, d,
                                      _dtype_code(x), _stream_ptr(stream))
    _lib.check_attn(rc, "mux_silu_and_mul")
    return out


_sample_workspaces = {}


def greedy_sample(embedding: torch.Tensor, hidden_states: torch.Tensor, vocab_size: int, num_rows: int,
                  row_index: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
                  workspace: Optional[torch.Tensor] = None, stream=None) -> torch.Tensor:
    """int64 [num_rows] on the device: argmax over v < vocab_size of
    hidden_states[row] . embedding[v], row = row_index[r] (int32, device) or r.
    A caller's own workspace must be zeroed once before its first use; every
    call leaves it zeroed."""
    _need_cuda(embedding, hidden_states)
    if embedding.dim() != 2 or hidden_states.dim() != 2 or embedding.shape[1] != hidden_states.shape[1]:
        raise ValueError("embedding [V, hidden] and hidden_states [T, hidden] expected")
    if embedding.dtype != hidden_states.dtype:
        raise TypeError("embedding and hidden_states dtypes differ")
    num_rows = int(num_rows)
    ri_ptr = None
    if row_index is not None:
        _need_cuda(row_index)
        if row_index.dtype != torch.int32 or row_index.dim() != 1 or not row_index.is_contiguous() \
                or row_index.shape[0] < num_rows:
            raise ValueError("row_index: expected contiguous int32 [>= num_rows]")
        ri_ptr = row_index.data_ptr()
    elif hidden_states.shape[0] < num_rows:
        raise ValueError("fewer rows of hidden states than sampled rows")
    if out is None:
        out = torch.empty((num_rows,), dtype=torch.int64, device=hidden_states.device)
    if out.dtype != torch.int64 or out.dim() != 1 or out.shape[0] < num_rows or not out.is_contiguous():
        raise ValueError("out: expected contiguous int64 [>= num_rows]")
    lib = _lib.attn()
    need = lib.mux_greedy_sample_workspace_bytes(int(vocab_size))
    sp = _stream_ptr(stream)
    if workspace is None:
        workspace = _scratch(_sample_workspaces, need, hidden_states.device, sp, 1)      # born zeroed
    rc = lib.mux_greedy_sample(out.data_ptr(), hidden_states.data_ptr(), _rows(hidden_states, "hidden_states"),
                               hidden_states.shape[0], ri_ptr, num_rows, embedding.data_ptr(),
                               _rows(embedding, "embedding"), embedding.shape[0],
                               int(vocab_size), hidden_states.shape[1], _dtype_code(hidden_states),
                               workspace.data_ptr(), workspace.numel(), sp)
    _lib.check_attn(rc, "mux_greedy_sample")
    return out[:num_rows]


class CUMaskedStream:
    """A HIP stream restricted to a share of the GPU's compute units (the
    replacement for a per-process MPS percentage).  Usable wherever a stream is
    accepted: ``with torch.cuda.stream(s.torch_stream): ...`` or ``stream=s``."""

    def __init__(self, lo_percent: Optional[int] = None, hi_percent: Optional[int] = None, parts=None):
        """Either a percent range [lo_percent, hi_percent) of the compute-unit
        mask, or `parts`: the tenths of the GPU a job holds (ids 0..9 in any
        combination, as muxserve_amd.cu_resource.CUResource hands them out)."""
        import ctypes as _c
        handle = _c.c_void_p()
        ncu = _c.c_int32()
        if parts is not None:
            if lo_percent is not None or hi_percent is not None:
                raise ValueError("give a percent range or a set of parts, not both")
            from .cu_resource import part_bits
            self.part_mask = part_bits(parts)
            rc = _lib.attn().mux_stream_create_cu_parts(_c.byref(handle), self.part_mask, _c.byref(ncu))
            _lib.check_attn(rc, "mux_stream_create_cu_parts")
            self.lo_percent = self.hi_percent = None
        else:
            rc = _lib.attn().mux_stream_create_cu_range(_c.byref(handle), int(lo_percent), int(hi_percent),
                                                        _c.byref(ncu))
            _lib.check_attn(rc, "mux_stream_create_cu_range")
            self.lo_percent, self.hi_percent = int(lo_percent), int(hi_percent)
            self.part_mask = None
        self.cuda_stream = handle.value
        self.num_cus = ncu.value
        self.torch_stream = torch.cuda.ExternalStream(self.cuda_stream)

    def synchronize(self):
        self.torch_stream.synchronize()

    def close(self):
        """Destroys the stream.  Scratch tensors this module allocated while the
        stream was current are dropped first: they must not outlive the stream
        they are tied to (nor be found again under a recycled handle value)."""
        if self.cuda_stream:
            self.torch_stream.synchronize()
            for cache in (_workspaces, _sample_workspaces):
                for key in [k for k in cache if k[1] == self.cuda_stream]:
                    del cache[key]
            _lib.attn().mux_stream_destroy(self.cuda_stream)
            self.cuda_stream = None


def device_cu_info():
    import ctypes as _c
    out = (_c.c_int32 * 2)()
    _lib.check_attn(_lib.attn().mux_device_cu_info(out), "mux_device_cu_info")
    return int(out[0]), int(out[1])
