"""The attention layer of the serving path, with the reference's call
signature, running on the HIP kernels of libmuxattn.so.

Drop-in for what muxserve/flexserver/models/llama.py:138-161 constructs and
calls:

    attn = PagedAttentionWithRoPE(num_heads, head_dim, scaling, base=...,
                                  max_position=..., rotary_dim=...,
                                  num_kv_heads=..., rope_scaling=...,
                                  layer_idx=...)
    out = attn(positions, q, k, v, k_cache, v_cache, input_metadata, cache_event)

k_cache / v_cache are the WHOLE unified pool (models/llama.py:276-288); the
layer index selects slot_mapping[:, l, :] and block_tables[l].  InputMetadata
carries the fields the reference fills at pipeworker.py:81-90.

In the reference both classes come from the external MuxServe-vLLM fork, which
is not available; behaviour here follows the call sites plus the published
vLLM v0.2.x semantics (prompt tokens first, then one generation token per
sequence; NeoX rotary applied to q and k before the cache write).
"""
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

import torch

from . import ops
from . import torch_ops as T

HEAD_SIZE = ops.HEAD_SIZE


@dataclass
class InputMetadata:
    """Fields as constructed at muxserve/flexserver/pipeworker.py:81-90."""
    prompt_lens: List[int]
    slot_mapping: torch.Tensor                 # int64 [num_tokens, L, H]
    context_lens: torch.Tensor                 # int32 [num_generation_tokens]
    max_context_len: int
    block_tables: torch.Tensor                 # int32 [L, num_seqs, H, max_blocks]
    seq_groups: Any = None
    seq_data: Any = None
    sliding_window: Optional[int] = None
    # Not in the reference: host-side sum of context_lens, if the caller has it
    # (prepare_inputs does); only tightens the decode grid.
    total_context_len: int = 0
    # Not in the reference either: a host copy of context_lens (CPU int32 [B];
    # the serving loop has the lengths on the host before they become a tensor,
    # llm_runtime.py:311-326).  Small decode batches are then enumerated on the
    # host.  Leave None when the step is recorded into a HIP graph.
    context_lens_host: Optional[torch.Tensor] = None
    is_muxserve: bool = True                   # read at models/llama.py:285
    _cu_seqlens: Optional[torch.Tensor] = field(default=None, repr=False)
    _prompt_order: Optional[torch.Tensor] = field(default=None, repr=False)
    _last_rows: Optional[torch.Tensor] = field(default=None, repr=False)
    _lens_array: Any = field(default=None, repr=False)

    def __post_init__(self):
        self.prompt_lens = [int(x) for x in self.prompt_lens]
        self.num_prompts = len(self.prompt_lens)
        self.num_prompt_tokens = sum(self.prompt_lens)
        self.max_prompt_len = max(self.prompt_lens) if self.prompt_lens else 0
        self.num_generation_tokens = int(self.context_lens.shape[0])
        self.num_valid_tokens = self.num_prompt_tokens + self.num_generation_tokens
        if self.sliding_window is not None:
            raise NotImplementedError("sliding_window is always None in the serving path")

    def cu_seqlens(self, device) -> torch.Tensor:
        """int32 [num_prompts + 1] on the device, built once per step and shared
        by every layer."""
        if self._cu_seqlens is None or self._cu_seqlens.device != torch.device(device):
            cu = [0]
            for n in self.prompt_lens:
                cu.append(cu[-1] + n)
            self._cu_seqlens = torch.tensor(cu, dtype=torch.int32, device=device)
        return self._cu_seqlens

    def last_token_rows(self, device) -> torch.Tensor:
        """int32 [num_prompts] on the device: the row of every prompt's last token
        (cumsum(prompt_lens) - 1, what the sampler looks at), built once per step."""
        if self._last_rows is None or self._last_rows.device != torch.device(device):
            rows, end = [], 0
            for n in self.prompt_lens:
                end += n
                rows.append(end - 1)
            self._last_rows = torch.tensor(rows, dtype=torch.int32, device=device)
        return self._last_rows

    def prompt_lens_array(self):
        """The prompt lengths as a host int32 array for the C ABI, built once per
        step and shared by every layer."""
        if self._lens_array is None:
            import ctypes
            self._lens_array = (ctypes.c_int32 * len(self.prompt_lens))(*self.prompt_lens)
        return self._lens_array

    def prompt_order(self, device) -> torch.Tensor:
        """int32 [num_prompts] on the device: the prompts longest first (the order
        their attention workgroups are started in), built once per step."""
        if self._prompt_order is None or self._prompt_order.device != torch.device(device):
            order = sorted(range(len(self.prompt_lens)), key=lambda i: -self.prompt_lens[i])
            self._prompt_order = torch.tensor(order, dtype=torch.int32, device=device)
        return self._prompt_order


def build_cos_sin_cache(rotary_dim: int, max_position: int, base: float, device) -> torch.Tensor:
    """fp32 [max_position, rotary_dim]: row p = [cos(p f_i) | sin(p f_i)],
    f_i = base^(-2i / rotary_dim)."""
    inv_freq = 1.0 / (base ** (torch.arange(0, rotary_dim, 2, dtype=torch.float64) / rotary_dim))
    t = torch.arange(max_position, dtype=torch.float64)
    freqs = torch.outer(t, inv_freq)
    return torch.cat([freqs.cos(), freqs.sin()], dim=-1).float().to(device)


class PagedAttention(torch.nn.Module):
    """Cache write + causal prefill attention + paged decode attention for one
    layer of one model over the unified pool."""

    def __init__(self, num_heads: int, head_size: int, scale: float, num_kv_heads: Optional[int] = None,
                 sliding_window: Optional[int] = None, layer_idx: int = -1):
        super().__init__()
        if head_size != HEAD_SIZE:
            raise ValueError(f"head size is fixed at {HEAD_SIZE} in the unified pool")
        if sliding_window is not None:
            raise NotImplementedError("sliding window attention is not part of this path")
        self.num_heads = int(num_heads)
        self.head_size = int(head_size)
        self.scale = float(scale)
        self.num_kv_heads = self.num_heads if num_kv_heads is None else int(num_kv_heads)
        if self.num_heads % self.num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        self.layer_idx = int(layer_idx)
        self.partition_size = 0   # 0 = library default

    def _layer(self, input_metadata: InputMetadata) -> int:
        # A single-layer index tensor is accepted with layer_idx left at -1.
        if self.layer_idx >= 0:
            return self.layer_idx
        if input_metadata.slot_mapping.shape[1] != 1:
            raise ValueError("layer_idx was not set and the index tensors hold several layers")
        return 0

    def forward(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                key_cache: Optional[torch.Tensor], value_cache: Optional[torch.Tensor],
                input_metadata: InputMetadata, cache_event: Optional[torch.cuda.Event] = None,
                _cache_written: bool = False) -> torch.Tensor:
        """query [T_pad, Hq*128], key/value [T_pad, Hkv*128] (rows past
        num_valid_tokens are padding) -> [T_pad, Hq*128]."""
        md = input_metadata
        layer = self._layer(md)
        out = torch.empty((query.shape[0], self.num_heads * self.head_size), dtype=query.dtype,
                          device=query.device)
        n_prompt = md.num_prompt_tokens
        n_valid = md.num_valid_tokens
        if cache_event is not None:
            cache_event.wait()
        # The new tokens' K/V go into the pool first (decode reads them back).
        if key_cache is not None and value_cache is not None and n_valid > 0 and not _cache_written:
            T.reshape_and_cache(key, value, key_cache, value_cache, md.slot_mapping, layer=layer,
                                  num_tokens=n_valid)
        if n_prompt > 0:
            T.prefill_causal(out[:n_prompt], query[:n_prompt], key[:n_prompt], value[:n_prompt],
                               md.cu_seqlens(query.device), md.max_prompt_len, self.scale, self.num_kv_heads,
                               prompt_lens=md.prompt_lens)
        if md.num_generation_tokens > 0:
            if key_cache is None or value_cache is None:
                raise ValueError("decode needs the KV pool")
            T.paged_decode(out[n_prompt:n_valid], query[n_prompt:n_valid], key_cache, value_cache,
                             md.block_tables, md.context_lens, md.max_context_len, self.scale, layer=layer,
                             partition_size=self.partition_size, total_context_len=md.total_context_len,
                             context_lens_host=md.context_lens_host)
        return out


class PagedAttentionWithRoPE(PagedAttention):
    """PagedAttention with NeoX rotary embedding applied to q and k in place
    first; constructor arguments as at muxserve/flexserver/models/llama.py:138-147."""

    def __init__(self, num_heads: int, head_size: int, scale: float, rotary_dim: Optional[int] = None,
                 max_position: int = 8192, base: float = 10000, num_kv_heads: Optional[int] = None,
                 is_neox_style: bool = True, rope_scaling: Optional[Dict[str, Any]] = None,
                 sliding_window: Optional[int] = None, layer_idx: int = -1):
        super().__init__(num_heads, head_size, scale, num_kv_heads, sliding_window, layer_idx)
        if not is_neox_style:
            raise NotImplementedError("only NeoX-style rotary embedding (LLaMA) is implemented")
        if rope_scaling is not None:
            raise NotImplementedError("rope_scaling is not implemented (LLaMA-1/2 checkpoints use none)")
        self.rotary_dim = int(head_size if rotary_dim is None else rotary_dim)
        self.fused_rope_max_tokens = 512
        self.max_position = int(max_position)
        self.base = float(base)
        self._cos_sin: Optional[torch.Tensor] = None

    def _cache(self, device) -> torch.Tensor:
        if self._cos_sin is None or self._cos_sin.device != torch.device(device):
            self._cos_sin = build_cos_sin_cache(self.rotary_dim, self.max_position, self.base, device)
        return self._cos_sin

    def forward(self, positions: torch.Tensor, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                key_cache: Optional[torch.Tensor], value_cache: Optional[torch.Tensor],
                input_metadata: InputMetadata, cache_event: Optional[torch.cuda.Event] = None) -> torch.Tensor:
        md = input_metadata
        n_valid = md.num_valid_tokens
        fused = False
        if n_valid > 0:
            # Rotation and cache write in one launch for small steps (decode: saves a
            # launch, 12.6 against 20.4 us per layer), when the whole head rotates and
            # the rows allow 16-byte accesses (q, k, v of one qkv row always do).  Large
            # prefill steps keep the two kernels: the fused one re-reads the cos/sin row
            # of a token once per kv head and is slower there (101 against 93 us for
            # 4096 tokens x 52 heads).
            fused = (key_cache is not None and value_cache is not None and self.rotary_dim == self.head_size
                     and n_valid <= self.fused_rope_max_tokens
                     and all(t.stride(0) % 8 == 0 and t.data_ptr() % 16 == 0 for t in (query, key, value)))
            if fused:
                if cache_event is not None:
                    cache_event.wait()
                T.rope_reshape_and_cache(positions, query, key, value, self._cache(query.device), key_cache,
                                           value_cache, md.slot_mapping, layer=self._layer(md), num_tokens=n_valid)
            else:
                T.rotary_neox(positions, query, key, self._cache(query.device), num_tokens=n_valid)
        return super().forward(query, key, value, key_cache, value_cache, md, cache_event, _cache_written=fused)
