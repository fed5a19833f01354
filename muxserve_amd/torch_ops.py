"""The package's TORCH_LIBRARY operators (libmuxtorch.so): the same entry
points as muxserve_amd.ops, registered with PyTorch's dispatcher as
``torch.ops.muxserve_amd.*`` for callers that bind the attention layer
(muxserve/flexserver/models/llama.py:159-161) through torch operators rather
than through ctypes.  The library is a thin layer over the C ABI of
libmuxattn.so: tensor checks, raw pointers, torch's current HIP stream.

    ops = muxserve_amd.torch_ops.load()
    ops.reshape_and_cache(k, v, k_cache, v_cache, slot_mapping, layer, num_tokens)

There is no fallback: a missing library raises, CPU tensors are refused by the
dispatcher (only the GPU key is registered).
"""
import os

import torch

from ._lib import MuxLibraryMissing

_PKG = os.path.dirname(os.path.abspath(__file__))
TORCH_LIB_PATH = os.environ.get("MUXSERVE_TORCH_LIB", os.path.join(_PKG, "libmuxtorch.so"))

OPERATORS = ("reshape_and_cache", "rope_reshape_and_cache", "multi_reshape_and_cache", "rotary_neox",
             "paged_decode_workspace_bytes",
             "paged_decode", "multi_decode_workspace_bytes", "multi_decode", "prefill_causal",
             "multi_prefill_causal", "rms_norm",
             "silu_and_mul", "greedy_sample_workspace_bytes", "greedy_sample")

_loaded = False


def load():
    """Loads libmuxtorch.so once and returns the ``torch.ops.muxserve_amd`` namespace."""
    global _loaded
    if not _loaded:
        if not os.path.exists(TORCH_LIB_PATH):
            raise MuxLibraryMissing(
                f"{TORCH_LIB_PATH} is not built; run `python -m muxserve_amd.build` (there is no fallback path)")
        torch.ops.load_library(TORCH_LIB_PATH)
        _loaded = True
    return torch.ops.muxserve_amd



# ---------------------------------------------------------------------------
# The serving path's calls.  muxserve_amd.attention and muxserve_amd.layers (the
# classes that stand in for the reference's attention layer, RMSNorm, SiluAndMul
# and GreedySampler) reach the GPU through these: registered operators of the
# extension, launched on torch's current stream, workspaces kept per (device,
# stream) by muxserve_amd.ops._scratch.
# ---------------------------------------------------------------------------

def _current_stream_ptr(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def reshape_and_cache(k, v, k_pool, v_pool, slot_mapping, layer: int = 0, num_tokens=None) -> None:
    load().reshape_and_cache(k, v, k_pool, v_pool, slot_mapping, int(layer), -1 if num_tokens is None else int(num_tokens))


def rope_reshape_and_cache(positions, q, k, v, cos_sin, k_pool, v_pool, slot_mapping, layer: int = 0,
                           num_tokens=None) -> None:
    load().rope_reshape_and_cache(positions, q, k, v, cos_sin, k_pool, v_pool, slot_mapping, int(layer),
                                  -1 if num_tokens is None else int(num_tokens))


def rotary_neox(positions, q, k, cos_sin, num_tokens=None) -> None:
    load().rotary_neox(positions, q, k, cos_sin, -1 if num_tokens is None else int(num_tokens))


def prefill_causal(out, q, k, v, cu_seqlens, max_prompt_len: int, scale: float, num_kv_heads: int,
                   prompt_lens=None) -> None:
    load().prefill_causal(out, q, k, v, cu_seqlens, [] if prompt_lens is None else [int(x) for x in prompt_lens],
                          int(max_prompt_len), float(scale), int(num_kv_heads))


def multi_prefill_causal(calls) -> None:
    """Causal prefill of several colocated models' prompts in one launch.  `calls`:
    muxserve_amd.ops.PrefillCall objects (out, q, k, v, cu_seqlens, prompt_lens,
    scale, num_kv_heads), one per model."""
    lens = [torch.tensor([int(x) for x in c.prompt_lens], dtype=torch.int32) for c in calls]
    load().multi_prefill_causal([c.out for c in calls], [c.q for c in calls], [c.k for c in calls],
                                [c.v for c in calls], [c.cu_seqlens for c in calls], lens,
                                [int(t.max()) if t.numel() else 0 for t in lens], [float(c.scale) for c in calls],
                                [int(c.num_kv_heads) for c in calls])


def paged_decode(out, q, k_pool, v_pool, block_tables, context_lens, max_context_len: int, scale: float,
                 layer: int = 0, partition_size: int = 0, total_context_len: int = 0, context_lens_host=None) -> None:
    from . import ops
    T = load()
    need = T.paged_decode_workspace_bytes(out, q, block_tables, context_lens, int(max_context_len), int(partition_size))
    ws = ops._workspace(need, q.device, _current_stream_ptr(q.device))
    if ws is None:
        ws = torch.empty((0,), dtype=torch.uint8, device=q.device)
    T.paged_decode(out, q, k_pool, v_pool, block_tables, context_lens, int(max_context_len), float(scale), int(layer),
                   int(partition_size), int(total_context_len), ws, context_lens_host)


def rms_norm(x, weight, eps: float):
    return load().rms_norm(x, weight, float(eps))


def silu_and_mul(x):
    return load().silu_and_mul(x)


def greedy_sample(embedding, hidden_states, vocab_size: int, num_rows: int, row_index=None):
    from . import ops
    T = load()
    need = T.greedy_sample_workspace_bytes(int(vocab_size))
    ws = ops._scratch(ops._sample_workspaces, need, hidden_states.device, _current_stream_ptr(hidden_states.device), 1)
    if row_index is None:
        row_index = torch.empty((0,), dtype=torch.int32, device=hidden_states.device)
    return T.greedy_sample(embedding, hidden_states, int(vocab_size), int(num_rows), row_index, ws)
