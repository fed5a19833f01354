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

OPERATORS = ("reshape_and_cache", "rope_reshape_and_cache", "rotary_neox", "paged_decode_workspace_bytes",
             "paged_decode", "multi_decode_workspace_bytes", "multi_decode", "prefill_causal", "rms_norm",
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
