"""The unified head-granular KV pool: geometry, sizing rule and allocation,
as FlexStore defines them (muxserve/flexstore/manager.py:444-498).

One pool entry ("head-block") holds block_size tokens of ONE head of ONE layer:
    K  [head_size/x, block_size, x]   x = 16 // element_size (8 for fp16/bf16)
    V  [head_size, block_size]
so models with different head and layer counts draw from the same free list.
"""
import torch

HEAD_SIZE = 128   # hard-wired in the reference (manager.py:337)


def key_block_shape(block_size: int, element_size: int = 2):
    x = 16 // element_size
    return (HEAD_SIZE // x, block_size, x)


def value_block_shape(block_size: int):
    return (HEAD_SIZE, block_size)


def block_bytes(block_size: int, element_size: int = 2) -> int:
    """Bytes of one K block plus one V block."""
    kn = 1
    for d in key_block_shape(block_size, element_size):
        kn *= d
    vn = HEAD_SIZE * block_size
    return element_size * (kn + vn)


def num_gpu_blocks(gpu_memory_utilization: float, total_mem_bytes: int, block_size: int) -> int:
    """N = ((round(util * total_mem) - 1) // block_bytes // 128) * 128."""
    available = round(gpu_memory_utilization * total_mem_bytes) - 1
    return (available // block_bytes(block_size) // 128) * 128


def allocate_gpu_cache(num_blocks: int, block_size: int, device="cuda:0", dtype=torch.float16):
    """(k_cache [N, 16, bs, 8], v_cache [N, 128, bs]); the reference hard-wires
    fp16, bf16 is accepted here with the same packing."""
    k = torch.empty((num_blocks, *key_block_shape(block_size)), dtype=dtype, device=device)
    v = torch.empty((num_blocks, *value_block_shape(block_size)), dtype=dtype, device=device)
    return k, v
