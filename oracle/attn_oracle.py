"""CPU restatement of the device half of the hot path: pool geometry, the
KV-cache write, paged decode attention and causal prefill attention.

TEST INFRASTRUCTURE ONLY.  Imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py; never by the product package.

Where the algorithm comes from.  The reference delegates this arithmetic to an
un-vendored, un-pinned dependency: module `vllm` = EfficientLLMSys/MuxServe-vLLM
(installed from a git URL, README.md:16-25; API of upstream vLLM v0.2.x).  It is
absent from the reference checkout and cannot be installed offline, and the
reference's own tests hold no vectors for it.  What the reference itself fixes,
and this file follows:
  * pool layout and sizing            muxserve/flexstore/manager.py:444-498
  * slot arithmetic                   csrc/batch_scheduler.h:42-67
  * tensor shapes at the call         muxserve/flexserver/llm_runtime.py:300-334
  * scale = head_dim**-0.5, q/k/v split, the call
                                      muxserve/flexserver/models/llama.py:118,157-161
The attention itself is restated from the published algorithm of upstream
vLLM's paged attention (single-query attention over a block table; GQA maps
query head hq to kv head hq // (Hq // Hkv)): gather, fp32 softmax(scale*q.K^T),
fp32 P.V.

Pinning (tests/test_attn_oracle.py): pool geometry against closed forms worked
by hand from manager.py; reshape_and_cache against a brute-force element loop
and gather(scatter(x)) == x; paged_decode against
torch.nn.functional.scaled_dot_product_attention on the gathered K/V, ctx == 1
=> out == V[0], identical keys => out == mean(V), invariance under relabelling
of physical blocks; prefill against per-prompt SDPA with is_causal=True and
block-diagonal independence.  PARITY UNPINNED against the absent dependency
itself: its internal rounding (fp16 vs fp32 in q.K and P.V) is only bounded by
the 2e-3 budget, not reproduced.
"""
from __future__ import annotations

import numpy as np
import torch

HEAD_SIZE = 128          # muxserve/flexstore/manager.py:337


# ---- pool geometry: muxserve/flexstore/manager.py:444-468 -------------------

def key_block_shape(block_size: int, head_size: int = HEAD_SIZE, element_size: int = 2):
    x = 16 // element_size                                   # manager.py:457
    return (head_size // x, block_size, x)                   # manager.py:458-462


def value_block_shape(block_size: int, head_size: int = HEAD_SIZE):
    return (head_size, block_size)                           # manager.py:464-468


def num_gpu_blocks(gpu_memory_utilization: float, total_mem_bytes: int, block_size: int,
                   head_size: int = HEAD_SIZE) -> int:
    available = round(gpu_memory_utilization * total_mem_bytes) - 1          # manager.py:448-449
    block_mem = 2 * (int(np.prod(key_block_shape(block_size, head_size))) +
                     int(np.prod(value_block_shape(block_size, head_size))))  # manager.py:451-452
    return (available // block_mem // 128) * 128                              # manager.py:453


def allocate_pool(num_blocks: int, block_size: int, dtype=torch.float16, device="cpu"):
    """manager.py:485-492 (dtype is hard-wired fp16 there)."""
    k = torch.empty((num_blocks, *key_block_shape(block_size)), dtype=dtype, device=device)
    v = torch.empty((num_blocks, *value_block_shape(block_size)), dtype=dtype, device=device)
    return k, v


# ---- KV-cache write -----------------------------------------------------------

def reshape_and_cache(k, v, k_pool, v_pool, slot_mapping, layer=0, num_tokens=None):
    """k, v: [T_pad, Hkv*D]; slot_mapping int64 [T, L, Hkv]; pools modified in
    place.  slot -> (block, offset) per csrc/batch_scheduler.h:50-53; element
    placement per manager.py:456-468."""
    T, L, H = slot_mapping.shape
    if num_tokens is not None:
        T = min(T, num_tokens)
    bs = k_pool.shape[2]
    x = k_pool.shape[3]
    D = v_pool.shape[1]
    slots = slot_mapping[:T, layer, :].reshape(-1)            # [(t,h)]
    keep = slots >= 0
    b = torch.div(slots, bs, rounding_mode="floor")[keep]
    o = (slots % bs)[keep]
    kk = k[:T].reshape(T * H, D // x, x)[keep]
    vv = v[:T].reshape(T * H, D)[keep]
    k_pool[b, :, o, :] = kk
    v_pool[b, :, o] = vv


def reshape_and_cache_loops(k, v, k_pool, v_pool, slot_mapping, layer=0):
    """Element-by-element form (tiny inputs only)."""
    T, L, H = slot_mapping.shape
    bs, x, D = k_pool.shape[2], k_pool.shape[3], v_pool.shape[1]
    for t in range(T):
        for h in range(H):
            slot = int(slot_mapping[t, layer, h])
            if slot < 0:
                continue
            b, o = slot // bs, slot % bs
            for d in range(D):
                k_pool[b, d // x, o, d % x] = k[t, h * D + d]
                v_pool[b, d, o] = v[t, h * D + d]


def gather_kv(k_pool, v_pool, table_row, ctx):
    """K, V [ctx, D] of one (sequence, kv head) through its block-table row."""
    bs = k_pool.shape[2]
    nblk = (ctx + bs - 1) // bs
    ids = table_row[:nblk].long()
    K = k_pool[ids].permute(0, 2, 1, 3).reshape(nblk * bs, -1)[:ctx]      # [nblk,bs,D/x,x]
    V = v_pool[ids].permute(0, 2, 1).reshape(nblk * bs, -1)[:ctx]         # [nblk,bs,D]
    return K, V


# ---- paged decode attention -----------------------------------------------------

def paged_decode(q, k_pool, v_pool, block_tables, context_lens, scale, layer=0):
    """q [>=B, Hq*D]; block_tables int32 [L, B, Hkv, maxBlk]; context_lens [B].
    Returns fp32 [B, Hq*D]."""
    L, B, Hkv, _ = block_tables.shape
    D = v_pool.shape[1]
    Hq = q.shape[1] // D
    ratio = Hq // Hkv
    out = torch.zeros((B, Hq * D), dtype=torch.float32)
    for s in range(B):
        ctx = int(context_lens[s])
        if ctx <= 0:
            continue
        for hk in range(Hkv):
            K, V = gather_kv(k_pool, v_pool, block_tables[layer, s, hk], ctx)
            K, V = K.float(), V.float()
            qq = q[s, hk * ratio * D:(hk + 1) * ratio * D].float().reshape(ratio, D)
            p = torch.softmax((qq @ K.T) * scale, dim=-1)
            out[s, hk * ratio * D:(hk + 1) * ratio * D] = (p @ V).reshape(-1)
    return out


# ---- causal prefill attention ---------------------------------------------------

def prefill_causal(q, k, v, prompt_lens, scale, num_kv_heads):
    """q [T_pad, Hq*D], k/v [T_pad, Hkv*D], packed prompts.  Returns fp32
    [T, Hq*D] for the first T = sum(prompt_lens) rows."""
    D = HEAD_SIZE
    Hq = q.shape[1] // D
    ratio = Hq // num_kv_heads
    T = int(sum(prompt_lens))
    out = torch.zeros((T, Hq * D), dtype=torch.float32)
    start = 0
    for n in prompt_lens:
        n = int(n)
        qs = q[start:start + n].float().reshape(n, Hq, D).permute(1, 0, 2)              # [Hq,n,D]
        ks = k[start:start + n].float().reshape(n, num_kv_heads, D).permute(1, 0, 2)
        vs = v[start:start + n].float().reshape(n, num_kv_heads, D).permute(1, 0, 2)
        ks = ks.repeat_interleave(ratio, dim=0)
        vs = vs.repeat_interleave(ratio, dim=0)
        sc = (qs @ ks.transpose(1, 2)) * scale
        mask = torch.ones(n, n, dtype=torch.bool).tril()
        sc = sc.masked_fill(~mask, float("-inf"))
        o = torch.softmax(sc, dim=-1) @ vs                                               # [Hq,n,D]
        out[start:start + n] = o.permute(1, 0, 2).reshape(n, Hq * D)
        start += n
    return out


# ---- algorithmic traffic (shared by bench.py and the tests) ---------------------

def decode_bytes(context_lens, num_q_heads, num_kv_heads, block_size, head_size=HEAD_SIZE, e=2):
    """Per timed layer: K+V over exact valid tokens, q read + out write, block
    table ints, context length."""
    total = 0
    for ctx in context_lens:
        ctx = int(ctx)
        total += 2 * ctx * num_kv_heads * head_size * e
        total += 2 * num_q_heads * head_size * e
        total += num_kv_heads * ((ctx + block_size - 1) // block_size) * 4 + 4
    return total


def cache_write_bytes(num_tokens, num_kv_heads, head_size=HEAD_SIZE, e=2):
    return num_tokens * num_kv_heads * (2 * head_size * e + 2 * head_size * e + 8)


# ---- rotary position embedding ---------------------------------------------------

def rotary_neox(positions, q, k, rotary_dim=HEAD_SIZE, base=10000.0, head_size=HEAD_SIZE):
    """Textbook NeoX-style RoPE (the reference constructs its attention layer
    with rotary_dim = head_dim, base = rope_theta,
    muxserve/flexserver/models/llama.py:138-147): for pair index i < r/2 with
    angle p * base^(-2i/r),  (x_i, x_{i+r/2}) -> (x_i cos - x_{i+r/2} sin,
    x_{i+r/2} cos + x_i sin).  fp64 angles, fp32 arithmetic; returns fp32
    copies of q and k ([T, H*head_size])."""
    T = positions.shape[0]
    half = rotary_dim // 2
    inv_freq = 1.0 / (base ** (torch.arange(0, rotary_dim, 2, dtype=torch.float64) / rotary_dim))
    ang = positions.double()[:, None] * inv_freq[None, :]              # [T, half]
    cos, sin = ang.cos().float()[:, None, :], ang.sin().float()[:, None, :]
    outs = []
    for t in (q, k):
        x = t[:T].float().reshape(T, -1, head_size).clone()
        a, b = x[..., :half].clone(), x[..., half:rotary_dim].clone()
        x[..., :half] = a * cos - b * sin
        x[..., half:rotary_dim] = b * cos + a * sin
        outs.append(x.reshape(T, -1))
    return outs[0], outs[1]
