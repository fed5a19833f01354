"""Synthetic workloads: the shapes and distributions the benchmark and the
parity tests run on.  Everything is seeded; index tensors are built on the
host with numpy exactly in the layout the serving loop hands to the attention
layer (muxserve/flexserver/llm_runtime.py:300-334) and then copied to the
device.
"""
from dataclasses import dataclass, field
from typing import List, Optional

import numpy as np
import torch

from .pool import HEAD_SIZE, num_gpu_blocks

# (name, query heads, kv heads, layers) - LLaMA-1 shapes are MHA.
LLAMA_SHAPES = {
    "7b": (32, 32, 32),
    "13b": (40, 40, 40),
    "30b": (52, 52, 60),
    "65b": (64, 64, 80),
    "70b-gqa": (64, 8, 80),
}

POISON_BLOCK = -1   # what table entries past a sequence's last block hold


def lognormal_lengths(rng, n, median, sigma, lo, hi):
    x = rng.lognormal(mean=np.log(median), sigma=sigma, size=n)
    return np.clip(np.rint(x), lo, hi).astype(np.int32)


@dataclass
class DecodeModel:
    """One model's share of a decode step, one layer."""
    name: str
    num_q_heads: int
    num_kv_heads: int
    context_lens: np.ndarray                  # int32 [B]
    block_tables: np.ndarray                  # int32 [1, B, Hkv, max_blocks]
    scale: float = HEAD_SIZE ** -0.5
    # device copies (filled by to_device)
    d_context_lens: Optional[torch.Tensor] = None
    d_block_tables: Optional[torch.Tensor] = None
    q: Optional[torch.Tensor] = None
    out: Optional[torch.Tensor] = None

    @property
    def batch(self):
        return int(self.context_lens.shape[0])

    @property
    def max_context_len(self):
        return int(self.context_lens.max()) if self.batch else 0

    def used_blocks(self, block_size):
        """All physical block ids this model's tables reference."""
        out = []
        for s, ctx in enumerate(self.context_lens):
            n = (int(ctx) + block_size - 1) // block_size
            out.append(self.block_tables[0, s, :, :n].reshape(-1))
        return np.concatenate(out) if out else np.zeros(0, np.int32)

    def to_device(self, device, dtype, seed):
        g = torch.Generator(device="cpu").manual_seed(seed)
        pad = (self.batch + 7) // 8 * 8          # llm_runtime.py:300
        q = torch.randn((pad, self.num_q_heads * HEAD_SIZE), generator=g, dtype=torch.float32).to(dtype)
        self.q = q.to(device)
        self.out = torch.zeros_like(self.q)
        self.d_context_lens = torch.from_numpy(self.context_lens).to(device)
        self.d_block_tables = torch.from_numpy(self.block_tables).to(device)
        return self


def build_tables(context_lens, num_kv_heads, block_size, ids, cursor=0, max_blocks=None):
    """Head-granular tables: every (sequence, kv head, logical block) takes the
    next id from `ids`.  Returns (tables int32 [1,B,Hkv,max_blocks], cursor)."""
    B = len(context_lens)
    nblk = (np.asarray(context_lens, dtype=np.int64) + block_size - 1) // block_size
    if max_blocks is None:
        max_blocks = int(nblk.max()) if B else 0
    bt = np.full((1, B, num_kv_heads, max_blocks), POISON_BLOCK, dtype=np.int32)
    for s in range(B):
        n = int(nblk[s])
        cnt = n * num_kv_heads
        bt[0, s, :, :n] = np.asarray(ids[cursor:cursor + cnt], dtype=np.int32).reshape(num_kv_heads, n)
        cursor += cnt
    return bt, cursor


def build_tables_token_groups(context_lens, num_kv_heads, block_size, group_perm):
    """Tables a fresh FlexStore allocation with L=1 yields: token-block group g
    owns head-blocks g*Hkv + h (runs ordered [token block][layer][head],
    csrc/memory_manager.cpp:104-135)."""
    B = len(context_lens)
    nblk = (np.asarray(context_lens, dtype=np.int64) + block_size - 1) // block_size
    max_blocks = int(nblk.max())
    bt = np.full((1, B, num_kv_heads, max_blocks), POISON_BLOCK, dtype=np.int32)
    cur = 0
    heads = np.arange(num_kv_heads, dtype=np.int64)
    for s in range(B):
        n = int(nblk[s])
        g = np.asarray(group_perm[cur:cur + n], dtype=np.int64)
        bt[0, s, :, :n] = (g[None, :] * num_kv_heads + heads[:, None]).astype(np.int32)
        cur += n
    return bt


def config1(seed=0, block_size=16):
    """Single 7B-shaped layer: 32 heads, batch 8, ctx ~ U{64..512}, tables from
    one seeded permutation of a 4096-group pool (4096*32 head-blocks)."""
    rng = np.random.Generator(np.random.PCG64(seed))
    ctx = rng.integers(64, 513, size=8).astype(np.int32)
    perm = rng.permutation(4096)
    bt = build_tables_token_groups(ctx, 32, block_size, perm)
    return [DecodeModel("7b", 32, 32, ctx, bt)], 4096 * 32


def config2(seed=0, num_pool_blocks=None, block_size=16, batches=(32, 16, 8), offset_ids=0,
            id_perm=None):
    """Three colocated models (7B/13B/30B shapes) over one pool; ctx lognormal
    (median 300, sigma 0.8) clipped to [16, 2048]; every (model, sequence,
    head, logical block) draws a distinct id from one seeded permutation of
    the whole pool."""
    rng = np.random.Generator(np.random.PCG64(seed))
    shapes = [("7b", 32, 32), ("13b", 40, 40), ("30b", 52, 52)]
    ctxs = [lognormal_lengths(rng, b, 300, 0.8, 16, 2048) for b in batches]
    need = sum(int(((c.astype(np.int64) + block_size - 1) // block_size).sum()) * hk
               for c, (_, _, hk) in zip(ctxs, shapes))
    if id_perm is None:
        # Distinct ids without materialising a permutation of a 20M-entry pool
        # for every batch: sample without replacement.
        id_perm = rng.choice(num_pool_blocks, size=need + offset_ids, replace=False)
    ids = id_perm[offset_ids:]
    models, cur = [], 0
    for (name, hq, hk), c in zip(shapes, ctxs):
        bt, cur = build_tables(c, hk, block_size, ids, cur)
        models.append(DecodeModel(name, hq, hk, c, bt))
    return models, need


def config5(seed=0, num_pool_blocks=None, block_size=16, batch=64, lo=2048, hi=8192):
    """Long-context GQA decode: 64 query heads, 8 kv heads, ctx ~ U{lo..hi},
    tables scattered over the whole pool."""
    rng = np.random.Generator(np.random.PCG64(seed))
    ctx = rng.integers(lo, hi + 1, size=batch).astype(np.int32)
    need = int(((ctx.astype(np.int64) + block_size - 1) // block_size).sum()) * 8
    ids = rng.choice(num_pool_blocks, size=need, replace=False)
    bt, _ = build_tables(ctx, 8, block_size, ids)
    return [DecodeModel("70b-gqa", 64, 8, ctx, bt)], need


def fill_blocks(k_pool, v_pool, block_ids, seed, chunk=8192):
    """Write N(0,1) data into the listed pool blocks (device side, seeded)."""
    g = torch.Generator(device=k_pool.device).manual_seed(seed)
    ids = torch.as_tensor(np.asarray(block_ids, dtype=np.int64), device=k_pool.device)
    for i in range(0, ids.numel(), chunk):
        sel = ids[i:i + chunk]
        k_pool[sel] = torch.randn((sel.numel(), *k_pool.shape[1:]), generator=g,
                                  device=k_pool.device, dtype=torch.float32).to(k_pool.dtype)
        v_pool[sel] = torch.randn((sel.numel(), *v_pool.shape[1:]), generator=g,
                                  device=v_pool.device, dtype=torch.float32).to(v_pool.dtype)


def compact_to_host(k_pool, v_pool, models, block_size):
    """Copy only the referenced blocks to the host and relabel the tables to
    index the compact copy (attention is invariant under such a relabelling).
    Returns (k_small, v_small, [tables int32 per model])."""
    used = np.unique(np.concatenate([m.used_blocks(block_size) for m in models]))
    remap = {int(b): i for i, b in enumerate(used)}
    sel = torch.as_tensor(used.astype(np.int64), device=k_pool.device)
    k_small = k_pool[sel].cpu()
    v_small = v_pool[sel].cpu()
    tables = []
    lut = np.vectorize(lambda b: remap.get(int(b), 0), otypes=[np.int32])
    for m in models:
        tables.append(torch.from_numpy(lut(m.block_tables)))
    return k_small, v_small, tables


@dataclass
class PrefillModel:
    name: str
    num_q_heads: int
    num_kv_heads: int
    prompt_lens: np.ndarray
    scale: float = HEAD_SIZE ** -0.5

    @property
    def num_tokens(self):
        return int(self.prompt_lens.sum())

    def cu_seqlens(self):
        return np.concatenate([[0], np.cumsum(self.prompt_lens)]).astype(np.int32)


def config3(seed=0, prompts=16):
    """Prefill for the three shapes: `prompts` prompts each, lengths lognormal
    (median 200, sigma 1.0) clipped to [8, 2048]."""
    rng = np.random.Generator(np.random.PCG64(seed))
    shapes = [("7b", 32, 32), ("13b", 40, 40), ("30b", 52, 52)]
    return [PrefillModel(n, hq, hk, lognormal_lengths(rng, prompts, 200, 1.0, 8, 2048))
            for n, hq, hk in shapes]


def prefill_slot_mapping(prompt_lens, num_kv_heads, block_size, ids):
    """Head-wise slots for packed prompts: prompt token i of a prompt uses its
    token block i // bs at offset i % bs (csrc/batch_scheduler.h:42-56); every
    (prompt, token block, head) takes the next id from `ids`.
    Returns int64 [T, 1, Hkv]."""
    rows, cur = [], 0
    for n in prompt_lens:
        n = int(n)
        nblk = (n + block_size - 1) // block_size
        blk = np.asarray(ids[cur:cur + nblk * num_kv_heads], dtype=np.int64).reshape(nblk, num_kv_heads)
        cur += nblk * num_kv_heads
        i = np.arange(n)
        rows.append(blk[i // block_size] * block_size + (i % block_size)[:, None])
    return np.concatenate(rows)[:, None, :].astype(np.int64), cur


# ---- algorithmic traffic and work (the figures throughput is priced in) ----------

def decode_bytes(context_lens, num_q_heads, num_kv_heads, block_size, head_size=HEAD_SIZE, e=2):
    """Bytes one decode step of one layer has to move: K and V of exactly the
    valid tokens, q read and output written, the block-table entries in use and
    the context length of every sequence."""
    ctx = np.asarray(context_lens, dtype=np.int64)
    kv = 2 * ctx * num_kv_heads * head_size * e
    qo = 2 * num_q_heads * head_size * e
    table = num_kv_heads * ((ctx + block_size - 1) // block_size) * 4 + 4
    return int((kv + qo + table).sum())


def cache_write_bytes(num_tokens, num_kv_heads, head_size=HEAD_SIZE, e=2):
    """k and v read, the same bytes written to the pool, one 8-byte slot per
    (token, head)."""
    return int(num_tokens) * num_kv_heads * (4 * head_size * e + 8)


def prefill_flops(prompt_lens, num_q_heads, head_size=HEAD_SIZE):
    """QK^T and PV over the causal triangle: 4 * Hq * D * sum L (L + 1) / 2."""
    lens = np.asarray(prompt_lens, dtype=np.float64)
    return 4.0 * num_q_heads * head_size * float((lens * (lens + 1) / 2).sum())


def probe_gather_read(k_pool: torch.Tensor, v_pool: torch.Tensor, block_ids: torch.Tensor,
                      sink: Optional[torch.Tensor] = None, stream=None) -> None:
    """Measuring aid (libmuxprobe.so, not the product library): reads the K and V
    head-blocks named by block_ids (int32, device) with the decode kernel's load
    pattern and nothing else.  Bytes read: block_ids.numel() * 8192 at block
    size 16."""
    from . import _lib, ops
    ops._need_cuda(k_pool, v_pool, block_ids)
    bs = ops._check_pools(k_pool, v_pool)
    if block_ids.dtype != torch.int32 or block_ids.dim() != 1 or not block_ids.is_contiguous():
        raise ValueError("block_ids: expected contiguous int32 [n]")
    if sink is None:
        sink = torch.zeros((1,), dtype=torch.int32, device=k_pool.device)
    rc = _lib.probe().mux_probe_gather_read(k_pool.data_ptr(), v_pool.data_ptr(), k_pool.shape[0],
                                            block_ids.data_ptr(), block_ids.numel(), bs, sink.data_ptr(),
                                            ops._stream_ptr(stream))
    _lib.check_attn(rc, "mux_probe_gather_read")


def where_workgroups_run(stream=None, num_workgroups: int = 8192, spin_microseconds: int = 20, device="cuda:0"):
    """Measuring aid (libmuxprobe.so): launches single-wave workgroups that idle
    for spin_microseconds on `stream` and returns the sorted set of compute units
    they ran on as (accelerator die, shader engine, shader array, compute unit)
    tuples, read from the XCC_ID and HW_ID registers."""
    from . import _lib, ops
    out = torch.zeros((num_workgroups, 2), dtype=torch.int32, device=device)
    torch.cuda.synchronize()
    rc = _lib.probe().mux_probe_where(out.data_ptr(), int(num_workgroups), int(spin_microseconds),
                                      ops._stream_ptr(stream))
    _lib.check_attn(rc, "mux_probe_where")
    torch.cuda.synchronize()
    o = out.cpu().numpy().astype(np.uint32)
    xcc, hw = o[:, 0] & 0xf, o[:, 1]
    return sorted(set(zip(xcc.tolist(), ((hw >> 13) & 7).tolist(), ((hw >> 12) & 1).tolist(),
                          ((hw >> 8) & 0xf).tolist())))
