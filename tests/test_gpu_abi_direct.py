"""The three entry points a binding of the attention call would link
(muxserve/flexserver/models/llama.py:159-161: cache write, paged decode,
causal prefill) driven DIRECTLY through ctypes - the library opened with
ctypes.CDLL, argument types written out here from include/muxserve_attn.h, raw
device pointers, no muxserve_amd.ops in between - on the single-model workload
(7B-shaped layer: 32 heads x 128, fp16, block size 16, batch 8, contexts
U{64..512}, tables from a seeded permutation of a 4096-group pool) and compared
with the CPU oracle: cache bit-exact, attention <= 2e-3 max-abs.
"""
import ctypes

import numpy as np
import pytest
import torch

from oracle import attn_oracle as orc
from muxserve_amd import _lib, workloads
from muxserve_amd.pool import HEAD_SIZE

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 2e-3

i32, i64, f32, vp, sz = ctypes.c_int32, ctypes.c_int64, ctypes.c_float, ctypes.c_void_p, ctypes.c_size_t


def _raw():
    lib = ctypes.CDLL(_lib.ATTN_LIB_PATH)
    lib.mux_reshape_and_cache.restype = i32
    lib.mux_reshape_and_cache.argtypes = [vp, vp, i64, vp, vp, i64, vp, i32, i32, i32, i32, i32, i32, i32, vp]
    lib.mux_paged_decode.restype = i32
    lib.mux_paged_decode.argtypes = [vp, i64, vp, i64, vp, vp, i64, vp, vp, i32, i32, i32, i32, i32, i32, i32, i32, i32,
                                     f32, i32, i32, vp, sz, vp]
    lib.mux_prefill_causal.restype = i32
    lib.mux_prefill_causal.argtypes = [vp, i64, vp, i64, vp, vp, i64, vp, vp, vp, i32, i32, i32, i32, i32, f32, i32, vp]
    return lib


def _stream():
    return torch.cuda.current_stream().cuda_stream


def test_cache_write_then_decode_through_the_bare_c_abi_on_the_single_model_workload():
    print("[case] bare C ABI: mux_reshape_and_cache + mux_paged_decode, config 1", flush=True)
    lib = _raw()
    bs, H = 16, 32
    (m,), N = workloads.config1(seed=0)
    ctx, bt = m.context_lens, m.block_tables                       # [8], [1, 8, 32, max_blocks]
    B, max_blocks = len(ctx), bt.shape[-1]
    g = torch.Generator().manual_seed(5)
    k_pool, v_pool = orc.allocate_pool(N, bs, torch.float16)
    k_pool.fill_(float("nan"))
    v_pool.fill_(float("nan"))
    dk, dv = k_pool.to(DEV), v_pool.to(DEV)
    # the contexts' K/V, written sequence by sequence through the cache write under test
    for s in range(B):
        n = int(ctx[s])
        kv = torch.randn((n, 2 * H * HEAD_SIZE), generator=g).half()
        k, v = kv[:, :H * HEAD_SIZE], kv[:, H * HEAD_SIZE:]
        i = np.arange(n)
        slots = torch.from_numpy((bt[0, s][:, i // bs].astype(np.int64).T * bs + (i % bs)[:, None])[:, None, :].copy())
        dkv, dslots = kv.to(DEV), slots.to(DEV)
        rc = lib.mux_reshape_and_cache(dkv.data_ptr(), dkv.data_ptr() + 2 * H * HEAD_SIZE, 2 * H * HEAD_SIZE,
                                       dk.data_ptr(), dv.data_ptr(), N, dslots.data_ptr(), 0, 1, n, H, HEAD_SIZE, bs,
                                       0, _stream())
        assert rc == 0, rc
        orc.reshape_and_cache(k, v, k_pool, v_pool, slots)
    torch.cuda.synchronize()
    assert torch.equal(dk.cpu().view(torch.int16), k_pool.view(torch.int16)), "K pool differs from the oracle's scatter"
    assert torch.equal(dv.cpu().view(torch.int16), v_pool.view(torch.int16)), "V pool differs from the oracle's scatter"

    q = torch.randn((B, H * HEAD_SIZE), generator=g).half()
    scale = HEAD_SIZE ** -0.5
    want = orc.paged_decode(q, k_pool, v_pool, torch.from_numpy(bt), ctx, scale)
    dq, dbt, dctx = q.to(DEV), torch.from_numpy(bt).to(DEV), torch.from_numpy(ctx).to(DEV)
    out = torch.zeros((B, H * HEAD_SIZE), dtype=torch.float16, device=DEV)
    ws = torch.zeros((64 << 20,), dtype=torch.uint8, device=DEV)        # zeroed: its head holds the arrival counters
    for partition in (0, 64):          # the library's choice, and one that splits every context
        out.zero_()
        rc = lib.mux_paged_decode(out.data_ptr(), H * HEAD_SIZE, dq.data_ptr(), H * HEAD_SIZE, dk.data_ptr(),
                                  dv.data_ptr(), N, dbt.data_ptr(), dctx.data_ptr(), 0, 1, B, H, H, HEAD_SIZE, bs,
                                  max_blocks, int(ctx.max()), scale, 0, partition, ws.data_ptr(), ws.numel(), _stream())
        assert rc == 0, rc
        torch.cuda.synchronize()
        err = (out.float().cpu() - want).abs().max().item()
        assert err <= TOL, f"partition {partition}: max-abs error {err:.3e}"


def test_prefill_through_the_bare_c_abi():
    print("[case] bare C ABI: mux_prefill_causal, 7B-shaped layer", flush=True)
    lib = _raw()
    H = 32
    lens = [70, 1, 200, 129, 16, 333]
    T = sum(lens)
    g = torch.Generator().manual_seed(6)
    qkv = torch.randn((T, 3 * H * HEAD_SIZE), generator=g).half()
    q, k, v = qkv.split([H * HEAD_SIZE] * 3, dim=-1)
    scale = HEAD_SIZE ** -0.5
    want = orc.prefill_causal(q, k, v, lens, scale, H)
    d = qkv.to(DEV)
    e = 2                                                             # bytes per element
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32, device=DEV)
    host_lens = (ctypes.c_int32 * len(lens))(*lens)
    out = torch.zeros((T, H * HEAD_SIZE), dtype=torch.float16, device=DEV)
    for lens_arg in (None, host_lens):           # grid sized by the longest prompt / the tiles that exist
        out.zero_()
        rc = lib.mux_prefill_causal(out.data_ptr(), H * HEAD_SIZE, d.data_ptr(), 3 * H * HEAD_SIZE,
                                    d.data_ptr() + H * HEAD_SIZE * e, d.data_ptr() + 2 * H * HEAD_SIZE * e,
                                    3 * H * HEAD_SIZE, cu.data_ptr(), None, lens_arg, len(lens), max(lens), H, H,
                                    HEAD_SIZE, scale, 0, _stream())
        assert rc == 0, rc
        torch.cuda.synchronize()
        err = (out.float().cpu() - want).abs().max().item()
        assert err <= TOL, f"max-abs error {err:.3e}"
