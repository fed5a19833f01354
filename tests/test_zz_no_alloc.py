"""GPU check of the entry point that allocates nothing
(mux_multi_decode_noalloc): through the C ABI its outputs must equal those of
mux_multi_decode on the same inputs bit for bit (same kernels, scratch in the
library's static per-GPU array instead of a caller's workspace), on two calls
in a row - the second with a smaller input, so that whatever the first call
left in the array (partials, counters, a pair table) must not leak into it -
and both must meet the 2e-3 bar against the CPU oracle.  Needs larger than the
array are refused before anything is launched.
"""
import numpy as np
import pytest
import torch

from oracle import attn_oracle as orc
from muxserve_amd import _lib, ops, workloads
from muxserve_amd.pool import allocate_gpu_cache

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 2e-3


def _models(rng, shapes, ids, bs):
    models, cur = [], 0
    for name, hq, hk, ctx in shapes:
        bt, cur = workloads.build_tables(ctx.astype(np.int32), hk, bs, ids, cur)
        models.append(workloads.DecodeModel(name, hq, hk, ctx.astype(np.int32), bt))
    return models


def _run_both(models, dk, dv, partition):
    calls = [ops.DecodeCall(m.out, m.q, m.d_block_tables, m.d_context_lens, m.max_context_len, m.scale)
             for m in models]
    for m in models:
        m.out.fill_(7.0)
    ops.multi_decode(calls, dk, dv, partition_size=partition)
    torch.cuda.synchronize()
    ref = [m.out.clone() for m in models]
    for m in models:
        m.out.fill_(7.0)
    # (a first call outside the check: the first launch of a kernel loads its code object)
    ops.multi_decode_noalloc(calls, dk, dv, partition_size=partition)
    torch.cuda.synchronize()
    for m in models:
        m.out.fill_(7.0)
    torch.cuda.synchronize()
    before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    ops.multi_decode_noalloc(calls, dk, dv, partition_size=partition)
    torch.cuda.synchronize()
    # neither torch's allocator nor the device's free memory (which a hipMalloc inside the library would move)
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before
    return ref, [m.out.clone() for m in models]


def test_noalloc_decode_equals_the_workspace_entry_point_on_two_calls_in_a_row():
    print("[case] no-alloc decode: large call then smaller call", flush=True)
    bs, N = 16, 30000
    rng = np.random.Generator(np.random.PCG64(77))
    ids = rng.permutation(N)
    # first call: grouped-query model + small multi-head model + a 300-sequence
    # batch (pair table), all with split contexts
    big = _models(rng, [("gqa", 16, 2, rng.integers(1, 900, size=6)),
                        ("mha", 4, 4, rng.integers(1, 700, size=9)),
                        ("mha-large", 1, 1, rng.integers(1, 300, size=300))], ids, bs)
    # second call: fewer, shorter sequences over other blocks of the same pool
    ids2 = ids[::-1].copy()
    small = _models(rng, [("gqa", 16, 2, rng.integers(1, 300, size=2)),
                          ("mha", 4, 4, rng.integers(100, 400, size=3))], ids2, bs)
    dk, dv = allocate_gpu_cache(N, bs, DEV)
    dk.fill_(float("nan"))
    dv.fill_(float("nan"))
    used = np.unique(np.concatenate([m.used_blocks(bs) for m in big + small]))
    workloads.fill_blocks(dk, dv, used, seed=5)
    for i, m in enumerate(big + small):
        m.to_device(DEV, torch.float16, seed=40 + i)
    for name, models in (("large", big), ("small", small)):
        ref, got = _run_both(models, dk, dv, partition=128)
        ks, vs, tables = workloads.compact_to_host(dk, dv, models, bs)
        for m, r, g, t in zip(models, ref, got, tables):
            assert torch.equal(r, g), f"{name} call, model {m.name}: outputs differ from mux_multi_decode"
            assert (g[m.batch:] == 7.0).all(), "padding rows must not be written"
            want = orc.paged_decode(m.q.cpu(), ks, vs, t, m.context_lens, m.scale)
            err = (g[:m.batch].float().cpu() - want).abs().max().item()
            assert err <= TOL, f"{name} call, model {m.name}: max-abs error {err:.3e} vs the oracle"


def test_noalloc_decode_refuses_what_the_static_array_cannot_hold():
    print("[case] no-alloc decode: size limit", flush=True)
    lib = _lib.attn()
    limit = lib.mux_multi_decode_noalloc_max_bytes()
    assert limit == 32 << 20
    bs = 16
    B, H, max_blocks = 256, 64, 256                    # 4096-token contexts: 16 partials of 520 B per head
    dk, dv = allocate_gpu_cache(64, bs, DEV)
    q = torch.zeros((B, H * 128), dtype=torch.float16, device=DEV)
    out = torch.full_like(q, 7.0)
    bt = torch.zeros((1, B, H, max_blocks), dtype=torch.int32, device=DEV)
    cl = torch.full((B,), 4096, dtype=torch.int32, device=DEV)
    call = ops.DecodeCall(out, q, bt, cl, 4096, 1.0)
    import ctypes
    items = (_lib.MuxDecodeItem * 1)(call.to_item())
    assert lib.mux_paged_decode_workspace_bytes(ctypes.addressof(items), 1, 256) > limit
    with pytest.raises(RuntimeError, match="static array"):
        ops.multi_decode_noalloc([call], dk, dv, partition_size=256)
    torch.cuda.synchronize()
    assert (out == 7.0).all(), "a refused call must not launch anything"


def test_noalloc_decode_refused_for_its_arguments_launches_nothing():
    """A call that is refused for a malformed argument (here: a block size the
    library does not have, then a table too narrow for max_context_len) must
    not have launched anything - not even the fill kernel that clears the
    static array's arrival counters."""
    print("[case] no-alloc decode: refused arguments", flush=True)
    import ctypes
    lib = _lib.attn()
    bs = 16
    dk, dv = allocate_gpu_cache(64, bs, DEV)
    q = torch.zeros((8, 4 * 128), dtype=torch.float16, device=DEV)
    out = torch.full_like(q, 7.0)
    bt = torch.zeros((1, 8, 4, 40), dtype=torch.int32, device=DEV)
    cl = torch.full((8,), 600, dtype=torch.int32, device=DEV)
    items = (_lib.MuxDecodeItem * 1)(ops.DecodeCall(out, q, bt, cl, 600, 1.0).to_item())
    st = torch.cuda.current_stream().cuda_stream
    rc = lib.mux_multi_decode_noalloc(ctypes.addressof(items), 1, dk.data_ptr(), dv.data_ptr(), 64, 128, 24, 0, 128, st)
    assert rc == -2
    items[0].max_blocks = 10                      # 160 tokens of table for 600-token contexts
    rc = lib.mux_multi_decode_noalloc(ctypes.addressof(items), 1, dk.data_ptr(), dv.data_ptr(), 64, 128, bs, 0, 128, st)
    assert rc == -1
    torch.cuda.synchronize()
    assert (out == 7.0).all()
