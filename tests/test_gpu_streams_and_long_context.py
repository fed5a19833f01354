"""GPU: CU-masked streams (prefill and decode colocated on disjoint CU shares)
and the long-context GQA decode shape (64 query heads over 8 kv heads, bf16,
contexts up to 8192, tables scattered over a ~200 GB pool)."""
import numpy as np
import pytest
import torch

from oracle import attn_oracle as orc
from muxserve_amd import ops, workloads
from muxserve_amd.pool import HEAD_SIZE, allocate_gpu_cache

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
D = HEAD_SIZE


def test_cu_masked_streams_run_prefill_and_decode_concurrently_and_correctly():
    print("[case] cu-masked streams", flush=True)
    ncu, nxcd = ops.device_cu_info()
    assert ncu >= 64 and ncu % nxcd == 0
    s_prefill = ops.CUMaskedStream(0, 40)
    s_decode = ops.CUMaskedStream(40, 100)
    assert s_prefill.num_cus + s_decode.num_cus == ncu
    bs, N = 16, 40000
    k_pool, v_pool = allocate_gpu_cache(N, bs, DEV)
    models, need = workloads.config2(seed=5, num_pool_blocks=N, batches=(16, 0, 0))
    dec = models[0]
    workloads.fill_blocks(k_pool, v_pool, dec.used_blocks(bs), seed=5)
    dec.to_device(DEV, torch.float16, seed=6)
    g = torch.Generator().manual_seed(8)
    lens = [700, 300]
    T = sum(lens)
    q = torch.randn((T, 4 * D), generator=g).half()
    k = torch.randn((T, 4 * D), generator=g).half()
    v = torch.randn((T, 4 * D), generator=g).half()
    dq, dk, dv = q.to(DEV), k.to(DEV), v.to(DEV)
    cu = torch.tensor([0, 700, 1000], dtype=torch.int32, device=DEV)
    pout = torch.zeros_like(dq)
    torch.cuda.synchronize()
    for _ in range(3):      # both streams busy at once, several rounds
        with torch.cuda.stream(s_prefill.torch_stream):
            ops.prefill_causal(pout, dq, dk, dv, cu, 700, D ** -0.5, 4)
        with torch.cuda.stream(s_decode.torch_stream):
            ops.paged_decode(dec.out, dec.q, k_pool, v_pool, dec.d_block_tables, dec.d_context_lens,
                             dec.max_context_len, dec.scale)
    s_prefill.synchronize()
    s_decode.synchronize()
    want_p = orc.prefill_causal(q, k, v, lens, D ** -0.5, 4)
    assert (pout.float().cpu() - want_p).abs().max().item() <= 2e-3
    ks, vs, tables = workloads.compact_to_host(k_pool, v_pool, [dec], bs)
    want_d = orc.paged_decode(dec.q.cpu(), ks, vs, tables[0], dec.context_lens, dec.scale)
    assert (dec.out[:dec.batch].float().cpu() - want_d).abs().max().item() <= 2e-3
    s_prefill.close()
    s_decode.close()
    with pytest.raises(RuntimeError):
        ops.CUMaskedStream(50, 50)


def test_part_set_streams_run_on_disjoint_compute_units_spread_over_every_die():
    """Streams made from sets of tenths of the GPU (what the scheduler's part
    bookkeeping hands out: any combination, not a contiguous range): the
    compute units their workgroups really run on - read from the XCC_ID / HW_ID
    registers by a recording kernel - are as many as the mask enables, differ
    between streams without a common part, and take every accelerator die's
    share within one compute unit per part."""
    print("[case] part-set cu masks, where workgroups run", flush=True)
    from muxserve_amd.cu_resource import CUResource
    ncu, nxcd = ops.device_cu_info()
    res = CUResource()
    held_a = res.allocate(3)                      # parts 9, 8, 7
    held_b = res.allocate(2)                      # parts 6, 5
    res.free(held_a[1:2])                         # part 8 back
    held_c = res.allocate(2)                      # parts 8, 4: not contiguous with each other
    sets = {"a": [held_a[0], held_a[2]], "b": held_b, "c": held_c, "one": [0]}
    seen = {}
    for name, parts in sets.items():
        st = ops.CUMaskedStream(parts=parts)
        where = workloads.where_workgroups_run(st)
        st.close()
        assert len(where) == st.num_cus, (name, len(where), st.num_cus)
        per_die = np.bincount([w[0] for w in where], minlength=nxcd)
        assert per_die.min() >= 1 and per_die.max() - per_die.min() <= len(parts), (name, per_die)
        seen[name] = set(where)
    for x in seen:
        for y in seen:
            if x < y:
                assert not seen[x] & seen[y], f"part sets {x} and {y} share a compute unit"
    whole = workloads.where_workgroups_run(None, num_workgroups=16384)
    assert len(whole) == ncu and set().union(*seen.values()) <= set(whole)
    # the percent ranges of the colocated configuration are disjoint as well
    s40, s60 = ops.CUMaskedStream(0, 40), ops.CUMaskedStream(40, 100)
    w40, w60 = workloads.where_workgroups_run(s40), workloads.where_workgroups_run(s60)
    s40.close()
    s60.close()
    assert not set(w40) & set(w60) and len(w40) + len(w60) == ncu
    for w in (w40, w60):
        per_die = np.bincount([x[0] for x in w], minlength=nxcd)
        assert per_die.max() - per_die.min() <= 1


def test_colocated_prefill_and_decode_at_the_benchmark_shapes():
    """The colocated configuration at its real shapes: a 30B-shaped prefill (52
    heads x 128, 4 prompts x 1024 tokens, fp16) on 40% of the compute units
    while a 7B-shaped decode (32 heads, batch 64, contexts uniform [512, 1024],
    block size 16) runs on the other 60%, both streams kept busy for several
    rounds, cache write of the prefill included (bit-exact).  The oracle runs
    on a subset: 4 heads of two prompts, and 6 sequences of the decode batch."""
    print("[case] colocated prefill + decode, benchmark shapes", flush=True)
    bs, N = 16, 160000
    Hp, Hd = 52, 32
    rng = np.random.Generator(np.random.PCG64(44))
    g = torch.Generator().manual_seed(44)
    k_pool, v_pool = allocate_gpu_cache(N, bs, DEV)
    ctx = rng.integers(512, 1025, size=64).astype(np.int32)
    need_d = int(((ctx + bs - 1) // bs).sum()) * Hd
    lens = [1024] * 4
    T = sum(lens)
    need_p = (T // bs) * Hp
    ids = rng.choice(N, size=need_d + need_p, replace=False)
    bt, _ = workloads.build_tables(ctx, Hd, bs, ids[:need_d])
    dec = workloads.DecodeModel("7b", Hd, Hd, ctx, bt)
    workloads.fill_blocks(k_pool, v_pool, dec.used_blocks(bs), seed=45)
    dec.to_device(DEV, torch.float16, seed=46)
    slots, _ = workloads.prefill_slot_mapping(lens, Hp, bs, ids[need_d:])       # int64 [T, 1, Hp]
    qkv = torch.randn((T, 3 * Hp * D), generator=g).half()
    dqkv = qkv.to(DEV)
    q, k, v = dqkv.split([Hp * D] * 3, dim=-1)
    dslots = torch.from_numpy(slots).to(DEV)
    cu = torch.tensor([0, 1024, 2048, 3072, 4096], dtype=torch.int32, device=DEV)
    pout = torch.zeros((T, Hp * D), dtype=torch.float16, device=DEV)
    s_prefill, s_decode = ops.CUMaskedStream(0, 40), ops.CUMaskedStream(40, 100)
    torch.cuda.synchronize()
    # Events at both ends of each stream's work, and one before all of it to measure from:
    # the two shares of the GPU must really have been busy at the same time.
    ev = {n: torch.cuda.Event(enable_timing=True) for n in ("t0", "p0", "p1", "d0", "d1")}
    for rnd in range(4):
        if rnd == 1:                    # the first round loads the kernels; the events bracket the other three
            s_prefill.synchronize()
            s_decode.synchronize()
            ev["t0"].record()
            ev["p0"].record(s_prefill.torch_stream)
            ev["d0"].record(s_decode.torch_stream)
        with torch.cuda.stream(s_prefill.torch_stream):
            ops.prefill_causal(pout, q, k, v, cu, 1024, D ** -0.5, Hp)
            ops.reshape_and_cache(k, v, k_pool, v_pool, dslots)
        with torch.cuda.stream(s_decode.torch_stream):
            for _ in range(4):          # a decode step is several times shorter than the prefill
                ops.paged_decode(dec.out, dec.q, k_pool, v_pool, dec.d_block_tables, dec.d_context_lens,
                                 dec.max_context_len, dec.scale, total_context_len=int(ctx.sum()),
                                 context_lens_host=torch.from_numpy(ctx))
    ev["p1"].record(s_prefill.torch_stream)
    ev["d1"].record(s_decode.torch_stream)
    s_prefill.synchronize()
    s_decode.synchronize()
    torch.cuda.synchronize()
    at = {n: ev["t0"].elapsed_time(e) for n, e in ev.items() if n != "t0"}      # ms since t0
    overlap = min(at["p1"], at["d1"]) - max(at["p0"], at["d0"])
    shorter = min(at["p1"] - at["p0"], at["d1"] - at["d0"])
    print(f"[colocated] prefill stream {at['p0']:.3f}..{at['p1']:.3f} ms, decode stream {at['d0']:.3f}..{at['d1']:.3f} ms, "
          f"overlap {overlap:.3f} ms", flush=True)
    assert overlap > 0.5 * shorter, (at, "the two streams did not run side by side")
    # prefill: heads 0, 17, 30, 51 of prompts 1 and 3 (causal attention is per head and per prompt)
    heads = [0, 17, 30, 51]
    cols = torch.cat([torch.arange(h * D, (h + 1) * D) for h in heads])
    qh, kh, vh = (qkv[:, o * Hp * D:(o + 1) * Hp * D] for o in range(3))
    for p in (1, 3):
        rows = slice(1024 * p, 1024 * (p + 1))
        want = orc.prefill_causal(qh[rows][:, cols], kh[rows][:, cols], vh[rows][:, cols], [1024], D ** -0.5,
                                  len(heads))
        got = pout[rows].float().cpu()[:, cols]
        assert (got - want).abs().max().item() <= 2e-3
    # the prefill's cache write, bit-exact on every slot it names
    hk, hv = orc.allocate_pool(N, bs, torch.float16)
    orc.reshape_and_cache(kh, vh, hk, hv, torch.from_numpy(slots))
    pblocks = torch.from_numpy(np.unique(slots // bs))
    assert torch.equal(k_pool.cpu()[pblocks].view(torch.int16), hk[pblocks].view(torch.int16))
    assert torch.equal(v_pool.cpu()[pblocks].view(torch.int16), hv[pblocks].view(torch.int16))
    # decode: six sequences (shortest, longest, four more), all heads
    pick = sorted({int(np.argmin(ctx)), int(np.argmax(ctx)), 0, 21, 42, 63})
    sub = workloads.DecodeModel("7b", Hd, Hd, ctx[pick].copy(), dec.block_tables[:, pick].copy(), dec.scale)
    ks, vs, tables = workloads.compact_to_host(k_pool, v_pool, [sub], bs)
    want_d = orc.paged_decode(dec.q[pick].cpu(), ks, vs, tables[0], sub.context_lens, dec.scale)
    assert (dec.out[pick].float().cpu() - want_d).abs().max().item() <= 2e-3
    assert torch.isfinite(dec.out[:64].float()).all() and torch.isfinite(pout.float()).all()
    s_prefill.close()
    s_decode.close()


def test_long_context_gqa_bf16_full_size_pool(full_size_pool_memory):
    """Config 5 at its real shape.  The oracle runs on a compact host copy of
    the referenced blocks for a subset of the sequences."""
    print("[case] long-context gqa", flush=True)
    bs = 16
    N = int(200e9) // 8192 // 128 * 128
    k_pool, v_pool = full_size_pool_memory(N, bs, torch.bfloat16)
    models, need = workloads.config5(seed=0, num_pool_blocks=N)
    m = models[0]
    used = m.used_blocks(bs)
    assert used.max() > N // 2
    workloads.fill_blocks(k_pool, v_pool, used, seed=1)
    m.to_device(DEV, torch.bfloat16, seed=2)
    for _ in range(2):
        ops.paged_decode(m.out, m.q, k_pool, v_pool, m.d_block_tables, m.d_context_lens, m.max_context_len,
                         m.scale, total_context_len=int(m.context_lens.sum()))
    torch.cuda.synchronize()
    assert torch.isfinite(m.out[:m.batch].float()).all()
    # The same launch with the units enumerated on the host (the prepared-launch path): same bits.
    device_enumerated = m.out.clone()
    launch = ops.DecodeLaunch([ops.DecodeCall(m.out, m.q, m.d_block_tables, m.d_context_lens, m.max_context_len, m.scale,
                                              total_context_len=int(m.context_lens.sum()),
                                              context_lens_host=torch.from_numpy(
                                                  np.ascontiguousarray(m.context_lens, dtype=np.int32)))],
                              k_pool, v_pool)
    assert launch.host_pairs > 0
    m.out.fill_(7.0)
    for _ in range(2):
        launch()
    torch.cuda.synchronize()
    assert torch.equal(m.out[:m.batch], device_enumerated[:m.batch])
    pick = [0, 17, int(np.argmax(m.context_lens)), int(np.argmin(m.context_lens))]
    sub = workloads.DecodeModel(m.name, m.num_q_heads, m.num_kv_heads, m.context_lens[pick].copy(),
                                m.block_tables[:, pick].copy(), m.scale)
    ks, vs, tables = workloads.compact_to_host(k_pool, v_pool, [sub], bs)
    want = orc.paged_decode(m.q[pick].cpu(), ks, vs, tables[0], sub.context_lens, m.scale)
    got = m.out[pick].float().cpu()
    bound = 2e-3 + want.abs() * 2.0 ** -8          # + rounding of the bf16 result
    assert ((got - want).abs() - bound).max().item() <= 0, (got - want).abs().max().item()


def test_decode_step_replays_from_a_hip_graph():
    """Cache write (fused with rotary) + fused three-model decode with split
    contexts and a 300-sequence model, captured once and replayed with new
    inputs; eager work and synchronisations between replays; every replay must
    equal the eager result bitwise (the split workspace's counters have to be
    back at zero after every run, eager or replayed)."""
    print("[case] hip graph replay of a decode step", flush=True)
    from muxserve_amd import _lib
    from muxserve_amd.attention import build_cos_sin_cache
    import ctypes
    bs, N = 16, 60000
    rng = np.random.Generator(np.random.PCG64(31))
    k_pool, v_pool = allocate_gpu_cache(N, bs, DEV)
    k_pool.zero_()
    v_pool.zero_()
    shapes = [("a", 4, 4, rng.integers(1, 900, size=6)), ("gqa", 8, 1, rng.integers(1, 900, size=5)),
              ("big", 1, 1, rng.integers(1, 400, size=300))]
    ids = rng.permutation(N)
    models, cur = [], 0
    for name, hq, hk, ctx in shapes:
        bt, cur = workloads.build_tables(ctx.astype(np.int32), hk, bs, ids, cur)
        models.append(workloads.DecodeModel(name, hq, hk, ctx.astype(np.int32), bt).to_device(DEV, torch.float16, seed=cur))
    workloads.fill_blocks(k_pool, v_pool, np.concatenate([m.used_blocks(bs) for m in models]), seed=31)
    calls = [ops.DecodeCall(m.out, m.q, m.d_block_tables, m.d_context_lens, m.max_context_len, m.scale)
             for m in models]
    items = (_lib.MuxDecodeItem * len(calls))(*[c.to_item() for c in calls])
    need = _lib.attn().mux_paged_decode_workspace_bytes(ctypes.addressof(items), len(calls), 128)
    ws = torch.zeros(need, dtype=torch.uint8, device=DEV)
    # the new token of model "a": k, v rows and the slot of its last context position
    a = models[0]
    cos_sin = build_cos_sin_cache(D, 2048, 10000.0, DEV)
    kv = torch.zeros((8, 2 * a.num_kv_heads * D), dtype=torch.float16, device=DEV)
    positions = torch.from_numpy(np.pad(a.context_lens.astype(np.int64) - 1, (0, 8 - a.batch))).to(DEV)
    last = (a.context_lens - 1)
    slots = (a.block_tables[0, np.arange(a.batch), :, last // bs].astype(np.int64) * bs + (last % bs)[:, None])
    dslots = torch.from_numpy(slots[:, None, :].copy()).to(DEV)

    def step():
        ops.rope_reshape_and_cache(positions, a.q, kv[:, :a.num_kv_heads * D], kv[:, a.num_kv_heads * D:], cos_sin,
                                   k_pool, v_pool, dslots, num_tokens=a.batch)
        ops.multi_decode(calls, k_pool, v_pool, partition_size=128, workspace=ws)

    def new_inputs(seed):
        g = torch.Generator(device=DEV).manual_seed(seed)
        for m in models:
            m.q.copy_(torch.randn(m.q.shape, generator=g, device=DEV).half())
        kv.copy_(torch.randn(kv.shape, generator=g, device=DEV).half())

    stream = torch.cuda.Stream()
    new_inputs(0)
    with torch.cuda.stream(stream):
        step()                                  # warm-up outside capture
    stream.synchronize()
    graph = torch.cuda.CUDAGraph()
    new_inputs(1)
    torch.cuda.synchronize()
    with torch.cuda.graph(graph, stream=stream):
        step()
    for rep in range(4):
        new_inputs(10 + rep)
        q_before = [m.q.clone() for m in models]
        kv_before = kv.clone()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [m.out.clone() for m in models]
        pools = (k_pool.clone(), v_pool.clone())
        # eager run on the same inputs (q and k of model a were rotated in place by the replay: restore them)
        kv.copy_(kv_before)
        for m, q0 in zip(models, q_before):
            m.q.copy_(q0)
            m.out.zero_()
        step()
        torch.cuda.synchronize()
        for m, o in zip(models, got):
            assert torch.equal(o, m.out), f"replay {rep}: model {m.name} differs from the eager run"
        assert torch.equal(pools[0], k_pool) and torch.equal(pools[1], v_pool)
    ks, vs, tables = workloads.compact_to_host(k_pool, v_pool, models, bs)
    for m, t in zip(models, tables):
        want = orc.paged_decode(m.q.cpu(), ks, vs, t, m.context_lens, m.scale)
        assert (m.out[:m.batch].float().cpu() - want).abs().max().item() <= 2e-3
