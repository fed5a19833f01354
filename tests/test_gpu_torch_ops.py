"""The TORCH_LIBRARY operators (libmuxtorch.so) against the ctypes path
(muxserve_amd.ops): both call the same C ABI, so every result must be
bit-identical; argument errors must surface as exceptions."""
import numpy as np
import pytest
import torch

from muxserve_amd import ops, torch_ops, workloads
from muxserve_amd.attention import build_cos_sin_cache
from muxserve_amd.pool import HEAD_SIZE, allocate_gpu_cache

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
D = HEAD_SIZE


def _bits(t):
    return t.view(torch.int16)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_torch_operators_equal_the_ctypes_path(dtype):
    print(f"[case] torch operators {dtype}", flush=True)
    T = torch_ops.load()
    bs, N, Hq, Hkv, L = 16, 4096, 8, 2, 2
    g = torch.Generator().manual_seed(5)
    rng = np.random.Generator(np.random.PCG64(5))
    # ---- prefill step: rotary + cache write, causal attention --------------------------
    lens = [37, 130, 5]
    n = sum(lens)
    pad = (n + 7) // 8 * 8
    qkv = torch.randn((pad, (Hq + 2 * Hkv) * D), generator=g).to(dtype).to(DEV)
    positions = torch.cat([torch.arange(x) for x in lens] + [torch.zeros(pad - n, dtype=torch.int64)]).to(DEV)
    cos_sin = build_cos_sin_cache(D, 512, 10000.0, DEV)
    ids = rng.permutation(N)
    slots_np, _ = workloads.prefill_slot_mapping(lens, Hkv, bs, ids)
    slots = torch.from_numpy(np.repeat(slots_np, L, axis=1).copy()).to(DEV)          # [n, L, Hkv]
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32, device=DEV)
    pools = []
    outs = []
    for path in ("ctypes", "torch"):
        k_pool, v_pool = allocate_gpu_cache(N, bs, DEV, dtype=dtype)
        k_pool.zero_()
        v_pool.zero_()
        qq, kk, v = qkv.clone().split([Hq * D, Hkv * D, Hkv * D], dim=-1)   # rotated in place: a copy per path
        out = torch.zeros((pad, Hq * D), dtype=dtype, device=DEV)
        if path == "ctypes":
            ops.rope_reshape_and_cache(positions, qq, kk, v, cos_sin, k_pool, v_pool, slots, layer=1, num_tokens=n)
            ops.reshape_and_cache(kk, v, k_pool, v_pool, slots, layer=0, num_tokens=n)
            ops.prefill_causal(out[:n], qq[:n], kk[:n], v[:n], cu, max(lens), D ** -0.5, Hkv, prompt_lens=lens)
        else:
            T.rope_reshape_and_cache(positions, qq, kk, v, cos_sin, k_pool, v_pool, slots, 1, n)
            T.reshape_and_cache(kk, v, k_pool, v_pool, slots, 0, n)
            T.prefill_causal(out[:n], qq[:n], kk[:n], v[:n], cu, lens, max(lens), D ** -0.5, Hkv)
        torch.cuda.synchronize()
        pools.append((k_pool, v_pool))
        outs.append((qq, kk, out))
    for a, b in zip(pools[0] + outs[0], pools[1] + outs[1]):
        assert torch.equal(_bits(a), _bits(b))
    assert outs[0][2][:n].float().abs().sum().item() > 0
    # ---- decode step over the pool just written (layer 1) ------------------------------
    ctx = np.asarray(lens, dtype=np.int32)
    nblk = (ctx + bs - 1) // bs
    bt = np.zeros((L, len(lens), Hkv, int(nblk.max())), dtype=np.int32)
    row = 0
    for s, x in enumerate(lens):
        blocks = slots_np[row:row + x:bs, 0, :] // bs                     # [nblk, Hkv]
        bt[:, s, :, :blocks.shape[0]] = blocks.T
        row += x
    d_bt, d_ctx = torch.from_numpy(bt).to(DEV), torch.from_numpy(ctx).to(DEV)
    dq = torch.randn((8, Hq * D), generator=g).to(dtype).to(DEV)
    k_pool, v_pool = pools[1]
    o1 = torch.zeros((8, Hq * D), dtype=dtype, device=DEV)
    o2 = torch.zeros_like(o1)
    ops.paged_decode(o1, dq, k_pool, v_pool, d_bt, d_ctx, int(ctx.max()), D ** -0.5, layer=1, partition_size=64)
    need = T.paged_decode_workspace_bytes(o2, dq, d_bt, d_ctx, int(ctx.max()), 64)
    assert need > 0                                                         # the 130-token context is split
    ws = torch.zeros((need,), dtype=torch.uint8, device=DEV)
    for _ in range(2):                                                      # the workspace is reusable as left
        T.paged_decode(o2, dq, k_pool, v_pool, d_bt, d_ctx, int(ctx.max()), D ** -0.5, 1, 64, 0, ws)
    torch.cuda.synchronize()
    assert torch.equal(_bits(o1), _bits(o2)) and o1[:3].float().abs().sum().item() > 0
    # ---- the fused launch over two "models" (the same tables twice, different queries) -----
    dq2 = torch.randn((8, Hq * D), generator=g).to(dtype).to(DEV)
    f1, f2 = torch.zeros_like(o1), torch.zeros_like(o1)
    lists = ([f1, f2], [dq, dq2], [d_bt, d_bt], [d_ctx, d_ctx], [int(ctx.max())] * 2)
    need2 = T.multi_decode_workspace_bytes(*lists, 64)
    ws2 = torch.zeros((need2,), dtype=torch.uint8, device=DEV)
    T.multi_decode(lists[0], lists[1], k_pool, v_pool, lists[2], lists[3], lists[4], [D ** -0.5] * 2, [1, 1],
                   [int(ctx.sum())] * 2, 64, ws2, [])
    # the same with the units enumerated on the host (CPU copies of the context lengths)
    h1, h2 = torch.zeros_like(o1), torch.zeros_like(o1)
    host = torch.from_numpy(ctx)
    T.multi_decode([h1, h2], lists[1], k_pool, v_pool, lists[2], lists[3], lists[4], [D ** -0.5] * 2, [1, 1],
                   [int(ctx.sum())] * 2, 64, ws2, [host, host])
    o4 = torch.zeros_like(o1)
    T.paged_decode(o4, dq, k_pool, v_pool, d_bt, d_ctx, int(ctx.max()), D ** -0.5, 1, 64, 0, ws, host)
    # the serving-path wrapper (workspace kept by the package)
    o5 = torch.zeros_like(o1)
    torch_ops.paged_decode(o5, dq, k_pool, v_pool, d_bt, d_ctx, int(ctx.max()), D ** -0.5, layer=1, partition_size=64,
                           total_context_len=int(ctx.sum()), context_lens_host=host)
    o3 = torch.zeros_like(o1)
    ops.paged_decode(o3, dq2, k_pool, v_pool, d_bt, d_ctx, int(ctx.max()), D ** -0.5, layer=1, partition_size=64)
    torch.cuda.synchronize()
    assert torch.equal(_bits(f1), _bits(o1)) and torch.equal(_bits(f2), _bits(o3))
    assert torch.equal(_bits(h1), _bits(o1)) and torch.equal(_bits(h2), _bits(o3))
    assert torch.equal(_bits(o4), _bits(o1)) and torch.equal(_bits(o5), _bits(o1))
    # ---- the fused cache write of two "models" against the ctypes path -----------------------
    pa, pb = [allocate_gpu_cache(N, bs, DEV, dtype=dtype) for _ in range(2)]
    for kp, vp in (pa, pb):
        kp.zero_()
        vp.zero_()
    xa, xb = qkv.clone(), qkv.clone()
    qa, ka, va = xa.split([Hq * D, Hkv * D, Hkv * D], dim=-1)
    qb, kb, vb = xb.split([Hq * D, Hkv * D, Hkv * D], dim=-1)
    ops.multi_reshape_and_cache([ops.CacheWriteCall(ka, va, slots, layer=1, positions=positions, cos_sin=cos_sin, q=qa,
                                                    num_tokens=n)], pa[0], pa[1])
    T.multi_reshape_and_cache([kb], [vb], pb[0], pb[1], [slots], [1], [n], [positions], [qb], [cos_sin])
    torch.cuda.synchronize()
    assert torch.equal(_bits(xa), _bits(xb)) and torch.equal(_bits(pa[0]), _bits(pb[0])) and \
        torch.equal(_bits(pa[1]), _bits(pb[1]))
    # ---- stand-alone rotary, greedy sampling ---------------------------------------------
    r1 = qkv.clone().split([Hq * D, Hkv * D, Hkv * D], dim=-1)
    r2 = qkv.clone().split([Hq * D, Hkv * D, Hkv * D], dim=-1)
    ops.rotary_neox(positions, r1[0], r1[1], cos_sin, num_tokens=n)
    T.rotary_neox(positions, r2[0], r2[1], cos_sin, n)
    assert torch.equal(_bits(r1[0]), _bits(r2[0])) and torch.equal(_bits(r1[1]), _bits(r2[1]))
    V = 1000
    emb = (torch.randn((V + 8, 512), generator=g) * 0.1).to(dtype).to(DEV)
    hid = torch.randn((12, 512), generator=g).to(dtype).to(DEV)
    ri = torch.tensor([11, 0, 5], dtype=torch.int32, device=DEV)
    wss = torch.zeros((T.greedy_sample_workspace_bytes(V),), dtype=torch.uint8, device=DEV)
    none = torch.empty((0,), dtype=torch.int32, device=DEV)
    assert torch.equal(T.greedy_sample(emb, hid, V, 3, ri, wss), ops.greedy_sample(emb, hid, V, 3, row_index=ri))
    assert torch.equal(T.greedy_sample(emb, hid, V, 12, none, wss), ops.greedy_sample(emb, hid, V, 12))
    # ---- layer operators -----------------------------------------------------------------
    x = (torch.randn((9, 1024), generator=g) * 2).to(dtype).to(DEV)
    w = (1 + 0.1 * torch.randn((1024,), generator=g)).to(dtype).to(DEV)
    assert torch.equal(_bits(T.rms_norm(x, w, 1e-6)), _bits(ops.rms_norm(x, w, 1e-6)))
    assert torch.equal(_bits(T.silu_and_mul(x)), _bits(ops.silu_and_mul(x)))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_fused_prefill_operator_equals_the_ctypes_path(dtype):
    """torch.ops.muxserve_amd.multi_prefill_causal (three models of different head
    counts, one of them grouped-query, one without prompts) against
    muxserve_amd.ops.multi_prefill_causal: the same C entry point, bitwise equal."""
    print(f"[case] fused prefill operator {dtype}", flush=True)
    shapes = [(4, 4, [70, 1, 200]), (8, 2, [129, 33]), (2, 2, [])]
    via_ops, via_torch = [], []
    for mi, (Hq, Hkv, lens) in enumerate(shapes):
        g = torch.Generator().manual_seed(90 + mi)
        T_ = sum(lens)
        pad = (T_ + 7) // 8 * 8
        qkv = torch.randn((pad, (Hq + 2 * Hkv) * D), generator=g).to(dtype).to(DEV)
        q, k, v = qkv.split([Hq * D, Hkv * D, Hkv * D], dim=-1)
        cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]).astype(np.int32), device=DEV)
        for calls in (via_ops, via_torch):
            calls.append(ops.PrefillCall(torch.zeros((pad, Hq * D), dtype=dtype, device=DEV), q, k, v, cu, lens,
                                         D ** -0.5, Hkv))
    ops.multi_prefill_causal(via_ops)
    torch_ops.multi_prefill_causal(via_torch)
    torch.cuda.synchronize()
    for a, b, (_, _, lens) in zip(via_ops, via_torch, shapes):
        assert torch.equal(_bits(a.out), _bits(b.out))
        if lens:
            assert a.out[:sum(lens)].float().abs().sum().item() > 0
    # one list shorter than the others is refused
    T = torch_ops.load()
    c = via_torch[0]
    with pytest.raises(RuntimeError):
        T.multi_prefill_causal([c.out], [c.q], [c.k], [c.v], [c.cu_seqlens], [], [200], [1.0, 1.0], [4])


def test_torch_operators_refuse_bad_arguments():
    print("[case] torch operators, bad arguments", flush=True)
    T = torch_ops.load()
    k_pool, v_pool = allocate_gpu_cache(64, 16, DEV)
    k = torch.zeros((8, 2 * D), dtype=torch.float16, device=DEV)
    slots = torch.zeros((8, 1, 2), dtype=torch.int64, device=DEV)
    with pytest.raises(RuntimeError):
        T.reshape_and_cache(k, k, k_pool, v_pool, slots.int(), 0, 8)             # slots must be int64
    with pytest.raises(RuntimeError):
        T.reshape_and_cache(k, k, k_pool, v_pool, slots, 3, 8)                   # layer outside [0, L)
    with pytest.raises(RuntimeError):
        T.reshape_and_cache(k.float(), k.float(), k_pool, v_pool, slots, 0, 8)   # fp32 is not a storage type
    with pytest.raises((RuntimeError, NotImplementedError)):
        T.silu_and_mul(torch.zeros((2, 16), dtype=torch.float16))                # no CPU path
