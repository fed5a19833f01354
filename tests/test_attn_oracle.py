"""Pins oracle/attn_oracle.py with checks that do not retype its formulas:
closed forms worked by hand from the reference's pool definition, a brute-force
element loop, library SDPA on gathered tensors, and special cases whose answer
is known without computing attention.  CPU only.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import attn_oracle as orc
from muxserve_amd import pool, workloads

D = 128


def test_pool_geometry_closed_forms():
    # manager.py:456-468 at block_size 16, fp16: K [16,16,8], V [128,16]; a
    # head-block pair is 2*(2048+2048) = 8192 bytes (16384 at block size 32).
    assert orc.key_block_shape(16) == (16, 16, 8)
    assert orc.value_block_shape(16) == (128, 16)
    assert orc.key_block_shape(32) == (16, 32, 8)
    assert pool.key_block_shape(16) == (16, 16, 8) and pool.value_block_shape(8) == (128, 8)
    assert pool.block_bytes(16) == 8192 and pool.block_bytes(32) == 16384
    # N = ((round(util*mem) - 1) // 8192 // 128) * 128, e.g. 0.5 * 80 GiB:
    mem = 80 * 2**30
    assert orc.num_gpu_blocks(0.5, mem, 16) == ((mem // 2 - 1) // 8192 // 128) * 128 == 5242752
    # exactly one block pair short of a multiple of 128 rounds down a full 128
    assert orc.num_gpu_blocks(1.0, 8192 * 256, 16) == 128
    assert orc.num_gpu_blocks(1.0, 8192 * 256 + 1, 16) == 256
    for util, m, bs in [(0.6, 288 * 10**9, 16), (0.9, 192 * 2**30, 32), (0.3, 10**9, 8)]:
        assert pool.num_gpu_blocks(util, m, bs) == orc.num_gpu_blocks(util, m, bs)


def test_element_offsets_match_documented_layout():
    """K element (b, o, d) sits at ((b*(D/8) + d//8)*bs + o)*8 + d%8, V element
    at (b*D + d)*bs + o (flat element offsets of the pool tensors)."""
    bs, N = 16, 5
    k_pool, v_pool = orc.allocate_pool(N, bs)
    k_pool.zero_()
    v_pool.zero_()
    k = torch.arange(1, 1 + 2 * D, dtype=torch.float32).reshape(1, 2 * D).half()
    slot = torch.tensor([[[3 * bs + 5, 1 * bs + 15]]], dtype=torch.int64)    # T=1, L=1, H=2
    orc.reshape_and_cache(k, k + 1000, k_pool, v_pool, slot)
    kf, vf = k_pool.reshape(-1), v_pool.reshape(-1)
    for h, (b, o) in enumerate([(3, 5), (1, 15)]):
        for d in (0, 1, 7, 8, 63, 127):
            assert kf[((b * 16 + d // 8) * bs + o) * 8 + d % 8] == k[0, h * D + d]
            assert vf[(b * D + d) * bs + o] == (k + 1000)[0, h * D + d]
    assert int((kf != 0).sum()) == 2 * D and int((vf != 0).sum()) == 2 * D   # nothing else touched


@pytest.mark.parametrize("bs", [8, 16, 32])
def test_cache_write_matches_element_loop_and_roundtrips(bs):
    rng = np.random.Generator(np.random.PCG64(bs))
    g = torch.Generator().manual_seed(bs)
    T, L, H, N = 9, 2, 3, 20
    slots = torch.from_numpy(rng.permutation(N * bs)[:T * L * H].reshape(T, L, H).astype(np.int64))
    slots[2, 1, 1] = -1
    k = torch.randn((T, H * D), generator=g).half()
    v = torch.randn((T, H * D), generator=g).half()
    a = [torch.zeros(s, dtype=torch.float16) for s in ((N, 16, bs, 8), (N, D, bs))]
    b = [t.clone() for t in a]
    orc.reshape_and_cache(k, v, a[0], a[1], slots, layer=1)
    orc.reshape_and_cache_loops(k, v, b[0], b[1], slots, layer=1)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    # read back through gather_kv: one-token "sequences"
    for t in range(T):
        for h in range(H):
            s = int(slots[t, 1, h])
            if s < 0:
                continue
            K, V = orc.gather_kv(a[0], a[1], torch.tensor([s // bs], dtype=torch.int32), bs)
            assert torch.equal(K[s % bs], k[t, h * D:(h + 1) * D])
            assert torch.equal(V[s % bs], v[t, h * D:(h + 1) * D])


def _dense_case(seed, ctx_lens, Hq, Hkv, bs):
    rng = np.random.Generator(np.random.PCG64(seed))
    g = torch.Generator().manual_seed(seed)
    ctx = np.asarray(ctx_lens, dtype=np.int32)
    need = int(((ctx + bs - 1) // bs).sum()) * Hkv
    N = need + 3
    ids = rng.permutation(N)[:need]
    bt, _ = workloads.build_tables(ctx, Hkv, bs, ids)
    k_pool = torch.full((N, 16, bs, 8), float("nan"), dtype=torch.float16)
    v_pool = torch.full((N, D, bs), float("nan"), dtype=torch.float16)
    dense = []
    for s, n in enumerate(ctx):
        n = int(n)
        kd = torch.randn((n, Hkv * D), generator=g).half()
        vd = torch.randn((n, Hkv * D), generator=g).half()
        i = np.arange(n)
        slots = bt[0, s][:, i // bs].astype(np.int64).T * bs + (i % bs)[:, None]
        orc.reshape_and_cache(kd, vd, k_pool, v_pool, torch.from_numpy(slots[:, None, :]))
        dense.append((kd, vd))
    q = torch.randn((len(ctx), Hq * D), generator=g).half()
    return q, k_pool, v_pool, bt, ctx, dense


@pytest.mark.parametrize("Hq,Hkv,bs", [(4, 4, 16), (8, 2, 16), (6, 3, 8), (4, 1, 32)])
def test_paged_decode_equals_library_sdpa_on_dense_kv(Hq, Hkv, bs):
    q, k_pool, v_pool, bt, ctx, dense = _dense_case(1, [1, 5, 16, 17, 100], Hq, Hkv, bs)
    scale = D ** -0.5
    got = orc.paged_decode(q, k_pool, v_pool, torch.from_numpy(bt), ctx, scale)
    ratio = Hq // Hkv
    for s, (kd, vd) in enumerate(dense):
        n = kd.shape[0]
        qs = q[s].float().reshape(1, Hq, 1, D)
        ks = kd.float().reshape(n, Hkv, D).permute(1, 0, 2).repeat_interleave(ratio, dim=0)[None]
        vs = vd.float().reshape(n, Hkv, D).permute(1, 0, 2).repeat_interleave(ratio, dim=0)[None]
        want = F.scaled_dot_product_attention(qs, ks, vs, scale=scale).reshape(-1)
        assert torch.allclose(got[s], want, atol=2e-6, rtol=1e-5)
    assert torch.isfinite(got).all()     # NaN poison outside valid tokens never leaks


def test_paged_decode_special_cases():
    q, k_pool, v_pool, bt, ctx, dense = _dense_case(2, [1, 40], 2, 2, 16)
    scale = D ** -0.5
    out = orc.paged_decode(q, k_pool, v_pool, torch.from_numpy(bt), ctx, scale)
    assert torch.equal(out[0], dense[0][1][0].float())            # ctx == 1  =>  out == V[0]
    # one key aligned with q and scaled up dominates: out ~= its value
    kd, vd = dense[1]
    j = 23
    kd2 = kd.clone()
    kd2[j] = (q[1].float() * 8).half()
    k2, v2 = k_pool.clone(), v_pool.clone()
    i = np.arange(40)
    slots = bt[0, 1][:, i // 16].astype(np.int64).T * 16 + (i % 16)[:, None]
    orc.reshape_and_cache(kd2, vd, k2, v2, torch.from_numpy(slots[:, None, :]))
    out2 = orc.paged_decode(q, k2, v2, torch.from_numpy(bt), ctx, scale)
    assert torch.allclose(out2[1], vd[j].float(), atol=1e-3)


def test_paged_decode_invariant_under_block_relabelling():
    q, k_pool, v_pool, bt, ctx, _ = _dense_case(3, [33, 70, 9], 4, 2, 16)
    N = k_pool.shape[0]
    perm = torch.from_numpy(np.random.Generator(np.random.PCG64(9)).permutation(N))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(N)
    # new pool: block perm[i] of the new pool holds old block i
    k2, v2 = torch.empty_like(k_pool), torch.empty_like(v_pool)
    k2[perm] = k_pool
    v2[perm] = v_pool
    bt2 = np.where(bt >= 0, perm.numpy()[np.clip(bt, 0, N - 1)], bt).astype(np.int32)
    a = orc.paged_decode(q, k_pool, v_pool, torch.from_numpy(bt), ctx, 0.1)
    b = orc.paged_decode(q, k2, v2, torch.from_numpy(bt2), ctx, 0.1)
    assert torch.equal(a, b)


@pytest.mark.parametrize("Hq,Hkv", [(3, 3), (4, 2)])
def test_prefill_equals_library_causal_sdpa_and_is_block_diagonal(Hq, Hkv):
    g = torch.Generator().manual_seed(4)
    lens = [1, 7, 64, 33]
    T = sum(lens)
    q = torch.randn((T + 3, Hq * D), generator=g).half()
    k = torch.randn((T + 3, Hkv * D), generator=g).half()
    v = torch.randn((T + 3, Hkv * D), generator=g).half()
    scale = D ** -0.5
    got = orc.prefill_causal(q, k, v, lens, scale, Hkv)
    ratio = Hq // Hkv
    start = 0
    for n in lens:
        qs = q[start:start + n].float().reshape(n, Hq, D).permute(1, 0, 2)[None]
        ks = k[start:start + n].float().reshape(n, Hkv, D).permute(1, 0, 2).repeat_interleave(ratio, 0)[None]
        vs = v[start:start + n].float().reshape(n, Hkv, D).permute(1, 0, 2).repeat_interleave(ratio, 0)[None]
        want = F.scaled_dot_product_attention(qs, ks, vs, is_causal=True, scale=scale)[0]
        assert torch.allclose(got[start:start + n], want.permute(1, 0, 2).reshape(n, -1), atol=3e-6, rtol=1e-5)
        start += n
    # first token of every prompt attends only to itself
    start = 0
    for n in lens:
        for h in range(Hq):
            assert torch.allclose(got[start, h * D:(h + 1) * D],
                                  v[start, (h // ratio) * D:(h // ratio + 1) * D].float(), atol=1e-6)
        start += n
    # changing one prompt leaves the others' outputs bit-identical
    k2 = k.clone()
    k2[lens[0]:lens[0] + lens[1]] += 1
    got2 = orc.prefill_causal(q, k2, v, lens, scale, Hkv)
    assert torch.equal(got2[:lens[0]], got[:lens[0]])
    assert torch.equal(got2[lens[0] + lens[1]:], got[lens[0] + lens[1]:])


def test_traffic_formulas():
    # one sequence of 100 tokens, 4 q heads over 2 kv heads, block size 16:
    # K+V 2*100*2*128*2 = 102400; q+out 2*4*128*2 = 2048; table 2*7*4 = 56; ctx 4
    assert orc.decode_bytes([100], 4, 2, 16) == 102400 + 2048 + 56 + 4
    assert orc.cache_write_bytes(10, 3) == 10 * 3 * 1032


def test_workload_generators_are_seeded_and_head_granular():
    m1, n1 = workloads.config1(seed=0)
    m1b, _ = workloads.config1(seed=0)
    assert np.array_equal(m1[0].block_tables, m1b[0].block_tables)
    ctx = m1[0].context_lens
    assert ctx.min() >= 64 and ctx.max() <= 512 and len(ctx) == 8
    used = m1[0].used_blocks(16)
    assert len(np.unique(used)) == len(used) and used.max() < n1
    # group g owns head-blocks g*32 + h
    bt = m1[0].block_tables[0, 0]
    assert (bt[:, 0] - bt[0, 0] == np.arange(32)).all() and bt[0, 0] % 32 == 0
    ms, need = workloads.config2(seed=1, num_pool_blocks=1_000_000)
    allu = np.concatenate([m.used_blocks(16) for m in ms])
    assert len(np.unique(allu)) == len(allu) == need
    assert [m.batch for m in ms] == [32, 16, 8] and [m.num_kv_heads for m in ms] == [32, 40, 52]
    for m in ms:
        assert m.context_lens.min() >= 16 and m.context_lens.max() <= 2048


def test_rotary_oracle_is_a_complex_rotation():
    """NeoX RoPE pairs (x_i, x_{i+64}) and multiplies x_i + j x_{i+64} by
    exp(j p f_i): checked with complex arithmetic, plus position 0 = identity,
    norm preservation and the relative-position property of q.k."""
    g = torch.Generator().manual_seed(7)
    T, H = 6, 3
    pos = torch.tensor([0, 1, 2, 17, 300, 2047])
    q = torch.randn((T, H * D), generator=g).half()
    k = torch.randn((T, 2 * D), generator=g).half()
    rq, rk = orc.rotary_neox(pos, q, k, rotary_dim=D, base=10000.0)
    f = 10000.0 ** (-torch.arange(0, D, 2, dtype=torch.float64) / D)
    x = q.double().reshape(T, H, D)
    z = torch.complex(x[..., :64], x[..., 64:]) * torch.polar(torch.ones(T, 64, dtype=torch.float64),
                                                               pos.double()[:, None] * f)[:, None, :]
    want = torch.cat([z.real, z.imag], dim=-1).reshape(T, H * D)
    assert torch.allclose(rq.double(), want, atol=2e-6)
    assert torch.equal(rq[0], q[0].float())                                  # position 0
    assert torch.allclose(rq.reshape(T, H, D).norm(dim=-1), q.float().reshape(T, H, D).norm(dim=-1), rtol=1e-5)
    # <rope(a, m), rope(b, n)> depends only on m - n
    a = torch.randn((1, D), generator=g)
    b = torch.randn((1, D), generator=g)
    def dot(m, n):
        ra, _ = orc.rotary_neox(torch.tensor([m]), a, a)
        rb, _ = orc.rotary_neox(torch.tensor([n]), b, b)
        return float((ra * rb).sum())
    assert abs(dot(5, 2) - dot(103, 100)) < 1e-3 and abs(dot(5, 2) - dot(6, 2)) > 1e-4


def test_traffic_formulas_of_the_package_agree_with_the_oracle():
    """bench.py prices throughput with muxserve_amd.workloads' formulas; the
    oracle holds its own statement of the same definitions."""
    from muxserve_amd import workloads
    rng = np.random.Generator(np.random.PCG64(5))
    for Hq, Hkv, bs in ((32, 32, 16), (64, 8, 16), (40, 40, 8), (52, 52, 32)):
        ctx = rng.integers(1, 3000, size=37)
        assert workloads.decode_bytes(ctx, Hq, Hkv, bs) == orc.decode_bytes(ctx, Hq, Hkv, bs)
        assert workloads.cache_write_bytes(int(ctx.sum()), Hkv) == orc.cache_write_bytes(int(ctx.sum()), Hkv)
    # one sequence by hand: 100 tokens, 2 kv heads, 4 q heads, 16-token blocks
    assert workloads.decode_bytes([100], 4, 2, 16) == 2 * 100 * 2 * 128 * 2 + 2 * 4 * 128 * 2 + 2 * 7 * 4 + 4
    assert workloads.cache_write_bytes(3, 2) == 3 * 2 * 1032
    assert workloads.prefill_flops([1, 3], 2) == 4.0 * 2 * 128 * (1 + 6)
