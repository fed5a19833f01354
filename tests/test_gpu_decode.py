"""GPU parity: KV-cache write (bit-exact) and paged decode attention (<= 2e-3
max-abs, fp16/bf16 storage with fp32 accumulation) against the CPU oracle, all
through the C ABI of libmuxattn.so.
"""
import numpy as np
import pytest
import torch

from oracle import attn_oracle as orc
from muxserve_amd import ops, workloads
from muxserve_amd.pool import HEAD_SIZE, allocate_gpu_cache, num_gpu_blocks

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 2e-3   # max-abs bar of the decode path


def _announce(msg):
    print(f"[case] {msg}", flush=True)


def _nan_pool(n, bs, dtype):
    k, v = orc.allocate_pool(n, bs, dtype)
    k.fill_(float("nan"))
    v.fill_(float("nan"))
    return k, v


def _decode_case(seed, ctx_lens, Hq, Hkv, bs, dtype=torch.float16, partition=0, num_layers=1, layer=0,
                 q_in_qkv=False, extra_blocks=7, hint=False, repeat=1, host_lens=False):
    """Builds pool + tables on the host with the oracle's cache write, runs the
    GPU decode, returns (gpu_out fp32, oracle_out fp32)."""
    rng = np.random.Generator(np.random.PCG64(seed))
    g = torch.Generator().manual_seed(seed)
    B = len(ctx_lens)
    ctx = np.asarray(ctx_lens, dtype=np.int32)
    nblk = (ctx.astype(np.int64) + bs - 1) // bs
    need = int(nblk.sum()) * Hkv
    N = need + extra_blocks
    ids = rng.permutation(N)[:need]
    bt1, _ = workloads.build_tables(ctx, Hkv, bs, ids)
    max_blocks = bt1.shape[-1]
    bt = np.full((num_layers, B, Hkv, max_blocks), workloads.POISON_BLOCK, dtype=np.int32)
    bt[layer] = bt1[0]
    k_pool, v_pool = _nan_pool(N, bs, dtype)
    # dense K/V per sequence -> written through the oracle's cache write
    for s in range(B):
        n = int(ctx[s])
        kd = torch.randn((n, Hkv * HEAD_SIZE), generator=g).to(dtype)
        vd = torch.randn((n, Hkv * HEAD_SIZE), generator=g).to(dtype)
        i = np.arange(n)
        slots = bt1[0, s][:, i // bs].astype(np.int64).T * bs + (i % bs)[:, None]     # [n, Hkv]
        orc.reshape_and_cache(kd, vd, k_pool, v_pool, torch.from_numpy(slots[:, None, :]))
    pad = (B + 7) // 8 * 8
    if q_in_qkv:
        qkv = torch.randn((pad, (Hq + 2 * Hkv) * HEAD_SIZE), generator=g).to(dtype)
        q = qkv[:, :Hq * HEAD_SIZE]
    else:
        q = torch.randn((pad, Hq * HEAD_SIZE), generator=g).to(dtype)
    scale = HEAD_SIZE ** -0.5
    want = orc.paged_decode(q, k_pool, v_pool, torch.from_numpy(bt), ctx, scale, layer=layer)

    dq = (qkv.to(DEV)[:, :Hq * HEAD_SIZE]) if q_in_qkv else q.to(DEV)
    out = torch.full((pad, Hq * HEAD_SIZE), 7.0, dtype=dtype, device=DEV)
    dkp, dvp, dbt, dctx = k_pool.to(DEV), v_pool.to(DEV), torch.from_numpy(bt).to(DEV), torch.from_numpy(ctx).to(DEV)
    for _ in range(repeat):     # repeated launches reuse the workspace (arrival counters must self-reset)
        out.fill_(7.0)
        ops.paged_decode(out, dq, dkp, dvp, dbt, dctx, int(ctx.max()), scale, layer=layer,
                         partition_size=partition, total_context_len=int(ctx.sum()) if hint else 0,
                         context_lens_host=torch.from_numpy(ctx) if host_lens else None)
    torch.cuda.synchronize()
    got = out.float().cpu()
    assert (got[B:] == 7.0).all(), "padding rows of out must not be written"
    return got[:B], want


def _check(got, want, tol=TOL, out_dtype=torch.float16):
    """|got - want| <= 2e-3, plus, for bf16 outputs only, the rounding of the
    result to its 8-bit mantissa (half an ulp = 2^-9 relative, taken as 2^-8
    to cover values just below a power of two)."""
    assert torch.isfinite(got).all()
    bound = torch.full_like(want, tol)
    if out_dtype == torch.bfloat16:
        bound = bound + want.abs() * 2.0 ** -8
    excess = ((got - want).abs() - bound).max().item()
    err = (got - want).abs().max().item()
    assert excess <= 0, f"max-abs error {err:.3e} exceeds {tol} (+ output rounding) by {excess:.3e}"
    return err


# ---- KV-cache write: bit-exact ---------------------------------------------------

@pytest.mark.parametrize("bs", [16, 8, 32])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_reshape_and_cache_bit_exact_random_slots(bs, dtype):
    _announce(f"reshape_and_cache random slots bs={bs} {dtype}")
    rng = np.random.Generator(np.random.PCG64(bs))
    g = torch.Generator().manual_seed(bs)
    T, L, H, layer, N = 37, 3, 5, 1, 300
    slots = rng.permutation(N * bs)[:T * L * H].reshape(T, L, H).astype(np.int64)
    slots[3, layer, 2] = -1                      # skipped slot
    pad = 40
    qkv = torch.randn((pad, (H + 2 * H) * HEAD_SIZE), generator=g).to(dtype)
    k = qkv[:, H * HEAD_SIZE:2 * H * HEAD_SIZE]
    v = qkv[:, 2 * H * HEAD_SIZE:]
    k_pool, v_pool = orc.allocate_pool(N, bs, dtype)
    k_pool.copy_(torch.randn(k_pool.shape, generator=g).to(dtype))
    v_pool.copy_(torch.randn(v_pool.shape, generator=g).to(dtype))
    dk, dv = k_pool.to(DEV), v_pool.to(DEV)
    dqkv = qkv.to(DEV)
    ops.reshape_and_cache(dqkv[:, H * HEAD_SIZE:2 * H * HEAD_SIZE], dqkv[:, 2 * H * HEAD_SIZE:], dk, dv,
                          torch.from_numpy(slots).to(DEV), layer=layer)
    torch.cuda.synchronize()
    orc.reshape_and_cache(k, v, k_pool, v_pool, torch.from_numpy(slots), layer=layer)
    assert torch.equal(dk.cpu().view(torch.int16), k_pool.view(torch.int16))
    assert torch.equal(dv.cpu().view(torch.int16), v_pool.view(torch.int16))


@pytest.mark.parametrize("bs", [16, 8, 32])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_reshape_and_cache_bit_exact_runs_of_consecutive_slots(bs, dtype):
    """Runs of consecutive slots take the 16-byte V store path when 8 tokens
    that the kernel groups together start a pool chunk; every way of almost
    qualifying (misaligned start, a skipped token inside, a run broken in the
    middle, a run cut by the end of the batch, reversed order) must fall back
    to the element path and still match the oracle bitwise."""
    _announce(f"reshape_and_cache slot runs bs={bs} {dtype}")
    g = torch.Generator().manual_seed(100 + bs)
    L, H, layer, N = 2, 3, 1, 64
    per_head = []
    for h in range(H):
        base = (h * 20 + 1) * bs                       # block-aligned, blocks disjoint between heads
        col = np.concatenate([
            base + np.arange(16),                      # tokens 0-15: two aligned chunks
            base + 16 + 3 + np.arange(8),              # 16-23: consecutive but misaligned start
            base + 32 + np.arange(8),                  # 24-31: aligned ...
            base + 48 + np.arange(8)[::-1],            # 32-39: right slots, reversed order
            base + 64 + np.arange(8),                  # 40-47: aligned, one token skipped below
            base + 80 + np.array([0, 1, 2, 3, 12, 13, 14, 15]),   # 48-55: broken in the middle
            base + 96 + np.arange(5),                  # 56-60: run cut by the end of the batch
        ]).astype(np.int64)
        per_head.append(col)
    T = len(per_head[0])
    slots = np.full((T, L, H), -1, dtype=np.int64)
    for h in range(H):
        slots[:, layer, h] = per_head[h]
    slots[43, layer, 1] = -1
    slots[:, 0, :] = 7                                 # another layer's column must be ignored
    pad = (T + 7) // 8 * 8
    k = torch.randn((pad, H * HEAD_SIZE), generator=g).to(dtype)
    v = torch.randn((pad, H * HEAD_SIZE), generator=g).to(dtype)
    k_pool, v_pool = orc.allocate_pool(N, bs, dtype)
    k_pool.copy_(torch.randn(k_pool.shape, generator=g).to(dtype))
    v_pool.copy_(torch.randn(v_pool.shape, generator=g).to(dtype))
    dk, dv = k_pool.to(DEV), v_pool.to(DEV)
    ops.reshape_and_cache(k.to(DEV), v.to(DEV), dk, dv, torch.from_numpy(slots).to(DEV), layer=layer, num_tokens=T)
    torch.cuda.synchronize()
    orc.reshape_and_cache(k, v, k_pool, v_pool, torch.from_numpy(slots), layer=layer, num_tokens=T)
    assert torch.equal(dk.cpu().view(torch.int16), k_pool.view(torch.int16))
    assert torch.equal(dv.cpu().view(torch.int16), v_pool.view(torch.int16))


@pytest.mark.parametrize("bs", [16, 8, 32])
def test_reshape_and_cache_bit_exact_packed_ragged_prompts(bs):
    """Prompts of every length 1..40 packed back to back: slot runs begin at
    every phase of the kernel's 16-token grid and end in partial chunks."""
    _announce(f"reshape_and_cache packed ragged prompts bs={bs}")
    rng = np.random.Generator(np.random.PCG64(200 + bs))
    g = torch.Generator().manual_seed(200 + bs)
    H = 3
    lens = rng.permutation(np.arange(1, 41)).astype(np.int32)
    T = int(lens.sum())
    N = int(((lens + bs - 1) // bs).sum()) * H + 9
    ids = rng.permutation(N)
    slots, used = workloads.prefill_slot_mapping(lens, H, bs, ids)
    assert slots.shape == (T, 1, H)
    pad = (T + 7) // 8 * 8
    k = torch.randn((pad, H * HEAD_SIZE), generator=g).half()
    v = torch.randn((pad, H * HEAD_SIZE), generator=g).half()
    k_pool, v_pool = orc.allocate_pool(N, bs, torch.float16)
    k_pool.copy_(torch.randn(k_pool.shape, generator=g).half())
    v_pool.copy_(torch.randn(v_pool.shape, generator=g).half())
    dk, dv = k_pool.to(DEV), v_pool.to(DEV)
    ops.reshape_and_cache(k.to(DEV), v.to(DEV), dk, dv, torch.from_numpy(slots).to(DEV), num_tokens=T)
    torch.cuda.synchronize()
    orc.reshape_and_cache(k, v, k_pool, v_pool, torch.from_numpy(slots), num_tokens=T)
    assert torch.equal(dk.cpu().view(torch.int16), k_pool.view(torch.int16))
    assert torch.equal(dv.cpu().view(torch.int16), v_pool.view(torch.int16))


def test_reshape_and_cache_prefill_pattern_roundtrip():
    """Prompt-shaped slots (token i -> block i//bs, offset i%bs per head), then
    gather back through the tables: gather(scatter(x)) == x bitwise."""
    _announce("reshape_and_cache prefill roundtrip")
    bs, H = 16, 4
    rng = np.random.Generator(np.random.PCG64(5))
    g = torch.Generator().manual_seed(5)
    lens = np.array([1, 16, 17, 100, 31], dtype=np.int32)
    N = 400
    ids = rng.permutation(N)
    slots, used = workloads.prefill_slot_mapping(lens, H, bs, ids)
    T = int(lens.sum())
    k = torch.randn((T, H * HEAD_SIZE), generator=g).half()
    v = torch.randn((T, H * HEAD_SIZE), generator=g).half()
    dk, dv = allocate_gpu_cache(N, bs, DEV)
    dk.zero_()
    dv.zero_()
    ops.reshape_and_cache(k.to(DEV), v.to(DEV), dk, dv, torch.from_numpy(slots).to(DEV))
    torch.cuda.synchronize()
    hk, hv = dk.cpu(), dv.cpu()
    start, cur = 0, 0
    for n in lens:
        n = int(n)
        nblk = (n + bs - 1) // bs
        blk = ids[cur:cur + nblk * H].reshape(nblk, H)
        cur += nblk * H
        for h in range(H):
            K, V = orc.gather_kv(hk, hv, torch.from_numpy(blk[:, h].astype(np.int32)), n)
            assert torch.equal(K, k[start:start + n, h * HEAD_SIZE:(h + 1) * HEAD_SIZE])
            assert torch.equal(V, v[start:start + n, h * HEAD_SIZE:(h + 1) * HEAD_SIZE])
        start += n


# ---- paged decode ------------------------------------------------------------------

def test_decode_config1_shape():
    """7B layer, 32 heads, batch 8, ctx ~ U{64..512}, block size 16."""
    _announce("decode config 1")
    models, N = workloads.config1(seed=0)
    m = models[0]
    got, want = _decode_case(1, m.context_lens, 32, 32, 16)
    _check(got, want)


def test_decode_config1_with_its_own_tables():
    """The same configuration with the tables the workload itself defines: one
    seeded permutation of a 4096-group pool (4096 * 32 head-blocks), a token
    block's 32 heads at ids group * 32 + head.  Checked against the oracle
    reading the same pool through the same tables."""
    _announce("decode config 1, own tables")
    bs = 16
    models, N = workloads.config1(seed=0)
    m = models[0]
    assert N == 4096 * 32 and m.block_tables.shape[:3] == (1, 8, 32)
    groups = m.block_tables[0, :, 0, :] // 32
    for s, c in enumerate(m.context_lens):
        n = (int(c) + bs - 1) // bs
        assert (m.block_tables[0, s, :, :n] == groups[s, :n][None, :] * 32 + np.arange(32)[:, None]).all()
    dk, dv = allocate_gpu_cache(N, bs, DEV)
    dk.fill_(float("nan"))
    dv.fill_(float("nan"))
    workloads.fill_blocks(dk, dv, m.used_blocks(bs), seed=1)
    m.to_device(DEV, torch.float16, seed=2)
    for host_lens in (None, torch.from_numpy(np.ascontiguousarray(m.context_lens, dtype=np.int32))):
        m.out.fill_(7.0)
        ops.paged_decode(m.out, m.q, dk, dv, m.d_block_tables, m.d_context_lens, m.max_context_len, m.scale,
                         context_lens_host=host_lens)
        torch.cuda.synchronize()
        want = orc.paged_decode(m.q.cpu(), dk.cpu(), dv.cpu(), torch.from_numpy(m.block_tables), m.context_lens,
                                m.scale)
        _check(m.out[:m.batch].float().cpu(), want)


@pytest.mark.parametrize("ctx", [[1], [2, 15, 16, 17], [63, 64, 65, 127, 128, 129], [255, 256, 257, 300]])
def test_decode_boundaries(ctx):
    _announce(f"decode boundaries ctx={ctx}")
    got, want = _decode_case(2, ctx, 4, 4, 16)
    _check(got, want)


@pytest.mark.parametrize("partition", [64, 128, 256, 512])
def test_decode_split_context_equals_single_pass(partition):
    _announce(f"decode split partition={partition}")
    ctx = [1, 64, 65, 200, 513, 777, 1024, 1500]
    got, want = _decode_case(3, ctx, 3, 3, 16, partition=partition)
    _check(got, want)


@pytest.mark.parametrize("Hq,Hkv,dtype,partition", [(3, 3, torch.float16, 0), (4, 2, torch.bfloat16, 64),
                                                     (8, 1, torch.float16, 128), (5, 5, torch.bfloat16, 512)])
def test_decode_units_enumerated_on_the_host_equal_units_enumerated_on_the_device(Hq, Hkv, dtype, partition):
    """With a host copy of the context lengths the (sequence, partition) pairs
    travel in the kernel argument; the result must be the one the device-side
    enumeration gives, bit for bit, and match the oracle.  Contexts cover no
    tokens at all, one token, tile and partition boundaries, exact multiples
    (no remainder unit) and long splits."""
    _announce(f"decode host-enumerated units Hq={Hq} Hkv={Hkv} {dtype} partition={partition}")
    ctx = [1, 0, 64, 65, 200, 256, 257, 512, 513, 777, 0, 1024, 1500, 16]
    dev_got, want = _decode_case(11, ctx, Hq, Hkv, 16, dtype=dtype, partition=partition, repeat=2)
    host_got, _ = _decode_case(11, ctx, Hq, Hkv, 16, dtype=dtype, partition=partition, repeat=2, host_lens=True)
    live = torch.tensor(ctx) > 0
    assert torch.equal(host_got[live], dev_got[live])
    _check(host_got[live], want[live], out_dtype=dtype)
    assert (host_got[~live] == 7.0).all(), "sequences without tokens must not be written"


def test_decode_host_lens_too_many_pairs_falls_back_to_the_device_enumeration():
    """More pairs than the kernel argument holds (here 400 sequences): the call
    silently takes the device-side path and still matches the oracle."""
    _announce("decode host lens, 400 sequences")
    rng = np.random.Generator(np.random.PCG64(5))
    ctx = rng.integers(1, 200, size=400)
    got, want = _decode_case(12, ctx, 2, 2, 16, partition=128, host_lens=True)
    _check(got, want)


@pytest.mark.parametrize("B", [65, 130, 300])
@pytest.mark.parametrize("hint", [False, True])
def test_decode_more_sequences_than_a_wave(B, hint):
    """Unit enumeration keeps up to 256 context lengths in registers and walks
    larger batches 64 sequences at a time."""
    _announce(f"decode B={B} hint={hint}")
    rng = np.random.Generator(np.random.PCG64(B))
    ctx = rng.integers(1, 400, size=B)
    ctx[::7] = 128          # exact multiples of the partition: no remainder unit
    ctx[3] = 1
    got, want = _decode_case(7, ctx, 2, 2, 16, partition=128, hint=hint, repeat=3)
    _check(got, want)


@pytest.mark.parametrize("bs", [8, 32])
def test_decode_other_block_sizes(bs):
    _announce(f"decode bs={bs}")
    got, want = _decode_case(4, [1, 7, 8, 9, 31, 32, 33, 100, 400], 3, 3, bs, partition=128)
    _check(got, want)


@pytest.mark.parametrize("Hq,Hkv", [(8, 4), (8, 2), (16, 2), (6, 2), (64, 8), (32, 2), (32, 1)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_decode_gqa(Hq, Hkv, dtype):
    _announce(f"decode gqa Hq={Hq} Hkv={Hkv} {dtype}")
    got, want = _decode_case(5, [5, 64, 130, 700], Hq, Hkv, 16, dtype=dtype, partition=256)
    _check(got, want, out_dtype=dtype)


@pytest.mark.parametrize("bs", [8, 32])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_decode_gqa_other_block_sizes(bs, dtype):
    """The matrix-core path (4 or more query heads per kv head) at every block size,
    with contexts around the block, tile and partition boundaries."""
    _announce(f"decode gqa bs={bs} {dtype}")
    got, want = _decode_case(8, [1, 7, 8, 9, 31, 32, 33, 63, 64, 65, 100, 128, 129, 400], 8, 2, bs,
                             dtype=dtype, partition=128, repeat=2)
    _check(got, want, out_dtype=dtype)


def test_decode_gqa_short_contexts_keep_probability_precision():
    """One to three keys: probabilities near 1 must not lose mantissa bits on
    their way into the P.V product (bf16 carries them as hi + lo parts)."""
    _announce("decode gqa short contexts bf16")
    got, want = _decode_case(11, [1, 2, 3, 2, 1, 3], 16, 2, 16, dtype=torch.bfloat16)
    _check(got, want, out_dtype=torch.bfloat16)


def test_decode_layer_slice_and_strided_q():
    """layer_idx selects block_tables[l]; q is a column slice of a qkv row."""
    _announce("decode layer slice + strided q")
    got, want = _decode_case(6, [40, 300, 17], 5, 5, 16, num_layers=3, layer=2, q_in_qkv=True)
    _check(got, want)


def test_decode_identical_keys_gives_mean_of_values():
    _announce("decode identical keys")
    bs, H, ctx = 16, 2, 150
    N = 64
    k_pool, v_pool = _nan_pool(N, bs, torch.float16)
    g = torch.Generator().manual_seed(9)
    key = torch.randn(H * HEAD_SIZE, generator=g).half()
    vals = torch.randn((ctx, H * HEAD_SIZE), generator=g).half()
    ids = np.arange(N)[::-1].copy()
    bt, _ = workloads.build_tables([ctx], H, bs, ids)
    i = np.arange(ctx)
    slots = bt[0, 0][:, i // bs].astype(np.int64).T * bs + (i % bs)[:, None]
    orc.reshape_and_cache(key.expand(ctx, -1).contiguous(), vals, k_pool, v_pool,
                          torch.from_numpy(slots[:, None, :]))
    q = torch.randn((8, H * HEAD_SIZE), generator=g).half()
    out = torch.zeros((8, H * HEAD_SIZE), dtype=torch.float16, device=DEV)
    ops.paged_decode(out, q.to(DEV), k_pool.to(DEV), v_pool.to(DEV), torch.from_numpy(bt).to(DEV),
                     torch.tensor([ctx], dtype=torch.int32, device=DEV), ctx, HEAD_SIZE ** -0.5,
                     partition_size=64)
    torch.cuda.synchronize()
    _check(out[:1].float().cpu(), vals.float().mean(dim=0, keepdim=True))


def test_multi_decode_three_models_one_launch_matches_separate_launches():
    _announce("multi decode 3 models")
    bs = 16
    models, need = workloads.config2(seed=3, num_pool_blocks=20000, batches=(6, 4, 3))
    N = 20000
    dk, dv = allocate_gpu_cache(N, bs, DEV)
    dk.fill_(float("nan"))
    dv.fill_(float("nan"))
    used = np.concatenate([m.used_blocks(bs) for m in models])
    assert len(np.unique(used)) == len(used) == need
    workloads.fill_blocks(dk, dv, used, seed=3)
    for i, m in enumerate(models):
        m.to_device(DEV, torch.float16, seed=10 + i)
    calls = [ops.DecodeCall(m.out, m.q, m.d_block_tables, m.d_context_lens, m.max_context_len, m.scale)
             for m in models]
    ops.multi_decode(calls, dk, dv, partition_size=256)
    torch.cuda.synchronize()
    fused = [m.out.clone() for m in models]
    for m in models:
        m.out.zero_()
        ops.paged_decode(m.out, m.q, dk, dv, m.d_block_tables, m.d_context_lens, m.max_context_len, m.scale,
                         partition_size=256)
    torch.cuda.synchronize()
    # The same fused launch with the units enumerated on the host.
    host_calls = [ops.DecodeCall(m.out, m.q, m.d_block_tables, m.d_context_lens, m.max_context_len, m.scale,
                                 context_lens_host=torch.from_numpy(np.ascontiguousarray(m.context_lens, dtype=np.int32)))
                  for m in models]
    separate = [m.out.clone() for m in models]
    for m in models:
        m.out.zero_()
    ops.multi_decode(host_calls, dk, dv, partition_size=256)
    torch.cuda.synchronize()
    for m, sep in zip(models, separate):
        assert torch.equal(m.out, sep), "host-enumerated and device-enumerated launches must agree bitwise"
    ks, vs, tables = workloads.compact_to_host(dk, dv, models, bs)
    for m, f, t in zip(models, fused, tables):
        assert torch.equal(f, m.out), "fused and separate launches must agree bitwise"
        want = orc.paged_decode(m.q.cpu(), ks, vs, t, m.context_lens, m.scale)
        _check(f[:m.batch].float().cpu(), want)


@pytest.mark.parametrize("n_models", [2, 4, 5, 8])
def test_multi_decode_layout_of_the_launch_changes_no_result(n_models):
    """Inside a fused launch the library lays the models out by sequence count and,
    with units enumerated on the host and at most four models, in two runs per
    model (units of split contexts of all models, then all single-unit contexts);
    with five to eight models each keeps one run.  Whatever the layout, every
    model's output is bitwise what its own launch gives - models with only
    single-unit contexts, only split contexts, one sequence, and equal sequence
    counts included."""
    _announce(f"multi decode layout, {n_models} models")
    bs, N = 16, 40000
    rng = np.random.Generator(np.random.PCG64(300 + n_models))
    ids = rng.permutation(N)
    kinds = [lambda: rng.integers(1, 900, size=9),          # mixed
             lambda: rng.integers(1, 257, size=12),         # single-unit contexts only
             lambda: rng.integers(300, 1200, size=5),       # split contexts only
             lambda: rng.integers(1, 700, size=1),          # one sequence
             lambda: rng.integers(1, 900, size=9),          # as many sequences as the first
             lambda: rng.integers(1, 600, size=3),
             lambda: rng.integers(200, 800, size=7),
             lambda: rng.integers(1, 300, size=16)]
    heads = [4, 2, 3, 5, 1, 2, 4, 3]
    models, cur = [], 0
    for k in range(n_models):
        ctx = kinds[k]().astype(np.int32)
        bt, cur = workloads.build_tables(ctx, heads[k], bs, ids, cur)
        models.append(workloads.DecodeModel(f"m{k}", heads[k], heads[k], ctx, bt))
    dk, dv = allocate_gpu_cache(N, bs, DEV)
    dk.fill_(float("nan"))
    dv.fill_(float("nan"))
    workloads.fill_blocks(dk, dv, np.concatenate([m.used_blocks(bs) for m in models]), seed=5)
    for i, m in enumerate(models):
        m.to_device(DEV, torch.float16, seed=40 + i)
    separate = []
    for m in models:
        m.out.zero_()
        ops.paged_decode(m.out, m.q, dk, dv, m.d_block_tables, m.d_context_lens, m.max_context_len, m.scale,
                         partition_size=256)
        torch.cuda.synchronize()
        separate.append(m.out.clone())
    for host in (True, False):
        calls = [ops.DecodeCall(m.out, m.q, m.d_block_tables, m.d_context_lens, m.max_context_len, m.scale,
                                total_context_len=int(m.context_lens.sum()),
                                context_lens_host=torch.from_numpy(np.ascontiguousarray(m.context_lens, dtype=np.int32))
                                if host else None) for m in models]
        for rep in range(2):            # twice: the arrival counters must come back to zero
            for m in models:
                m.out.zero_()
            ops.multi_decode(calls, dk, dv, partition_size=256)
            torch.cuda.synchronize()
            for m, sep in zip(models, separate):
                assert torch.equal(m.out, sep), (m.name, host, rep)
    ks, vs, tables = workloads.compact_to_host(dk, dv, models[:2], bs)
    for m, t in zip(models[:2], tables):
        want = orc.paged_decode(m.q.cpu(), ks, vs, t, m.context_lens, m.scale)
        _check(m.out[:m.batch].float().cpu(), want)


def test_multi_decode_mixed_head_groupings_and_a_large_batch_share_one_workspace():
    """One call with a grouped-query model (matrix-core kernel), a small
    multi-head model (register lookup) and a 300-sequence multi-head model
    (pair table), all with split contexts: their partials, counters and the
    table live in one workspace and must not overlap.  Run twice to check that
    the counters come back to zero."""
    _announce("multi decode mixed G + large batch")
    bs, N = 16, 30000
    rng = np.random.Generator(np.random.PCG64(21))
    shapes = [("gqa", 16, 2, rng.integers(1, 700, size=5)),
              ("mha-small", 3, 3, rng.integers(1, 500, size=7)),
              ("mha-large", 1, 1, rng.integers(1, 300, size=300))]
    ids = rng.permutation(N)
    models, cur = [], 0
    for name, hq, hk, ctx in shapes:
        bt, cur = workloads.build_tables(ctx.astype(np.int32), hk, bs, ids, cur)
        models.append(workloads.DecodeModel(name, hq, hk, ctx.astype(np.int32), bt))
    dk, dv = allocate_gpu_cache(N, bs, DEV)
    dk.fill_(float("nan"))
    dv.fill_(float("nan"))
    workloads.fill_blocks(dk, dv, np.concatenate([m.used_blocks(bs) for m in models]), seed=21)
    for i, m in enumerate(models):
        m.to_device(DEV, torch.float16, seed=30 + i)
    calls = [ops.DecodeCall(m.out, m.q, m.d_block_tables, m.d_context_lens, m.max_context_len, m.scale)
             for m in models]
    ks, vs, tables = workloads.compact_to_host(dk, dv, models, bs)
    for rep in range(2):
        for m in models:
            m.out.fill_(7.0)
        ops.multi_decode(calls, dk, dv, partition_size=128)
        torch.cuda.synchronize()
        for m, t in zip(models, tables):
            want = orc.paged_decode(m.q.cpu(), ks, vs, t, m.context_lens, m.scale)
            _check(m.out[:m.batch].float().cpu(), want)


@pytest.mark.parametrize("host_lens", [False, True])
def test_decode_large_single_model_batch_takes_the_long_partitions(host_lens):
    """One model's large batch (192 sequences of 600..1500 tokens, 8 heads: 1.6 M
    tokens x heads by the caller's bound): the library picks 1024-token
    partitions, waves walk several tiles, contexts beyond 1040 tokens are split
    in two.  Against the oracle, and against the same batch with the 256-token
    partitions of small launches."""
    _announce(f"large single-model batch, host lens {host_lens}")
    rng = np.random.Generator(np.random.PCG64(77))
    ctx = rng.integers(600, 1501, size=192).astype(np.int32)
    ctx[:4] = (1024, 1040, 1041, 1500)
    got, want = _decode_case(78, ctx, 8, 8, 16, hint=True, host_lens=host_lens)
    _check(got, want)
    short, _ = _decode_case(78, ctx, 8, 8, 16, partition=256, hint=True, host_lens=host_lens)
    assert (got - short).abs().max().item() <= 1e-3


@pytest.mark.parametrize("shape", ["a slot's share splits the long contexts", "a slot's share beyond every context",
                                   "two long contexts in many short units"])
def test_decode_grouped_query_launch_takes_a_slots_share_as_partition(shape):
    """Launches of grouped-query models only: with partition_size 0 the library
    takes tokens x kv heads / 768 workgroup slots, rounded up to 256 tokens, as
    partition.  Against the oracle, host- and device-enumerated (the same units:
    the same bits), and against the same batch in 256-token partitions."""
    _announce(f"grouped-query partition policy: {shape}")
    rng = np.random.Generator(np.random.PCG64(91))
    if shape.startswith("a slot's share splits"):
        ctx = rng.integers(150, 1301, size=96).astype(np.int32)      # 96 x ~725 x 8 / 768 -> 768-token partitions
        ctx[:4] = (768, 784, 785, 1300)
        hq, hkv = 32, 8
    elif shape.startswith("a slot's share beyond"):
        ctx = rng.integers(100, 701, size=300).astype(np.int32)      # 300 x ~400 x 8 / 768 -> 1280: nothing is split
        hq, hkv = 64, 8
    else:
        ctx = np.asarray([2500, 3100], dtype=np.int32)               # 5600 x 8 / 768 -> 256-token partitions
        hq, hkv = 64, 8
    got, want = _decode_case(92, ctx, hq, hkv, 16, hint=True, host_lens=True)
    _check(got, want)
    dev_enum, _ = _decode_case(92, ctx, hq, hkv, 16, hint=True, host_lens=False)
    assert torch.equal(got, dev_enum)
    short, _ = _decode_case(92, ctx, hq, hkv, 16, partition=256, hint=True, host_lens=True)
    assert (got - short).abs().max().item() <= 1e-3


def test_decode_rejects_bad_arguments():
    _announce("decode argument validation")
    dk, dv = allocate_gpu_cache(8, 16, DEV)
    q = torch.zeros((8, 256), dtype=torch.float16, device=DEV)
    out = torch.zeros_like(q)
    bt = torch.zeros((1, 2, 2, 4), dtype=torch.int32, device=DEV)
    cl = torch.ones(2, dtype=torch.int32, device=DEV)
    with pytest.raises(RuntimeError):   # max_context_len exceeds what a table row can hold
        ops.paged_decode(out, q, dk, dv, bt, cl, 4 * 16 + 1, 1.0)
    with pytest.raises(RuntimeError):   # partition must be a multiple of 64
        ops.paged_decode(out, q, dk, dv, bt, cl, 16, 1.0, partition_size=100)
    with pytest.raises(RuntimeError):   # CPU tensors: there is no CPU path
        ops.paged_decode(out.cpu(), q.cpu(), dk, dv, bt, cl, 16, 1.0)
    torch.cuda.synchronize()


def test_decode_config2_full_size_pool(full_size_pool_memory):
    """Headline workload at its real size: pool = 60% of HBM, three models,
    ids scattered over the whole pool.  Checked against the oracle on a compact
    host copy of the referenced blocks (attention is invariant under relabelling
    physical blocks)."""
    _announce("decode config 2 full size")
    bs = 16
    total = torch.cuda.get_device_properties(0).total_memory
    N = num_gpu_blocks(0.6, total, bs)
    dk, dv = full_size_pool_memory(N, bs, torch.float16)
    models, need = workloads.config2(seed=0, num_pool_blocks=N)
    used = np.concatenate([m.used_blocks(bs) for m in models])
    assert used.max() > N // 2, "ids must span the pool"
    workloads.fill_blocks(dk, dv, used, seed=0)
    for i, m in enumerate(models):
        m.to_device(DEV, torch.float16, seed=20 + i)
    calls = [ops.DecodeCall(m.out, m.q, m.d_block_tables, m.d_context_lens, m.max_context_len, m.scale,
                            total_context_len=int(m.context_lens.sum()))
             for m in models]
    for _ in range(3):
        ops.multi_decode(calls, dk, dv)
    torch.cuda.synchronize()
    device_enumerated = [m.out.clone() for m in models]
    # The path the benchmark times: the launch prepared once, the units enumerated on the host
    # from the host copy of the context lengths.  Same units, so the same bits.
    host_calls = [ops.DecodeCall(m.out, m.q, m.d_block_tables, m.d_context_lens, m.max_context_len, m.scale,
                                 total_context_len=int(m.context_lens.sum()),
                                 context_lens_host=torch.from_numpy(np.ascontiguousarray(m.context_lens, dtype=np.int32)))
                  for m in models]
    launch = ops.DecodeLaunch(host_calls, dk, dv)
    assert launch.host_pairs > 0, "the headline batch must take the host-enumerated path"
    for m in models:
        m.out.fill_(7.0)
    for _ in range(3):
        launch()
    torch.cuda.synchronize()
    for m, dev_out in zip(models, device_enumerated):
        assert torch.equal(m.out[:m.batch], dev_out[:m.batch]), "host- and device-enumerated launches must agree bitwise"
    ks, vs, tables = workloads.compact_to_host(dk, dv, models, bs)
    del dk, dv
    for m, t in zip(models, tables):
        want = orc.paged_decode(m.q.cpu(), ks, vs, t, m.context_lens, m.scale)
        _check(m.out[:m.batch].float().cpu(), want)


@pytest.mark.parametrize("Hq,Hkv,B,partition", [(2, 2, 9, 64), (8, 1, 7, 128), (1, 1, 300, 64)])
def test_decode_with_an_understated_sum_of_context_lengths_is_slow_not_wrong(Hq, Hkv, B, partition):
    """The caller's bound on the sum of the context lengths sizes the grid.  A
    bound that is far too small leaves most units without a workgroup of their
    own; the workgroups of the last unit that has one run them.  The outputs must
    match the oracle, and the NEXT launch on the same workspace - with a correct
    bound - must too (the arrival counters of the split contexts are back at
    zero).  Vector-ALU kernel, matrix-core kernel, and a batch large enough for
    the pair table."""
    _announce(f"decode, understated context sum Hq={Hq} Hkv={Hkv} B={B}")
    bs = 16
    rng = np.random.Generator(np.random.PCG64(77))
    g = torch.Generator().manual_seed(77)
    ctx = rng.integers(1, 5 * partition, size=B).astype(np.int32)
    nblk = (ctx.astype(np.int64) + bs - 1) // bs
    need = int(nblk.sum()) * Hkv
    N = need + 5
    bt, _ = workloads.build_tables(ctx, Hkv, bs, rng.permutation(N)[:need])
    k_pool, v_pool = orc.allocate_pool(N, bs, torch.float16)
    k_pool.copy_(torch.randn(k_pool.shape, generator=g).half())
    v_pool.copy_(torch.randn(v_pool.shape, generator=g).half())
    pad = (B + 7) // 8 * 8
    q = torch.randn((pad, Hq * HEAD_SIZE), generator=g).half()
    scale = HEAD_SIZE ** -0.5
    want = orc.paged_decode(q, k_pool, v_pool, torch.from_numpy(bt), ctx, scale)
    dq, dk, dv = q.to(DEV), k_pool.to(DEV), v_pool.to(DEV)
    dbt, dctx = torch.from_numpy(bt).to(DEV), torch.from_numpy(ctx).to(DEV)
    out = torch.full((pad, Hq * HEAD_SIZE), 7.0, dtype=torch.float16, device=DEV)
    ws = torch.zeros((64 << 20,), dtype=torch.uint8, device=DEV)
    for hint in (1, int(ctx.sum()) // 3, int(ctx.sum())):        # two understated sums, then the true one
        out.fill_(7.0)
        ops.paged_decode(out, dq, dk, dv, dbt, dctx, int(ctx.max()), scale, partition_size=partition,
                         total_context_len=hint, workspace=ws)
        torch.cuda.synchronize()
        _check(out[:B].float().cpu(), want)
        assert int(ws[:1 << 20].view(torch.int32).abs().max().item()) == 0, "arrival counters must be back at zero"


@pytest.mark.parametrize("n_pairs", [384, 385])
def test_decode_at_the_limit_of_host_enumerated_pairs(n_pairs):
    """The kernel argument holds 384 (sequence, unit) pairs.  A batch with
    exactly that many is enumerated on the host, one with a pair more on the
    device; both give the device-enumerated result bit for bit and match the
    oracle."""
    from muxserve_amd import _lib
    _announce(f"decode with {n_pairs} pairs")
    # 128 sequences of three units (two full partitions and a remainder) are 384 pairs
    ctx = [2 * 256 + 17 + (7 * i) % 200 for i in range(128)]        # remainders of 17 .. 216 tokens: units of their own
    if n_pairs == 385:
        ctx.append(33)
    dev_got, want = _decode_case(41, ctx, 1, 1, 16, partition=256)
    host_got, _ = _decode_case(41, ctx, 1, 1, 16, partition=256, host_lens=True)
    assert torch.equal(host_got, dev_got)
    _check(host_got, want)
    it = _lib.MuxDecodeItem()
    h = np.asarray(ctx, dtype=np.int32)
    it.num_seqs, it.num_q_heads, it.num_kv_heads, it.num_layers = len(ctx), 1, 1, 1
    it.max_context_len, it.max_blocks, it.context_lens_host = int(h.max()), 64, h.ctypes.data
    import ctypes
    pairs = _lib.attn().mux_paged_decode_host_pairs(ctypes.addressof(it), 1, 256)
    assert pairs == (384 if n_pairs == 384 else 0)


@pytest.mark.parametrize("Hq,Hkv,dtype", [(4, 4, torch.float16), (16, 2, torch.bfloat16)])
def test_decode_is_invariant_under_relabelling_of_the_physical_blocks(Hq, Hkv, dtype):
    """The same logical caches stored under different block ids (pool permuted,
    tables relabelled) give bit-identical outputs: nothing in the result may
    depend on where a block lives.  Contexts cover single-partition, split and
    remainder units; the write goes through the GPU cache-write kernel."""
    print(f"[case] decode block relabelling Hq={Hq} Hkv={Hkv} {dtype}", flush=True)
    bs = 16
    rng = np.random.Generator(np.random.PCG64(31))
    g = torch.Generator().manual_seed(31)
    ctx = np.asarray([1, 16, 70, 256, 257, 700, 1300, 33], dtype=np.int32)
    B = len(ctx)
    nblk = (ctx.astype(np.int64) + bs - 1) // bs
    need = int(nblk.sum()) * Hkv
    N = 3 * need + 11
    pad = (B + 7) // 8 * 8
    q = torch.randn((pad, Hq * HEAD_SIZE), generator=g).to(dtype).to(DEV)
    dense = [(torch.randn((int(n), Hkv * HEAD_SIZE), generator=g).to(dtype),
              torch.randn((int(n), Hkv * HEAD_SIZE), generator=g).to(dtype)) for n in ctx]
    outs = []
    for trial in range(3):
        ids = rng.permutation(N)[:need]
        bt1, _ = workloads.build_tables(ctx, Hkv, bs, ids)
        k_pool, v_pool = allocate_gpu_cache(N, bs, DEV, dtype=dtype)
        k_pool.fill_(float("nan"))
        v_pool.fill_(float("nan"))
        for s_, (kd, vd) in enumerate(dense):
            n = int(ctx[s_])
            i = np.arange(n)
            slots = bt1[0, s_][:, i // bs].astype(np.int64).T * bs + (i % bs)[:, None]
            ops.reshape_and_cache(kd.to(DEV), vd.to(DEV), k_pool, v_pool,
                                  torch.from_numpy(np.ascontiguousarray(slots[:, None, :])).to(DEV))
        out = torch.zeros((pad, Hq * HEAD_SIZE), dtype=dtype, device=DEV)
        ops.paged_decode(out, q, k_pool, v_pool, torch.from_numpy(bt1).to(DEV), torch.from_numpy(ctx).to(DEV),
                         int(ctx.max()), HEAD_SIZE ** -0.5)
        torch.cuda.synchronize()
        outs.append(out[:B].cpu().view(torch.int16))
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])


def test_gather_read_probe_runs_and_rejects_what_it_cannot_read():
    """The measuring aid next to the decode kernel: accepts any id list
    (duplicates, ids outside the pool are clamped, lengths that are no multiple
    of a wave's four blocks), never writes the pools, refuses other block sizes."""
    print("[case] gather-read probe", flush=True)
    from muxserve_amd import _lib
    N = 512
    k_pool, v_pool = allocate_gpu_cache(N, 16, DEV)
    k_pool.normal_()
    v_pool.normal_()
    k0, v0 = k_pool.clone(), v_pool.clone()
    sink = torch.zeros((1,), dtype=torch.int32, device=DEV)
    for n in (1, 3, 4, 17, 1000):
        ids = torch.randint(-5, N + 5, (n,), dtype=torch.int32, device=DEV)
        workloads.probe_gather_read(k_pool, v_pool, ids, sink)
    workloads.probe_gather_read(k_pool, v_pool, torch.zeros((0,), dtype=torch.int32, device=DEV), sink)
    torch.cuda.synchronize()
    assert torch.equal(k_pool, k0) and torch.equal(v_pool, v0)
    k8, v8 = allocate_gpu_cache(64, 8, DEV)
    with pytest.raises(RuntimeError):
        workloads.probe_gather_read(k8, v8, torch.zeros((4,), dtype=torch.int32, device=DEV), sink)
    assert _lib.probe().mux_probe_gather_read(None, v_pool.data_ptr(), N, sink.data_ptr(), 4, 16, sink.data_ptr(),
                                             None) == -1      # invalid argument


def test_copy_probe_copies_and_mfma_probe_reports_its_clocks():
    """The two other yardsticks of bench.py: the contiguous copy (next to the
    cache write) moves exactly the bytes it is given and refuses sizes and
    pointers that are no multiple of its 16-byte chunk; the matrix-core loop
    finishes, reports ticks of both clocks for every workgroup and refuses
    combinations that were not built."""
    print("[case] copy probe and mfma probe", flush=True)
    from muxserve_amd import _lib
    lib = _lib.probe()
    st = torch.cuda.current_stream().cuda_stream
    for n in (16, 4096, 16 * 257, 1 << 20):
        src = torch.randint(0, 256, (n,), dtype=torch.uint8, device=DEV)
        dst = torch.zeros(n + 32, dtype=torch.uint8, device=DEV)
        assert lib.mux_probe_copy(dst.data_ptr(), src.data_ptr(), n, st) == 0
        torch.cuda.synchronize()
        assert torch.equal(dst[:n], src) and int(dst[n:].sum()) == 0
    src = torch.zeros(64, dtype=torch.uint8, device=DEV)
    dst = torch.zeros(64, dtype=torch.uint8, device=DEV)
    assert lib.mux_probe_copy(dst.data_ptr(), src.data_ptr(), 0, st) == 0
    assert lib.mux_probe_copy(dst.data_ptr(), src.data_ptr(), 24, st) == -1
    assert lib.mux_probe_copy(dst.data_ptr() + 4, src.data_ptr(), 32, st) == -1
    assert lib.mux_probe_copy(None, src.data_ptr(), 32, st) == -1

    # the copy with scattered destinations: block b of the sources lands in pool block ids[b]
    N = 64
    k_pool, v_pool = allocate_gpu_cache(N, 16, DEV)
    k_pool.zero_()
    v_pool.zero_()
    ids = torch.tensor([5, 63, 0, 17, 99, -3], dtype=torch.int32, device=DEV)      # the last two are clamped to 63 and 0
    ks = torch.randint(-30000, 30000, (ids.numel(), 2048), dtype=torch.int16, device=DEV)
    vs = torch.randint(-30000, 30000, (ids.numel(), 2048), dtype=torch.int16, device=DEV)
    assert lib.mux_probe_scatter_copy(k_pool.data_ptr(), v_pool.data_ptr(), N, ks.data_ptr(), vs.data_ptr(),
                                      ids.data_ptr(), 4, st) == 0
    torch.cuda.synchronize()
    kp, vp = k_pool.view(torch.int16).view(N, 2048), v_pool.view(torch.int16).view(N, 2048)
    for b, i in enumerate((5, 63, 0, 17)):
        assert torch.equal(kp[i], ks[b]) and torch.equal(vp[i], vs[b])
    untouched = [i for i in range(N) if i not in (5, 63, 0, 17)]
    assert int(kp[untouched].abs().sum()) == 0 and int(vp[untouched].abs().sum()) == 0
    assert lib.mux_probe_scatter_copy(k_pool.data_ptr(), v_pool.data_ptr(), N, ks.data_ptr(), vs.data_ptr(),
                                      ids.data_ptr(), 6, st) == 0       # ids outside the pool: clamped, no stray write
    assert lib.mux_probe_scatter_copy(k_pool.data_ptr(), v_pool.data_ptr(), 0, ks.data_ptr(), vs.data_ptr(),
                                      ids.data_ptr(), 4, st) == -1
    assert lib.mux_probe_scatter_copy(k_pool.data_ptr(), v_pool.data_ptr(), N, ks.data_ptr(), vs.data_ptr(),
                                      None, 4, st) == -1
    torch.cuda.synchronize()

    sink = torch.zeros(1, dtype=torch.float32, device=DEV)
    for chains, valu, waves, mfma_waves in ((1, 0, 4, 4), (4, 8, 4, 4), (4, 0, 8, 4), (2, 0, 1, 0)):
        ticks = torch.zeros(8, 2, dtype=torch.int32, device=DEV)
        assert lib.mux_probe_mfma(chains, valu, 200, 8, waves, mfma_waves, ticks.data_ptr(), sink.data_ptr(), st) == 0
        torch.cuda.synchronize()
        assert bool((ticks > 0).all())
    ticks = torch.zeros(8, 2, dtype=torch.int32, device=DEV)
    assert lib.mux_probe_mfma(3, 0, 200, 8, 4, 4, ticks.data_ptr(), sink.data_ptr(), st) == -2     # not built
    assert lib.mux_probe_mfma(4, 0, 200, 8, 9, 4, ticks.data_ptr(), sink.data_ptr(), st) == -1
    assert lib.mux_probe_mfma(4, 0, 0, 8, 4, 4, ticks.data_ptr(), sink.data_ptr(), st) == -1
    torch.cuda.synchronize()
    assert int(ticks.sum()) == 0


def test_split_context_hand_off_is_stable_over_two_thousand_launches():
    """The hand-off of split contexts between workgroups (partial results
    published with device-coherent stores, one arrival counter per sequence and
    head group, the last arriver combines): 2000 launches of a split-heavy batch
    - partitions of 64 tokens, contexts 65..2048, so up to 32 partitions meet per
    head - alternating between two workspaces, every output compared bitwise
    with the first launch's.  The comparison stays on the device and is read
    back every 100 launches; the run stops at the first mismatch."""
    _announce("decode split hand-off, 2000 launches")
    bs, Hq, B = 16, 8, 48
    rng = np.random.Generator(np.random.PCG64(77))
    ctx = rng.integers(65, 2049, size=B).astype(np.int32)
    ctx[:4] = [65, 2048, 128, 1999]
    need = int(((ctx + bs - 1) // bs).sum()) * Hq
    N = need + 64
    bt, _ = workloads.build_tables(ctx, Hq, bs, rng.permutation(N)[:need])
    m = workloads.DecodeModel("m", Hq, Hq, ctx, bt)
    dk, dv = allocate_gpu_cache(N, bs, DEV)
    workloads.fill_blocks(dk, dv, m.used_blocks(bs), seed=3)
    m.to_device(DEV, torch.float16, seed=4)
    lib_need = (B * Hq * 32) * (128 + 2) * 4 + (2 << 20)
    spaces = [torch.zeros((lib_need,), dtype=torch.uint8, device=DEV) for _ in range(2)]
    host_lens = torch.from_numpy(ctx)

    def launch(i):
        ops.paged_decode(m.out, m.q, dk, dv, m.d_block_tables, m.d_context_lens, m.max_context_len, m.scale,
                         partition_size=64, workspace=spaces[i % 2],
                         context_lens_host=host_lens if (i // 2) % 2 else None)

    launch(0)
    torch.cuda.synchronize()
    first = m.out.clone()
    want = orc.paged_decode(m.q.cpu(), dk.cpu(), dv.cpu(), torch.from_numpy(bt), ctx, m.scale)
    _check(first[:B].float().cpu(), want)
    bad = torch.zeros((), dtype=torch.int32, device=DEV)
    for i in range(1, 2001):
        m.out.zero_()
        launch(i)
        bad += (m.out != first).any().to(torch.int32)
        if i % 100 == 0:
            assert int(bad.item()) == 0, f"a launch among {i - 99}..{i} differs from the first"


@pytest.mark.parametrize("seed", range(24))
def test_decode_random_shapes_against_the_oracle(seed):
    """Seeded draws over head grouping, block size, storage type, partition size,
    layer slice and context lengths (short, around tile and partition boundaries,
    long), each against the oracle at the 2e-3 bar."""
    rng = np.random.Generator(np.random.PCG64(1000 + seed))
    Hkv = int(rng.choice([1, 2, 3, 5]))
    ratio = int(rng.choice([1, 1, 2, 4, 8, 16, 3]))
    bs = int(rng.choice([8, 16, 16, 32]))
    dtype = [torch.float16, torch.bfloat16][int(rng.integers(2))]
    partition = int(rng.choice([0, 64, 128, 256, 512]))
    B = int(rng.integers(1, 12))
    kinds = rng.integers(0, 4, size=B)
    ctx = np.where(kinds == 0, rng.integers(1, 20, size=B),
                   np.where(kinds == 1, 64 * rng.integers(1, 9, size=B) + rng.integers(-1, 2, size=B),
                            np.where(kinds == 2, rng.integers(1, 600, size=B), rng.integers(600, 1500, size=B))))
    L = int(rng.integers(1, 4))
    layer = int(rng.integers(L))
    _announce(f"decode random seed={seed} Hq={Hkv * ratio} Hkv={Hkv} bs={bs} {dtype} partition={partition} "
              f"L={L} layer={layer} ctx={ctx.tolist()}")
    got, want = _decode_case(2000 + seed, ctx.tolist(), Hkv * ratio, Hkv, bs, dtype=dtype, partition=partition,
                             num_layers=L, layer=layer, q_in_qkv=bool(rng.integers(2)), hint=bool(rng.integers(2)),
                             repeat=2)
    _check(got, want, out_dtype=dtype)
