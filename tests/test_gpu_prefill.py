"""GPU parity: causal prefill attention (MFMA) against the CPU oracle
(<= 2e-3 max-abs, fp16/bf16 in, fp32 accumulate), then the prefill-shaped cache
write into head-wise slot mappings, bit-exact.  All through the C ABI.
"""
import numpy as np
import pytest
import torch

from oracle import attn_oracle as orc
from muxserve_amd import ops, workloads
from muxserve_amd.pool import HEAD_SIZE, allocate_gpu_cache

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 2e-3
D = HEAD_SIZE


def _announce(msg):
    print(f"[case] {msg}", flush=True)


def _bound(want, dtype):
    b = torch.full_like(want, TOL)
    if dtype == torch.bfloat16:      # + rounding of the result to bf16 (8-bit mantissa)
        b = b + want.abs() * 2.0 ** -8
    return b


def _run_prefill(seed, lens, Hq, Hkv, dtype, in_qkv=True, host_lens=False):
    g = torch.Generator().manual_seed(seed)
    T = int(sum(lens))
    pad = (T + 7) // 8 * 8
    if in_qkv:
        qkv = torch.randn((pad, (Hq + 2 * Hkv) * D), generator=g).to(dtype)
        q, k, v = qkv.split([Hq * D, Hkv * D, Hkv * D], dim=-1)     # models/llama.py:157-158
        dqkv = qkv.to(DEV)
        dq, dk, dv = dqkv.split([Hq * D, Hkv * D, Hkv * D], dim=-1)
    else:
        q = torch.randn((pad, Hq * D), generator=g).to(dtype)
        k = torch.randn((pad, Hkv * D), generator=g).to(dtype)
        v = torch.randn((pad, Hkv * D), generator=g).to(dtype)
        dq, dk, dv = q.to(DEV), k.to(DEV), v.to(DEV)
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32, device=DEV)
    out = torch.full((pad, Hq * D), 7.0, dtype=dtype, device=DEV)
    ops.prefill_causal(out, dq, dk, dv, cu, int(max(lens)), D ** -0.5, Hkv, prompt_lens=lens if host_lens else None)
    torch.cuda.synchronize()
    got = out.float().cpu()
    assert (got[T:] == 7.0).all(), "padding rows must not be written"
    return got[:T], q, k, v


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("Hq,Hkv", [(3, 3), (4, 2), (8, 1)])
def test_prefill_matches_oracle_ragged_prompts(Hq, Hkv, dtype):
    _announce(f"prefill ragged Hq={Hq} Hkv={Hkv} {dtype}")
    lens = [1, 7, 64, 33, 128, 129, 300, 31]
    got, q, k, v = _run_prefill(1, lens, Hq, Hkv, dtype)
    want = orc.prefill_causal(q, k, v, lens, D ** -0.5, Hkv)
    assert torch.isfinite(got).all()
    excess = ((got - want).abs() - _bound(want, dtype)).max().item()
    assert excess <= 0, f"max-abs error {(got - want).abs().max().item():.3e}"


@pytest.mark.parametrize("host_lens", [False, True])
@pytest.mark.parametrize("num_prompts", [64, 70, 150])
def test_prefill_many_prompts_ties_and_empty_prompts(num_prompts, host_lens):
    """Many prompts in one launch: equal lengths, empty prompts and lengths
    around the 128-row tile all appear; with the grid sized by the longest
    prompt and with the compact grid built from host-side lengths."""
    _announce(f"prefill {num_prompts} prompts host_lens={host_lens}")
    rng = np.random.Generator(np.random.PCG64(num_prompts))
    lens = rng.integers(1, 200, size=num_prompts)
    lens[::5] = 128
    lens[1::9] = 129
    lens[3] = 0
    lens[num_prompts - 2] = 0
    lens[7] = 260
    lens = [int(n) for n in lens]
    got, q, k, v = _run_prefill(3, lens, 2, 1, torch.float16, host_lens=host_lens)
    want = orc.prefill_causal(q, k, v, lens, D ** -0.5, 1)
    assert torch.isfinite(got).all()
    excess = ((got - want).abs() - _bound(want, torch.float16)).max().item()
    assert excess <= 0, f"max-abs error {(got - want).abs().max().item():.3e}"


@pytest.mark.parametrize("host_lens", [False, True])
@pytest.mark.parametrize("Hkv", [5, 9, 13])
def test_prefill_kv_head_counts_that_do_not_divide_by_eight(Hkv, host_lens):
    _announce(f"prefill Hkv={Hkv} host_lens={host_lens}")
    lens = [130, 17, 64]
    got, q, k, v = _run_prefill(4, lens, Hkv, Hkv, torch.float16, host_lens=host_lens)
    want = orc.prefill_causal(q, k, v, lens, D ** -0.5, Hkv)
    excess = ((got - want).abs() - _bound(want, torch.float16)).max().item()
    assert excess <= 0, f"max-abs error {(got - want).abs().max().item():.3e}"


def test_prefill_long_prompt_and_unstrided_inputs():
    _announce("prefill long prompt")
    lens = [2048, 5, 700]
    got, q, k, v = _run_prefill(2, lens, 2, 2, torch.float16, in_qkv=False)
    want = orc.prefill_causal(q, k, v, lens, D ** -0.5, 2)
    assert torch.isfinite(got).all()
    assert (got - want).abs().max().item() <= TOL


def test_prefill_prompt_order_changes_scheduling_only():
    """Longest-first, reversed and random start orders give bit-identical
    outputs (each workgroup computes the same tile whichever order it starts in)."""
    _announce("prefill prompt order")
    rng = np.random.Generator(np.random.PCG64(12))
    lens = [int(x) for x in rng.integers(1, 400, size=21)] + [0, 700]
    T = sum(lens)
    g = torch.Generator().manual_seed(12)
    q = torch.randn((T, 6 * D), generator=g).half().to(DEV)
    k = torch.randn((T, 3 * D), generator=g).half().to(DEV)
    v = torch.randn((T, 3 * D), generator=g).half().to(DEV)
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32, device=DEV)
    base = torch.zeros_like(q)
    ops.prefill_causal(base, q, k, v, cu, max(lens), D ** -0.5, 3)
    orders = [np.argsort(-np.asarray(lens), kind="stable"), np.arange(len(lens))[::-1].copy(),
              rng.permutation(len(lens))]
    for order in orders:
        out = torch.zeros_like(q)
        ops.prefill_causal(out, q, k, v, cu, max(lens), D ** -0.5, 3,
                           prompt_order=torch.from_numpy(order.astype(np.int32)).to(DEV))
        torch.cuda.synchronize()
        assert torch.equal(out, base)
    with pytest.raises(ValueError):
        ops.prefill_causal(base, q, k, v, cu, max(lens), D ** -0.5, 3,
                           prompt_order=torch.zeros((3,), dtype=torch.int32, device=DEV))
    # the compact grid built from host-side lengths: the same tiles again
    out = torch.zeros_like(q)
    ops.prefill_causal(out, q, k, v, cu, max(lens), D ** -0.5, 3, prompt_lens=lens)
    torch.cuda.synchronize()
    assert torch.equal(out, base)


def test_prefill_host_side_lengths_are_a_hint_not_an_address():
    """Host-side lengths only choose which query tiles are started: lengths that
    are too short leave the tiles they hide unwritten, lengths beyond the
    stated maximum are refused, and a batch with more query tiles than the
    kernel argument holds falls back to the grid sized by the longest prompt."""
    _announce("prefill host lengths")
    lens = [300, 40, 129]
    T = sum(lens)
    g = torch.Generator().manual_seed(13)
    q = torch.randn((T, 2 * D), generator=g).half().to(DEV)
    k = torch.randn((T, 2 * D), generator=g).half().to(DEV)
    v = torch.randn((T, 2 * D), generator=g).half().to(DEV)
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32, device=DEV)
    base = torch.full_like(q, 7.0)
    ops.prefill_causal(base, q, k, v, cu, 300, D ** -0.5, 2)
    out = torch.full_like(q, 7.0)
    ops.prefill_causal(out, q, k, v, cu, 300, D ** -0.5, 2, prompt_lens=[128, 40, 0])
    torch.cuda.synchronize()
    started = np.r_[0:128, 300:340]                     # rows of the tiles the short lengths still name
    hidden = np.r_[128:300, 340:T]
    assert torch.equal(out[started], base[started]) and (out[hidden] == 7.0).all()
    with pytest.raises(RuntimeError):
        ops.prefill_causal(out, q, k, v, cu, 300, D ** -0.5, 2, prompt_lens=[301, 40, 129])
    with pytest.raises(ValueError):
        ops.prefill_causal(out, q, k, v, cu, 300, D ** -0.5, 2, prompt_lens=[300, 40])
    # 1000 prompts of 129 tokens: 2000 query tiles, more than the compact list holds
    many = [129] * 1000
    got, q2, k2, v2 = _run_prefill(14, many, 1, 1, torch.float16, host_lens=True)
    want = orc.prefill_causal(q2, k2, v2, many, D ** -0.5, 1)
    assert (got - want).abs().max().item() <= TOL


def test_prefill_first_token_and_block_diagonal_properties():
    """Row 0 of every prompt equals its own v; changing one prompt's k leaves
    every other prompt's output bit-identical."""
    _announce("prefill properties")
    lens = [40, 130, 9]
    g = torch.Generator().manual_seed(3)
    T = sum(lens)
    q = torch.randn((T, 2 * D), generator=g).half().to(DEV)
    k = torch.randn((T, 2 * D), generator=g).half().to(DEV)
    v = torch.randn((T, 2 * D), generator=g).half().to(DEV)
    cu = torch.tensor([0, 40, 170, 179], dtype=torch.int32, device=DEV)
    out = torch.zeros_like(q)
    ops.prefill_causal(out, q, k, v, cu, 130, D ** -0.5, 2)
    k2 = k.clone()
    k2[40:170] += 1
    out2 = torch.zeros_like(q)
    ops.prefill_causal(out2, q, k2, v, cu, 130, D ** -0.5, 2)
    torch.cuda.synchronize()
    for s in (0, 40, 170):
        assert torch.equal(out[s], v[s])
    assert torch.equal(out[:40], out2[:40]) and torch.equal(out[170:], out2[170:])
    assert not torch.equal(out[40:170], out2[40:170])


def test_config3_prefill_then_cache_write_bit_exact():
    """Three shapes, 16 prompts each, lengths lognormal(200, 1.0) in [8, 2048]:
    attention checked on a subset of heads (the CPU oracle is O(n^2) per head),
    the cache scatter into seeded random head-wise slot mappings checked
    bit-exact over the whole pool."""
    _announce("config 3")
    bs = 16
    models = workloads.config3(seed=0)
    total_blocks = sum(int(((m.prompt_lens + bs - 1) // bs).sum()) * m.num_kv_heads for m in models)
    N = total_blocks + 1000
    rng = np.random.Generator(np.random.PCG64(0))
    ids = rng.permutation(N)
    dk_pool, dv_pool = allocate_gpu_cache(N, bs, DEV)
    dk_pool.zero_()
    dv_pool.zero_()
    hk_pool, hv_pool = dk_pool.cpu(), dv_pool.cpu()
    cur = 0
    for mi, m in enumerate(models):
        _announce(f"config 3 model {m.name} tokens={m.num_tokens}")
        g = torch.Generator().manual_seed(10 + mi)
        Hq, Hkv, T = m.num_q_heads, m.num_kv_heads, m.num_tokens
        pad = (T + 7) // 8 * 8
        qkv = torch.randn((pad, (Hq + 2 * Hkv) * D), generator=g).half()
        dqkv = qkv.to(DEV)
        dq, dk, dv = dqkv.split([Hq * D, Hkv * D, Hkv * D], dim=-1)
        q, k, v = qkv.split([Hq * D, Hkv * D, Hkv * D], dim=-1)
        cu = torch.from_numpy(m.cu_seqlens()).to(DEV)
        out = torch.zeros((pad, Hq * D), dtype=torch.float16, device=DEV)
        ops.prefill_causal(out, dq, dk, dv, cu, int(m.prompt_lens.max()), m.scale, Hkv)
        slots, used = workloads.prefill_slot_mapping(m.prompt_lens, Hkv, bs, ids[cur:])
        cur += used
        ops.reshape_and_cache(dk, dv, dk_pool, dv_pool, torch.from_numpy(slots).to(DEV), num_tokens=T)
        torch.cuda.synchronize()
        orc.reshape_and_cache(k, v, hk_pool, hv_pool, torch.from_numpy(slots), num_tokens=T)
        heads = sorted({0, Hq // 2, Hq - 1})
        sel = torch.cat([torch.arange(h * D, (h + 1) * D) for h in heads])
        want = orc.prefill_causal(q[:, sel], k[:, sel], v[:, sel], m.prompt_lens, m.scale, len(heads))
        got = out[:T].cpu()[:, sel].float()
        assert torch.isfinite(out[:T]).all()
        err = (got - want).abs().max().item()
        assert err <= TOL, f"{m.name}: prefill max-abs error {err:.3e}"
    assert torch.equal(dk_pool.cpu().view(torch.int16), hk_pool.view(torch.int16))
    assert torch.equal(dv_pool.cpu().view(torch.int16), hv_pool.view(torch.int16))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_fused_prefill_of_three_models_equals_one_launch_per_model(dtype):
    """mux_multi_prefill_causal over config 3's three shapes (plus a grouped-query
    model and a model without prompts) against one mux_prefill_causal per model:
    every output bitwise equal - the shared grid only changes which workgroup
    runs when - and the fused cache write of the same step bitwise equal to the
    oracle's scatter."""
    _announce(f"fused prefill, three models {dtype}")
    bs = 16
    models = workloads.config3(seed=1, prompts=6)
    shapes = [(m.num_q_heads, m.num_kv_heads, [int(x) for x in m.prompt_lens]) for m in models]
    shapes.append((16, 2, [300, 5, 129]))
    shapes.append((8, 8, []))
    total_blocks = sum(sum((n + bs - 1) // bs for n in lens) * hk for _, hk, lens in shapes)
    N = total_blocks + 50
    ids = np.random.Generator(np.random.PCG64(5)).permutation(N)
    dk_pool, dv_pool = allocate_gpu_cache(N, bs, DEV, dtype=dtype)
    dk_pool.zero_()
    dv_pool.zero_()
    hk_pool, hv_pool = dk_pool.cpu(), dv_pool.cpu()
    pcalls, wcalls, singles, cur = [], [], [], 0
    for mi, (Hq, Hkv, lens) in enumerate(shapes):
        g = torch.Generator().manual_seed(50 + mi)
        T = sum(lens)
        pad = (T + 7) // 8 * 8
        qkv = torch.randn((pad, (Hq + 2 * Hkv) * D), generator=g).to(dtype)
        dq, dk, dv = qkv.to(DEV).split([Hq * D, Hkv * D, Hkv * D], dim=-1)
        cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]).astype(np.int32), device=DEV)
        fused_out = torch.zeros((pad, Hq * D), dtype=dtype, device=DEV)
        single_out = torch.zeros_like(fused_out)
        pcalls.append(ops.PrefillCall(fused_out, dq, dk, dv, cu, lens, D ** -0.5, Hkv))
        if T:
            ops.prefill_causal(single_out, dq, dk, dv, cu, max(lens), D ** -0.5, Hkv, prompt_lens=lens)
            slots, used = workloads.prefill_slot_mapping(lens, Hkv, bs, ids[cur:])
            cur += used
            wcalls.append(ops.CacheWriteCall(dk, dv, torch.from_numpy(slots).to(DEV), num_tokens=T))
            _, k, v = qkv.split([Hq * D, Hkv * D, Hkv * D], dim=-1)
            orc.reshape_and_cache(k, v, hk_pool, hv_pool, torch.from_numpy(slots), num_tokens=T)
        singles.append((fused_out, single_out, T))
    ops.multi_prefill_causal(pcalls)
    ops.multi_reshape_and_cache(wcalls, dk_pool, dv_pool)
    torch.cuda.synchronize()
    for fused_out, single_out, T in singles:
        assert torch.equal(fused_out.view(torch.int16), single_out.view(torch.int16))
        if T:
            assert single_out[:T].float().abs().sum().item() > 0
    assert torch.equal(dk_pool.cpu().view(torch.int16), hk_pool.view(torch.int16))
    assert torch.equal(dv_pool.cpu().view(torch.int16), hv_pool.view(torch.int16))


def test_fused_prefill_falls_back_to_one_launch_per_model_when_the_tiles_do_not_fit():
    """More query tiles than the shared kernel argument lists (here 2 x 520): the
    call still returns every model's result, identical to the separate calls."""
    _announce("fused prefill, too many tiles")
    outs = []
    calls = []
    for mi in range(2):
        g = torch.Generator().manual_seed(70 + mi)
        lens = [100] * 520
        T = sum(lens)
        qkv = torch.randn((T, 3 * D), generator=g).half().to(DEV)
        q, k, v = qkv.split([D, D, D], dim=-1)
        cu = torch.arange(0, T + 1, 100, dtype=torch.int32, device=DEV)
        a, b = torch.zeros((T, D), dtype=torch.float16, device=DEV), torch.zeros((T, D), dtype=torch.float16, device=DEV)
        calls.append(ops.PrefillCall(a, q, k, v, cu, lens, D ** -0.5, 1))
        ops.prefill_causal(b, q, k, v, cu, 100, D ** -0.5, 1, prompt_lens=lens)
        outs.append((a, b))
    ops.multi_prefill_causal(calls)
    torch.cuda.synchronize()
    for a, b in outs:
        assert torch.equal(a.view(torch.int16), b.view(torch.int16)) and a.float().abs().sum().item() > 0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_prefill_row_maxima_that_jump_far_above_the_softmax_reference(dtype):
    """The kernel keeps the reference of its exponents until some row's maximum
    has risen by more than 8 (in the exponent) above it.  N(0,1) data never gets
    there after the first tile, so here the scores are made to jump: all queries
    share a strong component along one direction and a few keys, later and later
    in the prompt, point along it with growing length - the running maximum of
    every row then rises by 10 to 20 at those keys (several moves of the
    reference per wave, in different tiles), while the rows before a spike keep
    an ordinary mixture.  A second prompt has its spike in the very first tile."""
    _announce(f"prefill softmax reference moves {dtype}")
    Hq = Hkv = 2
    lens = [700, 190]
    g = torch.Generator().manual_seed(77)
    T = sum(lens)
    pad = (T + 7) // 8 * 8
    u = torch.randn((Hq, D), generator=g)
    u = u / u.norm(dim=-1, keepdim=True)
    q = torch.randn((pad, Hq, D), generator=g) + 4.0 * u
    k = torch.randn((pad, Hkv, D), generator=g)
    v = torch.randn((pad, Hkv, D), generator=g)
    for pos, beta in ((40, 20.0), (300, 45.0), (301, 44.0), (650, 80.0), (700 + 3, 30.0), (700 + 150, 60.0)):
        k[pos] = beta * u
    q, k, v = (x.reshape(pad, -1).to(dtype) for x in (q, k, v))
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32, device=DEV)
    out = torch.zeros((pad, Hq * D), dtype=dtype, device=DEV)
    ops.prefill_causal(out, q.to(DEV), k.to(DEV), v.to(DEV), cu, max(lens), D ** -0.5, Hkv, prompt_lens=lens)
    torch.cuda.synchronize()
    got = out.float().cpu()[:T]
    want = orc.prefill_causal(q, k, v, lens, D ** -0.5, Hkv)
    assert torch.isfinite(got).all()
    # the scores really jump: the spike keys dominate the rows after them
    s_spike = (q[651].float().reshape(Hq, D) * k[650].float().reshape(Hkv, D)).sum(-1) * D ** -0.5 * 1.4427
    assert (s_spike > 20).all()
    excess = ((got - want).abs() - _bound(want, dtype)).max().item()
    assert excess <= 0, f"max-abs error {(got - want).abs().max().item():.3e}"


def test_prefill_rejects_bad_arguments():
    q = torch.zeros((8, 256), dtype=torch.float16, device=DEV)
    cu = torch.tensor([0, 8], dtype=torch.int32, device=DEV)
    with pytest.raises(ValueError):
        ops.prefill_causal(q, q, q[:, :128], q, cu, 8, 1.0, 1)      # k/v shape mismatch
    with pytest.raises(RuntimeError):
        ops.prefill_causal(q.cpu(), q.cpu(), q.cpu(), q.cpu(), cu, 8, 1.0, 2)


@pytest.mark.parametrize("seed", range(16))
def test_prefill_random_shapes_against_the_oracle(seed):
    """Seeded draws over head grouping, storage type, number and lengths of the
    prompts (single tokens, around the 32/64/128-row tile edges, a few hundred
    tokens), inputs as slices of one qkv row or separate, with and without a
    start order; each against the oracle at the 2e-3 bar."""
    rng = np.random.Generator(np.random.PCG64(3000 + seed))
    Hkv = int(rng.choice([1, 2, 3, 5]))
    ratio = int(rng.choice([1, 1, 2, 4, 8]))
    dtype = [torch.float16, torch.bfloat16][int(rng.integers(2))]
    P = int(rng.integers(1, 10))
    kinds = rng.integers(0, 3, size=P)
    lens = np.where(kinds == 0, rng.integers(1, 6, size=P),
                    np.where(kinds == 1, 32 * rng.integers(1, 9, size=P) + rng.integers(-1, 2, size=P),
                             rng.integers(1, 500, size=P)))
    lens = [int(x) for x in lens]
    in_qkv = bool(rng.integers(2))
    _announce(f"prefill random seed={seed} Hq={Hkv * ratio} Hkv={Hkv} {dtype} lens={lens} in_qkv={in_qkv}")
    got, q, k, v = _run_prefill(4000 + seed, lens, Hkv * ratio, Hkv, dtype, in_qkv=in_qkv, host_lens=bool(seed % 2))
    want = orc.prefill_causal(q, k, v, lens, D ** -0.5, Hkv)
    assert torch.isfinite(got).all()
    excess = ((got - want).abs() - _bound(want, dtype)).max().item()
    assert excess <= 0, f"max-abs error {(got - want).abs().max().item():.3e}"
