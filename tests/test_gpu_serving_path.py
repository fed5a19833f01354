"""The drop-in boundary end to end on the GPU: two models of different head and
layer counts share ONE pool and ONE KVStorage; every step goes
BatchScheduler -> allocator -> prepare_inputs -> PagedAttentionWithRoPE.forward
for every layer, exactly as the reference's serving loop drives its attention
layer (llm_runtime.py:277-339, models/llama.py:149-163).  Checked per layer
against the oracle; the pool is compared bit-exact at the end.
"""
import numpy as np
import pytest
import torch

from oracle import attn_oracle as orc
from muxserve_amd import ops
from muxserve_amd.attention import PagedAttentionWithRoPE
from muxserve_amd.batch_scheduler import BatchScheduler
from muxserve_amd.device_tables import DeviceBlockTables
from muxserve_amd.memory_manager import KVStorage
from muxserve_amd.pool import HEAD_SIZE, allocate_gpu_cache
from muxserve_amd.prepare import prepare_inputs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
D = HEAD_SIZE
TOL = 2e-3


class _Model:
    def __init__(self, name, L, Hq, Hkv, storage, bs, seed, fused_rope_max_tokens=512, device_rows=0):
        self.name, self.L, self.Hq, self.Hkv = name, L, Hq, Hkv
        self.sched = BatchScheduler(L, Hkv, 512, bs)
        self.storage = storage
        self.layers = [PagedAttentionWithRoPE(Hq, D, D ** -0.5, base=10000, max_position=2048, rotary_dim=D,
                                              num_kv_heads=Hkv, rope_scaling=None, layer_idx=l) for l in range(L)]
        for layer in self.layers:
            layer.fused_rope_max_tokens = fused_rope_max_tokens
        self.g = torch.Generator().manual_seed(seed)
        self.device_tables = DeviceBlockTables(self.sched, device_rows, DEV) if device_rows else None

    def alloc(self, req):
        return self.storage.allocate_batch(req, self.L, self.Hkv)


def _step(m, ids, last_tokens, k_pool, v_pool, hk, hv, permuted):
    tokens, positions, md, batch_reqs, preempted = prepare_inputs(m.sched, m.alloc, ids, last_tokens, DEV,
                                                                  permuted_tables=permuted,
                                                                  device_tables=m.device_tables)
    assert not preempted
    T_pad = tokens.shape[0]
    n = md.num_valid_tokens
    worst = 0.0
    for l, layer in enumerate(m.layers):
        qkv = torch.randn((T_pad, (m.Hq + 2 * m.Hkv) * D), generator=m.g).half()
        dqkv = qkv.to(DEV)
        q, k, v = dqkv.split([m.Hq * D, m.Hkv * D, m.Hkv * D], dim=-1)          # models/llama.py:157-158
        q0, k0 = qkv[:, :m.Hq * D].clone(), qkv[:, m.Hq * D:(m.Hq + m.Hkv) * D].clone()
        out = layer(positions, q, k, v, k_pool, v_pool, md, None)
        torch.cuda.synchronize()
        # rotary: in place on q and k, against the textbook form (one fp16 rounding apart)
        rq, rk = orc.rotary_neox(positions[:n].cpu(), q0, k0)
        gq, gk = q[:n].cpu(), k[:n].cpu()
        assert (gq.float() - rq).abs().max() <= 4e-3 and (gk.float() - rk).abs().max() <= 4e-3
        assert torch.equal(q[n:].cpu(), q0[n:]) and torch.equal(k[n:].cpu(), k0[n:]), "padding rows rotated"
        # cache write + attention: the oracle consumes the GPU's rotated q, k so
        # that the comparison isolates the scatter (bit-exact) and the attention
        hv_in = qkv[:, (m.Hq + m.Hkv) * D:]
        orc.reshape_and_cache(gk, hv_in, hk, hv, md.slot_mapping.cpu(), layer=l, num_tokens=n)
        if md.num_prompt_tokens:
            want = orc.prefill_causal(gq, gk, hv_in[:n], md.prompt_lens, D ** -0.5, m.Hkv)
        else:
            want = orc.paged_decode(gq, hk, hv, md.block_tables.cpu(), md.context_lens.cpu().numpy(), D ** -0.5,
                                    layer=l)
        err = (out[:n].float().cpu() - want).abs().max().item()
        assert err <= TOL, f"{m.name} layer {l}: max-abs error {err:.3e}"
        worst = max(worst, err)
    return worst


@pytest.mark.parametrize("permuted,fused_max,device_rows", [(True, 512, 0), (False, 512, 0), (True, 0, 0),
                                                            (True, 60, 0), (True, 512, 8)])
def test_two_models_share_one_pool_prefill_then_decode(permuted, fused_max, device_rows):
    """fused_max: steps of up to that many tokens rotate and write the cache in
    one launch (0: always the two kernels; 60: decode steps fused, prefill not).
    device_rows > 0: slot mapping and block tables are built on the device."""
    print(f"[case] serving path permuted_tables={permuted} fused_rope_max_tokens={fused_max} "
          f"device_rows={device_rows}", flush=True)
    bs, N = 16, 6000
    storage = KVStorage(N)
    k_pool, v_pool = allocate_gpu_cache(N, bs, DEV)
    k_pool.zero_()
    v_pool.zero_()
    hk, hv = k_pool.cpu(), v_pool.cpu()
    a = _Model("small-mha", 2, 4, 4, storage, bs, seed=1, fused_rope_max_tokens=fused_max, device_rows=device_rows)
    b = _Model("gqa", 3, 8, 2, storage, bs, seed=2, fused_rope_max_tokens=fused_max, device_rows=device_rows)
    rng = np.random.Generator(np.random.PCG64(3))
    for m, lens, base_id in ((a, [5, 40, 17], 0), (b, [130, 16, 1, 33], 100)):
        for i, p in enumerate(lens):
            m.sched.add_request(rng.integers(0, 24000, size=p).astype(np.int32), base_id + i, 64)
    ids_a, ids_b = [0, 1, 2], [100, 101, 102, 103]
    _step(a, ids_a, [], k_pool, v_pool, hk, hv, permuted)           # prefill, model a
    _step(b, ids_b, [], k_pool, v_pool, hk, hv, permuted)           # prefill, model b (interleaved blocks)
    for step in range(20):                                          # decode, crossing block boundaries
        _step(a, ids_a, [7 + step] * 3, k_pool, v_pool, hk, hv, permuted)
        _step(b, ids_b[::-1], [9 + step] * 4, k_pool, v_pool, hk, hv, permuted)
    # one model's sequence finishes; its blocks are reused by a new request of the other model
    storage.free_batch([1])
    a.sched.release_requests([1])
    b.sched.add_request(rng.integers(0, 24000, size=70).astype(np.int32), 104, 64)
    _step(b, [104], [], k_pool, v_pool, hk, hv, permuted)
    for step in range(3):
        _step(a, [0, 2], [1, 2], k_pool, v_pool, hk, hv, permuted)
        _step(b, ids_b + [104], [3] * 5, k_pool, v_pool, hk, hv, permuted)
    assert torch.equal(k_pool.cpu().view(torch.int16), hk.view(torch.int16))
    assert torch.equal(v_pool.cpu().view(torch.int16), hv.view(torch.int16))
    assert storage.num_free() + sum(storage.num_held(i) for i in [0, 2, 100, 101, 102, 103, 104]) == N


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("Hq,Hkv", [(3, 3), (8, 2)])
@pytest.mark.parametrize("bs", [16, 8])
def test_fused_rotary_cache_write_equals_the_two_kernels(dtype, Hq, Hkv, bs):
    """mux_rope_reshape_and_cache against mux_rotary_neox followed by
    mux_reshape_and_cache on the same inputs: q, k and both pools bitwise equal.
    Packed ragged prompts (runs at every phase) plus tokens without a slot,
    which are rotated but not written."""
    print(f"[case] fused rope + cache write {dtype} Hq={Hq} Hkv={Hkv} bs={bs}", flush=True)
    from muxserve_amd import workloads
    from muxserve_amd.attention import build_cos_sin_cache
    from muxserve_amd.pool import allocate_gpu_cache
    rng = np.random.Generator(np.random.PCG64(77 + bs))
    g = torch.Generator().manual_seed(77 + bs)
    lens = rng.permutation(np.arange(1, 30)).astype(np.int32)
    T = int(lens.sum())
    N = int(((lens + bs - 1) // bs).sum()) * Hkv + 5
    slots, _ = workloads.prefill_slot_mapping(lens, Hkv, bs, rng.permutation(N))
    slots[5, 0, 0] = -1
    slots[T - 1, 0, :] = -1
    pad = (T + 7) // 8 * 8
    qkv = torch.randn((pad, (Hq + 2 * Hkv) * D), generator=g).to(dtype).to(DEV)
    positions = torch.from_numpy(rng.integers(0, 2048, size=pad)).to(DEV)
    cos_sin = build_cos_sin_cache(D, 2048, 10000.0, DEV)
    dslots = torch.from_numpy(slots).to(DEV)
    results = []
    for fused in (False, True):
        x = qkv.clone()
        q, k, v = x.split([Hq * D, Hkv * D, Hkv * D], dim=-1)
        kp, vp = allocate_gpu_cache(N, bs, DEV, dtype=dtype)
        kp.zero_()
        vp.zero_()
        if fused:
            ops.rope_reshape_and_cache(positions, q, k, v, cos_sin, kp, vp, dslots, num_tokens=T)
        else:
            ops.rotary_neox(positions, q, k, cos_sin, num_tokens=T)
            ops.reshape_and_cache(k, v, kp, vp, dslots, num_tokens=T)
        torch.cuda.synchronize()
        results.append((x.cpu().view(torch.int16), kp.cpu().view(torch.int16), vp.cpu().view(torch.int16)))
    for a, b, what in zip(results[0], results[1], ("qkv rows", "k pool", "v pool")):
        assert torch.equal(a, b), f"{what} differ between the fused launch and the two kernels"
    assert torch.equal(results[1][0][T:], qkv.cpu().view(torch.int16)[T:]), "padding rows must not be touched"


@pytest.mark.parametrize("rope", [True, False])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_multi_model_cache_write_equals_one_launch_per_model(rope, dtype):
    """mux_multi_rope_reshape_and_cache over three colocated models (7B, 13B, a
    grouped-query shape; a decode-shaped step of single tokens for two of them
    and packed ragged prompts for the third, one empty model in between) against
    one call per model: q, k rows and both pools bitwise equal, and the plain
    variant bitwise equal to the oracle's scatter."""
    print(f"[case] multi-model cache write rope={rope} {dtype}", flush=True)
    from oracle import attn_oracle as orc
    from muxserve_amd import workloads
    from muxserve_amd.attention import build_cos_sin_cache
    from muxserve_amd.pool import allocate_gpu_cache
    bs, L, layer = 16, 2, 1
    rng = np.random.Generator(np.random.PCG64(91))
    g = torch.Generator().manual_seed(91)
    shapes = [(32, 32, 32), (40, 40, 16), (8, 2, 0), (16, 4, None)]      # Hq, Hkv, decode tokens (None: prompts)
    lens3 = rng.permutation(np.arange(1, 24)).astype(np.int32)
    need = sum(hk * (t if t is not None else int(((lens3 + bs - 1) // bs).sum())) for _, hk, t in shapes)
    N = need + 11
    ids = rng.permutation(N)
    cos_sin = build_cos_sin_cache(D, 4096, 10000.0, DEV)
    models, cur = [], 0
    for hq, hk, t in shapes:
        if t is None:
            slots1, used = workloads.prefill_slot_mapping(lens3, hk, bs, ids[cur:])
            T = int(lens3.sum())
        else:
            # a decode step: every sequence writes one token somewhere inside its last block
            T = t
            blk = ids[cur:cur + T * hk].reshape(T, hk).astype(np.int64)
            slots1 = (blk * bs + rng.integers(0, bs, size=(T, 1)))[:, None, :]
            used = T * hk
        cur += used
        slots = np.full((T, L, hk), -1, dtype=np.int64)
        slots[:, layer, :] = slots1[:, 0, :]
        if T > 3:
            slots[2, layer, 0] = -1
        pad = (T + 7) // 8 * 8
        qkv = torch.randn((pad, (hq + 2 * hk) * D), generator=g).to(dtype).to(DEV)
        pos = torch.from_numpy(rng.integers(0, 4096, size=pad)).to(DEV)
        models.append((hq, hk, T, qkv, pos, torch.from_numpy(slots).to(DEV), slots))
    results = []
    for fused in (False, True):
        kp, vp = allocate_gpu_cache(N, bs, DEV, dtype=dtype)
        kp.zero_()
        vp.zero_()
        xs, calls = [], []
        for hq, hk, T, qkv, pos, dslots, _ in models:
            x = qkv.clone()
            xs.append(x)
            q, k, v = x.split([hq * D, hk * D, hk * D], dim=-1)
            if fused:
                calls.append(ops.CacheWriteCall(k, v, dslots, layer=layer, positions=pos if rope else None,
                                                cos_sin=cos_sin if rope else None, q=q if rope else None,
                                                num_tokens=T))
            elif rope:
                ops.rope_reshape_and_cache(pos, q, k, v, cos_sin, kp, vp, dslots, layer=layer, num_tokens=T)
            else:
                ops.reshape_and_cache(k, v, kp, vp, dslots, layer=layer, num_tokens=T)
        if fused:
            ops.multi_reshape_and_cache(calls, kp, vp)
        torch.cuda.synchronize()
        results.append(([x.cpu().view(torch.int16) for x in xs], kp.cpu(), vp.cpu()))
    for xa, xb in zip(results[0][0], results[1][0]):
        assert torch.equal(xa, xb), "q/k rows differ between the fused launch and the per-model launches"
    assert torch.equal(results[0][1].view(torch.int16), results[1][1].view(torch.int16))
    assert torch.equal(results[0][2].view(torch.int16), results[1][2].view(torch.int16))
    if not rope:
        hk_pool, hv_pool = orc.allocate_pool(N, bs, dtype)
        hk_pool.zero_()
        hv_pool.zero_()
        for hq, hk, T, qkv, pos, _, slots in models:
            if T == 0:
                continue
            _, k, v = qkv.cpu().split([hq * D, hk * D, hk * D], dim=-1)
            orc.reshape_and_cache(k[:T], v[:T], hk_pool, hv_pool, torch.from_numpy(slots), layer=layer)
        assert torch.equal(results[1][1].view(torch.int16), hk_pool.view(torch.int16))
        assert torch.equal(results[1][2].view(torch.int16), hv_pool.view(torch.int16))


def test_empty_steps_are_accepted():
    """No tokens, no sequences, no prompts, no sampled rows: every entry point
    returns without launching and without touching its outputs."""
    print("[case] empty steps", flush=True)
    from muxserve_amd.attention import build_cos_sin_cache
    H, bs, N = 2, 16, 64
    k_pool, v_pool = allocate_gpu_cache(N, bs, DEV)
    k_pool.fill_(3.0)
    v_pool.fill_(3.0)
    e16 = torch.empty((0, H * D), dtype=torch.float16, device=DEV)
    slots = torch.empty((0, 1, H), dtype=torch.int64, device=DEV)
    pos = torch.empty((0,), dtype=torch.int64, device=DEV)
    cos_sin = build_cos_sin_cache(D, 64, 10000.0, DEV)
    ops.reshape_and_cache(e16, e16, k_pool, v_pool, slots)
    ops.rotary_neox(pos, e16, e16, cos_sin)
    ops.rope_reshape_and_cache(pos, e16, e16, e16, cos_sin, k_pool, v_pool, slots)
    # a padded batch whose valid part is empty
    pad = torch.full((8, H * D), 5.0, dtype=torch.float16, device=DEV)
    ops.reshape_and_cache(pad, pad, k_pool, v_pool, torch.zeros((8, 1, H), dtype=torch.int64, device=DEV), num_tokens=0)
    out = torch.full((8, H * D), 7.0, dtype=torch.float16, device=DEV)
    ops.paged_decode(out, pad, k_pool, v_pool, torch.empty((1, 0, H, 4), dtype=torch.int32, device=DEV),
                     torch.empty((0,), dtype=torch.int32, device=DEV), 0, D ** -0.5)
    ops.prefill_causal(out, pad, pad, pad, torch.zeros((1,), dtype=torch.int32, device=DEV), 0, D ** -0.5, H)
    assert ops.rms_norm(e16[:, :64], torch.ones((64,), dtype=torch.float16, device=DEV), 1e-6).shape == (0, 64)
    assert ops.silu_and_mul(e16).shape == (0, H * D // 2)
    emb = torch.zeros((32, 256), dtype=torch.float16, device=DEV)
    assert ops.greedy_sample(emb, torch.zeros((8, 256), dtype=torch.float16, device=DEV), 32, 0).shape == (0,)
    torch.cuda.synchronize()
    assert (out == 7.0).all() and (k_pool == 3.0).all() and (v_pool == 3.0).all()
