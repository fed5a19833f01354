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
from muxserve_amd.attention import PagedAttentionWithRoPE
from muxserve_amd.batch_scheduler import BatchScheduler
from muxserve_amd.memory_manager import KVStorage
from muxserve_amd.pool import HEAD_SIZE, allocate_gpu_cache
from muxserve_amd.prepare import prepare_inputs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
D = HEAD_SIZE
TOL = 2e-3


class _Model:
    def __init__(self, name, L, Hq, Hkv, storage, bs, seed):
        self.name, self.L, self.Hq, self.Hkv = name, L, Hq, Hkv
        self.sched = BatchScheduler(L, Hkv, 512, bs)
        self.storage = storage
        self.layers = [PagedAttentionWithRoPE(Hq, D, D ** -0.5, base=10000, max_position=2048, rotary_dim=D,
                                              num_kv_heads=Hkv, rope_scaling=None, layer_idx=l) for l in range(L)]
        self.g = torch.Generator().manual_seed(seed)

    def alloc(self, req):
        return self.storage.allocate_batch(req, self.L, self.Hkv)


def _step(m, ids, last_tokens, k_pool, v_pool, hk, hv, permuted):
    tokens, positions, md, batch_reqs, preempted = prepare_inputs(m.sched, m.alloc, ids, last_tokens, DEV,
                                                                  permuted_tables=permuted)
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


@pytest.mark.parametrize("permuted", [True, False])
def test_two_models_share_one_pool_prefill_then_decode(permuted):
    print(f"[case] serving path permuted_tables={permuted}", flush=True)
    bs, N = 16, 6000
    storage = KVStorage(N)
    k_pool, v_pool = allocate_gpu_cache(N, bs, DEV)
    k_pool.zero_()
    v_pool.zero_()
    hk, hv = k_pool.cpu(), v_pool.cpu()
    a = _Model("small-mha", 2, 4, 4, storage, bs, seed=1)
    b = _Model("gqa", 3, 8, 2, storage, bs, seed=2)
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
