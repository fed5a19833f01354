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


def test_long_context_gqa_bf16_full_size_pool():
    """Config 5 at its real shape.  The oracle runs on a compact host copy of
    the referenced blocks for a subset of the sequences."""
    print("[case] long-context gqa", flush=True)
    bs = 16
    N = int(200e9) // 8192 // 128 * 128
    k_pool, v_pool = allocate_gpu_cache(N, bs, DEV, dtype=torch.bfloat16)
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
    pick = [0, 17, int(np.argmax(m.context_lens)), int(np.argmin(m.context_lens))]
    sub = workloads.DecodeModel(m.name, m.num_q_heads, m.num_kv_heads, m.context_lens[pick].copy(),
                                m.block_tables[:, pick].copy(), m.scale)
    ks, vs, tables = workloads.compact_to_host(k_pool, v_pool, [sub], bs)
    want = orc.paged_decode(m.q[pick].cpu(), ks, vs, tables[0], sub.context_lens, m.scale)
    got = m.out[pick].float().cpu()
    bound = 2e-3 + want.abs() * 2.0 ** -8          # + rounding of the bf16 result
    assert ((got - want).abs() - bound).max().item() <= 0, (got - want).abs().max().item()
