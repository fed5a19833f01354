"""A model runtime that lives in a process of its own and works on a KV pool it
does not own (started by tests/test_gpu_flexstore_ipc.py): asks the FlexStore
side for the pool ("cache_init"), maps it from the handle it is sent, then runs
a prefill step and decode steps of a small two-layer model through
prepare_inputs and PagedAttentionWithRoPE - cache writes and paged decode
attention over the other process's memory.  Records inputs and outputs of every
layer call for the parent to check.

    python flexstore_gpu_runtime_process.py ADDRESS OUT.pkl
"""
import os
import pickle
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)


def main():
    address, out_path = sys.argv[1], sys.argv[2]
    import torch
    from muxserve_amd.attention import PagedAttentionWithRoPE
    from muxserve_amd.batch_scheduler import BatchScheduler
    from muxserve_amd.flexstore import rebuild_tensor
    from muxserve_amd.flexstore_service import PipeClient
    from muxserve_amd.prepare import prepare_inputs

    client = None
    for _ in range(200):
        try:
            client = PipeClient(address)
            break
        except (FileNotFoundError, ConnectionRefusedError):
            time.sleep(0.05)
    assert client is not None
    model, L, Hq, Hkv, D, bs = "small", 2, 8, 4, 128, 16
    print("[runtime] asking for the pool", flush=True)
    k_meta, v_meta = client.request("cache_init", [0, model])
    k_pool, v_pool = rebuild_tensor(k_meta), rebuild_tensor(v_meta)
    print(f"[runtime] pool mapped: {tuple(k_pool.shape)} {k_pool.dtype} on {k_pool.device}", flush=True)
    assert client.request("get_num_blocks") == k_pool.shape[0]

    sched = BatchScheduler(L, Hkv, 512, bs)
    layers = [PagedAttentionWithRoPE(Hq, D, D ** -0.5, base=10000, max_position=2048, rotary_dim=D, num_kv_heads=Hkv,
                                     rope_scaling=None, layer_idx=l) for l in range(L)]
    rng = np.random.Generator(np.random.PCG64(5))
    g = torch.Generator().manual_seed(5)
    lens = [37, 300, 16, 1]
    for i, n in enumerate(lens):
        sched.add_request(rng.integers(0, 32000, size=n).astype(np.int32), i, 32)
    ids = list(range(len(lens)))
    alloc = client.cache_alloc_for(model)
    record = []
    for step, last in enumerate([[]] + [[5 + s] * len(ids) for s in range(3)]):
        tokens, positions, md, batch_reqs, preempted = prepare_inputs(sched, alloc, ids, last, "cuda:0")
        assert not preempted
        n = md.num_valid_tokens
        for l, layer in enumerate(layers):
            qkv = torch.randn((tokens.shape[0], (Hq + 2 * Hkv) * D), generator=g).half()
            dqkv = qkv.to("cuda:0")
            q, k, v = dqkv.split([Hq * D, Hkv * D, Hkv * D], dim=-1)
            out = layer(positions, q, k, v, k_pool, v_pool, md, None)
            torch.cuda.synchronize()
            record.append({"step": step, "layer": l, "n": n, "prompt_lens": list(md.prompt_lens),
                           "positions": positions.cpu(), "qkv_in": qkv, "q_rot": q.cpu(), "k_rot": k.cpu(),
                           "out": out.cpu(), "slot_mapping": md.slot_mapping.cpu(),
                           "block_tables": md.block_tables.cpu(), "context_lens": md.context_lens.cpu()})
        print(f"[runtime] step {step} done ({n} tokens)", flush=True)
    sched.release_requests(ids)
    client.request("free_cache", [model, ids])
    del k_pool, v_pool
    client.close()
    with open(out_path, "wb") as f:
        pickle.dump({"shape": (L, Hq, Hkv, D, bs), "record": record}, f)
    print("[runtime] finished", flush=True)


if __name__ == "__main__":
    main()
