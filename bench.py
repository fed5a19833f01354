#!/usr/bin/env python3
"""Headline benchmark: mixed three-model paged decode attention over one
head-granular KV pool on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload (config.workload = "mixed3_decode"): three colocated models sharing a
pool sized to 60% of HBM - 7B shape (32 heads, batch 32), 13B (40 heads, batch
16), 30B (52 heads, batch 8), head size 128, fp16, block size 16, context
lengths lognormal(median 300, sigma 0.8) clipped to [16, 2048]; every (model,
sequence, head, logical block) owns a distinct block id drawn from the whole
pool.  One "step" = one layer of each model = ONE fused launch over one batch.
`--sets` independent batches (disjoint blocks, ~0.43 GB each) are visited round
robin so the working set is several times the 256 MB last-level cache.

Prints one JSON line: tokens/s (sum of batch sizes / step time), the roofline
object for the decode kernel (algorithmic bytes / measured duration vs 8 TB/s)
and the CPU baseline (the oracle's restatement of the same path, timed on a
bounded sample on this box's host cores).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--sets", type=int, default=6, help="distinct batches rotated through")
    ap.add_argument("--partition", type=int, default=0, help="tokens per context split (0 = library default)")
    ap.add_argument("--pool-util", type=float, default=0.6)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-hint", action="store_true", help="do not pass the host-side sum of context lengths")
    ap.add_argument("--unfused", action="store_true", help="one launch per model instead of one fused launch")
    return ap.parse_args()


def cpu_baseline(models, k_pool, v_pool, block_size, budget_s=12.0):
    """Time the oracle (torch-CPU gather + fp32 softmax attention) on a bounded
    sample: the first sequences of each model in the mix's 4:2:1 ratio."""
    import torch
    from oracle import attn_oracle as orc
    from muxserve_amd import workloads

    take = (4, 2, 1)
    sample = []
    for m, n in zip(models, take):
        sub = workloads.DecodeModel(m.name, m.num_q_heads, m.num_kv_heads, m.context_lens[:n].copy(),
                                    m.block_tables[:, :n].copy(), m.scale)
        sub.q = m.q[:n]
        sample.append(sub)
    ks, vs, tables = workloads.compact_to_host(k_pool, v_pool, sample, block_size)
    qs = [s.q.cpu() for s in sample]
    threads = os.cpu_count() or 1
    torch.set_num_threads(threads)

    def once():
        for s, t, q in zip(sample, tables, qs):
            orc.paged_decode(q, ks, vs, t, s.context_lens, s.scale)

    once()
    reps, t0 = 0, time.perf_counter()
    while True:
        once()
        reps += 1
        dt = time.perf_counter() - t0
        if dt > budget_s or reps >= 50:
            break
    tokens = sum(take)
    return {
        "value": tokens * reps / dt,
        "unit": "tokens/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"first {take[0]}/{take[1]}/{take[2]} sequences of the 7b/13b/30b models "
                  f"(ctx {[int(c) for s in sample for c in s.context_lens]}), {reps} reps in {dt:.1f} s",
    }


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives or sharding); use --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import torch
    from muxserve_amd import ops, workloads
    from muxserve_amd.pool import allocate_gpu_cache, num_gpu_blocks
    from oracle import attn_oracle as orc   # traffic formula + cpu baseline only

    dev = "cuda:0"
    bs = 16
    total_mem = torch.cuda.get_device_properties(0).total_memory
    N = num_gpu_blocks(args.pool_util, total_mem, bs)
    k_pool, v_pool = allocate_gpu_cache(N, bs, dev)

    # Disjoint ids for all sets from one seeded draw over the whole pool.
    rng = np.random.Generator(np.random.PCG64(args.seed))
    probe = [workloads.config2(seed=args.seed + 1 + i, num_pool_blocks=N, id_perm=np.arange(1 << 20))[1]
             for i in range(args.sets)]
    ids = rng.choice(N, size=int(sum(probe)), replace=False)
    sets, off = [], 0
    for i in range(args.sets):
        models, need = workloads.config2(seed=args.seed + 1 + i, num_pool_blocks=N, id_perm=ids[off:off + probe[i]])
        off += need
        used = np.concatenate([m.used_blocks(bs) for m in models])
        workloads.fill_blocks(k_pool, v_pool, used, seed=args.seed + 100 + i)
        for j, m in enumerate(models):
            m.to_device(dev, torch.float16, seed=args.seed + 1000 + 10 * i + j)
        calls = [ops.DecodeCall(m.out, m.q, m.d_block_tables, m.d_context_lens, m.max_context_len, m.scale,
                                total_context_len=0 if args.no_hint else int(m.context_lens.sum()))
                 for m in models]
        sets.append((models, calls))
    torch.cuda.synchronize()

    def step(i):
        calls = sets[i % len(sets)][1]
        if args.unfused:
            for c in calls:
                ops.multi_decode([c], k_pool, v_pool, partition_size=args.partition)
        else:
            ops.multi_decode(calls, k_pool, v_pool, partition_size=args.partition)

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    for i in range(args.steps):
        step(i)
    ev1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    ev_ms = ev0.elapsed_time(ev1) / args.steps
    ms = max(wall_ms, ev_ms)

    tokens = sum(m.batch for m in sets[0][0])
    step_bytes = [sum(orc.decode_bytes(m.context_lens, m.num_q_heads, m.num_kv_heads, bs) for m in models)
                  for models, _ in sets]
    visits = [len(range(i, args.steps, len(sets))) for i in range(len(sets))]
    avg_bytes = sum(b * v for b, v in zip(step_bytes, visits)) / max(1, sum(visits))
    achieved = avg_bytes / (ev_ms * 1e-3) / 1e9

    result = {
        "metric": "multi-LLM decode attn tokens/s + achieved HBM GB/s (% of ~8 TB/s), 1 GPU",
        "value": tokens / (ms * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {
            "workload": "mixed3_decode",
            "models": "7b(H32,B32)+13b(H40,B16)+30b(H52,B8), one layer each, one fused launch per step",
            "head_size": 128, "block_size": bs, "pool_blocks": int(N), "pool_gb": round(N * 8192 / 1e9, 1),
            "tokens_per_step": tokens, "sets": args.sets, "partition": args.partition,
            "bytes_per_step": int(avg_bytes), "fused": not args.unfused, "seed": args.seed,
        },
        "roofline": {
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS,
            "traffic": None,
            "kernel": "paged_decode_kernel<F16,16,1>",
            "event_ms_per_step": ev_ms,
        },
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(sets[0][0], k_pool, v_pool, bs)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
