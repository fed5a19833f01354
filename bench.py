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
MFMA_PEAK_TFLOPS = 2500.0     # dense fp16 / bf16
# HBM bytes moved per algorithmic byte by the decode kernel on this workload,
# from the FETCH_SIZE / WRITE_SIZE counter passes summarised in
# profiles/paged_decode_mixed3_hbm_traffic.txt (420.6 MB measured / 410.6 MB).
MIXED3_TRAFFIC_RATIO = 1.024
# Same for the grouped-query decode kernel (profiles/paged_decode_gqa_long_kernel_trace_and_traffic.txt:
# 1369.5 MB / 1358.8 MB) and the prefill-shaped cache write
# (profiles/reshape_and_cache_write_kernel_trace_and_traffic.txt: 231.9 MB / 219.8 MB).
GQA_LONG_TRAFFIC_RATIO = 1.008
CACHE_WRITE_TRAFFIC_RATIO = 1.055


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--sets", type=int, default=6, help="distinct batches rotated through")
    ap.add_argument("--partition", type=int, default=0, help="tokens per context split (0 = library default)")
    ap.add_argument("--pool-util", type=float, default=0.6)
    ap.add_argument("--batch-scale", type=int, default=1,
                    help="mixed3_decode: multiply the three models' batches (32/16/8 sequences) by this; 1 is the "
                         "headline configuration, larger values show how the launch scales")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-hint", action="store_true", help="do not pass the host-side sum of context lengths")
    ap.add_argument("--no-host-lens", action="store_true",
                    help="do not pass the host copy of the context lengths (units are then enumerated on the device)")
    ap.add_argument("--no-prompt-order", action="store_true",
                    help="prefill3: start the prompts' workgroups as packed instead of longest first")
    ap.add_argument("--no-prompt-lens", action="store_true",
                    help="prefill3: do not pass the host-side prompt lengths (grid sized by the longest prompt)")
    ap.add_argument("--unfused", action="store_true", help="one launch per model instead of one fused launch")
    ap.add_argument("--prompt-cap", type=int, default=0,
                    help="prefill_timeline: cut the prompts of the three-model mix at this length (0 = as drawn)")
    ap.add_argument("--long-prompts", action="store_true",
                    help="prefill_timeline: 16 prompts of 2048 tokens, 32 heads, instead of the three-model mix")
    ap.add_argument("--workload", default="mixed3_decode",
                    choices=["mixed3_decode", "prefill3", "cache_write", "colocated", "gqa_long", "model_ops", "host_step",
                             "cu_masks", "prefill_long", "decode_timeline", "prefill_timeline", "gqa_timeline", "mfma_ceiling"],
                    help="mixed3_decode is the headline metric; the others are the remaining synthetic "
                         "shapes, each printing its own JSON line")
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
    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or min(os.cpu_count() or 1, 16)
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
        if dt > budget_s:
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


def _time(fn, steps, warmup, stream=None):
    """Average milliseconds per call of fn(i), HIP events on `stream` (torch's
    current stream if None)."""
    import torch
    st = stream if stream is not None else torch.cuda.current_stream()
    for i in range(warmup):
        fn(i)
    st.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(st)
    for i in range(steps):
        fn(i)
    e1.record(st)
    e1.synchronize()
    return e0.elapsed_time(e1) / steps


# The matrix-core kernels of a process start below their later rate: the first tens of launches run at a lower
# shader clock (SQ_BUSY_CU_CYCLES per launch stays the same while the launch takes up to a fifth longer).  The prefill
# workloads therefore warm up with at least this many launches and report the first launches' time beside the steady one.
PREFILL_MIN_WARMUP = 100


def _line(metric, value, unit, args, ms, config, roofline, dtype="f16", higher=True):
    return {"metric": metric, "value": value, "unit": unit, "n_gpus": 1, "steps": args.steps,
            "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": higher, "scaling": "weak",
            "vs_baseline": None, "dtype": dtype, "data": "synthetic", "config": config, "roofline": roofline}


def bench_prefill3(args):
    """Config 3: causal prefill attention (MFMA) of 16 prompts per model, then
    the cache write of the same tokens into head-wise slot mappings."""
    import torch
    from muxserve_amd import ops, workloads
    from muxserve_amd.pool import HEAD_SIZE as D, allocate_gpu_cache
    dev, bs = "cuda:0", 16
    models = workloads.config3(seed=args.seed)
    total_blocks = sum(int(((m.prompt_lens + bs - 1) // bs).sum()) * m.num_kv_heads for m in models)
    N = total_blocks + 4096
    ids = np.random.Generator(np.random.PCG64(args.seed)).permutation(N)
    k_pool, v_pool = allocate_gpu_cache(N, bs, dev)
    g = torch.Generator().manual_seed(args.seed)
    work, cur, flops, wbytes, tokens = [], 0, 0.0, 0, 0
    for m in models:
        T, Hq, Hkv = m.num_tokens, m.num_q_heads, m.num_kv_heads
        pad = (T + 7) // 8 * 8
        qkv = torch.randn((pad, (Hq + 2 * Hkv) * D), generator=g).half().to(dev)
        q, k, v = qkv.split([Hq * D, Hkv * D, Hkv * D], dim=-1)
        out = torch.empty((pad, Hq * D), dtype=torch.float16, device=dev)
        cu = torch.from_numpy(m.cu_seqlens()).to(dev)
        slots, used = workloads.prefill_slot_mapping(m.prompt_lens, Hkv, bs, ids[cur:])
        cur += used
        order = torch.from_numpy(np.argsort(-m.prompt_lens, kind="stable").astype(np.int32)).to(dev)
        work.append((m, q, k, v, out, cu, torch.from_numpy(slots).to(dev), T, order))
        flops += workloads.prefill_flops(m.prompt_lens, Hq)
        wbytes += workloads.cache_write_bytes(T, Hkv)
        tokens += T

    import ctypes
    lens_of = {w[0].name: (ctypes.c_int32 * len(w[0].prompt_lens))(*[int(x) for x in w[0].prompt_lens]) for w in work}

    def attn(_):
        for m, q, k, v, out, cu, slots, T, order in work:
            ops.prefill_causal(out, q, k, v, cu, int(m.prompt_lens.max()), m.scale, m.num_kv_heads,
                               prompt_order=None if args.no_prompt_order else order,
                               prompt_lens=None if (args.no_prompt_lens or args.no_prompt_order) else lens_of[m.name])

    def write(_):
        for m, q, k, v, out, cu, slots, T, order in work:
            ops.reshape_and_cache(k, v, k_pool, v_pool, slots, num_tokens=T)

    # the three models' prompts in ONE launch, and the three cache writes in one
    pcalls = [ops.PrefillCall(out, q, k, v, cu, [int(x) for x in m.prompt_lens], m.scale, m.num_kv_heads)
              for m, q, k, v, out, cu, slots, T, order in work]
    wcalls = [ops.CacheWriteCall(k, v, slots, num_tokens=T) for m, q, k, v, out, cu, slots, T, order in work]
    fused = (lambda _: ops.multi_prefill_causal(pcalls)) if not args.unfused else attn
    ms_first = _time(fused, 20, 0)
    warm = max(args.warmup, PREFILL_MIN_WARMUP)
    ms_separate = _time(attn, args.steps, warm)
    ms_a = ms_separate if args.unfused else _time(fused, args.steps, warm)
    ms_w_separate = _time(write, args.steps, args.warmup)
    ms_w = ms_w_separate if args.unfused else _time(lambda _: ops.multi_reshape_and_cache(wcalls, k_pool, v_pool),
                                                    args.steps, args.warmup)
    tf = flops / (ms_a * 1e-3) / 1e12
    gbs = wbytes / (ms_w * 1e-3) / 1e9
    cfg = {"workload": "prefill3", "prompts_per_model": 16, "tokens": tokens, "flops": flops,
           "fused": not args.unfused, "one_launch_per_model_ms": ms_separate, "warmup_launches": warm,
           "first_20_launches_of_the_process_ms": ms_first,
           "cache_write_one_launch_per_model_ms": ms_w_separate, "cache_write_ms": ms_w, "cache_write_gbs": gbs, "cache_write_frac_of_hbm": gbs / HBM_PEAK_GBS}
    roof = {"bound": "mfma", "achieved": tf, "peak": 2500.0, "unit": "TFLOP/s", "frac": tf / 2500.0,
            "traffic": None, "kernel": "prefill_causal_kernel<F16>"}
    return _line("prefill causal attention tokens/s (3 models, 16 prompts each)", tokens / (ms_a * 1e-3),
                 "tokens/s", args, ms_a, cfg, roof)


def bench_prefill_long(args):
    """The prefill kernel alone on long prompts: 16 prompts x 2048 tokens of a
    7B-shaped layer (32 heads x 128), fp16."""
    import torch
    from muxserve_amd import ops, workloads
    from muxserve_amd.pool import HEAD_SIZE as D
    dev, P, L, H = "cuda:0", 16, 2048, 32
    g = torch.Generator().manual_seed(args.seed)
    qkv = torch.randn((P * L, 3 * H * D), generator=g).half().to(dev)
    q, k, v = qkv.split([H * D] * 3, dim=-1)
    out = torch.empty((P * L, H * D), dtype=torch.float16, device=dev)
    cu = torch.arange(0, P * L + 1, L, dtype=torch.int32, device=dev)
    lens = [L] * P
    step = lambda _: ops.prefill_causal(out, q, k, v, cu, L, D ** -0.5, H,                          # noqa: E731
                                        prompt_lens=None if args.no_prompt_lens else lens)
    ms_first = _time(step, 20, 0)
    warm = max(args.warmup, PREFILL_MIN_WARMUP)
    ms = _time(step, args.steps, warm)
    flops = workloads.prefill_flops(np.asarray(lens), H)
    tf = flops / (ms * 1e-3) / 1e12
    cfg = {"workload": "prefill_long", "prompts": P, "prompt_len": L, "heads": H, "flops": flops,
           "warmup_launches": 20 + warm, "first_20_launches_of_the_process_ms": ms_first}
    roof = {"bound": "mfma", "achieved": tf, "peak": 2500.0, "unit": "TFLOP/s", "frac": tf / 2500.0,
            "traffic": None, "kernel": "prefill_causal_kernel<F16>"}
    return _line("prefill causal attention tokens/s (16 prompts x 2048 tokens, 32 heads)", P * L / (ms * 1e-3),
                 "tokens/s", args, ms, cfg, roof)


def bench_cache_write(args):
    """reshape_and_cache alone: decode-shaped (one token per sequence, the three
    models of the mix) and prefill-shaped (30B shape, 4 x 1024 tokens)."""
    import torch
    from muxserve_amd import ops, workloads
    from muxserve_amd.pool import HEAD_SIZE as D, allocate_gpu_cache
    dev, bs = "cuda:0", 16
    N = 1 << 20
    k_pool, v_pool = allocate_gpu_cache(N, bs, dev)
    rng = np.random.Generator(np.random.PCG64(args.seed))
    g = torch.Generator().manual_seed(args.seed)
    out = {}
    # decode-shaped: random distinct slots
    dec = []
    for (hk, b) in ((32, 32), (40, 16), (52, 8)):
        slots = rng.choice(N * bs, size=b * hk, replace=False).reshape(b, 1, hk).astype(np.int64)
        kv = torch.randn((b, 2 * hk * D), generator=g).half().to(dev)
        dec.append((kv[:, :hk * D], kv[:, hk * D:], torch.from_numpy(slots).to(dev), b, hk))
    ms_d = _time(lambda _: [ops.reshape_and_cache(k, v, k_pool, v_pool, s) for k, v, s, b, hk in dec],
                 args.steps, args.warmup)
    bytes_d = sum(workloads.cache_write_bytes(b, hk) for *_, b, hk in dec)
    # the same three writes in one launch; with the rotary embedding fused; and the whole
    # attention part of a three-model decode step: rope + cache write (one launch) + paged
    # decode attention (one launch) over the mix's contexts
    plain_calls = [ops.CacheWriteCall(k, v, s) for k, v, s, b, hk in dec]
    plain_items = ops.cache_write_items(plain_calls, k_pool.dtype)      # checked once, not per launch
    ms_d1 = _time(lambda _: ops.multi_reshape_and_cache(plain_items, k_pool, v_pool), args.steps, args.warmup)
    from muxserve_amd.attention import build_cos_sin_cache
    cos_sin = build_cos_sin_cache(D, 4096, 10000.0, dev)
    mix, _need = workloads.config2(seed=args.seed + 1, num_pool_blocks=N)
    rope_calls, dcalls = [], []
    for m, (k, v, s, b, hk) in zip(mix, dec):
        m.to_device(dev, torch.float16, seed=7)
        pos = torch.from_numpy(m.context_lens.astype(np.int64) - 1).to(dev)
        rope_calls.append(ops.CacheWriteCall(k, v, s, positions=pos, cos_sin=cos_sin, q=m.q[:b]))
        dcalls.append(ops.DecodeCall(m.out, m.q, m.d_block_tables, m.d_context_lens, m.max_context_len, m.scale,
                                     total_context_len=int(m.context_lens.sum()),
                                     context_lens_host=torch.from_numpy(np.ascontiguousarray(m.context_lens,
                                                                                             dtype=np.int32))))
    rope_items = ops.cache_write_items(rope_calls, k_pool.dtype)
    ms_dr = _time(lambda _: ops.multi_reshape_and_cache(rope_items, k_pool, v_pool), args.steps, args.warmup)

    def attention_part(_):
        ops.multi_reshape_and_cache(rope_items, k_pool, v_pool)
        ops.multi_decode(dcalls, k_pool, v_pool)

    ms_step = _time(attention_part, args.steps, args.warmup)
    # prefill-shaped
    # Five sources and five disjoint sets of pool blocks in rotation (1.1 GB), so
    # that neither k/v nor the pool lines come from the 256 MB last-level cache.
    lens = np.full(4, 1024)
    T = int(lens.sum())
    perm = rng.permutation(N)
    per_set = int(((lens + bs - 1) // bs).sum()) * 52
    psets = []
    for i in range(5):
        slots, _ = workloads.prefill_slot_mapping(lens, 52, bs, perm[i * per_set:])
        kv = torch.randn((T, 2 * 52 * D), generator=g).half().to(dev)
        psets.append((kv, torch.from_numpy(slots).to(dev)))

    def write(i):
        kv, dslots = psets[i % len(psets)]
        ops.reshape_and_cache(kv[:, :52 * D], kv[:, 52 * D:], k_pool, v_pool, dslots)

    ms_p = _time(write, args.steps, args.warmup)
    ms_warm = _time(lambda _: write(0), args.steps, args.warmup)
    bytes_p = workloads.cache_write_bytes(T, 52)
    # The yardstick: a contiguous copy of as many bytes in and out (the probe library's copy
    # kernel, and the framework's), rotated over buffers the same way.
    from muxserve_amd import _lib as _l
    half = T * 52 * 2 * D * 2
    srcs = [kv for kv, _ in psets]
    dsts = [torch.empty((half,), dtype=torch.uint8, device=dev) for _ in psets]
    st = torch.cuda.current_stream().cuda_stream
    ms_copy = _time(lambda i: _l.probe().mux_probe_copy(dsts[i % 5].data_ptr(), srcs[i % 5].data_ptr(), half, st),
                    args.steps, args.warmup)
    ms_tcopy = _time(lambda i: dsts[i % 5].copy_(srcs[i % 5].view(torch.uint8).view(-1)), args.steps, args.warmup)
    # ... and the same copy with the cache write's own destinations: sources read contiguously,
    # every 4 KiB written to the pool block the step's slots name (one K and one V block per
    # workgroup), no windows, no transposition.
    flat = [kv.view(-1) for kv, _ in psets]
    blk_ids = [(ds[::bs, 0, :] // bs).reshape(-1).to(torch.int32).contiguous() for _, ds in psets]
    n_blk = int(blk_ids[0].numel())

    def scatter(i):
        f, ids = flat[i % 5], blk_ids[i % 5]
        rc = _l.probe().mux_probe_scatter_copy(k_pool.data_ptr(), v_pool.data_ptr(), N, f.data_ptr(),
                                               f[n_blk * 2048:].data_ptr(), ids.data_ptr(), n_blk, st)
        if rc != 0:
            raise RuntimeError(f"mux_probe_scatter_copy returned {rc}")

    ms_scopy = _time(scatter, args.steps, args.warmup)
    # Where the blocks lie matters for writes (it does not for reads): the same step and the same
    # probe with the step's blocks (a) as runs of 52 consecutive ids - what a layer's slice of the
    # allocator's [token block][layer][head] order looks like (csrc/memory_manager.cpp:104-135) -
    # and (b) as one consecutive run of the pool.
    by_pattern = {"random_permutation": {"kernel_ms": ms_p, "probe_ms": ms_scopy}}
    n_tb = per_set // 52
    for name, make in (("runs_of_52_consecutive_blocks",
                        lambda: (rng.choice(N // 52 - 1, size=n_tb, replace=False)[:, None] * 52 + np.arange(52)).reshape(-1)),
                       ("one_consecutive_run", lambda: np.arange(per_set) + int(rng.integers(0, N - per_set)))):
        alt = []
        for i in range(5):
            slots, _ = workloads.prefill_slot_mapping(lens, 52, bs, make())
            alt.append(torch.from_numpy(slots).to(dev))
        alt_ids = [(ds[::bs, 0, :] // bs).reshape(-1).to(torch.int32).contiguous() for ds in alt]

        def write_alt(i):
            kv = psets[i % 5][0]
            ops.reshape_and_cache(kv[:, :52 * D], kv[:, 52 * D:], k_pool, v_pool, alt[i % 5])

        def scatter_alt(i):
            f, ids = flat[i % 5], alt_ids[i % 5]
            rc = _l.probe().mux_probe_scatter_copy(k_pool.data_ptr(), v_pool.data_ptr(), N, f.data_ptr(),
                                                   f[n_blk * 2048:].data_ptr(), ids.data_ptr(), n_blk, st)
            if rc != 0:
                raise RuntimeError(f"mux_probe_scatter_copy returned {rc}")

        by_pattern[name] = {"kernel_ms": _time(write_alt, args.steps, args.warmup),
                            "probe_ms": _time(scatter_alt, args.steps, args.warmup)}
    for v in by_pattern.values():
        v["kernel_frac_of_hbm"] = bytes_p / (v["kernel_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS
        v["probe_frac_of_hbm"] = 2 * half / (v["probe_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS
    for i in range(5):          # the pool holds the probe's bytes now: put the step's own back
        write(i)
    gbs = bytes_p / (ms_p * 1e-3) / 1e9
    cfg = {"workload": "cache_write", "prefill_shape": "52 heads x 4096 tokens", "prefill_bytes": bytes_p,
           "same_buffers_every_step_ms": ms_warm, "same_buffers_every_step_gbs": bytes_p / (ms_warm * 1e-3) / 1e9,
           "contiguous_copy_of_the_same_bytes": {"probe_copy_ms": ms_copy, "probe_copy_gbs": 2 * half / (ms_copy * 1e-3) / 1e9,
                                                 "torch_copy_ms": ms_tcopy, "torch_copy_gbs": 2 * half / (ms_tcopy * 1e-3) / 1e9,
                                                 "scattered_to_the_steps_pool_blocks_ms": ms_scopy,
                                                 "scattered_to_the_steps_pool_blocks_gbs": 2 * half / (ms_scopy * 1e-3) / 1e9},
           "by_where_the_blocks_lie": by_pattern,
           "decode_shape": "7b/13b/30b, 56 tokens, three launches", "decode_ms": ms_d, "decode_bytes": bytes_d,
           "decode_gbs": bytes_d / (ms_d * 1e-3) / 1e9,
           "decode_one_fused_launch_ms": ms_d1, "decode_one_fused_launch_with_rope_ms": ms_dr,
           "decode_step_rope_write_attention_two_launches_ms": ms_step}
    roof = {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
            "traffic": bytes_p * CACHE_WRITE_TRAFFIC_RATIO,
            "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, profiles/reshape_and_cache_write_kernel_trace_and_traffic.txt",
            "kernel": "reshape_and_cache_kernel"}
    return _line("KV-cache write tokens/s (prefill-shaped, 52 heads)", T / (ms_p * 1e-3), "tokens/s", args, ms_p,
                 cfg, roof, dtype="u16")


def bench_colocated(args):
    """Config 4: a 30B-shaped prefill on 40% of the CUs concurrently with a
    7B-shaped decode on the other 60%, via CU-masked streams."""
    import torch
    from muxserve_amd import ops, workloads
    from muxserve_amd.pool import HEAD_SIZE as D, allocate_gpu_cache, num_gpu_blocks
    dev, bs = "cuda:0", 16
    N = num_gpu_blocks(args.pool_util, torch.cuda.get_device_properties(0).total_memory, bs)
    k_pool, v_pool = allocate_gpu_cache(N, bs, dev)
    rng = np.random.Generator(np.random.PCG64(args.seed))
    g = torch.Generator().manual_seed(args.seed)
    # decode: 7B shape, batch 64, ctx U[512, 1024]; a few rotating batches
    dsets = []
    for i in range(4):
        ctx = rng.integers(512, 1025, size=64).astype(np.int32)
        need = int(((ctx + bs - 1) // bs).sum()) * 32
        bt, _ = workloads.build_tables(ctx, 32, bs, rng.choice(N, size=need, replace=False))
        m = workloads.DecodeModel("7b", 32, 32, ctx, bt).to_device(dev, torch.float16, seed=i)
        dsets.append(m)
    dbytes = float(np.mean([workloads.decode_bytes(m.context_lens, 32, 32, bs) for m in dsets]))
    # prefill: 30B shape, 4 prompts x 1024 tokens
    T = 4096
    qkv = torch.randn((T, 3 * 52 * D), generator=g).half().to(dev)
    q, k, v = qkv.split([52 * D] * 3, dim=-1)
    pout = torch.empty((T, 52 * D), dtype=torch.float16, device=dev)
    cu = torch.tensor([0, 1024, 2048, 3072, 4096], dtype=torch.int32, device=dev)
    pflops = 4.0 * 52 * D * 4 * (1024 * 1025 / 2)
    s_pre, s_dec = ops.CUMaskedStream(0, 40), ops.CUMaskedStream(40, 100)

    host_lens = [torch.from_numpy(np.ascontiguousarray(m.context_lens, dtype=np.int32)) for m in dsets]

    def decode(i, stream=None):
        m = dsets[i % len(dsets)]
        ops.paged_decode(m.out, m.q, k_pool, v_pool, m.d_block_tables, m.d_context_lens, m.max_context_len,
                         m.scale, total_context_len=int(m.context_lens.sum()), stream=stream,
                         context_lens_host=host_lens[i % len(dsets)])

    def prefill(i, stream=None):
        ops.prefill_causal(pout, q, k, v, cu, 1024, D ** -0.5, 52, stream=stream)

    steps, warm = args.steps, max(args.warmup, PREFILL_MIN_WARMUP)      # (the prefill's clock: see PREFILL_MIN_WARMUP)
    res = {"decode_alone_full_ms": _time(decode, steps, warm), "prefill_alone_full_ms": _time(prefill, steps, warm)}
    res["decode_alone_60pct_ms"] = _time(lambda i: decode(i, s_dec), steps, warm, s_dec.torch_stream)
    res["prefill_alone_40pct_ms"] = _time(lambda i: prefill(i, s_pre), steps, warm, s_pre.torch_stream)
    # concurrent: keep both streams busy; each is timed on its own stream
    n_pre = max(4, int(steps * res["decode_alone_60pct_ms"] / res["prefill_alone_40pct_ms"]) + 2)
    torch.cuda.synchronize()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
    ev[0].record(s_dec.torch_stream)
    ev[2].record(s_pre.torch_stream)
    done_pre = 0
    for i in range(steps):
        decode(i, s_dec)
        while done_pre < (i + 1) * n_pre // steps:
            prefill(done_pre, s_pre)
            done_pre += 1
    ev[1].record(s_dec.torch_stream)
    ev[3].record(s_pre.torch_stream)
    torch.cuda.synchronize()
    res["decode_concurrent_ms"] = ev[0].elapsed_time(ev[1]) / steps
    res["prefill_concurrent_ms"] = ev[2].elapsed_time(ev[3]) / max(1, done_pre)
    res["cus"] = [s_pre.num_cus, s_dec.num_cus]
    gbs = dbytes / (res["decode_concurrent_ms"] * 1e-3) / 1e9
    res.update({"workload": "colocated", "decode_bytes": dbytes, "prefill_flops": pflops,
                "prefill_concurrent_tflops": pflops / (res["prefill_concurrent_ms"] * 1e-3) / 1e12,
                "decode_alone_full_gbs": dbytes / (res["decode_alone_full_ms"] * 1e-3) / 1e9})
    roof = {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
            "traffic": None, "kernel": "paged_decode_kernel<F16,16,1,4> on 60% of CUs, prefill on the rest"}
    return _line("decode attn tokens/s on 60% of CUs while a prefill runs on 40%", 64 / (res["decode_concurrent_ms"] * 1e-3),
                 "tokens/s", args, res["decode_concurrent_ms"], res, roof)


def bench_cu_masks(args):
    """Where CU-masked streams run: for a set of masks, the compute units the
    workgroups of a recording kernel were started on (accelerator die, shader
    engine, compute unit from the XCC_ID / HW_ID registers), per die."""
    import torch
    from muxserve_amd import ops, workloads
    ncu, nxcd = ops.device_cu_info()
    rows = {}

    def record(name, stream):
        where = workloads.where_workgroups_run(stream)
        per_die = np.bincount([w[0] for w in where], minlength=nxcd).tolist()
        per_se = np.bincount([w[1] for w in where], minlength=4).tolist()
        rows[name] = {"compute_units": len(where), "per_die": per_die, "per_shader_engine": per_se,
                      "first": [list(w) for w in where[:6]]}
        return set(where)

    sets = {}
    # The two narrow ranges (mask bits 0-9 and 10-32) show how the driver deals consecutive
    # mask bits: over the dies first, the shader engines next.
    for name, kw in (("percent 0-4", dict(lo_percent=0, hi_percent=4)), ("percent 4-13", dict(lo_percent=4, hi_percent=13)),
                     ("percent 0-40", dict(lo_percent=0, hi_percent=40)), ("percent 40-100", dict(lo_percent=40, hi_percent=100)),
                     ("parts {0}", dict(parts=[0])), ("parts {9}", dict(parts=[9])), ("parts {0,3,7}", dict(parts=[0, 3, 7])),
                     ("parts {1,2,9}", dict(parts=[1, 2, 9])), ("parts {4,5,6,8}", dict(parts=[4, 5, 6, 8]))):
        st = ops.CUMaskedStream(**kw)
        sets[name] = record(name, st)
        st.close()
    sets["no mask"] = record("no mask", None)
    names = list(sets)
    overlaps = {f"{a} & {b}": len(sets[a] & sets[b]) for i, a in enumerate(names) for b in names[i + 1:]
                if a != "no mask" and b != "no mask"}
    cfg = {"workload": "cu_masks", "num_cus": ncu, "num_dies": nxcd, "masks": rows, "shared_compute_units": overlaps}
    return _line("compute units reached through CU-masked streams", float(ncu), "compute units", args, 0.0, cfg,
                 {"bound": "hbm", "achieved": None, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": None, "traffic": None,
                  "kernel": "probe_where_kernel (records XCC_ID / HW_ID per workgroup)"}, dtype="u32")


def bench_mfma_ceiling(args):
    """What the matrix cores sustain on this box (v_mfma_f32_32x32x16_f16 from
    register operands, nothing else in the loop) for one, two and four
    independent accumulation chains per wave, with vector-ALU work in the same
    wave and in other waves of the SIMD, and the shader clock each case ran at:
    the ceiling the causal prefill kernel is read against (probe_mfma_kernel in
    libmuxprobe.so)."""
    import torch
    from muxserve_amd import _lib, ops
    lib = _lib.probe()
    ncu, _ = ops.device_cu_info()
    iters = 40000
    sink = torch.zeros(1, dtype=torch.float32, device="cuda:0")
    rows = []
    # (label, chains, valu per iteration, waves per workgroup, mfma waves, workgroups per CU)
    cases = [("1 chain, 1 wave per SIMD", 1, 0, 4, 4, 1), ("2 chains, 1 wave per SIMD", 2, 0, 4, 4, 1),
             ("4 chains, 1 wave per SIMD", 4, 0, 4, 4, 1), ("1 chain, 2 waves per SIMD", 1, 0, 8, 8, 1),
             ("2 chains, 2 waves per SIMD", 2, 0, 8, 8, 1), ("4 chains, 2 waves per SIMD", 4, 0, 8, 8, 1),
             ("4 chains + 8 v_fma_f32 per iteration in the same wave", 4, 8, 4, 4, 1),
             ("4 chains + 32 v_fma_f32 per iteration in the same wave", 4, 32, 4, 4, 1),
             ("4 chains in one wave, 32 v_fma_f32 per iteration in the SIMD's other wave", 4, 0, 8, 4, 1),
             ("no MFMA: 32 v_fma_f32 per iteration, 1 wave per SIMD", 4, 0, 4, 0, 1)]
    for label, chains, valu, waves, mfma_waves, per_cu in cases:
        n_wg = ncu * per_cu
        ticks = torch.zeros(n_wg, 2, dtype=torch.int32, device="cuda:0")

        def launch(_i):
            rc = lib.mux_probe_mfma(chains, valu, iters, n_wg, waves, mfma_waves, ticks.data_ptr(), sink.data_ptr(),
                                    torch.cuda.current_stream().cuda_stream)
            if rc != 0:
                raise RuntimeError(f"mux_probe_mfma returned {rc}")
        ms = _time(launch, 10, 3)
        t = ticks.cpu().numpy().astype(np.int64) & 0xffffffff
        clock_ghz = float(np.median(t[:, 0] / np.maximum(t[:, 1], 1)) * 0.1)
        flops = float(n_wg) * mfma_waves * iters * chains * 32768.0
        rows.append({"case": label, "ms": ms, "tflops": flops / (ms * 1e-3) / 1e12, "shader_clock_ghz": clock_ghz})
    best = max(r["tflops"] for r in rows)
    cfg = {"workload": "mfma_ceiling", "instruction": "v_mfma_f32_32x32x16_f16", "iterations": iters, "cases": rows}
    roof = {"bound": "mfma", "achieved": best, "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": best / MFMA_PEAK_TFLOPS,
            "traffic": None, "kernel": "probe_mfma_kernel (register operands only)"}
    return _line("matrix-core rate sustained by independent MFMA chains", best, "TFLOP/s", args, rows[2]["ms"], cfg, roof)


def bench_decode_timeline(args):
    """Per-phase timeline of one launch of the headline kernel, from the tracing
    build of the library (libmuxattn_trace.so, `python -m muxserve_amd.build
    trace`): wave 0 of every workgroup stamps the 100 MHz clock at the ends of
    its phases.  Prints the phase statistics and the launch in 2 us bins."""
    import ctypes
    import torch
    from muxserve_amd import _lib, ops, workloads
    from muxserve_amd.build import TRACE_LIB
    from muxserve_amd.pool import allocate_gpu_cache, num_gpu_blocks
    if os.path.abspath(_lib.ATTN_LIB_PATH) != os.path.abspath(TRACE_LIB):
        raise SystemExit("decode_timeline needs the tracing build: python -m muxserve_amd.build trace, then run with "
                         f"MUXSERVE_ATTN_LIB={TRACE_LIB}")
    lib = _lib.attn()
    lib.mux_decode_trace_set.restype = ctypes.c_int32
    lib.mux_decode_trace_set.argtypes = [ctypes.c_void_p, ctypes.c_int64]
    dev, bs = "cuda:0", 16
    N = num_gpu_blocks(args.pool_util, torch.cuda.get_device_properties(0).total_memory, bs)
    k_pool, v_pool = allocate_gpu_cache(N, bs, dev)
    sets = []
    for i in range(3):
        models, need = workloads.config2(seed=args.seed + 1 + i, num_pool_blocks=N)
        for j, m in enumerate(models):
            m.to_device(dev, torch.float16, seed=j)
        calls = [ops.DecodeCall(m.out, m.q, m.d_block_tables, m.d_context_lens, m.max_context_len, m.scale,
                                total_context_len=int(m.context_lens.sum()),
                                context_lens_host=None if args.no_host_lens else
                                torch.from_numpy(np.ascontiguousarray(m.context_lens, dtype=np.int32)))
                 for m in models]
        sets.append((models, calls))
    rows = 20000
    table = torch.zeros((rows, 8), dtype=torch.int64, device=dev)
    for i in range(12):
        ops.multi_decode(sets[i % 3][1], k_pool, v_pool)
    torch.cuda.synchronize()
    ops.multi_decode(sets[1][1], k_pool, v_pool)            # a launch right before, as in the benchmark loop
    assert lib.mux_decode_trace_set(table.data_ptr(), rows) == 0
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    ops.multi_decode(sets[0][1], k_pool, v_pool)
    e1.record()
    torch.cuda.synchronize()
    lib.mux_decode_trace_set(None, 0)
    t = table.cpu().numpy()
    t = t[t[:, 6] > 0]
    t0 = t[:, 0].min()
    us = lambda x: (x - t0) / 100.0                                                    # noqa: E731
    a, b, c, d, e, f, g = (us(t[:, i]) for i in range(7))
    ntok, split = t[:, 7] & 0xffff, (t[:, 7] >> 16) & 1
    stats = {}
    for name, x, y in (("entry_to_unit_known", a, b), ("unit_known_to_ids_and_q", b, c), ("ids_and_q_to_kv_issued", c, d),
                       ("kv_issued_to_consumed", d, e), ("consumed_to_barrier", e, f), ("barrier_to_done", f, g),
                       ("life", a, g)):
        dd = y - x
        stats[name] = {"mean": float(dd.mean()), "p50": float(np.median(dd)), "p90": float(np.percentile(dd, 90))}
    bins = []
    for lo in np.arange(0.0, float(g.max()) + 2.0, 2.0):
        mid = lo + 1.0
        bins.append({"t_us": float(lo), "started": int(((a >= lo) & (a < lo + 2)).sum()),
                     "alive": int(((a <= mid) & (g > mid)).sum()), "kv_in_flight": int(((c <= mid) & (e > mid)).sum()),
                     "MB_consumed": float(ntok[(e >= lo) & (e < lo + 2)].sum() * 512 / 1e6)})
    first = slice(0, 768)
    cfg = {"workload": "decode_timeline", "kernel_ms_with_stamps": e0.elapsed_time(e1), "span_us": float(g.max()),
           "workgroups": int(len(t)), "MB": float(ntok.sum() * 512 / 1e6), "phases_us": stats,
           "split_units": {"n": int(split.sum()), "barrier_to_done_mean_us": float((g - f)[split == 1].mean())},
           "single_units": {"n": int((split == 0).sum()), "barrier_to_done_mean_us": float((g - f)[split == 0].mean())},
           "first_768_workgroups_mean_us": {"entry": float(a[first].mean()), "unit_known": float(b[first].mean()),
                                            "ids_and_q": float(c[first].mean()), "kv_issued": float(d[first].mean()),
                                            "consumed": float(e[first].mean())},
           "bins_2us": bins}
    return _line("decode kernel per-phase timeline (tracing build)", float(g.max()), "us", args, float(g.max()) * 1e-3, cfg,
                 {"bound": "hbm", "achieved": None, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": None, "traffic": None,
                  "kernel": "paged_decode_kernel<F16,16,1,4> with phase stamps"}, higher=False)


def bench_prefill_timeline(args):
    """Workgroup timeline of one launch of the prefill kernel, from the tracing
    build of the library (libmuxattn_trace.so): thread 0 of every workgroup
    stamps the 100 MHz clock at its entry, when the prompt's offsets are known,
    when its first key tile has landed, after its last key tile and after
    issuing its output stores.  Default: the three
    models' 16 prompts each in one launch (--prompt-cap N cuts them at N
    tokens); --long-prompts: 16 x 2048 tokens, 32 heads."""
    import ctypes
    import torch
    from muxserve_amd import _lib, ops, workloads
    from muxserve_amd.build import TRACE_LIB
    from muxserve_amd.pool import HEAD_SIZE as D
    if os.path.abspath(_lib.ATTN_LIB_PATH) != os.path.abspath(TRACE_LIB):
        raise SystemExit("prefill_timeline needs the tracing build: python -m muxserve_amd.build trace, then run with "
                         f"MUXSERVE_ATTN_LIB={TRACE_LIB}")
    lib = _lib.attn()
    lib.mux_prefill_trace_set.restype = ctypes.c_int32
    lib.mux_prefill_trace_set.argtypes = [ctypes.c_void_p, ctypes.c_int64]
    dev = "cuda:0"
    if args.long_prompts:
        models = [workloads.PrefillModel("7b", 32, 32, np.full(16, 2048, dtype=np.int64))]
    else:
        models = workloads.config3(seed=args.seed)
        if args.prompt_cap > 0:
            for m in models:
                m.prompt_lens = np.minimum(m.prompt_lens, args.prompt_cap)
    g = torch.Generator().manual_seed(args.seed)
    calls, flops = [], 0.0
    for m in models:
        T, Hq, Hkv = m.num_tokens, m.num_q_heads, m.num_kv_heads
        pad = (T + 7) // 8 * 8
        qkv = torch.randn((pad, (Hq + 2 * Hkv) * D), generator=g).half().to(dev)
        q, k, v = qkv.split([Hq * D, Hkv * D, Hkv * D], dim=-1)
        out = torch.empty((pad, Hq * D), dtype=torch.float16, device=dev)
        cu = torch.from_numpy(m.cu_seqlens()).to(dev)
        calls.append(ops.PrefillCall(out, q, k, v, cu, [int(x) for x in m.prompt_lens], m.scale, Hkv))
        flops += workloads.prefill_flops(m.prompt_lens, Hq)
    rows = 16384
    table = torch.zeros((rows, 8), dtype=torch.int64, device=dev)
    # What the stamps cost: the launches with the table switched off and on, after the warm-up.
    ms_off = _time(lambda _: ops.multi_prefill_causal(calls), 30, max(args.warmup, 150))
    assert lib.mux_prefill_trace_set(table.data_ptr(), rows) == 0
    ms_on = _time(lambda _: ops.multi_prefill_causal(calls), 30, 5)
    # Every launch stamps the same rows, so after a run of back-to-back launches the table holds
    # the last one's - a launch in the middle of a busy stream, as in the benchmark loop.
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    # (the first tens of launches of a process run up to a fifth slower than the later ones)
    for _ in range(20):
        ops.multi_prefill_causal(calls)
    e0.record()
    ops.multi_prefill_causal(calls)
    e1.record()
    torch.cuda.synchronize()
    lib.mux_prefill_trace_set(None, 0)
    t = table.cpu().numpy()
    t = t[t[:, 0] > 0]
    base = t[:, 0].min()
    us = lambda x: (x - base) / 100.0                                                   # noqa: E731
    a, known, b, c, d = (us(t[:, i]) for i in range(5))
    nt, plen, q0 = t[:, 5], t[:, 6], t[:, 7]
    span, life = float(d.max()), d - a
    slots = 3 * torch.cuda.get_device_properties(0).multi_processor_count
    # 32 x 32 score blocks the waves of a workgroup really compute (a wave skips the tiles in
    # its rows' future and rows past the prompt's end), against the causal triangle's share
    rows_left = np.clip(plen - q0, 0, 128)
    waves = (rows_left + 31) // 32
    blocks_done = sum(int(((q0 // 32 + w + 1) * (waves > w)).sum()) for w in range(4))
    blocks_ideal = float(sum(((q0[i] + np.arange(rows_left[i]) + 1).sum()) for i in range(len(t)))) / 1024.0
    by_tiles = []
    for lo, hi in ((1, 2), (2, 4), (4, 8), (8, 16), (16, 32), (32, 65)):
        m = (nt >= lo) & (nt < hi)
        if m.any():
            by_tiles.append({"key_tiles": f"{lo}..{hi - 1}", "workgroups": int(m.sum()), "life_us": float(life[m].mean()),
                             "prologue_us": float((b - a)[m].mean()),
                             "us_per_key_tile": float((c - b)[m].sum() / nt[m].sum()),
                             "epilogue_us": float((d - c)[m].mean())})
    bins, step = [], max(2.0, round(span / 24.0))
    for lo in np.arange(0.0, span + step, step):
        mid = lo + step / 2
        bins.append({"t_us": float(lo), "resident": int(((a <= mid) & (d > mid)).sum()),
                     "in_tile_loop": int(((b <= mid) & (c > mid)).sum())})
    cfg = {"workload": "prefill_timeline", "prompts": "16 x 2048, 32 heads" if args.long_prompts else
           f"three models x 16 prompts, cap {args.prompt_cap or None}", "flops": flops,
           "kernel_ms_with_stamps": e0.elapsed_time(e1), "ms_per_launch_table_off": ms_off,
           "ms_per_launch_table_on": ms_on, "span_us": span, "workgroups_with_work": int(len(t)),
           "workgroup_slots": int(slots), "slot_time_filled": float(life.sum() / (span * slots)),
           "share_of_workgroup_life": {"prologue": float((b - a).sum() / life.sum()),
                                       "tile_loop": float((c - b).sum() / life.sum()),
                                       "epilogue": float((d - c).sum() / life.sum())},
           "mean_us": {"prologue": float((b - a).mean()), "of_it_until_the_prompt_is_known": float((known - a).mean()),
                       "per_key_tile": float((c - b).sum() / nt.sum()),
                       "epilogue": float((d - c).mean()), "life": float(life.mean())},
           "key_tiles_per_workgroup": float(nt.mean()),
           "score_blocks_32x32": {"computed": int(blocks_done), "causal_triangle": blocks_ideal,
                                  "useful_fraction": blocks_ideal / blocks_done},
           "last_start_us": float(a.max()), "by_key_tiles": by_tiles, "bins": bins}
    return _line("prefill kernel workgroup timeline (tracing build)", span, "us", args, span * 1e-3, cfg,
                 {"bound": "mfma", "achieved": None, "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": None,
                  "traffic": None, "kernel": "prefill_causal_kernel<F16> with workgroup stamps"}, higher=False)


def bench_gqa_timeline(args):
    """Residency of the workgroups of one launch of the grouped-query decode
    kernel on the long-context workload, from the tracing build of the library
    (entry and end stamps of every workgroup, 100 MHz clock)."""
    import ctypes
    import torch
    from muxserve_amd import _lib, ops, workloads
    from muxserve_amd.build import TRACE_LIB
    from muxserve_amd.pool import allocate_gpu_cache
    if os.path.abspath(_lib.ATTN_LIB_PATH) != os.path.abspath(TRACE_LIB):
        raise SystemExit("gqa_timeline needs the tracing build: python -m muxserve_amd.build trace, then run with "
                         f"MUXSERVE_ATTN_LIB={TRACE_LIB}")
    lib = _lib.attn()
    lib.mux_decode_trace_set.restype = ctypes.c_int32
    lib.mux_decode_trace_set.argtypes = [ctypes.c_void_p, ctypes.c_int64]
    dev, bs = "cuda:0", 16
    N = int(200e9) // 8192 // 128 * 128
    k_pool, v_pool = allocate_gpu_cache(N, bs, dev, dtype=torch.bfloat16)
    sets = [workloads.config5(seed=args.seed + i, num_pool_blocks=N)[0][0].to_device(dev, torch.bfloat16, seed=i)
            for i in range(3)]
    launches = [ops.DecodeLaunch([ops.DecodeCall(m.out, m.q, m.d_block_tables, m.d_context_lens, m.max_context_len, m.scale,
                                                 total_context_len=int(m.context_lens.sum()),
                                                 context_lens_host=None if args.no_host_lens else torch.from_numpy(
                                                     np.ascontiguousarray(m.context_lens, dtype=np.int32)))],
                                 k_pool, v_pool, partition_size=args.partition) for m in sets]
    rows = 16384
    table = torch.zeros((rows, 8), dtype=torch.int64, device=dev)
    for i in range(30):
        launches[i % 3]()
    torch.cuda.synchronize()
    slots = 3 * torch.cuda.get_device_properties(0).multi_processor_count       # 142 registers: three workgroups per CU
    per_batch = []
    for which in range(3):
        table.zero_()
        launches[(which + 1) % 3]()                      # a launch right before, as in the benchmark loop
        assert lib.mux_decode_trace_set(table.data_ptr(), rows) == 0
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        launches[which]()
        e1.record()
        torch.cuda.synchronize()
        lib.mux_decode_trace_set(None, 0)
        t = table.cpu().numpy()
        t = t[(t[:, 6] > 0) & ((t[:, 7] & 0xffff) > 0)]      # workgroups that had a unit
        base = t[:, 0].min()
        a, g = (t[:, 0] - base) / 100.0, (t[:, 6] - base) / 100.0
        ntok = t[:, 7] & 0xffff
        span, life = float(g.max()), g - a
        full = ntok >= 0.95 * ntok.max()
        per_batch.append({"kernel_us_with_stamps": e0.elapsed_time(e1) * 1e3, "span_us": span, "workgroups": int(len(t)),
                          "life_us_mean": float(life.mean()), "life_us_of_the_full_units": float(life[full].mean()),
                          "tokens_of_a_full_unit": int(ntok.max()),
                          "slot_time_filled": float(life.sum() / (span * slots)), "last_start_us": float(a.max()),
                          "ends_us_p50_p90_max": [float(np.percentile(g, 50)), float(np.percentile(g, 90)), span],
                          "resident_every_10us": [int(((a <= lo + 5) & (g > lo + 5)).sum())
                                                  for lo in np.arange(0.0, span + 10.0, 10.0)]})
    span = float(np.mean([b["span_us"] for b in per_batch]))
    cfg = {"workload": "gqa_timeline", "partition": args.partition, "workgroup_slots": int(slots), "batches": per_batch}
    return _line("grouped-query decode kernel workgroup residency (tracing build)", span, "us", args, span * 1e-3, cfg,
                 {"bound": "hbm", "achieved": None, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": None, "traffic": None,
                  "kernel": "paged_decode_gqa_kernel<BF16,16,8,4> with entry and end stamps"}, dtype="bf16", higher=False)


def bench_gqa_long(args):
    """Config 5: 64 query heads over 8 kv heads, bf16, batch 64, ctx U[2048, 8192]."""
    import torch
    from muxserve_amd import ops, workloads
    from muxserve_amd.pool import allocate_gpu_cache
    dev, bs = "cuda:0", 16
    N = int(200e9) // 8192 // 128 * 128
    k_pool, v_pool = allocate_gpu_cache(N, bs, dev, dtype=torch.bfloat16)
    sets = []
    for i in range(3):
        m = workloads.config5(seed=args.seed + i, num_pool_blocks=N)[0][0].to_device(dev, torch.bfloat16, seed=i)
        sets.append(m)

    launches = [ops.DecodeLaunch([ops.DecodeCall(m.out, m.q, m.d_block_tables, m.d_context_lens, m.max_context_len, m.scale,
                                                 total_context_len=int(m.context_lens.sum()),
                                                 context_lens_host=None if args.no_host_lens else torch.from_numpy(
                                                     np.ascontiguousarray(m.context_lens, dtype=np.int32)))],
                                 k_pool, v_pool, args.partition) for m in sets]

    def step(i):
        launches[i % len(launches)]()

    ms = _time(step, args.steps, args.warmup)
    nbytes = float(np.mean([workloads.decode_bytes(m.context_lens, 64, 8, bs) for m in sets]))
    gbs = nbytes / (ms * 1e-3) / 1e9
    # The yardstick: the same blocks read by the bare gather-read probe.
    used = [torch.from_numpy(m.used_blocks(bs).astype(np.int32)).to(dev) for m in sets]
    sink = torch.zeros((1,), dtype=torch.int32, device=dev)
    probe_ms = _time(lambda i: workloads.probe_gather_read(k_pool, v_pool, used[i % len(used)], sink), args.steps, args.warmup)
    probe_bytes = float(np.mean([u.numel() * 8192 for u in used]))
    cfg = {"workload": "gqa_long", "shape": "Hq64/Hkv8, B=64, ctx U[2048,8192], bf16", "pool_gb": round(N * 8192 / 1e9, 1),
           "bytes_per_step": int(nbytes), "partition": args.partition,
           "units_enumerated_on_the_host": [l.host_pairs for l in launches]}
    roof = {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
            "traffic": nbytes * GQA_LONG_TRAFFIC_RATIO,
            "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, "
                              "profiles/paged_decode_gqa_long_kernel_trace_and_traffic.txt",
            "kernel": "paged_decode_gqa_kernel<BF16,16,8,4>",
            "bare_gather_read_of_the_same_blocks": {
                "ms": probe_ms, "bytes": int(probe_bytes), "GB/s": probe_bytes / (probe_ms * 1e-3) / 1e9,
                "kernel": "probe_gather_read_kernel (whole 4 KiB blocks, no arithmetic)"}}
    return _line("long-context GQA decode attn tokens/s", 64 / (ms * 1e-3), "tokens/s", args, ms, cfg, roof, dtype="bf16")


def bench_model_ops(args):
    """The per-step operators around the attention layer: greedy sampling
    (lm_head + argmax in one pass) for the three models of the mix, RMSNorm and
    SiluAndMul on a prefill-sized step of the 30B shape."""
    import torch
    import torch.nn.functional as F
    from muxserve_amd import ops
    dev = "cuda:0"
    g = torch.Generator().manual_seed(args.seed)
    V = 32000
    shapes = [("7b", 4096, 32), ("13b", 5120, 16), ("30b", 6656, 8)]
    heads = []
    sbytes = 0
    for name, hidden, R in shapes:
        emb = (torch.randn((V, hidden), generator=g) * 0.05).half().to(dev)
        hid = torch.randn(((R + 7) // 8 * 8, hidden), generator=g).half().to(dev)
        out = torch.empty((R,), dtype=torch.int64, device=dev)
        heads.append((emb, hid, R, out))
        sbytes += V * hidden * 2 + R * hidden * 2 + R * 8

    def sample(_):
        for emb, hid, R, out in heads:
            ops.greedy_sample(emb, hid, V, R, out=out)

    def sample_torch(_):
        for emb, hid, R, out in heads:
            torch.argmax(torch.matmul(hid[:R], emb.t())[:, :V], dim=-1, out=out)

    ms_s = _time(sample, args.steps, args.warmup)
    ms_st = _time(sample_torch, args.steps, args.warmup)

    T, hidden, d = 4096, 6656, 17920
    xs = [torch.randn((T, hidden), generator=g).half().to(dev) for _ in range(4)]
    outs = [torch.empty_like(x) for x in xs]
    w = (1 + 0.1 * torch.randn((hidden,), generator=g)).half().to(dev)
    ms_n = _time(lambda i: ops.rms_norm(xs[i % 4], w, 1e-6, out=outs[i % 4]), args.steps, args.warmup)
    ms_nt = _time(lambda i: F.rms_norm(xs[i % 4], (hidden,), w, 1e-6), args.steps, args.warmup)
    nbytes = 2 * T * hidden * 2 + hidden * 2
    del xs, outs
    gu = [torch.randn((T, 2 * d), generator=g).half().to(dev) for _ in range(2)]
    go = [torch.empty((T, d), dtype=torch.float16, device=dev) for _ in range(2)]
    ms_a = _time(lambda i: ops.silu_and_mul(gu[i % 2], out=go[i % 2]), args.steps, args.warmup)
    ms_at = _time(lambda i: torch.mul(F.silu(gu[i % 2][:, :d]), gu[i % 2][:, d:], out=go[i % 2]), args.steps,
                  args.warmup)
    abytes = 3 * T * d * 2

    gbs = sbytes / (ms_s * 1e-3) / 1e9
    cfg = {"workload": "model_ops",
           "sampler": "7b(hidden 4096, 32 rows)+13b(5120, 16)+30b(6656, 8), vocabulary 32000, three launches per step",
           "sampler_bytes_per_step": sbytes, "sampler_torch_matmul_argmax_ms": ms_st,
           "rms_norm": {"shape": [T, hidden], "ms": ms_n, "gbs": nbytes / (ms_n * 1e-3) / 1e9,
                        "frac_of_hbm": nbytes / (ms_n * 1e-3) / 1e9 / HBM_PEAK_GBS, "torch_ms": ms_nt},
           "silu_and_mul": {"shape": [T, 2 * d], "ms": ms_a, "gbs": abytes / (ms_a * 1e-3) / 1e9,
                            "frac_of_hbm": abytes / (ms_a * 1e-3) / 1e9 / HBM_PEAK_GBS, "torch_ms": ms_at}}
    roof = {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
            "traffic": None, "kernel": "lm_head_argmax_kernel<F16,NB,KT>"}
    return _line("greedy sampling tokens/s (lm_head + argmax, 3 models)", 56 / (ms_s * 1e-3), "tokens/s", args, ms_s,
                 cfg, roof)


def _host_step(sched, storage, L, H, ids, last_tokens, permuted):
    """One step of the host path with the reference's call sequence
    (llm_runtime.py:277-339): try_batch -> allocate_batch -> get_batch_info ->
    caller-allocated CPU tensors -> get_batch.  Works with the product's classes
    and with the compiled reference's."""
    import torch
    info = np.asarray(sched.try_batch(list(ids), list(last_tokens)), dtype=np.int32)
    req = np.ascontiguousarray(info[:-1])
    if int(info[-1]) > 0:
        block_info = np.asarray(storage.allocate_batch(req, L, H), dtype=np.int32)
    else:
        block_info = np.array([len(ids)], dtype=np.int32)
    bi = list(sched.get_batch_info(req, block_info))
    T, C, max_ctx, max_blk = bi[:4]
    slots = torch.empty((T, L, H), dtype=torch.int64)
    toks = torch.empty(((T + 7) // 8 * 8,), dtype=torch.int32)
    pos = torch.empty_like(toks)
    ctx = torch.empty((C,), dtype=torch.int32)
    if max_ctx > 0 and permuted:
        tables = torch.empty((L, C, H, max_blk), dtype=torch.int32)
        sched.get_batch_permuted(req, block_info, toks, pos, ctx, tables, slots)
    else:
        tables = torch.empty((T, max_blk, L, H) if max_ctx > 0 else (0, max_blk, 0, 0), dtype=torch.int32)
        sched.get_batch(req, block_info, toks, pos, ctx, tables, slots)
        if max_ctx > 0:
            tables = tables.permute(2, 0, 3, 1).contiguous()        # llm_runtime.py:327 (on the device there)
    return tables, slots


def _host_step_compact(sched, storage, L, H, ids, last_tokens, staging):
    """The host part of a step when the device builds the tables: the same
    calls up to get_batch_info, then 8 ints per sequence instead of tables and
    slots, everything packed into one staging buffer."""
    import torch
    info = np.asarray(sched.try_batch(list(ids), list(last_tokens)), dtype=np.int32)
    req = np.ascontiguousarray(info[:-1])
    if int(info[-1]) > 0:
        block_info = np.asarray(storage.allocate_batch(req, L, H), dtype=np.int32)
    else:
        block_info = np.array([len(ids)], dtype=np.int32)
    bi = list(sched.get_batch_info(req, block_info))
    T, C = bi[:2]
    pad = (T + 7) // 8 * 8
    n = max(int(block_info[0]), 0)
    o_ctx, o_desc = 2 * pad, 2 * pad + (C + 3) // 4 * 4
    o_info = o_desc + 8 * n
    sched.get_batch_compact(req, block_info, staging[:pad], staging[pad:o_ctx], staging[o_ctx:o_ctx + C],
                            staging[o_desc:o_info])
    staging[o_info:o_info + block_info.size] = torch.from_numpy(block_info)
    return o_info + block_info.size


def _time_host(make_storage, make_sched, L, H, lens, decode_steps, permuted, compact=False):
    """(prefill step seconds, mean decode step seconds[, ints uploaded per decode step]) for one batch."""
    import torch
    bs = 16
    need = sum((n + decode_steps + bs) // bs + 1 for n in lens) * L * H
    storage, sched = make_storage(need + 1024), make_sched(L, H, 2048, bs)
    rng = np.random.Generator(np.random.PCG64(1))
    ids = list(range(len(lens)))
    for i, n in enumerate(lens):
        sched.add_request(rng.integers(0, 32000, size=int(n)).astype(np.int32), i, decode_steps + 8)
    if compact:
        sched.enable_device_rows(len(lens))
        staging = torch.empty((need + 65536,), dtype=torch.int32)
        t0 = time.perf_counter()
        _host_step_compact(sched, storage, L, H, ids, [], staging)
        t1 = time.perf_counter()
        ints = 0
        for s in range(decode_steps):
            ints += _host_step_compact(sched, storage, L, H, ids, [7 + s] * len(ids), staging)
        t2 = time.perf_counter()
        return t1 - t0, (t2 - t1) / decode_steps, ints / decode_steps
    t0 = time.perf_counter()
    _host_step(sched, storage, L, H, ids, [], permuted)
    t1 = time.perf_counter()
    for s in range(decode_steps):
        _host_step(sched, storage, L, H, ids, [7 + s] * len(ids), permuted)
    t2 = time.perf_counter()
    return t1 - t0, (t2 - t1) / decode_steps


def _time_prepare_inputs(L, H, lens, decode_steps, mode):
    """Full prepare_inputs on the GPU box, wall clock per decode step including
    uploads and kernels (synchronised at the end).  mode: "device" (tables and
    slots built on the device), "lbhm" (host writes [L,B,H,maxBlk]) or
    "reference" (host writes the reference layout, permuted on the device)."""
    import torch
    from muxserve_amd.batch_scheduler import BatchScheduler
    from muxserve_amd.device_tables import DeviceBlockTables
    from muxserve_amd.memory_manager import KVStorage
    from muxserve_amd.prepare import prepare_inputs
    bs = 16
    need = sum((n + decode_steps + bs) // bs + 1 for n in lens) * L * H
    storage, sched = KVStorage(need + 1024), BatchScheduler(L, H, 2048, bs)
    kw = {"device_tables": DeviceBlockTables(sched, len(lens), "cuda:0")} if mode == "device" else \
         {"permuted_tables": mode == "lbhm"}
    rng = np.random.Generator(np.random.PCG64(1))
    ids = list(range(len(lens)))
    for i, n in enumerate(lens):
        sched.add_request(rng.integers(0, 32000, size=int(n)).astype(np.int32), i, decode_steps + 8)
    alloc = lambda r: storage.allocate_batch(r, L, H)   # noqa: E731
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    prepare_inputs(sched, alloc, ids, [], "cuda:0", **kw)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    for s in range(decode_steps):
        prepare_inputs(sched, alloc, ids, [7 + s] * len(ids), "cuda:0", **kw)
    torch.cuda.synchronize()
    t2 = time.perf_counter()
    return t1 - t0, (t2 - t1) / decode_steps


def bench_host_step(args):
    """The host side of a step at real layer counts, single-threaded as in the
    reference: the product's allocator + batch builder, and beside it the
    reference's own C++ compiled under oracle/_ref when that is present."""
    from muxserve_amd.batch_scheduler import BatchScheduler
    from muxserve_amd.memory_manager import KVStorage
    rng = np.random.Generator(np.random.PCG64(args.seed))
    shapes = {"7b (L32,H32), 32 sequences": (32, 32, 32), "13b (L40,H40), 16 sequences": (40, 40, 16),
              "30b (L60,H52), 8 sequences": (60, 52, 8)}
    ref = (None, None)
    if not args.no_cpu_baseline:
        from oracle import build_ref                                  # the checker: CPU baseline only
        if os.path.isdir(os.path.join(ROOT, "oracle", "_ref")):
            ref = build_ref.load()
    steps = 64
    import torch
    have_gpu = torch.cuda.is_available()
    rows, total_dec, total_ref = {}, 0.0, 0.0
    for name, (L, H, B) in shapes.items():
        lens = np.clip(np.rint(rng.lognormal(np.log(300), 0.8, size=B)), 16, 1900).astype(int)
        pre_p, dec_p = _time_host(KVStorage, BatchScheduler, L, H, lens, steps, True)
        pre_l, dec_l = _time_host(KVStorage, BatchScheduler, L, H, lens, steps, False)
        pre_c, dec_c, ints = _time_host(KVStorage, BatchScheduler, L, H, lens, steps, True, compact=True)
        row = {"compact_prefill_step_ms": pre_c * 1e3, "compact_decode_step_us": dec_c * 1e6,
               "compact_upload_bytes_per_decode_step": 4 * ints,
               "host_built_prefill_step_ms": pre_p * 1e3, "host_built_decode_step_us_lbhm": dec_p * 1e6,
               "host_built_decode_step_us_reference_layout_then_permute": dec_l * 1e6,
               "host_built_upload_bytes_per_decode_step":
                   int(B * L * H * (8 + 4 * ((int(lens.max()) + steps) // 16 + 1)))}
        if have_gpu:
            for mode in ("device", "lbhm", "reference"):
                pre_d, dec_d = _time_prepare_inputs(L, H, lens, steps, mode)
                row[f"prepare_inputs_{mode}_prefill_ms"] = pre_d * 1e3
                row[f"prepare_inputs_{mode}_decode_us"] = dec_d * 1e6
        total_dec += dec_c
        if ref[0] is not None:
            pre_r, dec_r = _time_host(ref[0].KVStorage, ref[1].BatchScheduler, L, H, lens, steps, False)
            row["reference_prefill_step_ms"] = pre_r * 1e3
            row["reference_decode_step_us"] = dec_r * 1e6
            total_ref += dec_r
        rows[name] = row
    line = _line("host path (compact step): decode step of the three models, microseconds", total_dec * 1e6, "us", args,
                 total_dec * 1e3, {"workload": "host_step", "decode_steps_timed": steps, "threads": 1, "models": rows},
                 None, dtype="int32", higher=False)
    if ref[0] is not None:
        line["cpu_baseline"] = {"value": total_ref * 1e6, "unit": "us", "cores": 1, "kind": "reference",
                                "sample": f"the same {steps} decode steps through the reference's compiled "
                                          "memory_manager / batch_scheduler, table permuted on the host"}
    return line


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives or sharding); use --gpus 1",
              file=sys.stderr)
        sys.exit(2)
    other = {"prefill3": bench_prefill3, "cache_write": bench_cache_write, "colocated": bench_colocated, "cu_masks": bench_cu_masks, "prefill_long": bench_prefill_long, "decode_timeline": bench_decode_timeline,
             "prefill_timeline": bench_prefill_timeline, "gqa_timeline": bench_gqa_timeline,
             "gqa_long": bench_gqa_long, "model_ops": bench_model_ops, "host_step": bench_host_step,
             "mfma_ceiling": bench_mfma_ceiling}
    if args.workload in other:
        print(json.dumps(other[args.workload](args)))
        return

    import torch
    from muxserve_amd import ops, workloads
    from muxserve_amd.pool import allocate_gpu_cache, num_gpu_blocks

    dev = "cuda:0"
    bs = 16
    total_mem = torch.cuda.get_device_properties(0).total_memory
    N = num_gpu_blocks(args.pool_util, total_mem, bs)
    k_pool, v_pool = allocate_gpu_cache(N, bs, dev)

    # Disjoint ids for all sets from one seeded draw over the whole pool.
    rng = np.random.Generator(np.random.PCG64(args.seed))
    if args.batch_scale < 1 or args.batch_scale > 8:
        raise SystemExit("--batch-scale takes 1..8")
    batches = tuple(b * args.batch_scale for b in (32, 16, 8))
    probe = [workloads.config2(seed=args.seed + 1 + i, num_pool_blocks=N, id_perm=np.arange(1 << 23),
                               batches=batches)[1]
             for i in range(args.sets)]
    ids = rng.choice(N, size=int(sum(probe)), replace=False)
    sets, off = [], 0
    for i in range(args.sets):
        models, need = workloads.config2(seed=args.seed + 1 + i, num_pool_blocks=N, id_perm=ids[off:off + probe[i]],
                                         batches=batches)
        off += need
        used = np.concatenate([m.used_blocks(bs) for m in models])
        workloads.fill_blocks(k_pool, v_pool, used, seed=args.seed + 100 + i)
        for j, m in enumerate(models):
            m.to_device(dev, torch.float16, seed=args.seed + 1000 + 10 * i + j)
        calls = [ops.DecodeCall(m.out, m.q, m.d_block_tables, m.d_context_lens, m.max_context_len, m.scale,
                                total_context_len=0 if args.no_hint else int(m.context_lens.sum()),
                                context_lens_host=None if (args.no_hint or args.no_host_lens)
                                else torch.from_numpy(np.ascontiguousarray(m.context_lens, dtype=np.int32)))
                 for m in models]
        sets.append((models, calls, torch.from_numpy(used.astype(np.int32)).to(dev)))
    torch.cuda.synchronize()

    # Every batch's launch is prepared once (tensor checks, descriptors, workspace): a step is
    # then a single call into the C ABI, as in a serving loop that runs the same step shape
    # layer after layer.
    launches = [[ops.DecodeLaunch([c], k_pool, v_pool, args.partition) for c in calls] if args.unfused
                else [ops.DecodeLaunch(calls, k_pool, v_pool, args.partition)] for _, calls, _ in sets]

    def step(i):
        for launch in launches[i % len(launches)]:
            launch()

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    for i in range(args.steps):
        step(i)
    t_enq = time.perf_counter()
    ev1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    enqueue_us = (t_enq - t0) * 1e6 / args.steps
    ev_ms = ev0.elapsed_time(ev1) / args.steps
    ms = max(wall_ms, ev_ms)

    # Outside the timed region: every batch's launch on its own between two events (a
    # launch with nothing queued behind it: kernel plus the dispatch latency around it).
    singles = []
    for r in range(3):
        for i in range(len(sets)):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            a.record()
            step(i)
            b.record()
            b.synchronize()
            singles.append((i, a.elapsed_time(b) * 1e3))
    single_us = [float(np.median([t for j, t in singles if j == i])) for i in range(len(sets))]

    # The yardstick: the same blocks read by the bare gather-read probe (the decode
    # kernel's loads, no table walk, no arithmetic), same rotation of the sets.
    sink = torch.zeros((1,), dtype=torch.int32, device=dev)
    probe_ms = _time(lambda i: workloads.probe_gather_read(k_pool, v_pool, sets[i % len(sets)][2], sink),
                     args.steps, args.warmup)
    probe_bytes = sum(int(s[2].numel()) * 8192 * v for s, v in
                      zip(sets, [len(range(i, args.steps, len(sets))) for i in range(len(sets))])) / args.steps
    # And what the chip reads at all in a launch of this size: the same probe over as many blocks
    # in one consecutive run of the pool (a different run per batch, far apart).
    runs = [torch.arange(int(s[2].numel()), dtype=torch.int32, device=dev) + int(i * (N // len(sets)))
            for i, s in enumerate(sets)]
    run_ms = _time(lambda i: workloads.probe_gather_read(k_pool, v_pool, runs[i % len(runs)], sink),
                   args.steps, args.warmup)

    tokens = sum(m.batch for m in sets[0][0])
    step_bytes = [sum(workloads.decode_bytes(m.context_lens, m.num_q_heads, m.num_kv_heads, bs) for m in models)
                  for models, _, _ in sets]
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
            "models": f"7b(H32,B{batches[0]})+13b(H40,B{batches[1]})+30b(H52,B{batches[2]}), one layer each, "
                      "one fused launch per step",
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
            "traffic": avg_bytes * MIXED3_TRAFFIC_RATIO if not args.unfused else None,
            "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, profiles/paged_decode_mixed3_hbm_traffic.txt",
            "kernel": "paged_decode_kernel<F16,16,1,4>",
            "event_ms_per_step": ev_ms,
            "wall_ms_per_step": wall_ms,
            "host_enqueue_us_per_step": enqueue_us,
            "units_enumerated_on_the_host": [[l.host_pairs for l in ls] for ls in launches],
            "single_launch_event_us_per_batch": single_us,
            "single_launch_event_us_weighted_mean": float(sum(t * v for t, v in zip(single_us, [len(range(i, args.steps, len(sets))) for i in range(len(sets))])) / args.steps),
            "bare_gather_read_of_the_same_blocks": {
                "ms": probe_ms, "bytes": int(probe_bytes), "GB/s": probe_bytes / (probe_ms * 1e-3) / 1e9,
                "kernel": "probe_gather_read_kernel (whole 4 KiB blocks, no arithmetic)"},
            "bare_read_of_as_many_consecutive_blocks": {
                "ms": run_ms, "bytes": int(probe_bytes), "GB/s": probe_bytes / (run_ms * 1e-3) / 1e9},
        },
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(sets[0][0], k_pool, v_pool, bs)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
