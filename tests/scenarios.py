"""Scripted serving scenarios for the host path (allocator + batch builder).

A scenario is a list of operations replayed against any implementation that
exposes the reference's method names: the compiled reference (oracle/_ref),
the CPU restatement (oracle/host_oracle.py) or the product
(muxserve_amd.memory_manager / batch_scheduler).  run_scenario() returns a
JSON-serialisable trace of everything those calls return, with memory the
reference leaves uninitialised masked out, so traces compare with ``==``.
"""
import hashlib
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from oracle.host_oracle import prepare_inputs  # noqa: E402  (test infrastructure)

FULL_ARRAY_LIMIT = 256   # larger arrays are recorded as shape + sha256


def _rec(a):
    a = np.ascontiguousarray(np.asarray(a))
    if a.size <= FULL_ARRAY_LIMIT:
        return {"shape": list(a.shape), "data": [int(x) for x in a.reshape(-1)]}
    return {"shape": list(a.shape), "sha256": hashlib.sha256(a.tobytes()).hexdigest()}


def _mask_table(block_tables_lbhm, context_lens, block_size):
    """Entries past ceil(ctx/bs) are uninitialised in the reference: set to -1."""
    bt = np.array(block_tables_lbhm, copy=True)
    if bt.size == 0:
        return bt
    for b, ctx in enumerate(np.asarray(context_lens).reshape(-1)):
        valid = (int(ctx) + block_size - 1) // block_size
        bt[:, b, :, valid:] = -1
    return bt


def run_scenario(make_storage, make_sched, sc):
    """sc = {"L","H","max_seq_len","block_size","num_blocks","ops":[...]}.

    ops:
      ["add", req_id, prompt_len, max_tokens]   prompt tokens are derived from req_id
      ["alloc", n]                              KVStorage.allocate(n)
      ["prefill", [ids]] / ["decode", [ids]]    one prepare_inputs round
      ["free", [ids]]                           free_batch + release_requests
    """
    L, H, bs = sc["L"], sc["H"], sc["block_size"]
    storage = make_storage(sc["num_blocks"])
    sched = make_sched(L, H, sc["max_seq_len"], bs)
    trace = []
    step = 0
    dead = set()     # ids the allocator preempted (the builder forgets them)
    for op in sc["ops"]:
        kind = op[0]
        if kind in ("prefill", "decode", "free"):
            op = [kind, [i for i in op[1] if i not in dead]]
            if not op[1]:
                continue
        if kind == "add":
            _, rid, plen, max_tokens = op
            dead.discard(rid)
            prompt = ((np.arange(plen, dtype=np.int64) * 7919 + rid * 104729) % 24000).astype(np.int32)
            sched.add_request(prompt, rid, max_tokens)
            trace.append({"op": "add", "id": rid})
        elif kind == "alloc":
            trace.append({"op": "alloc", "ids": _rec(storage.allocate(op[1]))})
        elif kind in ("prefill", "decode"):
            ids = list(op[1])
            step += 1
            last = [] if kind == "prefill" else [int((rid * 31 + step * 17) % 24000) for rid in ids]
            r = prepare_inputs(sched, storage, L, H, ids, last, fill=-7)
            ctx = r["context_lens"].numpy()
            rec = {
                "op": kind,
                "batch_block_request": _rec(r["batch_block_request"]),
                "block_info": _rec(r["block_info"]),
                "input_tensor": _rec(r["input_tensor"].numpy()),
                "input_positions": _rec(r["input_positions"].numpy()),
                "slot_mapping": _rec(r["slot_mapping"].numpy()),
                "context_lens": _rec(ctx),
                "block_tables": _rec(_mask_table(r["block_tables"].numpy(), ctx, bs)),
                "prompt_lens": [int(x) for x in r["prompt_lens"]],
                "max_context_len": int(r["max_context_len"]),
                "batch_reqs": [[int(a), int(b)] for a, b in r["batch_reqs"]],
                "preempted": [int(x) for x in r["preempted_reqs"]],
                "prompt_info": [int(x) for x in sched.get_prompt_info()],
                "new_blocks_allocated": int(storage.get_new_blocks_allocated()),
            }
            dead.update(rec["preempted"])
            trace.append(rec)
        elif kind == "free":
            ids = list(op[1])
            n = storage.free_batch(ids)
            sched.release_requests(ids)
            trace.append({"op": "free", "freed": int(n)})
        else:
            raise ValueError(kind)
    return trace


# ---------------------------------------------------------------------------
# Scenario library
# ---------------------------------------------------------------------------

def _decode_steps(ids, n):
    return [["decode", list(ids)] for _ in range(n)]


def scripted_scenarios():
    sc = {}
    sc["tiny_l1h1"] = {
        "L": 1, "H": 1, "max_seq_len": 128, "block_size": 16, "num_blocks": 64,
        "ops": [["add", 0, 5, 40], ["add", 1, 16, 40], ["prefill", [0, 1]],
                *_decode_steps([0, 1], 20), ["free", [0]], ["add", 2, 31, 8],
                ["prefill", [2]], *_decode_steps([1, 2], 6), ["free", [1, 2]]],
    }
    sc["l2h3_boundaries"] = {
        "L": 2, "H": 3, "max_seq_len": 256, "block_size": 16, "num_blocks": 1024,
        "ops": [*[["add", i, p, 64] for i, p in enumerate([1, 15, 16, 17, 33])],
                ["prefill", [0, 1, 2]], ["prefill", [3, 4]],
                *_decode_steps([0, 1, 2, 3, 4], 18), ["free", [1, 3]],
                ["add", 5, 48, 10], ["prefill", [5]],
                *_decode_steps([4, 0, 5, 2], 17), ["alloc", 5], ["free", [0, 2, 4, 5]]],
    }
    sc["bs8"] = {
        "L": 3, "H": 2, "max_seq_len": 64, "block_size": 8, "num_blocks": 512,
        "ops": [["add", 10, 7, 30], ["add", 11, 8, 30], ["add", 12, 9, 30],
                ["prefill", [10, 11, 12]], *_decode_steps([12, 10, 11], 20), ["free", [10, 11, 12]]],
    }
    sc["bs32"] = {
        "L": 2, "H": 2, "max_seq_len": 256, "block_size": 32, "num_blocks": 512,
        "ops": [["add", 1, 31, 50], ["add", 2, 32, 50], ["add", 3, 65, 50],
                ["prefill", [1, 2, 3]], *_decode_steps([1, 2, 3], 35), ["free", [2]],
                *_decode_steps([3, 1], 3)],
    }
    # Pool far too small for the third prompt: partial prefill preemption, then
    # decode preemption when the survivors outgrow the pool.
    sc["preempt_prefill_then_decode"] = {
        "L": 2, "H": 2, "max_seq_len": 128, "block_size": 16, "num_blocks": 24,
        "ops": [["add", 0, 16, 99], ["add", 1, 30, 99], ["add", 2, 40, 99],
                ["prefill", [0, 1, 2]],          # needs 4+8+12 = 24 -> fits exactly
                *_decode_steps([0, 1, 2], 3),    # seq 0 opens a block -> tail preempted
                ["add", 3, 3, 5], ["prefill", [3]],
                *_decode_steps([0, 1], 20)],
    }
    sc["preempt_everything"] = {
        "L": 1, "H": 4, "max_seq_len": 64, "block_size": 16, "num_blocks": 8,
        "ops": [["add", 0, 40, 9], ["prefill", [0]],     # needs 12 > 8 -> preemptIdx 0
                ["add", 1, 20, 9], ["add", 2, 20, 9], ["prefill", [1, 2]],   # 8 + 8 -> only first fits
                *_decode_steps([1], 14)],               # crosses into a third block -> preemptIdx 0
    }
    sc["reuse_after_free_order"] = {
        "L": 1, "H": 2, "max_seq_len": 128, "block_size": 16, "num_blocks": 40,
        "ops": [["add", 0, 20, 9], ["add", 1, 20, 9], ["add", 2, 20, 9], ["prefill", [0, 1, 2]],
                ["free", [1]], ["free", [0]], ["add", 3, 50, 9], ["prefill", [3]],
                ["alloc", 3], *_decode_steps([2, 3], 15)],
    }
    sc["llama7b_shape"] = {
        "L": 32, "H": 32, "max_seq_len": 2048, "block_size": 16, "num_blocks": 32 * 32 * 64,
        "ops": [["add", 0, 50, 9], ["add", 1, 17, 9], ["prefill", [0, 1]],
                *_decode_steps([0, 1], 16), ["free", [0, 1]]],
    }
    sc["llama30b_shape"] = {
        "L": 60, "H": 52, "max_seq_len": 2048, "block_size": 16, "num_blocks": 60 * 52 * 40,
        "ops": [["add", 7, 100, 9], ["add", 9, 31, 9], ["prefill", [7, 9]],
                *_decode_steps([9, 7], 3), ["free", [7]], *_decode_steps([9], 2)],
    }
    sc["gqa70b_shape_one_layer"] = {
        "L": 1, "H": 8, "max_seq_len": 8192, "block_size": 16, "num_blocks": 8 * 2048,
        "ops": [["add", 0, 2049, 9], ["add", 1, 4000, 9], ["prefill", [0, 1]],
                *_decode_steps([0, 1], 17)],
    }
    return sc


def random_scenario(seed):
    """A valid random op sequence: decode only live, prefilled requests; drop
    requests the allocator preempts (the serving loop re-queues them)."""
    rng = np.random.default_rng(seed)
    L = int(rng.integers(1, 4))
    H = int(rng.integers(1, 5))
    bs = int(rng.choice([8, 16, 32]))
    per = L * H
    num_blocks = int(rng.integers(6, 60)) * per
    max_seq = 160
    ops = []
    # The driver must know which requests survive; it mirrors the allocator's
    # bookkeeping with the restatement (cheap) to keep the script valid.
    from oracle.host_oracle import BatchScheduler as OS, KVStorage as OK
    st, sd = OK(num_blocks), OS(L, H, max_seq, bs)
    live, waiting, next_id, step = [], [], 0, 0

    def do(kind, ids):
        nonlocal step, live
        step += 1
        last = [] if kind == "prefill" else [int((rid * 31 + step * 17) % 24000) for rid in ids]
        r = prepare_inputs(sd, st, L, H, ids, last)
        ops.append([kind, list(ids)])
        gone = set(r["preempted_reqs"])
        live = [x for x in live if x not in gone]
        if kind == "prefill":
            live.extend(x for x in ids if x not in gone)

    for _ in range(int(rng.integers(15, 40))):
        roll = rng.random()
        if roll < 0.3 or (not live and not waiting):
            plen = int(rng.integers(1, 70))
            ops.append(["add", next_id, plen, 50])
            prompt = ((np.arange(plen, dtype=np.int64) * 7919 + next_id * 104729) % 24000).astype(np.int32)
            sd.add_request(prompt, next_id, 50)
            waiting.append(next_id)
            next_id += 1
        elif roll < 0.5 and waiting:
            k = int(rng.integers(1, len(waiting) + 1))
            ids, waiting = waiting[:k], waiting[k:]
            do("prefill", ids)
        elif roll < 0.9 and live:
            ids = [x for x in live if sd.requests[x].context_len < max_seq - 1]
            if ids:
                ids = [ids[i] for i in rng.permutation(len(ids))]
                do("decode", ids)
        elif live:
            k = int(rng.integers(1, len(live) + 1))
            ids = [live[i] for i in rng.permutation(len(live))[:k]]
            ops.append(["free", ids])
            st.free_batch(ids)
            sd.release_requests(ids)
            live = [x for x in live if x not in ids]
    return {"L": L, "H": H, "max_seq_len": max_seq, "block_size": bs,
            "num_blocks": num_blocks, "ops": ops}
