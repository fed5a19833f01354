"""A model runtime's side of the FlexStore protocol, as a process of its own
(started by tests/test_flexstore_process.py): connects to a FlexStore process,
goes through the start-up handshake, then drives its own BatchScheduler through
prefill and decode steps with prepare_inputs, every block allocation and every
release being a request over the transport (muxserve/flexserver/llm_runtime.py:
277-339, 585-599).  Writes what it asked and what it was told to a pickle.

    python flexstore_runtime_process.py ADDRESS MODEL L H SEED STEPS OUT.pkl
"""
import os
import pickle
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)


def main():
    address, model, L, H, seed, steps, out = sys.argv[1], sys.argv[2], *map(int, sys.argv[3:7]), sys.argv[7]
    from muxserve_amd.batch_scheduler import BatchScheduler
    from muxserve_amd.flexstore_service import PipeClient
    from muxserve_amd.prepare import prepare_inputs

    client = None
    for _ in range(200):                      # the FlexStore process may still be starting
        try:
            client = PipeClient(address)
            break
        except (FileNotFoundError, ConnectionRefusedError):
            time.sleep(0.05)
    assert client is not None, "FlexStore process not reachable"
    log = []

    def ask(kind, args=None):
        reply = client.request(kind, args)
        log.append(((kind, args), reply))
        return reply

    num_blocks = ask("get_num_blocks")
    assert ask("get_rank", 0) == 0
    while not ask("start_warmup"):            # one runtime warms up at a time (llm_runtime.py:600-640)
        time.sleep(0.01)
    ask("warmup_ready")
    while not ask("init_finished"):           # serve only once every runtime is up, so that the runtimes' steps interleave
        time.sleep(0.005)

    bs, max_seq = 16, 512
    rng = np.random.Generator(np.random.PCG64(seed))
    sched = BatchScheduler(L, H, max_seq, bs)
    alloc = lambda r: ask("cache_alloc", [model, r])      # noqa: E731
    # Request ids are unique across the models of a FlexStore: its one KVStorage keys the blocks by
    # request id alone (muxserve/flexstore/manager.py:776-790; the scheduler hands out global ids).
    next_id = 1000 * seed
    live = []
    steps_done = []
    for wave in range(3):
        new = []
        for _ in range(int(rng.integers(2, 5))):
            n = int(rng.integers(3, 70))
            sched.add_request(rng.integers(0, 32000, size=n).astype(np.int32), next_id, steps + 4)
            new.append(next_id)
            next_id += 1
        # prefill step for the newcomers, then decode steps for everybody alive
        _, _, md, batch_reqs, preempted = prepare_inputs(sched, alloc, new, [], "cpu")
        live = [i for i in live + new if i not in preempted]
        steps_done.append(("prefill", list(new), md.slot_mapping.numpy().copy(), list(preempted)))
        for s in range(steps):
            if not live:
                break
            _, _, md, batch_reqs, preempted = prepare_inputs(sched, alloc, live, [7 + s] * len(live), "cpu")
            steps_done.append(("decode", list(live), md.block_tables.numpy().copy(), list(preempted)))
            live = [i for i in live if i not in preempted]
        # the oldest requests finish: released here and at the store (llm_runtime.py:585-599)
        done, live = live[: len(live) // 2], live[len(live) // 2:]
        if done:
            sched.release_requests(done)
            ask("free_cache", [model, done])
    if live:
        sched.release_requests(live)
        ask("free_cache", [model, live])
    client.close()
    with open(out, "wb") as f:
        pickle.dump({"model": model, "num_blocks": num_blocks, "log": log, "steps": steps_done}, f)


if __name__ == "__main__":
    main()
