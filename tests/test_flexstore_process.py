"""FlexStore behind a real process boundary (CPU only): a FlexStore process
serves the request loop of muxserve/flexstore/manager.py:747-838 over a local
socket, two model runtimes - processes of their own, different layer and head
counts - run prefill and decode steps against it through prepare_inputs.  The
store answers one request at a time; its log of (request, reply) in the order
served, replayed through the in-process CacheRequestHandler over a fresh
allocator, must give the same replies, and every runtime must have been told
exactly what the log says it was told.
"""
import json
import os
import pickle
import subprocess
import sys
import time

import numpy as np

from muxserve_amd.flexstore import CacheRequestHandler
from muxserve_amd.flexstore_service import PipeClient
from muxserve_amd.memory_manager import KVStorage

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CHILD = os.path.join(ROOT, "tests", "helpers", "flexstore_runtime_process.py")


def _same(a, b):
    if isinstance(a, np.ndarray) or isinstance(b, np.ndarray):
        return isinstance(a, np.ndarray) and isinstance(b, np.ndarray) and a.dtype == b.dtype and np.array_equal(a, b)
    if isinstance(a, (list, tuple)) and isinstance(b, (list, tuple)):
        return len(a) == len(b) and all(_same(x, y) for x, y in zip(a, b))
    return a == b


def test_two_runtime_processes_share_one_flexstore_process(tmp_path):
    address = str(tmp_path / "flexstore.sock")
    log_path = str(tmp_path / "served.pkl")
    models = {"llama-a": [2, 4], "llama-b": [3, 2]}
    num_blocks = 1400                     # small enough that the two models contend for it
    env = dict(os.environ, PYTHONPATH=ROOT)
    store = subprocess.Popen([sys.executable, "-m", "muxserve_amd.flexstore_service", "--address", address,
                              "--num-blocks", str(num_blocks), "--models", json.dumps(models),
                              "--num-runtime-processes", "2", "--log", log_path], cwd=ROOT, env=env)
    outs, runtimes = [], []
    try:
        for i, (name, (L, H)) in enumerate(models.items()):
            out = str(tmp_path / f"runtime{i}.pkl")
            outs.append(out)
            runtimes.append(subprocess.Popen([sys.executable, CHILD, address, name, str(L), str(H), str(11 + i), "6", out],
                                             cwd=ROOT, env=env))
        for p in runtimes:
            assert p.wait(timeout=120) == 0
        # both runtimes are through their warm-up: the store says so, then it is told to stop
        me = None
        for _ in range(100):
            try:
                me = PipeClient(address)
                break
            except (FileNotFoundError, ConnectionRefusedError):
                time.sleep(0.05)
        assert me.request("init_finished") is True
        assert me.request("query_num_ready_processes") == 2
        assert me.request("not a request type", None) == "Incorrect format"
        me.send_pyobj(("exit", None))             # no reply to an exit (manager.py:823-827)
        assert store.wait(timeout=60) == 0
        me.close()
    finally:
        for p in runtimes + [store]:
            if p.poll() is None:
                p.kill()

    served = pickle.load(open(log_path, "rb"))
    results = [pickle.load(open(o, "rb")) for o in outs]
    # 1. the in-process handler, fed the same requests in the same order, answers the same
    handler = CacheRequestHandler(KVStorage(num_blocks), {k: tuple(v) for k, v in models.items()}, num_blocks,
                                  num_runtime_processes=2)
    kinds = {}
    for req, reply in served:
        kinds[req[0]] = kinds.get(req[0], 0) + 1
        if req[0] == "not a request type":
            assert handler.handle(req) == "Incorrect format"
            continue
        assert _same(handler.handle(req), reply), req
    assert kinds["cache_alloc"] >= 10 and kinds["free_cache"] >= 4 and kinds["warmup_ready"] == 2
    assert handler.block_manager.num_free() == num_blocks, "everything was released at the end"
    # 2. each runtime's own record is, in order, what the store's log holds for that model
    for res in results:
        mine = [(req, reply) for req, reply in served
                if req[0] in ("cache_alloc", "free_cache") and req[1][0] == res["model"]]
        theirs = [(req, reply) for req, reply in res["log"] if req[0] in ("cache_alloc", "free_cache")]
        assert len(mine) == len(theirs) > 0
        for (rq_a, rp_a), (rq_b, rp_b) in zip(mine, theirs):
            assert _same(rq_a[1][1], rq_b[1][1]) and _same(rp_a, rp_b)
        assert res["num_blocks"] == num_blocks
        assert any(kind == "decode" for kind, *_ in res["steps"])
