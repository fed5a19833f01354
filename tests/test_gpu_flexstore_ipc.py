"""The FlexStore process boundary with the pool on the GPU: this process owns a
SMALL pool (64 MiB; exporting the 185 GB one is excluded, see
muxserve_amd.flexstore.MAX_IPC_BYTES) and answers the request loop of
muxserve/flexstore/manager.py:747-838 over a local socket; a freshly started
runtime process asks for the pool ("cache_init", manager.py:789-793), maps it
from the IPC handle (as model_loader.py:46 maps the weights) and runs a prefill
step and three decode steps of a two-layer model on it.  Checked here, in the
owning process: the pool holds bit for bit what the oracle's cache write puts
there, every layer's attention output is within 2e-3 of the oracle, and the
allocator got everything back.
"""
import os
import pickle
import subprocess
import sys
import threading

import pytest
import torch

from oracle import attn_oracle as orc
from muxserve_amd.flexstore import MAX_IPC_BYTES, CacheRequestHandler, IpcExportExcluded
from muxserve_amd.flexstore_service import PipeServer, serve
from muxserve_amd.memory_manager import KVStorage
from muxserve_amd.pool import allocate_gpu_cache

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CHILD = os.path.join(ROOT, "tests", "helpers", "flexstore_gpu_runtime_process.py")
TOL = 2e-3


def test_a_runtime_process_works_on_the_pool_of_the_flexstore_process(tmp_path):
    print("[case] pool exported to a second process, cache write + decode there", flush=True)
    bs, N = 16, 8192                                   # 32 MiB of K + 32 MiB of V
    k_pool, v_pool = allocate_gpu_cache(N, bs, DEV)
    k_pool.zero_()
    v_pool.zero_()
    torch.cuda.synchronize()
    storage = KVStorage(N)
    handler = CacheRequestHandler(storage, {"small": (2, 4)}, N, gpu_cache=(k_pool, v_pool))
    address = str(tmp_path / "flexstore.sock")
    server = PipeServer(address)
    log = []
    failure = []

    def loop():
        try:
            serve(handler, server, log)
        except Exception as e:          # noqa: BLE001  (reported by the test below)
            failure.append(e)

    th = threading.Thread(target=loop, daemon=True)
    th.start()
    out_path = str(tmp_path / "runtime.pkl")
    child = subprocess.Popen([sys.executable, CHILD, address, out_path], cwd=ROOT, env=dict(os.environ, PYTHONPATH=ROOT))
    try:
        rc = child.wait(timeout=300)
    finally:
        if child.poll() is None:
            child.kill()
    assert not failure, failure
    assert rc == 0, "the runtime process failed"
    # stop the loop the way the reference's is stopped
    from muxserve_amd.flexstore_service import PipeClient
    me = PipeClient(address)
    me.send_pyobj(("exit", None))
    th.join(timeout=30)
    me.close()
    server.close()
    assert not th.is_alive() and not failure

    res = pickle.load(open(out_path, "rb"))
    L, Hq, Hkv, D, _ = res["shape"]
    hk, hv = orc.allocate_pool(N, bs, torch.float16)
    hk.zero_()
    hv.zero_()
    for r in res["record"]:
        n, l = r["n"], r["layer"]
        qkv = r["qkv_in"]
        rq, rk = orc.rotary_neox(r["positions"][:n], qkv[:, :Hq * D].clone(), qkv[:, Hq * D:(Hq + Hkv) * D].clone())
        gq, gk = r["q_rot"][:n], r["k_rot"][:n]
        assert (gq.float() - rq).abs().max() <= 4e-3 and (gk.float() - rk).abs().max() <= 4e-3
        v_in = qkv[:, (Hq + Hkv) * D:]
        orc.reshape_and_cache(gk, v_in, hk, hv, r["slot_mapping"], layer=l, num_tokens=n)
        if r["prompt_lens"]:
            want = orc.prefill_causal(gq, gk, v_in[:n], r["prompt_lens"], D ** -0.5, Hkv)
        else:
            want = orc.paged_decode(gq, hk, hv, r["block_tables"], r["context_lens"].numpy(), D ** -0.5, layer=l)
        err = (r["out"][:n].float() - want).abs().max().item()
        assert err <= TOL, f"step {r['step']} layer {l}: max-abs error {err:.3e}"
    torch.cuda.synchronize()
    assert torch.equal(k_pool.cpu().view(torch.int16), hk.view(torch.int16)), "K pool differs from the oracle's"
    assert torch.equal(v_pool.cpu().view(torch.int16), hv.view(torch.int16)), "V pool differs from the oracle's"
    assert storage.num_free() == N
    kinds = [req[0] for req, _ in log]
    assert kinds[0] == "cache_init" and kinds.count("cache_alloc") >= 2 and kinds[-2:] == ["free_cache", "exit"]


def test_a_pool_too_large_to_open_elsewhere_is_refused_by_name():
    """The export of a pool tensor of 2 GiB or more is refused before any handle
    is made (nothing that large is allocated here: the check reads the storage's
    size)."""
    class _Storage:
        def nbytes(self):
            return MAX_IPC_BYTES + 1

    class _Big:
        def untyped_storage(self):
            return _Storage()

    handler = CacheRequestHandler(KVStorage(16), {"m": (1, 1)}, 16, gpu_cache=(_Big(), _Big()))
    with pytest.raises(IpcExportExcluded, match="cannot be opened by another process"):
        handler.handle(("cache_init", [0, "m"]))
