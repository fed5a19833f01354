"""Host path parity: allocator + batch builder.

Three implementations are replayed through the scenarios of tests/scenarios.py:
  golden  - traces the COMPILED REFERENCE produced (tests/golden/host_traces.json,
            written by tests/golden/make_host_golden.py)
  oracle  - oracle/host_oracle.py (the CPU restatement; pinned here)
  product - muxserve_amd.memory_manager / batch_scheduler over libmuxhost.so
Bar: every returned integer identical (bit-exact).
"""
import json
import os

import numpy as np
import pytest

import scenarios
from oracle import host_oracle
from oracle import build_ref
from muxserve_amd.batch_scheduler import BatchScheduler
from muxserve_amd.memory_manager import KVStorage

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "host_traces.json")
with open(GOLDEN) as f:
    _GOLD = json.load(f)


def _first_diff(a, b):
    for i, (x, y) in enumerate(zip(a, b)):
        if x != y:
            keys = [k for k in x if x.get(k) != y.get(k)] if isinstance(x, dict) else []
            return f"record {i} differs in {keys}: {x if len(str(x)) < 400 else ''} vs {y if len(str(y)) < 400 else ''}"
    return f"length {len(a)} vs {len(b)}"


@pytest.mark.parametrize("name", sorted(_GOLD))
def test_oracle_matches_compiled_reference_golden(name):
    g = _GOLD[name]
    got = scenarios.run_scenario(host_oracle.KVStorage, host_oracle.BatchScheduler, g["scenario"])
    assert got == g["trace"], _first_diff(got, g["trace"])


@pytest.mark.parametrize("name", sorted(_GOLD))
def test_product_matches_compiled_reference_golden(name):
    g = _GOLD[name]
    got = scenarios.run_scenario(KVStorage, BatchScheduler, g["scenario"])
    assert got == g["trace"], _first_diff(got, g["trace"])


def test_scenario_definitions_match_fixture():
    """The fixture was generated from the scenario library in this tree."""
    for name, sc in scenarios.scripted_scenarios().items():
        assert _GOLD[name]["scenario"] == sc, name
    assert _GOLD["random_05"]["scenario"] == scenarios.random_scenario(5)


@pytest.mark.parametrize("seed", range(100, 300))
def test_product_matches_oracle_on_fresh_random_scenarios(seed):
    sc = scenarios.random_scenario(seed)
    a = scenarios.run_scenario(host_oracle.KVStorage, host_oracle.BatchScheduler, sc)
    b = scenarios.run_scenario(KVStorage, BatchScheduler, sc)
    assert a == b, _first_diff(a, b)


_REF = build_ref.load() if os.path.isdir(os.path.join(os.path.dirname(build_ref.__file__), "_ref")) else (None, None)


@pytest.mark.skipif(_REF[0] is None, reason="oracle/_ref not built (needs the reference checkout)")
@pytest.mark.parametrize("seed", range(200, 320))
def test_oracle_matches_live_compiled_reference(seed):
    sc = scenarios.random_scenario(seed)
    mm, bsm = _REF
    a = scenarios.run_scenario(mm.KVStorage, bsm.BatchScheduler, sc)
    b = scenarios.run_scenario(host_oracle.KVStorage, host_oracle.BatchScheduler, sc)
    assert a == b, _first_diff(a, b)


@pytest.mark.skipif(_REF[0] is None, reason="oracle/_ref not built (needs the reference checkout)")
@pytest.mark.parametrize("seed", range(400, 460))
def test_product_matches_live_compiled_reference(seed):
    sc = scenarios.random_scenario(seed)
    mm, bsm = _REF
    a = scenarios.run_scenario(mm.KVStorage, bsm.BatchScheduler, sc)
    b = scenarios.run_scenario(KVStorage, BatchScheduler, sc)
    assert a == b, _first_diff(a, b)


# ---- closed forms and invariants (pin the oracle where golden data is silent) ----

def test_fresh_pool_closed_form():
    """First batch needing M head-blocks on a fresh pool of N receives ids
    N-M..N-1 ascending, request 0 first, runs ordered [tokenBlock][layer][head]
    (csrc/memory_manager.cpp:104-135)."""
    N, L, H = 1000, 2, 5
    for cls in (host_oracle.KVStorage, KVStorage):
        s = cls(N)
        info = np.array([4, 3, 0, 9, 1, 0, 2, 2, 0], dtype=np.int32)
        r = s.allocate_batch(info, L, H)
        M = (3 + 1 + 2) * L * H
        assert r[0] == 3
        assert list(r[1:]) == list(range(N - M, N))
        assert s.get_new_blocks_allocated() == M


def test_allocate_pops_descending():
    for cls in (host_oracle.KVStorage, KVStorage):
        s = cls(10)
        assert list(s.allocate(4)) == [9, 8, 7, 6]
        assert list(s.allocate(0)) == []
        assert list(s.allocate(6)) == [5, 4, 3, 2, 1, 0]


def test_block_conservation_and_uniqueness():
    """No id is ever held twice and free + held == N, through a random run."""
    sc = scenarios.random_scenario(77)
    N, L, H = sc["num_blocks"], sc["L"], sc["H"]
    st, sd = KVStorage(N), BatchScheduler(L, H, sc["max_seq_len"], sc["block_size"])
    held = {}
    step = 0
    for op in sc["ops"]:
        if op[0] == "add":
            _, rid, plen, mt = op
            sd.add_request(np.arange(plen, dtype=np.int32), rid, mt)
        elif op[0] in ("prefill", "decode"):
            ids = [i for i in op[1] if sd.num_requests() and _alive(sd, i)]
            if not ids:
                continue
            step += 1
            last = [] if op[0] == "prefill" else [step] * len(ids)
            r = host_oracle.prepare_inputs(sd, st, L, H, ids, last)
            for rid in r["preempted_reqs"]:
                held.pop(rid, None)
            cut = int(r["block_info"][0])
            cur = 1
            for i in range(max(cut, 0)):
                n = int(r["batch_block_request"][3 * i + 1]) * L * H
                got = list(r["block_info"][cur:cur + n])
                cur += n
                if op[0] == "prefill":
                    held[ids[i]] = got
                else:
                    held.setdefault(ids[i], []).extend(got)
        elif op[0] == "free":
            st.free_batch(op[1])
            sd.release_requests(op[1])
            for rid in op[1]:
                held.pop(rid, None)
        flat = [x for v in held.values() for x in v]
        assert len(flat) == len(set(flat))
        assert st.num_free() + len(flat) == N
        for rid, v in held.items():
            assert st.num_held(rid) == len(v)


def _alive(sd, rid):
    try:
        sd.request_state(rid)
        return True
    except KeyError:
        return False


def test_slot_and_position_closed_forms():
    """slot = id*bs + offset; prompt token i -> (block i//bs, offset i%bs);
    decode token -> last block, offset (ctx-1)%bs; position = ctx-1
    (csrc/batch_scheduler.h:42-67, csrc/batch_scheduler.cpp:132-147)."""
    L, H, bs, N = 2, 3, 16, 4096
    for S, B in ((host_oracle.KVStorage, host_oracle.BatchScheduler), (KVStorage, BatchScheduler)):
        st, sd = S(N), B(L, H, 512, bs)
        sd.add_request(np.arange(37, dtype=np.int32), 5, 10)
        r = host_oracle.prepare_inputs(sd, st, L, H, [5], [])
        ids = np.asarray(r["block_info"][1:]).reshape(3, L, H)     # [tokenBlock][l][h]
        slots = r["slot_mapping"].numpy()
        for i in range(37):
            assert (slots[i] == ids[i // bs].astype(np.int64) * bs + i % bs).all()
        assert list(r["input_positions"][:37]) == list(range(37))
        assert r["input_tensor"].shape[0] == 40 and (r["input_tensor"][37:] == 0).all()
        assert tuple(r["block_tables"].shape) == (0, 0, 0, 0)      # permute of (0, maxBlk=0, 0, 0)
        for step in range(30):
            r = host_oracle.prepare_inputs(sd, st, L, H, [5], [123 + step])
            ctx = 38 + step
            assert list(r["context_lens"]) == [ctx]
            assert int(r["input_positions"][0]) == ctx - 1
            assert int(r["input_tensor"][0]) == 123 + step
            bt = r["block_tables"].numpy()                         # [L, 1, H, maxBlk]
            nblk = (ctx + bs - 1) // bs
            assert bt.shape == (L, 1, H, nblk)
            want = bt[:, 0, :, nblk - 1].astype(np.int64) * bs + (ctx - 1) % bs
            assert (r["slot_mapping"].numpy()[0] == want).all()


def test_permuted_table_equals_reference_permute():
    """get_batch_permuted == get_batch followed by permute(2,0,3,1).contiguous()
    (muxserve/flexserver/llm_runtime.py:327) on the valid entries."""
    import torch
    L, H, bs, N = 3, 4, 16, 8192
    a_st, a_sd = KVStorage(N), BatchScheduler(L, H, 256, bs)
    b_st, b_sd = KVStorage(N), BatchScheduler(L, H, 256, bs)
    lens = [5, 40, 17]
    for sd in (a_sd, b_sd):
        for i, p in enumerate(lens):
            sd.add_request(np.arange(p, dtype=np.int32), i, 9)
    host_oracle.prepare_inputs(a_sd, a_st, L, H, [0, 1, 2], [])
    host_oracle.prepare_inputs(b_sd, b_st, L, H, [0, 1, 2], [])
    for step in range(20):
        ra = host_oracle.prepare_inputs(a_sd, a_st, L, H, [2, 0, 1], [1, 2, 3], fill=-1)
        info = b_sd.try_batch([2, 0, 1], [1, 2, 3])
        req = np.ascontiguousarray(info[:-1])
        blk = b_st.allocate_batch(req, L, H) if info[-1] > 0 else np.array([3], dtype=np.int32)
        bi = b_sd.get_batch_info(req, blk)
        max_blk = bi[3] + 2     # caller may over-allocate the row
        tok = torch.empty(8, dtype=torch.int32)
        pos = torch.empty(8, dtype=torch.int32)
        ctx = torch.empty(3, dtype=torch.int32)
        bt = torch.full((L, 3, H, max_blk), -1, dtype=torch.int32)
        slot = torch.empty((3, L, H), dtype=torch.int64)
        b_sd.get_batch_permuted(req, blk, tok, pos, ctx, bt, slot)
        assert torch.equal(ctx, ra["context_lens"])
        assert torch.equal(slot, ra["slot_mapping"])
        assert torch.equal(tok.long(), ra["input_tensor"])
        want = torch.full_like(bt, -1)
        want[..., :bi[3]] = ra["block_tables"]
        for b in range(3):
            valid = (int(ctx[b]) + bs - 1) // bs
            want[:, b, :, valid:] = -1
        assert torch.equal(bt, want)


def test_error_paths_raise_instead_of_corrupting():
    st, sd = KVStorage(4), BatchScheduler(1, 1, 64, 16)
    with pytest.raises(MemoryError):
        st.allocate(5)
    with pytest.raises(KeyError):
        sd.try_batch([42], [])
    sd.add_request(np.arange(20, dtype=np.int32), 1, 4)
    info = sd.try_batch([1], [])
    blk = st.allocate_batch(info[:-1], 1, 1)
    sd.get_batch_info(info[:-1], blk)
    import torch
    small = torch.empty(8, dtype=torch.int32)
    with pytest.raises(MemoryError):   # 20 tokens do not fit 8
        sd.get_batch(info[:-1], blk, small, small.clone(), torch.empty(0, dtype=torch.int32),
                     torch.empty(0, dtype=torch.int32), torch.empty((20, 1, 1), dtype=torch.int64))
    with pytest.raises(TypeError):     # wrong dtype
        sd.get_batch(info[:-1], blk, torch.empty(24, dtype=torch.int64), torch.empty(24, dtype=torch.int32),
                     torch.empty(0, dtype=torch.int32), torch.empty(0, dtype=torch.int32),
                     torch.empty((20, 1, 1), dtype=torch.int64))
