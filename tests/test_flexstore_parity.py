"""The FlexStore request handler (muxserve_amd.flexstore) and the compute-share
bookkeeping (muxserve_amd.cu_resource) against the oracle's restatement of the
reference's loop body (muxserve/flexstore/manager.py:747-831) and of SMResource
(muxserve/muxsched/resource.py:15-81).  The oracle side allocates from the
COMPILED reference KVStorage when oracle/_ref is built, so the replies compared
here are the reference allocator's own.  CPU only.
"""
import os
import random

import numpy as np
import pytest

from oracle import build_ref, flexstore_oracle, host_oracle
from muxserve_amd import cu_resource
from muxserve_amd.batch_scheduler import BatchScheduler
from muxserve_amd.flexstore import INCORRECT_FORMAT, CacheRequestHandler, IpcExportExcluded
from muxserve_amd.memory_manager import KVStorage
from muxserve_amd.prepare import prepare_inputs

_REF = build_ref.load() if os.path.isdir(os.path.join(os.path.dirname(build_ref.__file__), "_ref")) else (None, None)
RefStorage = _REF[0].KVStorage if _REF[0] is not None else host_oracle.KVStorage

MODELS = {"llama-7b": (2, 3), "llama-13b": (3, 2), "llama-30b": (1, 5)}


def _pair(num_blocks, **kw):
    ref = flexstore_oracle.new_state(RefStorage(num_blocks), MODELS, num_blocks, **kw)
    got = CacheRequestHandler(KVStorage(num_blocks), MODELS, num_blocks, **kw)
    return ref, got


def _same(a, b):
    if a is None or b is None or isinstance(a, (bool, int, str)):
        assert a == b and type(a) is type(b), (a, b)
    else:
        assert np.array_equal(np.asarray(a), np.asarray(b)), (a, b)


def test_documented_request_formats_and_a_fresh_pool():
    """Tuple["cache_alloc", [model, batch_info]] on a fresh pool of N blocks that
    needs M head-blocks returns [number of requests served, N-M .. N-1]
    (csrc/memory_manager.cpp:104-135); free_cache returns None and the freed
    blocks are handed out again."""
    N = 600
    ref, got = _pair(N)
    L, H = MODELS["llama-7b"]
    info = np.array([4, 3, 0, 9, 1, 0, 2, 2, 0], dtype=np.int32)      # three requests: 3, 1, 2 new token blocks
    M = (3 + 1 + 2) * L * H
    for side in (lambda r: flexstore_oracle.deploy_step(ref, r), got.handle):
        reply = np.asarray(side(("cache_alloc", ["llama-7b", info])))
        assert reply[0] == 3 and list(reply[1:]) == list(range(N - M, N))
        assert side(("free_cache", ["llama-7b", [4, 2]])) is None
        assert side(("get_num_blocks", None)) == N
    assert got.model_occupy_info == ref["model_occupy_info"]
    assert got.model_occupy_info["llama-7b"] == -(3 + 2) * L * H      # the reference only ever subtracts (manager.py:818, 834-837)


@pytest.mark.parametrize("seed", range(12))
def test_request_streams_get_the_reference_replies(seed):
    """Three colocated models with their own batch builders share one pool
    through the handler: prefill and decode rounds, finished requests, a pool
    small enough to preempt.  Every reply equals the reference loop's."""
    rng = np.random.Generator(np.random.PCG64(seed))
    N = int(rng.integers(150, 900))
    ref, got = _pair(N)
    bs = 16
    scheds = {m: (BatchScheduler(L, H, 256, bs), BatchScheduler(L, H, 256, bs)) for m, (L, H) in MODELS.items()}
    live = {m: [] for m in MODELS}
    next_id = 0
    for step in range(40):
        m = list(MODELS)[int(rng.integers(3))]
        action = rng.integers(4)
        sa, sb = scheds[m]
        if action == 0 or not live[m]:
            ids = []
            for _ in range(int(rng.integers(1, 4))):
                prompt = rng.integers(0, 1000, size=int(rng.integers(1, 60))).astype(np.int32)
                for s in (sa, sb):
                    s.add_request(prompt, next_id, 64)
                ids.append(next_id)
                next_id += 1
            last = []
        elif action == 3:
            k = int(rng.integers(1, len(live[m]) + 1))
            done = [int(x) for x in rng.permutation(live[m])[:k]]
            _same(flexstore_oracle.deploy_step(ref, ("free_cache", [m, done])), got.handle(("free_cache", [m, done])))
            for s in (sa, sb):
                s.release_requests(done)
            live[m] = [r for r in live[m] if r not in done]
            continue
        else:
            ids, last = list(live[m]), [int(x) for x in rng.integers(0, 1000, size=len(live[m]))]
        info_a = np.asarray(sa.try_batch(ids, last), dtype=np.int32)
        info_b = np.asarray(sb.try_batch(ids, last), dtype=np.int32)
        assert np.array_equal(info_a, info_b)
        if int(info_a[-1]) > 0:
            ra = flexstore_oracle.deploy_step(ref, ("cache_alloc", [m, np.ascontiguousarray(info_a[:-1])]))
            rb = got.handle(("cache_alloc", [m, np.ascontiguousarray(info_b[:-1])]))
            _same(ra, rb)
        else:
            ra = rb = np.array([len(ids)], dtype=np.int32)
        for s, r, info in ((sa, ra, info_a), (sb, rb, info_b)):
            s.get_batch_info(np.ascontiguousarray(info[:-1]), np.asarray(r, dtype=np.int32))
        cut = list(sa.get_preempt_requests())
        assert cut == list(sb.get_preempt_requests())
        live[m] = [r for r in dict.fromkeys(live[m] + ids) if r not in cut]
        assert got.model_occupy_info == ref["model_occupy_info"]


def test_start_up_bookkeeping_and_the_edges_of_the_protocol():
    ref, got = _pair(64, num_runtime_processes=2, rank=1, local_world_size=4)
    stream = [("get_rank", 3), ("init_finished", None), ("start_warmup", None), ("start_warmup", None),
              ("warmup_ready", None), ("query_num_ready_processes", None), ("start_warmup", None),
              ("warmup_ready", None), ("init_finished", None), ("log_stats", None), ("no_such_request", 1)]
    want = [7, False, True, False, False, 1, True, True, True, None, INCORRECT_FORMAT]
    for req, w in zip(stream, want):
        a, b = flexstore_oracle.deploy_step(ref, req), got.handle(req)
        _same(a, b)
        _same(b, w)
    for req in (("blocktable_load", [3]), ("blocktable_store", [3, None])):     # listed, but the loop has no branch
        with pytest.raises(RuntimeError, match="Unknown request type"):
            flexstore_oracle.deploy_step(ref, req)
        with pytest.raises(RuntimeError, match="Unknown request type"):
            got.handle(req)
    for kind in ("weight", "cache_init", "lock_init"):
        with pytest.raises(IpcExportExcluded):
            got.handle((kind, [0, "llama-7b"]))
    assert got.handle(("exit", None)) is None and got.closed
    with pytest.raises(RuntimeError):
        got.handle(("get_num_blocks", None))


def test_prepare_inputs_through_the_handler_equals_the_direct_allocator_call():
    """prepare_inputs' cache_alloc callable bound to a model name is the
    runtime's request of llm_runtime.py:284-286 without the socket."""
    L, H = MODELS["llama-13b"]
    N = 500
    handler = CacheRequestHandler(KVStorage(N), MODELS, N)
    direct_store, s1, s2 = KVStorage(N), BatchScheduler(L, H, 256, 16), BatchScheduler(L, H, 256, 16)
    for i, p in enumerate([20, 7, 33]):
        prompt = np.arange(p, dtype=np.int32) + i
        s1.add_request(prompt, i, 32)
        s2.add_request(prompt, i, 32)
    for ids, last in (([0, 1, 2], []), ([0, 1, 2], [5, 6, 7]), ([2, 0, 1], [8, 9, 10])):
        a = prepare_inputs(s1, handler.cache_alloc_for("llama-13b"), ids, last, device="cpu")
        b = prepare_inputs(s2, lambda r: direct_store.allocate_batch(r, L, H), ids, last, device="cpu")
        assert np.array_equal(a[2].slot_mapping.numpy(), b[2].slot_mapping.numpy())
        assert np.array_equal(a[2].context_lens.numpy(), b[2].context_lens.numpy())


# ---- compute shares ------------------------------------------------------------------

@pytest.mark.parametrize("seed", range(20))
def test_cu_resource_hands_out_what_sm_resource_hands_out(seed):
    rng = np.random.Generator(np.random.PCG64(seed))
    thr = int(rng.integers(0, 6))
    ref, got = flexstore_oracle.SMResource(thr), cu_resource.CUResource(thr)
    held = []
    for step in range(200):
        if held and rng.integers(3) == 0:
            a, b = held.pop(int(rng.integers(len(held))))
            ref.free(a)
            got.free(b)
        else:
            n, over = int(rng.integers(0, 7)), bool(rng.integers(2))
            assert ref.can_allocate(n, over) == got.can_allocate(n, over)
            if ref.can_allocate(n, over) and (ref.num_free_sms >= n or (over and len(ref.unoverloaded_sms) >= n)):
                random.seed(1000 * seed + step)
                a = ref.allocate(n, over)
                random.seed(1000 * seed + step)
                b = got.allocate(n, over)
                assert [p.id for p in a] == [p.id for p in b]
                held.append((a, b))
        assert ref.num_free_sms == got.num_free_sms and ref.num_overloaded_sms == got.num_overloaded_sms
        assert [p.id for p in ref.free_sms] == [p.id for p in got.free_sms]
        assert ref.unoverloaded_sms == got.unoverloaded_sms
    # conservation: every part's reference count is the number of holders that name it
    count = [0] * 10
    for _, b in held:
        for p in b:
            count[p.id] += 1
    assert count == [p.ref_count for p in got._parts]


def test_fresh_cu_resource_closed_forms():
    r = cu_resource.CUResource()
    assert [p.id for p in r.allocate(3)] == [9, 8, 7]               # the free list is a stack (resource.py:58)
    assert r.num_free_sms == 7 and r.num_overloaded_sms == 0
    assert r.can_allocate(7) and not r.can_allocate(8) and r.can_allocate(11, overload=True)
    assert not r.can_allocate(12, overload=True)                     # 7 free + min(4, 10) extra


@pytest.mark.parametrize("num_cus", [256, 304, 64])
def test_part_masks_are_disjoint_cover_the_gpu_and_are_balanced_over_the_dies(num_cus):
    """Mask bit i enables a compute unit of die i % 8 (consecutive bits go
    round-robin over the 8 accelerator dies: measured with a kernel that records the die of every workgroup).
    Every part must therefore hold floor or ceil of its share of every die,
    parts must not overlap and all ten together are the whole GPU."""
    seen = set()
    for p in range(10):
        cus = cu_resource.enabled_cus([p], num_cus)
        assert len(cus) in (num_cus // 10, num_cus // 10 + 1)
        assert not seen & set(cus)
        seen |= set(cus)
        per_die = np.bincount(np.asarray(cus) % 8, minlength=8)
        assert per_die.max() - per_die.min() <= 1 and (per_die.min() >= 1 or num_cus < 80)
    assert seen == set(range(num_cus))
    a, b = [0, 3, 7], [1, 2, 9]
    ca, cb = cu_resource.enabled_cus(a, num_cus), cu_resource.enabled_cus(b, num_cus)
    assert not set(ca) & set(cb)
    for cus, parts in ((ca, a), (cb, b)):
        per_die = np.bincount(np.asarray(cus) % 8, minlength=8)
        assert per_die.max() - per_die.min() <= len(parts)
    words = cu_resource.cu_mask_words(a, num_cus)
    assert sum(bin(w).count("1") for w in words) == len(ca)
    with pytest.raises(ValueError):
        cu_resource.part_bits([])
    with pytest.raises(ValueError):
        cu_resource.part_bits([10])


def test_hsa_cu_mask_string_names_the_same_compute_units():
    s = cu_resource.hsa_cu_mask_env([0, 1, 5], 256, gpu_index=2)
    assert s.startswith("2:")
    cus = []
    for run in s[2:].split(","):
        lo, _, hi = run.partition("-")
        cus += list(range(int(lo), int(hi or lo) + 1))
    assert cus == cu_resource.enabled_cus([0, 1, 5], 256)
    assert s == "2:0-50,128-152"
