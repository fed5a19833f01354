"""muxserve_amd.prepare.prepare_inputs against the oracle's restatement of
LLMRuntime.prepare_inputs (muxserve/flexserver/llm_runtime.py:277-339), tensor
by tensor: padding of the token rows to a multiple of 8, the int64 widening, the
[T, L, H] slot mapping, the empty (0, maxBlk, 0, 0) table of a prompt-only step,
the permute(2, 0, 3, 1) of the block table and every InputMetadata field.  The
oracle side is driven by the compiled reference classes when oracle/_ref is
built (else by the oracle's own classes, which other tests pin to the compiled
reference's golden traces); the product side runs on the CPU device, through
libmuxhost.so, in both table layouts.
"""
import os

import numpy as np
import pytest
import torch

from oracle import build_ref, host_oracle
from muxserve_amd.batch_scheduler import BatchScheduler
from muxserve_amd.memory_manager import KVStorage
from muxserve_amd.prepare import prepare_inputs

_REF = build_ref.load() if os.path.isdir(os.path.join(os.path.dirname(build_ref.__file__), "_ref")) else (None, None)


def _reference_classes():
    if _REF[0] is not None:
        return _REF[0].KVStorage, _REF[1].BatchScheduler
    return host_oracle.KVStorage, host_oracle.BatchScheduler


def _compare(ref, got, bs, permuted):
    tok, pos, md, batch_reqs, preempted = got
    # token rows: int64, padded to a multiple of 8 (llm_runtime.py:300, 324-325)
    T = sum(ref["prompt_lens"]) + int(ref["context_lens"].numel())
    assert tok.dtype == torch.int64 and pos.dtype == torch.int64
    assert tok.shape == ref["input_tensor"].shape == ((T + 7) // 8 * 8,)
    assert torch.equal(tok[:T], ref["input_tensor"][:T]) and torch.equal(pos[:T], ref["input_positions"][:T])
    # slot mapping int64 [T, L, H] (llm_runtime.py:301-302)
    assert md.slot_mapping.dtype == torch.int64 and md.slot_mapping.shape == ref["slot_mapping"].shape
    assert torch.equal(md.slot_mapping, ref["slot_mapping"])
    # context lengths int32 [num_contexts]
    assert md.context_lens.dtype == torch.int32 and torch.equal(md.context_lens, ref["context_lens"])
    assert md.max_context_len == ref["max_context_len"]
    assert md.prompt_lens == [int(x) for x in ref["prompt_lens"]]
    assert md.total_context_len == int(ref["context_lens"].sum())
    if md.context_lens.numel():
        assert md.context_lens_host is not None and torch.equal(md.context_lens_host, ref["context_lens"])
    # block table [L, B, H, maxBlk] after permute(2, 0, 3, 1) (llm_runtime.py:327); entries past a
    # sequence's blocks are memory the reference never writes
    rt = ref["block_tables"]
    assert md.block_tables.dtype == torch.int32
    if ref["max_context_len"] > 0:
        assert md.block_tables.shape == rt.shape and md.block_tables.is_contiguous()
        for c, n_ctx in enumerate(ref["context_lens"].tolist()):
            valid = (n_ctx + bs - 1) // bs
            assert torch.equal(md.block_tables[:, c, :, :valid], rt[:, c, :, :valid])
    else:
        # a step without decoding sequences: an empty table whose only non-zero extent is maxBlk
        assert rt.numel() == 0 and md.block_tables.numel() == 0
        if not permuted:
            assert md.block_tables.shape == rt.shape
    assert [list(x) for x in batch_reqs] == [list(x) for x in ref["batch_reqs"]]
    assert list(preempted) == list(ref["preempted_reqs"])


@pytest.mark.parametrize("permuted", [False, True])
@pytest.mark.parametrize("L,H,bs", [(2, 3, 16), (1, 1, 8), (3, 2, 32)])
def test_prepare_inputs_equals_the_reference_restatement(L, H, bs, permuted):
    rng = np.random.Generator(np.random.PCG64(L * 1000 + H * 10 + bs))
    N = 3000
    RefStorage, RefSched = _reference_classes()
    ref_store, ref_sched = RefStorage(N), RefSched(L, H, 512, bs)
    store, sched = KVStorage(N), BatchScheduler(L, H, 512, bs)
    alloc = lambda r: store.allocate_batch(r, L, H)      # noqa: E731
    lens = [5, bs, bs + 1, 3 * bs - 1, 1, 2 * bs]
    for i, p in enumerate(lens):
        prompt = rng.integers(0, 1000, size=p).astype(np.int32)
        ref_sched.add_request(prompt, i, 64)
        sched.add_request(prompt, i, 64)
    ids = list(range(len(lens)))
    # a prompt-only step (the empty table), in two batches
    for part in (ids[:4], ids[4:]):
        _compare(host_oracle.prepare_inputs(ref_sched, ref_store, L, H, part, []),
                 prepare_inputs(sched, alloc, part, [], device="cpu", permuted_tables=permuted), bs, permuted)
    # decode steps across block boundaries, in a shuffled order
    order = [3, 0, 5, 4, 1, 2]
    for step in range(bs + 3):
        last = [100 + step + i for i in range(len(order))]
        _compare(host_oracle.prepare_inputs(ref_sched, ref_store, L, H, order, last),
                 prepare_inputs(sched, alloc, order, last, device="cpu", permuted_tables=permuted), bs, permuted)
    # a mixed step: two new prompts together with decoding sequences
    for rid, p in ((10, 2 * bs + 3), (11, 7)):
        prompt = rng.integers(0, 1000, size=p).astype(np.int32)
        ref_sched.add_request(prompt, rid, 64)
        sched.add_request(prompt, rid, 64)
    for s_, st_ in ((ref_sched, ref_store), (sched, store)):
        st_.free_batch([1, 4])
        s_.release_requests([1, 4])
    _compare(host_oracle.prepare_inputs(ref_sched, ref_store, L, H, [10, 11], []),
             prepare_inputs(sched, alloc, [10, 11], [], device="cpu", permuted_tables=permuted), bs, permuted)
    mixed = [0, 10, 2, 11, 3, 5]
    for step in range(3):
        last = [7 + step] * len(mixed)
        _compare(host_oracle.prepare_inputs(ref_sched, ref_store, L, H, mixed, last),
                 prepare_inputs(sched, alloc, mixed, last, device="cpu", permuted_tables=permuted), bs, permuted)


def test_prepare_inputs_under_allocator_preemption_equals_the_reference_restatement():
    """A pool too small for the batch: the allocator preempts from the tail and
    both sides must report the same survivors, tensors and preempted ids."""
    L, H, bs, N = 2, 2, 16, 2 * 2 * 9
    RefStorage, RefSched = _reference_classes()
    ref_store, ref_sched = RefStorage(N), RefSched(L, H, 256, bs)
    store, sched = KVStorage(N), BatchScheduler(L, H, 256, bs)
    alloc = lambda r: store.allocate_batch(r, L, H)      # noqa: E731
    for i, p in enumerate([40, 33, 50, 20]):
        prompt = (np.arange(p, dtype=np.int32) * 3 + i) % 997
        ref_sched.add_request(prompt, i, 32)
        sched.add_request(prompt, i, 32)
    ref = host_oracle.prepare_inputs(ref_sched, ref_store, L, H, [0, 1, 2, 3], [])
    got = prepare_inputs(sched, alloc, [0, 1, 2, 3], [], device="cpu")
    assert list(ref["preempted_reqs"]), "the scenario must preempt"
    _compare(ref, got, bs, False)
