"""The compact step (get_batch_compact + the device-side builder) against the
reference-shaped step (get_batch), on the host: descriptors are replayed with a
numpy restatement of the three device kernels and must reproduce the oracle's
slot_mapping and block table exactly, through prefill, decode across block
boundaries, release and row reuse, and allocator preemption."""
import numpy as np
import pytest
import torch

from oracle import host_oracle
from muxserve_amd.batch_scheduler import BatchScheduler
from muxserve_amd.memory_manager import KVStorage

D = BatchScheduler.STEP_DESC_INTS


class NumpyMirror:
    """What mux_build_step_inputs does, in numpy."""

    def __init__(self, rows, max_blocks, L, H, bs):
        self.m = np.zeros((rows, max_blocks, L * H), dtype=np.int32)
        self.L, self.H, self.bs = L, H, bs

    def build(self, desc, block_info, num_tokens, max_blocks_out):
        per = self.L * self.H
        for d in desc:
            row, nblk, first, new, off = (int(x) for x in d[:5])
            self.m[row, first:first + new] = block_info[off:off + new * per].reshape(new, per)
        slots = np.zeros((num_tokens, per), dtype=np.int64)
        for d in desc:
            row, nblk, _, _, _, length, t0, dec = (int(x) for x in d)
            if dec:
                slots[t0] = self.m[row, nblk - 1].astype(np.int64) * self.bs + (length - 1) % self.bs
            else:
                for k in range(length):
                    slots[t0 + k] = self.m[row, k // self.bs].astype(np.int64) * self.bs + k % self.bs
        tables = None
        if max_blocks_out > 0:
            tables = np.zeros((self.L, len(desc), self.H, max_blocks_out), dtype=np.int32)
            for c, d in enumerate(desc):
                nblk = int(d[1])
                tables[:, c, :, :nblk] = self.m[int(d[0]), :nblk].reshape(nblk, self.L, self.H).transpose(1, 2, 0)
        return slots.reshape(num_tokens, self.L, self.H), tables


def _compact_step(sched, storage, mirror, L, H, ids, last):
    info = sched.try_batch(list(ids), list(last))
    req = np.ascontiguousarray(info[:-1])
    block_info = (np.asarray(storage.allocate_batch(req, L, H), dtype=np.int32) if int(info[-1]) > 0
                  else np.array([len(ids)], dtype=np.int32))
    bi = sched.get_batch_info(req, block_info)
    T, C, max_ctx, max_blk = bi[:4]
    pad = (T + 7) // 8 * 8
    tok, pos = torch.full((pad,), -7, dtype=torch.int32), torch.full((pad,), -7, dtype=torch.int32)
    ctx = torch.full((C,), -7, dtype=torch.int32)
    n = max(int(block_info[0]), 0)
    desc = torch.full((n, D), -7, dtype=torch.int32)
    sched.get_batch_compact(req, block_info, tok, pos, ctx, desc)
    slots, tables = mirror.build(desc.numpy(), block_info, T, max_blk if max_ctx > 0 else 0)
    return {"tok": tok.long(), "pos": pos.long(), "ctx": ctx, "slots": slots, "tables": tables, "desc": desc.numpy(),
            "batch_reqs": sched.get_batch_reqs(), "preempted": sched.get_preempt_requests(),
            "prompt_info": sched.get_prompt_info()}


def _same(ref, got, bs):
    assert torch.equal(ref["input_tensor"], got["tok"]) and torch.equal(ref["input_positions"], got["pos"])
    assert torch.equal(ref["context_lens"], got["ctx"])
    assert np.array_equal(ref["slot_mapping"].numpy(), got["slots"])
    assert ref["batch_reqs"] == got["batch_reqs"] and ref["preempted_reqs"] == got["preempted"]
    if ref["max_context_len"] > 0:
        rt = ref["block_tables"].numpy()
        for c, n_ctx in enumerate(ref["context_lens"].tolist()):
            valid = (n_ctx + bs - 1) // bs
            assert np.array_equal(rt[:, c, :, :valid], got["tables"][:, c, :, :valid])
            assert (got["tables"][:, c, :, valid:] == 0).all()
    else:
        assert got["tables"] is None


@pytest.mark.parametrize("L,H,bs", [(2, 3, 16), (1, 1, 8), (4, 2, 32)])
def test_compact_step_reproduces_the_reference_step(L, H, bs):
    rng = np.random.Generator(np.random.PCG64(L * 100 + H))
    N = 4000
    ref_store, ref_sched = host_oracle.KVStorage(N), host_oracle.BatchScheduler(L, H, 512, bs)
    store, sched = KVStorage(N), BatchScheduler(L, H, 512, bs)
    sched.enable_device_rows(6)
    mirror = NumpyMirror(6, sched.max_blocks_per_seq, L, H, bs)
    lens = [5, bs, bs + 1, 3 * bs - 1, 1]
    for i, p in enumerate(lens):
        prompt = rng.integers(0, 1000, size=p).astype(np.int32)
        ref_sched.add_request(prompt, i, 64)
        sched.add_request(prompt, i, 64)
    ids = list(range(len(lens)))
    _same(host_oracle.prepare_inputs(ref_sched, ref_store, L, H, ids, []),
          _compact_step(sched, store, mirror, L, H, ids, []), bs)
    order = [3, 0, 4, 1, 2]
    for step in range(2 * bs + 3):                       # every sequence crosses block boundaries
        last = [100 + step] * 5
        got = _compact_step(sched, store, mirror, L, H, order, last)
        _same(host_oracle.prepare_inputs(ref_sched, ref_store, L, H, order, last), got, bs)
        assert sorted(int(d[0]) for d in got["desc"]) == [0, 1, 2, 3, 4]        # rows are stable
    # two requests finish; their rows are reused by new requests
    for s_, st_ in ((ref_sched, ref_store), (sched, store)):
        st_.free_batch([1, 3])
        s_.release_requests([1, 3])
    for rid, p in ((10, 2 * bs), (11, 7), (12, 9)):
        prompt = rng.integers(0, 1000, size=p).astype(np.int32)
        ref_sched.add_request(prompt, rid, 64)
        sched.add_request(prompt, rid, 64)
    got = _compact_step(sched, store, mirror, L, H, [10, 11, 12], [])
    _same(host_oracle.prepare_inputs(ref_sched, ref_store, L, H, [10, 11, 12], []), got, bs)
    assert sorted(int(d[0]) for d in got["desc"]) == [1, 3, 5]
    for step in range(bs + 2):
        idsd = [0, 10, 2, 11, 4, 12]
        last = [7] * 6
        _same(host_oracle.prepare_inputs(ref_sched, ref_store, L, H, idsd, last),
              _compact_step(sched, store, mirror, L, H, idsd, last), bs)
    with pytest.raises(MemoryError):                     # a seventh live request finds no row
        sched.add_request(np.arange(3, dtype=np.int32), 99, 8)
        _compact_step(sched, store, mirror, L, H, [99], [])


def test_compact_step_with_allocator_preemption():
    """A pool too small for the batch: the allocator cuts the batch, the cut
    requests are forgotten and their rows come back."""
    L, H, bs = 2, 2, 16
    per = L * H
    N = 9 * per                                          # room for 9 token blocks in all
    ref_store, ref_sched = host_oracle.KVStorage(N), host_oracle.BatchScheduler(L, H, 256, bs)
    store, sched = KVStorage(N), BatchScheduler(L, H, 256, bs)
    sched.enable_device_rows(4)
    mirror = NumpyMirror(4, sched.max_blocks_per_seq, L, H, bs)
    for i, p in enumerate([3 * bs, 3 * bs, 2 * bs + 5, 2 * bs]):
        prompt = np.arange(p, dtype=np.int32)
        ref_sched.add_request(prompt, i, 32)
        sched.add_request(prompt, i, 32)
    ref = host_oracle.prepare_inputs(ref_sched, ref_store, L, H, [0, 1, 2, 3], [])
    got = _compact_step(sched, store, mirror, L, H, [0, 1, 2, 3], [])
    assert ref["preempted_reqs"] and ref["preempted_reqs"] == got["preempted"]
    _same(ref, got, bs)
    alive = [r for r in [0, 1, 2, 3] if r not in ref["preempted_reqs"]]
    for step in range(bs + 1):                           # decode until the pool runs dry again
        last = [5] * len(alive)
        ref = host_oracle.prepare_inputs(ref_sched, ref_store, L, H, alive, last)
        got = _compact_step(sched, store, mirror, L, H, alive, last)
        _same(ref, got, bs)
        alive = [r for r in alive if r not in ref["preempted_reqs"]]
        if not alive:
            break
    assert sched.num_requests() == ref_sched.num_requests() if hasattr(ref_sched, "num_requests") else True


def test_compact_step_needs_rows_enabled():
    sched = BatchScheduler(1, 1, 64, 16)
    sched.add_request(np.arange(4, dtype=np.int32), 0, 4)
    store = KVStorage(64)
    info = sched.try_batch([0], [])
    req = np.ascontiguousarray(info[:-1])
    blk = store.allocate_batch(req, 1, 1)
    sched.get_batch_info(req, blk)
    with pytest.raises(ValueError):
        sched.get_batch_compact(req, blk, torch.zeros(8, dtype=torch.int32), torch.zeros(8, dtype=torch.int32),
                                torch.zeros(0, dtype=torch.int32), torch.zeros((1, D), dtype=torch.int32))
