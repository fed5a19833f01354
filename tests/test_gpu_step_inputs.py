"""prepare_inputs with the device-side builder (DeviceBlockTables) against
prepare_inputs on the reference-shaped host path and against the oracle's
restatement of the reference's prepare_inputs: the same scenario is driven
through three scheduler/allocator pairs in lockstep and every tensor the model
code receives must be bit-identical (block-table entries the reference leaves
undefined excepted)."""
import numpy as np
import pytest
import torch

from oracle import host_oracle
from muxserve_amd.batch_scheduler import BatchScheduler
from muxserve_amd.device_tables import DeviceBlockTables
from muxserve_amd.memory_manager import KVStorage
from muxserve_amd.prepare import prepare_inputs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _pair(L, H, bs, N, rows, max_seq_len=1024):
    a = (KVStorage(N), BatchScheduler(L, H, max_seq_len, bs))
    b = (KVStorage(N), BatchScheduler(L, H, max_seq_len, bs))
    dt = DeviceBlockTables(b[1], rows, DEV)
    _ORACLE[id(dt)] = (host_oracle.KVStorage(N), host_oracle.BatchScheduler(L, H, max_seq_len, bs))
    return a, b, dt


_ORACLE = {}       # the oracle's allocator and batch builder that shadow a pair


def _oracle_do(dt, fn):
    st, sc = _ORACLE[id(dt)]
    fn(st, sc)


def _against_oracle(ref, got, bs):
    """The device-built step against the oracle's reference-shaped tensors."""
    tok, pos, md, batch_reqs, preempted = got
    T = sum(ref["prompt_lens"]) + int(ref["context_lens"].numel())
    assert tok.dtype == torch.int64 and tok.shape == ref["input_tensor"].shape
    assert torch.equal(tok.cpu()[:T], ref["input_tensor"][:T]) and torch.equal(pos.cpu()[:T], ref["input_positions"][:T])
    assert md.slot_mapping.dtype == torch.int64 and torch.equal(md.slot_mapping.cpu(), ref["slot_mapping"])
    assert md.context_lens.dtype == torch.int32 and torch.equal(md.context_lens.cpu(), ref["context_lens"])
    assert md.max_context_len == ref["max_context_len"] and md.prompt_lens == [int(x) for x in ref["prompt_lens"]]
    assert [list(x) for x in batch_reqs] == [list(x) for x in ref["batch_reqs"]]
    assert list(preempted) == list(ref["preempted_reqs"])
    if ref["max_context_len"] > 0:
        rt, gt = ref["block_tables"], md.block_tables.cpu()
        assert gt.shape == rt.shape and gt.dtype == torch.int32
        for c, n in enumerate(ref["context_lens"].tolist()):
            valid = (n + bs - 1) // bs
            assert torch.equal(gt[:, c, :, :valid], rt[:, c, :, :valid]), f"sequence {c}"
    else:
        assert md.block_tables.numel() == 0 and ref["block_tables"].numel() == 0


def _both(a, b, dt, L, H, ids, last, bs):
    ra = prepare_inputs(a[1], lambda r: a[0].allocate_batch(r, L, H), ids, last, DEV, permuted_tables=False)
    rb = prepare_inputs(b[1], lambda r: b[0].allocate_batch(r, L, H), ids, last, DEV, device_tables=dt)
    torch.cuda.synchronize()
    ost, osc = _ORACLE[id(dt)]
    _against_oracle(host_oracle.prepare_inputs(osc, ost, L, H, ids, last), rb, bs)
    (ta, pa, ma, qa, ea), (tb, pb, mb, qb, eb) = ra, rb
    assert torch.equal(ta, tb) and torch.equal(pa, pb) and qa == qb and ea == eb
    assert ma.prompt_lens == mb.prompt_lens and ma.max_context_len == mb.max_context_len
    assert ma.total_context_len == mb.total_context_len
    assert torch.equal(ma.context_lens, mb.context_lens)
    assert ma.slot_mapping.shape == mb.slot_mapping.shape and torch.equal(ma.slot_mapping, mb.slot_mapping)
    if ma.max_context_len > 0:
        assert ma.block_tables.shape == mb.block_tables.shape
        xa, xb = ma.block_tables.cpu(), mb.block_tables.cpu()
        for c, n in enumerate(ma.context_lens.cpu().tolist()):
            valid = (n + bs - 1) // bs
            assert torch.equal(xa[:, c, :, :valid], xb[:, c, :, :valid]), f"sequence {c}"
    else:
        assert mb.block_tables.numel() == 0
    return ea


@pytest.mark.parametrize("L,H,bs", [(2, 4, 16), (32, 32, 16), (3, 5, 8), (60, 52, 16), (1, 1, 32)])
def test_device_built_step_inputs_equal_the_host_built_ones(L, H, bs):
    print(f"[case] device step inputs L={L} H={H} bs={bs}", flush=True)
    rng = np.random.Generator(np.random.PCG64(L + H))
    lens = [int(x) for x in rng.integers(1, 200, size=7)] + [bs, 2 * bs + 1]
    N = (sum((n + 40) // bs + 2 for n in lens)) * L * H + 256
    a, b, dt = _pair(L, H, bs, N, rows=12)
    for i, p in enumerate(lens):
        prompt = rng.integers(0, 32000, size=p).astype(np.int32)
        a[1].add_request(prompt, i, 64)
        b[1].add_request(prompt, i, 64)
        _oracle_do(dt, lambda st, sc: sc.add_request(prompt, i, 64))
    ids = list(range(len(lens)))
    _both(a, b, dt, L, H, ids[:5], [], bs)                         # two prefill steps
    _both(a, b, dt, L, H, ids[5:], [], bs)
    for step in range(bs + 3):                                      # decode across block boundaries
        order = ids[::-1] if step % 2 else ids
        _both(a, b, dt, L, H, order, [step + 1] * len(ids), bs)
    for st, sc in (a, b, _ORACLE[id(dt)]):                          # release, then new requests reuse rows
        st.free_batch([0, 4, 8])
        sc.release_requests([0, 4, 8])
    for rid, p in ((20, 33), (21, 1), (22, 3 * bs)):
        prompt = rng.integers(0, 32000, size=p).astype(np.int32)
        a[1].add_request(prompt, rid, 64)
        b[1].add_request(prompt, rid, 64)
        _oracle_do(dt, lambda st, sc: sc.add_request(prompt, rid, 64))
    _both(a, b, dt, L, H, [20, 21, 22], [], bs)
    live = [1, 2, 3, 5, 6, 7, 20, 21, 22]
    for step in range(4):
        _both(a, b, dt, L, H, live, [9] * len(live), bs)


def test_device_built_step_inputs_with_preemption():
    print("[case] device step inputs, preemption", flush=True)
    L, H, bs = 2, 2, 16
    N = 10 * L * H
    a, b, dt = _pair(L, H, bs, N, rows=4, max_seq_len=256)
    for i, p in enumerate([3 * bs, 3 * bs, 2 * bs + 5, 2 * bs]):
        prompt = np.arange(p, dtype=np.int32)
        a[1].add_request(prompt, i, 32)
        b[1].add_request(prompt, i, 32)
        _oracle_do(dt, lambda st, sc: sc.add_request(prompt, i, 32))
    cut = _both(a, b, dt, L, H, [0, 1, 2, 3], [], bs)
    assert cut, "the pool was meant to be too small for the batch"
    alive = [r for r in [0, 1, 2, 3] if r not in cut]
    for step in range(2 * bs):
        cut = _both(a, b, dt, L, H, alive, [3] * len(alive), bs)
        alive = [r for r in alive if r not in cut]
        if not alive:
            break


def test_descriptors_that_do_not_fit_are_skipped():
    """Descriptors pointing outside the mirror or the reply (row, block count,
    first new block, reply offset, sums that wrap in 32 bits) leave the mirror,
    the slots of their tokens and their table rows alone; the one well-formed
    descriptor among them is still carried out."""
    print("[case] device step inputs, malformed descriptors", flush=True)
    from muxserve_amd import _lib
    L, H, bs, rows, max_blk = 2, 3, 16, 4, 8
    per = L * H
    big = 2 ** 31 - 1
    mirror = torch.full((rows, max_blk, L, H), -7, dtype=torch.int32, device=DEV)
    reply = torch.arange(100, 100 + 1 + 2 * per, dtype=torch.int32)       # [preempt idx | 2 blocks of ids]
    # row, blocks, first new, new, reply offset, length, first token, decoding
    desc = torch.tensor([
        [rows, 1, 0, 1, 1, 5, 0, 0],            # row outside the mirror
        [0, max_blk + 1, 0, 1, 1, 5, 5, 0],     # more blocks than a row holds
        [0, 2, big, 1, 1, 5, 10, 0],            # first new + new wraps around
        [0, 2, 0, 2, 1 + per, 5, 15, 0],        # reply too short for the new blocks
        [0, 2, 1, 2, 1, 5, 20, 0],              # new blocks reach past the run
        [1, 2, 0, 2, 1, 20, 25, 0],             # well-formed: 20 prompt tokens, 2 new blocks
        [0, 1, 0, 0, 1, -3, 45, 1],             # negative length
    ], dtype=torch.int32)
    num_tokens = 50
    slots = torch.full((num_tokens, L, H), -1, dtype=torch.int64, device=DEV)
    tables = torch.full((L, desc.shape[0], H, max_blk), -9, dtype=torch.int32, device=DEV)
    d_desc, d_reply = desc.to(DEV), reply.to(DEV)
    rc = _lib.attn().mux_build_step_inputs(
        mirror.data_ptr(), rows, max_blk, L, H, bs, d_desc.data_ptr(), desc.shape[0], d_reply.data_ptr(),
        reply.numel(), 2, num_tokens, slots.data_ptr(), tables.data_ptr(), max_blk,
        torch.cuda.current_stream().cuda_stream)
    _lib.check_attn(rc, "mux_build_step_inputs")
    torch.cuda.synchronize()
    want_mirror = torch.full((rows, max_blk, L, H), -7, dtype=torch.int32)
    want_mirror[1, :2] = reply[1:].view(2, L, H)
    assert torch.equal(mirror.cpu(), want_mirror)
    want_slots = torch.full((num_tokens, L, H), -1, dtype=torch.int64)
    for k in range(20):
        want_slots[25 + k] = want_mirror[1, k // bs].long() * bs + k % bs
    assert torch.equal(slots.cpu(), want_slots)
    # no descriptor here is a decode step: every table row is defined and empty
    assert (tables.cpu() == 0).all()
