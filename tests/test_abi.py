"""The two C-ABI libraries load without a GPU and export every entry point the
headers under include/ declare (no compute calls here)."""
import ctypes
import os
import re

import pytest

from muxserve_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DECL = re.compile(r"^\s*(?:[A-Za-z_][\w\s\*]*?)\b(mux_\w+)\s*\(", re.M)


def _declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)          # drop comments
    return sorted(set(DECL.findall(text)))


@pytest.mark.parametrize("header,loader,path", [
    ("muxserve_host.h", _lib.host, _lib.HOST_LIB_PATH),
    ("muxserve_attn.h", _lib.attn, _lib.ATTN_LIB_PATH),
])
def test_library_exports_every_declared_symbol(header, loader, path):
    names = _declared(header)
    assert len(names) >= 10, names
    lib = loader()
    raw = ctypes.CDLL(path)
    for n in names:
        assert hasattr(raw, n), f"{n} declared in include/{header} but not exported by {os.path.basename(path)}"
    # every declared symbol also has a typed binding
    typed = set(_lib.ATTN_SIGNATURES) if header == "muxserve_attn.h" else None
    if typed is not None:
        assert set(names) <= typed, sorted(set(names) - typed)
    assert lib is loader()      # cached handle


def test_version_and_error_entry_points_work_without_a_gpu():
    lib = _lib.attn()
    assert lib.mux_attn_version() >= 100
    assert lib.mux_last_hip_error() == 0


def test_missing_library_fails_loudly(tmp_path, monkeypatch):
    monkeypatch.setattr(_lib, "_attn", None)
    monkeypatch.setattr(_lib, "ATTN_LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(_lib.MuxLibraryMissing):
        _lib.attn()


def test_decode_rejects_malformed_arguments_on_the_host_side():
    """Validation happens before any launch, so it can be exercised without a GPU."""
    lib = _lib.attn()
    item = _lib.MuxDecodeItem()
    rc = lib.mux_multi_decode(ctypes.addressof(item), 1, 16, 16, 8, 128, 16, 0, 0, None, 0, None)
    assert rc == -1          # null q/out/tables
    rc = lib.mux_multi_decode(ctypes.addressof(item), 9, 16, 16, 8, 128, 16, 0, 0, None, 0, None)
    assert rc == -1          # too many items
    rc = lib.mux_reshape_and_cache(16, 16, 128, 16, 16, 8, 16, 0, 1, 4, 1, 64, 16, 0, None)
    assert rc == -2          # head size other than 128
    assert lib.mux_stream_create_cu_range(None, 0, 50, None) == -1


def test_torch_operator_library_loads_and_registers_every_operator():
    """libmuxtorch.so loads without a GPU, registers its operators with the
    dispatcher, and has no CPU kernels to fall back to."""
    import pytest
    import torch
    from muxserve_amd import torch_ops
    ns = torch_ops.load()
    for name in torch_ops.OPERATORS:
        assert hasattr(ns, name), name
        assert getattr(ns, name).default._schema.name == f"muxserve_amd::{name}"
    with pytest.raises((NotImplementedError, RuntimeError)):
        ns.silu_and_mul(torch.zeros((2, 16), dtype=torch.float16))


def test_bench_refuses_more_than_one_gpu():
    """bench.py is a one-GPU benchmark: --gpus N > 1 exits with a message
    before anything touches a device."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode == 2 and "one GPU" in r.stderr and r.stdout.strip() == ""


def test_workspace_size_does_not_depend_on_the_hint_and_host_pairs_are_exact():
    """The caller's bound on the sum of the context lengths sizes the grid of a
    device-enumerated launch and nothing else: the pair table of a large batch
    has a row for every pair the shapes allow, so a bound that is too small can
    not make the table too small.  The host-side enumeration (the pairs carried
    in the kernel argument) is exact: for random batches it counts one unit per
    started partition, less the remainders of at most 16 tokens, which ride on
    the unit before them."""
    import numpy as np
    lib = _lib.attn()
    rng = np.random.Generator(np.random.PCG64(11))
    for partition in (64, 256, 512):
        for trial in range(20):
            B = 16 * int(rng.integers(17, 40))
            hi = int(rng.choice([partition // 2, partition, 3 * partition, 2000]))
            ctx = rng.integers(0, hi + 1, size=B).astype(np.int32)
            it = _lib.MuxDecodeItem()
            it.num_seqs, it.num_q_heads, it.num_kv_heads = B, 4, 4
            it.num_layers, it.layer = 1, 0
            it.max_context_len = int(ctx.max())
            it.max_blocks = (it.max_context_len + 15) // 16
            sizes = set()
            for hint in (0, 1, int(ctx.sum()) // 2, int(ctx.sum()), 10 * int(ctx.sum())):
                it.total_context_len = hint
                sizes.add(lib.mux_paged_decode_workspace_bytes(ctypes.addressof(it), 1, partition))
            assert len(sizes) == 1, (partition, trial, sizes)
            max_splits = max(1, -(-it.max_context_len // partition))
            assert sizes.pop() >= (1 << 20) + B * max_splits * 16
    for partition in (64, 256):
        for trial in range(20):
            B = int(rng.integers(1, 40))
            ctx = rng.integers(0, 4 * partition, size=B).astype(np.int32)
            it = _lib.MuxDecodeItem()
            it.num_seqs, it.num_q_heads, it.num_kv_heads, it.num_layers = B, 2, 2, 1
            it.max_context_len = max(int(ctx.max()), 1)
            it.max_blocks = (it.max_context_len + 15) // 16
            it.context_lens_host = ctx.ctypes.data
            want = 0
            for c in ctx.tolist():
                fg, rem = divmod(c, partition)
                want += fg + (1 if rem > 0 and not (fg > 0 and rem <= 16) else 0)
            assert lib.mux_paged_decode_host_pairs(ctypes.addressof(it), 1, partition) == (want if want <= 384 else 0)


def test_library_chosen_partition_follows_the_size_of_the_launch():
    """With partition_size 0 the library picks the partition: 256 tokens, but
    1024 for a large launch (at least 1.5 M tokens x heads over its models, by
    the caller's bound on the context sum, or by half the longest context per
    sequence without one) and 512 beyond 4096-token contexts; for launches of
    grouped-query models only, a workgroup slot's share of the launch.  Seen through the
    unit count of the host-side enumeration; the workspace asked for is never
    smaller than what the 256-token partition needs, whichever is picked."""
    import numpy as np
    lib = _lib.attn()

    def units(ctx, partition):
        n = 0
        for c in ctx:
            fg, rem = divmod(int(c), partition)
            n += fg + (1 if rem > 0 and not (fg > 0 and rem <= 16) else 0)
        return n

    def item(B, heads, ctx_value, hint):
        ctx = np.full(B, ctx_value, dtype=np.int32)
        it = _lib.MuxDecodeItem()
        it.num_seqs, it.num_q_heads, it.num_kv_heads, it.num_layers = B, heads, heads, 1
        it.max_context_len = ctx_value
        it.max_blocks = (ctx_value + 15) // 16
        it.total_context_len = hint
        it.context_lens_host = ctx.ctypes.data
        return it, ctx

    # 128 sequences x 700 tokens x 32 heads = 2.9 M: long partitions, one unit per sequence
    it, ctx = item(128, 32, 700, 128 * 700)
    assert lib.mux_paged_decode_host_pairs(ctypes.addressof(it), 1, 0) == units(ctx, 1024) == 128
    big = lib.mux_paged_decode_workspace_bytes(ctypes.addressof(it), 1, 0)
    assert big == lib.mux_paged_decode_workspace_bytes(ctypes.addressof(it), 1, 256)
    assert big >= lib.mux_paged_decode_workspace_bytes(ctypes.addressof(it), 1, 1024)
    # the same batch without the bound: 128 x 350 x 32 = 1.4 M, below the line
    it, ctx = item(128, 32, 700, 0)
    assert lib.mux_paged_decode_host_pairs(ctypes.addressof(it), 1, 0) == units(ctx, 256) == 128 * 3
    # a small batch keeps the short partitions
    it, ctx = item(8, 32, 700, 8 * 700)
    assert lib.mux_paged_decode_host_pairs(ctypes.addressof(it), 1, 0) == units(ctx, 256) == 24
    # the sizes of the models of one launch add up: 2 x (64 x 700 x 32) = 2.9 M
    pair = (_lib.MuxDecodeItem * 2)()
    keep = []
    for k in range(2):
        one, c = item(64, 32, 700, 64 * 700)
        keep.append(c)
        pair[k] = one
    assert lib.mux_paged_decode_host_pairs(ctypes.addressof(pair), 2, 0) == 2 * 64
    for k in range(2):
        pair[k].total_context_len = 0          # 2 x (64 x 350 x 32) = 1.4 M
    assert lib.mux_paged_decode_host_pairs(ctypes.addressof(pair), 2, 0) == 2 * 64 * 3
    # contexts beyond 4096 tokens: 512-token partitions for the vector-ALU kernel
    it, ctx = item(4, 32, 5000, 4 * 5000)
    assert lib.mux_paged_decode_host_pairs(ctypes.addressof(it), 1, 0) == units(ctx, 512)

    # Grouped-query launches (8 query heads per kv head): a workgroup slot's share of the launch -
    # tokens x kv heads / (3 x 256 slots), rounded up to 256 tokens, never under 256.
    def gqa_item(B, ctx_value, hint):
        it, ctx = item(B, 64, ctx_value, hint)
        it.num_kv_heads = 8
        return it, ctx

    it, ctx = gqa_item(64, 5120, 64 * 5120)          # 64 x 5120 x 8 / 768 = 3413 -> 3584 tokens
    assert lib.mux_paged_decode_host_pairs(ctypes.addressof(it), 1, 0) == units(ctx, 3584) == 2 * 64
    it, ctx = gqa_item(16, 5120, 16 * 5120)          # 853 -> 1024
    assert lib.mux_paged_decode_host_pairs(ctypes.addressof(it), 1, 0) == units(ctx, 1024) == 5 * 16
    it, ctx = gqa_item(2, 5120, 2 * 5120)            # 107 -> 256: a small launch is spread over many units
    assert lib.mux_paged_decode_host_pairs(ctypes.addressof(it), 1, 0) == units(ctx, 256) == 20 * 2
    it, ctx = gqa_item(256, 1000, 256 * 1000)        # 2667 -> 2816: beyond every context, nothing is split
    assert lib.mux_paged_decode_host_pairs(ctypes.addressof(it), 1, 0) == 256
    big = lib.mux_paged_decode_workspace_bytes(ctypes.addressof(it), 1, 0)
    assert big == lib.mux_paged_decode_workspace_bytes(ctypes.addressof(it), 1, 256)
    it, ctx = gqa_item(64, 5120, 0)                  # no bound: half the longest context each, 1707 -> 1792
    assert lib.mux_paged_decode_host_pairs(ctypes.addressof(it), 1, 0) == units(ctx, 1792) == 3 * 64


# ---------------------------------------------------------------------------
# Every entry point of include/muxserve_attn.h called once with well-formed
# arguments.  No device is present where this runs, so nothing can be launched:
# each call has to come back with a return code - MUXA_EHIP where it got as far
# as the HIP runtime, MUXA_OK where the host side had nothing to launch, a byte
# or pair count for the sizing helpers - and never crash the host on the way
# (an uninitialised field of a descriptor built inside the library once did).
# "Device" pointers are made-up aligned addresses: the host side must not
# dereference them.  Host arrays (context_lens_host, prompt_lens_host, the
# descriptor arrays, output words) are real.
# ---------------------------------------------------------------------------
def _call_table():
    import numpy as np
    P = lambda k: 0x7F0000000000 + 0x100000 * k          # noqa: E731  fake, 1 MiB apart, 16-byte aligned
    keep = []
    ctx_host = np.array([5, 200, 300, 17], dtype=np.int32)
    keep.append(ctx_host)

    def decode_items(n=1, host=True):
        arr = (_lib.MuxDecodeItem * n)()
        for it in arr:
            it.out, it.q, it.out_row_stride, it.q_row_stride = P(1), P(2), 4 * 128, 4 * 128
            it.block_tables, it.context_lens = P(3), P(4)
            it.total_context_len, it.layer, it.num_layers, it.num_seqs = 522, 0, 1, 4
            it.num_q_heads, it.num_kv_heads, it.max_blocks, it.max_context_len, it.scale = 4, 4, 19, 300, 0.088
            it.context_lens_host = ctx_host.ctypes.data if host else None
        keep.append(arr)
        return ctypes.addressof(arr)

    lens = (ctypes.c_int32 * 2)(40, 9)
    pit = (_lib.MuxPrefillItem * 1)()
    pit[0].out, pit[0].out_row_stride, pit[0].q, pit[0].q_row_stride = P(1), 512, P(2), 512
    pit[0].k, pit[0].v, pit[0].kv_row_stride, pit[0].cu_seqlens = P(3), P(4), 512, P(5)
    pit[0].prompt_lens_host, pit[0].num_prompts, pit[0].max_prompt_len = ctypes.addressof(lens), 2, 40
    pit[0].num_q_heads, pit[0].num_kv_heads, pit[0].scale = 4, 4, 0.088
    cw = (_lib.MuxCacheWriteItem * 1)()
    cw[0].k, cw[0].v, cw[0].kv_row_stride, cw[0].slot_mapping = P(3), P(4), 512, P(6)
    cw[0].layer, cw[0].num_layers, cw[0].num_tokens, cw[0].num_kv_heads = 0, 1, 8, 4
    words = (ctypes.c_uint32 * 8)()
    info = (ctypes.c_int32 * 2)()
    sout = ctypes.c_void_p()
    ncu = ctypes.c_int32()
    keep += [lens, pit, cw, words, info, sout, ncu]
    ws = 1 << 22
    table = {
        "mux_attn_version": lambda f: f(),
        "mux_last_hip_error": lambda f: f(),
        "mux_reshape_and_cache": lambda f: f(P(3), P(4), 512, P(7), P(8), 64, P(6), 0, 1, 8, 4, 128, 16, 0, None),
        "mux_paged_decode_workspace_bytes": lambda f: f(decode_items(2), 2, 0),
        "mux_paged_decode_host_pairs": lambda f: f(decode_items(2), 2, 0),
        "mux_paged_decode_workspace_init": lambda f: f(P(9), ws, None),
        "mux_multi_decode": lambda f: f(decode_items(2), 2, P(7), P(8), 64, 128, 16, 0, 0, P(9), ws, None),
        "mux_multi_decode_noalloc_max_bytes": lambda f: f(),
        "mux_multi_decode_noalloc": lambda f: f(decode_items(2, host=False), 2, P(7), P(8), 64, 128, 16, 0, 0, None),
        "mux_paged_decode": lambda f: f(P(1), 512, P(2), 512, P(7), P(8), 64, P(3), P(4), 0, 1, 4, 4, 4, 128, 16, 19,
                                        300, 0.088, 0, 0, P(9), ws, None),
        "mux_prefill_causal": lambda f: f(P(1), 512, P(2), 512, P(3), P(4), 512, P(5), None, ctypes.addressof(lens), 2,
                                          40, 4, 4, 128, 0.088, 0, None),
        "mux_multi_prefill_causal": lambda f: f(ctypes.addressof(pit), 1, 128, 0, None),
        "mux_rotary_neox": lambda f: f(P(5), P(2), 512, P(3), 512, P(6), 4096, 128, 8, 4, 4, 128, 0, None),
        "mux_rope_reshape_and_cache": lambda f: f(P(5), P(2), 512, P(3), P(4), 512, P(6), 4096, 128, P(7), P(8), 64,
                                                  P(10), 0, 1, 8, 4, 4, 128, 16, 0, None),
        "mux_multi_rope_reshape_and_cache": lambda f: f(ctypes.addressof(cw), 1, P(7), P(8), 64, 128, 16, 0, None),
        "mux_rms_norm": lambda f: f(P(1), 4096, P(2), 4096, P(3), 1e-6, 8, 4096, 0, None),
        "mux_silu_and_mul": lambda f: f(P(1), 1024, P(2), 2048, 8, 1024, 0, None),
        "mux_greedy_sample_workspace_bytes": lambda f: f(32000),
        "mux_greedy_sample_workspace_init": lambda f: f(P(9), ws, None),
        "mux_greedy_sample": lambda f: f(P(1), P(2), 4096, 8, None, 8, P(3), 4096, 32000, 32000, 4096, 0, P(9), ws,
                                         None),
        "mux_build_step_inputs": lambda f: f(P(1), 8, 16, 2, 4, 16, P(2), 4, P(3), 40, 1, 4, P(4), P(5), 16, None),
        "mux_cu_parts_mask": lambda f: f(0b1001, 256, ctypes.addressof(words), 8),
        "mux_stream_create_cu_parts": lambda f: f(ctypes.byref(sout), 0b11, ctypes.byref(ncu)),
        "mux_stream_create_cu_range": lambda f: f(ctypes.byref(sout), 0, 40, ctypes.byref(ncu)),
        "mux_stream_destroy": lambda f: f(None),
        "mux_device_cu_info": lambda f: f(ctypes.addressof(info)),
    }
    return table, keep


def test_every_attn_entry_point_returns_a_code_when_called_without_a_device():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a device is present: the made-up device pointers of this test must not reach a kernel")
    lib = _lib.attn()
    table, keep = _call_table()
    assert set(table) == set(_declared("muxserve_attn.h")), sorted(set(table) ^ set(_declared("muxserve_attn.h")))
    sizes = {"mux_paged_decode_workspace_bytes", "mux_multi_decode_noalloc_max_bytes",
             "mux_greedy_sample_workspace_bytes"}
    got = {}
    for name, call in table.items():
        got[name] = call(getattr(lib, name))
    assert got["mux_attn_version"] >= 300
    assert got["mux_paged_decode_host_pairs"] == 2 * 5          # per item: 300 -> 256 + 44, plus 5, 200, 17
    assert got["mux_cu_parts_mask"] > 0
    for name in sizes:
        assert got[name] > 0, name
    launches = set(table) - sizes - {"mux_attn_version", "mux_last_hip_error", "mux_paged_decode_host_pairs",
                                     "mux_cu_parts_mask", "mux_stream_destroy"}
    for name in sorted(launches):
        assert got[name] == -4, f"{name} returned {got[name]}, expected MUXA_EHIP (no device)"
    assert lib.mux_last_hip_error() != 0
    del keep


def test_single_model_decode_wrapper_equals_the_fused_entry_point_on_its_arguments():
    """mux_paged_decode is mux_multi_decode on one descriptor whose optional
    fields are absent: both must reject and accept the same calls."""
    import torch
    if torch.cuda.is_available():
        pytest.skip("made-up device pointers")
    lib = _lib.attn()
    P = 0x7F0000000000
    for max_ctx, max_blocks, want in ((300, 19, -4), (300, 18, -1), (0, 0, 0)):
        rc = lib.mux_paged_decode(P, 512, P + 4096, 512, P + 8192, P + 16384, 64, P + 32768, P + 65536, 0, 1, 4, 4, 4,
                                  128, 16, max_blocks, max_ctx, 0.088, 0, 0, P + (1 << 20), 1 << 22, None)
        assert rc == want, (max_ctx, max_blocks, rc)
