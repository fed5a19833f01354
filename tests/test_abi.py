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


def test_grid_bound_from_the_context_sum_covers_every_pair():
    """The host-side sum of context lengths tightens the number of (sequence,
    partition) pairs a launch reserves.  The reservation is visible, without a
    GPU, in the workspace size of a batch large enough to need a pair table
    (16 bytes per reserved pair): for random batches it must never be smaller
    than the true number of pairs, and never looser than floor(sum / partition)
    + sequences (the table is rounded up to 256 bytes = 16 pairs)."""
    import numpy as np
    lib = _lib.attn()
    rng = np.random.Generator(np.random.PCG64(11))
    for partition in (64, 256, 512):
        for trial in range(20):
            B = 16 * int(rng.integers(17, 40))      # a multiple of 16: the loose table has no rounding pad
            hi = int(rng.choice([partition // 2, partition, 3 * partition, 2000]))
            ctx = rng.integers(0, hi + 1, size=B).astype(np.int64)
            it = _lib.MuxDecodeItem()
            it.num_seqs, it.num_q_heads, it.num_kv_heads = B, 4, 4
            it.num_layers, it.layer = 1, 0
            it.max_context_len = int(ctx.max())
            it.max_blocks = (it.max_context_len + 15) // 16
            it.total_context_len = 0
            loose = lib.mux_paged_decode_workspace_bytes(ctypes.addressof(it), 1, partition)
            it.total_context_len = int(ctx.sum())
            tight = lib.mux_paged_decode_workspace_bytes(ctypes.addressof(it), 1, partition)
            max_splits = max(1, -(-it.max_context_len // partition))
            reserved = B * max_splits - (loose - tight) // 16          # pairs reserved with the hint, rounded up to 16
            true_pairs = int((-(-ctx // partition)).sum())
            assert reserved >= true_pairs, (partition, trial, reserved, true_pairs)
            assert reserved <= min(B * max_splits, int(ctx.sum()) // partition + B) + 15
