import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    """GPU tests are skipped, not failed, where no GPU is visible."""
    try:
        import torch
        has_gpu = torch.cuda.is_available()
    except Exception:   # pragma: no cover
        has_gpu = False
    if has_gpu:
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


_SESSION_POOL_BYTES = 0


@pytest.fixture(scope="session")
def full_size_pool_memory():
    """One raw allocation for every test that needs a pool of the benchmark's
    real size (185 GB fp16 for the mixed three-model decode, 200 GB bf16 for the
    long-context one): two 100 GB byte buffers, made once per test session and
    viewed by each such test as its K and V pools.  The suite therefore never
    frees and re-requests most of the device's memory between tests (a test run
    once crashed on the host inside torch's free-everything-and-retry path of
    such an allocation).  Returns view(num_blocks, block_size, dtype) ->
    (k_pool, v_pool)."""
    global _SESSION_POOL_BYTES
    import torch
    from muxserve_amd.pool import block_bytes, key_block_shape, value_block_shape
    half = int(200e9) // 2 // 4096 * 4096
    raw_k = torch.empty((half,), dtype=torch.uint8, device="cuda:0")
    raw_v = torch.empty((half,), dtype=torch.uint8, device="cuda:0")
    _SESSION_POOL_BYTES = 2 * half

    def view(num_blocks, block_size, dtype):
        nbytes = num_blocks * block_bytes(block_size) // 2
        assert nbytes <= half, "pool larger than the session's buffers"
        k = raw_k[:nbytes].view(dtype).view(num_blocks, *key_block_shape(block_size))
        v = raw_v[:nbytes].view(dtype).view(num_blocks, *value_block_shape(block_size))
        return k, v

    yield view
    del raw_k, raw_v
    _SESSION_POOL_BYTES = 0


@pytest.fixture(autouse=True)
def _return_large_caches_to_the_device(request):
    """Other large allocations of a GPU test (beyond the session's pool buffers)
    are handed back to the device after the test, so that no later allocation is
    made on the edge of the device's memory."""
    yield
    if "gpu" in request.keywords:
        import torch
        if torch.cuda.is_available() and torch.cuda.memory_reserved() - _SESSION_POOL_BYTES > (16 << 30):
            torch.cuda.synchronize()
            torch.cuda.empty_cache()
