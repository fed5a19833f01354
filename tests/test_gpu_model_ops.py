"""RMSNorm, SiluAndMul and the greedy sampler on the GPU, through the C ABI,
against oracle/layer_oracle.py.

Tolerances.  rms_norm and silu_and_mul round twice to the storage type T; the
GPU's reciprocal square root / exponential are accurate to about one fp32 ulp,
which can move the first-stage value across a rounding boundary of T, so
results must agree with the oracle within one such step (1 ulp of the result
plus |factor| x 1 ulp of the first-stage value) and exactly almost everywhere.  The
sampler is an index: it must be the oracle's token whenever the best logit
leads the runner-up by more than 2 ulp of T, and otherwise one whose exact
logit is within 2 ulp of the best."""
import numpy as np
import pytest
import torch

from oracle import layer_oracle as lo
from muxserve_amd import ops
from muxserve_amd.attention import InputMetadata
from muxserve_amd.layers import GreedySampler, RMSNorm, SiluAndMul

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _ulp(t, dtype):
    bits = 10 if dtype == torch.float16 else 7
    tiny = 2.0 ** -14 if dtype == torch.float16 else 2.0 ** -126
    mag = torch.clamp(t.abs().double(), min=tiny)
    return torch.pow(2.0, torch.floor(torch.log2(mag)) - bits)


def _close_in_ulps(got, want, dtype, what, first=None, factor=None):
    """Both operators round a first-stage value to T and multiply it by a
    factor: a first-stage value that lands one ulp away moves the product by
    |factor| ulp(first), on top of the product's own rounding."""
    got, want = got.double(), want.double()
    diff = (got - want).abs()
    tol = 1.001 * _ulp(want, dtype)
    if first is not None:
        tol = tol + factor.double().abs() * _ulp(first.double(), dtype)
    assert (diff <= tol).all(), f"{what}: beyond one rounding step (max {diff.max().item():.3e})"
    assert (diff == 0).double().mean().item() > 0.98, f"{what}: too many values differ from the oracle"


def _normalised(x, eps):
    xd = x.double()
    return xd / torch.sqrt((xd * xd).mean(-1, keepdim=True) + eps)


def _silu(x):
    a = x[:, :x.shape[1] // 2].double()
    return a / (1 + torch.exp(-a))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("T,hidden", [(1, 4096), (56, 4096), (300, 5120), (7, 6656), (33, 8192), (5, 128),
                                      (9, 16384), (4, 8000)])
def test_rms_norm(dtype, T, hidden):
    print(f"[case] rms_norm {dtype} T={T} hidden={hidden}", flush=True)
    g = torch.Generator().manual_seed(T * 7 + hidden)
    x = (torch.randn((T, hidden), generator=g) * 2).to(dtype)
    w = (1 + 0.3 * torch.randn((hidden,), generator=g)).to(dtype)
    got = ops.rms_norm(x.to(DEV), w.to(DEV), 1e-5)
    torch.cuda.synchronize()
    _close_in_ulps(got.cpu(), lo.rms_norm(x, w, 1e-5), dtype, "rms_norm", _normalised(x, 1e-5), w)


def test_rms_norm_strided_rows_padding_rows_and_module():
    print("[case] rms_norm strided", flush=True)
    g = torch.Generator().manual_seed(5)
    wide = torch.randn((24, 3 * 4096), generator=g).half()
    w = torch.randn((4096,), generator=g).half()
    dx = wide.to(DEV)[:, 4096:8192]                    # a column slice: row stride 3 * hidden
    out = torch.full((24, 4096), 7.0, dtype=torch.float16, device=DEV)
    ops.rms_norm(dx, w.to(DEV), 1e-6, out=out, num_tokens=21)
    torch.cuda.synchronize()
    xs = wide[:21, 4096:8192]
    _close_in_ulps(out[:21].cpu(), lo.rms_norm(xs, w, 1e-6), torch.float16, "rms_norm strided", _normalised(xs, 1e-6), w)
    assert (out[21:] == 7.0).all(), "rows past num_tokens were written"
    m = RMSNorm(4096, eps=1e-6).half().to(DEV)
    with torch.no_grad():
        m.weight.copy_(w)
    _close_in_ulps(m(wide.to(DEV)[:, :4096].contiguous()).cpu(), lo.rms_norm(wide[:, :4096], w, 1e-6),
                   torch.float16, "RMSNorm module", _normalised(wide[:, :4096], 1e-6), w)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("T,d", [(1, 11008), (56, 13824), (333, 17920), (3, 8), (17, 1000)])
def test_silu_and_mul(dtype, T, d):
    print(f"[case] silu_and_mul {dtype} T={T} d={d}", flush=True)
    g = torch.Generator().manual_seed(T + d)
    x = (torch.randn((T, 2 * d), generator=g) * 3).to(dtype)
    got = SiluAndMul()(x.to(DEV))
    torch.cuda.synchronize()
    assert got.shape == (T, d)
    _close_in_ulps(got.cpu(), lo.silu_and_mul(x), dtype, "silu_and_mul", _silu(x), x[:, d:])


def test_silu_and_mul_strided_and_partial():
    print("[case] silu_and_mul strided", flush=True)
    g = torch.Generator().manual_seed(9)
    wide = (torch.randn((40, 2 * 512 + 64), generator=g) * 3).half()
    out = torch.full((40, 512), -1.0, dtype=torch.float16, device=DEV)
    ops.silu_and_mul(wide.to(DEV)[:, :1024], out=out, num_tokens=33)
    torch.cuda.synchronize()
    xs = wide[:33, :1024]
    _close_in_ulps(out[:33].cpu(), lo.silu_and_mul(xs), torch.float16, "silu strided", _silu(xs), xs[:, 512:])
    assert (out[33:] == -1.0).all()


def _check_tokens(tokens, emb, hid_rows, V, dtype, what):
    """tokens: list[int]; hid_rows: the sampled hidden rows (CPU)."""
    exact = hid_rows.double() @ emb.double().t()
    exact = exact[:, :V]
    top2 = exact.topk(2, dim=-1).values
    tol = 2 * _ulp(top2[:, 0], dtype)
    want = exact.argmax(dim=-1)
    for r, tok in enumerate(tokens):
        assert 0 <= tok < V, f"{what}: row {r} token {tok} outside the vocabulary"
        if top2[r, 0] - top2[r, 1] > tol[r]:
            assert tok == int(want[r]), f"{what}: row {r} got {tok}, want {int(want[r])}"
        else:
            assert exact[r, tok] >= top2[r, 0] - tol[r], f"{what}: row {r} token {tok} is not a near-best logit"


@pytest.mark.parametrize("R", [1, 8, 16, 17, 32, 56, 64, 65, 130])
def test_greedy_sample_decode_rows_7b_shape(R):
    print(f"[case] greedy_sample decode R={R}", flush=True)
    g = torch.Generator().manual_seed(100 + R)
    V, Hd = 32000, 4096
    emb = (torch.randn((V, Hd), generator=g) * 0.05).half()
    hid = torch.randn(((R + 7) // 8 * 8, Hd), generator=g).half()
    toks = ops.greedy_sample(emb.to(DEV), hid.to(DEV), V, R)
    torch.cuda.synchronize()
    _check_tokens(toks.cpu().tolist(), emb, hid[:R], V, torch.float16, f"R={R}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("Hd", [5120, 6656, 8192, 256])
def test_greedy_sample_planted_winners_vocab_cut_and_ties(dtype, Hd):
    """Known answers: every sampled row has one embedding row planted as its
    clear best, at ids that sit on the edges of the kernel's 64-row and 16-row
    groups; rows past vocab_size hold larger logits and must be ignored; one
    sampled row has its best row duplicated at a higher id (lowest id wins)."""
    print(f"[case] greedy_sample planted {dtype} hidden={Hd}", flush=True)
    g = torch.Generator().manual_seed(Hd)
    V, V_pad = 5003, 5056
    emb = (torch.randn((V_pad, Hd), generator=g) * 0.02).to(dtype)
    ids = [0, 15, 16, 63, 64, 65, 1000, 4991, 4992, 5002, 77, 3]
    hid = torch.randn((len(ids) + 1, Hd), generator=g).to(dtype)
    for r, v in enumerate(ids):
        emb[v] = (hid[r].float() * 0.5).to(dtype)              # logit = |h|^2 / 2, far above the noise
    emb[V:] = (hid[0].float() * 2).to(dtype)                   # even larger, but outside the vocabulary
    dup = len(ids)
    emb[300] = (hid[dup].float() * 0.5).to(dtype)
    emb[4100] = emb[300]                                       # exact tie across workgroups
    emb[301] = emb[300]                                        # and inside one wave's 16 rows
    toks = ops.greedy_sample(emb.to(DEV), hid.to(DEV), V, len(ids) + 1).cpu().tolist()
    assert toks[:len(ids)] == ids
    assert toks[dup] == 300
    assert toks == lo.greedy_sample(emb, hid, [], len(ids) + 1, V)


def test_greedy_sampler_module_prompt_and_decode_steps():
    print("[case] GreedySampler module", flush=True)
    g = torch.Generator().manual_seed(11)
    V, V_pad, Hd = 32000, 32000, 4096
    emb = (torch.randn((V_pad, Hd), generator=g) * 0.05).half()
    demb = emb.to(DEV)
    sampler = GreedySampler(V)
    # prompt step: 5 prompts packed in 64 rows (padded to a multiple of 8)
    prompt_lens = [7, 1, 30, 12, 9]
    hid = torch.randn((64, Hd), generator=g).half()
    md = InputMetadata(prompt_lens=prompt_lens, slot_mapping=torch.empty((59, 1, 1), dtype=torch.int64),
                       context_lens=torch.empty((0,), dtype=torch.int32), max_context_len=0,
                       block_tables=torch.empty((0, 0, 0, 0), dtype=torch.int32))
    toks = sampler(demb, hid.to(DEV), md)
    assert isinstance(toks, list) and len(toks) == 5 and all(isinstance(t, int) for t in toks)
    rows = lo.sampled_rows(prompt_lens, 0)
    _check_tokens(toks, emb, hid[rows], V, torch.float16, "prompt step")
    # decode step: 13 sequences in 16 padded rows
    md = InputMetadata(prompt_lens=[], slot_mapping=torch.empty((13, 1, 1), dtype=torch.int64),
                       context_lens=torch.ones((13,), dtype=torch.int32), max_context_len=1,
                       block_tables=torch.empty((1, 13, 1, 1), dtype=torch.int32))
    toks = sampler(demb, hid[:16].to(DEV), md)
    assert len(toks) == 13
    _check_tokens(toks, emb, hid[:13], V, torch.float16, "decode step")


def test_greedy_sample_leaves_its_counter_zeroed_and_the_workspace_reusable():
    """One caller-owned workspace serves calls of different vocabulary sizes,
    batch sizes and workgroup shapes one after the other."""
    print("[case] greedy_sample workspace reuse", flush=True)
    from muxserve_amd import _lib
    g = torch.Generator().manual_seed(21)
    ws = torch.full((_lib.attn().mux_greedy_sample_workspace_bytes(32000),), 0xAB, dtype=torch.uint8, device=DEV)
    rc = _lib.attn().mux_greedy_sample_workspace_init(ws.data_ptr(), ws.numel(), torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    for V, Hd, R in ((32000, 256, 3), (700, 512, 40), (24593, 256, 64), (32000, 256, 20), (129, 256, 1)):
        emb = (torch.randn((V + 7, Hd), generator=g) * 0.1).half()
        hid = torch.randn((R, Hd), generator=g).half()
        toks = ops.greedy_sample(emb.to(DEV), hid.to(DEV), V, R, workspace=ws)
        torch.cuda.synchronize()
        _check_tokens(toks.cpu().tolist(), emb, hid, V, torch.float16, f"V={V} R={R}")
        assert int(ws[:256].count_nonzero()) == 0, "arrival counter not left at zero"


def test_model_ops_reject_malformed_arguments():
    x = torch.zeros((4, 4100), dtype=torch.float16, device=DEV)
    with pytest.raises(RuntimeError):
        ops.rms_norm(x, torch.ones(4100, dtype=torch.float16, device=DEV), 1e-6)      # hidden not a multiple of 8
    with pytest.raises(RuntimeError):
        ops.greedy_sample(torch.zeros((64, 4104), dtype=torch.float16, device=DEV)[:, :4100],
                          x, 64, 4)                                                  # hidden not a multiple of 256
    with pytest.raises(RuntimeError):
        ops.rms_norm(torch.zeros((4, 64)), torch.ones(64), 1e-6)                      # CPU tensors
