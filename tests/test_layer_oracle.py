"""Pins oracle/layer_oracle.py (RMSNorm, SiluAndMul, greedy sampling) by
mathematics: fp64 closed forms and torch's own operators within one rounding of
the storage type, scalar loops on tiny inputs, exact-integer cases, invariants.
The dependency that holds these operators is absent from the reference
checkout, so nothing here compares against it."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import layer_oracle as lo


def _ulp(t: torch.Tensor, dtype) -> torch.Tensor:
    """Spacing of dtype at |t| (fp64 in, fp64 out), with the normal-range floor."""
    bits = 10 if dtype == torch.float16 else 7
    tiny = 2.0 ** -14 if dtype == torch.float16 else 2.0 ** -126
    mag = torch.clamp(t.abs().double(), min=tiny)
    return torch.pow(2.0, torch.floor(torch.log2(mag)) - bits)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_rms_norm_against_fp64_closed_form_and_torch(dtype):
    g = torch.Generator().manual_seed(1)
    x = (torch.randn((37, 640), generator=g) * 3).to(dtype)
    w = (1 + 0.2 * torch.randn((640,), generator=g)).to(dtype)
    eps = 1e-5
    got = lo.rms_norm(x, w, eps).double()
    xd, wd = x.double(), w.double()
    want = xd / torch.sqrt((xd * xd).mean(-1, keepdim=True) + eps) * wd
    # two roundings to T (normalised value, then the product): within 1.5 ulp + the weight's share
    assert ((got - want).abs() <= 1.51 * _ulp(want, dtype) + _ulp(want / wd, dtype) * wd.abs()).all()
    lib = F.rms_norm(xd, (640,), wd, eps)
    assert torch.allclose(lib, want, rtol=1e-12, atol=0)


def test_rms_norm_scalar_loop_and_invariants():
    x = torch.tensor([[3.0, -4.0, 0.0, 12.0]], dtype=torch.float16)
    w = torch.tensor([1.0, 2.0, 3.0, 0.5], dtype=torch.float16)
    ms = (9 + 16 + 0 + 144) / 4
    want = []
    for xi, wi in zip(x[0].tolist(), w.tolist()):
        y = float(torch.tensor(xi / math.sqrt(ms), dtype=torch.float32).to(torch.float16))
        want.append(float(torch.tensor(y * wi, dtype=torch.float32).to(torch.float16)))
    assert lo.rms_norm(x, w, 0.0)[0].tolist() == want
    # a constant row normalises to +-1; scaling a row by a power of two changes nothing (eps = 0)
    c = torch.full((2, 64), -0.37, dtype=torch.float16)
    assert torch.equal(lo.rms_norm(c, torch.ones(64, dtype=torch.float16), 0.0), -torch.ones_like(c))
    g = torch.Generator().manual_seed(2)
    r = torch.randn((5, 128), generator=g).half()
    wr = torch.randn((128,), generator=g).half()
    assert torch.equal(lo.rms_norm(r, wr, 0.0), lo.rms_norm(r * 4, wr, 0.0))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_silu_and_mul_against_torch_silu(dtype):
    g = torch.Generator().manual_seed(3)
    x = (torch.randn((29, 2 * 96), generator=g) * 4).to(dtype)
    got = lo.silu_and_mul(x).double()
    a, b = x[:, :96].double(), x[:, 96:].double()
    s = F.silu(a)
    want = s * b
    assert ((got - want).abs() <= 0.51 * _ulp(want, dtype) + 0.51 * _ulp(s, dtype) * b.abs() + 1e-30).all()
    # silu(a) - silu(-a) = a; silu(0) = 0; large a: silu(a) = a
    ones = torch.ones((1, 4), dtype=dtype)
    v = torch.tensor([[0.0, 20.0, -20.0, 1.5]], dtype=dtype)
    out = lo.silu_and_mul(torch.cat([v, ones], dim=1))[0].float()
    assert out[0] == 0 and out[1] == 20 and abs(out[2]) < 1e-6
    neg = lo.silu_and_mul(torch.cat([-v, ones], dim=1))[0].float()
    assert abs((out[3] - neg[3]) - 1.5) <= 2 ** -7


def test_greedy_sample_brute_force_ties_vocab_cut_and_row_selection():
    rng = np.random.Generator(np.random.PCG64(4))
    V_pad, V, Hd = 24, 21, 16
    emb = torch.from_numpy(rng.integers(-3, 4, size=(V_pad, Hd)).astype(np.float32)).half()
    hid = torch.from_numpy(rng.integers(-3, 4, size=(11, Hd)).astype(np.float32)).half()
    emb[22] = 100.0                                   # a huge logit past the vocabulary must not win
    emb[7] = emb[3]                                   # exact tie between ids 3 and 7
    hid[4] = emb[3]                                   # row 4 is best matched by ids 3 and 7 ... unless beaten
    prompt_lens = [3, 2, 6]                           # sampled rows 2, 4, 10
    got = lo.greedy_sample(emb, hid, prompt_lens, 0, V)
    want = []
    for r in (2, 4, 10):
        best, arg = None, None
        for v in range(V):
            s = sum(float(hid[r, i]) * float(emb[v, i]) for i in range(Hd))      # small integers: exact
            if best is None or s > best:
                best, arg = s, v
        want.append(arg)
    assert got == want
    assert 22 not in got
    # decode step: rows 0 .. n-1
    got_d = lo.greedy_sample(emb, hid, [], 5, V)
    assert got_d == [lo.greedy_sample(emb, hid[r:r + 1], [], 1, V)[0] for r in range(5)]
    # the tie goes to the lower id
    e2 = torch.zeros((8, 16), dtype=torch.float16)
    e2[5] = 1.0
    e2[2] = 1.0
    assert lo.greedy_sample(e2, torch.ones((1, 16), dtype=torch.float16), [], 1, 8) == [2]
    assert lo.sampled_rows([3, 2, 6], 0).tolist() == [2, 4, 10]
    assert lo.sampled_rows([], 4).tolist() == [0, 1, 2, 3]
