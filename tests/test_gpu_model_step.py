"""The pieces composed the way the reference's model composes them
(muxserve/flexserver/models/llama.py:200-232, 265-292, 330-345): a small
LLaMA-shaped model - embedding, RMSNorm, qkv projection, PagedAttentionWithRoPE
over the shared pool, o_proj, residual, RMSNorm, gate/up projection,
SiluAndMul, down projection, final norm, GreedySampler - driven by
BatchScheduler / KVStorage / prepare_inputs through a prefill step and several
decode steps, against a plain fp32 PyTorch implementation of the same model
that recomputes full causal attention over the whole sequence every step (no
cache, no paging).  The projections are torch matmuls in both; everything else
on the tested side goes through this package's kernels.

Tolerances: final hidden states within 2e-2 (fp16 activations through two
layers against fp32); sampled tokens equal whenever the fp32 model's best logit
leads by more than 0.05."""
import numpy as np
import pytest
import torch

from muxserve_amd.attention import PagedAttentionWithRoPE
from muxserve_amd.batch_scheduler import BatchScheduler
from muxserve_amd.device_tables import DeviceBlockTables
from muxserve_amd.layers import GreedySampler, RMSNorm, SiluAndMul
from muxserve_amd.memory_manager import KVStorage
from muxserve_amd.pool import HEAD_SIZE, allocate_gpu_cache
from muxserve_amd.prepare import prepare_inputs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
D = HEAD_SIZE


class TinyLlama:
    """Weights shared by the tested model and the fp32 reference."""

    def __init__(self, L, Hq, Hkv, inter, vocab, seed):
        g = torch.Generator().manual_seed(seed)
        self.L, self.Hq, self.Hkv, self.inter, self.vocab = L, Hq, Hkv, inter, vocab
        self.hidden = Hq * D
        s = 0.5 / self.hidden ** 0.5

        def w(*shape, scale=s):
            return (torch.randn(shape, generator=g) * scale).half()

        self.embed = w(vocab, self.hidden, scale=0.5)
        self.layers = []
        for _ in range(L):
            self.layers.append({
                "ln1": (1 + 0.1 * torch.randn(self.hidden, generator=g)).half(),
                "qkv": w((Hq + 2 * Hkv) * D, self.hidden),
                "o": w(self.hidden, Hq * D),
                "ln2": (1 + 0.1 * torch.randn(self.hidden, generator=g)).half(),
                "gate_up": w(2 * inter, self.hidden),
                "down": w(self.hidden, inter, scale=0.5 / inter ** 0.5),
            })
        self.norm = (1 + 0.1 * torch.randn(self.hidden, generator=g)).half()
        self.lm_head = w((vocab + 63) // 64 * 64, self.hidden, scale=0.3)


def _rope_fp32(x, positions, n_heads):
    """NeoX rotary embedding, fp64 angles; x [T, n_heads * D] fp32."""
    T = x.shape[0]
    x = x.view(T, n_heads, D)
    inv = 1.0 / (10000.0 ** (torch.arange(0, D, 2, dtype=torch.float64) / D))
    ang = positions.double()[:, None] * inv[None, :]
    c, s_ = ang.cos().float()[:, None, :], ang.sin().float()[:, None, :]
    a, b = x[..., :D // 2], x[..., D // 2:]
    return torch.cat([a * c - b * s_, b * c + a * s_], dim=-1).reshape(T, n_heads * D)


def reference_logits(m: TinyLlama, tokens):
    """fp32, full recomputation: hidden state and logits of the LAST token."""
    x = m.embed.float()[torch.tensor(tokens)]
    T = len(tokens)
    pos = torch.arange(T)
    for w in m.layers:
        h = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + 1e-6) * w["ln1"].float()
        qkv = h @ w["qkv"].float().t()
        q, k, v = qkv.split([m.Hq * D, m.Hkv * D, m.Hkv * D], dim=-1)
        q, k = _rope_fp32(q, pos, m.Hq), _rope_fp32(k, pos, m.Hkv)
        q = q.view(T, m.Hq, D).transpose(0, 1)
        k = k.view(T, m.Hkv, D).transpose(0, 1).repeat_interleave(m.Hq // m.Hkv, dim=0)
        v = v.view(T, m.Hkv, D).transpose(0, 1).repeat_interleave(m.Hq // m.Hkv, dim=0)
        att = (q @ k.transpose(1, 2)) * D ** -0.5
        att = att.masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool), 1), float("-inf")).softmax(-1)
        x = x + (att @ v).transpose(0, 1).reshape(T, m.Hq * D) @ w["o"].float().t()
        h = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + 1e-6) * w["ln2"].float()
        gu = h @ w["gate_up"].float().t()
        x = x + (torch.nn.functional.silu(gu[:, :m.inter]) * gu[:, m.inter:]) @ w["down"].float().t()
    x = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + 1e-6) * m.norm.float()
    return x[-1], (x[-1] @ m.lm_head.float().t())[:m.vocab]


class Served:
    """The same model on the GPU, built from this package's layers."""

    def __init__(self, m: TinyLlama, storage, bs, rows):
        self.m = m
        self.sched = BatchScheduler(m.L, m.Hkv, 512, bs)
        self.storage = storage
        self.tables = DeviceBlockTables(self.sched, rows, DEV)
        self.attn = [PagedAttentionWithRoPE(m.Hq, D, D ** -0.5, base=10000, max_position=512, rotary_dim=D,
                                            num_kv_heads=m.Hkv, rope_scaling=None, layer_idx=l) for l in range(m.L)]
        self.ln1, self.ln2 = [], []
        for w in m.layers:
            for dst, key in ((self.ln1, "ln1"), (self.ln2, "ln2")):
                n = RMSNorm(m.hidden, eps=1e-6).half().to(DEV)
                with torch.no_grad():
                    n.weight.copy_(w[key])
                dst.append(n)
        self.norm = RMSNorm(m.hidden, eps=1e-6).half().to(DEV)
        with torch.no_grad():
            self.norm.weight.copy_(m.norm)
        self.act = SiluAndMul()
        self.sampler = GreedySampler(m.vocab)
        self.dev = {k: v.to(DEV) for k, v in (("embed", m.embed), ("lm_head", m.lm_head))}
        self.w = [{k: v.to(DEV) for k, v in w.items()} for w in m.layers]

    def step(self, ids, last_tokens, k_pool, v_pool):
        m = self.m
        tok, pos, md, _, preempted = prepare_inputs(self.sched, lambda r: self.storage.allocate_batch(r, m.L, m.Hkv),
                                                    ids, last_tokens, DEV, device_tables=self.tables)
        assert not preempted
        x = self.dev["embed"][tok]
        for l, w in enumerate(self.w):
            h = self.ln1[l](x)
            qkv = h @ w["qkv"].t()
            q, k, v = qkv.split([m.Hq * D, m.Hkv * D, m.Hkv * D], dim=-1)         # models/llama.py:157-158
            x = x + self.attn[l](pos, q, k, v, k_pool, v_pool, md, None) @ w["o"].t()
            h = self.ln2[l](x)
            x = x + self.act(h @ w["gate_up"].t()) @ w["down"].t()
        x = self.norm(x)
        tokens = self.sampler(self.dev["lm_head"], x, md)
        rows = (np.cumsum(md.prompt_lens) - 1) if md.num_prompts else np.arange(md.num_generation_tokens)
        return tokens, x[torch.as_tensor(rows, device=DEV)].float().cpu()


@pytest.mark.parametrize("Hq,Hkv", [(2, 2), (4, 1)])
def test_model_steps_match_an_fp32_model_without_a_cache(Hq, Hkv):
    print(f"[case] model step Hq={Hq} Hkv={Hkv}", flush=True)
    bs, N = 16, 2000
    m = TinyLlama(L=2, Hq=Hq, Hkv=Hkv, inter=512, vocab=1000, seed=Hq * 10 + Hkv)
    storage = KVStorage(N)
    k_pool, v_pool = allocate_gpu_cache(N, bs, DEV)
    served = Served(m, storage, bs, rows=4)
    rng = np.random.Generator(np.random.PCG64(7))
    seqs = {0: [int(t) for t in rng.integers(0, 1000, size=19)],
            1: [int(t) for t in rng.integers(0, 1000, size=33)],
            2: [int(t) for t in rng.integers(0, 1000, size=5)]}
    for rid, prompt in seqs.items():
        served.sched.add_request(np.asarray(prompt, dtype=np.int32), rid, 32)
    ids = [0, 1, 2]

    def check(tokens, hidden, what):
        agree = 0
        for i, rid in enumerate(ids):
            ref_h, ref_logits = reference_logits(m, seqs[rid])
            err = (hidden[i] - ref_h).abs().max().item()
            assert err <= 2e-2, f"{what}: request {rid}: final hidden state off by {err:.3e}"
            top2 = ref_logits.topk(2).values
            if top2[0] - top2[1] > 0.05:
                assert tokens[i] == int(ref_logits.argmax()), f"{what}: request {rid}: sampled {tokens[i]}"
                agree += 1
            else:
                assert ref_logits[tokens[i]] >= top2[0] - 0.05
        return agree

    tokens, hidden = served.step(ids, [], k_pool, v_pool)
    decided = check(tokens, hidden, "prefill")
    for step in range(18):                                  # crosses block boundaries of all three sequences
        for rid, t in zip(ids, tokens):
            seqs[rid].append(int(t))
        tokens, hidden = served.step(ids, list(tokens), k_pool, v_pool)
        decided += check(tokens, hidden, f"decode step {step}")
    assert decided >= 30, "too few steps had a clear best token to mean anything"
