"""CPU restatement of the per-step operators around the attention layer:
RMSNorm, SiluAndMul and the greedy sampler.

TEST INFRASTRUCTURE ONLY.  Nothing in muxserve_amd/ imports this file; it is
the checker for tests/, __graft_entry__.smoke() and bench.py's CPU baseline.

Where the algorithm lives
-------------------------
* GreedySampler is the reference's own file, muxserve/flexserver/sampler.py:9-35:
  on a prompt step keep the last row of every prompt (cumsum(prompt_lens) - 1,
  :18-24), logits = hidden . embedding^T cut to vocab_size (:26, through the
  dependency's _get_logits), argmax over the vocabulary (:33), first
  num_prompts / num_generation_tokens results (:28-35).
* RMSNorm, SiluAndMul and _get_logits are imported by the reference from the
  absent, unpinned dependency `vllm` = EfficientLLMSys/MuxServe-vLLM
  (muxserve/flexserver/models/llama.py:35-36, sampler.py:6; constructed at
  models/llama.py:75,200-203,257; applied at :79-81,217-232,283).  The functions
  below restate the published vLLM v0.2 operators:
      rms_norm:      out = (T)(x * rsqrt(mean(x^2) + eps)) * weight, fp32
                     statistics, the product with the weight taken in T
      silu_and_mul:  out = (T)(a / (1 + exp(-a))) * b for x = [a | b], the
                     product taken in T
      logits:        hidden @ embedding^T, fp32 accumulation, rounded to T
  PARITY UNPINNED against the dependency itself (its rounding points are taken
  from its published sources, which are not in the reference checkout).  Pinned
  by mathematics in tests/test_layer_oracle.py: torch's own rms_norm / silu in
  fp64, scalar loops on tiny inputs, brute-force argmax, exact-integer cases.
"""
import numpy as np
import torch


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """x [T, hidden] in fp16/bf16, weight [hidden] of the same type."""
    xf = x.float()
    var = xf.pow(2).mean(dim=-1, keepdim=True)
    y = (xf * torch.rsqrt(var + eps)).to(x.dtype)
    return (y.float() * weight.float()).to(x.dtype)          # product of two T values, rounded once


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    """x [T, 2 d] = [gate | up] -> [T, d]."""
    d = x.shape[-1] // 2
    a = x[..., :d].float()
    s = (a / (1.0 + torch.exp(-a))).to(x.dtype)
    return (s.float() * x[..., d:].float()).to(x.dtype)


def sampled_rows(prompt_lens, num_generation_tokens):
    """Rows of hidden_states the sampler looks at (sampler.py:18-32)."""
    if len(prompt_lens) > 0:
        assert num_generation_tokens == 0
        return (np.cumsum(np.asarray(prompt_lens, dtype=np.int64)) - 1).astype(np.int64)
    return np.arange(num_generation_tokens, dtype=np.int64)


def logits(embedding: torch.Tensor, hidden: torch.Tensor, vocab_size: int) -> torch.Tensor:
    """[R, vocab_size] in the storage type, fp64 accumulation then one rounding
    (what an fp32-accumulating GEMM returns up to the last bit)."""
    full = hidden.double() @ embedding.double().t()
    return full[:, :vocab_size].to(hidden.dtype)


def greedy_sample(embedding: torch.Tensor, hidden_states: torch.Tensor, prompt_lens,
                  num_generation_tokens: int, vocab_size: int):
    """list[int], one token per prompt (prompt step) or per sequence (decode
    step).  Ties go to the lowest token id."""
    rows = sampled_rows(prompt_lens, num_generation_tokens)
    h = hidden_states.index_select(0, torch.from_numpy(rows))
    lg = logits(embedding, h, vocab_size).float()
    best = lg.max(dim=-1, keepdim=True).values
    first = (lg == best).int().argmax(dim=-1)                # first occurrence of the maximum
    return first.tolist()
