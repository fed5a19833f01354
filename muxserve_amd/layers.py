"""The operators of a LLaMA step around the attention layer, with the class
names and call signatures the reference's model code uses
(muxserve/flexserver/models/llama.py:35-36,75-81,200-232,257,283 for RMSNorm and
SiluAndMul, which it imports from its vLLM fork; muxserve/flexserver/sampler.py
for GreedySampler).  Each forwards to one registered operator of the package's PyTorch extension
(libmuxtorch.so over libmuxattn.so's C ABI); there is no eager fallback.
"""
import numpy as np
import torch

from . import torch_ops as T


class RMSNorm(torch.nn.Module):
    """`RMSNorm(hidden_size, eps)`; `forward(x)` for x [num_tokens, hidden_size]."""

    def __init__(self, hidden_size: int, eps: float = 1e-6) -> None:
        super().__init__()
        self.weight = torch.nn.Parameter(torch.ones(hidden_size))
        self.variance_epsilon = eps

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return T.rms_norm(x, self.weight.data, self.variance_epsilon)


class SiluAndMul(torch.nn.Module):
    """`forward(x)`: x [num_tokens, 2 d] -> silu(x[:, :d]) * x[:, d:]."""

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return T.silu_and_mul(x)


class GreedySampler(torch.nn.Module):
    """`GreedySampler(vocab_size)`; `forward(embedding, hidden_states,
    input_metadata) -> list[int]` as in muxserve/flexserver/sampler.py:15-35: on a
    prompt step the last row of every prompt is sampled, on a decode step the
    first num_generation_tokens rows; the token is the argmax of
    hidden . embedding^T over the first vocab_size rows of `embedding`.
    The logits are not materialised."""

    def __init__(self, vocab_size: int) -> None:
        super().__init__()
        self.vocab_size = vocab_size

    def forward(self, embedding: torch.Tensor, hidden_states: torch.Tensor, input_metadata):
        row_index = None
        if input_metadata.num_prompts > 0:
            assert input_metadata.num_generation_tokens == 0           # sampler.py:19
            if hasattr(input_metadata, "last_token_rows"):              # cached per step by this package's metadata
                row_index = input_metadata.last_token_rows(hidden_states.device)
            else:
                indices = np.cumsum(input_metadata.prompt_lens) - 1     # sampler.py:20
                row_index = torch.tensor(indices, dtype=torch.int32, device=hidden_states.device)
            num_tokens = input_metadata.num_prompts
        else:
            num_tokens = input_metadata.num_generation_tokens
        if num_tokens == 0:
            return []
        next_tokens = T.greedy_sample(embedding, hidden_states, self.vocab_size, num_tokens, row_index=row_index)
        return next_tokens.cpu().numpy().tolist()
