"""Sampling parameters and the sampler (the role of vllm/sampling_params.py and
vllm/model_executor/layers/sampler.py for the options served here): greedy, temperature,
top-k, top-p, a seed per request."""
from dataclasses import dataclass, field
from typing import List, Optional

import torch


@dataclass
class SamplingParams:
    max_tokens: int = 16
    temperature: float = 0.0        # 0: greedy
    top_k: int = 0                  # 0: all
    top_p: float = 1.0
    seed: Optional[int] = None
    stop_token_ids: List[int] = field(default_factory=list)

    def __post_init__(self):
        if self.max_tokens < 1:
            raise ValueError("max_tokens must be at least 1")
        if self.temperature < 0 or not (0 < self.top_p <= 1) or self.top_k < 0:
            raise ValueError("temperature >= 0, 0 < top_p <= 1 and top_k >= 0 are required")


class Sampler:
    """logits fp32 [n, vocab] -> one token per row, each row under its own parameters."""

    def __call__(self, logits: torch.Tensor, params: List[SamplingParams],
                 generators: List[Optional[torch.Generator]]) -> List[int]:
        assert logits.dim() == 2 and logits.shape[0] == len(params) == len(generators)
        if all(p.temperature == 0 for p in params):
            return torch.argmax(logits, dim=-1).tolist()
        out = []
        for row, p, g in zip(logits, params, generators):
            if p.temperature == 0:
                out.append(int(torch.argmax(row)))
                continue
            row = row / p.temperature
            if p.top_k and p.top_k < row.numel():
                kth = torch.topk(row, p.top_k).values[-1]
                row = row.masked_fill(row < kth, float("-inf"))
            probs = torch.softmax(row, dim=-1)
            if p.top_p < 1.0:
                sp, idx = torch.sort(probs, descending=True)
                keep = torch.cumsum(sp, 0) - sp < p.top_p      # the first token always stays
                probs = torch.zeros_like(probs).scatter_(0, idx[keep], sp[keep])
                probs = probs / probs.sum()
            out.append(int(torch.multinomial(probs, 1, generator=g)))
        return out
