"""LLMEngine: the entry point that generation goes through (the role of
vllm/engine/llm_engine.py `add_request` / `step` and of vllm/entrypoints/llm.py `generate`)."""
from dataclasses import dataclass
from typing import Dict, List, Optional

import torch

from .cache_manager import CacheManager
from .model_runner import ModelRunner
from .sampling import Sampler, SamplingParams
from .scheduler import Scheduler, Sequence


@dataclass
class EngineConfig:
    block_size: int = 16
    num_blocks: int = 4096              # cache pool, in blocks
    max_num_seqs: int = 64              # live sequences = recurrent-state slots
    max_num_batched_tokens: int = 2048  # tokens per step


@dataclass
class RequestOutput:
    request_id: str
    prompt_token_ids: List[int]
    token_ids: List[int]
    finished: bool
    finish_reason: Optional[str]


class LLMEngine:

    def __init__(self, model, config: Optional[EngineConfig] = None, device="cuda") -> None:
        self.config = config or EngineConfig()
        c = self.config
        self.cache = CacheManager(c.num_blocks, c.block_size, c.max_num_seqs)
        self.scheduler = Scheduler(self.cache, c.max_num_batched_tokens, c.max_num_seqs)
        self.runner = ModelRunner(model, self.cache, device)
        self.sampler = Sampler()
        self._generators: Dict[str, Optional[torch.Generator]] = {}
        self._count = 0

    @classmethod
    def from_pretrained(cls, model_dir: str, dtype=torch.bfloat16, config: Optional[EngineConfig] = None,
                        device="cuda") -> "LLMEngine":
        from vllm_legacy_amd.model.registry import load_model
        return cls(load_model(model_dir, dtype, device), config, device)

    def add_request(self, prompt_token_ids: List[int], params: Optional[SamplingParams] = None,
                    request_id: Optional[str] = None) -> str:
        if not prompt_token_ids:
            raise ValueError("empty prompt")
        params = params or SamplingParams()
        if request_id is None:
            request_id = f"req-{self._count}"
        self._count += 1
        g = None
        if params.seed is not None:
            g = torch.Generator(device=self.runner.device).manual_seed(params.seed)
        self._generators[request_id] = g
        self.scheduler.add(Sequence(request_id, list(prompt_token_ids), params))
        return request_id

    def has_unfinished_requests(self) -> bool:
        return self.scheduler.has_unfinished()

    def step(self) -> List[RequestOutput]:
        """One scheduled step; returns the sequences that got a token in it."""
        scheduled = self.scheduler.schedule()
        if not scheduled:
            return []
        entries, want, sampled = [], [], []
        for seq, n in scheduled:
            tokens = seq.token_ids[seq.num_computed:seq.num_computed + n]
            entries.append((seq.seq_id, tokens, seq.num_computed))
            last = seq.num_computed + n == len(seq)      # the step reaches the sequence's end
            want.append([n - 1] if last else [])
            if last:
                sampled.append(seq)
        logits = self.runner.execute(entries, want)
        for seq, n in scheduled:
            seq.num_computed += n
        outputs = []
        if sampled:
            tokens = self.sampler(logits, [s.params for s in sampled],
                                  [self._generators[s.seq_id] for s in sampled])
            for seq, tok in zip(sampled, tokens):
                seq.output_token_ids.append(tok)
                if tok in seq.params.stop_token_ids:
                    self.scheduler.finish(seq, "stop")
                elif len(seq.output_token_ids) >= seq.params.max_tokens:
                    self.scheduler.finish(seq, "length")
                if seq.finished:
                    self._generators.pop(seq.seq_id, None)
                outputs.append(RequestOutput(seq.seq_id, seq.prompt_token_ids,
                                             list(seq.output_token_ids), seq.finished, seq.finish_reason))
        return outputs

    def generate(self, prompts: List[List[int]], params=None) -> List[RequestOutput]:
        """Run the prompts to completion; outputs in the order of the prompts."""
        if params is None or isinstance(params, SamplingParams):
            params = [params or SamplingParams()] * len(prompts)
        ids = [self.add_request(p, sp) for p, sp in zip(prompts, params)]
        done: Dict[str, RequestOutput] = {}
        while self.has_unfinished_requests():
            for out in self.step():
                if out.finished:
                    done[out.request_id] = out
        return [done[i] for i in ids]
