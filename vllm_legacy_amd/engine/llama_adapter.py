"""The Llama decode stack (model/llama_decode.py) behind the engine's model protocol.

The stack takes the reference's metadata -- prompt tokens first, decode tokens after them
(attention/backends/gfx950_paged.py) -- while the engine packs sequences in scheduling order with
any number of rows each.  This wrapper reorders a step (sequences that bring a run of rows, or
their first token, go first and take the prompt kernels over their cached prefix; sequences that
bring one row to a context go last and take paged attention), builds that metadata from the
step's host-side numbers, runs the stack and puts the rows back in the engine's order.
Weights are the stack's synthetic ones (it has no unquantized checkpoint format); the engine,
scheduler, cache manager and sampler are the ones every model uses.
"""
from dataclasses import asdict, fields
from typing import Dict, List, Optional

import torch
import torch.nn as nn

from vllm_legacy_amd.attention.backends.gfx950_paged import Gfx950PagedAttentionMetadata
from vllm_legacy_amd.attention.batch import SequenceBatch
from vllm_legacy_amd.model.llama_decode import LlamaConfig, LlamaDecodeModel


class LlamaEngineConfig:
    """config.json of a synthetic stack: LlamaConfig's fields plus `quant` (none / awq / gptq),
    `kv_cache_dtype` (auto / fp8) and `seed`."""

    def __init__(self, llama: LlamaConfig, quant: str = "none", kv_cache_dtype: str = "auto", seed: int = 0):
        self.llama, self.quant, self.kv_cache_dtype, self.seed = llama, quant, kv_cache_dtype, seed

    @staticmethod
    def from_dict(d: Dict) -> "LlamaEngineConfig":
        names = {f.name for f in fields(LlamaConfig)}
        return LlamaEngineConfig(LlamaConfig(**{k: v for k, v in d.items() if k in names}),
                                 d.get("quant", "none"), d.get("kv_cache_dtype", "auto"), int(d.get("seed", 0)))

    def to_dict(self) -> Dict:
        return dict(asdict(self.llama), architecture="LlamaDecodeStack", quant=self.quant,
                    kv_cache_dtype=self.kv_cache_dtype, seed=self.seed)


class PagedLlamaForEngine(nn.Module):
    architecture = "LlamaDecodeStack"

    def __init__(self, cfg: LlamaEngineConfig, dtype=torch.float16, device="cuda", seed: Optional[int] = None):
        super().__init__()
        self.cfg, self.dtype = cfg, dtype
        self.stack = LlamaDecodeModel(cfg.llama, quant=cfg.quant, kv_cache_dtype=cfg.kv_cache_dtype,
                                      device=device, seed=cfg.seed if seed is None else seed, dtype=dtype)
        self.block_size = 16

    def load_weights(self, tensors) -> int:
        return self.stack.load_weights(tensors)

    def allocate_caches(self, num_blocks: int, block_size: int, num_slots: int) -> List[torch.Tensor]:
        """One [2, blocks, block_size * kv_heads * head_dim] tensor per layer; the stack keeps no
        per-sequence state, so the slots are not used."""
        self.block_size = block_size
        dev = self.stack.lm_head.device
        dt = torch.uint8 if self.cfg.kv_cache_dtype == "fp8" else self.dtype
        shape = self.stack.kv_cache_shape(num_blocks, block_size)
        return [torch.zeros(shape, dtype=dt, device=dev) for _ in self.stack.layers]

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor, caches, batch: SequenceBatch) -> torch.Tensor:
        q, c = batch.host_query_lens, batch.host_context_lens
        assert q is not None and c is not None, "the step's host-side numbers are needed"
        dev = input_ids.device
        B = len(q)
        runs = [b for b in range(B) if q[b] > 1 or c[b] == 0]
        singles = [b for b in range(B) if not (q[b] > 1 or c[b] == 0)]
        order = runs + singles
        starts = [0]
        for n in q:
            starts.append(starts[-1] + n)
        perm = [r for b in order for r in range(starts[b], starts[b + 1])]
        identity = perm == list(range(len(perm)))
        if not identity:
            idx = torch.as_tensor(perm, dtype=torch.int64).to(dev)
            input_ids, positions = input_ids[idx], positions[idx]
            slot_mapping = batch.slot_mapping[idx]
            sel = torch.as_tensor(order, dtype=torch.int64).to(dev)
            tables = batch.block_tables[sel].contiguous()
        else:
            slot_mapping, tables = batch.slot_mapping, batch.block_tables
        seq_lens = [c[b] + q[b] for b in order]

        def i32(x):
            return torch.as_tensor(x, dtype=torch.int32).to(dev)

        cu_q, cu_s = [0], [0]
        for b in runs:
            cu_q.append(cu_q[-1] + q[b])
            cu_s.append(cu_s[-1] + c[b] + q[b])
        n_run_rows = cu_q[-1]
        meta = Gfx950PagedAttentionMetadata(
            num_prefills=len(runs), num_prefill_tokens=n_run_rows, num_decode_tokens=len(singles),
            slot_mapping=slot_mapping, seq_lens=seq_lens, seq_lens_tensor=i32(seq_lens),
            max_query_len=max([q[b] for b in runs], default=0),
            max_prefill_seq_len=max([c[b] + q[b] for b in runs], default=0),
            max_decode_seq_len=max([c[b] + 1 for b in singles], default=0),
            query_start_loc=i32(cu_q), seq_start_loc=i32(cu_s), use_cuda_graph=False,
            context_lens_tensor=i32([c[b] for b in runs] or [0]), block_tables=tables)
        hidden = self.stack(input_ids, positions, list(caches), meta)
        if identity:
            return hidden
        out = torch.empty_like(hidden)
        out[idx] = hidden
        return out

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return self.stack.compute_logits(hidden.contiguous()).float()
