"""Model runner: owns the model and its cache tensors and runs one step of a packed batch.

A model served by the engine provides
  allocate_caches(num_blocks, block_size, num_slots) -> per-layer-run cache tensors
  forward(input_ids, positions, caches, batch: SequenceBatch) -> hidden rows [T, width]
  compute_logits(hidden rows) -> fp32 logits
`execute` is the one step function: the engine's scheduled steps and a replayed trace's given
steps both go through it."""
from typing import List, Optional, Sequence as Seq, Tuple

import torch

from vllm_legacy_amd.attention.batch import SequenceBatch

from .cache_manager import CacheManager


class ModelRunner:

    def __init__(self, model, cache: CacheManager, device="cuda") -> None:
        self.model, self.cache, self.device = model, cache, torch.device(device)
        self.caches = model.allocate_caches(cache.num_blocks, cache.block_size, cache.num_slots)

    @torch.inference_mode()
    def execute(self, entries: Seq[Tuple[str, List[int], int]],
                want: Seq[Seq[int]]) -> Optional[torch.Tensor]:
        """entries: (sequence id, its next tokens, tokens of it already in the cache); the cache
        manager's table of each sequence must already cover them.  want: per entry, the indices
        among its tokens whose logits are asked for.  Returns fp32 [sum(len(want)), vocab] in
        the order of the entries, or None when nothing is asked for."""
        assert len(entries) == len(want) and entries
        ids: List[int] = []
        rows: List[int] = []
        for (seq_id, tokens, computed), w in zip(entries, want):
            assert tokens and all(0 <= i < len(tokens) for i in w)
            rows += [len(ids) + i for i in w]
            ids += tokens
        batch = SequenceBatch.build(
            [len(t) for _, t, _ in entries], [c for _, _, c in entries],
            [self.cache.block_table(s) for s, _, _ in entries],
            [self.cache.state_slot(s) for s, _, _ in entries], self.cache.block_size, self.device)
        input_ids = torch.as_tensor(ids, dtype=torch.int64).to(self.device, non_blocking=True)
        hidden = self.model(input_ids, batch.positions, self.caches, batch)
        if not rows:
            return None
        sel = torch.as_tensor(rows, dtype=torch.int64).to(self.device, non_blocking=True)
        return self.model.compute_logits(hidden.index_select(0, sel))
