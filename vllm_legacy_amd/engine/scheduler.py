"""Continuous-batching scheduler with prompts cut into portions.

Every step takes, in this order and under `max_num_batched_tokens`: one token for each running
sequence that is decoding, the next portion of each running sequence whose prompt is not through,
then new sequences from the waiting queue while slots, blocks and budget last (the policy of the
reference's chunked-prefill scheduler, vllm/core/scheduler.py `_schedule_chunked_prefill`:
decodes first, then prefills cut to the remaining budget).  A decoding sequence that cannot get
its next block preempts the most recently admitted sequence, which gives back everything and
starts over from the waiting queue's head (preemption by recomputation)."""
from collections import deque
from dataclasses import dataclass, field
from typing import Deque, List, Optional, Tuple

from .cache_manager import CacheManager
from .sampling import SamplingParams


@dataclass
class Sequence:
    seq_id: str
    prompt_token_ids: List[int]
    params: SamplingParams = field(default_factory=SamplingParams)
    output_token_ids: List[int] = field(default_factory=list)
    num_computed: int = 0           # tokens whose keys / state are in the cache
    finished: bool = False
    finish_reason: Optional[str] = None

    @property
    def token_ids(self) -> List[int]:
        return self.prompt_token_ids + self.output_token_ids

    def __len__(self) -> int:
        return len(self.prompt_token_ids) + len(self.output_token_ids)


class Scheduler:

    def __init__(self, cache: CacheManager, max_num_batched_tokens: int = 2048,
                 max_num_seqs: Optional[int] = None) -> None:
        self.cache = cache
        self.max_num_batched_tokens = max_num_batched_tokens
        self.max_num_seqs = min(max_num_seqs or cache.num_slots, cache.num_slots)
        self.waiting: Deque[Sequence] = deque()
        self.running: List[Sequence] = []
        self.num_preemptions = 0

    def add(self, seq: Sequence) -> None:
        if len(seq) + seq.params.max_tokens > self.cache.num_blocks * self.cache.block_size:
            raise ValueError("the request cannot fit the cache even alone")
        self.waiting.append(seq)

    def has_unfinished(self) -> bool:
        return bool(self.waiting or self.running)

    def _preempt_last(self, keep: Sequence) -> bool:
        for victim in reversed(self.running):
            if victim is not keep:
                self.running.remove(victim)
                self.cache.free(victim.seq_id)
                victim.num_computed = 0
                self.waiting.appendleft(victim)
                self.num_preemptions += 1
                return True
        return False

    def schedule(self) -> List[Tuple[Sequence, int]]:
        """[(sequence, number of its next tokens to run)]; blocks are allocated here."""
        budget = self.max_num_batched_tokens
        step: List[Tuple[Sequence, int]] = []
        for seq in list(self.running):          # decodes, oldest first
            if seq not in self.running or len(seq) - seq.num_computed != 1 or budget < 1:
                continue
            while not self.cache.can_grow(seq.seq_id, seq.num_computed + 1):
                if not self._preempt_last(seq):
                    raise RuntimeError("a single sequence has outgrown the cache")
            self.cache.grow(seq.seq_id, seq.num_computed + 1)
            step.append((seq, 1))
            budget -= 1
        # a preempted sequence may already be in `step`: drop it
        step = [(s, n) for s, n in step if s in self.running]
        for seq in self.running:                # prompts under way
            left = len(seq) - seq.num_computed
            if left <= 1 or budget < 1:
                continue
            n = min(left, budget)
            while n > 0 and not self.cache.can_grow(seq.seq_id, seq.num_computed + n):
                n = (self.cache.free_blocks + len(self.cache.block_table(seq.seq_id))) * \
                    self.cache.block_size - seq.num_computed
            if n <= 0:
                continue
            self.cache.grow(seq.seq_id, seq.num_computed + n)
            step.append((seq, n))
            budget -= n
        while self.waiting and budget > 0 and len(self.running) < self.max_num_seqs:
            seq = self.waiting[0]
            n = min(len(seq), budget)
            if not self.cache.can_admit(n):
                break
            self.waiting.popleft()
            self.cache.admit(seq.seq_id)
            self.cache.grow(seq.seq_id, n)
            self.running.append(seq)
            step.append((seq, n))
            budget -= n
        if not step and len(self.running) > 1:
            # every running prompt is stuck behind the others' blocks: the newest starts over
            self._preempt_last(self.running[0])
            return self.schedule()
        return step

    def finish(self, seq: Sequence, reason: str) -> None:
        seq.finished, seq.finish_reason = True, reason
        self.running.remove(seq)
        self.cache.free(seq.seq_id)
