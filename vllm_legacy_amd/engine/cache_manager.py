"""Cache manager: hands out the blocks of the paged cache and the slots of the recurrent state.

One pool of `num_blocks` blocks of `block_size` tokens serves every layer run (a block id means
the same block in each run's tensor, as in the reference's block manager,
vllm/core/block_manager_v1.py), and one pool of `num_slots` state slots serves every recurrent
layer.  Freed blocks and slots go back on a stack and are the first to be handed out again, so a
long-running engine keeps reusing the same few; nothing is cleared on reuse (the kernels never
read a cache position the sequence has not written, and a sequence that starts ignores what its
slot held)."""
from typing import Dict, List


class CacheManager:

    def __init__(self, num_blocks: int, block_size: int, num_slots: int) -> None:
        assert num_blocks > 0 and block_size > 0 and num_slots > 0
        self.num_blocks, self.block_size, self.num_slots = num_blocks, block_size, num_slots
        self._free_blocks: List[int] = list(range(num_blocks - 1, -1, -1))
        self._free_slots: List[int] = list(range(num_slots - 1, -1, -1))
        self._tables: Dict[str, List[int]] = {}
        self._slots: Dict[str, int] = {}

    # ---------------------------------------------------------------- queries
    @property
    def free_blocks(self) -> int:
        return len(self._free_blocks)

    @property
    def free_slots(self) -> int:
        return len(self._free_slots)

    def blocks_needed(self, seq_id: str, total_tokens: int) -> int:
        have = len(self._tables.get(seq_id, ()))
        return max(0, (total_tokens + self.block_size - 1) // self.block_size - have)

    def can_admit(self, total_tokens: int) -> bool:
        return (self.free_slots > 0 and
                (total_tokens + self.block_size - 1) // self.block_size <= self.free_blocks)

    def can_grow(self, seq_id: str, total_tokens: int) -> bool:
        return self.blocks_needed(seq_id, total_tokens) <= self.free_blocks

    # ---------------------------------------------------------------- changes
    def admit(self, seq_id: str) -> int:
        """Give a new sequence a state slot and an empty block table."""
        if seq_id in self._slots:
            raise KeyError(f"sequence {seq_id!r} is already live")
        if not self._free_slots:
            raise RuntimeError("no free state slot")
        self._slots[seq_id] = self._free_slots.pop()
        self._tables[seq_id] = []
        return self._slots[seq_id]

    def grow(self, seq_id: str, total_tokens: int) -> List[int]:
        """Make the sequence's table cover total_tokens; returns the table."""
        table = self._tables[seq_id]
        need = self.blocks_needed(seq_id, total_tokens)
        if need > len(self._free_blocks):
            raise RuntimeError(f"out of cache blocks: {need} needed, {len(self._free_blocks)} free")
        for _ in range(need):
            table.append(self._free_blocks.pop())
        return table

    def free(self, seq_id: str) -> None:
        for b in reversed(self._tables.pop(seq_id)):
            self._free_blocks.append(b)
        self._free_slots.append(self._slots.pop(seq_id))

    def is_live(self, seq_id: str) -> bool:
        return seq_id in self._slots

    def block_table(self, seq_id: str) -> List[int]:
        return self._tables[seq_id]

    def state_slot(self, seq_id: str) -> int:
        return self._slots[seq_id]
