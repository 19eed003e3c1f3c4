"""Step metadata of a packed batch in which every sequence brings any number of new tokens.

A prompt, a portion of a prompt and a decode step are the same thing here: sequence b continues
`context_lens[b]` cached tokens with the rows `query_start_loc[b] : query_start_loc[b + 1]` of
the step.  The layers that keep their history in a paged key cache or in a recurrent state slot
(attention/backends/windowed_keys.py, attention/recurrent.py) read nothing else.
Gfx950PagedAttentionMetadata (prompts first, decode tokens after them) describes the special case
the paged-attention decode kernels take; `SequenceBatch.build` is what an engine calls per step.
"""
from dataclasses import dataclass
from typing import List, Optional, Sequence

import torch


@dataclass
class SequenceBatch:
    num_seqs: int
    num_tokens: int
    positions: torch.Tensor         # int64 [T] position of each row in its sequence
    slot_mapping: torch.Tensor      # int64 [T] cache slot (block * block_size + offset) of each row
    token_seq: torch.Tensor         # int32 [T] batch index of each row's sequence
    query_start_loc: torch.Tensor   # int32 [B + 1]
    context_lens: torch.Tensor      # int32 [B] tokens cached before this step
    block_tables: torch.Tensor      # int32 [B, max_blocks]
    state_slots: torch.Tensor       # int32 [B] recurrent-state slot of each sequence
    max_query_len: int
    max_seq_len: int                # longest context + query of the step
    # host copies of the per-sequence numbers, for layers that plan their launches on the host
    host_query_lens: Optional[List[int]] = None
    host_context_lens: Optional[List[int]] = None
    host_state_slots: Optional[List[int]] = None

    @staticmethod
    def build(query_lens: Sequence[int], context_lens: Sequence[int],
              block_tables: Sequence[Sequence[int]], state_slots: Sequence[int], block_size: int,
              device) -> "SequenceBatch":
        """From host lists, one entry per sequence.  Every sequence's table must cover
        context + query tokens; everything is checked here, on the host, because the kernels
        trust it."""
        B = len(query_lens)
        assert B == len(context_lens) == len(block_tables) == len(state_slots) and B > 0
        positions: List[int] = []
        slots: List[int] = []
        token_seq: List[int] = []
        starts = [0]
        max_blocks = 1
        for b in range(B):
            n, c, table = int(query_lens[b]), int(context_lens[b]), block_tables[b]
            assert n > 0 and c >= 0
            need = (c + n + block_size - 1) // block_size
            assert len(table) >= need, "block table shorter than the sequence"
            max_blocks = max(max_blocks, need)
            for p in range(c, c + n):
                positions.append(p)
                slots.append(int(table[p // block_size]) * block_size + p % block_size)
                token_seq.append(b)
            starts.append(starts[-1] + n)
        tables = torch.zeros((B, max_blocks), dtype=torch.int32)
        for b in range(B):
            need = (int(context_lens[b]) + int(query_lens[b]) + block_size - 1) // block_size
            tables[b, :need] = torch.as_tensor(list(block_tables[b][:need]), dtype=torch.int32)

        def dev(x, dtype):
            return torch.as_tensor(x, dtype=dtype).to(device, non_blocking=True)

        return SequenceBatch(
            num_seqs=B, num_tokens=starts[-1], positions=dev(positions, torch.int64),
            slot_mapping=dev(slots, torch.int64), token_seq=dev(token_seq, torch.int32),
            query_start_loc=dev(starts, torch.int32), context_lens=dev(list(context_lens), torch.int32),
            block_tables=tables.to(device, non_blocking=True),
            state_slots=dev(list(state_slots), torch.int32), max_query_len=max(query_lens),
            max_seq_len=max(int(c) + int(n) for c, n in zip(context_lens, query_lens)),
            host_query_lens=[int(n) for n in query_lens], host_context_lens=[int(c) for c in context_lens],
            host_state_slots=[int(x) for x in state_slots])
