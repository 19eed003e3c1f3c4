"""Sliding-window attention whose values are its keys, over a paged key cache.

The layer keeps one cache tensor [num_blocks, block_size, kv_heads, dim] (no value half), scores
query i against the keys j of its window 0 <= i - j < window with an optional linear distance
bias slope_h * (i - j) and an optional query temperature that grows with the logarithm of the
position, and gates the concatenated heads with a sigmoid before the output projection.  Every
parameter is a constructor argument; `None` / 0 switch a term off.  Prompts, portions of prompts
and decode steps are one case: the step's keys are written to the cache, then every row reads
its window from there (csrc/seq_window_attention.hip: matrix-core kernels for 16-bit models --
tiles of 32 rows for runs of rows, all heads of a KV group at once for single rows -- and fp32
kernels for any dtype and head size).
"""
import os
from typing import List, Optional, Tuple

import torch
import torch.nn as nn

from vllm_legacy_amd import _seq_ops as ops
from vllm_legacy_amd.attention.batch import SequenceBatch


def geometric_slopes(num_heads: int, span: float = 8.0) -> List[float]:
    """slope_h = 2^(-span (h + 1) / H), h = 0 .. H - 1."""
    return [2.0**(-span * (h + 1) / num_heads) for h in range(num_heads)]


class WindowedKeyAttention(nn.Module):
    # steps whose longest run of rows is at least this long take the tiled kernel (16-bit models)
    TILE_MIN_QUERY = int(os.environ.get("VLA_TILE_MIN_QUERY", "4"))

    def __init__(self, num_heads: int, num_kv_heads: int, head_dim: int, scale: float,
                 window: Optional[int] = None, slopes: Optional[List[float]] = None,
                 temp_coef: float = 0.0, temp_every: float = 1.0, device=None) -> None:
        super().__init__()
        assert num_heads % num_kv_heads == 0
        self.num_heads, self.num_kv_heads, self.head_dim = num_heads, num_kv_heads, head_dim
        self.scale = float(scale)
        self.window = int(window) if window else 0
        self.temp_coef, self.temp_every = float(temp_coef), float(temp_every)
        self.register_buffer("slopes", None if slopes is None else
                             torch.tensor(slopes, dtype=torch.float32, device=device), persistent=False)

    @staticmethod
    def get_cache_shape(num_blocks: int, block_size: int, num_kv_heads: int,
                        head_dim: int) -> Tuple[int, ...]:
        return (num_blocks, block_size, num_kv_heads, head_dim)

    def forward(self, out: torch.Tensor, q: torch.Tensor, k: torch.Tensor, gate: Optional[torch.Tensor],
                cache: torch.Tensor, batch: SequenceBatch, out_scale: float = 1.0) -> torch.Tensor:
        """q, gate, out [T, H * D] and k [T, G * D]: views with free row strides.  Writes k into
        the cache, then attends; returns out (gated and scaled, in the activation dtype)."""
        ops.key_cache_write(cache, k, batch.slot_mapping)
        if batch.max_query_len >= self.TILE_MIN_QUERY and ops.window_attention_tiles_supported(q, self.head_dim):
            # a step with runs of rows (prompts, portions): 32-row tiles on the matrix cores
            ops.window_attention_tiles(out, q, gate, cache, batch.block_tables, batch.query_start_loc,
                                       batch.context_lens, batch.max_query_len, self.slopes, self.num_heads,
                                       self.window, self.scale, self.temp_coef, self.temp_every, out_scale)
        else:
            ops.window_attention(out, q, gate, cache, batch.block_tables, batch.token_seq, batch.positions,
                                 self.slopes, self.num_heads, self.window, self.scale, self.temp_coef,
                                 self.temp_every, out_scale)
        return out
