"""Gated linear attention as a recurrent layer with per-sequence state slots.

Per head S_t = diag(a_t) S_(t-1) + k_t v_t^T and o_t = S_t^T q_t, with a decay per key channel
a_t = sigmoid(z_t)^(1 / tau) from a low-rank projection z_t = W2 y_t + b.  The state lives in an
fp32 tensor [num_slots, heads, dim, vdim] that the engine's cache manager hands out by slot; a
sequence whose context length is 0 starts from zero whatever its slot held before.  The output of
each head is RMS-normed over vdim, gated with silu and scaled before the output projection.
Kernels: csrc/seq_linear_recurrence.hip, csrc/seq_stream_kernels.hip.
"""
from typing import Optional, Tuple

import torch
import torch.nn as nn

from vllm_legacy_amd import _seq_ops as ops
from vllm_legacy_amd.attention.batch import SequenceBatch


class GatedLinearRecurrence(nn.Module):

    def __init__(self, num_heads: int, head_dim: int, value_dim: int, tau: float, eps: float,
                 q_scale: Optional[float] = None) -> None:
        super().__init__()
        self.num_heads, self.head_dim, self.value_dim = num_heads, head_dim, value_dim
        self.inv_tau, self.eps = 1.0 / float(tau), float(eps)
        self.q_scale = head_dim**-0.5 if q_scale is None else float(q_scale)

    @staticmethod
    def get_state_shape(num_slots: int, num_heads: int, head_dim: int,
                        value_dim: int) -> Tuple[int, ...]:
        return (num_slots, num_heads, head_dim, value_dim)

    def forward(self, out: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                gate: torch.Tensor, y: torch.Tensor, w2: torch.Tensor, bias: Optional[torch.Tensor],
                norm_weight: torch.Tensor, state: torch.Tensor, batch: SequenceBatch,
                out_scale: float = 1.0) -> torch.Tensor:
        """q, k [T, H*D]; v, gate, out [T, H*V]; y [T, R] (views with free row strides);
        w2 [H*D, R]; bias fp32 [H*D]; norm_weight fp32 [V]."""
        T, H, D, V = q.shape[0], self.num_heads, self.head_dim, self.value_dim
        log_decay = torch.empty((T, H * D), dtype=torch.float32, device=q.device)
        ops.gla_log_decay(log_decay, y, w2, bias, self.inv_tau)
        o = torch.empty((T, H, V), dtype=torch.float32, device=q.device)
        ops.gla_scan(o, q, k, v, log_decay, state, batch.query_start_loc, batch.context_lens,
                     batch.state_slots, self.q_scale, batch.max_query_len)
        ops.gated_head_rms_norm(out, o, norm_weight, gate, self.eps, out_scale)
        return out
