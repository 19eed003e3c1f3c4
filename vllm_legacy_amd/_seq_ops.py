"""Python face of libvla_seq_gfx950.so (include/vla_sequence_ops.h): the row-wise layers of an
fp32 residual stream, sliding-window attention over a paged key cache, and the gated linear
recurrence.  Tensors stay torch tensors; raw pointers, sizes and the current HIP stream cross into
the library.  There is no eager fallback: without a GPU these raise."""
from typing import Optional

import torch

from . import _lib
from ._lib import seq_check

_DTYPE = {torch.float16: _lib.F16, torch.bfloat16: _lib.BF16, torch.float32: _lib.F32}


def _dt(dtype: torch.dtype) -> int:
    try:
        return _DTYPE[dtype]
    except KeyError:
        raise RuntimeError(f"Unsupported activation dtype: {dtype}") from None


def _stream(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def _gpu(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise RuntimeError("expected a tensor on the GPU")


def _rows(t: torch.Tensor, cols: int) -> int:
    """Row stride of a [T, cols] view whose rows may be slices of a wider matrix."""
    assert t.dim() == 2 and t.shape[1] == cols and (t.stride(1) == 1 or cols == 1), (t.shape, t.stride())
    return t.stride(0) if t.shape[0] > 1 else max(t.stride(0), cols)


def _p(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def embed_positions(out: torch.Tensor, table: torch.Tensor, ids: torch.Tensor,
                    positions: torch.Tensor, inv_freq: Optional[torch.Tensor]) -> None:
    _gpu(out, table, ids, positions, inv_freq)
    T, W = out.shape
    assert out.dtype == torch.float32 and out.is_contiguous() and table.is_contiguous()
    assert table.shape[1] == W and ids.dtype == torch.int64 and positions.dtype == torch.int64
    assert ids.numel() == T and positions.numel() == T and ids.is_contiguous() and positions.is_contiguous()
    if inv_freq is not None:
        assert inv_freq.dtype == torch.float32 and inv_freq.numel() >= (W + 1) // 2 and inv_freq.is_contiguous()
    with torch.cuda.device(out.device):
        seq_check(_lib.seq_lib().vla_seq_embed_positions(
            out.data_ptr(), table.data_ptr(), ids.data_ptr(), positions.data_ptr(), _p(inv_freq), T, W,
            table.shape[0], _dt(table.dtype), _stream(out.device)), "embed_positions")


def scalar_rms_norm(out: torch.Tensor, x: torch.Tensor, gain: torch.Tensor, eps: float,
                    add_rows: Optional[torch.Tensor] = None,
                    add_row: Optional[torch.Tensor] = None) -> None:
    """x (fp32, in place) += add_rows + add_row; out = x / sqrt(mean(x^2) + eps) * gain."""
    _gpu(out, x, gain, add_rows, add_row)
    T, W = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous() and out.is_contiguous() and out.shape == x.shape
    assert gain.dtype == torch.float32 and gain.numel() == 1
    if add_rows is not None:
        assert add_rows.dtype == torch.float32 and add_rows.is_contiguous() and add_rows.shape == x.shape
    if add_row is not None:
        assert add_row.dtype == torch.float32 and add_row.is_contiguous() and add_row.numel() == W
    with torch.cuda.device(x.device):
        seq_check(_lib.seq_lib().vla_seq_scalar_rms_norm(
            out.data_ptr(), x.data_ptr(), _p(add_rows), _p(add_row), gain.data_ptr(), eps, T, W,
            _dt(out.dtype), _stream(x.device)), "scalar_rms_norm")


def residual_add(x: torch.Tensor, y: torch.Tensor) -> None:
    _gpu(x, y)
    assert x.dtype == torch.float32 and x.is_contiguous() and y.is_contiguous() and x.numel() == y.numel()
    with torch.cuda.device(x.device):
        seq_check(_lib.seq_lib().vla_seq_residual_add(x.data_ptr(), y.data_ptr(), x.numel(),
                                                      _dt(y.dtype), _stream(x.device)), "residual_add")


def poly_norm(out: torch.Tensor, z: torch.Tensor, coef: torch.Tensor, eps: float) -> None:
    """out, z: [T, F] views (row strides free) of the activation dtype; coef fp32 [4]."""
    _gpu(out, z, coef)
    T, F = z.shape
    assert out.shape == z.shape and out.dtype == z.dtype
    assert coef.dtype == torch.float32 and coef.numel() == 4 and coef.is_contiguous()
    with torch.cuda.device(z.device):
        seq_check(_lib.seq_lib().vla_seq_poly_norm(out.data_ptr(), _rows(out, F), z.data_ptr(), _rows(z, F),
                                                   coef.data_ptr(), eps, T, F, _dt(z.dtype),
                                                   _stream(z.device)), "poly_norm")


def gated_head_rms_norm(out: torch.Tensor, o: torch.Tensor, weight: torch.Tensor, gate: torch.Tensor,
                        eps: float, scale: float) -> None:
    """o fp32 [T, H, V] -> out [T, H*V] = o / rms_V(o) * weight * silu(gate) * scale."""
    _gpu(out, o, weight, gate)
    T, H, V = o.shape
    assert o.dtype == torch.float32 and o.is_contiguous()
    assert weight.dtype == torch.float32 and weight.numel() == V and weight.is_contiguous()
    assert out.dtype == gate.dtype
    with torch.cuda.device(o.device):
        seq_check(_lib.seq_lib().vla_seq_gated_head_rms_norm(
            out.data_ptr(), _rows(out, H * V), o.data_ptr(), weight.data_ptr(), gate.data_ptr(),
            _rows(gate, H * V), eps, scale, T, H, V, _dt(out.dtype), _stream(o.device)),
            "gated_head_rms_norm")


def key_cache_write(cache: torch.Tensor, k: torch.Tensor, slot_mapping: torch.Tensor) -> None:
    """cache [NB, BS, G, D]; k [T, G*D] (row stride free); slot_mapping int64 [T]."""
    _gpu(cache, k, slot_mapping)
    NB, BS, G, D = cache.shape
    assert cache.is_contiguous() and cache.dtype == k.dtype
    assert slot_mapping.dtype == torch.int64 and slot_mapping.is_contiguous() and slot_mapping.numel() == k.shape[0]
    with torch.cuda.device(k.device):
        seq_check(_lib.seq_lib().vla_seq_key_cache_write(
            cache.data_ptr(), k.data_ptr(), _rows(k, G * D), slot_mapping.data_ptr(), k.shape[0], G, D, BS,
            NB, _dt(k.dtype), _stream(k.device)), "key_cache_write")


def window_attention(out: torch.Tensor, q: torch.Tensor, gate: Optional[torch.Tensor], cache: torch.Tensor,
                     block_tables: torch.Tensor, token_seq: torch.Tensor, positions: torch.Tensor,
                     slopes: Optional[torch.Tensor], heads: int, window: int, scale: float,
                     temp_coef: float = 0.0, temp_every: float = 1.0, out_scale: float = 1.0) -> None:
    _gpu(out, q, gate, cache, block_tables, token_seq, positions, slopes)
    NB, BS, G, D = cache.shape
    T = q.shape[0]
    assert cache.is_contiguous() and cache.dtype == q.dtype == out.dtype
    assert block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous()
    assert token_seq.dtype == torch.int32 and token_seq.numel() == T and token_seq.is_contiguous()
    assert positions.dtype == torch.int64 and positions.numel() == T and positions.is_contiguous()
    if slopes is not None:
        assert slopes.dtype == torch.float32 and slopes.numel() == heads and slopes.is_contiguous()
    if gate is not None:
        assert gate.dtype == q.dtype
    with torch.cuda.device(q.device):
        seq_check(_lib.seq_lib().vla_seq_window_attention(
            out.data_ptr(), _rows(out, heads * D), q.data_ptr(), _rows(q, heads * D), _p(gate),
            0 if gate is None else _rows(gate, heads * D), cache.data_ptr(), block_tables.data_ptr(),
            block_tables.shape[1], token_seq.data_ptr(), positions.data_ptr(), _p(slopes), T, heads, G, D, BS,
            NB, int(window), float(scale), float(temp_coef), float(temp_every), float(out_scale),
            _dt(q.dtype), _stream(q.device)), "window_attention")


def set_window_kernel(mode: int) -> None:
    """0: window_attention picks its kernel per shape; 1: always one wave per (row, head)."""
    seq_check(_lib.seq_lib().vla_seq_set_window_kernel(mode), "set_window_kernel")


def set_scan_kernel(mode: int) -> None:
    """0: gla_scan picks its kernel per shape; 1: always the token-by-token kernel."""
    seq_check(_lib.seq_lib().vla_seq_set_scan_kernel(mode), "set_scan_kernel")


def window_attention_tiles_supported(q: torch.Tensor, head_dim: int) -> bool:
    """Whether the matrix-core kernel for runs of query rows takes this query tensor."""
    return bool(_lib.seq_lib().vla_seq_window_attention_tiles_supported(head_dim, _dt(q.dtype))) and \
        q.data_ptr() % 8 == 0 and (q.stride(0) * q.element_size()) % 8 == 0


def window_attention_tiles(out: torch.Tensor, q: torch.Tensor, gate: Optional[torch.Tensor],
                           cache: torch.Tensor, block_tables: torch.Tensor, query_start_loc: torch.Tensor,
                           context_lens: torch.Tensor, max_query_len: int, slopes: Optional[torch.Tensor],
                           heads: int, window: int, scale: float, temp_coef: float = 0.0,
                           temp_every: float = 1.0, out_scale: float = 1.0) -> None:
    """The same attention as window_attention for 16-bit activations, tiled over runs of 32
    query rows of a sequence (rows query_start_loc[b] .. of sequence b sit at positions
    context_lens[b] ..)."""
    _gpu(out, q, gate, cache, block_tables, query_start_loc, context_lens, slopes)
    NB, BS, G, D = cache.shape
    B = context_lens.numel()
    assert cache.is_contiguous() and cache.dtype == q.dtype == out.dtype
    for t in (block_tables, query_start_loc, context_lens):
        assert t.dtype == torch.int32 and t.is_contiguous()
    assert block_tables.dim() == 2 and block_tables.shape[0] == B and query_start_loc.numel() == B + 1
    if slopes is not None:
        assert slopes.dtype == torch.float32 and slopes.numel() == heads and slopes.is_contiguous()
    with torch.cuda.device(q.device):
        seq_check(_lib.seq_lib().vla_seq_window_attention_tiles(
            out.data_ptr(), _rows(out, heads * D), q.data_ptr(), _rows(q, heads * D), _p(gate),
            0 if gate is None else _rows(gate, heads * D), cache.data_ptr(), block_tables.data_ptr(),
            block_tables.shape[1], query_start_loc.data_ptr(), context_lens.data_ptr(), _p(slopes), B,
            int(max_query_len), heads, G, D, BS, NB, int(window), float(scale), float(temp_coef),
            float(temp_every), float(out_scale), _dt(q.dtype), _stream(q.device)), "window_attention_tiles")


def gla_log_decay(out: torch.Tensor, y: torch.Tensor, w2: torch.Tensor, bias: Optional[torch.Tensor],
                  inv_tau: float) -> None:
    """out fp32 [T, C] = ln(sigmoid(y @ w2^T + bias)) * inv_tau; y [T, R], w2 [C, R]."""
    _gpu(out, y, w2, bias)
    T, R = y.shape
    Cn = w2.shape[0]
    assert out.dtype == torch.float32 and out.is_contiguous() and out.shape == (T, Cn)
    assert w2.is_contiguous() and w2.shape[1] == R and w2.dtype == y.dtype
    if bias is not None:
        assert bias.dtype == torch.float32 and bias.numel() == Cn and bias.is_contiguous()
    with torch.cuda.device(y.device):
        seq_check(_lib.seq_lib().vla_seq_gla_log_decay(out.data_ptr(), y.data_ptr(), _rows(y, R), w2.data_ptr(),
                                                       _p(bias), inv_tau, T, Cn, R, _dt(y.dtype),
                                                       _stream(y.device)), "gla_log_decay")


def gla_scan(o: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, log_decay: torch.Tensor,
             state: torch.Tensor, query_start_loc: torch.Tensor, context_lens: torch.Tensor,
             state_slots: torch.Tensor, q_scale: float, max_query_len: int = 0) -> None:
    """o fp32 [T, H, V]; q, k [T, H*D]; v [T, H*V]; log_decay fp32 [T, H*D]; state fp32
    [slots, H, D, V]; query_start_loc int32 [B+1], context_lens / state_slots int32 [B]."""
    _gpu(o, q, k, v, log_decay, state, query_start_loc, context_lens, state_slots)
    slots, H, D, V = state.shape
    T = q.shape[0]
    B = context_lens.numel()
    assert o.dtype == torch.float32 and o.is_contiguous() and o.shape == (T, H, V)
    assert state.dtype == torch.float32 and state.is_contiguous()
    assert log_decay.dtype == torch.float32 and log_decay.is_contiguous() and log_decay.shape == (T, H * D)
    assert q.dtype == k.dtype == v.dtype
    for t in (query_start_loc, context_lens, state_slots):
        assert t.dtype == torch.int32 and t.is_contiguous()
    assert query_start_loc.numel() == B + 1 and state_slots.numel() == B
    with torch.cuda.device(q.device):
        seq_check(_lib.seq_lib().vla_seq_gla_scan(
            o.data_ptr(), q.data_ptr(), _rows(q, H * D), k.data_ptr(), _rows(k, H * D), v.data_ptr(),
            _rows(v, H * V), log_decay.data_ptr(), state.data_ptr(), query_start_loc.data_ptr(),
            context_lens.data_ptr(), state_slots.data_ptr(), float(q_scale), B, slots, int(max_query_len), H, D, V,
            _dt(q.dtype), _stream(q.device)), "gla_scan")


def gla_piece_prefix(q_decayed: torch.Tensor, totals: torch.Tensor, q: torch.Tensor, log_decay: torch.Tensor,
                     piece_start_loc: torch.Tensor, q_scale: float) -> None:
    """q_decayed fp32 [T, C] = q * q_scale * exp(running sum of log_decay within each piece);
    totals fp32 [pieces, C] = exp(the piece's whole sum)."""
    _gpu(q_decayed, totals, q, log_decay, piece_start_loc)
    T, Cn = log_decay.shape
    P = piece_start_loc.numel() - 1
    assert q_decayed.dtype == torch.float32 and q_decayed.is_contiguous() and q_decayed.shape == (T, Cn)
    assert totals.dtype == torch.float32 and totals.is_contiguous() and totals.shape == (P, Cn)
    assert log_decay.dtype == torch.float32 and log_decay.is_contiguous()
    assert piece_start_loc.dtype == torch.int32 and piece_start_loc.is_contiguous()
    with torch.cuda.device(q.device):
        seq_check(_lib.seq_lib().vla_seq_gla_piece_prefix(
            q_decayed.data_ptr(), totals.data_ptr(), q.data_ptr(), _rows(q, Cn), log_decay.data_ptr(),
            piece_start_loc.data_ptr(), float(q_scale), P, Cn, _dt(q.dtype), _stream(q.device)), "gla_piece_prefix")


def gla_combine_states(state: torch.Tensor, slots: torch.Tensor, pieces: torch.Tensor, totals: torch.Tensor,
                       final_slot: int) -> None:
    _gpu(state, slots, pieces, totals)
    n, H, D, V = state.shape
    assert state.dtype == torch.float32 and state.is_contiguous() and totals.dtype == torch.float32
    assert totals.is_contiguous() and totals.shape[1] == H * D
    for t in (slots, pieces):
        assert t.dtype == torch.int32 and t.is_contiguous()
    assert slots.numel() == pieces.numel()
    with torch.cuda.device(state.device):
        seq_check(_lib.seq_lib().vla_seq_gla_combine_states(
            state.data_ptr(), slots.data_ptr(), pieces.data_ptr(), totals.data_ptr(), slots.numel(),
            int(final_slot), n, H, D, V, _stream(state.device)), "gla_combine_states")
