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


# ---------------------------------------------------------------- layers with norms on both sides
ACT = {"none": 0, "relu": 1, "relu2": 2, "silu": 3, "gelu_tanh": 4}


def residual_norms(x: torch.Tensor, y: Optional[torch.Tensor] = None, y_bias: Optional[torch.Tensor] = None,
                   post_weight: Optional[torch.Tensor] = None,
                   layer_scale: Optional[torch.Tensor] = None, add_row: Optional[torch.Tensor] = None,
                   out: Optional[torch.Tensor] = None, pre_weight: Optional[torch.Tensor] = None,
                   eps: float = 1e-5) -> None:
    """x (fp32 [T, W], in place) += y' / rms(y') * post_weight * layer_scale with y' = y + y_bias;
    x += add_row; out = x / rms(x) * pre_weight (pre_weight None: out = x).  Each part is optional."""
    _gpu(x, y, y_bias, post_weight, layer_scale, add_row, out, pre_weight)
    T, W = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous()
    for v in (y_bias, post_weight, layer_scale, add_row, pre_weight):
        assert v is None or (v.dtype == torch.float32 and v.numel() == W and v.is_contiguous())
    if y is not None:
        assert y.shape == x.shape and post_weight is not None
    if out is not None:
        assert out.shape == x.shape and out.is_contiguous()
    with torch.cuda.device(x.device):
        seq_check(_lib.seq_lib().vla_seq_residual_norms(
            x.data_ptr(), _p(y), 0 if y is None else _rows(y, W), _lib.F32 if y is None else _dt(y.dtype),
            _p(y_bias), _p(post_weight), _p(layer_scale), _p(add_row), _p(out), _p(pre_weight), float(eps), T, W,
            _lib.F32 if out is None else _dt(out.dtype), _stream(x.device)), "residual_norms")


def causal_conv(out: torch.Tensor, h: torch.Tensor, weight: torch.Tensor, state: Optional[torch.Tensor],
                query_start_loc: torch.Tensor, context_lens: torch.Tensor, state_slots: torch.Tensor,
                token_seq: torch.Tensor) -> None:
    """out = h + conv(h) along time per channel; h fp32 [T, W]; weight fp32 [W, taps]; state fp32
    [slots, taps - 1, W] holds every sequence's last inputs and is brought up to date."""
    _gpu(out, h, weight, state, query_start_loc, context_lens, state_slots, token_seq)
    T, W = h.shape
    taps = weight.shape[1]
    B = context_lens.numel()
    assert h.dtype == torch.float32 and h.is_contiguous() and out.is_contiguous() and out.shape == h.shape
    assert weight.dtype == torch.float32 and weight.is_contiguous() and weight.shape[0] == W
    slots = 0
    if taps > 1:
        assert state is not None and state.dtype == torch.float32 and state.is_contiguous()
        assert state.shape[1:] == (taps - 1, W)
        slots = state.shape[0]
    for t in (query_start_loc, context_lens, state_slots, token_seq):
        assert t.dtype == torch.int32 and t.is_contiguous()
    assert query_start_loc.numel() == B + 1 and state_slots.numel() == B and token_seq.numel() == T
    with torch.cuda.device(h.device):
        seq_check(_lib.seq_lib().vla_seq_causal_conv(
            out.data_ptr(), h.data_ptr(), weight.data_ptr(), _p(state), query_start_loc.data_ptr(),
            context_lens.data_ptr(), state_slots.data_ptr(), token_seq.data_ptr(), T, B, slots, W, taps,
            _dt(out.dtype), _stream(h.device)), "causal_conv")


def concat_cast(out: torch.Tensor, a: torch.Tensor, b: torch.Tensor) -> None:
    _gpu(out, a, b)
    T, W = a.shape
    assert a.dtype == b.dtype == torch.float32 and a.is_contiguous() and b.is_contiguous() and b.shape == a.shape
    assert out.shape == (T, 2 * W) and out.is_contiguous()
    with torch.cuda.device(a.device):
        seq_check(_lib.seq_lib().vla_seq_concat_cast(out.data_ptr(), a.data_ptr(), b.data_ptr(), T, W,
                                                     _dt(out.dtype), _stream(a.device)), "concat_cast")


def gated_act(out: torch.Tensor, gate: torch.Tensor, up: Optional[torch.Tensor], act: str) -> None:
    """out = act(gate) * up (up None: act(gate)); [T, F] views with free row strides."""
    _gpu(out, gate, up)
    T, F = gate.shape
    assert out.shape == gate.shape and out.dtype == gate.dtype and (up is None or (up.shape == gate.shape and up.dtype == gate.dtype))
    with torch.cuda.device(gate.device):
        seq_check(_lib.seq_lib().vla_seq_gated_act(
            out.data_ptr(), _rows(out, F), gate.data_ptr(), _rows(gate, F), _p(up),
            0 if up is None else _rows(up, F), T, F, ACT[act], _dt(gate.dtype), _stream(gate.device)), "gated_act")


def clamped_glu(out: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, limit: float, alpha: float,
                shift: float) -> None:
    """out = g * sigmoid(alpha g) * (u + shift), g = min(gate, limit), u = clamp(up, -limit, limit);
    [T, F] views with free row strides."""
    _gpu(out, gate, up)
    T, F = gate.shape
    assert out.shape == gate.shape == up.shape and out.dtype == gate.dtype == up.dtype
    with torch.cuda.device(gate.device):
        seq_check(_lib.seq_lib().vla_seq_clamped_glu(
            out.data_ptr(), _rows(out, F), gate.data_ptr(), _rows(gate, F), up.data_ptr(), _rows(up, F), T, F,
            float(limit), float(alpha), float(shift), _dt(gate.dtype), _stream(gate.device)), "clamped_glu")


def pair_hash_embed(out: torch.Tensor, table: torch.Tensor, pair_table: torch.Tensor, ids: torch.Tensor,
                    last_token: torch.Tensor, query_start_loc: torch.Tensor, context_lens: torch.Tensor,
                    state_slots: torch.Tensor, token_seq: torch.Tensor, mul_prev: int, mul_cur: int) -> None:
    """out fp32 [T, W] = table[ids] + pair_table[(prev * mul_prev + id * mul_cur) mod buckets], the
    table's last row (number buckets) for a sequence's first token; last_token int64 [slots] holds
    every sequence's last token between steps and is brought up to date."""
    _gpu(out, table, pair_table, ids, last_token, query_start_loc, context_lens, state_slots, token_seq)
    T, W = out.shape
    B = context_lens.numel()
    assert out.dtype == torch.float32 and out.is_contiguous()
    assert table.is_contiguous() and pair_table.is_contiguous() and table.dtype == pair_table.dtype
    assert table.shape[1] == W and pair_table.shape[1] == W and pair_table.shape[0] >= 2
    assert ids.dtype == torch.int64 and ids.numel() == T and ids.is_contiguous()
    assert last_token.dtype == torch.int64 and last_token.is_contiguous() and last_token.dim() == 1
    for t in (query_start_loc, context_lens, state_slots, token_seq):
        assert t.dtype == torch.int32 and t.is_contiguous()
    assert query_start_loc.numel() == B + 1 and state_slots.numel() == B and token_seq.numel() == T
    with torch.cuda.device(out.device):
        seq_check(_lib.seq_lib().vla_seq_pair_hash_embed(
            out.data_ptr(), table.data_ptr(), pair_table.data_ptr(), ids.data_ptr(), last_token.data_ptr(),
            query_start_loc.data_ptr(), context_lens.data_ptr(), state_slots.data_ptr(), token_seq.data_ptr(), T, B,
            last_token.numel(), W, table.shape[0], pair_table.shape[0] - 1, int(mul_prev), int(mul_cur),
            _dt(table.dtype), _stream(out.device)), "pair_hash_embed")


def rotary_kv_write(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, key_cache: torch.Tensor,
                    value_cache: torch.Tensor, positions: torch.Tensor, slot_mapping: torch.Tensor,
                    inv_freq: Optional[torch.Tensor], value_inv_freq: Optional[torch.Tensor], heads: int,
                    rot_dims: int, interleaved: bool, q_norm: Optional[torch.Tensor] = None,
                    k_norm: Optional[torch.Tensor] = None, norm_eps: float = 0.0,
                    v_other: Optional[torch.Tensor] = None, v_blend: Optional[torch.Tensor] = None) -> None:
    """q [T, H*D] rotated in place; k [T, G*D], v [T, G*V] rotated into the caches
    [NB, BS, G, D] / [NB, BS, G, V].  q_norm fp32 [H*D] / k_norm fp32 [G*D]: the whole query / key
    row is RMS-normed with these weights before the rotation.  v_other [T, G*V] with v_blend (fp32,
    one number on the device): the cached value is (1 - v_blend) v + v_blend v_other."""
    _gpu(q, k, v, key_cache, value_cache, positions, slot_mapping, inv_freq, value_inv_freq, q_norm, k_norm,
         v_other, v_blend)
    NB, BS, G, D = key_cache.shape
    V = value_cache.shape[3]
    T = q.shape[0]
    assert value_cache.shape[:3] == (NB, BS, G) and key_cache.is_contiguous() and value_cache.is_contiguous()
    assert q.dtype == k.dtype == v.dtype == key_cache.dtype == value_cache.dtype
    assert positions.dtype == torch.int64 and positions.numel() == T and positions.is_contiguous()
    assert slot_mapping.dtype == torch.int64 and slot_mapping.numel() == T and slot_mapping.is_contiguous()
    if rot_dims:
        assert inv_freq.dtype == torch.float32 and inv_freq.numel() == rot_dims // 2 and inv_freq.is_contiguous()
    if value_inv_freq is not None:
        assert value_inv_freq.dtype == torch.float32 and value_inv_freq.numel() == V // 2
    assert q_norm is None or (q_norm.dtype == torch.float32 and q_norm.numel() == heads * D and q_norm.is_contiguous())
    assert k_norm is None or (k_norm.dtype == torch.float32 and k_norm.numel() == G * D and k_norm.is_contiguous())
    if v_other is not None:
        assert v_other.dtype == v.dtype and v_other.shape == v.shape and value_inv_freq is None
        assert v_blend is not None and v_blend.dtype == torch.float32 and v_blend.numel() == 1
    with torch.cuda.device(q.device):
        seq_check(_lib.seq_lib().vla_seq_rotary_kv_write(
            q.data_ptr(), _rows(q, heads * D), k.data_ptr(), _rows(k, G * D), v.data_ptr(), _rows(v, G * V),
            key_cache.data_ptr(), value_cache.data_ptr(), positions.data_ptr(), slot_mapping.data_ptr(),
            _p(inv_freq), _p(value_inv_freq), T, heads, G, D, V, int(rot_dims), int(bool(interleaved)), BS, NB,
            _dt(q.dtype), _p(q_norm), _p(k_norm), float(norm_eps), _p(v_other),
            0 if v_other is None else _rows(v_other, G * V), _p(v_blend), _stream(q.device)), "rotary_kv_write")


def kv_attention(out: torch.Tensor, q: torch.Tensor, gate: Optional[torch.Tensor], key_cache: torch.Tensor,
                 value_cache: torch.Tensor, block_tables: torch.Tensor, token_seq: torch.Tensor,
                 positions: torch.Tensor, out_inv_freq: Optional[torch.Tensor], interleaved: bool, heads: int,
                 window: int, scale: float, keep_first: int = 0, softcap: float = 0.0) -> None:
    """out [T, H*V] = softmax attention of q [T, H*D] over the caches, output pairs turned back by
    the position, times sigmoid(gate [T, H]).  With a window the first keep_first tokens of a
    sequence stay visible; softcap > 0 caps the scores with softcap * tanh(score / softcap)."""
    _gpu(out, q, gate, key_cache, value_cache, block_tables, token_seq, positions, out_inv_freq)
    NB, BS, G, D = key_cache.shape
    V = value_cache.shape[3]
    T = q.shape[0]
    assert key_cache.is_contiguous() and value_cache.is_contiguous()
    assert key_cache.dtype == value_cache.dtype == q.dtype == out.dtype
    assert block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous()
    assert token_seq.dtype == torch.int32 and token_seq.numel() == T and token_seq.is_contiguous()
    assert positions.dtype == torch.int64 and positions.numel() == T and positions.is_contiguous()
    if out_inv_freq is not None:
        assert out_inv_freq.dtype == torch.float32 and out_inv_freq.numel() == V // 2
    if gate is not None:
        assert gate.dtype == q.dtype
    with torch.cuda.device(q.device):
        seq_check(_lib.seq_lib().vla_seq_kv_attention(
            out.data_ptr(), _rows(out, heads * V), q.data_ptr(), _rows(q, heads * D), _p(gate),
            0 if gate is None else _rows(gate, heads), key_cache.data_ptr(), value_cache.data_ptr(),
            block_tables.data_ptr(), block_tables.shape[1], token_seq.data_ptr(), positions.data_ptr(),
            _p(out_inv_freq), int(bool(interleaved)), T, heads, G, D, V, BS, NB, int(window), float(scale),
            _dt(q.dtype), int(keep_first), float(softcap), _stream(q.device)), "kv_attention")


def set_kv_attention_kernel(mode: int) -> None:
    """0: kv_attention picks its kernel per shape; 1: never the matrix-core kernels."""
    seq_check(_lib.seq_lib().vla_seq_set_kv_attention_kernel(mode), "set_kv_attention_kernel")


def kv_attention_tiles_supported(q: torch.Tensor, head_dim: int, value_dim: int) -> bool:
    """Whether the matrix-core kernel for runs of query rows takes this query tensor."""
    return bool(_lib.seq_lib().vla_seq_kv_attention_tiles_supported(head_dim, value_dim, _dt(q.dtype))) and \
        q.data_ptr() % 16 == 0 and (q.stride(0) * q.element_size()) % 16 == 0


def kv_attention_tiles(out: torch.Tensor, q: torch.Tensor, gate: Optional[torch.Tensor], key_cache: torch.Tensor,
                       value_cache: torch.Tensor, block_tables: torch.Tensor, query_start_loc: torch.Tensor,
                       context_lens: torch.Tensor, max_query_len: int, out_inv_freq: Optional[torch.Tensor],
                       interleaved: bool, heads: int, window: int, scale: float, keep_first: int = 0,
                       softcap: float = 0.0) -> None:
    """The same attention as kv_attention for 16-bit activations, tiled over runs of 32 query rows
    of a sequence."""
    _gpu(out, q, gate, key_cache, value_cache, block_tables, query_start_loc, context_lens, out_inv_freq)
    NB, BS, G, D = key_cache.shape
    V = value_cache.shape[3]
    B = context_lens.numel()
    assert key_cache.is_contiguous() and value_cache.is_contiguous()
    assert key_cache.dtype == value_cache.dtype == q.dtype == out.dtype
    for t in (block_tables, query_start_loc, context_lens):
        assert t.dtype == torch.int32 and t.is_contiguous()
    assert block_tables.dim() == 2 and block_tables.shape[0] == B and query_start_loc.numel() == B + 1
    if out_inv_freq is not None:
        assert out_inv_freq.dtype == torch.float32 and out_inv_freq.numel() == V // 2
    if gate is not None:
        assert gate.dtype == q.dtype
    with torch.cuda.device(q.device):
        seq_check(_lib.seq_lib().vla_seq_kv_attention_tiles(
            out.data_ptr(), _rows(out, heads * V), q.data_ptr(), _rows(q, heads * D), _p(gate),
            0 if gate is None else _rows(gate, heads), key_cache.data_ptr(), value_cache.data_ptr(),
            block_tables.data_ptr(), block_tables.shape[1], query_start_loc.data_ptr(), context_lens.data_ptr(),
            _p(out_inv_freq), int(bool(interleaved)), B, int(max_query_len), heads, G, D, V, BS, NB, int(window),
            float(scale), _dt(q.dtype), int(keep_first), float(softcap), _stream(q.device)), "kv_attention_tiles")


def mingru_scan(out: torch.Tensor, zp: torch.Tensor, up: torch.Tensor, gp: torch.Tensor, state: torch.Tensor,
                query_start_loc: torch.Tensor, context_lens: torch.Tensor, state_slots: torch.Tensor,
                max_query_len: int) -> None:
    """out, zp, up, gp: [T, R] views; state fp32 [slots, R]."""
    _gpu(out, zp, up, gp, state, query_start_loc, context_lens, state_slots)
    T, R = zp.shape
    B = context_lens.numel()
    assert state.dtype == torch.float32 and state.is_contiguous() and state.shape[1] == R
    assert out.dtype == zp.dtype == up.dtype == gp.dtype
    for t in (query_start_loc, context_lens, state_slots):
        assert t.dtype == torch.int32 and t.is_contiguous()
    L = _lib.seq_lib()
    need = L.vla_seq_mingru_scratch_floats(B, int(max_query_len), R)
    scratch = torch.empty(need, dtype=torch.float32, device=zp.device) if need else None
    with torch.cuda.device(zp.device):
        seq_check(L.vla_seq_mingru_scan(
            out.data_ptr(), _rows(out, R), zp.data_ptr(), _rows(zp, R), up.data_ptr(), _rows(up, R),
            gp.data_ptr(), _rows(gp, R), state.data_ptr(), query_start_loc.data_ptr(), context_lens.data_ptr(),
            state_slots.data_ptr(), B, state.shape[0], int(max_query_len), R, _p(scratch), need, _dt(zp.dtype),
            _stream(zp.device)), "mingru_scan")


def moe_route(h: torch.Tensor, router: torch.Tensor, correction: Optional[torch.Tensor],
              shared_gate_weight: Optional[torch.Tensor], top: int, logits: Optional[torch.Tensor] = None,
              bias: Optional[torch.Tensor] = None):
    """-> experts int32 [T, top], weights fp32 [T, top], shared gate fp32 [T] or None.  logits
    (fp32 [T, routed (+ 1, the shared gate's last)]): the router products, when the caller formed
    them as one matrix product."""
    _gpu(h, router, correction, shared_gate_weight, logits, bias)
    T, W = h.shape
    N = router.shape[0]
    assert bias is None or (bias.dtype == torch.float32 and bias.numel() == N and bias.is_contiguous())
    assert router.dtype == torch.float32 and router.is_contiguous() and router.shape[1] == W
    assert correction is None or (correction.dtype == torch.float32 and correction.numel() == N)
    assert shared_gate_weight is None or (shared_gate_weight.dtype == torch.float32 and shared_gate_weight.numel() == W)
    if logits is not None:
        assert logits.dtype == torch.float32 and logits.is_contiguous()
        assert logits.shape == (T, N + (0 if shared_gate_weight is None else 1))
    experts = torch.empty((T, top), dtype=torch.int32, device=h.device)
    weights = torch.empty((T, top), dtype=torch.float32, device=h.device)
    sg = None if shared_gate_weight is None else torch.empty((T, ), dtype=torch.float32, device=h.device)
    with torch.cuda.device(h.device):
        seq_check(_lib.seq_lib().vla_seq_moe_route(
            h.data_ptr(), _rows(h, W), router.data_ptr(), _p(logits), 0 if logits is None else logits.shape[1],
            _p(bias), _p(correction), _p(shared_gate_weight), experts.data_ptr(), weights.data_ptr(), _p(sg), T, W, N,
            int(top), _dt(h.dtype), _stream(h.device)), "moe_route")
    return experts, weights, sg


def moe_plan(experts: torch.Tensor, num_experts: int):
    """-> pair_row int32 [T, top], row_token int32 [rows], tile_expert int32 [tiles]."""
    _gpu(experts)
    T, top = experts.shape
    L = _lib.seq_lib()
    tile = L.vla_seq_moe_tile_rows()
    max_tiles = (T * top + (tile - 1) * min(num_experts, T * top) + tile - 1) // tile
    pair_row = torch.empty((T, top), dtype=torch.int32, device=experts.device)
    row_token = torch.empty((max_tiles * tile, ), dtype=torch.int32, device=experts.device)
    tile_expert = torch.empty((max_tiles, ), dtype=torch.int32, device=experts.device)
    assert experts.dtype == torch.int32 and experts.is_contiguous()
    with torch.cuda.device(experts.device):
        seq_check(L.vla_seq_moe_plan(experts.data_ptr(), T, top, int(num_experts), pair_row.data_ptr(),
                                     row_token.data_ptr(), tile_expert.data_ptr(), max_tiles,
                                     _stream(experts.device)), "moe_plan")
    return pair_row, row_token, tile_expert


def grouped_linear(out: torch.Tensor, a: torch.Tensor, row_token: Optional[torch.Tensor], weight: torch.Tensor,
                   tile_expert: torch.Tensor, act: str = "none") -> None:
    """out [tiles * tile rows, N] = act(weight[e] a[src(row)]); weight [E, N, K]; a rows of K."""
    _gpu(out, a, row_token, weight, tile_expert)
    E, N, K = weight.shape
    assert weight.is_contiguous() and weight.dtype == a.dtype and a.shape[1] == K
    L = _lib.seq_lib()
    tiles = tile_expert.numel()
    assert out.shape == (tiles * L.vla_seq_moe_tile_rows(), N) and out.is_contiguous()
    assert row_token is None or (row_token.dtype == torch.int32 and row_token.numel() == out.shape[0])
    if row_token is None:
        assert a.shape[0] == out.shape[0]
    with torch.cuda.device(a.device):
        seq_check(L.vla_seq_grouped_linear(
            out.data_ptr(), N, _dt(out.dtype), a.data_ptr(), _rows(a, K), _p(row_token), weight.data_ptr(),
            tile_expert.data_ptr(), tiles, N, K, ACT[act], _dt(a.dtype), _stream(a.device)), "grouped_linear")


def set_grouped_linear_form(mode: int) -> None:
    """0: grouped_linear picks its 16-bit form per shape; 1: one-wave workgroups; 2: runs of tiles."""
    seq_check(_lib.seq_lib().vla_seq_set_grouped_linear_form(mode), "set_grouped_linear_form")


def moe_combine(out: torch.Tensor, y: torch.Tensor, pair_row: torch.Tensor, weights: torch.Tensor,
                h: torch.Tensor, shared_y: Optional[torch.Tensor], shared_gate: Optional[torch.Tensor]) -> None:
    _gpu(out, y, pair_row, weights, h, shared_y, shared_gate)
    T, W = h.shape
    top = pair_row.shape[1]
    assert out.dtype == torch.float32 and out.shape == (T, W) and out.is_contiguous()
    assert y.dtype == torch.float32 and y.is_contiguous() and y.shape[1] == W
    assert shared_y is None or (shared_y.dtype == torch.float32 and shared_y.is_contiguous() and shared_y.shape == (T, W))
    with torch.cuda.device(h.device):
        seq_check(_lib.seq_lib().vla_seq_moe_combine(
            out.data_ptr(), y.data_ptr(), pair_row.data_ptr(), weights.data_ptr(), h.data_ptr(), _rows(h, W),
            _p(shared_y), _p(shared_gate), T, W, top, _dt(h.dtype), _stream(h.device)), "moe_combine")


# ---------------------------------------------------------------- layers that norm the stream itself
def post_norm(x: torch.Tensor, y: torch.Tensor, weight: torch.Tensor, alpha: float, eps: float,
              out: Optional[torch.Tensor] = None) -> None:
    """x (fp32 [T, W], in place) <- (alpha x + y) / rms(alpha x + y) * weight; out = the new x in
    out's dtype."""
    _gpu(x, y, weight, out)
    T, W = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous() and y.shape == x.shape
    assert weight.dtype == torch.float32 and weight.numel() == W and weight.is_contiguous()
    assert out is None or (out.shape == x.shape and out.is_contiguous())
    with torch.cuda.device(x.device):
        seq_check(_lib.seq_lib().vla_seq_post_norm(
            x.data_ptr(), float(alpha), y.data_ptr(), _rows(y, W), _dt(y.dtype), weight.data_ptr(), float(eps),
            _p(out), _lib.F32 if out is None else _dt(out.dtype), T, W, _stream(x.device)), "post_norm")


def rms_norm_rows(out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, eps: float) -> None:
    """out = x / rms(x) * weight per row; [T, n] views with free row strides, any dtypes."""
    _gpu(out, x, weight)
    T, n = x.shape
    assert out.shape == x.shape and weight.dtype == torch.float32 and weight.numel() == n and weight.is_contiguous()
    with torch.cuda.device(x.device):
        seq_check(_lib.seq_lib().vla_seq_rms_norm_rows(
            out.data_ptr(), _rows(out, n), _dt(out.dtype), x.data_ptr(), _rows(x, n), _dt(x.dtype),
            weight.data_ptr(), float(eps), T, n, _stream(x.device)), "rms_norm_rows")


def short_conv(out: torch.Tensor, u: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
               state: Optional[torch.Tensor], query_start_loc: torch.Tensor, context_lens: torch.Tensor,
               state_slots: torch.Tensor, token_seq: torch.Tensor, act: str = "none") -> None:
    """out = act(bias + conv(u)) along time per channel; out, u [T, C] views with free row strides;
    weight fp32 [C, taps]; state fp32 [slots, taps - 1, C] holds every sequence's last inputs and is
    brought up to date."""
    _gpu(out, u, weight, bias, state, query_start_loc, context_lens, state_slots, token_seq)
    T, Cn = u.shape
    taps = weight.shape[1]
    B = context_lens.numel()
    assert out.shape == u.shape
    assert weight.dtype == torch.float32 and weight.is_contiguous() and weight.shape[0] == Cn
    assert bias is None or (bias.dtype == torch.float32 and bias.numel() == Cn and bias.is_contiguous())
    slots = 0
    if taps > 1:
        assert state is not None and state.dtype == torch.float32 and state.is_contiguous()
        assert state.shape[1:] == (taps - 1, Cn)
        slots = state.shape[0]
    for t in (query_start_loc, context_lens, state_slots, token_seq):
        assert t.dtype == torch.int32 and t.is_contiguous()
    assert query_start_loc.numel() == B + 1 and state_slots.numel() == B and token_seq.numel() == T
    with torch.cuda.device(u.device):
        seq_check(_lib.seq_lib().vla_seq_short_conv(
            out.data_ptr(), _rows(out, Cn), _dt(out.dtype), u.data_ptr(), _rows(u, Cn), _dt(u.dtype),
            weight.data_ptr(), _p(bias), _p(state if taps > 1 else None), query_start_loc.data_ptr(),
            context_lens.data_ptr(), state_slots.data_ptr(), token_seq.data_ptr(), T, B, slots, Cn, taps, ACT[act],
            _stream(u.device)), "short_conv")


def gated_act_lookup(out: torch.Tensor, gate: torch.Tensor, table: torch.Tensor, ids: torch.Tensor,
                     first_col: int, act: str) -> None:
    """out[t] = act(gate[t]) * table[ids[t], first_col : first_col + F]; out, gate [T, F]."""
    _gpu(out, gate, table, ids)
    T, F = gate.shape
    assert out.shape == gate.shape and table.dim() == 2 and table.stride(1) == 1
    assert ids.dtype == torch.int64 and ids.numel() == T and ids.is_contiguous()
    assert 0 <= first_col and first_col + F <= table.shape[1]
    with torch.cuda.device(gate.device):
        seq_check(_lib.seq_lib().vla_seq_gated_act_lookup(
            out.data_ptr(), _rows(out, F), _dt(out.dtype), gate.data_ptr(), _rows(gate, F), _dt(gate.dtype),
            table.data_ptr(), table.stride(0), _dt(table.dtype), ids.data_ptr(), table.shape[0], int(first_col), T, F,
            ACT[act], _stream(gate.device)), "gated_act_lookup")


def embed_scaled(out: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, scale: float) -> None:
    _gpu(out, table, ids)
    T, W = out.shape
    assert out.dtype == torch.float32 and out.is_contiguous() and table.is_contiguous() and table.shape[1] == W
    assert ids.dtype == torch.int64 and ids.numel() == T and ids.is_contiguous()
    with torch.cuda.device(out.device):
        seq_check(_lib.seq_lib().vla_seq_embed_scaled(
            out.data_ptr(), table.data_ptr(), ids.data_ptr(), float(scale), T, W, table.shape[0], _dt(table.dtype),
            _stream(out.device)), "embed_scaled")


def softcap(z: torch.Tensor, cap: float) -> None:
    """z (fp32, in place) <- cap * tanh(z / cap)."""
    _gpu(z)
    assert z.dtype == torch.float32 and z.is_contiguous()
    with torch.cuda.device(z.device):
        seq_check(_lib.seq_lib().vla_seq_softcap(z.data_ptr(), z.numel(), float(cap), _stream(z.device)), "softcap")


def delta_rule_scan(out: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, gate: torch.Tensor,
                    beta: torch.Tensor, dt: torch.Tensor, a_log: torch.Tensor, dt_bias: torch.Tensor,
                    norm_weight: torch.Tensor, state: torch.Tensor, query_start_loc: torch.Tensor,
                    context_lens: torch.Tensor, state_slots: torch.Tensor, kv_heads: int, eps: float,
                    max_query_len: int = 0) -> None:
    """out [T, H*V]; q, k fp32 [T, G*D]; v, gate fp32 [T, H*V]; beta, dt fp32 [T, H] (views with free
    row strides); a_log, dt_bias fp32 [H]; norm_weight fp32 [V]; state fp32 [slots, H, V, D]."""
    _gpu(out, q, k, v, gate, beta, dt, a_log, dt_bias, norm_weight, state, query_start_loc, context_lens, state_slots)
    slots, H, V, D = state.shape
    B = context_lens.numel()
    assert state.dtype == torch.float32 and state.is_contiguous()
    for t in (q, k, v, gate, beta, dt):
        assert t.dtype == torch.float32
    for t in (a_log, dt_bias, norm_weight):
        assert t.dtype == torch.float32 and t.is_contiguous()
    assert a_log.numel() == H and dt_bias.numel() == H and norm_weight.numel() == V
    for t in (query_start_loc, context_lens, state_slots):
        assert t.dtype == torch.int32 and t.is_contiguous()
    assert query_start_loc.numel() == B + 1 and state_slots.numel() == B
    T = q.shape[0]
    scratch = torch.empty(_lib.seq_lib().vla_seq_delta_rule_scratch_floats(T, H, V), dtype=torch.float32, device=q.device)
    with torch.cuda.device(q.device):
        seq_check(_lib.seq_lib().vla_seq_delta_rule_scan(
            out.data_ptr(), _rows(out, H * V), _dt(out.dtype), q.data_ptr(), _rows(q, kv_heads * D), k.data_ptr(),
            _rows(k, kv_heads * D), v.data_ptr(), _rows(v, H * V), gate.data_ptr(), _rows(gate, H * V),
            beta.data_ptr(), _rows(beta, H), dt.data_ptr(), _rows(dt, H), _lib.F32, a_log.data_ptr(),
            dt_bias.data_ptr(), norm_weight.data_ptr(), state.data_ptr(), query_start_loc.data_ptr(),
            context_lens.data_ptr(), state_slots.data_ptr(), T, B, int(max_query_len), slots, H, int(kv_heads), D, V,
            float(eps),
            scratch.data_ptr(), _stream(q.device)), "delta_rule_scan")


def set_delta_kernel(mode: int) -> None:
    """0: delta_rule_scan picks its kernel per step; 1: always the one without staging; 2: never."""
    seq_check(_lib.seq_lib().vla_seq_set_delta_kernel(mode), "set_delta_kernel")


def rglru_scan(out: torch.Tensor, gates: torch.Tensor, u: torch.Tensor, y: torch.Tensor,
               rate: torch.Tensor, state: torch.Tensor, query_start_loc: torch.Tensor, context_lens: torch.Tensor,
               state_slots: torch.Tensor, max_query_len: int) -> None:
    """out [T, R]; gates fp32 [blocks, T, 2 * R / blocks] contiguous (per block: the recurrence
    gate's products, then the input gate's); u, y fp32 [T, R] views; rate fp32 [R]; state fp32
    [slots, R]."""
    _gpu(out, gates, u, y, rate, state, query_start_loc, context_lens, state_slots)
    T, R = u.shape
    B = context_lens.numel()
    blocks = gates.shape[0]
    bw = R // blocks
    assert gates.dtype == torch.float32 and gates.is_contiguous() and gates.shape == (blocks, T, 2 * bw)
    assert state.dtype == torch.float32 and state.is_contiguous() and state.shape[1] == R
    for t in (u, y):
        assert t.dtype == torch.float32 and t.shape == (T, R)
    assert rate.dtype == torch.float32 and rate.numel() == R and rate.is_contiguous()
    for t in (query_start_loc, context_lens, state_slots):
        assert t.dtype == torch.int32 and t.is_contiguous()
    L = _lib.seq_lib()
    need = L.vla_seq_mingru_scratch_floats(B, int(max_query_len), R)
    scratch = torch.empty(need, dtype=torch.float32, device=u.device) if need else None
    with torch.cuda.device(u.device):
        seq_check(L.vla_seq_rglru_scan(
            out.data_ptr(), _rows(out, R), _dt(out.dtype), gates.data_ptr(), 2 * bw, gates.data_ptr() + 4 * bw,
            2 * bw, bw, T * 2 * bw, u.data_ptr(), _rows(u, R), y.data_ptr(), _rows(y, R), rate.data_ptr(),
            state.data_ptr(), query_start_loc.data_ptr(), context_lens.data_ptr(), state_slots.data_ptr(), B,
            state.shape[0], int(max_query_len), R, _p(scratch), need, _stream(u.device)), "rglru_scan")


def latent_rotary_write(q: torch.Tensor, q_head_stride: int, q_first: int, heads: int, kv: torch.Tensor,
                        norm_weight: torch.Tensor, eps: float, cache: torch.Tensor, positions: torch.Tensor,
                        slot_mapping: torch.Tensor, inv_freq: Optional[torch.Tensor], magnitude: float,
                        rot_dims: int, interleaved: bool = True) -> None:
    """q [T, >= heads * q_head_stride]: the rotated part of head h starts at column h * q_head_stride +
    q_first; kv [T, rank + rot]; cache [NB, BS, rank + rot]."""
    _gpu(q, kv, norm_weight, cache, positions, slot_mapping, inv_freq)
    NB, BS, width = cache.shape
    rank = norm_weight.numel()
    rot = width - rank
    T = q.shape[0]
    assert cache.is_contiguous() and q.dtype == kv.dtype == cache.dtype and q.stride(1) == 1
    assert kv.shape == (T, width) and norm_weight.dtype == torch.float32 and norm_weight.is_contiguous()
    assert (heads - 1) * q_head_stride + q_first + rot <= q.shape[1]
    assert positions.dtype == torch.int64 and positions.numel() == T and positions.is_contiguous()
    assert slot_mapping.dtype == torch.int64 and slot_mapping.numel() == T and slot_mapping.is_contiguous()
    if rot_dims:
        assert inv_freq.dtype == torch.float32 and inv_freq.numel() == rot_dims // 2 and inv_freq.is_contiguous()
    with torch.cuda.device(q.device):
        seq_check(_lib.seq_lib().vla_seq_latent_rotary_write(
            q.data_ptr(), q.stride(0) if T > 1 else q.shape[1], int(q_head_stride), int(q_first), kv.data_ptr(),
            _rows(kv, width), norm_weight.data_ptr(), float(eps), cache.data_ptr(), positions.data_ptr(),
            slot_mapping.data_ptr(), _p(inv_freq), float(magnitude), T, int(heads), rank, rot, int(rot_dims), BS, NB,
            _dt(q.dtype), int(bool(interleaved)), _stream(q.device)), "latent_rotary_write")


def latent_attention(out: torch.Tensor, q_lat: torch.Tensor, q_rot: torch.Tensor, cache: torch.Tensor,
                     block_tables: torch.Tensor, token_seq: torch.Tensor, positions: torch.Tensor,
                     scale: float, window: int = 0, gate: Optional[torch.Tensor] = None) -> None:
    """out, q_lat [T, H, rank] and q_rot [T, H, rot] views (any token / head strides, unit stride
    along the last axis); cache [NB, BS, rank + rot]; window > 0: keys with position - j < window
    only; gate [T, H]: a head's sums times sigmoid(gate)."""
    _gpu(out, q_lat, q_rot, cache, block_tables, token_seq, positions, gate)
    assert gate is None or gate.dtype == q_lat.dtype
    NB, BS, width = cache.shape
    T, H, rank = q_lat.shape
    rot = width - rank
    assert out.shape == q_lat.shape and q_rot.shape == (T, H, rot) and cache.is_contiguous()
    assert out.dtype == q_lat.dtype == q_rot.dtype == cache.dtype
    for t in (out, q_lat, q_rot):
        assert t.stride(2) == 1 or t.shape[2] == 1
    assert block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous()
    assert token_seq.dtype == torch.int32 and token_seq.numel() == T and token_seq.is_contiguous()
    assert positions.dtype == torch.int64 and positions.numel() == T and positions.is_contiguous()
    with torch.cuda.device(q_lat.device):
        seq_check(_lib.seq_lib().vla_seq_latent_attention(
            out.data_ptr(), out.stride(0), out.stride(1), q_lat.data_ptr(), q_lat.stride(0), q_lat.stride(1),
            q_rot.data_ptr(), q_rot.stride(0), q_rot.stride(1), cache.data_ptr(), block_tables.data_ptr(),
            block_tables.shape[1], token_seq.data_ptr(), positions.data_ptr(), T, H, rank, rot, BS, NB, float(scale),
            _dt(q_lat.dtype), int(window), _p(gate), 0 if gate is None else _rows(gate, H),
            _stream(q_lat.device)), "latent_attention")


def set_latent_attention_kernel(mode: int) -> None:
    """0: latent attention picks its kernel per shape; 1: never the matrix-core kernel."""
    seq_check(_lib.seq_lib().vla_seq_set_latent_attention_kernel(mode), "set_latent_attention_kernel")


def latent_attention_tiles_supported(q_lat: torch.Tensor, q_rot: torch.Tensor, cache: torch.Tensor) -> bool:
    """Whether the matrix-core kernel takes these query tensors and this cache."""
    rank, rot = q_lat.shape[2], q_rot.shape[2]
    ok = bool(_lib.seq_lib().vla_seq_latent_attention_tiles_supported(rank, rot, _dt(q_lat.dtype)))
    for t in (q_lat, q_rot):
        if t.shape[2] == 0:
            continue
        ok = ok and t.data_ptr() % 16 == 0 and all(t.stride(d) % 8 == 0 or t.shape[d] == 1 for d in (0, 1))
    return ok and cache.data_ptr() % 16 == 0


def latent_attention_tiles(out: torch.Tensor, q_lat: torch.Tensor, q_rot: torch.Tensor, cache: torch.Tensor,
                           block_tables: torch.Tensor, query_start_loc: torch.Tensor, context_lens: torch.Tensor,
                           max_query_len: int, scale: float, key_splits: int = 1, window: int = 0,
                           gate: Optional[torch.Tensor] = None) -> None:
    """The same attention as latent_attention for 16-bit activations on the matrix cores; rows
    query_start_loc[b] .. of sequence b sit at positions context_lens[b] ...  key_splits > 1: the
    keys of every row tile are shared out to that many workgroups and merged."""
    _gpu(out, q_lat, q_rot, cache, block_tables, query_start_loc, context_lens, gate)
    NB, BS, width = cache.shape
    T, H, rank = q_lat.shape
    rot = width - rank
    B = context_lens.numel()
    assert gate is None or gate.dtype == q_lat.dtype
    assert out.shape == q_lat.shape and q_rot.shape == (T, H, rot) and cache.is_contiguous()
    assert out.dtype == q_lat.dtype == q_rot.dtype == cache.dtype
    for t in (out, q_lat, q_rot):
        assert t.stride(2) == 1 or t.shape[2] == 1
    for t in (block_tables, query_start_loc, context_lens):
        assert t.dtype == torch.int32 and t.is_contiguous()
    assert block_tables.dim() == 2 and block_tables.shape[0] == B and query_start_loc.numel() == B + 1

    def st(t, d):       # a stride that is never used may be anything: make it pass the alignment check
        return t.stride(d) if t.shape[d] > 1 else 8 * ((t.shape[2] + 7) // 8) * (H if d == 0 else 1)

    L = _lib.seq_lib()
    need = L.vla_seq_latent_attention_scratch_floats(int(key_splits), T, H, rank)
    scratch = torch.empty(need, dtype=torch.float32, device=q_lat.device) if need else None
    with torch.cuda.device(q_lat.device):
        seq_check(L.vla_seq_latent_attention_tiles(
            out.data_ptr(), st(out, 0), st(out, 1), q_lat.data_ptr(), st(q_lat, 0), st(q_lat, 1),
            q_rot.data_ptr(), st(q_rot, 0), st(q_rot, 1), cache.data_ptr(), block_tables.data_ptr(),
            block_tables.shape[1], query_start_loc.data_ptr(), context_lens.data_ptr(), B, int(max_query_len), H, rank,
            rot, BS, NB, float(scale), int(key_splits), _p(scratch), T, _dt(q_lat.dtype), int(window), _p(gate),
            0 if gate is None else _rows(gate, H), _stream(q_lat.device)),
            "latent_attention_tiles")
