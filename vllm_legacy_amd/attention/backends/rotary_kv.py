"""Causal softmax attention over paged key and value caches with rotary positions.

The layer keeps two cache tensors, keys [num_blocks, block_size, kv_heads, dim] and values
[num_blocks, block_size, kv_heads, vdim].  Queries and keys are rotated over their first `rot_dims`
elements (pairs (2i, 2i + 1) when interleaved, (i, i + rot_dims / 2) otherwise, pair i by
position * base^(-2i / rot_dims)).  With `rotate_values` the value of position j is rotated by j
over all vdim elements before it is cached (pair m by j * base^(-2m / vdim)) and a head's output
at position i is turned back by i, so that what a query reads of a value depends on their
distance.  An optional window keeps 0 <= i - j < window, and with `keep_first` also every j <
keep_first (a sequence's first tokens stay visible, at their true positions); `softcap` replaces a
score s by softcap * tanh(s / softcap); `freq_scale` divides every rotary frequency (linear position
scaling); `norm_rows` norms the whole query row and the whole key row (all heads at once, RMS with
a weight per element) before the rotation; an optional gate multiplies each head's output by the
sigmoid of one number per (token, head); forward's `v_other` / `v_blend` cache
(1 - v_blend) v + v_blend v_other instead of v (values blended with another layer's values of the
same tokens).  Every parameter is a constructor argument.  Prompts, portions of prompts and decode steps are one case: the step's keys and values
are written to the caches, then every row reads from there (csrc/seq_kv_attention.hip: matrix-core
kernels for 16-bit models whose head sizes are multiples of 32 -- tiles of 32 rows for runs of
rows, all heads of a KV group at once for single rows -- and an fp32 kernel for any dtype and head
size).
"""
from typing import Optional, Tuple

import torch
import torch.nn as nn

from vllm_legacy_amd import _seq_ops as ops
from vllm_legacy_amd.attention.batch import SequenceBatch


def inverse_frequencies(base: float, span: int, device=None, divide_by: float = 1.0) -> torch.Tensor:
    """base^(-2i / span) / divide_by, i = 0 .. span / 2 - 1: formed in float64, rounded once to fp32."""
    i = torch.arange(span // 2, dtype=torch.float64)
    f = torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / float(span)) / float(divide_by)
    return f.to(torch.float32).to(device)


class RotaryKVAttention(nn.Module):
    # steps whose longest run of rows is at least this long take the tiled kernel (16-bit models)
    TILE_MIN_QUERY = 4

    def __init__(self, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int, scale: float,
                 rot_dims: int, rot_base: float, interleaved: bool = True, rotate_values: bool = False,
                 window: Optional[int] = None, device=None, keep_first: int = 0, softcap: float = 0.0,
                 freq_scale: float = 1.0, norm_rows: bool = False, norm_eps: float = 1e-5) -> None:
        super().__init__()
        assert num_heads % num_kv_heads == 0 and 0 <= rot_dims <= head_dim and rot_dims % 2 == 0
        assert not rotate_values or value_dim % 2 == 0
        assert keep_first >= 0 and softcap >= 0.0 and freq_scale > 0.0
        self.keep_first = int(keep_first) if window else 0
        self.softcap, self.norm_eps = float(softcap), float(norm_eps)
        self.q_norm = nn.Parameter(torch.ones(num_heads * head_dim, dtype=torch.float32, device=device),
                                   requires_grad=False) if norm_rows else None
        self.k_norm = nn.Parameter(torch.ones(num_kv_heads * head_dim, dtype=torch.float32, device=device),
                                   requires_grad=False) if norm_rows else None
        self.num_heads, self.num_kv_heads = num_heads, num_kv_heads
        self.head_dim, self.value_dim = head_dim, value_dim
        self.scale, self.rot_dims, self.interleaved = float(scale), int(rot_dims), bool(interleaved)
        self.window = int(window) if window else 0
        self.register_buffer("inv_freq",
                             inverse_frequencies(rot_base, rot_dims, device, freq_scale) if rot_dims else None,
                             persistent=False)
        self.register_buffer("value_inv_freq",
                             inverse_frequencies(rot_base, value_dim, device) if rotate_values else None,
                             persistent=False)

    @staticmethod
    def get_cache_shapes(num_blocks: int, block_size: int, num_kv_heads: int, head_dim: int,
                         value_dim: int) -> Tuple[Tuple[int, ...], Tuple[int, ...]]:
        return ((num_blocks, block_size, num_kv_heads, head_dim),
                (num_blocks, block_size, num_kv_heads, value_dim))

    def forward(self, out: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                gate: Optional[torch.Tensor], key_cache: torch.Tensor, value_cache: torch.Tensor,
                batch: SequenceBatch, v_other: Optional[torch.Tensor] = None,
                v_blend: Optional[torch.Tensor] = None) -> torch.Tensor:
        """q [T, H * D] (normed and rotated in place), k [T, G * D], v [T, G * V], gate [T, H], out
        [T, H * V], v_other [T, G * V]: views with free row strides; v_blend one fp32 number on the
        device."""
        ops.rotary_kv_write(q, k, v, key_cache, value_cache, batch.positions, batch.slot_mapping,
                            self.inv_freq, self.value_inv_freq, self.num_heads, self.rot_dims, self.interleaved,
                            None if self.q_norm is None else self.q_norm.data,
                            None if self.k_norm is None else self.k_norm.data, self.norm_eps, v_other, v_blend)
        if batch.max_query_len >= self.TILE_MIN_QUERY and \
                ops.kv_attention_tiles_supported(q, self.head_dim, self.value_dim):
            # a step with runs of rows (prompts, portions): 32-row tiles on the matrix cores
            ops.kv_attention_tiles(out, q, gate, key_cache, value_cache, batch.block_tables,
                                   batch.query_start_loc, batch.context_lens, batch.max_query_len,
                                   self.value_inv_freq, self.interleaved, self.num_heads, self.window, self.scale,
                                   self.keep_first, self.softcap)
        else:
            ops.kv_attention(out, q, gate, key_cache, value_cache, batch.block_tables, batch.token_seq,
                             batch.positions, self.value_inv_freq, self.interleaved, self.num_heads, self.window,
                             self.scale, self.keep_first, self.softcap)
        return out
