"""The elementwise layers on either side of attention, on the gfx950 library.

Host-side mirrors of the reference's RMSNorm (vllm/model_executor/layers/layernorm.py:11-71),
RotaryEmbedding (vllm/model_executor/layers/rotary_embedding.py:47-170: cos/sin cache in the
model dtype, [max_position, rot_dim], cos half then sin half) and SiluAndMul
(vllm/model_executor/layers/activation.py:15-38).  forward() always runs the HIP kernels; there
is no eager fallback.
"""
from typing import Optional, Tuple, Union

import torch
import torch.nn as nn

from vllm_legacy_amd import _custom_ops as ops
from vllm_legacy_amd import _seq_ops as seq_ops
from vllm_legacy_amd.distributed.communication_op import (
    PendingAllReduce, tensor_model_parallel_all_reduce_add_rms_norm)


class RMSNorm(nn.Module):

    def __init__(self, hidden_size: int, eps: float = 1e-6, dtype=torch.float16, device=None):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size, dtype=dtype, device=device),
                                   requires_grad=False)
        self.variance_epsilon = eps

    def forward(self, x, residual: Optional[torch.Tensor] = None
                ) -> Union[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]]:
        if isinstance(x, PendingAllReduce):
            # a row-parallel linear's output under tensor parallelism: the all-reduce happens here
            assert residual is not None
            return tensor_model_parallel_all_reduce_add_rms_norm(x, residual, self.weight.data,
                                                                 self.variance_epsilon)
        if isinstance(x, ops.SplitKSlabs):
            # the producing GEMM left its split-K partial sums for this kernel to add up
            assert residual is not None
            out = torch.empty_like(residual)
            ops.fused_add_rms_norm_splitk(x, out, residual, self.weight.data,
                                          self.variance_epsilon)
            return out, residual
        if residual is not None:
            ops.fused_add_rms_norm(x, residual, self.weight.data, self.variance_epsilon)
            return x, residual
        out = torch.empty_like(x)
        ops.rms_norm(out, x, self.weight.data, self.variance_epsilon)
        return out


class RotaryEmbedding(nn.Module):

    def __init__(self, head_size: int, rotary_dim: int, max_position_embeddings: int, base: float,
                 is_neox_style: bool, dtype=torch.float16, device=None):
        super().__init__()
        self.head_size, self.rotary_dim, self.is_neox_style = head_size, rotary_dim, is_neox_style
        inv_freq = 1.0 / (base**(torch.arange(0, rotary_dim, 2, dtype=torch.float32, device=device)
                                 / rotary_dim))
        t = torch.arange(max_position_embeddings, dtype=torch.float32, device=device)
        freqs = torch.outer(t, inv_freq)
        self.register_buffer("cos_sin_cache",
                             torch.cat([freqs.cos(), freqs.sin()], dim=-1).to(dtype),
                             persistent=False)

    def forward(self, positions: torch.Tensor, query: torch.Tensor,
                key: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        ops.rotary_embedding(positions, query, key, self.head_size, self.cos_sin_cache,
                             self.is_neox_style)
        return query, key


class SiluAndMul(nn.Module):

    def forward(self, x, dtype: torch.dtype = torch.float16) -> torch.Tensor:
        if isinstance(x, ops.SplitKSlabs):
            # the merged gate|up GEMM left its split-K partial sums for this kernel to add up
            out = torch.empty((x.m, x.n // 2), dtype=dtype, device=x.workspace.device)
            ops.silu_and_mul_splitk(x, out)
            return out
        d = x.shape[-1] // 2
        out = torch.empty(x.shape[:-1] + (d, ), dtype=x.dtype, device=x.device)
        ops.silu_and_mul(out, x)
        return out


class ScalarRMSNorm(nn.Module):
    """RMS norm of an fp32 residual stream with one gain for all coordinates:
    out = x / sqrt(mean(x^2) + eps) * g, written in `out_dtype`.  add_rows ([T, W] fp32) and
    add_row ([W] fp32) are added to the stream first, in place (the additions that open a pass
    over looped layers ride in this launch)."""

    def __init__(self, eps: float, device=None):
        super().__init__()
        self.weight = nn.Parameter(torch.ones((), dtype=torch.float32, device=device),
                                   requires_grad=False)
        self.variance_epsilon = float(eps)

    def forward(self, x: torch.Tensor, out_dtype: torch.dtype, add_rows: Optional[torch.Tensor] = None,
                add_row: Optional[torch.Tensor] = None) -> torch.Tensor:
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        seq_ops.scalar_rms_norm(out, x, self.weight.data.view(1), self.variance_epsilon, add_rows,
                                add_row)
        return out


class PolyNorm(nn.Module):
    """out = c0 N(z) + c1 N(z^2) + c2 N(z^3) + c3, powers element by element, N(u) = u divided by
    the root mean square of a token's vector u (eps inside the root)."""

    def __init__(self, eps: float, device=None):
        super().__init__()
        self.weight = nn.Parameter(torch.tensor([1.0, 0.0, 0.0, 0.0], dtype=torch.float32,
                                                device=device), requires_grad=False)
        self.variance_epsilon = float(eps)

    def forward(self, z: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        if out is None:
            out = torch.empty(z.shape, dtype=z.dtype, device=z.device)
        seq_ops.poly_norm(out, z, self.weight.data, self.variance_epsilon)
        return out


class SinusoidalEmbedding(nn.Module):
    """Token embedding plus the sinusoidal position vector (entry 2i sin, entry 2i + 1 cos of
    p * base^(-2i / width)), written as the fp32 residual stream."""

    def __init__(self, vocab_size: int, width: int, dtype=torch.bfloat16, device=None,
                 base: float = 10000.0):
        super().__init__()
        self.weight = nn.Parameter(torch.zeros((vocab_size, width), dtype=dtype, device=device),
                                   requires_grad=False)
        i2 = torch.arange(0, width, 2, dtype=torch.float32)
        inv_freq = torch.pow(torch.tensor(base, dtype=torch.float32), -i2 / width)
        self.register_buffer("inv_freq", inv_freq.to(device), persistent=False)

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        out = torch.empty((input_ids.numel(), self.weight.shape[1]), dtype=torch.float32,
                          device=self.weight.device)
        seq_ops.embed_positions(out, self.weight.data, input_ids, positions, self.inv_freq)
        return out


class CausalConvMix(nn.Module):
    """h + conv(h): a causal convolution over time on each channel (weight [width, taps], no bias,
    tap j reads the input taps - 1 - j tokens back), added to its input.  The last taps - 1 inputs
    of every sequence live in a state slot [num_slots, taps - 1, width] (fp32), so a sequence may be
    cut anywhere.  Reads the fp32 rows a norm left and writes the activation dtype."""

    def __init__(self, width: int, taps: int, device=None):
        super().__init__()
        self.taps = int(taps)
        self.weight = nn.Parameter(torch.zeros((width, taps), dtype=torch.float32, device=device),
                                   requires_grad=False)

    @staticmethod
    def get_state_shape(num_slots: int, width: int, taps: int) -> Tuple[int, ...]:
        return (num_slots, max(taps - 1, 0), width)

    def forward(self, h: torch.Tensor, state: Optional[torch.Tensor], batch, out_dtype: torch.dtype) -> torch.Tensor:
        out = torch.empty(h.shape, dtype=out_dtype, device=h.device)
        seq_ops.causal_conv(out, h, self.weight.data, state if self.taps > 1 else None, batch.query_start_loc,
                            batch.context_lens, batch.state_slots, batch.token_seq)
        return out


class ShortConv(nn.Module):
    """act(bias + conv(u)): a causal convolution over time on each channel (weight [channels, taps],
    the last column weighs the current token, zeros before a sequence's start), with an optional
    bias and activation.  The last taps - 1 inputs of every sequence live in a state slot
    [num_slots, taps - 1, channels] (fp32), so a sequence may be cut anywhere.  Input and output are
    views with free row strides, of any dtype."""

    def __init__(self, channels: int, taps: int, bias: bool = False, act: str = "none", device=None):
        super().__init__()
        if act not in seq_ops.ACT:
            raise ValueError(f"unknown activation {act!r}")
        self.channels, self.taps, self.act = int(channels), int(taps), act
        self.weight = nn.Parameter(torch.zeros((channels, taps), dtype=torch.float32, device=device),
                                   requires_grad=False)
        self.bias = nn.Parameter(torch.zeros(channels, dtype=torch.float32, device=device),
                                 requires_grad=False) if bias else None

    @staticmethod
    def get_state_shape(num_slots: int, channels: int, taps: int) -> Tuple[int, ...]:
        return (num_slots, max(taps - 1, 0), channels)

    def forward(self, out: torch.Tensor, u: torch.Tensor, state: Optional[torch.Tensor], batch) -> torch.Tensor:
        seq_ops.short_conv(out, u, self.weight.data, None if self.bias is None else self.bias.data,
                           state if self.taps > 1 else None, batch.query_start_loc, batch.context_lens,
                           batch.state_slots, batch.token_seq, self.act)
        return out


class TokenGatedInput(nn.Module):
    """A per-token side input to an fp32 stream: with e the token's row of a side embedding table
    (columns first_col .. first_col + dim - 1), g = act(W_gate x) * e, y = W_proj g,
    x += y / rms(y) * weight.  Returns the new stream in the activation dtype as well (what the next
    sublayer's projections read)."""

    def __init__(self, width: int, dim: int, first_col: int, eps: float, act: str = "gelu_tanh",
                 dtype=torch.bfloat16, device=None):
        super().__init__()
        self.dim, self.first_col, self.eps, self.act, self.dtype = int(dim), int(first_col), float(eps), act, dtype
        self.gate = nn.Parameter(torch.zeros((dim, width), dtype=dtype, device=device), requires_grad=False)
        self.proj = nn.Parameter(torch.zeros((width, dim), dtype=dtype, device=device), requires_grad=False)
        self.weight = nn.Parameter(torch.ones(width, dtype=torch.float32, device=device), requires_grad=False)

    def forward(self, x: torch.Tensor, h: torch.Tensor, table: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
        """x fp32 [T, width] (in place), h the same rows in the activation dtype; table the side
        embedding [vocab, columns]."""
        gate = torch.mm(h, self.gate.data.t())
        g = torch.empty_like(gate)
        seq_ops.gated_act_lookup(g, gate, table, ids, self.first_col, self.act)
        y = torch.mm(g, self.proj.data.t()) if g.dtype == torch.float32 else \
            torch.mm(g, self.proj.data.t(), out_dtype=torch.float32)
        seq_ops.residual_norms(x, y, None, self.weight.data, None, None, h, None, self.eps)
        return h


class GatedActivation(nn.Module):
    """act(gate) * up on the two halves of a merged projection [T, 2 F] (gate | up), or act(z) on
    a plain one; act: relu, relu2 (the square of relu), silu, gelu_tanh.  The gated form
    "clamped_glu" is g sigmoid(alpha g) (u + shift) with g = min(gate, limit) and
    u = clamp(up, -limit, limit)."""

    def __init__(self, act: str, gated: bool = True, limit: float = 0.0, alpha: float = 1.702, shift: float = 1.0):
        super().__init__()
        if act == "clamped_glu":
            if not (gated and limit > 0):
                raise ValueError("clamped_glu is a gated activation with a positive limit")
        elif act not in seq_ops.ACT or act == "none":
            raise ValueError(f"unknown activation {act!r}")
        self.act, self.gated = act, gated
        self.limit, self.alpha, self.shift = float(limit), float(alpha), float(shift)

    def forward(self, z: torch.Tensor) -> torch.Tensor:
        F = z.shape[1] // 2 if self.gated else z.shape[1]
        out = torch.empty((z.shape[0], F), dtype=z.dtype, device=z.device)
        if self.act == "clamped_glu":
            seq_ops.clamped_glu(out, z[:, :F], z[:, F:], self.limit, self.alpha, self.shift)
        else:
            seq_ops.gated_act(out, z[:, :F], z[:, F:] if self.gated else None, self.act)
        return out


class PairHashEmbedding(nn.Module):
    """Token embedding plus a hashed embedding of the (previous token, token) pair, written as the
    fp32 stream: row (prev * mul_prev + token * mul_cur) mod buckets of a second table, its last row
    (number `buckets`) for a sequence's first token.  A sequence's last token lives in a state slot
    (int64 [num_slots]) between steps, so a sequence may be cut anywhere."""

    def __init__(self, vocab_size: int, width: int, buckets: int, mul_prev: int, mul_cur: int,
                 dtype=torch.bfloat16, device=None):
        super().__init__()
        if buckets < 1 or mul_prev < 0 or mul_cur < 0:
            raise ValueError("buckets must be positive and the multipliers non-negative")
        self.buckets, self.mul_prev, self.mul_cur = int(buckets), int(mul_prev), int(mul_cur)
        self.weight = nn.Parameter(torch.zeros((vocab_size, width), dtype=dtype, device=device),
                                   requires_grad=False)
        self.pair_weight = nn.Parameter(torch.zeros((buckets + 1, width), dtype=dtype, device=device),
                                        requires_grad=False)

    @staticmethod
    def get_state_shape(num_slots: int) -> Tuple[int, ...]:
        return (num_slots, )

    def forward(self, input_ids: torch.Tensor, last_token: torch.Tensor, batch) -> torch.Tensor:
        out = torch.empty((input_ids.numel(), self.weight.shape[1]), dtype=torch.float32,
                          device=self.weight.device)
        seq_ops.pair_hash_embed(out, self.weight.data, self.pair_weight.data, input_ids, last_token,
                                batch.query_start_loc, batch.context_lens, batch.state_slots, batch.token_seq,
                                self.mul_prev, self.mul_cur)
        return out
