"""Gated linear attention as a recurrent layer with per-sequence state slots.

Per head S_t = diag(a_t) S_(t-1) + k_t v_t^T and o_t = S_t^T q_t, with a decay per key channel
a_t = sigmoid(z_t)^(1 / tau) from a low-rank projection z_t = W2 y_t + b.  The state lives in an
fp32 tensor [num_slots, heads, dim, vdim] that the engine's cache manager hands out by slot; a
sequence whose context length is 0 starts from zero whatever its slot held before.  The output of
each head is RMS-normed over vdim, gated with silu and scaled before the output projection.

A long run of rows (a prompt, a large portion) is cut into pieces of PIECE_ROWS rows that are
walked at the same time, each from a zero state in a scratch slot behind the sequences' slots;
the state a piece should have started from then reaches its outputs through one batched matrix
product (o_t += (q_t exp(c_t))^T S_start, c_t the log decays summed from the piece's first row)
and the pieces' states are chained by a cheap walk.  The result is the long walk's, to rounding.
Kernels: csrc/seq_linear_recurrence.hip, csrc/seq_stream_kernels.hip.
"""
import os
from typing import Optional, Tuple

import torch
import torch.nn as nn

from vllm_legacy_amd import _seq_ops as ops
from vllm_legacy_amd.attention.batch import SequenceBatch


class GatedLinearRecurrence(nn.Module):
    # rows of a piece; runs of at least two pieces are cut (VLA_GLA_PIECE_ROWS: another size, for studies)
    PIECE_ROWS = int(os.environ.get("VLA_GLA_PIECE_ROWS", "256"))
    SCRATCH_SLOTS = 64      # state slots behind the sequences' own, for the pieces of a step

    def __init__(self, num_heads: int, head_dim: int, value_dim: int, tau: float, eps: float,
                 q_scale: Optional[float] = None) -> None:
        super().__init__()
        self.num_heads, self.head_dim, self.value_dim = num_heads, head_dim, value_dim
        self.inv_tau, self.eps = 1.0 / float(tau), float(eps)
        self.q_scale = head_dim**-0.5 if q_scale is None else float(q_scale)

    @staticmethod
    def get_state_shape(num_slots: int, num_heads: int, head_dim: int,
                        value_dim: int) -> Tuple[int, ...]:
        """num_slots sequence slots, then SCRATCH_SLOTS slots that only live within a step."""
        return (num_slots + GatedLinearRecurrence.SCRATCH_SLOTS, num_heads, head_dim, value_dim)

    def _plan_pieces(self, batch: SequenceBatch, num_slots: int):
        """None when no run of the step is long enough (or scratch would not suffice); else
        (piece_start_loc, piece_context, piece_slots, [per cut sequence: (first piece, count, own
        slot, first row)])."""
        q, c, sl = batch.host_query_lens, batch.host_context_lens, batch.host_state_slots
        L = self.PIECE_ROWS
        if q is None or max(q) < 2 * L:
            return None
        # the plan depends on the step and on where the scratch slots start, not on the layer:
        # it is made (and copied to the device, in one transfer) once per step
        cache = batch.__dict__.setdefault("_piece_plans", {})
        key = (num_slots, L)
        if key not in cache:
            cache[key] = self._make_plan(q, c, sl, L, num_slots, batch.positions.device)
        return cache[key]

    def _make_plan(self, q, c, sl, L, num_slots, device):
        first_scratch = num_slots - self.SCRATCH_SLOTS
        starts, ctx, slots, cut, row, scratch = [0], [], [], [], 0, first_scratch
        for n, cb, sb in zip(q, c, sl):
            if n < 2 * L:
                ctx.append(cb)
                slots.append(sb)
                starts.append(starts[-1] + n)
            else:
                count = (n + L - 1) // L
                if scratch + count > num_slots:
                    return None
                cut.append((len(ctx), count, sb, row, cb))
                for i in range(count):
                    ctx.append(cb if i == 0 else 0)
                    slots.append(scratch + i)
                    starts.append(starts[-1] + min(L, n - i * L))
                scratch += count
            row += n
        # one int32 transfer: piece_start_loc | piece contexts | piece slots | 0 .. pieces - 1
        flat = torch.tensor(starts + ctx + slots + list(range(len(ctx))), dtype=torch.int32).to(device)
        n = len(ctx)
        dev = (flat[:n + 1], flat[n + 1:2 * n + 1], flat[2 * n + 1:3 * n + 1], flat[3 * n + 1:])
        return starts, ctx, slots, cut, dev

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
        plan = self._plan_pieces(batch, state.shape[0])
        if plan is None:
            ops.gla_scan(o, q, k, v, log_decay, state, batch.query_start_loc, batch.context_lens,
                         batch.state_slots, self.q_scale, batch.max_query_len)
        else:
            self._scan_in_pieces(o, q, k, v, log_decay, state, plan)
        ops.gated_head_rms_norm(out, o, norm_weight, gate, self.eps, out_scale)
        return out

    def _scan_in_pieces(self, o, q, k, v, log_decay, state, plan) -> None:
        starts, ctx, slots, cut, (start_loc, ctx_dev, slots_dev, index_dev) = plan
        dev, L = q.device, self.PIECE_ROWS
        H, D, V = self.num_heads, self.head_dim, self.value_dim
        for first, count, own, row, cb in cut:      # a continuing sequence starts from its state
            if cb > 0:
                state[slots[first]].copy_(state[own])
        ops.gla_scan(o, q, k, v, log_decay, state, start_loc, ctx_dev, slots_dev, self.q_scale,
                     max(b - a for a, b in zip(starts, starts[1:])))
        q_decayed = torch.empty((q.shape[0], H * D), dtype=torch.float32, device=dev)
        totals = torch.empty((len(ctx), H * D), dtype=torch.float32, device=dev)
        ops.gla_piece_prefix(q_decayed, totals, q, log_decay, start_loc, self.q_scale)
        for first, count, own, row, cb in cut:
            piece_slots = slots[first:first + count]
            ops.gla_combine_states(state, slots_dev[first:first + count], index_dev[first:first + count], totals, own)
            n = starts[first + count] - starts[first]
            full = n // L                           # pieces of exactly L rows
            # pieces 1 .. full - 1 start from the states at the end of pieces 0 .. full - 2
            if full > 1:
                r0, r1 = row + L, row + full * L
                s_start = state[piece_slots[0]:piece_slots[0] + full - 1]              # [p, H, D, V]
                qd = q_decayed[r0:r1].view(full - 1, L, H, D).permute(0, 2, 1, 3)       # [p, H, L, D]
                o[r0:r1].view(full - 1, L, H, V).permute(0, 2, 1, 3).add_(torch.matmul(qd, s_start))
            if n > full * L:                        # the shorter last piece
                r0 = row + full * L
                qd = q_decayed[r0:row + n].view(n - full * L, H, D).permute(1, 0, 2)    # [H, l, D]
                o[r0:row + n].permute(1, 0, 2).add_(torch.matmul(qd, state[piece_slots[full - 1]]))


class MinGRURecurrence(nn.Module):
    """Element-wise gated recurrence whose gates read only the current token:
    S_t = (1 - z_t) S_(t-1) + z_t c_t with z = sigmoid(zp) and the candidate c = up + 1/2 where
    up >= 0, sigmoid(up) below; the output is S_t * silu(gp).  zp, up, gp are projections of the
    token (biases included).  One fp32 number per channel and sequence lives in a state slot
    [num_slots, channels]; a sequence whose context length is 0 starts from zero.  Long runs of
    rows are walked in pieces at the same time (csrc/seq_gated_recurrence.hip)."""

    def __init__(self, channels: int) -> None:
        super().__init__()
        self.channels = channels

    @staticmethod
    def get_state_shape(num_slots: int, channels: int) -> Tuple[int, ...]:
        return (num_slots, channels)

    def forward(self, out: torch.Tensor, zp: torch.Tensor, up: torch.Tensor, gp: torch.Tensor,
                state: torch.Tensor, batch: SequenceBatch) -> torch.Tensor:
        ops.mingru_scan(out, zp, up, gp, state, batch.query_start_loc, batch.context_lens, batch.state_slots,
                        batch.max_query_len)
        return out


class GatedDeltaRule(nn.Module):
    """Gated delta rule with per-sequence state slots.  Per head, on a state S [dim, vdim]:
    S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q -- the read-out sees the token's
    own write.  k and q are unit vectors per key head (q also times dim^-1/2), `heads / kv_heads`
    value heads share a key head, beta = sigmoid(b), g = exp(-exp(A_log) softplus(dt + dt_bias)),
    and o leaves RMS-normed over vdim, weighted (one weight vector for all heads) and times
    silu(gate).  All inputs are fp32 rows (the caller's projections and short convolutions leave
    them so); the state is fp32 [num_slots, heads, vdim, dim] and a sequence whose context length
    is 0 starts from zero whatever its slot held (csrc/seq_delta_rule.hip)."""

    def __init__(self, heads: int, kv_heads: int, dim: int, vdim: int, eps: float, device=None) -> None:
        super().__init__()
        assert heads % kv_heads == 0
        self.heads, self.kv_heads, self.dim, self.vdim, self.eps = heads, kv_heads, dim, vdim, float(eps)

        def par(n, fill=0.0):
            return nn.Parameter(torch.full((n, ), fill, dtype=torch.float32, device=device), requires_grad=False)

        self.a_log, self.dt_bias, self.norm_weight = par(heads), par(heads), par(vdim, 1.0)

    @staticmethod
    def get_state_shape(num_slots: int, heads: int, dim: int, vdim: int) -> Tuple[int, ...]:
        return (num_slots, heads, vdim, dim)

    def forward(self, out: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, gate: torch.Tensor,
                beta: torch.Tensor, dt: torch.Tensor, state: torch.Tensor, batch: SequenceBatch) -> torch.Tensor:
        """q, k [T, G*D]; v, gate, out [T, H*V]; beta, dt [T, H]: views with free row strides."""
        ops.delta_rule_scan(out, q, k, v, gate, beta, dt, self.a_log.data, self.dt_bias.data, self.norm_weight.data,
                            state, batch.query_start_loc, batch.context_lens, batch.state_slots, self.kv_heads,
                            self.eps, batch.max_query_len)
        return out


class RealGatedLRU(nn.Module):
    """Real-gated linear recurrent unit: per channel S_t = a_t S_(t-1) + sqrt(1 - a_t^2) i_t u_t with
    a_t = exp(-c r_t softplus(lam)), r = sigmoid(W_a u + b_a), i = sigmoid(W_i u + b_i), where W_a and
    W_i are block-diagonal (`blocks` square blocks [out, in]); the output is S_t * gelu_tanh(y_t).
    u and y are fp32 rows; the gates' products are fp32 batched matrix products; the state is fp32
    [num_slots, channels] and a sequence whose context length is 0 starts from zero.  Long runs of
    rows are walked in pieces at the same time (csrc/seq_gated_recurrence.hip)."""

    def __init__(self, channels: int, blocks: int, c: float = 8.0, device=None) -> None:
        super().__init__()
        assert channels % blocks == 0
        self.channels, self.blocks, self.c = channels, blocks, float(c)
        bw = channels // blocks
        # both gates' blocks side by side: [blocks, in, 2 * out] (recurrence gate | input gate)
        self.gate_weight = nn.Parameter(torch.zeros((blocks, bw, 2 * bw), dtype=torch.float32, device=device),
                                        requires_grad=False)
        self.gate_bias = nn.Parameter(torch.zeros((blocks, 1, 2 * bw), dtype=torch.float32, device=device),
                                      requires_grad=False)
        self.rate = nn.Parameter(torch.zeros(channels, dtype=torch.float32, device=device), requires_grad=False)

    def set_weights(self, ra, ra_b, ri, ri_b, lam) -> None:
        """ra, ri [blocks, out, in]; ra_b, ri_b [blocks, out]; lam [channels]."""
        dev = self.rate.device
        w = torch.cat([ra.float().transpose(1, 2), ri.float().transpose(1, 2)], 2)
        b = torch.cat([ra_b.float(), ri_b.float()], 1)[:, None, :]
        self.gate_weight.data = w.to(dev).contiguous()
        self.gate_bias.data = b.to(dev).contiguous()
        self.rate.data = (self.c * torch.nn.functional.softplus(lam.float())).to(dev).contiguous()

    @staticmethod
    def get_state_shape(num_slots: int, channels: int) -> Tuple[int, ...]:
        return (num_slots, channels)

    def forward(self, out: torch.Tensor, u: torch.Tensor, y: torch.Tensor, state: torch.Tensor,
                batch: SequenceBatch) -> torch.Tensor:
        """u fp32 [T, R] contiguous (the recurrent branch after its convolution), y fp32 [T, R] view (the
        other branch before its activation), out [T, R]."""
        T, R = u.shape
        B, bw = self.blocks, R // self.blocks
        gates = torch.baddbmm(self.gate_bias.data, u.view(T, B, bw).transpose(0, 1), self.gate_weight.data)
        ops.rglru_scan(out, gates, u, y, self.rate.data, state, batch.query_start_loc, batch.context_lens,
                       batch.state_slots, batch.max_query_len)
        return out
