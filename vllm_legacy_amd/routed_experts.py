"""Mixture-of-experts feed-forward in the activation dtype, routed on the device.

Router: z = W_r h (+ a bias) in fp32 over all routed experts, s = softmax(z); the `top` experts
with the largest s + correction are chosen and weighted by their s renormalized to sum 1 (without a
correction: the softmax over the chosen logits).  The last `identity` routed experts have no
weights: their output is the token's input.  An expert is W_down act(W_up h), or, `gated`,
W_down (act(W_gate h) * W_up h); with act "clamped_glu" the gated form is
g sigmoid(alpha g) (u + shift), g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit).  An
optional shared expert runs for every token: plain, multiplied by sigmoid(w_sg . h), or
(`shared_gated`) of the gated form with a limit of its own and nothing in front.  The output is
fp32 (the caller norms it and adds it to its stream).

Execution (csrc/seq_moe_kernels.hip): route (the logits of a large step come from one fp32 matrix
product) -> plan (pairs grouped by expert into row tiles) ->
grouped up-projection with the activation fused (rows gathered from the tokens) -> grouped
down-projection in fp32 -> combine (weighted sum per token in the order of its choices, identity
experts and the shared expert added there).  Nothing synchronises with the host.
"""
from typing import Dict, Optional

import torch
import torch.nn as nn

from vllm_legacy_amd import _seq_ops as ops


def mm_f32(a: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """a [T, K] x w [N, K]^T with an fp32 result (16-bit operands keep the fp32 accumulator)."""
    if a.dtype == torch.float32:
        return torch.mm(a, w.t())
    return torch.mm(a, w.t(), out_dtype=torch.float32)


class RoutedExperts(nn.Module):
    # steps with at least this many tokens form the router logits as one matrix product; below,
    # the routing kernel forms them itself (one launch)
    ROUTE_PRODUCT_MIN_TOKENS = 256

    def __init__(self, width: int, num_experts: int, num_identity: int, top: int, expert_ff: int,
                 shared_ff: int = 0, act: str = "relu2", shared_act: Optional[str] = None,
                 dtype=torch.bfloat16, device=None, gated: bool = False, router_bias: bool = False,
                 act_limit: float = 0.0, act_alpha: float = 1.702, act_shift: float = 1.0,
                 shared_gated: bool = False, shared_limit: float = 0.0) -> None:
        super().__init__()
        if act == "clamped_glu" and not (gated and act_limit > 0):
            raise ValueError("clamped_glu needs gated experts and a limit")
        if shared_gated and shared_ff and (shared_act or act) == "clamped_glu" and not shared_limit > 0:
            raise ValueError("a clamped_glu shared expert needs a limit")
        self.act_limit, self.act_alpha, self.act_shift = float(act_limit), float(act_alpha), float(act_shift)
        self.shared_gated, self.shared_limit = bool(shared_gated), float(shared_limit)
        if top > num_experts + num_identity:
            raise ValueError("top exceeds the number of routed experts")
        self.width, self.num_experts, self.num_identity, self.top = width, num_experts, num_identity, top
        self.expert_ff, self.shared_ff, self.act = expert_ff, shared_ff, act
        self.shared_act = shared_act or act
        self.dtype = dtype
        self.gated = bool(gated)
        self._router_rows = None
        routed = num_experts + num_identity

        def par(shape, dt):
            return nn.Parameter(torch.zeros(shape, dtype=dt, device=device), requires_grad=False)

        self.router = par((routed, width), torch.float32)
        self.correction = par((routed, ), torch.float32)
        self.router_bias = par((routed, ), torch.float32) if router_bias else None
        # gated experts keep W_gate's rows ahead of W_up's in one matrix per expert
        self.w_up = par((num_experts, (2 if gated else 1) * expert_ff, width), dtype)
        self.w_down = par((num_experts, width, expert_ff), dtype)
        self.shared_gate = None
        if shared_ff:
            # a gated shared expert keeps W_gate's rows ahead of W_up's and has no sigmoid in front
            self.shared_up = par(((2 if shared_gated else 1) * shared_ff, width), dtype)
            self.shared_down = par((width, shared_ff), dtype)
            self.shared_gate = None if shared_gated else par((width, ), torch.float32)

    def set_weights(self, t: Dict[str, torch.Tensor]) -> None:
        """t: router, router.b (with a router bias), correction (optional), e<i>.up / e<i>.down
        (gated: also e<i>.gate), shared.up / shared.down and shared.sg or (gated) shared.gate."""
        dev, dt = self.router.device, self.dtype
        routed = self.num_experts + self.num_identity

        def put(param, value, name):
            if tuple(value.shape) != tuple(param.shape):
                raise ValueError(f"{name}: shape {tuple(value.shape)}, expected {tuple(param.shape)}")
            param.data = value.to(param.dtype).to(dev).contiguous()

        self._router_rows = None
        put(self.router, t["router"], "router")
        if "correction" in t:
            put(self.correction, t["correction"].reshape(routed), "correction")
        if self.router_bias is not None:
            put(self.router_bias, t["router.b"].reshape(routed), "router.b")
        if self.num_experts and self.gated:
            put(self.w_up, torch.stack([torch.cat([t[f"e{e}.gate"], t[f"e{e}.up"]], 0)
                                        for e in range(self.num_experts)]).to(dt), "e*.gate | e*.up")
        elif self.num_experts:
            put(self.w_up, torch.stack([t[f"e{e}.up"] for e in range(self.num_experts)]).to(dt), "e*.up")
        if self.num_experts:
            put(self.w_down, torch.stack([t[f"e{e}.down"] for e in range(self.num_experts)]).to(dt), "e*.down")
        if self.shared_ff:
            if self.shared_gated:
                put(self.shared_up, torch.cat([t["shared.gate"], t["shared.up"]], 0), "shared.gate | shared.up")
            else:
                put(self.shared_up, t["shared.up"], "shared.up")
                put(self.shared_gate, t["shared.sg"].reshape(self.width), "shared.sg")
            put(self.shared_down, t["shared.down"], "shared.down")

    def router_rows(self) -> torch.Tensor:
        """fp32 [routed (+ 1), width]: the router and, last, the shared expert's gate."""
        if self._router_rows is None:
            self._router_rows = torch.cat([self.router.data, self.shared_gate.data[None]], 0).contiguous() \
                if self.shared_gate is not None else self.router.data
        return self._router_rows

    def _glu(self, out: torch.Tensor, both: torch.Tensor, ff: int, act: str, limit: float) -> None:
        if act == "clamped_glu":
            ops.clamped_glu(out, both[:, :ff], both[:, ff:], limit, self.act_alpha, self.act_shift)
        else:
            ops.gated_act(out, both[:, :ff], both[:, ff:], act)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        """h [T, width] in the activation dtype -> fp32 [T, width]."""
        T = h.shape[0]
        logits = None
        if T >= self.ROUTE_PRODUCT_MIN_TOKENS:
            # many tokens: the router rows (and the shared gate's) as one fp32 matrix product
            logits = torch.mm(h if h.dtype == torch.float32 else h.float(), self.router_rows().t())
        experts, weights, sg = ops.moe_route(h, self.router.data, self.correction.data,
                                             None if self.shared_gate is None else self.shared_gate.data, self.top, logits,
                                             None if self.router_bias is None else self.router_bias.data)
        if self.num_experts:
            pair_row, row_token, tile_expert = ops.moe_plan(experts, self.num_experts)
            rows = row_token.numel()
            u = torch.empty((rows, self.expert_ff), dtype=h.dtype, device=h.device)
            if self.gated:
                both = torch.empty((rows, 2 * self.expert_ff), dtype=h.dtype, device=h.device)
                ops.grouped_linear(both, h, row_token, self.w_up.data, tile_expert)
                self._glu(u, both, self.expert_ff, self.act, self.act_limit)
            else:
                ops.grouped_linear(u, h, row_token, self.w_up.data, tile_expert, self.act)
            y = torch.empty((rows, self.width), dtype=torch.float32, device=h.device)
            ops.grouped_linear(y, u, None, self.w_down.data, tile_expert)
        else:   # identity experts only
            pair_row = torch.full((T, self.top), -1, dtype=torch.int32, device=h.device)
            y = torch.zeros((1, self.width), dtype=torch.float32, device=h.device)
        shared_y = None
        if self.shared_ff:
            su = torch.mm(h, self.shared_up.data.t())
            if self.shared_gated:
                sa = torch.empty((T, self.shared_ff), dtype=su.dtype, device=su.device)
                self._glu(sa, su, self.shared_ff, self.shared_act, self.shared_limit)
            else:
                sa = torch.empty_like(su)
                ops.gated_act(sa, su, None, self.shared_act)
            shared_y = mm_f32(sa, self.shared_down.data)
        out = torch.empty((T, self.width), dtype=torch.float32, device=h.device)
        ops.moe_combine(out, y, pair_row, weights, h, shared_y, sg)
        return out
