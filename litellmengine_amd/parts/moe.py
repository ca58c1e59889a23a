"""Mixture of experts: every token runs through the `top` of `experts` small gated
feed-forwards that its router picks, and through one shared expert that all tokens use.

    logits = W_router h + b            32-bit
    chosen = the `top` largest logits (the lower index wins a tie)
    weights = softmax over the chosen logits only
    out = sum_k weights_k * expert_k(h) + shared(h),   expert(h) = down(silu(gate h) * (up h))

The experts' weights are stacked into one tensor per kind, so the kernels index them by the
chosen ids on the device: no expert's token list ever comes back to the host, and a decode step
can be captured into a graph.  The routed sum is left in 32-bit; with a shared expert the result is
the pair (routed sum, shared result), which the norm's kernel adds up.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..weights.spec import INIT_NORMAL, TensorSpec
from .base import BuildContext, FeedForward
from .feed_forward import GatedMLP
from .linear import Linear


class RoutedMLP(FeedForward):
    def __init__(self, prefix: str, hidden_size: int, expert_size: int, num_experts: int, top: int,
                 shared: Optional[GatedMLP] = None, expert_prefix: str = "e{}.",
                 names=("gate", "up", "down"), router_names=("router", "router.b")):
        """Expert e's tensors are `prefix + expert_prefix.format(e) + name`; `shared` is the
        feed-forward that every token runs through (None: none)."""
        if not 0 < top <= num_experts:
            raise ValueError("every token uses between one and all of the experts")
        self.prefix, self.hidden, self.ff, self.E, self.top = prefix, hidden_size, expert_size, num_experts, top
        self.shared = shared
        self.expert_names = [[prefix + expert_prefix.format(e) + n for n in names] for e in range(num_experts)]
        self.router = Linear([prefix + router_names[0]], hidden_size, [num_experts])
        self.router_bias_name = prefix + router_names[1]
        self.router_bias = self.gate_up = self.down = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs = dict(self.router.tensor_specs())
        specs[self.router_bias_name] = TensorSpec((self.E,), INIT_NORMAL)
        for gate, up, down in self.expert_names:
            specs[gate] = TensorSpec((self.ff, self.hidden), INIT_NORMAL)
            specs[up] = TensorSpec((self.ff, self.hidden), INIT_NORMAL)
            specs[down] = TensorSpec((self.hidden, self.ff), INIT_NORMAL)
        if self.shared is not None:
            specs.update(self.shared.tensor_specs())
        return specs

    def bind(self, weights, ctx: BuildContext) -> None:
        self.ctx = ctx
        self.router.bind(weights, ctx)
        self.router_bias = weights[self.router_bias_name].float().contiguous()
        # [E, 2 ff, hidden] (gate rows, then up rows) and [E, hidden, ff]
        self.gate_up = torch.stack(
            [torch.cat([weights[g].to(ctx.dtype), weights[u].to(ctx.dtype)], dim=0) for g, u, _ in self.expert_names]
        ).contiguous()
        self.down = torch.stack([weights[d].to(ctx.dtype) for _, _, d in self.expert_names]).contiguous()
        if self.shared is not None:
            self.shared.bind(weights, ctx)

    def forward(self, x):
        ops = self.ctx.ops
        logits = self.router.forward(x, out_dtype=torch.float32)
        ids, gains = ops.moe_route(logits, self.router_bias, self.top)
        routed = ops.moe_experts(x, ids, gains, self.gate_up, self.down)  # float32 [N, hidden]
        if self.shared is None:
            return routed
        return routed, self.shared.forward(x)
