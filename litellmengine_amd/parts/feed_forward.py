"""Dense gated feed-forward: down(silu(gate(x)) * up(x)), no biases
(src/model/qwen3.cpp:88-105, :143-152; src/ops/silu_and_mul.cu:44-46).  gate and
up are one stacked product here; the activation is computed in 32-bit."""
from __future__ import annotations

from typing import Dict

import torch

from ..weights.spec import TensorSpec
from .base import BuildContext, FeedForward
from .linear import Linear


class GatedMLP(FeedForward):
    def __init__(self, prefix: str, hidden_size: int, intermediate_size: int,
                 names=("gate_proj.weight", "up_proj.weight", "down_proj.weight"), to_residual: bool = True):
        """`names`: the checkpoint's names of the gate, up and down weights after `prefix`.
        `to_residual`: the result goes nowhere but into Norm.forward(hidden, delta) (it may then
        come as PartialSums); an arrangement that does anything else with it says False."""
        # the products that do a folded norm's work read their inner dimension eight elements at a time
        self.folds_norm = intermediate_size % 8 == 0 and to_residual
        gate, up, down = names
        self.gate_up = Linear([prefix + gate, prefix + up], hidden_size, [intermediate_size] * 2)
        self.down = Linear([prefix + down], intermediate_size, [hidden_size], to_residual=to_residual)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {**self.gate_up.tensor_specs(), **self.down.tensor_specs()}

    def bind(self, weights, ctx: BuildContext) -> None:
        self.ctx = ctx
        self.gate_up.bind(weights, ctx)
        self.down.bind(weights, ctx)

    def forward(self, x, fold=None):
        return self.down.forward(self.ctx.ops.gate_up_silu(x, self.gate_up.weight), fold=fold)
