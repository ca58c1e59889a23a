"""minGRU: a gated recurrence whose gates read the current token only.

    z_t = sigmoid(W_z h_t + b_z)            how much of the state is replaced
    c_t = g(W_x h_t + b_x)                  the candidate; g(u) = u + 1/2 for u >= 0, sigmoid(u) below
    S_t = (1 - z_t) S_(t-1) + z_t c_t       element by element, S_(-1) = 0
    y_t = W_o (S_t * silu(W_g h_t))

The three input projections are one stacked product whose result stays in 32-bit; biases,
gates, candidate and state are 32-bit in every mode.  The state is one row per request slot
(`StateSpec`), carried from step to step by the cache manager; a step's tokens of one request
are scanned in order by one kernel launch, whatever the mix of portions and single tokens.
"""
from __future__ import annotations

from typing import Dict, Sequence

import torch

from ..weights.spec import INIT_NORMAL, TensorSpec
from .base import BuildContext, Mixer, StateSpec
from .linear import Linear


class MinGRU(Mixer):
    graph_safe = True

    def __init__(self, prefix: str, hidden_size: int, width: int,
                 names: Sequence[str] = ("z", "x", "g", "o"), bias_names: Sequence[str] = ("z.b", "x.b")):
        """`names`: the checkpoint's names after `prefix` of the update-gate, candidate, output-gate
        and output projections; `bias_names` those of the update gate's and the candidate's biases."""
        z, x, g, o = names
        self.prefix = prefix
        self.width = int(width)
        self.zxg = Linear([prefix + z, prefix + x, prefix + g], hidden_size, [width] * 3)
        self.o = Linear([prefix + o], width, [hidden_size])
        self.bias_names = [prefix + n for n in bias_names]
        self.z_bias = self.x_bias = None

    def state_spec(self) -> StateSpec:
        return StateSpec((self.width,), torch.float32)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs = {**self.zxg.tensor_specs(), **self.o.tensor_specs()}
        for n in self.bias_names:
            specs[n] = TensorSpec((self.width,), INIT_NORMAL)
        return specs

    def bind(self, weights, ctx: BuildContext) -> None:
        self.ctx = ctx
        self.zxg.bind(weights, ctx)
        self.o.bind(weights, ctx)
        self.z_bias, self.x_bias = (weights[n].float().contiguous() for n in self.bias_names)

    def forward(self, x, step, cache):
        ops = self.ctx.ops
        zxg = self.zxg.forward(x, out_dtype=torch.float32)
        y = ops.mingru_scan(zxg, self.z_bias, self.x_bias, cache.state, step.seq_slots, step.cu_tokens,
                            self.ctx.dtype, step.max_q_len)
        return self.o.forward(y)
