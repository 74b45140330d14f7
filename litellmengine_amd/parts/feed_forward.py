"""Dense feed-forwards.  Gated: down(act(gate(x)) * up(x)); silu without biases is the
reference's (src/model/qwen3.cpp:88-105, :143-152; src/ops/silu_and_mul.cu:44-46), other
activations and biases are parameters.  Plain: down(act(up(x))).  gate and up are one stacked
product here; the activations are computed in 32-bit."""
from __future__ import annotations

from typing import Dict, Optional, Sequence

import torch

from ..weights.spec import TensorSpec
from .base import BuildContext, FeedForward
from .linear import Linear


class GatedMLP(FeedForward):
    def __init__(self, prefix: str, hidden_size: int, intermediate_size: int,
                 names=("gate_proj.weight", "up_proj.weight", "down_proj.weight"), to_residual: bool = True,
                 activation: str = "silu", bias_names: Optional[Sequence[str]] = None):
        """`names`: the checkpoint's names of the gate, up and down weights after `prefix`.
        `to_residual`: the result goes nowhere but into Norm.forward(hidden, delta) (it may then
        come as PartialSums); an arrangement that does anything else with it says False.
        `activation`: silu, relu or gelu_tanh (gelu in its tanh form).  `bias_names`: the three projections' biases after `prefix`
        (none: no biases); the gate's and up's are added inside the activation's kernel."""
        if activation not in ("silu", "relu", "gelu_tanh"):
            raise ValueError(f"a gated feed-forward's activation is silu, relu or gelu_tanh, not {activation!r}")
        self.activation = activation
        biased = bool(bias_names)
        if biased and len(bias_names) != 3:
            raise ValueError("bias_names holds three names (gate, up, down)")
        # the products that do a folded norm's work read their inner dimension eight elements at a time
        self.folds_norm = intermediate_size % 8 == 0 and to_residual and activation == "silu" and not biased
        self.fused = activation == "silu" and not biased  # one launch may do the product and the activation
        gate, up, down = names
        self.gate_up = Linear([prefix + gate, prefix + up], hidden_size, [intermediate_size] * 2,
                              bias_names=[prefix + b for b in bias_names[:2]] if biased else None)
        self.down = Linear([prefix + down], intermediate_size, [hidden_size], to_residual=to_residual and not biased,
                           bias_names=[prefix + bias_names[2]] if biased else None)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {**self.gate_up.tensor_specs(), **self.down.tensor_specs()}

    def bind(self, weights, ctx: BuildContext) -> None:
        self.ctx = ctx
        self.gate_up.bind(weights, ctx)
        self.down.bind(weights, ctx)

    def forward(self, x, fold=None):
        ops = self.ctx.ops
        if self.fused:
            return self.down.forward(ops.gate_up_silu(x, self.gate_up.weight), fold=fold)
        a = ops.bias_act(ops.linear(x, self.gate_up.weight), self.activation, gated=True, bias=self.gate_up.bias)
        return self.down.forward(a)


class PlainMLP(FeedForward):
    """Feed-forward without a gate: down(act(up(x))), no biases; act is relu2 (the square of relu), relu or silu.
    `forward(x, row_gate=(t, col))`: row n of the result is multiplied by sigmoid(t[n, col]) (t float32 [N, any]);
    the factor enters with the activation, in 32-bit, since the last product is linear in it."""

    def __init__(self, prefix: str, hidden_size: int, intermediate_size: int, names=("up", "down"),
                 activation: str = "relu2"):
        if activation not in ("relu2", "relu", "silu"):
            raise ValueError(f"a plain feed-forward's activation is relu2, relu or silu, not {activation!r}")
        self.activation = activation
        up, down = names
        self.up = Linear([prefix + up], hidden_size, [intermediate_size])
        self.down = Linear([prefix + down], intermediate_size, [hidden_size])

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {**self.up.tensor_specs(), **self.down.tensor_specs()}

    def bind(self, weights, ctx: BuildContext) -> None:
        self.ctx = ctx
        self.up.bind(weights, ctx)
        self.down.bind(weights, ctx)

    def forward(self, x, row_gate=None):
        ops = self.ctx.ops
        return self.down.forward(ops.bias_act(ops.linear(x, self.up.weight), self.activation, gated=False, row_gate=row_gate))
