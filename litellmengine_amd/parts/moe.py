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
from .feed_forward import GatedMLP, PlainMLP
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


class GroupLimitedMLP(FeedForward):
    """Mixture of experts whose router scores ALL experts with one softmax and limits its choice to groups:

        s = softmax(W_router h)                        32-bit, over experts and identity experts alike
        c = s + correction                             the choice scores; the gains never see the correction
        the experts form `groups` equal groups of neighbours; a group's score is its largest c, and only
        the experts of the `groups_kept` best groups can be chosen (the others count as minus infinity)
        chosen = the `top` largest c among those;  gains = s[chosen] / (sum of s[chosen] + 1e-20)
        out = sum_k gains_k * expert_k(h),  expert(h) = down(silu(gate h) * (up h))

    The last `identity` router outputs are identity experts: no tensors, their result is h itself.  The
    experts' weights are stacked, the choice stays on the device, the sum is left in 32-bit.

    Parameters for other routers and experts of the same shape: `score="sigmoid"` (s = sigmoid(W_router h), every
    expert scored on its own), `correction=False` (no correction tensor: c = s), `group_top=n` (a group's score
    is the sum of its n largest c), `form="gated_clamp"` with `limit` (g = min(gate h, limit),
    u = clamp(up h, -limit, limit), expert(h) = down(g sigmoid(1.702 g) (u + 1)))."""

    def __init__(self, prefix: str, hidden_size: int, expert_size: int, num_experts: int, top: int, identity: int = 0,
                 groups: int = 1, groups_kept: int = 1, expert_prefix: str = "e{}.", names=("gate", "up", "down"),
                 router_names=("router", "correction"), score: str = "softmax", correction: bool = True,
                 group_top: int = 1, form: str = "gated_silu", limit: float = 0.0):
        total = num_experts + identity
        if num_experts <= 0 or identity < 0 or groups <= 0 or total % groups or not 0 < groups_kept <= groups:
            raise ValueError("experts and identity experts together form equal groups, of which some are kept")
        if not 0 < top <= groups_kept * (total // groups):
            raise ValueError("every token uses between one and all of the experts of the kept groups")
        self.prefix, self.hidden, self.ff, self.E, self.identity, self.top = (prefix, hidden_size, expert_size,
                                                                             num_experts, identity, top)
        if score not in ("softmax", "sigmoid"):
            raise ValueError(f"a router's scores are a softmax over all experts or sigmoids, not {score!r}")
        if form not in ("gated_silu", "gated_clamp") or (form == "gated_clamp" and not limit > 0.0):
            raise ValueError("the experts are gated_silu, or gated_clamp with a positive limit")
        if group_top < 1:
            raise ValueError("a group's score adds up at least one of its experts' scores")
        self.groups, self.groups_kept = groups, groups_kept
        self.score, self.group_top, self.form, self.limit = score, int(group_top), form, float(limit)
        self.expert_names = [[prefix + expert_prefix.format(e) + n for n in names] for e in range(num_experts)]
        self.router = Linear([prefix + router_names[0]], hidden_size, [total])
        self.correction_name = prefix + router_names[1] if correction else None
        self.correction = self.gate_up = self.down = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs = dict(self.router.tensor_specs())
        if self.correction_name is not None:
            specs[self.correction_name] = TensorSpec((self.E + self.identity,), INIT_NORMAL)
        for gate, up, down in self.expert_names:
            specs[gate] = TensorSpec((self.ff, self.hidden), INIT_NORMAL)
            specs[up] = TensorSpec((self.ff, self.hidden), INIT_NORMAL)
            specs[down] = TensorSpec((self.hidden, self.ff), INIT_NORMAL)
        return specs

    def bind(self, weights, ctx: BuildContext) -> None:
        self.ctx = ctx
        self.router.bind(weights, ctx)
        if self.correction_name is not None:
            self.correction = weights[self.correction_name].float().contiguous()
        self.gate_up = torch.stack(
            [torch.cat([weights[g].to(ctx.dtype), weights[u].to(ctx.dtype)], dim=0) for g, u, _ in self.expert_names]
        ).contiguous()
        self.down = torch.stack([weights[d].to(ctx.dtype) for _, _, d in self.expert_names]).contiguous()

    def forward(self, x):
        ops = self.ctx.ops
        logits = self.router.forward(x, out_dtype=torch.float32)
        ids, gains = ops.moe_route_grouped(logits, self.correction, self.top, self.groups, self.groups_kept,
                                           score=self.score, group_top=self.group_top)
        # float32 [N, hidden]; ids from E on: x itself
        return ops.moe_experts(x, ids, gains, self.gate_up, self.down, form=self.form, limit=self.limit)


class ScoreRoutedMLP(FeedForward):
    """Mixture of experts whose router scores every expert on its own and weighs the experts' INPUTS:

        s = sigmoid(W_router h)                        32-bit
        chosen = the `top` largest s (the lower index wins a tie); their weights are s itself, not renormalised
        out = sum_k expert_k(s_k * h) + sigmoid(w_sg . h) * shared(h),   expert(x) = down(act(up x)), act = relu squared

    The experts have no gate and no biases; their weights are stacked, the choice stays on the device.  A weight on
    an expert's input is a factor on its first product's result, where the kernels apply it in 32-bit before the
    activation.  The shared expert (None: none) has the same form and one gate number per token, which comes out of
    the router's product (its row is stacked under the router's).  The routed sum is left in 32-bit; with a shared
    expert the result is the pair (routed sum, gated shared result), which the norm's kernel adds up."""

    def __init__(self, prefix: str, hidden_size: int, expert_size: int, num_experts: int, top: int,
                 shared: Optional[PlainMLP] = None, shared_gate_name: str = "shared.sg", expert_prefix: str = "e{}.",
                 names=("up", "down"), router_name: str = "router"):
        if not 0 < top <= num_experts:
            raise ValueError("every token uses between one and all of the experts")
        self.prefix, self.hidden, self.ff, self.E, self.top = prefix, hidden_size, expert_size, num_experts, top
        self.shared = shared
        self.expert_names = [[prefix + expert_prefix.format(e) + n for n in names] for e in range(num_experts)]
        rows, sizes = [prefix + router_name], [num_experts]
        if shared is not None:
            rows.append(prefix + shared_gate_name)
            sizes.append(1)
        self.router = Linear(rows, hidden_size, sizes)
        self.up = self.down = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs = dict(self.router.tensor_specs())
        for up, down in self.expert_names:
            specs[up] = TensorSpec((self.ff, self.hidden), INIT_NORMAL)
            specs[down] = TensorSpec((self.hidden, self.ff), INIT_NORMAL)
        if self.shared is not None:
            specs.update(self.shared.tensor_specs())
        return specs

    def bind(self, weights, ctx: BuildContext) -> None:
        self.ctx = ctx
        self.router.bind(weights, ctx)
        self.up = torch.stack([weights[u].to(ctx.dtype) for u, _ in self.expert_names]).contiguous()  # [E, ff, hidden]
        self.down = torch.stack([weights[d].to(ctx.dtype) for _, d in self.expert_names]).contiguous()  # [E, hidden, ff]
        if self.shared is not None:
            self.shared.bind(weights, ctx)

    def forward(self, x):
        ops = self.ctx.ops
        logits = self.router.forward(x, out_dtype=torch.float32)  # [N, E (+ 1: the shared expert's gate)]
        ids, gains = ops.moe_route(logits, None, self.top, score="sigmoid", experts=self.E)
        routed = ops.moe_experts(x, ids, gains, self.up, self.down, form="relu2", gain_on_input=True)  # float32 [N, hidden]
        if self.shared is None:
            return routed
        return routed, self.shared.forward(x, row_gate=(logits, self.E))
