"""A recurrence with a matrix state per head whose decay is made from the data.

With h' the previous token's h (zeros before a request's first token), every input reads its own
mix of the two, mix_s = h + (h' - h) * mu_s for s of r, k, v, g, w:

    r, k, v = W_r mix_r, W_k mix_k, W_v mix_v            [heads, dim] each
    gate    = silu(W_g mix_g)
    decay   = exp(-exp(W_w2 tanh(W_w1 mix_w) + w0))      per head and key channel, in (0, 1)
    o_t     = (S + diag(u) k_t v_t^T)^T r_t              the bonus u counts for the current token only
    S      <- diag(decay_t) S + k_t v_t^T
    y_t     = W_o (o_t / rms(o_t) per head * norm * gate)

The state is one float32 row per request slot (`StateSpec`): the heads' matrices and, behind them,
the last token's h, which the next step's first token is mixed with.  The projections' results that
enter the recurrence (r, k, v and the decay's exponent) stay in 32-bit, as do the decay, the state
and the unit norm, in every mode.  A step's tokens of one request are walked in order by one kernel
(long portions in pieces side by side), whatever the mix of portions and single tokens.
"""
from __future__ import annotations

from typing import Dict, Sequence

import torch

from ..weights.spec import INIT_NORM, INIT_NORMAL, TensorSpec
from ..csrc.limits import MAX_WKV_HEAD_DIM
from .base import BuildContext, Mixer, StateSpec
from .linear import Linear

MAX_HEAD_CHANNELS = MAX_WKV_HEAD_DIM


class WKVMixer(Mixer):
    graph_safe = True

    def __init__(self, prefix: str, hidden_size: int, heads: int, dim: int, decay_rank: int, norm_eps: float,
                 names: Sequence[str] = ("r", "k", "v", "g", "w1", "w2", "w0", "u", "norm", "o"), mu_prefix: str = "mu.",
                 out_scale: float = 1.0):
        """`out_scale`: the result is multiplied by it; it is folded into the 32-bit output norm's weight, so it
        costs no operation and no rounding of its own.  `names`: the checkpoint's names after `prefix` of the four input projections, the decay's two
        projections and its offset, the bonus, the output norm's weight and the output projection; the mixing
        weights are `mu_prefix` + r, k, v, g, w."""
        if not 0 < dim <= MAX_HEAD_CHANNELS:
            raise ValueError(f"a head of the recurrence holds between 1 and {MAX_HEAD_CHANNELS} channels, not {dim}")
        if decay_rank <= 0:
            raise ValueError("the decay's inner rank must be positive")
        self.prefix, self.hidden, self.H, self.dim, self.rank = prefix, hidden_size, heads, dim, int(decay_rank)
        self.eps = float(norm_eps)
        self.out_scale = float(out_scale)
        r, k, v, g, w1, w2, w0, u, norm, o = (prefix + n for n in names)
        hd = heads * dim
        self.r, self.k, self.v, self.g = (Linear([n], hidden_size, [hd]) for n in (r, k, v, g))
        self.w1 = Linear([w1], hidden_size, [self.rank])
        self.w2 = Linear([w2], self.rank, [hd])
        self.o = Linear([o], hd, [hidden_size])
        self.w0_name, self.u_name, self.norm_name = w0, u, norm
        self.mu_names = [prefix + mu_prefix + s for s in ("r", "k", "v", "g", "w")]
        self.mu = self.w0 = self.u = self.norm_w = None

    def state_spec(self) -> StateSpec:
        return StateSpec((self.H * self.dim * self.dim + self.hidden,), torch.float32)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs: Dict[str, TensorSpec] = {}
        for p in (self.r, self.k, self.v, self.g, self.w1, self.w2, self.o):
            specs.update(p.tensor_specs())
        for n in self.mu_names:
            specs[n] = TensorSpec((self.hidden,), INIT_NORMAL)
        specs[self.w0_name] = TensorSpec((self.H * self.dim,), INIT_NORMAL)
        specs[self.u_name] = TensorSpec((self.H, self.dim), INIT_NORMAL)
        specs[self.norm_name] = TensorSpec((self.H * self.dim,), INIT_NORM)
        return specs

    def bind(self, weights, ctx: BuildContext) -> None:
        self.ctx = ctx
        for p in (self.r, self.k, self.v, self.g, self.w1, self.w2, self.o):
            p.bind(weights, ctx)
        self.mu = torch.stack([weights[n].float() for n in self.mu_names]).contiguous()
        self.w0 = weights[self.w0_name].float().reshape(-1).contiguous()
        self.u = weights[self.u_name].float().reshape(-1).contiguous()
        self.norm_w = (weights[self.norm_name].float() * self.out_scale).contiguous()

    def forward(self, x, step, cache):
        ops = self.ctx.ops
        state = cache.state
        mixes = ops.shift_mix(x, state, self.H * self.dim * self.dim, self.mu, step.token_seq, step.cu_tokens,
                              step.seq_slots)
        r = self.r.forward(mixes[0], out_dtype=torch.float32)
        k = self.k.forward(mixes[1], out_dtype=torch.float32)
        v = self.v.forward(mixes[2], out_dtype=torch.float32)
        g = self.g.forward(mixes[3])
        wraw = self.w2.forward(ops.tanh_(self.w1.forward(mixes[4])), out_dtype=torch.float32)
        y = ops.wkv_scan(r, k, v, wraw, self.w0, self.u, g, self.norm_w, self.eps, x, state, self.H, self.dim,
                         step.seq_slots, step.cu_tokens, self.ctx.dtype, step.max_q_len)
        return self.o.forward(y)
