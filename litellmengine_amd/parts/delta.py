"""The gated delta rule: a recurrence with a matrix state per head that is decayed and then corrected
towards each new value.

    u      = (W_q h, W_k h, W_v h)                       one stacked product, no biases
    c      = silu(conv(u))                                per channel over time, J taps, zeros before a request's start
    q, k   = the heads of c's q and k parts as unit vectors, x / sqrt(sum x^2 + unit_eps); q also times dim^(-1/2)
    beta   = sigmoid(W_b h)                               one per value head
    g      = exp(-exp(A_log) * softplus(W_a h + dt_bias)) one decay per value head, in (0, 1)
    S     <- g S;  w = beta (v - S^T k);  S <- S + k w^T;  o = S^T q      (the read-out sees the token's own write)
    y      = W_o [heads' o / rms(o) * norm * silu(W_g h)]

There are `kv_heads` query/key heads of `dim` channels and `heads` value heads of `vdim`; value head h reads
query/key head h // (heads // kv_heads).  The state is one float32 row per request slot (`StateSpec`): the heads'
matrices (transposed, [head][value][key], the way the walk's kernel reads them) and, behind them, the last J - 1
rows of u, which the next step's first tokens are convolved with.  What enters the recurrence beyond the
projections and the convolution's results is 32-bit in every mode: unit vectors, beta, the decay and its
exponentials, the state, the read-out and its norm.  A step's tokens of one request are walked in order by one
kernel, whatever the mix of portions and single tokens.
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence

import torch

from ..csrc.limits import MAX_DELTA_HEAD_DIM
from ..weights.spec import INIT_NORM, INIT_NORMAL, INIT_WIDE, TensorSpec
from .base import BuildContext, Mixer, StateSpec
from .linear import Linear


class GatedDeltaMixer(Mixer):
    graph_safe = True

    def __init__(self, prefix: str, hidden_size: int, heads: int, kv_heads: int, dim: int, vdim: int, taps: int,
                 norm_eps: float, unit_eps: float = 1e-6, q_scale: Optional[float] = None,
                 names: Sequence[str] = ("q", "k", "v", "b", "a", "A_log", "dt_bias", "g", "norm", "o"),
                 conv_suffix: str = ".conv"):
        """`taps`: the convolution's length J (with one tap the state keeps no rows; the tensor [channels, 1] still
        scales the channels).  `q_scale`: the factor on the unit queries (default dim^(-1/2)).
        `names`: the checkpoint's names after `prefix` of the three convolved projections (their taps are
        + `conv_suffix`, [channels, J], the last column the current token's), beta's and the decay's projections,
        the decay's two vectors, the output gate's projection, the output norm's weight [vdim] (one for all heads)
        and the output projection."""
        if heads <= 0 or kv_heads <= 0 or heads % kv_heads:
            raise ValueError("the value heads are a multiple of the query/key heads")
        if not 0 < dim <= MAX_DELTA_HEAD_DIM or not 0 < vdim <= MAX_DELTA_HEAD_DIM:
            raise ValueError(f"a head of the delta rule holds between 1 and {MAX_DELTA_HEAD_DIM} channels, not {dim} and {vdim}")
        if taps < 1:
            raise ValueError("a convolution has at least one tap")
        self.prefix, self.hidden = prefix, hidden_size
        self.H, self.G, self.dim, self.vdim, self.taps = heads, kv_heads, dim, vdim, int(taps)
        self.eps, self.unit_eps = float(norm_eps), float(unit_eps)
        self.q_scale = float(dim) ** -0.5 if q_scale is None else float(q_scale)
        q, k, v, b, a, a_log, dt_bias, g, norm, o = (prefix + n for n in names)
        self.proj_names = (q, k, v)
        self.widths = (kv_heads * dim, kv_heads * dim, heads * vdim)
        self.cols = sum(self.widths)
        self.conv_suffix = conv_suffix
        self.qkv = Linear([q, k, v], hidden_size, list(self.widths))
        self.ba = Linear([b, a], hidden_size, [heads, heads])
        self.g = Linear([g], hidden_size, [heads * vdim])
        self.o = Linear([o], heads * vdim, [hidden_size])
        self.a_log_name, self.dt_bias_name, self.norm_name = a_log, dt_bias, norm
        self.conv_w = self.a_log = self.dt_bias = self.norm_w = None

    @property
    def matrix_floats(self) -> int:
        return self.H * self.vdim * self.dim

    @property
    def kept_rows(self) -> int:
        """Rows of the projections that a request keeps from step to step."""
        return self.taps - 1

    def state_spec(self) -> StateSpec:
        return StateSpec((self.matrix_floats + self.kept_rows * self.cols,), torch.float32)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs: Dict[str, TensorSpec] = {}
        for p in (self.qkv, self.ba, self.g, self.o):
            specs.update(p.tensor_specs())
        for name, rows in zip(self.proj_names, self.widths):
            specs[name + self.conv_suffix] = TensorSpec((rows, self.taps), INIT_WIDE)
        specs[self.a_log_name] = TensorSpec((self.H,), INIT_NORMAL)
        specs[self.dt_bias_name] = TensorSpec((self.H,), INIT_NORMAL)
        specs[self.norm_name] = TensorSpec((self.vdim,), INIT_NORM)
        return specs

    def bind(self, weights, ctx: BuildContext) -> None:
        self.ctx = ctx
        for p in (self.qkv, self.ba, self.g, self.o):
            p.bind(weights, ctx)
        self.conv_w = torch.cat([weights[n + self.conv_suffix].float() for n in self.proj_names], dim=0).contiguous()
        self.a_log = weights[self.a_log_name].float().reshape(-1).contiguous()
        self.dt_bias = weights[self.dt_bias_name].float().reshape(-1).contiguous()
        self.norm_w = weights[self.norm_name].float().contiguous()

    def forward(self, x, step, cache):
        ops = self.ctx.ops
        state = cache.state
        kept = state[:, self.matrix_floats:] if self.kept_rows else None  # (a view: the kernels take a row stride)
        u = self.qkv.forward(x)
        ba = self.ba.forward(x, out_dtype=torch.float32)
        gate = self.g.forward(x)
        q, k, v = ops.delta_conv(u, self.conv_w, kept, step.token_seq, step.cu_tokens, step.seq_slots, self.G, self.dim,
                                 self.H, self.vdim, self.unit_eps, self.q_scale)
        if self.kept_rows:
            ops.conv_state_update(u, kept, self.kept_rows, step.cu_tokens, step.seq_slots)
        o = ops.delta_scan(q, k, v, ba, self.a_log, self.dt_bias, state, self.H, self.G, self.dim, self.vdim,
                           step.seq_slots, step.cu_tokens)
        return self.o.forward(ops.delta_out_norm(o, gate, self.norm_w, self.eps, self.H, self.vdim))
