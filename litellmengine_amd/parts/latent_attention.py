"""Latent attention: keys and values of all heads are made from one small vector per token,
and only that vector (and one rotated key part shared by the heads) is cached.

    q = W_q h                          per head [dim plain | rot_dim rotated]
    W_dkv h = [kv_rank | rot_dim]      c = RMSNorm(first part) * w   (the latent)
                                       k_rot = rotated(second part)  (one for all heads)
    per head: k_plain = W_uk c, v = W_uv c
    score = (q_plain . k_plain + q_rot . k_rot) * scale
    softmax over the keys AND one sink per head: the denominator also holds exp(sink_h)  (`sink=False`: the keys alone)
    out = W_o [heads' sum_j p_j v_j]

With `q_rank` the queries pass a latent of their own first, q = W_uq (RMSNorm(W_dq h) * w), and with `head_gate`
head a's result is multiplied by sigmoid(W_g h)_a, a gate that reads the mixer's input.

Nothing per head is ever made for a cached token.  Since q_plain . (W_uk c) = (W_uk^T q_plain) . c
and sum_j p_j (W_uv c_j) = W_uv (sum_j p_j c_j), a query is carried into the latent space once
(`q_lat`, one small product per head), all heads of a token attend to the same cached rows
[c | k_rot] as one multi-query attention whose values are the c rows themselves, and the
result is expanded by W_uv once per query.  Prompt portions, decoded tokens and whole prompts
are one case: the step's latents are written to their pages first, then every token attends
through the block table.  Scores, softmax and sums are 32-bit in every mode.
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence

import torch

from ..weights.spec import INIT_NORM, INIT_NORMAL, TensorSpec
from .base import BuildContext, CacheField, CacheSpec, Mixer
from .linear import Linear
from .position import RotaryInterleaved


class LatentAttention(Mixer):
    graph_safe = True

    def __init__(self, prefix: str, hidden_size: int, heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int,
                 scale: float, norm_eps: float, position: RotaryInterleaved, window: Optional[int] = None,
                 names: Sequence[str] = ("q", "dkv", "dkv.norm", "uk", "uv", "sink", "o"), sink: bool = True,
                 q_rank: Optional[int] = None, q_names: Sequence[str] = ("dq", "dq.norm", "uq"),
                 head_gate: Optional[str] = None):
        """`position` rotates the first `position.rotary_dim` of the `rot_dim` elements.  `names`: the
        checkpoint's names after `prefix` of the query projection, the down projection to
        [latent | rotated key], the latent's norm weight, the up projections to plain keys and to
        values, the sinks and the output projection.  `sink=False`: no sink tensor, an ordinary softmax.
        `q_rank`: the queries' latent size; then `q_names` are the names of the down projection, the latent's
        norm weight and the up projection to the heads' queries, and names[0] is not read.  `head_gate`: the name
        of the projection [heads, hidden] whose sigmoids gate the heads' results (None: no gate)."""
        if position.rotary_dim > rot_dim:
            raise ValueError("the rotation covers more elements than the rotated part has")
        self.prefix = prefix
        self.H, self.dim, self.rot, self.vdim, self.rank = heads, dim, rot_dim, vdim, kv_rank
        self.scale = float(scale)
        self.eps = float(norm_eps)
        self.window = window
        self.position = position
        q, dkv, dkv_norm, uk, uv, sink_name, o = (prefix + n for n in names)
        self.q_rank = None if q_rank is None else int(q_rank)
        self.has_sink = bool(sink)
        if self.q_rank is None:
            self.q = Linear([q], hidden_size, [heads * (dim + rot_dim)])
            self.dq = self.q_norm_name = None
        else:
            dq, dq_norm, uq = (prefix + n for n in q_names)
            self.dq = Linear([dq], hidden_size, [self.q_rank])
            self.q = Linear([uq], self.q_rank, [heads * (dim + rot_dim)])
            self.q_norm_name = dq_norm
        self.dkv = Linear([dkv], hidden_size, [kv_rank + rot_dim])
        self.gate = Linear([prefix + head_gate], hidden_size, [heads]) if head_gate else None
        self.o = Linear([o], heads * vdim, [hidden_size])
        self.norm_name, self.uk_name, self.uv_name, self.sink_name = dkv_norm, uk, uv, sink_name
        self.norm_w = self.uk_t = self.uv = self.sink = self.q_norm_w = None

    def _linears(self):
        return [p for p in (self.q, self.dq, self.dkv, self.gate, self.o) if p is not None]

    def cache_spec(self) -> CacheSpec:
        # the latents twice: token after token for the scores, transposed (the keys of one element
        # side by side) for the weighted sum, which the matrix cores contract over keys
        return CacheSpec((CacheField("c", 1, self.rank), CacheField("c_t", 1, self.rank, True),
                          CacheField("k_rot", 1, self.rot)), self.window)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs: Dict[str, TensorSpec] = {}
        for p in self._linears():
            specs.update(p.tensor_specs())
        specs[self.norm_name] = TensorSpec((self.rank,), INIT_NORM)
        specs[self.uk_name] = TensorSpec((self.H * self.dim, self.rank), INIT_NORMAL)
        specs[self.uv_name] = TensorSpec((self.H * self.vdim, self.rank), INIT_NORMAL)
        if self.has_sink:
            specs[self.sink_name] = TensorSpec((self.H,), INIT_NORMAL)
        if self.q_norm_name is not None:
            specs[self.q_norm_name] = TensorSpec((self.q_rank,), INIT_NORM)
        return specs

    def bind(self, weights, ctx: BuildContext) -> None:
        self.ctx = ctx
        for p in self._linears() + [self.position]:
            p.bind(weights, ctx)
        self.norm_w = weights[self.norm_name].contiguous()
        if self.q_norm_name is not None:
            self.q_norm_w = weights[self.q_norm_name].contiguous()
        # per head, ready for `x . W^T`: W_uk^T [rank, dim] (queries into the latent space) and W_uv [vdim, rank]
        uk = weights[self.uk_name].to(ctx.dtype).view(self.H, self.dim, self.rank)
        self.uk_t = uk.transpose(1, 2).contiguous()
        self.uv = weights[self.uv_name].to(ctx.dtype).view(self.H, self.vdim, self.rank).contiguous()
        self.sink = weights[self.sink_name].float().contiguous() if self.has_sink else None

    def forward(self, x, step, cache):
        ops = self.ctx.ops
        group = cache.group
        cos_sin = self.position.table(step)
        rot_dims = self.position.rotary_dim
        if self.dq is None:
            q = self.q.forward(x)
        else:  # the queries' latent: its norm reads the product's 32-bit result
            q = self.q.forward(ops.rmsnorm(self.dq.forward(x, out_dtype=torch.float32), self.q_norm_w, self.eps,
                                           out_dtype=self.ctx.dtype))
        dkv = self.dkv.forward(x)
        if cache.writes:
            ops.latent_kv_write(dkv, self.norm_w, self.eps, cos_sin, rot_dims, group.slot_mapping, cache.pages,
                                group.page_size, self.rank, self.rot)
        q_rot = ops.latent_q_rope(q, cos_sin, rot_dims, self.H, self.dim, self.rot)
        q_lat = ops.heads_linear(q, self.H, 0, self.dim, self.uk_t,
                                 ops.latent_query_dtype(self.ctx.dtype, group.page_size, self.rank, self.rot))  # [N, H, rank]
        o_lat = ops.latent_attention(
            q_lat, q_rot, cache.pages, group.page_size, self.rank, self.rot, group.block_table, step.seq_slots,
            step.cu_tokens, step.kv_lens, step.token_seq, self.sink, self.window, self.scale, step.max_q_len,
            step.max_kv_len, self.ctx.dtype,
        )
        v = ops.heads_linear(o_lat, self.H, 0, self.rank, self.uv, self.ctx.dtype)  # [N, H, vdim]
        v = v.reshape(v.shape[0], self.H * self.vdim)
        if self.gate is not None:
            v = ops.head_gate(v, self.gate.forward(x), 0, self.H, self.vdim)
        return self.o.forward(v)
