"""Grouped-query attention over the paged cache.

q/k/v projections (no bias) -> RMSNorm of each q and k head over head_dim with
one weight [head_dim] for all heads, before the position encoding; v untouched
-> position encoding of q and k -> K (ready to dot) and V written to the pages
-> attention of every token of the step through the block table -> output
projection.  src/model/qwen3.cpp:375-377, :391-407, :443-449, :464-481,
:498-557, :565-567.  scale = 1/sqrt(head_dim) (src/ops/attention.cu:201); kv
head of q head h is h // (nq // nkv) (:196-199).  The q/k norm is optional and
the position encoding is a part of its own, so the same mixer serves models
without either; `window` limits a query to the last `window` keys (the
reference has full attention only).
"""
from __future__ import annotations

import math
from typing import Dict, Optional, Sequence

import torch

from ..csrc.limits import check_head_dim
from ..weights.spec import INIT_NORM, INIT_NORMAL, TensorSpec
from ..weights.spec import INIT_WIDE
from .base import BuildContext, CacheSpec, KVCacheSpec, Mixer, PositionEncoding, StateSpec
from .linear import Linear


class PagedAttention(Mixer):
    graph_safe = True
    folds_norm = True

    def __init__(
        self,
        prefix: str,
        hidden_size: int,
        num_q_heads: int,
        num_kv_heads: int,
        head_dim: int,
        position: PositionEncoding,
        qk_norm_eps: Optional[float] = None,
        window: Optional[int] = None,
        scale: Optional[float] = None,
        qkv_names: Optional[Sequence[str]] = None,
        o_name: Optional[str] = None,
        qkv_bias: bool = False,
        o_bias: bool = False,
        qk_norm_names: Optional[Sequence[str]] = None,
    ):
        """`qkv_names`: the checkpoint's names of the projections' weights after `prefix`, three
        (q, k, v; default q_proj.weight, k_proj.weight, v_proj.weight) or one that holds the three
        stacked in that order; `o_name` the output projection's (default o_proj.weight);
        `qk_norm_names` the two norm weights' (default q_norm.weight, k_norm.weight).  With
        `qkv_bias` / `o_bias` every weight `x.weight` has a bias `x.bias`."""
        if num_q_heads % num_kv_heads:
            raise ValueError("num_q_heads must be a multiple of num_kv_heads")
        check_head_dim(head_dim, getattr(position, "rotary_dim", 0))  # what no kernel takes is refused now, not at the first step
        self.prefix = prefix
        self.nq, self.nkv, self.d = num_q_heads, num_kv_heads, head_dim
        self.position = position
        self.qk_norm_eps = qk_norm_eps
        self.window = window
        self.scale = 1.0 / math.sqrt(head_dim) if scale is None else float(scale)
        widths = [num_q_heads * head_dim, num_kv_heads * head_dim, num_kv_heads * head_dim]
        names = list(qkv_names) if qkv_names else ["q_proj.weight", "k_proj.weight", "v_proj.weight"]
        if len(names) == 1:
            widths = [sum(widths)]  # the three stacked in one checkpoint tensor
        elif len(names) != 3:
            raise ValueError("qkv_names holds three names (q, k, v) or one (the three stacked)")
        o_name = o_name or "o_proj.weight"
        bias_of = lambda name: prefix + (name[: -len("weight")] + "bias" if name.endswith("weight") else name + ".bias")
        self.qkv = Linear([prefix + n for n in names], hidden_size, widths,
                          bias_names=[bias_of(n) for n in names] if qkv_bias else None)
        self.o = Linear([prefix + o_name], num_q_heads * head_dim, [hidden_size], to_residual=True,
                        bias_names=[bias_of(o_name)] if o_bias else None)
        self.folds_norm = not o_bias  # (the product before a folded norm adds into the residual stream itself)
        self.qk_norm_names = list(qk_norm_names) if qk_norm_names else ["q_norm.weight", "k_norm.weight"]
        if len(self.qk_norm_names) != 2:
            raise ValueError("qk_norm_names holds two names (q, k)")
        self.q_norm_w = None
        self.k_norm_w = None

    def cache_spec(self) -> CacheSpec:
        return KVCacheSpec(self.nkv, self.d, self.window)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs = {**self.qkv.tensor_specs(), **self.o.tensor_specs()}
        if self.qk_norm_eps is not None:
            for name in self.qk_norm_names:
                specs[self.prefix + name] = TensorSpec((self.d,), INIT_NORM)
        return specs

    def bind(self, weights, ctx: BuildContext) -> None:
        self.ctx = ctx
        self.qkv.bind(weights, ctx)
        self.o.bind(weights, ctx)
        self.position.bind(weights, ctx)
        if self.qk_norm_eps is not None:
            qw = weights[self.prefix + self.qk_norm_names[0]]
            kw = weights[self.prefix + self.qk_norm_names[1]]
            if qw.dtype != kw.dtype:
                qw, kw = qw.float(), kw.float()
            self.q_norm_w, self.k_norm_w = qw.contiguous(), kw.contiguous()

    def forward(self, x, step, cache, fold=None):
        ops = self.ctx.ops
        qkv = self.qkv.forward(x)
        fused = self.position.fused_rotary(step)
        eps = self.qk_norm_eps if self.qk_norm_eps is not None else 0.0
        group = cache.group
        if fused is not None:
            cos_sin, rot = fused
            if ops.can_fuse_rope_attention(qkv.dtype, self.d, rot, cache.kv.shape[3], self.nq // self.nkv,
                                           step.max_q_len, step.max_kv_len, step.seq_slots.shape[0]):
                # a decode step: norm, rotation, cache write and attention in one launch
                a = ops.qk_norm_rope_attention(
                    qkv, group.slot_mapping, self.q_norm_w, self.k_norm_w, cos_sin, eps, cache.kv, self.nq,
                    self.nkv, self.d, cache.writes, group.block_table, step.seq_slots, step.cu_tokens,
                    step.kv_lens, step.token_seq, self.window, self.scale, step.max_kv_len,
                )
                return self.o.forward(a, fold=fold)
            q = ops.qk_norm_rope_write(
                qkv, group.slot_mapping, self.q_norm_w, self.k_norm_w, cos_sin, rot, eps,
                cache.kv, self.nq, self.nkv, self.d, cache.writes,
            )
        else:
            # an encoding the fused kernel does not know: norm, encode, then write
            N = qkv.shape[0]
            qw, kw = self.nq * self.d, self.nkv * self.d
            q = qkv[:, :qw].reshape(N * self.nq, self.d).contiguous()
            k = qkv[:, qw : qw + kw].reshape(N * self.nkv, self.d).contiguous()
            if self.qk_norm_eps is not None:
                q = ops.rmsnorm(q, self.q_norm_w, eps)
                k = ops.rmsnorm(k, self.k_norm_w, eps)
            q, k = self.position.apply(q.view(N, self.nq, self.d), k.view(N, self.nkv, self.d), step.positions)
            packed = torch.cat([q.reshape(N, qw), k.reshape(N, kw), qkv[:, qw + kw :]], dim=1).contiguous()
            q = ops.qk_norm_rope_write(
                packed, group.slot_mapping, None, None, None, 0, 0.0,
                cache.kv, self.nq, self.nkv, self.d, cache.writes,
            )
        a = ops.paged_attention(
            q, cache.kv, group.block_table, step.seq_slots, step.cu_tokens, step.kv_lens, step.token_seq,
            self.window, self.scale, step.min_q_len, step.max_q_len, step.max_kv_len,
        )
        return self.o.forward(a, fold=fold)


class SinkAttention(Mixer):
    """Grouped-query attention over the paged cache whose softmax has a sink and whose heads are gated:

        q = W_q h + b_q, k = W_k h + b_k, v = W_v h + b_v
        q, k <- divided by the root mean square of the WHOLE projection (all heads at once), times a
                weight per element; then the position encoding on the first elements of every head
                (`norm_over="head"`: every head by its own root mean square; `norm_weights=False`: no
                weight tensors, the division alone)
        p_j = exp(s_j) / (exp(sink) + sum_j exp(s_j)),  s_j = (q . k_j) * scale,  over the last `window` keys
        out = W_o [heads' (sum_j p_j v_j) * sigmoid(W_g h)_head]        (`gate=False`: no gate, no W_g)

    Keys may be `dim` wide and values `vdim`: the cache's heads hold `cache_dim` >= both elements (a
    multiple of 32, which the matrix-core kernels take), the rest zeros, so the kernels of
    `PagedAttention` serve.  With `own_kv=False` the mixer has no key and value tensors: its plan
    entry reads the cache that another layer's mixer writes, with queries, window and gate of its
    own.  `cache_window` is what the cache keeps (the largest window of all mixers that read it;
    default: this mixer's own)."""

    graph_safe = True
    UNBOUNDED = object()  # cache_window: keep every position, whatever this mixer's own window

    def __init__(self, prefix: str, hidden_size: int, num_q_heads: int, num_kv_heads: int, dim: int, vdim: int,
                 position: PositionEncoding, norm_eps: float, scale: float, window: Optional[int] = None,
                 sink: Optional[float] = 0.0, own_kv: bool = True, cache_window=None,
                 names: Sequence[str] = ("q", "k", "v", "g", "o"), bias_suffix: str = ".b", norm_suffix: str = ".norm",
                 norm_over: str = "projection", norm_weights: bool = True, gate: bool = True):
        if num_q_heads % num_kv_heads:
            raise ValueError("num_q_heads must be a multiple of num_kv_heads")
        self.cache_dim = -(-max(dim, vdim) // 32) * 32
        check_head_dim(self.cache_dim, getattr(position, "rotary_dim", 0))
        if getattr(position, "rotary_dim", 0) > dim:
            raise ValueError("the rotation covers more elements than a key has")
        self.prefix = prefix
        self.hidden = hidden_size
        self.nq, self.nkv, self.dim, self.vdim = num_q_heads, num_kv_heads, dim, vdim
        self.position = position
        self.eps = float(norm_eps)
        self.scale = float(scale)
        self.window = window
        self.sink = sink
        self.own_kv = bool(own_kv)
        if norm_over not in ("projection", "head"):
            raise ValueError(f"q and k are normed over the whole projection or head by head, not over {norm_over!r}")
        self.per_head, self.norm_weights, self.gated = norm_over == "head", bool(norm_weights), bool(gate)
        if cache_window is SinkAttention.UNBOUNDED:
            self._cache_window = None
        else:
            self._cache_window = window if cache_window is None else cache_window
        q, k, v, g, o = (prefix + n for n in names)
        self.q_name, self.k_name, self.v_name, self.g_name = q, k, v, g
        self.bias_suffix, self.norm_suffix = bias_suffix, norm_suffix
        self.o = Linear([o], num_q_heads * vdim, [hidden_size])
        self.weight = self.bias = self.q_norm_w = self.k_norm_w = self.sinks = None

    def _widths(self):
        w = [(self.q_name, self.nq * self.dim, True)]
        if self.own_kv:
            w += [(self.k_name, self.nkv * self.dim, True), (self.v_name, self.nkv * self.vdim, True)]
        return w + ([(self.g_name, self.nq, False)] if self.gated else [])  # (name, rows, has a bias)

    def cache_spec(self) -> CacheSpec:
        return KVCacheSpec(self.nkv, self.cache_dim, self._cache_window)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs = dict(self.o.tensor_specs())
        for name, rows, biased in self._widths():
            specs[name] = TensorSpec((rows, self.hidden), INIT_NORMAL)
            if biased:
                specs[name + self.bias_suffix] = TensorSpec((rows,), INIT_NORMAL)
        if self.norm_weights:
            specs[self.q_name + self.norm_suffix] = TensorSpec((self.nq * self.dim,), INIT_NORM)
            if self.own_kv:
                specs[self.k_name + self.norm_suffix] = TensorSpec((self.nkv * self.dim,), INIT_NORM)
        return specs

    def bind(self, weights, ctx: BuildContext) -> None:
        self.ctx = ctx
        if self.gated or self.cache_dim == self.vdim:
            self.o.bind(weights, ctx)
        else:  # without gates nothing drops the cache's padding: the output projection gets zero columns there
            o = weights[self.o.names[0]].to(ctx.dtype)
            o = torch.nn.functional.pad(o.view(self.hidden, self.nq, self.vdim), (0, self.cache_dim - self.vdim))
            self.o.bind_tensor(o.reshape(self.hidden, self.nq * self.cache_dim).contiguous(), ctx)
        self.position.bind(weights, ctx)
        # one product for q, (k, v,) and the gates' inputs; the gates have no bias
        self.weight = torch.cat([weights[name].to(ctx.dtype) for name, _, _ in self._widths()], dim=0).contiguous()
        self.bias = torch.cat([
            weights[name + self.bias_suffix].to(ctx.dtype).reshape(-1) if biased
            else torch.zeros(rows, dtype=ctx.dtype, device=ctx.device)
            for name, rows, biased in self._widths()]).contiguous()
        self.q_norm_w = self.k_norm_w = None
        if self.norm_weights:
            self.q_norm_w = weights[self.q_name + self.norm_suffix].float().contiguous()
            self.k_norm_w = weights[self.k_name + self.norm_suffix].float().contiguous() if self.own_kv else None
        self.sinks = None if self.sink is None else torch.full((self.nq,), float(self.sink), dtype=torch.float32,
                                                               device=ctx.device)

    def forward(self, x, step, cache):
        ops = self.ctx.ops
        if cache.writes != self.own_kv:
            raise ValueError("a mixer with keys and values of its own writes its cache, one without reads another's")
        group = cache.group
        qkvg = ops.linear(x, self.weight)
        cos_sin, rot = self.position.fused_rotary(step)
        q = ops.proj_norm_rope_write(qkvg, self.bias, group.slot_mapping, self.q_norm_w, self.k_norm_w, cos_sin, rot,
                                     self.eps, cache.kv, self.nq, self.nkv, self.dim, self.vdim, self.own_kv, cache.writes,
                                     per_head=self.per_head)
        a = ops.paged_attention(q, cache.kv, group.block_table, step.seq_slots, step.cu_tokens, step.kv_lens,
                                step.token_seq, self.window, self.scale, step.min_q_len, step.max_q_len, step.max_kv_len,
                                sinks=self.sinks)
        if self.gated:  # (the gates' kernel also drops the cache's padding)
            return self.o.forward(ops.head_gate(a, qkvg, qkvg.shape[1] - self.nq, self.nq, self.vdim))
        return self.o.forward(a)  # heads of cache_dim elements, zeros past vdim, against zero columns of the weight


class ConvAttention(Mixer):
    """Grouped-query attention whose projections pass a short causal convolution over time first:

        u = (W_q h, W_k h, W_v h)                         one stacked product, no biases
        c_t = sum_j taps[:, j] * u_(t - J + 1 + j)        per channel, J taps, zeros before a request's start
        q, k <- every head of c's q and k parts divided by its root mean square, times one weight [dim]
                for all heads; then the position encoding on the first elements of every head
        p_j = softmax_j((q . k_j) * scale) over every earlier token and the token itself
        out = out_scale * W_o [heads' sum_j p_j v_j]

    Keys may be `dim` wide and values `vdim`: the cache's heads hold `cache_dim` >= both elements (a
    multiple of 32, which the matrix-core kernels take), the rest zeros, so the kernels of
    `PagedAttention` serve; the output projection reads zeros against zero columns there.  The last
    J - 1 rows of u of every request are its state (`StateSpec`, float32): what the next step's first
    tokens are convolved with.  The taps are kept in 32-bit, and `out_scale` is folded into the taps of
    v (the result is linear in v), so it costs no operation and no rounding of its own."""

    graph_safe = True

    def __init__(self, prefix: str, hidden_size: int, num_q_heads: int, num_kv_heads: int, dim: int, vdim: int,
                 position: PositionEncoding, norm_eps: float, scale: float, taps: int = 0, out_scale: float = 1.0,
                 names: Sequence[str] = ("q", "k", "v", "o"), conv_suffix: str = ".conv", norm_suffix: str = ".norm"):
        """`taps`: the convolution's length J (0 or 1 without a tensor: none).  The checkpoint's tensors are
        `prefix` + q, k, v (projections), + `conv_suffix` (their taps, [channels, J]), + `norm_suffix` (q and k: the
        heads' norm weight [dim]) and o."""
        if num_q_heads % num_kv_heads:
            raise ValueError("num_q_heads must be a multiple of num_kv_heads")
        self.cache_dim = -(-max(dim, vdim) // 32) * 32
        check_head_dim(self.cache_dim, getattr(position, "rotary_dim", 0))
        if getattr(position, "rotary_dim", 0) > dim:
            raise ValueError("the rotation covers more elements than a key has")
        if taps < 0:
            raise ValueError("a convolution has no negative number of taps")
        self.prefix, self.hidden = prefix, hidden_size
        self.nq, self.nkv, self.dim, self.vdim = num_q_heads, num_kv_heads, dim, vdim
        self.position = position
        self.eps, self.scale, self.out_scale = float(norm_eps), float(scale), float(out_scale)
        self.taps = int(taps)
        q, k, v, o = (prefix + n for n in names)
        self.proj_names = (q, k, v)
        self.widths = (num_q_heads * dim, num_kv_heads * dim, num_kv_heads * vdim)
        self.cols = sum(self.widths)
        self.conv_suffix, self.norm_suffix = conv_suffix, norm_suffix
        self.o_name = o
        self.o = Linear([o], num_q_heads * vdim, [hidden_size])
        self.weight = self.conv_w = self.q_norm_w = self.k_norm_w = None

    @property
    def kept_rows(self) -> int:
        """Rows of the projections that a request keeps from step to step."""
        return max(0, self.taps - 1)

    def cache_spec(self) -> CacheSpec:
        return KVCacheSpec(self.nkv, self.cache_dim, None)

    def state_spec(self) -> Optional[StateSpec]:
        return StateSpec((self.kept_rows * self.cols,), torch.float32) if self.kept_rows else None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs = dict(self.o.tensor_specs())
        for name, rows in zip(self.proj_names, self.widths):
            specs[name] = TensorSpec((rows, self.hidden), INIT_NORMAL)
            if self.taps:
                specs[name + self.conv_suffix] = TensorSpec((rows, self.taps), INIT_WIDE)
        for name in self.proj_names[:2]:
            specs[name + self.norm_suffix] = TensorSpec((self.dim,), INIT_NORM)
        return specs

    def bind(self, weights, ctx: BuildContext) -> None:
        self.ctx = ctx
        self.position.bind(weights, ctx)
        self.weight = torch.cat([weights[n].to(ctx.dtype) for n in self.proj_names], dim=0).contiguous()
        if self.taps:
            taps = torch.cat([weights[n + self.conv_suffix].float() for n in self.proj_names], dim=0)
        else:  # one tap of one: the projection itself
            taps = torch.ones((self.cols, 1), dtype=torch.float32, device=self.weight.device)
        taps = taps.clone()
        taps[self.widths[0] + self.widths[1]:] *= self.out_scale  # the attention's result is linear in v
        self.conv_w = taps.to(ctx.device).contiguous()
        self.q_norm_w = weights[self.proj_names[0] + self.norm_suffix].float().contiguous()
        self.k_norm_w = weights[self.proj_names[1] + self.norm_suffix].float().contiguous()
        o = weights[self.o_name].to(ctx.dtype)
        if self.cache_dim != self.vdim:  # the attention hands out heads of cache_dim elements, zeros past vdim
            o = torch.nn.functional.pad(o.view(self.hidden, self.nq, self.vdim), (0, self.cache_dim - self.vdim))
            o = o.reshape(self.hidden, self.nq * self.cache_dim)
        self.o.bind_tensor(o.contiguous(), ctx)

    def forward(self, x, step, cache):
        ops = self.ctx.ops
        group = cache.group
        u = ops.linear(x, self.weight)
        cos_sin, rot = self.position.fused_rotary(step)
        q = ops.conv_norm_rope_write(u, self.conv_w, cache.state if self.kept_rows else None, step.token_seq,
                                     step.cu_tokens, step.seq_slots, group.slot_mapping, self.q_norm_w, self.k_norm_w,
                                     cos_sin, rot, self.eps, cache.kv, self.nq, self.nkv, self.dim, self.vdim, cache.writes)
        if self.kept_rows:
            ops.conv_state_update(u, cache.state, self.kept_rows, step.cu_tokens, step.seq_slots)
        a = ops.paged_attention(q, cache.kv, group.block_table, step.seq_slots, step.cu_tokens, step.kv_lens,
                                step.token_seq, None, self.scale, step.min_q_len, step.max_q_len, step.max_kv_len)
        return self.o.forward(a)
