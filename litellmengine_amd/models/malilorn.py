"""Malilorn: how its configuration becomes parts.

The layers are listed one by one in the configuration; layer i's tensors start with `l<i>.`, its
mixer's with `l<i>.mix.`, its feed-forward's with `l<i>.mlp.`, its four norms are `l<i>.norm1`,
`norm1b` (before and after the mixer), `norm2`, `norm2b` (before and after the feed-forward).  The
mixer is two mixers side by side (`mix.left.`: attention behind a short convolution; `mix.right.`: a
recurrence with a matrix state per head), each times a constant of the configuration; the
feed-forward is dense (gated, relu, with biases), routed by sigmoid scores with a shared expert, or
absent.  The output head is the embedding table; the logits are capped smoothly.
"""
from __future__ import annotations

from ..config.malilorn_config import DenseSizes, MalilornConfig, MalilornLayer
from ..config.registry import register_architecture
from ..parts import (ConvAttention, Embedding, GatedMLP, Linear, NoPositionEncoding, PlainMLP, RMSNorm, RotaryHalfSplit,
                     SandwichBlock, ScoreRoutedMLP, SideBySideMixer, WKVMixer)
from .decoder import DecoderLM, PlanEntry


def _mixer(c: MalilornConfig, layer: MalilornLayer, prefix: str):
    m = layer.mixer
    a, r = m.left, m.right
    if r.decay_rank is None:
        raise ValueError("the decay's inner rank is not known yet: it is read from the checkpoint's shapes "
                         "(MalilornConfig.with_tensor_shapes) or given as `decay_rank`")
    position = (RotaryHalfSplit(a.dim, a.rot_base, a.rot_dims, scaling=a.rot_scaling) if a.rot_dims
                else NoPositionEncoding())
    left = ConvAttention(prefix + "left.", c.width, a.heads, a.kv_heads, a.dim, a.vdim, position, c.norm_eps, a.scale,
                         taps=a.conv, out_scale=m.left_scale)
    right = WKVMixer(prefix + "right.", c.width, r.heads, r.dim, r.decay_rank, c.norm_eps, out_scale=m.right_scale)
    return SideBySideMixer(left, right)


def _feed_forward(c: MalilornConfig, f, prefix: str):
    if isinstance(f, DenseSizes):
        return GatedMLP(prefix, c.width, f.ff, names=("gate", "up", "down"), to_residual=False, activation="relu",
                        bias_names=("gate.b", "up.b", "down.b"))
    shared = PlainMLP(prefix + "shared.", c.width, f.shared_ff) if f.shared_ff is not None else None
    return ScoreRoutedMLP(prefix, c.width, f.ff, f.experts, f.top, shared=shared)


def build_malilorn(config: MalilornConfig) -> DecoderLM:
    c = config
    norm = lambda name: RMSNorm(name, c.width, c.norm_eps)
    blocks = []
    for i, layer in enumerate(c.layers):
        p = f"l{i}."
        mixer = _mixer(c, layer, p + "mix.")
        if layer.mlp is None:
            blocks.append(SandwichBlock(norm(p + "norm1"), mixer, norm(p + "norm1b")))
        else:
            blocks.append(SandwichBlock(norm(p + "norm1"), mixer, norm(p + "norm1b"), norm(p + "norm2"),
                                        _feed_forward(c, layer.mlp, p + "mlp."), norm(p + "norm2b")))
    return DecoderLM(
        config=c,
        embedding=Embedding("embed", c.vocab, c.width),
        blocks=blocks,
        plan=[PlanEntry(i) for i in range(len(blocks))],
        final_norm=norm("final.norm"),
        head=Linear(["head"], c.width, [c.vocab], optional=True),
        tied_head=True,
        logit_softcap=c.logit_softcap,
    )


register_architecture(MalilornConfig.ARCHITECTURE, MalilornConfig, build_malilorn)
