"""Birelix: how its configuration becomes parts.

The layers are listed one by one in the configuration; layer i's tensors start with `l<i>.`, its mixer's
with `l<i>.mix.`, its feed-forward's with `l<i>.mlp.`, its norms are `l<i>.norm1` (before the mixer) and
`l<i>.norm2` (before the feed-forward).  Every layer is a pre-norm block; the mixer is latent attention whose
queries pass a latent of their own and whose heads are gated, grouped-query attention over a sliding window
(biases, q and k divided by their heads' root mean square, no rotation, one more place in the softmax's
sum), or the gated delta rule; the feed-forward is dense (gated, tanh-gelu), routed (sigmoid scores, the
best groups by their two largest scores, clamped experts), or absent.  The embedding's rows are scaled; the
output head is the embedding table as it is stored.
"""
from __future__ import annotations

from ..config.birelix_config import ATTENTION, DELTA, LATENT, BirelixConfig, BirelixLayer, DenseSizes
from ..config.registry import register_architecture
from ..parts import (Embedding, GatedDeltaMixer, GatedMLP, GroupLimitedMLP, LatentAttention, Linear, NoPositionEncoding,
                     PreNormBlock, RMSNorm, RotaryInterleaved, SinkAttention)
from .decoder import DecoderLM, PlanEntry

GROUP_TOP = 2  # a group of experts is worth the sum of its two largest scores


def _mixer(c: BirelixConfig, layer: BirelixLayer, prefix: str):
    m = layer.mixer
    if layer.type == LATENT:
        if m.kv_rank is None or m.q_rank is None:
            raise ValueError("the latents' sizes are not known yet: they are read from the checkpoint's shapes "
                             "(BirelixConfig.with_tensor_shapes) or given as `kv_rank` and `q_rank`")
        return LatentAttention(prefix, c.width, m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank, m.scale, c.norm_eps,
                               RotaryInterleaved(m.rot_dims, m.rot_base), sink=False, q_rank=m.q_rank, head_gate="g")
    if layer.type == ATTENTION:
        return SinkAttention(prefix, c.width, m.heads, m.kv_heads, m.dim, m.vdim, NoPositionEncoding(), c.norm_eps, m.scale,
                             window=m.window, sink=0.0, norm_over="head", norm_weights=False, gate=False)
    if layer.type == DELTA:
        if m.conv is None:
            raise ValueError("the convolution's length is not known yet: it is read from the checkpoint's shapes "
                             "(BirelixConfig.with_tensor_shapes) or given as `conv`")
        return GatedDeltaMixer(prefix, c.width, m.heads, m.kv_heads, m.dim, m.vdim, m.conv, c.norm_eps)
    raise ValueError(f"unknown mixer {layer.type!r}")


def _feed_forward(c: BirelixConfig, f, prefix: str):
    if isinstance(f, DenseSizes):
        return GatedMLP(prefix, c.width, f.ff, names=("gate", "up", "down"), activation="gelu_tanh")
    return GroupLimitedMLP(prefix, c.width, f.ff, f.experts, f.top, groups=f.groups, groups_kept=f.groups_kept,
                           score="sigmoid", correction=False, group_top=GROUP_TOP, form="gated_clamp", limit=f.limit)


def build_birelix(config: BirelixConfig) -> DecoderLM:
    c = config
    norm = lambda name: RMSNorm(name, c.width, c.norm_eps)
    blocks = []
    for i, layer in enumerate(c.layers):
        p = f"l{i}."
        mixer = _mixer(c, layer, p + "mix.")
        if layer.mlp is None:
            blocks.append(PreNormBlock(norm(p + "norm1"), mixer))
        else:
            blocks.append(PreNormBlock(norm(p + "norm1"), mixer, norm(p + "norm2"), _feed_forward(c, layer.mlp, p + "mlp.")))
    return DecoderLM(
        config=c,
        embedding=Embedding("embed", c.vocab, c.width, scale=c.embedding_scale),
        blocks=blocks,
        plan=[PlanEntry(i) for i in range(len(blocks))],
        final_norm=norm("final.norm"),
        head=Linear(["head"], c.width, [c.vocab], optional=True),
        tied_head=True,
    )


register_architecture(BirelixConfig.ARCHITECTURE, BirelixConfig, build_birelix)
