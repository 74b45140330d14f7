"""Birelix: a decoder whose layers are listed one by one in config.json.  Every layer is pre-norm,
`x <- x + mixer(norm1(x))`, then `x <- x + ff(norm2(x))` (or no second line).  The mixer is latent
attention with a query latent and a gate per head, grouped-query attention over a sliding window
whose softmax has one more place in its sum, or a gated delta rule (a matrix state per head that is
corrected towards each new value); the feed-forward is dense (gated, tanh-gelu), a mixture of clamped
experts chosen by sigmoid scores among the best groups, or absent.  The embedding's rows are scaled and
the embedding table is the output head.

config.json keys: `architecture` (a string), `vocab`, `width`, `embedding.scale`, `norm.eps`, and
`layers`: a list of `{type, mixer: {...}, mlp: {...} | null}`:

  latent_attention  mixer: heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, rot.{base, dims}
                    (kv_rank and q_rank may be left to the shapes of `mix.dkv.norm` and `mix.dq.norm`)
  attention         mixer: heads, kv_heads, dim, vdim, scale, mask.size (absent: every earlier token is seen)
  delta             mixer: heads, kv_heads, dim, vdim, conv (taps; may be left to the shape of `mix.q.conv`)
  mlp               kind "dense": ff
                    kind "moe":   router.{experts, top, groups.{count, keep}}, expert.{ff, limit}

Every size and every constant that may differ between models is read from there (or from a
tensor's shape); nothing of it stands in code.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, Mapping, Optional, Tuple

from .model_config import ConfigError, _optional, _required

LATENT, ATTENTION, DELTA = "latent_attention", "attention", "delta"
MIXER_TYPES = (LATENT, ATTENTION, DELTA)
DENSE, MOE = "dense", "moe"


def _section(d: Dict[str, Any], key: str, where: str) -> Dict[str, Any]:
    v = d.get(key)
    if not isinstance(v, dict):
        raise ConfigError(f"{where} needs an object `{key}`")
    return v


def _positive(value, what: str):
    if not value > 0:
        raise ConfigError(f"Birelix config {what} must be positive")
    return value


@dataclasses.dataclass(frozen=True)
class LatentSizes:
    heads: int
    dim: int  # unrotated query/key elements per head
    rot_dim: int  # rotated query/key elements per head (the key's are shared by the heads)
    vdim: int
    scale: float
    rot_base: float
    rot_dims: int  # how many of the rot_dim elements the rotation covers
    kv_rank: Optional[int] = None  # None until a checkpoint's shapes have said it
    q_rank: Optional[int] = None


@dataclasses.dataclass(frozen=True)
class WindowSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: Optional[int] = None  # None: every earlier token is seen


@dataclasses.dataclass(frozen=True)
class DeltaSizes:
    heads: int  # value heads (and states)
    kv_heads: int  # query/key heads
    dim: int
    vdim: int
    conv: Optional[int] = None  # taps; None until a checkpoint's shapes have said it


@dataclasses.dataclass(frozen=True)
class DenseSizes:
    ff: int


@dataclasses.dataclass(frozen=True)
class RoutedSizes:
    experts: int
    top: int
    ff: int
    limit: float
    groups: int = 1
    groups_kept: int = 1


@dataclasses.dataclass(frozen=True)
class BirelixLayer:
    type: str
    mixer: Any  # LatentSizes, WindowSizes or DeltaSizes
    mlp: Any  # DenseSizes, RoutedSizes or None


def _heads(m: Dict[str, Any], where: str):
    heads = _positive(_required(m, "heads", int), f"{where}.heads")
    kv_heads = _positive(_optional(m, "kv_heads", int, heads), f"{where}.kv_heads")
    if heads % kv_heads:
        raise ConfigError(f"{where}.heads must be a multiple of kv_heads")
    return heads, kv_heads


def _mixer_from(kind: str, m: Dict[str, Any], where: str):
    dim = _positive(_required(m, "dim", int), f"{where}.dim")
    vdim = _positive(_optional(m, "vdim", int, dim), f"{where}.vdim")
    if kind == LATENT:
        rot_dim = _positive(_required(m, "rot_dim", int), f"{where}.rot_dim")
        rot = m.get("rot") if isinstance(m.get("rot"), dict) else {}
        rot_dims = _optional(rot, "dims", int, rot_dim)
        if rot_dims % 2 or not 0 <= rot_dims <= rot_dim:
            raise ConfigError(f"{where}.rot.dims must be even and at most rot_dim")
        ranks = []
        for key in ("kv_rank", "q_rank"):
            r = _optional(m, key, int, None)
            ranks.append(None if r is None else _positive(r, f"{where}.{key}"))
        return LatentSizes(
            heads=_positive(_required(m, "heads", int), f"{where}.heads"), dim=dim, rot_dim=rot_dim, vdim=vdim,
            scale=_optional(m, "scale", float, float(dim + rot_dim) ** -0.5),
            rot_base=_positive(_optional(rot, "base", float, 10000.0), f"{where}.rot.base"), rot_dims=rot_dims,
            kv_rank=ranks[0], q_rank=ranks[1])
    heads, kv_heads = _heads(m, where)
    if kind == ATTENTION:
        mask = m.get("mask") if isinstance(m.get("mask"), dict) else {}
        window = _optional(mask, "size", int, None)
        if window is not None:
            _positive(window, f"{where}.mask.size")
        return WindowSizes(heads, kv_heads, dim, vdim, _optional(m, "scale", float, float(dim) ** -0.5), window)
    conv = _optional(m, "conv", int, None)
    if conv is not None:
        _positive(conv, f"{where}.conv")
    return DeltaSizes(heads, kv_heads, dim, vdim, conv)


def _mlp_from(m: Optional[Dict[str, Any]], where: str):
    if m is None:
        return None
    if not isinstance(m, dict):
        raise ConfigError(f"{where}.mlp must be an object or null")
    kind = m.get("kind")
    if kind == DENSE:
        return DenseSizes(_positive(_required(m, "ff", int), f"{where}.mlp.ff"))
    if kind != MOE:
        raise ConfigError(f"{where}.mlp.kind={kind!r} is unknown ({DENSE}, {MOE})")
    router = _section(m, "router", f"{where}.mlp")
    expert = _section(m, "expert", f"{where}.mlp")
    experts = _positive(_required(router, "experts", int), f"{where}.mlp.router.experts")
    top = _positive(_required(router, "top", int), f"{where}.mlp.router.top")
    groups = router.get("groups") if isinstance(router.get("groups"), dict) else {}
    count = _positive(_optional(groups, "count", int, 1), f"{where}.mlp.router.groups.count")
    keep = _positive(_optional(groups, "keep", int, count), f"{where}.mlp.router.groups.keep")
    if experts % count or keep > count:
        raise ConfigError(f"{where}.mlp.router: the experts form `groups.count` equal groups, of which at most all are kept")
    if top > keep * (experts // count):
        raise ConfigError(f"{where}.mlp.router.top is larger than the number of experts in the kept groups")
    return RoutedSizes(experts, top, _positive(_required(expert, "ff", int), f"{where}.mlp.expert.ff"),
                       _positive(_required(expert, "limit", float), f"{where}.mlp.expert.limit"), count, keep)


@dataclasses.dataclass(frozen=True)
class BirelixConfig:
    architecture: str
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    layers: Tuple[BirelixLayer, ...]

    ARCHITECTURE = "Birelix"

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "BirelixConfig":
        layers = d.get("layers")
        if not isinstance(layers, list):
            raise ConfigError("Missing required config field: layers")
        out = []
        for i, layer in enumerate(layers):
            where = f"layers[{i}]"
            if not isinstance(layer, dict) or layer.get("type") not in MIXER_TYPES:
                kind = layer.get("type") if isinstance(layer, dict) else layer
                raise ConfigError(f"{where}.type={kind!r} is unknown ({', '.join(MIXER_TYPES)})")
            out.append(BirelixLayer(layer["type"], _mixer_from(layer["type"], _section(layer, "mixer", where), f"{where}.mixer"),
                                    _mlp_from(layer.get("mlp"), where)))
        embedding = d.get("embedding") if isinstance(d.get("embedding"), dict) else {}
        return cls(
            architecture=str(d.get("architecture") or (d.get("architectures") or [cls.ARCHITECTURE])[0]),
            vocab=_positive(_required(d, "vocab", int), "vocab"),
            width=_positive(_required(d, "width", int), "width"),
            embedding_scale=_optional(embedding, "scale", float, 1.0),
            norm_eps=_positive(_required(_section(d, "norm", "Birelix config"), "eps", float), "norm.eps"),
            layers=tuple(out),
        )

    def with_tensor_shapes(self, shapes: Mapping[str, Tuple[int, ...]]) -> "BirelixConfig":
        """The sizes that config.json may leave to the checkpoint, read from its tensors' shapes: the two ranks of
        a latent attention (`l<i>.mix.dkv.norm`, `l<i>.mix.dq.norm`) and the taps of a delta layer's convolutions
        (columns of `l<i>.mix.q.conv`)."""
        def shape_of(name, dims):
            shape = shapes.get(name)
            if shape is None or len(shape) != dims:
                raise ConfigError(f"the checkpoint has no tensor {name} of {dims} dimension(s) to read a size from")
            return shape

        layers = []
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            if layer.type == LATENT and (m.kv_rank is None or m.q_rank is None):
                m = dataclasses.replace(
                    m, kv_rank=m.kv_rank if m.kv_rank is not None else int(shape_of(f"l{i}.mix.dkv.norm", 1)[0]),
                    q_rank=m.q_rank if m.q_rank is not None else int(shape_of(f"l{i}.mix.dq.norm", 1)[0]))
            elif layer.type == DELTA and m.conv is None:
                m = dataclasses.replace(m, conv=int(shape_of(f"l{i}.mix.q.conv", 2)[1]))
            layers.append(dataclasses.replace(layer, mixer=m))
        return dataclasses.replace(self, layers=tuple(layers))

    def to_dict(self) -> Dict[str, Any]:
        layers = []
        for layer in self.layers:
            m = layer.mixer
            if isinstance(m, LatentSizes):
                mixer: Dict[str, Any] = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim, "scale": m.scale,
                                         "rot": {"base": m.rot_base, "dims": m.rot_dims}}
                if m.kv_rank is not None:
                    mixer["kv_rank"] = m.kv_rank
                if m.q_rank is not None:
                    mixer["q_rank"] = m.q_rank
            elif isinstance(m, WindowSizes):
                mixer = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale}
                if m.window is not None:
                    mixer["mask"] = {"size": m.window}
            else:
                mixer = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim}
                if m.conv is not None:
                    mixer["conv"] = m.conv
            f = layer.mlp
            if f is None:
                mlp = None
            elif isinstance(f, DenseSizes):
                mlp = {"kind": DENSE, "ff": f.ff}
            else:
                mlp = {"kind": MOE, "expert": {"ff": f.ff, "limit": f.limit},
                       "router": {"experts": f.experts, "top": f.top, "groups": {"count": f.groups, "keep": f.groups_kept}}}
            layers.append({"type": layer.type, "mixer": mixer, "mlp": mlp})
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps}, "layers": layers}
