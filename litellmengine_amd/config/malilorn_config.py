"""Malilorn: a decoder whose layers are listed one by one in config.json.  Every layer is
`x <- x + norm1b(mixer(norm1(x)))`, then `x <- x + norm2b(ff(norm2(x)))`: a norm before and a norm
after each sublayer.  The mixer is two mixers side by side on the same input, attention behind a
short convolution (`left`) and a recurrence with a matrix state per head (`right`), whose results
are added with a constant each; the feed-forward is dense, routed, or absent.  The output head
is the embedding table, and the logits pass through `cap * tanh(logits / cap)`.

config.json keys: `architecture` (a string), `vocab`, `width`, `norm.eps`, `logit_softcap` (absent or 0:
none), and `layers`: a list of `{type, mixer: {...}, mlp: {...} | null}`:

  parallel   mixer: left_scale, right_scale,
             left:  heads, kv_heads, dim, vdim, scale, conv (taps of the short convolution; absent or 0:
                    none), rot.{base, dims, scaling.{factor, low, high, original}}
             right: heads, dim   (the decay's inner rank is the shape of `mix.right.w1`; a config may
                    also say it as `decay_rank`)
  mlp        kind "dense": ff
             kind "moe":   router.{experts, top}, expert.ff, shared.ff (absent: no shared expert)

Every size and every constant that may differ between models is read from there (or from a
tensor's shape); nothing of it stands in code.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, Mapping, Optional, Tuple

from .kezasun_config import FrequencyScaling
from .model_config import ConfigError, _optional, _required

PARALLEL = "parallel"
MIXER_TYPES = (PARALLEL,)
DENSE, MOE = "dense", "moe"


def _section(d: Dict[str, Any], key: str, where: str) -> Dict[str, Any]:
    v = d.get(key)
    if not isinstance(v, dict):
        raise ConfigError(f"{where} needs an object `{key}`")
    return v


def _positive(value, what: str):
    if not value > 0:
        raise ConfigError(f"Malilorn config {what} must be positive")
    return value


@dataclasses.dataclass(frozen=True)
class ConvAttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    conv: int  # taps of the short convolution on q, k and v; 0: none
    rot_base: float
    rot_dims: int
    rot_scaling: Optional[FrequencyScaling] = None


@dataclasses.dataclass(frozen=True)
class MatrixStateSizes:
    heads: int
    dim: int
    decay_rank: Optional[int] = None  # None until a checkpoint's shapes have said it


@dataclasses.dataclass(frozen=True)
class SideBySideSizes:
    left: ConvAttentionSizes
    right: MatrixStateSizes
    left_scale: float
    right_scale: float


@dataclasses.dataclass(frozen=True)
class DenseSizes:
    ff: int


@dataclasses.dataclass(frozen=True)
class RoutedSizes:
    experts: int
    top: int
    ff: int
    shared_ff: Optional[int] = None  # None: no shared expert


@dataclasses.dataclass(frozen=True)
class MalilornLayer:
    type: str
    mixer: SideBySideSizes
    mlp: Any  # DenseSizes, RoutedSizes or None


def _left_from(m: Dict[str, Any], where: str) -> ConvAttentionSizes:
    heads = _positive(_required(m, "heads", int), f"{where}.heads")
    dim = _positive(_required(m, "dim", int), f"{where}.dim")
    kv_heads = _positive(_optional(m, "kv_heads", int, heads), f"{where}.kv_heads")
    if heads % kv_heads:
        raise ConfigError(f"{where}.heads must be a multiple of kv_heads")
    rot = m.get("rot") if isinstance(m.get("rot"), dict) else {}
    rot_dims = _optional(rot, "dims", int, 0)
    if rot_dims % 2 or not 0 <= rot_dims <= dim:
        raise ConfigError(f"{where}.rot.dims must be even and at most dim")
    scaling = None
    if isinstance(rot.get("scaling"), dict):
        s = rot["scaling"]
        scaling = FrequencyScaling(_required(s, "factor", float), _required(s, "low", float), _required(s, "high", float),
                                   _required(s, "original", float))
        if not (scaling.factor > 0 and scaling.high > scaling.low and scaling.original > 0):
            raise ConfigError(f"{where}.rot.scaling needs factor > 0, high > low and original > 0")
    conv = _optional(m, "conv", int, 0) or 0
    if conv < 0:
        raise ConfigError(f"{where}.conv counts taps: it cannot be negative")
    sizes = ConvAttentionSizes(
        heads=heads, kv_heads=kv_heads, dim=dim,
        vdim=_positive(_optional(m, "vdim", int, dim), f"{where}.vdim"),
        scale=_optional(m, "scale", float, float(dim) ** -0.5), conv=conv,
        rot_base=_optional(rot, "base", float, 10000.0), rot_dims=rot_dims, rot_scaling=scaling,
    )
    _positive(sizes.rot_base, f"{where}.rot.base")
    return sizes


def _right_from(m: Dict[str, Any], where: str) -> MatrixStateSizes:
    rank = _optional(m, "decay_rank", int, None)
    if rank is not None:
        _positive(rank, f"{where}.decay_rank")
    return MatrixStateSizes(_positive(_required(m, "heads", int), f"{where}.heads"),
                            _positive(_required(m, "dim", int), f"{where}.dim"), rank)


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
    experts = _positive(_required(router, "experts", int), f"{where}.mlp.router.experts")
    top = _positive(_required(router, "top", int), f"{where}.mlp.router.top")
    if top > experts:
        raise ConfigError(f"{where}.mlp.router.top is larger than the number of experts")
    shared = m.get("shared")
    shared_ff = None
    if isinstance(shared, dict):
        shared_ff = _positive(_required(shared, "ff", int), f"{where}.mlp.shared.ff")
    return RoutedSizes(experts, top, _positive(_required(_section(m, "expert", f"{where}.mlp"), "ff", int),
                                               f"{where}.mlp.expert.ff"), shared_ff)


@dataclasses.dataclass(frozen=True)
class MalilornConfig:
    architecture: str
    vocab: int
    width: int
    norm_eps: float
    logit_softcap: Optional[float]
    layers: Tuple[MalilornLayer, ...]

    ARCHITECTURE = "Malilorn"

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "MalilornConfig":
        layers = d.get("layers")
        if not isinstance(layers, list):
            raise ConfigError("Missing required config field: layers")
        out = []
        for i, layer in enumerate(layers):
            where = f"layers[{i}]"
            if not isinstance(layer, dict) or layer.get("type") not in MIXER_TYPES:
                kind = layer.get("type") if isinstance(layer, dict) else layer
                raise ConfigError(f"{where}.type={kind!r} is unknown ({', '.join(MIXER_TYPES)})")
            mixer = _section(layer, "mixer", where)
            sizes = SideBySideSizes(
                _left_from(_section(mixer, "left", f"{where}.mixer"), f"{where}.mixer.left"),
                _right_from(_section(mixer, "right", f"{where}.mixer"), f"{where}.mixer.right"),
                _optional(mixer, "left_scale", float, 1.0), _optional(mixer, "right_scale", float, 1.0))
            out.append(MalilornLayer(layer["type"], sizes, _mlp_from(layer.get("mlp"), where)))
        cap = _optional(d, "logit_softcap", float, None)
        if cap is not None and cap < 0.0:
            raise ConfigError("Malilorn config logit_softcap cannot be negative")
        cfg = cls(
            architecture=str(d.get("architecture") or (d.get("architectures") or [cls.ARCHITECTURE])[0]),
            vocab=_positive(_required(d, "vocab", int), "vocab"),
            width=_positive(_required(d, "width", int), "width"),
            norm_eps=_positive(_required(_section(d, "norm", "Malilorn config"), "eps", float), "norm.eps"),
            logit_softcap=cap or None,
            layers=tuple(out),
        )
        return cfg

    def with_tensor_shapes(self, shapes: Mapping[str, Tuple[int, ...]]) -> "MalilornConfig":
        """The sizes that config.json leaves to the checkpoint, read from its tensors' shapes: the
        inner rank of every recurrence's decay (rows of `l<i>.mix.right.w1`)."""
        layers = []
        for i, layer in enumerate(self.layers):
            if layer.mixer.right.decay_rank is None:
                shape = shapes.get(f"l{i}.mix.right.w1")
                if shape is None or len(shape) != 2:
                    raise ConfigError(f"layers[{i}]: the checkpoint has no matrix l{i}.mix.right.w1 to read the decay's rank from")
                right = dataclasses.replace(layer.mixer.right, decay_rank=int(shape[0]))
                layer = dataclasses.replace(layer, mixer=dataclasses.replace(layer.mixer, right=right))
            layers.append(layer)
        return dataclasses.replace(self, layers=tuple(layers))

    def to_dict(self) -> Dict[str, Any]:
        layers = []
        for layer in self.layers:
            a, r = layer.mixer.left, layer.mixer.right
            rot: Dict[str, Any] = {"base": a.rot_base, "dims": a.rot_dims}
            if a.rot_scaling is not None:
                s = a.rot_scaling
                rot["scaling"] = {"factor": s.factor, "low": s.low, "high": s.high, "original": s.original}
            left = {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim, "scale": a.scale, "rot": rot}
            if a.conv:
                left["conv"] = a.conv
            right: Dict[str, Any] = {"heads": r.heads, "dim": r.dim}
            if r.decay_rank is not None:
                right["decay_rank"] = r.decay_rank
            f = layer.mlp
            if f is None:
                mlp = None
            elif isinstance(f, DenseSizes):
                mlp = {"kind": DENSE, "ff": f.ff}
            else:
                mlp = {"kind": MOE, "expert": {"ff": f.ff}, "router": {"experts": f.experts, "top": f.top}}
                if f.shared_ff is not None:
                    mlp["shared"] = {"ff": f.shared_ff}
            layers.append({"type": layer.type, "mlp": mlp,
                           "mixer": {"left": left, "right": right, "left_scale": layer.mixer.left_scale,
                                     "right_scale": layer.mixer.right_scale}})
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
               "norm": {"eps": self.norm_eps}, "layers": layers}
        if self.logit_softcap:
            out["logit_softcap"] = self.logit_softcap
        return out
